"""The recording of one layer's library calls and their repetition for like layers: the host-side pieces."""
import ctypes

import pytest
import torch

from tokenizer_amd.kernels import KernelError, LaunchTape, _RecordingLibrary
from tokenizer_amd.parts.base import Repeatable, repeatable_of
from tokenizer_amd.parts.model import _addresses_put, _coming, _Make


class FakeLibrary:
    """Stands in for the loaded library: remembers what it was called with."""

    def __init__(self):
        self.seen = []
        self.status = 0

    def ta_something(self, *args):
        self.seen.append(tuple(a.value if isinstance(a, (ctypes.c_void_p, ctypes.c_float)) else a for a in args))
        return self.status


def test_recorded_calls_are_made_again_with_addresses_put_in_place():
    fake, tape = FakeLibrary(), LaunchTape()
    lib = _RecordingLibrary(fake, tape)
    assert lib.ta_something(ctypes.c_void_p(1000), ctypes.c_void_p(0), 7, ctypes.c_float(0.5), ctypes.c_void_p(2000)) == 0
    assert lib.ta_something(ctypes.c_void_p(3000), 1000) == 0          # the plain integer 1000 is no address
    assert len(tape.calls) == 2 and fake.seen[0] == (1000, None, 7, 0.5, 2000)
    fake.seen.clear()
    tape.replay({1000: 1111, 3000: 3333, 7: 8})
    assert fake.seen == [(1111, None, 7, 0.5, 2000), (3333, 1000)]
    fake.seen.clear()
    tape.replay({})
    assert fake.seen == [(1000, None, 7, 0.5, 2000), (3000, 1000)]
    fake.status = -3                                                  # a call that ends otherwise than when recorded
    with pytest.raises(KernelError, match="returned -3 where it had returned 0"):
        tape.replay({})


def test_one_address_cannot_stand_for_two():
    assert _addresses_put((10, 20, 0, 30), (11, 21, 0, 30)) == {10: 11, 20: 21}
    assert _addresses_put((10, 10), (11, 11)) == {10: 11}
    assert _addresses_put((10, 10), (11, 12)) is False               # one tensor twice there, two tensors here
    assert _addresses_put((10, 20), (11, 11)) == {10: 11, 20: 11}


def test_what_a_layer_is_handed_has_a_form_and_addresses():
    assert _coming(None) == ("none", ())
    x = torch.zeros(3, 8)
    form, addresses = _coming(x)
    assert form[0] == "tensor" and addresses == (x.data_ptr(),)
    assert _coming(torch.zeros(3, 8))[0] == form and _coming(torch.zeros(4, 8))[0] != form

    class Parts:
        partial, bias, dtype = torch.zeros(2, 3, 8), None, torch.bfloat16

    form, addresses = _coming(Parts())
    assert form[0] == "parts" and addresses == (Parts.partial.data_ptr(),)

    class Odd:
        pass

    assert _coming(Odd())[0] is None                                  # an unknown form: the layer runs on its own


def test_the_promise_is_the_class_own_and_layout_is_part_of_a_make():
    class Base:
        def repeatable(self):
            return Repeatable(("base",), ())

    class Child(Base):                    # overrides nothing, promises nothing
        pass

    class Again(Base):
        def repeatable(self):
            return Repeatable(("again",), ())

    assert repeatable_of(Base()).constants == ("base",)
    assert repeatable_of(Child()) is None
    assert repeatable_of(Again()).constants == ("again",)
    assert repeatable_of(None).constants == ("absent",)
    a, b = torch.zeros(4, 8), torch.zeros(4, 8)
    assert _Make(("k",), (a, None)).key == _Make(("k",), (b, None)).key
    assert _Make(("k",), (a, None)).key != _Make(("k",), (b.t(), None)).key          # another layout
    assert _Make(("k",), (a, None)).key != _Make(("k",), (torch.zeros(4, 8, dtype=torch.float64), None)).key
    assert _Make(("k",), (a, None)).key != _Make(("j",), (b, None)).key
