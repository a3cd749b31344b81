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


# ---------------------------------------------------------------- the model's use of the tape, on a stand-in library
class _ToyLibrary:
    """A library of one function that notes the addresses it is given."""

    def __init__(self):
        self.seen = []

    def ta_toy(self, *args):
        self.seen.append(tuple(a.value for a in args))
        return 0


def _toy_model(kind: str, n_layers: int = 4):
    """A model of `n_layers` layers of one toy mixer (registered under `kind`), on the CPU, whose only library call
    is `ta_toy(w1, w2, key pages, out)`; returns (model, library)."""
    from tokenizer_amd import kernels
    from tokenizer_amd.parts import DecoderModel, Runtime
    from tokenizer_amd.parts.spec import LayerSpec, MixerSpec, ModelSpec, NormSpec, ScheduleEntry

    class ToyOps(kernels.Ops):
        def __init__(self):
            self._loaded = _ToyLibrary()

        def embedding(self, ids, table, out):
            return out.copy_(table[ids.long()].float())

        def add_rmsnorm(self, residual, delta, weight, eps, out, rows=None, store_residual=True):
            return out.zero_()

        def linear(self, x, weight, bias=None, out=None, out_dtype=None, pending=False):
            return x.float() @ weight.float().t()

    norm = NormSpec("rmsnorm", 8, 1e-6)
    layers = tuple(LayerSpec("pre_norm", MixerSpec(kind, 8), None, norm, None, mixer_prefix=f"l{i}.mix",
                             mixer_norm_prefix=f"l{i}.norm") for i in range(n_layers))
    spec = ModelSpec("Toy", 16, 8, 64, "embed", layers, tuple(ScheduleEntry(i) for i in range(n_layers)), norm,
                     "norm", True, "head")
    tensors = {"embed": torch.randn(16, 8), "norm.weight": torch.ones(8)}
    for i in range(n_layers):
        tensors.update({f"l{i}.norm.weight": torch.ones(8), f"l{i}.mix.w1": torch.randn(8, 8),
                        f"l{i}.mix.w2": torch.randn(8, 8)})
    ops = ToyOps()
    return DecoderModel(spec, tensors, Runtime(torch.float32, torch.device("cpu"), ops)), ops._loaded


def _register_toy_mixers():
    from tokenizer_amd.kernels import _ptr
    from tokenizer_amd.parts.base import MIXERS, Mixer
    from tokenizer_amd.parts.spec import TensorSpec
    if "toy_honest" in MIXERS.kinds():
        return

    class Toy(Mixer):
        def __init__(self, spec, tensors, runtime):
            self.w1, self.w2, self.runtime = tensors["w1"], tensors["w2"], runtime

        @staticmethod
        def tensor_specs(spec):
            return {"w1": TensorSpec((8, 8)), "w2": TensorSpec((8, 8))}

        def forward_normed(self, residual, delta, norm, ctx, cache):
            x = norm.apply(residual, delta)
            out = torch.empty_like(x)
            self.runtime.ops.lib.ta_toy(_ptr(self.w1), _ptr(self.w2), _ptr(cache.k_pages), _ptr(out))
            return out

    @MIXERS.register("toy_honest")
    class Honest(Toy):
        def repeatable(self):
            return Repeatable(("toy",), (self.w1, self.w2))

    @MIXERS.register("toy_hiding")
    class Hiding(Toy):
        def repeatable(self):
            return Repeatable(("toy",), (self.w1,))             # w2 goes into the call too, and is not said


def _toy_step(model, pages):
    from types import SimpleNamespace
    from tokenizer_amd.parts import LayerCache
    ctx = SimpleNamespace(n_tokens=3, token_ids=torch.tensor([1, 2, 3], dtype=torch.int32),
                          want_rows=torch.tensor([2], dtype=torch.int32))
    caches = [LayerCache(group=0, k_pages=k, v_pages=v) for k, v in pages]
    return caches, ctx


def test_like_layers_are_given_their_own_tensors_and_a_hidden_tensor_stops_the_repeating():
    _register_toy_mixers()
    for kind, repeats in (("toy_honest", True), ("toy_hiding", False)):
        model, library = _toy_model(kind)
        pages = [(torch.zeros(4), torch.zeros(4)) for _ in model.blocks]
        caches, ctx = _toy_step(model, pages)
        for _ in range(2):
            library.seen.clear()
            model.forward(ctx, caches)
            assert len(library.seen) == len(model.blocks)
            for block, (k, _), call in zip(model.blocks, pages, library.seen):
                assert call[:3] == (block.mixer.w1.data_ptr(), block.mixer.w2.data_ptr(), k.data_ptr())
        # The first layer is handed nothing and is a make of its own; the second is recorded; the rest repeat it,
        # unless the recording shows a tensor the parts hold and did not list.
        assert (model.layers_repeated > 0) == repeats
        assert (model.promises_broken > 0) == (not repeats)


def test_a_model_outlives_its_engines_and_their_address_maps_go_with_them():
    """One model under one cache after another (as a benchmark that makes an engine per batch size does): the maps
    from a recorded layer's addresses to a like layer's belong to the cache entries, so a later engine's layers are
    never given an earlier engine's pages, whatever ids its objects happen to get."""
    import gc
    _register_toy_mixers()
    model, library = _toy_model("toy_honest", n_layers=6)
    for round_ in range(12):
        pages = [(torch.zeros(4 + round_), torch.zeros(4)) for _ in model.blocks]
        caches, ctx = _toy_step(model, pages)
        library.seen.clear()
        model.forward(ctx, caches)
        model.forward(ctx, caches)
        for call, (k, _), block in zip(library.seen[len(model.blocks):], pages, model.blocks):
            assert call[:3] == (block.mixer.w1.data_ptr(), block.mixer.w2.data_ptr(), k.data_ptr()), round_
        del caches, pages
        gc.collect()
    assert model.layers_repeated > 0 and not hasattr(model, "_put")
