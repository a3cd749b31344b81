"""Bindings of the hand-written HIP kernels (loaded through ctypes).

There is no fallback: without a GPU and the built library `get_ops()` raises.
Every wrapper checks on the host that its operands have the shapes, dtypes and
layout its kernel and grid assume, and launches on torch's current stream.
"""
from __future__ import annotations

import contextlib
import ctypes
import math
import threading

import torch

from . import build as _build

_F32, _BF16 = 0, 1
_CODES = {torch.float32: _F32, torch.bfloat16: _BF16}


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def _raw_stream(device_index: int) -> int:
    return torch._C._cuda_getCurrentRawStream(device_index)


class _Recording(threading.local):
    """What the thread that records a layer's calls is recording into (nothing, for every other thread)."""
    library = None        # the `_RecordingLibrary` that stands in for the loaded one
    keep: list | None = None      # every tensor whose address went into a recorded call


_RECORDING = _Recording()


def _ptr(tensor: torch.Tensor | None) -> ctypes.c_void_p:
    if tensor is None:
        return ctypes.c_void_p(0)
    keep = _RECORDING.keep
    if keep is not None:
        keep.append(tensor)
    return ctypes.c_void_p(tensor.data_ptr())


def _need(cond: bool, message: str) -> None:
    if not cond:
        raise KernelError(message)


def _dev(*tensors: torch.Tensor | None) -> None:
    for tensor in tensors:
        if tensor is not None:
            _need(tensor.is_cuda, "kernel operands must live on the GPU")
            _need(tensor.is_contiguous(), "kernel operands must be contiguous")


def _parts_of_k(k: int, splits: int, step: int) -> int:
    """Into how many parts K really falls when `splits` are asked for and a part is a multiple of `step`."""
    if splits <= 1:
        return 1
    chunk = -(-(-(-k // splits)) // step) * step
    return -(-k // chunk)


class PendingSum:
    """A product whose K was cut over workgroups, before its parts are added: float32 slabs [parts, M, N] and
    the bias that joins their sum.  `Ops.add_rmsnorm` takes it as the delta and adds the parts, the bias and the
    residual and normalises in one kernel; `resolve()` adds the parts on their own and gives the product."""

    def __init__(self, ops: "Ops", partial: torch.Tensor, bias: torch.Tensor | None, dtype: torch.dtype):
        self.ops, self.partial, self.bias, self.dtype = ops, partial, bias, dtype
        self.shape = tuple(partial.shape[1:])

    def resolve(self) -> torch.Tensor:
        parts, m, n = self.partial.shape
        out = torch.empty((m, n), dtype=self.dtype, device=self.partial.device)
        self.ops._check(self.ops.lib.ta_splitk_reduce(_ptr(self.partial), _ptr(self.bias), _ptr(out), m, n, n, parts,
                                                      _code(self.dtype), self.ops._stream()), "splitk_reduce")
        return out


class LaunchTape:
    """The library calls that one layer made, in order, each with its arguments and the status it returned.

    Layers of the same make (the same parts with the same sizes and constants) make the same calls on a step's
    batch; only the addresses of their own tensors differ.  `replay(put)` makes the calls again with every
    address found in `put` replaced: the Python between the calls (checks, choices of kernel and split, buffers)
    ran once, for the recorded layer.  The tape keeps every tensor whose address it holds, so the recorded
    layer's buffers are there for the layers that use them again (all on one stream, one after another).
    """

    def __init__(self):
        self.calls: list[tuple] = []          # (function, arguments, status, ((index, address), ...))
        self.keep: list[torch.Tensor] = []

    def replay(self, put: dict[int, int]) -> None:
        for function, args, status, addresses in self.calls:
            changed = None
            for index, address in addresses:
                to = put.get(address)
                if to is not None:
                    if changed is None:
                        changed = list(args)
                    changed[index] = ctypes.c_void_p(to)
            got = function(*args) if changed is None else function(*changed)
            if got != status:
                raise KernelError(f"a recorded call returned {got} where it had returned {status}")

    def addresses(self) -> set:
        """Every address that went into a recorded call."""
        return {address for _, _, _, addresses in self.calls for _, address in addresses}


class _RecordingLibrary:
    """Stands in for the loaded library while a tape is recorded: every call goes through and onto the tape."""

    def __init__(self, lib, tape: LaunchTape):
        self._lib, self._tape = lib, tape

    def __getattr__(self, name):
        function = getattr(self._lib, name)
        calls = self._tape.calls

        def call(*args):
            status = function(*args)
            calls.append((function, args, status,
                          tuple((i, a.value) for i, a in enumerate(args) if isinstance(a, ctypes.c_void_p) and a.value)))
            return status
        return call


class Ops:
    """The kernel library.  One instance per process; see `get_ops()`."""

    def __init__(self, path: str):
        self.path = path
        self._loaded = ctypes.CDLL(path)
        for name in ("ta_embedding", "ta_add_rmsnorm", "ta_silu_gate", "ta_rope_store",
                     "ta_paged_attention_generic", "ta_decode_attention_bf16", "ta_prefill_attention_bf16",
                     "ta_prefill_attention_shared_plan", "ta_prefill_attention_key_splits",
                     "ta_gemm_f32", "ta_gemm_bf16", "ta_gemm_bf16_splitk", "ta_gemm_skinny_bf16",
                     "ta_gemm_skinny_bf16_splitk", "ta_gemm_skinny_qkv_rope", "ta_fused_norm_qkv_rope",
                     "ta_fused_norm_gated", "ta_fused_linear_residual", "ta_fused_qkv_rope", "ta_fused_gated",
                     "ta_splitk_reduce", "ta_splitk_add_rmsnorm", "ta_argmax", "ta_argmax_next_step", "ta_sample",
                     "ta_sample_workspace_words", "ta_library_gemm_bf16", "ta_compute_units", "ta_read_stream"):
            getattr(self.lib, name).restype = ctypes.c_int
        self.lib.ta_library_gemm_bf16.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 + [
            ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
        self._workspaces: dict[int, torch.Tensor] = {}
        self.compute_units = int(self._loaded.ta_compute_units())     # what the splits below aim to fill

    @staticmethod
    def _stream() -> ctypes.c_void_p:
        """The current HIP stream of the current device (the raw handle, which costs far less to ask for
        than a stream object; every launch asks)."""
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))

    LIBRARY_WORKSPACE = 128 << 20      # bytes the vendor's matrix library may use per device (its first choice for
    #                                    the widest products of a 7B model wants some 60 MB)

    def _workspace(self, device: torch.device) -> torch.Tensor:
        index = device.index if device.index is not None else torch.cuda.current_device()
        space = self._workspaces.get(index)
        if space is None:
            space = self._workspaces[index] = torch.empty(self.LIBRARY_WORKSPACE, dtype=torch.uint8, device=device)
        return space

    @staticmethod
    def _check(status: int, what: str) -> None:
        if status != 0:
            raise KernelError(f"{what} failed with status {status}"
                              + (" (sizes the kernel does not take)" if status < 0 else " (HIP error)"))

    @property
    def lib(self):
        """The loaded library, or, on a thread that is recording a layer's calls, the recorder in front of it."""
        return _RECORDING.library or self._loaded

    @contextlib.contextmanager
    def record_launches(self):
        """Record every library call this thread makes inside the block on a `LaunchTape` (which the block
        receives).  Other threads' calls are not touched; a recording inside a recording takes over until it ends."""
        tape = LaunchTape()
        before = _RECORDING.library, _RECORDING.keep
        _RECORDING.library, _RECORDING.keep = _RecordingLibrary(self._loaded, tape), tape.keep
        try:
            yield tape
        finally:
            _RECORDING.library, _RECORDING.keep = before

    # ------------------------------------------------------------------ yardstick
    def read_stream(self, data: torch.Tensor, workgroups: int | None = None) -> torch.Tensor:
        """Read every byte of `data` once in the access pattern of the weight-streaming kernels; returns the xor
        of its 32-bit words per workgroup (uint32 as int32 [workgroups]).  A yardstick for what a kernel bound by
        HBM reaches on this device; no model code calls it."""
        _dev(data)
        nbytes = data.numel() * data.element_size()
        _need(nbytes % 16 == 0 and data.data_ptr() % 16 == 0, "the buffer must be whole 16-byte words")
        workgroups = workgroups or 8 * self.compute_units
        out = torch.empty(workgroups, dtype=torch.int32, device=data.device)
        self._check(self.lib.ta_read_stream(_ptr(data), ctypes.c_size_t(nbytes), _ptr(out), workgroups, self._stream()),
                    "read_stream")
        return out

    # ------------------------------------------------------------------ embedding
    def embedding(self, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out[t] = table[ids[t]] as float32.  ids int32 [T]; table [V, H]; out float32 [T, H]."""
        _dev(ids, table, out)
        n, (vocab, hidden) = ids.numel(), table.shape
        _need(ids.dtype == torch.int32 and ids.dim() == 1, "ids must be int32 [T]")
        _need(out.dtype == torch.float32 and tuple(out.shape) == (n, hidden), "out must be float32 [T, H]")
        self._check(self.lib.ta_embedding(_ptr(ids), _ptr(table), _ptr(out), n, hidden, vocab,
                                          _code(table.dtype), self._stream()), "embedding")
        return out

    # ---------------------------------------------------------------------- norm
    def add_rmsnorm(self, residual: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor,
                    eps: float, out: torch.Tensor, rows: torch.Tensor | None = None,
                    store_residual: bool = True) -> torch.Tensor:
        """x = residual[r] (+ delta[r]); optionally residual[r] = x; out[i] = rmsnorm(x) * weight.

        residual float32 [T, H]; delta [T, H] in out's dtype, None, or a `PendingSum` (the parts of a product
        still to be added: they are added here, in the same kernel); weight float32 [H];
        rows int32 [R] picks the rows (None: all, R = T); out [R, H].
        """
        if isinstance(delta, PendingSum):
            n_tokens, hidden = residual.shape
            if (rows is not None or not store_residual or hidden % 4 or hidden > 4096
                    or delta.shape != (n_tokens, hidden)):
                delta = delta.resolve()
            else:
                _dev(residual, weight, out)
                _need(residual.dtype == torch.float32, "the residual stream is float32")
                _need(weight.dtype == torch.float32 and weight.numel() == hidden, "norm weight must be float32 [H]")
                _need(tuple(out.shape) == (n_tokens, hidden) and out.dtype == delta.dtype, "norm output has the wrong shape")
                self._check(self.lib.ta_splitk_add_rmsnorm(
                    _ptr(residual), _ptr(delta.partial), delta.partial.shape[0], _ptr(delta.bias), _ptr(weight),
                    _ptr(out), n_tokens, hidden, ctypes.c_float(eps), _code(out.dtype), self._stream()),
                    "splitk_add_rmsnorm")
                return out
        _dev(residual, delta, weight, out, rows)
        n_tokens, hidden = residual.shape
        n_rows = n_tokens if rows is None else rows.numel()
        _need(residual.dtype == torch.float32, "the residual stream is float32")
        _need(weight.dtype == torch.float32 and weight.numel() == hidden, "norm weight must be float32 [H]")
        _need(tuple(out.shape) == (n_rows, hidden), "norm output has the wrong shape")
        if delta is not None:
            _need(delta.shape == residual.shape and delta.dtype == out.dtype, "delta must match residual and out")
        if rows is not None:
            _need(rows.dtype == torch.int32, "rows must be int32")
            _need(not store_residual, "a row subset never stores the residual")
        self._check(self.lib.ta_add_rmsnorm(_ptr(residual), _ptr(delta), _ptr(weight), _ptr(out), _ptr(rows),
                                            n_rows, hidden, ctypes.c_float(eps), int(store_residual),
                                            _code(out.dtype), self._stream()), "add_rmsnorm")
        return out

    # ------------------------------------------------------------- gated activation
    def silu_gate(self, gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out = silu(gate_up[:, :I]) * gate_up[:, I:].  gate_up [T, 2I]; out [T, I]."""
        _dev(gate_up, out)
        n_tokens, two_inner = gate_up.shape
        _need(two_inner % 2 == 0 and tuple(out.shape) == (n_tokens, two_inner // 2) and out.dtype == gate_up.dtype,
              "silu_gate shapes do not fit")
        self._check(self.lib.ta_silu_gate(_ptr(gate_up), _ptr(out), n_tokens, two_inner // 2,
                                          _code(out.dtype), self._stream()), "silu_gate")
        return out

    # ----------------------------------------------------------------------- rope
    def rope_store(self, qkv: torch.Tensor, bias: torch.Tensor | None, positions: torch.Tensor,
                   cos_sin: torch.Tensor | None, slots: torch.Tensor | None,
                   k_pages: torch.Tensor | None, v_pages: torch.Tensor | None,
                   n_q: int, n_kv: int, head_dim: int) -> None:
        """Add bias, rotate q and k heads in place, store k and v heads into their pages.

        qkv [T, (n_q + 2 n_kv) d]; bias float32 or None; positions int32 [T];
        cos_sin float32 [P, d] (cos half, sin half) or None for no rotation;
        slots int32 [T] (page * page_size + offset, negative = skip) or None;
        key pages [n_pages, n_kv, page_size, d], value pages [n_pages, n_kv, d, page_size].
        """
        _dev(qkv, bias, positions, cos_sin, slots, k_pages, v_pages)
        n_tokens, width = qkv.shape
        _need(width == (n_q + 2 * n_kv) * head_dim, "qkv width does not match the head counts")
        _need(head_dim % 2 == 0, "head size must be even")
        _need(positions.dtype == torch.int32 and positions.numel() == n_tokens, "positions must be int32 [T]")
        page_size = 1
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() == width, "bias must be float32 of the qkv width")
        if cos_sin is not None:
            _need(cos_sin.dtype == torch.float32 and cos_sin.shape[1] == head_dim, "cos_sin must be float32 [P, d]")
        if slots is not None:
            _need(slots.dtype == torch.int32 and slots.numel() == n_tokens, "slots must be int32 [T]")
            _need(k_pages is not None and v_pages is not None, "slots without pages")
            _need(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "pages must have the dtype of qkv")
            page_size = self._page_size(k_pages, v_pages, n_kv, head_dim)
        self._check(self.lib.ta_rope_store(_ptr(qkv), width, _ptr(bias), _ptr(positions), _ptr(cos_sin),
                                           _ptr(slots), _ptr(k_pages), _ptr(v_pages), n_tokens, n_q, n_kv,
                                           head_dim, page_size, _code(qkv.dtype), self._stream()), "rope_store")

    @staticmethod
    def _page_size(k_pages: torch.Tensor, v_pages: torch.Tensor, n_kv: int, head_dim: int) -> int:
        _need(k_pages.dim() == 4 and k_pages.shape[1] == n_kv and k_pages.shape[3] == head_dim,
              "key pages must be [n_pages, n_kv, page_size, d]")
        page_size = k_pages.shape[2]
        _need(tuple(v_pages.shape) == (k_pages.shape[0], n_kv, head_dim, page_size),
              "value pages must be [n_pages, n_kv, d, page_size]")
        _need(k_pages.numel() < 2 ** 31, "a layer's pages must hold fewer than 2^31 elements")
        return page_size

    # ------------------------------------------------------------------ attention
    def paged_attention(self, qkv: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor,
                        v_pages: torch.Tensor, positions: torch.Tensor, entry_of_token: torch.Tensor,
                        block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int,
                        window: int | None, scale: float, max_position: int | None = None,
                        batch=None) -> torch.Tensor:
        """Causal attention of every token over the pages of its request.

        qkv [T, >= n_q d] (query heads first); out [T, n_q d]; key pages [n_pages, n_kv, page_size, d],
        value pages [n_pages, n_kv, d, page_size];
        positions, entry_of_token int32 [T]; block_table int32 [E, P]; a token at position p sees keys
        max(0, p - window)..p.  `max_position` (host) lets the wrapper check that the table is wide enough.
        `batch` (a StepContext of the same tokens) lets bfloat16 batches run the tiled kernel on prompt
        portions and the split kernel on single tokens; without it every token goes through the latter.
        """
        _dev(qkv, out, k_pages, v_pages, positions, entry_of_token, block_table)
        n_tokens = qkv.shape[0]
        _need(qkv.shape[1] >= n_q * head_dim, "qkv is narrower than the query heads")
        _need(tuple(out.shape) == (n_tokens, n_q * head_dim) and out.dtype == qkv.dtype, "attention output shape")
        _need(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "pages must have the dtype of qkv")
        page_size = self._page_size(k_pages, v_pages, n_kv, head_dim)
        _need(positions.dtype == torch.int32 and positions.numel() == n_tokens, "positions must be int32 [T]")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() == n_tokens, "entry_of_token must be int32 [T]")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 [E, P]")
        _need(n_kv > 0 and n_q % n_kv == 0, "query heads must be a multiple of kv heads")
        _need(0 < head_dim <= 256, "head sizes up to 256 are supported")
        if max_position is not None:
            _need(max_position // page_size < block_table.shape[1], "block table is too narrow for the positions")
        if (qkv.dtype == torch.bfloat16 and head_dim in self.DECODE_HEAD_DIMS and page_size % 16 == 0
                and qkv.shape[1] % 8 == 0 and self.use_fast_attention):
            args = (qkv, out, k_pages, v_pages, positions, entry_of_token, block_table, n_q, n_kv, head_dim,
                    page_size, window, scale, max_position)
            if batch is None:
                return self._decode_attention(*args)
            if batch.q_tiles.numel() == 0:
                # One token per request: request e is row e, the kernel needs no entry-of-token lookup.
                return self._decode_attention(*args, identity_entries=batch.n_tokens == block_table.shape[0])
            _need(batch.n_tokens == n_tokens and batch.cu_q.numel() == block_table.shape[0] + 1,
                  "the batch description does not belong to these tokens")
            n_tiles, choice = batch.q_tiles.shape[0], (
                -1 if window is None else int(window), self.prefill_shape, int(batch.max_position) + 1,
                self.prefill_waves, self.prefill_shared)
            # A few tiles behind a long context: the launcher cuts each tile's keys over workgroups, whose states
            # a second kernel merges; it says into how many parts, and gets the buffers for them.
            parts = self.lib.ta_prefill_attention_key_splits(n_tiles, n_q, n_kv, head_dim, *choice) if self.prefill_key_splits else 1
            part_o = part_ml = None
            if parts > 1:
                part_o = torch.empty((n_tiles * 16, n_q, parts, head_dim), dtype=torch.float32, device=qkv.device)
                part_ml = torch.empty((n_tiles * 16, n_q, parts, 2), dtype=torch.float32, device=qkv.device)
            self._check(self.lib.ta_prefill_attention_bf16(
                _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(batch.q_tiles),
                n_tiles, _ptr(batch.cu_q), _ptr(batch.first_position), _ptr(block_table),
                block_table.shape[1], n_q, n_kv, head_dim, page_size, choice[0], ctypes.c_float(scale), *choice[1:],
                _ptr(part_o), _ptr(part_ml), self._stream()), "prefill_attention")
            if batch.decode_rows.numel():
                self._decode_attention(*args, rows=batch.decode_rows)
            return out
        self._check(self.lib.ta_paged_attention_generic(
            _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(positions),
            _ptr(entry_of_token), _ptr(block_table), block_table.shape[1], n_tokens, n_q, n_kv, head_dim,
            page_size, -1 if window is None else int(window), ctypes.c_float(scale), _code(qkv.dtype),
            self._stream()), "paged_attention")
        return out

    DECODE_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256)
    use_fast_attention = True     # tests switch it off to reach the generic kernel in bfloat16
    prefill_waves = 0             # waves that share a tile's keys in the per-wave prompt kernel: 0 lets the launcher choose;
    #                               asking for a number asks for that kernel
    prefill_shape = 0             # shape of the workgroup-shared prompt kernel when it is asked for: heads a wave
    #                               (1 or 2), + 10 for two key groups in a workgroup; 0: its own choice
    prefill_shared = 0            # the prompt kernel whose waves share a block of keys through LDS: 1 = wherever it has
    #                               an instance, -1 = never, 0 = where the launcher expects it to be the faster one
    prefill_key_splits = True     # whether the prompt kernel may cut a tile's keys over workgroups (tests switch it off)
    target_workgroups = 1024      # what the split of the key range aims at
    min_split_keys = 128          # ... in parts of at least so many keys (a block of 32 for each of a workgroup's four waves)
    PLAN_KEYS = 512               # launch shapes depend on the context only through its multiple of this

    def _decode_attention(self, qkv, out, k_pages, v_pages, positions, entry_of_token, block_table,
                          n_q, n_kv, head_dim, page_size, window, scale, max_position, rows=None,
                          identity_entries=False):
        """Matrix-core attention of single tokens with the key range split over workgroups."""
        n_items = qkv.shape[0] if rows is None else rows.numel()
        max_keys = (block_table.shape[1] * page_size) if max_position is None else max_position + 1
        # The split is planned for the context rounded up to a multiple of 512 keys: a step that replays a
        # graph captured for a whole range of contexts then splits exactly as the same step run on its own.
        max_keys = -(-max_keys // self.PLAN_KEYS) * self.PLAN_KEYS
        if window is not None:
            max_keys = min(max_keys, window + 32)
        head_blocks = -(-(n_q // n_kv) // 16)
        per_split = max(1, self.target_workgroups // max(1, n_items * n_kv * head_blocks))
        split_keys = max(self.min_split_keys, -(-max_keys // per_split))
        split_keys = -(-split_keys // 32) * 32
        splits = max(1, -(-(max_keys + 31) // split_keys))
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty((n_items, n_q, splits, head_dim), dtype=torch.float32, device=qkv.device)
            part_ml = torch.empty((n_items, n_q, splits, 2), dtype=torch.float32, device=qkv.device)
        self._check(self.lib.ta_decode_attention_bf16(
            _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(rows), _ptr(positions),
            _ptr(None if identity_entries and rows is None else entry_of_token), _ptr(block_table),
            block_table.shape[1], _ptr(part_o), _ptr(part_ml), n_items,
            n_q, n_kv, head_dim, page_size, -1 if window is None else int(window), ctypes.c_float(scale),
            split_keys, splits, self._stream()), "decode_attention")
        return out

    # --------------------------------------------------------------------- linear
    takes_pending = True      # `linear(pending=True)` and `add_rmsnorm` with a `PendingSum` exist here

    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
               out: torch.Tensor | None = None, out_dtype: torch.dtype | None = None,
               pending: bool = False) -> "torch.Tensor | PendingSum":
        """out = x @ weight.T (+ bias).  x [M, K] (rows may be strided); weight [N, K]; bias float32 [N].

        float32 operands run on plain multiply-adds; bfloat16 operands on the matrix cores with
        float accumulation and a bfloat16 or float32 result.  `pending=True` allows the result to come back
        as a `PendingSum` when K is cut over workgroups: whoever takes it next (the norm that follows) adds the
        parts in its own kernel and the addition's launch is saved.
        """
        _need(x.is_cuda and weight.is_cuda, "kernel operands must live on the GPU")
        _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "linear shapes do not fit")
        _need(x.stride(1) == 1 and weight.is_contiguous(), "linear operands must have contiguous rows")
        _need(x.dtype == weight.dtype, "x and weight must share a dtype")
        m, k = x.shape
        n = weight.shape[0]
        lda = x.stride(0) if m > 1 else k
        if out_dtype is None:
            out_dtype = x.dtype if out is None else out.dtype
        pending = pending and out is None and x.dtype == torch.bfloat16
        if out is None and not pending:
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        if out is not None:
            _need(tuple(out.shape) == (m, n) and out.is_contiguous() and out.dtype == out_dtype, "linear output shape")
        if bias is not None:
            _need(bias.is_cuda and bias.dtype == torch.float32 and bias.numel() == n, "bias must be float32 [N]")
        if x.dtype == torch.float32:
            _need(out_dtype == torch.float32, "float32 products give float32")
            status = self.lib.ta_gemm_f32(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), m, n, k, lda, n,
                                          self._stream())
        else:
            _need(x.dtype == torch.bfloat16, "linear takes float32 or bfloat16")
            _need(k % 8 == 0 and lda % 8 == 0, "bfloat16 products need K and the row stride to be multiples of 8")
            _need(x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
            streaming_splits = self._streaming_splits(m, n, k, pending)
            if streaming_splits > 1 and self.split_k_kind == "streaming":
                # 17 to 64 rows, a long K and few output columns (the down projection of a decode batch): the
                # weight-streaming kernel with K cut over workgroups, so that every compute unit streams a share
                # of the weights; the parts are added in a fixed order by a second small kernel.
                parts = _parts_of_k(k, streaming_splits, 32)
                leave = pending and parts > 1
                if out is None and not leave:
                    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
                partial = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
                self._check(self.lib.ta_gemm_skinny_bf16_splitk(
                    _ptr(x), lda, _ptr(weight), _ptr(bias), _ptr(None if leave else out), n, _ptr(partial), m, n, k,
                    _code(out_dtype), streaming_splits, self.skinny_column_blocks, self._stream()), "linear")
                return PendingSum(self, partial, bias, out_dtype) if leave else out
            splits = self._k_splits(m, n, k, pending)
            if splits > 1:
                # The same with the tiled kernel.
                parts = _parts_of_k(k, splits, 64)
                leave = pending and parts > 1
                if out is None and not leave:
                    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
                partial = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
                self._check(self.lib.ta_gemm_bf16_splitk(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(None if leave else out), _ptr(partial), m, n, k, lda, n,
                    _code(out_dtype), splits, self._stream()), "linear")
                return PendingSum(self, partial, bias, out_dtype) if leave else out
            if out is None:
                out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            if m > self.SKINNY_ROWS:
                to_library = self.capturing or m * n * k >= self.EAGER_LIBRARY_WORK
            else:
                to_library = m > self.FUSED_ROWS and ((k >= 2048 and n <= 4096) or n * k >= self.LIBRARY_WEIGHT)
            if to_library and self.use_library_gemm and out_dtype == torch.bfloat16:
                # Plain products of more than 64 rows go to the vendor's library (hipBLASLt, called from
                # library_gemm.hip), as the reference's engine uses a library for its matrix products: on the
                # device's own clock (launches recorded in a graph, weights cold) it is ahead of the tiled
                # kernel of this package for nearly every shape of the 0.5B to 7B models.  So do products of 17
                # to 64 rows with a big weight matrix (every tile of the weight-streaming kernel reads all the
                # rows again, which costs more than the weights once there are more than sixteen of them), and
                # those with a long K and few output columns that the kernels above did not take.  The float32 bias
                # joins the library's float accumulator as it joins the kernels' own.  A launch of the library
                # costs the host some 15 us against 4 us for a kernel of this package: outside graph capture,
                # products of more than 64 rows that are over on the device in about that time stay with the
                # tiled kernel (steps of small models with few tokens are bound by the host's launches).
                # In the run that warms a step up before it is recorded the library is told that the shape
                # will come again: it then times its candidates for a big product and keeps the fastest.
                space = self._workspace(x.device)
                status = self.lib.ta_library_gemm_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), m, n, k, lda, n,
                                                       _ptr(space), space.numel(), int(self.capturing),
                                                       self._stream())
                if status != -3:                  # -3: no algorithm for this shape, the kernels below take it
                    self._check(status, "linear (vendor library)")
                    return out
            if m <= self.FUSED_ROWS or (m <= self.SKINNY_ROWS and n < self.WIDE_OUTPUT):
                status = self.lib.ta_gemm_skinny_bf16(_ptr(x), lda, _ptr(weight), _ptr(bias), _ptr(out), n, m, n, k,
                                                      _code(out_dtype), 0, self.skinny_column_blocks, self._stream())
            else:
                status = self.lib.ta_gemm_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), m, n, k, lda, n,
                                               _code(out_dtype), self._stream())
        self._check(status, "linear")
        return out

    use_split_k = True
    skinny_column_blocks = 0   # blocks of sixteen output columns per workgroup of the weight-streaming kernel: 0 = its choice

    def _k_splits(self, m: int, n: int, k: int, pending: bool = False) -> int:
        """Into how many parts the tiled kernel cuts K.  17 to 64 rows: more than one with a K so long, and so few
        output tiles of 64 x 64, that the library (which cuts K as well) falls behind.  65 to 256 rows (portions of
        prompts beside decoded tokens): few tiles again, far fewer than compute units, and a whole K for each is
        a long walk (137 rows x 896 columns over a K of 4,864: 32 us in one piece).  Where the parts may be left
        for the norm that follows (`pending`) and K is 2,048 or more, eight parts beat the library as well (the same
        product: 10 us against 10 us; 137 x 1,536 over 8,960: 17 us against 23 us).  Launched eagerly, small
        products do not go to the library at all (its launch costs the host more than they take): those are cut
        whenever K allows, into parts for the next norm or, with a long K, into four that the kernel adds itself
        (14 us)."""
        if not self.use_split_k or n % 4:
            return 1
        tiles = -(-m // 64) * -(-n // 64)
        if self.SKINNY_ROWS < m <= 256:
            if tiles >= 128:
                return 1
            if pending and k >= 2048:
                return min(8, k // 512)
            if self.capturing or m * n * k >= self.EAGER_LIBRARY_WORK:
                return 1                   # the library's
            if pending and k >= 768:
                return min(8, k // 384)
            return 4 if k >= 2048 else 1
        if not (self.FUSED_ROWS < m <= self.SKINNY_ROWS) or k < self.SPLIT_K_FROM:
            return 1
        if tiles >= self.compute_units:
            return 1
        return max(1, min(-(-2 * self.compute_units // tiles), k // 256))

    split_k_kind = "streaming"     # which kernel cuts K for 17 to 64 rows ("tiled": only the tiled one)

    def _streaming_splits(self, m: int, n: int, k: int, pending: bool = False) -> int:
        """Into how many parts the weight-streaming kernel cuts K for 17 to 64 rows and a K of 2,048 up to where
        the tiled kernel takes over: so many that its tiles of sixteen output columns times the parts give every
        compute unit a workgroup, each part at least 512 long.  (Measured with cold weights for the down
        projections of the 0.5B to 7B models: one of the two beats the library at every row count from 17 to 64,
        the streaming kernel while a part is a few steps per wave, the tiled one, which reads the rows a quarter
        as often, for longer K.)  When the parts may be left for the next norm to add (`pending`), the addition
        costs no launch, and a K from 512 on is cut as well, into parts of at least 224 (the output projection of
        a decode batch: every workgroup reads all the rows, and a quarter of K is a quarter of them)."""
        shortest, part = (self.PENDING_SHORTEST_K, 224) if pending else (2048, 512)
        if (not self.use_split_k or not (self.FUSED_ROWS < m <= self.SKINNY_ROWS) or n % 4
                or not (shortest <= k < self.SPLIT_K_FROM)):
            return 1
        tiles = -(-n // 16)
        if tiles >= 128:
            return 1
        if m > 32:
            tiles = -(-n // 32)        # more than 32 rows: a workgroup takes two blocks of sixteen columns
        return max(1, min(-(-self.compute_units // tiles), k // part))

    PENDING_SHORTEST_K = 512   # the shortest K that is cut when the parts may be left for the next norm
    SPLIT_K_FROM = 8192        # the shortest K that the tiled kernel cuts (shorter ones are the weight-streaming kernel's)

    EAGER_LIBRARY_WORK = 2 ** 30   # multiply-adds from which a product launched eagerly goes to the library
    capturing = False          # set while a graph is recorded (and in the run that warms it up): launches are free then
    LIBRARY_WEIGHT = 2 ** 21   # weight elements from which products of 17 to 64 rows go to the library
    GATED_LIBRARY_WEIGHT = 2 ** 24   # ... and the gated product (its activation then is a kernel of its own)
    SKINNY_ROWS = 64    # up to this many rows the weight-streaming kernel runs ...
    WIDE_OUTPUT = 32768  # ... unless there are more than 16 rows and this many output columns (the vocabulary
    #                      projection): there the rows' re-reading per tile of 16 columns costs more than tiling
    use_library_gemm = True

    def linear_silu_gate(self, x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """out = silu(x @ Wg.T) * (x @ Wu.T) for weight = [Wg; Wu] of shape [2I, K]; out [M, I].

        Few bfloat16 rows run in one kernel; otherwise the product and the gated activation are two."""
        _need(weight.dim() == 2 and weight.shape[0] % 2 == 0, "the joined gate and up matrix has an even row count")
        m, inner = x.shape[0], weight.shape[0] // 2
        if out is None:
            out = torch.empty((m, inner), dtype=x.dtype, device=x.device)
        _need(tuple(out.shape) == (m, inner) and out.dtype == x.dtype and out.is_contiguous(), "gated output shape")
        if (x.dtype == torch.bfloat16 and m <= self.SKINNY_ROWS
                and not (self.use_library_gemm and m > self.FUSED_ROWS
                         and weight.shape[0] * weight.shape[1] >= self.GATED_LIBRARY_WEIGHT)):
            _need(x.is_cuda and weight.is_cuda and x.dim() == 2 and x.shape[1] == weight.shape[1], "linear shapes do not fit")
            _need(x.stride(1) == 1 and weight.is_contiguous() and weight.dtype == torch.bfloat16, "linear operands")
            k = x.shape[1]
            lda = x.stride(0) if m > 1 else k
            _need(k % 8 == 0 and lda % 8 == 0, "bfloat16 products need K and the row stride to be multiples of 8")
            _need(x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
            self._check(self.lib.ta_gemm_skinny_bf16(_ptr(x), lda, _ptr(weight), None, _ptr(out), inner, m, 2 * inner,
                                                     k, _BF16, 1, self.skinny_column_blocks, self._stream()),
                        "linear_silu_gate")
            return out
        return self.silu_gate(self.linear(x, weight), out)

    # ------------------------------------------------------- fused decode products
    FUSED_ROWS = 16
    use_fused_decode = True
    fused_rows = 0            # 0: the launcher picks the weight rows per workgroup (1..32; 16, 8, 4 with rotation) ...
    fused_waves = 0           # ... and how many waves share a tile's K (4, 8, 16)

    FUSED_LDS_BYTES = 140 * 1024     # what the norm prologue may take of a compute unit's 160 KB of LDS

    def can_fuse_decode(self, rows: int, dtype: torch.dtype, hidden: int = 0) -> bool:
        """Batches of few bfloat16 rows can run the products that take the norm, the rotation with the
        cache write, the gated activation and the residual add into the same kernel.  The norm prologue
        keeps sixteen normalised rows of `hidden` elements in LDS, which bounds `hidden`."""
        return (self.use_fused_decode and dtype == torch.bfloat16 and 0 < rows <= self.FUSED_ROWS
                and (not self.fold_norm(hidden) or 16 * (hidden + 8) * 2 <= self.FUSED_LDS_BYTES))

    FOLD_NORM_WIDTH = 2048    # up to this model width the decode products normalise their rows themselves

    def fold_norm(self, hidden: int) -> bool:
        """Whether the fused decode products should take the norm into their prologue: every workgroup then reads
        and normalises all rows again, which pays for narrow models (one kernel fewer) and costs more than the
        norm's own small kernel for wide ones."""
        return hidden <= self.FOLD_NORM_WIDTH

    def fused_norm_qkv_rope(self, residual, norm_weight, eps, weight, bias, positions, cos_sin, slots,
                            k_pages, v_pages, n_q: int, n_kv: int, head_dim: int) -> torch.Tensor:
        """q, k, v = rmsnorm(residual) @ weight.T + bias; q and k rotated; k and v stored into their pages
        (when `slots` is given); returns q [M, n_q * d] in bfloat16.  residual float32 [M, K]; or, with
        `norm_weight` None, `residual` holds the normalised rows in bfloat16 already."""
        _dev(norm_weight, weight, bias, positions, cos_sin, slots, k_pages, v_pages)
        _need(residual.is_cuda and residual.dim() == 2, "the rows must live on the GPU")
        m, k = residual.shape
        if norm_weight is None:
            _need(residual.dtype == torch.bfloat16 and residual.stride(1) == 1 and residual.stride(0) % 8 == 0
                  and residual.data_ptr() % 16 == 0, "normalised rows are bfloat16 with 16-byte aligned rows")
        else:
            _need(residual.dtype == torch.float32 and residual.is_contiguous() and norm_weight.dtype == torch.float32
                  and norm_weight.numel() == k, "the residual and the norm weight are float32")
        _need(weight.dtype == torch.bfloat16 and tuple(weight.shape) == ((n_q + 2 * n_kv) * head_dim, k),
              "the joined q/k/v matrix has the wrong shape")
        _need(k % 8 == 0 and head_dim % 32 == 0
              and (m <= self.FUSED_ROWS or (norm_weight is None and m <= self.SKINNY_ROWS)),
              "sizes the fused projection does not take")
        _need(positions.dtype == torch.int32 and positions.numel() == m, "positions must be int32 [M]")
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() == weight.shape[0], "bias must be float32")
        if cos_sin is not None:
            _need(cos_sin.dtype == torch.float32 and cos_sin.shape[1] == head_dim, "cos_sin must be float32 [P, d]")
        page_size = 1
        if slots is not None:
            _need(slots.dtype == torch.int32 and slots.numel() == m, "slots must be int32 [M]")
            _need(k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16, "pages must be bfloat16")
            page_size = self._page_size(k_pages, v_pages, n_kv, head_dim)
        q = torch.empty((m, n_q * head_dim), dtype=torch.bfloat16, device=residual.device)
        tail = (_ptr(weight), _ptr(bias), _ptr(q), _ptr(positions), _ptr(cos_sin), _ptr(slots),
                _ptr(k_pages if slots is not None else None), _ptr(v_pages if slots is not None else None),
                m, k, n_q, n_kv, head_dim, page_size, self.fused_rows, self.fused_waves, self._stream())
        if m > self.FUSED_ROWS:
            # 17 to 64 rows: the weight-streaming kernel with the same epilogue.
            status = self.lib.ta_gemm_skinny_qkv_rope(_ptr(residual), residual.stride(0), *tail[:-3], self._stream())
        elif norm_weight is None:
            status = self.lib.ta_fused_qkv_rope(_ptr(residual), residual.stride(0) if m > 1 else k, *tail)
        else:
            status = self.lib.ta_fused_norm_qkv_rope(_ptr(residual), _ptr(norm_weight), ctypes.c_float(eps), *tail)
        self._check(status, "fused_norm_qkv_rope")
        return q

    ROPE_STORE_WEIGHT = 2 ** 22   # joined q/k/v matrices up to this many elements take the route below at 17-64 rows

    def can_rope_store(self, rows: int, dtype: torch.dtype, weight_elements: int = 0) -> bool:
        """Whether `fused_norm_qkv_rope` should take this many normalised bfloat16 rows: 17 to 64 go through the
        weight-streaming kernel, which then needs no rotation kernel after it.  That pays while the matrix is
        small (measured: 0.5B and 1.5B sizes); a big one is better off with the library's product and the
        rotation kernel."""
        return (self.use_fused_decode and dtype == torch.bfloat16 and self.FUSED_ROWS < rows <= self.SKINNY_ROWS
                and weight_elements <= self.ROPE_STORE_WEIGHT)

    def fused_norm_gated(self, residual, norm_weight, eps, weight) -> torch.Tensor:
        """silu(x @ Wg.T) * (x @ Wu.T) with x = rmsnorm(residual), weight = [Wg; Wu]; bfloat16 [M, I].  With
        `norm_weight` None, `residual` holds the normalised rows in bfloat16 already."""
        _dev(norm_weight, weight)
        _need(residual.is_cuda and residual.dim() == 2, "the rows must live on the GPU")
        m, k = residual.shape
        if norm_weight is None:
            _need(residual.dtype == torch.bfloat16 and residual.stride(1) == 1 and residual.stride(0) % 8 == 0
                  and residual.data_ptr() % 16 == 0, "normalised rows are bfloat16 with 16-byte aligned rows")
        else:
            _need(residual.dtype == torch.float32 and residual.is_contiguous() and norm_weight.dtype == torch.float32
                  and norm_weight.numel() == k, "the residual and the norm weight are float32")
        _need(weight.dtype == torch.bfloat16 and weight.shape[1] == k and weight.shape[0] % 2 == 0, "gate/up matrix shape")
        _need(m <= self.FUSED_ROWS and k % 8 == 0, "sizes the fused product does not take")
        out = torch.empty((m, weight.shape[0] // 2), dtype=torch.bfloat16, device=residual.device)
        tail = (_ptr(weight), _ptr(out), m, weight.shape[0], k, self.fused_rows, self.fused_waves, self._stream())
        if norm_weight is None:
            status = self.lib.ta_fused_gated(_ptr(residual), residual.stride(0) if m > 1 else k, *tail)
        else:
            status = self.lib.ta_fused_norm_gated(_ptr(residual), _ptr(norm_weight), ctypes.c_float(eps), *tail)
        self._check(status, "fused_norm_gated")
        return out

    def linear_add(self, x, weight, bias, residual) -> None:
        """residual += x @ weight.T (+ bias), in place, in float32.  x bfloat16 [M, K], M <= 16."""
        _dev(weight, bias, residual)
        _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and x.dtype == torch.bfloat16, "x must be bfloat16 rows")
        m, k = x.shape
        n = weight.shape[0]
        lda = x.stride(0) if m > 1 else k
        _need(weight.dtype == torch.bfloat16 and weight.shape[1] == k, "weight shape")
        _need(residual.dtype == torch.float32 and tuple(residual.shape) == (m, n), "the residual must be float32 [M, N]")
        _need(m <= self.FUSED_ROWS and k % 8 == 0 and lda % 8 == 0 and x.data_ptr() % 16 == 0, "sizes not taken")
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() == n, "bias must be float32 [N]")
        self._check(self.lib.ta_fused_linear_residual(_ptr(x), lda, _ptr(weight), _ptr(bias), _ptr(residual), m, n, k,
                                                      self.fused_rows, self.fused_waves, self._stream()), "linear_add")

    # ------------------------------------------------------------------- sampling
    def argmax(self, logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """First maximum of each row.  logits float32 [B, V] -> int32 [B]."""
        _dev(logits, out)
        _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be float32 [B, V]")
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        _need(out.dtype == torch.int32 and out.numel() == logits.shape[0], "argmax output must be int32 [B]")
        n_rows, vocab = logits.shape
        chunks = max(1, min(256, vocab // 2048, 2048 // max(1, n_rows)))
        partial_v = torch.empty((n_rows, chunks), dtype=torch.float32, device=logits.device)
        partial_i = torch.empty((n_rows, chunks), dtype=torch.int32, device=logits.device)
        self._check(self.lib.ta_argmax(_ptr(logits), _ptr(out), _ptr(partial_v), _ptr(partial_i), n_rows, vocab,
                                       chunks, self._stream()), "argmax")
        return out

    NEXT_STEP_GROUPS = 4          # cache groups `argmax_next_step` can advance

    def argmax_next_step(self, logits: torch.Tensor, token_ids: torch.Tensor, positions: torch.Tensor,
                         first_position: torch.Tensor, slots: list[torch.Tensor], block_tables: list[torch.Tensor],
                         page_size: int) -> torch.Tensor:
        """`argmax` for a decode step of one token per request (row i of the logits = request i), which also turns
        the step's description into the next step's, in place: the picked ids become `token_ids`, `positions` and
        `first_position` go up by one, and every cache group's `slots` are looked up for the new positions in its
        block table [B, width] (a position past the table's width takes the last entry; a page that is not there
        gives slot -1).  All int32 [B]."""
        _dev(logits, token_ids, positions, first_position, *slots, *block_tables)
        _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be float32 [B, V]")
        n_rows, vocab = logits.shape
        _need(len(slots) == len(block_tables) <= self.NEXT_STEP_GROUPS, "one table per group of slots, four at most")
        for t in (token_ids, positions, first_position, *slots):
            _need(t.dtype == torch.int32 and t.numel() == n_rows and t.is_contiguous(), "the description is int32 [B]")
        for table in block_tables:
            _need(table.dtype == torch.int32 and table.dim() == 2 and table.shape[0] == n_rows and table.shape[1] >= 1
                  and table.is_contiguous(), "block tables are int32 [B, width]")
        _need(page_size >= 1, "page size")
        out = torch.empty(n_rows, dtype=torch.int32, device=logits.device)
        chunks = max(1, min(256, vocab // 2048, 2048 // max(1, n_rows)))
        partial_v = torch.empty((n_rows, chunks), dtype=torch.float32, device=logits.device)
        partial_i = torch.empty((n_rows, chunks), dtype=torch.int32, device=logits.device)
        groups = []
        for g in range(self.NEXT_STEP_GROUPS):
            if g < len(slots):
                groups += [_ptr(slots[g]), _ptr(block_tables[g]), int(block_tables[g].shape[1])]
            else:
                groups += [_ptr(None), _ptr(None), 0]
        self._check(self.lib.ta_argmax_next_step(_ptr(logits), _ptr(out), _ptr(partial_v), _ptr(partial_i), n_rows, vocab,
                                                 chunks, _ptr(token_ids), _ptr(positions), _ptr(first_position),
                                                 int(page_size), len(slots), *groups, self._stream()), "argmax_next_step")
        return out

    def sample(self, logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, uniform: torch.Tensor,
               out: torch.Tensor | None = None, any_cut: bool = True) -> torch.Tensor:
        """Temperature / nucleus draw per row with the reference's rules (tokens by falling logit, lower
        index first among equals; the shortest prefix reaching top_p; the uniform number walks its mass).
        logits float32 [B, V]; temperature (> 0), top_p, uniform: float32 [B]; returns int32 [B].
        `any_cut=False` promises that no row has top_p < 1: the rounds that look for the nucleus's end are
        then not launched."""
        _dev(logits, temperature, top_p, uniform, out)
        _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be float32 [B, V]")
        n_rows = logits.shape[0]
        for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
            _need(t.dtype == torch.float32 and t.numel() == n_rows, f"{name} must be float32 [B]")
        if out is None:
            out = torch.empty(n_rows, dtype=torch.int32, device=logits.device)
        _need(out.dtype == torch.int32 and out.numel() == n_rows, "sample output must be int32 [B]")
        workspace = torch.empty(max(1, n_rows) * self.lib.ta_sample_workspace_words(), dtype=torch.float32,
                                device=logits.device)
        self._check(self.lib.ta_sample(_ptr(logits), _ptr(temperature), _ptr(top_p), _ptr(uniform), _ptr(out),
                                       _ptr(workspace), n_rows, logits.shape[1], 1 if any_cut else 0, self._stream()),
                    "sample")
        return out


_OPS: Ops | None = None
_LOCK = threading.Lock()


def get_ops() -> Ops:
    """The loaded kernel library; builds it on first use if no built library is found."""
    global _OPS
    if _OPS is not None:
        return _OPS
    with _LOCK:
        if _OPS is None:
            if not torch.cuda.is_available():
                raise KernelError("tokenizer_amd runs on an AMD GPU through its HIP kernels; "
                                  "no GPU is visible and there is no CPU path")
            path = _build.find_library()
            if path is None:
                path = _build.build_library()
            _OPS = Ops(path)
    return _OPS


def default_scale(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)
