"""Each HIP kernel alone against its plain torch reference, at sizes other than the engine's."""
import math

import pytest
import torch

from tokenizer_amd.kernels import KernelError, PendingSum

from kernel_refs import PlainOps

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from tokenizer_amd.kernels import get_ops
    return get_ops()


@pytest.fixture(scope="module")
def ref():
    return PlainOps(torch.float64)


def tol(dtype):
    # float32: rounding of sums of a few hundred terms; bfloat16: one rounding of the output (2^-9 relative).
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=8e-3, atol=1e-3)


def rand(shape, dtype, seed, scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=gen) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(ops, ref, dtype):
    table = rand((1000, 200), dtype, 1)
    ids = torch.tensor([0, 999, 5, 5, 17, 400, 123] * 5 + [1, 2], dtype=torch.int32).cuda()
    out = torch.empty((ids.numel(), 200), dtype=torch.float32).cuda()
    ops.embedding(ids, table, out)
    want = torch.empty_like(out)
    ref.embedding(ids, table, want)
    assert torch.equal(out, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [200, 896, 72, 2048, 3000, 4096, 4100])
@pytest.mark.parametrize("n", [33, 301])
def test_add_rmsnorm(ops, ref, dtype, hidden, n):
    # (few and many rows; rows that fit the registers of a workgroup and rows that do not)
    residual = rand((n, hidden), torch.float32, 2, 3.0)
    delta = rand((n, hidden), dtype, 3)
    weight = rand((hidden,), torch.float32, 4) + 1
    for use_delta in (True, False):
        res_a, res_b = residual.clone(), residual.clone()
        out_a = torch.empty((n, hidden), dtype=dtype).cuda()
        out_b = torch.empty_like(out_a)
        ops.add_rmsnorm(res_a, delta if use_delta else None, weight, 1e-5, out_a)
        ref.add_rmsnorm(res_b, delta if use_delta else None, weight, 1e-5, out_b)
        torch.testing.assert_close(res_a, res_b, rtol=1e-6, atol=1e-6)
        torch.testing.assert_close(out_a.float(), out_b.float(), **tol(dtype))
    picked = [n - 1, 0, 7, 7] if n < 256 else [n - 1, 0, 7, 7] + list(range(2, 2 + 256))
    rows = torch.tensor(picked, dtype=torch.int32).cuda()
    res_a = residual.clone()
    out_a = torch.empty((len(picked), hidden), dtype=dtype).cuda()
    out_b = torch.empty_like(out_a)
    ops.add_rmsnorm(res_a, delta, weight, 1e-6, out_a, rows, store_residual=False)
    ref.add_rmsnorm(residual.clone(), delta, weight, 1e-6, out_b, rows, store_residual=False)
    assert torch.equal(res_a, residual), "a row subset must leave the residual alone"
    torch.testing.assert_close(out_a.float(), out_b.float(), **tol(dtype))


def test_rmsnorm_eps_matters(ops):
    # Tiny inputs: the result is x / sqrt(eps) when mean(x^2) << eps, so a misplaced eps shows.
    x = torch.full((1, 64), 1e-6).cuda()
    w = torch.ones(64).cuda()
    out = torch.empty((1, 64)).cuda()
    ops.add_rmsnorm(x, None, w, 1e-4, out)
    torch.testing.assert_close(out, torch.full((1, 64), 1e-6 / math.sqrt(1e-12 + 1e-4)).cuda(), rtol=1e-5, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_gate(ops, ref, dtype):
    x = rand((19, 2 * 272), dtype, 5, 2.0)
    out_a = torch.empty((19, 272), dtype=dtype).cuda()
    out_b = torch.empty_like(out_a)
    ops.silu_gate(x, out_a)
    ref.silu_gate(x, out_b)
    torch.testing.assert_close(out_a.float(), out_b.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geometry", [(6, 2, 48, 16), (3, 1, 32, 16), (4, 4, 128, 32)])
def test_rope_store(ops, ref, dtype, geometry):
    n_q, n_kv, d, page_size = geometry
    n_tokens, n_pages, max_pos = 21, 9, 400
    width = (n_q + 2 * n_kv) * d
    qkv = rand((n_tokens, width), dtype, 6)
    bias = rand((width,), torch.float32, 7)
    positions = torch.randint(0, max_pos, (n_tokens,), generator=torch.Generator().manual_seed(8)).int().cuda()
    inv = torch.tensor([1.0 / (10000.0 ** (i / d)) for i in range(0, d, 2)], dtype=torch.float64).float()
    ang = torch.arange(max_pos).float()[:, None] * inv[None]
    cos_sin = torch.cat([ang.cos(), ang.sin()], 1).cuda()
    perm = torch.randperm(n_pages * page_size, generator=torch.Generator().manual_seed(9))[:n_tokens]
    slots = perm.int().cuda()
    slots[3] = -1
    for use_bias, use_rot in ((True, True), (False, True), (True, False), (False, False)):
        a, b = qkv.clone(), qkv.clone()
        ka = torch.zeros((n_pages, n_kv, page_size, d), dtype=dtype).cuda()
        kb = ka.clone()
        va = torch.zeros((n_pages, n_kv, d, page_size), dtype=dtype).cuda()
        vb = va.clone()
        args = (bias if use_bias else None, positions, cos_sin if use_rot else None, slots)
        ops.rope_store(a, *args, ka, va, n_q, n_kv, d)
        ref.rope_store(b, *args, kb, vb, n_q, n_kv, d)
        torch.testing.assert_close(a.float(), b.float(), **tol(dtype))
        torch.testing.assert_close(ka.float(), kb.float(), **tol(dtype))
        torch.testing.assert_close(va.float(), vb.float(), **tol(dtype))
    # Without slots nothing is stored.
    a = qkv.clone()
    ops.rope_store(a, None, positions, cos_sin, None, None, None, n_q, n_kv, d)
    b = qkv.clone()
    ref.rope_store(b, None, positions, cos_sin, None, None, None, n_q, n_kv, d)
    torch.testing.assert_close(a.float(), b.float(), **tol(dtype))


def make_paged_case(dtype, n_q, n_kv, d, page_size, lengths, q_lens, seed):
    """Requests of the given lengths whose last q_lens tokens are queried; pages scattered at random."""
    gen = torch.Generator().manual_seed(seed)
    n_entries = len(lengths)
    pages_each = [-(-n // page_size) for n in lengths]
    n_pages = sum(pages_each) + 3
    order = torch.randperm(n_pages, generator=gen).tolist()
    width = max(pages_each)
    table = torch.full((n_entries, width), -1, dtype=torch.int32)
    k_pages = torch.randn((n_pages, n_kv, page_size, d), generator=gen).to(dtype)
    v_pages = torch.randn((n_pages, n_kv, d, page_size), generator=gen).to(dtype)
    positions, entry_of_token = [], []
    used = torch.zeros(n_pages, page_size, dtype=torch.bool)
    for e, (length, q_len) in enumerate(zip(lengths, q_lens)):
        for i in range(pages_each[e]):
            table[e, i] = order.pop()
            used[table[e, i], :max(0, min(page_size, length - i * page_size))] = True
        positions += list(range(length - q_len, length))
        entry_of_token += [e] * q_len
    # Slots no request wrote hold NaN: a kernel that lets them into a sum shows it.
    k_pages[~used[:, None, :, None].expand_as(k_pages)] = float("nan")
    v_pages[~used[:, None, None, :].expand_as(v_pages)] = float("nan")
    n_tokens = len(positions)
    qkv = torch.randn((n_tokens, (n_q + 2 * n_kv) * d), generator=gen).to(dtype)
    return (qkv.cuda(), k_pages.cuda(), v_pages.cuda(), torch.tensor(positions, dtype=torch.int32).cuda(),
            torch.tensor(entry_of_token, dtype=torch.int32).cuda(), table.cuda())


def make_batch(lengths, q_lens):
    """What the engine's step context tells the attention kernels about a batch."""
    import types
    cu_q, first, tiles, rows = [0], [], [], []
    for e, (length, q_len) in enumerate(zip(lengths, q_lens)):
        first.append(length - q_len)
        if q_len == 1:
            rows.append(cu_q[-1])
        else:
            for offset in range(0, q_len, 16):
                tiles += [e, offset]
        cu_q.append(cu_q[-1] + q_len)
    as_int = lambda values: torch.tensor(values, dtype=torch.int32).cuda()
    return types.SimpleNamespace(n_tokens=cu_q[-1], cu_q=as_int(cu_q), first_position=as_int(first),
                                 q_tiles=as_int(tiles).reshape(-1, 2), decode_rows=as_int(rows),
                                 max_position=max(lengths) - 1)


def dense_attention(qkv, k_pages, v_pages, table, lengths, q_lens, n_q, n_kv, d, window, scale):
    """Attention of each request's last q_len tokens over its keys as one masked matrix product per request
    (float32): what the per-token reference computes, fast enough for thousands of tokens."""
    page_size, group = k_pages.shape[2], n_q // n_kv
    out, row = [], 0
    for e, (length, q_len) in enumerate(zip(lengths, q_lens)):
        pages = table[e, :-(-length // page_size)].long()
        k = k_pages[pages].float().permute(1, 0, 2, 3).reshape(n_kv, -1, d)[:, :length]          # [n_kv, L, d]
        v = v_pages[pages].float().permute(1, 0, 3, 2).reshape(n_kv, -1, d)[:, :length]
        q = qkv[row:row + q_len, :n_q * d].float().reshape(q_len, n_kv, group, d).permute(1, 2, 0, 3)   # [n_kv, g, T, d]
        scores = torch.einsum("kgtd,kld->kgtl", q, k) * scale
        pos = torch.arange(length - q_len, length, device=qkv.device)[:, None]
        key = torch.arange(length, device=qkv.device)[None, :]
        seen = key <= pos
        if window is not None:
            seen &= key >= pos - window
        probs = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
        out.append(torch.einsum("kgtl,kld->tkgd", probs, v).reshape(q_len, n_q * d))
        row += q_len
    return torch.cat(out)


# (dtype, fast): the generic kernel in both dtypes, the matrix-core kernels in bfloat16.
ATTENTION_MODES = [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)]


@pytest.fixture()
def attention_mode(ops, request):
    dtype, fast = request.param
    before = ops.use_fast_attention
    ops.use_fast_attention = fast
    yield dtype
    ops.use_fast_attention = before


def attention_tol(dtype, fast):
    # The matrix-core kernels round the probabilities to bfloat16 before the product with the values.
    return dict(rtol=2e-2, atol=8e-3) if fast else tol(dtype)


@pytest.mark.parametrize("attention_mode", ATTENTION_MODES, indirect=True)
@pytest.mark.parametrize("geometry", [(6, 3, 48, 16), (3, 1, 32, 16), (8, 2, 128, 32), (14, 2, 64, 16),
                                      (20, 1, 16, 16), (4, 4, 80, 48), (2, 1, 256, 16)])
@pytest.mark.parametrize("window", [None, 37])
def test_paged_attention(ops, ref, attention_mode, geometry, window):
    dtype = attention_mode
    n_q, n_kv, d, page_size = geometry
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        dtype, n_q, n_kv, d, page_size, lengths=[1, 300, 64, 17], q_lens=[1, 5, 64, 1], seed=11)
    out_a = torch.empty((qkv.shape[0], n_q * d), dtype=dtype).cuda()
    out_b = torch.empty_like(out_a)
    scale = 1.0 / math.sqrt(d)
    ops.paged_attention(qkv, out_a, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=int(positions.max()))
    ref.paged_attention(qkv, out_b, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale)
    torch.testing.assert_close(out_a.float(), out_b.float(), **attention_tol(dtype, ops.use_fast_attention))
    if ops.use_fast_attention:
        # With the batch described, prompt portions take the tiled kernel and single tokens the split one.
        out_c = torch.full_like(out_a, float("nan"))
        ops.paged_attention(qkv, out_c, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window,
                            scale, max_position=int(positions.max()), batch=make_batch([1, 300, 64, 17], [1, 5, 64, 1]))
        torch.testing.assert_close(out_c.float(), out_b.float(), **attention_tol(dtype, True))


@pytest.mark.parametrize("geometry,waves", [((14, 2, 64, 16), 0), ((14, 2, 64, 16), 1), ((14, 2, 64, 16), 4),
                                            ((14, 2, 64, 16), 8), ((6, 3, 48, 32), 8),
                                            ((12, 2, 128, 16), 0), ((3, 1, 32, 32), 2), ((5, 5, 16, 16), 4)])
@pytest.mark.parametrize("window", [None, 100])
def test_prefill_attention_on_long_and_ragged_portions(ops, ref, geometry, window, waves, monkeypatch):
    # Portions that start in the middle of a page, end in the middle of a tile, and a long whole prompt;
    # with one wave per tile and with several that share its keys (some of them without a key of their own).
    monkeypatch.setattr(ops, "prefill_waves", waves)
    n_q, n_kv, d, page_size = geometry
    lengths, q_lens = [700, 333, 40, 16, 1000], [700, 50, 33, 16, 2]
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        torch.bfloat16, n_q, n_kv, d, page_size, lengths=lengths, q_lens=q_lens, seed=17)
    out_a = torch.full((qkv.shape[0], n_q * d), float("nan"), dtype=torch.bfloat16).cuda()
    out_b = torch.empty_like(out_a)
    scale = 1.0 / math.sqrt(d)
    ops.paged_attention(qkv, out_a, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=max(lengths) - 1, batch=make_batch(lengths, q_lens))
    ref.paged_attention(qkv, out_b, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale)
    torch.testing.assert_close(out_a.float(), out_b.float(), **attention_tol(torch.bfloat16, True))


@pytest.mark.parametrize("geometry,shape,window", [
    ((28, 4, 128, 16), 0, None), ((12, 2, 128, 32), 0, None), ((28, 4, 128, 16), 2, None), ((12, 2, 128, 16), 12, None),
    ((14, 2, 64, 16), 11, None), ((6, 2, 64, 48), 1, None), ((28, 4, 128, 16), 0, 4150), ((14, 2, 64, 16), 11, 4150),
    ((12, 2, 128, 32), 0, 600), ((6, 2, 64, 48), 1, 600)])
def test_few_tiles_behind_a_long_context_cut_their_keys_over_workgroups(ops, ref, geometry, shape, window, monkeypatch):
    """A portion of 70 tokens behind 4,150 cached ones and a second request's 20 behind 320: fewer workgroups than
    compute units, thousands of keys each.  The workgroup-shared kernel then cuts every tile's keys over several
    workgroups (whole turns each; the short request's later parts are empty) and a second kernel merges their
    states.  Every shape of the kernel, a window that reaches nearly as far and one that does not (no cut then);
    unwritten slots hold NaN."""
    n_q, n_kv, d, page_size = geometry
    lengths, q_lens = [4220, 340], [70, 20]
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        torch.bfloat16, n_q, n_kv, d, page_size, lengths=lengths, q_lens=q_lens, seed=29)
    if shape:
        monkeypatch.setattr(ops, "prefill_shared", 1)
        monkeypatch.setattr(ops, "prefill_shape", shape)
    tiles = sum(-(-n // 16) for n in q_lens)
    parts = ops.lib.ta_prefill_attention_key_splits(tiles, n_q, n_kv, d, -1 if window is None else window,
                                                    ops.prefill_shape, max(lengths), ops.prefill_waves, ops.prefill_shared)
    assert (parts > 1) == (window != 600), parts
    out_a = torch.full((qkv.shape[0], n_q * d), float("nan"), dtype=torch.bfloat16).cuda()
    out_b = torch.empty_like(out_a)
    scale = 1.0 / math.sqrt(d)
    ops.paged_attention(qkv, out_a, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=max(lengths) - 1, batch=make_batch(lengths, q_lens))
    ref.paged_attention(qkv, out_b, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale)
    torch.testing.assert_close(out_a.float(), out_b.float(), **attention_tol(torch.bfloat16, True))
    # The same launch with the keys in one piece: the same attention, up to the order of the sums.
    monkeypatch.setattr(ops, "prefill_key_splits", False)
    out_c = torch.full_like(out_a, float("nan"))
    ops.paged_attention(qkv, out_c, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=max(lengths) - 1, batch=make_batch(lengths, q_lens))
    torch.testing.assert_close(out_c.float(), out_b.float(), **attention_tol(torch.bfloat16, True))


@pytest.mark.parametrize("window", [None, 600])
def test_a_short_portion_behind_a_long_context_takes_eight_waves_a_tile(ops, ref, window, monkeypatch):
    """A portion of 70 tokens behind 4,150 cached ones (and a second request's 20 behind 320): few tiles with a
    long walk each, for which the per-wave kernel's launcher gives a tile eight waves at head size 64 (with a window
    of 600 nobody looks that far back and it stays at fewer).  Keys the waves share out unevenly, waves without a key of their
    own at the short request, unwritten slots holding NaN."""
    n_q, n_kv, d, page_size = 14, 2, 64, 16
    lengths, q_lens = [4220, 340], [70, 20]
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        torch.bfloat16, n_q, n_kv, d, page_size, lengths=lengths, q_lens=q_lens, seed=23)
    assert ops.prefill_waves == 0
    monkeypatch.setattr(ops, "prefill_shared", -1)        # the per-wave kernel (where it has the launch to itself)
    out_a = torch.full((qkv.shape[0], n_q * d), float("nan"), dtype=torch.bfloat16).cuda()
    out_b = torch.empty_like(out_a)
    scale = 1.0 / math.sqrt(d)
    ops.paged_attention(qkv, out_a, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=max(lengths) - 1, batch=make_batch(lengths, q_lens))
    ref.paged_attention(qkv, out_b, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale)
    torch.testing.assert_close(out_a.float(), out_b.float(), **attention_tol(torch.bfloat16, True))


@pytest.mark.parametrize("geometry,lengths,q_lens,shape", [((14, 2, 64, 16), [4500, 333], [4400, 50], 11),
                                                           ((28, 2, 64, 16), [2300, 40], [2200, 33], 11),
                                                           ((28, 4, 128, 16), [2300, 40], [2200, 33], 12),
                                                           ((28, 4, 128, 16), [4300, 40], [4200, 33], 2),
                                                           ((14, 2, 64, 16), [1100, 40], [1000, 33], 11),
                                                           ((16, 4, 128, 16), [2300, 40], [2200, 33], 11)])
@pytest.mark.parametrize("window", [None, 1000])
def test_the_launcher_takes_the_workgroup_shared_kernel_for_many_tiles(ops, ref, geometry, lengths, q_lens, shape, window):
    # Seven (or twice seven) query heads per kv head and dozens to hundreds of tiles: the launcher's own choice is
    # the kernel whose waves share their blocks of keys, with one head a wave or two and one or two key groups by
    # the number of workgroups (shape = heads a wave + 10 for two key groups).  Portions that start and end inside
    # pages and tiles, beside a short one, with and without a window.
    n_q, n_kv, d, page_size = geometry
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        torch.bfloat16, n_q, n_kv, d, page_size, lengths=lengths, q_lens=q_lens, seed=23)
    batch = make_batch(lengths, q_lens)
    assert ops.prefill_shared == 0 and ops.prefill_waves == 0 and ops.prefill_shape == 0
    plan = ops.lib.ta_prefill_attention_shared_plan
    reach = -(-max(lengths) // 512) * 512 if window is None else window + 16
    assert plan(batch.q_tiles.shape[0], n_q, n_kv, d, reach) == shape
    scale = 1.0 / math.sqrt(d)
    out_a = torch.full((qkv.shape[0], n_q * d), float("nan"), dtype=torch.bfloat16).cuda()
    ops.paged_attention(qkv, out_a, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=max(lengths) - 1, batch=batch)
    out_b = dense_attention(qkv, k_pages, v_pages, table, lengths, q_lens, n_q, n_kv, d, window, scale)
    torch.testing.assert_close(out_a.float(), out_b, **attention_tol(torch.bfloat16, True))
    # The plain per-token reference on a few rows pins the dense one used above.
    rows = torch.tensor([0, 17, q_lens[0] - 1, q_lens[0], qkv.shape[0] - 1]).cuda()
    out_c = torch.empty((len(rows), n_q * d), dtype=torch.bfloat16).cuda()
    ref.paged_attention(qkv[rows], out_c, k_pages, v_pages, positions[rows], entry_of_token[rows], table, n_q, n_kv, d,
                        window, scale)
    torch.testing.assert_close(out_c.float(), out_b[rows], **tol(torch.bfloat16))


@pytest.mark.parametrize("seed", range(8))
def test_shared_block_prompt_attention_on_random_batches(ops, seed, monkeypatch):
    # Random head counts, page sizes, windows and batches of portions (whole prompts, portions after cached tokens,
    # two-token portions, single tokens beside them), unwritten slots holding NaN: the kernel whose waves share
    # their blocks, in all its four shapes, against one masked matrix product per request.
    import random
    rng = random.Random(seed)
    d = rng.choice([64, 128])
    n_kv = rng.choice([1, 2, 3])
    n_q = n_kv * rng.choice([3, 4, 5, 6, 7, 8, 12])
    page_size = rng.choice([16, 32, 48, 64])
    window = rng.choice([None, None, rng.randint(1, 40), rng.randint(41, 900)])
    lengths, q_lens = [], []
    for _ in range(rng.randint(1, 5)):
        length = rng.choice([rng.randint(2, 70), rng.randint(71, 1500)])
        lengths.append(length)
        q_lens.append(rng.choice([length, rng.randint(1, length), min(length, 2), 1]))
    if all(q == 1 for q in q_lens):
        q_lens[0] = min(lengths[0], 17)
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        torch.bfloat16, n_q, n_kv, d, page_size, lengths=lengths, q_lens=q_lens, seed=100 + seed)
    scale = 1.0 / math.sqrt(d)
    want = dense_attention(qkv, k_pages, v_pages, table, lengths, q_lens, n_q, n_kv, d, window, scale)
    monkeypatch.setattr(ops, "prefill_shared", 1)
    for heads in (1, 2, 11, 12):
        monkeypatch.setattr(ops, "prefill_shape", heads)
        out = torch.full((qkv.shape[0], n_q * d), float("nan"), dtype=torch.bfloat16).cuda()
        ops.paged_attention(qkv, out, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                            max_position=max(lengths) - 1, batch=make_batch(lengths, q_lens))
        torch.testing.assert_close(out.float(), want, **attention_tol(torch.bfloat16, True),
                                   msg=lambda m: f"{m}\n{(n_q, n_kv, d, page_size, window, lengths, q_lens, heads)}")


def test_where_the_workgroup_shared_kernel_is_planned(ops):
    plan = ops.lib.ta_prefill_attention_shared_plan
    # (tiles, query heads, kv heads, head size, reach) -> heads a wave + 10 for two key groups, 0 = the per-wave kernel
    assert plan(32, 14, 2, 64, 512) == 0 and plan(64, 14, 2, 64, 1024) == 11       # 512 and 1,024 tokens at 0.5B sizes
    assert plan(128, 14, 2, 64, 2048) == 11 and plan(256, 14, 2, 64, 4096) == 11 and plan(512, 14, 2, 64, 8192) == 2
    assert plan(32, 28, 4, 128, 512) == 11 and plan(64, 28, 4, 128, 1024) == 11 and plan(64, 28, 4, 128, 8192) == 12
    assert plan(128, 28, 4, 128, 2048) == 12 and plan(256, 28, 4, 128, 4096) == 2
    assert plan(31, 28, 4, 128, 512) == 0 and plan(31, 28, 4, 128, 1024) == 11      # few tiles: only behind some context ...
    assert plan(1, 12, 2, 128, 4096) == 11 and plan(8, 32, 8, 128, 8192) == 11 and plan(31, 14, 2, 64, 2560) == 0   # ... at head size 128,
    assert plan(31, 14, 2, 64, 3072) == 11 and plan(2, 16, 4, 64, 8192) == 11           # behind 3,072 keys and more at head size 64
    # behind 6,144 keys and more two heads a wave read each block half as often; the shortest portions stay at one
    assert plan(16, 28, 4, 128, 8704) == 12 and plan(4, 28, 4, 128, 8704) == 11 and plan(16, 28, 4, 128, 5632) == 11
    assert plan(32, 28, 4, 128, 8704) == 12 and plan(64, 12, 2, 128, 9216) == 12 and plan(64, 14, 2, 64, 9216) == 12
    assert plan(128, 14, 2, 64, 10240) == 11 and plan(32, 14, 2, 64, 8704) == 12 and plan(8, 14, 2, 64, 8704) == 11
    splits = ops.lib.ta_prefill_attention_shared_key_splits
    # (tiles, query heads, kv heads, reach, shape) -> parts of a tile's keys: fewer workgroups than compute units and a long reach
    assert splits(8, 28, 4, 8704, 11) == 4 and splits(1, 28, 4, 8704, 11) == 8 and splits(32, 12, 2, 8704, 11) == 2
    assert splits(32, 28, 4, 8704, 11) == 1 and splits(8, 28, 4, 3584, 11) == 3 and splits(8, 28, 4, 4096, 11) == 4
    assert splits(8, 28, 4, 2048, 11) == 2 and splits(8, 28, 4, 1536, 11) == 1 and splits(1, 28, 4, 2048, 1) == 4
    assert splits(2, 28, 4, 30720, 2) == 16 and splits(8, 28, 4, 8704, 0) == 1
    assert plan(128, 12, 2, 128, 2048) == 11 and plan(128, 12, 2, 128, 10240) == 12
    assert plan(128, 32, 8, 128, 2048) == 1 and plan(64, 32, 8, 128, 1024) == 11 and plan(31, 32, 8, 128, 512) == 0   # four heads per kv head: one a wave
    assert plan(128, 16, 4, 64, 2048) == 11 and plan(512, 16, 4, 64, 8192) == 1 and plan(512, 24, 8, 128, 8192) == 1
    assert plan(4096, 16, 8, 128, 8192) == 0        # two heads per kv head
    assert plan(4096, 28, 4, 96, 8192) == 0         # no instance


@pytest.mark.parametrize("geometry", [(28, 4, 128, 16), (12, 2, 128, 32), (5, 1, 64, 48), (16, 2, 128, 16),
                                      (24, 2, 128, 64), (3, 1, 128, 16), (14, 2, 64, 16), (8, 2, 64, 32)])
@pytest.mark.parametrize("window", [None, 100])
@pytest.mark.parametrize("heads", [1, 2, 11, 12])
def test_prefill_attention_with_a_block_of_keys_shared_by_a_workgroup(ops, ref, geometry, window, heads, monkeypatch):
    # The kernel whose four waves take one block of keys from LDS for up to eight query heads of a kv head: five,
    # six, seven and eight heads (a wave with one head, a wave without any), twelve (two workgroups a tile) and
    # three; portions that start in the middle of a page, end in the middle of a tile, lie under a window whose
    # first pages hold nothing any more, and unwritten slots that hold NaN.  With two heads a wave and with one,
    # with one group of waves and with two that take the blocks in turn (shape = heads a wave + 10 for two groups).
    monkeypatch.setattr(ops, "prefill_shared", 1)
    monkeypatch.setattr(ops, "prefill_shape", heads)
    n_q, n_kv, d, page_size = geometry
    lengths, q_lens = [700, 333, 40, 16, 1000], [700, 50, 33, 16, 2]
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        torch.bfloat16, n_q, n_kv, d, page_size, lengths=lengths, q_lens=q_lens, seed=29)
    scale = 1.0 / math.sqrt(d)
    out_a = torch.full((qkv.shape[0], n_q * d), float("nan"), dtype=torch.bfloat16).cuda()
    ops.paged_attention(qkv, out_a, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=max(lengths) - 1, batch=make_batch(lengths, q_lens))
    out_b = dense_attention(qkv, k_pages, v_pages, table, lengths, q_lens, n_q, n_kv, d, window, scale)
    torch.testing.assert_close(out_a.float(), out_b, **attention_tol(torch.bfloat16, True))
    rows = torch.tensor([0, 17, 699, 700, 749, 750, qkv.shape[0] - 1]).cuda()
    out_c = torch.empty((len(rows), n_q * d), dtype=torch.bfloat16).cuda()
    ref.paged_attention(qkv[rows], out_c, k_pages, v_pages, positions[rows], entry_of_token[rows], table, n_q, n_kv, d,
                        window, scale)
    torch.testing.assert_close(out_c.float(), out_b[rows], **tol(torch.bfloat16))
    # The other prompt kernel rounds at other places; both stay within the same distance of the float32 result.
    monkeypatch.setattr(ops, "prefill_shared", -1)
    monkeypatch.setattr(ops, "prefill_shape", 0)
    out_d = torch.full_like(out_a, float("nan"))
    ops.paged_attention(qkv, out_d, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, scale,
                        max_position=max(lengths) - 1, batch=make_batch(lengths, q_lens))
    torch.testing.assert_close(out_d.float(), out_b, **attention_tol(torch.bfloat16, True))


@pytest.mark.parametrize("target", [1024, 16])
@pytest.mark.parametrize("window", [None, 1000])
def test_decode_attention_long_contexts_and_many_splits(ops, ref, window, target, monkeypatch):
    # Batches of single tokens at long, unequal contexts: the key range is cut into many splits (a wave has a few
    # blocks and asks for the next one ahead), or, aiming at few workgroups, into one or two long ones (a wave
    # walks dozens of blocks one after the other).
    monkeypatch.setattr(ops, "target_workgroups", target)
    n_q, n_kv, d, page_size = 14, 2, 64, 16
    for lengths in ([3000], [2049, 1, 777, 4096, 31, 32, 33, 2500]):
        qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
            torch.bfloat16, n_q, n_kv, d, page_size, lengths=lengths, q_lens=[1] * len(lengths), seed=13)
        out_a = torch.empty((qkv.shape[0], n_q * d), dtype=torch.bfloat16).cuda()
        out_b = torch.empty_like(out_a)
        ops.paged_attention(qkv, out_a, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window,
                            0.125, max_position=max(lengths) - 1)
        ref.paged_attention(qkv, out_b, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, 0.125)
        torch.testing.assert_close(out_a.float(), out_b.float(), rtol=2e-2, atol=4e-3)


@pytest.mark.parametrize("attention_mode", ATTENTION_MODES, indirect=True)
def test_paged_attention_finds_one_far_key(ops, attention_mode):
    dtype = attention_mode
    # One key far back is made to dominate: the output must be its value row.
    n_q, n_kv, d, page_size = 4, 2, 64, 16
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        dtype, n_q, n_kv, d, page_size, lengths=[700], q_lens=[1], seed=12)
    target = 123
    page, off = int(table[0, target // page_size]), target % page_size
    q = qkv[0, :n_q * d].reshape(n_q, d).float()
    for h in range(n_q):
        k_pages[page, h // 2, off] = 0
    k_pages[page, 0, off] = (q[0] * 40 / q[0].norm()).to(dtype)
    qkv[0, d:2 * d] = qkv[0, :d]            # head 1 shares kv head 0 and looks the same way
    k_pages[page, 1, off] = (q[2] * 40 / q[2].norm()).to(dtype)
    qkv[0, 3 * d:4 * d] = qkv[0, 2 * d:3 * d]
    out = torch.empty((1, n_q * d), dtype=dtype).cuda()
    ops.paged_attention(qkv, out, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, None, 1.0)
    got = out.reshape(n_q, d).float()
    for h in range(n_q):
        torch.testing.assert_close(got[h], v_pages[page, h // 2, :, off].float(), rtol=2e-2, atol=2e-2)
    # With a window that ends just after the key, it is gone: position 699 sees keys >= 699 - w.
    ops.paged_attention(qkv, out, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, 699 - target - 1, 1.0)
    assert (out.reshape(n_q, d).float()[0] - v_pages[page, 0, :, off].float()).abs().max() > 0.1
    ops.paged_attention(qkv, out, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, 699 - target, 1.0)
    torch.testing.assert_close(out.reshape(n_q, d).float()[0], v_pages[page, 0, :, off].float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("attention_mode", ATTENTION_MODES, indirect=True)
@pytest.mark.parametrize("waves,heads,shared", [(0, (4, 2, 64), 0), (1, (4, 2, 64), 0), (0, (10, 2, 128), 1)])
def test_every_row_of_a_portion_sees_exactly_to_its_window_edge(ops, attention_mode, waves, heads, shared, monkeypatch):
    """A portion of 100 prompt tokens under a window of 77: the query at position p is made to look at the key
    at p - 77, the farthest it may see; those keys cross page and tile edges.  The output must be that key's
    value row; with a window of 76 the key is out of sight and the output is something else."""
    dtype = attention_mode
    monkeypatch.setattr(ops, "prefill_waves", waves)
    monkeypatch.setattr(ops, "prefill_shared", shared)
    (n_q, n_kv, d), page_size, window = heads, 16, 77
    lengths, q_lens = [700], [100]
    qkv, k_pages, v_pages, positions, entry_of_token, table = make_paged_case(
        dtype, n_q, n_kv, d, page_size, lengths=lengths, q_lens=q_lens, seed=21)
    group = n_q // n_kv
    want = torch.empty((q_lens[0], n_q, d))
    for row in range(q_lens[0]):
        target = int(positions[row]) - window
        page, off = int(table[0, target // page_size]), target % page_size
        for h in range(n_q):
            key = k_pages[page, h // group, off].float()
            qkv[row, h * d:(h + 1) * d] = (key * (30.0 / float(key.dot(key)))).to(dtype)   # its score is 30
            want[row, h] = v_pages[page, h // group, :, off].float().cpu()
    batch = make_batch(lengths, q_lens) if ops.use_fast_attention else None
    out = torch.full((q_lens[0], n_q * d), float("nan"), dtype=dtype).cuda()
    ops.paged_attention(qkv, out, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window, 1.0,
                        max_position=lengths[0] - 1, batch=batch)
    torch.testing.assert_close(out.float().cpu().reshape(q_lens[0], n_q, d), want, rtol=2e-2, atol=2e-2)
    ops.paged_attention(qkv, out, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, window - 1, 1.0,
                        max_position=lengths[0] - 1, batch=batch)
    off_by = (out.float().cpu().reshape(q_lens[0], n_q, d) - want).abs().amax(dim=(1, 2))
    assert float(off_by.min()) > 0.1          # every row lost its key


def linear_tol(out_dtype, x, w):
    # A float32 sum of K products errs by about sqrt(K) * 2^-24 * |x||w| per term, also where the
    # result cancels to nearly zero; allow eight times that.  bfloat16 output adds its own rounding.
    k = x.shape[1]
    typical = float(x.float().pow(2).mean().sqrt() * w.float().pow(2).mean().sqrt()) * k ** 0.5
    base = tol(out_dtype)
    return dict(rtol=base["rtol"], atol=max(base["atol"], 8 * k ** 0.5 * 2.0 ** -24 * typical))


@pytest.mark.parametrize("shape", [(40, 200, 2304), (64, 96, 4864), (17, 1028, 2048), (33, 64, 2056)])
def test_linear_with_k_cut_over_workgroups(ops, ref, shape, monkeypatch):
    """17 to 64 rows, a long K and few output tiles: the tiled kernel cuts K over workgroups and adds the parts
    in a fixed order; the result is the same product, the same on every run."""
    monkeypatch.setattr(ops, "SPLIT_K_FROM", 2048)
    monkeypatch.setattr(ops, "split_k_kind", "tiled")
    m, n, k = shape
    assert ops._k_splits(m, n, k) > 1
    x = rand((m, k), torch.bfloat16, 24)
    w = rand((n, k), torch.bfloat16, 25, 0.1)
    bias = rand((n,), torch.float32, 26)
    for use_bias in (True, False):
        for out_dtype in (torch.bfloat16, torch.float32):
            got = ops.linear(x, w, bias if use_bias else None, out_dtype=out_dtype)
            want = ref.linear(x, w, bias if use_bias else None, out_dtype=torch.float64)
            torch.testing.assert_close(got.double(), want, **linear_tol(out_dtype, x, w))
            again = ops.linear(x, w, bias if use_bias else None, out_dtype=out_dtype)
            assert torch.equal(got, again)


@pytest.mark.parametrize("shape", [(137, 896, 4864), (65, 100, 2056), (256, 1536, 8960), (100, 896, 896), (200, 60, 776)])
def test_linear_of_a_few_hundred_rows_with_k_cut(ops, ref, shape, monkeypatch):
    """65 to 256 rows (a portion of a prompt beside decoded tokens) and few output tiles: K is cut where the parts
    may stay for the next norm (long K: recorded or not; shorter K: when launched eagerly, where small products
    do not go to the library), or into four parts that the kernel adds itself.  The same product either way, the
    same on every run; the parts, added, are the product too."""
    m, n, k = shape
    x = rand((m, k), torch.bfloat16, 34)
    w = rand((n, k), torch.bfloat16, 35, 0.1)
    bias = rand((n,), torch.float32, 36)
    want = ref.linear(x, w, bias, out_dtype=torch.float64)
    for capturing in (False, True):
        monkeypatch.setattr(ops, "capturing", capturing)
        expect_parts = k >= 2048 or (not capturing and k >= 768)
        assert (ops._k_splits(m, n, k, True) > 1) == expect_parts
        assert (ops._k_splits(m, n, k, False) > 1) == (not capturing and k >= 2048 and m * n * k < ops.EAGER_LIBRARY_WORK)
        left = ops.linear(x, w, bias, pending=True)
        assert isinstance(left, PendingSum) == expect_parts
        got = left.resolve() if expect_parts else left
        torch.testing.assert_close(got.double(), want, **linear_tol(torch.bfloat16, x, w))
        added = ops.linear(x, w, bias)
        torch.testing.assert_close(added.double(), want, **linear_tol(torch.bfloat16, x, w))
        assert torch.equal(added, ops.linear(x, w, bias))
        if expect_parts:
            # The parts go into the norm that follows as they are: sum + bias + residual, then the norm.
            residual = rand((m, n), torch.float32, 37)
            weight = rand((n,), torch.float32, 38).abs() + 0.5
            out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
            stream = residual.clone()
            ops.add_rmsnorm(stream, left, weight, 1e-6, out)
            total = residual.double() + want
            torch.testing.assert_close(stream.double(), total, rtol=1e-5, atol=linear_tol(torch.float32, x, w)["atol"])
            normed = total / (total.pow(2).mean(dim=1, keepdim=True) + 1e-6).sqrt() * weight.double()
            torch.testing.assert_close(out.double(), normed, rtol=1e-2, atol=2e-2)


@pytest.mark.parametrize("shape", [(40, 200, 2304), (64, 96, 4864), (17, 1028, 2048), (33, 64, 2056), (20, 52, 4104)])
def test_linear_with_k_cut_over_streaming_workgroups(ops, ref, shape):
    """The same for the weight-streaming kernel (K of 2,048 up to 8,192): parts that are no multiple of 32 long in
    all, a last part with a tail of K, output columns that do not fill the last tile of sixteen."""
    m, n, k = shape
    assert ops._streaming_splits(m, n, k) > 1
    x = rand((m, k), torch.bfloat16, 24)
    w = rand((n, k), torch.bfloat16, 25, 0.1)
    bias = rand((n,), torch.float32, 26)
    for use_bias in (True, False):
        for out_dtype in (torch.bfloat16, torch.float32):
            got = ops.linear(x, w, bias if use_bias else None, out_dtype=out_dtype)
            want = ref.linear(x, w, bias if use_bias else None, out_dtype=torch.float64)
            torch.testing.assert_close(got.double(), want, **linear_tol(out_dtype, x, w))
            assert torch.equal(got, ops.linear(x, w, bias if use_bias else None, out_dtype=out_dtype))


@pytest.mark.parametrize("shape", [(17, 1152, 896), (64, 896, 4864), (200, 264, 136), (2048, 1152, 896)])
def test_linear_through_the_library_and_through_own_kernels(ops, ref, shape, monkeypatch):
    """More than sixteen bfloat16 rows may go to the vendor's library, the float32 bias in its accumulator; the
    package's own kernels give the same product.  Rows of the input may be strided."""
    m, n, k = shape
    wide = rand((m, k + 24), torch.bfloat16, 27)
    x = wide[:, 8:8 + k]                                 # strided rows, 16-byte aligned
    w = rand((n, k), torch.bfloat16, 28, 0.1)
    bias = rand((n,), torch.float32, 29)
    for use_bias in (True, False):
        b = bias if use_bias else None
        want = ref.linear(x, w, b, out_dtype=torch.float64)
        monkeypatch.setattr(ops, "use_library_gemm", True)
        monkeypatch.setattr(ops, "LIBRARY_WEIGHT", 0)    # every product of more than sixteen rows
        through_library = ops.linear(x, w, b)
        monkeypatch.setattr(ops, "use_library_gemm", False)
        own = ops.linear(x, w, b)
        for got in (through_library, own):
            torch.testing.assert_close(got.double(), want, **linear_tol(torch.bfloat16, x, w))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 100, 72), (37, 200, 136), (130, 260, 272), (300, 1000, 64), (64, 151, 896),
                                   (8, 384, 96), (513, 130, 40)])
def test_linear(ops, ref, dtype, shape):
    m, n, k = shape
    x = rand((m, k), dtype, 20)
    w = rand((n, k), dtype, 21, 0.1)
    bias = rand((n,), torch.float32, 22)
    for use_bias in (True, False):
        for out_dtype in ([torch.float32] if dtype == torch.float32 else [torch.bfloat16, torch.float32]):
            got = ops.linear(x, w, bias if use_bias else None, out_dtype=out_dtype)
            want = ref.linear(x, w, bias if use_bias else None, out_dtype=torch.float64)
            torch.testing.assert_close(got.double(), want, **linear_tol(out_dtype, x, w))
    # Rows of a wider buffer.
    wide = rand((m, k + 24), dtype, 23)
    got = ops.linear(wide[:, :k], w, None, out_dtype=torch.float32)
    want = ref.linear(wide[:, :k], w, None, out_dtype=torch.float64)
    torch.testing.assert_close(got.double(), want, **linear_tol(torch.float32, x, w))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 272, 96), (8, 4864, 896), (33, 130, 72), (64, 176, 80), (100, 128, 64)])
def test_linear_silu_gate(ops, ref, dtype, shape):
    m, inner, k = shape
    x = rand((m, k), dtype, 30)
    w = rand((2 * inner, k), dtype, 31, 0.1)
    got = ops.linear_silu_gate(x, w)
    want = torch.empty((m, inner), dtype=torch.float64).cuda()
    gate_up = ref.linear(x, w, None, out_dtype=torch.float64)
    ref.silu_gate(gate_up, want)
    # Unfused, the products are rounded to the storage dtype before the activation; allow for that.
    base = linear_tol(dtype, x, w)
    torch.testing.assert_close(got.double(), want, rtol=2 * base["rtol"], atol=4 * base["atol"] + (2e-2 if dtype == torch.bfloat16 else 0))


@pytest.mark.parametrize("shape", [(1, 1152, 896), (8, 896, 4864), (64, 151, 896), (17, 100, 40), (48, 3000, 264)])
def test_skinny_rows_agree_with_the_tiled_kernel(ops, shape):
    # The same product through the weight-streaming kernel and through the tiled one.
    m, n, k = shape
    x = rand((m, k), torch.bfloat16, 32)
    w = rand((n, k), torch.bfloat16, 33, 0.1)
    bias = rand((n,), torch.float32, 34)
    skinny = ops.linear(x, w, bias, out_dtype=torch.float32)
    before = ops.SKINNY_ROWS
    try:
        ops.SKINNY_ROWS = 0
        tiled = ops.linear(x, w, bias, out_dtype=torch.float32)
    finally:
        ops.SKINNY_ROWS = before
    torch.testing.assert_close(skinny, tiled, **linear_tol(torch.float32, x, w))


@pytest.mark.parametrize("geometry", [(14, 2, 64, 896, 16), (3, 1, 32, 96, 16), (4, 4, 128, 520, 32), (20, 2, 96, 264, 16),
                                      (2, 1, 64, 1280, 16), (4, 2, 32, 2304, 16), (12, 2, 128, 1536, 16),
                                      (3, 1, 64, 2048, 16), (2, 2, 32, 1800, 16)])
@pytest.mark.parametrize("rows", [1, 8, 16, 17, 40, 64])
def test_fused_norm_qkv_rope(ops, ref, geometry, rows):
    # Up to 16 rows: the fused decode kernel, from the residual or from normalised rows; 17 to 64 rows: the
    # weight-streaming kernel with the same epilogue, from normalised rows.
    n_q, n_kv, d, hidden, page_size = geometry
    n_pages, max_pos = 7, 300
    gen = torch.Generator().manual_seed(40)
    residual = rand((rows, hidden), torch.float32, 41, 2.0)
    norm_w = rand((hidden,), torch.float32, 42) * 0.1 + 1
    w = rand(((n_q + 2 * n_kv) * d, hidden), torch.bfloat16, 43, 0.05)
    bias = rand(((n_q + 2 * n_kv) * d,), torch.float32, 44)
    positions = torch.randint(0, max_pos, (rows,), generator=gen).int().cuda()
    inv = torch.tensor([1.0 / (1e6 ** (i / d)) for i in range(0, d, 2)], dtype=torch.float64).float()
    ang = torch.arange(max_pos).float()[:, None] * inv[None]
    cos_sin = torch.cat([ang.cos(), ang.sin()], 1).cuda()
    slots = torch.randperm(n_pages * page_size, generator=gen)[:rows].int().cuda()
    if rows > 2:
        slots[1] = -1
    for use_bias, table, store in ((True, cos_sin, True), (False, cos_sin, True), (True, None, True), (True, cos_sin, False)):
        ka = torch.zeros((n_pages, n_kv, page_size, d), dtype=torch.bfloat16).cuda()
        va = torch.zeros((n_pages, n_kv, d, page_size), dtype=torch.bfloat16).cuda()
        kb, vb = ka.clone(), va.clone()
        args = (residual, norm_w, 1e-6, w, bias if use_bias else None, positions, table, slots if store else None)
        before = residual.clone()
        qb = ref.fused_norm_qkv_rope(*args, kb, vb, n_q, n_kv, d)
        # The norm's output is rounded to bfloat16 in both; what differs is the summation order.
        tolerance = dict(rtol=2e-2, atol=2e-2)
        if rows <= 16:
            qa = ops.fused_norm_qkv_rope(*args, ka, va, n_q, n_kv, d)
            assert torch.equal(residual, before)
            torch.testing.assert_close(qa.float(), qb.float(), **tolerance)
            torch.testing.assert_close(ka.float(), kb.float(), **tolerance)
            torch.testing.assert_close(va.float(), vb.float(), **tolerance)
            if not store:
                assert float(ka.abs().max()) == 0 and float(va.abs().max()) == 0
        # The same from rows that are normalised already (the route of wide models): rows of a wider buffer.
        wide = torch.zeros((rows, hidden + 8), dtype=torch.bfloat16).cuda()
        normed = wide[:, :hidden]
        ref.add_rmsnorm(residual.clone(), None, norm_w, 1e-6, normed)
        kc, vc = torch.zeros_like(ka), torch.zeros_like(va)
        qc = ops.fused_norm_qkv_rope(normed, None, 1e-6, w, bias if use_bias else None, positions, table,
                                     slots if store else None, kc, vc, n_q, n_kv, d)
        torch.testing.assert_close(qc.float(), qb.float(), **tolerance)
        torch.testing.assert_close(kc.float(), kb.float(), **tolerance)
        torch.testing.assert_close(vc.float(), vb.float(), **tolerance)
        if not store:
            assert float(kc.abs().max()) == 0 and float(vc.abs().max()) == 0


# Rows of 1,280 and 2,304 elements give the waves unequal shares of K in the kernels that ask for
# a wave's whole share at once (some waves then have steps past the end, which must add nothing); rows of 1,536 to
# 2,048 are one trip of six or eight steps from normalised rows in LDS (in one block of weight rows, or in two where
# the matrix has more than sixteen rows for every compute unit).
@pytest.mark.parametrize("shape", [(1, 4864, 896), (8, 272, 96), (16, 176, 80), (5, 136, 72), (6, 1280, 2304),
                                   (8, 2304, 1280), (8, 8960, 1536), (3, 1104, 1536), (16, 600, 2048), (7, 5000, 1800)])
def test_fused_norm_gated_and_linear_add(ops, ref, shape):
    rows, inner, hidden = shape
    residual = rand((rows, hidden), torch.float32, 50, 2.0)
    norm_w = rand((hidden,), torch.float32, 51) * 0.1 + 1
    w = rand((2 * inner, hidden), torch.bfloat16, 52, 0.1)
    got = ops.fused_norm_gated(residual, norm_w, 1e-5, w)
    want = ref.fused_norm_gated(residual, norm_w, 1e-5, w)
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    normed = torch.empty((rows, hidden), dtype=torch.bfloat16).cuda()
    ref.add_rmsnorm(residual.clone(), None, norm_w, 1e-5, normed)
    torch.testing.assert_close(ops.fused_norm_gated(normed, None, 1e-5, w).float(), want.float(), rtol=2e-2, atol=2e-2)
    # residual += act @ down.T + bias
    down = rand((hidden, inner), torch.bfloat16, 53, 0.05)
    bias = rand((hidden,), torch.float32, 54)
    for use_bias in (True, False):
        res_a, res_b = residual.clone(), residual.clone()
        ops.linear_add(got, down, bias if use_bias else None, res_a)
        ref.linear_add(got, down, bias if use_bias else None, res_b)
        torch.testing.assert_close(res_a, res_b, **linear_tol(torch.float32, got, down))
    wide = rand((rows, inner + 8), torch.bfloat16, 55)
    res_a, res_b = residual.clone(), residual.clone()
    ops.linear_add(wide[:, :inner], down, None, res_a)
    ref.linear_add(wide[:, :inner], down, None, res_b)
    torch.testing.assert_close(res_a, res_b, **linear_tol(torch.float32, wide[:, :inner], down))


@pytest.mark.parametrize("shape", [(40, 896, 4864), (64, 1536, 8960), (17, 2048, 11008), (33, 100, 2048)])
def test_product_left_in_parts_and_added_by_the_norm(ops, ref, shape):
    # A product of 17 to 64 rows whose K is cut over workgroups may come back in parts; the norm that takes it as
    # its delta adds the parts, the bias and the residual and normalises in one kernel.  Both that and the parts
    # added on their own agree with the plain product and the plain norm.
    from tokenizer_amd.kernels import PendingSum
    m, n, k = shape
    x, w = rand((m, k), torch.bfloat16, 1), rand((n, k), torch.bfloat16, 2, 0.05)
    bias, gain = rand((n,), torch.float32, 3), 1 + rand((n,), torch.float32, 4, 0.1)
    residual = rand((m, n), torch.float32, 5, 2.0)
    got = ops.linear(x, w, bias, pending=True)
    assert isinstance(got, PendingSum) and got.shape == (m, n) and got.partial.shape[0] > 1
    plain_product = ref.linear(x, w, bias, out_dtype=torch.float32)
    torch.testing.assert_close(got.resolve().float(), plain_product, rtol=2e-2, atol=2e-2)
    # (the product that adds its parts itself may cut K differently: equal up to the rounding of the sums)
    torch.testing.assert_close(got.resolve().float(), ops.linear(x, w, bias).float(), **tol(torch.bfloat16))
    assert torch.equal(got.resolve(), got.resolve())
    res_a, res_b = residual.clone(), residual.clone()
    out_a = ops.add_rmsnorm(res_a, got, gain, 1e-6, torch.empty((m, n), dtype=torch.bfloat16).cuda())
    out_b = ref.add_rmsnorm(res_b, plain_product, gain, 1e-6, torch.empty((m, n), dtype=torch.float32).cuda())
    torch.testing.assert_close(res_a, res_b, rtol=1e-4, atol=1e-3)
    torch.testing.assert_close(out_a.float(), out_b, rtol=2e-2, atol=2e-2)
    # A row subset (the final norm) has the parts added first.
    rows = torch.tensor([m - 1, 0], dtype=torch.int32).cuda()
    res_c = residual.clone()
    out_c = ops.add_rmsnorm(res_c, got, gain, 1e-6, torch.empty((2, n), dtype=torch.bfloat16).cuda(), rows,
                            store_residual=False)
    assert torch.equal(res_c, residual)
    torch.testing.assert_close(out_c.float(), out_b[rows.long()], rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("hidden", [896, 1028, 2048, 3000, 3584, 4096])
@pytest.mark.parametrize("splits", [1, 3, 8, 11, 20])
@pytest.mark.parametrize("with_bias", [False, True])
def test_parts_of_every_count_added_by_the_norm_at_every_row_length(ops, hidden, splits, with_bias):
    # The norm that adds a product's parts has an instance for every 1,024 floats of a row's length and asks for its
    # first parts, the bias, the residual and the norm weight at once: every count of parts around the eight (or four)
    # it asks for first, with and without a bias, against sums in the same order in float32.
    from tokenizer_amd.kernels import PendingSum
    m = 19
    parts = rand((splits, m, hidden), torch.float32, 11, 1.5)
    bias = rand((hidden,), torch.float32, 12) if with_bias else None
    gain = 1 + rand((hidden,), torch.float32, 13, 0.1)
    residual = rand((m, hidden), torch.float32, 14, 2.0)
    total = torch.zeros((m, hidden), dtype=torch.float32).cuda()
    for part in parts:
        total = total + part
    if with_bias:
        total = total + bias
    want_residual = residual + total
    want = want_residual * torch.rsqrt(want_residual.pow(2).mean(dim=1, keepdim=True) + 1e-6) * gain
    for dtype in (torch.bfloat16, torch.float32):
        got_residual = residual.clone()
        out = ops.add_rmsnorm(got_residual, PendingSum(ops, parts, bias, dtype), gain, 1e-6,
                              torch.empty((m, hidden), dtype=dtype).cuda())
        assert torch.equal(got_residual, want_residual)
        torch.testing.assert_close(out.float(), want, **tol(dtype))


@pytest.mark.parametrize("shape", [(33, 48, 264), (64, 100, 896), (50, 900, 40), (64, 1000, 2048)])
def test_weight_streaming_product_with_two_column_blocks(ops, ref, shape, monkeypatch):
    # More than 32 rows may take two blocks of sixteen output columns per workgroup (the rows are then read half as
    # often): with one block and with two, plain, gated and with K cut over workgroups, at widths that end inside
    # a block and inside a pair of blocks.
    m, n, k = shape
    x, w = rand((m, k), torch.bfloat16, 31), rand((n, k), torch.bfloat16, 32, 0.05)
    bias = rand((n,), torch.float32, 33)
    monkeypatch.setattr(ops, "use_library_gemm", False)
    want = ref.linear(x, w, bias, out_dtype=torch.float32)
    gated_want = ref.linear_silu_gate(x.float(), w.float(), None)
    results = []
    for blocks in (1, 2):
        monkeypatch.setattr(ops, "skinny_column_blocks", blocks)
        got = ops.linear(x, w, bias)
        torch.testing.assert_close(got.float(), want, **tol(torch.bfloat16))
        gated = ops.linear_silu_gate(x, w)
        torch.testing.assert_close(gated.float(), gated_want, rtol=2e-2, atol=2e-3)
        parts = ops.linear(x, w, bias, pending=True)
        if not isinstance(parts, torch.Tensor):
            parts = parts.resolve()
        torch.testing.assert_close(parts.float(), want, **tol(torch.bfloat16))
        results.append((got, gated))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])


@pytest.mark.parametrize("rows", [1, 7, 8, 9, 16])
@pytest.mark.parametrize("k", [896, 72, 200, 64, 40])
def test_vocabulary_projection_of_few_rows_reads_its_weights_line_by_line(ops, rows, k):
    """Up to sixteen rows against tens of thousands of output columns: the weight-streaming kernel with four column
    blocks a workgroup, whose weight loads touch eight rows' whole cache lines and are put right for the matrix
    instruction by an exchange between lanes.  Against the plain product and against the same kernel with the older
    loads (the same sums in another order): widths that end inside a workgroup's 64 columns, a K of whole lines, of
    a line and a piece, of less than a line, one to sixteen rows (the upper half of the row block empty or not),
    rows of a wider buffer, float32 and bfloat16 results."""
    n = 70_003
    x = rand((rows, k + 8), torch.bfloat16, 161)[:, :k]
    w = rand((n, k), torch.bfloat16, 162, 0.1)
    bias = rand((n,), torch.float32, 163)
    want = x.float() @ w.float().t() + bias
    results = []
    for lines in (1, 0):
        ops.lib.ta_skinny_lines(lines)
        try:
            got = ops.linear(x, w, bias, out_dtype=torch.float32)
            half = ops.linear(x, w, bias)
        finally:
            ops.lib.ta_skinny_lines(1)
        torch.testing.assert_close(got, want, **linear_tol(torch.float32, x, w))
        torch.testing.assert_close(half.float(), want, **linear_tol(torch.bfloat16, x, w))
        results.append(got)
    torch.testing.assert_close(results[0], results[1], rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("shape", [(1, 151, 37), (3, 50, 1000), (16, 33, 130), (9, 1000, 896), (16, 4, 8)])
def test_linear_float32_of_few_rows(ops, ref, shape):
    # Up to sixteen float32 rows take the kernel that walks the weights once: widths that end inside a wave's four
    # weight rows, K that is and is not a multiple of four, rows of A with a stride.
    m, n, k = shape
    wide = rand((m, k + 12), torch.float32, 41)
    x, w, bias = wide[:, 4:4 + k], rand((n, k), torch.float32, 42, 0.1), rand((n,), torch.float32, 43)
    want = (x.double() @ w.double().t() + bias.double()).float()
    torch.testing.assert_close(ops.linear(x, w, bias), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(ops.linear(x.contiguous(), w), (x.double() @ w.double().t()).float(), rtol=1e-5, atol=1e-5)


def test_linear_float32_is_true_float32(ops):
    # Inputs that need 13 mantissa bits: a reduced-precision matrix mode (10 or 7 bits) would be off by
    # about 1e-2 here, float32 accumulation by less than 3e-4.
    k = 64
    x = (1 + torch.arange(k, dtype=torch.float64) * 2.0 ** -12).float().reshape(1, k).cuda()
    w = (1 - torch.arange(k, dtype=torch.float64) * 2.0 ** -13).float().reshape(1, k).cuda()
    got = ops.linear(x, w, None)
    want = (x.double() * w.double()).sum()
    assert abs(float(got) - float(want)) < 1e-3


@pytest.mark.parametrize("rows", [1, 16, 17, 64, 65, 200])
def test_linear_float32_is_true_float32_at_every_row_count(ops, rows):
    """The same probe for each of the 32-bit product's kernels (one row, up to sixteen rows, the tiled kernel for
    more): operands that need 13 mantissa bits, over a K long enough for the tile loop to turn, in every row and
    column of a tile and past its edge.  A reduced-precision matrix mode would be off by
    about 2e-2; true 32-bit products and sums are within a few 1e-4 of the 64-bit result of sums near 500."""
    k, n = 520, 150
    x = (1 + torch.arange(k, dtype=torch.float64)[None, :] * 2.0 ** -12
         + torch.arange(rows, dtype=torch.float64)[:, None] * 2.0 ** -13).float().cuda()
    w = (1 - torch.arange(k, dtype=torch.float64)[None, :] * 2.0 ** -13
         - torch.arange(n, dtype=torch.float64)[:, None] * 2.0 ** -12).float().cuda()
    got = ops.linear(x, w, None)
    want = x.double() @ w.double().t()
    assert float((got.double() - want).abs().max()) < 2e-3
    # What rounding the operands to bfloat16 would do to the same sums: several times the bound.
    low = x.bfloat16().double() @ w.bfloat16().double().t()
    assert float((low - want).abs().max()) > 1e-2


def test_argmax_first_maximum_wins(ops):
    logits = torch.full((5, 3000), -1.0)
    logits[0, 2999] = 3.0
    logits[1, 7] = 2.0
    logits[1, 2000] = 2.0          # tie: the lower index
    logits[2, 1500] = 2.0
    logits[2, 1499] = 2.0
    logits[3] = 0.0                # all equal: index 0
    logits[4] = float("-inf")      # a scan with `>` from -inf never moves: index 0
    out = ops.argmax(logits.cuda()).cpu().tolist()
    assert out == [2999, 7, 1499, 0, 0]
    small = torch.tensor([[0.2, 1.5, 1.5, -3.0, 0.0]]).cuda()   # qwen-infer/src/sample.rs:191-192
    assert ops.argmax(small).item() == 1


def test_sampling_kernel_follows_the_reference_rules(ops, ref):
    import numpy as np
    rng = np.random.default_rng(3)
    rows = []
    for case in range(48):
        vocab_row = rng.normal(size=3000).astype(np.float32) * float(rng.choice([0.5, 2.0, 6.0]))
        if case % 4 == 0:
            vocab_row[100:160] = vocab_row[7]                 # many equal logits: the index order decides
        if case % 6 == 1:
            vocab_row[::2] = -np.inf
        rows.append(vocab_row)
    logits = torch.tensor(np.stack(rows)).cuda()
    temperature = torch.tensor(rng.choice([0.3, 0.7, 1.0, 1.8], size=48).astype(np.float32)).cuda()
    top_p = torch.tensor(rng.choice([0.05, 0.5, 0.9, 0.999, 1.0, 4.0], size=48).astype(np.float32)).cuda()
    uniform = torch.tensor(rng.random(48).astype(np.float32)).cuda()
    got = ops.sample(logits, temperature, top_p, uniform).cpu().tolist()
    want = ref.sample(logits, temperature, top_p, uniform).cpu().tolist()
    # Sums run in another order on the device, so a draw that falls within rounding of a boundary may land
    # on the neighbouring token; everywhere else the ids are equal.
    same = sum(int(a == b) for a, b in zip(got, want))
    assert same >= 46, (got, want)
    for row, (a, b) in enumerate(zip(got, want)):
        if a != b:
            order = sorted(range(3000), key=lambda i: (-float(logits[row, i]), i))
            assert abs(order.index(a) - order.index(b)) <= 1, (row, a, b)
    # qwen-infer/src/sample.rs:211-230: a tiny top_p keeps the top token; top_p above one is one.
    small = torch.tensor([[0.0, 2.0, 0.5, -1.0]] * 8).cuda()
    us = torch.linspace(0.01, 0.99, 8).cuda()
    ones = torch.ones(8).cuda()
    assert ops.sample(small, ones, ones * 1e-6, us).cpu().tolist() == [1] * 8
    assert ops.sample(small, ones * 0.7, ones * 0.0, us).cpu().tolist() == [1] * 8
    assert ops.sample(small, ones * 0.8, ones, us).cpu().tolist() == ops.sample(small, ones * 0.8, ones * 4, us).cpu().tolist()
    flat = torch.zeros(8, 8).cuda()
    assert ops.sample(flat, ones, ones, torch.arange(8).cuda() / 8 + 0.01).cpu().tolist() == list(range(8))
    # All -inf: nothing to weigh, the first index, as the greedy scan gives.
    assert ops.sample(torch.full((1, 50), float("-inf")).cuda(), ones[:1], ones[:1], us[:1]).item() == 0


@pytest.mark.parametrize("rows, vocab, widths, page_size", [(1, 33, [3], 16), (8, 5000, [40, 7], 16), (37, 151936, [9], 32),
                                                            (64, 700, [5, 5, 2, 11], 48)])
def test_greedy_pick_that_writes_the_next_steps_description(ops, rows, vocab, widths, page_size):
    """The pick itself is `argmax`'s; the ids become the next tokens, positions and first positions go up by one,
    and each group's slots are page * page size + offset of the new position, looked up in the request's row of
    that group's table: -1 where the page is not there, the row's last entry where the position lies past the
    table (what the host never relies on)."""
    import numpy as np
    rng = np.random.default_rng(rows + vocab)
    logits = torch.tensor(rng.normal(size=(rows, vocab)).astype(np.float32)).cuda()
    ids = torch.full((rows,), -7, dtype=torch.int32).cuda()
    reach = min(widths) * page_size
    start = rng.integers(0, reach + 40, size=rows).astype(np.int32)          # some past the narrowest table's end
    start[0] = page_size - 1                                                  # the next position opens a page
    positions, first = torch.tensor(start).cuda(), torch.tensor(start).cuda()
    tables, slots = [], []
    for width in widths:
        table = rng.permutation(rows * width).astype(np.int32).reshape(rows, width)
        table[rng.random((rows, width)) < 0.2] = -1
        tables.append(torch.tensor(table).cuda())
        slots.append(torch.full((rows,), -5, dtype=torch.int32).cuda())
    picked = ops.argmax_next_step(logits, ids, positions, first, slots, tables, page_size)
    assert torch.equal(picked, ops.argmax(logits)) and torch.equal(ids, picked)
    after = start + 1
    assert positions.cpu().numpy().tolist() == after.tolist() and first.cpu().numpy().tolist() == after.tolist()
    for width, table, slot in zip(widths, tables, slots):
        page = table.cpu().numpy()[np.arange(rows), np.minimum(after // page_size, width - 1)]
        want = np.where(page < 0, -1, page * page_size + after % page_size)
        assert slot.cpu().numpy().tolist() == want.tolist()
    with pytest.raises(KernelError):                                          # five groups; positions of another size
        ops.argmax_next_step(logits, ids, positions, first, (slots * 5)[:5], (tables * 5)[:5], page_size)
    with pytest.raises(KernelError):
        ops.argmax_next_step(logits, ids, torch.zeros(rows + 1, dtype=torch.int32).cuda(), first, slots, tables, page_size)


@pytest.mark.parametrize("vocab", [151936, 50257, 33])
def test_sampling_kernel_over_large_and_tiny_vocabularies(ops, ref, vocab):
    """A row is cut into slices that are summed by workgroups of their own, round after round: vocabularies that
    fill every slice, that leave the last slice short, and that leave most slices empty; peaked rows (a nucleus
    of a few tokens) and flat ones (the crossing deep in the bulk, among many tokens in one range of keys); rows
    with and without a nucleus cut in one batch; the same draw on every run."""
    import numpy as np
    rng = np.random.default_rng(vocab)
    rows, temps, tops = [], [], []
    for case in range(12):
        scale = [0.05, 1.0, 4.0][case % 3]
        row = rng.normal(size=vocab).astype(np.float32) * scale
        if case % 4 == 1:
            row[rng.integers(0, vocab, size=5)] += 12.0            # a few tokens hold nearly all the mass
        if case % 4 == 2:
            row[vocab // 3:vocab // 3 + 20] = row.max()             # equal maxima: the index order decides
        if case == 11:
            row[:] = -np.inf
            row[vocab - 1] = 0.5                                    # a single token that can be drawn, in the last slice
        rows.append(row)
        temps.append([0.6, 1.0, 1.5][case % 3])
        tops.append([0.9, 1.0, 0.5, 1.0][case % 4])
    logits = torch.tensor(np.stack(rows)).cuda()
    temperature, top_p = torch.tensor(temps).cuda(), torch.tensor(tops).cuda()
    uniform = torch.tensor(rng.random(12).astype(np.float32)).cuda()
    got = ops.sample(logits, temperature, top_p, uniform).cpu().tolist()
    assert got == ops.sample(logits, temperature, top_p, uniform).cpu().tolist()
    want = ref.sample(logits, temperature, top_p, uniform).cpu().tolist()

    def agree(got, want):
        # The two may differ by how float32 sums of `vocab` weights round (the reference adds them one after the
        # other in falling order, where the small ones at the end are partly lost; here slices are summed apart):
        # the target, a share of the whole mass, moves by that.  In the reference's order the running mass (in
        # float64 here) at the two tokens must lie closer together than such a sum can be off; and a token that
        # weighs far more than that must be drawn by both.
        heavy = 0
        for row, (a, b) in enumerate(zip(got, want)):
            order = np.lexsort((np.arange(vocab), -rows[row].astype(np.float64)))
            weights = np.exp((rows[row][order].astype(np.float64) - float(rows[row].max())) / temps[row])
            running = np.cumsum(weights)
            place = np.empty(vocab, dtype=np.int64)
            place[order] = np.arange(vocab)
            slack = vocab * 2.0 ** -24 * running[-1]
            assert abs(running[place[a]] - running[place[b]]) <= slack, (row, a, b)
            if weights[place[b]] > 10 * slack:
                heavy += 1
                assert a == b, (row, a, b)
        assert heavy >= 2

    agree(got, want)
    assert got[11] == vocab - 1
    # Without any cut in the batch the rounds of the nucleus are not launched at all.
    ones = torch.ones(12).cuda()
    free = ops.sample(logits, temperature, ones, uniform, any_cut=False).cpu().tolist()
    assert free == ops.sample(logits, temperature, ones, uniform, any_cut=True).cpu().tolist()
    agree(free, ref.sample(logits, temperature, ones, uniform).cpu().tolist())


@pytest.mark.parametrize("rows", [1, 3, 4, 7, 16, 19, 32])
@pytest.mark.parametrize("waves", [0, 4, 8, 16])
def test_fused_products_for_every_cut(ops, ref, rows, waves):
    """Weight rows per workgroup (one or two blocks of up to sixteen, the last one partly filled) and waves per
    workgroup are the launcher's choice; every choice gives the same numbers.  Sizes chosen so that waves
    are left without a step, K has a tail, and the last workgroup reaches past the matrix."""
    m, inner, hidden = 7, 328, 104
    residual = rand((m, hidden), torch.float32, 60, 2.0)
    norm_w = rand((hidden,), torch.float32, 61) * 0.1 + 1
    w = rand((2 * inner, hidden), torch.bfloat16, 62, 0.1)
    down = rand((hidden, inner), torch.bfloat16, 63, 0.05)
    bias = rand((hidden,), torch.float32, 64)
    ops.fused_rows, ops.fused_waves = rows, waves
    try:
        got = ops.fused_norm_gated(residual, norm_w, 1e-5, w)
        res_a = residual.clone()
        ops.linear_add(got, down, bias, res_a)
    finally:
        ops.fused_rows, ops.fused_waves = 0, 0
    want = ref.fused_norm_gated(residual, norm_w, 1e-5, w)
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    res_b = residual.clone()
    ref.linear_add(got, down, bias, res_b)
    torch.testing.assert_close(res_a, res_b, **linear_tol(torch.float32, got, down))


def test_read_stream_reads_every_word_once(ops):
    """The bandwidth yardstick leaves the xor of all it read: equal to the xor of the buffer's words, at sizes that
    are and are not multiples of its eight loads a lane, with few and many workgroups."""
    import numpy as np
    for words, workgroups in ((4, 1), (256 * 8 * 4 * 3, 3), (1_000_000, 64), (12_345_680, None)):
        data = torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), dtype=torch.int32, device="cuda")
        parts = ops.read_stream(data, workgroups).cpu().numpy().view(np.uint32)
        assert int(np.bitwise_xor.reduce(parts)) == int(np.bitwise_xor.reduce(data.cpu().numpy().view(np.uint32))), words
