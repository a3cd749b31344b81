"""The plain implementation pinned by what fixes it beside the reference's text: library special
cases, invariants and the vectors the reference's own tests hold.  A real checkpoint is not
available here, so agreement with the reference's float32 fixture of Qwen2.5-0.5B
(tests/fixtures/qwen_last_logits.f32 of the reference) is parity unpinned.

How the parts sit in a layer and in the model (`self_attention`, `decoder_layer`, `hidden_states`,
`greedy_generate`) is pinned by special cases in which the whole thing reduces to a handful of library
routines applied in an order written out here: a sequence of one token (its softmax is 1, so attention is
the value row passed through the output projection), layers whose output matrices are zero (the residual
stream must pass through untouched), and one sub-layer switched off at a time.  Norm scales, biases and
inputs are random and far from 0 and 1, so a norm taken from the wrong tensor or put after the sub-layer
instead of before it, a residual taken after the norm, a feed-forward that reads the layer's input instead
of the attention's sum, or a bias dropped from one of the three projections, each fails one of them."""
import math

import pytest
import torch
import torch.nn.functional as F

from plain import qwen2_plain as plain
from tiny_configs import TINY, random_ids


def test_mask_value_truth_table():
    # qwen-infer/src/model.rs:1389-1399
    inf = -math.inf
    assert plain.mask_value(0, 0, None) == 0.0
    assert plain.mask_value(2, 1, None) == 0.0
    assert plain.mask_value(1, 2, None) == inf
    assert plain.mask_value(5, 0, 4) == inf     # distance 5 with window 4 is blocked
    assert plain.mask_value(5, 1, 4) == 0.0     # distance 4 is kept
    assert plain.mask_value(5, 5, 4) == 0.0
    assert plain.mask_value(5, 6, 4) == inf


def test_rms_norm_is_the_library_routine_and_eps_sits_inside_the_root():
    x = torch.randn(5, 48, dtype=torch.float64)
    w = torch.randn(48, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5))
    ones = torch.ones(48, dtype=torch.float64)
    y = plain.rms_norm(x, ones, 1e-3)
    sq = (x * x).sum(-1)
    torch.testing.assert_close((y * y).sum(-1), 48 * sq / (sq + 48 * 1e-3))
    tiny = torch.full((1, 8), 1e-6, dtype=torch.float64)
    torch.testing.assert_close(plain.rms_norm(tiny, torch.ones(8, dtype=torch.float64), 1e-4),
                               tiny / math.sqrt(1e-12 + 1e-4))


def test_linear_has_its_bias():
    w = torch.randn(7, 5)
    b = torch.randn(7)
    torch.testing.assert_close(plain.linear(torch.zeros(3, 5), w, b), b.expand(3, 7))
    x = torch.randn(3, 5)
    torch.testing.assert_close(plain.linear(x, w, b), F.linear(x, w, b))


def test_rope_pairs_the_halves_and_only_distances_count():
    d = 16
    cos, sin = plain.rope_tables(10000.0, d, 64, torch.float64)
    assert cos.shape == (64, 8)
    x = torch.randn(2, 5, d, dtype=torch.float64)
    torch.testing.assert_close(plain.apply_rope(x, cos[[0] * 5], sin[[0] * 5]), x)   # position 0 is the identity
    rows = torch.tensor([3, 9, 27, 40, 63])
    y = plain.apply_rope(x, cos[rows], sin[rows])
    for i in range(d // 2):                                                          # each (i, i + d/2) pair keeps its length
        torch.testing.assert_close(y[..., i] ** 2 + y[..., i + 8] ** 2, x[..., i] ** 2 + x[..., i + 8] ** 2)
    # Complex form: (x1 + i x2) * exp(i p f), f = theta^(-2i/d).
    freq = torch.tensor([10000.0 ** (-2 * i / d) for i in range(8)], dtype=torch.float64)
    z = torch.complex(x[..., :8], x[..., 8:]) * torch.polar(torch.ones(5, 8, dtype=torch.float64), rows[:, None] * freq)
    torch.testing.assert_close(torch.cat([z.real, z.imag], -1), y)
    # An interleaved pairing would move x[0] into y[1]; the half-split one moves it into y[d/2].
    e0 = torch.zeros(1, 1, d, dtype=torch.float64)
    e0[..., 0] = 1
    out = plain.apply_rope(e0, cos[[7]], sin[[7]])
    assert out[0, 0, 1] == 0 and abs(float(out[0, 0, 8]) - math.sin(7.0)) < 1e-12
    assert abs(float(out[0, 0, 0]) - math.cos(7.0)) < 1e-12                          # the sign: x1 cos - x2 sin
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)
    def score(m, n):
        return float((plain.apply_rope(q, cos[[m]], sin[[m]]) * plain.apply_rope(k, cos[[n]], sin[[n]])).sum())
    assert abs(score(5, 2) - score(45, 42)) < 1e-10 and abs(score(5, 2) - score(2, 5)) > 1e-6


def test_attention_is_the_library_routine_without_rotation():
    n_q, n_kv, seq, d = 6, 2, 11, 8
    q, k, v = (torch.randn(n, seq, d, dtype=torch.float64) for n in (n_q, n_kv, n_kv))
    mask = plain.attention_mask(range(seq), range(seq), None, torch.float64)
    ours = plain.attend(q, plain.repeat_kv(k, 3), plain.repeat_kv(v, 3), mask)
    want = F.scaled_dot_product_attention(q[None], k.repeat_interleave(3, 0)[None], v.repeat_interleave(3, 0)[None],
                                          is_causal=True, scale=1 / math.sqrt(d))[0]
    torch.testing.assert_close(ours, want)
    # one head, one key: the output is the value row
    torch.testing.assert_close(plain.attend(q[:1, :1], k[:1, :1], v[:1, :1], torch.zeros(1, 1, dtype=torch.float64)), v[:1, :1])
    probs = torch.softmax(q @ plain.repeat_kv(k, 3).transpose(-1, -2) / math.sqrt(d) + mask, -1)
    torch.testing.assert_close(probs.sum(-1), torch.ones(n_q, seq, dtype=torch.float64))
    assert torch.equal(plain.repeat_kv(k, 3), k.repeat_interleave(3, dim=0))


def test_swiglu():
    z = torch.randn(4, 6)
    torch.testing.assert_close(plain.silu(z), F.silu(z))
    assert float(plain.silu(torch.zeros(1))) == 0.0
    t = {"m.gate_proj.weight": torch.randn(10, 6), "m.up_proj.weight": torch.randn(10, 6),
         "m.down_proj.weight": torch.randn(6, 10)}
    want = F.linear(F.silu(F.linear(z, t["m.gate_proj.weight"])) * F.linear(z, t["m.up_proj.weight"]), t["m.down_proj.weight"])
    torch.testing.assert_close(plain.mlp(z, t, "m"), want)


@pytest.fixture(scope="module")
def loaded(model_folders):
    return {name: plain.load_folder(model_folders[name], torch.float64) for name in TINY}


@pytest.mark.parametrize("name", list(TINY))
def test_later_tokens_do_not_change_earlier_logits(loaded, name):
    cfg, tensors = loaded[name]
    ids = random_ids(cfg["vocab_size"], 30, 1)
    base = plain.all_logits(cfg, tensors, ids)
    changed = list(ids)
    changed[20] = (changed[20] + 1) % cfg["vocab_size"]
    other = plain.all_logits(cfg, tensors, changed)
    torch.testing.assert_close(other[:20], base[:20], rtol=0, atol=0)
    assert float((other[20:] - base[20:]).abs().max()) > 1e-6
    torch.testing.assert_close(plain.all_logits(cfg, tensors, ids[:12]), base[:12], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_shift_of_all_positions_changes_nothing(loaded, name):
    # Only distances enter the scores (rotary), and the mask is causal: moving the whole sequence is invisible.
    cfg, tensors = loaded[name]
    ids = random_ids(cfg["vocab_size"], 20, 2)
    torch.testing.assert_close(plain.all_logits(cfg, tensors, ids, 0), plain.all_logits(cfg, tensors, ids, 37),
                               rtol=1e-9, atol=1e-9)
    with pytest.raises(ValueError):
        plain.all_logits(cfg, tensors, ids, cfg["max_position_embeddings"] - 5)


def test_window_edge(loaded):
    # Config C: layers 1..3 see keys at distance <= 21.  With one windowed layer alone on top of embeddings,
    # a token at distance 22 would be invisible; here the full layer 0 still passes information on, so the
    # pin is on the attention part: the key at distance 21 counts, the one at 22 does not.
    seq, d = 30, 8
    q, k, v = (torch.randn(1, seq, d, dtype=torch.float64) for _ in range(3))
    mask = plain.attention_mask(range(seq), range(seq), 21, torch.float64)
    base = plain.attend(q, k, v, mask)[0, 29]
    v2 = v.clone(); v2[0, 7] += 1.0                  # distance 22 from the last query
    torch.testing.assert_close(plain.attend(q, k, v2, mask)[0, 29], base, rtol=0, atol=0)
    v3 = v.clone(); v3[0, 8] += 1.0                  # distance 21
    assert float((plain.attend(q, k, v3, mask)[0, 29] - base).abs().max()) > 1e-9
    cfg, _ = loaded["C"]
    assert [plain.window_for_layer(cfg, i) for i in range(4)] == [None, 21, 21, 21]


def test_zero_weights_give_equal_finite_logits_and_id_zero():
    # qwen-infer/src/model.rs:1420-1432
    cfg = dict(TINY["A"][0], num_hidden_layers=1)
    shapes = {"model.embed_tokens.weight": (256, 64), "model.norm.weight": (64,)}
    p = "model.layers.0"
    shapes.update({f"{p}.self_attn.q_proj.weight": (64, 64), f"{p}.self_attn.q_proj.bias": (64,),
                   f"{p}.self_attn.k_proj.weight": (32, 64), f"{p}.self_attn.k_proj.bias": (32,),
                   f"{p}.self_attn.v_proj.weight": (32, 64), f"{p}.self_attn.v_proj.bias": (32,),
                   f"{p}.self_attn.o_proj.weight": (64, 64), f"{p}.mlp.gate_proj.weight": (128, 64),
                   f"{p}.mlp.up_proj.weight": (128, 64), f"{p}.mlp.down_proj.weight": (64, 128),
                   f"{p}.input_layernorm.weight": (64,), f"{p}.post_attention_layernorm.weight": (64,)})
    tensors = {k: torch.zeros(s) for k, s in shapes.items()}
    logits = plain.all_logits(cfg, tensors, [1, 2, 3])[-1]
    assert logits.shape == (256,) and bool(torch.isfinite(logits).all()) and float(logits.abs().max()) == 0
    assert plain.greedy_token(logits) == 0


def test_untied_head_is_used(loaded):
    cfg, tensors = loaded["B"]
    ids = random_ids(cfg["vocab_size"], 6, 3)
    hidden = plain.hidden_states(cfg, tensors, ids)
    torch.testing.assert_close(plain.all_logits(cfg, tensors, ids), hidden @ tensors["lm_head.weight"].t())
    cfg_a, tensors_a = loaded["A"]
    ids_a = random_ids(cfg_a["vocab_size"], 4, 3)
    hidden = plain.hidden_states(cfg_a, tensors_a, ids_a)
    torch.testing.assert_close(plain.all_logits(cfg_a, tensors_a, ids_a), hidden @ tensors_a["model.embed_tokens.weight"].t())


def test_plain_sampling_vectors():
    # qwen-infer/src/sample.rs:188-230
    logits = [0.2, 1.5, 1.5, -3.0, 0.0]
    assert plain.greedy_token(logits) == 1
    for u in (0.0, 0.3, 0.99):
        assert plain.sample_token(logits, 0.0, 1.0, u) == 1
        assert plain.sample_token(logits, 0.0, 1.5, u) == 1
    peaked = [0.0, 2.0, 0.5, -1.0]
    for u in (0.0, 0.5, 0.999):
        assert plain.sample_token(peaked, 1.0, 1e-6, u) == 1
        assert plain.sample_token(peaked, 0.7, 0.0, u) == 1
        assert plain.sample_token(peaked, 0.8, 1.0, u) == plain.sample_token(peaked, 0.8, 4.0, u)
    flat = [0.0] * 8
    assert len({plain.sample_token(flat, 1.0, 1.0, u / 40) for u in range(40)}) == 8
    with pytest.raises(ValueError):
        plain.sample_token([], 1.0, 1.0, 0.5)
    with pytest.raises(ValueError):
        plain.sample_token([1.0], -0.1, 1.0, 0.5)


# ---- how the parts sit together -----------------------------------------------------------------------
def _layer_tensors(cfg, seed, dtype=torch.float64):
    """Random tensors of one decoder layer (index 0) with norm scales and biases far from 1 and 0."""
    gen = torch.Generator().manual_seed(seed)
    hidden, n_q, n_kv = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d, inner = hidden // n_q, cfg["intermediate_size"]
    draw = lambda *shape, scale=0.3: torch.randn(*shape, generator=gen, dtype=dtype) * scale
    p = "model.layers.0"
    return {
        f"{p}.input_layernorm.weight": 1 + draw(hidden, scale=0.5),
        f"{p}.post_attention_layernorm.weight": 1 + draw(hidden, scale=0.5),
        f"{p}.self_attn.q_proj.weight": draw(n_q * d, hidden), f"{p}.self_attn.q_proj.bias": draw(n_q * d, scale=1.0),
        f"{p}.self_attn.k_proj.weight": draw(n_kv * d, hidden), f"{p}.self_attn.k_proj.bias": draw(n_kv * d, scale=1.0),
        f"{p}.self_attn.v_proj.weight": draw(n_kv * d, hidden), f"{p}.self_attn.v_proj.bias": draw(n_kv * d, scale=1.0),
        f"{p}.self_attn.o_proj.weight": draw(hidden, n_q * d),
        f"{p}.mlp.gate_proj.weight": draw(inner, hidden), f"{p}.mlp.up_proj.weight": draw(inner, hidden),
        f"{p}.mlp.down_proj.weight": draw(hidden, inner),
    }


_LAYER_CFG = {"hidden_size": 24, "num_attention_heads": 6, "num_key_value_heads": 2, "intermediate_size": 40,
              "rms_norm_eps": 1e-3, "rope_theta": 100.0, "use_sliding_window": False, "max_position_embeddings": 64}


def _library_mlp(t, z):
    p = "model.layers.0.mlp"
    return F.linear(F.silu(F.linear(z, t[f"{p}.gate_proj.weight"])) * F.linear(z, t[f"{p}.up_proj.weight"]),
                    t[f"{p}.down_proj.weight"])


def _library_attention_of_one_token(t, z, cfg):
    """A sequence of one token attends to itself with weight 1 whatever its query and key are: every query head
    gets the value row of its kv head (head h of the kv heads serves query heads h*r..(h+1)*r-1,
    qwen-infer/src/model.rs:571-580), then the output projection, which has no bias (model.rs:272)."""
    p = "model.layers.0.self_attn"
    n_q, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg["hidden_size"] // n_q
    v = F.linear(z, t[f"{p}.v_proj.weight"], t[f"{p}.v_proj.bias"]).reshape(n_kv, d)
    return F.linear(v.repeat_interleave(n_q // n_kv, dim=0).reshape(1, n_q * d), t[f"{p}.o_proj.weight"])


def test_a_layer_of_one_token_is_five_library_calls_in_this_order():
    # qwen-infer/src/model.rs:615-622: r = x; a = attn(norm1(x)); h = a + r; m = mlp(norm2(h)); out = m + h.
    cfg, hidden = _LAYER_CFG, _LAYER_CFG["hidden_size"]
    t = _layer_tensors(cfg, 1)
    cos, sin = plain.rope_tables(cfg["rope_theta"], hidden // cfg["num_attention_heads"], 64, torch.float64)
    x = torch.randn(1, hidden, dtype=torch.float64) * 2
    for position in (0, 17):
        got = plain.decoder_layer(x, cfg, t, 0, cos, sin, [position])
        n1 = F.rms_norm(x, (hidden,), t["model.layers.0.input_layernorm.weight"], cfg["rms_norm_eps"])
        h = x + _library_attention_of_one_token(t, n1, cfg)
        n2 = F.rms_norm(h, (hidden,), t["model.layers.0.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
        want = h + _library_mlp(t, n2)
        torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    # The plausible mistakes all give something else (so the comparison above can tell them apart):
    swapped = dict(t)
    swapped["model.layers.0.input_layernorm.weight"], swapped["model.layers.0.post_attention_layernorm.weight"] = \
        t["model.layers.0.post_attention_layernorm.weight"], t["model.layers.0.input_layernorm.weight"]
    assert float((plain.decoder_layer(x, cfg, swapped, 0, cos, sin, [0]) - want).abs().max()) > 1e-3
    parallel = h + _library_mlp(t, F.rms_norm(x, (hidden,), t["model.layers.0.post_attention_layernorm.weight"],
                                              cfg["rms_norm_eps"]))       # feed-forward reading the layer's input
    post_norm = F.rms_norm(h, (hidden,), t["model.layers.0.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    post_norm = post_norm + _library_mlp(t, post_norm)                    # residual taken after the norm
    no_v_bias = dict(t, **{"model.layers.0.self_attn.v_proj.bias": torch.zeros_like(t["model.layers.0.self_attn.v_proj.bias"])})
    for other in (parallel, post_norm, plain.decoder_layer(x, cfg, no_v_bias, 0, cos, sin, [0])):
        assert float((other - want).abs().max()) > 1e-3


def test_attention_of_a_sequence_is_the_library_routine_on_biased_rotated_projections():
    # qwen-infer/src/model.rs:279-328: bias on q, k and v, rotation of q and k only, kv heads repeated, no
    # bias on the output projection.  (Rotation, mask and head repetition are pinned on their own above.)
    cfg, hidden = _LAYER_CFG, _LAYER_CFG["hidden_size"]
    n_q, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d, seq = hidden // n_q, 9
    t = _layer_tensors(cfg, 2)
    p = "model.layers.0.self_attn"
    cos, sin = plain.rope_tables(cfg["rope_theta"], d, 64, torch.float64)
    x = torch.randn(seq, hidden, dtype=torch.float64)
    positions = list(range(5, 5 + seq))
    got = plain.self_attention(x, t, p, n_q, n_kv, d, cos, sin, positions, None)

    def heads(name, n):
        return F.linear(x, t[f"{p}.{name}.weight"], t[f"{p}.{name}.bias"]).reshape(seq, n, d).transpose(0, 1)

    def rotate(y):          # the complex form of the half-split rotation: (y1 + i y2) * e^{i angle}
        half = d // 2
        angle = torch.tensor(positions, dtype=torch.float64)[:, None] * \
            torch.tensor([cfg["rope_theta"] ** (-2 * i / d) for i in range(half)], dtype=torch.float64)[None, :]
        z = torch.complex(y[..., :half], y[..., half:]) * torch.polar(torch.ones_like(angle), angle)
        return torch.cat([z.real, z.imag], dim=-1)

    q, k, v = rotate(heads("q_proj", n_q)), rotate(heads("k_proj", n_kv)), heads("v_proj", n_kv)
    k, v = k.repeat_interleave(n_q // n_kv, dim=0), v.repeat_interleave(n_q // n_kv, dim=0)
    mixed = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True, scale=1 / math.sqrt(d))[0]
    want = F.linear(mixed.transpose(0, 1).reshape(seq, n_q * d), t[f"{p}.o_proj.weight"])
    torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-10)
    for name in ("q_proj", "k_proj", "v_proj"):                          # each of the three biases counts
        dropped = dict(t, **{f"{p}.{name}.bias": torch.zeros_like(t[f"{p}.{name}.bias"])})
        other = plain.self_attention(x, dropped, p, n_q, n_kv, d, cos, sin, positions, None)
        assert float((other - want).abs().max()) > 1e-3, name


def test_layers_with_zero_output_matrices_pass_the_stream_through_and_the_final_norm_comes_before_the_head(loaded):
    # qwen-infer/src/model.rs:832-848 and 1210-1242: embedding, layers, `model.norm`, head.  With every
    # o_proj and down_proj zero each layer adds nothing, whatever its norms hold (a norm applied to the stream
    # itself instead of to the sub-layer's input would show), and the logits are the head of the final norm
    # of the embedding rows.
    for name in ("A", "B"):
        cfg, tensors = loaded[name]
        muted = {key: (torch.zeros_like(value) if key.endswith(("o_proj.weight", "down_proj.weight")) else value)
                 for key, value in tensors.items()}
        ids = random_ids(cfg["vocab_size"], 11, 5)
        embedded = tensors["model.embed_tokens.weight"][torch.tensor(ids)]
        normed = F.rms_norm(embedded, (cfg["hidden_size"],), tensors["model.norm.weight"], cfg["rms_norm_eps"])
        head = tensors["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else tensors["lm_head.weight"]
        torch.testing.assert_close(plain.all_logits(cfg, muted, ids), F.linear(normed, head), rtol=1e-12, atol=1e-12)
        assert float((tensors["model.norm.weight"] - 1).abs().max()) > 0.1           # the fixture's scales are not 1
        # ... and the full model is not that (the layers do something).
        assert float((plain.all_logits(cfg, tensors, ids) - F.linear(normed, head)).abs().max()) > 1e-3


def test_one_sub_layer_at_a_time(loaded):
    """The whole model A with every feed-forward muted, then with every attention muted: what is left is a
    chain of library calls per token (muted attention: rows do not see each other at all)."""
    cfg, tensors = loaded["A"]
    hidden, eps, layers = cfg["hidden_size"], cfg["rms_norm_eps"], cfg["num_hidden_layers"]
    ids = random_ids(cfg["vocab_size"], 7, 6)
    no_attention = {k: (torch.zeros_like(v) if k.endswith("o_proj.weight") else v) for k, v in tensors.items()}
    x = tensors["model.embed_tokens.weight"][torch.tensor(ids)]
    for i in range(layers):
        p = f"model.layers.{i}"
        z = F.rms_norm(x, (hidden,), tensors[f"{p}.post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(z, tensors[f"{p}.mlp.gate_proj.weight"])) *
                         F.linear(z, tensors[f"{p}.mlp.up_proj.weight"]), tensors[f"{p}.mlp.down_proj.weight"])
    want = F.linear(F.rms_norm(x, (hidden,), tensors["model.norm.weight"], eps), tensors["model.embed_tokens.weight"])
    torch.testing.assert_close(plain.all_logits(cfg, no_attention, ids), want, rtol=1e-11, atol=1e-11)
    # One token, feed-forwards muted: attention of a single token is its value row through the output projection.
    no_mlp = {k: (torch.zeros_like(v) if k.endswith("down_proj.weight") else v) for k, v in tensors.items()}
    n_q, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = hidden // n_q
    x = tensors["model.embed_tokens.weight"][torch.tensor(ids[:1])]
    for i in range(layers):
        p = f"model.layers.{i}"
        z = F.rms_norm(x, (hidden,), tensors[f"{p}.input_layernorm.weight"], eps)
        v = F.linear(z, tensors[f"{p}.self_attn.v_proj.weight"], tensors[f"{p}.self_attn.v_proj.bias"]).reshape(n_kv, d)
        x = x + F.linear(v.repeat_interleave(n_q // n_kv, dim=0).reshape(1, n_q * d), tensors[f"{p}.self_attn.o_proj.weight"])
    want = F.linear(F.rms_norm(x, (hidden,), tensors["model.norm.weight"], eps), tensors["model.embed_tokens.weight"])
    torch.testing.assert_close(plain.all_logits(cfg, no_mlp, ids[:1]), want, rtol=1e-11, atol=1e-11)


def test_greedy_generation_appends_the_first_maximum_of_the_last_row(loaded):
    # qwen-infer/src/lib.rs:116-130
    cfg, tensors = loaded["B"]
    prompt = random_ids(cfg["vocab_size"], 6, 8)
    got = plain.greedy_generate(cfg, tensors, prompt, 4)
    ids = list(prompt)
    for token in got:
        row = plain.all_logits(cfg, tensors, ids)[-1]
        assert token == int(torch.argmax(row)) and float(row[token]) == float(row.max())
        ids.append(token)
    assert len(got) == 4
