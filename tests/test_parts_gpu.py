"""Each part of a layer alone against the plain implementation, and parts defined here, outside the package:
a mixer with state of its own, a model whose layers have different mixers, a schedule that runs a layer twice
on one cache."""
import dataclasses
import math

import pytest
import torch

from plain import qwen2_plain as plain
from tiny_configs import random_ids

pytestmark = pytest.mark.gpu

TOL = {torch.float32: dict(rtol=1e-4, atol=2e-5), torch.bfloat16: dict(rtol=3e-2, atol=3e-2)}


def close(got, want, dtype):
    """float32: elementwise.  bfloat16: every rounding is 2^-9 relative to the values around it, and a few of
    them pile up, so the bound is relative to the largest value of the result (2 %), not to each element."""
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, **TOL[dtype])
    else:
        err, scale = float((got - want).abs().max()), float(want.abs().max())
        assert err <= 2e-2 * scale, f"max abs error {err} against values up to {scale}"


def runtime(dtype):
    from tokenizer_amd.kernels import get_ops
    from tokenizer_amd.parts import Runtime
    return Runtime(dtype, torch.device("cuda:0"), get_ops())


def context_for(needs, lengths, dtype, page_size=16, chunks=None):
    """A cache manager, pools and the step context of whole sequences of the given lengths."""
    from tokenizer_amd.cache import CacheManager, CachePools
    from tokenizer_amd.engine.batch import StepEntry, build_context
    manager = CacheManager(needs, num_pages=sum(-(-n // page_size) for n in lengths) + 2, page_size=page_size,
                           max_requests=len(lengths))
    pools = CachePools(manager, needs, dtype, "cuda:0")
    pools.poison()
    entries = []
    for rid, n in enumerate(lengths):
        manager.add_request(rid)
        assert manager.reserve(rid, n)
        entries.append(StepEntry(rid, [0] * n, []))
    return manager, pools, build_context(entries, manager, "cuda:0")


def rand(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from tokenizer_amd.parts import NORMS, NormSpec
    spec = NormSpec("rmsnorm", 72, 3e-5)
    weight = rand((72,), 1) * 0.1 + 1
    norm = NORMS.get("rmsnorm")(spec, {"weight": weight.cuda()}, runtime(dtype))
    residual, delta = rand((9, 72), 2, 3.0), rand((9, 72), 3).to(dtype)
    res = residual.cuda().clone()
    out = norm.apply(res, delta.cuda())
    want_res = residual + delta.float()
    torch.testing.assert_close(res.cpu(), want_res, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.float().cpu(), plain.rms_norm(want_res, weight, 3e-5), **TOL[dtype])
    rows = torch.tensor([8, 2], dtype=torch.int32).cuda()
    out = norm.apply(res, None, rows=rows)
    torch.testing.assert_close(out.float().cpu(), plain.rms_norm(want_res[[8, 2]], weight, 3e-5), **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_position_part_rotates_and_stores(dtype):
    from tokenizer_amd.parts import POSITIONS, CacheNeed, LayerCache, PositionSpec
    n_q, n_kv, d = 3, 1, 32
    need = CacheNeed("full", n_kv, d)
    manager, pools, ctx = context_for([need], [21, 5], dtype)
    k_pages, v_pages = pools.layer_pages(0)
    cache = LayerCache(group=0, k_pages=k_pages, v_pages=v_pages)
    rope = POSITIONS.get("rope_half_split")(PositionSpec("rope_half_split", d, 1e6, 64), runtime(dtype))
    qkv = rand((26, (n_q + 2 * n_kv) * d), 4).to(dtype)
    work = qkv.cuda().clone()
    rope.encode_and_store(work, None, n_q, n_kv, d, ctx, cache)
    cos, sin = plain.rope_tables(1e6, d, 64)
    positions = list(range(21)) + list(range(5))
    heads = qkv.float().reshape(26, n_q + 2 * n_kv, d).transpose(0, 1)
    want = plain.apply_rope(heads[:n_q + n_kv], cos[positions], sin[positions])
    got = work.float().cpu().reshape(26, n_q + 2 * n_kv, d).transpose(0, 1)
    torch.testing.assert_close(got[:n_q + n_kv], want, **TOL[dtype])
    torch.testing.assert_close(got[n_q + n_kv:], heads[n_q + n_kv:], rtol=0, atol=0)     # values are not rotated
    # Request 0's token 17 sits in its second page at offset 1: keys row-wise, values transposed.
    page = manager.table(0, 0)[1]
    torch.testing.assert_close(k_pages[page, 0, 1].float().cpu(), want[n_q, 17], **TOL[dtype])
    torch.testing.assert_close(v_pages[page, 0, :, 1].float().cpu(), heads[n_q + n_kv, 17], rtol=0, atol=0)
    # "none" leaves the heads as they are and still stores them.
    none = POSITIONS.get("none")(PositionSpec("none"), runtime(dtype))
    work = qkv.cuda().clone()
    none.encode_and_store(work, None, n_q, n_kv, d, ctx, cache)
    torch.testing.assert_close(work.float().cpu(), qkv.float(), rtol=0, atol=0)
    torch.testing.assert_close(k_pages[page, 0, 1].float().cpu(), heads[n_q, 17], rtol=0, atol=0)


def attention_tensors(n_q, n_kv, d, hidden, seed):
    names = {"q_proj.weight": (n_q * d, hidden), "k_proj.weight": (n_kv * d, hidden), "v_proj.weight": (n_kv * d, hidden),
             "o_proj.weight": (hidden, n_q * d), "q_proj.bias": (n_q * d,), "k_proj.bias": (n_kv * d,),
             "v_proj.bias": (n_kv * d,)}
    return {name: rand(shape, seed + i, 0.2).to(torch.bfloat16).float() for i, (name, shape) in enumerate(names.items())}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geometry", [(6, 2, 16, 40, None), (4, 4, 32, 72, 9), (14, 2, 64, 96, None)])
def test_attention_mixer_alone(dtype, geometry):
    from tokenizer_amd.parts import MIXERS, LayerCache, MixerSpec, PositionSpec
    n_q, n_kv, d, hidden, window = geometry
    spec = MixerSpec("gqa_attention", hidden, n_q, n_kv, d, qkv_bias=True, window=window,
                     position=PositionSpec("rope_half_split", d, 10000.0, 128))
    mixer_cls = MIXERS.get("gqa_attention")
    tensors = attention_tensors(n_q, n_kv, d, hidden, 10)
    assert set(mixer_cls.tensor_specs(spec)) == set(tensors)
    assert {k: v.shape for k, v in mixer_cls.tensor_specs(spec).items()} == {k: tuple(v.shape) for k, v in tensors.items()}
    need = mixer_cls.cache_need(spec)
    assert need.kind == ("window" if window else "full") and (need.n_kv_heads, need.head_dim) == (n_kv, d)
    held = {k: (v.to(dtype) if v.dim() == 2 else v).cuda() for k, v in tensors.items()}
    mixer = mixer_cls(spec, held, runtime(dtype))
    lengths = [37, 16, 3]
    manager, pools, ctx = context_for([need], lengths, dtype)
    k_pages, v_pages = pools.layer_pages(0)
    x = rand((sum(lengths), hidden), 20).to(dtype)
    out = mixer.forward(x.cuda(), ctx, LayerCache(group=0, k_pages=k_pages, v_pages=v_pages)).float().cpu()
    cos, sin = plain.rope_tables(10000.0, d, 128)
    named = {f"a.{k}": v for k, v in tensors.items()}
    at = 0
    for n in lengths:
        want = plain.self_attention(x[at:at + n].float(), named, "a", n_q, n_kv, d, cos, sin, list(range(n)), window)
        close(out[at:at + n], want, dtype)
        at += n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [5, 130])
def test_feed_forward_alone(dtype, rows):
    from tokenizer_amd.parts import FEED_FORWARDS, FeedForwardSpec
    spec = FeedForwardSpec("gated_dense", 72, 136, "silu")
    tensors = {"gate_proj.weight": rand((136, 72), 1, 0.2), "up_proj.weight": rand((136, 72), 2, 0.2),
               "down_proj.weight": rand((72, 136), 3, 0.2)}
    tensors = {k: v.to(torch.bfloat16).float() for k, v in tensors.items()}
    part = FEED_FORWARDS.get("gated_dense")(spec, {k: v.to(dtype).cuda() for k, v in tensors.items()}, runtime(dtype))
    x = rand((rows, 72), 4).to(dtype)
    out = part.forward(x.cuda(), None).float().cpu()
    want = plain.mlp(x.float(), {f"m.{k}": v for k, v in tensors.items()}, "m")
    close(out, want, dtype)
    with pytest.raises(ValueError):
        FEED_FORWARDS.get("gated_dense")(FeedForwardSpec("gated_dense", 72, 136, "gelu"), {}, runtime(dtype))


@pytest.mark.parametrize("hidden", [1024, 2304])
def test_wide_models_take_the_norm_out_of_the_fused_decode_products(hidden):
    """Up to a width the fused decode products normalise their rows themselves; wider models run the norm's own
    kernel once and hand the products normalised rows.  The numbers agree either way."""
    from tokenizer_amd.parts import FEED_FORWARDS, NORMS, FeedForwardSpec, NormSpec
    dtype, rows, inner = torch.bfloat16, 6, 48
    rt = runtime(dtype)
    assert rt.ops.can_fuse_decode(rows, dtype, hidden) and rt.ops.fold_norm(hidden) == (hidden == 1024)
    tensors = {"gate_proj.weight": rand((inner, hidden), 1, 0.05), "up_proj.weight": rand((inner, hidden), 2, 0.05),
               "down_proj.weight": rand((hidden, inner), 3, 0.2)}
    tensors = {k: v.to(dtype).float() for k, v in tensors.items()}
    part = FEED_FORWARDS.get("gated_dense")(FeedForwardSpec("gated_dense", hidden, inner, "silu"),
                                            {k: v.to(dtype).cuda() for k, v in tensors.items()}, rt)
    norm = NORMS.get("rmsnorm")(NormSpec("rmsnorm", hidden, 1e-6), {"weight": torch.ones(hidden).cuda()}, rt)
    residual = rand((rows, hidden), 4).float()
    on_device = residual.cuda().clone()
    assert part.forward_normed(on_device, None, norm, None) is None      # fused: added into the stream in place
    want = residual + plain.mlp(plain.rms_norm(residual, torch.ones(hidden), 1e-6), {f"m.{k}": v for k, v in tensors.items()}, "m")
    close(on_device.cpu(), want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_alone(dtype):
    # One pre-norm block with its own sizes: norm, attention, add, norm, feed-forward, add (the last add is
    # left to the next norm, so the block hands back the stream and what is still to be added).
    from tokenizer_amd.parts import as_tensor
    from tokenizer_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, FeedForwardSpec, LayerCache, MixerSpec,
                                     NormSpec, PositionSpec)
    n_q, n_kv, d, hidden, inner = 3, 1, 32, 96, 136
    rt = runtime(dtype)
    cfg = {"rms_norm_eps": 2e-5, "num_attention_heads": n_q, "num_key_value_heads": n_kv, "hidden_size": hidden}
    t = {f"model.layers.0.self_attn.{k}": v for k, v in attention_tensors(n_q, n_kv, d, hidden, 30).items()}
    for name, shape, seed in (("mlp.gate_proj.weight", (inner, hidden), 40), ("mlp.up_proj.weight", (inner, hidden), 41),
                              ("mlp.down_proj.weight", (hidden, inner), 42)):
        t[f"model.layers.0.{name}"] = rand(shape, seed, 0.1).to(torch.bfloat16).float()
    t["model.layers.0.input_layernorm.weight"] = rand((hidden,), 43) * 0.1 + 1
    t["model.layers.0.post_attention_layernorm.weight"] = rand((hidden,), 44) * 0.1 + 1

    def held(prefix):
        return {k[len(prefix) + 1:]: (v.to(dtype) if v.dim() == 2 else v.float()).cuda() for k, v in t.items()
                if k.startswith(prefix + ".")}
    mixer_spec = MixerSpec("gqa_attention", hidden, n_q, n_kv, d, qkv_bias=True,
                           position=PositionSpec("rope_half_split", d, 10000.0, 64))
    norm_spec = NormSpec("rmsnorm", hidden, 2e-5)
    block = BLOCKS.get("pre_norm")(
        NORMS.get("rmsnorm")(norm_spec, held("model.layers.0.input_layernorm"), rt),
        MIXERS.get("gqa_attention")(mixer_spec, held("model.layers.0.self_attn"), rt),
        NORMS.get("rmsnorm")(norm_spec, held("model.layers.0.post_attention_layernorm"), rt),
        FEED_FORWARDS.get("gated_dense")(FeedForwardSpec("gated_dense", hidden, inner), held("model.layers.0.mlp"), rt))
    for lengths in ([29, 7], [1, 1, 1]):           # the second batch is small enough for the fused decode kernels
        need = MIXERS.get("gqa_attention").cache_need(mixer_spec)
        manager, pools, ctx = context_for([need], lengths, dtype)
        k_pages, v_pages = pools.layer_pages(0)
        x = rand((sum(lengths), hidden), 45)
        residual = x.cuda().clone()
        delta = block.forward(residual, None, ctx, LayerCache(group=0, k_pages=k_pages, v_pages=v_pages))
        got = residual.cpu() + (0 if delta is None else as_tensor(delta).float().cpu())
        cos, sin = plain.rope_tables(10000.0, d, 64)
        at = 0
        for n in lengths:
            want = plain.decoder_layer(x[at:at + n], cfg, t, 0, cos, sin, list(range(n)))
            close(got[at:at + n], want, dtype)
            at += n


# ------------------------------------------------------------------------------------------------
# Parts and an architecture defined here, not in the package.
def register_toys():
    from tokenizer_amd.config import get_architecture, register_architecture, registered_architectures
    from tokenizer_amd.config.base import ModelConfig
    if "ToyMixedForCausalLM" in registered_architectures():
        return get_architecture("ToyMixedForCausalLM").config_class
    from tokenizer_amd.parts import (MIXERS, CacheNeed, FeedForwardSpec, LayerSpec, Mixer, MixerSpec, ModelSpec,
                                     NormSpec, PositionSpec, ScheduleEntry, TensorSpec)

    if "running_mean" not in MIXERS.kinds():
        @MIXERS.register("running_mean")
        class RunningMean(Mixer):
            """y_t = W * mean(x_0 .. x_t): the sum so far is the request's state, one slot of fixed size."""

            def __init__(self, spec, tensors, rt):
                self.hidden, self.rt, self.w = spec.hidden_size, rt, tensors["mix.weight"]

            @staticmethod
            def tensor_specs(spec):
                return {"mix.weight": TensorSpec((spec.hidden_size, spec.hidden_size), std=0.1)}

            @staticmethod
            def cache_need(spec):
                return CacheNeed(kind="none", state_shape=(spec.hidden_size,), state_dtype="float32")

            def forward(self, x, ctx, cache):
                means = torch.empty(x.shape, dtype=torch.float32, device=x.device)
                for info in ctx.entries:
                    rows = slice(info.q_start, info.q_start + info.q_len)
                    state = cache.state[info.slot]
                    if info.position == 0:
                        state.zero_()                      # a new request starts from nothing, whoever had the slot
                    sums = torch.cumsum(x[rows].float(), dim=0) + state
                    counts = torch.arange(info.position + 1, info.position + info.q_len + 1, device=x.device)
                    means[rows] = sums / counts[:, None]
                    state.copy_(sums[-1])
                return self.rt.ops.linear(means.to(x.dtype), self.w)

    @dataclasses.dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        vocab_size: int
        hidden_size: int
        heads: int
        inner: int
        twice: bool = False

    def toy_spec(cfg):
        d = cfg.hidden_size // cfg.heads
        norm = NormSpec("rmsnorm", cfg.hidden_size, 1e-5)
        ff = FeedForwardSpec("gated_dense", cfg.hidden_size, cfg.inner, "silu")
        mixers = [MixerSpec("running_mean", cfg.hidden_size),
                  MixerSpec("gqa_attention", cfg.hidden_size, cfg.heads, cfg.heads, d, qkv_bias=False,
                            position=PositionSpec("rope_half_split", d, 10000.0, 256))]
        layers = tuple(LayerSpec("pre_norm", m, ff, norm, norm, f"l.{i}.mix", f"l.{i}.ff", f"l.{i}.n1", f"l.{i}.n2")
                       for i, m in enumerate(mixers))
        # `twice`: the attention layer runs a second time and then reads the keys and values of its first run.
        schedule = (ScheduleEntry(0), ScheduleEntry(1)) + ((ScheduleEntry(1, cache_of=1),) if cfg.twice else ())
        return ModelSpec("ToyMixedForCausalLM", cfg.vocab_size, cfg.hidden_size, 256, "emb.weight", layers, schedule,
                         norm, "final", tied_head=True, head_name="head.weight")

    register_architecture("ToyMixedForCausalLM", ToyConfig, toy_spec)
    return ToyConfig


def toy_plain_logits(tensors, ids, heads, twice):
    """The toy model on whole sequences with the plain parts."""
    t = {k: v.float() for k, v in tensors.items()}
    hidden = t["emb.weight"].shape[1]
    d = hidden // heads
    x = t["emb.weight"][ids]
    n = len(ids)

    def ff(x, i):
        h = plain.rms_norm(x, t[f"l.{i}.n2.weight"], 1e-5)
        return x + plain.mlp(h, {f"m.{k.split('.ff.')[1]}": v for k, v in t.items() if f"l.{i}.ff." in k}, "m")

    h = plain.rms_norm(x, t["l.0.n1.weight"], 1e-5)
    means = torch.cumsum(h, 0) / torch.arange(1, n + 1)[:, None]
    x = ff(x + means @ t["l.0.mix.mix.weight"].t(), 0)
    cos, sin = plain.rope_tables(10000.0, d, 256)
    pos = list(range(n))

    def heads_of(h, name, rotate):
        v = (h @ t[f"l.1.mix.{name}.weight"].t()).reshape(n, heads, d).transpose(0, 1)
        return plain.apply_rope(v, cos[pos], sin[pos]) if rotate else v

    mask = plain.attention_mask(pos, pos, None)
    h = plain.rms_norm(x, t["l.1.n1.weight"], 1e-5)
    k, v = heads_of(h, "k_proj", True), heads_of(h, "v_proj", False)
    mixed = plain.attend(heads_of(h, "q_proj", True), k, v, mask).transpose(0, 1).reshape(n, hidden)
    x = ff(x + mixed @ t["l.1.mix.o_proj.weight"].t(), 1)
    if twice:
        h = plain.rms_norm(x, t["l.1.n1.weight"], 1e-5)
        mixed = plain.attend(heads_of(h, "q_proj", True), k, v, mask).transpose(0, 1).reshape(n, hidden)   # first run's k, v
        x = ff(x + mixed @ t["l.1.mix.o_proj.weight"].t(), 1)
    return plain.rms_norm(x, t["final.weight"], 1e-5) @ t["emb.weight"].t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("twice", [False, True])
def test_toy_architecture_registers_builds_and_steps(tmp_path, dtype, twice):
    import trace_tools as tt
    import tokenizer_amd as ta
    from safetensors.torch import load_file
    from tokenizer_amd.engine import Engine, Scheduler, SchedulerConfig, GenerateParams, load_model

    config_cls = register_toys()
    cfg = config_cls.from_dict({"vocab_size": 96, "hidden_size": 64, "heads": 2, "inner": 88, "twice": twice})
    folder = ta.write_random_model(cfg, 3, str(tmp_path / "toy"))
    tensors = load_file(folder + "/model.safetensors")
    assert "l.0.mix.mix.weight" in tensors and "l.1.mix.q_proj.weight" in tensors and "l.1.mix.q_proj.bias" not in tensors
    model = load_model(folder, dtype)
    assert [n.kind for n in model.cache_needs] == ["none", "full"] and model.cache_needs[0].state_shape == (64,)
    assert not model.decoder.graph_safe           # the toy mixer loops over requests on the host
    requests = {f"r{i}": random_ids(96, n, 60 + i) for i, n in enumerate([1, 23, 64, 40, 9])}
    steps = tt.mixed(requests, 7, max_live=3)
    engine = Engine(model, max_tokens=tt.peak_tokens(steps), max_requests=3)
    assert len(engine.cache.groups) == 1 and engine.cache.state_layers == [0]
    engine.pools.poison()
    got = tt.run_in_process(engine, steps)
    for rid, ids in requests.items():
        want = toy_plain_logits(tensors, ids, 2, twice)
        err = float((got[rid] - want).abs().max())
        assert err <= (2e-5 if dtype == "float32" else 4e-2) * max(1.0, float(want.abs().max())), (rid, err)
    engine.cache.check_invariants()
    # The scheduler, preemption included, works on it unchanged: few pages, outputs equal to running alone.
    small = Engine(model, num_pages=5, max_requests=3)
    sched = Scheduler(small, SchedulerConfig(num_blocks=5, prefix_cache=False, max_batch_size=3))
    prompts = [random_ids(96, n, 80 + n) for n in (30, 28, 14)]
    rids = [sched.add_request(p, GenerateParams.greedy(6)) for p in prompts]
    results = sched.run()
    assert sched.stats.preemptions >= 1
    if dtype == "float32":
        for rid, prompt in zip(rids, prompts):
            ids = list(prompt)
            for _ in range(6):
                ids.append(plain.greedy_token(toy_plain_logits(tensors, ids, 2, twice)[-1]))
            assert results[rid].tokens == ids[len(prompt):]
    sched.assert_idle()


# ------------------------------------------------------------------------------------------------
# A second toy architecture: a feed-forward with routing and another position encoding, again defined
# here.  Layer 0: attention with distance decay + two routed experts; layer 1: windowed attention with
# rotation + a dense feed-forward.  So one model has different mixers' options, position encodings and
# feed-forwards in different layers, and two cache groups.
def register_routed_toys():
    from tokenizer_amd.config import get_architecture, register_architecture, registered_architectures
    from tokenizer_amd.config.base import ModelConfig
    if "ToyRoutedForCausalLM" in registered_architectures():
        return get_architecture("ToyRoutedForCausalLM").config_class
    from tokenizer_amd.parts import (FEED_FORWARDS, POSITIONS, FeedForward, FeedForwardSpec, LayerSpec, MixerSpec,
                                     ModelSpec, NormSpec, PositionSpec, ScheduleEntry, TensorSpec)
    from tokenizer_amd.parts.position import NoPosition

    if "distance_decay" not in POSITIONS.kinds():
        @POSITIONS.register("distance_decay")
        class DistanceDecay(NoPosition):
            """q_i is scaled by g^-i and k_j by g^j, so that a score is q_i.k_j * g^(j - i): only distances
            count.  The scaling is this test's own torch code; the store into the pages is the package's."""
            graph_safe = False

            def __init__(self, spec, runtime):
                super().__init__(spec, runtime)
                self.gamma = float(spec.options["gamma"])

            def encode_and_store(self, qkv, bias, n_q, n_kv, head_dim, ctx, cache):
                assert bias is None
                pos = ctx.positions.to(torch.float32)[:, None]
                q_end, k_end = n_q * head_dim, (n_q + n_kv) * head_dim
                qkv[:, :q_end] = (qkv[:, :q_end].float() * self.gamma ** (-pos)).to(qkv.dtype)
                qkv[:, q_end:k_end] = (qkv[:, q_end:k_end].float() * self.gamma ** pos).to(qkv.dtype)
                super().encode_and_store(qkv, None, n_q, n_kv, head_dim, ctx, cache)

    if "top1_experts" not in FEED_FORWARDS.kinds():
        @FEED_FORWARDS.register("top1_experts")
        class Top1Experts(FeedForward):
            """Router logits in float32, the first maximum picks one expert a token, its output is scaled by the
            softmax weight of that expert.  Every expert is the package's dense gated part."""

            def __init__(self, spec, tensors, runtime):
                self.runtime, self.n = runtime, int(spec.options["experts"])
                self.router = tensors["router.weight"].float()
                dense = FEED_FORWARDS.get("gated_dense")
                inner = FeedForwardSpec("gated_dense", spec.hidden_size, spec.intermediate_size, "silu")
                self.experts = [dense(inner, {k[len(f"experts.{e}."):]: v for k, v in tensors.items()
                                              if k.startswith(f"experts.{e}.")}, runtime) for e in range(self.n)]

            @staticmethod
            def tensor_specs(spec):
                dense = FEED_FORWARDS.get("gated_dense")
                inner = FeedForwardSpec("gated_dense", spec.hidden_size, spec.intermediate_size, "silu")
                specs = {"router.weight": TensorSpec((int(spec.options["experts"]), spec.hidden_size), std=0.5,
                                                     role="keep")}
                for e in range(int(spec.options["experts"])):
                    specs.update({f"experts.{e}.{k}": v for k, v in dense.tensor_specs(inner).items()})
                return specs

            def forward(self, x, ctx):
                logits = x.float() @ self.router.t()
                choice = torch.argmax(logits, dim=-1)
                weight = torch.softmax(logits, dim=-1).gather(1, choice[:, None])
                out = torch.zeros_like(x)
                for e, expert in enumerate(self.experts):
                    rows = torch.nonzero(choice == e).flatten()
                    if rows.numel():
                        out[rows] = expert.forward(x[rows].contiguous(), ctx)
                return (out.float() * weight).to(x.dtype)

    @dataclasses.dataclass(frozen=True)
    class RoutedConfig(ModelConfig):
        vocab_size: int
        hidden_size: int
        heads: int
        kv_heads: int
        inner: int
        experts: int
        gamma: float
        window: int

    def routed_spec(cfg):
        d = cfg.hidden_size // cfg.heads
        norm = NormSpec("rmsnorm", cfg.hidden_size, 1e-5)
        decay = PositionSpec("distance_decay", d, options={"gamma": cfg.gamma})
        rope = PositionSpec("rope_half_split", d, 10000.0, 512)
        mixers = [MixerSpec("gqa_attention", cfg.hidden_size, cfg.heads, cfg.kv_heads, d, qkv_bias=False, position=decay),
                  MixerSpec("gqa_attention", cfg.hidden_size, cfg.heads, cfg.kv_heads, d, qkv_bias=False, position=rope,
                            window=cfg.window)]
        ffs = [FeedForwardSpec("top1_experts", cfg.hidden_size, cfg.inner, "silu", options={"experts": cfg.experts}),
               FeedForwardSpec("gated_dense", cfg.hidden_size, 2 * cfg.inner, "silu")]
        layers = tuple(LayerSpec("pre_norm", m, f, norm, norm, f"l.{i}.mix", f"l.{i}.ff", f"l.{i}.n1", f"l.{i}.n2")
                       for i, (m, f) in enumerate(zip(mixers, ffs)))
        return ModelSpec("ToyRoutedForCausalLM", cfg.vocab_size, cfg.hidden_size, 512, "emb.weight", layers,
                         (ScheduleEntry(0), ScheduleEntry(1)), norm, "final", tied_head=True, head_name="head.weight")

    register_architecture("ToyRoutedForCausalLM", RoutedConfig, routed_spec)
    return RoutedConfig


def routed_plain_logits(tensors, ids, cfg):
    """The routed toy model on whole sequences with the plain parts."""
    t = {k: v.float() for k, v in tensors.items()}
    hidden, heads, kv = cfg["hidden_size"], cfg["heads"], cfg["kv_heads"]
    d, n = hidden // heads, len(ids)
    pos = list(range(n))
    x = t["emb.weight"][ids]

    def attention(x, i, window, encode):
        h = plain.rms_norm(x, t[f"l.{i}.n1.weight"], 1e-5)
        def heads_of(name, count):
            return (h @ t[f"l.{i}.mix.{name}.weight"].t()).reshape(n, count, d).transpose(0, 1)
        q, k, v = encode(heads_of("q_proj", heads), True), encode(heads_of("k_proj", kv), False), heads_of("v_proj", kv)
        k, v = plain.repeat_kv(k, heads // kv), plain.repeat_kv(v, heads // kv)
        mixed = plain.attend(q, k, v, plain.attention_mask(pos, pos, window)).transpose(0, 1).reshape(n, hidden)
        return x + mixed @ t[f"l.{i}.mix.o_proj.weight"].t()

    def dense(h, prefix):
        return plain.mlp(h, {f"m.{k[len(prefix):]}": v for k, v in t.items() if k.startswith(prefix)}, "m")

    steps = torch.tensor(pos, dtype=torch.float32)[None, :, None]
    x = attention(x, 0, None, lambda v, is_q: v * cfg["gamma"] ** (-steps if is_q else steps))
    h = plain.rms_norm(x, t["l.0.n2.weight"], 1e-5)
    logits = h @ t["l.0.ff.router.weight"].t()
    choice = [plain.greedy_token(row) for row in logits]
    top2 = torch.topk(logits, 2, dim=-1).values
    routed_plain_logits.smallest_gap = float((top2[:, 0] - top2[:, 1]).min())
    weight = torch.softmax(logits, dim=-1)
    out = torch.stack([dense(h[j:j + 1], f"l.0.ff.experts.{choice[j]}.")[0] * weight[j, choice[j]] for j in range(n)])
    x = x + out
    cos, sin = plain.rope_tables(10000.0, d, 512)
    x = attention(x, 1, cfg["window"], lambda v, is_q: plain.apply_rope(v, cos[pos], sin[pos]))
    x = x + dense(plain.rms_norm(x, t["l.1.n2.weight"], 1e-5), "l.1.ff.")
    return plain.rms_norm(x, t["final.weight"], 1e-5) @ t["emb.weight"].t()


def test_distance_decay_counts_only_distances():
    """What pins the toy position encoding's plain form: shifting every position changes no score."""
    q, k = rand((1, 5, 8), 90).cpu(), rand((1, 5, 8), 91).cpu()
    def scores(first):
        steps = torch.arange(first, first + 5, dtype=torch.float32)[None, :, None]
        return (q * 0.97 ** -steps) @ (k * 0.97 ** steps).transpose(1, 2)
    torch.testing.assert_close(scores(0), scores(40), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_architecture(tmp_path, dtype):
    import trace_tools as tt
    import tokenizer_amd as ta
    from safetensors.torch import load_file
    from tokenizer_amd.engine import Engine, load_model

    config_cls = register_routed_toys()
    values = {"vocab_size": 80, "hidden_size": 96, "heads": 6, "kv_heads": 2, "inner": 56, "experts": 3,
              "gamma": 0.97, "window": 19}
    cfg = config_cls.from_dict(values)
    folder = ta.write_random_model(cfg, 5, str(tmp_path / "routed"))
    tensors = load_file(folder + "/model.safetensors")
    assert tensors["l.0.ff.router.weight"].dtype == torch.float32 and "l.0.ff.experts.2.down_proj.weight" in tensors
    model = load_model(folder, dtype)
    assert [n.kind for n in model.cache_needs] == ["full", "window"]
    # Seeds picked (on the CPU, with the plain model) so that the narrowest router decision is clear.
    requests = {f"r{i}": random_ids(80, n, seed) for i, (n, seed) in enumerate([(50, 92), (3, 70), (77, 99), (34, 123)])}
    steps = tt.mixed(requests, 9, max_live=3)
    engine = Engine(model, max_tokens=tt.peak_tokens(steps), max_requests=3)
    assert len(engine.cache.groups) == 2
    engine.pools.poison()
    got = tt.run_in_process(engine, steps)
    for rid, ids in requests.items():
        want = routed_plain_logits(tensors, ids, values)
        # The inputs are chosen so that no router decision is near a tie, which bfloat16 could turn the other way.
        assert routed_plain_logits.smallest_gap > 0.2, routed_plain_logits.smallest_gap
        err = float((got[rid] - want).abs().max())
        assert err <= (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(want.abs().max())), (rid, err)
    engine.cache.check_invariants()


# ------------------------------------------------------------------------------------------------
# A third toy architecture: layers that lack a sub-layer, and a norm and a position encoding defined here
# that say themselves that the fused decode kernels can compute them.  Layer 0 is attention alone, layer 1 a
# feed-forward alone, layer 2 has both.
def register_chain_toys():
    from tokenizer_amd.config import get_architecture, register_architecture, registered_architectures
    from tokenizer_amd.config.base import ModelConfig
    if "ToyChainForCausalLM" in registered_architectures():
        return get_architecture("ToyChainForCausalLM").config_class
    from tokenizer_amd.parts import (NORMS, POSITIONS, FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, Norm,
                                     NormFold, NormSpec, PositionEncoding, PositionSpec, ScheduleEntry, StoreEpilogue,
                                     TensorSpec)

    if "rms_one_plus" not in NORMS.kinds():
        @NORMS.register("rms_one_plus")
        class OnePlus(Norm):
            """x / sqrt(mean(x^2) + eps) * (1 + gain): the file holds the gain's distance from one."""
            graph_safe = True

            def __init__(self, spec, tensors, rt):
                self.size, self.eps, self.rt = spec.size, float(spec.eps), rt
                self.scale = (1.0 + tensors["gain"].float()).contiguous()

            @staticmethod
            def tensor_specs(spec):
                return {"gain": TensorSpec((spec.size,), std=0.3, role="vector")}

            def fold(self):
                return NormFold(self.scale, self.eps)

            def apply(self, residual, delta, rows=None):
                n_rows = residual.shape[0] if rows is None else rows.numel()
                out = torch.empty((n_rows, self.size), dtype=self.rt.dtype, device=residual.device)
                return self.rt.ops.add_rmsnorm(residual, delta, self.scale, self.eps, out, rows,
                                               store_residual=rows is None)

    if "rope_half_speed" not in POSITIONS.kinds():
        @POSITIONS.register("rope_half_speed")
        class HalfSpeed(PositionEncoding):
            """The half-split rotation with every angle halved: another table, the same kernels."""
            graph_safe = True

            def __init__(self, spec, rt):
                self.rt = rt
                cos, sin = half_speed_tables(spec.theta, spec.head_dim, spec.max_positions)
                self.cos_sin = torch.cat([cos, sin], dim=1).contiguous().to(rt.device)

            def epilogue(self):
                return StoreEpilogue(self.cos_sin)

            def encode_and_store(self, qkv, bias, n_q, n_kv, head_dim, ctx, cache):
                slots = ctx.slots[cache.group] if cache.writes else None
                self.rt.ops.rope_store(qkv, bias, ctx.positions, self.cos_sin, slots,
                                       cache.k_pages if cache.writes else None,
                                       cache.v_pages if cache.writes else None, n_q, n_kv, head_dim)

    @dataclasses.dataclass(frozen=True)
    class ChainConfig(ModelConfig):
        vocab_size: int
        hidden_size: int
        heads: int
        inner: int

    def chain_spec(cfg):
        d = cfg.hidden_size // cfg.heads
        norm = NormSpec("rms_one_plus", cfg.hidden_size, 1e-4)
        mixer = MixerSpec("gqa_attention", cfg.hidden_size, cfg.heads, 1, d, qkv_bias=True,
                          position=PositionSpec("rope_half_speed", d, 100.0, 256))
        ff = FeedForwardSpec("gated_dense", cfg.hidden_size, cfg.inner, "silu")
        layers = (LayerSpec("pre_norm", mixer, None, norm, None, mixer_prefix="l.0.mix", mixer_norm_prefix="l.0.n1"),
                  LayerSpec("pre_norm", None, ff, None, norm, feed_forward_prefix="l.1.ff", feed_forward_norm_prefix="l.1.n2"),
                  LayerSpec("pre_norm", mixer, ff, norm, norm, "l.2.mix", "l.2.ff", "l.2.n1", "l.2.n2"))
        return ModelSpec("ToyChainForCausalLM", cfg.vocab_size, cfg.hidden_size, 256, "emb.weight", layers,
                         tuple(ScheduleEntry(i) for i in range(3)), norm, "final", tied_head=True, head_name="head.weight")

    register_architecture("ToyChainForCausalLM", ChainConfig, chain_spec)
    return ChainConfig


def half_speed_tables(theta, d, n_positions):
    inv_freq = torch.tensor([1.0 / (float(theta) ** (i / d)) for i in range(0, d, 2)], dtype=torch.float64).float()
    angles = torch.arange(n_positions, dtype=torch.float32)[:, None] * 0.5 * inv_freq[None, :]
    return angles.cos(), angles.sin()


def chain_plain_logits(tensors, ids, heads):
    t = {k: v.float() for k, v in tensors.items()}
    hidden = t["emb.weight"].shape[1]
    d, n = hidden // heads, len(ids)
    pos = list(range(n))
    cos, sin = half_speed_tables(100.0, d, 256)
    norm = lambda x, name: plain.rms_norm(x, 1.0 + t[f"{name}.gain"], 1e-4)

    def attention(x, i):
        named = {f"a.{k[len(f'l.{i}.mix.'):]}": v for k, v in t.items() if k.startswith(f"l.{i}.mix.")}
        return x + plain.self_attention(norm(x, f"l.{i}.n1"), named, "a", heads, 1, d, cos, sin, pos, None)

    def feed_forward(x, i):
        named = {f"m.{k[len(f'l.{i}.ff.'):]}": v for k, v in t.items() if k.startswith(f"l.{i}.ff.")}
        return x + plain.mlp(norm(x, f"l.{i}.n2"), named, "m")

    x = feed_forward(attention(feed_forward(attention(t["emb.weight"][ids], 0), 1), 2), 2)
    return norm(x, "final") @ t["emb.weight"].t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_without_a_sub_layer_and_parts_that_offer_their_fused_form(tmp_path, dtype):
    import trace_tools as tt
    import tokenizer_amd as ta
    from safetensors.torch import load_file
    from tokenizer_amd.engine import Engine, load_model

    config_cls = register_chain_toys()
    cfg = config_cls.from_dict({"vocab_size": 72, "hidden_size": 64, "heads": 2, "inner": 40})
    folder = ta.write_random_model(cfg, 8, str(tmp_path / "chain"))
    tensors = load_file(folder + "/model.safetensors")
    assert "l.0.mix.q_proj.weight" in tensors and "l.1.ff.down_proj.weight" in tensors and "l.2.n2.gain" in tensors
    assert not any(k.startswith(("l.0.ff", "l.0.n2", "l.1.mix", "l.1.n1")) for k in tensors)
    model = load_model(folder, dtype)
    assert [n.kind for n in model.cache_needs] == ["full", "none", "full"] and model.decoder.graph_safe
    ops = model.runtime.ops
    folded = {"qkv": 0, "gated": 0}
    inner_qkv, inner_gated = ops.fused_norm_qkv_rope, ops.fused_norm_gated

    def count_qkv(rows, norm_weight, *rest, **kw):
        folded["qkv"] += norm_weight is not None
        return inner_qkv(rows, norm_weight, *rest, **kw)

    def count_gated(rows, norm_weight, *rest, **kw):
        folded["gated"] += norm_weight is not None
        return inner_gated(rows, norm_weight, *rest, **kw)

    ops.fused_norm_qkv_rope, ops.fused_norm_gated = count_qkv, count_gated
    try:
        requests = {f"r{i}": random_ids(72, n, 130 + i) for i, n in enumerate([2, 31, 64, 17, 40])}
        steps = tt.mixed(requests, 11, max_live=3)
        engine = Engine(model, max_tokens=tt.peak_tokens(steps), max_requests=3)
        engine.pools.poison()
        got = tt.run_in_process(engine, steps)
    finally:
        del ops.fused_norm_qkv_rope, ops.fused_norm_gated          # back to the class's methods
    for rid, ids in requests.items():
        want = chain_plain_logits(tensors, ids, 2)
        err = float((got[rid] - want).abs().max())
        assert err <= (3e-5 if dtype == "float32" else 4e-2) * max(1.0, float(want.abs().max())), (rid, err)
    engine.cache.check_invariants()
    if dtype == "bfloat16":
        # Steps of few rows took the norm into the products' prologue and the rotation into their epilogue,
        # for parts the package has never heard of.
        assert folded["qkv"] >= 2 and folded["gated"] >= 2, folded
    else:
        assert folded == {"qkv": 0, "gated": 0}


# ------------------------------------------------------------------------------------------------
# A model frame defined outside the package (tests/toy_scaled_frame.py): a scaled embedding, capped logits.
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_frame_of_its_own_registers_and_runs_through_engine_scheduler_and_replay(tmp_path, dtype):
    """What stands around the layers is chosen by the spec (`ModelSpec.frame`), as every part is: a toy frame that
    multiplies its embedding by a constant from its own config.json key and caps its logits is registered from a
    test's file and runs through the engine (mixed batches with reused pages, decode steps replayed from graphs),
    through the scheduler, and through `bin/trace_run` as a child process (which imports the file because the
    environment names it), against the plain model with the embedding scaled by hand."""
    import os
    import trace_tools as tt
    import tokenizer_amd as ta
    import toy_scaled_frame as toy
    from tiny_configs import TINY, random_ids
    from tokenizer_amd.engine import Engine, GenerateParams, load_model

    kind = torch.float32 if dtype == "float32" else torch.bfloat16
    raw = dict(TINY["B"][0], architectures=[toy.ARCHITECTURE], embedding_scale=3.5, logit_cap=1.5)
    folder = ta.write_random_model(toy.ToyScaledConfig.from_dict(raw), 5, str(tmp_path / "scaled"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    scaled = dict(tensors)
    scaled["model.embed_tokens.weight"] = tensors["model.embed_tokens.weight"].float() * 3.5     # (the head is untied)
    assert not raw["tie_word_embeddings"]

    def want_logits(ids):
        return torch.tanh(plain.all_logits(cfg, scaled, ids) / 1.5) * 1.5

    reqs = {f"r{i}": random_ids(raw["vocab_size"], n, 90 + i) for i, n in enumerate([40, 7, 64, 33, 21])}
    want = {rid: want_logits(ids) for rid, ids in reqs.items()}
    # The scale matters: without it the logits are far away.
    unscaled = torch.tanh(plain.all_logits(cfg, tensors, reqs["r0"]) / 1.5) * 1.5
    assert float((unscaled - want["r0"]).abs().max()) > 0.1
    model = load_model(folder, dtype)
    assert type(model.decoder).__name__ == "ToyScaledDecoder"
    for steps in (tt.mixed(reqs, 3), tt.decode_tail(reqs, 20)):
        eng = Engine(model, max_tokens=tt.peak_tokens(steps), max_requests=4)
        eng.pools.poison()
        got = tt.run_in_process(eng, steps)
        for rid in reqs:
            close(got[rid], want[rid], kind)
    # The scheduler: greedy ids against the plain model's (32-bit), and equal to the same request alone.
    eng = Engine(model, num_pages=24, max_requests=3, max_num_batched_tokens=48)
    ids = {eng.add_request(reqs[rid][:30], GenerateParams.greedy(6)): rid for rid in ("r0", "r2", "r3")}
    results = eng.run()
    for request, rid in ids.items():
        tokens, seq = [], list(reqs[rid][:30])
        for _ in range(6):
            tokens.append(int(want_logits(seq)[-1].argmax()))
            seq.append(tokens[-1])
        if dtype == "float32":
            assert results[request].tokens == tokens, rid
        assert len(results[request].tokens) == 6
    # bin/trace_run in a child process: the environment names the module that registers the frame.
    steps = tt.portions({rid: reqs[rid] for rid in ("r0", "r1")}, 5)
    env = dict(os.environ, TOKENIZER_AMD_PLUGINS="toy_scaled_frame",
               PYTHONPATH=os.path.dirname(os.path.abspath(__file__)) + os.pathsep + os.environ.get("PYTHONPATH", ""))
    got = tt.run_program(folder, dtype, steps, str(tmp_path / "out"), tt.peak_tokens(steps), raw["vocab_size"], env=env)
    for rid in ("r0", "r1"):
        close(got[rid], want[rid], kind)
