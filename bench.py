"""Decode and prefill throughput of the engine at Qwen2.5-0.5B sizes with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--dtype bfloat16]

A step is one decode step of the whole batch.  The default run prefills 8 prompts of 2,048
random ids and decodes every request on to 4,096 tokens (8 warm-up steps, 2,040 timed ones); it
also times a prefill of 2,048 tokens, the same decoding at batch 1 and 64 and, at the record's own sizes, the
serving workload mixed-0.5b under a token budget of 512 (with decoding and with prompts first) and the decoding
at batch 8 at Qwen2.5-1.5B and 7B sizes, and prints one JSON line.

    python bench.py --workload mixed-1.5b | mixed-0.5b | prefix-7b [--token-budget N] [--prompts-first]

runs a whole serving workload through the scheduler instead (64 requests at Qwen2.5-1.5B or 0.5B sizes
with prompts of 128 to 2,048 ids and 256 new tokens each; 64 requests at Qwen2.5-7B sizes that
share a prefix of 1,024 ids, with the prefix cache) and prints one JSON line for it.

    python bench.py [--size 0.5b|1.5b|7b] --attention TOKENS [--cached C] [--attention-kernel auto|per-wave|shared]

times the prompt attention kernel alone on a portion of TOKENS tokens after C cached ones.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Published peaks of MI355X.
HBM_GBS = 8000.0
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}

QWEN2_0_5B = {"architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 24, "hidden_size": 896,
              "num_attention_heads": 14, "num_key_value_heads": 2, "intermediate_size": 4864,
              "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
              "max_position_embeddings": 32768, "sliding_window": 32768, "use_sliding_window": False,
              "max_window_layers": 21, "hidden_act": "silu"}
QWEN2_1_5B = dict(QWEN2_0_5B, num_hidden_layers=28, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2,
                  intermediate_size=8960, max_window_layers=21)
QWEN2_7B = dict(QWEN2_0_5B, num_hidden_layers=28, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4,
                intermediate_size=18944, vocab_size=152064, tie_word_embeddings=False, max_window_layers=28)
FULL_LAYERS = 24
PROMPT_LEN = 2048
CONTEXT_LEN = 4096


def log(message: str) -> None:
    print(f"[bench] {message}", file=sys.stderr, flush=True)


def weight_bytes_per_step(model) -> int:
    """Bytes of every weight a decode step reads once (the embedding table is read whole by the tied head)."""
    import torch
    seen, total = set(), 0
    decoder = model.decoder
    tensors = [decoder.head]
    for block in decoder.blocks:
        for part in (block.mixer_norm, block.mixer, block.feed_forward_norm, block.feed_forward):
            if part is not None:
                tensors.extend(v for v in vars(part).values() if isinstance(v, torch.Tensor))
    tensors.extend(v for v in vars(decoder.final_norm).values() if isinstance(v, torch.Tensor))
    for tensor in tensors:
        if tensor.data_ptr() not in seen:
            seen.add(tensor.data_ptr())
            total += tensor.numel() * tensor.element_size()
    return total


def kv_bytes_per_token(cfg, itemsize: int) -> int:
    d = cfg.hidden_size // cfg.num_attention_heads
    return cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * d * itemsize


def prefill_flops(cfg, tokens: int, logit_rows: int = 1) -> float:
    d = cfg.hidden_size // cfg.num_attention_heads
    h, i = cfg.hidden_size, cfg.intermediate_size
    linear = h * (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d + cfg.num_attention_heads * d * h + 3 * h * i
    flops = 2.0 * tokens * cfg.num_hidden_layers * linear
    flops += cfg.num_hidden_layers * 4.0 * cfg.num_attention_heads * d * tokens * (tokens + 1) / 2
    flops += 2.0 * h * cfg.vocab_size * logit_rows
    return flops


def make_prompts(batch: int, vocab: int, seed: int):
    import numpy as np
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, vocab, size=PROMPT_LEN)] for _ in range(batch)]


def run_decode(model, batch: int, steps: int, warmup: int):
    """Prefill `batch` prompts, then time `steps` decode steps (greedy, ids picked on the device).  When the
    timed steps reach into further 512-token ranges of context than the warm-up did, the whole run is done once
    untimed before: a range's first step records its graph, which is set-up, not a decode step."""
    import torch
    from tokenizer_amd.engine import Engine, StepEntry

    page_size = 16
    longest = PROMPT_LEN + warmup + steps
    pages_each = -(-max(CONTEXT_LEN, longest) // page_size)
    engine = Engine(model, num_pages=batch * pages_each + 8, page_size=page_size, max_requests=batch)
    prompts = make_prompts(batch, model.vocab_size, seed=1)
    rids = list(range(batch))

    def one_pass():
        last = []
        for rid, prompt in enumerate(prompts):
            engine.add_request(rid)
            for at in range(0, len(prompt), 2048):                  # long prompts in portions
                portion = prompt[at:at + 2048]
                logits = engine.step([StepEntry(rid, portion, [len(portion) - 1] if at + 2048 >= len(prompt) else [])])
            last.append(engine.argmax(logits)[0])
        # Greedy decode steps back to back: each step's ids feed the next on the device and reach the host one
        # step late (`Engine.decode_greedy`), so the host's work on a step hides behind the device's.
        if warmup:
            last = engine.decode_greedy(rids, last, warmup)[-1]
        torch.cuda.synchronize()
        kv_start = engine.cache.seq_len(0)
        started = time.perf_counter()
        picked = engine.decode_greedy(rids, last, steps)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        assert len(picked) == steps and all(len(ids) == batch for ids in picked)
        for rid in rids:
            engine.end_request(rid)
        return elapsed, kv_start

    bucket = engine.GRAPH_BUCKET
    if engine.use_graphs and -(-longest // bucket) > -(-(PROMPT_LEN + warmup + 1) // bucket):
        one_pass()
    elapsed, kv_start = one_pass()
    kv_mean = kv_start + (steps - 1) / 2 + 1          # keys each step reads, averaged over the timed steps
    del engine
    torch.cuda.empty_cache()
    return elapsed, kv_mean


def run_prefill(model, repeats: int = 7, portion: int | None = None):
    """The prompt in one step, or cut into portions of `portion` tokens, one step each (the best of the repeats)."""
    import torch
    from tokenizer_amd.engine import Engine, StepEntry
    engine = Engine(model, num_pages=PROMPT_LEN // 16 + 8, page_size=16, max_requests=1)
    import numpy as np
    prompt = np.asarray(make_prompts(1, model.vocab_size, seed=2)[0], dtype=np.int64)   # ids as a tokenizer hands them on
    portion = portion or PROMPT_LEN
    best = None
    for _ in range(repeats + 1):
        engine.add_request("p")
        torch.cuda.synchronize()
        started = time.perf_counter()
        for at in range(0, PROMPT_LEN, portion):
            tokens = prompt[at:at + portion]
            logits = engine.step([StepEntry("p", tokens, [len(tokens) - 1] if at + portion >= PROMPT_LEN else [])])
        engine.argmax(logits)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        engine.end_request("p")
        best = elapsed if best is None else min(best, elapsed)
    return best


def run_workload(name: str, layers: int | None, dtype: str, temperature: float = 0.0, token_budget: int = 2048,
                 prompts_first: bool = False, decode_burst: int | None = None, model=None) -> dict:
    """A serving workload through the scheduler: every request is admitted, its prompt cut into portions under
    the token budget beside the others' decode tokens (or, `prompts_first`, ahead of them), decoded greedily to
    its length, and freed."""
    import numpy as np
    import torch
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import Engine, GenerateParams, Generated, Scheduler, SchedulerConfig, random_model

    rng = np.random.default_rng(7)
    if name in ("mixed-1.5b", "mixed-0.5b"):
        raw, new_tokens, prefix_cache = (QWEN2_1_5B if name == "mixed-1.5b" else QWEN2_0_5B), 256, False
        lengths = [int(n) for n in rng.integers(128, 2049, size=64)]
        prompts = [[int(t) for t in rng.integers(0, raw["vocab_size"], size=n)] for n in lengths]
    elif name == "prefix-7b":
        raw, new_tokens, prefix_cache = QWEN2_7B, 512, True
        shared = [int(t) for t in rng.integers(0, raw["vocab_size"], size=1024)]
        prompts = [shared + [int(t) for t in rng.integers(0, raw["vocab_size"], size=512)] for _ in range(64)]
    else:
        raise SystemExit(f"unknown workload {name!r}")
    full_layers = raw["num_hidden_layers"]
    cfg = Qwen2Config.from_dict(dict(raw, num_hidden_layers=layers or full_layers))
    if model is None:
        log(f"building random weights ({cfg.num_hidden_layers} of {full_layers} layers, {dtype})")
        model = random_model(cfg, seed=0, dtype=dtype, device="cuda:0")
    pages = sum(-(-(len(p) + new_tokens) // 16) for p in prompts) + 16
    engine = Engine(model, num_pages=pages, page_size=16, max_requests=64, prefix_cache=prefix_cache)
    log(f"{name}: {len(prompts)} requests, {sum(len(p) for p in prompts)} prompt tokens, {new_tokens} new tokens each")
    tokens_of_pass = []
    for attempt in ("warm-up", "timed"):        # the first pass captures the decode graphs and warms the library
        sched = Scheduler(engine, SchedulerConfig(max_batch_size=64, max_waiting=64, num_blocks=pages,
                                                  prefix_cache=prefix_cache, max_num_batched_tokens=token_budget,
                                                  prompts_first=prompts_first,
                                                  **({} if decode_burst is None else {"decode_burst": decode_burst})))
        torch.cuda.synchronize()
        started = time.perf_counter()
        params = lambda i: (GenerateParams.greedy(new_tokens) if temperature == 0 else
                            GenerateParams(max_tokens=new_tokens, temperature=temperature, top_p=0.95, seed=i))
        ids = [sched.add_request(prompts[0], params(0))]
        if prefix_cache:
            sched.step()                         # the first request's prompt is in the cache when the others arrive
        ids += [sched.add_request(p, params(i + 1)) for i, p in enumerate(prompts[1:])]
        results = sched.run()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        done = [results[i] for i in ids]
        assert all(isinstance(r, Generated) and r.completion_tokens == new_tokens for r in done)
        tokens_of_pass.append([r.tokens for r in done])
        sched.assert_idle()                      # also gives the cached prefix pages back: the timed pass starts cold
        log(f"{attempt} pass: {elapsed:.3f} s; steps so far {engine.steps}, replayed {engine.steps_replayed}, "
            f"graphs captured {engine.graphs_captured}")
    generated = sum(r.completion_tokens for r in done)
    stats = sched.stats
    return {"metric": f"output tokens/s of the workload {name} through the scheduler", "value": round(generated / elapsed, 1),
            "unit": "tokens/s", "n_gpus": 1, "seconds": round(elapsed, 3), "higher_is_better": True,
            "dtype": "bf16" if dtype == "bfloat16" else "fp32", "data": "synthetic (random weights, uniform random ids)",
            "config": {"model": name, "layers": cfg.num_hidden_layers, "layers_of_model": full_layers,
                       "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                       "head_dim": cfg.derived_head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                       "requests": len(prompts), "prompt_tokens": sum(len(p) for p in prompts),
                       "new_tokens_each": new_tokens, "token_budget": token_budget, "prompts_first": prompts_first,
                       "decode_burst": sched.config.decode_burst,
                       "prefix_cache": prefix_cache,
                       "pages": pages, "page_size": 16, "temperature": temperature},
            "scheduler": {"steps": stats.steps, "tokens_forwarded": stats.tokens_forwarded, "max_running": stats.max_running,
                          "preemptions": stats.preemptions, "peak_pages": stats.peak_blocks,
                          "forwarded_tokens_per_s": round(stats.tokens_forwarded / elapsed, 1),
                          "engine_steps": engine.steps, "steps_replayed": engine.steps_replayed,
                          "graphs_captured": engine.graphs_captured,
                          # Requests whose ids are the same in both passes (the first pass runs most steps eagerly,
                          # the second replays them; a recorded step's products may be other kernels', which round
                          # differently, so a greedy request may part ways at a near tie).
                          "requests_with_equal_ids_in_both_passes": sum(
                              a == b for a, b in zip(*tokens_of_pass))}}


def measure_peaks() -> dict:
    """What this device reaches on the two yardsticks of the rooflines: reading a large buffer once (4 GiB, by a
    library reduction and by the package's own read loop in the access pattern of its weight-streaming kernels;
    the higher of the two counts) and a large square bf16 product through the library."""
    import torch
    from tokenizer_amd.kernels import get_ops
    out = {}
    big = torch.empty(1 << 30, dtype=torch.float32, device="cuda:0").fill_(1.0)
    for name, read in (("hbm_read_library_gbs", big.sum), ("hbm_read_loop_gbs", lambda: get_ops().read_stream(big))):
        for _ in range(2):
            read()
        torch.cuda.synchronize()
        started = time.perf_counter()
        for _ in range(10):
            read()
        torch.cuda.synchronize()
        out[name] = round(10 * big.numel() * 4 / (time.perf_counter() - started) / 1e9, 1)
    out["hbm_read_gbs"] = max(out["hbm_read_library_gbs"], out["hbm_read_loop_gbs"])
    del big
    n = 8192
    a = torch.randn(n, n, device="cuda:0").to(torch.bfloat16)
    b = torch.randn(n, n, device="cuda:0").to(torch.bfloat16)
    for _ in range(3):
        a @ b
    torch.cuda.synchronize()
    started = time.perf_counter()
    for _ in range(20):
        a @ b
    torch.cuda.synchronize()
    out["bf16_gemm_tflops"] = round(20 * 2.0 * n ** 3 / (time.perf_counter() - started) / 1e12, 1)
    return out


def run_attention(sizes: dict, tokens: int, cached: int, kernel: str, repeats: int = 20) -> dict:
    """The prompt attention kernel alone at a size's head shape: a portion of `tokens` tokens after `cached` cached
    ones, timed back to back on random keys and values (bfloat16, pages of 16).  kernel: "auto" (the launcher's
    choice), "per-wave" or "shared" (with the launcher's shape where it plans one, else two heads a wave)."""
    import types
    import torch
    from tokenizer_amd.kernels import get_ops
    ops = get_ops()
    n_q, n_kv = sizes["num_attention_heads"], sizes["num_key_value_heads"]
    d = sizes["hidden_size"] // n_q
    page, length = 16, cached + tokens
    n_pages = length // page + 1
    dev, bf = "cuda:0", torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(0)
    k_pages = torch.randn((n_pages, n_kv, page, d), generator=gen, device=dev).to(bf)
    v_pages = torch.randn((n_pages, n_kv, d, page), generator=gen, device=dev).to(bf)
    qkv = torch.randn((tokens, (n_q + 2 * n_kv) * d), generator=gen, device=dev).to(bf)
    out = torch.empty((tokens, n_q * d), dtype=bf, device=dev)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device=dev)
    table = torch.arange(n_pages, dtype=torch.int32, device=dev).reshape(1, n_pages)
    positions = torch.arange(cached, length, dtype=torch.int32, device=dev)
    entry_of_token = torch.zeros(tokens, dtype=torch.int32, device=dev)
    batch = types.SimpleNamespace(n_tokens=tokens, cu_q=ints([0, tokens]), first_position=ints([cached]),
                                  q_tiles=ints([[0, o] for o in range(0, tokens, 16)]), decode_rows=ints([]),
                                  max_position=length - 1)
    tiles = batch.q_tiles.shape[0]
    plan = ops.lib.ta_prefill_attention_shared_plan(tiles, n_q, n_kv, d, -(-length // 512) * 512)
    ops.prefill_shared = {"auto": 0, "per-wave": -1, "shared": 1}[kernel]

    def run():
        ops.paged_attention(qkv, out, k_pages, v_pages, positions, entry_of_token, table, n_q, n_kv, d, None, d ** -0.5,
                            max_position=length - 1, batch=batch)
    run()
    torch.cuda.synchronize()
    started = time.perf_counter()
    for _ in range(repeats):
        run()
    torch.cuda.synchronize()
    seconds = (time.perf_counter() - started) / repeats
    ops.prefill_shared = 0
    flops = 4.0 * n_q * d * (tokens * cached + tokens * (tokens + 1) / 2)
    return {"attention_us": round(seconds * 1e6, 1), "tflops": round(flops / seconds / 1e12, 1), "tokens": tokens,
            "cached": cached, "q_heads": n_q, "kv_heads": n_kv, "head_dim": d, "kernel": kernel,
            "planned_shape": plan}


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=None,
                        help="timed decode steps (default: from the prompt's end to the context the record names, "
                             "2,048 -> 4,096 tokens per request)")
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--layers", type=int, default=None)
    parser.add_argument("--size", default="0.5b", choices=["0.5b", "1.5b", "7b"],
                        help="layer sizes of the decode benchmark (the default is the one the record is for)")
    parser.add_argument("--peaks", action="store_true", help="measure what the device reaches in HBM reads and bf16 products")
    parser.add_argument("--workload", default=None, choices=["mixed-1.5b", "mixed-0.5b", "prefix-7b"],
                        help="run a serving workload through the scheduler instead of the decode benchmark")
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    parser.add_argument("--only-prefill", action="store_true", help="time the prefill alone (for profiling)")
    parser.add_argument("--portion", type=int, default=None,
                        help="with --only-prefill: cut the prompt into portions of this many tokens, one step each")
    parser.add_argument("--attention", type=int, default=None, metavar="TOKENS",
                        help="time the prompt attention kernel alone on a portion of this many tokens at --size's head shape")
    parser.add_argument("--cached", type=int, default=0, help="with --attention: tokens already in the cache")
    parser.add_argument("--attention-kernel", default="auto", choices=["auto", "per-wave", "shared"],
                        help="with --attention: the launcher's choice, or one of the two prompt kernels")
    parser.add_argument("--token-budget", type=int, default=2048,
                        help="with --workload: the most tokens a step of the scheduler may hold")
    parser.add_argument("--prompts-first", action="store_true",
                        help="with --workload: portions of prompts take the token budget before decoding requests do")
    parser.add_argument("--decode-burst", type=int, default=None,
                        help="with --workload: decode steps the scheduler lets run back to back (its default: 16)")
    parser.add_argument("--temperature", type=float, default=0.0,
                        help="with --workload: draw with this temperature and top_p 0.95 instead of greedy picks")
    parser.add_argument("--prompt-len", type=int, default=None,
                        help="tokens of every prompt before decoding (default 2,048, the record's; the context the "
                             "record names is then twice that, else the prompt plus the decoded tokens)")
    args = parser.parse_args()
    global PROMPT_LEN, CONTEXT_LEN
    if args.prompt_len:
        PROMPT_LEN = args.prompt_len
        if args.steps is None:
            args.steps = 128
        CONTEXT_LEN = -(-(args.prompt_len + args.warmup + max(args.steps, 64) + 1) // 16) * 16
    if args.steps is None:
        args.steps = CONTEXT_LEN - PROMPT_LEN - args.warmup
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; runs with --gpus > 1 are not supported")
        return 2

    if args.peaks:
        print(json.dumps(measure_peaks()), flush=True)
        return 0
    if args.workload:
        print(json.dumps(run_workload(args.workload, args.layers, args.dtype, args.temperature, args.token_budget,
                                      args.prompts_first, args.decode_burst)), flush=True)
        return 0
    sizes = {"0.5b": QWEN2_0_5B, "1.5b": QWEN2_1_5B, "7b": QWEN2_7B}[args.size]
    if args.attention:
        print(json.dumps(run_attention(sizes, args.attention, args.cached, args.attention_kernel)), flush=True)
        return 0
    full_layers = sizes["num_hidden_layers"]
    args.layers = args.layers or full_layers

    import torch
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import random_model

    cfg = Qwen2Config.from_dict(dict(sizes, num_hidden_layers=args.layers))
    log(f"building random weights ({args.layers} layers, {args.dtype})")
    model = random_model(cfg, seed=0, dtype=args.dtype, device="cuda:0")
    itemsize = 2 if args.dtype == "bfloat16" else 4
    weights = weight_bytes_per_step(model)
    kv_token = kv_bytes_per_token(cfg, itemsize)

    if args.only_prefill:
        seconds = run_prefill(model, repeats=3 if args.portion else 7, portion=args.portion)
        print(json.dumps({"prefill_ms": round(seconds * 1e3, 3), "tokens": PROMPT_LEN, "portion": args.portion or PROMPT_LEN,
                          "tokens_per_s": round(PROMPT_LEN / seconds, 1)}), flush=True)
        return 0
    log(f"decode at batch {args.batch}: {args.warmup} warmup + {args.steps} timed steps")
    elapsed, kv_mean = run_decode(model, args.batch, args.steps, args.warmup)
    ms_per_step = elapsed / args.steps * 1e3
    value = args.batch * args.steps / elapsed
    step_bytes = weights + args.batch * kv_mean * kv_token
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9

    decoded_to = PROMPT_LEN + args.warmup + args.steps
    first_timed = PROMPT_LEN + args.warmup
    record = {
        # The contexts the timed steps really ran at: a short run sits at the cheap end of the range.
        "metric": "decode tokens/s (Qwen2.5-%s sizes, batch %d, contexts %d to %d of prompts of %d)"
                  % (args.size.upper(), args.batch, first_timed + 1, decoded_to, PROMPT_LEN),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform random ids)",
        "config": {"model": "qwen2.5-%s-sizes" % args.size, "layers": args.layers, "layers_of_model": full_layers,
                   "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.derived_head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "tied_head": cfg.tie_word_embeddings, "global_batch": args.batch, "prompt_len": PROMPT_LEN,
                   "seq_len": decoded_to, "decoded_to": decoded_to, "page_size": 16,
                   "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
    }
    if not args.no_points:
        log("prefill of 2,048 tokens")
        seconds = run_prefill(model)
        flops = prefill_flops(cfg, PROMPT_LEN)
        record["prefill"] = {"value": round(PROMPT_LEN / seconds, 1), "tokens": PROMPT_LEN, "ms": round(seconds * 1e3, 3),
                             "frac": round(flops / seconds / (PEAK_TFLOPS[args.dtype] * 1e12), 5)}
        points = {}
        for batch, steps in ((1, args.steps), (64, args.steps)):
            log(f"decode at batch {batch}: {steps} timed steps")
            e, kv = run_decode(model, batch, steps, min(args.warmup, 4))
            points[f"decode_b{batch}"] = round(batch * steps / e, 1)
            # The same roofline figures as for the main batch: a step's time, the bytes it has to read (weights
            # once, the live requests' keys and values), and their quotient against the published bandwidth.
            gb = (weights + batch * kv * kv_token) / 1e9
            points[f"decode_b{batch}_ms"] = round(e / steps * 1e3, 4)
            points[f"decode_b{batch}_gb"] = round(gb, 4)
            points[f"decode_b{batch}_hbm_frac"] = round(gb / (e / steps) / HBM_GBS, 4)
        record["points"] = points
        # The same two fractions against what this device reaches on the yardsticks themselves (a large read,
        # a large square product through the library), beside those against the published peaks.
        log("what the device reaches: a 4 GiB read and an 8,192-cubed bf16 product")
        reached = measure_peaks()
        record["roofline"]["step_gb"] = round(step_bytes / 1e9, 4)
        record["roofline"]["measured_peak"] = reached["hbm_read_gbs"]
        record["roofline"]["measured_peak_library_sum"] = reached["hbm_read_library_gbs"]
        record["roofline"]["frac_of_measured"] = round(achieved / reached["hbm_read_gbs"], 4)
        if args.dtype == "bfloat16":
            record["prefill"]["measured_peak_tflops"] = reached["bf16_gemm_tflops"]
            record["prefill"]["frac_of_measured"] = round(flops / seconds / (reached["bf16_gemm_tflops"] * 1e12), 5)
        if args.size == "0.5b" and args.layers == full_layers:
            # The serving workload at these sizes through the scheduler (64 requests, prompts of 128 to 2,048 ids,
            # 256 new tokens each, a token budget of 512), with decoding and with prompts first.  What goes wrong
            # here is said in the record and does not cost it the figures above.
            try:
                serving = {"workload": "mixed-0.5b", "token_budget": 512, "unit": "output tokens/s"}
                for key, first in (("decoding_first", False), ("prompts_first", True)):
                    log(f"serving workload mixed-0.5b, budget 512, {key.replace('_', ' ')}")
                    run = run_workload("mixed-0.5b", None, args.dtype, token_budget=512, prompts_first=first, model=model)
                    serving[key] = run["value"]
                    serving[key + "_s"] = run["seconds"]
                record["serving"] = serving
            except Exception as err:                                  # noqa: BLE001 (whatever it is, it is reported)
                record["serving"] = {"error": f"{type(err).__name__}: {err}"[:300]}
            # The same decoding at batch 8 at the sizes of the larger models of the family (all their layers), whose
            # steps are nearer to what the memory can deliver: tokens/s, a step's time, the bytes it has to read and
            # their quotient against the published bandwidth, as for the record's own sizes.
            del model
            torch.cuda.empty_cache()
            larger = {}
            for name, raw in (("1.5b", QWEN2_1_5B), ("7b", QWEN2_7B)):
                try:
                    log(f"decode at batch 8 at Qwen2.5-{name.upper()} sizes: {args.steps} timed steps")
                    other_cfg = Qwen2Config.from_dict(dict(raw))
                    other = random_model(other_cfg, seed=0, dtype=args.dtype, device="cuda:0")
                    e, kv = run_decode(other, 8, args.steps, min(args.warmup, 4))
                    gb = (weight_bytes_per_step(other) + 8 * kv * kv_bytes_per_token(other_cfg, itemsize)) / 1e9
                    larger[f"decode_b8_{name}"] = round(8 * args.steps / e, 1)
                    larger[f"decode_b8_{name}_ms"] = round(e / args.steps * 1e3, 4)
                    larger[f"decode_b8_{name}_gb"] = round(gb, 4)
                    larger[f"decode_b8_{name}_hbm_frac"] = round(gb / (e / args.steps) / HBM_GBS, 4)
                    del other
                    torch.cuda.empty_cache()
                except Exception as err:                              # noqa: BLE001
                    larger[f"decode_b8_{name}_error"] = f"{type(err).__name__}: {err}"[:300]
            record["larger_sizes"] = larger
    print(json.dumps(record), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
