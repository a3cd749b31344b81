"""The scheduler on the device: preemption with recomputation, shared prefix pages, prompts cut into portions
whose shape recurs (so that captured graphs replay them), against the plain implementation's tokens."""
import pytest
import torch

from plain import qwen2_plain as plain
from tiny_configs import TINY, random_ids

pytestmark = pytest.mark.gpu


def engine_for(folder, dtype, **kw):
    from tokenizer_amd.engine import Engine, load_model
    return Engine(load_model(folder, dtype), **kw)


def check_greedy(cfg, tensors, prompt, tokens, dtype, n_tokens):
    """The tokens a greedy request produced, against the plain implementation.  float32: the same ids.
    bfloat16: rounding may pick another of two nearly equal logits, after which the sequences differ for good;
    so every token is checked against the plain logits of the sequence the engine itself went along: it must
    be the maximum of its row up to what bfloat16 rounding can move a logit."""
    assert len(tokens) == n_tokens
    if dtype == "float32":
        assert tokens == plain.greedy_generate(cfg, tensors, prompt, n_tokens)
        return
    logits = plain.all_logits(cfg, tensors, list(prompt) + list(tokens))
    for k, token in enumerate(tokens):
        row = logits[len(prompt) - 1 + k]
        assert float(row.max() - row[token]) <= 4e-2 * max(1.0, float(row.abs().max())), (k, token)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_few_pages_a_shared_prefix_and_portions_on_the_device(model_folders, dtype):
    """Six requests, three of which start with the same 40 tokens, through a pool of eight pages with prompts cut
    into portions of sixteen: some are preempted and recomputed, the later sharers take over the prefix's pages,
    decode steps and recurring portion shapes replay captured graphs.  Every request gets the plain
    implementation's tokens, and nothing is left over.  (Cases of qwen-server/src/engine.rs:1833-1908,
    1965-2320 and 2470-2529, run on the kernels.)"""
    from tokenizer_amd.engine import Generated, GenerateParams, Scheduler, SchedulerConfig
    name = "B"
    cfg, tensors = plain.load_folder(model_folders[name])
    vocab = cfg["vocab_size"]
    prefix = random_ids(vocab, 40, 7)
    prompts = [prefix + random_ids(vocab, 6, 1), random_ids(vocab, 21, 2), prefix + random_ids(vocab, 9, 3),
               random_ids(vocab, 33, 4), prefix + random_ids(vocab, 3, 5), random_ids(vocab, 17, 6)]
    eng = engine_for(model_folders[name], dtype, num_pages=8, max_requests=3, prefix_cache=True)
    eng.pools.poison()
    sched = Scheduler(eng, SchedulerConfig(max_batch_size=3, num_blocks=8, prefix_cache=True, prefill_chunk=16,
                                           max_num_batched_tokens=48))
    rids = [sched.add_request(p, GenerateParams.greedy(12)) for p in prompts]
    results = sched.run()
    for rid, prompt in zip(rids, prompts):
        assert isinstance(results[rid], Generated), results[rid]
        check_greedy(cfg, tensors, prompt, results[rid].tokens, dtype, 12)
    assert sched.stats.preemptions >= 1 and sched.stats.prefix_hits >= 2 and sched.stats.prefix_tokens_reused >= 64
    assert eng.use_graphs and eng.graphs
    sched.assert_idle()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_long_prompts_replay_graphs_narrower_than_their_tables(tmp_path, dtype):
    """Prompts longer than a graph's context bucket, one after another, cut into equal portions: the pages of a
    whole prompt are reserved at admission, so during its first portions a request's block table is wider than
    the table of the graph that the recurring shape replays.  Tokens with graphs equal tokens without, and the
    plain implementation's."""
    import tokenizer_amd as ta
    from tokenizer_amd.config import Qwen2Config
    from tokenizer_amd.engine import GenerateParams, Scheduler, SchedulerConfig
    raw = dict(TINY["A"][0], max_position_embeddings=2048, sliding_window=2048)
    folder = ta.write_random_model(Qwen2Config.from_dict(raw), 21, str(tmp_path / "long"), norm_spread=0.3)
    cfg, tensors = plain.load_folder(folder)
    prompts = [random_ids(raw["vocab_size"], 1100, 300 + i) for i in range(4)]
    tokens = {}
    for use_graphs in (True, False):
        eng = engine_for(folder, dtype, num_pages=80, max_requests=1, use_graphs=use_graphs)
        eng.pools.poison()
        sched = Scheduler(eng, SchedulerConfig(max_batch_size=1, num_blocks=80, prefix_cache=False, prefill_chunk=256,
                                               max_num_batched_tokens=256))
        rids = [sched.add_request(p, GenerateParams.greedy(6)) for p in prompts]
        results = sched.run()
        tokens[use_graphs] = [results[rid].tokens for rid in rids]
        if use_graphs:
            portion_graphs = [key for key in eng.graphs if not isinstance(key[0], int)]
            assert portion_graphs, "no portion shape was captured"
            # The first portions replay graphs for contexts of 512 tokens: 32 pages, where the request holds 69.
            assert any(eng.graphs[key].width < 69 for key in portion_graphs)
        sched.assert_idle()
    if dtype == "float32":        # (bfloat16 portions of this many rows go to different products when recorded)
        assert tokens[True] == tokens[False]
    for use_graphs in (True, False):
        for prompt, got in zip(prompts, tokens[use_graphs]):
            check_greedy(cfg, tensors, prompt, got, dtype, 6)
