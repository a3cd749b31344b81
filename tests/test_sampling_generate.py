"""Sampling, the streaming decoder, the stop-string hold and the generation loop (vectors of
qwen-infer/src/sample.rs:159-255, stream.rs:95-141 and generate.rs:519-748)."""
import pytest

from cpu_engine import cpu_engine
from plain import qwen2_plain as plain
from tokenizer_amd.engine import (Control, GenerateParams, SampleCursor, StopHold, StopReason, StreamDecoder,
                                  generate, generate_with, greedy_tokens, parse_eos_token_ids)
from tokenizer_amd.sampling import Rng, SampleError, greedy_token, sample_token, sample_with_uniform


def draw(logits, temperature, top_p, seed):
    return sample_token(logits, temperature, top_p, Rng(seed))


def sequence(logits, temperature, top_p, seed, n):
    rng = Rng(seed)
    return [sample_token(logits, temperature, top_p, rng) for _ in range(n)]


def test_seeded_sampling_is_deterministic():
    logits = [0.2, 1.0, 0.5, 0.7, 0.1, 0.9, 0.4, 0.8]
    first = sequence(logits, 1.0, 0.9, 7, 32)
    assert first == sequence(logits, 1.0, 0.9, 7, 32)
    assert first != sequence(logits, 1.0, 0.9, 8, 32)


def test_temperature_zero_is_greedy_and_ties_keep_the_lower_id():
    logits = [0.2, 1.5, 1.5, -3.0, 0.0]
    assert greedy_token(logits) == 1
    assert draw(logits, 0.0, 1.0, 99) == 1
    assert draw(logits, 0.0, 1.0, 1) == draw(logits, 0.0, 1.0, 2)
    assert draw(logits, 0.0, 1.5, 4) == 1
    rng = Rng(3)
    sample_token(logits, 0.0, 1.0, rng)
    assert rng.counter == 0                     # greedy never draws
    assert greedy_token([float("nan"), 1.0, float("nan")]) == 1
    assert greedy_token([float("-inf")] * 3) == 0


def test_top_p_keeps_at_least_the_top_token_and_full_mass_keeps_everyone():
    logits = [0.0, 2.0, 0.5, -1.0]
    for seed in range(30):
        assert draw(logits, 1.0, 1e-6, seed) == 1
        assert draw(logits, 0.7, 0.0, seed) == 1
    flat = [0.0] * 8
    assert len({draw(flat, 1.0, 1.0, seed) for seed in range(40)}) > 1
    assert draw(logits, 0.8, 1.0, 3) == draw(logits, 0.8, 4.0, 3)


def test_sampling_rejects_bad_arguments():
    rng = Rng(1)
    for args in (([], 1.0, 1.0), ([1.0], -0.1, 1.0), ([1.0], float("nan"), 1.0), ([1.0], 1.0, -0.2),
                 ([1.0], float("inf"), 1.0), ([1.0], 1.0, float("nan"))):
        with pytest.raises(SampleError):
            sample_token(*args, rng)


def test_host_sampler_agrees_with_the_plain_one():
    import numpy as np
    rng = np.random.default_rng(0)
    for case in range(200):
        logits = rng.normal(size=50).astype(np.float32) * 3
        if case % 5 == 0:
            logits[10:20] = logits[3]            # ties
        t = float(rng.choice([0.3, 1.0, 2.5]))
        p = float(rng.choice([0.1, 0.5, 0.9, 1.0]))
        u = float(rng.random())
        assert sample_with_uniform(logits, t, p, u) == plain.sample_token(logits, t, p, u)
    assert 0.0 <= Rng(5).random_f32() < 1.0
    values = [Rng(9).random_f32() for _ in range(3)]
    assert values[0] == values[1] == values[2]
    stream = Rng(9)
    assert len({stream.random_f32() for _ in range(100)}) == 100


# ---- stream decoder ------------------------------------------------------------------------------
def test_stream_decoder_buffers_partial_utf8():
    text = "aé中🦀b"
    decoder, acc, held = StreamDecoder(), "", False
    for byte in text.encode():
        chunk = decoder.push(bytes([byte]))
        assert "�" not in chunk
        if decoder.pending:
            held = True
        acc += chunk
    assert held and not decoder.pending and acc == text and decoder.finish() == ""
    for case in ("é", "中", "🦀", "a中b🦀"):
        d = StreamDecoder()
        assert "".join(d.push(bytes([b])) for b in case.encode()) == case and not d.pending
    d = StreamDecoder()
    assert d.push(b"\xf0") == "" and bytes(d.pending) == b"\xf0"
    assert d.push(b"\x9f\xa6") == ""
    assert d.finish() == "�" and not d.pending
    d = StreamDecoder()
    assert d.push(b"a\xffb") == "a�b"      # a byte that can never start a character


def test_stop_hold_releases_a_suffix_that_was_not_the_stop():
    held = StopHold()
    assert held.push("aba", ["abc"]) == (False, "ab")
    assert held.push("bc", ["abc"]) == (True, "")
    assert held.handed_out == 2 and held.tail == "" and held.push("more", ["abc"]) == (True, "")


# ---- generation loop -----------------------------------------------------------------------------
def scripted(data: bytes):
    state = {"at": 0}

    def token_bytes(_token):
        at = state["at"]
        state["at"] += 1
        return data[at:at + 1]
    return token_bytes


@pytest.fixture()
def engine(model_folders):
    return cpu_engine(model_folders["A"])


def test_stops_on_max_tokens_and_skips_the_unused_forward(engine, model_folders):
    out = generate(engine, [1, 2, 3], GenerateParams.greedy(5), scripted(b"abcdefgh"))
    assert out.reason == StopReason.MaxTokens and len(out.tokens) == 5 and out.completion_tokens == 5
    assert out.text == "abcde" and "".join(out.chunks) == out.text
    assert engine.forwards == [[3], [1], [1], [1], [1]]           # generate.rs:686-704
    cfg, tensors = plain.load_folder(model_folders["A"])
    assert out.tokens == plain.greedy_generate(cfg, tensors, [1, 2, 3], 5)
    assert greedy_tokens(engine, [1, 2, 3], 5) == out.tokens
    assert not engine.cache.requests


def test_max_tokens_zero_still_runs_the_prompt(engine):
    out = generate(engine, [4, 5, 6], GenerateParams.greedy(0))
    assert out.reason == StopReason.MaxTokens and out.tokens == [] and out.completion_tokens == 0
    assert engine.forwards == [[3]]


def test_eos_is_counted_but_neither_stored_nor_forwarded(engine):
    free = generate(engine, [4, 5, 6], GenerateParams.greedy(6), scripted(b"abcdefghij"))
    engine.forwards.clear()
    params = GenerateParams.greedy(6)
    params.eos = [free.tokens[2] + 97, free.tokens[2]]
    first_hit = free.tokens.index(free.tokens[2])
    out = generate(engine, [4, 5, 6], params, scripted(b"abcdefghij"))
    assert out.reason == StopReason.Eos
    assert out.tokens == free.tokens[:first_hit] and out.completion_tokens == first_hit + 1
    assert out.text == "abcdefghij"[:first_hit]
    assert engine.forwards == [[3]] + [[1]] * first_hit


def test_stop_string_is_excluded_even_when_it_spans_tokens(engine):
    data = b"hello world"
    params = GenerateParams.greedy(len(data))
    params.stop = ["world", "lo "]
    out = generate(engine, [1, 2], params, scripted(data))
    assert out.reason == StopReason.StopString and out.text == "hel" and "".join(out.chunks) == "hel"
    params.stop, params.max_tokens = ["abc"], 2
    flushed = generate(engine, [1, 2], params, scripted(b"abZZ"))
    assert flushed.reason == StopReason.MaxTokens and flushed.text == "ab"
    emoji = b"a" + "🦀".encode() + b"b"
    params.stop, params.max_tokens = ["🦀"], len(emoji)
    cut = generate(engine, [1, 2], params, scripted(emoji))
    assert cut.reason == StopReason.StopString and cut.text == "a"


def test_cancel_skips_the_next_forward(engine):
    seen = []

    def on_chunk(piece):
        seen.append(piece)
        return Control.Stop if len(seen) == 3 else Control.Continue     # the probe, then two tokens
    out = generate_with(engine, [1, 2, 3], GenerateParams.greedy(8), scripted(b"abcdefgh"), on_chunk)
    assert out.reason == StopReason.Cancelled and len(out.tokens) == 2
    assert engine.forwards == [[3], [1]]
    engine.forwards.clear()
    gone = generate_with(engine, [1, 2, 3], GenerateParams.greedy(8), scripted(b"ab"), lambda piece: Control.Stop)
    assert gone.reason == StopReason.Cancelled and gone.tokens == [] and engine.forwards == [[3]]


def test_warm_generation_is_seeded(engine):
    params = GenerateParams(max_tokens=24, temperature=1.1, top_p=1.0, seed=11)
    a = generate(engine, [1, 2, 3, 4], params)
    b = generate(engine, [1, 2, 3, 4], params)
    assert a.tokens == b.tokens and len(a.tokens) == 24
    params.seed = 12
    assert generate(engine, [1, 2, 3, 4], params).tokens != a.tokens
    with pytest.raises(ValueError):
        generate(engine, [], params)
    with pytest.raises(SampleError):
        SampleCursor(GenerateParams(stop=[""]))
    with pytest.raises(SampleError):
        SampleCursor(GenerateParams(temperature=-1.0))


def test_parse_eos_token_ids():
    # qwen-infer/src/lib.rs:136-147
    assert parse_eos_token_ids('{"eos_token_id":[151645,151643],"do_sample":true}') == [151645, 151643]
    assert parse_eos_token_ids('{"bos_token_id":1,"eos_token_id":151643}') == [151643]
    for bad in ('{"bos_token_id":1}', '{"eos_token_id":[]}', '{"eos_token_id":"x"}'):
        with pytest.raises(ValueError):
            parse_eos_token_ids(bad)


def test_engine_queues_and_runs_generations(model_folders):
    """The entry point in the reference's manner: requests with their parameters go to the engine, `run()` returns
    what each generated; the same as generating each alone."""
    from cpu_engine import cpu_engine
    from tiny_configs import random_ids
    from tokenizer_amd.engine import Engine, GenerateParams, Generated, generate, load_model
    from kernel_refs import PlainOps
    folder = model_folders["A"]
    model = load_model(folder, "float32", "cpu", ops=PlainOps())
    engine = Engine(model, num_blocks=32, max_batch_size=3, max_num_batched_tokens=24, prefix_cache=True)
    assert engine.cache.num_pages == 32 and engine.cache.max_requests == 3
    prompts = [random_ids(256, n, 300 + n) for n in (5, 30, 17, 2)]
    ids = [engine.add_request(p, GenerateParams.greedy(4 + i)) for i, p in enumerate(prompts)]
    results = engine.run()
    for rid, prompt, n in zip(ids, prompts, range(4, 8)):
        assert isinstance(results[rid], Generated)
        assert results[rid].tokens == generate(cpu_engine(folder), prompt, GenerateParams.greedy(n)).tokens
    engine.scheduler.assert_idle()
