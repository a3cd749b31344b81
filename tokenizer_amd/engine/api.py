"""Entry points in the manner of qwen-infer's library (qwen-infer/src/lib.rs:14-24, 116-130):
`generate`, `generate_with`, `greedy_tokens`."""
from __future__ import annotations

import time

from .batch import StepEntry
from .generate import Control, GenerateParams, Generated, SampleCursor, Sampled, StopReason, _go_on, _no_bytes


def _next(engine, cursor: SampleCursor, logits, token_bytes, on_chunk):
    """Pick the next id on the device (greedy, or a warm draw with the cursor's next uniform number) and hand
    it to the cursor; an engine without a device sampler gets the logits row drawn on the host."""
    if cursor.exhausted:
        return cursor.push_token(0, token_bytes, on_chunk)        # finishes, nothing is drawn
    if cursor.is_greedy:
        token = engine.argmax(logits, [0])[0]
    elif hasattr(engine, "sample"):
        token = engine.sample(logits, [0], [cursor.params.temperature], [cursor.params.top_p],
                              [cursor.next_uniform()])[0]
    else:
        return cursor.push_logits(engine.rows_to_host(logits, [0])[0], token_bytes, on_chunk)
    return cursor.push_token(token, token_bytes, on_chunk)


def _engine_for(model_or_engine, prompt, params):
    """`generate(model, ...)` as in the reference: a bare model gets an engine sized for this one request."""
    if hasattr(model_or_engine, "step"):
        return model_or_engine
    from .engine import Engine
    return Engine(model_or_engine, max_tokens=len(prompt) + params.max_tokens + 1, max_requests=1)


def generate_with(engine, prompt: list[int], params: GenerateParams, token_bytes=_no_bytes,
                  on_chunk=_go_on) -> Generated:
    """Prefill `prompt`, then sample up to `params.max_tokens` ids, one cached forward per id.

    The forward after the last allowed sample is not run; `max_tokens == 0` still runs the prompt;
    the chunk callback is probed once with "" after the prompt so that a caller who is gone
    cancels before the first draw (qwen-infer/src/generate.rs:340-394).
    """
    if not prompt:
        raise ValueError("prompt encoded to no tokens")
    engine = _engine_for(engine, prompt, params)
    cursor = SampleCursor(params)
    rid = ("generate", id(cursor))
    engine.add_request(rid)
    try:
        started = time.perf_counter()
        logits = engine.step([StepEntry(rid, list(prompt), [len(prompt) - 1] if params.max_tokens > 0 else [])])
        if params.max_tokens > 0:
            engine.argmax(logits, [0])                 # waits for the prompt's forward, so the clock is honest
        prefill = time.perf_counter() - started
        started = time.perf_counter()
        if params.max_tokens == 0:
            done = cursor.finish_without_sample(on_chunk)
        elif on_chunk("") == Control.Stop:
            done = Sampled([], "", [], StopReason.Cancelled, 0)
        else:
            outcome = _next(engine, cursor, logits, token_bytes, on_chunk)
            on_device = hasattr(engine, "decode_greedy") and (
                cursor.is_greedy or (hasattr(engine, "decode_sampled") and hasattr(engine, "sample")))
            if not isinstance(outcome, Sampled) and on_device:
                # The remaining steps run back to back on the device, greedy picks or draws (the cursor gives a
                # step's uniform number when it is launched); the cursor sees each id one step late and ends the
                # run when it stops (at most one forward is then run for nothing).
                ended = []

                def on_step(_k, ids):
                    result = cursor.push_token(ids[0], token_bytes, on_chunk)
                    if isinstance(result, Sampled):
                        ended.append(result)
                        return False
                    return True

                if cursor.is_greedy:
                    engine.decode_greedy([rid], [int(outcome)], params.max_tokens - cursor.produced, on_step)
                else:
                    draw = lambda _k: ([params.temperature], [params.top_p], [cursor.next_uniform()])
                    engine.decode_sampled([rid], [int(outcome)], params.max_tokens - cursor.produced, draw, on_step)
                outcome = ended[0]
            while not isinstance(outcome, Sampled):
                logits = engine.step([StepEntry(rid, [int(outcome)], [0])])
                outcome = _next(engine, cursor, logits, token_bytes, on_chunk)
            done = outcome
        decode = time.perf_counter() - started
    finally:
        engine.end_request(rid)
    return Generated(done.tokens, done.text, done.chunks, done.reason, done.completion_tokens, prefill, decode)


def generate(engine, prompt, params: GenerateParams, token_bytes=_no_bytes, tokenizer=None) -> Generated:
    """Generate from token ids, or from text when a `tokenizer` (tokenizer_amd.Tokenizer) is given: the text is
    encoded with it and the sampled ids are decoded with it.  `engine`: an `Engine` or a bare model."""
    if isinstance(prompt, str):
        if tokenizer is None:
            raise ValueError("a text prompt needs a tokenizer")
        prompt = tokenizer.encode(prompt)
    if tokenizer is not None and token_bytes is _no_bytes:
        token_bytes = lambda token: tokenizer.decode_bytes([token])
    return generate_with(engine, prompt, params, token_bytes, _go_on)


def greedy_tokens(engine, prompt: list[int], new_tokens: int) -> list[int]:
    """Greedy ids through the cache (the reference's `greedy_tokens` recomputes everything each step;
    the ids are the same)."""
    return generate(engine, prompt, GenerateParams.greedy(new_tokens)).tokens
