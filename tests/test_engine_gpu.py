"""The engine on the GPU against the plain implementation: whole prompts, decoding, portions, mixed batches."""
import pytest
import torch

from plain import qwen2_plain as plain
from tiny_configs import TINY, random_ids

pytestmark = pytest.mark.gpu

# float32: the reference's own tolerance between its paths is 1e-4 (qwen-infer/src/model.rs:1455-1531);
# logits here are of order 1.  bfloat16: rounding to 8 bits at every layer boundary, a few percent of the
# largest logit at most.
TOL = {"float32": 2e-5, "bfloat16": 4e-2}


@pytest.fixture(scope="module")
def oracle(model_folders):
    cache = {}

    def get(name, ids):
        key = (name, tuple(ids))
        if key not in cache:
            cfg, tensors = plain.load_folder(model_folders[name])
            cache[key] = plain.all_logits(cfg, tensors, ids)
        return cache[key]
    return get


def engine_for(folder, dtype, **kw):
    from tokenizer_amd.engine import Engine, load_model
    return Engine(load_model(folder, dtype), **kw)


def close(got, want, dtype):
    got = got.float().cpu()
    err = float((got - want).abs().max())
    scale = float(want.abs().max())
    assert err <= TOL[dtype] * max(scale, 1.0), f"max abs error {err} against logits up to {scale}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_whole_prompts(model_folders, oracle, name, dtype):
    from tokenizer_amd.engine import StepEntry
    vocab = TINY[name][0]["vocab_size"]
    eng = engine_for(model_folders[name], dtype, num_pages=16, max_requests=4)
    for seed, length in enumerate([1, 5, 17, 31, 64, 100]):
        ids = random_ids(vocab, length, seed)
        eng.add_request(seed)
        got = eng.step([StepEntry(seed, ids, list(range(length)))])
        close(got, oracle(name, ids), dtype)
        eng.end_request(seed)
    eng.cache.check_invariants()
