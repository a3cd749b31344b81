"""A real `Engine` on the CPU for host-side tests: the kernel library is replaced by the plain torch ops
of kernel_refs (a test double; the package has no CPU path of its own)."""
import torch

from kernel_refs import PlainOps


def cpu_engine(folder, num_pages=64, max_requests=8, prefix_cache=False, page_size=16, counting=True):
    from tokenizer_amd.engine import Engine, load_model
    model = load_model(folder, "float32", "cpu", ops=PlainOps())
    engine = Engine(model, num_pages=num_pages, page_size=page_size, max_requests=max_requests, prefix_cache=prefix_cache)
    engine.forwards = []          # token count per entry of every step, in order

    inner = engine.step

    def step(entries, **kw):
        engine.forwards.append([len(e.tokens) for e in entries])
        return inner(entries, **kw)

    if counting:
        engine.step = step
    return engine
