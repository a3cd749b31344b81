"""A real `Engine` on the CPU for host-side tests: the kernel library is replaced by the plain torch ops
of kernel_refs (a test double; the package has no CPU path of its own)."""
import torch

from kernel_refs import PlainOps


def cpu_engine(folder, num_pages=64, max_requests=8, prefix_cache=False, page_size=16, counting=True, bursts=False):
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

    def decode_run(rids, tokens, n_steps, on_step=None, draw=None):
        """`Engine.decode_greedy` (and, with `draw`, `Engine.decode_sampled`) as it behaves with captured graphs, one
        step at a time on the CPU: the ids of a step reach `on_step` one step late, when the next step has already
        run (and taken its uniform numbers), and when `on_step` returns False the run ends behind that further
        step, whose ids are returned as well."""
        from tokenizer_amd.engine import StepEntry
        if n_steps <= 0:
            return []
        ran, picked, current, go_on = [], [], [int(t) for t in tokens], True
        for k in range(n_steps):
            entries = [StepEntry(rid, [token], [0]) for rid, token in zip(rids, current)]
            logits = engine.step(entries)
            current = [int(t) for t in engine.argmax(logits)]
            if draw is not None:                              # rows with temperature 0 keep the greedy pick
                temperature, top_p, uniform = draw(k)
                warm = [row for row, t in enumerate(temperature) if t != 0]
                drawn = engine.sample(logits, warm, [temperature[r] for r in warm], [top_p[r] for r in warm],
                                      [uniform[r] for r in warm]) if warm else []
                for row, token in zip(warm, drawn):
                    current[row] = int(token)
            ran.append(current)
            if k > 0:
                picked.append(ran[k - 1])
                if on_step is not None and on_step(k - 1, picked[-1]) is False:
                    go_on = False
            if not go_on:
                break
        picked.append(ran[len(picked)])
        if on_step is not None and go_on:
            on_step(len(picked) - 1, picked[-1])
        return picked

    # The scheduler runs greedy decode steps in bursts only over an engine that says it replays graphs; nothing is
    # captured here, the double only takes the scheduler (and greedy `generate`) down that road when asked to.
    if bursts:
        engine.decode_greedy = lambda rids, tokens, n_steps, on_step=None: decode_run(rids, tokens, n_steps, on_step)
        engine.decode_sampled = lambda rids, tokens, n_steps, draw, on_step=None: decode_run(rids, tokens, n_steps, on_step, draw)
        engine.use_graphs = True
        engine._replays = lambda entries: False
    return engine
