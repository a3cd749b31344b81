"""Command line in the manner of the reference's `qwen-infer` (qwen-infer/src/main.rs:12-148).

    qwen-infer --model DIR [--max-tokens N] [--temperature T] [--top-p P] [--seed N] [--stop STRING]... <prompt>

Flags, defaults and the lines printed are the reference's: the generated text on standard
output; prompt ids, parameters, generated ids, the stop reason and the timings on standard
error.  The model comes from a folder (config.json, model.safetensors, tokenizer.json and,
if present, generation_config.json) instead of a download.  `--token-ids` takes the prompt as
comma-separated ids for folders without a tokenizer; `--random-weights SEED` needs only the folder's
config.json; `--dtype` is bf16 (default) or fp32; `--num-blocks` is the size of the page pool.
"""
from __future__ import annotations

import os
import sys
import time

USAGE = ("usage: qwen-infer --model DIR [--dtype bf16|fp32] [--num-blocks N] [--random-weights SEED] [--max-tokens N] "
         "[--temperature T] [--top-p P] [--seed N] [--stop STRING]... [--token-ids] <prompt>")


class ArgError(ValueError):
    pass


def parse_args(argv: list[str]) -> dict:
    args = {"prompt": None, "max_tokens": 20, "temperature": 0.0, "top_p": 1.0, "seed": 0, "stop": [],
            "model": None, "dtype": "bfloat16", "num_blocks": 256, "token_ids": False, "help": False,
            "random_weights": None}
    it = iter(argv)

    def value(flag: str) -> str:
        try:
            return next(it)
        except StopIteration:
            raise ArgError(f"{flag} needs a value") from None

    for arg in it:
        if arg in ("--help", "-h"):
            args["help"] = True
        elif arg == "--max-tokens":
            raw = value(arg)
            try:
                args["max_tokens"] = int(raw)
                if args["max_tokens"] < 0:
                    raise ValueError
            except ValueError:
                raise ArgError(f"--max-tokens {raw}") from None
        elif arg == "--temperature":
            raw = value(arg)
            try:
                args["temperature"] = float(raw)
            except ValueError:
                raise ArgError(f"--temperature {raw}") from None
        elif arg == "--top-p":
            try:
                args["top_p"] = float(value(arg))
            except ValueError:
                raise ArgError("--top-p wants a number") from None
        elif arg == "--seed":
            try:
                args["seed"] = int(value(arg))
            except ValueError:
                raise ArgError("--seed wants an integer") from None
        elif arg == "--num-blocks":
            try:
                args["num_blocks"] = int(value(arg))
            except ValueError:
                raise ArgError("--num-blocks wants an integer") from None
        elif arg == "--random-weights":
            try:
                args["random_weights"] = int(value(arg))
            except ValueError:
                raise ArgError("--random-weights wants an integer seed") from None
        elif arg == "--stop":
            args["stop"].append(value(arg))
        elif arg == "--model":
            args["model"] = value(arg)
        elif arg == "--dtype":
            args["dtype"] = value(arg)
        elif arg == "--token-ids":
            args["token_ids"] = True
        elif arg.startswith("-") and len(arg) > 1:
            raise ArgError(f"unknown argument {arg}")
        else:
            if args["prompt"] is not None:
                raise ArgError(f"only one prompt is accepted (got {arg!r} as well)")
            args["prompt"] = arg
    return args


def _plain_number(value: float) -> str:
    """A float as the reference's `{}` prints it (qwen-infer/src/main.rs:33-36): whole numbers without a
    fraction ("0", "1"), others as short as they read back ("0.7")."""
    text = repr(float(value))
    return text[:-2] if text.endswith(".0") else text


def main(argv: list[str] | None = None) -> int:
    try:
        args = parse_args(sys.argv[1:] if argv is None else argv)
    except ArgError as err:
        print(f"error: {err}", file=sys.stderr)
        return 2
    if args["help"]:
        print(USAGE, file=sys.stderr)
        return 0
    if args["prompt"] is None or args["model"] is None:
        print(USAGE, file=sys.stderr)
        return 1

    from .config import load_config
    from .engine import Engine, Failure, GenerateParams, StopReason, load_eos_token_ids, load_model, random_model
    from .tokenizer import load_tokenizer

    folder = args["model"]
    tokenizer = None
    if args["token_ids"]:
        prompt_ids = [int(part) for part in args["prompt"].replace(",", " ").split()]
    else:
        tokenizer = load_tokenizer(folder)          # of the kind the folder's tokenizer.json declares
        prompt_ids = tokenizer.encode(args["prompt"])
    if not prompt_ids:
        print("error: prompt encoded to no tokens", file=sys.stderr)
        return 1
    print(f"prompt ids ({len(prompt_ids)}): {prompt_ids}", file=sys.stderr)

    params = GenerateParams.greedy(args["max_tokens"])
    params.temperature, params.top_p, params.seed, params.stop = (args["temperature"], args["top_p"],
                                                                   args["seed"], args["stop"])
    eos_path = os.path.join(folder, "generation_config.json")
    if os.path.exists(eos_path):
        params.eos = load_eos_token_ids(eos_path)
    print(f"max_tokens {params.max_tokens} temperature {_plain_number(params.temperature)} "
          f"top_p {_plain_number(params.top_p)} seed {params.seed} eos {params.eos}", file=sys.stderr)

    if args["random_weights"] is not None:      # the folder then needs its config.json only
        model = random_model(load_config(folder), args["random_weights"], args["dtype"])
    else:
        model = load_model(folder, args["dtype"])
    engine = Engine(model, num_pages=args["num_blocks"], max_requests=1)
    token_bytes = (lambda token: tokenizer.decode_bytes([token])) if tokenizer else \
        (lambda token: f"{token} ".encode())
    started = time.perf_counter()
    # The request takes the way every request of a serving engine takes: queued, admitted with pages for its whole
    # prompt, the prompt run in portions under the token budget, decoded (greedy steps in bursts), finished, freed.
    request = engine.add_request(prompt_ids, params, token_bytes=token_bytes)
    generated = engine.run()[request]
    elapsed = time.perf_counter() - started
    if isinstance(generated, Failure):
        print(f"error: {generated.message}", file=sys.stderr)
        return 1
    print(generated.text)
    print(f"generated ids: {generated.tokens}", file=sys.stderr)
    print(f"stop: {generated.reason.value}", file=sys.stderr)
    n = len(generated.tokens)
    if n == 0 or generated.decode == 0:
        print(f"prefill {generated.prefill:.4f} s, decode {generated.decode:.4f} s, {n} tokens "
              f"(KV cache, total {elapsed:.4f} s)", file=sys.stderr)
    else:
        print(f"prefill {generated.prefill:.4f} s, decode {generated.decode:.4f} s, {n / generated.decode:.4f} tok/s "
              f"({n} tokens, KV cache, total {elapsed:.4f} s)", file=sys.stderr)
    if generated.reason == StopReason.Eos:
        print("stopped on eos before max_tokens", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
