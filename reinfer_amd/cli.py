"""Command line in the reference's manner (bin/reinfer/src/main.rs:247-293).

    reinfer run MODEL [-n MAX_TOKENS] [-t TEMP] [--top-k K] [--top-p P] [--repeat-penalty X]
                      [--seed S] [--max-model-len N] [--perf] [PROMPT ...]

``run`` keeps the reference's option names and meanings (default 256 new
tokens, temperature 1.0). MODEL is a folder with config.json and
model.safetensors. The prompt is the trailing words (else standard input): token
ids as integers, or text if the folder holds a tokenizer.json. Generated token
ids (and text, with a tokenizer) go to standard output, statistics and the
``PERF`` line to standard error (main.rs:700-727). ``generate`` is an alias of
``run``; ``init`` writes a random-weights model folder; ``bench`` measures.
The reference's serve, download, model and doctor verbs have no counterpart here.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List, Optional


def _backend(name: str) -> str:
    """``--backend`` as the reference parses it (bin/reinfer/src/main.rs:80-90): a known name or an
    error that lists the names. Only ``auto`` and ``hip`` exist here."""
    if name in ("auto", "hip"):
        return name
    raise argparse.ArgumentTypeError(f"unknown backend '{name}' (auto|hip)")


def _add_run_args(p: argparse.ArgumentParser) -> None:
    p.add_argument("model", help="model folder (config.json + model.safetensors)")
    p.add_argument("--backend", type=_backend, default="auto", metavar="BACKEND",
                   help="auto|hip: this engine has one backend, the MI355X (main.rs:252 names auto|cuda|ascend|cpu)")
    p.add_argument("-n", dest="max_tokens", type=int, default=256, metavar="MAX_TOKENS",
                   help="max new tokens (hard cap)")
    p.add_argument("-t", dest="temperature", type=float, default=1.0, metavar="TEMP",
                   help="sampling temperature (0 = greedy)")
    p.add_argument("--top-k", type=int, default=None, metavar="K", help="top-k truncation (default: off)")
    p.add_argument("--top-p", type=float, default=None, metavar="P", help="nucleus sampling (default: off)")
    p.add_argument("--min-p", type=float, default=None, metavar="P", help="min-p filter (default: off)")
    p.add_argument("--repeat-penalty", type=float, default=None, metavar="PENALTY",
                   help="repeat penalty (> 1.0 to act, e.g. 1.1)")
    p.add_argument("--seed", type=int, default=None, metavar="SEED", help="RNG seed (deterministic when set)")
    p.add_argument("--max-model-len", type=int, default=None, metavar="N",
                   help="effective context window (default: max_position_embeddings)")
    p.add_argument("--perf", action="store_true", help="print a machine-parseable perf line")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--allow-extra-tensors", action="store_true",
                   help="leave tensors of the folder that the model does not declare unread instead of refusing them")
    p.add_argument("--num-blocks", type=int, default=None, help="cache blocks (default: from free memory)")
    p.add_argument("--max-num-seqs", type=int, default=64)
    p.add_argument("--max-num-batched-tokens", type=int, default=2048)
    p.add_argument("--prompt-len", type=int, default=None, metavar="N",
                   help="use N seeded random token ids as the prompt")


def _load_tokenizer(model_dir: str):
    import os
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    try:
        from tokenizers import Tokenizer
        return Tokenizer.from_file(path)
    except Exception as e:   # a broken tokenizer file must not stop id-based use
        print(f"reinfer: tokenizer.json not usable ({e}); token ids only", file=sys.stderr)
        return None


def _prompt_ids(args, vocab: int, tokenizer) -> List[int]:
    if args.prompt_len is not None:
        import torch
        g = torch.Generator().manual_seed(args.seed if args.seed is not None else 0)
        return torch.randint(0, vocab, (args.prompt_len,), generator=g).tolist()
    words = [w for w in args.prompt if w != "--"]
    if not words:
        words = sys.stdin.read().split()
    if not words:
        raise SystemExit("reinfer: empty prompt")
    try:
        return [int(w.strip(",")) for w in words]
    except ValueError:
        if tokenizer is None:
            raise SystemExit("reinfer: the prompt is not a list of token ids and the model folder has no tokenizer.json")
        return tokenizer.encode(" ".join(words)).ids


def cmd_run(args) -> int:
    from .engine import LLMEngine
    from .sampling import SamplingParams
    t_load = time.perf_counter()
    engine = LLMEngine(args.model, dtype=args.dtype, max_model_len=args.max_model_len,
                       block_size=args.block_size, num_blocks=args.num_blocks,
                       max_num_seqs=args.max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens,
                       seed=args.seed or 0, allow_unexpected=args.allow_extra_tensors)
    extra = engine.runner.load_report.get("unexpected") or []
    if extra:
        print(f"reinfer: {len(extra)} tensors of the folder are not part of the model and were left unread "
              f"({', '.join(extra[:4])}{', ...' if len(extra) > 4 else ''})", file=sys.stderr)
    t_load = time.perf_counter() - t_load
    tokenizer = _load_tokenizer(args.model)
    ids = _prompt_ids(args, engine.runner.spec.vocab_size, tokenizer)
    params = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            min_p=args.min_p, repeat_penalty=args.repeat_penalty, seed=args.seed,
                            max_tokens=args.max_tokens)
    import torch
    t0 = time.perf_counter()
    out = engine.generate([ids], params)[0]
    torch.cuda.synchronize() if engine.device.type == "cuda" else None
    total = time.perf_counter() - t0
    print(" ".join(str(t) for t in out.token_ids))
    if tokenizer is not None:
        print(tokenizer.decode(out.token_ids))
    n = len(out.token_ids)
    first = engine.timings.get("first_step_s", 0.0)
    tpot = (total - first) / max(n - 1, 1)           # excludes the first token (main.rs:704-711)
    print(f"{n} tokens in {total:.3f}s, {n / total:.1f} tok/s, first-token {first * 1e3:.1f}ms "
          f"(load {t_load:.1f}s, finish: {out.finish_reason})", file=sys.stderr)
    if args.perf:
        print(f"PERF model={args.model} tokens={n} tpot_ms={tpot * 1e3:.3f} tok_s={1.0 / tpot if tpot > 0 else 0:.2f} "
              f"first_token_ms={first * 1e3:.3f} dtype={args.dtype} preemptions={out.preemptions}", file=sys.stderr)
    return 0


def cmd_init(args) -> int:
    from .config import config_from_dict
    from .weights import write_model_folder
    with open(args.config, "r", encoding="utf-8") as f:
        cfg = config_from_dict(json.load(f))
    out = write_model_folder(cfg, args.seed, args.out, dtype=args.dtype)
    print(out)
    return 0


def cmd_bench(args) -> int:
    import os
    import runpy
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.argv = ["bench.py"] + args.rest
    runpy.run_path(os.path.join(root, "bench.py"), run_name="__main__")
    return 0


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="reinfer", description="Qwen3-class inference on one MI355X")
    sub = ap.add_subparsers(dest="verb", required=True)
    for verb in ("run", "generate"):
        p = sub.add_parser(verb, help="generate from a prompt")
        _add_run_args(p)
        p.set_defaults(fn=cmd_run)
    p = sub.add_parser("init", help="write a random-weights model folder from a config.json and a seed")
    p.add_argument("config", help="a config.json")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--out", required=True)
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.set_defaults(fn=cmd_init)
    p = sub.add_parser("bench", help="throughput measurement (see bench.py --help)")
    p.add_argument("rest", nargs=argparse.REMAINDER)
    p.set_defaults(fn=cmd_bench)
    argv = list(sys.argv[1:] if argv is None else argv)
    # the prompt is what follows "--", else the trailing words no option takes
    # (the reference's trailing_var_arg, bin/reinfer/src/main.rs:290-292)
    prompt: List[str] = []
    if "--" in argv:
        cut = argv.index("--")
        argv, prompt = argv[:cut], argv[cut + 1:]
    if argv and argv[0] == "bench":
        # everything behind the verb is bench.py's, options first or not
        args = argparse.Namespace(verb="bench", rest=argv[1:] + (["--"] + prompt if prompt else []), fn=cmd_bench)
        return args.fn(args)
    args, extra = ap.parse_known_args(argv)
    if extra:
        if args.verb not in ("run", "generate") or any(w.startswith("-") and not w.lstrip("-").isdigit() for w in extra):
            ap.error("unrecognized arguments: " + " ".join(extra))
        prompt = extra + prompt
    args.prompt = prompt
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
