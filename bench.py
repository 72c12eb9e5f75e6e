#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run is the Qwen3-8B shape (36 layers, width 4096, 32 query heads over
8 KV heads of 128, feed-forward 12288, vocabulary 151936, separate head) in
bfloat16 with random weights N(0, 0.02) and uniform-random prompts: 8 requests
with 2,048-token prompts are prefilled, then W untimed and K timed decode steps
run through the engine's own loop (scheduler, step function, GPU sampler). One
JSON line goes to standard output: ``value`` is decoded tokens a second at batch
8; ``prefill`` is one 2,048-token prompt in one step; ``roofline`` prices the
decode step against 8 TB/s by the bytes it must read (every weight once and the
keys and values of the live requests); ``points`` holds batch 1 and batch 64 and the further sizes
(the same shape at batch 8 over 14,000-token and at batch 64 over 8,000-token contexts and an 8,192-token
prompt; the Qwen3-32B shape, all 64 layers, at batch 1, 8 and 64 and prompts of 2,048 and 16,384 tokens; the
Qwen3-4B shape serving 128 requests, whose other figures are in ``serve_128_4b``), ``points_frac`` each
point's fraction of its roofline; ``kernel_ms`` the decode step's GPU time by kernel class with the bytes
each class reads. A run whose logits are not finite or whose tokens lie outside the vocabulary prints no line.
``--serve N`` runs a continuous-batching workload of N requests instead (the reference's replay harness
feeds its scheduler synthetic arrivals the same way, crates/scheduler/src/replay.rs:180-217).
``--shape 4b`` and ``--shape 32b`` run the same measurement at the Qwen3-4B and Qwen3-32B layer sizes.
The reference publishes no number at this size (its own are Qwen3-0.6B on a
laptop GPU, bench/gate-fixture.md:66-74), so ``vs_baseline`` is null.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12                       # bytes a second
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN3_8B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 36,
    "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "intermediate_size": 12288, "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "max_position_embeddings": 4096, "attention_bias": False,
}


# the other two full-size shapes the engine is sized for (tied head at 2560 wide; 64 query heads at 5120 wide)
QWEN3_4B = dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, tie_word_embeddings=True,
                max_position_embeddings=8192)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64,
                 intermediate_size=25600, max_position_embeddings=16384)
SHAPES = {"8b": ("Qwen3-8B", QWEN3_8B), "4b": ("Qwen3-4B", QWEN3_4B), "32b": ("Qwen3-32B", QWEN3_32B)}


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def linear_params(raw: dict) -> int:
    """Matrix elements a token passes through: layers and head (the embedding is a row read)."""
    h, L = raw["hidden_size"], raw["num_hidden_layers"]
    nq = raw["num_attention_heads"] * raw["head_dim"]
    nkv = raw["num_key_value_heads"] * raw["head_dim"]
    per_layer = h * (nq + 2 * nkv) + nq * h + 3 * h * raw["intermediate_size"]
    return L * per_layer + raw["vocab_size"] * h


def kv_bytes_per_token(raw: dict, elem: int) -> int:
    return 2 * raw["num_hidden_layers"] * raw["num_key_value_heads"] * raw["head_dim"] * elem


class InvalidRun(RuntimeError):
    """A timed run whose results are not those of a working model: no line is printed for it."""


def check_run(engine, raw, requests, what: str) -> None:
    """Refuse a timed run unless the logits of its last step are all finite and every token its requests were
    given lies in the vocabulary (the reference's parity harness asserts finiteness before any figure,
    crates/cuda/tests/parity.rs:42-45)."""
    import torch
    logits = engine.runner.last_logits
    if logits is None or logits.numel() == 0 or not bool(torch.isfinite(logits).all()):
        raise InvalidRun(f"{what}: the last step's logits are not all finite")
    V = raw["vocab_size"]
    for r in requests:
        bad = [t for t in r.output if not 0 <= t < V]
        if bad or not r.output:
            raise InvalidRun(f"{what}: request {r.rid!r} was given {len(r.output)} tokens, "
                             f"{len(bad)} of them outside the vocabulary")


def decode_run(engine, raw, batch: int, prompt_len: int, steps: int, warmup: int, seed: int, max_tokens: int):
    """Prefill ``batch`` prompts, then time ``steps`` decode steps. -> (ms a step, mean context)."""
    import torch
    from reinfer_amd.sampling import SamplingParams
    g = torch.Generator().manual_seed(seed)
    # the cap on new tokens is what the run needs: the scheduler admits by what requests may come to hold
    params = SamplingParams(temperature=0.0, max_tokens=max_tokens, ignore_eos=True)
    rids = []
    for _ in range(batch):
        ids = torch.randint(0, raw["vocab_size"], (prompt_len,), generator=g).tolist()
        rids.append(engine.add_request(ids, params))
    sched = engine.scheduler
    # prompts first: until every request is decoding
    while any(not r.decoding for r in sched.running) or sched.waiting:
        engine.step()
    for _ in range(warmup):
        engine.step()
    ctx0 = statistics.mean(r.num_tokens for r in sched.running)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert len(sched.running) == batch, "a request ended inside the timed steps"
    check_run(engine, raw, list(sched.running), f"decode at batch {batch}")
    ctx1 = statistics.mean(r.num_tokens for r in sched.running)
    for r in rids:
        engine.abort(r)
    return dt * 1e3 / steps, 0.5 * (ctx0 + ctx1)


def prefill_run(engine, raw, tokens: int, reps: int, seed: int) -> float:
    """Median milliseconds of one ``tokens``-long prompt run as one step (its first token sampled)."""
    import torch
    from reinfer_amd.sampling import SamplingParams
    g = torch.Generator().manual_seed(seed)
    times = []
    for i in range(reps + 2):
        ids = torch.randint(0, raw["vocab_size"], (tokens,), generator=g).tolist()
        rid = engine.add_request(ids, SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        check_run(engine, raw, list(engine.scheduler.running), f"prefill of {tokens} tokens")
        engine.abort(rid)
        if i >= 2:
            times.append(dt * 1e3)
    return statistics.median(times)


def profile_run(engine, raw, batch: int, prompt_len: int, steps: int, seed: int, max_tokens: int, elem: int):
    """GPU time of a decode step by kernel class: ``steps`` steps run without the captured graph, every call
    into the kernel set between two events, queued behind work that keeps the GPU busy meanwhile so that the
    kernels run back to back as they do in a replayed graph. -> class -> {"ms", "calls", "bytes", "flops"} a
    step (``bytes``: what the class must read, ``flops``: its products; 0 where neither says much)."""
    import torch
    from reinfer_amd import kernels
    from reinfer_amd.kernels.profile import TimedKernels
    from reinfer_amd.sampling import SamplingParams
    g = torch.Generator().manual_seed(seed)
    params = SamplingParams(temperature=0.0, max_tokens=max_tokens, ignore_eos=True)
    rids = [engine.add_request(torch.randint(0, raw["vocab_size"], (prompt_len,), generator=g).tolist(), params)
            for _ in range(batch)]
    sched = engine.scheduler
    while any(not r.decoding for r in sched.running) or sched.waiting:
        engine.step()
    engine.step()
    model = engine.runner.model
    timed = TimedKernels(kernels.current())
    for b in model.blocks:
        for part, attr, role in ((getattr(b, "mixer", None), "w_qkv", "qkv"), (getattr(b, "mixer", None), "w_o", "o_proj"),
                                 (getattr(b, "ffn", None), "w_gate_up", "gate_up"), (getattr(b, "ffn", None), "w_down", "down")):
            w = getattr(part, attr, None)
            if w is not None:
                timed.name_weight(w, role)
    timed.name_weight(model.head, "head")
    graphs, engine.runner.graphs = engine.runner.graphs, None
    try:
        with kernels.use(timed):
            for _ in range(steps):
                timed.hold_back(25.0, engine.device)
                engine.step()
        rows = timed.report()
    finally:
        engine.runner.graphs = graphs
    ctx = statistics.mean(r.num_tokens for r in sched.running)
    for r in rids:
        engine.abort(r)
    h, L, I, V = raw["hidden_size"], raw["num_hidden_layers"], raw["intermediate_size"], raw["vocab_size"]
    nq = raw["num_attention_heads"] * raw["head_dim"]
    nkv = raw["num_key_value_heads"] * raw["head_dim"]
    weights = {"qkv": L * h * (nq + 2 * nkv), "o_proj": L * nq * h, "gate_up": L * 2 * h * I, "down": L * I * h,
               "head": V * h}
    out = {}
    for label, row in sorted(rows.items(), key=lambda kv: -kv[1]["ms"]):
        rec = {"ms": round(row["ms"] / steps, 4), "calls": round(row["calls"] / steps, 1), "bytes": 0, "flops": 0}
        if label in weights:
            rec["bytes"] = weights[label] * elem
            rec["flops"] = 2 * batch * weights[label]
        elif label == "attention":
            rec["bytes"] = int(batch * ctx * kv_bytes_per_token(raw, elem))
            rec["flops"] = int(4 * batch * ctx * nq * L)
        out[label] = rec
    return out


def prefill_flops(raw: dict, T: int) -> float:
    """Every row through every matrix but the head (one row), causal attention (scores and values)."""
    nq = raw["num_attention_heads"] * raw["head_dim"]
    n_lin = linear_params(raw)
    return 2.0 * (n_lin - raw["vocab_size"] * raw["hidden_size"]) * T + 2.0 * raw["vocab_size"] * raw["hidden_size"] \
        + 2.0 * nq * T * T * raw["num_hidden_layers"]


def further_points(args, points: dict, fracs: dict) -> dict:
    """The other sizes the engine is sized for, into ``points`` (tokens a second) and ``fracs`` (the same
    keys: a decode step's bytes a second over the HBM peak, a prompt's flops a second over the matrix peak),
    each with an engine of its own so that the headline's engine keeps the limits it is measured with:
    the Qwen3-8B shape decoding at batch 8 over 14,000-token and at batch 64 over 8,000-token contexts and one
    8,192-token prompt as one step; the Qwen3-32B shape (all 64 layers) decoding at batch 1, 8 and 64 behind
    2,048-token prompts and prompts of 2,048 and 16,384 tokens, each one step; and the Qwen3-4B shape serving
    128 requests by continuous batching (returned: generated tokens a second, preemptions, tokens computed)."""
    import gc
    import torch
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.engine import LLMEngine
    block = 16
    steps, warmup = max(16, args.steps // 4), min(args.warmup, 16)
    elem = 2 if args.dtype == "bfloat16" else 4
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"

    def engine_for(raw, batch, prompt_len, budget, runs=1):
        """Room for ``runs`` decode runs of up to ``batch`` requests one after the other (a run's requests are
        gone before the next starts) and for one prompt of ``budget`` tokens."""
        prompt_steps = batch * -(-prompt_len // budget) if budget < prompt_len else -(-batch * prompt_len // budget) + batch
        max_new = prompt_steps + warmup + steps + 16
        ctx = -(-(max(prompt_len, budget) + max_new + 32) // 1024) * 1024
        raw = dict(raw, max_position_embeddings=ctx)
        blocks = batch * (-(-(prompt_len + max_new + 32) // block) + 1) + -(-(budget + 16) // block) + 8
        log(f"building {raw['num_hidden_layers']} layers, width {raw['hidden_size']}: {batch} requests of "
            f"{prompt_len} tokens, steps of up to {budget} tokens ...")
        eng = LLMEngine(config=config_from_dict(raw), seed=args.seed, dtype=args.dtype, block_size=block,
                        num_blocks=blocks, max_num_seqs=batch, max_num_batched_tokens=budget, max_model_len=ctx)
        return eng, raw, max_new

    def release(eng):
        del eng
        gc.collect()
        torch.cuda.empty_cache()

    def decode_point(key, eng, raw, batch, prompt_len, max_new, seed, what):
        ms, ctx = decode_run(eng, raw, batch, prompt_len, steps, warmup, seed, max_new)
        points[key] = round(batch / (ms * 1e-3), 1)
        step_bytes = linear_params(raw) * elem + batch * ctx * kv_bytes_per_token(raw, elem)
        fracs[key] = round(step_bytes / (ms * 1e-3) / HBM_PEAK, 4)
        log(f"decode batch {batch}, {what}, contexts of {ctx:.0f} tokens: {ms:.3f} ms a step, {points[key]:.0f} tok/s, "
            f"{fracs[key]:.3f} of the HBM peak")

    def prefill_point(key, eng, raw, T, seed, what):
        ms = prefill_run(eng, raw, T, reps=3, seed=seed)
        points[key] = round(T / (ms * 1e-3), 1)
        fracs[key] = round(prefill_flops(raw, T) / (ms * 1e-3) / MFMA_PEAK[dkey], 4)
        log(f"prefill {T} tokens, {what}: {ms:.2f} ms, {points[key]:.0f} tok/s, {fracs[key]:.3f} of the MFMA peak")

    eng, raw, max_new = engine_for(QWEN3_8B, 8, 14000, 8192)
    prefill_point("prefill_8192", eng, raw, 8192, args.seed + 11, "Qwen3-8B shape")
    decode_point("decode_b8_ctx14000", eng, raw, 8, 14000, max_new, args.seed + 12, "Qwen3-8B shape")
    release(eng)
    eng, raw, max_new = engine_for(QWEN3_8B, 64, 8000, 8192)
    decode_point("decode_b64_ctx8000", eng, raw, 64, 8000, max_new, args.seed + 14, "Qwen3-8B shape")
    release(eng)
    eng, raw, max_new = engine_for(QWEN3_32B, 64, 2048, 16384)
    name = f"Qwen3-32B shape ({raw['num_hidden_layers']} layers)"
    prefill_point("prefill_2048_32b", eng, raw, 2048, args.seed + 15, name)
    prefill_point("prefill_16384_32b", eng, raw, 16384, args.seed + 16, name)
    decode_point("decode_b1_32b", eng, raw, 1, 2048, max_new, args.seed + 17, name)
    decode_point("decode_b8_32b", eng, raw, 8, 2048, max_new, args.seed + 13, name)
    decode_point("decode_b64_32b", eng, raw, 64, 2048, max_new, args.seed + 18, name)
    release(eng)
    serve = serve_measure(args, dict(QWEN3_4B), "Qwen3-4B", 128, None)
    points["serve_128_4b"] = serve["value"]
    return {k: serve[k] for k in ("value", "total_tok_s", "seconds", "steps", "preemptions", "tokens_computed",
                                  "prompt_tokens", "generated_tokens")}


def serve_measure(args, raw, shape_name: str, n_requests: int, num_blocks) -> dict:
    """Continuous batching: ``n_requests`` requests arrive at once, prompts uniform in [64, 4096] tokens and
    outputs uniform in [32, 512], prompts cut into portions under a 2,048-token step budget beside the
    decoding requests. -> the figures of the whole run."""
    import gc
    import random
    import torch
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.engine import LLMEngine
    from reinfer_amd.sampling import SamplingParams
    rng = random.Random(args.seed)
    reqs = [(rng.randint(64, 4096), rng.randint(32, 512)) for _ in range(n_requests)]
    raw["max_position_embeddings"] = max(raw["max_position_embeddings"], 4096 + 512 + 1)
    block = 16
    num_blocks = num_blocks or sum((p + o + block - 1) // block + 1 for p, o in reqs)
    max_seqs = min(n_requests, 128)
    log(f"building {raw['num_hidden_layers']} layers of the {shape_name} shape in {args.dtype}, {num_blocks} cache blocks ...")
    engine = LLMEngine(config=config_from_dict(raw), seed=args.seed, dtype=args.dtype, block_size=block,
                       num_blocks=num_blocks, max_num_seqs=max_seqs, max_num_batched_tokens=2048,
                       max_model_len=raw["max_position_embeddings"])
    g = torch.Generator().manual_seed(args.seed + 1)
    V = raw["vocab_size"]
    for p, o in reqs:
        engine.add_request(torch.randint(0, V, (p,), generator=g).tolist(),
                           SamplingParams(temperature=0.0, max_tokens=o, ignore_eos=True))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps, generated, bad = 0, 0, 0
    while engine.has_unfinished():
        for o in engine.step():
            generated += len(o.token_ids)
            bad += sum(1 for t in o.token_ids if not 0 <= t < V)
        steps += 1
        if steps % 200 == 0:
            log(f"step {steps}: {len(engine.scheduler.running)} running, {len(engine.scheduler.waiting)} waiting")
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    t_in, t_out = sum(p for p, _ in reqs), sum(o for _, o in reqs)
    if generated != t_out or bad:
        raise InvalidRun(f"serving {n_requests} requests: {generated} tokens came back for {t_out} asked for, "
                         f"{bad} of them outside the vocabulary")
    if not bool(torch.isfinite(engine.runner.last_logits).all()):
        raise InvalidRun(f"serving {n_requests} requests: the last step's logits are not all finite")
    stats = engine.cache_stats()
    out = {"value": round(t_out / dt, 1), "total_tok_s": round((t_in + t_out) / dt, 1), "seconds": round(dt, 3),
           "steps": steps, "ms_per_step": round(dt * 1e3 / steps, 4), "preemptions": stats["preemptions"],
           "held_back": stats["held_back"], "tokens_computed": stats["tokens"], "prompt_tokens": t_in,
           "generated_tokens": t_out, "cache_blocks": num_blocks, "block_size": block, "max_num_seqs": max_seqs,
           "layers": raw["num_hidden_layers"]}
    log(f"serving {n_requests} requests, {shape_name} shape: {dt:.2f} s, {out['value']:.0f} generated tok/s, "
        f"{stats['preemptions']} preemptions, {stats['tokens']} tokens computed for {t_in + t_out}")
    del engine
    gc.collect()
    torch.cuda.empty_cache()
    return out


def serve_run(args, raw, shape_name: str) -> int:
    """``--serve N``: one JSON line with generated and total tokens a second over the whole run."""
    m = serve_measure(args, raw, shape_name, args.serve, args.num_blocks)
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": f"generated tok/s, continuous batching of {args.serve} requests ({shape_name} shape, {dkey})",
        "value": m["value"], "unit": "tok/s", "n_gpus": 1, "steps": m["steps"], "warmup": 0,
        "ms_per_step": m["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dkey, "data": "synthetic (uniform-random token ids and lengths, random weights N(0, 0.02))",
        "config": {"model": f"{shape_name} shape", "layers": m["layers"], "requests": args.serve,
                   "prompt_tokens": m["prompt_tokens"], "generated_tokens": m["generated_tokens"], "step_budget": 2048,
                   "max_num_seqs": m["max_num_seqs"], "cache_blocks": m["cache_blocks"], "block_size": m["block_size"],
                   "parallelism": "single GPU"},
        "total_tok_s": m["total_tok_s"], "seconds": m["seconds"],
        "preemptions": m["preemptions"], "held_back": m["held_back"], "tokens_computed": m["tokens_computed"],
    }), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1, 64 and 128 points and the further sizes")
    ap.add_argument("--no-profile", action="store_true", help="skip the per-kernel-class times of the decode step")
    ap.add_argument("--profile-steps", type=int, default=4, help="decode steps timed kernel by kernel")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--serve", type=int, default=0, metavar="REQUESTS",
                    help="instead of the decode measurement: continuous batching of this many requests")
    ap.add_argument("--num-blocks", type=int, default=None, help="with --serve: cache blocks (default: room for all)")
    ap.add_argument("--max-model-len", type=int, default=None, metavar="N",
                    help="context length (default: the shape's: 4096 at 8b, 8192 at 4b, 16384 at 32b)")
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="layer sizes (default: the Qwen3-8B shape)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from reinfer_amd import kernels
    from reinfer_amd.config import config_from_dict
    from reinfer_amd.engine import LLMEngine

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    kernels.current()
    shape_name, shape = SHAPES[args.shape]
    raw = dict(shape)
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    if args.max_model_len:
        raw["max_position_embeddings"] = args.max_model_len
    if args.serve:
        return serve_run(args, raw, shape_name)
    cfg = config_from_dict(raw)
    ctx_len = raw["max_position_embeddings"]
    max_batch = max(args.batch, 1 if args.no_points else 128)
    block = 16
    # a request decodes while later prompts are still being prefilled: one step a portion of a prompt
    budget = max(2048, args.prefill_tokens)
    prompt_steps = max_batch * -(-args.prompt_len // budget)
    need_ctx = max(args.prompt_len + prompt_steps + args.warmup + args.steps + 16, args.prefill_tokens + 8)
    if need_ctx > ctx_len:
        # exactly the steps asked for are timed: a run that outgrows the shape's context gets a longer one
        ctx_len = -(-need_ctx // 1024) * 1024
        raw["max_position_embeddings"] = ctx_len
        cfg = config_from_dict(raw)
        log(f"{max_batch} prompts of {args.prompt_len} tokens, {args.warmup + args.steps} decode steps and a prefill of "
            f"{args.prefill_tokens} need a context of {ctx_len}")
    max_new = prompt_steps + args.warmup + args.steps + 16
    blocks_per_req = -(-(args.prompt_len + max_new + 32) // block) + 1
    num_blocks = max(max_batch * blocks_per_req, -(-(args.prefill_tokens + 16) // block)) + 8
    log(f"building {raw['num_hidden_layers']} layers of the {shape_name} shape in {args.dtype}, random weights ...")
    t0 = time.perf_counter()
    engine = LLMEngine(config=cfg, seed=args.seed, dtype=args.dtype, block_size=block, num_blocks=num_blocks,
                       max_num_seqs=max_batch, max_num_batched_tokens=budget,
                       max_model_len=ctx_len)
    torch.cuda.synchronize()
    log(f"model ready in {time.perf_counter() - t0:.1f} s; {num_blocks} cache blocks of {block}")

    elem = 2 if args.dtype == "bfloat16" else 4
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    n_lin = linear_params(raw)
    kv_tok = kv_bytes_per_token(raw, elem)

    # prefill: one prompt, one step
    T = args.prefill_tokens
    pf_ms = prefill_run(engine, raw, T, reps=5, seed=args.seed + 1)
    pf_flops = prefill_flops(raw, T)
    prefill = {"value": round(T / (pf_ms * 1e-3), 1), "tokens": T, "ms": round(pf_ms, 3),
               "frac": round(pf_flops / (pf_ms * 1e-3) / MFMA_PEAK[dkey], 4)}
    log(f"prefill {T} tokens: {pf_ms:.2f} ms, {prefill['value']:.0f} tok/s, {prefill['frac']:.3f} of the MFMA peak")

    ms, ctx = decode_run(engine, raw, args.batch, args.prompt_len, args.steps, args.warmup, args.seed + 2, max_new)
    value = args.batch / (ms * 1e-3)
    step_bytes = n_lin * elem + args.batch * ctx * kv_tok
    achieved = step_bytes / (ms * 1e-3)
    log(f"decode batch {args.batch}: {ms:.3f} ms a step, {value:.0f} tok/s, {achieved / 1e9:.0f} GB/s")

    points, fracs, serve = {}, {}, None
    if not args.no_points:
        for b in (1, 64, 128):
            steps_b = args.steps if b == 1 else max(16, args.steps // (2 if b == 64 else 4))
            pms, pctx = decode_run(engine, raw, b, args.prompt_len, steps_b, min(args.warmup, 16), args.seed + 3 + b, max_new)
            points[f"decode_b{b}"] = round(b / (pms * 1e-3), 1)
            fracs[f"decode_b{b}"] = round((n_lin * elem + b * pctx * kv_tok) / (pms * 1e-3) / HBM_PEAK, 4)
            log(f"decode batch {b}: {pms:.3f} ms a step, {points[f'decode_b{b}']:.0f} tok/s, "
                f"{fracs[f'decode_b{b}']:.3f} of the HBM peak")

    kernel_ms = None
    if not args.no_profile:
        kernel_ms = profile_run(engine, raw, args.batch, args.prompt_len, args.profile_steps, args.seed + 90, max_new, elem)
        total = sum(r["ms"] for r in kernel_ms.values())
        log(f"decode batch {args.batch}, kernel by kernel (events, no graph): {total:.3f} ms a step: " +
            ", ".join(f"{k} {r['ms'] * 1e3:.0f} us" + (f" ({r['bytes'] / r['ms'] / 1e6:.0f} GB/s)" if r["bytes"] else "")
                      for k, r in kernel_ms.items()))

    peaks = kernels.current().measure_peaks(engine.device)
    if not args.no_points and args.shape == "8b" and not args.layers and args.dtype == "bfloat16":
        import gc
        del engine          # each further size builds an engine of its own
        gc.collect()
        torch.cuda.empty_cache()
        serve = further_points(args, points, fracs)
    log(f"measured on this GPU: a plain read {peaks['hbm_read_GBps']:.0f} GB/s, bfloat16 matrix cores "
        f"{peaks['mfma_bf16_32x32x16_TFLOPs']:.0f} TFLOP/s with 32x32x16 products, {peaks['mfma_bf16_16x16x32_TFLOPs']:.0f} with "
        f"16x16x32 (nominal: {HBM_PEAK / 1e9:.0f} GB/s, {MFMA_PEAK['bf16'] / 1e12:.0f} TFLOP/s)")
    out = {
        "metric": f"decode tok/s at batch {args.batch} ({shape_name} shape, {dkey}, {args.prompt_len}-token prompts)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dkey, "data": "synthetic (uniform-random token ids, random weights N(0, 0.02))",
        "config": {
            "model": f"{shape_name} shape", "layers": raw["num_hidden_layers"], "layers_of_model": full_layers,
            "hidden": raw["hidden_size"], "q_heads": raw["num_attention_heads"],
            "kv_heads": raw["num_key_value_heads"], "head_dim": raw["head_dim"],
            "intermediate": raw["intermediate_size"], "vocab": raw["vocab_size"],
            "tied_head": raw["tie_word_embeddings"], "global_batch": args.batch, "seq_len": ctx_len,
            "prompt_len": args.prompt_len, "mean_context": round(ctx, 1), "block_size": block,
            "parallelism": "single GPU",
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 4)},
        "points": points,
        # the same keys: a decode point's bytes a second over the HBM peak, a prompt point's flops over the matrix peak
        "points_frac": fracs,
        # the Qwen3-4B shape serving 128 requests by continuous batching (prompts 64..4096, outputs 32..512 tokens)
        "serve_128_4b": serve,
        # GPU time of the decode step by kernel class (events around every kernel, outside the captured graph)
        "kernel_ms": kernel_ms,
        # what this GPU gives at best, beside the published peaks that the fractions above use
        "measured_peaks": {k: round(v, 1) for k, v in peaks.items()},
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    try:
        sys.exit(main())
    except InvalidRun as e:
        print(f"bench.py: {e}; no line is printed for an invalid run", file=sys.stderr)
        sys.exit(4)
