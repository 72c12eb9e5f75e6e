"""Plain, slow Qwen3 dense decoder: whole sequences, no cache, one function a part.

Written from the reference's formulas; each function cites where the reference
computes the same thing. It shares no code with ``reinfer_amd``: it reads the
raw config.json dictionary and a ``name -> tensor`` dictionary and works in
float64 (or any dtype asked for) on the CPU.

Paths are into the reference tree (LeonRust/reinfer).
"""
from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional, Sequence

import torch


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w over the last axis.

    crates/kernels/src/refs.rs:10-18 (rms_norm_ref); GPU twin
    crates/cuda/kernels/dense_kernels.cu:59-88: eps inside the root, the weight
    multiplies after the normalisation.
    """
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(mean_sq + eps) * w


def head_norm(u: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """Per-head RMSNorm: every head vector [d] on its own, one weight [d] for all heads.

    u: [T, heads, d]. crates/cuda/tests/engine_vs_cpu.rs:185-195 (q and k, not v,
    same eps as the layer norms); crates/cuda/kernels/dense_kernels.cu:92-123.
    """
    return rms_norm(u, w, eps)


def rope_neox(u: torch.Tensor, positions: torch.Tensor, theta: float) -> torch.Tensor:
    """Half-split rotation of pairs (j, j + d/2) by angle pos * theta^(-2j/d).

    u: [T, heads, d]; positions: [T]. crates/kernels/src/refs.rs:25-37 (rope_ref)
    and crates/cuda/tests/engine_vs_cpu.rs:291-299:
        out[j]       = u[j] cos - u[j+half] sin
        out[j+half]  = u[j] sin + u[j+half] cos
    The frequency denominator is the full head size (2*half).
    """
    d = u.shape[-1]
    half = d // 2
    j = torch.arange(half, dtype=u.dtype)
    inv = torch.pow(torch.tensor(theta, dtype=u.dtype), -2.0 * j / d)
    ang = positions.to(u.dtype)[:, None] * inv[None, :]          # [T, half]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = u[..., :half], u[..., half:]
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     window: int = 0) -> torch.Tensor:
    """Grouped-query causal attention of one sequence.

    q: [T, Hq, d]; k, v: [T, Hkv, d] -> [T, Hq, d]. Query head a reads KV head
    a // (Hq / Hkv) (crates/cuda/kernels/decode_gqa_kernels.cu:84;
    engine_vs_cpu.rs:213). s_t = (q . k_t) * scale for t <= p, softmax with the
    row maximum subtracted, o = sum_t P_t v_t (engine_vs_cpu.rs:210-241;
    crates/kernels/src/refs.rs:99-160). ``window`` W > 0 keeps keys with
    p - t < W; the reference has no window (full causal only).
    """
    T, Hq, d = q.shape
    Hkv = k.shape[1]
    ratio = Hq // Hkv
    out = torch.zeros_like(q)
    for a in range(Hq):
        kh = a // ratio
        s = (q[:, a, :] @ k[:, kh, :].T) * scale                  # [T, T]
        p_idx = torch.arange(T)[:, None]
        t_idx = torch.arange(T)[None, :]
        keep = t_idx <= p_idx
        if window > 0:
            keep = keep & (p_idx - t_idx < window)
        s = torch.where(keep, s, torch.full_like(s, float("-inf")))
        m = s.max(dim=-1, keepdim=True).values
        e = torch.exp(s - m)
        e = torch.where(keep, e, torch.zeros_like(e))
        out[:, a, :] = (e / e.sum(dim=-1, keepdim=True)) @ v[:, kh, :]
    return out


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """down( silu(gate(x)) * up(x) ), silu(g) = g / (1 + exp(-g)); no bias.

    crates/cuda/tests/engine_vs_cpu.rs:246-255; crates/cpu/src/ops.rs:75-92;
    crates/cuda/kernels/dense_kernels.cu:202-213.
    """
    g = x @ w_gate.T
    u = x @ w_up.T
    return (g / (1.0 + torch.exp(-g)) * u) @ w_down.T


def attention_block(xn: torch.Tensor, positions: torch.Tensor, w: Mapping[str, torch.Tensor], prefix: str,
                    Hq: int, Hkv: int, d: int, theta: float, eps: float, window: int) -> torch.Tensor:
    """q/k/v projections, head norm of q and k, rotation, attention, output projection.

    crates/cuda/tests/engine_vs_cpu.rs:179-244 in that order: projections without
    bias, head norm BEFORE rotation, v untouched, scale 1/sqrt(d) on the score.
    """
    T = xn.shape[0]
    q = (xn @ w[prefix + "self_attn.q_proj.weight"].T).reshape(T, Hq, d)
    k = (xn @ w[prefix + "self_attn.k_proj.weight"].T).reshape(T, Hkv, d)
    v = (xn @ w[prefix + "self_attn.v_proj.weight"].T).reshape(T, Hkv, d)
    q = head_norm(q, w[prefix + "self_attn.q_norm.weight"], eps)
    k = head_norm(k, w[prefix + "self_attn.k_norm.weight"], eps)
    q = rope_neox(q, positions, theta)
    k = rope_neox(k, positions, theta)
    o = causal_attention(q, k, v, 1.0 / math.sqrt(d), window)
    return o.reshape(T, Hq * d) @ w[prefix + "self_attn.o_proj.weight"].T


def layer_windows(cfg: Mapping) -> List[int]:
    n = cfg["num_hidden_layers"]
    types = cfg.get("layer_types")
    if types is not None:
        return [cfg["sliding_window"] if t == "sliding_attention" else 0 for t in types]
    if cfg.get("use_sliding_window", False):
        first = cfg.get("max_window_layers", n)
        return [cfg["sliding_window"] if i >= first else 0 for i in range(n)]
    return [0] * n


def forward(cfg: Mapping, weights: Mapping[str, torch.Tensor], tokens: Sequence[int],
            dtype: torch.dtype = torch.float64, start_pos: int = 0,
            rows: Optional[Sequence[int]] = None) -> torch.Tensor:
    """Logits [T, V] of one whole sequence (with ``rows``: of those positions only, [len(rows), V]; the
    layers still run every position, only the head's product is smaller).

    Order of work: crates/cuda/tests/engine_vs_cpu.rs:162-281 (embedding row,
    per layer: norm, attention, residual add, norm, SwiGLU, residual add; final
    norm; head). Tied head: the embedding matrix (crates/cpu/src/model.rs:218-225).
    ``start_pos`` shifts all positions (only distances count in the result).
    """
    x = hidden_states(cfg, weights, tokens, dtype, start_pos)[-1]
    w = {k: weights[k].to(dtype) for k in ("model.norm.weight", "model.embed_tokens.weight", "lm_head.weight")
         if k in weights}
    eps = cfg.get("rms_norm_eps", 1e-5)
    if rows is not None:
        x = x[torch.tensor(list(rows), dtype=torch.long)]
    xn = rms_norm(x, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return xn @ head.T


def hidden_states(cfg: Mapping, weights: Mapping[str, torch.Tensor], tokens: Sequence[int],
                  dtype: torch.dtype = torch.float64, start_pos: int = 0) -> List[torch.Tensor]:
    """The hidden state [T, hidden] behind the embedding and behind every layer (layers + 1 tensors):
    what the reference reads back layer by layer when it looks for the first layer that differs
    (crates/cuda/src/engine.rs:3744-3765); same order of work as :func:`forward`."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    h = cfg["hidden_size"]
    Hq = cfg["num_attention_heads"]
    Hkv = cfg.get("num_key_value_heads", Hq)
    d = cfg.get("head_dim", h // Hq)
    eps = cfg.get("rms_norm_eps", 1e-5)
    theta = cfg.get("rope_theta", 1_000_000.0)
    windows = layer_windows(cfg)
    ids = torch.tensor(list(tokens), dtype=torch.long)
    positions = torch.arange(len(tokens)) + start_pos
    x = w["model.embed_tokens.weight"][ids]
    out = [x]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        xn = rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_block(xn, positions, w, p, Hq, Hkv, d, theta, eps, windows[i])
        xn = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"])
        out.append(x)
    return out


def argmax_first(logits: torch.Tensor) -> int:
    """Lowest id among equal maxima (crates/cuda/src/engine.rs:6512-6520, strict '>')."""
    best, idx = float("-inf"), 0
    for i, v in enumerate(logits.tolist()):
        if v > best:
            best, idx = v, i
    return idx


def greedy_generate(cfg: Mapping, weights: Mapping[str, torch.Tensor], prompt: Sequence[int], n: int,
                    dtype: torch.dtype = torch.float64) -> List[int]:
    """n greedy tokens; the first comes from the logits at the prompt's last
    position (the aligned loop of crates/cuda/tests/parity.rs:14-20)."""
    toks = list(prompt)
    out: List[int] = []
    for _ in range(n):
        nxt = argmax_first(forward(cfg, weights, toks, dtype)[-1])
        out.append(nxt)
        toks.append(nxt)
    return out


# ---- sampling (pure functions of seed, position and token id) -----------------

_M = (1 << 64) - 1


def splitmix64(x: int) -> int:
    """crates/scheduler/src/rng.rs:17-32; vectors at rng.rs:83-87."""
    z = (x + 0x9E3779B97F4A7C15) & _M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
    return z ^ (z >> 31)


def mix64(z: int) -> int:
    """The z stage alone (crates/cuda/kernels/sampler_kernel.cu:62-66, smix_mix)."""
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
    return z ^ (z >> 31)


def unit_from_u64(x: int) -> float:
    """Top 24 bits over 2^24 (crates/cuda/kernels/sampler_kernel.cu:68-70)."""
    return (x >> 40) / 16777216.0


def filter_logits(logits: torch.Tensor, temperature: float, *, top_k: int = 0, top_p: float = 0.0,
                  min_p: float = 0.0, repeat_penalty: float = 0.0, frequency_penalty: float = 0.0,
                  presence_penalty: float = 0.0, window: Sequence[int] = (),
                  logit_bias: Sequence = ()) -> torch.Tensor:
    """Logit bias, penalties, then the filters on softmax(logits / T); removed tokens are -inf.

    Bias (crates/cuda/kernels/sampler_kernel.cu:189-203): logit[id] += bias for the
    listed ids, before anything else; a logit that is not finite stays as it is.

    Penalties (crates/cuda/kernels/sampler_kernel.cu:207-221): for a token that
    occurs cnt > 0 times in the window, logit -= cnt * freq + pres, then logit > 0
    is divided by the repetition penalty, else multiplied. Filters, if T > 0
    (sampler_kernel.cu:20-43): min_p keeps p >= min_p * max p; top_k keeps the k
    largest, lower id first among equals; top_p keeps, within what is left, the
    values p >= theta with theta the largest value whose kept mass reaches
    top_p times the mass left (ties at the boundary are all kept).
    """
    l = logits.clone().double()
    V = l.numel()
    for t, b in logit_bias:
        if 0 <= t < V and torch.isfinite(l[t]):
            l[t] = l[t] + float(torch.tensor(b, dtype=torch.float32))
    if window and (repeat_penalty > 1 or frequency_penalty > 0 or presence_penalty > 0):
        counts: Dict[int, int] = {}
        for t in window:
            counts[t] = counts.get(t, 0) + 1
        for t, c in counts.items():
            x = float(l[t])
            x -= frequency_penalty * c + presence_penalty
            if repeat_penalty > 1:
                x = x / repeat_penalty if x > 0 else x * repeat_penalty
            l[t] = x
    if not temperature > 0:
        return l
    p = torch.softmax(l / temperature, dim=0)
    keep = torch.ones(V, dtype=torch.bool)
    if min_p > 0:
        keep &= p >= min_p * p.max()
    if 0 < top_k < V:
        order = torch.sort(l, descending=True, stable=True).indices[:top_k]      # stable: lower id first among equals
        kk = torch.zeros(V, dtype=torch.bool)
        kk[order] = True
        keep &= kk
    if 0 < top_p < 1:
        need = top_p * float(p[keep].sum())
        vals, _ = torch.sort(p[keep], descending=True)
        first = int((torch.cumsum(vals, dim=0) >= need).nonzero()[0])   # the largest theta whose mass reaches the need
        keep &= p >= vals[first]
    l[~keep] = float("-inf")
    return l
