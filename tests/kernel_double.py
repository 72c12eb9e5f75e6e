"""A CPU stand-in for the kernel library, for tests of the engine's bookkeeping.

It has the method names and argument meaning of ``reinfer_amd.kernels.ops.HipKernels``
and computes with torch on the CPU, reading and writing the same paged cache
through the same index arrays. With it the ``not gpu`` tests can run the step
function, the cache manager and the scheduler end to end where there is no GPU.
It is not part of the product and nothing in ``reinfer_amd`` imports it; on a GPU
box the tests use the real kernels.
"""
from __future__ import annotations

import torch

from reinfer_amd.cache.layout import unpack_k, unpack_v


def k_index(off, e, d):
    """Element (slot off, e) of a (block, KV head) slab, as csrc/common.h cache_k_index."""
    return (off >> 4) * 16 * d + ((e >> 3) * 16 + (off & 15)) * 8 + (e & 7)


def v_index(off, e, d):
    s = off & 15
    return (off >> 4) * 16 * d + (((e >> 4) * 4 + (s >> 2)) * 16 + (e & 15)) * 4 + (s & 3)


class KernelDouble:
    name = "cpu-double"

    def embed(self, table, ids, out):
        out.copy_(table[ids.long()].float())

    def add_rmsnorm(self, resid, delta, weight, eps, out, rows=None):
        if rows is None:
            if delta is not None:
                resid.add_(delta.float())
            x = resid
        else:
            x = resid[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].float()
        rstd = torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)
        out.copy_((x * rstd * weight.float()).to(out.dtype))

    def qk_norm_rope_cache(self, qkv, q_weight, k_weight, eps, positions, inv_freq, rotary_dim,
                           rope_style, slots, kcache, vcache, num_heads, num_kv_heads, head_dim):
        T = qkv.shape[0]
        d = head_dim
        u = qkv.view(T, num_heads + 2 * num_kv_heads, d).float()
        q, k, v = u[:, :num_heads], u[:, num_heads:num_heads + num_kv_heads], u[:, num_heads + num_kv_heads:]

        def norm(x, w):
            if w is None:
                return x
            return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w.float()

        def rot(x):
            if rotary_dim == 0:
                return x
            half = rotary_dim // 2
            ang = positions.float()[:, None] * inv_freq[:half].float()[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            out = x.clone()
            if rope_style == 0:
                a, b = x[..., :half], x[..., half:rotary_dim]
                out[..., :half] = a * c - b * s
                out[..., half:rotary_dim] = a * s + b * c
            else:
                a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
                out[..., 0:rotary_dim:2] = a * c - b * s
                out[..., 1:rotary_dim:2] = a * s + b * c
            return out

        q = rot(norm(q, q_weight))
        k = rot(norm(k, k_weight))
        qkv.view(T, -1, d)[:, :num_heads] = q.to(qkv.dtype)
        bs = kcache.shape[2] * 16
        kflat, vflat = kcache.view(kcache.shape[0], num_kv_heads, -1), vcache.view(vcache.shape[0], num_kv_heads, -1)
        e = torch.arange(d)
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            kflat[s // bs][:, k_index(s % bs, e, d)] = k[t].to(kcache.dtype)
            vflat[s // bs][:, v_index(s % bs, e, d)] = v[t].to(vcache.dtype)

    GATE_GROUP = 8

    def silu_mul(self, gate_up, out, group=0):
        T, I = out.shape
        if group:
            v = gate_up.view(T, I // group, 2, group).float()
            g, u = v[:, :, 0].reshape(T, I), v[:, :, 1].reshape(T, I)
        else:
            g, u = gate_up[:, :I].float(), gate_up[:, I:].float()
        out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))

    def gated_linear(self, x, weight, out, row_sums=None):
        gu = torch.empty((x.shape[0], weight.shape[0]), dtype=torch.float32)
        self.linear(x, weight, gu)
        if row_sums is not None:
            gu *= self._rstd(row_sums)[:, None]
        self.silu_mul(gu.to(out.dtype), out, self.GATE_GROUP)

    # the accumulating epilogue and the norm that rides on products, so that the parts' use of
    # them runs on the CPU too
    def can_accumulate(self, x, weight):
        return x.shape[0] <= 64

    ROW_PART = 16         # columns of one emitted partial sum
    NORM_ON_PRODUCTS_ROWS = 64

    def skinny_row_parts(self, M, N):
        return -(-N // self._row_part(M))

    def _row_part(self, M):
        return self.ROW_PART if M <= 16 else 1024

    @staticmethod
    def _rstd(row_sums):
        ss, eps, width = row_sums
        return torch.rsqrt(ss.double().sum(0) / width + eps).float()

    def linear_skinny(self, x, weight, out, bias=None, accumulate=False, row_sums=None, emit=None):
        y = x.float() @ weight.float().T
        if row_sums is not None:
            y = y * self._rstd(row_sums)[:, None]
        if bias is not None:
            y = y + bias.float()
        if not accumulate:
            assert emit is None
            out.copy_(y.to(out.dtype))
            return
        out.add_(y.to(out.dtype))
        if emit is not None:
            w, xo, so = emit
            xo.copy_((out.float() * w.float()).to(xo.dtype))
            sq = out.float() ** 2
            part = self._row_part(x.shape[0])
            for p in range(so.shape[0]):
                so[p] = sq[:, p * part:(p + 1) * part].sum(1)

    def attention(self, q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads, head_dim,
                  scale, window, group):
        T = batch.num_tokens
        bs = kcache.shape[2] * 16
        kl, vl = unpack_k(kcache, head_dim), unpack_v(vcache, head_dim)      # [blocks, Hkv, bs, d]
        tables = batch.block_tables[group]
        ratio = num_heads // num_kv_heads
        qh = q[:, :num_heads * head_dim].reshape(T, num_heads, head_dim).float()
        for t in range(T):
            seq = int(batch.seq_of_token[t])
            p = int(batch.positions[t])
            lo = max(0, p - window + 1) if window > 0 else 0
            keys = torch.arange(lo, p + 1)
            blk = tables[seq, keys // bs].long()
            K = kl[blk, :, keys % bs, :].float()        # [n, Hkv, d]
            V = vl[blk, :, keys % bs, :].float()
            for a in range(num_heads):
                s = (K[:, a // ratio, :] @ qh[t, a]) * scale
                pr = torch.softmax(s, dim=0)
                out[t, a * head_dim:(a + 1) * head_dim] = (pr @ V[:, a // ratio, :]).to(out.dtype)

    attention_plain = attention

    def linear(self, x, weight, out, bias=None):
        y = x.float() @ weight.float().T
        if bias is not None:
            y = y + bias.float()
        out.copy_(y.to(out.dtype))

    linear_plain = linear

    def filter_logits(self, logits, params, histories):
        import plain_qwen3 as plain
        for i, (p, hist) in enumerate(zip(params, histories)):
            win = list(hist[-p.repeat_last_n:]) if p.repeat_last_n > 0 else []
            logits[i] = plain.filter_logits(
                logits[i], max(0.0, p.temperature), top_k=p.top_k or 0, top_p=p.top_p or 0.0,
                min_p=p.min_p or 0.0, repeat_penalty=p.repeat_penalty or 0.0,
                frequency_penalty=p.frequency_penalty or 0.0, presence_penalty=p.presence_penalty or 0.0,
                window=win, logit_bias=p.logit_bias).float()

    def sample(self, logits, temperature, seeds, positions, tokens):
        from plain_qwen3 import mix64, splitmix64, unit_from_u64
        import math
        for r in range(logits.shape[0]):
            T = float(temperature[r])
            best, idx = float("-inf"), -1
            base = splitmix64((int(seeds[r]) & ((1 << 64) - 1)) ^ ((int(positions[r]) * 0x9E3779B97F4A7C15) & ((1 << 64) - 1)))
            for v, x in enumerate(logits[r].tolist()):
                if not math.isfinite(x):
                    continue
                if T > 0:
                    u = unit_from_u64(mix64(base ^ mix64(v)))
                    if u <= 0:
                        continue
                    x = torch.tensor(x, dtype=torch.float32) / torch.tensor(T, dtype=torch.float32) \
                        - torch.log(-torch.log(torch.tensor(u, dtype=torch.float32)))
                    x = float(x)
                if x > best:
                    best, idx = x, v
            tokens[r] = idx
