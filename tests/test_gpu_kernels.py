"""Each kernel alone against a plain float reference of the same operation, at
sizes other than the engine's tiny models: widths and vocabularies that are no
power of two, head sizes in steps of 16, odd head counts and groups."""
import math

import pytest
import torch

import plain_qwen3 as plain
from reinfer_amd import kernels
from reinfer_amd.cache.layout import pack_k, pack_v, unpack_k, unpack_v

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# one rounding of the result to bfloat16 is 2^-9 relative; float results differ by summation order only
OUT_TOL = {"float32": 1e-5, "bfloat16": 2 ** -8}


def ops():
    k = kernels.current()
    assert k.name == "hip-gfx950"
    return k


def close(got, ref, tol):
    got, ref = got.double().cpu(), ref.double().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs().max().item()
    scale = ref.abs().max().item()
    assert err <= tol * max(scale, 1e-6), f"max error {err} against scale {scale}"


def kt(kc):
    """The tests build caches as [blocks, kv heads, slot, d]; the kernels take them in
    tiles of 16 slots in matrix-core operand order."""
    return pack_k(kc)


def vt(vc):
    return pack_v(vc)


class FakeBatch:
    def __init__(self, q_lens, starts, tables):
        self.num_seqs = len(q_lens)
        self.num_tokens = sum(q_lens)
        self.q_lens, self.starts = list(q_lens), list(starts)
        seq, pos = [], []
        for i, (q, s) in enumerate(zip(q_lens, starts)):
            seq += [i] * q
            pos += list(range(s, s + q))
        self.seq_of_token = torch.tensor(seq, dtype=torch.int32, device=DEV)
        self.positions = torch.tensor(pos, dtype=torch.int32, device=DEV)
        cu = [0]
        for q in q_lens:
            cu.append(cu[-1] + q)
        self.cu_tokens = torch.tensor(cu, dtype=torch.int32, device=DEV)
        self.start_pos = torch.tensor(starts, dtype=torch.int32, device=DEV)
        self.ctx_lens = torch.tensor([s + q for s, q in zip(starts, q_lens)], dtype=torch.int32, device=DEV)
        self.block_tables = [tables]
        self.max_q_len = max(q_lens)
        self.max_ctx_len = max(s + q for s, q in zip(starts, q_lens))
        self.extra = {}


# ------------------------------------------------------------------ rows
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed(dtype):
    table = torch.randn(77, 200, device=DEV).to(DT[dtype])
    ids = torch.tensor([0, 76, 5, 5, 13], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 200, device=DEV)
    ops().embed(table, ids, out)
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("dtype,wdtype", [("float32", "float32"), ("bfloat16", "bfloat16"), ("bfloat16", "float32")])
@pytest.mark.parametrize("h", [100, 98, 4096, 4104, 20000])
def test_add_rmsnorm(dtype, wdtype, h):
    torch.manual_seed(h)
    T, eps = 7, 1e-5
    resid = torch.randn(T, h, device=DEV) * 3
    delta = torch.randn(T, h, device=DEV).to(DT[dtype])
    w = (torch.rand(h, device=DEV) + 0.5).to(DT[wdtype])
    want_resid = resid + delta.float()
    ref = plain.rms_norm(want_resid.double().cpu(), w.double().cpu(), eps)
    # gathered form leaves the residual alone
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    out_g = torch.empty(3, h, device=DEV, dtype=DT[dtype])
    keep = resid.clone()
    ops().add_rmsnorm(resid, delta, w, eps, out_g, rows)
    assert torch.equal(resid, keep)
    close(out_g, ref[[6, 0, 3]], OUT_TOL[dtype])
    # in place
    out = torch.empty(T, h, device=DEV, dtype=DT[dtype])
    ops().add_rmsnorm(resid, delta, w, eps, out)
    assert torch.allclose(resid, want_resid, rtol=0, atol=1e-6)
    close(out, ref, OUT_TOL[dtype])
    # no addend: norm only (reference vector: rms_norm_ref([3,4],[1,2],0) = [3,8]/sqrt(12.5),
    # crates/kernels/src/refs.rs:168-178)
    r2 = torch.tensor([[3.0, 4.0]], device=DEV)
    o2 = torch.empty(1, 2, device=DEV)
    ops().add_rmsnorm(r2, None, torch.tensor([1.0, 2.0], device=DEV), 0.0, o2)
    assert torch.allclose(o2.cpu(), torch.tensor([[3.0, 8.0]]) / math.sqrt(12.5), atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_silu_mul(dtype):
    T, I = 5, 333
    gu = (torch.randn(T, 2 * I, device=DEV) * 4).to(DT[dtype])
    out = torch.empty(T, I, device=DEV, dtype=DT[dtype])
    ops().silu_mul(gu, out)
    g, u = gu[:, :I].double(), gu[:, I:].double()
    close(out, g / (1 + torch.exp(-g)) * u, OUT_TOL[dtype])
    # gate and up interleaved in runs of 3
    I2 = 330
    gu2 = gu[:, :2 * I2].contiguous()
    out2 = torch.empty(T, I2, device=DEV, dtype=DT[dtype])
    ops().silu_mul(gu2, out2, 3)
    v = gu2.view(T, I2 // 3, 2, 3).double()
    g, u = v[:, :, 0].reshape(T, I2), v[:, :, 1].reshape(T, I2)
    close(out2, g / (1 + torch.exp(-g)) * u, OUT_TOL[dtype])
    # widths in steps of 8 take the vector kernel: both layouts
    I3 = 328
    gu3 = gu[:, :2 * I3].contiguous()
    out3 = torch.empty(T, I3, device=DEV, dtype=DT[dtype])
    ops().silu_mul(gu3, out3)
    g, u = gu3[:, :I3].double(), gu3[:, I3:].double()
    close(out3, g / (1 + torch.exp(-g)) * u, OUT_TOL[dtype])
    ops().silu_mul(gu3, out3, 8)
    v = gu3.view(T, I3 // 8, 2, 8).double()
    g, u = v[:, :, 0].reshape(T, I3), v[:, :, 1].reshape(T, I3)
    close(out3, g / (1 + torch.exp(-g)) * u, OUT_TOL[dtype])


def rope_reference(x, positions, theta, rotary_dim, style):
    """x [T, H, d] double; rotates the first rotary_dim entries of every head."""
    half = rotary_dim // 2
    j = torch.arange(half, dtype=torch.float64)
    ang = positions.double()[:, None] * theta ** (-2.0 * j / rotary_dim)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if style == 0:
        a, b = x[..., :half], x[..., half:rotary_dim]
        out[..., :half], out[..., half:rotary_dim] = a * c - b * s, a * s + b * c
    else:
        a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        out[..., 0:rotary_dim:2], out[..., 1:rotary_dim:2] = a * c - b * s, a * s + b * c
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,Hkv,d,rot,style,norm", [
    (4, 2, 16, 16, 0, True), (14, 2, 48, 48, 0, True), (5, 5, 128, 128, 0, True),
    (3, 1, 80, 32, 0, False), (6, 3, 64, 64, 1, True), (32, 8, 128, 128, 0, True), (2, 1, 256, 256, 0, True)])
@pytest.mark.parametrize("T", [11, 45, 200])  # few tokens: a wave per head; from 192: a workgroup per token
def test_qk_norm_rope_cache(dtype, Hq, Hkv, d, rot, style, norm, T):
    torch.manual_seed(d + Hq)
    bs, nblk, eps, theta = 16, max(9, T // 16 + 3), 1e-6, 10000.0
    width = (Hq + 2 * Hkv) * d
    qkv = torch.randn(T, width, device=DEV).to(DT[dtype])
    src = qkv.clone()
    qw = (torch.rand(d, device=DEV) + 0.5).to(DT[dtype]) if norm else None
    kw = (torch.rand(d, device=DEV) + 0.5).to(DT[dtype]) if norm else None
    pos_l = [0, 1, 15, 16, 17, 100, 255, 3, 4, 5, 6]
    slots_l = [5 * bs + 3, 0, 8 * bs + 15, -1, 2 * bs, 2 * bs + 1, 7 * bs + 9, 1 * bs + 1, 1 * bs + 2, 1 * bs + 3, 4 * bs]
    g = torch.Generator().manual_seed(T)
    free = [x for x in torch.randperm(nblk * bs, generator=g).tolist() if x not in slots_l]
    while len(pos_l) < T:
        pos_l.append(int(torch.randint(0, 128, (1,), generator=g)))   # float angles: their rounding grows with the position
        slots_l.append(-1 if len(pos_l) % 7 == 0 else free.pop())
    positions = torch.tensor(pos_l, dtype=torch.int32, device=DEV)
    slots = torch.tensor(slots_l, dtype=torch.int32, device=DEV)
    kc = torch.full((nblk, Hkv, bs // 16, 16 * d), float("nan"), device=DEV, dtype=DT[dtype])
    vc = torch.full_like(kc, float("nan"))
    j = torch.arange(max(rot // 2, 1), dtype=torch.float64)
    inv_freq = (theta ** (-2.0 * j / max(rot, 1))).float().to(DEV)
    ops().qk_norm_rope_cache(qkv, qw, kw, eps, positions, inv_freq, rot, style, slots, kc, vc, Hq, Hkv, d)

    u = src.double().cpu().view(T, Hq + 2 * Hkv, d)
    q, k, v = u[:, :Hq], u[:, Hq:Hq + Hkv], u[:, Hq + Hkv:]
    if norm:
        q = plain.head_norm(q, qw.double().cpu(), eps)
        k = plain.head_norm(k, kw.double().cpu(), eps)
    if style == 0 and rot == d:
        q_ref, k_ref = plain.rope_neox(q, positions.cpu(), theta), plain.rope_neox(k, positions.cpu(), theta)
    else:
        q_ref = rope_reference(q, positions.cpu(), theta, rot, style)
        k_ref = rope_reference(k, positions.cpu(), theta, rot, style)
    tol = OUT_TOL[dtype]
    kc, vc = unpack_k(kc, d), unpack_v(vc, d)         # [blocks, kv heads, slot, d]
    close(qkv.view(T, -1, d)[:, :Hq], q_ref, tol)
    written = torch.zeros(nblk, bs, dtype=torch.bool)
    for t, s in enumerate(slots_l):
        if s < 0:
            continue
        written[s // bs, s % bs] = True
        close(kc[s // bs, :, s % bs, :], k_ref[t], tol)
        assert torch.equal(vc[s // bs, :, s % bs, :].cpu().double(), v[t])
    # nothing else was touched
    untouched = ~written
    assert torch.isnan(kc.float().cpu().permute(0, 2, 1, 3)[untouched]).all()
    assert torch.isnan(vc.float().cpu().permute(0, 2, 1, 3)[untouched]).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,Hkv,d", [(4, 2, 16), (5, 5, 128), (32, 8, 128), (2, 1, 256), (6, 3, 64), (40, 40, 128),
                                      (9, 9, 32)])
def test_qk_norm_rope_cache_values_of_four_slots_in_a_row(dtype, Hq, Hkv, d):
    """A prompt's tokens sit in slots that follow each other: where four tokens in a row fill slots 4k .. 4k + 3
    the per-token kernel writes their values in one piece. Runs of slots that start at a multiple of 4, one that
    starts beside it, one with a token that stores nothing inside a group of four, and a ragged end."""
    T, bs = 203, 16
    nblk = 40
    torch.manual_seed(d)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * d, device=DEV).to(DT[dtype])
    src = qkv.clone()
    slots_l = [32 + t for t in range(80)] + [321 + t for t in range(40)] + [480 + t for t in range(83)]
    slots_l[50] = -1
    slots = torch.tensor(slots_l, dtype=torch.int32, device=DEV)
    # every token another position, all below 128: the kernel's angles are floats, whose rounding grows with the position
    positions = ((torch.arange(T, dtype=torch.int32) * 5) % 128).to(DEV)
    kc = torch.full((nblk, Hkv, bs // 16, 16 * d), float("nan"), device=DEV, dtype=DT[dtype])
    vc = torch.full_like(kc, float("nan"))
    inv_freq = (10000.0 ** (-torch.arange(0, d, 2).double() / d)).float().to(DEV)
    qw = (torch.rand(d, device=DEV) + 0.5).to(DT[dtype])
    kw = (torch.rand(d, device=DEV) + 0.5).to(DT[dtype])
    ops().qk_norm_rope_cache(qkv, qw, kw, 1e-6, positions, inv_freq, d, 0, slots, kc, vc, Hq, Hkv, d)
    u = src.view(T, Hq + 2 * Hkv, d)
    v = u[:, Hq + Hkv:]
    # the four tokens of such a group also share the work on their keys, each with the angles of its own position
    q_ref = plain.rope_neox(plain.head_norm(u[:, :Hq].double().cpu(), qw.double().cpu(), 1e-6), positions.cpu(), 10000.0)
    k_ref = plain.rope_neox(plain.head_norm(u[:, Hq:Hq + Hkv].double().cpu(), kw.double().cpu(), 1e-6),
                            positions.cpu(), 10000.0)
    close(qkv.view(T, -1, d)[:, :Hq], q_ref, OUT_TOL[dtype])
    vc, kc = unpack_v(vc, d), unpack_k(kc, d)
    written = torch.zeros(nblk, bs, dtype=torch.bool)
    for t, sl in enumerate(slots_l):
        if sl < 0:
            continue
        written[sl // bs, sl % bs] = True
        assert torch.equal(vc[sl // bs, :, sl % bs, :], v[t]), t
        close(kc[sl // bs, :, sl % bs, :], k_ref[t], OUT_TOL[dtype])
    assert torch.isnan(vc.float().cpu().permute(0, 2, 1, 3)[~written]).all()
    assert torch.isnan(kc.float().cpu().permute(0, 2, 1, 3)[~written]).all()


@pytest.mark.parametrize("Hq,Hkv,d,rot,style,norm", [(4, 2, 16, 16, 0, True), (3, 1, 80, 32, 0, False),
                                                      (6, 3, 64, 64, 1, True), (32, 8, 128, 128, 0, True)])
@pytest.mark.parametrize("T,S,carried", [(5, 1, False), (33, 4, True), (64, 3, True), (20, 2, False), (40, 6, True),
                                         (18, 7, False), (64, 11, True)])
def test_qk_norm_rope_cache_from_the_ranges_of_a_split_product(Hq, Hkv, d, rot, style, norm, T, S, carried):
    """The same kernel fed with the float results of the K ranges of a split product, which it adds
    itself, and with the partial sums of squares of an RMSNorm carried by that product: equal to
    the plain kernel on the sum, scaled."""
    torch.manual_seed(d + Hq + T)
    bs, nblk, eps, theta = 16, T // 16 + 3, 1e-6, 10000.0
    width = (Hq + 2 * Hkv) * d
    ranges = torch.randn(S, T, width, device=DEV)
    total = ranges.double().sum(0)
    row_sums = None
    if carried:
        parts, hidden, neps = 3, 100, 1e-5
        ss = torch.rand(parts, T, device=DEV) * hidden
        row_sums = (ss, neps, hidden)
        total = total * torch.rsqrt(ss.double().sum(0) / hidden + neps)[:, None]
    qw = (torch.rand(d, device=DEV) + 0.5).to(torch.bfloat16) if norm else None
    kw = (torch.rand(d, device=DEV) + 0.5).to(torch.bfloat16) if norm else None
    g = torch.Generator().manual_seed(T)
    positions = torch.randint(0, 128, (T,), generator=g).to(torch.int32).to(DEV)
    slots_l = torch.randperm(nblk * bs, generator=g)[:T].tolist()
    slots_l[T // 2] = -1
    slots = torch.tensor(slots_l, dtype=torch.int32, device=DEV)
    kc = torch.full((nblk, Hkv, bs // 16, 16 * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    vc = torch.full_like(kc, float("nan"))
    j = torch.arange(max(rot // 2, 1), dtype=torch.float64)
    inv_freq = (theta ** (-2.0 * j / max(rot, 1))).float().to(DEV)
    q_out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().qk_norm_rope_cache_ranges(ranges, row_sums, q_out, qw, kw, eps, positions, inv_freq, rot, style, slots,
                                    kc, vc, Hq, Hkv, d)
    u = total.cpu().view(T, Hq + 2 * Hkv, d)
    q, k, v = u[:, :Hq], u[:, Hq:Hq + Hkv], u[:, Hq + Hkv:]
    if norm:
        q = plain.head_norm(q, qw.double().cpu(), eps)
        k = plain.head_norm(k, kw.double().cpu(), eps)
    q_ref = rope_reference(q, positions.cpu(), theta, rot, style)
    k_ref = rope_reference(k, positions.cpu(), theta, rot, style)
    tol = OUT_TOL["bfloat16"]
    kc, vc = unpack_k(kc, d), unpack_v(vc, d)
    close(q_out.view(T, Hq, d), q_ref, tol)
    for t, sl in enumerate(slots_l):
        if sl < 0:
            continue
        close(kc[sl // bs, :, sl % bs, :], k_ref[t], tol)
        close(vc[sl // bs, :, sl % bs, :], v[t], tol)
    assert int(torch.isnan(kc.float()).any(-1).sum()) == (nblk * bs - (T - 1)) * Hkv


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotation_by_hand_through_the_position_part_and_the_cache_index(dtype):
    """Numbers written out, not computed by the expression under test: head size 16, theta 10000, so pair j
    turns by position * 10^(-j/2) (crates/kernels/src/refs.rs:25-37: the exponent is -2j over the whole head
    size). Position 3: pair 6 turns by 0.003, pair 2 by 0.3. The frequencies come from the position part the
    engine builds, and the key is read back from the cache by the index formula of csrc/common.h
    (K tile [d/8][16 slots][8], V tile [d/16][4][16][4]) spelt out here, not through cache.layout."""
    from reinfer_amd.config.schema import PositionSpec
    from reinfer_amd.parts import lookup
    d, bs, nblk = 16, 32, 3
    part = lookup("position", "rope_neox")(PositionSpec("rope_neox", rotary_dim=d, theta=10000.0), torch.device(DEV))
    assert torch.allclose(part.inv_freq.cpu().double(), torch.tensor(
        [1.0, 0.31622776601683794, 0.1, 0.031622776601683794, 0.01, 0.0031622776601683794, 0.001,
         0.00031622776601683794], dtype=torch.float64), rtol=1e-7, atol=0)
    qkv = torch.zeros(1, 3 * d, device=DEV)
    qkv[0, 6] = 1.0                     # q = e_6: a of pair 6
    qkv[0, d + 10] = 2.0                # k = 2 e_10: b of pair 2
    qkv[0, 2 * d:] = torch.arange(1, d + 1)
    qkv = qkv.to(DT[dtype])
    kc = torch.full((nblk, 1, bs // 16, 16 * d), float("nan"), device=DEV, dtype=DT[dtype])
    vc = torch.full_like(kc, float("nan"))
    block, off = 1, 21                  # the second tile of the block, slot 5 of the tile
    ops().qk_norm_rope_cache(qkv, None, None, 0.0, torch.tensor([3], dtype=torch.int32, device=DEV), part.inv_freq,
                             part.rotary_dim, part.style, torch.tensor([block * bs + off], dtype=torch.int32, device=DEV),
                             kc, vc, 1, 1, d)
    tol = 1e-6 if dtype == "float32" else 2 ** -8
    q = qkv[0, :d].double().cpu()
    want_q = torch.zeros(d, dtype=torch.float64)
    want_q[6], want_q[14] = 0.999995500003375, 0.002999995500002025            # cos 0.003, sin 0.003
    assert (q - want_q).abs().max().item() <= tol
    want_k = torch.zeros(d, dtype=torch.float64)
    want_k[2], want_k[10] = -2 * 0.29552020666133955, 2 * 0.955336489125606    # -b sin 0.3, b cos 0.3
    kflat, vflat = kc[block, 0].reshape(-1).double().cpu(), vc[block, 0].reshape(-1).double().cpu()
    seen_k, seen_v = set(), set()
    for e in range(d):
        ik = (off // 16) * 16 * d + ((e // 8) * 16 + off % 16) * 8 + e % 8
        iv = (off // 16) * 16 * d + (((e // 16) * 4 + (off % 16) // 4) * 16 + e % 16) * 4 + (off % 16) % 4
        assert abs(kflat[ik].item() - want_k[e].item()) <= tol, (e, kflat[ik].item(), want_k[e].item())
        assert vflat[iv].item() == float(e + 1)
        seen_k.add(ik)
        seen_v.add(iv)
    assert len(seen_k) == d and len(seen_v) == d
    # nothing else of the cache was written
    assert int((~torch.isnan(kflat)).sum()) == d and int((~torch.isnan(vflat)).sum()) == d
    assert torch.isnan(kc[[0, 2]].float()).all() and torch.isnan(vc[[0, 2]].float()).all()


def test_rotation_depends_on_distance_only():
    """<R_p q, R_t k> is a function of p - t: shift all positions and nothing changes."""
    Hq, Hkv, d, bs = 2, 1, 32, 16
    torch.manual_seed(0)
    base = torch.randn(2, (Hq + 2 * Hkv) * d, device=DEV)
    j = torch.arange(d // 2, dtype=torch.float64)
    inv_freq = (10000.0 ** (-2.0 * j / d)).float().to(DEV)
    dots = []
    for shift in (0, 37):
        qkv = base.clone()
        kc = torch.zeros(4, Hkv, bs // 16, 16 * d, device=DEV)
        vc = torch.zeros_like(kc)
        pos = torch.tensor([5 + shift, 9 + shift], dtype=torch.int32, device=DEV)
        slots = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
        ops().qk_norm_rope_cache(qkv, None, None, 0.0, pos, inv_freq, d, 0, slots, kc, vc, Hq, Hkv, d)
        dots.append((qkv[1, :d] * unpack_k(kc, d)[0, 0, 0]).sum().item())
    assert abs(dots[0] - dots[1]) < 1e-4 * max(1.0, abs(dots[0]))


# ------------------------------------------------------------- attention
def attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window):
    """Gathers each request's keys through its block table and calls the plain attention."""
    bs = kc.shape[2]
    out, t0 = [], 0
    for i, (ql, st) in enumerate(zip(q_lens, starts)):
        n = st + ql
        keys = torch.arange(n)
        blk = tables[i, keys // bs].long().cpu()
        K = kc.double().cpu()[blk, :, keys % bs, :]
        V = vc.double().cpu()[blk, :, keys % bs, :]
        K = torch.nan_to_num(K)          # positions a window has passed may hold anything
        V = torch.nan_to_num(V)
        Q = torch.zeros(n, Hq, d, dtype=torch.float64)
        Q[st:] = q[t0:t0 + ql].double().cpu()
        out.append(plain.causal_attention(Q, K, V, scale, window)[st:])
        t0 += ql
    return torch.cat(out).reshape(-1, Hq * d)


def make_paged_case(dtype, Hq, Hkv, d, q_lens, starts, bs=16, seed=0, poison=True, window=0):
    g = torch.Generator().manual_seed(seed)
    n_seqs = len(q_lens)
    ctx = [s + q for s, q in zip(starts, q_lens)]
    need = [-(-c // bs) for c in ctx]
    total = sum(need) + 3
    perm = torch.randperm(total, generator=g).tolist()          # shuffled physical blocks
    if window > 0:
        perm = [b for b in perm if b != 0]                      # block 0 is nobody's: it stays NaN (see below)
        total += 1
    width = max(need)
    tables = torch.zeros(n_seqs, width, dtype=torch.int32)
    kc = torch.full((total, Hkv, bs, d), float("nan") if poison else 0.0)
    vc = kc.clone()
    p = 0
    for i in range(n_seqs):
        for b in range(need[i]):
            # As in the engine: a block that lies wholly below the window of the request's first query has
            # been given back, and its table entry reads 0. Here block 0 holds NaN, so a kernel that reads
            # a tile below the window's lower edge shows, whatever its mask then does with the score.
            if window > 0 and (b + 1) * bs - 1 < starts[i] - window + 1:
                tables[i, b] = 0
                continue
            blk = perm[p]
            p += 1
            tables[i, b] = blk
            fill = min(bs, ctx[i] - b * bs)
            kc[blk, :, :fill] = torch.randn(Hkv, fill, d, generator=g)
            vc[blk, :, :fill] = torch.randn(Hkv, fill, d, generator=g)
    T = sum(q_lens)
    q = torch.randn(T, Hq, d, generator=g)
    return (q.to(DT[dtype]).to(DEV), kc.to(DT[dtype]).to(DEV), vc.to(DT[dtype]).to(DEV), tables.to(DEV))


ATT_SHAPES = [(4, 2, 16), (14, 2, 64), (12, 2, 48), (5, 5, 32), (8, 1, 128), (32, 8, 128), (2, 1, 256), (6, 3, 80)]
ATT_BATCHES = [
    ([1], [0]), ([1], [15]), ([1], [16]), ([1, 1, 1], [31, 32, 700]),
    ([33], [0]), ([2, 17, 1, 64], [0, 30, 99, 1]), ([130], [5]), ([200, 1], [0, 257]),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,Hkv,d", ATT_SHAPES)
def test_attention_plain(dtype, Hq, Hkv, d):
    for bi, (q_lens, starts) in enumerate(ATT_BATCHES):
        for window in (0, 19):
            q, kc, vc, tables = make_paged_case(dtype, Hq, Hkv, d, q_lens, starts, seed=bi)
            batch = FakeBatch(q_lens, starts, tables)
            T = sum(q_lens)
            out = torch.empty(T, Hq * d, device=DEV, dtype=DT[dtype])
            scale = 1.0 / math.sqrt(d)
            ops().attention_plain(q.view(T, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window, 0)
            ref = attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window)
            close(out, ref, OUT_TOL[dtype])


def test_attention_reduces_to_library_routine():
    """No rotation, full heads (Hkv = Hq), whole prompt: torch's own attention."""
    Hq, d, n = 3, 32, 50
    q, kc, vc, tables = make_paged_case("float32", Hq, Hq, d, [n], [0], seed=5, poison=False)
    batch = FakeBatch([n], [0], tables)
    out = torch.empty(n, Hq * d, device=DEV)
    ops().attention_plain(q.view(n, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hq, d, 1 / math.sqrt(d), 0, 0)
    keys = torch.arange(n)
    K = kc[tables[0, keys // 16].long(), :, keys % 16, :].transpose(0, 1)     # [H, n, d]
    V = vc[tables[0, keys // 16].long(), :, keys % 16, :].transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1)[None], K[None], V[None], is_causal=True)
    close(out, ref[0].transpose(0, 1).reshape(n, Hq * d), 1e-5)


# ---------------------------------------------------------------- linear
@pytest.mark.parametrize("M,N,K", [(1, 100, 64), (7, 333, 129), (64, 1000, 96), (130, 257, 515), (3, 5, 1)])
@pytest.mark.parametrize("din,dout", [("float32", "float32"), ("bfloat16", "bfloat16"), ("bfloat16", "float32")])
def test_linear_plain(M, N, K, din, dout):
    torch.manual_seed(M * N)
    x = torch.randn(M, K, device=DEV).to(DT[din])
    w = torch.randn(N, K, device=DEV).to(DT[din])
    b = torch.randn(N, device=DEV).to(DT[din])
    out = torch.empty(M, N, device=DEV, dtype=DT[dout])
    ops().linear_plain(x, w, out)
    ref = x.double() @ w.double().T
    close(out, ref, OUT_TOL[dout])
    ops().linear_plain(x, w, out, b)
    close(out, ref + b.double(), OUT_TOL[dout])


def test_float32_linear_is_true_float32():
    """(1 + 2^-12)^2 - 1 = 2^-11 + 2^-24: inputs rounded to 10 or 7 mantissa bits give 0."""
    a = 1.0 + 2.0 ** -12
    x = torch.tensor([[a, 1.0]], device=DEV)
    w = torch.tensor([[a, -1.0]], device=DEV)
    out = torch.empty(1, 1, device=DEV)
    ops().linear_plain(x, w, out)
    assert abs(out.item() - (2.0 ** -11 + 2.0 ** -24)) < 1e-7     # float rounding of a*a itself


# -------------------------------------------------------------- sampling
def test_sample_greedy_first_maximum():
    V = 151936 // 8 + 5
    logits = torch.randn(4, V, device=DEV)
    logits[0, 77] = 50.0
    logits[0, 9000] = 50.0                  # equal maxima: the lowest id wins
    logits[1, V - 1] = 60.0
    logits[2, :] = float("nan")
    logits[3, 5] = float("inf")             # non-finite never wins
    logits[3, 4000] = 40.0
    tokens = torch.empty(4, dtype=torch.int32, device=DEV)
    zeros = torch.zeros(4, device=DEV)
    seeds = torch.zeros(4, dtype=torch.int64, device=DEV)
    pos = torch.zeros(4, dtype=torch.int32, device=DEV)
    ops().sample(logits, zeros, seeds, pos, tokens)
    assert tokens.tolist() == [77, V - 1, -1, 4000]


def gumbel_reference(logits_row, T, seed, position):
    M = (1 << 64) - 1
    base = plain.splitmix64((seed & M) ^ ((position * 0x9E3779B97F4A7C15) & M))
    best, idx, second = -1e30, -1, -1e30
    for v, x in enumerate(logits_row):
        u = plain.unit_from_u64(plain.mix64(base ^ plain.mix64(v)))
        if u <= 0:
            continue
        key = x / T - math.log(-math.log(u))
        if key > best:
            second, best, idx = best, key, v
        elif key > second:
            second = key
    return idx, best - second


def test_sample_temperature_matches_formula_and_ignores_batch():
    V, n = 1000, 12
    torch.manual_seed(3)
    logits = torch.randn(n, V, device=DEV) * 2
    temps = torch.full((n,), 0.8, device=DEV)
    seeds = torch.arange(1000, 1000 + n, dtype=torch.int64, device=DEV)
    pos = torch.arange(5, 5 + n, dtype=torch.int32, device=DEV)
    tokens = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample(logits, temps, seeds, pos, tokens)
    rows = logits.cpu().tolist()
    checked = 0
    for r in range(n):
        idx, gap = gumbel_reference(rows[r], 0.8, 1000 + r, 5 + r)
        if gap > 1e-4:                      # float and double keys can only disagree on near ties
            assert tokens[r].item() == idx
            checked += 1
    assert checked >= n - 2
    # the same row alone, in another place of the batch: the same token
    alone = torch.empty(1, dtype=torch.int32, device=DEV)
    ops().sample(logits[7:8], temps[:1], seeds[7:8], pos[7:8], alone)
    assert alone.item() == tokens[7].item()


def test_sample_distribution_is_softmax():
    """Gumbel-max draws from softmax(logits / T): frequencies over many seeds."""
    V, n, T = 6, 20000, 0.7
    row = torch.tensor([0.0, 1.0, -1.0, 2.0, 0.5, -3.0])
    logits = row.repeat(n, 1).to(DEV)
    temps = torch.full((n,), T, device=DEV)
    seeds = torch.arange(n, dtype=torch.int64, device=DEV) * 7919 + 13
    pos = torch.zeros(n, dtype=torch.int32, device=DEV)
    tokens = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample(logits, temps, seeds, pos, tokens)
    freq = torch.bincount(tokens.cpu().long(), minlength=V).double() / n
    p = torch.softmax(row.double() / T, dim=0)
    # 4 standard deviations of a binomial frequency
    assert ((freq - p).abs() <= 4 * torch.sqrt(p * (1 - p) / n) + 1e-4).all(), (freq, p)


@pytest.mark.parametrize("V", [1000, 151936])
def test_filter_logits_against_plain(V):
    """Penalties, min-p, top-k and top-p against the plain chain; spaced logits keep every boundary clear."""
    from reinfer_amd.sampling import SamplingParams
    g = torch.Generator().manual_seed(V)
    base = torch.randn(V, generator=g) * 3
    cases = [
        dict(temperature=0.7, top_k=5), dict(temperature=1.0, top_p=0.8), dict(temperature=1.3, min_p=0.05),
        dict(temperature=0.9, top_k=40, top_p=0.5, min_p=0.01),
        dict(temperature=1.0, repeat_penalty=1.3, frequency_penalty=0.4, presence_penalty=0.2, top_k=7),
        dict(temperature=0.0, repeat_penalty=1.5, top_k=3),          # greedy: penalties only
        dict(temperature=1.0, top_k=1),
        # a bias lifts an unlikely token over the favourite and sinks the favourite; with penalties and a filter
        dict(temperature=0.0, logit_bias=((3, 40.0), (int(base.argmax()), -50.0))),
        dict(temperature=0.8, logit_bias=((5, 25.0), (999, -3.5), (0, 1.25)), top_k=4, frequency_penalty=0.3),
    ]
    hist = torch.randint(0, V, (90,), generator=g).tolist()
    hist += hist[:10] + [int(base.argmax())] * 3                    # repeats, and the favourite three times
    params = [SamplingParams(**c) for c in cases]
    logits = base.repeat(len(cases), 1).to(DEV)
    logits[0, 17] = float("nan")                                     # a non-finite logit is never kept
    ops().filter_logits(logits, params, [hist] * len(cases))
    for i, c in enumerate(cases):
        row = base.clone()
        if i == 0:
            row[17] = float("-inf")
        kw = {k: v for k, v in c.items() if k != "temperature"}
        ref = plain.filter_logits(row, c["temperature"], window=hist[-64:], **kw)
        if i == 7:
            assert int(ref.argmax()) == 3                                # the bias decides the greedy token
        got = logits[i].cpu().double()
        kept_ref, kept_got = torch.isfinite(ref), torch.isfinite(got)
        if i == 0:
            kept_got[17] = False
        assert torch.equal(kept_ref, kept_got), (i, int(kept_ref.sum()), int(kept_got.sum()))
        assert torch.allclose(got[kept_got], ref[kept_ref], rtol=1e-6, atol=1e-6)


def test_filtered_sampling_stays_inside_top_k():
    from reinfer_amd.sampling import Sampler, SamplingParams
    V, n = 500, 300
    torch.manual_seed(3)
    row = torch.randn(V, device=DEV)
    top = set(torch.topk(row, 4).indices.tolist())
    sampler = Sampler(torch.device(DEV))
    params = [SamplingParams(temperature=1.5, top_k=4)] * n
    toks = sampler.sample(row.repeat(n, 1), params, list(range(n)), [7] * n, [[1, 2, 3]] * n)
    assert set(toks) <= top and len(set(toks)) >= 3


# ------------------------------------------------- bfloat16 kernels of serving
@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 32, 33, 40, 48, 49, 64])
@pytest.mark.parametrize("N,K", [(100, 64), (333, 136), (1000, 96), (6144, 4096), (257, 520), (16, 8),
                                 (48, 12288), (130, 1160)])
@pytest.mark.parametrize("dout", ["bfloat16", "float32"])
@pytest.mark.parametrize("wide", [False, True])
def test_linear_skinny(M, N, K, dout, wide):
    """Both kernels for few rows (waves split K / waves share the activations), at every row count."""
    torch.manual_seed(M * N + K)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    b = torch.randn(N, device=DEV).to(torch.bfloat16)
    out = torch.full((M, N), float("nan"), device=DEV, dtype=DT[dout])
    ops().linear_skinny(x, w, out, wide=wide)
    ref = x.double() @ w.double().T
    close(out, ref, OUT_TOL[dout])
    ops().linear_skinny(x, w, out, b, wide=wide)
    close(out, ref + b.double(), OUT_TOL[dout])
    # the row of a token does not depend on its neighbours: row r of the batch = the single-row product
    one = torch.empty(1, N, device=DEV, dtype=DT[dout])
    ops().linear_skinny(x[M - 1:M], w, one, wide=wide)
    ops().linear_skinny(x, w, out, wide=wide)
    close(one, out[M - 1:M], 1e-6 if dout == "float32" else 2 ** -8)
    # the accumulating epilogue: C += A . W^T into a float matrix
    c0 = torch.randn(M, N, device=DEV)
    c = c0.clone()
    ops().linear_skinny(x, w, c, b, accumulate=True, wide=wide)
    close(c, c0.double() + ref + b.double(), 1e-5)


@pytest.mark.parametrize("M", [1, 7, 16, 20, 33, 48, 64, 65, 200])
@pytest.mark.parametrize("I,K", [(8, 8), (40, 64), (176, 80), (320, 96), (12288, 512), (72, 1032)])
@pytest.mark.parametrize("wide", [False, True])
def test_gated_linear(M, I, K, wide):
    """silu(x Wg^T) * (x Wu^T) with gate and up rows interleaved in runs of 8: the fused epilogue
    (up to 64 rows) and the two-kernel form (more rows) against the separate float products."""
    torch.manual_seed(M + I + K)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    wg = (torch.randn(I, K, device=DEV) * 2 / math.sqrt(K)).to(torch.bfloat16)
    wu = (torch.randn(I, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    w = torch.stack([wg.view(I // 8, 8, K), wu.view(I // 8, 8, K)], dim=1).reshape(2 * I, K).contiguous()
    out = torch.full((M, I), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().gated_linear(x, w, out, wide=wide if M <= 64 else None)
    g = x.double() @ wg.double().T
    u = x.double() @ wu.double().T
    # the two-kernel form rounds gate and up to bfloat16 before the gate: two more roundings
    close(out, g / (1 + torch.exp(-g)) * u, 2 ** -8 if M <= 64 else 3 * 2 ** -8)


@pytest.mark.parametrize("M,N,K,wdt", [(1, 64, 64, torch.float32), (8, 4096, 1024, torch.float32),
                                       (13, 200, 264, torch.bfloat16), (16, 96, 4096, torch.float32),
                                       (23, 1000, 512, torch.bfloat16), (40, 328, 256, torch.float32),
                                       (64, 9000, 128, torch.bfloat16), (64, 48, 1024, torch.float32),
                                       (17, 4096, 4096, torch.bfloat16), (33, 4096, 1024, torch.float32),
                                       (64, 4096, 4096, torch.bfloat16), (48, 5120, 512, torch.bfloat16),
                                       (64, 4096, 12288, torch.bfloat16), (8, 10240, 64, torch.bfloat16)])
def test_rmsnorm_carried_by_two_products(M, N, K, wdt):
    """stream += a . W1^T, then y = rmsnorm(stream; w, eps) . W2^T with no norm kernel: the first
    product also writes bf16(stream * w) and partial sums of squares, the second applies the
    row factor; plain and gated second products, against the same in double precision."""
    torch.manual_seed(M * 7 + N)
    eps = 1e-5
    a = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w1 = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    stream = torch.randn(M, N, device=DEV) * 3
    stream[M // 2] *= 50                                       # one row far larger than the rest
    nw = (1 + 0.3 * torch.randn(N, device=DEV)).to(wdt)
    parts = ops().skinny_row_parts(M, N)
    xs = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    ss = torch.full((parts, M), float("nan"), device=DEV)
    want_stream = stream.double() + a.double() @ w1.double().T
    written = ops().linear_skinny(a, w1, stream, accumulate=True, emit=(nw, xs, ss))
    assert 1 <= written <= parts and torch.isnan(ss[written:]).all()      # room for either kernel's sums; one wrote its own
    ss = ss[:written]
    close(stream, want_stream, 2 ** -8)
    close(xs, stream.double() * nw.double(), 2 ** -8)
    close(ss.sum(0), (stream.double() ** 2).sum(1), 1e-5)
    normed = stream.double() * torch.rsqrt((stream.double() ** 2).mean(1, keepdim=True) + eps) * nw.double()
    if N % 8 == 0:
        J = 80
        w2 = (torch.randn(J, N, device=DEV) / math.sqrt(N)).to(torch.bfloat16)
        bias = torch.randn(J, device=DEV).to(torch.bfloat16)
        for dout in (torch.bfloat16, torch.float32):
            y = torch.full((M, J), float("nan"), device=DEV, dtype=dout)
            ops().linear_skinny(xs, w2, y, bias, row_sums=(ss, eps, N))
            close(y, normed @ w2.double().T + bias.double(), 3 * 2 ** -8)
        wg = (torch.randn(J, N, device=DEV) * 2 / math.sqrt(N)).to(torch.bfloat16)
        wu = (torch.randn(J, N, device=DEV) / math.sqrt(N)).to(torch.bfloat16)
        w = torch.stack([wg.view(J // 8, 8, N), wu.view(J // 8, 8, N)], dim=1).reshape(2 * J, N).contiguous()
        out = torch.full((M, J), float("nan"), device=DEV, dtype=torch.bfloat16)
        ops().gated_linear(xs, w, out, row_sums=(ss, eps, N))
        g, u = normed @ wg.double().T, normed @ wu.double().T
        close(out, g / (1 + torch.exp(-g)) * u, 3 * 2 ** -8)


@pytest.mark.parametrize("M", [3, 16, 24, 32])
def test_wide_gated_product_takes_the_many_partial_sums_of_a_narrow_producer(M):
    """A small product before the norm (up to 32 rows; from 17 on, one that the other kernel would have to
    cut into K ranges) writes one partial sum per 16 columns (256 for a width of 4096); a gated product wide
    enough to fill the chip goes to the kernel whose waves share the activations, and adds them up itself."""
    torch.manual_seed(M)
    N, J, eps = 4096, 12288, 1e-6              # 24576 gated features: 256 workgroups of 96, one a CU
    K = 256 if M <= 16 else 4096               # above 16 rows the producer stays narrow only if the other would cut K
    a = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w1 = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    stream = torch.randn(M, N, device=DEV) * 3
    stream[M // 2] *= 30
    nw = (1 + 0.3 * torch.randn(N, device=DEV)).to(torch.bfloat16)
    parts = ops().skinny_row_parts(M, N)
    assert parts == N // 16
    xs = torch.empty((M, N), device=DEV, dtype=torch.bfloat16)
    ss = torch.empty((parts, M), device=DEV)
    assert ops().linear_skinny(a, w1, stream, accumulate=True, emit=(nw, xs, ss)) == parts
    normed = stream.double() * torch.rsqrt((stream.double() ** 2).mean(1, keepdim=True) + eps) * nw.double()
    wg = (torch.randn(J, N, device=DEV) * 2 / math.sqrt(N)).to(torch.bfloat16)
    wu = (torch.randn(J, N, device=DEV) / math.sqrt(N)).to(torch.bfloat16)
    w = torch.stack([wg.view(J // 8, 8, N), wu.view(J // 8, 8, N)], dim=1).reshape(2 * J, N).contiguous()
    # from 9 rows on this gated product goes to the kernel whose waves share the activations, below that
    # to the one whose workgroups stay: either must take the producer's 256 partial sums a row
    assert kernels.library.load().ra_gemm_wide_preferred(1, M, 2 * J, N) == (1 if M > 8 else 0)
    assert kernels.library.load().ra_gemm_wide_preferred(2, M, N, K) == 0
    out = torch.full((M, J), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().gated_linear(xs, w, out, row_sums=(ss, eps, N))
    g, u = normed @ wg.double().T, normed @ wu.double().T
    close(out, g / (1 + torch.exp(-g)) * u, 3 * 2 ** -8)
    plain_out = torch.full((M, J), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().gated_linear(xs, w, plain_out)                      # and without the carried norm
    g, u = xs.double() @ wg.double().T, xs.double() @ wu.double().T
    close(plain_out, g / (1 + torch.exp(-g)) * u, 3 * 2 ** -8)


@pytest.mark.parametrize("M", [65, 96, 97, 128])
def test_accumulating_product_over_k_ranges_above_64_rows(M):
    """65 to 128 rows: a product that adds into the float stream over a long K is cut into K ranges (six or
    eight row tiles) where that beats the library's product; other products of that many rows are not offered
    (asked for all the same, they add into the stream through the library's product)."""
    lib = kernels.library.load()
    N, K = 2048, 12288
    assert lib.ra_gemm_wide_preferred(2, M, N, K) == 1
    assert lib.ra_gemm_wide_preferred(0, M, N, K) == 0 and lib.ra_gemm_wide_preferred(2, M, 512, 1024) == 0
    assert lib.ra_gemm_wide_preferred(2, 129, N, K) == 0
    torch.manual_seed(M)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    stream = torch.randn(M, N, device=DEV)
    want = stream.double() + x.double() @ w.double().T
    assert ops().can_accumulate(x, w)
    ops().linear_skinny(x, w, stream, accumulate=True)
    close(stream, want, 2 ** -8)
    small = (torch.randn(512, 1024, device=DEV) / 32).to(torch.bfloat16)
    assert not ops().can_accumulate(x[:, :1024], small)         # the library's product and the norm kernel's add are faster
    stream = torch.randn(M, 512, device=DEV)
    want = stream.double() + x[:, :1024].double() @ small.double().T
    ops().linear_skinny(x[:, :1024], small, stream, accumulate=True)
    close(stream, want, 2 ** -8)
    with pytest.raises(kernels.KernelLibraryError, match="rows"):          # the kernel whose waves split K, asked by name
        ops().linear_skinny(x[:, :1024], small, stream, accumulate=True, wide=False)
    ops().linear_skinny(x[:, :1024], small, stream, accumulate=True, wide=True)      # and the other one
    close(stream, want + x[:, :1024].double() @ small.double().T, 2 ** -8)


@pytest.mark.parametrize("M", [65, 100, 128])
@pytest.mark.parametrize("N,K", [(4096, 4096), (2048, 12288), (5120, 8192), (8200, 2560)])
def test_accumulating_product_finishes_the_norm_that_follows(M, N, K):
    """65 to 128 rows: the kernel that adds the K ranges into the stream holds a whole row a workgroup and
    writes the RMSNorm of the new row as well (one, two and four chunks of columns a thread; a width that is
    no multiple of 1024). A product it does not take adds only and says so."""
    torch.manual_seed(M + N)
    eps = 1e-5
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    g = (torch.rand(N, device=DEV) + 0.5).to(torch.bfloat16)
    stream = torch.randn(M, N, device=DEV)
    new = stream.double() + x.double() @ w.double().T
    want = new * torch.rsqrt((new * new).mean(dim=1, keepdim=True) + eps) * g.double()
    assert ops().can_finish_norm(M, N, K)
    normed = torch.full((M, N), float("nan"), device=DEV, dtype=torch.bfloat16)
    assert ops().linear_skinny(x, w, stream, accumulate=True, finish=(g, normed, eps)) is True
    close(stream, new, 2 ** -8)
    close(normed, want, OUT_TOL["bfloat16"])
    # the same rows through the norm kernel
    ref = torch.empty_like(normed)
    ops().add_rmsnorm(stream, None, g, eps, ref)
    close(normed, ref.double(), OUT_TOL["bfloat16"])
    # a small product goes to the library: added, not normed
    small = (torch.randn(512, 1024, device=DEV) / 32).to(torch.bfloat16)
    assert not ops().can_finish_norm(M, 512, 1024) and not ops().can_finish_norm(64, N, K) and not ops().can_finish_norm(129, N, K)
    s2 = torch.randn(M, 512, device=DEV)
    want2 = s2.double() + x[:, :1024].double() @ small.double().T
    n2 = torch.empty(M, 512, device=DEV, dtype=torch.bfloat16)
    assert ops().linear_skinny(x[:, :1024], small, s2, accumulate=True, finish=(g[:512].contiguous(), n2, eps)) is False
    close(s2, want2, 2 ** -8)


@pytest.mark.parametrize("M,N,K", [(129, 520, 264), (700, 96, 1000), (2048, 1024, 4096), (3072, 80, 176)])
def test_accumulating_product_of_many_rows_adds_in_the_library(M, N, K):
    """More rows than the weight-streaming kernels take: the library's product reads and writes the float
    stream itself (bfloat16 operands, float sums), so the addend is never rounded to bfloat16."""
    torch.manual_seed(M + N)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    stream = torch.randn(M, N, device=DEV) * 100                # a bfloat16 addend beside 100 would show at 2**-8
    want = stream.double() + x.double() @ w.double().T
    assert ops().can_accumulate(x, w)
    assert not ops().can_accumulate(torch.empty(ops().LIBRARY_ACCUMULATES_ROWS + 1, K, device=DEV, dtype=torch.bfloat16), w)
    assert ops().linear_skinny(x, w, stream, accumulate=True) is None
    assert (stream.double() - want).abs().max().item() < 2e-3


@pytest.mark.parametrize("M", [3, 12, 40])
def test_linear_over_a_matrix_above_4_gib(M):
    """A vocabulary of 262144 at a width of 8192 is 4.3 GB of weights: past what one 32-bit buffer offset
    spans. The weight-streaming kernels take it (each through the form that addresses it in 64 bits or by
    workgroup), rows at both ends of the matrix included."""
    N, K = 262144, 8192
    g = torch.Generator(device=DEV).manual_seed(M)
    w = torch.empty(N, K, device=DEV, dtype=torch.bfloat16)
    for lo in range(0, N, 32768):                      # in pieces: the float draw of the whole would be 8.6 GB
        w[lo:lo + 32768] = (torch.randn(32768, K, device=DEV, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    x = torch.randn(M, K, device=DEV, generator=g).to(torch.bfloat16)
    out = torch.full((M, N), float("nan"), device=DEV)
    ops().linear(x, w, out)
    for lo in (0, 131072 - 512, N - 1024):             # first rows, rows around the 2 GiB and 4 GiB marks, last rows
        ref = x.double() @ w[lo:lo + 1024].double().T
        close(out[:, lo:lo + 1024], ref, 2 ** -8)
    assert torch.isfinite(out).all()


def test_linear_dispatch_refuses_nothing_silently():
    """Sizes the MFMA kernel does not take go to the plain kernel, not to a wrong result."""
    x = torch.randn(5, 100, device=DEV).to(torch.bfloat16)[:, :99]       # K = 99, odd row stride
    w = torch.randn(7, 99, device=DEV).to(torch.bfloat16)
    out = torch.empty(5, 7, device=DEV, dtype=torch.bfloat16)
    ops().linear(x, w, out)
    close(out, x.double() @ w.double().T, 2 ** -8)
    with pytest.raises(kernels.KernelLibraryError, match="multiples of 8"):
        ops().linear_skinny(x.contiguous(), w, out)
    big = torch.randn(65, 64, device=DEV).to(torch.bfloat16)
    with pytest.raises(kernels.KernelLibraryError, match="at most 64"):
        ops().linear_skinny(big, torch.randn(8, 64, device=DEV).to(torch.bfloat16),
                            torch.empty(65, 8, device=DEV, dtype=torch.bfloat16))


@pytest.mark.parametrize("M,N,K", [(65, 1003, 200), (130, 333, 72), (300, 5001, 264)])
def test_linear_float_result_from_bfloat16_above_64_rows(M, N, K):
    """The head's logits for more than 64 wanted rows: float out of bfloat16 operands, summed in
    float (a rounded bfloat16 result would be off by 2^-9 of the value), 64 rows at a time
    through the weight-streaming kernel; a row stride it does not take goes to the plain kernel."""
    g = torch.Generator(device="cpu").manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.05).to(DEV).to(torch.bfloat16)
    out = torch.full((M, N), float("nan"), device=DEV)
    ops().linear(x, w, out)
    close(out, x.double() @ w.double().T, 2e-5)
    odd = torch.randn(M, K + 1, generator=g).to(DEV).to(torch.bfloat16)[:, :K]      # row stride K + 1
    ops().linear(odd, w, out)
    close(out, odd.double() @ w.double().T, 2e-5)


DEC_SHAPES = [(4, 2, 16), (14, 2, 64), (12, 2, 48), (5, 5, 32), (8, 1, 128), (32, 8, 128), (2, 1, 256), (6, 3, 80)]
DEC_BATCHES = [
    ([1], [0]), ([1], [15]), ([1], [16]), ([1, 1, 1], [31, 32, 700]), ([1] * 5, [63, 64, 65, 1000, 2]),
    ([2, 1, 3, 1], [0, 257, 30, 99]), ([1, 1, 1], [2047, 3000, 130]),
]


@pytest.mark.parametrize("Hq,Hkv,d", DEC_SHAPES)
def test_attention_decode(Hq, Hkv, d):
    for bi, (q_lens, starts) in enumerate(DEC_BATCHES):
        for window in (0, 19):
            # (least chunk, waves a workgroup); None: what the dispatch would choose (12 waves: few pairs)
            for chunk, waves in ((None, None), (128, 4), (256, 4), (1024, 4), (128, 12), (512, 12), (2048, 12)):
                q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=10 + bi)
                batch = FakeBatch(q_lens, starts, tables)
                T = sum(q_lens)
                out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
                scale = 1.0 / math.sqrt(d)
                ops().attention_decode(q.view(T, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window, 0,
                                       chunk=chunk, waves=waves)
                ref = attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window)
                close(out, ref, 2 ** -7)     # probabilities and values are bfloat16 products summed in float


def test_attention_decode_more_tokens_than_one_launch_numbers():
    """The kernel numbers the work items of at most 1024 tokens a launch; longer
    lists go in slices, with and without a token list."""
    Hq, Hkv, d = 4, 2, 32
    q_lens, starts = [700, 500], [5, 300]
    q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=31)
    batch = FakeBatch(q_lens, starts, tables)
    T = sum(q_lens)
    ref = attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, d ** -0.5, 0)
    out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().attention_decode(q.view(T, -1), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, d ** -0.5, 0, 0, chunk=128)
    close(out, ref, 2 ** -7)
    rows = list(range(T - 1, 60, -1))                      # 1139 tokens, in descending order
    lst = torch.tensor(rows, dtype=torch.int32, device=DEV)
    out = torch.full((T, Hq * d), 7.0, device=DEV, dtype=torch.bfloat16)
    ops().attention_decode(q.view(T, -1), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, d ** -0.5, 0, 0, lst,
                           len(rows), max(s + n for s, n in zip(starts, q_lens)), chunk=256)
    close(out[rows], ref[rows], 2 ** -7)
    assert (out[:61] == 7.0).all()


def test_attention_decode_token_list_leaves_other_rows_alone():
    Hq, Hkv, d = 8, 2, 64
    q_lens, starts = [1, 6, 1], [40, 3, 99]
    q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=3)
    batch = FakeBatch(q_lens, starts, tables)
    T = sum(q_lens)
    out = torch.full((T, Hq * d), 7.0, device=DEV, dtype=torch.bfloat16)
    lst = torch.tensor([0, 7], dtype=torch.int32, device=DEV)
    ops().attention_decode(q.view(T, -1), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, d ** -0.5, 0, 0, lst, 2, 100)
    ref = attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, d ** -0.5, 0)
    close(out[[0, 7]], ref[[0, 7]], 2 ** -7)
    assert (out[1:7] == 7.0).all()


PRE_BATCHES = [
    ([5], [0]), ([64], [0]), ([65], [0]), ([17, 130], [30, 5]), ([200], [0]), ([33, 7, 64], [1, 700, 16]),
    ([300], [213]),
]


@pytest.mark.parametrize("Hq,Hkv,d", [(4, 2, 16), (14, 2, 64), (12, 2, 48), (5, 5, 32), (8, 1, 128), (32, 8, 128),
                                      (6, 3, 80), (3, 1, 112)])
def test_attention_prefill(Hq, Hkv, d):
    tile = kernels.library.load().ra_attention_prefill_tile(Hq, Hkv, d)
    for bi, (q_lens, starts) in enumerate(PRE_BATCHES):
        for window in (0, 19, 100):
            q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=20 + bi)
            batch = FakeBatch(q_lens, starts, tables)
            T = sum(q_lens)
            out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
            info, t = [], 0
            for i, (ql, st) in enumerate(zip(q_lens, starts)):
                for q0 in range(0, ql, tile):
                    info += [i, t + q0, min(tile, ql - q0), st + q0]
                t += ql
            tiles = torch.tensor(info, dtype=torch.int32, device=DEV)
            scale = 1.0 / math.sqrt(d)
            ops().attention_prefill(q.view(T, Hq * d), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window, 0,
                                    tiles, len(info) // 4)
            ref = attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, window)
            close(out, ref, 2 ** -7)
            # the same tiles cut by keys into parts of 1, 2 or 3 rounds of 64 (every other tile whole), listed in
            # another order, their sums added by the second kernel
            for per in (1, 2, 3):
                items, ranges, merge, n_slots = [], [], [], 0
                for k in range(len(info) // 4):
                    i, row, n, pos = info[4 * k:4 * k + 4]
                    r = -(-(pos + n) // 64)
                    parts = -(-r // per)
                    if k % 2 == 1 or parts < 2:
                        items.append(((i, row, n, pos), (0, 1 << 30, -1)))
                        continue
                    merge += [row, n, n_slots, parts]
                    for c in range(parts):
                        items.append(((i, row, n, pos), (c * per * 64, (c + 1) * per * 64 if c + 1 < parts else 1 << 30, n_slots + c)))
                    n_slots += parts
                if not merge:
                    continue
                items = items[::-1]
                out3 = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
                ops().attention_prefill(q.view(T, Hq * d), Hq * d, out3, kt(kc), vt(vc), batch, Hq, Hkv, d, scale, window, 0,
                                        torch.tensor([v for it in items for v in it[0]], dtype=torch.int32, device=DEV), len(items),
                                        torch.tensor([v for it in items for v in it[1]], dtype=torch.int32, device=DEV),
                                        torch.tensor(merge, dtype=torch.int32, device=DEV), len(merge) // 4, n_slots)
                close(out3, ref, 2 ** -7)
            if kernels.library.load().ra_attention_prefill_columns(Hq, Hkv, d) == 2 and window != 100:
                # every other tile given to two workgroups, each with one of a wave's two column tiles
                cut = []
                for k in range(len(info) // 4):
                    i, row, n, pos = info[4 * k:4 * k + 4]
                    cut += [i, row, n | (1 << 16), pos, i, row, n | (2 << 16), pos] if k % 2 == 0 else [i, row, n, pos]
                out2 = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
                ops().attention_prefill(q.view(T, Hq * d), Hq * d, out2, kt(kc), vt(vc), batch, Hq, Hkv, d, scale,
                                        window, 0, torch.tensor(cut, dtype=torch.int32, device=DEV), len(cut) // 4)
                assert torch.equal(out2, out)             # the same arithmetic, column tile by column tile


def test_attention_and_cache_write_in_a_cache_above_4_gib():
    """K and V of one layer at 4.9 GB each (150,000 blocks of 16 slots, 8 KV heads of 128): the attention
    kernels and the cache write address blocks at the far end of it as they do the first."""
    Hq, Hkv, d, NB = 32, 8, 128, 150000
    q_lens, starts = [1, 70, 1, 3], [700, 200, 15, 40]
    q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=77)
    small_k, small_v = kt(kc), vt(vc)                      # [blocks, kv heads, 1, 16 d]
    n_small = small_k.shape[0]
    far = torch.tensor([NB - 1 - 997 * b for b in range(n_small)])      # spread downwards from the last block
    far[::3] = torch.arange(1, n_small + 1)[::3] * 11                   # and a third of them near the start
    big_k = torch.full((NB, Hkv, 1, 16 * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    big_v = torch.full((NB, Hkv, 1, 16 * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    big_k[far.to(DEV)] = small_k
    big_v[far.to(DEV)] = small_v
    big_tables = far[tables.long().cpu()].to(torch.int32).to(DEV)
    batch = FakeBatch(q_lens, starts, big_tables)
    T = sum(q_lens)
    scale = d ** -0.5
    ref = attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, scale, 0)
    out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().attention(q.view(T, Hq * d), Hq * d, out, big_k, big_v, batch, Hq, Hkv, d, scale, 0, 0)   # decode and prefill kernels
    close(out, ref, 2 ** -7)
    out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().attention_plain(q.view(T, Hq * d), Hq * d, out, big_k, big_v, batch, Hq, Hkv, d, scale, 0, 0)
    close(out, ref, 2 ** -7)
    # the cache write, few tokens (a wave a head) and many (a workgroup a token), into the last blocks
    for n_tok in (5, 200):
        qkv = torch.randn(n_tok, (Hq + 2 * Hkv) * d, device=DEV).to(torch.bfloat16)
        src = qkv.clone()
        slots = torch.arange(n_tok, dtype=torch.int32, device=DEV) + (NB - 40) * 16
        pos = torch.arange(n_tok, dtype=torch.int32, device=DEV)
        inv_freq = (10000.0 ** (-torch.arange(0, d, 2).double() / d)).float().to(DEV)
        ops().qk_norm_rope_cache(qkv, None, None, 1e-6, pos, inv_freq, d, 0, slots, big_k, big_v, Hq, Hkv, d)
        v_rows = unpack_v(big_v[NB - 40:NB - 40 + (n_tok + 15) // 16], d)          # [blocks, kv heads, slot, d]
        got = v_rows.permute(0, 2, 1, 3).reshape(-1, Hkv, d)[:n_tok]
        assert torch.equal(got, src.view(n_tok, Hq + 2 * Hkv, d)[:, Hq + Hkv:])
        k_rows = unpack_k(big_k[NB - 40:NB - 40 + (n_tok + 15) // 16], d).permute(0, 2, 1, 3).reshape(-1, Hkv, d)[:n_tok]
        k_ref = plain.rope_neox(src.view(n_tok, Hq + 2 * Hkv, d)[:, Hq:Hq + Hkv].double().cpu(), pos.cpu(), 10000.0)
        close(k_rows, k_ref, 2 ** -7)


def test_attention_dispatch_mixed_batch():
    """Single tokens, a short portion and long portions in one call: each token gets
    the kernel its portion calls for, and every row is written once."""
    Hq, Hkv, d = 8, 2, 64
    q_lens, starts = [1, 3, 70, 1, 5], [100, 0, 11, 15, 64]
    q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=9)
    batch = FakeBatch(q_lens, starts, tables)
    T = sum(q_lens)
    out = torch.full((T, Hq * d), float("nan"), device=DEV, dtype=torch.bfloat16)
    ops().attention(q.view(T, -1), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, d ** -0.5, 0, 0)
    tile = kernels.library.load().ra_attention_prefill_tile(Hq, Hkv, d)
    (plan,) = [v for k, v in batch.extra.items() if isinstance(k, tuple) and k[:2] == ("attention_plan", tile)]
    listed = plan["tiles"].view(-1, 4).tolist()
    assert plan["n_decode"] == 5 and plan["n_tiles"] == len(listed)
    rows = sorted({t[1] for t in listed})
    assert len(rows) == -(-70 // tile) + 1                  # the query tiles themselves
    for row in rows:                                        # each listed whole, or once for each half of the heads
        marks = sorted(t[2] >> 16 for t in listed if t[1] == row)
        assert marks in ([0], [1, 2])
    close(out, attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, d ** -0.5, 0), 2 ** -7)


def test_far_key_among_hundreds_decode_and_prefill():
    """One key far back matches the query much better than all others: losing it
    (a wrong block, a dropped split, a wrong running maximum) changes the output."""
    Hq, Hkv, d = 4, 1, 128
    for q_lens, starts in (([1], [900]), ([80], [821])):
        q, kc, vc, tables = make_paged_case("bfloat16", Hq, Hkv, d, q_lens, starts, seed=4)
        far = 37
        blk = int(tables[0, far // 16])
        kc[blk, 0, far % 16] = (q[-1, 0].float() * 3).to(torch.bfloat16)      # the last query's first head points at it
        vc[blk, 0, far % 16] = 5.0
        batch = FakeBatch(q_lens, starts, tables)
        T = sum(q_lens)
        out = torch.empty((T, Hq * d), device=DEV, dtype=torch.bfloat16)
        ops().attention(q.view(T, -1), Hq * d, out, kt(kc), vt(vc), batch, Hq, Hkv, d, d ** -0.5, 0, 0)
        ref = attention_reference(q, kc, vc, tables, q_lens, starts, Hq, Hkv, d, d ** -0.5, 0)
        assert ref[-1, :d].mean() > 4.0           # the far value dominates the reference
        close(out, ref, 2 ** -7)


def test_measured_peaks_are_plausible():
    """The two measurement kernels (a plain read, matrix-core products on registers) run, and what they
    report is not above the published peaks: a mistake in their byte or flop count would show there. How
    close a box comes to the peaks is a measurement, not a test: the lower bounds only say that a
    figure was computed at all (a twentieth of the peak)."""
    p = ops().measure_peaks(DEV, read_bytes=1 << 30)
    print(p)
    assert 400.0 < p["hbm_read_GBps"] < 8000.0 * 1.05, p
    assert 125.0 < p["mfma_bf16_32x32x16_TFLOPs"] < 2500.0 * 1.05, p
    assert 125.0 < p["mfma_bf16_16x16x32_TFLOPs"] < 2500.0 * 1.05, p
    with pytest.raises(kernels.KernelLibraryError, match="multiple of 16"):
        from reinfer_amd.kernels import library
        library.call("ra_stream_read", 0, 8, 0, 0)
