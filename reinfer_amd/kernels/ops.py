"""Tensor-level entry points of the kernel library.

Each function checks on the host that shapes, dtypes, devices and strides are
what the kernel assumes, and only then launches on torch's current stream. The
parts call these through :func:`reinfer_amd.kernels.current`.
"""
from __future__ import annotations

import heapq
from typing import Optional

import torch

from . import library

_TAG = {torch.float32: 0, torch.bfloat16: 1}


def _tag(t: torch.Tensor, what: str) -> int:
    try:
        return _TAG[t.dtype]
    except KeyError:
        raise TypeError(f"{what}: dtype {t.dtype} is not float32 or bfloat16") from None


def _dev(*tensors) -> None:
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise library.KernelLibraryError(
                "the kernels run on the GPU only: got a tensor on " + str(t.device))


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _int32(t: torch.Tensor, what: str, n: Optional[int] = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{what}: expected a contiguous int32 tensor, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise ValueError(f"{what}: {t.numel()} entries, need {n}")


class HipKernels:
    """The product's kernels. Stateless apart from the loaded library."""

    name = "hip-gfx950"

    def __init__(self):
        library.load()
        self._decode_slots = {}     # (heads, KV heads, head size) -> workgroups of the decode kernel's grid
        self._cu_count = {}
        self._side_streams = {}     # device -> the stream for the second kernel of a mixed step

    # ------------------------------------------------------------------ rows
    def embed(self, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
        _dev(table, ids, out)
        T, h = out.shape
        if table.dim() != 2 or table.shape[1] != h or not table.is_contiguous():
            raise ValueError(f"embed: table {tuple(table.shape)} does not have rows of width {h}")
        if out.dtype != torch.float32 or not out.is_contiguous():
            raise TypeError("embed: the residual stream is contiguous float32")
        _int32(ids, "embed ids", T)
        library.call("ra_embed", table.data_ptr(), _tag(table, "embed table"), ids.data_ptr(),
                     out.data_ptr(), T, h, _stream())

    def add_rmsnorm(self, resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor,
                    eps: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        _dev(resid, delta, weight, out, rows)
        h = resid.shape[-1]
        n = out.shape[0]
        if resid.dtype != torch.float32 or not resid.is_contiguous():
            raise TypeError("add_rmsnorm: the residual stream is contiguous float32")
        if weight.shape != (h,) or out.shape[-1] != h or not out.is_contiguous():
            raise ValueError(f"add_rmsnorm: width {h}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
        if delta is not None:
            if delta.shape != resid.shape or delta.dtype != out.dtype or not delta.is_contiguous():
                raise ValueError("add_rmsnorm: delta must match the residual's shape and the output's dtype")
        if rows is None:
            if n != resid.shape[0]:
                raise ValueError("add_rmsnorm: in-place form needs one output row per residual row")
        else:
            _int32(rows, "add_rmsnorm rows", n)
        library.call("ra_add_rmsnorm", resid.data_ptr(), _ptr(delta), weight.data_ptr(),
                     _tag(weight, "norm weight"), out.data_ptr(), _tag(out, "add_rmsnorm out"),
                     _ptr(rows), n, h, float(eps), _stream())

    def qk_norm_rope_cache(self, qkv: torch.Tensor, q_weight: Optional[torch.Tensor],
                           k_weight: Optional[torch.Tensor], eps: float, positions: torch.Tensor,
                           inv_freq: torch.Tensor, rotary_dim: int, rope_style: int,
                           slots: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor,
                           num_heads: int, num_kv_heads: int, head_dim: int) -> None:
        _dev(qkv, q_weight, k_weight, positions, inv_freq, slots, kcache, vcache)
        T = qkv.shape[0]
        width = (num_heads + 2 * num_kv_heads) * head_dim
        if qkv.shape != (T, width) or not qkv.is_contiguous():
            raise ValueError(f"qk_norm_rope_cache: qkv {tuple(qkv.shape)}, expected [T, {width}] contiguous")
        self._check_cache("qk_norm_rope_cache", kcache, vcache, num_kv_heads, head_dim)
        if kcache.dtype != qkv.dtype or vcache.dtype != qkv.dtype:
            raise TypeError("qk_norm_rope_cache: the cache has the activations' dtype")
        _int32(positions, "positions", T)
        _int32(slots, "cache slots", T)
        if inv_freq.dtype != torch.float32 or inv_freq.numel() < rotary_dim // 2:
            raise ValueError("qk_norm_rope_cache: inv_freq is float32 with rotary_dim/2 entries")
        wtag = 0
        for w in (q_weight, k_weight):
            if w is not None:
                if w.shape != (head_dim,):
                    raise ValueError(f"qk_norm_rope_cache: head-norm weight {tuple(w.shape)}, expected [{head_dim}]")
                wtag = _tag(w, "head-norm weight")
        if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
            raise TypeError("qk_norm_rope_cache: q and k norm weights differ in dtype")
        library.call("ra_qk_norm_rope_cache", qkv.data_ptr(), _tag(qkv, "qkv"), _ptr(q_weight),
                     _ptr(k_weight), wtag, float(eps), positions.data_ptr(), inv_freq.data_ptr(),
                     int(rotary_dim), int(rope_style), slots.data_ptr(), kcache.data_ptr(),
                     vcache.data_ptr(), kcache.shape[2] * 16, T, num_heads, num_kv_heads, head_dim, _stream())

    # ---- the q/k/v product left in K ranges for the kernel that consumes it
    def linear_ranges(self, x: torch.Tensor, weight: torch.Tensor):
        """x . weight^T as the float results of the K ranges it was cut into, [ranges, M, N], not yet
        added, or None where that does not pay: only the products the split kernel takes (bfloat16,
        17 to 64 rows) and cuts (few output features), whose adding kernel a consumer can save by
        adding the ranges itself (``qk_norm_rope_cache(..., ranges=)``)."""
        if not (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.dim() == 2):
            return None
        M, K = x.shape
        N = weight.shape[0]
        if not (self.NORM_SKINNY_ROWS < M <= 64) or K % 8 or x.stride(1) != 1 or x.stride(0) % 8 \
                or weight.shape != (N, K) or not weight.is_contiguous():
            return None
        lib = library.load()
        S = int(lib.ra_gemm_wide_ranges(M, N, K))
        if S < 2 or not lib.ra_gemm_wide_preferred(0, M, N, K):
            return None
        parts = torch.empty((S, M, N), dtype=torch.float32, device=x.device)
        library.call("ra_gemm_wide_partial", x.data_ptr(), weight.data_ptr(), parts.data_ptr(), parts.numel(),
                     M, N, K, x.stride(0), _stream())
        return parts

    def qk_norm_rope_cache_ranges(self, ranges: torch.Tensor, row_sums, q_out: torch.Tensor,
                                  q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                                  positions: torch.Tensor, inv_freq: torch.Tensor, rotary_dim: int,
                                  rope_style: int, slots: torch.Tensor, kcache: torch.Tensor,
                                  vcache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int) -> None:
        """``qk_norm_rope_cache`` on the result of ``linear_ranges``: the ranges are added here (in
        range order), the rows scaled by the RMSNorm that the product carried (``row_sums`` = (ss
        [parts, T], eps, width) or None), q normalised and rotated into ``q_out`` [T, heads * head_dim]."""
        _dev(ranges, q_weight, k_weight, positions, inv_freq, slots, kcache, vcache, q_out)
        S, T, width = ranges.shape
        if width != (num_heads + 2 * num_kv_heads) * head_dim or ranges.dtype != torch.float32 \
                or not ranges.is_contiguous():
            raise ValueError(f"qk_norm_rope_cache: ranges {tuple(ranges.shape)} {ranges.dtype}, expected float32 "
                             f"[ranges, T, {(num_heads + 2 * num_kv_heads) * head_dim}]")
        self._check_cache("qk_norm_rope_cache", kcache, vcache, num_kv_heads, head_dim)
        if q_out.dtype != kcache.dtype or q_out.shape != (T, num_heads * head_dim) or q_out.stride(1) != 1:
            raise ValueError("qk_norm_rope_cache: q_out is [T, heads * head_dim] in the cache's dtype")
        _int32(positions, "positions", T)
        _int32(slots, "cache slots", T)
        if inv_freq.dtype != torch.float32 or inv_freq.numel() < rotary_dim // 2:
            raise ValueError("qk_norm_rope_cache: inv_freq is float32 with rotary_dim/2 entries")
        wtag = 0
        for w in (q_weight, k_weight):
            if w is not None:
                if w.shape != (head_dim,):
                    raise ValueError(f"qk_norm_rope_cache: head-norm weight {tuple(w.shape)}, expected [{head_dim}]")
                wtag = _tag(w, "head-norm weight")
        ss = None
        parts, in_eps, in_width = 0, 0.0, 0
        if row_sums is not None:
            ss, in_eps, in_width = row_sums
            _dev(ss)
            if ss.dtype != torch.float32 or ss.dim() != 2 or ss.shape[1] != T or not ss.is_contiguous():
                raise ValueError(f"qk_norm_rope_cache: row sums {tuple(ss.shape)} {ss.dtype}, expected float32 [parts, {T}]")
            parts = ss.shape[0]
        library.call("ra_qk_norm_rope_cache_sums", ranges.data_ptr(), S, _ptr(ss), parts, float(in_eps),
                     int(in_width), q_out.data_ptr(), q_out.stride(0), _tag(q_out, "q"), _ptr(q_weight),
                     _ptr(k_weight), wtag, float(eps), positions.data_ptr(), inv_freq.data_ptr(),
                     int(rotary_dim), int(rope_style), slots.data_ptr(), kcache.data_ptr(), vcache.data_ptr(),
                     kcache.shape[2] * 16, T, num_heads, num_kv_heads, head_dim, _stream())

    def silu_mul(self, gate_up: torch.Tensor, out: torch.Tensor, group: int = 0) -> None:
        """out = silu(gate) * up. ``group`` 0: gate_up is [gate | up]; ``group`` g > 0: runs of g
        gate columns and g up columns alternate."""
        _dev(gate_up, out)
        T, I = out.shape
        if gate_up.shape != (T, 2 * I) or gate_up.dtype != out.dtype \
                or not gate_up.is_contiguous() or not out.is_contiguous():
            raise ValueError(f"silu_mul: gate_up {tuple(gate_up.shape)} against out {tuple(out.shape)}")
        if group < 0 or (group > 0 and I % group != 0):
            raise ValueError(f"silu_mul: width {I} is not a whole number of runs of {group}")
        library.call("ra_silu_mul", gate_up.data_ptr(), out.data_ptr(), _tag(out, "silu_mul"), T, I,
                     int(group), _stream())

    # ------------------------------------------------------------- attention
    SHORT_PORTION = 4     # portions up to this many tokens go token by token through the decode kernel
    TWO_STREAMS_FROM = 8  # decode tokens of a mixed step from which their attention runs beside the prompt portions'

    def attention(self, q: torch.Tensor, q_stride: int, out: torch.Tensor, kcache: torch.Tensor,
                  vcache: torch.Tensor, batch, num_heads: int, num_kv_heads: int, head_dim: int,
                  scale: float, window: int, group: int) -> None:
        """Attention of every token of the step over its request's cache.

        ``q`` is the buffer whose row ``t`` holds the query heads of token t at
        its start (row stride ``q_stride`` elements); ``batch`` is the step's
        :class:`reinfer_amd.engine.batch.StepBatch`; ``group`` picks the block
        tables of the cache group this layer belongs to. bfloat16: single tokens
        and short portions take the split-KV decode kernel, longer portions the
        MFMA prefill kernel in tiles of queries; sizes neither takes, and
        float32, go to the plain kernel.
        """
        lib = library.load()
        if q.dtype != torch.bfloat16:
            return self.attention_plain(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                        head_dim, scale, window, group)
        bs = kcache.shape[2] * 16
        tile = lib.ra_attention_prefill_tile(num_heads, num_kv_heads, head_dim)
        # query tiles that give every CU one workgroup
        room = self._cus(q.device) // max(1, lib.ra_attention_prefill_groups(num_heads, num_kv_heads, head_dim))
        halves = lib.ra_attention_prefill_columns(num_heads, num_kv_heads, head_dim) == 2
        # the plan's fixed costs are priced in rounds of this shape: a round's time goes with the columns of a
        # query tile times the head size the kernel is built for
        cols = 128 * max(1, lib.ra_attention_prefill_columns(num_heads, num_kv_heads, head_dim))
        built_for = 64 if head_dim <= 64 else 128 if head_dim <= 128 else 256
        plan = self._attention_plan(batch, q.device, tile, room, halves, (256 * 128) / (cols * built_for))
        dec_ok = bool(lib.ra_attention_decode_supports(num_heads, num_kv_heads, head_dim, bs))
        pre_ok = bool(lib.ra_attention_prefill_supports(num_heads, num_kv_heads, head_dim, bs))
        side = None
        if plan["n_decode"] >= self.TWO_STREAMS_FROM and plan["n_tiles"] and dec_ok and pre_ok \
                and not torch.cuda.is_current_stream_capturing():
            # a mixed step: the decoding requests' attention streams keys and values, the prompt
            # portions' attention computes; on two streams (both of default priority) the two kernels
            # share the chip (128 requests at the Qwen3-4B shape, 2048-token steps: 0.7 ms a mixed step)
            side = self._side_stream(q.device)
            cur = torch.cuda.current_stream()
            side.wait_stream(cur)
            with torch.cuda.stream(side):           # its scratch comes from, and goes back to, the side stream's pool
                self.attention_decode(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                      head_dim, scale, window, group, plan["decode_list"], plan["n_decode"],
                                      plan["decode_max_ctx"])
        elif plan["n_decode"]:
            if dec_ok:
                self.attention_decode(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                      head_dim, scale, window, group, plan["decode_list"], plan["n_decode"],
                                      plan["decode_max_ctx"])
            else:
                self.attention_plain(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                     head_dim, scale, window, group, plan["decode_list"], plan["n_decode"])
        if plan["n_tiles"]:
            if pre_ok:
                self.attention_prefill(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                       head_dim, scale, window, group, plan["tiles"], plan["n_tiles"],
                                       plan.get("ranges"), plan.get("merge"), plan.get("n_merge", 0),
                                       plan.get("n_slots", 0))
            else:
                self.attention_plain(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                     head_dim, scale, window, group, plan["prefill_list"], plan["n_prefill"])
        if side is not None:
            torch.cuda.current_stream().wait_stream(side)

    def _side_stream(self, device):
        s = self._side_streams.get(device)
        if s is None:
            s = self._side_streams[device] = torch.cuda.Stream(device=device)      # default priority
        return s

    def _cus(self, device) -> int:
        n = self._cu_count.get(device)
        if n is None:
            n = self._cu_count[device] = int(torch.cuda.get_device_properties(device).multi_processor_count)
        return n

    # What the prompt kernel's plan is chosen by, in rounds of 64 keys of a whole query tile of 256 columns
    # and head size 128 (2.1 us: 64 queries of 4 heads): a tile listed with half of its heads costs 0.76 of the
    # whole one, every listed item one such round to start and end, and the kernel that adds the parts of cut
    # tiles 3 rounds and 0.15 for each part; for another shape the three fixed costs are scaled by how much
    # shorter or longer its rounds are (``fixed``: the reference round's work over this shape's) (measured: a portion of 512 tokens behind 3584: 142 us as it is, 115 with the tiles
    # listed twice, 57 cut by keys; 256 behind 7936: 277 / 223 / 58; a whole prompt of 2048: 83 / 69 / 83,
    # of 1024: 43 / 35 / 40; 2048 behind 2048: 152 / 195 / 146)
    PREFILL_ROUND = 64
    PREFILL_HALF_HEADS = 0.76
    PREFILL_ITEM = 1.0
    PREFILL_MERGE = (3.0, 0.15)
    PREFILL_PART_ROUNDS = 4     # a part of a cut tile has at least this many rounds
    PREFILL_MAX_PARTS = 8

    @staticmethod
    def _span(costs, room: int) -> float:
        """When the last of ``costs`` ends if ``room`` run at a time, the heaviest started first and each
        further one where room is first free."""
        if len(costs) <= room:
            return max(costs)
        costs = sorted(costs, reverse=True)
        ends = costs[:room]
        heapq.heapify(ends)
        for c in costs[room:]:
            heapq.heappush(ends, heapq.heappop(ends) + c)
        return max(ends)

    def _prefill_items(self, tiles, room: int, halves: bool, fixed: float = 1.0):
        """The prompt kernel's work items for ``tiles`` of (request, row, queries, position), and the list
        for the kernel that adds the parts of tiles cut by keys: ``(items, merge, n_slots)``, an item being
        (cost, tile, first key, one past the last key, slot or -1).

        A launch lasts as long as its heaviest item while the CUs of the light ones idle: a whole prompt of
        2048 tokens is one tile a CU, the last with 32 times the keys of the first; a portion of 512 tokens
        deep in a long prompt is eight tiles of thousands of keys each on a chip with room for 32. Three
        ways to list the tiles are priced by ``_span`` and the cheapest is taken. As they are. Where the
        kernel can give a workgroup half of a tile's heads (``halves``), the tiles with the most keys
        twice, each time with half of the heads (as many as there is room for and at
        least a quarter of ``room``; from ``room`` to 5/4 of it 3/16 of ``room``): a half that queues behind
        a light tile still ends before a whole heavy one would, which pays for a prompt from its start. Or,
        while there are fewer tiles than ``room``, the heaviest cut by keys into parts, each an item whose
        float sums a second kernel adds up; the spare room goes, one part at a time, to the tile whose
        parts are longest. (Windows are not known here, one plan serving all layers: a part below a
        layer's window finds nothing to do.)"""
        R = self.PREFILL_ROUND
        n = len(tiles)
        item_cost = self.PREFILL_ITEM * fixed
        rounds = [-(-(pos + q) // R) for (_, _, q, pos) in tiles]
        whole = [(r + item_cost, tl, 0, 0, -1) for tl, r in zip(tiles, rounds)]
        if room <= 0 or n == 0:
            return whole, [], 0
        best, best_span = (whole, [], 0), self._span([it[0] for it in whole], room)
        # the heaviest twice, by heads
        n_twice = 0
        if not halves:
            pass
        elif n <= room:
            n_twice = min(n, max(room - n, room // 4))
        elif n <= room + room // 4:
            n_twice = (3 * room) // 16
        if n_twice:
            twice = set(sorted(range(n), key=lambda k: -rounds[k])[:n_twice])
            items = []
            for k, (tl, r) in enumerate(zip(tiles, rounds)):
                if k in twice:
                    i, row, q, pos = tl
                    c = r * self.PREFILL_HALF_HEADS + item_cost
                    items.append((c, (i, row, q | (1 << 16), pos), 0, 0, -1))
                    items.append((c, (i, row, q | (2 << 16), pos), 0, 0, -1))
                else:
                    items.append(whole[k])
            span = self._span([it[0] for it in items], room)
            if span < best_span:
                best, best_span = (items, [], 0), span
        # the heaviest cut by keys
        if n < room:
            parts = [1] * n
            heap = [(-r, k) for k, r in enumerate(rounds)]
            heapq.heapify(heap)
            used = n
            while used < room and heap:
                _, k = heapq.heappop(heap)
                if parts[k] >= self.PREFILL_MAX_PARTS or rounds[k] < self.PREFILL_PART_ROUNDS * (parts[k] + 1):
                    continue
                parts[k] += 1
                used += 1
                heapq.heappush(heap, (-rounds[k] / parts[k], k))
            items, merge, n_slots = [], [], 0
            for k, (tl, r) in enumerate(zip(tiles, rounds)):
                per = -(-r // parts[k])
                p = -(-r // per)
                if p <= 1:
                    items.append(whole[k])
                    continue
                merge.extend((tl[1], tl[2], n_slots, p))
                for j in range(p):
                    hi = (j + 1) * per * R if j + 1 < p else 1 << 30
                    items.append((min(per, r - j * per) + item_cost, tl, j * per * R, hi, n_slots + j))
                n_slots += p
            if n_slots:
                span = self._span([it[0] for it in items], room) + (self.PREFILL_MERGE[0]
                                                                      + self.PREFILL_MERGE[1] * n_slots) * fixed
                if span < best_span:
                    best, best_span = (items, merge, n_slots), span
        return best

    def plan_captured_step(self, batch, num_rows: int, ctx_cap: int) -> None:
        """The attention plan of a captured decode step: ``num_rows`` single tokens over contexts of at most
        ``ctx_cap``, whatever the step that is replayed holds (the grids are chosen from these)."""
        batch.extra["attention_plan"] = {
            "n_decode": num_rows, "decode_max_ctx": ctx_cap, "decode_list": None, "n_prefill": 0,
            "prefill_list": None, "n_tiles": 0, "tiles": None}

    def _attention_plan(self, batch, device, tile: int, room: int = 0, halves: bool = False, fixed: float = 1.0):
        """Which tokens go to which kernel; made once per step and query-tile size, shared by the
        layers. ``room`` is the number of query tiles whose workgroups fill the chip once (0: the tiles
        are listed as they are)."""
        plan = batch.extra.get("attention_plan")
        if plan is not None and plan.get("tile", tile) == tile:
            return plan
        plan = batch.extra.get(("attention_plan", tile, room, halves, fixed))
        if plan is not None:
            return plan
        dec, pre, tiles = [], [], []
        dec_max_ctx = 0
        t = 0
        for i, (ql, st) in enumerate(zip(batch.q_lens, batch.starts)):
            if ql <= self.SHORT_PORTION:
                dec.extend(range(t, t + ql))
                dec_max_ctx = max(dec_max_ctx, st + ql)
            else:
                pre.extend(range(t, t + ql))
                for q0 in range(0, ql, tile):
                    tiles.append((i, t + q0, min(tile, ql - q0), st + q0))
            t += ql
        items, merge, n_slots = self._prefill_items(tiles, room, halves, fixed)
        items.sort(key=lambda it: it[0])                     # the heaviest last: the kernel starts the last listed first
        listed = [v for it in items for v in it[1]]
        ranges = [v for it in items for v in ((it[2], it[3], it[4]) if it[4] >= 0 else (0, 1 << 30, -1))] if merge else []
        all_decode = len(dec) == batch.num_tokens
        flat = ([] if all_decode else dec) + pre + listed + ranges + merge
        dev = torch.tensor(flat, dtype=torch.int32).to(device, non_blocking=True) if flat else None
        n_dec_listed = 0 if all_decode else len(dec)
        o_tiles = n_dec_listed + len(pre)
        o_ranges = o_tiles + len(listed)
        o_merge = o_ranges + len(ranges)
        plan = {
            "n_decode": len(dec), "decode_max_ctx": dec_max_ctx,
            "decode_list": None if all_decode or not dec else dev[:n_dec_listed],
            "n_prefill": len(pre),
            "prefill_list": dev[n_dec_listed:o_tiles] if pre else None,
            "n_tiles": len(items),
            "tiles": dev[o_tiles:o_ranges] if items else None,
            "ranges": dev[o_ranges:o_merge] if merge else None,
            "merge": dev[o_merge:] if merge else None,
            "n_merge": len(merge) // 4, "n_slots": n_slots,
            "tile": tile,
        }
        batch.extra[("attention_plan", tile, room, halves, fixed)] = plan
        return plan

    @staticmethod
    def _check_cache(what: str, kcache, vcache, num_kv_heads: int, head_dim: int) -> None:
        """K and V of a layer: [blocks, kv heads, block_size // 16, 16 * head_dim], tiled."""
        if kcache.dim() != 4 or kcache.shape != vcache.shape or kcache.shape[1] != num_kv_heads \
                or head_dim % 16 != 0 or kcache.shape[3] != 16 * head_dim \
                or not kcache.is_contiguous() or not vcache.is_contiguous():
            raise ValueError(f"{what}: cache K {tuple(kcache.shape)}, V {tuple(vcache.shape)}: expected "
                             f"[blocks, {num_kv_heads}, block_size // 16, 16 * {head_dim}] "
                             "(head sizes in steps of 16)")

    def _check_attention(self, q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads, head_dim, group):
        _dev(q, out, kcache, vcache)
        T = batch.num_tokens
        tables = batch.block_tables[group]
        if out.shape != (T, num_heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
            raise ValueError(f"attention: out {tuple(out.shape)}, expected [{T}, {num_heads * head_dim}]")
        if q.shape[0] != T or q_stride < num_heads * head_dim or q.stride(0) != q_stride:
            raise ValueError("attention: query rows do not match the step's tokens")
        if kcache.dtype != q.dtype or vcache.dtype != q.dtype:
            raise TypeError("attention: the cache has the activations' dtype")
        self._check_cache("attention", kcache, vcache, num_kv_heads, head_dim)
        _int32(tables, "block tables")
        if tables.dim() != 2 or tables.shape[0] < batch.num_seqs:
            raise ValueError("attention: one block-table row per request of the step")
        # every key a query may read must have a table entry
        if tables.shape[1] * kcache.shape[2] * 16 < batch.max_ctx_len:
            raise ValueError("attention: block tables shorter than the longest context")
        return tables

    def attention_plain(self, q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads, head_dim,
                        scale, window, group, token_list=None, n_listed=None) -> None:
        tables = self._check_attention(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                       head_dim, group)
        n = batch.num_tokens if token_list is None else int(n_listed)
        library.call("ra_attention_plain", q.data_ptr(), q_stride, out.data_ptr(), out.stride(0),
                     kcache.data_ptr(), vcache.data_ptr(), _tag(q, "attention"), tables.data_ptr(),
                     tables.shape[1], _ptr(token_list), batch.seq_of_token.data_ptr(),
                     batch.positions.data_ptr(), n, kcache.shape[2] * 16, num_heads, num_kv_heads, head_dim,
                     float(scale), int(window), _stream())

    # The decode kernel runs in workgroups of 12 waves from this many (token, KV head) pairs on, or over
    # contexts longer than this; below both, in workgroups of 4 (measured with 32 query heads over 8 KV
    # heads of 128, flash decode and merge together: 2200 keys a token, 1 / 4 / 8 / 16 / 32 / 64 tokens: 4 waves
    # 10.6 / 13.1 / 23.3 / 40.4 / 61.3 / 107 us, 12 waves 13.6 / 14.5 / 21.5 / 33.8 / 56.2 / 107; 8000 keys,
    # 1 / 4 / 16 / 64 tokens: 17.9 / 35.9 / 113 / 370 against 14.7 / 31.2 / 101 / 364)
    DECODE_WIDE_PAIRS = 64
    DECODE_WIDE_CTX = 4096      # keys of head size 128: what counts is the bytes of a (token, KV head) pair
    DECODE_WIDE_FILL = 0.9      # of the last round of large workgroups that the pairs must fill
    # Fewer pairs than the chip holds large workgroups: one large workgroup a pair, nothing to merge, from this
    # share of them on (20 to 28 requests over 8 KV heads, 1000 to 7000 keys: 8 to 14 % faster than the small
    # workgroups with their chunks and merge, 16 requests: equal), and at any number over contexts up to
    # DECODE_SHORT_CTX keys of head size 128 (600 keys, 1 to 24 requests: 7.8 to 15.2 us against 9.3 to 20.6)
    DECODE_WIDE_FILL_ONE = 0.6
    DECODE_SHORT_CTX = 768

    def _slots_of_decode(self, num_heads: int, num_kv_heads: int, head_dim: int, waves: int) -> int:
        """Workgroups of the decode kernel's form with ``waves`` waves that the chip holds at once (0: that
        form does not take these sizes)."""
        key = (num_heads, num_kv_heads, head_dim, waves)
        slots = self._decode_slots.get(key)
        if slots is None:
            slots = int(library.load().ra_attention_decode_slots(num_heads, num_kv_heads, head_dim, waves))
            self._decode_slots[key] = slots
        return slots

    def decode_chunk(self, n_tokens: int, num_heads: int, num_kv_heads: int, head_dim: int, max_ctx: int):
        """How the decode kernel cuts a token's keys: (least chunk length, most chunks a token, waves a
        workgroup). The kernel cuts every token into equal chunks of its own length, so only their
        number is chosen here: as many as fill the kernel's grid once (the workgroups the chip holds at
        once, whatever the batch). Then all work items run side by side and the launch lasts as long as
        one of them; more items than that cost a start and a partial result each (measured at 2200
        and 8000 keys a token, 1 to 128 tokens). Workgroups of 12 waves, one a CU, each with three times
        the keys in flight, need a third of the chunks to keep the memory as busy, which leaves fewer
        partial results to merge (none at 32 tokens and more); a small step over short contexts has too
        little work for them, and a step with more (token, KV head) pairs than the chip holds such
        workgroups would give some of them two pairs one after the other while the rest idle (33
        requests over 8 KV heads: 68 us a layer against 47 with the small workgroups, of which three fit
        a CU)."""
        pairs = max(1, n_tokens * num_kv_heads)
        waves = 4
        wide = self._slots_of_decode(num_heads, num_kv_heads, head_dim, 12)
        if 0 < pairs <= wide and (pairs >= self.DECODE_WIDE_FILL_ONE * wide
                                  or max_ctx * head_dim <= self.DECODE_SHORT_CTX * 128):
            return 512, 1, 12
        if pairs >= self.DECODE_WIDE_PAIRS or max_ctx * head_dim > self.DECODE_WIDE_CTX * 128:
            # whole rounds of the large workgroups, or nearly (64 requests over 8 KV heads are two rounds
            # of 256: 8.45 ms a step against 8.65 with the small workgroups)
            if wide > 0 and pairs >= self.DECODE_WIDE_FILL * (-(-pairs // wide) * wide):
                waves = 12
        slots = self._slots_of_decode(num_heads, num_kv_heads, head_dim, waves) or 768
        least = 256 if waves == 4 else 512
        return least, max(1, min(slots // pairs, -(-max_ctx // least))), waves

    def attention_decode(self, q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads, head_dim,
                         scale, window, group, token_list=None, n_listed=None, max_ctx=None,
                         chunk=None, waves=None) -> None:
        tables = self._check_attention(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                       head_dim, group)
        if q.dtype != torch.bfloat16:
            raise TypeError("attention_decode: bfloat16 only")
        n = batch.num_tokens if token_list is None else int(n_listed)
        max_ctx = int(max_ctx or batch.max_ctx_len)
        if chunk is None:
            chunk, max_chunks, waves = self.decode_chunk(n, num_heads, num_kv_heads, head_dim, max_ctx)
        else:
            waves = int(waves or 4)
            max_chunks = max(1, -(-max_ctx // int(chunk)))
        part_o = part_ml = None
        if max_chunks > 1:
            pairs = n * num_kv_heads
            G = num_heads // num_kv_heads
            part_o = torch.empty((pairs, max_chunks, G, head_dim), dtype=torch.float32, device=q.device)
            part_ml = torch.empty((pairs, max_chunks, G, 2), dtype=torch.float32, device=q.device)
        # every request of the step brings one token: token t is request t, and the kernel need not look it up
        one_each = token_list is None and batch.num_tokens == batch.num_seqs
        library.call("ra_attention_decode", q.data_ptr(), q_stride, out.data_ptr(), out.stride(0),
                     kcache.data_ptr(), vcache.data_ptr(), tables.data_ptr(), tables.shape[1],
                     _ptr(token_list), None if one_each else batch.seq_of_token.data_ptr(), batch.positions.data_ptr(), n,
                     kcache.shape[2] * 16, num_heads, num_kv_heads, head_dim, float(scale), int(window),
                     int(chunk), int(max_chunks), int(waves), _ptr(part_o), _ptr(part_ml), _stream())

    def attention_prefill(self, q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads, head_dim,
                          scale, window, group, tiles, n_tiles, ranges=None, merge=None, n_merge: int = 0,
                          n_slots: int = 0) -> None:
        """``tiles``: four ints a listed query tile (request row, first token row, queries, first
        position). With ``ranges`` (three ints a listed tile: first key, one past the last, the part's
        slot or -1) some tiles are listed in several parts by keys, and ``merge`` (four ints a cut tile:
        first token row, queries, first slot, parts) says which to add up."""
        tables = self._check_attention(q, q_stride, out, kcache, vcache, batch, num_heads, num_kv_heads,
                                       head_dim, group)
        if q.dtype != torch.bfloat16:
            raise TypeError("attention_prefill: bfloat16 only")
        _int32(tiles, "query tiles", 4 * n_tiles)
        if ranges is not None:
            _int32(ranges, "key ranges", 3 * n_tiles)
            _int32(merge, "cut tiles", 4 * n_merge)
            if n_merge <= 0 or n_slots <= 0:
                raise ValueError("attention_prefill: key ranges without cut tiles")
            lib = library.load()
            part_o = torch.empty(int(lib.ra_attention_prefill_part_floats(num_heads, num_kv_heads, head_dim, n_slots, 0)),
                                 dtype=torch.float32, device=q.device)
            part_ml = torch.empty(int(lib.ra_attention_prefill_part_floats(num_heads, num_kv_heads, head_dim, n_slots, 1)),
                                  dtype=torch.float32, device=q.device)
            library.call("ra_attention_prefill_split", q.data_ptr(), q_stride, out.data_ptr(), out.stride(0),
                         kcache.data_ptr(), vcache.data_ptr(), tables.data_ptr(), tables.shape[1],
                         tiles.data_ptr(), int(n_tiles), ranges.data_ptr(), merge.data_ptr(), int(n_merge),
                         part_o.data_ptr(), part_ml.data_ptr(), kcache.shape[2] * 16, num_heads, num_kv_heads,
                         head_dim, float(scale), int(window), _stream())
            return
        library.call("ra_attention_prefill", q.data_ptr(), q_stride, out.data_ptr(), out.stride(0),
                     kcache.data_ptr(), vcache.data_ptr(), tables.data_ptr(), tables.shape[1],
                     tiles.data_ptr(), int(n_tiles), kcache.shape[2] * 16, num_heads, num_kv_heads, head_dim,
                     float(scale), int(window), _stream())

    # ---------------------------------------------------------------- linear
    def linear(self, x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor,
               bias: Optional[torch.Tensor] = None) -> None:
        """out[M, N] = x[M, K] . weight[N, K]^T (+ bias), float accumulation.

        bfloat16 with up to 64 rows: the weight-streaming MFMA kernel. bfloat16
        with more rows and a bfloat16 result: the library product (hipBLASLt
        through torch), as the reference calls cuBLAS for its prompt products
        (crates/cuda/src/gemm.rs:226-292). bfloat16 with more rows and a float
        result (the head's logits for more than 64 wanted rows): the library
        product again, bfloat16 operands and a float result.
        Everything else, all of float32 included: the plain FMA kernel.
        """
        if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
            M, K = x.shape
            if M <= 64 and K % 8 == 0 and x.stride(0) % 8 == 0 and x.stride(1) == 1:
                return self.linear_skinny(x, weight, out, bias)
            if out.dtype == torch.bfloat16 and x.is_cuda:
                self._check_linear(x, weight, out, bias)
                if bias is None:
                    torch.mm(x, weight.t(), out=out)
                else:
                    torch.addmm(bias, x, weight.t(), out=out)
                return
            if out.dtype == torch.float32 and x.is_cuda:
                # the library's product with a float result: one pass over the weights (a head of 151936 x
                # 4096 at 128 rows: 285 us against 530 for two passes of the weight-streaming kernel)
                self._check_linear(x, weight, out, bias)
                torch.mm(x, weight.t(), out_dtype=torch.float32, out=out)
                if bias is not None:
                    out.add_(bias)
                return
        self.linear_plain(x, weight, out, bias)

    @staticmethod
    def _check_linear(x, weight, out, bias):
        _dev(x, weight, out, bias)
        M, K = x.shape
        N = weight.shape[0]
        if weight.shape != (N, K) or out.shape != (M, N) or x.dtype != weight.dtype:
            raise ValueError(f"linear: x {tuple(x.shape)} {x.dtype}, weight {tuple(weight.shape)} "
                             f"{weight.dtype}, out {tuple(out.shape)}")
        if x.stride(1) != 1 or out.stride(1) != 1 or not weight.is_contiguous():
            raise ValueError("linear: rows must be contiguous")
        if bias is not None and (bias.shape != (N,) or bias.dtype != weight.dtype):
            raise ValueError("linear: bias must be [N] in the weight's dtype")
        return M, N, K

    def linear_plain(self, x, weight, out, bias=None) -> None:
        M, N, K = self._check_linear(x, weight, out, bias)
        library.call("ra_gemm_plain", x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(),
                     _tag(x, "linear input"), _tag(out, "linear output"), M, N, K, x.stride(0),
                     out.stride(0), _stream())

    def linear_skinny(self, x, weight, out, bias=None, accumulate: bool = False, row_sums=None,
                      emit=None, wide: Optional[bool] = None, finish=None):
        """The weight-streaming product; with ``accumulate`` the float32 ``out`` is added to (with more rows
        than the weight-streaming kernels take, by the library's product).

        An RMSNorm can ride on the products around it, y = rstd[m] * ((x .* w) . W^T):
        ``row_sums`` = (ss float32 [parts, M], eps, width) scales result row m by
        rsqrt(sum_p ss[p, m] / width + eps); ``emit`` = (w [N], x_out bfloat16 [M, N],
        ss_out float32 [at least skinny_row_parts(M, N), M]), with ``accumulate`` only, also writes
        bf16(out * w) and each workgroup's sums of squares of its columns of ``out``: into the first
        rows of ss_out, as many as the kernel that ran has workgroups a row; that number comes back.
        ``finish`` = (w [N], x_out bfloat16 [M, N], eps), with ``accumulate`` and 65 to 128 rows, asks for the
        finished norm of the new ``out`` instead, x_out = bf16(rmsnorm(out, eps) * w): True comes back where
        the product that ran wrote it (``can_finish_norm``), False where it only added."""
        M, N, K = self._check_linear(x, weight, out, bias)
        if x.dtype != torch.bfloat16:
            raise TypeError("linear_skinny: bfloat16 only")
        if accumulate and out.dtype != torch.float32:
            raise TypeError("linear_skinny: accumulation is into a float32 matrix")
        if finish is not None:
            if not accumulate or row_sums is not None or emit is not None:
                raise ValueError("linear_skinny: a finished norm rides on a plain accumulating product only")
            if self.can_finish_norm(M, N, K):
                w, xo, eps = finish
                _dev(w, xo)
                if w.shape != (N,) or not w.is_contiguous() or xo.dtype != torch.bfloat16 or xo.shape != (M, N) \
                        or xo.stride(1) != 1:
                    raise ValueError(f"linear_skinny: norm weight {tuple(w.shape)}, finished rows {tuple(xo.shape)} "
                                     f"{xo.dtype}; expected [{N}] and bfloat16 [{M}, {N}]")
                need = int(library.load().ra_gemm_wide_scratch(2, M, N, K, 1))
                scratch = torch.empty(need, dtype=torch.float32, device=x.device)
                library.call("ra_gemm_wide_normed", x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(),
                             _tag(out, "linear output"), 2, M, N, K, x.stride(0), out.stride(0), scratch.data_ptr(),
                             need, None, 0, 0.0, 0, w.data_ptr(), _tag(w, "norm weight"), xo.data_ptr(),
                             xo.stride(0), None, float(eps), _stream())
                return True
            self.linear_skinny(x, weight, out, bias, accumulate=True, wide=wide)
            return False
        if accumulate and M > 64 and bias is None and row_sums is None and emit is None and wide is None \
                and not bool(library.load().ra_gemm_wide_preferred(2, M, N, K)):
            # more rows than the weight-streaming kernels take: the library's product, adding in place
            torch.addmm(out, x, weight.t(), out_dtype=torch.float32, out=out)
            return None
        if row_sums is None and emit is None:
            self._few_rows("linear output", x, weight, bias, out, 2 if accumulate else 0, M, N, K, wide)
            return None
        return self._skinny_normed(x, weight, bias, out, 2 if accumulate else 0, M, N, K, row_sums, emit)

    # Rows up to which an RMSNorm rides on the products around it (``row_sums`` / ``emit``) rather
    # than running as a kernel of its own: all that the weight-streaming products take. Up to 16
    # rows the kernel whose waves split K carries it, above that the other one, which has the
    # registers to spare (the first, at 32 and 64 rows, got slower than with a norm kernel).
    NORM_ON_PRODUCTS_ROWS = 64
    NORM_SKINNY_ROWS = 16
    # Rows up to which the adding kernel of a product cut into K ranges can finish the norm that follows
    # (a whole row a workgroup): the decode steps above the weight-streaming products' rows, whose other
    # products are the library's and can apply no row factor.
    NORM_FINISHED_ROWS = 128

    def can_finish_norm(self, M: int, N: int, K: int) -> bool:
        """True where ``linear_skinny(..., accumulate=True, finish=)`` writes the finished norm: the rows
        between the two limits, a product that the kernel with K ranges takes at these rows, rows of up to
        16384 columns in steps of 8."""
        return self.NORM_ON_PRODUCTS_ROWS < M <= self.NORM_FINISHED_ROWS and N % 8 == 0 and N <= 16384 \
            and K % 8 == 0 and bool(library.load().ra_gemm_wide_preferred(2, M, N, K))

    def _few_rows(self, what, x, weight, bias, out, epilogue, M, N, K, wide: Optional[bool] = None) -> None:
        """The weight-streaming product for up to 64 rows, by one of two kernels: the one whose
        waves split K (best up to 16 rows) or the one whose waves share the activations (it may
        need scratch for partial sums). ``wide`` forces the choice; the library knows where each
        is faster."""
        lib = library.load()
        if wide is None:
            wide = bool(lib.ra_gemm_wide_preferred(epilogue, M, N, K))
        if not wide:
            library.call("ra_gemm_skinny", x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(),
                         _tag(out, what), epilogue, M, N, K, x.stride(0), out.stride(0), _stream())
            return
        need = int(lib.ra_gemm_wide_scratch(epilogue, M, N, K, 0))
        scratch = torch.empty(need, dtype=torch.float32, device=x.device) if need else None
        library.call("ra_gemm_wide", x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(),
                     _tag(out, what), epilogue, M, N, K, x.stride(0), out.stride(0), _ptr(scratch), need,
                     _stream())

    def skinny_row_parts(self, M: int, N: int) -> int:
        """Partial sums a row that ``linear_skinny(..., emit=)`` writes for an [M, N] result at most:
        which of the two kernels runs, and with it the number, depends on the product's K as well."""
        lib = library.load()
        return max(int(lib.ra_gemm_skinny_row_parts(int(M), int(N))), int(lib.ra_gemm_wide_row_parts(int(N))))

    def _emits_from_skinny(self, epilogue: int, M: int, N: int, K: int) -> bool:
        """Whether an emitting product goes to the kernel whose waves split K: up to 16 rows always; up to
        32 where the other kernel would have to cut K into ranges and add them with a second launch for a
        small product (an output projection of 4096 x 4096 at 32 rows: 10 us against 16; the decode step of
        32 requests 6.19 -> 6.01 ms). With more rows the step gains nothing from it (33 and 64 requests:
        within 0.5 %), and the consumer has 16 times the partial sums to add."""
        if M <= self.NORM_SKINNY_ROWS:
            return True
        lib = library.load()
        return M <= 32 and not bool(lib.ra_gemm_wide_preferred(epilogue, M, N, K)) \
            and int(lib.ra_gemm_skinny_row_parts(M, N)) * 16 == N

    def _skinny_normed(self, x, weight, bias, out, epilogue, M, N, K, row_sums, emit) -> None:
        ss = eps = width = None
        parts = 0
        if row_sums is not None:
            ss, eps, width = row_sums
            _dev(ss)
            if ss.dtype != torch.float32 or ss.dim() != 2 or ss.shape[1] != M or not ss.is_contiguous():
                raise ValueError(f"linear_skinny: row sums {tuple(ss.shape)} {ss.dtype}, expected float32 [parts, {M}]")
            parts = ss.shape[0]
        w = xo = so = None
        parts_out = None
        if emit is not None:
            if epilogue != 2:
                raise ValueError("linear_skinny: only an accumulating product emits for a norm")
            w, xo, so = emit
            _dev(w, xo, so)
            lib = library.load()
            parts_out = int(lib.ra_gemm_skinny_row_parts(M, N)) if self._emits_from_skinny(epilogue, M, N, K) \
                else int(lib.ra_gemm_wide_row_parts(N))
            if w.shape != (N,) or not w.is_contiguous():
                raise ValueError(f"linear_skinny: norm weight {tuple(w.shape)}, expected [{N}]")
            if xo.dtype != torch.bfloat16 or xo.shape != (M, N) or xo.stride(1) != 1:
                raise ValueError(f"linear_skinny: scaled copy {tuple(xo.shape)} {xo.dtype}, expected bfloat16 [{M}, {N}]")
            if so.dtype != torch.float32 or so.dim() != 2 or so.shape[0] < parts_out or so.shape[1] != M or not so.is_contiguous():
                raise ValueError(f"linear_skinny: emitted sums {tuple(so.shape)}, expected float32 [{parts_out} or more, {M}]")
        norm_args = (_ptr(ss), parts, float(eps or 0.0), int(width or 0), _ptr(w),
                     _tag(w, "norm weight") if w is not None else 0, _ptr(xo),
                     xo.stride(0) if xo is not None else 0, _ptr(so))
        # the gated product of a wide feed-forward goes to the other kernel at every row count; it
        # takes row sums (any number of parts) and never emits
        gated_wide = epilogue == 1 and emit is None and bool(library.load().ra_gemm_wide_preferred(epilogue, M, N, K))
        to_skinny = self._emits_from_skinny(epilogue, M, N, K) if emit is not None else M <= self.NORM_SKINNY_ROWS
        if to_skinny and not gated_wide:
            library.call("ra_gemm_skinny_normed", x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(),
                         _tag(out, "linear output"), epilogue, M, N, K, x.stride(0), out.stride(0), *norm_args,
                         _stream())
            return parts_out
        need = int(library.load().ra_gemm_wide_scratch(epilogue, M, N, K, 1 if emit is not None else 0))
        scratch = torch.empty(need, dtype=torch.float32, device=x.device) if need else None
        library.call("ra_gemm_wide_normed", x.data_ptr(), weight.data_ptr(), _ptr(bias), out.data_ptr(),
                     _tag(out, "linear output"), epilogue, M, N, K, x.stride(0), out.stride(0), _ptr(scratch),
                     need, *norm_args, -1.0, _stream())
        return parts_out

    def can_accumulate(self, x: torch.Tensor, weight: torch.Tensor) -> bool:
        """True if ``linear_skinny(..., accumulate=True)`` takes this product (out += x . W^T):
        the residual add of an output projection then costs no kernel and no round trip."""
        if not (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and x.stride(1) == 1):
            return False
        M, K = x.shape
        # above 64 rows where the kernel that cuts K into ranges beats the library's product and an add,
        # or where the library's own product adds into the float matrix
        return M <= 64 or self.LIBRARY_ACCUMULATES_FROM <= M <= self.LIBRARY_ACCUMULATES_ROWS \
            or bool(library.load().ra_gemm_wide_preferred(2, M, weight.shape[0], K))

    # Rows up to which the library's product adds into the float residual stream itself (bfloat16 operands, a
    # float matrix read and written): up to here it takes as long as the product with a bfloat16 result
    # (2048 rows, 4096 x 4096: 67 against 69 us; 4096 x 12288: 187 against 191), and the norm kernel behind it
    # reads one matrix less (3072 rows: 95 against 85 and 248 against 275 us); from 4096 rows on it is the slower one
    # (4096: 116 against 95 and 314 against 279 us; 8192: 218 against 179, 620 against 539).
    # Below 129 rows (decode steps of 65 to 128 requests) it is a wash (a step of 96 requests 11.78 against
    # 11.69 ms with the norm kernel's add, of 128 requests 14.28 against 14.36): those steps stay as they were.
    LIBRARY_ACCUMULATES_FROM = 129
    LIBRARY_ACCUMULATES_ROWS = 3072

    GATE_GROUP = 8        # rows of gate, then rows of up, in the weight of gated_linear

    def gated_linear(self, x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, row_sums=None,
                     wide: Optional[bool] = None) -> None:
        """out[M, I] = silu(x . Wg^T) * (x . Wu^T) for ``weight`` [2I, K] whose rows alternate in
        runs of GATE_GROUP: 8 gate rows, the 8 up rows of the same features, and so on.

        bfloat16 with up to 64 rows: one kernel, the gate applied in the product's
        epilogue. Otherwise the product into a [M, 2I] buffer, then the gate kernel."""
        _dev(x, weight, out)
        M, K = x.shape
        I = out.shape[1]
        if weight.shape != (2 * I, K) or out.shape != (M, I) or I % self.GATE_GROUP != 0:
            raise ValueError(f"gated_linear: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
        if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 \
                and M <= 64 and K % 8 == 0 and x.stride(0) % 8 == 0 and x.stride(1) == 1 \
                and weight.is_contiguous() and out.stride(1) == 1:
            if row_sums is None:
                self._few_rows("linear output", x, weight, None, out, 1, M, 2 * I, K, wide)
            else:
                self._skinny_normed(x, weight, None, out, 1, M, 2 * I, K, row_sums, None)
            return
        if row_sums is not None:
            raise ValueError("gated_linear: row sums ride on the weight-streaming product only (bfloat16, <= 64 rows)")
        gu = torch.empty((M, 2 * I), dtype=out.dtype, device=x.device)
        self.linear(x, weight, gu)
        self.silu_mul(gu, out, self.GATE_GROUP)

    # -------------------------------------------------------------- sampling
    def sample(self, logits: torch.Tensor, temperature: torch.Tensor, seeds: torch.Tensor,
               positions: torch.Tensor, tokens: torch.Tensor) -> None:
        _dev(logits, temperature, seeds, positions, tokens)
        n, V = logits.shape
        if logits.dtype != torch.float32 or logits.stride(1) != 1:
            raise TypeError("sample: logits are float32 rows")
        if temperature.dtype != torch.float32 or seeds.dtype != torch.int64:
            raise TypeError("sample: temperature float32, seeds int64")
        _int32(positions, "sample positions", n)
        _int32(tokens, "sampled tokens", n)
        if temperature.numel() < n or seeds.numel() < n:
            raise ValueError("sample: one temperature and seed per row")
        slices = library.load().ra_sample_slices(V)
        val = torch.empty((n, slices), dtype=torch.float32, device=logits.device)
        idx = torch.empty((n, slices), dtype=torch.int32, device=logits.device)
        library.call("ra_sample", logits.data_ptr(), n, V, logits.stride(0), temperature.data_ptr(),
                     seeds.data_ptr(), positions.data_ptr(), val.data_ptr(), idx.data_ptr(),
                     tokens.data_ptr(), _stream())

    def filter_logits(self, logits: torch.Tensor, params, histories) -> None:
        """Logit bias, penalties and top-k / top-p / min-p of every row's SamplingParams, in
        place (removed tokens become -inf); ``histories[i]`` are row i's tokens so far."""
        import numpy as np
        _dev(logits)
        n, V = logits.shape
        if logits.dtype != torch.float32 or logits.stride(1) != 1:
            raise TypeError("filter_logits: logits are float32 rows")
        rec = np.zeros((n, 12), dtype=np.float32)
        irec = rec.view(np.int32)
        window, off = [], 0
        for i, (p, hist) in enumerate(zip(params, histories)):
            rec[i, 0] = max(0.0, float(p.temperature))
            rec[i, 1] = float(p.top_p or 0.0)
            rec[i, 2] = float(p.min_p or 0.0)
            rec[i, 3] = float(p.repeat_penalty or 0.0)
            rec[i, 4] = max(0.0, float(p.frequency_penalty or 0.0))
            rec[i, 5] = max(0.0, float(p.presence_penalty or 0.0))
            irec[i, 6] = int(p.top_k or 0)
            win = list(hist[-p.repeat_last_n:]) if (p.penalties and p.repeat_last_n > 0) else []
            irec[i, 7], irec[i, 8] = off, len(win)
            window += win
            off += len(win)
            bias = getattr(p, "logit_bias", ())
            if bias:
                pairs = np.zeros((len(bias), 2), dtype=np.int32)
                pairs[:, 0] = [int(t) for t, _ in bias]
                pairs[:, 1] = np.asarray([float(b) for _, b in bias], dtype=np.float32).view(np.int32)
                irec[i, 9], irec[i, 10] = off, len(bias)
                window += pairs.reshape(-1).tolist()
                off += 2 * len(bias)
        rows_t = torch.from_numpy(rec).to(logits.device)
        win_t = torch.tensor(window or [0], dtype=torch.int32).to(logits.device)
        library.call("ra_filter_logits", logits.data_ptr(), n, V, logits.stride(0), rows_t.data_ptr(),
                     win_t.data_ptr(), _stream())

    # ------------------------------------------------------------ measurement
    def measure_peaks(self, device="cuda:0", read_bytes: int = 4 << 30) -> dict:
        """What the machine gives at best: GB/s of a plain read of ``read_bytes`` of device memory
        (more than the chip's caches hold) and TFLOP/s of bfloat16 matrix-core products on
        registers, in both instruction shapes. For pricing measured kernels beside the published peaks; not on the product path."""
        import ctypes
        buf = torch.empty(read_bytes // 4, dtype=torch.int32, device=device).random_()
        sink = torch.zeros(1, dtype=torch.int32, device=device)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

        def timed(fn, reps):
            fn()
            torch.cuda.synchronize(device)
            best = float("inf")
            for _ in range(reps):
                e0.record()
                fn()
                e1.record()
                torch.cuda.synchronize(device)
                best = min(best, e0.elapsed_time(e1) * 1e-3)
            return best

        with torch.cuda.device(device):
            t_read = timed(lambda: library.call("ra_stream_read", buf.data_ptr(), read_bytes, sink.data_ptr(), _stream()), 5)
            out = {"hbm_read_GBps": read_bytes / t_read / 1e9}
            for shape, name in ((32, "mfma_bf16_32x32x16_TFLOPs"), (16, "mfma_bf16_16x16x32_TFLOPs")):
                flops = ctypes.c_double(0.0)
                t = timed(lambda: library.call("ra_mfma_loop", shape, 10000, 16, sink.data_ptr(),
                                               ctypes.byref(flops), _stream()), 3)
                out[name] = flops.value / t / 1e12
        del buf
        return out
