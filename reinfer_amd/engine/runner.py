"""The step function: model + cache on one GPU.

``ModelRunner.step(entries)`` runs exactly the tokens it is given, as one
batch, from the cache that earlier steps left, and returns float32 logits at
the wanted places. Generation (scheduler + sampler) and trace replay both call
this one function; neither has a forward pass of its own.
"""
from __future__ import annotations

import math
from typing import Dict, Hashable, List, Optional, Sequence

import torch

from ..cache import CacheManager, OutOfBlocks, plan_groups
from ..config import load_config
from ..config.schema import ModelSpec
from ..models import DecoderModel, declare_params
from ..parts import KVNeed, LayerCache, PagedNeed, StateNeed
from ..weights import check_tensors, load_weights, random_tensor, random_tensors, storage_dtype, weight_from_folder
from .._hostlib import StepError
from .batch import StepBatch, StepEntry, build_step_batch
from .graphs import MAX_GRAPH_BATCH

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
           "fp32": torch.float32, "f32": torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype {dtype}: the engine runs in bfloat16 or float32")
        return dtype
    try:
        return _DTYPES[str(dtype)]
    except KeyError:
        raise ValueError(f"dtype {dtype!r}: expected bfloat16 or float32") from None


class ModelRunner:
    def __init__(self, spec: ModelSpec, weights: Dict[str, torch.Tensor], dtype: torch.dtype,
                 device: torch.device, *, block_size: int = 16, num_blocks: Optional[int] = None,
                 max_tokens: Optional[int] = None, max_seqs: int = 64,
                 max_model_len: Optional[int] = None, memory_fraction: float = 0.9,
                 use_graphs: Optional[bool] = None):
        self.spec = spec
        self.dtype = dtype
        self.device = device
        self._poison = False
        self.last_logits: Optional[torch.Tensor] = None
        self._weight_source = ("given", weights)       # replaced by from_folder / from_config; see get_weight
        self.load_report: Dict[str, object] = {}
        self.block_size = int(block_size)
        self.max_model_len = min(max_model_len or spec.max_positions, spec.max_positions)
        self.max_seqs = int(max_seqs)
        self.model = DecoderModel(spec, weights, dtype, device)
        needs = self.model.cache_needs()

        # which run-order entries keep keys of their own, and with which window
        windows: List[Optional[int]] = []
        for e, need in zip(spec.run_order, needs):
            if isinstance(need, (KVNeed, PagedNeed)) and e.cache_from is None:
                windows.append(need.window)
            else:
                windows.append(None)
        # no layer with keys of its own: no group, no pool, no block tables; requests then hold a state
        # slot each and are admitted by slots alone
        groups = plan_groups(windows)
        self.groups = groups
        group_of = {i: g for g, gs in enumerate(groups) for i in gs.entries}

        if num_blocks is None:
            if max_tokens is not None:
                num_blocks = max(1, -(-int(max_tokens) // self.block_size))
            else:
                num_blocks = self._blocks_that_fit(needs, windows, memory_fraction)
        self.num_blocks = int(num_blocks)
        self.manager = CacheManager(groups, self.block_size, [self.num_blocks] * len(groups), max_seqs)

        # device side of the cache: what each mixer's need names, a tensor of [blocks, *one block] each
        self.caches: List[Optional[LayerCache]] = []
        for i, (e, need) in enumerate(zip(spec.run_order, needs)):
            if isinstance(need, (KVNeed, PagedNeed)):
                if e.cache_from is None:
                    tensors = {}
                    for name, shape, tdtype in need.block_tensors(self.block_size):
                        tensors[name] = torch.zeros((self.num_blocks, *shape), dtype=tdtype or dtype, device=device)
                    self.caches.append(LayerCache(k=tensors.get("k"), v=tensors.get("v"), group=group_of[i],
                                                  writes=True, tensors=tensors))
                else:
                    src = self.caches[e.cache_from]
                    src_need = needs[e.cache_from]
                    if not isinstance(src_need, (KVNeed, PagedNeed)) or \
                            tuple(src_need.block_tensors(self.block_size)) != tuple(need.block_tensors(self.block_size)):
                        raise ValueError(f"run entry {i} cannot read the cache of entry {e.cache_from}: "
                                         "different heads")
                    self.caches.append(LayerCache(k=src.k, v=src.v, group=src.group, writes=False,
                                                  tensors=src.tensors))
            elif isinstance(need, StateNeed):
                state = torch.zeros((max_seqs, *need.shape), dtype=need.dtype, device=device)
                self.caches.append(LayerCache(state=state))
            else:
                self.caches.append(None)

        # decode steps replay captured graphs when every part says it can be captured
        # (a block arrangement says so itself with ``graph_safe``, or it is asked of its ``mixer`` and ``ffn``)
        def block_safe(b) -> bool:
            if hasattr(b, "graph_safe"):
                return bool(b.graph_safe)
            return bool(getattr(getattr(b, "mixer", None), "graph_safe", False)
                        and getattr(getattr(b, "ffn", None), "graph_safe", False))
        safe = all(block_safe(b) for b in self.model.blocks) and \
            (self.model.input_position is None or bool(getattr(self.model.input_position, "graph_safe", False)))
        if use_graphs is None:
            use_graphs = True
        self.graphs = None
        if use_graphs and safe and device.type == "cuda":
            from .graphs import DecodeGraphs
            self.graphs = DecodeGraphs(self)

    # ------------------------------------------------------------ building
    @classmethod
    def from_folder(cls, model_dir: str, dtype="bfloat16", device="cuda:0", allow_unexpected: bool = False,
                    **limits) -> "ModelRunner":
        """``allow_unexpected``: tensors of the folder that the model does not declare are left unread
        (``load_report["unexpected"]`` names them) instead of refused."""
        cfg = load_config(model_dir)
        spec = cfg.to_spec()
        tdtype = parse_dtype(dtype)
        dev = torch.device(device)
        report: Dict[str, object] = {}
        weights = load_weights(model_dir, declare_params(spec), tdtype, dev, allow_unexpected, report)
        runner = cls(spec, weights, tdtype, dev, **limits)
        runner._weight_source = ("folder", model_dir)
        runner.load_report = report
        return runner

    @classmethod
    def from_config(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0",
                    weights: Optional[Dict[str, torch.Tensor]] = None, **limits) -> "ModelRunner":
        """Random weights drawn on ``device`` (or the tensors given), no folder."""
        spec = config.to_spec()
        tdtype = parse_dtype(dtype)
        dev = torch.device(device)
        decls = declare_params(spec)
        source = ("seed", int(seed))
        if weights is None:
            weights = random_tensors(decls, seed, tdtype, dev)
        else:
            check_tensors("weights", decls, weights)
            by = {d.name: d for d in decls}
            source = ("given", weights)
            weights = {n: t.to(storage_dtype(by[n], t.dtype, tdtype)).to(dev) for n, t in weights.items()}
        runner = cls(spec, weights, tdtype, dev, **limits)
        runner._weight_source = source
        return runner

    def get_weight(self, name: str) -> torch.Tensor:
        """The tensor ``name`` as the model was given it (before any fusing or re-laying by the parts), on
        the CPU: read from the folder again, drawn again from the seed, or the caller's own tensor. For
        checking the engine against another implementation with the very same weights
        (crates/cuda/tests/engine_vs_cpu.rs:80-118 reads them back for that)."""
        decls = {d.name: d for d in declare_params(self.spec)}
        if name not in decls:
            raise KeyError(f"{name}: the model declares no such tensor")
        kind, what = self._weight_source
        if kind == "folder":
            return weight_from_folder(what, name)
        if kind == "seed":
            d = decls[name]
            if d.optional:
                raise KeyError(f"{name}: not part of this random model (a tied head)")
            return random_tensor(d, what, self.dtype)
        if name not in what:
            raise KeyError(f"{name}: not among the tensors the model was built from")
        return what[name].detach().cpu()

    def _blocks_that_fit(self, needs, windows, fraction: float) -> int:
        """Blocks per group from free device memory: the reference's budget,
        capacity = utilisation * total - weights, pages = capacity / page bytes
        (crates/memory/src/budget.rs:99-117)."""
        per_block = 0
        for need, w in zip(needs, windows):
            if w is not None:
                for _, shape, tdtype in need.block_tensors(self.block_size):
                    per_block += math.prod(shape) * torch.empty((), dtype=tdtype or self.dtype).element_size()
        if per_block == 0:
            return 1
        if self.device.type != "cuda":
            return 256
        free, total = torch.cuda.mem_get_info(self.device)
        usable = free - (1.0 - fraction) * total
        blocks = int(usable // per_block)
        # no request can hold more than max_model_len tokens, and max_seqs requests are live at most
        cap = self.max_seqs * (-(-self.max_model_len // self.block_size))
        return max(1, min(blocks, cap))

    # ----------------------------------------------------------- requests
    def add_request(self, rid: Hashable) -> None:
        self.manager.add(rid)

    def free_request(self, rid: Hashable) -> None:
        self.manager.free(rid)
        if self._poison:
            self._poison_freed()

    def poison_freed_blocks(self, on: bool = True) -> None:
        """A hook for tests: from now on the keys and values of every block that goes back to its pool (a
        request ended, a window passed it) are overwritten with NaN at once, so that a kernel that reads a
        slot its request no longer holds gives NaN instead of stale values that look right."""
        self._poison = bool(on)
        self.manager.log_freed(self._poison)

    def _poison_freed(self) -> None:
        for g, blocks in enumerate(self.manager.take_freed()):
            if not blocks:
                continue
            idx = torch.tensor(sorted(set(blocks)), dtype=torch.long, device=self.device)
            for cache in self.caches:
                if cache is not None and cache.tensors and cache.writes and cache.group == g:
                    for t in cache.tensors.values():
                        if t.is_floating_point():
                            t[idx] = float("nan")

    def has_request(self, rid: Hashable) -> bool:
        return rid in self.manager

    def num_tokens(self, rid: Hashable) -> int:
        return self.manager.get(rid).num_tokens

    # --------------------------------------------------------------- step
    def step(self, entries: Sequence[StepEntry], observer=None) -> torch.Tensor:
        """Run the entries' tokens as one batch; logits [wanted, vocab] float32,
        in the order of the entries and of each entry's ``want``. The result may be
        a view of a buffer that the next step overwrites: use it before stepping again.
        ``observer(i, hidden)`` sees the hidden state of all the step's tokens behind the embedding
        and behind every layer (such a step never replays a captured graph)."""
        return self.step_sampled(entries, None, observer)[0]

    def can_chain(self, n_entries: int) -> bool:
        """Whether a step of ``n_entries`` single tokens can take its tokens from the device (``token_source``)."""
        return self.graphs is not None and 0 < n_entries <= MAX_GRAPH_BATCH

    def step_sampled(self, entries: Sequence[StepEntry], sampling=None, observer=None, token_source=None):
        """As :meth:`step`; ``sampling`` = (temperatures, seeds, positions), one per entry,
        asks for a token from each entry's single wanted row where the step can draw it
        itself. -> (logits, tokens): ``tokens`` is an int32 device tensor, one per
        entry, or None when the caller has to sample from the logits. ``token_source`` (only for a step
        of single tokens that replays a captured graph, see :meth:`can_chain`): the entries' tokens are
        taken from this device tensor, not from the entries."""
        if not isinstance(entries, list):
            entries = list(entries)
        if token_source is not None and not (self.can_chain(len(entries)) and observer is None
                                             and all(len(e.tokens) == 1 for e in entries)):
            raise ValueError("token_source: only a step of single tokens that replays a captured graph takes its "
                             "tokens from the device")
        # checks every entry (StepError), then takes the blocks of all of them or raises OutOfBlocks
        one_token, one_want, longest = self.manager.begin_step(entries, self.spec.vocab_size,
                                                               self.max_model_len)
        tokens = None
        graphed = self.graphs is not None and one_token and len(entries) <= MAX_GRAPH_BATCH and observer is None
        if graphed:
            all_logits, all_tokens = self.graphs.run(entries, longest, sampling, token_source)
            n = len(entries)
            if one_want:
                logits = all_logits[:n]
                if sampling is not None:
                    tokens = all_tokens[:n]
            else:
                rows = [i for i, e in enumerate(entries) for _ in e.want]
                logits = all_logits[torch.tensor(rows, dtype=torch.long, device=self.device)] if rows \
                    else all_logits[:0]
        else:
            batch = build_step_batch(entries, self.manager, self.device, pin=self.device.type == "cuda")
            logits = self.forward(batch, observer)
        self.manager.end_step(entries)
        if self._poison:
            self._poison_freed()           # blocks a window has passed
        self.last_logits = logits          # for a caller that checks a run's results after timing it
        return logits, tokens

    def forward(self, batch: StepBatch, observer=None) -> torch.Tensor:
        with torch.no_grad():
            if batch.num_logit_rows == 0:
                # still run the layers: the step's keys and values must be stored
                self.model.forward_layers(batch, self.caches, observer)
                return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
            return self.model.forward(batch, self.caches, observer)
