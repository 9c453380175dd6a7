"""The model on the GPU and the one step function.

``ModelRunner`` reads the configuration, builds the model from parts, loads the
weights, makes the cache (pages per group of layers, state pools per slot) and
offers ``step``: a batch of (request, its next tokens, the places whose logits are
wanted). A step runs only the tokens it is given, all requests as one packed
batch, against what earlier steps left in the cache, and returns float32 logits
for the wanted places. Prompt portions of any length and single decoded tokens are
the same kind of entry. Sampling is not done here.

The reference's runner builds two kinds of batch (nanovllm/engine/model_runner.py:
924-1146) and never mixes them in one forward pass; its index tensors
(``slot_mapping``, ``block_tables``, ``cu_seqlens_q``, ``context_lens``, positions)
have the same meaning here.
"""
from __future__ import annotations

import sys
from dataclasses import dataclass, field
from typing import Hashable

import numpy as np
import torch

from ..cache.manager import NO_PAGE, CacheManager, OutOfPages, PagedGroupSpec
from ..config.model_config import read_config_json
from ..config.registry import resolve_architecture
from ..native.ops import AttentionBatch
from ..parts.base import CacheView, PagedKVNeed, StateNeed
from ..parts.context import GroupTables, StepContext
from ..parts.model import DecoderModel
from ..weights.loader import load_weights

_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass
class StepEntry:
    """One request's share of a step."""

    request_id: Hashable
    tokens: list[int]                       # its next tokens (at least one)
    want: list[int] = field(default_factory=list)   # places among ``tokens`` whose logits are returned
    # the tokens' positions as the position encodings see them, [axes][tokens]; None: on every axis a token's
    # position is its index in the request. (Where a token's key is stored and which keys it may read follows
    # from its index alone.)
    positions: list[list[int]] | None = None


class ModelRunner:
    def __init__(self, model_dir: str, dtype: str = "bfloat16", device: str = "cuda:0", page_size: int = 256,
                 num_pages: int | None = None, num_state_slots: int = 512, gpu_memory_utilization: float = 0.9,
                 max_num_batched_tokens: int = 16384, model=None, arch=None, cfg=None, use_graphs: bool = False,
                 max_model_len: int | None = None, max_graph_batch: int = 64, poison_freed_pages: bool = False,
                 share_prefixes: bool = False, residual_float32: bool = True, max_graph_tokens: int = 256,
                 gemm_table: dict | None = None, measure_gemms: bool = True, fuse_norms: bool = True):
        """``model``/``arch``/``cfg`` may be given ready-made (weights already bound)
        instead of being read from ``model_dir``.
        ``gemm_table``: this engine's own table of how each shape of bfloat16 matrix product is done (None: the
        process-wide table, in which a shape is timed once for all engines); ``measure_gemms``: whether shapes that
        the table lacks may be timed. Both are put in force whenever this runner steps, so engines of one process
        do not change each other's products."""
        if dtype not in _TORCH_DTYPES:
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}")
        self.dtype = _TORCH_DTYPES[dtype]
        self.device = torch.device(device)
        if model is None:
            raw = read_config_json(model_dir)
            arch = resolve_architecture(raw)
            cfg = arch.parse_config(raw)
            # engine options that parts may care for are offered to every part's constructor
            model = DecoderModel(arch.build_spec(cfg), options={"residual_float32": bool(residual_float32)})
            load_weights(model, arch, cfg, model_dir, self.dtype, self.device)
        self.arch, self.cfg, self.model = arch, cfg, model
        self.model.to(self.device)
        # what the engine above needs to know of the model comes from the model's description, not from the
        # architecture's typed configuration (whose fields are the architecture's own affair)
        self.vocab_size = model.spec.vocab_size
        self.max_position = model.spec.max_position
        self.eos_token_id = model.spec.eos_token_id
        self.page_size = page_size
        # a model whose positions have several coordinates gets them as an array of their own in every step; for the
        # others the tokens' indices are the positions, unless an entry brings positions of its own
        self.position_axes = model.spec.position_axes
        if share_prefixes and poison_freed_pages:
            raise ValueError("a freed page keeps its content for later requests when prefixes are shared; "
                             "poison_freed_pages would destroy it")
        self.share_prefixes = share_prefixes
        self.gemm_table, self.measure_gemms = gemm_table, bool(measure_gemms)
        # bfloat16 products of up to 16 rows may make the residual addition that follows them and the norm that comes
        # before them in their own kernels (two kernels fewer a layer in a decoding step)
        self.fuse_norms = bool(fuse_norms)
        self._pinned = None
        self._pinned_free = None
        # a debugging aid: pages that are given back are filled with NaN, so that a read of a page that a
        # request no longer owns shows up in its logits
        self.poison_freed_pages = poison_freed_pages
        # decode-only steps replay a HIP graph per batch-size bucket (the reference captures CUDA graphs for
        # the same batch sizes, nanovllm/engine/model_runner.py:2559-2594). In bfloat16 a graph may hold the
        # library's matrix products beside the own kernels: from 17 rows on always (measured faster than the own
        # kernel there), for fewer rows where a measurement of the shape says so. Run eagerly, a step of 17 to 48
        # requests is bound by its launches (8.3 ms at every size). A graph with a library call in it is checked
        # when it is recorded: replayed three times, with eager work and waits between, and compared bit by bit
        # with the eager result; a bucket whose graph fails runs eagerly from then on.
        self.use_graphs = bool(use_graphs) and self.device.type == "cuda" and self.model.recordable()
        self.max_model_len = min(max_model_len or self.max_position, self.max_position)
        self.max_graph_batch = max_graph_batch
        # batch sizes that have a graph: a step is padded to the next one
        self.graph_buckets = self._bucket_sizes(max_graph_batch)
        self._graphs: dict[int, dict | None] = {}     # None: the bucket's graph failed its check
        # Short steps of any make (portions of prompts, beside decoded tokens or alone) are bound by their launches as
        # well: some 350 kernels of a few microseconds each against 15 to 20 us of host work a launch. A step of up to
        # ``max_graph_tokens`` tokens in which every request wants at most one place replays a graph too, recorded for
        # (tokens, requests) rounded up to the next sizes of ``mixed_token_buckets`` and ``mixed_request_buckets``: the tokens
        # that fill the bucket belong to a request of their own, whose keys are the zeros of the spare page and which
        # stores nothing, and the requests that fill it have no tokens. 0 switches this off.
        self.max_graph_tokens = max_graph_tokens if self.use_graphs else 0
        self.mixed_token_buckets = self._token_bucket_sizes(self.max_graph_tokens)
        self.mixed_request_buckets = [b for b in (1, 4, 16, 64) if b < max_graph_batch] + [max_graph_batch]
        self._mixed_graphs: dict[tuple[int, int], dict | None] = {}
        self.graph_check = torch.equal                # (replay, eager) -> bool; a test replaces it to force a refusal
        self.graphs_rerecorded = 0                    # graphs recorded again because the contexts had outgrown their layout
        # all recorded steps share one pool of memory: they replay one after the other on one stream, so what one
        # needs between its kernels can be what another needed; each keeps only its own logits and index arrays
        self._graph_pool = None
        self.probe = None                             # what the cache's sizing measured (see _pages_from_free_memory)
        self._make_cache(page_size, num_pages, num_state_slots, gpu_memory_utilization, max_num_batched_tokens)

    # ------------------------------------------------------------------ cache
    def _make_cache(self, page_size, num_pages, num_state_slots, utilization, max_tokens):
        needs = self.model.cache_needs()
        windows: list[int | None] = []                 # one group per distinct window
        self._entry_group: dict[int, int] = {}
        for i, need in enumerate(needs):
            if isinstance(need, PagedKVNeed):
                if need.window not in windows:
                    windows.append(need.window)
                self._entry_group[i] = windows.index(need.window)
        if not windows:
            windows = [None]                           # a model without paged layers still has one (empty) group
        self._windows = windows
        if self.share_prefixes and any(isinstance(n, StateNeed) for n in needs):
            # state of fixed size summarises all earlier tokens: pages alone do not bring a prefix back
            # (the reference switches the page hashes off for such models, nanovllm/config.py:384-399)
            raise ValueError("prefixes cannot be shared by a model with per-request state")
        # the pools of per-request state come first, so that the pages are counted from what is left
        # (the reference splits its budget between the two, nanovllm/engine/model_runner.py:723-775).
        # One row more than there are slots: the padding rows of a recorded step work on it.
        self.state_pools: list[dict] = []
        self._state_views: dict[int, CacheView] = {}
        self.num_state_slots = num_state_slots
        for i, need in enumerate(needs):
            if isinstance(need, StateNeed):
                pool = {name: torch.zeros((num_state_slots + 1, *shape), dtype=dt, device=self.device)
                        for name, (shape, dt) in need.tensors.items()}
                self.state_pools.append(pool)
                self._state_views[i] = CacheView(kind="state", state=pool)
        item = torch.empty((), dtype=self.dtype).element_size()
        page_bytes = sum(2 * page_size * n.num_kv_heads * n.head_dim * item
                         for n in needs if isinstance(n, PagedKVNeed))
        if num_pages is None:
            num_pages = self._pages_from_free_memory(page_bytes, utilization, max_tokens)
        self._allocate_pages(num_pages)

    def _allocate_pages(self, num_pages: int) -> None:
        """The cache manager and the key/value tensors for ``num_pages`` pages per group, attached to the model."""
        needs = self.model.cache_needs()
        page_size = self.page_size
        self.num_pages = num_pages
        groups = [PagedGroupSpec(name="all keys" if w is None else f"window {w}", page_size=page_size,
                                 num_pages=num_pages, window=w) for w in self._windows]
        self.cache = CacheManager(groups, self.num_state_slots, share_prefixes=self.share_prefixes)
        views: list[CacheView | None] = [None] * len(needs)
        views[:] = [self._state_views.get(i) for i in range(len(needs))]
        self.kv_tensors: list[torch.Tensor] = []       # the pages that requests may hold, per cache unit
        for i, need in enumerate(needs):
            if isinstance(need, PagedKVNeed):
                # [2, pages + 1, page_size, kv_heads, head_dim]: one token's heads lie together
                # (nanovllm/engine/model_runner.py:870-906). The last page is handed to no request and holds zeros:
                # the padding rows of a recorded step read their one key there.
                kv = torch.empty((2, num_pages + 1, page_size, need.num_kv_heads, need.head_dim),
                                 dtype=self.dtype, device=self.device)
                kv[:, num_pages].zero_()
                self.kv_tensors.append(kv[:, :num_pages])
                views[i] = CacheView(kind="paged", group=self._entry_group[i], k=kv[0], v=kv[1], writes=True)
        for i, e in enumerate(self.model.run_order):
            if e.cache is not None:
                lender = views[e.cache]
                views[i] = CacheView(kind=lender.kind, group=lender.group, k=lender.k, v=lender.v, writes=False,
                                     state=lender.state)
            elif views[i] is None:
                views[i] = CacheView(kind="none")
        self.model.attach_cache(views)

    def _pages_from_free_memory(self, page_bytes, utilization, max_tokens) -> int:
        """budget = total * utilization - used - room for a step's activations - room for the recorded steps
        (nanovllm/engine/model_runner.py:654-699,839-861). As the reference does, the room is measured, not
        computed: on a cache just large enough for it, the largest step that the engine can be asked for is run
        once eagerly (``max_tokens`` tokens of as many requests as there are state slots, every request wanting
        a row of logits) and the allocator's peak over what it held before is the activations' room; the
        largest recorded steps of both kinds are recorded once, and what they add to the allocator's reserve
        beyond their own logits is the room of the pool that all recorded steps share. Every recorded step's own
        logits and index arrays are counted by their sizes. Then the probe's cache is given back and the pages
        are what the budget has left. The weights and the state pools are allocated already and count as used."""
        if page_bytes == 0:
            return 1
        free, total = torch.cuda.mem_get_info(self.device)
        # the probe's step: single tokens of all but one request, the rest of the tokens in requests as long as allowed
        tokens = max(1, max_tokens)
        slots = max(1, self.num_state_slots)
        lengths = [1] * min(slots - 1, max(0, tokens - 1))
        rest = tokens - len(lengths)
        while rest > 0 and len(lengths) < slots:
            n = min(rest, self.max_model_len)
            lengths.append(n)
            rest -= n
        probe_pages = sum(-(-n // self.page_size) for n in lengths)
        if (probe_pages + 1) * page_bytes > total * utilization - (total - free):
            raise RuntimeError(f"no memory left for the cache: {free / 2**30:.1f} GiB free of {total / 2**30:.1f}; the "
                               f"largest step alone needs {probe_pages} pages of {page_bytes / 2**20:.1f} MiB")
        self._allocate_pages(probe_pages)
        try:
            torch.cuda.synchronize(self.device)
            torch.cuda.reset_peak_memory_stats(self.device)
            held = torch.cuda.memory_allocated(self.device), torch.cuda.memory_reserved(self.device)
            entries = [StepEntry(("probe", i), [0] * n, [n - 1]) for i, n in enumerate(lengths)]
            logits = self.step(entries)
            torch.cuda.synchronize(self.device)
            del logits
            activations = max(torch.cuda.max_memory_allocated(self.device) - held[0],
                              torch.cuda.max_memory_reserved(self.device) - held[1])
            for e in entries:
                self.finish(e.request_id)
            shared_pool, own = 0, 0
            s = self.model.spec
            if self.use_graphs:
                width = -(-self.max_model_len // self.page_size)
                # the largest recorded step of single tokens and the largest of any other make, recorded here once
                most = min(self.max_graph_batch, slots, probe_pages)
                bucket = max([b for b in self.graph_buckets if b <= most], default=None)
                def reserved() -> int:                 # what the allocator holds, without blocks it only keeps for later
                    torch.cuda.synchronize(self.device)
                    torch.cuda.empty_cache()
                    return torch.cuda.memory_reserved(self.device)

                if bucket is not None:
                    before = reserved()
                    ids = [("probe", i) for i in range(bucket)]
                    self.step([StepEntry(r, [0], []) for r in ids])
                    self.step([StepEntry(r, [0], [0]) for r in ids])
                    for r in ids:
                        self.finish(r)
                    shared_pool += max(0, reserved() - before - bucket * s.vocab_size * 4)
                t = max([t for t in self.mixed_token_buckets if t - 1 <= min(self.max_model_len, probe_pages * self.page_size)],
                        default=None)
                if t is not None and t >= 2:
                    before = reserved()
                    self.step([StepEntry(("probe", 0), [0] * (t - 1), [t - 2])])
                    self.finish(("probe", 0))
                    shared_pool += max(0, reserved() - before - s.vocab_size * 4)
                # every recorded step's own: float32 logits of its rows, and its index arrays (block tables of full width)
                row = s.vocab_size * 4 + (width * len(self._windows) + 16) * 4
                own = sum(b * row for b in self.graph_buckets)
                own += sum(rb * row + tb * 16 for tb in self.mixed_token_buckets for rb in self.mixed_request_buckets)
                # and the matrix products of every new size of step are timed once: a sweep of the caches and a workspace
                from ..native import ops
                backend = ops.backend()
                if self.measure_gemms and hasattr(backend, "library_workspace"):
                    own += (512 << 20) + 2 * getattr(backend, "library_workspace", 0)
        finally:
            # the probe's cache, its graphs and whatever the allocator kept go back to the device
            self._graphs.clear()
            self._mixed_graphs.clear()
            self._graph_pool = None
            self.graphs_rerecorded = 0
            self.model.attach_cache([CacheView(kind="none") for _ in self.model.run_order])
            self.kv_tensors = []
            self.cache = None
            self._pinned = self._pinned_free = None
            torch.cuda.synchronize(self.device)
            torch.cuda.empty_cache()
        free, total = torch.cuda.mem_get_info(self.device)
        budget = total * utilization - (total - free) - activations - shared_pool - own
        pages = int(budget // page_bytes)
        self.probe = {"tokens": tokens, "requests": len(lengths), "activation_bytes": int(activations),
                      "graph_pool_bytes": int(shared_pool), "graph_own_bytes": int(own)}
        if pages <= 0:
            raise RuntimeError(f"no memory left for the cache: {free / 2**30:.1f} GiB free of {total / 2**30:.1f}, "
                               f"one page needs {page_bytes / 2**20:.1f} MiB")
        return pages

    @staticmethod
    def _token_bucket_sizes(largest: int) -> list[int]:
        """Token counts that have a recorded short step: powers of two from 16 on and the sizes half way between, up to
        ``largest`` (a step is padded to the next one: at the 8B shape a token of padding costs about 13 us)."""
        sizes = sorted({t for p in range(4, 24) for t in (1 << p, 3 << p >> 1)})
        return [t for t in sizes if t < largest] + [largest] if largest else []

    @staticmethod
    def _bucket_sizes(largest: int) -> list[int]:
        """Batch sizes that have a recorded step: powers of two and the sizes half way between, up to ``largest``."""
        sizes = sorted({b for p in range(24) for b in (1 << p, 3 << p >> 1) if b >= 1})
        return [b for b in sizes if b < largest] + [largest]

    # ------------------------------------------------------------------ the step
    def _fill_host_buffer(self, arrays: list[np.ndarray]) -> torch.Tensor:
        """The step's index arrays one after the other in host memory (pinned, and reused from step to step, where
        the device is a GPU)."""
        total = sum(a.size for a in arrays)
        if self.device.type == "cuda":
            if self._pinned is None or self._pinned.numel() < total:
                self._pinned = torch.empty(max(total, 4096) * 2, dtype=torch.int32, pin_memory=True)
                self._pinned_free = None
            if self._pinned_free is not None:
                self._pinned_free.synchronize()      # the last step's copy has read the buffer
            host = self._pinned[:total]
        else:
            host = torch.empty(total, dtype=torch.int32)
        flat = host.numpy()
        offset = 0
        for a in arrays:
            flat[offset:offset + a.size] = a.reshape(-1)
            offset += a.size
        return host

    def _copy_issued(self) -> None:
        """Marks the point after which the host buffer may be written again."""
        if self.device.type == "cuda":
            self._pinned_free = torch.cuda.Event()
            self._pinned_free.record()

    def _stage(self, arrays: list[np.ndarray]) -> list[torch.Tensor]:
        """All index arrays of a step go to the device in one copy."""
        sizes = [a.size for a in arrays]
        host = self._fill_host_buffer(arrays)
        dev = host.to(self.device, non_blocking=True)
        self._copy_issued()
        out, offset = [], 0
        for a, n in zip(arrays, sizes):
            out.append(dev[offset:offset + n].view(a.shape))
            offset += n
        return out

    def _layout(self, entries: list[StepEntry], pad_to: int | None = None, table_width: int | None = None,
                pad_tokens_to: int | None = None):
        """Reserves pages and lays the batch out as int32 arrays on the host.
        ``pad_to``: number of requests the arrays are made for (a graph's bucket; only for
        single-token entries): the padding rows store nothing and their results are dropped.
        ``table_width``: fixed width of the block tables.
        Everything that can be wrong with the entries is found before anything is taken from the cache: a step
        that is refused leaves no request admitted and no page reserved."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        cache = self.cache
        seen = set()
        need = [0] * len(cache.groups)
        new_requests = 0
        for e in entries:
            if e.request_id in seen:
                raise ValueError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.request_id!r}: a step entry needs at least one token")
            low, high = (e.tokens[0], e.tokens[0]) if n == 1 else (min(e.tokens), max(e.tokens))
            if low < 0 or high >= self.vocab_size:
                bad = low if low < 0 else high
                raise ValueError(f"token id {bad} is outside the vocabulary of {self.vocab_size}")
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"request {e.request_id!r}: wanted place {w} is outside its {n} tokens")
            if e.positions is not None:
                if len(e.positions) != self.position_axes or any(len(row) != n for row in e.positions):
                    raise ValueError(f"request {e.request_id!r}: positions must be [{self.position_axes}][{n}] "
                                     f"(axes of the model, tokens of the entry)")
                for row in e.positions:
                    if min(row) < 0 or max(row) >= self.max_position:
                        raise ValueError(f"request {e.request_id!r}: a position is outside the model's "
                                         f"{self.max_position} positions")
            known = e.request_id in cache
            new_requests += not known
            new_len = (cache.num_tokens(e.request_id) if known else 0) + n
            if new_len > self.max_position:
                raise ValueError(f"request {e.request_id!r}: {new_len} tokens exceed the model's "
                                 f"{self.max_position} positions")
            for gi, g in enumerate(cache.groups):
                if table_width is not None and -(-new_len // g.page_size) > table_width:
                    raise ValueError(f"request {e.request_id!r}: {new_len} tokens need more than the {table_width} "
                                     f"pages of {g.page_size} that max_model_len {self.max_model_len} allows")
            for gi, k in enumerate(cache.pages_needed(e.request_id if known else None, new_len)):
                need[gi] += k
        for gi, k in enumerate(need):
            if k > cache.num_free_pages(gi):
                raise OutOfPages(f"group '{cache.groups[gi].name}': the step needs {k} more pages, "
                                 f"{cache.num_free_pages(gi)} are free")
        if new_requests > cache.num_free_slots():
            raise OutOfPages(f"the step brings {new_requests} new requests, {cache.num_free_slots()} state slots are free")
        if pad_tokens_to is not None:
            return self._layout_general(entries, pad_to, table_width, pad_tokens_to)
        if all(len(e.tokens) == 1 for e in entries):
            return self._layout_single_tokens(entries, pad_to, table_width)
        return self._layout_general(entries, pad_to, table_width)

    def _layout_general(self, entries: list[StepEntry], pad_to: int | None, table_width: int | None,
                        pad_tokens_to: int | None = None):
        """``pad_to`` requests of one token each fill the batch (a graph of single tokens); or, with ``pad_tokens_to``
        (a graph of a short step of any make), ``pad_to`` requests without tokens and one more that owns the
        ``pad_tokens_to - T`` tokens which fill the bucket."""
        cache = self.cache
        starts, new_lens = [], []
        for e in entries:
            if e.request_id not in cache:
                cache.admit(e.request_id)
            start = cache.num_tokens(e.request_id)
            new_len = start + len(e.tokens)
            cache.reserve(e.request_id, new_len)
            starts.append(start)
            new_lens.append(new_len)

        B = len(entries)
        pad = 0 if pad_to is None else pad_to - B
        real_tokens = sum(len(e.tokens) for e in entries)
        if pad_tokens_to is None:
            pad_q = [1] * pad
        else:
            pad_q = [0] * pad + [pad_tokens_to - real_tokens]
            pad += 1
        q_lens = np.array([len(e.tokens) for e in entries] + pad_q, dtype=np.int32)
        T = int(q_lens.sum())
        cu = np.zeros(B + pad + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu[1:])
        input_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries] + [np.zeros(T - real_tokens, np.int32)])
        token_req = np.repeat(np.arange(B + pad, dtype=np.int32), q_lens)
        positions = (np.arange(T, dtype=np.int32) - np.repeat(cu[:-1], q_lens)
                     + np.repeat(np.array(starts + [0] * pad, dtype=np.int32), q_lens))
        context_lens = np.array(new_lens + pad_q, dtype=np.int32)
        # (padding rows work on the spare row of the state pools)
        state_slots = np.array([cache.state_slot(e.request_id) for e in entries] + [self.num_state_slots] * pad,
                               dtype=np.int32)
        rows = [int(cu[i]) + w for i, e in enumerate(entries) for w in e.want]

        arrays = [input_ids, positions, token_req, cu, context_lens, state_slots]
        for gi, g in enumerate(cache.groups):
            tables = [cache.block_table(e.request_id, gi) for e in entries]
            width = table_width or max(1, max(len(t) for t in tables))
            # padding rows read their keys on the spare page (zeros) and store nothing (slot -1)
            bt = np.full((B + pad, width), NO_PAGE, dtype=np.int32)
            if pad_tokens_to is None:
                bt[B:, 0] = self.num_pages
            else:
                bt[-1, :max(1, -(-int(pad_q[-1]) // g.page_size))] = self.num_pages
            slot_mapping = np.full(T, -1, dtype=np.int32)
            for i, t in enumerate(tables):
                ta = np.asarray(t, dtype=np.int32)
                bt[i, :len(t)] = ta
                p = positions[cu[i]:cu[i + 1]]
                pages = ta[p // g.page_size]
                if (pages == NO_PAGE).any():
                    raise RuntimeError(f"request {entries[i].request_id!r}: a new token falls on a page that was given back")
                slot_mapping[cu[i]:cu[i + 1]] = pages * g.page_size + p % g.page_size
            arrays += [slot_mapping, bt]
        arrays += self._position_rows(entries, positions, cu)
        meta = {"B": B + pad, "T": T, "rows": rows, "starts": starts, "new_lens": new_lens,
                "q_lens": q_lens.tolist(), "state_slots": state_slots.tolist(),
                "max_q_len": int(q_lens.max()), "max_context_len": int(max(new_lens))}
        return arrays, meta

    def _position_rows(self, entries: list[StepEntry], index: np.ndarray, cu) -> list[np.ndarray]:
        """The positions as the position encodings see them, [axes, T], as one more array of the step; nothing for a
        model of one axis whose entries bring no positions of their own (the tokens' indices are the positions).
        Padding tokens keep their index."""
        explicit = any(e.positions is not None for e in entries)
        if self.position_axes == 1 and not explicit:
            return []
        rows = np.repeat(index[None, :], self.position_axes, axis=0)
        for i, e in enumerate(entries):
            if e.positions is not None:
                rows[:, int(cu[i]):int(cu[i + 1])] = np.asarray(e.positions, dtype=np.int32)
        return [np.ascontiguousarray(rows, dtype=np.int32)]

    def _layout_single_tokens(self, entries: list[StepEntry], pad_to: int | None, table_width: int | None):
        """``_layout`` for a step in which every request brings one token (a decoding step): the same arrays,
        built from plain lists (this runs between two steps, while the GPU waits)."""
        cache = self.cache
        B = len(entries)
        pad = 0 if pad_to is None else pad_to - B
        starts, ids, slots, rows = [], [], [], []
        for i, e in enumerate(entries):
            if e.request_id not in cache:
                cache.admit(e.request_id)
            start = cache.num_tokens(e.request_id)
            cache.reserve(e.request_id, start + 1)
            starts.append(start)
            ids.append(e.tokens[0])
            slots.append(cache.state_slot(e.request_id))
            rows += [i] * len(e.want)
        n = B + pad
        new_lens = [s + 1 for s in starts]
        zeros = [0] * pad
        arrays = [np.array(ids + zeros, dtype=np.int32), np.array(starts + zeros, dtype=np.int32),
                  np.arange(n, dtype=np.int32), np.arange(n + 1, dtype=np.int32),
                  np.array(new_lens + [1] * pad, dtype=np.int32),
                  np.array(slots + [self.num_state_slots] * pad, dtype=np.int32)]
        for gi, g in enumerate(cache.groups):
            tables = [cache.block_table(e.request_id, gi) for e in entries]
            width = table_width or max(1, max(len(t) for t in tables))
            # padding rows read their one key on the spare page (zeros) and store nothing (slot -1)
            flat, slot_mapping = [], [-1] * n
            ps = g.page_size
            for i, t in enumerate(tables):
                flat += t
                flat += [NO_PAGE] * (width - len(t))
                page = t[starts[i] // ps]
                if page == NO_PAGE:
                    raise RuntimeError(f"request {entries[i].request_id!r}: a new token falls on a page that was given back")
                slot_mapping[i] = page * ps + starts[i] % ps
            flat += ([self.num_pages] + [NO_PAGE] * (width - 1)) * pad
            bt = np.array(flat, dtype=np.int32).reshape(n, width)
            arrays += [np.array(slot_mapping, dtype=np.int32), bt]
        arrays += self._position_rows(entries, arrays[1], arrays[3])
        meta = {"B": n, "T": n, "rows": rows, "starts": starts, "new_lens": new_lens, "q_lens": [1] * n,
                "state_slots": slots + [self.num_state_slots] * pad, "max_q_len": 1, "max_context_len": max(new_lens)}
        return arrays, meta

    def _context(self, dev: list[torch.Tensor], meta: dict, logit_rows: torch.Tensor | None, num_logit_rows: int,
                 max_context_len: int) -> StepContext:
        d_ids, d_pos, d_req, d_cu, d_ctx, d_slots = dev[:6]
        num_groups = len(self.cache.groups)
        groups = [GroupTables(slot_mapping=dev[6 + 2 * gi], block_tables=dev[7 + 2 * gi]) for gi in range(num_groups)]
        # the positions of the position encodings: an array of their own if the step carries one, else the indices
        positions = dev[6 + 2 * num_groups] if len(dev) > 6 + 2 * num_groups else d_pos.view(1, -1)
        attention = AttentionBatch(num_tokens=meta["T"], num_requests=meta["B"], token_req=d_req, positions=d_pos,
                                   cu_seqlens_q=d_cu, context_lens=d_ctx, max_q_len=meta["max_q_len"],
                                   max_context_len=max_context_len)
        return StepContext(num_tokens=meta["T"], num_requests=meta["B"], input_ids=d_ids, positions=positions,
                           token_positions=positions[0], attention=attention, groups=groups, state_slots=d_slots, logit_rows=logit_rows,
                           num_logit_rows=num_logit_rows,
                           host={k: meta[k] for k in ("starts", "new_lens", "q_lens", "state_slots")})

    def build_context(self, entries: list[StepEntry]) -> tuple[StepContext, list[int]]:
        """Reserves pages, lays out the batch and copies it to the device. Returns the context and every
        request's new length."""
        arrays, meta = self._layout(entries)
        rows = np.array(meta["rows"], dtype=np.int32)
        dev = self._stage(arrays + [rows])
        ctx = self._context(dev[:-1], meta, dev[-1] if len(rows) else None, len(rows), meta["max_context_len"])
        return ctx, meta["new_lens"]

    @torch.no_grad()
    def step(self, entries: list[StepEntry], keep: bool = True) -> torch.Tensor | None:
        """Runs the batch and returns float32 logits [wanted, vocab] in the order of the
        entries and of each entry's ``want`` (None if nothing is wanted). With ``keep=False`` the result may be
        memory that the next step overwrites (a caller that samples at once saves the copy)."""
        self._use_own_choices()
        # (a recorded step of a model with one position axis has no array for positions of an entry's own)
        recorded = self.use_graphs and (self.position_axes > 1 or all(e.positions is None for e in entries))
        if recorded and len(entries) <= self.max_graph_batch and all(len(e.tokens) == 1 for e in entries):
            bucket = next(b for b in self.graph_buckets if b >= len(entries))
            if self._graphs.get(bucket, ...) is not None:
                return self._graph_step(entries, bucket, keep)
        elif recorded and self.max_graph_tokens and len(entries) <= self.max_graph_batch and all(len(e.want) <= 1 for e in entries):
            tokens = sum(len(e.tokens) for e in entries)
            # the bucket is strictly larger than the step: the request that owns the filling tokens has at least one,
            # so every request of the padded batch, also one without tokens, has its first row inside the batch
            # (a part may index rows by ``cu_seqlens_q[:-1]``)
            token_bucket = next((t for t in self.mixed_token_buckets if t > tokens), None)
            if token_bucket is not None:
                key = (token_bucket, next(b for b in self.mixed_request_buckets if b >= len(entries)))
                # (the tokens that fill a bucket stand at positions below the bucket's size: the model must have them)
                if key[0] <= self.max_model_len and self._mixed_graphs.get(key, ...) is not None:
                    return self._mixed_graph_step(entries, key, keep)
        ctx, new_lens = self.build_context(entries)
        if self.device.type == "cuda":
            from ..native import ops
            backend = ops.backend()
            backend.step_number = getattr(backend, "step_number", 0) + 1      # (shapes that come again, step after step, are measured)
        hidden = self.model.forward(ctx)
        logits = self.model.logits(hidden) if hidden is not None else None
        for e, n in zip(entries, new_lens):
            self._poison(self.cache.commit(e.request_id, n, e.tokens))
        return logits

    def _use_own_choices(self) -> None:
        """This engine's table of matrix-product choices, and its leave to time, are the ones in force from here on."""
        from ..native import ops
        backend = ops.backend()
        backend.fuse_norms = self.fuse_norms
        if self.device.type == "cuda" and hasattr(backend, "use_choices"):
            backend.use_choices(self.gemm_table, self.measure_gemms)

    def _poison(self, given_back: list[list[int]]) -> None:
        if not self.poison_freed_pages or not any(given_back):
            return
        for view in self.model.cache_views:
            if view.kind == "paged" and view.writes and given_back[view.group]:
                pages = torch.tensor(given_back[view.group], device=self.device)
                view.k[pages] = float("nan")
                view.v[pages] = float("nan")

    # ------------------------------------------------------------------ decode steps as HIP graphs
    def _graph_step(self, entries: list[StepEntry], bucket: int, keep: bool = True) -> torch.Tensor | None:
        """A step of single tokens: the batch is padded to the bucket, written into the bucket's fixed index
        buffer, and the bucket's graph (embedding to logits of every row) is replayed."""
        width = -(-self.max_model_len // self.page_size)
        arrays, meta = self._layout(entries, pad_to=bucket, table_width=width)
        g = self._graphs.get(bucket)
        # a graph's kernels are laid out for the context lengths of the step that recorded it, g["planned"]; when the
        # longest context is half as long again, or less than half of it, a new graph is recorded (the old one is dropped)
        # (no graph is made for less than 256 keys: short contexts share one)
        longest = max(256, meta["max_context_len"])
        if g is None or not g["planned"] // 2 < longest <= g["covered"]:
            self.graphs_rerecorded += g is not None
            # (a graph recorded again holds the same library calls as the one before it, which passed its check:
            # it is replayed and compared once, not three times with eager work between)
            g = self._capture(bucket, arrays, meta, width, len(entries), checks=3 if g is None else 1)
            self._graphs[bucket] = g if g["graph"] is not None else None
        if g["graph"] is not None:
            g["index"].copy_(self._fill_host_buffer(arrays), non_blocking=True)
            self._copy_issued()
            g["graph"].replay()
        # (a graph that failed its check leaves the eager result of this very step in g["logits"])
        for e, n in zip(entries, meta["new_lens"]):
            self._poison(self.cache.commit(e.request_id, n, e.tokens))
        rows = meta["rows"]
        if not rows:
            return None
        if rows == list(range(len(entries))):
            return g["logits"][:len(entries)].clone() if keep else g["logits"][:len(entries)]
        return g["logits"][torch.tensor(rows, device=self.device)]

    def _mixed_graph_step(self, entries: list[StepEntry], key: tuple[int, int], keep: bool = True) -> torch.Tensor | None:
        """A short step of any make: padded to the bucket (tokens, requests), written into the bucket's fixed index
        buffer, and the bucket's graph is replayed. One graph serves every context length: nothing in such a step is
        laid out for the lengths (the attention of prompt portions takes its bounds from the device)."""
        token_bucket, request_bucket = key
        width = -(-self.max_model_len // self.page_size)
        arrays, meta = self._layout(entries, pad_to=request_bucket, table_width=width, pad_tokens_to=token_bucket)
        # the places whose logits are wanted, one row per request of the bucket (unused rows repeat row 0)
        rows = meta["rows"]
        arrays.append(np.array(rows + [0] * (request_bucket - len(rows)), dtype=np.int32))
        g = self._mixed_graphs.get(key)
        if g is None:
            # (a step that wants no logits still has its first token's row computed by the graph: that row is compared)
            g = self._capture_mixed(key, arrays, meta, width, max(len(rows), 1))
            self._mixed_graphs[key] = g if g["graph"] is not None else None
        if g["graph"] is not None:
            g["index"].copy_(self._fill_host_buffer(arrays), non_blocking=True)
            self._copy_issued()
            g["graph"].replay()
        for e, n in zip(entries, meta["new_lens"]):
            self._poison(self.cache.commit(e.request_id, n, e.tokens))
        if not rows:
            return None
        return g["logits"][:len(rows)].clone() if keep else g["logits"][:len(rows)]

    def _capture_mixed(self, key: tuple[int, int], arrays: list[np.ndarray], meta: dict, width: int, num_real: int) -> dict:
        index, dev = self._index_buffer(arrays)
        token_bucket, request_bucket = key
        meta = dict(meta, max_q_len=token_bucket)            # (the launch is made for the longest portion the bucket can hold)
        ctx = self._context(dev[:-1], meta, dev[-1], request_bucket, max_context_len=width * self.page_size)
        graph, logits = self._record(ctx, f"{token_bucket} tokens of {request_bucket} requests", num_real, planned=0)
        return {"graph": graph, "index": index, "logits": logits, "ctx": ctx}

    # ------------------------------------------------------------------ a decoding step issued ahead of its tokens
    def can_step_ahead(self, request_ids: list) -> bool:
        """Whether the next tokens of these requests can be run before the host knows them (``step_ahead``):
        a recorded graph for their number, laid out for their lengths, and a cache whose commits can be taken back."""
        if not (self.use_graphs and request_ids and len(request_ids) <= self.max_graph_batch
                and not self.cache.share_prefixes and all(g.window is None for g in self.cache.groups)):
            return False
        g = self._graphs.get(next(b for b in self.graph_buckets if b >= len(request_ids)))
        if g is None or g["graph"] is None:
            return False
        real = max(self.cache.num_tokens(r) for r in request_ids) + 1
        longest = max(256, real)                       # (short contexts share one graph, as in _graph_step)
        need = [0] * len(self.cache.groups)
        for r in request_ids:
            for gi, n in enumerate(self.cache.pages_needed(r, self.cache.num_tokens(r) + 1)):
                need[gi] += n
        return (g["planned"] // 2 < longest <= g["covered"] and real <= self.max_model_len
                and real <= self.max_position and all(n <= self.cache.num_free_pages(gi) for gi, n in enumerate(need)))

    @torch.no_grad()
    def step_ahead(self, request_ids: list, tokens: torch.Tensor) -> dict:
        """Issues the decoding step that feeds ``tokens[i]`` (int32, on the device: what the sampling kernel has
        just been asked for, not yet known to the host) to ``request_ids[i]``, by the graph of that size; only after
        ``can_step_ahead``. The GPU goes from one step into the next while the host still waits for the tokens,
        finishes the step before and plans: between two steps that the host issues in turn the GPU waits 0.1 to
        0.3 ms. Returns what ``logits_ahead`` and ``undo_ahead`` need."""
        self._use_own_choices()
        entries = [StepEntry(r, [0], [0]) for r in request_ids]
        bucket = next(b for b in self.graph_buckets if b >= len(entries))
        g = self._graphs[bucket]
        width = -(-self.max_model_len // self.page_size)
        arrays, meta = self._layout(entries, pad_to=bucket, table_width=width)
        g["index"].copy_(self._fill_host_buffer(arrays), non_blocking=True)
        self._copy_issued()
        g["index"][:len(entries)].copy_(tokens[:len(entries)])     # the token ids are the first of the index arrays
        # state of fixed size cannot be stepped back: what these requests' rows hold now is kept until the step's
        # turn has come (a few rows per pool)
        slots = meta["state_slots"][:len(entries)]
        kept = None
        if self.state_pools:
            at = g["ctx"].state_slots[:len(entries)].long()
            kept = [{name: t[at] for name, t in pool.items()} for pool in self.state_pools]
        g["graph"].replay()
        for e, n in zip(entries, meta["new_lens"]):
            self.cache.commit(e.request_id, n)
        return {"requests": list(request_ids), "starts": meta["starts"], "logits": g["logits"], "slots": slots,
                "kept_state": kept}

    def logits_ahead(self, ahead: dict, request_ids: list) -> torch.Tensor:
        """The logits of ``request_ids`` (some or all of the step's, in any order) from a step issued ahead."""
        if request_ids == ahead["requests"]:
            return ahead["logits"][:len(request_ids)]
        place = {r: i for i, r in enumerate(ahead["requests"])}
        return ahead["logits"][torch.tensor([place[r] for r in request_ids], device=self.device)]

    def undo_ahead(self, ahead: dict, request_ids: list) -> None:
        """Takes a step issued ahead back for these of its requests, as far as they still hold anything: their
        tokens count as not fed (the keys and values it stored are stored again, the same, when the step is run
        in its turn)."""
        rows, slots = [], []
        for i, (r, start) in enumerate(zip(ahead["requests"], ahead["starts"])):
            if r in request_ids and r in self.cache and self.cache.num_tokens(r) == start + 1:
                self.cache.rewind(r, start)
                rows.append(i)
                slots.append(ahead["slots"][i])
        if rows and ahead["kept_state"] is not None:
            rows_t = torch.tensor(rows, device=self.device)
            slots_t = torch.tensor(slots, device=self.device)
            for pool, kept in zip(self.state_pools, ahead["kept_state"]):
                for name, t in pool.items():
                    t[slots_t] = kept[name][rows_t]

    def _index_buffer(self, arrays: list[np.ndarray]) -> tuple[torch.Tensor, list[torch.Tensor]]:
        """A graph's fixed buffer of index arrays, filled with these, and the views of the arrays in it."""
        sizes = [a.size for a in arrays]
        index = torch.zeros(sum(sizes), dtype=torch.int32, device=self.device)
        index.copy_(torch.from_numpy(np.concatenate([a.reshape(-1) for a in arrays])))
        dev, offset = [], 0
        for a, n in zip(arrays, sizes):
            dev.append(index[offset:offset + n].view(a.shape))
            offset += n
        return index, dev

    def _capture(self, bucket: int, arrays: list[np.ndarray], meta: dict, width: int, num_real: int, checks: int = 3) -> dict:
        """The graph of a step of single tokens for ``bucket`` requests."""
        index, dev = self._index_buffer(arrays)
        all_rows = torch.arange(bucket, dtype=torch.int32, device=self.device)
        ctx = self._context(dev, meta, all_rows, bucket, max_context_len=width * self.page_size)
        # the graph's launches are fixed: kernels that split the keys plan for this step's longest context, and their
        # splits (and the splits' results) cover contexts of up to half as much again; the block tables are made for
        # max_model_len. The graph serves contexts from half of ``planned`` to ``covered`` and is replaced beyond.
        planned = max(256, meta["max_context_len"])
        covered = planned + planned // 2                   # (the kernels cut it down to what the block tables can hold)
        graph, logits = self._record(ctx, f"{bucket} requests", num_real, planned, checks, covered)
        return {"graph": graph, "index": index, "logits": logits, "ctx": ctx, "planned": planned, "covered": covered}

    def _record(self, ctx: StepContext, what: str, num_real: int, planned: int, checks: int = 3, covered: int = 0):
        """Runs the step of ``ctx`` once eagerly on its fixed buffers (so that every kernel library is loaded
        and the allocator is warm), then records it, and checks the graph if a library call went into it. Returns
        (graph, its logits), or (None, the eager step's logits) if the step cannot be recorded or its graph fails.
        A model with per-request state is stepped several times here on the same tokens: the state that the
        step found is put back before each run, so that all of them, and the caller's, start from it."""
        from ..native import ops
        backend = ops.backend()
        with_library = self.dtype == torch.bfloat16           # (the float32 path has kernels of its own throughout)
        old = (getattr(backend, "own_kernels_only", False), getattr(backend, "planned_context", 0),
               getattr(backend, "measure_linears", False), getattr(backend, "covered_context", 0))
        backend.own_kernels_only = False
        backend.measure_linears = True                        # few-rows products of new shapes are timed both ways, once
        backend.planned_context = planned
        backend.covered_context = covered
        state_slots = ctx.state_slots.long()
        found = [{name: t[state_slots] for name, t in pool.items()} for pool in self.state_pools]

        def put_state_back():
            for pool, rows in zip(self.state_pools, found):
                for name, t in pool.items():
                    t[state_slots] = rows[name]

        try:
            # warm-up; it writes the same cache slots as every replay will. A run in which a product's shape was
            # measured is run again: how one product is done can depend on what was found out about a later one, and
            # the recorded step is compared with an eager one that was done the same way throughout
            for _ in range(3):
                known = len(getattr(backend, "chosen", ()))
                eager = self.model.logits(self.model.forward(ctx)).clone()
                torch.cuda.synchronize()
                if len(getattr(backend, "chosen", ())) == known:
                    break
                put_state_back()
            graph = torch.cuda.CUDAGraph()
            try:
                if self._graph_pool is None:
                    self._graph_pool = torch.cuda.graph_pool_handle()
                with torch.cuda.graph(graph, pool=self._graph_pool):
                    logits = self.model.logits(self.model.forward(ctx))
            except RuntimeError as err:                       # something in the step cannot be recorded
                print(f"[nanohybrid_vlm_amd] no graph for {what} ({str(err).splitlines()[0][:200]}); "
                      "steps of this size run eagerly", file=sys.stderr, flush=True)
                return None, eager
            if with_library or self.state_pools:
                for _ in range(checks):
                    logits.fill_(float("nan"))
                    put_state_back()
                    graph.replay()
                    torch.cuda.synchronize()
                    # (the rows of the requests: what the padding rows hold is nobody's result)
                    if not self.graph_check(logits[:num_real], eager[:num_real]):
                        print(f"[nanohybrid_vlm_amd] the graph for {what} differs from the eager step when "
                              "replayed; steps of this size run eagerly", file=sys.stderr, flush=True)
                        return None, eager
                    if checks > 1:
                        put_state_back()
                        self.model.logits(self.model.forward(ctx))      # eager work between the replays
                        torch.cuda.synchronize()
            put_state_back()                                  # the caller replays the graph for this very step
        finally:
            backend.own_kernels_only, backend.planned_context, backend.measure_linears, backend.covered_context = old
            if hasattr(backend, "end_measurements"):
                backend.end_measurements()
        return graph, logits

    def get_memory_stats(self) -> dict:
        """Bytes of weights, cache and state pools, pages per group, and the allocator's and the device's view
        (nanovllm/engine/model_runner.py:260-371 reports the same kinds of figures)."""
        params = getattr(self.model, "parameters", {}) or {}
        seen, weight_bytes = set(), 0
        for t in params.values():
            if t.data_ptr() not in seen:                    # a tied head shares the embedding's storage
                seen.add(t.data_ptr())
                weight_bytes += t.numel() * t.element_size()
        stats = {
            "weight_bytes": weight_bytes,
            "kv_cache_bytes": sum(t.numel() * t.element_size() for t in self.kv_tensors),
            "state_pool_bytes": sum(t.numel() * t.element_size() for pool in self.state_pools for t in pool.values()),
            "page_size": self.page_size,
            "groups": [{"name": g.name, "window": g.window, "pages": g.num_pages,
                        "free_pages": self.cache.num_free_pages(i)} for i, g in enumerate(self.cache.groups)],
            "live_requests": len(self.cache.requests),
            "prefix_cache": {"enabled": self.cache.share_prefixes, "known_pages": len(self.cache.page_of_hash),
                             "shared_tokens": self.cache.num_shared_tokens},
            "graphs_recorded": sorted(b for b, g in self._graphs.items() if g is not None),
            "graphs_refused": sorted(b for b, g in self._graphs.items() if g is None),
            "graphs_rerecorded": self.graphs_rerecorded,
            "cache_sizing_probe": self.probe,
            "mixed_graphs_recorded": sorted(k for k, g in self._mixed_graphs.items() if g is not None),
            "mixed_graphs_refused": sorted(k for k, g in self._mixed_graphs.items() if g is None),
        }
        if self.device.type == "cuda":
            free, total = torch.cuda.mem_get_info(self.device)
            stats.update(device_free_bytes=free, device_total_bytes=total,
                         torch_allocated_bytes=torch.cuda.memory_allocated(self.device),
                         torch_reserved_bytes=torch.cuda.memory_reserved(self.device))
        return stats

    def finish(self, request_id) -> None:
        """The request is over: its pages and its state slot are given back."""
        if request_id in self.cache:
            self._poison(self.cache.release(request_id))
