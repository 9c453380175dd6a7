"""A decoder as data, and the one class that runs any such description.

``ModelSpec`` says which parts every layer is made of and in which order layers
run. ``DecoderModel`` builds the parts through the registries and runs them over
the step's packed tokens. An architecture is a function from its configuration to
a ``ModelSpec`` plus the names of its checkpoint tensors (``config/registry.py``).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..native import ops
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheView, PagedKVNeed, ParamSpec, Part,
                   StateNeed)


@dataclass
class LayerSpec:
    """One layer: each entry is {"kind": registered name, ...constructor arguments}.

    Which norms a layer has is the block arrangement's affair: a registered block names its norm slots
    (``norm_slots``, the names of its constructor's arguments) and gets one norm built for each, from
    ``norms[slot]`` if the layer names that slot, else from ``norm``."""

    mixer: dict
    feed_forward: dict
    norm: dict | None = None              # the norm of every slot that ``norms`` does not name
    block: dict = field(default_factory=lambda: {"kind": "prenorm"})
    position: str | None = "default"      # name in ModelSpec.positions that the mixer gets, or None
    norms: dict = field(default_factory=dict)   # slot name -> {"kind": ..., ...}

    def norm_spec(self, slot: str) -> dict:
        spec = self.norms.get(slot, self.norm)
        if spec is None:
            raise ValueError(f"the layer's block has a norm slot '{slot}' and the layer names no norm for it")
        return spec


@dataclass
class RunEntry:
    """One step of the run order. ``cache`` names the entry (by its index in the run
    order) whose cache this entry reads without writing; None: the entry has a
    cache of its own and fills it."""

    layer: int
    cache: int | None = None


@dataclass
class ModelSpec:
    vocab_size: int
    hidden_size: int
    layers: list[LayerSpec]
    final_norm: dict
    positions: dict                        # name -> {"kind": ..., ...}; layers refer to these by name
    max_position: int
    tie_embeddings: bool
    run_order: list[RunEntry] | None = None   # None: every layer once, in order
    eos_token_id: int | None = None           # the token that ends a request, if the checkpoint names one
    embed_scale: float | None = None          # the embedding's rows are multiplied by this (in float, then rounded)
    logit_cap: float | None = None            # logits become cap * tanh(logits / cap)
    position_axes: int = 1                    # coordinates of a token's position (a step carries [axes, tokens])

    def order(self) -> list[RunEntry]:
        if self.run_order is None:
            return [RunEntry(i) for i in range(len(self.layers))]
        return self.run_order


class DecoderModel(Part):
    """Embedding, the layers in run order, final norm, and the head on the wanted rows."""

    def __init__(self, spec: ModelSpec, options: dict | None = None):
        """``options``: engine options that are offered to every part's constructor (a part takes those it names,
        see ``Registry.build``); today ``residual_float32``."""
        self.spec = spec
        self.options = options = dict(options or {})
        if spec.position_axes < 1:
            raise ValueError(f"a model has at least one position axis, got {spec.position_axes}")
        self.positions = {name: POSITION_ENCODINGS.build(p, offered=options, max_position=spec.max_position)
                          for name, p in spec.positions.items()}
        self.layers = []
        for ls in spec.layers:
            mixer_args = {}
            if ls.position is not None:
                mixer_args["position"] = self.positions[ls.position]
            mixer = MIXERS.build(ls.mixer, offered=options, **mixer_args)
            ff = FEED_FORWARDS.build(ls.feed_forward, offered=options)
            # the block says which norms it takes; the layer says what each of them is
            slots = getattr(BLOCKS.maker(ls.block.get("kind")), "norm_slots", ())
            norms = {slot: NORMS.build(ls.norm_spec(slot), offered=options) for slot in slots}
            unknown = set(ls.norms) - set(slots)
            if unknown:
                raise ValueError(f"the layer names norms {sorted(unknown)}; its block '{ls.block.get('kind')}' has the "
                                 f"slots {list(slots)}")
            self.layers.append(BLOCKS.build(ls.block, offered=options, mixer=mixer, feed_forward=ff, **norms))
        self.final_norm = NORMS.build(spec.final_norm, offered=options)
        self.run_order = spec.order()
        for i, e in enumerate(self.run_order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run order entry {i} names layer {e.layer}; there are {len(self.layers)}")
            if e.cache is not None:
                if not 0 <= e.cache < i or self.run_order[e.cache].cache is not None:
                    raise ValueError(f"run order entry {i} reads the cache of entry {e.cache}, which must be an "
                                     f"earlier entry with a cache of its own")
                if self.layers[e.layer].mixer.cache_need() != self.layers[self.run_order[e.cache].layer].mixer.cache_need():
                    raise ValueError(f"run order entry {i} and entry {e.cache} need different caches")
        self.embed_weight = None
        self.head_weight = None
        self.cache_views: list[CacheView] = []

    # -- parameters -------------------------------------------------------
    def param_specs(self):
        s = self.spec
        specs = {"embed.weight": ParamSpec((s.vocab_size, s.hidden_size))}
        if not s.tie_embeddings:
            specs["head.weight"] = ParamSpec((s.vocab_size, s.hidden_size))
        return specs

    def children(self):
        out = {f"layers.{i}": layer for i, layer in enumerate(self.layers)}
        out["final_norm"] = self.final_norm
        return out

    def bind(self, params):
        self.embed_weight = params["embed.weight"]
        # tied: the head reads the embedding's own storage (nanovllm/models/qwen3.py:202-203)
        self.head_weight = params["embed.weight"] if self.spec.tie_embeddings else params["head.weight"]

    def to(self, device):
        for p in self.positions.values():
            p.to(device)
        return self

    def recordable(self) -> bool:
        """Whether a step of this model can be recorded into a HIP graph and replayed with other index
        tensors: every part works from the step's device tensors alone."""
        def ok(part) -> bool:
            return part.recordable and all(ok(c) for c in part.children().values())
        return ok(self)

    # -- cache ------------------------------------------------------------
    def cache_needs(self) -> list[PagedKVNeed | StateNeed | None]:
        """Per run-order entry: what cache of its own it needs (None when it has none or borrows one)."""
        out = []
        for e in self.run_order:
            out.append(self.layers[e.layer].mixer.cache_need() if e.cache is None else None)
        return out

    def attach_cache(self, views: list[CacheView]) -> None:
        """``views[i]`` is the cache of run-order entry i (for a borrowing entry: the lender's, with writes off)."""
        if len(views) != len(self.run_order):
            raise ValueError(f"{len(views)} cache views for {len(self.run_order)} run-order entries")
        self.cache_views = views

    # -- the forward pass -------------------------------------------------
    def forward(self, step) -> torch.Tensor:
        """Hidden states after the final norm, for the rows whose logits are wanted only: [n, hidden]."""
        hidden = ops.embed(step.input_ids, self.embed_weight, self.spec.embed_scale)
        residual = None
        order = self.run_order
        for i, (entry, cache) in enumerate(zip(order, self.cache_views)):
            layer = self.layers[entry.layer]
            # a block that knows ``ops.Summed`` (a sum that a product has made already, in place of a tensor still to be
            # added) may hand one on to the norm that comes next, if that knows it too: the next block's first norm, or
            # this model's last
            more = {}
            if getattr(layer, "takes_summed", False):
                if i + 1 == len(order):
                    more["next_norm"] = self.final_norm if getattr(self.final_norm, "takes_summed", False) else None
                else:
                    nxt = self.layers[order[i + 1].layer]
                    if getattr(nxt, "takes_summed", False):
                        more["next_norm"], more["next_reader"] = nxt.mixer_norm, nxt.mixer
            hidden, residual = layer.forward(hidden, residual, step, cache, **more)
        if step.num_logit_rows == 0:
            return None
        # only the wanted rows go through the last norm and the head (nanovllm/layers/embed_head.py:56-61)
        if isinstance(hidden, ops.Summed):    # the last product has added itself to the residual stream already
            hidden, _ = self.final_norm.forward_add(hidden, residual)
            return ops.gather_rows(hidden, step.logit_rows)
        hidden = ops.gather_rows(hidden, step.logit_rows)
        if residual is None:                  # the last block has made its additions itself
            return self.final_norm.forward(hidden)
        residual = ops.gather_rows(residual, step.logit_rows)
        hidden, _ = self.final_norm.forward_add(hidden, residual)
        return hidden

    def logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """float32 logits [n, vocab] (the reference's sampler casts to float first, nanovllm/layers/sampler.py:12)."""
        logits = ops.linear(hidden, self.head_weight, out_dtype=torch.float32)
        if self.spec.logit_cap is not None:
            ops.soft_cap_(logits, self.spec.logit_cap)
        return logits
