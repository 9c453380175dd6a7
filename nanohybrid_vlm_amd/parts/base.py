"""What every part of a model is: a thing with sizes given at construction, a list
of the tensors it needs, and a ``forward`` over the step's packed tokens.

No part reads a model configuration or knows which model it is in: the
architecture's builder turns the configuration into constructor arguments
(as the reference's layers take theirs, nanovllm/models/qwen3.py:16-27,93-98).
"""
from __future__ import annotations

import inspect
from dataclasses import dataclass, field
from typing import Callable

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One tensor that a part needs."""

    shape: tuple[int, ...]
    init: str = "normal"          # random-weights mode: "normal" N(0, 0.02^2), "norm" 1 + N(0, 0.1^2), "zeros"
    keeps_float32: bool = False   # a tensor stored in 32-bit stays so even in a bfloat16 run


@dataclass(frozen=True)
class PagedKVNeed:
    """A mixer that stores a key and a value per token."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None     # None: all keys; n: only the last n are read


@dataclass(frozen=True)
class StateNeed:
    """A mixer with state of fixed size per request: name -> (shape of one request's state, dtype)."""

    tensors: dict = field(default_factory=dict)

    def __hash__(self):
        return hash(tuple(sorted((k, tuple(v[0]), str(v[1])) for k, v in self.tensors.items())))


@dataclass
class CacheView:
    """The cache that one entry of the run order works on."""

    kind: str                              # "paged" | "state" | "none"
    group: int = 0                         # paged: which block tables and slot mapping of the step
    k: torch.Tensor | None = None          # paged: [pages, page_size, kv_heads, head_dim]
    v: torch.Tensor | None = None
    writes: bool = True                    # False: the entry reads a cache that another entry fills
    state: dict | None = None              # state: name -> [slots, ...]


class Part:
    """Base of mixers, feed-forwards, norms, position encodings and blocks."""

    # True: ``forward`` reads the step only through its device tensors and launches the same kernels whatever
    # they hold, so a step can be recorded into a HIP graph and replayed. A part that loops over the step's
    # host lists (``step.host``), or whose launches depend on values, says False; steps of a model with such a
    # part always run eagerly.
    recordable = True

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def children(self) -> dict[str, "Part"]:
        return {}

    def bind(self, params: dict[str, torch.Tensor]) -> None:
        """Receives this part's own tensors (names as in ``param_specs``)."""
        for name, tensor in params.items():
            setattr(self, name.replace(".", "_"), tensor)

    # -- walking the tree -------------------------------------------------
    def walk(self):
        """This part and every part below it."""
        yield self
        for child in self.children().values():
            yield from child.walk()

    def all_param_specs(self, prefix: str = "") -> dict[str, ParamSpec]:
        out = {prefix + k: v for k, v in self.param_specs().items()}
        for cname, child in self.children().items():
            out.update(child.all_param_specs(f"{prefix}{cname}."))
        return out

    def bind_all(self, params: dict[str, torch.Tensor], prefix: str = "") -> None:
        if prefix == "":
            self.parameters = params            # the whole tree's tensors by name, kept at the root
        own = {k: params[prefix + k] for k in self.param_specs()}
        self.bind(own)
        for cname, child in self.children().items():
            child.bind_all(params, f"{prefix}{cname}.")


class Registry:
    """Name -> constructor for one kind of part."""

    def __init__(self, what: str):
        self.what = what
        self._makers: dict[str, Callable] = {}

    def register(self, kind: str):
        def deco(maker):
            if kind in self._makers:
                raise ValueError(f"{self.what} '{kind}' is already registered")
            self._makers[kind] = maker
            return maker
        return deco

    def unregister(self, kind: str) -> None:
        self._makers.pop(kind, None)

    def kinds(self) -> list[str]:
        return sorted(self._makers)

    def maker(self, kind: str):
        if kind not in self._makers:
            raise KeyError(f"unknown {self.what} '{kind}'; registered: {self.kinds()}")
        return self._makers[kind]

    def build(self, spec: dict, offered: dict | None = None, **extra):
        """``spec`` = {"kind": name, ...constructor arguments}. ``extra``: further arguments that the maker must
        take. ``offered``: engine options that every part is offered; a maker gets those it names among its
        parameters (or all of them if it takes ``**kwargs``) and never hears of the others."""
        spec = dict(spec)
        maker = self.maker(spec.pop("kind", None))
        if offered:
            params = inspect.signature(maker).parameters
            takes_any = any(p.kind is inspect.Parameter.VAR_KEYWORD for p in params.values())
            extra = dict({k: v for k, v in offered.items() if (takes_any or k in params) and k not in spec}, **extra)
        return maker(**spec, **extra)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block")
