"""The step's batch as the parts see it: packed tokens of several requests, with
the index tensors that the kernels need. Built once per step by the engine
(the reference passes the same facts through a module-global ``Context``,
nanovllm/utils/context.py:6-104; here it is an argument)."""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..native.ops import AttentionBatch


@dataclass
class GroupTables:
    """Per cache group: where this step's tokens are stored and where each request's pages are."""

    slot_mapping: torch.Tensor     # [T] int32: page * page_size + offset of every token
    block_tables: torch.Tensor     # [B, max_pages] int32, -1 where there is no page


@dataclass
class StepContext:
    num_tokens: int
    num_requests: int
    input_ids: torch.Tensor        # [T] int32
    positions: torch.Tensor        # [axes, T] int32: every token's position as the position encodings see it
    token_positions: torch.Tensor  # [T] int32: the first axis (all there is for a model of one axis)
    attention: AttentionBatch      # (its ``positions`` are the tokens' indices in their requests: storage and causality)
    groups: list[GroupTables]
    state_slots: torch.Tensor      # [B] int32: each request's row in the state pools
    logit_rows: torch.Tensor | None  # [n] int32: the tokens whose logits are wanted
    num_logit_rows: int = 0
    host: dict = field(default_factory=dict)   # the same facts as Python lists, for parts that work on the host
