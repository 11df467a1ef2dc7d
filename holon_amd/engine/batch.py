"""What a step is given and what its parts see. core/holon/api/batch.py:123-181 (`BatchPlan`, `DeviceBatch`)."""
from __future__ import annotations

import dataclasses
from typing import Any

import numpy as np
import torch

from ..kernels.api import AttnRows


@dataclasses.dataclass
class StepRow:
    """One request's share of a step: its next `tokens`, the first of them at position `start` (= tokens it already
    has in the cache), and `want`: indices among these tokens whose logits are asked for."""

    slot: int
    start: int
    tokens: list[int]
    want: list[int] = dataclasses.field(default_factory=list)
    on_device: bool = False                      # its one token is the one the previous step drew for this slot and
                                                 # left on the device (`tokens` then holds a placeholder)


@dataclasses.dataclass
class PagedView:
    """A paged group during one step."""

    page_size: int
    table: torch.Tensor                          # [max_seqs + 1, max_pages] int32, device
    write_page: torch.Tensor                     # [T] int32: where each of the step's tokens is stored
    write_off: torch.Tensor                      # [T] int32


@dataclasses.dataclass
class Step:
    """The context parts are called with: the step's tokens as flat device tensors, rows as ranges of them."""

    kernels: Any
    n_tokens: int
    n_rows: int
    token_ids: torch.Tensor                      # [T] int32
    positions: torch.Tensor                      # [T] int32
    token_row: torch.Tensor                      # [T] int32: the row each token belongs to
    slots: torch.Tensor                          # [B] int32
    starts: torch.Tensor                         # [B] int32: tokens the row had before this step
    rows: AttnRows
    paged: dict[int, PagedView]
    h_slots: np.ndarray                          # host copies, for parts that plan on the host
    h_starts: np.ndarray
    h_counts: np.ndarray
    token_take: tuple[torch.Tensor, torch.Tensor] | None = None   # (take_slot [T], last_token [S+1]): tokens that the
                                                 # previous step drew and left on the device replace token_ids there

    @property
    def query_start(self) -> torch.Tensor:
        return self.rows.query_start

    @property
    def lens(self) -> torch.Tensor:
        return self.rows.lens
