"""The kernel contract: every device operation the parts call, with shapes, dtypes and in-place rules.

`holon_amd.kernels.hip.HipKernels` is the only implementation the product has (hand-written gfx950 HIP, loaded from
the in-tree library; it fails loudly when the library is missing). A plain twin with the same methods lives under
`tests/` and is handed to the engine only by tests. The shapes follow the reference's op contracts
(std/holon_std/ops/kernels.py:1-45, std/holon_std/mixers/gqa/kernels.py:1-52), with this engine's cache layout.

Conventions: T tokens in the step, B rows (requests in the step), Hq/Hkv heads, D head_dim, P page size. Activations
and weights are `dtype` (bfloat16 or float32) unless stated; index tensors are int32. Norms, softmax, rotation angles
and every sum are computed in float32 and rounded once to `dtype`.

Cache layout of one page of one site, `pages[page]` = `[2, Hkv, P * D]`: keys as rows `[P, D]` (token-major),
values as columns `[D, P]` (transposed inside the page, so that a matrix-core operand of the value product is one
contiguous 16-byte load). Block table row `slot` lists the page of token positions `i*P .. i*P+P-1` at index i.
"""
from __future__ import annotations

import dataclasses
from typing import Protocol

import torch


@dataclasses.dataclass
class AttnRows:
    """The rows of a step, as attention sees them. Row b reads block table row `slots[b]`, holds `lens[b]` tokens
    including this step's, and owns query tokens `query_start[b]:query_start[b+1]`, the last of its sequence
    ("bottom-right causal": query i of the row sits at position lens[b] - n_query[b] + i). Rows with one query token
    are listed in `decode_rows`, the others in `chunk_rows` (row indices, int32, device). `in_order` says that the
    step is decode rows alone, listed as they lie (a kernel then need not read the lists)."""

    slots: torch.Tensor                  # [B] int32
    lens: torch.Tensor                   # [B] int32
    query_start: torch.Tensor            # [B+1] int32
    decode_rows: torch.Tensor            # [n_decode] int32
    chunk_rows: torch.Tensor             # [n_chunk] int32
    n_decode: int
    n_chunk: int
    max_decode_len: int                  # host bounds for launch shapes
    max_chunk_query: int
    max_chunk_len: int
    in_order: bool = False               # every row is a decode row, and decode_rows[i] = query_start[i] = i


class Kernels(Protocol):
    name: str

    def embedding(self, ids: torch.Tensor, table: torch.Tensor,
                  take: tuple[torch.Tensor, torch.Tensor] | None = None, want_stats: bool = False):
        """ids [T] int32, table [V, H] -> [T, H] (rows of the table). `take` = (take_slot [T] int32, last_token [S]
        int32): token t is last_token[take_slot[t]] where take_slot[t] >= 0 (a token the previous step drew and left
        on the device), ids[t] otherwise. With `want_stats` -> (rows, row statistics or None): see `row_sumsq`."""

    def row_sumsq(self, x: torch.Tensor) -> torch.Tensor:
        """Row statistics of x [M <= 16, H]: float32 [parts, 16] whose column m sums to the sum of squares of row m
        (here parts = 1). A kernel that writes rows may leave the same thing in several parts (`linear_add`); a
        product with a folded norm (`linear(..., row_scale=)`) adds the parts in a fixed order."""

    def folds_norm(self, rows: int, weight: torch.Tensor, tiled: torch.Tensor | None) -> bool:
        """Whether `linear(x, weight, tiled=tiled, row_scale=...)` serves `rows` rows."""

    def rmsnorm(self, x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
        """x [..., dim] contiguous -> a new tensor; x is not modified."""

    def add_rmsnorm(self, x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
        """residual += x in place (sum rounded to dtype), returns rmsnorm(residual) as a new tensor. `x` may be what
        `linear_parts` returned, float32 [S, *residual.shape]: what is added is then the parts' sum in order, rounded
        to the residual's dtype first (the product that `linear` would have returned)."""

    def linear(self, x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype | None = None,
               tiled: torch.Tensor | None = None, row_scale: tuple[torch.Tensor, float] | None = None) -> torch.Tensor:
        """x [T, K] @ weight [N, K].T -> [T, N], float32 accumulation, rounded to x's dtype; with another `out_dtype`
        that rounded product is then cast (the reference's `F.linear(...).float()`, std/holon_std/ops/units.py:348): one
        rule for every number of rows. `tiled`: what `tile_weight(weight)` returned, if anything.
        `row_scale` = (row statistics of x, eps): an RMSNorm folded into the product. `tiled` is then
        `tile_weight(weight, norm_weight)`, x the un-normed rows, and row m of the float32 sums is scaled by
        rsqrt(mean(x[m]^2) + eps) before it is rounded: norm(x) W^T with the rounding of the normed activations
        moved to the folded weights."""

    def tile_weight(self, weight: torch.Tensor, scale: torch.Tensor | None = None) -> torch.Tensor | None:
        """Once per weight after loading: a copy in the layout steps of few rows stream fastest, or None. With
        `scale` [K] the copy holds weight * scale[None, :] (rounded): a norm's weight folded in."""

    def serves_rows(self, rows: int, weight: torch.Tensor, tiled: torch.Tensor | None, gated: bool = False) -> bool:
        """Whether `linear` (gated: `linear_silu_mul`) reads `tiled` for a step of `rows` rows beyond the few-row
        kernels' (17 to 64): a caller whose tiled copy has a norm folded in then passes rows normed without the
        norm's weight."""
        return False

    def linear_parts(self, x: torch.Tensor, weight: torch.Tensor, tiled: torch.Tensor | None) -> torch.Tensor | None:
        """linear(x, weight) as float32 sums over S shares of K, [S, T, N], for a reader that adds them up itself
        (`add_rmsnorm`; `sum_parts` for anyone else): their sum in order, rounded to x's dtype, is the product. None
        when this step is not served that way (then nothing was done); a kernel set serves it only where that is
        faster than `linear` even with the reader's extra reads."""
        return None

    def sum_parts(self, parts: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        """float32 [S, ...] -> [...] in `dtype`: the parts added up in order, rounded once."""

    def linear_add(self, x: torch.Tensor, weight: torch.Tensor, tiled: torch.Tensor | None, residual: torch.Tensor,
                   want_stats: bool = False) -> "bool | torch.Tensor":
        """residual += linear(x, weight) in place in one kernel: the product rounded to dtype, then the sum rounded,
        as the add of `add_rmsnorm` does. False when not fused for this shape; then nothing was done. Otherwise
        True, or with `want_stats` the row statistics of the residual rows as they now are, when the kernel can
        leave them."""

    def linear_silu_mul(self, x: torch.Tensor, weight: torch.Tensor, tiled: torch.Tensor | None = None,
                        row_scale: tuple[torch.Tensor, float] | None = None) -> torch.Tensor | None:
        """silu_mul(linear(x, weight)) fused, with the composition's roundings; None when not fused for this shape.
        `row_scale` as in `linear`."""

    def silu_mul(self, gate_up: torch.Tensor) -> torch.Tensor:
        """gate_up [T, 2I] (gate columns first) -> [T, I] = round(silu(gate)) * up."""

    def rope(self, x: torch.Tensor, positions: torch.Tensor, table: torch.Tensor) -> None:
        """Rotate the first table.shape[1] dims of x [T, heads, D] in place, half-split pairing; table
        [max_positions, rotary_dim] float32 = cos of the rotary_dim/2 angles, then their sin."""

    def kv_write(self, k: torch.Tensor, v: torch.Tensor, pages: torch.Tensor, write_page: torch.Tensor,
                 write_off: torch.Tensor, page_size: int) -> None:
        """k, v [T, Hkv, D] into the cache layout at (write_page[t], write_off[t])."""

    def qk_norm_rope_write(self, qkv: torch.Tensor, heads: int, kv_heads: int, head_dim: int,
                           q_weight: torch.Tensor | None, k_weight: torch.Tensor | None, eps: float,
                           table: torch.Tensor | None, positions: torch.Tensor, pages: torch.Tensor | None,
                           write_page: torch.Tensor | None, write_off: torch.Tensor | None, page_size: int
                           ) -> torch.Tensor:
        """The fused form of per-head rmsnorm (if weights), rope (if table) and kv_write (if pages) on the merged
        projection qkv [T, (Hq + 2 Hkv) D]: q and k heads are normed and rounded, rotated and rounded; k and v go to
        the cache; returns q' [T, Hq, D], a new tensor. Same roundings as the three ops one after the other."""

    def check_attention(self, head_dim: int, page_size: int, dtype: torch.dtype) -> None:
        """Raise, with a message that names the limit, when no attention kernel serves this head size, page size and
        dtype. Mixers call it when they are built, so that a model is refused before it takes a request."""

    def paged_attention(self, q: torch.Tensor, pages: torch.Tensor, table: torch.Tensor, rows: AttnRows,
                        page_size: int, scale: float, window: int) -> torch.Tensor:
        """softmax(q k^T * scale) v per row over its cached tokens, causal; with window W > 0 a query at position p
        sees keys p-W+1 .. p. q [T, Hq, D] -> [T, Hq, D]. This step's keys are already in the cache."""

    def qkv_attention(self, qkv: torch.Tensor, heads: int, kv_heads: int, head_dim: int,
                      q_weight: torch.Tensor | None, k_weight: torch.Tensor | None, eps: float,
                      rope_table: torch.Tensor | None, positions: torch.Tensor, pages: torch.Tensor | None,
                      table: torch.Tensor, write_page: torch.Tensor, write_off: torch.Tensor, rows: AttnRows,
                      page_size: int, scale: float, window: int, writes: bool = True) -> torch.Tensor:
        """`paged_attention(qk_norm_rope_write(qkv, ...), pages, table, rows, ...)` as one operation, with that
        composition's roundings; a kernel set may run it in fewer kernels (a step of decode rows alone). `writes`
        False: the keys and values are not stored (a run that reads another run's cache)."""

    def argmax(self, logits: torch.Tensor) -> torch.Tensor:
        """logits [R, V] float32 -> [R] int32, the first maximal index of each row."""

    def store_tokens(self, last_token: torch.Tensor, slots: torch.Tensor, tokens: torch.Tensor) -> None:
        """last_token[slots[r]] = tokens[r] (all int32, slots distinct): drawn tokens kept on the device by slot."""

    def logprobs(self, logits: torch.Tensor, tokens: torch.Tensor, k: int
                 ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """log_softmax of the raw logits [R, V]: (the log-probability of tokens[r] [R], the k largest ids [R, k] int32,
        their log-probabilities [R, k]); k <= 32; ties go to the lower id."""

    def sample(self, logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
               min_p: torch.Tensor, seeds: torch.Tensor, positions: torch.Tensor,
               slots: torch.Tensor | None = None) -> torch.Tensor:
        """One token per row [R] int32. temperature/top_p/min_p float32, top_k int32, seeds int64: [R], row r's own;
        or, with `slots` [R] int32, tables [S] of which row r reads entry slots[r]. positions [R] int32 or int64 (the
        position of the token being drawn). Rows with temperature 0 take the argmax; the others draw by inverse CDF
        at the hashed uniform of (seed, position): in vocabulary order when the row has no filter (top_k 0, top_p 1,
        min_p 0), else in sorted order (scaled logit descending, equal ones by index)."""

    def scatter_rows(self, dst: torch.Tensor, idx: torch.Tensor, src: torch.Tensor) -> None:
        """dst[idx[r]] = src[r] for int32 rows: dst [N, W], idx [n], src n * W values."""
