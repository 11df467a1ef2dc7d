"""Plain twins of the device kernels: one slow torch function per operation of `holon_amd.kernels.api.Kernels`, with
the same arguments and the same cache layout. Two uses: the yardstick each HIP kernel is compared with, alone, on the
GPU; and a stand-in that lets the engine's logic (cache, step function, scheduler) run on the CPU in tests. The product
never falls back to it.

Formulas: std/holon_std/ops/reference.py:7-30 (norms, rope), std/holon_std/ffn/reference.py:7-12 (silu_mul),
std/holon_std/mixers/gqa/reference.py:26-60 (paged attention), :91-101 (kv write),
std/holon_std/sampling/sampler.py:24-61 (uniform, inverse CDF).
"""
from __future__ import annotations

import torch


def _up(x):
    """float32 for the arithmetic; float64 inputs (a test's exact yardstick) stay float64."""
    return x if x.dtype == torch.float64 else x.float()


def _rmsnorm(x, w, eps):
    x32 = _up(x)
    return (x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps) * _up(w)).to(x.dtype)


def _rope(x, positions, table):
    rd = table.shape[1]
    cs = table[positions.long()]
    cos, sin = cs[:, None, : rd // 2], cs[:, None, rd // 2:]
    a, b = _up(x[..., : rd // 2]), _up(x[..., rd // 2: rd])
    return torch.cat(((a * cos - b * sin).to(x.dtype), (b * cos + a * sin).to(x.dtype), x[..., rd:]), dim=-1)


def _mix32(x):
    m = 0xFFFFFFFF
    x = x ^ (x >> 16)
    x = (x * 0x7FEB352D) & m
    x = x ^ (x >> 15)
    x = (x * 0x846CA68B) & m
    return x ^ (x >> 16)


class TorchKernels:
    name = "torch-plain"

    fold_norms = False       # a test may switch the folded-norm path on: the twin then stands in for the tiled copy
    split_products = 0       # a test may set a number of shares: steps of 17 to 128 rows then get their products that
                             # are added to the residual stream as partial sums over that many shares of K

    def __getattr__(self, name):
        """An operation a part registered for itself (`holon_amd.kernels.registry`): its plain form."""
        from holon_amd.kernels.registry import kernel_op
        op = kernel_op(name) if not name.startswith("_") else None
        if op is None:
            raise AttributeError(f"TorchKernels has no operation {name!r}")
        return op.plain

    def embedding(self, ids, table, take=None, want_stats=False):
        if take is not None:
            take_slot, last_token = take
            ids = torch.where(take_slot >= 0, last_token[take_slot.clamp(min=0).long()], ids)
        rows = table[ids.long()]
        if not want_stats:
            return rows
        return rows, (self.row_sumsq(rows) if self.fold_norms and rows.shape[0] <= 16 else None)

    def row_sumsq(self, x):
        stats = torch.zeros(1, 16, dtype=torch.float32, device=x.device)
        stats[0, : x.shape[0]] = x.float().pow(2).sum(-1)
        return stats

    def rmsnorm(self, x, weight, eps):
        return _rmsnorm(x, weight, eps)

    def add_rmsnorm(self, x, residual, weight, eps):
        if x.dim() == residual.dim() + 1:                    # partial sums of a product: added up in order, rounded
            x = self.sum_parts(x, residual.dtype)
        residual.add_(x)
        return _rmsnorm(residual, weight, eps)

    def tile_weight(self, weight, scale=None):
        """No tile layout here. With `scale` (and `fold_norms`) the stand-in for a folded copy: the scaled rows."""
        if scale is None or not self.fold_norms:
            return None
        return (_up(weight) * _up(scale)[None, :]).to(weight.dtype)

    def folds_norm(self, rows, weight, tiled):
        return tiled is not None and rows <= 16

    def serves_rows(self, rows, weight, tiled, gated=False):
        """With `fold_norms`, steps of 17 to 64 rows read the stand-in for the tiled copy, as the HIP kernels do for
        weights with many tiles."""
        return tiled is not None and self.fold_norms and 16 < rows <= 64

    @staticmethod
    def _scaled(x, folded, row_scale):
        stats, eps = row_scale
        inv = torch.rsqrt(stats.sum(0)[: x.shape[0]] / x.shape[1] + eps)
        return (_up(x) @ _up(folded).T) * inv[:, None].to(_up(x).dtype)

    def linear(self, x, weight, out_dtype=None, tiled=None, row_scale=None):
        if row_scale is not None:
            return self._scaled(x, tiled, row_scale).to(x.dtype).to(out_dtype or x.dtype)
        if self.serves_rows(x.shape[0], weight, tiled):
            weight = tiled                                   # (folded or not: what the caller's rows were prepared for)
        return (_up(x) @ _up(weight).T).to(x.dtype).to(out_dtype or x.dtype)      # rounded to x's dtype, then cast

    def linear_parts(self, x, weight, tiled):
        s, k = self.split_products, x.shape[1]
        if not s or not 16 < x.shape[0] <= 128 or k % s:
            return None
        share = k // s
        return torch.stack([_up(x[:, i * share:(i + 1) * share]) @ _up(weight[:, i * share:(i + 1) * share]).T
                            for i in range(s)])

    def sum_parts(self, parts, dtype):
        total = parts[0].clone()
        for part in parts[1:]:
            total += part
        return total.to(dtype)

    def linear_add(self, x, weight, tiled, residual, want_stats=False):
        if self.split_products and 16 < x.shape[0] <= 128:
            return False                                     # as the HIP kernels: not fused at these row counts
        residual.copy_((_up(residual) + _up(self.linear(x, weight))).to(residual.dtype))
        if want_stats and self.fold_norms and residual.shape[0] <= 16:
            return self.row_sumsq(residual)
        return True

    def linear_silu_mul(self, x, weight, tiled=None, row_scale=None):
        if row_scale is None and self.serves_rows(x.shape[0], weight, tiled, gated=True):
            return self.silu_mul(self.linear(x, weight, None, tiled))
        if row_scale is None:
            return None
        return self.silu_mul(self._scaled(x, tiled, row_scale).to(x.dtype))

    def silu_mul(self, gate_up):
        gate, up = gate_up.chunk(2, dim=-1)
        return torch.nn.functional.silu(_up(gate)).to(gate.dtype) * up

    def rope(self, x, positions, table):
        x.copy_(_rope(x, positions, table))

    def kv_write(self, k, v, pages, write_page, write_off, page_size):
        t, hkv, d = k.shape
        kp = pages[:, 0].view(-1, hkv, page_size, d)
        vp = pages[:, 1].view(-1, hkv, d, page_size)
        kp[write_page.long(), :, write_off.long()] = k
        vp[write_page.long(), :, :, write_off.long()] = v

    def qk_norm_rope_write(self, qkv, heads, kv_heads, head_dim, q_weight, k_weight, eps, table, positions, pages,
                           write_page, write_off, page_size):
        t = qkv.shape[0]
        q = qkv[:, : heads * head_dim].reshape(t, heads, head_dim)
        k = qkv[:, heads * head_dim: (heads + kv_heads) * head_dim].reshape(t, kv_heads, head_dim)
        v = qkv[:, (heads + kv_heads) * head_dim:].reshape(t, kv_heads, head_dim)
        if q_weight is not None:
            q, k = _rmsnorm(q, q_weight, eps), _rmsnorm(k, k_weight, eps)
        if table is not None:
            q, k = _rope(q, positions, table), _rope(k, positions, table)
        if pages is not None:
            self.kv_write(k, v, pages, write_page, write_off, page_size)
        return q.contiguous()

    def check_attention(self, head_dim, page_size, dtype):
        return None

    def paged_attention(self, q, pages, table, rows, page_size, scale, window):
        t, hq, d = q.shape
        hkv = pages.shape[2]
        kp = pages[:, 0].view(-1, hkv, page_size, d)
        vp = pages[:, 1].view(-1, hkv, d, page_size)
        out = torch.zeros_like(q)
        qs = rows.query_start.tolist()
        for b, (slot, n) in enumerate(zip(rows.slots.tolist(), rows.lens.tolist())):
            s, e = qs[b], qs[b + 1]
            if n == 0 or s == e:
                continue
            units = table[slot, : -(-n // page_size)].long()
            k = _up(kp[units].transpose(1, 2).reshape(-1, hkv, d)[:n]).repeat_interleave(hq // hkv, dim=1)
            v = _up(vp[units].permute(0, 3, 1, 2).reshape(-1, hkv, d)[:n]).repeat_interleave(hq // hkv, dim=1)
            scores = torch.einsum("qhd,khd->hqk", _up(q[s:e]), k) * scale
            pos = torch.arange(n - (e - s), n, device=q.device)[:, None]
            key = torch.arange(n, device=q.device)[None, :]
            hidden = key > pos
            if window:
                hidden = hidden | (pos - key >= window)
            probs = scores.masked_fill(hidden, float("-inf")).softmax(-1)
            out[s:e] = torch.einsum("hqk,khd->qhd", probs, v).to(q.dtype)
        return out

    def argmax(self, logits):
        return logits.argmax(-1).to(torch.int32)

    def store_tokens(self, last_token, slots, tokens):
        last_token[slots.long()] = tokens

    def logprobs(self, logits, tokens, k):
        lp = (logits if logits.dtype == torch.float64 else logits.float()).log_softmax(-1)
        order = lp.argsort(dim=-1, descending=True, stable=True)[:, :k]
        return lp.gather(-1, tokens.long()[:, None])[:, 0], order.to(torch.int32), lp.gather(-1, order)

    def qkv_attention(self, qkv, heads, kv_heads, head_dim, q_weight, k_weight, eps, rope_table, positions, pages,
                      table, write_page, write_off, rows, page_size, scale, window, writes=True):
        q = self.qk_norm_rope_write(qkv, heads, kv_heads, head_dim, q_weight, k_weight, eps, rope_table, positions,
                                    pages if writes else None, write_page, write_off, page_size)
        return self.paged_attention(q, pages, table, rows, page_size, scale, window)

    def scatter_rows(self, dst, idx, src):
        dst[idx.long()] = src.view(idx.shape[0], dst.shape[1])

    def sample(self, logits, temperature, top_k, top_p, min_p, seeds, positions, slots=None):
        if slots is not None:
            at = slots.long()
            temperature, top_k, top_p, min_p, seeds = (t[at] for t in (temperature, top_k, top_p, min_p, seeds))
        positions = positions.long()
        m = 0xFFFFFFFF
        h = _mix32(seeds & m) ^ ((seeds >> 32) & m) ^ _mix32(positions & m)
        h = _mix32(h)
        u = (((h >> 8).float() + 0.5) * 2.0 ** -24).clamp(max=1 - 2.0 ** -24)
        out = logits.argmax(-1)
        for r in range(logits.shape[0]):
            temp = float(temperature[r])
            if temp == 0:
                continue
            x = logits[r].float() / torch.full_like(logits[r], temp, dtype=torch.float32)   # (a tensor: a true division)
            keep = torch.ones_like(x, dtype=torch.bool)
            order = x.argsort(descending=True, stable=True)
            if int(top_k[r]) > 0:
                keep[order[int(top_k[r]):]] = False
            q = torch.where(keep, x, float("-inf")).softmax(-1)
            if float(top_p[r]) < 1:
                sq = q[order]
                keep[order[sq.cumsum(-1) - sq > float(top_p[r])]] = False
            if float(min_p[r]) > 0:
                keep &= q >= float(min_p[r]) * q.max()
            q = torch.where(keep, q, 0.0)
            filtered = int(top_k[r]) > 0 or float(top_p[r]) < 1 or float(min_p[r]) > 0
            c = (q[order] if filtered else q).cumsum(-1)      # a filtered row is walked in the filters' sorted order
            idx = torch.searchsorted(c, (u[r] * c[-1]).reshape(1), right=True)[0].clamp(max=x.numel() - 1)
            out[r] = order[idx] if filtered else idx
        return out.to(torch.int32)
