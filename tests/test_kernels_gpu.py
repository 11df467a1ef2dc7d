"""Each HIP kernel alone against its plain twin (tests/plain/ops.py) on the same inputs, at sizes other than the tiny
models': the reference's own test shapes (plugins/tests/test_op_kernels.py:28-72, test_attention_kernels.py:20-66)
and awkward ones (widths that are no power of two, head sizes in steps of 16, page sizes from 1 up)."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from holon_amd.kernels.api import AttnRows
from tests import helpers as H
from tests.plain.ops import TorchKernels

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]
PLAIN = TorchKernels()


@pytest.fixture(scope="module")
def hip():
    from holon_amd.kernels import load_hip
    return load_hip()


def _randn(*shape, dtype, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(37, 4096), (37, 8, 128), (5, 100), (3, 7, 48), (1, 12288), (130, 16)])
def test_rmsnorm_and_add(hip, dtype, shape):
    x, r = _randn(*shape, dtype=dtype, seed=1), _randn(*shape, dtype=dtype, seed=2)
    w = (1 + 0.1 * torch.randn(shape[-1], generator=torch.Generator().manual_seed(3))).to(dtype).cuda()
    x0 = x.clone()
    for eps in (1e-6, 1e-2):
        got, want = hip.rmsnorm(x, w, eps), PLAIN.rmsnorm(x.double(), w.double(), eps)
        assert torch.equal(x, x0), "rmsnorm wrote its input"
        assert H.op_budget_usage(got, want, dtype, shape[-1]) <= 1
    x2, r_hip, r_ref = x.reshape(-1, shape[-1]), r.reshape(-1, shape[-1]).clone(), r.reshape(-1, shape[-1]).clone()
    got = hip.add_rmsnorm(x2, r_hip, w, 1e-6)
    want = PLAIN.add_rmsnorm(x2, r_ref, w, 1e-6)
    assert torch.equal(r_hip, r_ref), "the residual sum is one rounding of x + r"
    assert H.op_budget_usage(got, want.float(), dtype, shape[-1]) <= 1


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_silu_mul(hip, dtype):
    table = _randn(1000, 120, dtype=dtype, seed=4)
    ids = torch.tensor([0, 999, 5, 5, 123], dtype=torch.int32).cuda()
    assert torch.equal(hip.embedding(ids, table), table[ids.long()])
    table = _randn(333, 4096, dtype=dtype, seed=5)
    assert torch.equal(hip.embedding(ids[2:], table), table[ids[2:].long()])
    # tokens that the last step drew and left on the device: kept by slot, taken where a row says so
    last = torch.zeros(9, dtype=torch.int32).cuda()
    hip.store_tokens(last, torch.tensor([7, 2, 5], dtype=torch.int32).cuda(), torch.tensor([330, 11, 0], dtype=torch.int32).cuda())
    assert last.tolist() == [0, 0, 11, 0, 0, 0, 0, 330, 0]
    take = torch.tensor([-1, 7, -1, 2, 5], dtype=torch.int32).cuda()
    want = table[torch.tensor([0, 330, 5, 11, 0])]
    assert torch.equal(hip.embedding(ids, table, (take, last)), want)
    assert torch.equal(PLAIN.embedding(ids, table, (take, last)), want)
    for t, inter in ((17, 12288), (3, 100), (1, 7)):
        gu = _randn(t, 2 * inter, dtype=dtype, seed=6, scale=3.0)
        got, want = hip.silu_mul(gu), PLAIN.silu_mul(gu.double())
        assert H.op_budget_usage(got, want, dtype, 1) <= 1
    gu = torch.zeros(2, 8, dtype=dtype).cuda()
    gu[:, 4:] = 1
    assert torch.equal(hip.silu_mul(gu), torch.zeros(2, 4, dtype=dtype).cuda())


def test_silu_is_rounded_before_the_multiply(hip):
    """The reference multiplies silu(gate), rounded to the activation dtype, by up (std/holon_std/ffn/reference.py:
    7-12). Where rounding first and rounding only the product give different bfloat16 results, the kernels give the
    first: alone and fused into the gated product."""
    bf = torch.bfloat16
    g = torch.Generator().manual_seed(60)
    gate = (torch.randn(64, 4096, generator=g) * 2).to(bf)
    up = torch.randn(64, 4096, generator=g).to(bf)
    s64 = gate.double() * torch.sigmoid(gate.double())
    first = (s64.to(bf).float() * up.float()).to(bf)                   # rounded, then multiplied (one more rounding)
    late = (s64 * up.double()).to(bf)                                  # only the product rounded
    half_ulp = torch.exp2(torch.frexp(s64.to(bf).double())[1].double() - 1 - 8)      # of silu's bfloat16 neighbour
    edge = half_ulp - (s64 - s64.to(bf).double()).abs() < 1e-2 * half_ulp            # silu on a rounding edge: skip
    tell = (first != late) & ~edge
    assert tell.sum() > 10000                                          # the two orders differ in thousands of places
    got = hip.silu_mul(torch.cat((gate, up), dim=-1).cuda()).cpu()
    assert torch.equal(got[tell], first[tell])
    # the gated product: weights that copy x into gate and up make the product exact, the activation is what is left
    k = 256
    x = torch.cat((gate[:16, :128], up[:16, :128]), dim=-1).contiguous()                 # [16, 256]
    w = torch.zeros(256, k)
    w[:128, :128] = torch.eye(128)                                     # gate_i = x_i
    w[128:, 128:] = torch.eye(128)                                     # up_i = x_(128 + i)
    fused = hip.linear_silu_mul(x.cuda(), w.to(bf).cuda()).cpu()
    t = tell[:16, :128]
    assert t.sum() > 20 and torch.equal(fused[t], first[:16, :128][t])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize(("head_dim", "rotary_dim", "theta"), [(128, 128, 1e6), (256, 64, 1e7), (48, 48, 1e4), (16, 8, 1e4)])
def test_rope(hip, dtype, head_dim, rotary_dim, theta):
    from holon_amd.parts.positions import rope_table
    table = rope_table(8192, rotary_dim, theta).cuda()
    pos = torch.tensor([0, 1, 2, 15, 16, 1000, 4095, 8191] + list(range(100, 121)), dtype=torch.int32).cuda()
    q = _randn(29, 24, head_dim, dtype=dtype, seed=7)
    want = q.clone()
    PLAIN.rope(want, pos, table)
    got = q.clone()
    hip.rope(got, pos, table)
    assert H.op_budget_usage(got, want, dtype, 2) <= 1
    assert torch.equal(got[..., rotary_dim:], q[..., rotary_dim:])          # the rest passes through untouched
    assert torch.equal(got[0], q[0])                                         # position 0: identity
    # against the formula itself, in float64, half-split pairing
    inv = theta ** (-torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim)
    ang = pos.double().cpu()[:, None] * inv
    a, b = q[..., : rotary_dim // 2].double().cpu(), q[..., rotary_dim // 2: rotary_dim].double().cpu()
    ref = torch.cat((a * ang.cos()[:, None] - b * ang.sin()[:, None], b * ang.cos()[:, None] + a * ang.sin()[:, None]), -1)
    assert (got[..., :rotary_dim].double().cpu() - ref).abs().max() < (4e-3 if dtype == torch.float32 else 4e-2)


def _paged_case(rows, heads, kv_heads, head_dim, page, dtype, seed=0, max_seqs=8, scale_q=1.0):
    """rows: (tokens before this step, tokens this step). A shuffled block table with spare pages."""
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    assert len(rows) <= max_seqs
    slots = rng.permutation(max_seqs)[: len(rows)].astype(np.int32)
    max_pages = -(-max(s + n for s, n in rows) // page)
    units = max_seqs * max_pages + 7
    table = torch.from_numpy(rng.permutation(units)[: max_seqs * max_pages].reshape(max_seqs, max_pages).astype(np.int32))
    pages = torch.randn(units, 2, kv_heads, page * head_dim, generator=g).to(dtype).cuda()
    counts = np.array([n for _, n in rows])
    lens = np.array([s + n for s, n in rows])
    qstart = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    q = (torch.randn(int(counts.sum()), heads, head_dim, generator=g) * scale_q).to(dtype).cuda()
    dec, chk = np.flatnonzero(counts == 1), np.flatnonzero(counts > 1)
    i32 = lambda a: torch.as_tensor(np.asarray(a, dtype=np.int32)).cuda()
    attn = AttnRows(slots=i32(slots), lens=i32(lens), query_start=i32(qstart), decode_rows=i32(dec), chunk_rows=i32(chk),
                    n_decode=len(dec), n_chunk=len(chk), max_decode_len=int(lens[dec].max()) if len(dec) else 0,
                    max_chunk_query=int(counts[chk].max()) if len(chk) else 0,
                    max_chunk_len=int(lens[chk].max()) if len(chk) else 0, in_order=len(chk) == 0)
    return q, pages, table.cuda(), attn


GEOMETRIES = [(32, 8, 128), (16, 4, 256), (16, 8, 64), (6, 3, 32), (4, 1, 16), (5, 5, 48), (12, 2, 80),
              (10, 2, 64), (40, 2, 128), (7, 7, 64), (6, 1, 128), (48, 2, 64),   # groups of 5, 20, 1, 6 and 24 heads
              (40, 1, 128), (66, 1, 64),                                         # and of more heads than a tile has rows
              (64, 8, 128)]                                                      # groups of 8 at head_dim 128
ROWSETS = [[(0, 1), (0, 17), (5, 16), (31, 33), (0, 64), (100, 7), (16, 16)],
           [(0, 1), (15, 1), (16, 1), (99, 1), (999, 1), (4096, 1)],
           [(63, 1), (200, 2), (17, 1), (0, 130), (1, 1)]]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [16, 8, 64, 1, 5])
@pytest.mark.parametrize("geometry", GEOMETRIES)
def test_paged_attention(hip, dtype, page, geometry):
    heads, kv_heads, head_dim = geometry
    for seed, rows in enumerate(ROWSETS):
        if page < 8:
            rows = [(min(s, 300), n) for s, n in rows]
        q, pages, table, attn = _paged_case(rows, heads, kv_heads, head_dim, page, dtype, seed)
        scale = head_dim ** -0.5
        want = PLAIN.paged_attention(q.double(), pages.double(), table, attn, page, scale, 0)
        got = hip.paged_attention(q, pages, table, attn, page, scale, 0)
        again = hip.paged_attention(q, pages, table, attn, page, scale, 0)
        assert torch.equal(got, again), "two runs differ"
        # sums over head_dim (scores) and over the keys (softmax, values)
        assert H.op_budget_usage(got, want, dtype, head_dim + max(s + n for s, n in rows)) <= 1, (geometry, page, rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geometry", [(32, 8, 128), (6, 3, 32), (8, 2, 64), (32, 1, 64)])
def test_attention_never_touches_what_lies_beyond_a_row(hip, dtype, geometry):
    """Every cache slot that no row of the step holds a token in (the rest of a row's last page, pages of other
    requests, spare pages) is filled with NaN: a kernel that lets such a slot into a product, even with weight zero,
    gives NaN. Decode rows, short portions and portions long enough for the kernels that stage through LDS."""
    heads, kv_heads, head_dim = geometry
    page = 16
    for rows in ([(0, 1), (14, 1), (16, 1), (99, 1), (1000, 1)], [(0, 17), (5, 16), (31, 33), (100, 7)],
                 [(3, 700), (0, 530)]):
        q, pages, table, attn = _paged_case(rows, heads, kv_heads, head_dim, page, dtype, seed=len(rows))
        held = torch.zeros(pages.shape[0], page, dtype=torch.bool)
        for slot, (s, n) in zip(attn.slots.tolist(), rows):
            pos = torch.arange(s + n)
            held[table[slot, pos // page].cpu().long(), pos % page] = True
        kp, vp = pages[:, 0].view(-1, kv_heads, page, head_dim), pages[:, 1].view(-1, kv_heads, head_dim, page)
        free = (~held).cuda()
        kp.masked_fill_(free[:, None, :, None], float("nan"))
        vp.masked_fill_(free[:, None, None, :], float("nan"))
        want = PLAIN.paged_attention(q.double(), pages.double(), table, attn, page, head_dim ** -0.5, 0)
        got = hip.paged_attention(q, pages, table, attn, page, head_dim ** -0.5, 0)
        assert torch.isfinite(got.float()).all(), (geometry, rows)
        assert H.op_budget_usage(got, want, dtype, head_dim + max(s + n for s, n in rows)) <= 1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geometry", [(32, 8, 128), (8, 2, 64)])
def test_sixty_four_decode_rows(hip, dtype, geometry):
    """A decode step of 64 rows of unequal lengths (one key to 4,096, on and off page edges), with the launch shaped
    for a longer row than any has (as a graph's length bucket shapes it), and again with 11 of the rows empty rows on
    a table row of one page (as a graph's padding rows are)."""
    heads, kv_heads, head_dim = geometry
    rng = np.random.default_rng(5)
    longest = 4095 if head_dim == 64 else 1030
    rows = [(int(n), 1) for n in rng.integers(0, longest, 60)] + [(0, 1), (15, 1), (16, 1), (longest, 1)]
    q, pages, table, attn = _paged_case(rows, heads, kv_heads, head_dim, 16, dtype, seed=9, max_seqs=64)
    scale = head_dim ** -0.5
    want = PLAIN.paged_attention(q.double(), pages.double(), table, attn, 16, scale, 0)
    got = hip.paged_attention(q, pages, table, attn, 16, scale, 0)
    assert H.op_budget_usage(got, want, dtype, head_dim + longest) <= 1
    attn.max_decode_len = 1 << (longest).bit_length()                   # the bucket's length, not the rows'
    assert H.op_budget_usage(hip.paged_attention(q, pages, table, attn, 16, scale, 0), want, dtype,
                             head_dim + longest) <= 1
    lens = attn.lens.clone()
    lens[53:] = 0                                                       # rows that hold nothing give zeros
    attn.lens = lens
    got = hip.paged_attention(q, pages, table, attn, 16, scale, 0)
    assert not got[53:].any() and H.op_budget_usage(got[:53], want[:53], dtype, head_dim + longest) <= 1


@pytest.mark.parametrize("geometry", [(32, 8, 128), (64, 8, 128), (16, 8, 64), (16, 4, 256), (40, 1, 128), (7, 7, 64)])
@pytest.mark.parametrize("norm,rope", [(True, True), (False, True), (True, False), (False, False)])
def test_decode_attention_from_the_raw_projection(hip, geometry, norm, rope):
    """A step of decode rows alone, from the raw q/k/v projection: per-head norm, rotation and the cache write of each
    row's new token inside the attention kernel, against the three operations one after the other in float64. The
    cache afterwards holds what the separate write would have stored (every page compared: nothing else is touched),
    the rest of each row's last page holds NaN (the new key is read back, its neighbours never), rows differ in
    length (one key, page edges, thousands), one row holds nothing, and a window."""
    from holon_amd.parts.positions import rope_table
    heads, kv_heads, head_dim = geometry
    bf, page = torch.bfloat16, 16
    for seed, (starts, window) in enumerate((([0, 15, 16, 99, 1000, 4100, 31], 0), ([0, 5, 300, 2049], 64))):
        rows = [(s0, 1) for s0 in starts]
        _, pages, table, attn = _paged_case(rows, heads, kv_heads, head_dim, page, bf, seed=40 + seed)
        t = len(rows)
        held = torch.zeros(pages.shape[0], page, dtype=torch.bool)
        wp, wo = [], []
        for slot, (s0, _) in zip(attn.slots.tolist(), rows):
            pos = torch.arange(s0)                                    # the tokens before this step's
            held[table[slot, pos // page].cpu().long(), pos % page] = True
            wp.append(int(table[slot, s0 // page]))
            wo.append(s0 % page)
        kp, vp = pages[:, 0].view(-1, kv_heads, page, head_dim), pages[:, 1].view(-1, kv_heads, head_dim, page)
        free = (~held).cuda()
        kp.masked_fill_(free[:, None, :, None], float("nan"))
        vp.masked_fill_(free[:, None, None, :], float("nan"))
        i32 = lambda a: torch.tensor(a, dtype=torch.int32).cuda()
        wp, wo, pos = i32(wp), i32(wo), i32(starts)
        qkv = _randn(t, (heads + 2 * kv_heads) * head_dim, dtype=bf, seed=50 + seed)
        qw = (_randn(head_dim, dtype=bf, seed=51) + 1) if norm else None
        kw = (_randn(head_dim, dtype=bf, seed=52) + 1) if norm else None
        tab = rope_table(8192, head_dim, 1e4).cuda() if rope else None
        scale = head_dim ** -0.5
        pages_plain = pages.double()
        want = PLAIN.qkv_attention(qkv.double(), heads, kv_heads, head_dim, qw.double() if norm else None,
                                   kw.double() if norm else None, 1e-6, tab, pos, pages_plain, table, wp, wo, attn, page,
                                   scale, window)
        stored = pages.clone()
        ref_q = hip.qk_norm_rope_write(qkv, heads, kv_heads, head_dim, qw, kw, 1e-6, tab, pos, stored, wp, wo, page)
        unfused = hip.paged_attention(ref_q, stored, table, attn, page, scale, window)
        got = hip.qkv_attention(qkv, heads, kv_heads, head_dim, qw, kw, 1e-6, tab, pos, pages, table, wp, wo, attn, page,
                                scale, window)
        assert torch.isfinite(got.float()).all(), (geometry, starts)
        same = (pages == stored) | (pages.isnan() & stored.isnan())
        assert same.all(), "the cache differs from what the separate write stores"
        assert H.op_budget_usage(got, want, bf, head_dim + max(starts) + 1) <= 1, (geometry, starts, window)
        assert H.op_budget_usage(got, unfused.double(), bf, head_dim + max(starts) + 1) <= 1
        attn.lens = attn.lens.clone()
        attn.lens[1] = 0                                              # a row that holds nothing gives zeros, writes nothing
        before = pages.clone()
        got = hip.qkv_attention(qkv, heads, kv_heads, head_dim, qw, kw, 1e-6, tab, pos, pages, table, wp, wo, attn, page,
                                scale, window)
        assert not got[1].any() and ((pages == before) | before.isnan()).all()
        assert H.op_budget_usage(torch.cat((got[:1], got[2:])), torch.cat((want[:1], want[2:])), bf,
                                 head_dim + max(starts) + 1) <= 1


@pytest.mark.parametrize("geometry", [(32, 8, 128), (16, 8, 64), (8, 1, 128), (7, 7, 64), (6, 2, 64), (5, 1, 128),
                                      (24, 1, 64), (32, 1, 128), (40, 1, 128), (66, 1, 64), (80, 2, 64)])
def test_long_prompt_portions_two_tiles_a_wave(hip, geometry):
    """Portions long enough for the kernels that stage keys and values through LDS (tiles of 32 rows, one or two a
    wave, for groups of up to 32 heads; tiles of 16 rows, one or two a wave, for larger groups): one row of 4,500 tokens from position 0, two
    rows continuing earlier tokens (so the keys start before the queries), and a window. Groups of 1, 3, 5, 24, 32
    (tiles that hold one position or several, whole or in part), 40 and 66 heads."""
    heads, kv_heads, head_dim = geometry
    bf = torch.bfloat16
    for rows, window in (([(0, 4500)], 0), ([(300, 4200), (77, 2300)], 0), ([(1000, 4100)], 600)):
        q, pages, table, attn = _paged_case(rows, heads, kv_heads, head_dim, 16, bf, seed=len(rows) + window)
        scale = head_dim ** -0.5
        want = PLAIN.paged_attention(q.double(), pages.double(), table, attn, 16, scale, window)
        # one tile of 32 rows a wave, its stages copied into LDS by the memory pipeline (head_dim 128) or through
        # registers, and two tiles a wave (groups of up to 32 heads)
        for form, direct in ((0, 1), (0, 0), (2, 0)):
            before = hip.lib.holon_attention_prefill_form(form)
            copies = hip.lib.holon_attention_prefill_copies(direct)
            try:
                got = hip.paged_attention(q, pages, table, attn, 16, scale, window)
                again = hip.paged_attention(q, pages, table, attn, 16, scale, window)
            finally:
                hip.lib.holon_attention_prefill_form(before)
                hip.lib.holon_attention_prefill_copies(copies)
            # rows that see few keys are averages of few values and much larger than rows that see thousands: each
            # stretch of rows is held to the budget of its own size and of the keys it sees
            at = 0
            for start, n in rows:
                for lo, hi in ((0, 64), (64, 512), (512, n)):
                    part = slice(at + lo, at + min(hi, n))
                    span = head_dim + (min(window, start + hi) if window else start + min(hi, n))
                    assert H.op_budget_usage(got[part], want[part], bf, span) <= 1, (geometry, rows, window, lo, form, direct)
                at += n
            assert torch.equal(got, again)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 7, 16, 100])
def test_paged_attention_window(hip, dtype, window):
    for geometry, page in (((16, 8, 64), 16), ((6, 3, 32), 8), ((32, 8, 128), 16)):
        heads, kv_heads, head_dim = geometry
        q, pages, table, attn = _paged_case(ROWSETS[0] + [(300, 1), (98, 1)], heads, kv_heads, head_dim, page, dtype, 3,
                                            max_seqs=12)
        want = PLAIN.paged_attention(q.double(), pages.double(), table, attn, page, head_dim ** -0.5, window)
        got = hip.paged_attention(q, pages, table, attn, page, head_dim ** -0.5, window)
        assert H.op_budget_usage(got, want, dtype, head_dim + window) <= 1, (geometry, window)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_key(hip, dtype):
    """One key among thousands carries the weight: its query is aligned with it and scaled up. A kernel that skips or
    misplaces a page, a tile edge or the last key shows here."""
    heads, kv_heads, head_dim, page = 8, 2, 64, 16
    for n, target in ((4097, 0), (4097, 4096), (1000, 511), (1000, 512), (2049, 1023), (130, 64), (130, 63)):
        q, pages, table, attn = _paged_case([(n - 1, 1)], heads, kv_heads, head_dim, page, dtype, seed=n + target)
        slot = int(attn.slots[0])
        unit, off = int(table[slot, target // page]), target % page
        kp = pages[:, 0].view(-1, kv_heads, page, head_dim)
        for h in range(heads):
            q[0, h] = kp[unit, h // (heads // kv_heads), off].float().mul(4.0).to(dtype)
        want = PLAIN.paged_attention(q.double(), pages.double(), table, attn, page, head_dim ** -0.5, 0)
        vp = pages[:, 1].view(-1, kv_heads, head_dim, page)
        assert (want[0, 0] - vp[unit, 0, :, off].double()).abs().max() < 0.05       # the test itself singles the key out
        got = hip.paged_attention(q, pages, table, attn, page, head_dim ** -0.5, 0)
        assert H.op_budget_usage(got, want, dtype, head_dim + n) <= 1, (n, target)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geometry", [(32, 8, 128, 16), (6, 3, 32, 8), (4, 1, 16, 16), (5, 5, 48, 4), (16, 4, 256, 32)])
def test_fused_norm_rope_write_is_the_three_ops(hip, dtype, geometry):
    from holon_amd.parts.positions import rope_table
    heads, kv_heads, head_dim, page = geometry
    table = rope_table(4096, head_dim, 1e6).cuda()
    rng = np.random.default_rng(0)
    qw, kw = _randn(head_dim, dtype=dtype, seed=9), _randn(head_dim, dtype=dtype, seed=10)
    # few tokens at scattered places; many tokens at consecutive places (whole pages and ragged ends); many scattered
    layouts = [(45, rng.permutation(40 * page)[:45]), (200, np.arange(200) + 3 * page), (130, np.arange(130) + 5),
               (100, rng.permutation(40 * page)[:100]), (300, np.arange(300) + 2 * page + 3),
               (260, rng.permutation(80 * page)[:260])]      # from 256 tokens on a block walks all heads of its token
    for t, where in layouts:
        units = int(where.max()) // page + 2
        qkv = _randn(t, (heads + 2 * kv_heads) * head_dim, dtype=dtype, seed=8)
        pos = torch.as_tensor(rng.integers(0, 4096, t).astype(np.int32)).cuda()
        wp, wo = (torch.as_tensor((where // page).astype(np.int32)).cuda(), torch.as_tensor((where % page).astype(np.int32)).cuda())
        for use_norm, use_rope in ((True, True), (False, True), (True, False), (False, False)):
            pages_h = torch.zeros(units, 2, kv_heads, page * head_dim, dtype=dtype).cuda()
            pages_p = pages_h.clone()
            args = (heads, kv_heads, head_dim, qw if use_norm else None, kw if use_norm else None, 1e-6,
                    table if use_rope else None, pos)
            got = hip.qk_norm_rope_write(qkv, *args, pages_h, wp, wo, page)
            want = PLAIN.qk_norm_rope_write(qkv, *args, pages_p, wp, wo, page)
            assert H.op_budget_usage(got, want, dtype, head_dim) <= 1
            assert H.op_budget_usage(pages_h, pages_p, dtype, head_dim) <= 1
            assert torch.equal(pages_h == 0, pages_p == 0), "a cache entry outside the written ones changed"
            assert torch.equal(pages_h[:, 1], pages_p[:, 1]), "values are copied bit for bit"
    t, where = layouts[0]
    units = 42
    qkv = _randn(t, (heads + 2 * kv_heads) * head_dim, dtype=dtype, seed=8)
    pos = torch.as_tensor(rng.integers(0, 4096, t).astype(np.int32)).cuda()
    wp, wo = (torch.as_tensor((where // page).astype(np.int32)).cuda(), torch.as_tensor((where % page).astype(np.int32)).cuda())
    # queries only (a run that reads another run's cache)
    got = hip.qk_norm_rope_write(qkv, heads, kv_heads, head_dim, qw, kw, 1e-6, table, pos, None, None, None, page)
    want = PLAIN.qk_norm_rope_write(qkv, heads, kv_heads, head_dim, qw, kw, 1e-6, table, pos, None, None, None, page)
    assert H.op_budget_usage(got, want, dtype, head_dim) <= 1
    # the unfused write
    k, v = _randn(t, kv_heads, head_dim, dtype=dtype, seed=11), _randn(t, kv_heads, head_dim, dtype=dtype, seed=12)
    pages_h, pages_p = torch.zeros_like(pages_h), torch.zeros_like(pages_p)
    hip.kv_write(k, v, pages_h, wp, wo, page)
    PLAIN.kv_write(k, v, pages_p, wp, wo, page)
    assert torch.equal(pages_h, pages_p)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("geometry", [(32, 8, 128, 16), (16, 4, 256, 32), (6, 2, 64, 16)])
def test_values_of_many_tokens_are_written_16_tokens_a_block(hip, dtype, geometry):
    """From 256 tokens on, the norm + rotation + write kernel's launch has blocks behind the tokens' own that write the
    values, 16 tokens of one kv head each, transposed through LDS: whole groups inside one page, groups that straddle
    pages or start off a multiple of 8, a ragged last group, scattered places. Values bit for bit, nothing else touched,
    queries and keys within the budget."""
    from holon_amd.parts.positions import rope_table
    heads, kv_heads, head_dim, page = geometry
    table = rope_table(4096, head_dim, 1e6).cuda()
    rng = np.random.default_rng(1)
    qw, kw = _randn(head_dim, dtype=dtype, seed=9), _randn(head_dim, dtype=dtype, seed=10)
    for t, where in ((530, np.arange(530) + page + 5), (1040, np.arange(1040) + 2 * page),
                     (257, rng.permutation(60 * page)[:257]), (300, np.arange(300) * 2)):
        units = int(where.max()) // page + 2
        qkv = _randn(t, (heads + 2 * kv_heads) * head_dim, dtype=dtype, seed=t)
        pos = torch.as_tensor(rng.integers(0, 4096, t).astype(np.int32)).cuda()
        wp, wo = (torch.as_tensor((where // page).astype(np.int32)).cuda(), torch.as_tensor((where % page).astype(np.int32)).cuda())
        pages_h = torch.zeros(units, 2, kv_heads, page * head_dim, dtype=dtype).cuda()
        pages_p = pages_h.clone()
        got = hip.qk_norm_rope_write(qkv, heads, kv_heads, head_dim, qw, kw, 1e-6, table, pos, pages_h, wp, wo, page)
        want = PLAIN.qk_norm_rope_write(qkv, heads, kv_heads, head_dim, qw, kw, 1e-6, table, pos, pages_p, wp, wo, page)
        assert torch.equal(pages_h[:, 1], pages_p[:, 1]), (geometry, t, "values are copied bit for bit")
        assert torch.equal(pages_h == 0, pages_p == 0), "a cache entry outside the written ones changed"
        assert H.op_budget_usage(got, want, dtype, head_dim) <= 1
        assert H.op_budget_usage(pages_h[:, 0], pages_p[:, 0], dtype, head_dim) <= 1


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear(hip, dtype):
    # up to 16 rows the few-row kernel runs (bfloat16, K >= 256), above that the vendor library's product
    for t, k, n in ((1, 4096, 6144), (8, 4096, 1000), (17, 100, 333), (64, 12288, 4096), (300, 120, 1000), (2, 96, 384),
                    (1, 4096, 4096), (16, 12288, 4096), (3, 4096, 24576), (9, 512, 208), (33, 1024, 4096),
                    (48, 4096, 512), (5, 12288, 151936 // 8), (65, 4096, 512),
                    (1, 8192, 5120), (12, 4096, 8192),                   # 320 and 512 tiles: two tiles a block
                    (5, 512, 80_000), (12, 512, 80_000), (16, 256, 65_568)):  # a vocabulary's worth: two from ten rows up
        x, w = _randn(t, k, dtype=dtype, seed=13), _randn(n, k, dtype=dtype, seed=14, scale=0.05)
        want = x.double() @ w.double().T
        got = hip.linear(x, w)
        assert got.dtype == dtype and H.op_budget_usage(got, want, dtype, k) <= 1, (t, k, n)
        got32 = hip.linear(x, w, torch.float32)
        assert got32.dtype == torch.float32 and H.op_budget_usage(got32, want, dtype, k) <= 1
        assert torch.equal(got32, got.float())         # one rule for every number of rows: the product, then the cast
        tiled = hip.tile_weight(w)
        assert (tiled is None) == (dtype != torch.bfloat16 or n % 16 != 0 or k % 32 != 0 or k < 256)
        if tiled is not None:                          # the tile layout is a permutation: the same bits come out
            assert torch.equal(hip.linear(x, w, None, tiled), got)
            assert torch.equal(hip.linear(x, w, torch.float32, tiled), got32)
    # exact arithmetic: activations in {-1, 0, 1} and weights in {-1, 0, 1} / 8 make every partial sum exact, so any
    # order of summation gives the same bits (plugins/tests/test_attention_kv_quant.py:244-261)
    g = torch.Generator().manual_seed(15)
    x = torch.randint(-1, 2, (5, 512), generator=g).to(dtype).cuda()
    for n in (200, 208, 4096):
        w = (torch.randint(-1, 2, (n, 512), generator=g).float() / 8).to(dtype).cuda()
        assert torch.equal(hip.linear(x, w).float(), x.float() @ w.float().T)
    # a row's result does not depend on the rows beside it, beyond rounding
    x = _randn(64, 4096, dtype=dtype, seed=16)
    w = _randn(512, 4096, dtype=dtype, seed=17, scale=0.02)
    assert H.op_budget_usage(hip.linear(x[:1].contiguous(), w), hip.linear(x, w)[:1].float(), dtype, 4096) <= 1


def test_product_for_17_to_64_rows_over_many_tiles(hip):
    """Steps of 17 to 64 rows over weights with at least 1,024 tiles of 16 rows read the tiled copy through the kernel
    that shares the rows through LDS: plain, with a float32 result (the bfloat16 one cast up), and gated; against
    float64 and against the same product over the rows as they are. A row's result is bit for bit the same whatever
    rows lie beside it, and fewer tiles, other row counts and other K stay where they were."""
    bf = torch.bfloat16
    for m, k, n in ((17, 256, 16384), (64, 4096, 24576), (33, 1024, 16512), (48, 512, 65536), (64, 768, 65664), (20, 256, 131072)):
        x, w = _randn(m, k, dtype=bf, seed=80), _randn(n, k, dtype=bf, seed=81, scale=0.05)
        tiled = hip.tile_weight(w)
        timed = hip.configured("timed")
        assert timed.serves_rows(m, w, tiled)                                          # outside an engine's start: untimed, ours
        assert timed.plan.how == {f"rows:{n}x{k}:{32 if m <= 32 else 64}": "untimed"}
        timed = hip.configured("timed")
        timed.plan.resolving = True                                                    # as while an engine starts: timed once
        timed.serves_rows(m, w, tiled)
        bucket = 32 if m <= 32 else 64
        assert timed.plan.how == {f"rows:{n}x{k}:{bucket}": "timed"} and timed.plan.seconds > 0
        assert timed.plan.report()[f"rows:{n}x{k}:{32 if m <= 32 else 64}"] in ("rows", "vendor")
        assert not hip.configured("vendor").serves_rows(m, w, tiled)
        assert hip.serves_rows(m, w, tiled) and not hip.serves_rows(16, w, tiled) and not hip.serves_rows(65, w, tiled)
        want = x.double() @ w.double().T
        got = hip.linear(x, w, None, tiled)
        assert got.dtype == bf and H.op_budget_usage(got, want, bf, k) <= 1, (m, k, n)
        assert H.op_budget_usage(got, hip.linear(x, w).double(), bf, k) <= 1          # the vendor library's, over the rows
        assert torch.equal(hip.linear(x, w, torch.float32, tiled), got.float())
        fewer = hip.linear(x[3:21].contiguous(), w, None, tiled)                       # 18 rows, other places
        assert torch.equal(fewer, got[3:21]) if m >= 21 else True
    for m, k, inter in ((64, 4096, 12288), (17, 256, 8192), (40, 1024, 8320), (33, 512, 16384), (64, 768, 16512)):   # the last two: eight waves a block
        x, w = _randn(m, k, dtype=bf, seed=82), _randn(2 * inter, k, dtype=bf, seed=83, scale=0.05)
        tiled = hip.tile_weight(w)
        assert hip.serves_rows(m, w, tiled, gated=True)
        pinned = hip.configured("own", {f"glu:{2 * inter}x{k}:{32 if m <= 32 else 64}": "vendor"})
        assert not pinned.serves_rows(m, w, tiled, gated=True) and pinned.plan.how.popitem()[1] == "pinned"
        exact = PLAIN.silu_mul(PLAIN.linear(x.double(), w.double()))
        got = hip.linear_silu_mul(x, w, tiled)
        assert got is not None and got.shape == (m, inter) and H.op_budget_usage(got, exact, bf, k) <= 1, (m, k, inter)
        two = hip.silu_mul(hip.linear(x, w))                                           # the same roundings in two kernels
        assert (got != two).float().mean() < 0.02
    w = _randn(4096, 4096, dtype=bf, seed=84)
    tiled = hip.tile_weight(w)
    assert not hip.serves_rows(32, w, tiled) and not hip.serves_rows(32, w, None)      # 256 tiles: the vendor library's
    w = _randn(16384, 384, dtype=bf, seed=85)
    assert not hip.serves_rows(32, w, hip.tile_weight(w))                              # K no multiple of 256


def test_product_in_shares_of_k_for_narrow_weights(hip):
    """Steps of 17 to 64 rows over narrow weights (a few hundred tiles: output and down projections) may have K split
    over blocks: float32 sums of every share, which the residual add + norm kernel (or `sum_parts`) adds up in order.
    Every share against float64 over its columns; the sum, rounded once, against the whole product; the norm that
    reads the parts against the norm over their rounded sum (the residual rows bit for bit), in both of its kernels
    (rows of 1,024 values and more, and narrower ones); a row's result whatever rows lie beside it; and the timed
    choice."""
    from holon_amd.kernels.hip import KernelError
    bf = torch.bfloat16
    for m, k, n in ((64, 4096, 4096), (17, 12288, 4096), (33, 1024, 5120), (48, 25600, 5120), (40, 512, 320), (64, 256, 64),
                    (65, 4096, 4096), (100, 12288, 4096), (128, 1024, 5120), (90, 256, 64), (113, 2560, 1024)):
        x, w = _randn(m, k, dtype=bf, seed=90), _randn(n, k, dtype=bf, seed=91, scale=0.05)
        tiled = hip.tile_weight(w)
        splits = hip.lib.holon_gemm_rows_splits(m, n, k)
        assert splits in (2, 4, 8) and k % (128 * splits) == 0, (m, k, n, splits)
        parts = hip._rows_parts(x, w, tiled, splits)
        assert parts.shape == (splits, m, n) and parts.dtype == torch.float32
        share = k // splits
        for s in range(splits):
            want = x[:, s * share:(s + 1) * share].double() @ w[:, s * share:(s + 1) * share].double().T
            assert H.op_budget_usage(parts[s], want, torch.float32, share) <= 1, (m, k, n, s)
        total = hip.sum_parts(parts)
        in_order = parts[0].clone()
        for s in range(1, splits):
            in_order += parts[s]
        assert torch.equal(total, in_order.to(bf))
        assert H.op_budget_usage(total, x.double() @ w.double().T, bf, k) <= 1
        assert H.op_budget_usage(total, hip.linear(x, w).double(), bf, k) <= 1           # the vendor library's product
        fewer = hip._rows_parts(x[3:21].contiguous(), w, tiled, splits) if m >= 21 else None
        assert fewer is None or torch.equal(fewer, parts[:, 3:21])
        weight, eps = _randn(n, dtype=bf, seed=92) + 1, 1e-5
        res_a, res_b = _randn(m, n, dtype=bf, seed=93), _randn(m, n, dtype=bf, seed=93)
        normed_a = hip.add_rmsnorm(parts, res_a, weight, eps)                             # reads the parts itself
        normed_b = hip.add_rmsnorm(total, res_b, weight, eps)
        assert torch.equal(res_a, res_b), (m, k, n)                                       # the same sums, bit for bit
        assert H.op_budget_usage(normed_a, normed_b.double(), bf, 1) <= 1, (m, k, n)      # (squares summed in another order)
        plain_res = _randn(m, n, dtype=bf, seed=93)
        plain_normed = PLAIN.add_rmsnorm(parts, plain_res, weight, eps)                   # the twin takes parts as well
        assert torch.equal(plain_res, res_a) and H.op_budget_usage(normed_a, plain_normed.double(), bf, 1) <= 1
    x, w = _randn(32, 4096, dtype=bf, seed=94), _randn(4096, 4096, dtype=bf, seed=95, scale=0.05)
    tiled = hip.tile_weight(w)
    timed = hip.configured("timed")
    timed.plan.resolving = True
    got = timed.linear_parts(x, w, tiled)                                                 # timed once, then kept
    assert timed.plan.report()["parts:4096x4096:32"] in ("parts", "vendor")
    assert (got is None) == (timed.plan.report()["parts:4096x4096:32"] == "vendor")
    assert hip.configured("vendor").linear_parts(x, w, tiled) is None
    assert hip.configured("vendor", {"parts:4096x4096:32": "parts"}).linear_parts(x, w, tiled).shape == (8, 32, 4096)
    assert hip.linear_parts(x, w, tiled).shape == (8, 32, 4096)
    assert hip.linear_parts(x[:16].contiguous(), w, tiled) is None and hip.linear_parts(x, w, None) is None
    assert hip.linear_parts(_randn(129, 4096, dtype=bf, seed=99), w, tiled) is None            # beyond 128 rows, K < 2 N
    assert hip.linear_parts(_randn(32, 4096, dtype=torch.float32, seed=96), w.float(), tiled) is None          # float32 rows: not this path
    w = _randn(4096, 4224, dtype=bf, seed=97)                                             # K = 33 x 128: no equal shares
    assert hip.linear_parts(_randn(32, 4224, dtype=bf, seed=98), w, hip.tile_weight(w)) is None
    with pytest.raises(KernelError):
        hip._rows_parts(x, w[:, :4096].contiguous(), tiled, 3)                            # 4096 / 128 = 32 chunks, not by 3
    with pytest.raises(KernelError):
        hip._rows_parts(x.cpu(), w[:, :4096].contiguous(), tiled, 8)
    with pytest.raises(KernelError):
        hip.add_rmsnorm(torch.zeros(8, 32, 4000, device="cuda"), _randn(32, 4096, dtype=bf), _randn(4096, dtype=bf), 1e-5)


def test_choices_are_timed_over_the_same_shaped_weights_of_other_layers(hip):
    """Every weight that got a tiled copy is known by shape (weakly: a weight that is gone is forgotten), and a timing
    calls its candidates on them in turn, the given one first, up to 16 of them or a gigabyte: one weight called over
    and over would be read from the memory-side cache, which a step's weights never are."""
    import gc
    bf = torch.bfloat16
    ws = [_randn(2048, 512, dtype=bf, seed=300 + i) for i in range(5)]
    ts = [hip.tile_weight(w) for w in ws]
    pairs = hip._alike(ws[2], ts[2])
    assert pairs[0][0] is ws[2] and pairs[0][1] is ts[2] and len(pairs) == 5
    assert {id(w) for w, _ in pairs} == {id(w) for w in ws} and all(t is ts[[id(x) for x in ws].index(id(w))] for w, t in pairs)
    assert all(t is None for _, t in hip._alike(ws[0], None)) and len(hip._alike(ws[0], None)) == 5
    assert len(hip._alike(ws[0], ts[0], most=3)) == 3 and len(hip._alike(ws[0], ts[0], most_bytes=2 * 2048 * 512 * 2)) == 2
    folded = hip.tile_weight(ws[1], _randn(512, dtype=bf, seed=310))      # a new copy of a known weight replaces the old
    assert [t for w, t in hip._alike(ws[0], ts[0]) if w is ws[1]] == [folded]
    del pairs, ws[3:], ts[3:]
    gc.collect()
    assert len(hip._alike(ws[0], ts[0])) == 3
    calls = hip._in_turn(hip._alike(ws[0], ts[0]), lambda w, t: (w, t))
    assert len(calls) == 9 and calls[0]()[0] is ws[0] and calls[3]()[0] is ws[0]          # three rounds over three weights
    assert {id(c()[0]) for c in calls[:3]} == {id(w) for w in ws}
    x = _randn(32, 512, dtype=bf, seed=311)
    ms = hip._graph_time(hip._in_turn(hip._alike(ws[0], ts[0]), lambda w, t: torch.matmul(x, w.t())))
    assert 0 < ms < 5


def test_vendor_product_forms_for_steps_of_17_to_64_rows(hip):
    """Steps of 17 to 64 bfloat16 rows (over deep weights also prompt portions of up to 1,024 rows) take the vendor
    library's product in the fastest of three forms, timed once per weight shape and row bucket: each is the product
    rounded once, whichever is kept, and the float32 output is the bfloat16 one cast up."""
    bf = torch.bfloat16
    for m, k, n in ((32, 25600, 5120), (24, 4096, 6144), (64, 1024, 512), (300, 25600, 5120), (1000, 8192, 512)):
        x, w = _randn(m, k, dtype=bf, seed=70), _randn(n, k, dtype=bf, seed=71, scale=0.02)
        want = x.double() @ w.double().T
        key = f"vendor:{n}x{k}:{32 if m <= 32 else 1 << (m - 1).bit_length()}"
        timed = hip.configured("timed")
        timed.plan.resolving = True
        got = timed.linear(x, w)
        assert timed.plan.report()[key] in ("bf16", "f32", "f32x2")       # timed and kept
        for form in ("bf16", "f32", "f32x2"):
            y = hip.configured("own", {key: form}).linear(x, w)
            assert y.dtype == bf and H.op_budget_usage(y, want, bf, k) <= 1, (m, k, n, form)
            assert torch.equal(hip.configured("own", {key: form}).linear(x, w, torch.float32), y.float())
        assert torch.equal(hip.linear(x, w), hip.configured("vendor").linear(x, w))          # both: the plain form
        assert H.op_budget_usage(got, want, bf, k) <= 1
    timed = hip.configured("timed")
    timed.plan.resolving = True
    timed.linear(_randn(300, 4096, dtype=bf, seed=72), _randn(512, 4096, dtype=bf, seed=73))    # a shallow weight, and
    timed.linear(_randn(1025, 8192, dtype=bf, seed=74), _randn(512, 8192, dtype=bf, seed=75))   # more rows: no choice
    assert timed.plan.report() == {}


def test_float32_product_is_true_32_bit_and_its_order_is_fixed(hip):
    """The 32-bit path's own product: close to the float64 product as only true float32 arithmetic is (a
    reduced-precision matrix mode would be a thousand times off), at odd sizes (K no multiple of 4 or 32, N and M
    off the tile edges), and bit for bit independent of the rows beside a row and of the row's place in the batch."""
    f32 = torch.float32
    for m, k, n in ((1, 64, 256), (5, 30, 97), (33, 33, 65), (70, 200, 120), (64, 4096, 64), (130, 72, 1000),
                    (3, 12288, 4096), (257, 4096, 192)):
        x, w = _randn(m, k, dtype=f32, seed=40), _randn(n, k, dtype=f32, seed=41, scale=0.05)
        got, want = hip.linear(x, w), x.double() @ w.double().T
        assert got.dtype == f32 and H.op_budget_usage(got, want, f32, k) <= 1, (m, k, n)
        rel = ((got.double() - want).abs().max() / want.abs().max()).item()
        assert rel < 2e-6 * max(1.0, (k / 64) ** 0.5), (m, k, n, rel)            # bfloat16 or tf32 operands give 1e-3
        rows = torch.tensor(sorted({0, m // 2, m - 1}))
        alone = hip.linear(x[rows.cuda()].contiguous(), w)                        # other company, other places
        assert torch.equal(alone, got[rows.cuda()]), (m, k, n)
        if m > 1:
            shifted = hip.linear(torch.cat((x[-1:], x)).contiguous(), w)          # every row one place further down
            assert torch.equal(shifted[1:], got), (m, k, n)
    x = torch.randint(-1, 2, (7, 100), generator=torch.Generator().manual_seed(42)).float().cuda()
    w = (torch.randint(-1, 2, (50, 100), generator=torch.Generator().manual_seed(43)).float() / 8).cuda()
    assert torch.equal(hip.linear(x, w), x @ w.T)                                 # exact arithmetic: any order, same bits


def test_norm_folded_into_the_product(hip):
    """The norm's weight folded into the tiled copy, the rows scaled inside the product from statistics another kernel
    left: against norm then product in float64, within the budget of the two operations; the statistics from the
    residual add's kernel, from the embedding and from `row_sumsq` are the rows' sums of squares; the gated form too."""
    bf = torch.bfloat16
    for m, k, n in ((1, 4096, 6144), (8, 4096, 1024), (16, 512, 208), (5, 12288, 4096), (3, 4096, 24576)):
        h = _randn(m, k, dtype=bf, seed=50, scale=2.0)
        g = (1 + 0.2 * torch.randn(k, generator=torch.Generator().manual_seed(51))).to(bf).cuda()
        w = _randn(n, k, dtype=bf, seed=52, scale=0.05)
        eps = 1e-5
        exact = PLAIN.rmsnorm(h.double(), g.double(), eps) @ w.double().T
        composed = hip.linear(hip.rmsnorm(h, g, eps), w)
        folded = hip.tile_weight(w, g)
        assert hip.folds_norm(m, w, folded)
        stats = hip.row_sumsq(h)
        assert stats.shape == (1, 16)
        assert torch.allclose(stats[0, :m], h.float().pow(2).sum(-1), rtol=1e-5)
        got = hip.linear(h, w, None, folded, row_scale=(stats, eps))
        assert got.dtype == bf and H.op_budget_usage(got, exact, bf, 2 * k) <= 1, (m, k, n)
        assert H.rel_rms(got, exact) <= 1.5 * H.rel_rms(composed, exact) + 1e-4          # no worse than norm, then product
        split = torch.zeros(7, 16, device="cuda")                                      # the same sums in seven parts
        split[:, :m] = (h.float().pow(2).sum(-1) / 7)[None, :]
        assert H.op_budget_usage(hip.linear(h, w, None, folded, row_scale=(split, eps)), exact, bf, 2 * k) <= 1
        got32 = hip.linear(h, w, torch.float32, folded, row_scale=(stats, eps))
        assert torch.equal(got32, got.float())
        if n % 32 == 0 and k % 128 == 0:                                               # the gated form
            want = PLAIN.silu_mul((PLAIN.rmsnorm(h.double(), g.double(), eps) @ w.double().T))
            glu = hip.linear_silu_mul(h, w, folded, row_scale=(stats, eps))
            assert glu.shape == (m, n // 2) and H.op_budget_usage(glu, want, bf, 2 * k) <= 1, (m, k, n)
    # the residual add leaves the statistics of the rows it wrote, one part per 16 columns
    for m, k, n in ((8, 4096, 4096), (1, 12288, 4096), (16, 512, 208), (7, 8192, 5120), (16, 1024, 6144)):
        x, r = _randn(m, k, dtype=bf, seed=53), _randn(m, n, dtype=bf, seed=54)
        w = _randn(n, k, dtype=bf, seed=55, scale=0.05)
        tiled = hip.tile_weight(w)
        want = r.clone()
        assert hip.linear_add(x, w, tiled, want) is True
        stats = hip.linear_add(x, w, tiled, r, want_stats=True)
        assert torch.equal(r, want) and stats.shape == (n // 16, 16)
        assert torch.allclose(stats.sum(0)[:m], r.float().pow(2).sum(-1), rtol=1e-5) and not stats[:, m:].any()
    table = _randn(500, 4096, dtype=bf, seed=56)
    ids = torch.tensor([3, 499, 0, 3, 77], dtype=torch.int32).cuda()
    rows, stats = hip.embedding(ids, table, None, want_stats=True)
    assert torch.equal(rows, table[ids.long()]) and torch.allclose(stats[0, :5], rows.float().pow(2).sum(-1), rtol=1e-5)
    rows, stats = hip.embedding(torch.zeros(40, dtype=torch.int32).cuda(), table, None, want_stats=True)
    assert stats is None                                                               # more rows than a folded norm serves


def test_fused_gate_up_is_the_two_kernels(hip, monkeypatch):
    for m, k, inter in ((1, 4096, 12288), (8, 4096, 12288), (16, 512, 208), (3, 1024, 1024), (5, 256, 48)):
        x = _randn(m, k, dtype=torch.bfloat16, seed=30)
        w = _randn(2 * inter, k, dtype=torch.bfloat16, seed=31, scale=0.05)
        exact = PLAIN.silu_mul(PLAIN.linear(x.double(), w.double()))
        want = hip.silu_mul(hip.linear(x, w))
        assert H.op_budget_usage(want, exact, torch.bfloat16, k) <= 1
        both = []
        for tiled in (None, hip.tile_weight(w)):
            got = hip.linear_silu_mul(x, w, tiled)
            assert got is not None and H.op_budget_usage(got, exact, torch.bfloat16, k) <= 1, (m, k, inter)
            # the same roundings as the two kernels; the sums over K may be split differently
            assert (got != want).float().mean() < 0.02
            both.append(got)
        assert torch.equal(both[0], both[1])           # the tile layout is a permutation of the same reads
    assert hip.linear_silu_mul(_randn(40, 256, dtype=torch.bfloat16), _randn(64, 256, dtype=torch.bfloat16)) is None
    assert hip.linear_silu_mul(_randn(4, 256, dtype=torch.float32), _randn(64, 256, dtype=torch.float32)) is None


def test_product_added_into_the_residual(hip):
    """`linear_add` = the few-row product, rounded, added into the residual, rounded: the bits of the two kernels one
    after the other, since the product is the same kernel's."""
    from holon_amd.kernels.hip import KernelError
    bf = torch.bfloat16
    for m, k, n in ((1, 4096, 6144), (8, 4096, 4096), (16, 12288, 4096), (3, 256, 48), (5, 1024, 208), (2, 4096, 24576)):
        x, w = _randn(m, k, dtype=bf, seed=50), _randn(n, k, dtype=bf, seed=51, scale=0.05)
        tiled = hip.tile_weight(w)
        res = _randn(m, n, dtype=bf, seed=53, scale=2.0)
        exact = res.double() + (x.double() @ w.double().T).to(bf).double()
        want = (res.float() + hip.linear(x, w, None, tiled).float()).to(bf)
        mine = res.clone()
        assert hip.linear_add(x, w, tiled, mine) is True
        assert torch.equal(mine, want), (m, k, n)
        assert H.op_budget_usage(mine, exact, bf, k) <= 1, (m, k, n)
    # what is not served is left to the kernels one after the other, and nothing is touched
    w = _randn(512, 4096, dtype=bf, seed=55, scale=0.02)
    tiled = hip.tile_weight(w)
    res = _randn(17, 512, dtype=bf)
    keep = res.clone()
    assert hip.linear_add(_randn(17, 4096, dtype=bf), w, tiled, res) is False and torch.equal(res, keep)
    assert hip.linear_add(_randn(4, 4096, dtype=bf), w, None, res[:4].contiguous()) is False
    f32 = torch.float32
    assert hip.linear_add(_randn(4, 256, dtype=f32), _randn(64, 256, dtype=f32), None, _randn(4, 64, dtype=f32)) is False
    with pytest.raises(KernelError):
        hip.linear_add(_randn(16, 4096, dtype=bf), w, tiled, _randn(16, 500, dtype=bf))


def test_logprobs_kernel(hip):
    g = torch.Generator().manual_seed(40)
    for rows, vocab, k in ((3, 151_936, 20), (5, 97, 5), (2, 40, 0), (1, 33, 32)):
        logits = (torch.randn(rows, vocab, generator=g) * 3).cuda()
        logits[0, 7] = logits[0, 3] = logits[0].max() + 1                 # a tie at the top: the lower id first
        tokens = torch.randint(0, vocab, (rows,), generator=g).to(torch.int32).cuda()
        lp, ids, top = hip.logprobs(logits, tokens, k)
        want_lp, want_ids, want_top = PLAIN.logprobs(logits.double(), tokens, k)
        assert ids.tolist() == want_ids.tolist()
        torch.testing.assert_close(lp.double(), want_lp.double(), rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(top.double(), want_top.double(), rtol=1e-5, atol=1e-5)


def test_argmax_and_sampling(hip):
    from tests.plain import sampling as S
    g = torch.Generator().manual_seed(20)
    logits = (torch.randn(9, 151_936, generator=g) * 3).cuda()
    logits[3, 777] = logits[3, 90_000] = 50.0                     # a tie: the first index wins
    assert hip.argmax(logits).tolist() == logits.argmax(-1).tolist()
    assert int(hip.argmax(logits)[3]) == 777
    # wide rows are searched in pieces of 4,096: ties across pieces, rows of -inf and of NaN, widths that are no
    # multiple of 4 (or of the piece), a best value at a piece's first and last place
    for rows, vocab in ((3, 16_385), (70, 20_001), (2, 16_384), (5, 9_001)):
        x = torch.randn(rows, vocab, generator=g).cuda()
        x[0, 4095] = x[0, 4096] = x[0, vocab - 1] = 9.0
        x[1, :] = float("-inf")
        x[1, 5000:5003] = float("nan")
        if rows > 2:
            x[2, :] = float("nan")
        if rows > 3:
            x[3, :4100] = float("nan")
            x[3, 4100:] = float("-inf")
            x[4, 8192] = 30.0
        got = hip.argmax(x).tolist()
        want = torch.where(x.isnan(), torch.full_like(x, float("-inf")), x).cpu().argmax(-1).tolist()
        if rows > 2:
            want[2] = 0                        # nothing to choose from: the first token
        if rows > 3:
            want[3] = 4100                     # the first value that is a number
        assert got == want, (rows, vocab, got[:5], want[:5])
        assert got[0] == 4095 and got[1] == 0
    # the law, by counting: one row of 40 logits drawn 100,000 times at consecutive positions
    v, n = 40, 100_000
    row = torch.randn(v, generator=torch.Generator().manual_seed(0)) * 2
    row[7] = row[11]                                              # equal logits straddling a top-k edge
    cases = [(0.7, 0, 1.0, 0.0), (1.0, 5, 1.0, 0.0), (1.0, 0, 0.8, 0.0), (1.3, 0, 1.0, 0.1), (0.9, 12, 0.9, 0.02),
             (1.0, 1, 1.0, 0.0), (1.0, 0, 1e-6, 0.0)]
    for temp, top_k, top_p, min_p in cases:
        f = lambda x, dt: torch.full((n,), x, dtype=dt).cuda()
        tokens = hip.sample(row.expand(n, v).contiguous().cuda(), f(temp, torch.float32), f(top_k, torch.int32),
                            f(top_p, torch.float32), f(min_p, torch.float32), f(1234, torch.int64),
                            torch.arange(n, dtype=torch.int64).cuda())
        freq = torch.bincount(tokens.long().cpu(), minlength=v).double() / n
        p = S.probs(row, temp, top_k, top_p, min_p)
        assert (freq[p == 0] == 0).all(), (temp, top_k, top_p, min_p, "a filtered token was drawn")
        assert 0.5 * (freq - p).abs().sum() < 0.02, (temp, top_k, top_p, min_p)
    # a draw depends on (seed, position) only: not on the row's place in the batch or on the other rows
    logits = torch.randn(6, v, generator=torch.Generator().manual_seed(1)).cuda()
    one = lambda x, dt, r: torch.full((r,), x, dtype=dt).cuda()
    seeds = torch.tensor([100, 101, 102, 103, 100, 101], dtype=torch.int64).cuda()
    pos = torch.tensor([5, 5, 5, 5, 9, 9], dtype=torch.int64).cuda()
    together = hip.sample(logits, one(1.0, torch.float32, 6), one(0, torch.int32, 6), one(1.0, torch.float32, 6),
                          one(0.0, torch.float32, 6), seeds, pos)
    alone = hip.sample(logits[[1, 5]].contiguous(), one(1.0, torch.float32, 2), one(0, torch.int32, 2),
                       one(1.0, torch.float32, 2), one(0.0, torch.float32, 2), seeds[[1, 5]].contiguous(),
                       pos[[1, 5]].contiguous())
    assert together[[1, 5]].tolist() == alone.tolist()
    # the draw is the inverse CDF at the hashed uniform, in vocabulary order, at the full vocabulary
    big = (torch.randn(4, 151_936, generator=g) * 3).cuda()
    toks = hip.sample(big, one(1.0, torch.float32, 4), one(0, torch.int32, 4), one(1.0, torch.float32, 4),
                      one(0.0, torch.float32, 4), one(77, torch.int64, 4), torch.arange(4, dtype=torch.int64).cuda())
    for r in range(4):
        cdf = big[r].double().softmax(-1).cumsum(0).cpu()
        u, t = S.uniform(77, r), int(toks[r])
        assert (cdf[t - 1] if t else 0.0) - 1e-5 <= u < cdf[t] + 1e-5
    # temperature 0 rows take the argmax beside sampled rows
    mixed_t = torch.tensor([0.0, 1.0, 0.0, 1.0], dtype=torch.float32).cuda()
    toks = hip.sample(big, mixed_t, one(0, torch.int32, 4), one(1.0, torch.float32, 4), one(0.0, torch.float32, 4),
                      one(5, torch.int64, 4), torch.arange(4, dtype=torch.int64).cuda())
    assert toks[[0, 2]].tolist() == big[[0, 2]].argmax(-1).tolist()


def test_temperature_divides_the_logits_as_the_reference_does(hip):
    """logit / t and logit * (1 / t) differ in the last place for some values, and with them which of two nearly equal
    logits count as equal at a filter's edge (equal ones go by index). Two such pairs, found by search: one that is a
    tie only under division, one only under multiplication; top-k = 1 then keeps the token the division says
    (std/holon_std/sampling/sampler.py:137 divides)."""
    from tests.plain import sampling as S
    g = torch.Generator().manual_seed(3)
    t = torch.tensor(1.7, dtype=torch.float32)
    inv = torch.tensor(1.0, dtype=torch.float32) / t
    a = torch.rand(200_000, generator=g) * 8 + 4
    b = torch.nextafter(a, torch.tensor(0.0))                        # the float just below
    tie_div, tie_mul = (a / t) == (b / t), (a * inv) == (b * inv)
    only_div, only_mul = int((tie_div & ~tie_mul).nonzero()[0]), int((tie_mul & ~tie_div).nonzero()[0])
    for at, first in ((only_div, 3), (only_mul, 9)):                 # b sits at index 3, a (larger) at index 9
        row = torch.full((1000,), -30.0)
        row[3], row[9] = b[at], a[at]
        f = lambda x, dt: torch.full((16,), x, dtype=dt).cuda()
        got = hip.sample(row.expand(16, 1000).contiguous().cuda(), f(1.7, torch.float32), f(1, torch.int32),
                         f(1.0, torch.float32), f(0.0, torch.float32), f(5, torch.int64), torch.arange(16).cuda())
        assert got.tolist() == [first] * 16, (at, got.tolist())      # a tie: the lower index; no tie: the larger value
        assert int(S.probs(row, 1.7, 1).argmax()) == first and int(PLAIN.sample(
            row[None].cuda(), f(1.7, torch.float32)[:1], f(1, torch.int32)[:1], f(1.0, torch.float32)[:1],
            f(0.0, torch.float32)[:1], f(5, torch.int64)[:1], torch.arange(1).cuda())[0]) == first


def _at_uniform(law, order, token, u, slack=2e-5):
    """Whether `token` is where the inverse CDF of `law`, walked in `order` (None: as it lies), puts the uniform `u`."""
    walk = law if order is None else law[order]
    at = token if order is None else int((order == token).nonzero()[0])
    cdf = walk.cumsum(0)
    return (cdf[at - 1] if at else 0.0) - slack <= u < cdf[at] + slack


def test_sampling_filters_at_the_full_vocabulary(hip):
    """Every draw is the plain sampler's (float64 law, inverse CDF at the hashed uniform, a filtered row walked in
    sorted order) at 151,936 tokens: peaked
    rows whose kept set is small (the fast form: candidates collected and sorted), flat rows and a large k (the
    general form), ties at the edge of top-k and of top-p, k = 1, a tiny top-p."""
    from tests.plain import sampling as S
    v = 151_936
    g = torch.Generator().manual_seed(60)
    peaked = torch.randn(v, generator=g) * 3
    flat = torch.randn(v, generator=g) * 0.3
    tied = peaked.clone()
    order = peaked.argsort(descending=True)
    tied[order[45:55]] = peaked[order[49]]                       # ten equal values around the 50th place
    tied[order[2:5]] = peaked[order[3]]
    plateau = peaked.clone()
    plateau[order[:6000]] = peaked[order[0]]
    coarse = (torch.randn(v, generator=g) * 0.4).round() / 4     # five values, tens of thousands of each; +0 and -0 are one
    assert (coarse == 0).sum() > 50_000 and ((coarse == 0) & coarse.signbit()).sum() > 10_000
    cases = [(peaked, 0.8, 50, 1.0, 0.0), (peaked, 0.8, 0, 0.9, 0.0), (peaked, 1.0, 50, 0.9, 0.02), (peaked, 0.7, 0, 1.0, 0.05),
             (peaked, 1.0, 1, 1.0, 0.0), (peaked, 1.0, 0, 1e-6, 0.0), (peaked, 1.2, 2048, 0.99, 0.0), (peaked, 1.0, 5000, 1.0, 0.0),
             (flat, 1.0, 0, 0.9, 0.0), (flat, 1.0, 300, 0.5, 0.0), (tied, 1.0, 50, 1.0, 0.0), (tied, 1.0, 48, 0.95, 0.0),
             (tied, 0.9, 4, 1.0, 0.0), (tied, 1.0, 0, 0.5, 0.0), (peaked, 1.0, 0, 1.0, 0.0),
             (peaked * 8, 1.0, 50, 1.0, 0.0), (peaked * 8, 1.0, 0, 0.999, 0.0), (peaked * 8, 0.5, 20, 0.9, 0.0),
             (peaked * 40, 1.0, 50, 0.9, 0.0),      # sharp rows: the 50th token lies tens, or hundreds, below the first
             (flat, 1.0, 0, 1.0, 0.2), (peaked, 1.0, 200_000, 1.0, 0.0),   # kept sets too long to collect: min-p alone, all
             (plateau, 1.0, 0, 0.5, 0.0), (plateau, 1.0, 0, 1.0, 0.5), (plateau, 1.0, 7000, 1.0, 0.0),   # 6,000 equal values
             (flat, 0.8, 50, 0.9, 0.0), (flat, 0.8, 20, 0.95, 0.05), (peaked, 1.0, 5000, 0.9, 0.01),    # cuts found by halving
             (plateau, 1.0, 3000, 1.0, 0.0), (peaked * 40, 1.0, 5000, 1.0, 0.0),   # a cut inside equal values; k beyond what weighs
             (coarse, 0.3, 0, 0.9, 0.0), (coarse, 1.0, 0, 0.5, 0.0), (coarse, 1.0, 70_000, 1.0, 0.0), (coarse, 0.3, 0, 1.0, 0.15)]
    n = 48
    for at, (row, temp, top_k, top_p, min_p) in enumerate(cases):
        f = lambda x, dt: torch.full((n,), x, dtype=dt).cuda()
        seed = 900 + at
        tokens = hip.sample(row.expand(n, v).contiguous().cuda(), f(temp, torch.float32), f(top_k, torch.int32),
                            f(top_p, torch.float32), f(min_p, torch.float32), f(seed, torch.int64),
                            torch.arange(n, dtype=torch.int64).cuda()).tolist()
        law = S.probs(row, temp, top_k, top_p, min_p)
        order = S.drawing_order(row, temp, top_k, top_p, min_p)
        assert (order is None) == (top_k == 0 and top_p == 1.0 and min_p == 0.0)
        assert all(law[t] > 0 for t in tokens), (at, "a filtered token was drawn")
        for pos, t in enumerate(tokens):                   # the inverse CDF at the hashed uniform, to float32 rounding
            assert _at_uniform(law, order, t, S.uniform(seed, pos)), (at, pos, t)
        if row is not flat and row is not coarse and top_k < v:   # few tokens carry the mass: a draw then sits well inside its token's share
            want = [S.draw(law, S.uniform(seed, pos), order) for pos in range(n)]
            assert sum(a != b for a, b in zip(tokens, want)) <= 1, (at, temp, top_k, top_p, min_p)
    # rows of one batch with different settings do not disturb each other
    rows = torch.stack([peaked, flat, tied, peaked]).cuda()
    t = torch.tensor([0.8, 1.0, 0.0, 1.0], dtype=torch.float32).cuda()
    k = torch.tensor([50, 0, 0, 1], dtype=torch.int32).cuda()
    p = torch.tensor([1.0, 0.9, 1.0, 1.0], dtype=torch.float32).cuda()
    m = torch.zeros(4, dtype=torch.float32).cuda()
    got = hip.sample(rows, t, k, p, m, torch.full((4,), 5, dtype=torch.int64).cuda(), torch.arange(4).cuda()).tolist()
    assert got[0] == S.draw(S.probs(peaked, 0.8, 50), S.uniform(5, 0), S.drawing_order(peaked, 0.8, 50))
    assert _at_uniform(S.probs(flat, 1.0, 0, 0.9), S.drawing_order(flat, 1.0, 0, 0.9), got[1], S.uniform(5, 1))
    assert got[2] == int(tied.argmax()) and got[3] == int(peaked.argmax())


def test_sampling_under_random_settings(hip):
    """Many rows with settings drawn at random, a row each its own: vocabularies of 1,000 to 33,000, flat to sharp
    rows, every filter alone and together, k beyond what is collected. A drawn token lies in the plain law's kept set
    and at the hashed uniform of the plain CDF."""
    import random
    from tests.plain import sampling as S
    rng = random.Random(7)
    for vocab in (1000, 5003, 33000):
        g = torch.Generator().manual_seed(vocab)
        rows = 48
        scales = [rng.choice([0.3, 1.0, 3.0, 10.0]) for _ in range(rows)]
        logits = torch.randn(rows, vocab, generator=g) * torch.tensor(scales)[:, None]
        temp = [rng.choice([0.3, 0.7, 1.0, 1.5]) for _ in range(rows)]
        top_k = [rng.choice([0, 0, 1, 5, 50, 500, 3000, 5000]) for _ in range(rows)]
        top_p = [rng.choice([1.0, 1.0, 0.99, 0.9, 0.5, 0.1]) for _ in range(rows)]
        min_p = [rng.choice([0.0, 0.0, 0.01, 0.2]) for _ in range(rows)]
        t = lambda v, dt: torch.tensor(v, dtype=dt).cuda()
        got = hip.sample(logits.cuda(), t(temp, torch.float32), t(top_k, torch.int32), t(top_p, torch.float32),
                         t(min_p, torch.float32), t([11] * rows, torch.int64), torch.arange(rows).cuda()).tolist()
        for r in range(rows):
            law = S.probs(logits[r], temp[r], top_k[r], top_p[r], min_p[r])
            case = (vocab, r, scales[r], temp[r], top_k[r], top_p[r], min_p[r])
            assert law[got[r]] > 0, case
            order = S.drawing_order(logits[r], temp[r], top_k[r], top_p[r], min_p[r])
            assert _at_uniform(law, order, got[r], S.uniform(11, r)), case


def test_product_in_shares_of_k_for_prompt_portions(hip):
    """129 to 1,024 rows over a weight whose K is at least twice its N (a feed-forward's second product): blocks of
    128 rows against 256 columns, K in shares. Every share against float64 over its columns, for every number of
    shares the kernel takes; the sum against the whole product and the vendor library's; rows whatever rows lie beside
    them (another number of row blocks); the norm that reads the parts; what the kernel does not take."""
    from holon_amd.kernels.hip import KernelError
    bf = torch.bfloat16
    for m, k, n in ((129, 512, 256), (200, 1024, 512), (512, 12288, 4096), (1000, 2048, 512), (1024, 1536, 768),
                    (300, 25600, 5120), (640, 9728, 2560)):
        x, w = _randn(m, k, dtype=bf, seed=190), _randn(n, k, dtype=bf, seed=191, scale=0.05)
        tiled = hip.tile_weight(w)
        auto = hip.lib.holon_gemm_tiles_splits(m, n, k)
        assert auto in (0, 1, 2, 4, 8) and (auto > 0 or n <= 512), (m, k, n, auto)    # (0: too few blocks to be worth taking)
        whole = x.double() @ w.double().T
        for splits in (1, 2, 4, 8):
            if not hip.lib.holon_gemm_tiles_parts_supported(m, n, k, splits):
                assert splits != auto
                continue
            parts = hip._rows_parts(x, w, tiled, splits)
            assert parts.shape == (splits, m, n) and parts.dtype == torch.float32
            share = k // splits
            for s in range(splits):
                want = x[:, s * share:(s + 1) * share].double() @ w[:, s * share:(s + 1) * share].double().T
                assert H.op_budget_usage(parts[s], want, torch.float32, share) <= 1, (m, k, n, splits, s)
            total = hip.sum_parts(parts)
            assert H.op_budget_usage(total, whole, bf, k) <= 1
            if splits == (auto or 2):
                assert H.op_budget_usage(total, hip.linear(x, w).double(), bf, k) <= 1       # the vendor library's product
                some = hip._rows_parts(x[5:200].contiguous(), w, tiled, splits) if m >= 200 else None
                assert some is None or torch.equal(some, parts[:, 5:200])
                weight, eps = _randn(n, dtype=bf, seed=192) + 1, 1e-5
                res_a, res_b = _randn(m, n, dtype=bf, seed=193), _randn(m, n, dtype=bf, seed=193)
                normed_a = hip.add_rmsnorm(parts, res_a, weight, eps)
                normed_b = hip.add_rmsnorm(total, res_b, weight, eps)
                assert torch.equal(res_a, res_b), (m, k, n)
                assert H.op_budget_usage(normed_a, normed_b.double(), bf, 1) <= 1, (m, k, n)
    x, w = _randn(512, 12288, dtype=bf, seed=194), _randn(4096, 12288, dtype=bf, seed=195, scale=0.05)
    tiled = hip.tile_weight(w)
    assert hip.linear_parts(x, w, tiled).shape == (8, 512, 4096)                            # mode `own`
    assert hip.configured("vendor").linear_parts(x, w, tiled) is None
    assert hip.configured("vendor", {"parts:4096x12288:512": "parts"}).linear_parts(x, w, tiled).shape == (8, 512, 4096)
    assert hip.linear_parts(_randn(1025, 12288, dtype=bf, seed=196), w, tiled) is None     # beyond 1,024 rows
    wide = _randn(8192, 4096, dtype=bf, seed=197)
    assert hip.linear_parts(_randn(512, 4096, dtype=bf, seed=198), wide, hip.tile_weight(wide)) is None   # K < 2 N
    with pytest.raises(KernelError):
        hip._rows_parts(x, w, tiled, 5)
    with pytest.raises(KernelError):
        hip._rows_parts(x, w[:4000].contiguous(), hip.tile_weight(w[:4000].contiguous()), 4)   # 4,000 columns: no whole blocks


def test_kernels_refuse_what_they_do_not_serve(hip):
    from holon_amd.kernels.hip import KernelError
    with pytest.raises(KernelError):
        hip.rmsnorm(torch.zeros(4, 8), torch.ones(8), 1e-6)                         # a CPU tensor: no fallback
    with pytest.raises(KernelError):
        hip.rmsnorm(torch.zeros(4, 8, dtype=torch.float16).cuda(), torch.ones(8, dtype=torch.float16).cuda(), 1e-6)
    q, pages, table, attn = _paged_case([(0, 4)], 2, 1, 12, 16, torch.float32)     # head_dim 12: not a multiple of 8
    with pytest.raises(KernelError, match="head_dim"):
        hip.paged_attention(q, pages, table, attn, 16, 1.0, 0)
    # the products run on raw pointers: an operand off the GPU, or a tiled copy that is not this weight's, is refused
    bf = torch.bfloat16
    w, other = _randn(512, 1024, dtype=bf, seed=1), _randn(256, 1024, dtype=bf, seed=2)
    tiled = hip.tile_weight(w)
    big = _randn(16384, 256, dtype=bf, seed=3)
    for rows, weight in ((4, w), (32, big)):
        with pytest.raises(KernelError):
            hip.linear(torch.zeros(rows, weight.shape[1], dtype=bf), weight, None, hip.tile_weight(weight))   # rows on the CPU
    with pytest.raises(KernelError, match="tiled"):
        hip.linear(_randn(32, 256, dtype=bf), big, None, hip.tile_weight(_randn(8192, 256, dtype=bf)))
    with pytest.raises(KernelError, match="tiled"):
        hip.linear(_randn(4, 1024, dtype=bf), w, None, hip.tile_weight(other))
    with pytest.raises(KernelError, match="tiled"):
        hip.linear_add(_randn(4, 1024, dtype=bf), w, hip.tile_weight(other), _randn(4, 512, dtype=bf))
    with pytest.raises(KernelError):
        hip.linear_add(_randn(4, 1024, dtype=bf), w, tiled, torch.zeros(4, 512, dtype=bf))   # residual on the CPU
