"""Pins for the plain implementation: each check is chosen so that a plausible misreading of the reference's
formulas (a wrong sign or pairing in the rotation, a norm in the wrong place, a wrong mask or scale) fails it."""
from __future__ import annotations

import math

import torch

from tests.plain import qwen3 as plain
from tests.plain import sampling as plain_sampling


def test_rms_norm_is_the_library_routine():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(7, 3, 48, generator=g), torch.randn(48, generator=g)
    for eps in (1e-6, 1e-2):
        want = torch.nn.functional.rms_norm(x, (48,), w, eps)
        torch.testing.assert_close(plain.rms_norm(x, w, eps), want, rtol=1e-6, atol=1e-6)
    # weight 1, eps 0, unit-rms input: identity
    unit = x / x.pow(2).mean(-1, keepdim=True).sqrt()
    torch.testing.assert_close(plain.rms_norm(unit, torch.ones(48), 0.0), unit, rtol=1e-6, atol=1e-6)
    # eps sits inside the square root, beside the mean (not added to the root, not multiplied by dim)
    tiny = torch.full((1, 48), 1e-3)
    want = 1e-3 / math.sqrt(1e-6 + 1e-2)
    torch.testing.assert_close(plain.rms_norm(tiny, torch.ones(48), 1e-2), torch.full((1, 48), want))


def test_rms_norm_rounds_once_in_low_precision():
    g = torch.Generator().manual_seed(1)
    x, w = torch.randn(5, 64, generator=g).bfloat16(), (1 + 0.1 * torch.randn(64, generator=g)).bfloat16()
    exact = plain.rms_norm(x.float(), w.float(), 1e-6)
    assert torch.equal(plain.rms_norm(x, w, 1e-6), exact.bfloat16())


def test_rope_is_a_complex_rotation_of_the_half_split_pairs():
    g = torch.Generator().manual_seed(2)
    d, theta = 32, 1e4
    x = torch.randn(9, 3, d, generator=g)
    pos = torch.tensor([0, 1, 2, 15, 16, 100, 1000, 4095, 8191])
    got = plain.rope_neox(x, pos, theta)
    inv_freq = theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    ang = pos.double()[:, None] * inv_freq[None, :]
    z = torch.complex(x[..., : d // 2].double(), x[..., d // 2:].double()) * torch.polar(torch.ones_like(ang), ang)[:, None]
    want = torch.cat((z.real, z.imag), -1)
    # float32 angles at position 8191 carry about 8191 * 2^-24 of error
    torch.testing.assert_close(got.double(), want, rtol=0, atol=3e-3)
    torch.testing.assert_close(got[:5].double(), want[:5], rtol=0, atol=1e-5)
    assert torch.equal(got[0], x[0])                                       # position 0: identity
    torch.testing.assert_close(got.norm(dim=-1), x.norm(dim=-1), rtol=1e-5, atol=1e-5)


def test_rope_scores_depend_on_distances_only():
    g = torch.Generator().manual_seed(3)
    q, k = torch.randn(1, 2, 64, generator=g), torch.randn(1, 2, 64, generator=g)
    def score(pq, pk):
        a = plain.rope_neox(q, torch.tensor([pq]), 1e6)
        b = plain.rope_neox(k, torch.tensor([pk]), 1e6)
        return (a * b).sum(-1)
    torch.testing.assert_close(score(7, 3), score(107, 103), rtol=1e-4, atol=1e-4)
    assert not torch.allclose(score(7, 3), score(3, 7), rtol=1e-3, atol=1e-3)     # the sign of the angle matters


def test_attention_is_sdpa_with_grouped_heads():
    g = torch.Generator().manual_seed(4)
    for hq, hkv, d, t in ((6, 3, 32, 19), (4, 1, 16, 33), (5, 5, 48, 8)):
        q, k, v = (torch.randn(t, h, d, generator=g) for h in (hq, hkv, hkv))
        want = torch.nn.functional.scaled_dot_product_attention(
            q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], is_causal=True,
            enable_gqa=True)[0].transpose(0, 1)
        torch.testing.assert_close(plain.causal_attention(q, k, v), want, rtol=1e-5, atol=1e-5)


def test_attention_special_cases():
    g = torch.Generator().manual_seed(5)
    q, k, v = torch.randn(6, 4, 16, generator=g), torch.randn(6, 2, 16, generator=g), torch.randn(6, 2, 16, generator=g)
    out = plain.causal_attention(q, k, v)
    # the first token sees one key: its output is v[0] of its kv head (head j reads kv head j // group)
    torch.testing.assert_close(out[0], v[0].repeat_interleave(2, dim=0))
    # equal scores: the mean of the visible values
    flat = plain.causal_attention(torch.zeros_like(q), k, v)
    want = (v.cumsum(0) / torch.arange(1, 7)[:, None, None]).repeat_interleave(2, dim=1)
    torch.testing.assert_close(flat, want, rtol=1e-5, atol=1e-5)
    # a window of 2: each query sees itself and the key before it
    win = plain.causal_attention(torch.zeros_like(q), k, v, window=2)
    want = torch.cat((v[:1], (v[1:] + v[:-1]) / 2)).repeat_interleave(2, dim=1)
    torch.testing.assert_close(win, want, rtol=1e-5, atol=1e-5)


def test_attention_scale_is_one_over_sqrt_head_dim():
    q = torch.zeros(2, 1, 16); k = torch.zeros(2, 1, 16); v = torch.zeros(2, 1, 16)
    q[1, 0, 0], k[1, 0, 0], v[1, 0, 0] = 4.0, 4.0, 1.0           # score 16 / sqrt(16) = 4 against 0
    out = plain.causal_attention(q, k, v)
    torch.testing.assert_close(out[1, 0, 0], torch.tensor(math.exp(4) / (1 + math.exp(4))))


def test_swiglu_parts():
    g = torch.Generator().manual_seed(6)
    gate, up = torch.randn(5, 40, generator=g), torch.randn(5, 40, generator=g)
    torch.testing.assert_close(plain.silu_mul(gate, up), torch.nn.functional.silu(gate) * up)
    assert torch.equal(plain.silu_mul(torch.zeros(3), torch.ones(3)), torch.zeros(3))
    x, wg, wu, wd = (torch.randn(*s, generator=g) for s in ((4, 24), (40, 24), (40, 24), (24, 40)))
    want = (torch.nn.functional.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    torch.testing.assert_close(plain.swiglu(x, wg, wu, wd), want, rtol=1e-5, atol=1e-5)


def _tiny(seed=0, tied=False):
    cfg = {"num_hidden_layers": 2, "hidden_size": 48, "num_attention_heads": 6, "num_key_value_heads": 2,
           "head_dim": 16, "intermediate_size": 80, "vocab_size": 101, "rope_theta": 1e4, "rms_norm_eps": 1e-5,
           "tie_word_embeddings": tied}
    g = torch.Generator().manual_seed(seed)
    def lin(o, i): return torch.randn(o, i, generator=g) * 0.2
    def nrm(n): return 1 + 0.3 * torch.randn(n, generator=g)
    w = {"model.embed_tokens.weight": lin(101, 48), "model.norm.weight": nrm(48)}
    if not tied:
        w["lm_head.weight"] = lin(101, 48)
    for i in range(2):
        p = f"model.layers.{i}."
        w |= {p + "input_layernorm.weight": nrm(48), p + "post_attention_layernorm.weight": nrm(48),
              p + "self_attn.q_proj.weight": lin(96, 48), p + "self_attn.k_proj.weight": lin(32, 48),
              p + "self_attn.v_proj.weight": lin(32, 48), p + "self_attn.o_proj.weight": lin(48, 96),
              p + "self_attn.q_norm.weight": nrm(16), p + "self_attn.k_norm.weight": nrm(16),
              p + "mlp.gate_proj.weight": lin(80, 48), p + "mlp.up_proj.weight": lin(80, 48),
              p + "mlp.down_proj.weight": lin(48, 80)}
    return cfg, w


def test_attention_layer_sees_distances_only():
    """q/k norm comes before the rotation: with norm weights that differ inside a rotated pair, norming after the
    rotation would make the output depend on absolute positions."""
    cfg, w = _tiny()
    x = torch.randn(11, 48, generator=torch.Generator().manual_seed(7))
    a = plain.attention_layer(x, torch.arange(11), w, "model.layers.0.self_attn.", cfg)
    b = plain.attention_layer(x, torch.arange(11) + 300, w, "model.layers.0.self_attn.", cfg)
    torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-4)

    def wrong_order(x, positions):
        t = x.shape[0]
        p = "model.layers.0.self_attn."
        q = plain.linear(x, w[p + "q_proj.weight"]).view(t, 6, 16)
        k = plain.linear(x, w[p + "k_proj.weight"]).view(t, 2, 16)
        v = plain.linear(x, w[p + "v_proj.weight"]).view(t, 2, 16)
        q = plain.rms_norm(plain.rope_neox(q, positions, 1e4), w[p + "q_norm.weight"], 1e-5)
        k = plain.rms_norm(plain.rope_neox(k, positions, 1e4), w[p + "k_norm.weight"], 1e-5)
        return plain.causal_attention(q, k, v)
    assert not torch.allclose(wrong_order(x, torch.arange(11)), wrong_order(x, torch.arange(11) + 300),
                              rtol=1e-3, atol=1e-3)


def test_model_is_causal_and_uses_the_tied_head():
    cfg, w = _tiny(tied=True)
    ids = [5, 17, 3, 99, 0, 42, 7, 7, 23]
    full = plain.logits_of(ids, w, cfg)
    assert full.dtype == torch.float32 and full.shape == (9, 101)
    torch.testing.assert_close(plain.logits_of(ids[:4], w, cfg), full[:4], rtol=1e-5, atol=1e-5)
    # the head of a tied model is the embedding: the final hidden state of token t scores E rows
    h = full @ torch.linalg.pinv(w["model.embed_tokens.weight"]).T
    torch.testing.assert_close(h @ w["model.embed_tokens.weight"].T, full, rtol=1e-3, atol=1e-3)


def test_one_layer_by_hand():
    """The block's wiring against a direct transcription with library routines: residual around attention, then
    around the MLP, each reading a normed copy."""
    cfg, w = _tiny(seed=3)
    cfg = dict(cfg, num_hidden_layers=1)
    ids = [1, 2, 3, 4, 5, 6]
    F = torch.nn.functional
    h = w["model.embed_tokens.weight"][torch.tensor(ids)]
    p = "model.layers.0."
    a = F.rms_norm(h, (48,), w[p + "input_layernorm.weight"], 1e-5)
    q = F.rms_norm((a @ w[p + "self_attn.q_proj.weight"].T).view(6, 6, 16), (16,), w[p + "self_attn.q_norm.weight"], 1e-5)
    k = F.rms_norm((a @ w[p + "self_attn.k_proj.weight"].T).view(6, 2, 16), (16,), w[p + "self_attn.k_norm.weight"], 1e-5)
    v = (a @ w[p + "self_attn.v_proj.weight"].T).view(6, 2, 16)
    inv = 1e4 ** (-torch.arange(0, 16, 2, dtype=torch.float32) / 16)
    rot = torch.polar(torch.ones(6, 8), torch.arange(6, dtype=torch.float32)[:, None] * inv)[:, None]
    def rope(x):
        z = torch.complex(x[..., :8], x[..., 8:]) * rot
        return torch.cat((z.real, z.imag), -1)
    o = F.scaled_dot_product_attention(rope(q).transpose(0, 1)[None], rope(k).transpose(0, 1)[None],
                                       v.transpose(0, 1)[None], is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    h = h + o.reshape(6, 96) @ w[p + "self_attn.o_proj.weight"].T
    x = F.rms_norm(h, (48,), w[p + "post_attention_layernorm.weight"], 1e-5)
    h = h + (F.silu(x @ w[p + "mlp.gate_proj.weight"].T) * (x @ w[p + "mlp.up_proj.weight"].T)) @ w[p + "mlp.down_proj.weight"].T
    want = F.rms_norm(h, (48,), w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T
    torch.testing.assert_close(plain.logits_of(ids, w, cfg), want, rtol=1e-4, atol=1e-4)


def test_sampling_oracle():
    assert plain_sampling.mix32(0) == 0
    assert plain_sampling.mix32(1) != 1 and 0 <= plain_sampling.mix32(123456789) < 2 ** 32
    assert plain_sampling.sequence_seed(2 ** 63 + 5, 0) == 5                  # core/holon/api/batch.py:71-73
    assert plain_sampling.sequence_seed(5, 1) != plain_sampling.sequence_seed(5, 2)
    us = [plain_sampling.uniform(11, p) for p in range(2000)]
    assert 0 < min(us) and max(us) < 1 and abs(sum(us) / 2000 - 0.5) < 0.03
    logits = torch.tensor([2.0, 1.0, 0.0, -1.0, 3.0])
    assert plain_sampling.probs(logits, 0.0).tolist() == [0, 0, 0, 0, 1]
    torch.testing.assert_close(plain_sampling.probs(logits, 0.5), (logits.double() / 0.5).softmax(-1))
    k2 = plain_sampling.probs(logits, 1.0, top_k=2)
    assert (k2 > 0).tolist() == [True, False, False, False, True]
    # top-p keeps the smallest prefix reaching p; the most likely token always stays
    assert (plain_sampling.probs(logits, 1.0, top_p=1e-6) > 0).sum() == 1
    p = logits.double().softmax(-1)
    kept = plain_sampling.probs(logits, 1.0, top_p=float(p[4] + p[0]) - 1e-9) > 0
    assert kept.tolist() == [True, False, False, False, True]
    assert (plain_sampling.probs(logits, 1.0, min_p=1.0) > 0).sum() == 1
    assert plain_sampling.draw(torch.tensor([0.2, 0.0, 0.8]), 0.1) == 0
    assert plain_sampling.draw(torch.tensor([0.2, 0.0, 0.8]), 0.2) == 2        # zero-mass entries are never drawn
    assert plain_sampling.draw(torch.tensor([0.2, 0.0, 0.8]), 0.999999) == 2
    # a row with a filter is walked in the filters' order (largest first, equal ones by index); one without, as it lies
    assert plain_sampling.drawing_order(logits, 1.0) is None and plain_sampling.drawing_order(logits, 0.0, top_k=2) is None
    order = plain_sampling.drawing_order(torch.tensor([1.0, 3.0, 3.0, -1.0]), 0.5, min_p=0.01)
    assert order.tolist() == [1, 2, 0, 3]
    q = torch.tensor([0.1, 0.4, 0.4, 0.1])
    assert [plain_sampling.draw(q, u, order) for u in (0.0, 0.39, 0.41, 0.79, 0.81, 0.95)] == [1, 1, 2, 2, 0, 3]
    assert [plain_sampling.draw(q, u) for u in (0.0, 0.39, 0.41, 0.79, 0.81, 0.95)] == [0, 1, 1, 2, 2, 3]
