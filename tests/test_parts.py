"""The parts alone, and models put together from them in ways Qwen3 does not use: a layer that runs twice, a run that
reads another run's cache, windowed beside full attention, another position encoding, and toy parts defined here (a
mixer with state of its own in the request's slot, a feed-forward with routing) that are registered, built and stepped
without touching the framework's files. Each is compared with a computation written out here from the plain functions.
CPU cases run the plain kernel twins, `gpu` cases the HIP kernels."""
from __future__ import annotations

import pytest
import torch

from holon_amd.engine.batch import StepRow
from holon_amd.engine.loading import attach_cache, build_from_spec
from holon_amd.parts import Build, Part, PartialSums, SlotState, Stream
from holon_amd.parts.linear import Linear
from holon_amd.registry import register_part, unregister_part
from holon_amd.spec import LayerSpec, ModelSpec, PartRef, Run, in_order
from holon_amd.weights.loader import finalize
from tests import helpers as H
from tests.plain import qwen3 as plain
from tests.plain.ops import TorchKernels

DEVICES = [pytest.param("cpu", id="cpu-twin"), pytest.param("cuda", marks=pytest.mark.gpu, id="hip")]
DTYPES = [torch.float32, torch.bfloat16]


def _kernels(device):
    if device == "cpu":
        return TorchKernels()
    from holon_amd.kernels import load_hip
    return load_hip()


def _close(got, want, dtype, k, what=""):
    assert H.op_budget_usage(got, want, dtype, k) <= 1, what


def _several_ops_close(got, want64, floor, dtype, k, what):
    """A chain of operations: float32 within one operation's budget of the exact result; bfloat16 no further from it
    than twice the plain functions' own bfloat16 run."""
    if dtype == torch.float32:
        return _close(got, want64, dtype, k, what)
    r, fr = H.rel_rms(got, want64), H.rel_rms(floor, want64)
    m, fm = H.max_over_rms(got, want64), H.max_over_rms(floor, want64)
    assert r <= 2 * fr + 1e-3 and m <= 2 * fm + 5e-3, f"{what}: rms {r:.3g} (floor {fr:.3g}), max {m:.3g} (floor {fm:.3g})"


def _build(device, dtype, **kw):
    return Build(kernels=_kernels(device), device=torch.device(device), dtype=dtype, max_model_len=256, **kw)


def _fill(part, seed, dtype, device, std=0.2):
    """Random tensors into every declared parameter; returns them by path (float32 copies of the rounded values)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for path, owner, name, decl in part.named_params():
        t = torch.randn(decl.shape, generator=g)
        t = (1 + 0.2 * t) if decl.init == "norm" else std * t
        t = t.to(dtype)
        setattr(owner, name, t.to(device))
        out[path] = t.float()
    finalize(part)
    return out


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_position_ffn_embedding_alone(device, dtype):
    b = _build(device, dtype)
    g = torch.Generator().manual_seed(0)
    norm = b.make(PartRef("norm", "rmsnorm", eps=1e-5), dim=1536)
    w = _fill(norm, 1, dtype, device)
    x, r = torch.randn(9, 1536, generator=g).to(dtype), torch.randn(9, 1536, generator=g).to(dtype)
    _close(norm(x.to(device)), plain.rms_norm(x.double(), w["weight"].double(), 1e-5), dtype, 1536)
    r_dev = r.clone().to(device)
    y, r2 = norm.add(x.to(device), r_dev)
    assert r2 is r_dev and torch.equal(r_dev.cpu(), x + r)
    _close(y, plain.rms_norm((x + r).double(), w["weight"].double(), 1e-5), dtype, 1536)

    rope = b.make(PartRef("position", "rope", theta=1e4), head_dim=48)
    q, k = torch.randn(7, 5, 48, generator=g).to(dtype), torch.randn(7, 2, 48, generator=g).to(dtype)
    pos = torch.tensor([0, 1, 17, 100, 255, 3, 3], dtype=torch.int32)
    qd, kd = q.clone().to(device), k.clone().to(device)
    rope.apply(qd, kd, pos.to(device))
    _close(qd, plain.rope_neox(q.double(), pos, 1e4), dtype, 2)
    _close(kd, plain.rope_neox(k.double(), pos, 1e4), dtype, 2)

    ffn = b.make(PartRef("ffn", "swiglu", inter=200), hidden=120, layer=0)
    w = _fill(ffn, 2, dtype, device)
    x = torch.randn(11, 120, generator=g).to(dtype)
    want = plain.swiglu(x, w["gate_proj.weight"].to(dtype), w["up_proj.weight"].to(dtype), w["down_proj.weight"].to(dtype))
    _close(ffn(x.to(device)), want.double(), dtype, 200)
    assert ffn.gate_proj is None and ffn.gate_up.weight.shape == (400, 120)

    embed = b.make(PartRef("embed", "table"), vocab=333, hidden=40)
    w = _fill(embed, 3, dtype, device)
    ids = torch.tensor([0, 332, 7, 7], dtype=torch.int32)
    assert torch.equal(embed(ids.to(device)).cpu().float(), w["weight"][ids.long()])
    for tied in (True, False):
        head = b.make(PartRef("head", "linear", tied=tied), vocab=333, hidden=40, embed=embed)
        hw = _fill(head, 4, dtype, device) if not tied else {}
        h = torch.randn(3, 40, generator=g).to(dtype)
        logits = head(h.to(device))
        assert logits.dtype == torch.float32
        _close(logits, h.double() @ (w["weight"] if tied else hw["weight"]).double().T, dtype, 40)


def _spec(layers, order=None, hidden=64, vocab=97, eps=1e-6):
    norm = PartRef("norm", "rmsnorm", eps=eps)
    full = tuple(LayerSpec(block=PartRef("block", "prenorm"), mixer=m, ffn=f, norm=norm) for m, f in layers)
    return ModelSpec(hidden=hidden, vocab=vocab, layers=full, order=tuple(order) if order else in_order(len(full)),
                     embed=PartRef("embed", "table"), norm=norm, head=PartRef("head", "linear", tied=False), rules=())


def _model(spec, device, dtype, seed, page_size=8, cache_tokens=256, max_seqs=4, std=0.2):
    shape = dict(device=torch.device(device), dtype=dtype, kernels=_kernels(device), page_size=page_size,
                 max_seqs=max_seqs, max_model_len=256, max_step_tokens=256)
    model, _ = build_from_spec(spec, **shape)
    weights = _fill(model, seed, dtype, device, std)
    cache, runner = attach_cache(model, cache_tokens=cache_tokens, **shape)
    return model, weights, cache, runner


def _gqa(heads, kv_heads, head_dim, eps=1e-6, theta=1e4, **kw):
    return PartRef("mixer", "gqa", heads=heads, kv_heads=kv_heads, head_dim=head_dim,
                   qk_norm=PartRef("norm", "rmsnorm", eps=eps), position=PartRef("position", "rope", theta=theta), **kw)


def _run_cut(cache, runner, ids, cuts, also=()):
    """One request through the step function in portions `cuts`; `also`: other requests run whole beside the first
    portion (mixed batch). Returns logits of every token of the request."""
    slot = cache.admit()
    others = []
    for other in also:
        s = cache.admit()
        cache.reserve(s, len(other))
        others.append(StepRow(s, 0, other, []))
    out, at = [], 0
    for n in cuts:
        cache.reserve(slot, at + n)
        rows = [StepRow(slot, at, ids[at: at + n], list(range(n)))] + (others if at == 0 else [])
        out.append(runner.run(rows).float().cpu())
        at += n
    assert at == len(ids)
    cache.release(slot)
    for r in others:
        cache.release(r.slot)
    cache.check()
    return torch.cat(out)


def _plain_attention(x, positions, w, p, heads, kv_heads, head_dim, eps, theta, window=0, kv_from=None, rotary=None):
    """The attention layer from plain parts; `kv_from`: (k, v) of another run to read instead of its own."""
    t, dt = x.shape[0], x.dtype
    q = plain.rms_norm(plain.linear(x, w[p + "q_proj.weight"].to(dt)).view(t, heads, head_dim), w[p + "q_norm.weight"].to(dt), eps)
    rope = (lambda z: plain.rope_neox(z, positions, theta)) if rotary is None else rotary
    q = rope(q)
    if kv_from is None:
        k = plain.rms_norm(plain.linear(x, w[p + "k_proj.weight"].to(dt)).view(t, kv_heads, head_dim), w[p + "k_norm.weight"].to(dt), eps)
        k, v = rope(k), plain.linear(x, w[p + "v_proj.weight"].to(dt)).view(t, kv_heads, head_dim)
    else:
        k, v = kv_from
    o = plain.causal_attention(q, k, v, window)
    return plain.linear(o.reshape(t, heads * head_dim), w[p + "o_proj.weight"].to(dt)), (k, v)


def _plain_ffn(x, w, p):
    dt = x.dtype
    return plain.swiglu(x, w[p + "gate_proj.weight"].to(dt), w[p + "up_proj.weight"].to(dt), w[p + "down_proj.weight"].to(dt))


def _plain_model(ids, w, dtype, runs, eps, mix):
    """Pre-norm residual wiring over `runs` (layer index per run); `mix(run, layer, normed_x) -> attention output`."""
    h = w["embed.weight"].to(dtype)[torch.tensor(ids)]
    for at, layer in enumerate(runs):
        p = f"layers.{layer}."
        h = h + mix(at, layer, plain.rms_norm(h, w[p + "input_norm.weight"].to(dtype), eps))
        h = h + _plain_ffn(plain.rms_norm(h, w[p + "post_norm.weight"].to(dtype), eps), w, p + "ffn.")
    return plain.linear(plain.rms_norm(h, w["norm.weight"].to(dtype), eps), w["lm_head.weight"].to(dtype)).float()


def _check_logits(got, want32, floor16, dtype, what):
    if dtype == torch.float32:
        H.assert_fp32_close(got, want32, what)
    else:
        H.assert_bf16_close(got, want32, floor16, what)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_windows_a_layer_twice_and_a_shared_cache(device, dtype):
    """Layer 0: full attention, layer 1: a window of 11 (its pages are given back as the window passes). Order:
    0, 1, 0 again with a cache of its own, then 1 again reading the cache its first run wrote."""
    hq, hkv, d, eps, theta, win = 4, 2, 16, 1e-6, 1e4, 11
    ffn = PartRef("ffn", "swiglu", inter=96)
    spec = _spec([(_gqa(hq, hkv, d), ffn), (_gqa(hq, hkv, d, window=win), ffn)],
                 order=[Run(0), Run(1), Run(0), Run(1, reads=1)])
    model, w, cache, runner = _model(spec, device, dtype, 5, page_size=4, cache_tokens=96)
    assert len(cache.groups) == 2 and sorted(len(g.sites) for g in cache.groups) == [1, 2]
    ids = H.random_ids(70, 97, 1)

    def logits(dt):
        kept = {}
        def mix(at, layer, x):
            out, kv = _plain_attention(x, torch.arange(len(ids)), w, f"layers.{layer}.mixer.", hq, hkv, d, eps, theta,
                                       window=win if layer == 1 else 0, kv_from=kept.get(1) if at == 3 else None)
            kept[at] = kv
            return out
        return _plain_model(ids, w, dt, [0, 1, 0, 1], eps, mix)
    want, floor = logits(torch.float32), logits(torch.bfloat16)
    for cuts, also in (([70], ()), ([38] + [1] * 32, ()), ([5, 2, 9, 24, 3, 2, 25], (H.random_ids(9, 97, 2),))):
        got = _run_cut(cache, runner, ids, cuts, also)
        _check_logits(got, want, floor, dtype, f"cuts {cuts[:4]}")
    windowed = next(g for g in cache.groups if g.decl.window)
    slot = cache.admit()
    cache.reserve(slot, 70)
    runner.run([StepRow(slot, 0, ids, [])])
    assert windowed.first[slot] == (70 - win + 1) // 4 and windowed.pool.usable - windowed.pool.free <= 4
    cache.release(slot)


class _Alibi(Part):
    """A position encoding defined by the test, with no fused form: it scales query and key dims by a power of the
    position's parity, so the unfused path (norm, encode, write) runs."""

    def __init__(self, build: Build, *, head_dim: int, gain: float) -> None:
        super().__init__(build)
        self.gain = gain

    def apply(self, q, k, positions):
        s = (1 + self.gain * (positions % 3).to(q.dtype))[:, None, None]
        q.mul_(s)
        if k is not None:
            k.mul_(s)

    def fusion(self):
        return None


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_other_position_encodings(device, dtype):
    """Partial rotary (the first 8 of 16 dims), no encoding at all, and one defined here without a fused kernel."""
    register_part("position", "test-scale")(_Alibi)
    try:
        hq, hkv, d, eps = 4, 4, 16, 1e-5
        norm = PartRef("norm", "rmsnorm", eps=eps)
        def mixer(position):
            return PartRef("mixer", "gqa", heads=hq, kv_heads=hkv, head_dim=d, qk_norm=norm, position=position)
        ffn = PartRef("ffn", "swiglu", inter=80)
        spec = _spec([(mixer(PartRef("position", "rope", theta=1e4, rotary_dim=8)), ffn),
                      (mixer(PartRef("position", "none")), ffn),
                      (mixer(PartRef("position", "test-scale", gain=0.5)), ffn)], eps=eps)
        model, w, cache, runner = _model(spec, device, dtype, 6)
        assert model.blocks[2].mixer._fused is None and model.blocks[0].mixer._fused is not None
        ids = H.random_ids(45, 97, 3)
        pos = torch.arange(len(ids))

        def logits(dt):
            def partial(z):
                return torch.cat((plain.rope_neox(z[..., :8], pos, 1e4), z[..., 8:]), -1)
            def scale(z):
                return z * (1 + 0.5 * (pos % 3).to(z.dtype))[:, None, None]
            rot = {0: partial, 1: lambda z: z, 2: scale}
            def mix(at, layer, x):
                return _plain_attention(x, pos, w, f"layers.{layer}.mixer.", hq, hkv, d, eps, 1e4, rotary=rot[layer])[0]
            return _plain_model(ids, w, dt, [0, 1, 2], eps, mix)
        want, floor = logits(torch.float32), logits(torch.bfloat16)
        for cuts in ([45], [13, 2, 30], [20] + [1] * 25):
            _check_logits(_run_cut(cache, runner, ids, cuts), want, floor, dtype, f"cuts {cuts[:3]}")
    finally:
        unregister_part("position", "test-scale")


class _RunningMean(Part):
    """A toy mixer with state of its own: y[t] = W (decay * s[t-1] + x[t]), s kept per request in its slot between
    steps (float32), reset when the request starts at position 0."""

    def __init__(self, build: Build, *, hidden: int, layer: int, decay: float) -> None:
        super().__init__(build)
        self.decay, self.hidden = decay, hidden
        self.attach("proj", Linear(build, inp=hidden, out=hidden))

    def state(self):
        return [SlotState("s", (self.hidden,), torch.float32)]

    def forward(self, x, step, site):
        state = site.slot_state["s"]
        mixed = torch.empty_like(x, dtype=torch.float32)
        at = 0
        for slot, start, n in zip(step.h_slots.tolist(), step.h_starts.tolist(), step.h_counts.tolist()):
            s = torch.zeros_like(state[slot]) if start == 0 else state[slot].clone()
            for i in range(at, at + n):
                s = self.decay * s + x[i].float()
                mixed[i] = s
            state[slot] = s
            at += n
        return self.proj(mixed.to(x.dtype))

    __call__ = forward


class _TopOne(Part):
    """A toy feed-forward with routing: a float32 router picks one of `experts` small SwiGLUs per token."""

    def __init__(self, build: Build, *, hidden: int, layer: int, inter: int, experts: int) -> None:
        super().__init__(build)
        self.attach("router", Linear(build, inp=hidden, out=experts))
        self.experts = [self.attach(f"experts.{e}", build.make(PartRef("ffn", "swiglu", inter=inter), hidden=hidden, layer=layer))
                        for e in range(experts)]

    def forward(self, x, step=None):
        choice = self.router(x, torch.float32).argmax(-1)
        out = torch.zeros_like(x)
        for e, expert in enumerate(self.experts):
            idx = torch.nonzero(choice == e)[:, 0]
            if len(idx):
                out[idx] = expert(x[idx].contiguous())
        return out

    __call__ = forward


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_slot_state_and_toy_routed_ffn(device, dtype):
    register_part("mixer", "test-running-mean")(_RunningMean)
    register_part("ffn", "test-top-one")(_TopOne)
    try:
        hq, hkv, d, eps, decay = 4, 1, 16, 1e-6, 0.75
        spec = _spec([(PartRef("mixer", "test-running-mean", decay=decay), PartRef("ffn", "swiglu", inter=96)),
                      (_gqa(hq, hkv, d), PartRef("ffn", "test-top-one", inter=48, experts=3)),
                      (PartRef("mixer", "test-running-mean", decay=decay), PartRef("ffn", "swiglu", inter=96))],
                     order=[Run(0), Run(1), Run(2), Run(0)])
        model, w, cache, runner = _model(spec, device, dtype, 7, std=0.3)
        assert len(cache.slot_states) == 3 and len(cache.groups) == 1           # three runs keep a state, one keeps pages
        ids = H.random_ids(50, 97, 4)
        pos = torch.arange(len(ids))

        def logits(dt):
            def ema(layer, x):
                s, rows = torch.zeros(64), []
                for t in range(x.shape[0]):
                    s = decay * s + x[t].float()
                    rows.append(s)
                return plain.linear(torch.stack(rows).to(dt), w[f"layers.{layer}.mixer.proj.weight"].to(dt))
            def mix(at, layer, x):
                if layer == 1:
                    return _plain_attention(x, pos, w, "layers.1.mixer.", hq, hkv, d, eps, 1e4)[0]
                return ema(layer, x)
            h = w["embed.weight"].to(dt)[torch.tensor(ids)]
            for at, layer in enumerate([0, 1, 2, 0]):
                p = f"layers.{layer}."
                h = h + mix(at, layer, plain.rms_norm(h, w[p + "input_norm.weight"].to(dt), eps))
                x = plain.rms_norm(h, w[p + "post_norm.weight"].to(dt), eps)
                if layer == 1:
                    choice = (x.float() @ w[p + "ffn.router.weight"].to(dt).float().T).argmax(-1)
                    y = torch.stack([_plain_ffn(x[t: t + 1], w, p + f"ffn.experts.{int(choice[t])}.")[0] for t in range(len(ids))])
                else:
                    y = _plain_ffn(x, w, p + "ffn.")
                h = h + y
            return plain.linear(plain.rms_norm(h, w["norm.weight"].to(dt), eps), w["lm_head.weight"].to(dt)).float()
        want, floor = logits(torch.float32), logits(torch.bfloat16)
        for cuts, also in (([50], ()), ([18] + [1] * 32, ()), ([7, 2, 19, 2, 20], (H.random_ids(12, 97, 5),))):
            got = _run_cut(cache, runner, ids, cuts, also)
            if dtype == torch.float32:
                H.assert_fp32_close(got, want, f"toy parts, cuts {cuts[:3]}")
            else:     # a routed token may flip expert in bfloat16: compare the bulk
                close = ((got - want).abs().amax(-1) / want.pow(2).mean().sqrt()) < 0.1
                assert close.float().mean() > 0.9
        # a slot handed to a new request starts from a clean state
        again = _run_cut(cache, runner, ids, [50])
        assert torch.equal(again, _run_cut(cache, runner, ids, [50]))
    finally:
        unregister_part("mixer", "test-running-mean")
        unregister_part("ffn", "test-top-one")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_gqa_mixer_and_block_alone(device, dtype):
    """One attention mixer, then one pre-norm block, stepped whole and in portions against the plain functions; the
    query and key weights are scaled up so that attention is peaked."""
    for hq, hkv, d, page in ((8, 2, 64, 16), (6, 3, 32, 8), (5, 5, 48, 4)):
        hidden, eps = 72, 1e-5
        spec = _spec([(_gqa(hq, hkv, d, eps=eps, theta=1e6), PartRef("ffn", "swiglu", inter=56))], hidden=hidden, eps=eps)
        model, w, cache, runner = _model(spec, device, dtype, 8 + d, page_size=page, std=0.3)
        block = model.blocks[0]
        for name in ("q_norm", "k_norm"):
            getattr(block.mixer, name).weight.mul_(2.0)
            w[f"layers.0.mixer.{name}.weight"] *= 2.0
        g = torch.Generator().manual_seed(d)
        x = torch.randn(37, hidden, generator=g).to(dtype)
        pos = torch.arange(37)
        w64 = {k: v.double() for k, v in w.items()}
        want_mix = _plain_attention(x.double(), pos, w64, "layers.0.mixer.", hq, hkv, d, eps, 1e6)[0]
        floor_mix = _plain_attention(x, pos, w, "layers.0.mixer.", hq, hkv, d, eps, 1e6)[0]     # the same in `dtype`
        slot = cache.admit()
        got, at = [], 0
        for n in (20, 2, 15):
            cache.reserve(slot, at + n)
            step, _ = runner.prepare([StepRow(slot, at, [0] * n, [])])
            got.append(block.mixer(x[at: at + n].contiguous().to(device), step, model.sites[0]))
            cache.advance(slot, at + n)
            at += n
        _several_ops_close(torch.cat(got), want_mix, floor_mix, dtype, hidden + 37, f"mixer {hq}/{hkv}/{d}")
        cache.release(slot)
        # the block: residual stream in, (stream, pending term) out
        slot = cache.admit()
        cache.reserve(slot, 37)
        step, _ = runner.prepare([StepRow(slot, 0, [0] * 37, [])])
        out = block(Stream(x.clone().to(device)), step, model.sites[0])
        delta = out.delta.value() if isinstance(out.delta, PartialSums) else out.delta
        stream = out.h.float() + (delta.float() if delta is not None else 0)    # the last add may be done or pending
        def whole(xd, wd):
            a = xd + _plain_attention(plain.rms_norm(xd, wd["layers.0.input_norm.weight"], eps), pos, wd,
                                      "layers.0.mixer.", hq, hkv, d, eps, 1e6)[0]
            return a + _plain_ffn(plain.rms_norm(a, wd["layers.0.post_norm.weight"], eps), wd, "layers.0.ffn.")
        _several_ops_close(stream, whole(x.double(), w64), whole(x, w), dtype, 4 * hidden, f"block {hq}/{hkv}/{d}")
        cache.release(slot)


# -- the seams another architecture would need, each with a toy part from tests/toy_parts.py ---------------------------
def _weights_of(model):
    """Every parameter of a built model by path, as float32 copies on the host (after merging)."""
    return {path: getattr(owner, name).detach().float().cpu() for path, owner, name, _ in model.named_params()}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_two_paged_states_of_different_widths(device, dtype):
    from tests.toy_parts import TwoCaches
    register_part("mixer", "test-two-caches")(TwoCaches)
    try:
        hq, hkv, d, eps = 4, 1, 16, 1e-6
        ffn = PartRef("ffn", "swiglu", inter=96)
        spec = _spec([(PartRef("mixer", "test-two-caches"), ffn), (_gqa(hq, hkv, d), ffn),
                      (PartRef("mixer", "test-two-caches"), ffn)])
        model, w, cache, runner = _model(spec, device, dtype, 11, page_size=4, cache_tokens=96)
        widths = sorted((g.decl.elems, len(g.members)) for g in cache.groups)
        assert widths == [(1, 2), (2 * hkv * d, 1), (64, 2)]                 # three groups, three block tables
        assert not runner.use_graphs and "TwoCaches" in runner.not_graph_safe
        ids = H.random_ids(61, 97, 8)
        pos = torch.arange(len(ids))

        def logits(dt):
            def mix(at, layer, x):
                if layer == 1:
                    return _plain_attention(x, pos, w, "layers.1.mixer.", hq, hkv, d, eps, 1e4)[0]
                weight = 1 + x[:, :1].float() ** 2
                mean = (weight * x.float()).cumsum(0) / weight.cumsum(0)
                return plain.linear(mean.to(dt), w[f"layers.{layer}.mixer.proj.weight"].to(dt))
            return _plain_model(ids, w, dt, [0, 1, 2], eps, mix)
        want, floor = logits(torch.float32), logits(torch.bfloat16)
        for cuts, also in (([61], ()), ([29] + [1] * 32, ()), ([3, 2, 17, 9, 30], (H.random_ids(13, 97, 9),))):
            _check_logits(_run_cut(cache, runner, ids, cuts, also), want, floor, dtype, f"two caches, cuts {cuts[:3]}")
        assert all(g.pool.free == g.pool.usable for g in cache.groups)
    finally:
        unregister_part("mixer", "test-two-caches")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_ffn_with_stacked_expert_weights(device, dtype):
    from tests.toy_parts import StackedTopOne
    register_part("ffn", "test-stacked-top-one")(StackedTopOne)
    try:
        hq, hkv, d, eps, inter, experts = 4, 1, 16, 1e-6, 40, 3
        spec = _spec([(_gqa(hq, hkv, d), PartRef("ffn", "test-stacked-top-one", inter=inter, experts=experts)),
                      (_gqa(hq, hkv, d), PartRef("ffn", "swiglu", inter=96))])
        model, w, cache, runner = _model(spec, device, dtype, 12, std=0.3)
        assert model.blocks[0].ffn.gate_up.shape == (experts, 2 * inter, 64)
        ids = H.random_ids(40, 97, 10)
        pos = torch.arange(len(ids))

        def logits(dt):
            h = w["embed.weight"].to(dt)[torch.tensor(ids)]
            for layer in (0, 1):
                p = f"layers.{layer}."
                x = plain.rms_norm(h, w[p + "input_norm.weight"].to(dt), eps)
                h = h + _plain_attention(x, pos, w, p + "mixer.", hq, hkv, d, eps, 1e4)[0]
                x = plain.rms_norm(h, w[p + "post_norm.weight"].to(dt), eps)
                if layer == 1:
                    h = h + _plain_ffn(x, w, p + "ffn.")
                    continue
                choice = (x.float() @ w[p + "ffn.router.weight"].to(dt).float().T).argmax(-1)
                rows = []
                for t in range(len(ids)):
                    gu, down = w[p + "ffn.gate_up"][int(choice[t])].to(dt), w[p + "ffn.down"][int(choice[t])].to(dt)
                    rows.append(plain.swiglu(x[t: t + 1], gu[:inter], gu[inter:], down)[0])
                h = h + torch.stack(rows)
            return plain.linear(plain.rms_norm(h, w["norm.weight"].to(dt), eps), w["lm_head.weight"].to(dt)).float()
        want = logits(torch.float32)
        for cuts in ([40], [8] + [1] * 32, [7, 2, 31]):
            got = _run_cut(cache, runner, ids, cuts)
            if dtype == torch.float32:
                H.assert_fp32_close(got, want, f"stacked experts, cuts {cuts[:3]}")
            else:     # a routed token may flip expert in bfloat16: compare the bulk
                close = ((got - want).abs().amax(-1) / want.pow(2).mean().sqrt()) < 0.1
                assert close.float().mean() > 0.9
    finally:
        unregister_part("ffn", "test-stacked-top-one")


@pytest.mark.parametrize("device", DEVICES)
def test_toy_architecture_through_the_engine_with_a_portion_grid_and_graphs_asked_for(device):
    """A toy architecture registered here (its own config.json keys, recipe and mixer) generates through the engine.
    Its mixer keeps a running sum in the request's slot, lets prompt portions end only on a grid of 8 positions (the
    step budget of 13 does not fall on it) and plans on the host, so although graphs are asked for every step runs
    eagerly. Greedy tokens equal a computation written out here from the plain functions."""
    from holon_amd.config import EngineConfig, SamplingParams
    from holon_amd.engine.engine import Engine
    from holon_amd.registry import register_architecture, unregister_architecture
    from tests.toy_parts import GridRunningMean, ToyConfig, toy_recipe
    register_part("mixer", "test-grid-mean")(GridRunningMean)
    register_architecture("ToyGridModel", ToyConfig, toy_recipe)
    try:
        config = {"architectures": ["ToyGridModel"], "width": 48, "tokens": 61, "depth": 2, "grid": 8, "eps": 1e-5}
        engine = Engine.from_random(config, 3, EngineConfig(
            model="random:toy", device=device, dtype="float32", page_size=4, max_seqs=3, max_model_len=64,
            max_step_tokens=13, graphs=True, overlap=True), kernels=_kernels(device))
        assert not engine.runner.use_graphs and engine.runner.not_graph_safe == ["GridRunningMean"]
        assert engine.cache.prefix is None and not engine.cache.groups           # nothing paged, nothing shared
        w = _weights_of(engine.model)

        def greedy(ids, n):
            ids, out = list(ids), []
            for _ in range(n):
                h = w["embed.weight"][torch.tensor(ids)]
                for layer in (0, 1):
                    p = f"layers.{layer}."
                    x = plain.rms_norm(h, w[p + "input_norm.weight"], 1e-5)
                    mean = x.cumsum(0) / torch.arange(1, len(ids) + 1)[:, None]
                    h = h + plain.linear(mean, w[p + "mixer.proj.weight"])
                    x = plain.rms_norm(h, w[p + "post_norm.weight"], 1e-5)
                    gu = w[p + "ffn.gate_up.weight"]
                    h = h + plain.swiglu(x, gu[:96], gu[96:], w[p + "ffn.down_proj.weight"])
                logits = plain.linear(plain.rms_norm(h, w["norm.weight"], 1e-5), w["embed.weight"])
                out.append(int(logits[-1].argmax()))
                ids.append(out[-1])
            return out
        prompts = [H.random_ids(n, 61, 20 + n) for n in (30, 5, 21, 9)]
        got = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
        assert got == [greedy(p, 10) for p in prompts]
        portions = engine.model.blocks[0].mixer.portions
        assert (0, 8) in portions and (8, 8) in portions and (24, 6) in portions     # the prompt of 30: 8, 8, 8, 6
        assert all(start % 8 == 0 for start, n in portions if n > 1)
        with pytest.raises(ValueError, match="no prompt portion"):               # a budget that reaches no grid position
            Engine.from_random(config, 3, EngineConfig(model="random:toy", device=device, dtype="float32", page_size=4,
                                                       max_seqs=3, max_model_len=64, max_step_tokens=7),
                               kernels=_kernels(device))
    finally:
        unregister_part("mixer", "test-grid-mean")
        unregister_architecture("ToyGridModel")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_that_brings_a_kernel_of_its_own(device, dtype):
    """A toy mixer under tests/ registers the operation it needs beside itself: the plain form, and a HIP symbol with
    its argument types and its own source file, which is compiled into a library of its own. Every kernel set then
    answers `kernels.decay_scan(...)`: the plain twin runs the plain form, the HIP kernels the symbol. The toy
    architecture generates through the engine (prompt portions under a small step budget, then decode steps, replayed
    from graphs on the GPU) and its greedy tokens equal a whole-sequence computation written out here. No file of
    the framework names the operation."""
    from holon_amd.config import EngineConfig, SamplingParams
    from holon_amd.engine.engine import Engine
    from holon_amd.kernels.registry import kernel_ops, register_kernel, unregister_kernel
    from holon_amd.registry import register_architecture, unregister_architecture
    from tests.toy_parts import DecayScan, ToyScanConfig, decay_scan_op, toy_scan_recipe
    register_kernel(decay_scan_op())
    register_part("mixer", "test-decay-scan")(DecayScan)
    register_architecture("ToyScanModel", ToyScanConfig, toy_scan_recipe)
    try:
        assert "decay_scan" in kernel_ops()
        with pytest.raises(KeyError, match="twice"):
            register_kernel(decay_scan_op())
        config = {"architectures": ["ToyScanModel"], "width": 64, "tokens": 97, "depth": 2, "decay": 0.75, "eps": 1e-5}
        kernels = _kernels(device)
        engine = Engine.from_random(config, 5, EngineConfig(
            model="random:toy-scan", device=device, dtype=dtype, page_size=4, max_seqs=4, max_model_len=96,
            max_step_tokens=16, graphs=True, overlap=True), kernels=kernels)
        assert engine.runner.use_graphs == (device == "cuda") and not engine.runner.not_graph_safe
        with pytest.raises(AttributeError, match="no operation"):
            kernels.an_operation_nobody_registered
        w = _weights_of(engine.model)
        dt = getattr(torch, dtype)

        def logits(ids):
            h = w["embed.weight"].to(dt)[torch.tensor(ids)]
            for layer in (0, 1):
                p = f"layers.{layer}."
                x = plain.rms_norm(h, w[p + "input_norm.weight"].to(dt), 1e-5)
                s, rows = torch.zeros(64), []
                for t in range(len(ids)):
                    s = 0.75 * s + x[t].float()
                    rows.append(s.to(dt))
                h = h + plain.linear(torch.stack(rows), w[p + "mixer.proj.weight"].to(dt))
                x = plain.rms_norm(h, w[p + "post_norm.weight"].to(dt), 1e-5)
                gu = w[p + "ffn.gate_up.weight"].to(dt)
                h = h + plain.swiglu(x, gu[:128], gu[128:], w[p + "ffn.down_proj.weight"].to(dt))
            return plain.linear(plain.rms_norm(h, w["norm.weight"].to(dt), 1e-5), w["embed.weight"].to(dt)).float()

        def greedy_follows(prompt, got):
            ids = list(prompt)
            for token in got:
                last = logits(ids)[-1]
                top = last.topk(2).values
                if float(top[0] - top[1]) > (1e-4 if dtype == "float32" else 0.05) * float(last.std()):
                    assert token == int(last.argmax()), (len(ids), token, int(last.argmax()))
                ids.append(token)
        prompts = [H.random_ids(n, 97, 30 + n) for n in (37, 5, 21, 9)]
        got = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
        for prompt, tokens in zip(prompts, got):
            assert len(tokens) == 12
            greedy_follows(prompt, tokens)
        if device == "cuda":
            from tests.toy_parts import DECAY_SCAN_SOURCE
            assert str(DECAY_SCAN_SOURCE) in kernels._part_libs and engine.runner.graph_replays > 5
    finally:
        unregister_architecture("ToyScanModel")
        unregister_part("mixer", "test-decay-scan")
        unregister_kernel("decay_scan")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_norm_and_an_embedding_that_implement_only_their_base_class(device, dtype):
    """Another norm (no weight: x centred, over its root mean square) and another embedding (the table's rows times a
    constant) written as the base classes ask: `NormPart.forward`, `EmbedPart.rows`. What the model and the blocks
    call beside these (the residual add in front of a norm, tokens taken from the device, row statistics, deferral,
    fusion into other kernels) comes from the base classes' defaults: nothing is folded or fused, every step gives the
    plain computation. A part of a family the framework does not know opens it."""
    from holon_amd.parts import EmbedPart, NormPart
    from holon_amd.registry import RegistryError, part_class

    class Centred(NormPart):
        graph_safe = True

        def __init__(self, build, *, eps, dim):
            super().__init__(build)
            self.eps = eps

        def forward(self, x):
            x32 = x.float() - x.float().mean(-1, keepdim=True)
            return (x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + self.eps)).to(x.dtype)

    class ScaledTable(EmbedPart):
        graph_safe = True

        def __init__(self, build, *, vocab, hidden, scale):
            super().__init__(build)
            self.scale = scale
            self.declare("weight", (vocab, hidden))

        def rows(self, ids):
            return (self.weight[ids.long()].float() * self.scale).to(self.weight.dtype)

    register_part("norm", "test-centred")(Centred)
    register_part("embed", "test-scaled-table")(ScaledTable)
    register_part("test-family", "thing")(Centred)
    try:
        assert part_class(PartRef("test-family", "thing")) is Centred
        with pytest.raises(RegistryError, match="test-family"):
            part_class(PartRef("test-family", "other"))
        hq, hkv, d, eps = 4, 2, 16, 1e-5
        norm = PartRef("norm", "test-centred", eps=eps)
        layer = LayerSpec(block=PartRef("block", "prenorm"), mixer=_gqa(hq, hkv, d), ffn=PartRef("ffn", "swiglu", inter=96),
                          norm=norm)
        spec = ModelSpec(hidden=64, vocab=97, layers=(layer, layer), order=in_order(2),
                         embed=PartRef("embed", "test-scaled-table", scale=1.5), norm=norm,
                         head=PartRef("head", "linear", tied=False), rules=())
        model, w, cache, runner = _model(spec, device, dtype, 21, page_size=4, cache_tokens=96)
        assert not model.blocks[0]._mixer_defers and not model.blocks[0]._ffn_defers        # nothing to fold
        ids = H.random_ids(45, 97, 22)
        pos = torch.arange(len(ids))

        def centred(x):
            x32 = x.float() - x.float().mean(-1, keepdim=True)
            return (x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype)

        def logits(dt):
            h = (w["embed.weight"].to(dt)[torch.tensor(ids)].float() * 1.5).to(dt)
            for layer_at in (0, 1):
                p = f"layers.{layer_at}."
                h = h + _plain_attention(centred(h), pos, w, p + "mixer.", hq, hkv, d, 1e-6, 1e4)[0]
                h = h + _plain_ffn(centred(h), w, p + "ffn.")
            return plain.linear(centred(h), w["lm_head.weight"].to(dt)).float()
        want, floor = logits(torch.float32), logits(torch.bfloat16)
        for cuts, also in (([45], ()), ([13] + [1] * 32, ()), ([3, 2, 17, 9, 14], (H.random_ids(13, 97, 9),))):
            _check_logits(_run_cut(cache, runner, ids, cuts, also), want, floor, dtype, f"base-class parts, cuts {cuts[:3]}")
    finally:
        unregister_part("norm", "test-centred")
        unregister_part("embed", "test-scaled-table")
        unregister_part("test-family", "thing")
