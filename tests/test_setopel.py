"""Setopel decoders (mistralrs_amd.hybrid: residual streams, GatedSinkAttention, RetentionMixer, LatentAttention, GluFeedForward; the kernels added to csrc/hyb_kernels.hip and
the batched products of csrc/hyb_gemm.hip) against the plain float64 restatement in tests/setopel_oracle.py.

Every test builds its own small configuration with random bf16-representable weights.  The sharp comparisons run in the all-f32 mode (a wrong key, a lost state, a sink left
out is an O(1) error there, rounding is 1e-6); the bf16 mode is held to a rounding-sized bar.  CPU tests cover what needs no device.
"""
import io
import json
import math
import os

import numpy as np
import pytest
import torch

import mistralrs_amd  # noqa: F401
from mistralrs_amd import _lib
from tests import setopel_oracle as O


# ---------------------------------------------------------------------------------------------------------------- configurations and weights
def glu(ff=56):
    return {"kind": "dense", "ff": ff}


def attn(heads=4, kv_heads=2, dim=16, vdim=8, conv=3, cap=6.0, coef=0.25, every=16, kv_from=None, mlp="glu", scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if conv:
        m["conv"] = conv
    if cap:
        m["softcap"] = cap
    if coef:
        m["q_temp"] = {"coef": coef, "every": every}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": glu() if mlp == "glu" else mlp}


def ret(heads=2, dim=8, vdim=16, decay=(0.9375, 0.998046875), dims=6, base=500.0, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if dims:
        m["rot"] = {"dims": dims, "base": base}
    return {"type": "retention", "mixer": m, "mlp": glu() if mlp == "glu" else mlp}


def lat(heads=3, dim=16, vdim=8, rank=24, mlp="glu", scale=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)},
            "mlp": glu() if mlp == "glu" else mlp}


def config(layers, vocab=96, width=40, eps=1e-5, streams=3, mult=0.4):
    c = {"architecture": "Setopel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams:
        c["streams"] = streams
    if mult is not None:
        c["residual_mult"] = mult
    return c


def weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg.get("streams", 0)
    w = {}

    def rnd(*shape, scale=1.0, shift=0.0):
        return (torch.randn(*shape, generator=g) * scale + shift).to(torch.bfloat16)
    w["embed"], w["head"] = rnd(cfg["vocab"], W), rnd(cfg["vocab"], W, scale=W ** -0.5)
    w["embed.norm"], w["final.norm"] = rnd(W, scale=0.2), rnd(W, scale=0.2)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for q in (1, 2) if L.get("mlp") else (1,):
            w[f"{p}norm{q}"] = rnd(W, scale=0.2)
            if S:
                w[f"{p}hc{q}.in"], w[f"{p}hc{q}.out"] = rnd(S, scale=0.3, shift=1.0 / S), rnd(S, scale=0.4, shift=1.0)
                w[f"{p}hc{q}.mix"] = (torch.eye(S) * 0.8 + 0.25 * torch.randn(S, S, generator=g)).to(torch.bfloat16)
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "attention":
            G = m["kv_heads"]
            names = {"q": H * D, "k": G * D, "v": G * Dv} if m.get("kv_from") is None else {"q": H * D}
            for n, rows in names.items():
                w[f"{p}mix.{n}"], w[f"{p}mix.{n}.b"] = rnd(rows, W, scale=(1.0 if n == "v" else 1.5) * W ** -0.5), rnd(rows, scale=0.3)
                if m.get("conv"):
                    w[f"{p}mix.{n}.conv"] = rnd(rows, m["conv"], scale=0.6)
            w[p + "mix.g"], w[p + "mix.o"] = rnd(H * Dv, W, scale=2.0 * W ** -0.5), rnd(W, H * Dv, scale=(H * Dv) ** -0.5)
        elif L["type"] == "retention":
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = rnd(H * D, W, scale=1.5 * W ** -0.5), rnd(H * D, W, scale=1.5 * W ** -0.5), rnd(H * Dv, W, scale=W ** -0.5)
            w[p + "mix.g"], w[p + "mix.o"] = rnd(H * Dv, W, scale=2.0 * W ** -0.5), rnd(W, H * Dv, scale=(H * Dv) ** -0.5)
        else:
            R = m["kv_rank"]
            w[p + "mix.q"], w[p + "mix.dkv"], w[p + "mix.dkv.norm"] = rnd(H * D, W, scale=1.5 * W ** -0.5), rnd(R, W, scale=W ** -0.5), rnd(R, scale=0.2, shift=1.0)
            w[p + "mix.uk"], w[p + "mix.uv"] = rnd(H * D, R, scale=1.5 * R ** -0.5), rnd(H * Dv, R, scale=R ** -0.5)
            w[p + "mix.o"] = rnd(W, H * Dv, scale=(H * Dv) ** -0.5)
        f = L.get("mlp")
        if f:
            w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = rnd(f["ff"], W, scale=2 * W ** -0.5), rnd(f["ff"], W, scale=2 * W ** -0.5), rnd(W, f["ff"], scale=f["ff"] ** -0.5)
    return w


def f64(w):
    return {k: v.to(torch.float64) for k, v in w.items()}


STACK = [lat(), attn(), ret(), lat(heads=2, dim=8, vdim=12, rank=16, mlp=None), attn(kv_from=1, every=5, cap=0.0), ret(heads=3, dim=16, vdim=8, decay=(0.5, 0.96875, 1.0), dims=16, mlp="glu"),
         attn(heads=6, kv_heads=3, dim=8, vdim=12, conv=0, coef=0.0, mlp=None)]


class Served:
    """A model on the device with its caches, stepped the way the engine and the trace runner step it."""

    def __init__(self, cfg, w, dev, dtype="float32", max_tokens=512, slots=4, block_size=32):
        from mistralrs_amd.hybrid import SPEC_READERS, HybridCache, HybridDecoder
        self.bs = block_size
        self.m = HybridDecoder(SPEC_READERS[cfg["architecture"]](cfg), dev, dtype, num_blocks=-(-max_tokens // block_size) + slots + 1, block_size=block_size, state_slots=slots)
        self.m.load_weights(w.__getitem__)
        self.cache = HybridCache(self.m)
        self.len = {}

    def step(self, parts):
        """parts: [(request id, tokens)]; logits of every row, split per part"""
        from mistralrs_amd.hybrid import RaggedBatch
        entries = []
        for rid, tk in parts:
            p0 = self.len.get(rid, 0)
            assert self.cache.reserve(rid, p0 + len(tk)), "out of pages / slots"
            entries.append(self.cache.entry(rid, tk, p0, range(len(tk))))
            self.len[rid] = p0 + len(tk)
        out = self.m.forward_batch(RaggedBatch.build(entries, self.bs, self.m.device)).double().cpu()
        res, r = [], 0
        for _, tk in parts:
            res.append(out[r:r + len(tk)])
            r += len(tk)
        return res

    def end(self, rid):
        self.cache.release(rid)
        self.len.pop(rid, None)


def rel(a, b):
    return float((a - b).norm() / (b.norm() + 1e-30))


def close(a, b, bar):
    """f32 mode (bar < 1e-3): the whole tensor within `bar`.  bf16 mode: the typical row within `bar`, at most one row in ten above five times that."""
    if bar < 1e-3:
        return rel(a, b) < bar
    rows = (a - b).reshape(-1, a.shape[-1]).norm(dim=1) / (b.reshape(-1, b.shape[-1]).norm(dim=1) + 1e-30)
    return float(rows.median()) < bar and float((rows > 5 * bar).double().mean()) <= 0.1


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _model(layers, dev, dtype="float32", seed=1, **kw):
    cfg = config(layers, **{k: v for k, v in kw.items() if k in ("vocab", "width", "eps", "streams", "mult")})
    w = weights(cfg, seed)
    return cfg, w, Served(cfg, w, dev, dtype, **{k: v for k, v in kw.items() if k in ("max_tokens", "slots", "block_size")})


def _batch(dev, parts, bs=32, blocks=None):
    """a RaggedBatch of [(first position, rows, state slot)] over made-up block tables"""
    from mistralrs_amd.hybrid import RaggedBatch
    entries, nb = [], 0
    for k, (p0, n, slot) in enumerate(parts):
        need = -(-(p0 + n) // bs)
        blk = blocks[k] if blocks else list(range(nb + 1, nb + 1 + need))
        nb += need
        entries.append({"tokens": [0] * n, "pos0": p0, "slot": slot, "blocks": blk, "want": []})
    return RaggedBatch.build(entries, bs, dev)


# ---------------------------------------------------------------------------------------------------------------- no device needed
def test_config_reader_takes_every_size_and_constant_from_the_file():
    from mistralrs_amd.hybrid import GluSpec, LatentAttentionSpec, RetentionSpec, SinkAttentionSpec, setopel_spec
    cfg = config([attn(heads=6, kv_heads=3, dim=10, vdim=14, conv=5, cap=11.0, coef=0.75, every=9, mlp=glu(77), scale=0.3),
                  attn(heads=6, kv_heads=3, dim=10, vdim=14, conv=0, cap=0.0, coef=0.0, kv_from=0, mlp=None),
                  ret(heads=3, dim=12, vdim=20, decay=(0.5, 0.75, 0.875), dims=4, base=77.0, mlp="glu"), ret(dims=0),
                  lat(heads=5, dim=6, vdim=7, rank=9, mlp=glu(3), scale=0.7)], vocab=123, width=56, eps=3e-4, streams=4, mult=0.125)
    sp = setopel_spec(cfg)
    assert (sp.vocab, sp.width, sp.eps, sp.norm, sp.post_norms, sp.embed_norm, sp.residual_mult, sp.streams) == (123, 56, 3e-4, "rms_one_plus", False, "embed.norm", 0.125, 4)
    a, b, c, d, e = sp.layers
    assert [l.kind for l in sp.layers] == ["sink_attention", "sink_attention", "retention", "retention", "latent_attention"]
    assert isinstance(a.mixer, SinkAttentionSpec) and isinstance(c.mixer, RetentionSpec) and isinstance(e.mixer, LatentAttentionSpec)
    assert (a.mixer.heads, a.mixer.kv_heads, a.mixer.dim, a.mixer.vdim, a.mixer.scale, a.mixer.conv, a.mixer.softcap, a.mixer.temp_coef, a.mixer.temp_every, a.mixer.kv_from,
            a.mixer.sink) == (6, 3, 10, 14, 0.3, 5, 11.0, 0.75, 9, None, True)
    assert isinstance(a.ff, GluSpec) and a.ff.ff == 77 and b.ff is None
    assert (b.mixer.conv, b.mixer.softcap, b.mixer.temp_every, b.mixer.kv_from) == (0, 0.0, 0, 0)
    assert (c.mixer.heads, c.mixer.dim, c.mixer.vdim, c.mixer.decay, c.mixer.rotary.dims, c.mixer.rotary.base, c.mixer.rotary.layout) == (3, 12, 20, [0.5, 0.75, 0.875], 4, 77.0, "half")
    assert d.mixer.rotary is None and c.ff.ff == 56
    assert (e.mixer.heads, e.mixer.dim, e.mixer.vdim, e.mixer.kv_rank, e.mixer.scale, e.ff.ff) == (5, 6, 7, 9, 0.7, 3)
    assert [l.prefix for l in sp.layers] == ["l0.", "l1.", "l2.", "l3.", "l4."]
    plain = setopel_spec(config([lat()], streams=0, mult=None))
    assert (plain.streams, plain.residual_mult) == (0, 1.0)
    for bad in ([attn(kv_from=0)], [attn(), attn(kv_from=1)], [attn(), attn(kv_from=0), attn(kv_from=1)], [attn(), attn(dim=8, kv_from=0)], [lat(), attn(kv_from=0)],
                [ret(decay=(0.5,))], [{"type": "mamba2", "mixer": {}, "mlp": None}], [lat(mlp={"kind": "moe"})]):
        with pytest.raises(ValueError):
            setopel_spec(config(bad))


def test_registry_and_synthetic_weights_know_the_architecture():
    from mistralrs_amd import registry
    from mistralrs_amd.hybrid import FEED_FORWARDS, MIXERS, SPEC_READERS, setopel_spec, synthetic_weights
    assert "Setopel" in registry.ARCHITECTURES and "Setopel" in SPEC_READERS
    assert {"sink_attention", "retention", "latent_attention"} <= set(MIXERS) and "dense_glu_silu" in FEED_FORWARDS
    for streams in (3, 0):
        cfg = config(STACK, streams=streams)
        get = synthetic_weights(setopel_spec(cfg), "cpu", 1)
        for name, t in weights(cfg).items():
            assert tuple(get(name).shape) == tuple(t.shape), name
        with pytest.raises(KeyError):
            get("l4.mix.k")   # a layer that reads another layer's pages has no key projection


def test_restatement_pieces():
    """the oracle's own building blocks on hand-computed values"""
    D = torch.float64
    u = torch.tensor([[1.0], [2.0], [4.0], [8.0]], dtype=D)
    assert O.causal_conv(u, torch.tensor([[100.0, 10.0, 1.0]], dtype=D)).reshape(-1).tolist() == [1.0, 12.0, 124.0, 248.0]
    x = torch.zeros(3, 1, 6, dtype=D)
    x[:, 0, 0], x[:, 0, 5] = 1.0, 7.0
    y = O.rotate_half(x, 4, 1.0)     # pairs (0, 2) and (1, 3); frequencies 1 and 1 / sqrt(1) ** ... = base^(-2 i / 4)
    assert torch.allclose(y[:, 0, 0], torch.cos(torch.arange(3, dtype=D))) and torch.allclose(y[:, 0, 2], torch.sin(torch.arange(3, dtype=D)))
    assert y[:, 0, 5].tolist() == [7.0] * 3 and float(y[:, 0, 1].abs().max()) == 0.0
    assert O.query_temperature(9, 0.5, 4).tolist() == [1.0] * 3 + [1 + 0.5 * math.log(2)] * 4 + [1 + 0.5 * math.log(3)] * 2
    xs = torch.tensor([[[1.0]], [[10.0]]], dtype=D)
    new = O.hyper_write(xs, torch.tensor([[100.0]], dtype=D), torch.tensor([[1.0, 2.0], [3.0, 4.0]], dtype=D), torch.tensor([1.0, -1.0], dtype=D), 0.5)
    assert new.reshape(-1).tolist() == [1 + 30 + 50, 2 + 40 - 50]
    assert float(O.hyper_read(xs, torch.tensor([2.0, 0.5], dtype=D))) == 7.0
    # retention against its closed form o_t = sum_{j <= t} decay^(t - j) (q_t . k_j) v_j
    m = {"heads": 1, "dim": 2, "vdim": 3, "decay": [0.5]}
    g = torch.Generator().manual_seed(0)
    h = torch.randn(5, 4, generator=g, dtype=D)
    w = {"q": torch.randn(2, 4, generator=g, dtype=D), "k": torch.randn(2, 4, generator=g, dtype=D), "v": torch.randn(3, 4, generator=g, dtype=D),
         "g": torch.randn(3, 4, generator=g, dtype=D), "o": torch.eye(3, dtype=D)}
    q, k, v = h @ w["q"].T, (h @ w["k"].T) * 2 ** -0.5, h @ w["v"].T
    o = torch.stack([sum(0.5 ** (t - j) * float(q[t] @ k[j]) * v[j] for j in range(t + 1)) for t in range(5)])
    gate = h @ w["g"].T
    want = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6) * (gate * torch.sigmoid(gate))
    assert torch.allclose(O.retention(h, w, "", m, 1e-6), want, atol=1e-12)


# ---------------------------------------------------------------------------------------------------------------- kernels alone (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("parts,width", [(1, 40), (4, 52), (3, 39)])
def test_unit_norm_with_gate_behind_it(dev, parts, width):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(width)
    x, gate, w = torch.randn(9, width, generator=g) * 3, torch.randn(9, width + 5, generator=g), torch.randn(width, generator=g)
    xd, gd = x.double().view(9, parts, -1), gate[:, :width].double()
    unit = (xd / O.rms(xd, 1e-5)).reshape(9, width)
    out32, out = torch.empty(9, width, device=dev), torch.empty(9, width, device=dev)
    _call("mrs_hyb_rmsnorm", x.to(dev), width, None, out, out32, None, 9, width, parts, 1e-5, 0, 2, gate.to(dev), width + 5, 1)
    assert rel(out32.double().cpu(), unit * gd * torch.sigmoid(gd)) < 2e-6 and rel(out.double().cpu(), out32.double().cpu()) == 0
    _call("mrs_hyb_rmsnorm", x.to(dev), width, None, out, out32, None, 9, width, parts, 1e-5, 0, 2, None, 0, 0)
    assert rel(out32.double().cpu(), unit) < 2e-6
    _call("mrs_hyb_rmsnorm", x.to(dev), width, w.to(dev), out, out32, None, 9, width, parts, 1e-5, 1, 2, None, 0, 0)
    assert rel(out32.double().cpu(), unit * (1 + w.double())) < 2e-6
    # the gate in front of the norm (the other order) is still what it was
    _call("mrs_hyb_rmsnorm", x.to(dev), width, w.to(dev), out, out32, None, 9, width, parts, 1e-5, 0, 2, gate.to(dev), width + 5, 0)
    xg = (x.double() * gd * torch.sigmoid(gd)).view(9, parts, -1)
    assert rel(out32.double().cpu(), (xg / O.rms(xg, 1e-5)).reshape(9, width) * w.double()) < 2e-6


@pytest.mark.gpu
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_convolution_without_activation_carries_biased_rows(dev, taps):
    """three sequences in one batch (one starting, two continuing from their slots), then single rows: against the convolution over each whole sequence"""
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    C, ld = 37, 45
    g = torch.Generator().manual_seed(taps)
    seqs = [torch.randn(n, ld, generator=g) for n in (30, 12, 9)]
    bias, cw = torch.randn(C, generator=g), torch.randn(C, taps, generator=g)
    want = [O.causal_conv(s[:, :C].double() + bias.double(), cw.double()) for s in seqs]
    state = torch.full((5, C, max(taps - 1, 1)), float("nan"), device=dev)      # whatever an earlier owner of the slot left
    got = [[] for _ in seqs]
    at = [0, 0, 0]

    def run(lens, slots=(3, 0, 4)):
        parts = [(k, n) for k, n in enumerate(lens) if n]
        b = _batch(dev, [(at[k], n, slots[k]) for k, n in parts])
        u = torch.cat([seqs[k][at[k]:at[k] + n] for k, n in parts]).to(dev)
        out = torch.empty(u.shape[0], C, device=dev)
        _call("mrs_hyb_conv", u, ld, bias.to(dev), cw.to(dev), None, state, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, out, u.shape[0], len(parts), C, taps, 0)
        r = 0
        for k, n in parts:
            got[k].append(out[r:r + n].double().cpu())
            r += n
            at[k] += n
    run([20, 2, 0])
    run([1, 1, 1])        # one row each: the step kernel
    run([2, 5, 3])
    run([1, 0, 2])
    run([6, 4, 3])
    for k in range(3):
        assert rel(torch.cat(got[k]), want[k]) < 2e-6, k


@pytest.mark.gpu
@pytest.mark.parametrize("heads,D,rot", [(2, 8, 8), (3, 10, 4), (1, 6, 0), (4, 16, 2)])
def test_half_split_rotary_in_place(dev, heads, D, rot):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    n, ld, qc, kc = 13, 3 + 2 * heads * D + 4, 3 + heads * D, 3
    u = torch.randn(n, ld, generator=torch.Generator().manual_seed(D))
    pos = torch.tensor([0, 1, 2, 3, 70, 71, 900, 5, 6, 7, 8, 9, 4000], dtype=torch.int32)
    base = 300.0
    freq = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)] or [0.0], dtype=torch.float64).float()
    d = u.to(dev)
    _call("mrs_hyb_rotary_half", d, ld, qc, kc, heads, D, rot, freq.to(dev), pos.to(dev), 0.3, n)
    got = d.double().cpu()

    def turned(x):
        x = x.double().view(n, heads, D)
        half = rot // 2
        ang = pos.double().view(n, 1, 1) * freq.double()[:half] if rot else None
        if not rot:
            return x
        a, b = x[..., :half], x[..., half:rot]
        return torch.cat([a * torch.cos(ang) - b * torch.sin(ang), b * torch.cos(ang) + a * torch.sin(ang), x[..., rot:]], -1)
    assert (got[:, qc:qc + heads * D] - turned(u[:, qc:qc + heads * D]).reshape(n, -1)).abs().max() < 2e-4      # angles up to 4000 rad in f32
    assert (got[:, kc:kc + heads * D] - 0.3 * turned(u[:, kc:kc + heads * D]).reshape(n, -1)).abs().max() < 2e-4
    assert torch.equal(got[:, :3], u[:, :3].double()) and torch.equal(got[:, qc + heads * D:], u[:, qc + heads * D:].double())


@pytest.mark.gpu
@pytest.mark.parametrize("S,W", [(1, 40), (2, 33), (3, 64), (4, 300), (8, 24)])
def test_stream_write_read_and_norm_in_one_launch(dev, S, W):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(S)
    T = 7
    x, y = torch.randn(T, S, W, generator=g), torch.randn(T, W, generator=g)
    mix, wo, wi, nw = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g), torch.randn(W, generator=g) * 0.3
    xs = x.double().permute(1, 0, 2)
    new = O.hyper_write(xs, y.double(), mix.double(), wo.double(), 1.0)
    d = x.to(dev)
    out, out32 = torch.empty(T, W, device=dev), torch.empty(T, W, device=dev)
    _call("mrs_hyb_hyper_step", d, y.to(dev), mix.to(dev), wo.to(dev), wi.to(dev), nw.to(dev), out, out32, T, S, W, 1e-5, 1, 2)
    assert rel(d.double().cpu().permute(1, 0, 2), new) < 2e-6
    assert rel(out32.double().cpu(), O.norm_one_plus(O.hyper_read(new, wi.double()), nw.double(), 1e-5)) < 3e-6 and torch.equal(out, out32)
    # the streams' start (every stream = out[r] * y), and the closing sum without a norm
    _call("mrs_hyb_hyper_step", d, y.to(dev), None, wo.to(dev), None, None, None, None, T, S, W, 1e-5, 1, 2)
    assert rel(d.double().cpu(), wo.double().view(1, S, 1) * y.double().view(T, 1, W)) < 1e-6
    d = x.to(dev)
    _call("mrs_hyb_hyper_step", d, y.to(dev), mix.to(dev), wo.to(dev), torch.ones(S, device=dev), None, None, out32, T, S, W, 1e-5, 1, 2)
    assert rel(out32.double().cpu(), new.sum(0)) < 2e-6
    # reading alone
    d = x.to(dev)
    _call("mrs_hyb_hyper_step", d, None, None, None, wi.to(dev), nw.to(dev), out, None, T, S, W, 1e-5, 1, 2)
    assert torch.equal(d.cpu(), x) and rel(out.double().cpu(), O.norm_one_plus(O.hyper_read(xs, wi.double()), nw.double(), 1e-5)) < 3e-6


@pytest.mark.gpu
@pytest.mark.parametrize("M", [1, 3, 8, 9, 70, 300])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_per_head_products_in_one_launch(dev, M, dtype):
    """heads as column blocks of one row-major operand, the result rounded once to the operand type"""
    from mistralrs_amd.hybrid import DTYPES, _call
    _lib.load("hybrid")
    code, td = DTYPES[dtype]
    for H, N, K in ((3, 24, 16), (5, 7, 9), (2, 130, 40)):
        g = torch.Generator().manual_seed(M + N)
        a, w = torch.randn(M, H * K, generator=g).to(td), (torch.randn(H, N, K, generator=g) * K ** -0.5).to(td)
        out = torch.full((M, H * N), float("nan"), dtype=td, device=dev)
        _call("mrs_hyb_gemm_batched", a.to(dev), w.to(dev), out, M, N, K, H * K, K, H * N, code, H, K, N * K, N, 1)
        want = torch.einsum("mhk,hnk->mhn", a.double().view(M, H, K), w.double()).reshape(M, H * N)
        assert rel(out.double().cpu(), want) < (3e-6 if dtype == "float32" else 4e-3), (H, N, K)
        out32 = torch.full((M, H * N), float("nan"), device=dev)
        _call("mrs_hyb_gemm_batched", a.to(dev), w.to(dev), out32, M, N, K, H * K, K, H * N, code, H, K, N * K, N, 0)
        assert rel(out32.double().cpu(), want) < 3e-6


@pytest.mark.gpu
def test_latent_rows_are_normed_into_their_pages(dev):
    from mistralrs_amd.hybrid import _call
    H, D, R, bs = 3, 6, 20, 32
    _, _, sv = _model([lat(heads=H, dim=D, vdim=5, rank=R, mlp=None)], dev)
    la = sv.m.layers[0].mixer
    assert sv.cache.reserve(1, 70)
    blocks = sv.cache.kv.get_block_ids(1)
    p0, n = 27, 40
    b = _batch(dev, [(p0, n, 0)], bs, [blocks])
    g = torch.Generator().manual_seed(5)
    u, w = torch.randn(n, H * D + R + 3, generator=g), torch.randn(R, generator=g)
    q = torch.empty(n, H * D, device=dev)
    _call("mrs_hyb_latent_norm_cache", u.to(dev), u.shape[1], H * D, R, w.to(dev), b.slot_mapping, q, la.c_cache, 1e-5, n, 2)
    assert torch.equal(q.cpu(), u[:, :H * D])
    want = O.norm_plain(u[:, H * D:H * D + R].double(), w.double(), 1e-5)
    for i in (0, 4, 5, 39):
        pos = p0 + i
        assert rel(la.c_cache[blocks[pos // bs], 0, pos % bs].double().cpu(), want[i]) < 2e-6
    sv.end(1)


# ---------------------------------------------------------------------------------------------------------------- mixers alone (GPU)
def _alone(layer, dev, dtype, bar, prompt=150, total=180, seed=2, **kw):
    """one layer without a feed-forward: a prompt (tiles of several queries, several passes of 64 keys, several segments of the recurrence), then decoded tokens one by one"""
    cfg, w, sv = _model([layer], dev, dtype, seed=seed, **kw)
    t = toks(total, cfg["vocab"], 9)
    want = O.forward(cfg, f64(w), t)
    got = sv.step([(1, t[:prompt])])[0]
    assert close(got, want[:prompt], bar)
    got = torch.cat([sv.step([(1, [t[i]])])[0] for i in range(prompt, total)])
    assert close(got, want[prompt:], bar)


ATTN_SHAPES = [dict(), dict(heads=3, kv_heads=3, dim=10, vdim=7, conv=2, every=3), dict(heads=6, kv_heads=2, dim=24, vdim=40, conv=5, cap=2.0, every=50),
               dict(heads=2, kv_heads=1, dim=8, vdim=4, conv=0, cap=0.0, coef=0.0), dict(heads=8, kv_heads=4, dim=16, vdim=160, cap=0.5), dict(heads=5, kv_heads=1, dim=9, vdim=3, every=1),
               dict(heads=4, kv_heads=4, dim=32, vdim=130, conv=1), dict(heads=2, kv_heads=2, dim=8, vdim=300, conv=0)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", ATTN_SHAPES, ids=lambda s: "-".join(f"{k}{v}" for k, v in s.items()) or "default")
@pytest.mark.parametrize("dtype,bar", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_sink_attention_alone(dev, shape, dtype, bar):
    _alone(attn(mlp=None, **shape), dev, dtype, bar)


RET_SHAPES = [dict(), dict(heads=3, dim=10, vdim=7, decay=(0.25, 0.9, 1.0), dims=10), dict(heads=1, dim=32, vdim=24, decay=(0.99609375,), dims=8, base=2e5),
              dict(heads=4, dim=4, vdim=130, decay=(0.5, 0.75, 0.875, 0.9375), dims=0), dict(heads=2, dim=72, vdim=8, dims=2), dict(heads=2, dim=136, vdim=16, dims=136)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", RET_SHAPES, ids=lambda s: "-".join(f"{k}{v}" for k, v in s.items() if k != "decay") or "default")
@pytest.mark.parametrize("dtype,bar", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_retention_alone(dev, shape, dtype, bar):
    _alone(ret(**shape), dev, dtype, bar, prompt=200, total=230)


LAT_SHAPES = [dict(), dict(heads=1, dim=8, vdim=8, rank=8), dict(heads=5, dim=10, vdim=7, rank=13), dict(heads=2, dim=24, vdim=40, rank=136), dict(heads=2, dim=16, vdim=8, rank=264),
              dict(heads=8, dim=32, vdim=16, rank=64)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", LAT_SHAPES, ids=lambda s: "-".join(f"{k}{v}" for k, v in s.items()) or "default")
@pytest.mark.parametrize("dtype,bar", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_latent_attention_alone(dev, shape, dtype, bar):
    _alone(lat(mlp=None, **shape), dev, dtype, bar)


@pytest.mark.gpu
@pytest.mark.parametrize("ff", [56, 9, 300, 1])
def test_feed_forward_alone(dev, ff):
    """a retention layer that forgets at once (decay 0) in front, so every row depends on its own token only: 70 rows at once (tile products) and 1 - 3 rows (the streamed
    products of decode steps, the GLU in their operand load)"""
    cfg, w, sv = _model([ret(heads=1, decay=(0.0,), dims=0, mlp=glu(ff))], dev, seed=4)
    t = toks(70, cfg["vocab"], 10)
    want = O.forward(cfg, f64(w), t)
    assert rel(sv.step([(1, t)])[0], want) < 2e-5
    sv.end(1)
    assert rel(sv.step([(2, t[:1])])[0], want[:1]) < 2e-5
    got = torch.cat(sv.step([(2, [t[1]]), (3, [t[0]]), (4, [t[0]])]))
    assert rel(got, torch.stack([want[1], want[0], want[0]])) < 2e-5


# ---------------------------------------------------------------------------------------------------------------- planted keys and states (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_planted_keys_sink_and_cap(dev, dtype):
    """The attention kernel with hand-made pages.  One key scores far above the rest, so whether the kernel sees it decides the output: the query itself, the first token, both
    sides of a page border and of a pass of 64 keys, a key hundreds of tokens back, a key one step in the future (never seen) -- for prompt tiles and single decoded rows.
    Then the sink: with every score far below zero the output vanishes (without the sink it is the mean of the values); and the cap: scores of 30 and 60 under a cap of 2
    weigh almost alike."""
    from mistralrs_amd.hybrid import _call
    H, G, D, Dv, bs, T = 2, 1, 8, 4, 32, 300
    _, _, sv = _model([attn(heads=H, kv_heads=G, dim=D, vdim=Dv, mlp=None)], dev, dtype)
    m, td = sv.m, sv.m.torch_dtype
    att = m.layers[0].mixer
    assert sv.cache.reserve(1, T)
    blocks = sv.cache.kv.get_block_ids(1)
    g = torch.Generator().manual_seed(11)
    v = torch.randn(T, G, Dv, generator=g).to(torch.bfloat16)
    blk, off = torch.tensor([blocks[t // bs] for t in range(T)], device=dev), torch.arange(T, device=dev) % bs
    att.v_cache[blk, :, off] = v.to(dev, td)
    tol = 1e-4 if dtype == "float32" else 2e-2

    def run(i, k, q, rows, cap=0.0, sink=1, gate=None, splits=0):
        att.k_cache[blk, :, off] = k.to(dev, td)
        p0 = i if rows == "decode" else max(0, i - 20)
        n = i - p0 + 1
        b = _batch(dev, [(p0, n, 0)], bs, [blocks])
        qq = torch.zeros(n, H * D, dtype=td, device=dev)
        qq[n - 1] = q.reshape(-1).to(dev, td)
        out = torch.empty(n, H * Dv, dtype=td, device=dev)
        if rows == "decode" and not splits:
            splits = 1 + (i + j0) % 6                         # the keys dealt to several workgroups (some of them without a share), or all to one
        scratch = torch.full((max(splits, 1), n, H, Dv + 2), float("nan"), device=dev) if splits > 1 else None
        _call("mrs_hyb_paged_attn_opts", qq, att.k_cache, att.v_cache, b.block_tables, b.tok_seq, b.tok_pos, out, n, H, G, D, Dv, bs, b.max_blocks, 0, 0, 1.0, m.dt,
              b.seg_entry, b.seg_row0, b.seg_len, b.segments, 64, cap, sink, gate, H * Dv if gate is not None else 0, scratch, splits if splits > 1 else 0, 0)
        return out[n - 1].double().cpu().view(H, Dv)
    j0 = 0
    for i in (60, 64, 95, 96, 299):
        for j in (0, i, 31, 32, i - 1, i - 63, i - 64, i - 65, i + 1, 3):
            if j < 0 or j >= T:
                continue
            k = torch.randn(T, G, D, generator=g).to(torch.bfloat16) * 0.05
            k[j, 0, 0] = 6.0
            q = torch.zeros(H, D, dtype=torch.bfloat16)
            q[1, 0] = 6.0                                    # head 1 asks for key j; head 0 asks for nothing and averages what it sees with the sink
            j0 = j
            for rows in ("decode", "prompt"):
                got = run(i, k, q, rows)
                if j <= i:
                    assert float((got[1] - v[j, 0].double()).abs().max()) < tol, (i, j, rows)
                else:
                    assert float((got[1] - v[j, 0].double()).abs().max()) > 0.1, (i, j, rows)
                assert float((got[0] - v[:i + 1, 0].double().sum(0) / (i + 2)).abs().max()) < tol, (i, j, rows)
    k = torch.zeros(T, G, D, dtype=torch.bfloat16)
    k[:, 0, 0] = -5.0
    q = torch.zeros(H, D, dtype=torch.bfloat16)
    q[:, 0] = 6.0
    for rows in ("decode", "prompt"):
        assert float(run(100, k, q, rows).abs().max()) < 1e-6                                                      # the sink takes all the weight
        assert float((run(100, k, q, rows, sink=0)[0] - v[:101, 0].double().mean(0)).abs().max()) < tol            # without it: the mean
    k = torch.zeros(T, G, D, dtype=torch.bfloat16)
    k[:, 0, 0] = -6.0
    k[7, 0, 0], k[90, 0, 0] = 5.0, 10.0
    e = [math.exp(2 * math.tanh(s / 2)) for s in (30.0, 60.0, -36.0)]
    den = 1 + e[0] + e[1] + 99 * e[2]
    want = (e[0] * v[7, 0].double() + e[1] * v[90, 0].double() + e[2] * (v[:101, 0].double().sum(0) - v[7, 0].double() - v[90, 0].double())) / den
    gate = torch.randn(1, H * Dv, generator=g)
    for rows in ("decode", "prompt"):
        assert float((run(100, k, q, rows, cap=2.0)[0] - want).abs().max()) < tol
        n = 1 if rows == "decode" else 21
        gd = torch.zeros(n, H * Dv)
        gd[n - 1] = gate[0]
        got = run(100, k, q, rows, cap=2.0, gate=gd.to(dev))
        assert float((got[0] - want * torch.sigmoid(gate[0, :Dv].double())).abs().max()) < tol
    sv.end(1)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_decoding_with_the_keys_dealt_to_several_workgroups(dev, dtype, bar, monkeypatch):
    """single-row steps over a few hundred keys with a small share per workgroup: three sequences of unequal length in one step (the shortest leaves most workgroups without
    keys), against the restatement; and the same step without the split"""
    from mistralrs_amd.hybrid import HybridDecoder
    cfg = config([attn(), lat(), attn(kv_from=0, conv=0), lat(heads=2, dim=8, vdim=8, rank=136, mlp=None)])
    w = weights(cfg, 31)
    wd = f64(w)
    req = {1: toks(330, cfg["vocab"], 81), 2: toks(70, cfg["vocab"], 82), 3: toks(9, cfg["vocab"], 83)}
    full = {r: O.forward(cfg, wd, t) for r, t in req.items()}
    for per in (64, 10 ** 9):
        monkeypatch.setattr(HybridDecoder, "KEYS_PER_SPLIT", per)
        sv = Served(cfg, w, dev, dtype, max_tokens=512)
        sv.step([(r, t[:-8]) for r, t in req.items()])
        assert (sv.m.key_splits(_batch(dev, [(320, 1, 0)]), 4, 8)[1] > 1) == (per == 64)
        for i in range(8):
            outs = sv.step([(r, [t[len(t) - 8 + i]]) for r, t in req.items()])
            for (r, t), o in zip(req.items(), outs):
                assert close(o, full[r][len(t) - 8 + i:len(t) - 7 + i], bar), (per, r, i)


@pytest.mark.gpu
def test_latent_attention_finds_a_far_row(dev):
    """the whole mixer: one token's latent row is made to stand out for one head by scaling one row of the key expansion and the matching query weights; the head's output then is that
    token's value (hundreds of tokens back, over page borders), in a prompt and in decoded rows"""
    cfg = config([lat(heads=2, dim=8, vdim=8, rank=16, mlp=None, scale=1.0)], streams=0, mult=1.0)
    w = weights(cfg, 21)
    w["l0.mix.q"] = (w["l0.mix.q"].float() * 6).to(torch.bfloat16)
    w["l0.mix.uk"] = (w["l0.mix.uk"].float() * 4).to(torch.bfloat16)
    t = toks(300, cfg["vocab"], 22)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    got = sv.step([(1, t[:270])]) + [sv.step([(1, [x])])[0] for x in t[270:]]
    assert rel(torch.cat(got), want) < 3e-5
    # the softmax is sharp here: most rows put nearly all weight on one key, often far back
    h = O.norm_one_plus(O.norm_one_plus(f64(w)["embed"][torch.tensor(t)], f64(w)["embed.norm"], 1e-5), f64(w)["l0.norm1"], 1e-5)
    c = O.norm_plain(h @ f64(w)["l0.mix.dkv"].T, f64(w)["l0.mix.dkv.norm"], 1e-5)
    s = ((h @ f64(w)["l0.mix.q"].T)[:, :8] @ (c @ f64(w)["l0.mix.uk"].T)[:, :8].T).tril() + torch.full((300, 300), -1e9, dtype=torch.float64).triu(1)
    p = torch.softmax(s, -1)
    far = (p.argmax(-1) < torch.arange(300) - 100) & (p.max(-1).values > 0.5)
    assert int(far.sum()) >= 3


@pytest.mark.gpu
def test_retention_keeps_a_planted_token_for_hundreds_of_steps(dev):
    """the scan kernel with hand-made rows: key e_0 with value u at one row, nothing elsewhere; a later query e_0 reads decay^(distance) u -- over segment borders (64 rows), over
    portions cut at 63 / 64 / 65 / 2 rows, from a slot that another sequence used before, and in single decoded rows"""
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    H, N, P = 2, 8, 4
    ld = H * P + 2 * H * N
    dec = torch.tensor([0.99609375, 0.5])
    state = torch.full((3, H, N, P), float("nan"), device=dev)
    state[1] = 1e6                                          # the slot's former owner; a sequence that starts must not read it
    uval = torch.tensor([1.0, -2.0, 3.0, 0.5], dtype=torch.float64)
    T, plant = 400, 5
    rows = torch.zeros(T, ld)
    rows[plant, :P] = uval.float()                          # v of head 0
    rows[plant, H * P] = 1.0                                # k of head 0 = e_0
    rows[:, H * P + H * N] = 1.0                            # every q of head 0 = e_0
    rows[:, P:2 * P] = 1.0                                  # head 1: v = 1, k = q = e_0 everywhere: o = sum of 0.5^d = 2 - 0.5^t
    rows[:, H * P + N] = 1.0
    rows[:, H * P + H * N + N] = 1.0
    at, outs = 0, []
    for n in (63, 1, 64, 2, 65, 1, 1, 130, 3, 70):
        b = _batch(dev, [(at, n, 1)])
        y = torch.empty(n, H * P, device=dev)
        steps = torch.empty(n, H, 2, device=dev)
        carry = torch.empty(b.segments, H, N, P, device=dev)
        dk = torch.empty(b.segments, H, device=dev)
        _call("mrs_hyb_decay_scan", rows[at:at + n].to(dev), ld, dec.to(dev), state, y, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0, steps, carry, dk,
              n, 1, b.segments, H, P, N, H)
        outs.append(y.double().cpu())
        at += n
    assert at == T
    y = torch.cat(outs)
    t = torch.arange(T, dtype=torch.float64)
    want0 = torch.where(t >= plant, 0.99609375 ** (t - plant), torch.zeros_like(t)).view(T, 1) * uval
    assert float((y[:, :P] - want0).abs().max()) < 1e-5 and float(want0[-1].abs().max()) > 0.2
    assert float((y[:, P:] - (2 - 0.5 ** t).view(T, 1)).abs().max()) < 1e-5
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()


@pytest.mark.gpu
def test_first_tokens_see_zeros_not_the_slots_former_owner(dev):
    """two slots, four requests one after the other: convolution taps and retention states of finished requests stay in the slots; a new request's first tokens must not read them"""
    cfg = config([attn(conv=4), ret(mlp="glu"), attn(kv_from=0, conv=2)])
    w = weights(cfg, 23)
    sv = Served(cfg, w, dev, max_tokens=128, slots=2)
    wd = f64(w)
    for r in range(1, 5):
        t = toks(40 + r, cfg["vocab"], 30 + r)
        want = O.forward(cfg, wd, t)
        got = sv.step([(r, t[:1])]) + sv.step([(r, t[1:3])]) + sv.step([(r, t[3:])])
        assert rel(torch.cat(got), want) < 3e-5, r
        sv.end(r)


# ---------------------------------------------------------------------------------------------------------------- whole models (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
@pytest.mark.parametrize("streams,mult", [(3, 0.4), (1, 0.7), (0, 0.6), (0, None)], ids=["streams3", "streams1", "scaled", "plain"])
def test_whole_prompt_every_layer(dev, dtype, bar, streams, mult):
    cfg = config(STACK, streams=streams, mult=mult)
    w = weights(cfg, 5)
    sv = Served(cfg, w, dev, dtype)
    t = toks(150, cfg["vocab"], 14)
    lo = []
    want = O.forward(cfg, f64(w), t, lo)
    sv.m.trace_layers = []
    got = sv.step([(1, t)])[0]
    assert len(sv.m.trace_layers) == len(lo)
    for i, (a, b) in enumerate(zip(sv.m.trace_layers, lo)):
        assert close(a.double().cpu(), b, bar), f"residual stream after layer {i}"
    assert close(got, want, bar)


@pytest.mark.gpu
def test_portions_and_decoding_equal_the_whole_prompt(dev):
    """the same 200 tokens: whole; in portions of changing sizes down to two tokens and single tokens; token by token from the start"""
    cfg = config(STACK)
    w = weights(cfg, 6)
    t = toks(200, cfg["vocab"], 15)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    assert rel(sv.step([(1, t)])[0], want) < 3e-5
    cuts = [2, 3, 1, 64, 2, 31, 1, 1, 65, 7, 2, 21]
    assert sum(cuts) == 200
    got, at = [], 0
    for c in cuts:
        got += sv.step([(2, t[at:at + c])])
        at += c
    assert rel(torch.cat(got), want) < 3e-5
    got = [sv.step([(3, [x])])[0] for x in t[:80]]
    assert rel(torch.cat(got), want[:80]) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_mixed_batches_with_reused_pages_and_slots(dev, dtype, bar):
    """five requests of unequal length through a pool of 192 tokens and three slots: portions beside single tokens, a request left out of a step, pages and slots of finished
    requests taken by later ones -- every row against the request alone in the restatement"""
    cfg = config(STACK)
    w = weights(cfg, 7)
    wd = f64(w)
    sv = Served(cfg, w, dev, dtype, max_tokens=192, slots=3)
    req = {r: toks(n, cfg["vocab"], 20 + r) for r, n in ((1, 70), (2, 9), (3, 64), (4, 33), (5, 90))}
    full = {r: O.forward(cfg, wd, t) for r, t in req.items()}
    plan = [[(1, 40), (2, 1)], [(1, 1), (2, 3), (3, 33)], [(2, 5), (3, 1)], [(1, 29), (3, 30)], [(4, 2), (3, 0)], [(4, 31), (5, 60)], [(5, 1), (4, 0)], [(5, 29)]]
    at = {r: 0 for r in req}
    for step in plan:
        parts = [(r, req[r][at[r]:at[r] + n]) for r, n in step if n]
        outs = sv.step(parts)
        for (r, tk), o in zip(parts, outs):
            assert close(o, full[r][at[r]:at[r] + len(tk)], bar), (r, at[r])
            at[r] += len(tk)
            if at[r] == len(req[r]):
                sv.end(r)
    assert at == {r: len(t) for r, t in req.items()}


@pytest.mark.gpu
def test_long_decoding_past_temperature_steps_and_slow_decays(dev):
    cfg = config([attn(every=11, conv=4), ret(decay=(0.9990234375, 0.9), dims=8, base=1e4, mlp="glu"), lat(), attn(kv_from=0, every=64, conv=2)])
    w = weights(cfg, 8)
    t = toks(260, cfg["vocab"], 16)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev)
    got = sv.step([(1, t[:5])]) + [sv.step([(1, [x])])[0] for x in t[5:]]
    assert rel(torch.cat(got), want) < 3e-5


@pytest.mark.gpu
def test_sizes_that_coincide_or_equal_one(dev):
    """one stream, one head, one tap, a latent as wide as the model, key and value sizes equal to the width, a temperature step at every token, rotation over the whole head,
    a multiplier of one, one-token prompts"""
    for layers, kw in (([attn(heads=1, kv_heads=1, dim=24, vdim=24, conv=1, every=1, mlp=glu(24)), lat(heads=1, dim=24, vdim=24, rank=24, mlp=glu(24)),
                         ret(heads=1, dim=24, vdim=24, decay=(1.0,), dims=24, mlp="glu")], dict(width=24, vocab=24, streams=1, mult=1.0)),
                       ([attn(heads=2, kv_heads=2, dim=2, vdim=1, conv=2, every=2, mlp=glu(1)), attn(heads=2, kv_heads=2, dim=2, vdim=1, kv_from=0, mlp=None), ret(heads=1, dim=2, vdim=1, decay=(0.5,), dims=2),
                         lat(heads=1, dim=1, vdim=1, rank=1, mlp=None)], dict(width=8, vocab=5, streams=2, mult=0.5))):
        cfg = config(layers, **kw)
        w = weights(cfg, 9)
        t = toks(40, cfg["vocab"], 17)
        want = O.forward(cfg, f64(w), t)
        sv = Served(cfg, w, dev)
        assert rel(sv.step([(1, t[:1])])[0], want[:1]) < 3e-5
        got = sv.step([(2, t[:1])]) + sv.step([(2, t[1:3])]) + sv.step([(2, t[3:])])
        assert rel(torch.cat(got), want) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 5e-2)])
def test_sizes_off_every_vector_width(dev, dtype, bar):
    """width, vocabulary, head sizes, ranks and feed-forward sizes that no 16-byte load divides: the element-wise paths of every kernel, prompt and decode"""
    cfg = config([attn(heads=3, kv_heads=1, dim=11, vdim=13, conv=3, every=7, mlp=glu(27)), lat(heads=3, dim=7, vdim=5, rank=11, mlp=glu(15)), ret(heads=3, dim=6, vdim=9, decay=(0.9, 0.8, 0.7), dims=4),
                  attn(heads=3, kv_heads=1, dim=11, vdim=13, conv=5, kv_from=0, mlp=None)], vocab=77, width=50, streams=5)
    w = weights(cfg, 13)
    t = toks(100, cfg["vocab"], 18)
    want = O.forward(cfg, f64(w), t)
    sv = Served(cfg, w, dev, dtype)
    got = sv.step([(1, t[:67])]) + sv.step([(1, t[67:90])]) + [sv.step([(1, [x])])[0] for x in t[90:]]
    assert close(torch.cat(got), want, bar)


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_greedy_generation_through_scheduler_and_engine(dev, graphs):
    """the package's own entry point: scheduler (pages + slots), engine, sampler; five prompts through three slots, against greedy decoding of the restatement"""
    from mistralrs_amd.cli import make_engine
    from mistralrs_amd.hybrid import HybridDecoder, setopel_spec
    from mistralrs_amd.sampler import SequenceSampler
    from mistralrs_amd.scheduler import Sequence
    cfg = config([lat(), attn(), ret(mlp="glu"), attn(kv_from=1, mlp=None)])
    w = weights(cfg, 10)
    m = HybridDecoder(setopel_spec(cfg), dev, "float32", num_blocks=12, block_size=32, state_slots=3)
    m.load_weights(w.__getitem__)
    assert m.has_recurrent_state and m.has_paged_kv
    core = os.path.exists(_lib.path("core"))
    eng = make_engine(m, 12 * 32, 3, sampler=SequenceSampler(cfg["vocab"], dev, top_k=1) if core else None, max_batched_tokens=48, use_graphs=graphs)
    prompts = [toks(n, cfg["vocab"], 30 + n) for n in (5, 40, 1, 23, 60)]
    seqs = [Sequence(id=i + 1, tokens=list(p), max_new_tokens=6) for i, p in enumerate(prompts)]
    for s in seqs:
        eng.s.add_seq(s)
    eng.run()
    wd = f64(w)
    for p, s in zip(prompts, seqs):
        ref = list(p)
        for _ in range(6):
            lg = O.forward(cfg, wd, ref)[-1]
            top2 = torch.topk(lg, 2).values
            if float(top2[0] - top2[1]) < 1e-3:
                break  # a tie within rounding: the comparison stops here
            ref.append(int(lg.argmax()))
        assert s.error is None and s.generated[:len(ref) - len(p)] == ref[len(p):], (s.id, s.generated, ref[len(p):])
    assert eng.steps["prompt"] >= 2 and eng.steps["completion"] >= 6 and bool(eng._graphs) == graphs


@pytest.mark.gpu
def test_captured_decode_steps_equal_eager_steps(dev):
    """a HIP graph of one decode step for three sequences, captured while two of them are live: every replay (eager work and synchronisation between replays) against the
    eager step function on a second copy of the model, and the pages and slots the warm-up touched are intact"""
    cfg = config(STACK)
    w = weights(cfg, 11)
    a, b = Served(cfg, w, dev), Served(cfg, w, dev)
    prompts = {1: toks(37, cfg["vocab"], 41), 2: toks(3, cfg["vocab"], 42), 3: toks(64, cfg["vocab"], 43)}
    for sv in (a, b):
        sv.step([(1, prompts[1]), (2, prompts[2])])
    g = a.m.capture_decode(3, 8)
    for sv in (a, b):
        sv.step([(3, prompts[3])])
    nxt = {r: toks(12, cfg["vocab"], 50 + r) for r in prompts}
    for i in range(12):
        parts = [(r, [nxt[r][i]]) for r in (1, 2, 3)]
        want = torch.cat(b.step(parts))
        entries = []
        for r, tk in parts:
            assert a.cache.reserve(r, a.len[r] + 1)
            entries.append(a.cache.entry(r, tk, a.len[r]))
            a.len[r] += 1
        got = g.replay(entries).double().cpu()
        assert rel(got, want) < 1e-6, f"replay {i}"
        torch.cuda.synchronize()


@pytest.mark.gpu
def test_checkpoint_folder_through_registry_command_line_and_trace_replay(dev, tmp_path, monkeypatch, capsys):
    """config.json + model.safetensors on disk -> registry -> `trace` (steps from standard input, logits to files, pages and slots given back and reused) and `generate`
    (scheduler, engine, sampler) -- both against the restatement"""
    from safetensors.torch import save_file
    from mistralrs_amd import cli, registry, trace
    cfg = config([attn(), lat(mlp=None), ret(mlp="glu"), attn(kv_from=0)])
    w = weights(cfg, 12)
    folder = tmp_path / "model"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(folder / "model.safetensors"))
    assert registry.architecture_of(str(folder)) == "Setopel"
    wd = f64(w)
    reqs = {"a": toks(45, cfg["vocab"], 61), "b": toks(20, cfg["vocab"], 62), "c": toks(33, cfg["vocab"], 63)}
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": reqs["a"][:30], "want": [0, 29]}, {"id": "b", "tokens": reqs["b"][:19], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": reqs["a"][30:31], "want": [0]}, {"id": "b", "tokens": reqs["b"][19:], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "c", "tokens": reqs["c"][:2], "want": [1]}, {"id": "a", "tokens": reqs["a"][31:], "want": [13]}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "c", "tokens": reqs["c"][2:], "want": [0, 30]}], "end": ["c"]}]
    out = tmp_path / "out"
    monkeypatch.setattr("sys.stdin", io.StringIO("\n".join(json.dumps(s) for s in steps) + "\n"))
    assert trace.main(["--model", str(folder), "--dtype", "float32", "--out", str(out), "--max-tokens", "128", "--state-slots", "2"]) == 0
    printed = capsys.readouterr().out.split("\n")
    assert [l for l in printed if l.startswith("done")] == [f"done {i}" for i in range(4)]
    full = {r: O.forward(cfg, wd, t) for r, t in reqs.items()}
    want = {0: [full["a"][0], full["a"][29]], 1: [full["a"][30], full["b"][19]], 2: [full["c"][1], full["a"][44]], 3: [full["c"][2], full["c"][32]]}
    for n, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"]).astype(np.float64))
        assert rel(got, torch.stack(rows)) < 3e-5, f"step {n}"
    if not os.path.exists(_lib.path("core")):
        pytest.skip("the sampler's library is not built")
    prompts = [toks(12, cfg["vocab"], 71), toks(3, cfg["vocab"], 72)]
    args = ["generate", "--model", str(folder), "--dtype", "float32", "--max-new-tokens", "4", "--max-tokens", "256", "--max-seqs", "2"]
    for p in prompts:
        args += ["--prompt-ids", ",".join(map(str, p))]
    assert cli.main(args) == 0
    lines = [json.loads(l) for l in capsys.readouterr().out.split("\n") if l.startswith("{")]
    assert len(lines) == 2
    for p, line in zip(prompts, lines):
        ref = list(p)
        for _ in range(4):
            lg = O.forward(cfg, wd, ref)[-1]
            t2 = torch.topk(lg, 2).values
            if float(t2[0] - t2[1]) < 1e-3:
                break
            ref.append(int(lg.argmax()))
        assert line["error"] is None and line["tokens"][:len(ref) - len(p)] == ref[len(p):]
