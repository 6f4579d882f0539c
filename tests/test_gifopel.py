"""Gifopel decoders (mistralrs_amd.hybrid: paired norms, DeltaRuleMixer, MlstmMixer, ParallelMixer over chunked sink attention and a delta rule, TopkSoftmaxReluSqMoe, layers that
borrow another layer's tensors, the tied head; csrc/hyb_recur.hip and the options added to csrc/hyb_kernels.hip / hyb_gemm.hip) against the plain float64 restatement in
tests/gifopel_oracle.py.

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
from tests import gifopel_oracle as O

D64 = torch.float64


# ---------------------------------------------------------------------------------------------------------------- configurations and weights
def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=24):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def _ff(mlp):
    return moe() if mlp == "moe" else dense() if mlp == "dense" else mlp


def cdelta(heads=4, kv_heads=2, dim=16, vdim=8, conv=3, mlp="moe", weights_of=None):
    L = {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": _ff(mlp)}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def mlstm(heads=2, dim=12, vdim=16, cap=9.0, mlp="dense", weights_of=None):
    L = {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": _ff(mlp)}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def par(heads=4, kv_heads=2, dim=16, vdim=8, size=24, dims=8, base=300.0, scale=None, rheads=2, rkv=1, rdim=8, rvdim=12, rconv=4, mlp="moe", weights_of=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if size:
        left["mask"] = {"size": size}
    if dims:
        left["rot"] = {"dims": dims, "base": base}
    L = {"type": "parallel", "mixer": {"left": left, "right": {"heads": rheads, "kv_heads": rkv, "dim": rdim, "vdim": rvdim, "conv": rconv}}, "mlp": _ff(mlp)}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def config(layers, vocab=96, width=40, eps=1e-5):
    return {"architecture": "Gifopel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def weights(cfg, seed=0, rank=5, slow=False):
    """slow: decays close to one and forget gates close to open, so that a state written early is still read hundreds of tokens later"""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def rnd(*shape, scale=1.0, shift=0.0):
        return (torch.randn(*shape, generator=g) * scale + shift).to(torch.bfloat16)

    def delta(p, m, channel):
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for n, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
            w[p + n], w[p + n + ".conv"] = rnd(rows, W, scale=1.5 * W ** -0.5), rnd(rows, m["conv"], scale=0.6)
        w[p + "b"], w[p + "A_log"], w[p + "norm"] = rnd(H, W, scale=2 * W ** -0.5), rnd(H, scale=0.5, shift=-5.0 if slow else 0.0), rnd(Dv, scale=0.2, shift=1.0)
        if channel:
            w[p + "a1"], w[p + "a2"], w[p + "dt_bias"] = rnd(rank, W, scale=W ** -0.5), rnd(H * D, rank, scale=rank ** -0.5), rnd(H * D, scale=0.5, shift=-1.0)
            w[p + "g1"], w[p + "g2"] = rnd(rank + 1, W, scale=W ** -0.5), rnd(H * Dv, rank + 1, scale=2 * (rank + 1) ** -0.5)
        else:
            w[p + "a"], w[p + "dt_bias"], w[p + "g"] = rnd(H, W, scale=W ** -0.5), rnd(H, scale=0.5, shift=-1.0), rnd(H * Dv, W, scale=2 * W ** -0.5)
        w[p + "o"] = rnd(W, H * Dv, scale=(H * Dv) ** -0.5)
    w["embed"], w["final.norm"] = rnd(cfg["vocab"], W), rnd(W, scale=0.2, shift=1.0)
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", L["mixer"]
        w[p + "norm1"] = rnd(W, scale=0.2, shift=1.0)
        if L["type"] == "channel_delta":
            delta(p + "mix.", m, True)
        elif L["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            q = p + "mix."
            w[q + "q"], w[q + "k"], w[q + "v"] = rnd(H * D, W, scale=2 * W ** -0.5), rnd(H * D, W, scale=2 * W ** -0.5), rnd(H * Dv, W, scale=W ** -0.5)
            w[q + "g"], w[q + "o"], w[q + "norm"] = rnd(H * Dv, W, scale=2 * W ** -0.5), rnd(W, H * Dv, scale=(H * Dv) ** -0.5), rnd(H * Dv, scale=0.2, shift=1.0)
            w[q + "i"], w[q + "i.b"] = rnd(H, W, scale=3 * W ** -0.5), rnd(H, scale=0.5)
            w[q + "f"], w[q + "f.b"] = rnd(H, W, scale=3 * W ** -0.5), rnd(H, scale=0.5, shift=6.0 if slow else 2.0)
        else:
            l, q = m["left"], p + "mix.left."
            H, G, D, Dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            w[q + "q"], w[q + "k"], w[q + "v"] = rnd(H * D, W, scale=2 * W ** -0.5), rnd(G * D, W, scale=2 * W ** -0.5), rnd(G * Dv, W, scale=W ** -0.5)
            w[q + "q.norm"], w[q + "k.norm"] = rnd(D, scale=0.3, shift=1.5), rnd(D, scale=0.3, shift=1.5)
            w[q + "sink"], w[q + "g"], w[q + "o"] = rnd(H, scale=1.0, shift=0.5), rnd(H, W, scale=2 * W ** -0.5), rnd(W, H * Dv, scale=(H * Dv) ** -0.5)
            delta(p + "mix.right.", m["right"], False)
            w[p + "mix.left.out"], w[p + "mix.right.out"] = rnd(W, scale=0.2, shift=1.0), rnd(W, scale=0.2, shift=1.0)
        f = L.get("mlp")
        if f:
            w[p + "norm2"] = rnd(W, scale=0.2, shift=1.0)
            if f["kind"] == "dense":
                w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = rnd(f["ff"], W, scale=2 * W ** -0.5), rnd(f["ff"], W, scale=2 * W ** -0.5), rnd(W, f["ff"], scale=f["ff"] ** -0.5)
            else:
                E, ff = f["router"]["experts"], f["expert"]["ff"]
                w[p + "mlp.router"], w[p + "mlp.router.b"] = rnd(E, W, scale=3 * W ** -0.5), rnd(E, scale=0.5)
                for e in range(E):
                    w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = rnd(ff, W, scale=2 * W ** -0.5), rnd(W, ff, scale=ff ** -0.5)
    return w


def f64(w):
    return {k: v.to(D64) for k, v in w.items()}


STACK = [mlstm(), par(), cdelta(), mlstm(heads=3, dim=8, vdim=8, cap=4.0, mlp="moe"), par(heads=6, kv_heads=3, dim=8, vdim=12, size=9, dims=4, rheads=4, rkv=4, rdim=12, rvdim=4, rconv=2, mlp=None),
         cdelta(weights_of=2), par(weights_of=1), cdelta(heads=2, kv_heads=2, dim=8, vdim=20, conv=5, mlp=dense(30))]


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


def logits_of(cfg, wd, t):
    return O.forward(cfg, wd, t)[0]


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
    from mistralrs_amd.hybrid import AttentionSpec, DeltaRuleSpec, GluSpec, MlstmSpec, ParallelSpec, TopkSoftmaxMoeSpec, gifopel_spec
    cfg = config([par(heads=6, kv_heads=3, dim=10, vdim=14, size=17, dims=6, base=77.0, scale=0.3, rheads=4, rkv=2, rdim=6, rvdim=10, rconv=5, mlp=moe(9, 3, 21)),
                  mlstm(heads=5, dim=6, vdim=7, cap=3.5, mlp=dense(77)), cdelta(heads=6, kv_heads=2, dim=4, vdim=6, conv=2, mlp=None), par(size=0, dims=0, mlp=None),
                  cdelta(heads=6, kv_heads=2, dim=4, vdim=6, conv=2, mlp=None, weights_of=2)], vocab=123, width=56, eps=3e-4)
    sp = gifopel_spec(cfg)
    assert (sp.vocab, sp.width, sp.eps, sp.norm, sp.parallel_sublayers, sp.head, sp.embed, sp.post_norms, sp.streams) == (123, 56, 3e-4, "rms", True, "embed", "embed", False, 0)
    a, b, c, d, e = sp.layers
    assert [l.kind for l in sp.layers] == ["parallel", "mlstm", "delta_rule", "parallel", "delta_rule"]
    assert isinstance(a.mixer, ParallelSpec) and isinstance(a.mixer.left, AttentionSpec) and isinstance(a.mixer.right, DeltaRuleSpec) and isinstance(b.mixer, MlstmSpec)
    l, r = a.mixer.left, a.mixer.right
    assert (a.mixer.left_kind, a.mixer.right_kind) == ("attention", "delta_rule")
    assert (l.heads, l.kv_heads, l.dim, l.vdim, l.scale, l.window, l.keep_first, l.chunk, l.head_norm, l.sink, l.head_gate, l.rotary.dims, l.rotary.base, l.rotary.layout) == \
        (6, 3, 10, 14, 0.3, 0, 0, 17, True, True, True, 6, 77.0, "interleaved")
    assert (r.heads, r.kv_heads, r.dim, r.vdim, r.conv, r.decay, r.gate) == (4, 2, 6, 10, 5, "head", "silu")
    assert isinstance(a.ff, TopkSoftmaxMoeSpec) and (a.ff.experts, a.ff.top, a.ff.ff) == (9, 3, 21)
    assert (b.mixer.heads, b.mixer.dim, b.mixer.vdim, b.mixer.gate_cap) == (5, 6, 7, 3.5) and isinstance(b.ff, GluSpec) and b.ff.ff == 77
    assert (c.mixer.heads, c.mixer.kv_heads, c.mixer.dim, c.mixer.vdim, c.mixer.conv, c.mixer.decay, c.mixer.gate) == (6, 2, 4, 6, 2, "channel", "sigmoid_lowrank") and c.ff is None
    assert d.mixer.left.chunk == 0 and d.mixer.left.rotary is None
    assert [x.prefix for x in sp.layers] == ["l0.", "l1.", "l2.", "l3.", "l2."] and [x.weights_of for x in sp.layers] == [None, None, None, None, 2]
    for bad in ([cdelta(weights_of=0)], [cdelta(), cdelta(weights_of=0), cdelta(weights_of=1)], [cdelta(), cdelta(dim=8, weights_of=0)], [cdelta(), mlstm(weights_of=0)],
                [cdelta(weights_of=3)], [{"type": "mamba2", "mixer": {}, "mlp": None}], [mlstm(mlp={"kind": "glu"})]):
        with pytest.raises(ValueError):
            gifopel_spec(config(bad))


def test_registry_and_synthetic_weights_know_the_architecture():
    from mistralrs_amd import registry
    from mistralrs_amd.hybrid import FEED_FORWARDS, MIXERS, SPEC_READERS, gifopel_spec, synthetic_weights
    assert "Gifopel" in registry.ARCHITECTURES and "Gifopel" in SPEC_READERS
    assert {"delta_rule", "mlstm", "parallel"} <= set(MIXERS) and "moe_topk_softmax_relu2" in FEED_FORWARDS
    cfg = config(STACK)
    get = synthetic_weights(gifopel_spec(cfg), "cpu", 1)
    for name, t in weights(cfg).items():
        if name.endswith((".a1", ".a2", ".g1", ".g2")):
            assert get(name).shape[0 if name.endswith("2") else 1] == t.shape[0 if name.endswith("2") else 1], name   # the inner sizes are the generator's choice
        else:
            assert tuple(get(name).shape) == tuple(t.shape), name
    with pytest.raises(KeyError):
        get("l5.mix.q")   # a layer that borrows another layer's tensors has none
    with pytest.raises(KeyError):
        get("head")


def test_restatement_pieces():
    """the oracle's own building blocks on hand-computed values"""
    u = torch.tensor([[1.0], [2.0], [4.0], [8.0]], dtype=D64)
    y, taps = O.conv_silu(u, torch.tensor([[100.0, 10.0, 1.0]], dtype=D64), None)
    pre = torch.tensor([1.0, 12.0, 124.0, 248.0], dtype=D64)
    assert torch.allclose(y.reshape(-1), pre * torch.sigmoid(pre)) and taps.reshape(-1).tolist() == [4.0, 8.0]
    y2, _ = O.conv_silu(torch.tensor([[16.0]], dtype=D64), torch.tensor([[100.0, 10.0, 1.0]], dtype=D64), taps)
    assert torch.allclose(y2.reshape(-1), torch.tensor([496.0], dtype=D64) * torch.sigmoid(torch.tensor(496.0, dtype=D64)))
    # delta rule: with beta = 1 and no decay, writing (k, v) makes S^T k = v; writing the same key again replaces the value; an orthogonal key is untouched
    e0, e1 = torch.tensor([1.0, 0.0], dtype=D64), torch.tensor([0.0, 1.0], dtype=D64)
    k = torch.stack([e0, e1, e0, e0]).view(4, 1, 2)
    v = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0], [7.0, 8.0, 9.0], [0.0, 0.0, 0.0]], dtype=D64).view(4, 1, 3)
    q = torch.stack([e0, e0, e0, e1]).view(4, 1, 2)
    one = torch.ones(4, 1, dtype=D64)
    o, S = O.delta_rule(q, k, v, one, torch.ones(4, 1, 2, dtype=D64), torch.zeros(1, 2, 3, dtype=D64))
    assert o.view(4, 3).tolist() == [[1.0, 2.0, 3.0], [1.0, 2.0, 3.0], [7.0, 8.0, 9.0], [4.0, 5.0, 6.0]] and S[0].tolist() == [[0.0, 0.0, 0.0], [4.0, 5.0, 6.0]]
    # half-strength writes move the stored value half way; a decay of 1 / 2 on channel 0 halves what sits there before the correction is taken
    o, _ = O.delta_rule(q[:2], torch.stack([e0, e0]).view(2, 1, 2), v[:2], 0.5 * one[:2], torch.tensor([[[1.0, 1.0]], [[0.5, 1.0]]], dtype=D64), torch.zeros(1, 2, 3, dtype=D64))
    first = 0.5 * v[0, 0]
    assert torch.allclose(o[1, 0], 0.5 * first + 0.5 * (v[1, 0] - 0.5 * first))
    # matrix memory: one head, scalar keys; the stabiliser never changes the read-out while max(|n q|, e^-m) = |n q|
    ig, fg = torch.tensor([[0.0], [2.0], [-1.0]], dtype=D64), torch.tensor([[-0.1], [-0.2], [-0.3]], dtype=D64)
    kk, vv, qq = torch.tensor([1.0, 2.0, 3.0], dtype=D64).view(3, 1, 1), torch.tensor([5.0, 7.0, 11.0], dtype=D64).view(3, 1, 1), torch.ones(3, 1, 1, dtype=D64) * 4
    o, (S, n, m) = O.mlstm_cell(qq, kk, vv, ig, fg, (torch.zeros(1, 1, 1, dtype=D64), torch.zeros(1, 1, dtype=D64), torch.zeros(1, dtype=D64)))
    c = [math.exp(0.0) * 1 * 5]
    nn = [math.exp(0.0) * 1]
    c.append(math.exp(-0.2) * c[0] + math.exp(2.0) * 2 * 7)
    nn.append(math.exp(-0.2) * nn[0] + math.exp(2.0) * 2)
    c.append(math.exp(-0.3) * c[1] + math.exp(-1.0) * 3 * 11)
    nn.append(math.exp(-0.3) * nn[1] + math.exp(-1.0) * 3)
    ms = [0.0, 2.0, 1.7]
    want = [4 * c[i] / (max(abs(4 * nn[i]), 1.0) + 1e-6 * math.exp(ms[i])) for i in range(3)]     # the unstabilised form of the same cell
    assert torch.allclose(o.view(3), torch.tensor(want, dtype=D64), rtol=1e-12) and torch.allclose(m, torch.tensor([1.7], dtype=D64))
    # rotary: a pair turns by position times its frequency; dimensions past `dims` pass
    x = torch.zeros(3, 1, 6, dtype=D64)
    x[:, 0, 2], x[:, 0, 5] = 1.0, 7.0
    r = O.rotary_interleaved(x, torch.arange(3), 4, 100.0)
    assert torch.allclose(r[:, 0, 2], torch.cos(torch.arange(3, dtype=D64) * 0.1)) and torch.allclose(r[:, 0, 3], torch.sin(torch.arange(3, dtype=D64) * 0.1))
    assert r[:, 0, 5].tolist() == [7.0] * 3 and float(r[:, 0, :2].abs().max()) == 0.0
    # routing: the largest logits, ties to the lower index, weights over the chosen only
    w = {"router": torch.eye(4, dtype=D64), "router.b": torch.tensor([0.0, 0.0, 1.0, 0.0], dtype=D64)}
    ids, wts = O.route(torch.tensor([[2.0, 2.0, 0.5, -1.0]], dtype=D64), w, "", {"router": {"top": 3}})
    assert ids.tolist() == [[0, 1, 2]] and torch.allclose(wts, torch.softmax(torch.tensor([[2.0, 2.0, 1.5]], dtype=D64), -1))


def test_restatement_decodes_token_by_token_like_whole_prompts():
    """the oracle carries states between calls: whole prompt == portions == single tokens (chunks counted from position 0, taps and states carried)"""
    cfg = config(STACK)
    wd = f64(weights(cfg, 3))
    t = toks(50, cfg["vocab"], 4)
    want, after, _ = O.forward(cfg, wd, t)
    got, st, at = [], None, 0
    for n in (1, 2, 20, 1, 26):
        lg, _, st = O.forward(cfg, wd, t[at:at + n], st, at)
        got.append(lg)
        at += n
    assert rel(torch.cat(got), want) < 1e-12 and after.shape == (len(STACK), 50, cfg["width"])


# ---------------------------------------------------------------------------------------------------------------- kernels alone (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("W,one_plus", [(40, 0), (257, 1), (1030, 0)])
def test_two_norms_of_the_same_rows_in_one_launch(dev, W, one_plus):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(W)
    x, w1, w2 = torch.randn(7, W + 3, generator=g) * 3, torch.randn(W, generator=g), torch.randn(W, generator=g)
    unit = x[:, :W].double() / O.rms(x[:, :W].double(), 1e-5)
    for dt, T in ((2, torch.float32), (1, torch.bfloat16)):
        o1, o2, o32 = torch.empty(7, W, dtype=T, device=dev), torch.empty(7, W, dtype=T, device=dev), torch.empty(7, W, device=dev)
        _call("mrs_hyb_rmsnorm_pair", x.to(dev), W + 3, w1.to(dev), w2.to(dev), o1, o2, o32, 7, W, 1e-5, one_plus, dt)
        a, b = unit * (one_plus + w1.double()), unit * (one_plus + w2.double())
        assert rel(o32.double().cpu(), b) < 2e-6
        assert rel(o1.double().cpu(), a) < (2e-6 if dt == 2 else 4e-3) and rel(o2.double().cpu(), b) < (2e-6 if dt == 2 else 4e-3)
        if dt == 1:
            assert torch.equal(o2.cpu(), o32.cpu().to(torch.bfloat16))   # rounded once


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,per_channel", [(4, 2, 16, True), (3, 3, 7, True), (6, 2, 32, False), (1, 1, 130, True), (5, 1, 3, False)])
def test_delta_operands(dev, H, G, D, per_channel):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(H * D)
    T, per = 9, D if per_channel else 1
    ldc, ldu, b_col = 2 * G * D + 5, H + 3 + (0 if per_channel else H), 2
    c, u = torch.randn(T, ldc, generator=g), torch.randn(T, ldu, generator=g)
    a = torch.randn(T, H * per + 2, generator=g) if per_channel else None
    A_log, dtb = torch.randn(H, generator=g) * 0.5, torch.randn(H * per, generator=g)
    cd, ud = c.to(dev), u.to(dev)
    ad = a.to(dev) if per_channel else ud[:, b_col + H:]
    beta, dec = torch.empty(T, H, device=dev), torch.empty(T, H * per, device=dev)
    _call("mrs_hyb_delta_prep", cd, ldc, ud, ldu, b_col, ad, ad.stride(0), A_log.to(dev), dtb.to(dev), beta, dec, T, H, G, D, per)
    qk = c[:, :2 * G * D].double().view(T, 2 * G, D)
    unit = qk / torch.sqrt((qk * qk).sum(-1, keepdim=True) + 1e-6)
    unit[:, :G] *= D ** -0.5
    got = cd.double().cpu()
    assert rel(got[:, :2 * G * D], unit.reshape(T, -1)) < 2e-6 and torch.equal(got[:, 2 * G * D:], c[:, 2 * G * D:].double())
    assert rel(beta.double().cpu(), torch.sigmoid(u[:, b_col:b_col + H].double())) < 2e-6
    raw = (a[:, :H * per] if per_channel else u[:, b_col + H:b_col + 2 * H]).double()
    want = torch.exp(-torch.exp(A_log.double()).repeat_interleave(per) * O.softplus(raw + dtb.double()))
    assert rel(dec.double().cpu(), want) < 2e-6


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,taps,per_channel", [(4, 2, 16, 8, 3, True), (3, 1, 7, 5, 1, False), (2, 2, 64, 32, 4, True), (2, 1, 130, 3, 6, False)])
def test_single_row_steps_convolve_shift_taps_and_make_operands_in_one_launch(dev, H, G, D, Dv, taps, per_channel):
    """three entries of one row each (one at position 0 over a NaN-filled slot, two continuing): convolution + SiLU from the slots' taps, the taps shifted, unit vectors, write
    strengths and decays -- against the restatement; two steps in a row so that the shifted taps are read back"""
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(D + taps)
    per, C, keep = (D if per_channel else 1), 2 * G * D + H * Dv, max(taps - 1, 1)
    ldu, b_col = C + H + 2, C + 1
    cw, A_log, dtb = torch.randn(C, taps, generator=g) * 0.6, torch.randn(H, generator=g) * 0.5, torch.randn(H * per, generator=g)
    before = [None, torch.randn(taps - 1, C, generator=g), torch.randn(taps - 1, C, generator=g)]
    state = torch.full((4, C, keep), float("nan"), device=dev)
    slots = (2, 0, 3)
    for e in (1, 2):
        if taps > 1:
            state[slots[e]] = before[e].T.to(dev)
    pos = [0, 9, 40]
    for step in range(2):
        u, a = torch.randn(3, ldu, generator=g), torch.randn(3, H * per + 3, generator=g)
        b = _batch(dev, [(pos[e] + step, 1, slots[e]) for e in range(3)])
        c, beta, dec = torch.empty(3, C + 2, device=dev), torch.empty(3, H, device=dev), torch.empty(3, H * per, device=dev)
        _call("mrs_hyb_delta_step_prep", u.to(dev), ldu, cw.to(dev), state, c, C + 2, C, taps, b_col, a.to(dev), H * per + 3, A_log.to(dev), dtb.to(dev), beta, dec, b.seq_start,
              b.seq_pos0, b.seq_slot, 3, 3, H, G, D, per)
        for e in range(3):
            y, before[e] = O.conv_silu(u[e:e + 1, :C].double(), cw.double(), before[e].double() if before[e] is not None else None)
            qk = y[0, :2 * G * D].view(2 * G, D)
            unit = qk / torch.sqrt((qk * qk).sum(-1, keepdim=True) + 1e-6)
            unit[:G] *= D ** -0.5
            got = c[e].double().cpu()
            assert rel(got[:2 * G * D], unit.reshape(-1)) < 3e-6 and rel(got[2 * G * D:C], y[0, 2 * G * D:]) < 3e-6, (step, e)
            assert rel(beta[e].double().cpu(), torch.sigmoid(u[e, b_col:b_col + H].double())) < 2e-6
            want = torch.exp(-torch.exp(A_log.double()).repeat_interleave(per) * O.softplus(a[e, :H * per].double() + dtb.double()))
            assert rel(dec[e].double().cpu(), want) < 2e-6
            if taps > 1:
                assert rel(state[slots[e]].double().cpu(), before[e].T) < 1e-7, (step, e)
    assert bool(torch.isnan(state[1]).all())


def _delta_rows(T, H, G, D, Dv, per, seed, slow=False):
    g = torch.Generator().manual_seed(seed)
    q, k = torch.randn(T, G, D, generator=g), torch.randn(T, G, D, generator=g)
    q, k = q / q.norm(dim=-1, keepdim=True) * D ** -0.5, k / k.norm(dim=-1, keepdim=True)
    v = torch.randn(T, H, Dv, generator=g)
    beta = torch.rand(T, H, generator=g)
    dec = (1 - 0.02 * torch.rand(T, H, per, generator=g)) if slow else torch.rand(T, H, per, generator=g) * 0.6 + 0.4
    return q, k, v, beta, dec


@pytest.mark.gpu
@pytest.mark.parametrize("segmented", [False, True], ids=["chains", "segments"])
@pytest.mark.parametrize("H,G,D,Dv,per_channel,lanes", [(4, 2, 16, 8, True, 0), (2, 1, 32, 32, False, 4), (2, 2, 64, 16, True, 16), (3, 1, 7, 5, True, 0), (1, 1, 130, 3, False, 16),
                                                         (2, 2, 128, 40, True, 4), (2, 1, 256, 130, True, 0), (5, 5, 1, 1, False, 0)])
def test_delta_recurrence_over_portions_single_rows_and_reused_slots(dev, H, G, D, Dv, per_channel, lanes, segmented):
    """three sequences through slots that hold a former owner's numbers: portions of several sizes (some longer than two segments of 64 rows) beside single rows, every entry
    as one chain or its segments side by side, every row against the restatement on the whole sequence"""
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    per = D if per_channel else 1
    lens = (250, 151, 9)
    seqs = [_delta_rows(n, H, G, D, Dv, per, 10 * D + k, slow=k == 0) for k, n in enumerate(lens)]   # the longest one decays slowly: what a segment is handed matters
    rep = H // G
    want = []
    for q, k, v, beta, dec in seqs:
        o, _ = O.delta_rule(q.double().repeat_interleave(rep, 1), k.double().repeat_interleave(rep, 1), v.double(), beta.double(), dec.double().expand(-1, H, D),
                            torch.zeros(H, D, Dv, dtype=D64))
        want.append(o.reshape(-1, H * Dv))
    ldc = 2 * G * D + H * Dv + 3
    state = torch.full((5, H, D, Dv), 1e6, device=dev)
    state[1] = float("nan")
    got, at = [[] for _ in seqs], [0, 0, 0]

    def run(ns, slots=(3, 0, 4)):
        parts = [(j, n) for j, n in enumerate(ns) if n]
        b = _batch(dev, [(at[j], n, slots[j]) for j, n in parts])
        rows = []
        for j, n in parts:
            q, k, v, _, _ = seqs[j]
            s = slice(at[j], at[j] + n)
            rows.append(torch.cat([q[s].reshape(n, -1), k[s].reshape(n, -1), v[s].reshape(n, -1), torch.zeros(n, 3)], 1))
        c = torch.cat(rows).to(dev)
        beta = torch.cat([seqs[j][3][at[j]:at[j] + n] for j, n in parts]).to(dev)
        dec = torch.cat([seqs[j][4][at[j]:at[j] + n].reshape(n, -1) for j, n in parts]).to(dev)
        y = torch.empty(c.shape[0], H * Dv, device=dev)
        if segmented:
            carry, trans = torch.empty(b.segments, H, D, Dv, device=dev), torch.empty(b.segments, H, D, D, device=dev)
            _call("mrs_hyb_delta_scan", c, ldc, beta, dec, state, y, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0, carry, trans, c.shape[0], len(parts),
                  b.segments, H, G, D, Dv, per, lanes)
        else:
            _call("mrs_hyb_delta_scan", c, ldc, beta, dec, state, y, b.seq_pos0, b.seq_slot, *b.entry_table(), None, None, c.shape[0], len(parts), len(parts), H, G, D, Dv, per, lanes)
        r = 0
        for j, n in parts:
            got[j].append(y[r:r + n].double().cpu())
            r += n
            at[j] += n
    run([30, 2, 0])
    run([1, 1, 1])
    run([2, 5, 3])
    run([1, 0, 2])
    run([150, 64, 3])      # three segments (64 + 64 + 22) beside exactly one beside a short one
    run([66, 79, 0])
    assert at == list(lens)
    for j in range(3):
        assert rel(torch.cat(got[j]), want[j]) < 2e-5, j
    assert bool((state[2] == 1e6).all()) and bool(torch.isnan(state[1]).all())


@pytest.mark.gpu
def test_delta_state_keeps_a_planted_pair_for_hundreds_of_rows_and_replaces_it(dev):
    """hand-made rows: key e_0 with value u at row 5, other rows write along e_1 only; a query e_0 reads g^distance u hundreds of rows later (over portions of 63 / 64 / 65 / 2 / 1
    rows, from a slot another sequence left full); at row 300 the same key comes again with value w and full strength: from then on the read-out is w, not u + w"""
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    H, D, Dv, T = 2, 8, 4, 400
    ldc = 2 * H * D + H * Dv
    uval, wval = torch.tensor([1.0, -2.0, 3.0, 0.5], dtype=D64), torch.tensor([-4.0, 0.25, 0.0, 2.0], dtype=D64)
    c = torch.zeros(T, ldc)
    c[:, 0] = 1.0                                           # every q of head 0 = e_0
    c[:, H * D + 1] = 1.0                                   # k of head 0 = e_1 ...
    c[:, 2 * H * D:2 * H * D + Dv] = 9.0                    # ... with some value
    for row, val in ((5, uval), (300, wval)):
        c[row, H * D + 1], c[row, H * D] = 0.0, 1.0         # k of head 0 = e_0
        c[row, 2 * H * D:2 * H * D + Dv] = val.float()
    beta, dec = torch.ones(T, H), torch.ones(T, H, D)
    dec[:, 0, 0] = 0.99609375                               # channel 0 of head 0 decays; channel 1 (where the other rows write) would vanish at once
    dec[:, 0, 1] = 0.0
    state = torch.full((3, H, D, Dv), float("nan"), device=dev)
    state[1] = 1e6
    at, outs = 0, []
    for n in (63, 1, 64, 2, 65, 1, 1, 130, 3, 70):
        b = _batch(dev, [(at, n, 1)])
        y = torch.empty(n, H * Dv, device=dev)
        carry, trans = torch.empty(b.segments, H, D, Dv, device=dev), torch.empty(b.segments, H, D, D, device=dev)
        _call("mrs_hyb_delta_scan", c[at:at + n].to(dev), ldc, beta[at:at + n].to(dev), dec[at:at + n].reshape(n, -1).to(dev), state, y, b.seq_pos0, b.seq_slot, b.seg_entry,
              b.seg_row0, b.seg_len, b.ent_seg0, carry, trans, n, 1, b.segments, H, H, D, Dv, D, 0)
        outs.append(y.double().cpu())
        at += n
    y = torch.cat(outs)[:, :Dv]
    t = torch.arange(T, dtype=D64)
    want = torch.where((t >= 5).view(T, 1), (0.99609375 ** (t - 5)).view(T, 1) * uval, torch.zeros(T, Dv, dtype=D64))
    want[300:] = (0.99609375 ** (t[300:] - 300)).view(-1, 1) * wval
    assert float((y - want).abs().max()) < 1e-5 and float(want[299].abs().max()) > 0.5
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("H,D,Dv,cap", [(2, 12, 16, 9.0), (3, 7, 5, 2.5), (1, 64, 64, 15.0), (4, 16, 127, 6.0), (2, 130, 8, 30.0), (2, 64, 256, 8.0), (1, 128, 300, 8.0), (1, 20, 257, 8.0)])
def test_exponential_gates_and_matrix_memory_over_segments_and_single_rows(dev, H, D, Dv, cap):
    """gate kernel + gated scan with the normaliser column + head norm, two sequences through reused slots, portions longer than a segment (64 rows), a portion that ends a
    segment exactly, single rows: against the restatement's cell on the whole sequences"""
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(D * Dv)
    lens = (210, 77)
    nv, nk = H * Dv, H * D
    ld = 2 * nv + 2 * nk + 2 * H + 1
    q_col, g_col, i_col, f_col = nv + nk, nv + 2 * nk, 2 * nv + 2 * nk, 2 * nv + 2 * nk + H
    seqs = [torch.randn(n, ld, generator=g) for n in lens]
    for s in seqs:
        s[:, i_col:f_col] *= 3
        s[:, f_col:f_col + H] = s[:, f_col:f_col + H] * 3 + 2
    bi, bf, nw = torch.randn(H, generator=g), torch.randn(H, generator=g), torch.randn(nv, generator=g)
    want = []
    for s in seqs:
        d = s.double()
        n = d.shape[0]
        ig = cap * torch.tanh((d[:, i_col:f_col] + bi.double()) / cap)
        fg = O.logsigmoid(cap * torch.tanh((d[:, f_col:f_col + H] + bf.double()) / cap))
        o, _ = O.mlstm_cell(d[:, q_col:g_col].view(n, H, D) * D ** -0.5, d[:, nv:q_col].view(n, H, D), d[:, :nv].view(n, H, Dv), ig, fg,
                            (torch.zeros(H, D, Dv, dtype=D64), torch.zeros(H, D, dtype=D64), torch.zeros(H, dtype=D64)))
        want.append((o / O.rms(o, 1e-5)).reshape(n, nv) * nw.double() * torch.sigmoid(d[:, g_col:i_col]))
    state = torch.full((4, H, D, Dv + 1), 1e6, device=dev)
    m_state = torch.full((4, H), 50.0, device=dev)
    got, at = [[], []], [0, 0]

    def run(ns, slots=(2, 0)):
        parts = [(j, n) for j, n in enumerate(ns) if n]
        b = _batch(dev, [(at[j], n, slots[j]) for j, n in parts])
        u = torch.cat([seqs[j][at[j]:at[j] + n] for j, n in parts]).to(dev)
        T = u.shape[0]
        steps, mbuf, mexp = torch.empty(T, H, 2, device=dev), torch.empty(T + len(parts), H, device=dev), torch.empty(T, H, device=dev)
        _call("mrs_hyb_exp_gates", u, ld, i_col, f_col, bi.to(dev), bf.to(dev), cap, m_state, steps, mbuf, mexp, b.tok_seq, b.seq_start, b.seq_pos0, b.seq_slot, T, len(parts), H)
        y = torch.empty(T, H * (Dv + 1), device=dev)
        carry, dk = torch.empty(b.segments, H, D, Dv + 1, device=dev), torch.empty(b.segments, H, device=dev)
        _call("mrs_hyb_gated_scan", u, ld, steps, state, y, b.seq_pos0, b.seq_slot, b.seg_entry, b.seg_row0, b.seg_len, b.ent_seg0, carry, dk, T, len(parts), b.segments,
              H, Dv, D, H, 1, float(np.float32(D) ** np.float32(-0.5)))
        o = torch.empty(T, nv, device=dev)
        _call("mrs_hyb_head_norm_gate", y, Dv + 1, mexp, nw.to(dev), 1, u[:, g_col:], ld, 1, o, T, H, Dv, 1e-5, 2)
        r = 0
        for j, n in parts:
            got[j].append(o[r:r + n].double().cpu())
            r += n
            at[j] += n
    run([130, 3])
    run([1, 1])
    run([62, 64])       # the first sequence now stands at 193, the second at 68
    run([1, 0])
    run([2, 9])
    run([14, 0])
    assert at == list(lens)
    for j in range(2):
        assert rel(torch.cat(got[j]), want[j]) < 2e-5, j
    assert bool((state[1] == 1e6).all()) and bool((m_state[3] == 50.0).all())


@pytest.mark.gpu
@pytest.mark.parametrize("H,Dv,full,mode", [(3, 8, 0, 1), (2, 70, 1, 2), (5, 1, 0, 0), (1, 129, 1, 1)])
def test_head_norm_with_shared_or_full_weight_and_either_gate(dev, H, Dv, full, mode):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(H * Dv)
    y, gate, w = torch.randn(6, H * Dv, generator=g) * 2, torch.randn(6, H * Dv + 4, generator=g), torch.randn(H * Dv if full else Dv, generator=g)
    yd = y.double().view(6, H, Dv)
    want = yd / O.rms(yd, 1e-4) * (w.double().view(H, Dv) if full else w.double())
    gd = gate[:, :H * Dv].double().view(6, H, Dv)
    want = want * (torch.sigmoid(gd) if mode == 1 else O.silu(gd) if mode == 2 else 1.0)
    out = torch.empty(6, H * Dv, device=dev)
    _call("mrs_hyb_head_norm_gate", y.to(dev), Dv, None, w.to(dev), full, gate.to(dev) if mode else None, H * Dv + 4, mode, out, 6, H, Dv, 1e-4, 2)
    assert rel(out.double().cpu(), want.reshape(6, -1)) < 2e-6
    ob = torch.empty(6, H * Dv, dtype=torch.bfloat16, device=dev)
    _call("mrs_hyb_head_norm_gate", y.to(dev), Dv, None, w.to(dev), full, gate.to(dev) if mode else None, H * Dv + 4, mode, ob, 6, H, Dv, 1e-4, 1)
    assert torch.equal(ob.cpu(), out.cpu().to(torch.bfloat16))


@pytest.mark.gpu
@pytest.mark.parametrize("W", [40, 513])
def test_normed_average_rounded_columns_and_squared_relu(dev, W):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(W)
    x, y1, y2, w1, w2 = (torch.randn(5, W, generator=g) for _ in range(5))
    w1, w2 = w1[0], w2[0]
    avg = 0.5 * (O.norm_plain(y1.double(), w1.double(), 1e-5) + O.norm_plain(y2.double(), w2.double(), 1e-5))
    for acc in (1, 0):
        xd = x.to(dev)
        _call("mrs_hyb_norm_pair_add", xd, W, y1.to(dev), w1.to(dev), y2.to(dev), w2.to(dev), 5, W, 1e-5, 0.5, acc)
        assert rel(xd.double().cpu(), avg + (x.double() if acc else 0)) < 2e-6
    out = torch.empty(5, W - 7, dtype=torch.bfloat16, device=dev)
    _call("mrs_hyb_round_cols", x.to(dev)[:, 3:], W, out, 5, W - 7, 1)
    assert torch.equal(out.cpu(), x[:, 3:W - 4].to(torch.bfloat16))
    sq = torch.empty(5, W, device=dev)
    _call("mrs_hyb_relu_sq", x.to(dev), sq, 5, W, 2)
    assert torch.equal(sq.cpu(), torch.clamp(x, min=0) ** 2)


@pytest.mark.gpu
@pytest.mark.parametrize("E,top,W", [(6, 2, 40), (16, 4, 64), (70, 7, 33), (3, 3, 8), (5, 1, 12)])
def test_router_softmax_over_the_chosen_logits(dev, E, top, W):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(E)
    h, wr, br = torch.randn(11, W, generator=g), torch.randn(E, W, generator=g), torch.randn(E, generator=g) * 2
    h[3] = 0.0              # all logits = the bias
    ids, wts = torch.empty(11 * top, dtype=torch.int32, device=dev), torch.empty(11 * top, device=dev)
    _call("mrs_hyb_route_topk_softmax", h.to(dev), wr.to(dev), br.to(dev), 11, W, E, top, 1.0, ids, wts)
    want_ids, want_w = O.route(h.double(), {"router": wr.double(), "router.b": br.double()}, "", {"router": {"top": top}})
    assert torch.equal(ids.cpu().view(11, top).long(), want_ids) and rel(wts.double().cpu().view(11, top), want_w) < 2e-6
    assert float((wts.view(11, top).sum(-1) - 1).abs().max()) < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,rot", [(4, 2, 16, 8, 8), (3, 1, 10, 6, 4), (2, 2, 64, 64, 64), (5, 5, 6, 3, 0)])
def test_query_key_norm_per_head_then_rotary_then_pages(dev, H, G, D, Dv, rot):
    from mistralrs_amd.hybrid import _call
    _lib.load("hybrid")
    g = torch.Generator().manual_seed(D)
    T, bs = 6, 4
    ld = H * D + G * D + G * Dv + 2
    u, qw, kw = torch.randn(T, ld, generator=g), torch.randn(D, generator=g), torch.randn(D, generator=g)
    pos = torch.tensor([0, 1, 5, 300, 2, 3], dtype=torch.int32)
    slots = torch.tensor([4, 5, 9, 0, 14, 15], dtype=torch.int64)
    freq = torch.tensor([50.0 ** (-2.0 * i / rot) for i in range(rot // 2)] or [0.0], dtype=D64).float()
    q = torch.empty(T, H * D, device=dev)
    kc, vc = torch.zeros(4, G, bs, D, device=dev), torch.zeros(4, G, bs, Dv, device=dev)
    _call("mrs_hyb_qk_headnorm_rope_cache", u.to(dev), ld, qw.to(dev), kw.to(dev), freq.to(dev), pos.to(dev), slots.to(dev), q, kc, vc, T, H, G, D, Dv, rot, bs, 1e-5, 2)
    ud = u.double()
    wq = O.rotary_interleaved(O.norm_plain(ud[:, :H * D].view(T, H, D), qw.double(), 1e-5), pos, rot, 50.0)
    wk = O.rotary_interleaved(O.norm_plain(ud[:, H * D:H * D + G * D].view(T, G, D), kw.double(), 1e-5), pos, rot, 50.0)
    assert rel(q.double().cpu().view(T, H, D), wq) < 3e-5
    for t in range(T):
        blk, off = int(slots[t]) // bs, int(slots[t]) % bs
        assert rel(kc[blk, :, off].double().cpu(), wk[t]) < 3e-5
        assert torch.equal(vc[blk, :, off].cpu(), u[t, H * D + G * D:H * D + G * D + G * Dv].view(G, Dv))


def _attend(dev, q, keys, vals, pos0s, lens, chunk, sink, gate, scale, bs=8, dtype=2):
    """q [rows, H, D] of several entries (rows of entry e at positions pos0s[e] ...); keys / vals [e] = [P_e, G, D | Dv] of every position of the entry's sequence, scattered
    over shuffled pages"""
    from mistralrs_amd.hybrid import _call
    rows, H, D = q.shape
    G, Dv = keys[0].shape[1], vals[0].shape[2]
    order = torch.randperm(64, generator=torch.Generator().manual_seed(5)).tolist()
    kc, vc = torch.zeros(65, G, bs, D, device=dev), torch.zeros(65, G, bs, Dv, device=dev)
    blocks = []
    for e, (k, v) in enumerate(zip(keys, vals)):
        need = -(-k.shape[0] // bs)
        blk = [order.pop() + 1 for _ in range(need)]
        blocks.append(blk)
        for j in range(k.shape[0]):
            kc[blk[j // bs], :, j % bs], vc[blk[j // bs], :, j % bs] = k[j].to(dev), v[j].to(dev)
    b = _batch(dev, [(p0, n, 0) for p0, n in zip(pos0s, lens)], bs, blocks)
    out = torch.empty(rows, H * Dv, device=dev)
    _call("mrs_hyb_paged_attn_chunked", q.reshape(rows, -1).to(dev), kc, vc, b.block_tables, b.tok_seq, b.tok_pos, out, rows, H, G, D, Dv, bs, b.max_blocks, chunk, scale, dtype,
          b.seg_entry, b.seg_row0, b.seg_len, b.segments, 64, 0.0, 1 if sink is not None else 0, sink.to(dev) if sink is not None else None,
          gate.to(dev) if gate is not None else None, H if gate is not None else 0, 1, None, 0)
    return out.double().cpu().view(rows, H, Dv)


@pytest.mark.gpu
@pytest.mark.parametrize("single", [False, True], ids=["portion", "single_rows"])
@pytest.mark.parametrize("chunk", [7, 8, 24, 0])
def test_planted_keys_at_the_chunk_edges(dev, single, chunk):
    """one key per query gets a score far above the rest: the first key of the query's chunk (must be read), the key just before it (must not be), the query itself, a key on
    a page border; the value of that key is recognisable.  Without any visible planted key the output is the plain average behind a large sink."""
    _lib.load("hybrid")
    H, G, D, Dv, P = 2, 1, 8, 4, 61
    g = torch.Generator().manual_seed(chunk)
    keys = torch.randn(P, G, D, generator=g) * 0.05
    vals = torch.zeros(P, G, Dv)
    vals[:, 0, 0] = torch.arange(P).float()                       # the value names its position
    vals[:, 0, 1] = 1.0
    q0 = 30 if single else 20
    rows = P - q0
    q = torch.zeros(rows, H, D)
    targets = []
    for r in range(rows):
        i = q0 + r
        lo = (i // chunk) * chunk if chunk else 0
        tgt = [lo, lo - 1, i, (i // 8) * 8][r % 4]                # inside edge, outside edge, itself, the first slot of its page
        targets.append(tgt)
        if tgt >= 0:
            q[r, :, :] = keys[tgt, 0] / keys[tgt, 0].norm() * 40.0
            keys[tgt, 0] = keys[tgt, 0] / keys[tgt, 0].norm() * 8.0
    # a planted key is loud for every query that points along it; the restatement below knows that too
    sink = torch.tensor([-30.0, 2.0])
    gate = torch.randn(rows, H, generator=g)
    if single:
        outs = [_attend(dev, q[r:r + 1], [keys[:q0 + r + 1]], [vals[:q0 + r + 1]], [q0 + r], [1], chunk, sink, gate[r:r + 1], 1.0) for r in range(rows)]
        got = torch.cat(outs)
    else:
        got = _attend(dev, q, [keys], [vals], [q0], [rows], chunk, sink, gate, 1.0)
    kd, vd, qd = keys.double(), vals.double(), q.double()
    seen_inside = seen_outside = 0
    for r in range(rows):
        i = q0 + r
        lo = (i // chunk) * chunk if chunk else 0
        for h in range(H):
            s = kd[lo:i + 1, 0] @ qd[r, h]
            top = max(float(s.max()), float(sink[h]))
            e = torch.exp(s - top)
            want = (e[:, None] * vd[lo:i + 1, 0]).sum(0) / (e.sum() + math.exp(float(sink[h]) - top)) * torch.sigmoid(gate[r, h].double())
            assert float((got[r, h] - want).abs().max()) < 2e-4 * max(1.0, float(want.abs().max())), (r, h, targets[r])
        read = float(got[r, 0, 0] / got[r, 0, 1])                 # head 0 has next to no sink: the weighted mean of the positions read
        if targets[r] >= lo and targets[r] >= 0:
            assert abs(read - targets[r]) < 0.05, (r, targets[r], read)
            seen_inside += targets[r] == lo
        else:
            assert read >= lo - 1e-3, (r, targets[r], read)      # nothing before the chunk leaks in
            seen_outside += 1
    assert seen_inside >= 3 and (seen_outside >= 3 or not chunk)


@pytest.mark.gpu
def test_sink_alone_and_gate_per_head(dev):
    """a query that matches nothing next to a large sink returns (almost) nothing; without the sink term the same rows return the average value; the gate scales whole heads"""
    _lib.load("hybrid")
    H, D, Dv, P = 3, 8, 6, 20
    g = torch.Generator().manual_seed(1)
    keys, vals = torch.zeros(P, 1, D), torch.randn(P, 1, Dv, generator=g) + 3
    q = torch.zeros(4, H, D)
    sink = torch.tensor([10.0, 0.0, -40.0])
    gate = torch.tensor([[0.0, 0.0, 0.0], [50.0, -50.0, 0.0], [0.0, 0.0, 0.0], [0.0, 0.0, 0.0]])
    got = _attend(dev, q, [keys], [vals], [P - 4], [4], 0, sink, gate, 1.0)
    for r in range(4):
        n = P - 4 + r + 1
        mean = vals[:n, 0].double().mean(0)
        for h in range(H):
            want = mean * n / (n + math.exp(float(sink[h]))) * (1 / (1 + math.exp(-float(gate[r, h]))))
            assert float((got[r, h] - want).abs().max()) < 1e-5, (r, h)
    assert float(got[0, 0].abs().max()) < 1e-2 and float(got[1, 1].abs().max()) < 1e-12 and float(got[0, 2].abs().min()) > 0.4


# ---------------------------------------------------------------------------------------------------------------- mixers alone (GPU)
def _one_layer(layer, dev, t_len=90, seed=1, dtype="float32", **kw):
    cfg = config([layer], **kw)
    w = weights(cfg, seed)
    t = toks(t_len, cfg["vocab"], seed + 100)
    want = logits_of(cfg, f64(w), t)
    sv = Served(cfg, w, dev, dtype)
    got = sv.step([(1, t[:t_len - 12])]) + sv.step([(1, t[t_len - 12:t_len - 9])]) + [sv.step([(1, [x])])[0] for x in t[t_len - 9:]]
    return torch.cat(got), want


@pytest.mark.gpu
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=64, vdim=64, conv=4), dict(heads=6, kv_heads=2, dim=7, vdim=5, conv=2), dict(heads=2, kv_heads=1, dim=128, vdim=16, conv=1),
                                dict(heads=3, kv_heads=3, dim=40, vdim=130, conv=7), dict(heads=8, kv_heads=4, dim=32, vdim=32, conv=4, mlp=None)])
def test_delta_mixer_with_channel_decays_alone(dev, kw):
    got, want = _one_layer(cdelta(**kw), dev)
    assert rel(got, want) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, dim=64, vdim=64, cap=15.0), dict(heads=5, dim=7, vdim=5, cap=1.5), dict(heads=2, dim=130, vdim=16), dict(heads=2, dim=16, vdim=255, mlp=None),
                                dict(heads=4, dim=32, vdim=127, mlp="moe")])
def test_matrix_memory_mixer_alone(dev, kw):
    got, want = _one_layer(mlstm(**kw), dev, t_len=150)
    assert rel(got, want) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("kw", [dict(), dict(heads=8, kv_heads=1, dim=32, vdim=32, size=32, dims=32), dict(heads=3, kv_heads=3, dim=10, vdim=7, size=5, dims=6, rheads=3, rkv=1, rdim=5, rvdim=3, rconv=1),
                                dict(size=0, dims=0), dict(heads=2, kv_heads=2, dim=128, vdim=160, size=64, dims=2, rheads=1, rkv=1, rdim=64, rvdim=64), dict(size=1), dict(size=1000, mlp=None)])
def test_parallel_mixer_alone(dev, kw):
    got, want = _one_layer(par(**kw), dev, t_len=120)
    assert rel(got, want) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("f", [moe(6, 2, 24), moe(16, 4, 40), moe(3, 3, 7), moe(9, 1, 130), dense(56), dense(7)])
def test_feed_forwards_alone_at_prompt_and_decode_sizes(dev, f):
    """70 rows (grouped products over expert-sorted rows) and 1 - 3 rows (every route streams its expert's slabs)"""
    got, want = _one_layer(mlstm(heads=1, dim=4, vdim=4, mlp=f), dev, t_len=82)
    assert rel(got, want) < 3e-5


@pytest.mark.gpu
def test_sharp_attention_lands_on_chunk_edges_and_needs_the_mask_and_the_sink(dev):
    """queries and keys scaled until most rows put their weight on one key: the restatement with a chunk size one off, or without the sink, is far away; the served model is not"""
    layer = par(heads=2, kv_heads=1, dim=8, vdim=8, size=13, dims=4, scale=1.0, mlp=None)
    cfg = config([layer])
    w = weights(cfg, 21)
    w["l0.mix.left.q.norm"] = (w["l0.mix.left.q.norm"].float() * 3).to(torch.bfloat16)
    w["l0.mix.right.out"] = (w["l0.mix.right.out"].float() * 0).to(torch.bfloat16)     # the attention side alone
    t = toks(200, cfg["vocab"], 22)
    wd = f64(w)
    want = logits_of(cfg, wd, t)
    sv = Served(cfg, w, dev)
    got = sv.step([(1, t[:150])]) + [sv.step([(1, [x])])[0] for x in t[150:]]
    assert rel(torch.cat(got), want) < 3e-5
    for size in (12, 14):
        other = json.loads(json.dumps(cfg))
        other["layers"][0]["mixer"]["left"]["mask"]["size"] = size
        assert rel(logits_of(other, wd, t), want) > 0.05
    no_sink = dict(wd)
    no_sink["l0.mix.left.sink"] = wd["l0.mix.left.sink"] - 60.0
    assert rel(logits_of(cfg, no_sink, t), want) > 0.01


@pytest.mark.gpu
def test_slow_states_carry_the_first_tokens_across_a_long_prompt_and_decoding(dev):
    """decays and forget gates close to one: the logits of the last rows depend on the first tokens (the restatement fed another beginning is far away), over portions and
    300 single rows"""
    cfg = config([cdelta(mlp=None), mlstm(mlp=None), par(mlp=None)])
    w = weights(cfg, 31, slow=True)
    wd = f64(w)
    t = toks(420, cfg["vocab"], 32)
    want = logits_of(cfg, wd, t)
    other = logits_of(cfg, wd, toks(6, cfg["vocab"], 33) + t[6:])
    assert rel(other[-40:], want[-40:]) > 1e-3
    sv = Served(cfg, w, dev, max_tokens=448)
    got = sv.step([(1, t[:63])]) + sv.step([(1, t[63:65])]) + sv.step([(1, t[65:120])]) + [sv.step([(1, [x])])[0] for x in t[120:]]
    assert rel(torch.cat(got), want) < 5e-5


@pytest.mark.gpu
@pytest.mark.parametrize("size", [0, 600, 300])
def test_decoding_with_split_keys_inside_a_long_chunk(dev, size):
    """single-row steps over hundreds of keys deal a row's keys to several workgroups (some shares empty right behind a chunk border); two sequences of unequal length"""
    cfg = config([par(heads=4, kv_heads=2, dim=16, vdim=8, size=size, dims=8, scale=0.6, mlp=None)])
    w = weights(cfg, 41)
    wd = f64(w)
    ta, tb = toks(640, cfg["vocab"], 42), toks(290, cfg["vocab"], 43)
    wa, wb = logits_of(cfg, wd, ta), logits_of(cfg, wd, tb)
    sv = Served(cfg, w, dev, max_tokens=1024)
    sv.step([(1, ta[:590]), (2, tb[:240])])
    assert sv.m.key_splits(_batch(dev, [(600, 1, 0)]), 4, 8, size)[1] >= 2 if size != 300 else True
    for i in range(50):
        ga, gb = sv.step([(1, [ta[590 + i]]), (2, [tb[240 + i]])])
        assert rel(ga, wa[590 + i:591 + i]) < 3e-5 and rel(gb, wb[240 + i:241 + i]) < 3e-5, i


@pytest.mark.gpu
def test_first_tokens_see_zeros_not_the_slots_former_owner(dev):
    """two slots, four requests one after the other: taps, matrices, normalisers and stabilisers of finished requests stay in the slots; a new request must not read them"""
    cfg = config([cdelta(), mlstm(), par()])
    w = weights(cfg, 23)
    sv = Served(cfg, w, dev, max_tokens=128, slots=2)
    wd = f64(w)
    for r in range(1, 5):
        t = toks(40 + r, cfg["vocab"], 30 + r)
        want = logits_of(cfg, wd, t)
        got = sv.step([(r, t[:1])]) + sv.step([(r, t[1:3])]) + sv.step([(r, t[3:])])
        assert rel(torch.cat(got), want) < 3e-5, r
        sv.end(r)


# ---------------------------------------------------------------------------------------------------------------- whole models (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_whole_prompt_every_layer(dev, dtype, bar):
    cfg = config(STACK)
    w = weights(cfg, 5)
    sv = Served(cfg, w, dev, dtype)
    t = toks(150, cfg["vocab"], 14)
    want, after, _ = O.forward(cfg, f64(w), t)
    sv.m.trace_layers = []
    got = sv.step([(1, t)])[0]
    assert len(sv.m.trace_layers) == len(STACK)
    for i, (a, b) in enumerate(zip(sv.m.trace_layers, after)):
        assert close(a.double().cpu(), b, bar), f"residual stream after layer {i}"
    assert close(got, want, bar)


@pytest.mark.gpu
def test_layers_that_borrow_tensors_hold_no_copy_and_their_own_state(dev):
    cfg = config(STACK)
    sv = Served(cfg, weights(cfg, 5), dev)
    L = sv.m.layers
    assert L[5].mixer.w_in is L[2].mixer.w_in and L[5].ff is L[2].ff and L[5].norm1 is L[2].norm1 and L[5].mixer.state is not L[2].mixer.state
    assert L[6].mixer.left.w_qkv is L[1].mixer.left.w_qkv and L[6].mixer.left.k_cache is not L[1].mixer.left.k_cache and L[6].mixer.right.conv_state is not L[1].mixer.right.conv_state
    assert sv.m.head is sv.m.embed
    assert sv.m.has_recurrent_state and sv.m.has_paged_kv


@pytest.mark.gpu
def test_portions_and_decoding_equal_the_whole_prompt(dev):
    """the same 200 tokens: whole; in portions of changing sizes down to two tokens and single tokens; token by token from the start"""
    cfg = config(STACK)
    w = weights(cfg, 6)
    t = toks(200, cfg["vocab"], 15)
    want = logits_of(cfg, f64(w), t)
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
    full = {r: logits_of(cfg, wd, t) for r, t in req.items()}
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
def test_sizes_that_coincide_or_equal_one(dev):
    """one head, one tap, one expert, chunks of one position, key and value sizes equal to the width, rotation over the whole head, one-token prompts"""
    for layers, kw in (([cdelta(heads=1, kv_heads=1, dim=24, vdim=24, conv=1, mlp=moe(1, 1, 24)), mlstm(heads=1, dim=24, vdim=24, mlp=dense(24)),
                         par(heads=1, kv_heads=1, dim=24, vdim=24, size=24, dims=24, rheads=1, rkv=1, rdim=24, rvdim=24, rconv=1, mlp=moe(2, 2, 24))], dict(width=24, vocab=24)),
                       ([cdelta(heads=2, kv_heads=2, dim=1, vdim=1, conv=2, mlp=moe(2, 1, 1)), mlstm(heads=1, dim=1, vdim=1, cap=1.0, mlp=dense(1)),
                         par(heads=2, kv_heads=2, dim=2, vdim=1, size=1, dims=2, rheads=1, rkv=1, rdim=1, rvdim=1, rconv=2, mlp=None)], dict(width=8, vocab=5))):
        cfg = config(layers, **kw)
        w = weights(cfg, 9, rank=1)
        t = toks(40, cfg["vocab"], 17)
        want = logits_of(cfg, f64(w), t)
        sv = Served(cfg, w, dev)
        assert rel(sv.step([(1, t[:1])])[0], want[:1]) < 3e-5
        got = sv.step([(2, t[:1])]) + sv.step([(2, t[1:3])]) + sv.step([(2, t[3:])])
        assert rel(torch.cat(got), want) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,bar", [("float32", 3e-5), ("bfloat16", 5e-2)])
def test_sizes_off_every_vector_width(dev, dtype, bar):
    """width, vocabulary, head sizes, inner sizes and feed-forward sizes that no 16-byte load divides: the element-wise paths of every kernel, prompt and decode"""
    cfg = config([cdelta(heads=3, kv_heads=1, dim=11, vdim=13, conv=3, mlp=moe(5, 2, 27)), mlstm(heads=3, dim=7, vdim=5, mlp=dense(15)),
                  par(heads=3, kv_heads=1, dim=10, vdim=13, size=11, dims=6, rheads=3, rkv=3, rdim=9, rvdim=7, rconv=5, mlp=moe(3, 2, 9)), cdelta(heads=3, kv_heads=1, dim=11, vdim=13, conv=3, mlp=moe(5, 2, 27),
                                                                                                                                weights_of=0)], vocab=77, width=50)
    w = weights(cfg, 13, rank=3)
    t = toks(100, cfg["vocab"], 18)
    want = logits_of(cfg, f64(w), t)
    sv = Served(cfg, w, dev, dtype)
    got = sv.step([(1, t[:67])]) + sv.step([(1, t[67:90])]) + [sv.step([(1, [x])])[0] for x in t[90:]]
    assert close(torch.cat(got), want, bar)


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_greedy_generation_through_scheduler_and_engine(dev, graphs):
    """the package's own entry point: scheduler (pages + slots), engine, sampler; five prompts through three slots, against greedy decoding of the restatement"""
    from mistralrs_amd.cli import make_engine
    from mistralrs_amd.hybrid import HybridDecoder, gifopel_spec
    from mistralrs_amd.sampler import SequenceSampler
    from mistralrs_amd.scheduler import Sequence
    cfg = config([mlstm(), par(), cdelta(), par(weights_of=1, mlp="moe")])
    w = weights(cfg, 10)
    m = HybridDecoder(gifopel_spec(cfg), dev, "float32", num_blocks=12, block_size=32, state_slots=3)
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
            lg = logits_of(cfg, wd, ref)[-1]
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
    cfg = config([par(), mlstm(mlp=None), cdelta(), par(weights_of=0)])
    w = weights(cfg, 12)
    folder = tmp_path / "model"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(folder / "model.safetensors"))
    assert registry.architecture_of(str(folder)) == "Gifopel"
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
    full = {r: logits_of(cfg, wd, t) for r, t in reqs.items()}
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
            lg = logits_of(cfg, wd, ref)[-1]
            t2 = torch.topk(lg, 2).values
            if float(t2[0] - t2[1]) < 1e-3:
                break
            ref.append(int(lg.argmax()))
        assert line["error"] is None and line["tokens"][:len(ref) - len(p)] == ref[len(p):]
