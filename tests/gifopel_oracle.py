"""TEST INFRASTRUCTURE: a plain, slow restatement of the Gifopel decoder, one function per mechanism, in float64 on the CPU: layers whose mixer and feed-forward read two
norms of the SAME residual row and join it together, a gated delta-rule mixer (short causal convolutions with SiLU on q / k / v, unit-length queries and keys, per-head or
per-key-channel decays, a written-then-read outer-product state, a per-head output norm with a sigmoid or SiLU gate), a matrix-memory mixer with exponential gates and a
running stabiliser (mLSTM), a mixer that averages two normed sub-mixers (attention inside position chunks with a learned per-head sink, per-head query / key norms,
interleaved rotary and a per-head output gate, next to a delta-rule mixer), dense SiLU-GLU feed-forwards and routed squared-ReLU experts whose weights are a softmax over the
chosen logits, layers that borrow another layer's tensors, and a head tied to the embedding.  Shares no code with the product path (mistral.rs_amd/hybrid.py, csrc/hyb_*.hip).

A model is `(cfg, w)`: `cfg` the parsed config dictionary, `w` a dict name -> float64 torch tensor.  Every mixer takes the rows of ONE sequence [T, ...] and the state the
sequence carried before them (None: a fresh sequence), and returns its output and the new state, so the same functions restate whole prompts and token-by-token decoding.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x, eps):
    return torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return x / rms(x, eps) * w


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.clamp(x, min=0.0) + torch.log1p(torch.exp(-x.abs()))


def logsigmoid(x):
    return -softplus(-x)


# ------------------------------------------------------------------------------------------------------------------ short convolution
def conv_silu(u, cw, before):
    """u [T, C], cw [C, taps] (the LAST column multiplies the current row), before [taps - 1, C] = the rows that came before u (None: zeros).  Returns silu(conv) and the
    last taps - 1 rows of (before ++ u)."""
    T, C = u.shape
    taps = cw.shape[1]
    if before is None:
        before = torch.zeros(taps - 1, C, dtype=F)
    full = torch.cat([before, u], 0)
    y = torch.zeros(T, C, dtype=F)
    for j in range(taps):
        y = y + cw[:, j] * full[j:j + T]
    return silu(y), full[full.shape[0] - (taps - 1):]


# ------------------------------------------------------------------------------------------------------------------ gated delta rule
def delta_rule(q, k, v, beta, g, S):
    """q, k [T, H, D]; v [T, H, Dv]; beta [T, H]; g [T, H, D] (a decay per key channel; a per-head decay is the same number in every channel); S [H, D, Dv].
    Per row: S <- g S (rows of S scaled); u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, _ = q.shape
    S = S.clone()
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for t in range(T):
        for h in range(H):
            Sh = S[h] * g[t, h][:, None]
            u = beta[t, h] * (v[t, h] - Sh.T @ k[t, h])
            Sh = Sh + torch.outer(k[t, h], u)
            out[t, h] = Sh.T @ q[t, h]
            S[h] = Sh
    return out, S


def delta_mixer(h, w, p, m, eps, state, channel_decay):
    """The whole mixer on rows h [T, W] with tensors `p + name`.  channel_decay: decays per (head, key channel) from a two-step projection and a sigmoid gate from a two-step
    projection; else one decay per head from one projection and a SiLU gate from a full projection.  state = (taps of q, k, v; S) or None."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    taps_in = state[0] if state is not None else (None, None, None)
    S = state[1] if state is not None else torch.zeros(H, D, Dv, dtype=F)
    q, tq = conv_silu(h @ w[p + "q"].T, w[p + "q.conv"], taps_in[0])
    k, tk = conv_silu(h @ w[p + "k"].T, w[p + "k.conv"], taps_in[1])
    v, tv = conv_silu(h @ w[p + "v"].T, w[p + "v.conv"], taps_in[2])
    q, k, v = q.view(T, G, D), k.view(T, G, D), v.view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)     # head h reads q / k head h // rep
    beta = torch.sigmoid(h @ w[p + "b"].T)
    rate = torch.exp(w[p + "A_log"])                                    # [H]
    if channel_decay:
        step = softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).view(T, H, D)
        g = torch.exp(-rate[None, :, None] * step)
        gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, Dv)
    else:
        step = softplus(h @ w[p + "a"].T + w[p + "dt_bias"])            # [T, H]
        g = torch.exp(-rate[None, :] * step)[:, :, None].expand(T, H, D)
        gate = silu(h @ w[p + "g"].T).view(T, H, Dv)
    o, S = delta_rule(q, k, v, beta, g, S)
    o = o / rms(o, eps) * w[p + "norm"] * gate
    return o.reshape(T, H * Dv) @ w[p + "o"].T, ((tq, tk, tv), S)


# ------------------------------------------------------------------------------------------------------------------ matrix memory with exponential gates
def mlstm_cell(q, k, v, ig, fg, state):
    """q, k [T, H, D]; v [T, H, Dv]; ig, fg [T, H] log gates; state = (S [H, D, Dv], n [H, D], m [H]).  m' = max(fg + m, ig); S' = e^{fg + m - m'} S + e^{ig - m'} k v^T;
    n' likewise with k; o = S'^T q / (max(|n' . q|, e^{-m'}) + 1e-6)."""
    T, H, _ = q.shape
    S, n, m = (t.clone() for t in state)
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for t in range(T):
        m_new = torch.maximum(fg[t] + m, ig[t])
        keep, put = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
        S = keep[:, None, None] * S + put[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + put[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = num / den[:, None]
    return out, (S, n, m)


def mlstm_mixer(h, w, p, m, eps, state):
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    if state is None:
        state = (torch.zeros(H, D, Dv, dtype=F), torch.zeros(H, D, dtype=F), torch.zeros(H, dtype=F))
    q = (h @ w[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, Dv)
    ig = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    fg = logsigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    o, state = mlstm_cell(q, k, v, ig, fg, state)
    o = (o / rms(o, eps)).reshape(T, H * Dv) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T, state


# ------------------------------------------------------------------------------------------------------------------ attention inside chunks, with a learned sink
def rotary_interleaved(x, pos, dims, base):
    """x [T, H, D]: in the first `dims` of every head the pair (2i, 2i + 1) turns by pos * base^(-2i / dims)."""
    if not dims:
        return x
    i = torch.arange(dims // 2, dtype=F)
    ang = pos.to(F)[:, None] * (float(base) ** (-2.0 * i / dims))[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    y = x.clone()
    y[..., 0:dims:2] = a * c - b * s
    y[..., 1:dims:2] = b * c + a * s
    return y


def chunk_attention(h, w, p, m, eps, state, pos0):
    """state = (keys [P, G, D], values [P, G, Dv]) of the positions before these rows (None: none).  Position i sees j <= i of its own chunk floor(i / size); the softmax's
    denominator has one more term e^{sink_h}; head h's output is multiplied by sigmoid(Wg h)_h."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(pos0, pos0 + T)
    q = norm_plain((h @ w[p + "q"].T).view(T, H, D), w[p + "q.norm"], eps)
    k = norm_plain((h @ w[p + "k"].T).view(T, G, D), w[p + "k.norm"], eps)
    v = (h @ w[p + "v"].T).view(T, G, Dv)
    rot = m.get("rot") or {}
    q = rotary_interleaved(q, pos, int(rot.get("dims", 0) or 0), rot.get("base", 1.0))
    k = rotary_interleaved(k, pos, int(rot.get("dims", 0) or 0), rot.get("base", 1.0))
    if state is not None:
        k, v = torch.cat([state[0], k], 0), torch.cat([state[1], v], 0)
    size = int((m.get("mask") or {}).get("size", 0) or 0)
    gate = torch.sigmoid(h @ w[p + "g"].T)                                # [T, H]
    out = torch.zeros(T, H, Dv, dtype=F)
    for t in range(T):
        i = pos0 + t
        lo = (i // size) * size if size else 0
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo:i + 1, g] @ q[t, hh]) * float(m["scale"])
            top = torch.maximum(s.max(), w[p + "sink"][hh])
            e = torch.exp(s - top)
            out[t, hh] = (e[:, None] * v[lo:i + 1, g]).sum(0) / (e.sum() + torch.exp(w[p + "sink"][hh] - top)) * gate[t, hh]
    return out.reshape(T, H * Dv) @ w[p + "o"].T, (k, v)


def parallel_mixer(h, w, p, m, eps, state, pos0):
    """Half the sum of the two sub-mixers' outputs, each normed over the model width with its own plain weight."""
    sl, sr = state if state is not None else (None, None)
    left, sl = chunk_attention(h, w, p + "left.", m["left"], eps, sl, pos0)
    right, sr = delta_mixer(h, w, p + "right.", m["right"], eps, sr, channel_decay=False)
    return 0.5 * (norm_plain(left, w[p + "left.out"], eps) + norm_plain(right, w[p + "right.out"], eps)), (sl, sr)


# ------------------------------------------------------------------------------------------------------------------ feed-forwards
def glu_ff(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, f):
    """The chosen experts of every row and their weights: the `top` largest logits (ties: the lower index), softmax over the chosen logits only."""
    z = h @ w[p + "router"].T + w[p + "router.b"]
    top = int(f["router"]["top"])
    order = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.softmax(torch.gather(z, 1, order), -1)


def moe_ff(h, w, p, f):
    ids, wts = route(h, w, p, f)
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            a = torch.clamp(w[f"{p}e{e}.up"] @ h[t], min=0.0) ** 2
            out[t] += wts[t, j] * (w[f"{p}e{e}.down"] @ a)
    return out


# ------------------------------------------------------------------------------------------------------------------ the model
def mixer(kind, h, w, p, m, eps, state, pos0):
    if kind == "channel_delta":
        return delta_mixer(h, w, p, m, eps, state, channel_decay=True)
    if kind == "mlstm":
        return mlstm_mixer(h, w, p, m, eps, state)
    if kind == "parallel":
        return parallel_mixer(h, w, p, m, eps, state, pos0)
    raise ValueError(kind)


def forward(cfg, w, tokens, states=None, pos0=0):
    """Rows `tokens` of one sequence that starts them at position pos0 with the per-layer states `states` (None: fresh).  Returns (logits [T, vocab], the residual stream
    after every layer [L, T, W], new states)."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    states = list(states) if states is not None else [None] * len(cfg["layers"])
    after = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{L.get('weights_of', i)}."
        y, states[i] = mixer(L["type"], norm_plain(x, w[p + "norm1"], eps), w, p + "mix.", L["mixer"], eps, states[i], pos0)
        f = L.get("mlp")
        if f:
            h2 = norm_plain(x, w[p + "norm2"], eps)
            y = y + (glu_ff(h2, w, p + "mlp.") if f["kind"] == "dense" else moe_ff(h2, w, p + "mlp.", f))
        x = x + y
        after.append(x)
    return norm_plain(x, w["final.norm"], eps) @ w["embed"].T, torch.stack(after), states
