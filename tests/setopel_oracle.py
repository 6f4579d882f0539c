"""TEST INFRASTRUCTURE: a plain, slow restatement of the Setopel decoder, one function per mechanism, in float64 on the CPU: several residual streams that every sublayer
reads through a weighted sum and writes back through a mixing matrix (hyper-connections), an attention mixer with projection biases, a short causal convolution on q / k / v,
a query temperature, tanh-capped scores, a softmax with a zero-score sink and an elementwise sigmoid gate (optionally reading another layer's keys and values), a retention
mixer (decayed outer-product state, half-split rotary, per-head unit norm, SiLU gate), a latent attention mixer (keys and values expanded from one normed low-rank row),
and a SiLU-GLU feed-forward.  Shares no code with the product path (mistral.rs_amd/hybrid.py and csrc/hyb_*.hip).

A model is `(cfg, w)`: `cfg` the parsed config dictionary, `w` a dict name -> float64 torch tensor.  Everything works on one whole sequence [T, ...], positions 0 .. T-1.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x, eps):
    return torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """x / rms(x) * (1 + w)"""
    return x / rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return x / rms(x, eps) * w


def causal_conv(u, cw):
    """u [T, C], cw [C, taps]: y[t] = sum_j cw[:, j] u[t - (taps - 1) + j], zeros before the start (the LAST tap multiplies the current token)."""
    T, C = u.shape
    taps = cw.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F), u], 0)
    y = torch.zeros(T, C, dtype=F)
    for j in range(taps):
        y = y + cw[:, j] * pad[j:j + T]
    return y


def query_temperature(T, coef, every):
    """Factor on the query at position p: 1 + coef ln(floor((p + 1) / every) + 1)."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in range(T)], dtype=F)


def attention_kv(h, w, p, m):
    """Keys [T, G, D] and values [T, G, Dv] of a layer with projections of its own: bias, then the convolution when the layer has one."""
    T = h.shape[0]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    if m.get("conv"):
        k, v = causal_conv(k, w[p + "k.conv"]), causal_conv(v, w[p + "v.conv"])
    return k.view(T, m["kv_heads"], m["dim"]), v.view(T, m["kv_heads"], m["vdim"])


def sink_attention(h, k, v, w, p, m):
    """Causal grouped-head attention: s = cap tanh(scale (q . k) / cap) (no cap: s = scale q . k); p_j = e^{s_j} / (1 + sum_j' e^{s_j'}); heads concatenated,
    times sigmoid(Wg h) element by element, then the output projection."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    if m.get("conv"):
        q = causal_conv(q, w[p + "q.conv"])
    q = q.view(T, H, D)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, float(qt["coef"]), int(qt["every"])).view(T, 1, 1)
    cap = float(m.get("softcap") or 0.0)
    rep = H // G
    seen = torch.arange(T).view(1, T) <= torch.arange(T).view(T, 1)
    heads = []
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh // rep].T) * float(m["scale"])
        if cap:
            s = cap * torch.tanh(s / cap)
        e = torch.exp(s) * seen
        heads.append((e / (1.0 + e.sum(-1, keepdim=True))) @ v[:, hh // rep])
    o = torch.cat(heads, -1) * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def rotate_half(x, dims, base):
    """x [T, heads, D]: in the first `dims` dimensions, (x_i, x_{i + dims/2}) turns by the angle t * base^(-2 i / dims); the rest passes."""
    if not dims:
        return x
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = torch.arange(T, dtype=F).view(T, 1, 1) * f
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def retention(h, w, p, m, eps, state=None):
    """Per head: S_t = decay S_{t-1} + k_t v_t^T, o_t = S_t^T q_t, o_t / rms(o_t); heads concatenated, times silu(Wg h), projected.  `state` [H, D, Dv]: the start (zeros)."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    dims, base = int(rot.get("dims", 0) or 0), float(rot.get("base", 1.0))
    q = rotate_half((h @ w[p + "q"].T).view(T, H, D), dims, base)
    k = rotate_half((h @ w[p + "k"].T).view(T, H, D), dims, base) * D ** -0.5
    v = (h @ w[p + "v"].T).view(T, H, Dv)
    S = torch.zeros(H, D, Dv, dtype=F) if state is None else state.clone()
    dec = torch.tensor([float(d) for d in m["decay"]], dtype=F).view(H, 1, 1)
    o = torch.zeros(T, H, Dv, dtype=F)
    for t in range(T):
        S = dec * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = o / rms(o, eps)
    g = h @ w[p + "g"].T
    return (o.reshape(T, H * Dv) * (g * torch.sigmoid(g))) @ w[p + "o"].T


def latent_attention(h, w, p, m, eps):
    """c = norm_plain(Wdkv h); per head k = Wuk c, v = Wuv c; causal softmax attention with s = scale q . k."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, D)
    c = norm_plain(h @ w[p + "dkv"].T, w[p + "dkv.norm"], eps)
    k = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, Dv)
    seen = torch.arange(T).view(1, T) <= torch.arange(T).view(T, 1)
    heads = []
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh].T) * float(m["scale"])
        s = s.masked_fill(~seen, -math.inf)
        heads.append(torch.softmax(s, -1) @ v[:, hh])
    return torch.cat(heads, -1) @ w[p + "o"].T


def glu_ff(h, w, p):
    g = h @ w[p + "gate"].T
    return ((g * torch.sigmoid(g)) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def hyper_read(xs, w_in):
    """xs [S, T, W]: the sublayer's input sum_s in[s] xs[s]."""
    return torch.einsum("s,stw->tw", w_in, xs)


def hyper_write(xs, y, mix, w_out, mult):
    """new[t] = sum_s mix[s, t] xs[s] + mult out[t] y, all from the old streams."""
    return torch.einsum("sr,stw->rtw", mix, xs) + mult * w_out.view(-1, 1, 1) * y.unsqueeze(0)


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence; layers_out (a list) receives the sum of the streams after every layer."""
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg.get("residual_mult", 1.0))
    S = cfg.get("streams")
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = norm_one_plus(x, w["embed.norm"], eps)
    xs = x.unsqueeze(0).repeat(int(S), 1, 1) if S else x.unsqueeze(0)
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        for q, sub in ((1, "mix"), (2, "mlp")):
            if sub == "mlp" and not L.get("mlp"):
                continue
            u = hyper_read(xs, w[f"{p}hc{q}.in"]) if S else xs[0]
            h = norm_one_plus(u, w[f"{p}norm{q}"], eps)
            if sub == "mlp":
                y = glu_ff(h, w, p + "mlp.")
            elif L["type"] == "attention":
                if m.get("kv_from") is not None:
                    k, v = kv[int(m["kv_from"])]
                else:
                    k, v = kv[i] = attention_kv(h, w, p + "mix.", m)
                y = sink_attention(h, k, v, w, p + "mix.", m)
            elif L["type"] == "retention":
                y = retention(h, w, p + "mix.", m, eps)
            elif L["type"] == "latent_attention":
                y = latent_attention(h, w, p + "mix.", m, eps)
            else:
                raise ValueError(L["type"])
            xs = hyper_write(xs, y, w[f"{p}hc{q}.mix"], w[f"{p}hc{q}.out"], mult) if S else xs + mult * y.unsqueeze(0)
        if layers_out is not None:
            layers_out.append(xs.sum(0))
    x = norm_one_plus(xs.sum(0), w["final.norm"], eps)
    return x @ w["head"].T
