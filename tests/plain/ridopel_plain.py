"""A plain, slow Ridopel: whole sequences, no cache, one function per mechanism.

It shares no code with the engine.  Every function works on one sequence, [tokens, ...] torch tensors on
the CPU, in the precision of the tensors it is given (float32, or float64 to see how much of a
difference is rounding).  Weights come as a dict from tensor name to tensor; `cfg` is config.json as a
dict.

Notation: T tokens, W the model's width, H heads; `p(name)` is a layer's tensor.
"""
from __future__ import annotations

import math

import torch


# ----------------------------------------------------------------------------
# small pieces
# ----------------------------------------------------------------------------

def rms_norm(x, weight, eps):
    """y = x / sqrt(mean(x^2) + eps) [* weight], over the last dimension."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def short_conv(h, w):
    """h [T, W], w [W, taps]: y_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j); nothing before the first token."""
    T, taps = h.shape[0], w.shape[1]
    y = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * h[s]
    return y


def turn_pairs(x, positions, base, dims):
    """x [T, n, d]: of each vector's first `dims` entries, entry 2i and 2i+1 are turned by the angle
    position * base^(-2i/dims); the rest stay."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    ang = positions.to(torch.float64)[:, None] * freq[None, :]
    cos, sin = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


# ----------------------------------------------------------------------------
# mixers
# ----------------------------------------------------------------------------

def latent_attention(h, p, m, eps):
    """Keys and values are made from one small vector per token (c, kv_rank wide) and one turned key part
    that all heads share; each query head has an unturned part against W_uk c and a turned part."""
    T = h.shape[0]
    H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ p("mix.q").T).view(T, H, dn + dr)
    q_plain, q_turn = q[..., :dn], q[..., dn:]
    low = h @ p("mix.dkv").T
    c = rms_norm(low[:, :rank], p("mix.dkv.norm"), eps)
    k_turn = low[:, rank:].view(T, 1, dr)
    rot = m["rot"]
    q_turn = turn_pairs(q_turn, pos, rot["base"], rot["dims"])
    k_turn = turn_pairs(k_turn, pos, rot["base"], rot["dims"])[:, 0]
    k_plain = (c @ p("mix.uk").T).view(T, H, dn)
    v = (c @ p("mix.uv").T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        s = (torch.einsum("hd,jhd->hj", q_plain[t], k_plain[:t + 1])
             + torch.einsum("hd,jd->hj", q_turn[t], k_turn[:t + 1])) * m["scale"]
        a = torch.softmax(s, dim=-1)
        out[t] = torch.einsum("hj,jhd->hd", a, v[:t + 1])
    gate = torch.sigmoid(h @ p("mix.g").T)
    return (out.reshape(T, H * dv) * gate) @ p("mix.o").T


def wkv(h, p, m, eps):
    """A matrix state per head with a decay per key channel that the token itself decides; the current
    token's own key-value product counts with a bonus u and only for itself."""
    T, W = h.shape
    H, d = m["heads"], m["dim"]
    before = torch.cat([torch.zeros(1, W, dtype=h.dtype), h[:-1]], dim=0)

    def mixed(s):
        return h + (before - h) * p("mix.mu." + s)
    r = (mixed("r") @ p("mix.r").T).view(T, H, d)
    k = (mixed("k") @ p("mix.k").T).view(T, H, d)
    v = (mixed("v") @ p("mix.v").T).view(T, H, d)
    gate = silu(mixed("g") @ p("mix.g").T)
    decay = torch.exp(-torch.exp(torch.tanh(mixed("w") @ p("mix.w1").T) @ p("mix.w2").T + p("mix.w0"))).view(T, H, d)
    u = p("mix.u")
    S = torch.zeros(H, d, d, dtype=h.dtype)
    out = torch.zeros(T, H, d, dtype=h.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hi,hij->hj", r[t], S + u[:, :, None] * kv)
        S = decay[t][:, :, None] * S + kv
    out = rms_norm(out, None, eps).reshape(T, H * d) * p("mix.norm") * gate
    return out @ p("mix.o").T


def hgrn2(h, p, m, eps):
    """A matrix state per head whose forget gate f also decides what is written: row i keeps f_i of itself and
    takes 1 - f_i of the new value."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ p("mix.q").T).view(T, H, d)
    v = (h @ p("mix.v").T).view(T, H, dv)
    low = p("mix.lower")
    f = (low + (1.0 - low) * torch.sigmoid(h @ p("mix.f").T + p("mix.f.b"))).view(T, H, d)
    S = torch.zeros(H, d, dv, dtype=h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hi,hij->hj", q[t], S)
    out = rms_norm(out, p("mix.norm"), eps).reshape(T, H * dv)
    return out @ p("mix.o").T


MIXERS = {"latent_attention": latent_attention, "wkv": wkv, "hgrn2": hgrn2}


# ----------------------------------------------------------------------------
# feed-forward
# ----------------------------------------------------------------------------

def expert(h, gate_w, up_w, down_w, limit):
    g = torch.clamp(h @ gate_w.T, max=limit)
    u = torch.clamp(h @ up_w.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down_w.T


def routed_experts(h, p, f):
    """Each token takes its `top` experts by softmax score + correction and weighs them by their softmax
    scores alone, made to add up to one."""
    n, top, limit = f["router"]["experts"], f["router"]["top"], f["expert"]["limit"]
    s = torch.softmax(h @ p("mlp.router").T, dim=-1)
    chosen = torch.topk(s + p("mlp.correction"), top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        ws = s[t, chosen[t]]
        ws = ws / (ws.sum() + 1e-20)
        for e, wt in zip(chosen[t].tolist(), ws):
            out[t] += wt * expert(h[t], p(f"mlp.e{e}.gate"), p(f"mlp.e{e}.up"), p(f"mlp.e{e}.down"), limit)
    return out


# ----------------------------------------------------------------------------
# the model
# ----------------------------------------------------------------------------

def run_order(cfg):
    """[(layer, first of a pass)] in the order in which layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg, weights, tokens, dtype=torch.float32, keep_layers=False):
    """-> logits [T, vocab] (and the residual stream after every layer run, [runs, T, W])."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = rms_norm(w["embed"][torch.as_tensor(tokens)], w["embed.norm"], eps)
    x0 = x
    streams = []
    for i, first in run_order(cfg):
        layer = cfg["layers"][i]

        def p(name, i=i):
            return w[f"l{i}.{name}"]
        if first:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        h = rms_norm(x, p("norm1"), eps)
        if cfg.get("canon"):
            h = short_conv(h, p("canon1"))
        x = x + MIXERS[layer["type"]](h, p, layer["mixer"], eps)
        if layer.get("mlp"):
            x = x + routed_experts(rms_norm(x, p("norm2"), eps), p, layer["mlp"])
        streams.append(x)
    x = rms_norm(x, w["final.norm"], eps)
    logits = x @ w["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return (logits, torch.stack(streams)) if keep_layers else logits
