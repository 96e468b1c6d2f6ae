"""A plain, slow Pafivik: whole sequences, no cache, one function per mechanism.

It shares no code with the engine.  Every function works on one sequence, [tokens, ...] torch tensors on
the CPU, in the precision of the tensors it is given (float32, or float64 to see how much of a
difference is rounding).  Weights come as a dict from tensor name to tensor; `cfg` is config.json as a
dict.

Notation: T tokens, W the model's width, H heads, G heads of queries and keys where they are fewer; `p(name)`
is a layer's tensor.
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


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def xielu(z, pq):
    """pq = (p, q).  z > 0: softplus(p) z^2 + z / 2;  else: (1/2 + softplus(q)) (e^z - 1 - z) + z / 2."""
    ap, aq = softplus(pq[0]), 0.5 + softplus(pq[1])
    neg = torch.clamp(z, max=0)
    return torch.where(z > 0, ap * z * z + 0.5 * z, aq * (torch.expm1(neg) - neg) + 0.5 * z)


def causal_taps(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_(t - taps + 1 + j), the last column weighs the token itself;
    nothing before the first token."""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def turn_pairs(x, positions, base, dims):
    """x [T, n, d]: of each vector's first `dims` entries, entry 2i and 2i+1 are turned by the angle
    position * base^(-2i/dims); the rest stay."""
    out = x.clone()
    if dims == 0:
        return out
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

def lightning(h, p, m, eps):
    """A matrix per head that fades by a constant of the head: S <- decay_h S + k v^T, o = S^T q, with q, k, v
    through silu; all heads' o normed as one vector, gated by sigmoid(W_g h), projected."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ p("mix.q").T).view(T, H, dk)
    k = silu(h @ p("mix.k").T).view(T, H, dk)
    v = silu(h @ p("mix.v").T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, dk, dv, dtype=h.dtype)
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    y = rms_norm(o.reshape(T, H * dv), p("mix.norm"), eps) * torch.sigmoid(h @ p("mix.g").T)
    return y @ p("mix.o").T


def channel_delta(h, p, m, eps):
    """The delta rule with a decay per head and key channel.  q and k (G heads) and v (H heads) pass a short
    convolution over time and silu; q and k become unit vectors, q times dim^(-1/2).  Per head:
    S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rep = H // G
    q = silu(causal_taps(h @ p("mix.q").T, p("mix.q.conv"))).view(T, G, dk)
    k = silu(causal_taps(h @ p("mix.k").T, p("mix.k.conv"))).view(T, G, dk)
    v = silu(causal_taps(h @ p("mix.v").T, p("mix.v.conv"))).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ p("mix.b").T)                                   # [T, H]
    step = softplus((h @ p("mix.a1").T) @ p("mix.a2").T + p("mix.dt_bias")).view(T, H, dk)
    g = torch.exp(-torch.exp(p("mix.A_log"))[None, :, None] * step)         # [T, H, dk]
    S = torch.zeros(H, dk, dv, dtype=h.dtype)
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        qt = q[t].repeat_interleave(rep, dim=0)
        kt = k[t].repeat_interleave(rep, dim=0)
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, kt))
        S = S + kt[:, :, None] * u[:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, qt)
    gate = torch.sigmoid((h @ p("mix.g1").T) @ p("mix.g2").T).view(T, H, dv)
    y = rms_norm(o, p("mix.norm"), eps) * gate
    return y.reshape(T, H * dv) @ p("mix.o").T


def attention(h, p, m):
    """Causal softmax attention; G key heads for H query heads, keys `dim` and values `vdim` wide, biases on q, k, v,
    pairs of the first rot.dims entries of q and k turned by the position."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rep = H // G
    pos = torch.arange(T)
    q = (h @ p("mix.q").T + p("mix.q.b")).view(T, H, dk)
    k = (h @ p("mix.k").T + p("mix.k.b")).view(T, G, dk)
    v = (h @ p("mix.v").T + p("mix.v.b")).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        q = turn_pairs(q, pos, rot["base"], rot["dims"])
        k = turn_pairs(k, pos, rot["base"], rot["dims"])
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        for hh in range(H):
            s = (k[:t + 1, hh // rep] @ q[t, hh]) * m["scale"]
            out[t, hh] = torch.softmax(s, dim=0) @ v[:t + 1, hh // rep]
    return out.reshape(T, H * dv) @ p("mix.o").T


# ----------------------------------------------------------------------------
# feed-forwards
# ----------------------------------------------------------------------------

def dense_ff(h, p):
    return xielu(h @ p("mlp.up").T + p("mlp.up.b"), p("mlp.act")) @ p("mlp.down").T + p("mlp.down.b")


def gated_ff(h, p, name):
    return (silu(h @ p(name + ".gate").T) * (h @ p(name + ".up").T)) @ p(name + ".down").T


def expert_ff(h, p, mlp):
    """Scores sigmoid(W_router h); the `top` largest are a token's experts, their scores its weights as they are;
    a weight multiplies what the expert reads.  A shared expert, if any, is added times sigmoid(W_sg h)."""
    T = h.shape[0]
    top = mlp["router"]["top"]
    s = torch.sigmoid(h @ p("mlp.router").T)
    out = torch.zeros_like(h)
    for t in range(T):
        val, idx = torch.topk(s[t], top)
        for w, e in zip(val, idx):
            out[t] += gated_ff((w * h[t])[None], p, f"mlp.e{int(e)}")[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, p, "mlp.shared") * torch.sigmoid(h @ p("mlp.shared.sg").T)
    return out


# ----------------------------------------------------------------------------
# the model
# ----------------------------------------------------------------------------

def forward(cfg, weights, tokens, dtype=torch.float32, streams=None):
    """-> logits [T, vocab].  streams: a list that receives the stream after every layer (after the averaging)."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    history = [x]
    for i, layer in enumerate(cfg["layers"]):
        p = lambda name, i=i: W[f"l{i}.{name}"]       # noqa: E731
        h = rms_norm(x, p("norm1"), eps)
        if layer["type"] == "lightning":
            y = lightning(h, p, layer["mixer"], eps)
        elif layer["type"] == "channel_delta":
            y = channel_delta(h, p, layer["mixer"], eps)
        else:
            y = attention(h, p, layer["mixer"])
        x = x + m * (rms_norm(y, p("norm1b"), eps) * p("ls1"))
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, p("norm2"), eps)
            y = dense_ff(h, p) if mlp["kind"] == "dense" else expert_ff(h, p, mlp)
            x = x + m * (rms_norm(y, p("norm2b"), eps) * p("ls2"))
        history.append(x)
        x = sum(p("dwa")[j] * history[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x)
    return rms_norm(x, W["final.norm"], eps) @ W["embed"].T
