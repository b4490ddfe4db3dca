"""The Zarinex decoder as a plain function of a whole sequence, in double precision: one function
per mechanism, no cache, no batching, no kernels.  What the engine computes is held against this.

Notation: h [T, D] rows of one sequence in order; W a dict of arrays by tensor name; weights are
stored [out, in] and applied as W x.

    x0        = embed[token] + pe(position)        pe[2i] = sin(p b^(-2i/D)), pe[2i+1] = cos(p b^(-2i/D)), b = 10000
    layer     : u = mixer(shifted(x)) * sigmoid(Rg1 x + b1);  x = rms(alpha x + u) w1
                u = ff(x) * sigmoid(Rg2 x + b2);               x = rms(alpha x + u) w2      (if it has a feed-forward)
    shifted(x)= x + (x_prev - x) * mu                x_prev: the row before, zeros before the first
    logits    = embed @ rms(x) w_final
"""
from __future__ import annotations

import math

import numpy as np


def rms_norm(x, w, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def position_rows(positions, width, base=10000.0):
    pe = np.zeros((len(positions), width))
    for r, p in enumerate(positions):
        for c in range(width):
            angle = p * base ** (-(2 * (c // 2)) / width)
            pe[r, c] = math.sin(angle) if c % 2 == 0 else math.cos(angle)
    return pe


def token_shift(h, mu):
    prev = np.vstack([np.zeros((1, h.shape[1])), h[:-1]])
    return h + (prev - h) * mu


def causal_conv(x, weight, bias):
    """y[t, c] = bias[c] + sum_j weight[c, taps-1-j] x[t-j, c]: the last column meets the current token."""
    T, C = x.shape
    taps = weight.shape[1]
    y = np.tile(bias, (T, 1)).astype(np.float64)
    for t in range(T):
        for j in range(taps):
            if t - j >= 0:
                y[t] += weight[:, taps - 1 - j] * x[t - j]
    return y


def mamba1(h, W, p, m):
    """Selective scan.  m: {inner, state, dt_rank, conv}."""
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ W[p + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, W[p + "conv"], W[p + "conv.b"]))
    low = x @ W[p + "x"].T
    dt = softplus(low[:, :R] @ W[p + "dt"].T + W[p + "dt.b"])
    B, C = low[:, R:R + N], low[:, R + N:R + 2 * N]
    A = -np.exp(W[p + "A_log"])                      # [inner, N]
    S = np.zeros((inner, N))
    y = np.zeros_like(x)
    for t in range(h.shape[0]):
        S = np.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + W[p + "D"] * x[t]
    return (y * silu(z)) @ W[p + "o"].T


def latent_attention(h, W, p, m, eps):
    """Attention through latents, no positions.  m: {heads, dim, vdim, kv_rank, q_rank, scale}."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).reshape(T, H, d)
    c = rms_norm(h @ W[p + "dkv"].T, W[p + "dkv.norm"], eps)
    k = (c @ W[p + "uk"].T).reshape(T, H, d)
    v = (c @ W[p + "uv"].T).reshape(T, H, dv)
    out = np.zeros((T, H, dv))
    for i in range(T):
        s = np.einsum("hd,jhd->hj", q[i], k[:i + 1]) * m["scale"]
        s = np.exp(s - s.max(axis=1, keepdims=True))
        s /= s.sum(axis=1, keepdims=True)
        out[i] = np.einsum("hj,jhe->he", s, v[:i + 1])
    out = out.reshape(T, H * dv) * sigmoid(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


def hgrn2(h, W, p, m, eps):
    """A matrix state per head whose forget gate also weighs what is written.  m: {heads, dim, vdim}."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ W[p + "q"].T).reshape(T, H, d)
    v = (h @ W[p + "v"].T).reshape(T, H, dv)
    low = W[p + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).reshape(T, H, d)
    S = np.zeros((H, d, dv))
    o = np.zeros((T, H, dv))
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hde,hd->he", S, q[t])
    o = rms_norm(o, W[p + "norm"], eps)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def gated_expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def routed_experts(h, W, p, mlp):
    """Each row goes to the `top` experts with the largest router logits, weighted by the softmax
    over those logits alone; a shared expert, if there is one, takes every row."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ W[p + "router"].T + W[p + "router.b"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = np.argsort(-z[t], kind="stable")[:top]
        w = np.exp(z[t, chosen] - z[t, chosen].max())
        w /= w.sum()
        for e, we in zip(chosen, w):
            out[t] += we * gated_expert(h[t:t + 1], W, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out += gated_expert(h, W, p + "shared.")
    return out


def router_margins(h, W, p, mlp):
    """Per row, how far the last picked logit lies above the first one that is not picked (inf where
    every expert is picked): a row with a small margin may pick otherwise after a rounding."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    if top >= E:
        return np.full(h.shape[0], np.inf)
    z = -np.sort(-(h @ W[p + "router"].T + W[p + "router.b"]), axis=1)
    return z[:, top - 1] - z[:, top]


MIXERS = {"mamba1": lambda h, W, p, m, eps: mamba1(h, W, p, m), "latent_attention": latent_attention, "hgrn2": hgrn2}


def layer(x, W, p, entry, alpha, eps, margins=None):
    u = MIXERS[entry["type"]](token_shift(x, W[p + "shift"]), W, p + "mix.", entry["mixer"], eps)
    u = u * sigmoid(x @ W[p + "rg1"].T + W[p + "rg1.b"])
    x = rms_norm(alpha * x + u, W[p + "norm1"], eps)
    if entry.get("mlp"):
        if margins is not None:
            margins.append(router_margins(x, W, p + "mlp.", entry["mlp"]))
        u = routed_experts(x, W, p + "mlp.", entry["mlp"]) * sigmoid(x @ W[p + "rg2"].T + W[p + "rg2.b"])
        x = rms_norm(alpha * x + u, W[p + "norm2"], eps)
    return x


def forward(config: dict, W: dict, tokens, return_layers: bool = False, margins: list | None = None):
    """logits [T, vocab] of one sequence from its first token; with return_layers also the rows
    after every layer run; `margins` collects every routed layer run's margins per row."""
    W = {k: np.asarray(v, np.float64) for k, v in W.items()}
    D, eps, alpha = config["width"], config["norm"]["eps"], config["postln_alpha"]
    x = W["embed"][np.asarray(tokens)] + position_rows(range(len(tokens)), D)
    after = []
    for i, entry in enumerate(config["layers"]):
        owner = entry.get("weights_of")
        x = layer(x, W, f"l{i if owner is None else owner}.", entry, alpha, eps, margins)
        after.append(x)
    logits = rms_norm(x, W["final.norm"], eps) @ W["embed"].T
    return (logits, np.stack(after)) if return_layers else logits
