"""A plain, slow Begopel in double precision on the CPU: one function per mechanism, written from
the design's equations and sharing no code with the library.  The tests hold the engine to it.

Notation: x[t] is the residual row of position t (positions count from 0), h the input of a
mixer, W matrices are [out, in] and applied as W h.  Everything is a loop over positions or a
dense matrix over all pairs of positions; nothing is cached, so prefill, decoding and batches
have one meaning: the function of the whole sequence.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance table for a key n positions back: one row per distance up to half of
    the rows, then rows spaced evenly in the logarithm of the distance up to `far`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def short_conv(x, w, bias=None):
    """x [T, C], w [C, taps]: y[t, c] = sum_j w[c, taps-1-j] x[t-j, c], with x[t] = 0 for t < 0."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            if t - j >= 0:
                y[t] += w[:, taps - 1 - j] * x[t - j]
    if bias is not None:
        y = y + bias
    return y


def sink_attention(h, W, cfg, eps):
    """Causal softmax attention whose scores get a learned bias by distance and whose denominator
    holds one more term exp(sink) per head; heads are gated by sigmoid(W_g h) before W_o."""
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = (h @ W["q"].T).view(T, H, d)
    k = (h @ W["k"].T).view(T, G, d)
    v = (h @ W["v"].T).view(T, G, dv)
    q = rms(q, eps) * W["q.norm"]
    k = rms(k, eps) * W["k.norm"]
    rel = W["rel"]
    rows = rel.shape[0]
    by_distance = torch.stack([rel[distance_bucket(n, rows, cfg["bias_max"])] for n in range(T)])     # [T, H]
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        sink = W["sink"][head]
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, head]) * cfg["scale"] + by_distance[:i + 1, head].flip(0)
            m = torch.maximum(s.max(), sink)
            e = torch.exp(s - m)
            den = e.sum() + torch.exp(sink - m)
            out[i, head] = (e[:, None] * v[: i + 1, g]).sum(0) / den
    gate = torch.sigmoid(h @ W["g"].T)
    return (out.reshape(T, H * dv) * gate) @ W["o"].T


def gated_delta(h, W, cfg, eps):
    """The gated delta rule: a matrix state per head that decays, is corrected towards the new
    value along the new key, and is read with the query after the write."""
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ W["q"].T, W["q.conv"])).view(T, G, d)
    k = silu(short_conv(h @ W["k"].T, W["k.conv"])).view(T, G, d)
    v = silu(short_conv(h @ W["v"].T, W["v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W["b"].T)
    decay = torch.exp(-torch.exp(W["A_log"]) * softplus(h @ W["a"].T + W["dt_bias"]))
    gate = silu(h @ W["g"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(d, dv, dtype=F)
        for t in range(T):
            S = decay[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, head] = S.T @ q[t, g]
    o = rms(o, eps) * W["norm"] * gate
    return o.reshape(T, H * dv) @ W["o"].T


def parallel_mixer(h, W, cfg, eps):
    left = sink_attention(h, {k[5:]: v for k, v in W.items() if k.startswith("left.") and k != "left.out"}, cfg["left"], eps)
    right = gated_delta(h, {k[6:]: v for k, v in W.items() if k.startswith("right.") and k != "right.out"}, cfg["right"], eps)
    return 0.5 * (rms(left, eps) * W["left.out"] + rms(right, eps) * W["right.out"])


def mamba2(h, W, cfg, eps):
    """State-space layer with a scalar decay per head: S_t = a_t S_(t-1) + dt_t B_t x_t^T,
    y_t = S_t^T C_t + D x_t, gated by silu(z) and normed in equal parts of the inner width."""
    H, P, N, G, parts = cfg["heads"], cfg["vdim"], cfg["state"], cfg["groups"], cfg["norm_groups"]
    inner = H * P
    T = h.shape[0]
    u = h @ W["in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, W["conv"], W["conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W["dt_bias"])
    a = torch.exp(-torch.exp(W["A_log"]) * dt)
    y = torch.zeros(T, H, P, dtype=F)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(N, P, dtype=F)
        for t in range(T):
            S = a[t, head] * S + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S.T @ C[t, g] + W["D"][head] * x[t, head]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W["norm"]
    return y @ W["o"].T


def relu2_mlp(h, W):
    return torch.relu(h @ W["up"].T) ** 2 @ W["down"].T


def one_plus_norm(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def layer_runs(config):
    """The layers in the order they run, as (layer index, pass number or None): the looped
    stretch `times` times in a row, then the rest."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            runs.append((i, t, i == loop["start"]))
    runs += [(i, None, False) for i in range(loop["stop"], n)]
    return runs


def forward(config, weights, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; `layers_out`: a list that takes the residual rows
    after every layer run."""
    W = {k: v.to(F) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    x0 = x.clone()
    for i, t, first in layer_runs(config):
        if first:
            x = torch.cat([x, x0], dim=-1) @ W["loop.in"].T + W["loop.step"][t]
        L = config["layers"][i]
        p = f"l{i}."
        mix = {k[len(p) + 4:]: v for k, v in W.items() if k.startswith(p + "mix.")}
        h = one_plus_norm(x, W[p + "norm1"], eps)
        if L["type"] == "parallel":
            x = x + parallel_mixer(h, mix, L["mixer"], eps)
        elif L["type"] == "mamba2":
            x = x + mamba2(h, mix, L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            h = one_plus_norm(x, W[p + "norm2"], eps)
            x = x + relu2_mlp(h, {"up": W[p + "mlp.up"], "down": W[p + "mlp.down"]})
        if layers_out is not None:
            layers_out.append(x.clone())
    h = one_plus_norm(x, W["final.norm"], eps)
    logits = h @ W["embed"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits
