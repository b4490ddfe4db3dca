"""Small Begopel configurations with weights made for the tests, their model folders, and the plain
model's logits for them.

The weights are not the library's random ones: every kind of tensor gets a spread that makes its
mechanism count (distance biases and sinks of order one, decays between 0.1 and 0.9, norm weights
away from their neutral value), and all are rounded to bfloat16 first, so that both runtimes and the
plain model read the same numbers.  The configurations differ from each other in every size, and
none has two sizes equal that the code could mix up (heads and key heads, key and value sizes,
groups, taps, rows of the distance table)."""
from __future__ import annotations

import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, scale, bias_max, bias_rows):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, bias_max=bias_max, bias_rows=bias_rows)


def delta(heads, kv_heads, dim, vdim, conv):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)


def parallel(left, right, ff):
    return dict(type="parallel", mixer=dict(left=left, right=right), mlp=None if ff is None else dict(kind="dense", ff=ff))


def mamba(heads, vdim, state, groups, norm_groups, conv, ff):
    return dict(type="mamba2", mixer=dict(heads=heads, vdim=vdim, state=state, groups=groups, norm_groups=norm_groups, conv=conv),
                mlp=None if ff is None else dict(kind="dense", ff=ff))


def config(vocab, width, layers, loop=None, scale=1.0, eps=1e-6, softcap=None):
    c = dict(architecture="Begopel", vocab=vocab, width=width, embedding=dict(scale=scale), norm=dict(eps=eps), layers=layers)
    if loop is not None:
        c["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    if softcap is not None:
        c["logit_softcap"] = softcap
    return c


# P: both kinds of layer, a loop over the first two that runs twice, grouped heads everywhere, a
# layer without feed-forward, sharp attention (scale 0.5 on normed heads of 24)
CONFIG_P = config(211, 72, [
    parallel(attention(4, 2, 24, 40, 0.5, 50.0, 12), delta(4, 2, 24, 20, 3), 100),
    mamba(4, 12, 16, 2, 2, 4, None),
    parallel(attention(3, 3, 16, 8, 0.7, 30.0, 6), delta(2, 1, 40, 24, 2), 56),
], loop=(0, 2, 2), scale=3.0, eps=1e-5, softcap=20.0)

# Q: the loop starts after the first layer and runs three times over one layer; no cap on the logits;
# a state-space layer with one group and one norm part next to one with several; five taps
CONFIG_Q = config(97, 128, [
    mamba(2, 64, 48, 1, 1, 5, 192),
    parallel(attention(2, 1, 80, 32, 0.2, 100.0, 20), delta(6, 3, 72, 16, 4), None),
    mamba(8, 16, 24, 4, 8, 2, 64),
], loop=(1, 2, 3), scale=1.0, eps=1e-6)

# R: no loop at all, sizes of real layers' kind (multiples of 64 and 128)
CONFIG_R = config(515, 256, [
    parallel(attention(4, 2, 64, 128, 0.125, 200.0, 32), delta(4, 2, 128, 64, 4), 512),
    mamba(4, 64, 128, 2, 1, 4, 512),
], scale=16.0, eps=1e-6, softcap=30.0)

# S: no size is a multiple of 8 (width 50, heads of 10, 6, 5 and 7, three heads, three norm parts)
CONFIG_S = config(77, 50, [
    parallel(attention(3, 1, 10, 6, 0.3, 11.0, 5), delta(3, 1, 10, 5, 3), 33),
    mamba(3, 5, 7, 1, 3, 3, 21),
], loop=(0, 2, 2), scale=2.0, softcap=9.0)

CONFIGS = {"P": CONFIG_P, "Q": CONFIG_Q, "R": CONFIG_R, "S": CONFIG_S}


def tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a configuration's tensors, written out from the design's naming (the
    library's own list is held against this one)."""
    D, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],)}
    if cfg.get("loop"):
        out["loop.in"] = (D, 2 * D)
        out["loop.step"] = (cfg["loop"]["times"], D)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (D,)
        if layer["type"] == "parallel":
            l, r = m["left"], m["right"]
            q = p + "mix.left."
            out.update({q + "q": (l["heads"] * l["dim"], D), q + "k": (l["kv_heads"] * l["dim"], D), q + "v": (l["kv_heads"] * l["vdim"], D),
                        q + "q.norm": (l["dim"],), q + "k.norm": (l["dim"],), q + "rel": (l["bias_rows"], l["heads"]), q + "sink": (l["heads"],),
                        q + "g": (l["heads"] * l["vdim"], D), q + "o": (D, l["heads"] * l["vdim"]), q + "out": (D,)})
            q = p + "mix.right."
            qk, vv = r["kv_heads"] * r["dim"], r["heads"] * r["vdim"]
            out.update({q + "q": (qk, D), q + "q.conv": (qk, r["conv"]), q + "k": (qk, D), q + "k.conv": (qk, r["conv"]),
                        q + "v": (vv, D), q + "v.conv": (vv, r["conv"]), q + "b": (r["heads"], D), q + "a": (r["heads"], D),
                        q + "A_log": (r["heads"],), q + "dt_bias": (r["heads"],), q + "norm": (r["vdim"],), q + "g": (vv, D),
                        q + "o": (D, vv), q + "out": (D,)})
        else:
            q = p + "mix."
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            out.update({q + "in": (2 * inner + 2 * gn + m["heads"], D), q + "conv": (inner + 2 * gn, m["conv"]),
                        q + "conv.b": (inner + 2 * gn,), q + "dt_bias": (m["heads"],), q + "A_log": (m["heads"],), q + "D": (m["heads"],),
                        q + "norm": (inner,), q + "o": (D, inner)})
        if layer["mlp"]:
            out[p + "norm2"] = (D,)
            out[p + "mlp.up"] = (layer["mlp"]["ff"], D)
            out[p + "mlp.down"] = (D, layer["mlp"]["ff"])
    return out


def make_weights(cfg: dict, seed: int) -> dict:
    """bfloat16 tensors by name."""
    gen = torch.Generator().manual_seed(seed)
    randn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = randn(*shape)
        elif last in ("norm1", "norm2") or name == "final.norm":
            t = 0.2 * randn(*shape)                                  # the norm adds one
        elif name.endswith(("q.norm", "k.norm", "left.out", "right.out", ".norm")):
            t = 1.0 + 0.2 * randn(*shape)
        elif last == "rel":
            t = 1.5 * randn(*shape)
        elif last == "sink":
            t = 1.0 + randn(*shape)
        elif last == "A_log":
            t = torch.rand(*shape, generator=gen, dtype=torch.float64) * 2.0 - 1.5
        elif last == "dt_bias":
            t = 0.5 * randn(*shape)
        elif last == "D":
            t = 1.0 + 0.3 * randn(*shape)
        elif name.endswith("conv.b"):
            t = 0.2 * randn(*shape)
        elif last == "conv":
            t = 0.6 * randn(*shape)
        elif name == "loop.step":
            t = 0.3 * randn(*shape)
        elif last in ("a", "b"):
            t = 2.0 * randn(*shape) / shape[1] ** 0.5                # decays and strengths that differ from token to token
        else:
            t = randn(*shape) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_folder(path: str, cfg: dict, weights: dict) -> str:
    from picolm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(path, "model.safetensors"), {k: v.contiguous() for k, v in weights.items()})
    return path


def plain_logits(cfg: dict, weights: dict, tokens) -> np.ndarray:
    from plain import begopel_plain as P
    return P.forward(cfg, weights, list(tokens)).numpy()


def load(cfg: dict, weights: dict, dtype: str):
    """The library's model of `cfg` with `weights` bound, on the GPU."""
    from picolm_amd.engine.builder import build_from_config_dict, parse_dtype
    from picolm_amd.parts.base import Runtime
    from picolm_amd.weights import TensorDict
    model = build_from_config_dict(cfg)
    model.load(TensorDict(weights), Runtime(torch.device("cuda:0"), parse_dtype(dtype)))
    return model


def distance(got: np.ndarray, want: np.ndarray) -> float:
    """The largest distance of a row of logits from the plain model's: means taken off, root mean
    square over the vocabulary, in units of the plain rows' own root mean square."""
    got, want = np.atleast_2d(got).astype(np.float64), np.atleast_2d(want)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    spread = np.sqrt(((want - want.mean(-1, keepdims=True)) ** 2).mean())
    return float(np.sqrt((d ** 2).mean(-1)).max() / spread)


# in 32-bit the engine's sums differ from the plain model's double precision by rounding alone; in
# bfloat16 every product's input is rounded to eight bits, which sharp attention and several passes
# over a loop multiply
LIMIT = {"float32": 2e-4, "bfloat16": 0.08}
