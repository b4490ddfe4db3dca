"""Small Zarinex configurations with weights made for the tests, and the plain model's logits for
them.

The weights are not the library's random ones: every kind of tensor gets a spread that makes its
mechanism count (forget gates between their lower bounds and one, step sizes and decays that differ
from channel to channel, blends, gates and norm weights away from their neutral values), and all are
rounded to bfloat16 first, so that both runtimes and the plain model read the same numbers.  The
configurations differ from each other in every size, and none has two sizes equal that the code
could mix up (key and value sizes, the two ranks, heads, the experts' and the shared expert's
widths); layers run with the tensors of layers before and after them."""
from __future__ import annotations

import numpy as np
import torch

from begopel_tiny import distance, load, write_folder  # noqa: F401  (the same helpers serve both designs)


def mamba(inner, state, dt_rank, conv):
    return "mamba1", dict(inner=inner, state=state, dt_rank=dt_rank, conv=conv)


def latent(heads, dim, vdim, kv_rank, q_rank, scale):
    return "latent_attention", dict(heads=heads, dim=dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale)


def hgrn(heads, dim, vdim):
    return "hgrn2", dict(heads=heads, dim=dim, vdim=vdim)


def moe(experts, top, ff, shared=None):
    return dict(kind="moe", router=dict(experts=experts, top=top), expert=dict(ff=ff), shared=None if shared is None else dict(ff=shared))


def layer(mixer, mlp=None, weights_of=None):
    d = dict(type=mixer[0], mixer=mixer[1], mlp=mlp)
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def config(vocab, width, layers, alpha=1.0, eps=1e-6):
    return dict(architecture="Zarinex", vocab=vocab, width=width, norm=dict(eps=eps), postln_alpha=alpha, layers=layers)


# A: every mixer, a layer without feed-forward, one without a shared expert, one pick and several,
# a layer that runs with the tensors of a later one, two that run with those of an earlier one
CONFIG_A = config(211, 72, [
    layer(hgrn(3, 24, 20), moe(5, 1, 32)),
    layer(latent(4, 16, 24, 40, 56, 0.3), moe(6, 2, 40, 56), weights_of=3),
    layer(mamba(100, 12, 6, 3), None),
    layer(latent(4, 16, 24, 40, 56, 0.3), moe(6, 2, 40, 56)),
    layer(hgrn(3, 24, 20), moe(5, 1, 32), weights_of=0),
    layer(mamba(100, 12, 6, 3), None, weights_of=2),
], alpha=2.0, eps=1e-5)

# B: sizes of real layers' kind (multiples of 64; latents of 64 go through the matrix cores in
# bfloat16), every expert picked (top = experts), alpha 1
CONFIG_B = config(515, 256, [
    layer(latent(8, 32, 64, 64, 96, 0.18), moe(4, 4, 128, 256)),
    layer(mamba(512, 16, 16, 4), moe(8, 2, 64, 128)),
    layer(hgrn(2, 128, 64), moe(8, 3, 128)),
    layer(latent(8, 32, 64, 64, 96, 0.18), moe(4, 4, 128, 256), weights_of=0),
], alpha=1.0)

# C: no size is a multiple of 8; one tap; a state of one; one head
CONFIG_C = config(77, 50, [
    layer(mamba(30, 1, 3, 1), moe(3, 2, 14, 9)),
    layer(hgrn(1, 10, 7), None),
    layer(latent(3, 5, 7, 9, 11, 0.45), moe(7, 3, 6)),
    layer(mamba(21, 5, 2, 5), moe(2, 1, 13, 22)),
], alpha=4.0, eps=1e-4)

CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C}


def tensor_shapes(cfg: dict) -> dict:
    """Names and shapes of a configuration's tensors, written out from the design's naming (the
    library's own list is held against this one)."""
    D = cfg["width"]
    out = {"embed": (cfg["vocab"], D), "final.norm": (D,)}
    for i, l in enumerate(cfg["layers"]):
        if l.get("weights_of") is not None:
            continue
        p, q, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
        out.update({p + "norm1": (D,), p + "shift": (D,), p + "rg1": (D, D), p + "rg1.b": (D,)})
        if l["type"] == "mamba1":
            n, s, r = m["inner"], m["state"], m["dt_rank"]
            out.update({q + "in": (2 * n, D), q + "conv": (n, m["conv"]), q + "conv.b": (n,), q + "x": (r + 2 * s, n), q + "dt": (n, r),
                        q + "dt.b": (n,), q + "A_log": (n, s), q + "D": (n,), q + "o": (D, n)})
        elif l["type"] == "latent_attention":
            H, d, dv, r, rq = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({q + "dq": (rq, D), q + "dq.norm": (rq,), q + "uq": (H * d, rq), q + "dkv": (r, D), q + "dkv.norm": (r,),
                        q + "uk": (H * d, r), q + "uv": (H * dv, r), q + "g": (H * dv, D), q + "o": (D, H * dv)})
        else:
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({q + "q": (H * d, D), q + "f": (H * d, D), q + "f.b": (H * d,), q + "lower": (H * d,), q + "v": (H * dv, D),
                        q + "norm": (dv,), q + "o": (D, H * dv)})
        if l["mlp"]:
            f, mlp = p + "mlp.", l["mlp"]
            out.update({p + "norm2": (D,), p + "rg2": (D, D), p + "rg2.b": (D,), f + "router": (mlp["router"]["experts"], D),
                        f + "router.b": (mlp["router"]["experts"],)})
            names = [(f"e{e}.", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
            if mlp.get("shared"):
                names.append(("shared.", mlp["shared"]["ff"]))
            for n, ff in names:
                out.update({f + n + "gate": (ff, D), f + n + "up": (ff, D), f + n + "down": (D, ff)})
    return out


def make_weights(cfg: dict, seed: int) -> dict:
    """bfloat16 tensors by name."""
    gen = torch.Generator().manual_seed(seed)
    randn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    rand = lambda *s: torch.rand(*s, generator=gen, dtype=torch.float64)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = randn(*shape)
        elif last in ("norm1", "norm2", "norm") or name == "final.norm":
            t = 1.0 + 0.2 * randn(*shape)
        elif last == "shift":
            t = rand(*shape)
        elif name.endswith(("rg1.b", "rg2.b", "f.b")):
            t = 0.7 * randn(*shape)
        elif last == "lower":
            t = 0.9 * rand(*shape)
        elif last == "A_log":
            t = rand(*shape) * 2.0 - 1.5
        elif name.endswith("dt.b"):
            t = randn(*shape) - 1.0
        elif last == "dt":
            t = 2.0 * randn(*shape) / shape[1] ** 0.5                # step sizes that differ from token to token
        elif last == "D":
            t = 1.0 + 0.3 * randn(*shape)
        elif name.endswith("conv.b"):
            t = 0.2 * randn(*shape)
        elif last == "conv":
            t = 0.6 * randn(*shape)
        elif name.endswith("router.b"):
            t = 0.5 * randn(*shape)
        elif last == "router":
            t = 2.0 * randn(*shape) / shape[1] ** 0.5
        elif last == "down":
            t = 2.0 * randn(*shape) / shape[1] ** 0.5                # experts that weigh as much as the mixers
        else:
            t = randn(*shape) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def plain_logits(cfg: dict, weights: dict, tokens) -> np.ndarray:
    from plain import zarinex_plain as P
    return P.forward(cfg, {k: v.to(torch.float64).numpy() for k, v in weights.items()}, list(tokens))


class Truth:
    """The plain model's logits of a sequence, and per token the smallest margin by which any of
    its routers picked."""

    def __init__(self, cfg: dict, weights: dict, tokens):
        from plain import zarinex_plain as P
        margins = []
        self.logits = P.forward(cfg, {k: v.to(torch.float64).numpy() for k, v in weights.items()}, list(tokens), margins=margins)
        self.margins = np.min(margins, axis=0) if margins else np.full(len(tokens), np.inf)

    def __getitem__(self, rows):
        return self.logits[rows]


def near(got, truth: Truth, rows, dtype: str) -> bool:
    """Whether the engine's rows lie within the limit of the plain model's.  A token whose router
    picked by less than CLOSE_CALL is held to LOOSE instead, and so are the AFTER tokens behind it:
    rounding may give it another expert, and then its row is another function's value, which the
    next tokens read through the blend, the convolution and the states."""
    rows = np.arange(len(truth.logits))[rows]
    got, want = np.atleast_2d(np.asarray(got, np.float64)), np.atleast_2d(truth.logits[rows])
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    spread = np.sqrt(((want - want.mean(-1, keepdims=True)) ** 2).mean())
    e = np.sqrt((d ** 2).mean(-1)) / spread
    close = truth.margins < CLOSE_CALL[dtype]
    shaky = np.array([close[max(0, r - AFTER):r + 1].any() for r in np.atleast_1d(rows)])
    limit = np.where(shaky, LOOSE, LIMIT[dtype])
    return bool((e <= limit).all())


# in 32-bit the engine's sums differ from the plain model's double precision by rounding alone; in
# bfloat16 every product's input is rounded to eight bits, and a router's logits that lie close
# together may then pick another expert for a token
LIMIT = {"float32": 2e-4, "bfloat16": 0.08}
CLOSE_CALL = {"float32": 1e-4, "bfloat16": 0.06}     # router logits have a spread of about two
LOOSE, AFTER = 1.5, 8
