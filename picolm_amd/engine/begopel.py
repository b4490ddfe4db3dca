"""The Begopel decoder as a list of parts, and its entry in the architecture registry.

A scaled embedding; pre-norm layers (norms whose weights are offsets from one) whose mixer is either
two branches on one input, a softmax attention with a sink and a gated delta rule, or a Mamba-2
state-space layer, each followed by a feed-forward with a squared relu (or none); a stretch of
layers that runs several times in a row with the same weights, every pass entered through a
product over [x ; embedding output] and with a cache entry of its own per layer; a head tied to
the embedding table, with capped logits."""
from __future__ import annotations

from ..config import register_architecture
from ..config.begopel import BegopelConfig, Mamba2Config, ParallelConfig
from ..parts import LMHead, Part, PreNormBlock, RMSNorm, TokenEmbedding
from ..parts.block import LoopEntry
from ..parts.feedforward import ActivatedMLP
from ..parts.linear import Linear
from ..parts.parallel import ParallelMixer
from ..parts.recurrent import GatedDeltaRule, Mamba2
from ..parts.sink_attention import SinkAttention
from ..weights import TensorSpec
from .model import DecoderModel, LayerCall


def _mixer(prefix: str, kind, D: int, eps: float):
    if isinstance(kind, ParallelConfig):
        l, r = kind.left, kind.right
        left = SinkAttention(prefix + "left.", D, l.heads, l.kv_heads, l.dim, l.vdim, l.scale, eps, bias_rows=l.bias_rows,
                             bias_max=l.bias_max, has_bias=True)
        right = GatedDeltaRule(prefix + "right.", D, r.heads, r.kv_heads, r.dim, r.vdim, r.conv, eps)
        return ParallelMixer(left, right, prefix + "left.out", prefix + "right.out", D, eps)
    if isinstance(kind, Mamba2Config):
        return Mamba2(prefix, D, kind.heads, kind.vdim, kind.state, kind.groups, kind.conv, kind.norm_groups, eps)
    raise ValueError(f"no mixer for {type(kind).__name__}")


class _UnusedTensors(Part):
    """Tensors that a checkpoint may carry and the model never reads (the second norm of a layer
    that has no feed-forward): named, so that the check of the checkpoint passes them by."""

    def __init__(self, specs):
        self._specs = list(specs)

    def tensor_specs(self):
        return self._specs


def build_begopel(cfg: BegopelConfig) -> DecoderModel:
    D, eps = cfg.width, cfg.norm_eps
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        has_ff = layer.ff is not None
        blocks.append(PreNormBlock(RMSNorm(p + "norm1", D, eps, weight_offset=1.0), _mixer(p + "mix.", layer.mixer, D, eps),
                                   RMSNorm(p + "norm2", D, eps, weight_offset=1.0) if has_ff else None,
                                   ActivatedMLP(p + "mlp.", D, layer.ff, "relu_squared") if has_ff else None))
    n_layers = len(blocks)
    order = []
    unused = _UnusedTensors(TensorSpec(f"l{i}.norm2", (D,), optional=True, init=None)
                            for i, layer in enumerate(cfg.layers) if layer.ff is None)
    if cfg.loop is not None:
        w_in = Linear(["loop.in"], [D], 2 * D)
        blocks += [LoopEntry(w_in, "loop.step", D, cfg.loop.times, t) for t in range(cfg.loop.times)]
    for i, t, first in cfg.layer_runs():
        if first:
            order.append(LayerCall(n_layers + t))
        order.append(LayerCall(i))
    emb = TokenEmbedding("embed", cfg.vocab, D, scale=cfg.embedding_scale, keeps_output=cfg.loop is not None)
    model = DecoderModel(cfg, emb, blocks, RMSNorm("final.norm", D, eps, weight_offset=1.0),
                         LMHead("lm_head", cfg.vocab, D, emb, tied=True, softcap=cfg.logit_softcap), order)
    model.extra_parts = [unused]
    return model


register_architecture("Begopel", BegopelConfig.from_dict, build_begopel, replace=True)
