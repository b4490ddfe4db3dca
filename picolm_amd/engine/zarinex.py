"""The Zarinex decoder as a list of parts, and its entry in the architecture registry.

An embedding plus a sinusoid per position; layers that norm after the sum, whose branches read the
residual rows themselves (the mixer a blend of each row with the one before it) and are gated by a
sigmoid of a product of those rows; a mixer that is a selective scan, an attention over cached
latents, or a matrix state with a forget gate per key channel; a routed feed-forward with a shared
expert; layers that run with another layer's tensors and a cache of their own; a head tied to the
embedding table."""
from __future__ import annotations

from ..config import register_architecture
from ..config.zarinex import HGRN2Config, LatentAttentionConfig, Mamba1Config, ZarinexConfig
from ..parts import LMHead, RMSNorm, TokenEmbedding
from ..parts.block import PostNormBlock
from ..parts.embedding import SinusoidalPositions
from ..parts.feedforward import RoutedExperts
from ..parts.latent_attention import LatentAttention
from ..parts.recurrent import HGRN2, Mamba1
from ..weights import TensorSpec
from .begopel import _UnusedTensors
from .model import DecoderModel, LayerCall


def _mixer(prefix: str, m, D: int, eps: float):
    if isinstance(m, Mamba1Config):
        return Mamba1(prefix, D, m.inner, m.state, m.dt_rank, m.conv)
    if isinstance(m, LatentAttentionConfig):
        return LatentAttention(prefix, D, m.heads, m.dim, m.vdim, m.kv_rank, m.q_rank, m.scale, eps)
    if isinstance(m, HGRN2Config):
        return HGRN2(prefix, D, m.heads, m.dim, m.vdim, eps)
    raise ValueError(f"no mixer for {type(m).__name__}")


def build_zarinex(cfg: ZarinexConfig) -> DecoderModel:
    D, eps = cfg.width, cfg.norm_eps
    blocks, block_of, unused = [], {}, []
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p = f"l{i}."
        ffn = None
        if layer.mlp is not None:
            ffn = RoutedExperts(p + "mlp.", D, layer.mlp.experts, layer.mlp.top, layer.mlp.ff, layer.mlp.shared_ff)
        else:
            unused.append(TensorSpec(p + "norm2", (D,), optional=True, init=None))
        block_of[i] = len(blocks)
        blocks.append(PostNormBlock(D, RMSNorm(p + "norm1", D, eps), _mixer(p + "mix.", layer.mixer, D, eps),
                                    RMSNorm(p + "norm2", D, eps) if ffn is not None else None, ffn, alpha=cfg.postln_alpha,
                                    shift_name=p + "shift", gate_names=(p + "rg1", p + "rg2")))
    order = [LayerCall(block_of[cfg.owner_of(i)]) for i in range(len(cfg.layers))]
    emb = TokenEmbedding("embed", cfg.vocab, D, positions=SinusoidalPositions(D))
    model = DecoderModel(cfg, emb, blocks, RMSNorm("final.norm", D, eps), LMHead("lm_head", cfg.vocab, D, emb, tied=True), order)
    model.extra_parts = [_UnusedTensors(unused)]
    return model


register_architecture("Zarinex", ZarinexConfig.from_dict, build_zarinex, replace=True)
