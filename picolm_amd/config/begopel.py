"""Typed configuration of the Begopel decoder, read from the keys of its config.json.

    architecture        "Begopel"
    vocab, width        sizes of the embedding table
    embedding.scale     the embedding's rows are multiplied by it
    norm.eps            eps of every RMS norm of a layer
    logit_softcap       c: logits <- c tanh(logits / c) (absent or 0: none)
    layers[i]           {"type": "parallel" | "mamba2", "mixer": {...}, "mlp": {"kind": "dense", "ff": F} | null}
        parallel        mixer.left  {heads, kv_heads, dim, vdim, scale, bias_max}: softmax attention with a sink
                        mixer.right {heads, kv_heads, dim, vdim, conv}: gated delta rule
        mamba2          mixer {heads, vdim, state, groups, norm_groups, conv}
    loop                {start, stop, times}: layers start .. stop-1 run `times` times in a row (absent: no loop)

The rows of an attention's distance table are a tensor's shape, not a key; a configuration that
is written out for random weights names them in `bias_rows`, which a reader takes if it is there.
Every size the model uses comes from an instance of `BegopelConfig` or from a tensor's shape.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .llama import ConfigError

MAX_HEAD_DIM = 1024          # the largest head the vector-ALU attention kernels take
MAX_STATE_KEY_DIM = 256      # the largest key (or state size) of a matrix state
MAX_CONV_TAPS = 16


def _integer(d: dict, where: str, key: str, default=None, least: int = 1) -> int:
    v = d.get(key, default)
    if v is None:
        raise ConfigError(f"{where}{key}: missing")
    if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
        raise ConfigError(f"{where}{key}: expected an integer, got {v!r}")
    if int(v) < least:
        raise ConfigError(f"{where}{key}: must be at least {least}, got {v}")
    return int(v)


def _number(d: dict, where: str, key: str, default=None) -> float:
    v = d.get(key, default)
    if v is None:
        raise ConfigError(f"{where}{key}: missing")
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{where}{key}: expected a number, got {v!r}")
    return float(v)


def _object(d: dict, where: str, key: str) -> dict:
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}{key}: expected an object")
    return v


@dataclass(frozen=True)
class SinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: float
    bias_rows: int | None = None     # rows of the distance table; None: the tensor's shape says

    @staticmethod
    def from_dict(d: dict, where: str) -> "SinkAttentionConfig":
        c = SinkAttentionConfig(_integer(d, where, "heads"), _integer(d, where, "kv_heads"), _integer(d, where, "dim"),
                                _integer(d, where, "vdim"), _number(d, where, "scale"), _number(d, where, "bias_max"),
                                _integer(d, where, "bias_rows") if d.get("bias_rows") is not None else None)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}kv_heads: {c.kv_heads} does not divide heads = {c.heads}")
        for key in ("dim", "vdim"):
            if getattr(c, key) > MAX_HEAD_DIM:
                raise ConfigError(f"{where}{key}: {getattr(c, key)} exceeds {MAX_HEAD_DIM}, the largest head the attention kernels take")
        if not c.bias_max > 0:
            raise ConfigError(f"{where}bias_max: must be positive")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "bias_max": self.bias_max}
        if self.bias_rows is not None:
            d["bias_rows"] = self.bias_rows
        return d


@dataclass(frozen=True)
class GatedDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @staticmethod
    def from_dict(d: dict, where: str) -> "GatedDeltaConfig":
        c = GatedDeltaConfig(_integer(d, where, "heads"), _integer(d, where, "kv_heads"), _integer(d, where, "dim"),
                             _integer(d, where, "vdim"), _integer(d, where, "conv"))
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}kv_heads: {c.kv_heads} does not divide heads = {c.heads}")
        if c.dim > MAX_STATE_KEY_DIM:
            raise ConfigError(f"{where}dim: {c.dim} exceeds {MAX_STATE_KEY_DIM}, the largest key of a matrix state")
        if c.conv > MAX_CONV_TAPS:
            raise ConfigError(f"{where}conv: {c.conv} taps exceed {MAX_CONV_TAPS}")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class ParallelConfig:
    left: SinkAttentionConfig
    right: GatedDeltaConfig

    @staticmethod
    def from_dict(d: dict, where: str) -> "ParallelConfig":
        return ParallelConfig(SinkAttentionConfig.from_dict(_object(d, where, "left"), where + "left."),
                              GatedDeltaConfig.from_dict(_object(d, where, "right"), where + "right."))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class Mamba2Config:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @staticmethod
    def from_dict(d: dict, where: str) -> "Mamba2Config":
        c = Mamba2Config(_integer(d, where, "heads"), _integer(d, where, "vdim"), _integer(d, where, "state"),
                         _integer(d, where, "groups"), _integer(d, where, "norm_groups"), _integer(d, where, "conv"))
        if c.heads % c.groups:
            raise ConfigError(f"{where}groups: {c.groups} does not divide heads = {c.heads}")
        if (c.heads * c.vdim) % c.norm_groups:
            raise ConfigError(f"{where}norm_groups: {c.norm_groups} does not divide heads * vdim = {c.heads * c.vdim}")
        if c.state > MAX_STATE_KEY_DIM:
            raise ConfigError(f"{where}state: {c.state} exceeds {MAX_STATE_KEY_DIM}, the largest of a matrix state")
        if c.conv > MAX_CONV_TAPS:
            raise ConfigError(f"{where}conv: {c.conv} taps exceed {MAX_CONV_TAPS}")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups,
                "norm_groups": self.norm_groups, "conv": self.conv}


_MIXERS = {"parallel": ParallelConfig, "mamba2": Mamba2Config}
_MLP_KINDS = ("dense",)


@dataclass(frozen=True)
class BegopelLayer:
    type: str
    mixer: object                    # ParallelConfig | Mamba2Config
    ff: int | None                   # the feed-forward's inner width; None: the layer has none

    @staticmethod
    def from_dict(d: dict, where: str) -> "BegopelLayer":
        if not isinstance(d, dict):
            raise ConfigError(f"{where[:-1]}: expected an object")
        kind = d.get("type")
        if kind not in _MIXERS:
            raise ConfigError(f"{where}type: '{kind}' is not a known mixer (known: {', '.join(_MIXERS)})")
        mixer = _MIXERS[kind].from_dict(_object(d, where, "mixer"), where + "mixer.")
        mlp = d.get("mlp")
        ff = None
        if mlp is not None:
            if not isinstance(mlp, dict):
                raise ConfigError(f"{where}mlp: expected an object or null")
            if mlp.get("kind") not in _MLP_KINDS:
                raise ConfigError(f"{where}mlp.kind: '{mlp.get('kind')}' is not supported (known: {', '.join(_MLP_KINDS)})")
            ff = _integer(mlp, where + "mlp.", "ff")
        return BegopelLayer(kind, mixer, ff)

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int

    def to_dict(self) -> dict:
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclass(frozen=True)
class BegopelConfig:
    vocab: int
    width: int
    layers: tuple
    embedding_scale: float = 1.0
    norm_eps: float = 1e-6
    logit_softcap: float = 0.0
    loop: LoopConfig | None = None
    torch_dtype: str = "bfloat16"
    max_position_embeddings: int | None = None       # the design has no position tables: a sequence is as long as the cache allows
    bos_token_id: int | None = None
    eos_token_ids: tuple = field(default=())

    @staticmethod
    def from_dict(root: dict) -> "BegopelConfig":
        if not isinstance(root, dict):
            raise ConfigError("config.json: expected an object")
        layers = root.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("layers: expected a list of at least one layer")
        loop = root.get("loop")
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("loop: expected an object or null")
            loop = LoopConfig(_integer(loop, "loop.", "start", least=0), _integer(loop, "loop.", "stop", least=0),
                              _integer(loop, "loop.", "times"))
        emb = root.get("embedding") or {}
        norm = root.get("norm") or {}
        eos = root.get("eos_token_id")
        cfg = BegopelConfig(
            vocab=_integer(root, "", "vocab"), width=_integer(root, "", "width"),
            layers=tuple(BegopelLayer.from_dict(l, f"layers[{i}].") for i, l in enumerate(layers)),
            embedding_scale=_number(emb, "embedding.", "scale", 1.0),
            norm_eps=_number(norm, "norm.", "eps", 1e-6),
            logit_softcap=_number(root, "", "logit_softcap", 0.0) if root.get("logit_softcap") is not None else 0.0,
            loop=loop, torch_dtype=str(root.get("torch_dtype", "bfloat16")),
            max_position_embeddings=(_integer(root, "", "max_position_embeddings")
                                     if root.get("max_position_embeddings") is not None else None),
            bos_token_id=None if root.get("bos_token_id") is None else int(root["bos_token_id"]),
            eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos])))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps: must be positive")
        if self.logit_softcap < 0:
            raise ConfigError("logit_softcap: must not be negative")
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            raise ConfigError(f"torch_dtype: '{self.torch_dtype}' is not one of bfloat16, float32, float16")
        if self.loop is not None:
            lp = self.loop
            if not 0 <= lp.start < lp.stop <= len(self.layers):
                raise ConfigError(f"loop: layers {lp.start} .. {lp.stop - 1} are no stretch of the {len(self.layers)} layers")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"eos_token_id: {e} is outside the vocabulary of {self.vocab}")

    def to_dict(self) -> dict:
        d = {"architecture": "Begopel", "vocab": self.vocab, "width": self.width,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
             "layers": [l.to_dict() for l in self.layers], "torch_dtype": self.torch_dtype}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d

    # -- derived ---------------------------------------------------------------------------
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    def layer_runs(self) -> list:
        """The layers in the order they run, as (layer, pass number or None, first of its pass):
        the looped stretch `times` times in a row, then the rest."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None, False) for i in range(n)]
        lp = self.loop
        runs = [(i, None, False) for i in range(lp.start)]
        for t in range(lp.times):
            runs += [(i, t, i == lp.start) for i in range(lp.start, lp.stop)]
        return runs + [(i, None, False) for i in range(lp.stop, n)]
