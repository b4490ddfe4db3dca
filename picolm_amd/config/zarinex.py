"""Typed configuration of the Zarinex decoder, read from the keys of its config.json.

    architecture        "Zarinex"
    vocab, width        sizes of the embedding table
    norm.eps            eps of every RMS norm
    postln_alpha        alpha of  x <- norm(alpha x + branch)
    layers[i]           {"type": "mamba1" | "latent_attention" | "hgrn2", "mixer": {...}, "mlp": {...} | null,
                         "weights_of": j}       weights_of: the layer runs with layer j's tensors and a state of its own
        mamba1            mixer {inner, state, dt_rank, conv}
        latent_attention  mixer {heads, dim, vdim, kv_rank, q_rank, scale}
        hgrn2             mixer {heads, dim, vdim}
        mlp               {"kind": "moe", "router": {experts, top}, "expert": {ff}, "shared": {ff} | null}

Every size the model uses comes from an instance of `ZarinexConfig`.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .begopel import MAX_CONV_TAPS, MAX_HEAD_DIM, MAX_STATE_KEY_DIM, _integer, _number, _object
from .llama import ConfigError


@dataclass(frozen=True)
class Mamba1Config:
    inner: int
    state: int
    dt_rank: int
    conv: int

    @staticmethod
    def from_dict(d: dict, where: str) -> "Mamba1Config":
        c = Mamba1Config(_integer(d, where, "inner"), _integer(d, where, "state"), _integer(d, where, "dt_rank"), _integer(d, where, "conv"))
        if c.state > MAX_STATE_KEY_DIM:
            raise ConfigError(f"{where}state: {c.state} exceeds {MAX_STATE_KEY_DIM}, the largest of a matrix state")
        if c.conv > MAX_CONV_TAPS:
            raise ConfigError(f"{where}conv: {c.conv} taps exceed {MAX_CONV_TAPS}")
        return c

    def to_dict(self) -> dict:
        return {"inner": self.inner, "state": self.state, "dt_rank": self.dt_rank, "conv": self.conv}


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float

    @staticmethod
    def from_dict(d: dict, where: str) -> "LatentAttentionConfig":
        c = LatentAttentionConfig(_integer(d, where, "heads"), _integer(d, where, "dim"), _integer(d, where, "vdim"),
                                  _integer(d, where, "kv_rank"), _integer(d, where, "q_rank"), _number(d, where, "scale"))
        if not c.scale > 0:
            raise ConfigError(f"{where}scale: must be positive")
        if c.kv_rank > MAX_HEAD_DIM:        # the attention runs over the latents: they are its keys
            raise ConfigError(f"{where}kv_rank: {c.kv_rank} exceeds {MAX_HEAD_DIM}, the largest key the attention kernels take")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
                "scale": self.scale}


@dataclass(frozen=True)
class HGRN2Config:
    heads: int
    dim: int
    vdim: int

    @staticmethod
    def from_dict(d: dict, where: str) -> "HGRN2Config":
        c = HGRN2Config(_integer(d, where, "heads"), _integer(d, where, "dim"), _integer(d, where, "vdim"))
        if c.dim > MAX_STATE_KEY_DIM:
            raise ConfigError(f"{where}dim: {c.dim} exceeds {MAX_STATE_KEY_DIM}, the largest key of a matrix state")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}


@dataclass(frozen=True)
class RoutedConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int = 0               # 0: no shared expert

    @staticmethod
    def from_dict(d: dict, where: str) -> "RoutedConfig":
        if d.get("kind") != "moe":
            raise ConfigError(f"{where}kind: '{d.get('kind')}' is not supported (known: moe)")
        router = _object(d, where, "router")
        shared = d.get("shared")
        if shared is not None and not isinstance(shared, dict):
            raise ConfigError(f"{where}shared: expected an object or null")
        c = RoutedConfig(_integer(router, where + "router.", "experts"), _integer(router, where + "router.", "top"),
                         _integer(_object(d, where, "expert"), where + "expert.", "ff"),
                         _integer(shared, where + "shared.", "ff") if shared else 0)
        if c.top > c.experts:
            raise ConfigError(f"{where}router.top: {c.top} exceeds router.experts = {c.experts}")
        return c

    def to_dict(self) -> dict:
        return {"kind": "moe", "router": {"experts": self.experts, "top": self.top}, "expert": {"ff": self.ff},
                "shared": {"ff": self.shared_ff} if self.shared_ff else None}


_MIXERS = {"mamba1": Mamba1Config, "latent_attention": LatentAttentionConfig, "hgrn2": HGRN2Config}


@dataclass(frozen=True)
class ZarinexLayer:
    type: str
    mixer: object                    # Mamba1Config | LatentAttentionConfig | HGRN2Config
    mlp: RoutedConfig | None         # None: the layer has no feed-forward
    weights_of: int | None = None    # the layer whose tensors this one runs with

    @staticmethod
    def from_dict(d: dict, where: str) -> "ZarinexLayer":
        if not isinstance(d, dict):
            raise ConfigError(f"{where[:-1]}: expected an object")
        kind = d.get("type")
        if kind not in _MIXERS:
            raise ConfigError(f"{where}type: '{kind}' is not a known mixer (known: {', '.join(_MIXERS)})")
        mixer = _MIXERS[kind].from_dict(_object(d, where, "mixer"), where + "mixer.")
        mlp = d.get("mlp")
        if mlp is not None and not isinstance(mlp, dict):
            raise ConfigError(f"{where}mlp: expected an object or null")
        owner = d.get("weights_of")
        return ZarinexLayer(kind, mixer, RoutedConfig.from_dict(mlp, where + "mlp.") if mlp is not None else None,
                            None if owner is None else _integer(d, where, "weights_of", least=0))

    def to_dict(self) -> dict:
        d = {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class ZarinexConfig:
    vocab: int
    width: int
    layers: tuple
    norm_eps: float = 1e-6
    postln_alpha: float = 1.0
    torch_dtype: str = "bfloat16"
    max_position_embeddings: int | None = None       # positions are computed, not tabled: a sequence is as long as the cache allows
    bos_token_id: int | None = None
    eos_token_ids: tuple = field(default=())

    @staticmethod
    def from_dict(root: dict) -> "ZarinexConfig":
        if not isinstance(root, dict):
            raise ConfigError("config.json: expected an object")
        layers = root.get("layers")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError("layers: expected a list of at least one layer")
        norm = root.get("norm") or {}
        eos = root.get("eos_token_id")
        cfg = ZarinexConfig(
            vocab=_integer(root, "", "vocab"), width=_integer(root, "", "width"),
            layers=tuple(ZarinexLayer.from_dict(l, f"layers[{i}].") for i, l in enumerate(layers)),
            norm_eps=_number(norm, "norm.", "eps", 1e-6), postln_alpha=_number(root, "", "postln_alpha", 1.0),
            torch_dtype=str(root.get("torch_dtype", "bfloat16")),
            max_position_embeddings=(_integer(root, "", "max_position_embeddings")
                                     if root.get("max_position_embeddings") is not None else None),
            bos_token_id=None if root.get("bos_token_id") is None else int(root["bos_token_id"]),
            eos_token_ids=() if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos])))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps: must be positive")
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            raise ConfigError(f"torch_dtype: '{self.torch_dtype}' is not one of bfloat16, float32, float16")
        for i, layer in enumerate(self.layers):
            if layer.weights_of is None:
                continue
            j, seen = i, set()
            while self.layers[j].weights_of is not None:       # a layer may name one that names another
                seen.add(j)
                j = self.layers[j].weights_of
                if not 0 <= j < len(self.layers) or j in seen:
                    raise ConfigError(f"layers[{i}].weights_of: {layer.weights_of} leads to no layer with tensors of its own")
            owner = self.layers[j]
            if (owner.type, owner.mixer, owner.mlp) != (layer.type, layer.mixer, layer.mlp):
                raise ConfigError(f"layers[{i}].weights_of: layer {j} has other sizes than this one")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab:
                raise ConfigError(f"eos_token_id: {e} is outside the vocabulary of {self.vocab}")

    def to_dict(self) -> dict:
        d = {"architecture": "Zarinex", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "postln_alpha": self.postln_alpha, "layers": [l.to_dict() for l in self.layers], "torch_dtype": self.torch_dtype}
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

    def owner_of(self, i: int) -> int:
        """The layer whose tensors layer i runs with."""
        while self.layers[i].weights_of is not None:
            i = self.layers[i].weights_of
        return i
