"""Typed configuration of the Gimozen architecture: a list of layers, each with its own kind of mixer and its own sizes.

config.json keys: ``architecture`` ("Gimozen"), ``vocab``, ``width``, ``embedding.scale``, ``norm.eps``, ``postln_alpha`` and
``layers``, a list of {``type``, ``mixer``, ``mlp``}. ``type`` "attention": mixer = {heads, kv_heads, dim, vdim, scale,
q_temp: {coef, every}}; ``type`` "latent_attention": mixer = {heads, dim, rot_dim, vdim, kv_rank, scale, rot: {dims, base,
scaling: {factor, original, fast, slow} | absent}, kv_from: index of an earlier latent layer | absent}. ``mlp`` is {kind:
"dense", ff} or null."""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ModelConfig, take_float, take_int

MAX_HEAD_SIZE = 256  # the widest head the paged attention kernels take
MAX_LATENT_RANK = 512  # the widest latent the latent attention kernel sums


def _section(raw: dict, key: str, where: str, optional: bool = False):
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"{where}'{key}' must be an object, not {value!r}")
    return value


@dataclass(frozen=True)
class RotaryConfig:
    dims: int
    base: float
    scaling: tuple | None   # (factor, original, fast, slow)

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "RotaryConfig":
        dims = take_int(raw, "dims", minimum=0)
        if dims % 2:
            raise ConfigError(f"{where}rot.dims = {dims} is not even")
        base = take_float(raw, "base")
        if not base > 1:
            raise ConfigError(f"{where}rot.base must be above 1, not {base}")
        scaling = _section(raw, "scaling", where + "rot.", optional=True)
        if scaling is not None:
            scaling = tuple(take_float(scaling, key) for key in ("factor", "original", "fast", "slow"))
            if not (scaling[0] > 0 and scaling[1] > 0 and scaling[2] > 0 and scaling[3] > 0):
                raise ConfigError(f"{where}rot.scaling holds a number that is not positive")
        return cls(dims, base, scaling)

    def scaling_dict(self):
        return None if self.scaling is None else dict(zip(("factor", "original", "fast", "slow"), self.scaling))

    def to_dict(self) -> dict:
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = self.scaling_dict()
        return out


@dataclass(frozen=True)
class AttentionMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    temp_coef: float
    temp_every: int

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "AttentionMixerConfig":
        heads, kv_heads = take_int(raw, "heads"), take_int(raw, "kv_heads")
        if heads % kv_heads:
            raise ConfigError(f"{where}{heads} heads do not divide into {kv_heads} key/value heads")
        dim, vdim = take_int(raw, "dim"), take_int(raw, "vdim")
        if max(dim, vdim) > MAX_HEAD_SIZE:
            raise ConfigError(f"{where}heads of {max(dim, vdim)} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        temp = _section(raw, "q_temp", where, optional=True) or {"coef": 0.0, "every": 1}
        return cls(heads, kv_heads, dim, vdim, take_float(raw, "scale"), take_float(temp, "coef"), take_int(temp, "every"))

    def to_dict(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "q_temp": {"coef": self.temp_coef, "every": self.temp_every},
                "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: RotaryConfig
    kv_from: int | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "LatentMixerConfig":
        rot_dim, kv_rank = take_int(raw, "rot_dim", minimum=0), take_int(raw, "kv_rank")
        rot = RotaryConfig.from_dict(_section(raw, "rot", where), where)
        if rot.dims > rot_dim:
            raise ConfigError(f"{where}rot.dims = {rot.dims} exceeds rot_dim = {rot_dim}")
        if kv_rank > MAX_LATENT_RANK:
            raise ConfigError(f"{where}a latent of {kv_rank} is wider than the latent attention kernel takes ({MAX_LATENT_RANK})")
        kv_from = raw.get("kv_from")
        if kv_from is not None:
            kv_from = take_int(raw, "kv_from", minimum=0)
        return cls(take_int(raw, "heads"), take_int(raw, "dim"), rot_dim, take_int(raw, "vdim"), kv_rank, take_float(raw, "scale"), rot, kv_from)

    def to_dict(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "rot": self.rot.to_dict(), "rot_dim": self.rot_dim,
               "scale": self.scale, "vdim": self.vdim}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


MIXERS = {"attention": AttentionMixerConfig, "latent_attention": LatentMixerConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: object
    ff: int | None   # the feed-forward's inner size; None: the layer has none

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"}, "type": self.type}


@dataclass(frozen=True)
class GimozenConfig(ModelConfig):
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    postln_alpha: float
    layers: tuple
    eos_token_id: int | None = None

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, raw: dict) -> "GimozenConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json has no list of 'layers'")
        layers = []
        for index, entry in enumerate(layers_raw):
            where = f"layer {index}: "
            if not isinstance(entry, dict):
                raise ConfigError(f"{where}must be an object")
            kind = entry.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{where}unknown type {kind!r}; known: {', '.join(sorted(MIXERS))}")
            mixer = MIXERS[kind].from_dict(_section(entry, "mixer", where), where)
            mlp = _section(entry, "mlp", where, optional=True)
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}unknown mlp.kind {mlp.get('kind')!r}; known: dense")
                ff = take_int(mlp, "ff")
            if kind == "latent_attention" and mixer.kv_from is not None:
                source = layers[mixer.kv_from].mixer if mixer.kv_from < index else None
                if not isinstance(source, LatentMixerConfig) or source.kv_from is not None:
                    raise ConfigError(f"{where}kv_from = {mixer.kv_from} does not name an earlier latent layer with a latent of its own")
                if (source.kv_rank, source.rot_dim, source.rot) != (mixer.kv_rank, mixer.rot_dim, mixer.rot):
                    raise ConfigError(f"{where}kv_rank, rot_dim and rot differ from those of layer {mixer.kv_from}, whose latent it reads")
            layers.append(LayerConfig(kind, mixer, ff))
        eps = take_float(_section(raw, "norm", ""), "eps")
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, not {eps}")
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer or null, not {eos!r}")
        return cls(
            architecture=raw.get("architecture") or "Gimozen",
            vocab=take_int(raw, "vocab"),
            width=take_int(raw, "width"),
            embedding_scale=take_float(_section(raw, "embedding", "", optional=True) or {"scale": 1.0}, "scale", 1.0),
            norm_eps=eps,
            postln_alpha=take_float(raw, "postln_alpha", 1.0),
            layers=tuple(layers),
            eos_token_id=eos,
        )

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale}, "layers": [layer.to_dict() for layer in self.layers],
               "norm": {"eps": self.norm_eps}, "postln_alpha": self.postln_alpha, "vocab": self.vocab, "width": self.width}
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out
