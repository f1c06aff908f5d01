"""Typed configuration of the Ketolix architecture: a list of layers, each with its own kind of mixer and its own sizes.

config.json keys: ``architecture`` ("Ketolix"), ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list of {``type``, ``mixer``,
``mlp``}; ``mlp`` is {kind: "dense", ff} or null. By ``type``:

- "mlstm": mixer = {heads, dim, vdim, gate_cap | absent}.
- "attention": mixer = {heads, kv_heads, dim, vdim, scale, softcap | absent, mask: {size} | absent, rot: {dims, base, scaling:
  {factor, low, high, original} | absent} | absent, v_mix: true | absent}.
- "parallel": mixer = {left_scale, right_scale, left: {heads, kv_heads, dim, vdim, scale, conv | absent, mask, rot}, right: {heads,
  dim, vdim, decay: [one number a head]}}; the left mixer's values are its keys, so its vdim equals its dim."""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ModelConfig, take_float, take_int

MAX_HEAD_SIZE = 256   # the widest head the paged attention kernels take
MAX_TAPS = 16         # the longest short convolution


def _section(raw: dict, key: str, where: str, optional: bool = False):
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"{where}'{key}' must be an object, not {value!r}")
    return value


def recurrence_fits(dim: int, vdim: int) -> bool:
    """Whether the recurrence kernel takes heads of dim x vdim: a block holds tiles of up to 64 value columns, up to 512 / tile
    parts along dim and up to 64 rows of the matrix a thread."""
    return 1 <= dim <= 64 * max(1, min(dim, 512 // min(vdim, 64))) and vdim >= 1


@dataclass(frozen=True)
class PairRotaryConfig:
    dims: int
    base: float
    scaling: tuple | None   # (factor, low, high, original)

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "PairRotaryConfig":
        dims = take_int(raw, "dims", minimum=0)
        if dims % 2:
            raise ConfigError(f"{where}rot.dims = {dims} is not even")
        base = take_float(raw, "base")
        if not base > 1:
            raise ConfigError(f"{where}rot.base must be above 1, not {base}")
        scaling = _section(raw, "scaling", where + "rot.", optional=True)
        if scaling is not None:
            scaling = tuple(take_float(scaling, key) for key in ("factor", "low", "high", "original"))
            if not (scaling[0] > 0 and scaling[3] > 0 and scaling[2] > scaling[1] >= 0):
                raise ConfigError(f"{where}rot.scaling needs factor > 0, original > 0 and high > low >= 0")
        return cls(dims, base, scaling)

    def scaling_dict(self):
        return None if self.scaling is None else {"kind": "wavelength", **dict(zip(("factor", "low", "high", "original"), self.scaling))}

    def to_dict(self) -> dict:
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return out


def _rot(raw: dict, where: str, dim: int):
    rot = _section(raw, "rot", where, optional=True)
    if rot is None:
        return None
    rot = PairRotaryConfig.from_dict(rot, where)
    if rot.dims > dim:
        raise ConfigError(f"{where}rot.dims = {rot.dims} exceeds the heads' {dim} elements")
    return rot


def _window(raw: dict, where: str):
    mask = _section(raw, "mask", where, optional=True)
    return None if mask is None else take_int(mask, "size")


def _grouped_heads(raw: dict, where: str):
    heads, kv_heads = take_int(raw, "heads"), take_int(raw, "kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"{where}{heads} heads do not divide into {kv_heads} key/value heads")
    return heads, kv_heads


@dataclass(frozen=True)
class MlstmMixerConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "MlstmMixerConfig":
        dim, vdim = take_int(raw, "dim"), take_int(raw, "vdim")
        if not recurrence_fits(dim, vdim):
            raise ConfigError(f"{where}heads of {dim} x {vdim} are larger than the recurrence kernel takes")
        cap = raw.get("gate_cap")
        if cap is not None:
            cap = take_float(raw, "gate_cap")
            if not cap > 0:
                raise ConfigError(f"{where}gate_cap must be positive, not {cap}")
        return cls(take_int(raw, "heads"), dim, vdim, cap)

    def to_dict(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "vdim": self.vdim}
        if self.gate_cap is not None:
            out["gate_cap"] = self.gate_cap
        return out


@dataclass(frozen=True)
class AttentionMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None
    window: int | None
    rot: PairRotaryConfig | None
    v_mix: bool

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "AttentionMixerConfig":
        heads, kv_heads = _grouped_heads(raw, where)
        dim, vdim = take_int(raw, "dim"), take_int(raw, "vdim")
        if max(dim, vdim) > MAX_HEAD_SIZE:
            raise ConfigError(f"{where}heads of {max(dim, vdim)} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        softcap = raw.get("softcap")
        if softcap is not None:
            softcap = take_float(raw, "softcap")
            if not softcap > 0:
                raise ConfigError(f"{where}softcap must be positive, not {softcap}")
        v_mix = raw.get("v_mix", False)
        if not isinstance(v_mix, bool):
            raise ConfigError(f"{where}'v_mix' must be true or false, not {v_mix!r}")
        return cls(heads, kv_heads, dim, vdim, take_float(raw, "scale"), softcap, _window(raw, where), _rot(raw, where, dim), v_mix)

    def to_dict(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        if self.v_mix:
            out["v_mix"] = True
        return out


@dataclass(frozen=True)
class KeyValueAttentionConfig:
    """The attention side of a parallel mixer: its values are its keys."""

    heads: int
    kv_heads: int
    dim: int
    scale: float
    conv: int | None
    window: int | None
    rot: PairRotaryConfig | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "KeyValueAttentionConfig":
        heads, kv_heads = _grouped_heads(raw, where)
        dim = take_int(raw, "dim")
        if raw.get("vdim", dim) != dim:
            raise ConfigError(f"{where}the values are the keys: vdim = {raw.get('vdim')} must equal dim = {dim}")
        if dim > MAX_HEAD_SIZE:
            raise ConfigError(f"{where}heads of {dim} are wider than the attention kernels take ({MAX_HEAD_SIZE})")
        conv = raw.get("conv")
        if conv is not None:
            conv = take_int(raw, "conv")
            if conv > MAX_TAPS:
                raise ConfigError(f"{where}a convolution of {conv} taps is longer than the kernel takes ({MAX_TAPS})")
        return cls(heads, kv_heads, dim, take_float(raw, "scale"), conv, _window(raw, where), _rot(raw, where, dim))

    def to_dict(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.dim}
        if self.conv is not None:
            out["conv"] = self.conv
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.rot is not None:
            out["rot"] = self.rot.to_dict()
        return out


@dataclass(frozen=True)
class DecayedMixerConfig:
    heads: int
    dim: int
    vdim: int
    decay: tuple

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DecayedMixerConfig":
        heads, dim, vdim = take_int(raw, "heads"), take_int(raw, "dim"), take_int(raw, "vdim")
        if not recurrence_fits(dim, vdim):
            raise ConfigError(f"{where}heads of {dim} x {vdim} are larger than the recurrence kernel takes")
        decay = raw.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"{where}'decay' must list one number for each of the {heads} heads")
        return cls(heads, dim, vdim, tuple(float(d) for d in decay))

    def to_dict(self) -> dict:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: KeyValueAttentionConfig
    right: DecayedMixerConfig
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "ParallelMixerConfig":
        return cls(KeyValueAttentionConfig.from_dict(_section(raw, "left", where), where + "left: "),
                   DecayedMixerConfig.from_dict(_section(raw, "right", where), where + "right: "),
                   take_float(raw, "left_scale", 1.0), take_float(raw, "right_scale", 1.0))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(), "right_scale": self.right_scale}


MIXERS = {"mlstm": MlstmMixerConfig, "attention": AttentionMixerConfig, "parallel": ParallelMixerConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: object
    ff: int | None   # the feed-forward's inner size; None: the layer has none

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"}, "type": self.type}


@dataclass(frozen=True)
class KetolixConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    layers: tuple
    eos_token_id: int | None = None

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, raw: dict) -> "KetolixConfig":
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json has no list of 'layers'")
        layers, mixed_values = [], None
        for index, entry in enumerate(layers_raw):
            where = f"layer {index}: "
            if not isinstance(entry, dict):
                raise ConfigError(f"{where}must be an object")
            kind = entry.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{where}unknown type {kind!r}; known: {', '.join(sorted(MIXERS))}")
            mixer = MIXERS[kind].from_dict(_section(entry, "mixer", where), where)
            if kind == "attention" and mixer.v_mix:
                if mixed_values is None:
                    mixed_values = (index, mixer.kv_heads * mixer.vdim)
                elif mixed_values[1] != mixer.kv_heads * mixer.vdim:
                    raise ConfigError(f"{where}its values ({mixer.kv_heads} x {mixer.vdim}) cannot be mixed with those of layer {mixed_values[0]} ({mixed_values[1]} in all)")
            mlp = _section(entry, "mlp", where, optional=True)
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}unknown mlp.kind {mlp.get('kind')!r}; known: dense")
                ff = take_int(mlp, "ff")
            layers.append(LayerConfig(kind, mixer, ff))
        eps = take_float(_section(raw, "norm", ""), "eps")
        if not eps > 0:
            raise ConfigError(f"norm.eps must be positive, not {eps}")
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer or null, not {eos!r}")
        return cls(architecture=raw.get("architecture") or "Ketolix", vocab=take_int(raw, "vocab"), width=take_int(raw, "width"), norm_eps=eps,
                   layers=tuple(layers), eos_token_id=eos)

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers], "norm": {"eps": self.norm_eps},
               "vocab": self.vocab, "width": self.width}
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out
