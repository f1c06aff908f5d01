"""The Gimozen architecture as a recipe of parts: a scaled token embedding, layers that norm after their sums (each with the
mixer its configuration names: attention with normed heads and a query temperature, or attention over a shared latent, which a
later layer may borrow), gated feed-forwards, a final RMS norm and a head of its own.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<name>``, ``l<i>.mlp.{gate,up,down}``, ``final.norm``, ``head``."""

from __future__ import annotations

from ..config.gimozen import AttentionMixerConfig, GimozenConfig, LatentMixerConfig
from ..config.registry import register_architecture
from ..parts import LinearHead, TokenEmbedding, make_part
from .base import LayerCall, Model


def _mixer(config: GimozenConfig, mixer):
    if isinstance(mixer, AttentionMixerConfig):
        return make_part("mixer", "normed_head_attention", width=config.width, n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, dim=mixer.dim,
                         vdim=mixer.vdim, scale=mixer.scale, eps=config.norm_eps, temp_coef=mixer.temp_coef, temp_every=mixer.temp_every)
    if isinstance(mixer, LatentMixerConfig):
        rotary = make_part("position_encoding", "rotary", dims=mixer.rot.dims, base=mixer.rot.base, scaling=mixer.rot.scaling_dict())
        return make_part("mixer", "latent_attention", width=config.width, n_heads=mixer.heads, dim=mixer.dim, rot_dim=mixer.rot_dim,
                         vdim=mixer.vdim, kv_rank=mixer.kv_rank, scale=mixer.scale, eps=config.norm_eps, rotary=rotary,
                         own_latent=mixer.kv_from is None)
    raise TypeError(f"no mixer for {type(mixer).__name__}")


def build_gimozen(config: GimozenConfig, precision) -> Model:
    width, eps = config.width, config.norm_eps
    norm = lambda: make_part("norm", "rmsnorm", width=width, eps=eps, one_plus=True, tensor_name="")
    blocks, schedule = [], []
    for index, layer in enumerate(config.layers):
        has_mlp = layer.ff is not None
        blocks.append(make_part(
            "block", "post_norm", norm_1=norm(), mixer=_mixer(config, layer.mixer), norm_2=norm() if has_mlp else None,
            feed_forward=make_part("feed_forward", "gated_mlp", width=width, inner=layer.ff) if has_mlp else None,
            alpha=config.postln_alpha, compute_dtype=precision.compute,
        ))
        borrowed = getattr(layer.mixer, "kv_from", None)
        schedule.append(LayerCall(block=index, cache=index if borrowed is None else borrowed, write_cache=borrowed is None))
    return Model(
        config, precision,
        embedding=TokenEmbedding(config.vocab, width, scale=config.embedding_scale, tensor_name="", std=1.0 / max(config.embedding_scale, 1e-6)),
        position_encoding=None,
        blocks=blocks, schedule=schedule,
        final_norm=make_part("norm", "rmsnorm", width=width, eps=eps, one_plus=True, tensor_name=""),
        head=LinearHead(config.vocab, width, tensor_name=""),
        names={"embedding": "embed", "block": "l{i}.", "final_norm": "final.norm", "head": "head"},
    )


register_architecture("Gimozen", GimozenConfig, build_gimozen)
