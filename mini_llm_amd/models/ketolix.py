"""The Ketolix architecture as a recipe of parts: a token embedding that is also the head, layers that norm each branch's output
before it joins the stream (x <- x + norm1(mixer(x)), x <- x + norm2(ff(x))), per layer the mixer its configuration names (a
matrix memory, attention with normed projections, a softcap and a sink whose values may be mixed with an earlier layer's, or
attention and a decayed linear recurrence side by side), gated feed-forwards, and a final RMS norm.

Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<name>`` (``left.`` / ``right.`` inside a parallel mixer),
``l<i>.mlp.{gate,up,down}``, ``final.norm``."""

from __future__ import annotations

from ..config.ketolix import AttentionMixerConfig, KetolixConfig, MlstmMixerConfig, ParallelMixerConfig
from ..config.registry import register_architecture
from ..parts import TiedHead, TokenEmbedding, make_part
from .base import LayerCall, Model

VALUE_MIX_GROUP = "mixed_values"


def _rotary(rot):
    if rot is None or rot.dims == 0:
        return None
    return make_part("position_encoding", "rotary", dims=rot.dims, base=rot.base, scaling=rot.scaling_dict(), pairing="neighbours")


def _mixer(config: KetolixConfig, mixer, first_value_mixer: bool):
    width, eps = config.width, config.norm_eps
    if isinstance(mixer, MlstmMixerConfig):
        return make_part("mixer", "matrix_memory", width=width, n_heads=mixer.heads, dim=mixer.dim, vdim=mixer.vdim, eps=eps, gate_cap=mixer.gate_cap)
    if isinstance(mixer, AttentionMixerConfig):
        return make_part("mixer", "projection_norm_attention", width=width, n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, dim=mixer.dim,
                         vdim=mixer.vdim, scale=mixer.scale, eps=eps, rotary=_rotary(mixer.rot), window=mixer.window, softcap=mixer.softcap,
                         sink=True, value_mix=VALUE_MIX_GROUP if mixer.v_mix else None, value_mix_first=first_value_mixer)
    if isinstance(mixer, ParallelMixerConfig):
        left, right = mixer.left, mixer.right
        return make_part(
            "mixer", "parallel",
            left=make_part("mixer", "projection_norm_attention", width=width, n_heads=left.heads, n_kv_heads=left.kv_heads, dim=left.dim, vdim=None,
                           scale=left.scale, eps=eps, rotary=_rotary(left.rot), window=left.window, values="keys", biases=True,
                           conv_taps=left.conv, head_gate=True, out_scale=mixer.left_scale),
            right=make_part("mixer", "decayed_linear_attention", width=width, n_heads=right.heads, dim=right.dim, vdim=right.vdim,
                            decay=right.decay, eps=eps, out_scale=mixer.right_scale),
        )
    raise TypeError(f"no mixer for {type(mixer).__name__}")


def build_ketolix(config: KetolixConfig, precision) -> Model:
    width, eps = config.width, config.norm_eps
    norm = lambda: make_part("norm", "rmsnorm", width=width, eps=eps, tensor_name="")
    blocks, schedule = [], []
    value_mixers = 0
    for index, layer in enumerate(config.layers):
        mixes = isinstance(layer.mixer, AttentionMixerConfig) and layer.mixer.v_mix
        has_mlp = layer.ff is not None
        blocks.append(make_part(
            "block", "branch_norm", norm_1=norm(), mixer=_mixer(config, layer.mixer, mixes and value_mixers == 0), norm_2=norm() if has_mlp else None,
            feed_forward=make_part("feed_forward", "gated_mlp", width=width, inner=layer.ff) if has_mlp else None, compute_dtype=precision.compute,
        ))
        value_mixers += mixes
        schedule.append(LayerCall(block=index, cache=index))
    embedding = TokenEmbedding(config.vocab, width, tensor_name="", std=1.0)
    return Model(
        config, precision, embedding=embedding, position_encoding=None, blocks=blocks, schedule=schedule,
        final_norm=make_part("norm", "rmsnorm", width=width, eps=eps, tensor_name=""), head=TiedHead(embedding),
        names={"embedding": "embed", "block": "l{i}.", "final_norm": "final.norm"},
    )


register_architecture("Ketolix", KetolixConfig, build_ketolix)
