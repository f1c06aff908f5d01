"""A plain, slow forward pass of the Gimozen design: whole sequences, no cache, one function per mechanism.

numpy only, float64 by default, and no code shared with ``mini_llm_amd``: the tests compare the engine with it.
Notation: T tokens, d the model's width, H query heads, G key/value heads, r the latent rank, n the rotated part."""

from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np

import plain_gpt2  # the safetensors reader/writer and the bfloat16 rounding helpers (plain numpy too)


def _keep(x):
    return x


# --------------------------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------------------------
def rms_norm(x, weight, eps, one_plus=False):
    """y = x / sqrt(mean(x^2) + eps) * g, with g = weight, or 1 + weight where the gain is stored around zero."""
    inverse = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    return x * inverse * ((1.0 + weight) if one_plus else weight)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gated_mlp(h, gate, up, down, stored=_keep):
    """down @ (silu(gate @ h) * (up @ h)); matrices are [out, in]."""
    inner = stored(stored(silu(stored(h @ gate.T))) * stored(h @ up.T))
    return inner @ down.T


def query_temperature(positions, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    positions = np.asarray(positions, dtype=np.int64)
    return 1.0 + coef * np.log(((positions + 1) // every) + 1.0)


def softmax_rows(scores, visible, sink=None):
    """Row softmax over the keys marked visible; with ``sink`` the denominator holds exp(sink) once more (a key without
    a value)."""
    out = np.zeros_like(scores)
    for i in range(scores.shape[0]):
        keys = np.nonzero(visible[i])[0]
        row = scores[i, keys]
        top = row.max() if sink is None else max(row.max(), sink)
        e = np.exp(row - top)
        total = e.sum() + (0.0 if sink is None else math.exp(sink - top))
        out[i, keys] = e / total
    return out


def causal_mask(n_queries, n_keys, first_position=0):
    q = first_position + np.arange(n_queries)[:, None]
    return np.arange(n_keys)[None, :] <= q


def normed_attention(h, w, mixer, eps, first_position=0, stored=_keep):
    """Grouped-head attention without rotation: per-head RMS norm of queries and keys (one gain vector for all heads),
    a temperature on the queries that grows with the logarithm of the position, a given score scale, ordinary softmax."""
    T = h.shape[0]
    H, G, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = stored(h @ w["q"].T).reshape(T, H, dim)
    k = stored(h @ w["k"].T).reshape(T, G, dim)
    v = stored(h @ w["v"].T).reshape(T, G, vdim)
    q = rms_norm(q, w["q.norm"], eps)
    k = stored(rms_norm(k, w["k.norm"], eps))
    temp = query_temperature(first_position + np.arange(T), mixer["q_temp"]["coef"], mixer["q_temp"]["every"])
    q = stored(q * temp[:, None, None])
    visible = causal_mask(T, T)
    out = np.zeros((T, H, vdim), dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        scores = (q[:, head] @ k[:, g].T) * mixer["scale"]
        out[:, head] = softmax_rows(scores, visible) @ v[:, g]
    return stored(out.reshape(T, H * vdim)) @ w["o"].T


def rotary_frequencies(rot):
    """The angle per position of each of dims/2 pairs: base^(-2i/dims), and with ``scaling`` the YaRN blend: pairs that
    turn fast keep their frequency, slow ones are divided by the factor, a linear ramp between. Returns (frequencies,
    the factor that multiplies cos and sin)."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    i = np.arange(half, dtype=np.float64)
    freq = base ** (-2.0 * i / dims)
    scaling = rot.get("scaling")
    if not scaling:
        return freq, 1.0
    factor, original = scaling["factor"], scaling["original"]

    def pair_of(turns):   # the pair whose wavelength fits `turns` times into the original length
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(scaling["fast"])), 0)
    hi = min(math.ceil(pair_of(scaling["slow"])), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    freq = freq / factor * ramp + freq * (1.0 - ramp)
    return freq, 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, rot):
    """x [..., T, heads?, dims]: element i pairs with i + dims/2: (u, v) -> (u c - v s, v c + u s). x is [T, ..., dims]
    with the positions along the first axis."""
    freq, magnitude = rotary_frequencies(rot)
    half = rot["dims"] // 2
    angle = np.asarray(positions, dtype=np.float64)[:, None] * freq[None, :]
    c, s = np.cos(angle) * magnitude, np.sin(angle) * magnitude
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (half,)
    c, s = c.reshape(shape), s.reshape(shape)
    u, v = x[..., :half], x[..., half : 2 * half]
    return np.concatenate([u * c - v * s, v * c + u * s, x[..., 2 * half :]], axis=-1)


def latent_of(h, w, mixer, eps, first_position=0, stored=_keep):
    """What a latent-attention layer keeps per token: the normed latent c [T, r] and the rotated key part [T, n]."""
    r = mixer["kv_rank"]
    T = h.shape[0]
    both = stored(h @ w["dkv"].T)
    c = stored(rms_norm(both[:, :r], w["dkv.norm"], eps))
    k_rot = stored(rotate_half(both[:, r:], first_position + np.arange(T), mixer["rot"]))
    return c, k_rot


def latent_attention(h, w, mixer, eps, latent, first_position=0, stored=_keep):
    """Attention whose keys and values are expanded per head from a shared latent; a rotated part shared by all heads;
    a sink in the softmax; a sigmoid gate on the heads' outputs. ``latent`` = (c, k_rot) of this layer or of the layer
    it borrows from."""
    T = h.shape[0]
    H, dim, n, vdim, r = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"], mixer["kv_rank"]
    c, k_rot = latent
    q = stored(h @ w["q"].T).reshape(T, H, dim + n)
    q_plain = q[:, :, :dim]
    q_rot = stored(rotate_half(q[:, :, dim:], first_position + np.arange(T), mixer["rot"]))
    k_plain = stored(c @ w["uk"].T).reshape(-1, H, dim)
    v = stored(c @ w["uv"].T).reshape(-1, H, vdim)
    visible = causal_mask(T, c.shape[0], first_position)
    out = np.zeros((T, H, vdim), dtype=h.dtype)
    for head in range(H):
        scores = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * mixer["scale"]
        out[:, head] = softmax_rows(scores, visible, sink=float(w["sink"][head])) @ v[:, head]
    gate = sigmoid(stored(h @ w["g"].T))
    return stored(stored(out.reshape(T, H * vdim)) * gate) @ w["o"].T


# --------------------------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------------------------
def layer_weights(weights, index, part):
    prefix = f"l{index}.{part}."
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def forward(config, weights, tokens, dtype=np.float64, stored=_keep, layer_outputs=None):
    """Logits [T, vocab] of a whole sequence from position 0. ``stored``: the rounding applied where a run in reduced
    precision stores activations. ``layer_outputs``: a list that receives the stream after every layer."""
    weights = {name: np.asarray(value).astype(dtype) if np.asarray(value).dtype.kind == "f" else value for name, value in weights.items()}
    eps, alpha = config["norm"]["eps"], config["postln_alpha"]
    x = weights["embed"][np.asarray(tokens, dtype=np.int64)] * config["embedding"]["scale"]
    latents = {}
    for index, layer in enumerate(config["layers"]):
        mixer, w = layer["mixer"], layer_weights(weights, index, "mix")
        h = stored(x)
        if layer["type"] == "attention":
            mixed = normed_attention(h, w, mixer, eps, stored=stored)
        elif layer["type"] == "latent_attention":
            source = mixer.get("kv_from")
            if source is None:
                latents[index] = latent_of(h, w, mixer, eps, stored=stored)
                source = index
            mixed = latent_attention(h, w, mixer, eps, latents[source], stored=stored)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = rms_norm(alpha * x + mixed, weights[f"l{index}.norm1"], eps, one_plus=True)
        if layer.get("mlp") is not None:
            m = layer_weights(weights, index, "mlp")
            x = rms_norm(alpha * x + gated_mlp(stored(x), m["gate"], m["up"], m["down"], stored), weights[f"l{index}.norm2"], eps, one_plus=True)
        if layer_outputs is not None:
            layer_outputs.append(x.copy())
    x = stored(rms_norm(x, weights["final.norm"], eps, one_plus=True))
    return x @ weights["head"].T


def greedy(config, weights, prompt, n_new, dtype=np.float64):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(np.argmax(forward(config, weights, tokens, dtype)[-1])))
    return tokens[len(prompt):]


# --------------------------------------------------------------------------------------------
# random models
# --------------------------------------------------------------------------------------------
def tensor_shapes(config):
    d, out = config["width"], {}
    out["embed"] = (config["vocab"], d)
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}."
        out[p + "norm1"] = (d,)
        if layer["type"] == "attention":
            out[p + "mix.q"] = (m["heads"] * m["dim"], d)
            out[p + "mix.k"] = (m["kv_heads"] * m["dim"], d)
            out[p + "mix.v"] = (m["kv_heads"] * m["vdim"], d)
            out[p + "mix.q.norm"] = (m["dim"],)
            out[p + "mix.k.norm"] = (m["dim"],)
            out[p + "mix.o"] = (d, m["heads"] * m["vdim"])
        else:
            out[p + "mix.q"] = (m["heads"] * (m["dim"] + m["rot_dim"]), d)
            if m.get("kv_from") is None:
                out[p + "mix.dkv"] = (m["kv_rank"] + m["rot_dim"], d)
                out[p + "mix.dkv.norm"] = (m["kv_rank"],)
            out[p + "mix.uk"] = (m["heads"] * m["dim"], m["kv_rank"])
            out[p + "mix.uv"] = (m["heads"] * m["vdim"], m["kv_rank"])
            out[p + "mix.sink"] = (m["heads"],)
            out[p + "mix.g"] = (m["heads"] * m["vdim"], d)
            out[p + "mix.o"] = (d, m["heads"] * m["vdim"])
        if layer.get("mlp") is not None:
            out[p + "norm2"] = (d,)
            out[p + "mlp.gate"] = (layer["mlp"]["ff"], d)
            out[p + "mlp.up"] = (layer["mlp"]["ff"], d)
            out[p + "mlp.down"] = (d, layer["mlp"]["ff"])
    out["final.norm"] = (d,)
    out["head"] = (config["vocab"], d)
    return out


def random_weights(config, seed, bf16=True):
    """Weights whose activations stay of order one through the layers: matrices ~ N(0, 1/in), gains stored around
    zero, norm gains of the heads around one, sinks of order one. Rounded to bfloat16 values (as files hold them)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        if name.endswith(".sink"):
            value = rng.normal(0.0, 1.0, shape)
        elif name.endswith("q.norm") or name.endswith("k.norm") or name.endswith("dkv.norm"):
            value = 1.0 + rng.normal(0.0, 0.1, shape)
        elif len(shape) == 1:
            value = rng.normal(0.0, 0.1, shape)
        elif name == "embed":
            value = rng.normal(0.0, 1.0 / max(config["embedding"]["scale"], 1e-6), shape)
        else:
            value = rng.normal(0.0, 1.0 / math.sqrt(shape[1]), shape)
        value = value.astype(np.float32)
        out[name] = plain_gpt2.round_to_bf16(value) if bf16 else value
    return out


def write_model_dir(path, config, weights, bf16=True):
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(config, indent=1))
    plain_gpt2.write_safetensors(path / "model.safetensors", {k: np.asarray(v, dtype=np.float32) for k, v in weights.items()}, bf16=bf16)
    return path


def load_model_dir(path):
    path = Path(path)
    config = json.loads((path / "config.json").read_text())
    return config, plain_gpt2.read_safetensors(path / "model.safetensors")
