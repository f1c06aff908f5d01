"""A plain, slow implementation of the Ketolix design: numpy, float64, whole sequences, token by token where the design
is recurrent, no cache, no batching. One function per mechanism; the framework's parts and kernels are compared with these.

A model is (config, tensors): ``config`` the dictionary that config.json holds, ``tensors`` name -> float64 array. A layer is
x <- x + norm1(mixer(x)), then x <- x + norm2(ff(x)): the branches read the stream itself and the norm sits on their output.

``round_to`` (optional, a function array -> array) is applied where a bfloat16 run stores something in bfloat16: the inputs
of matrix products and what lies in the cache. None: exact arithmetic."""

from __future__ import annotations

import numpy as np


def _same(x):
    return x


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def product(x, w, rnd=_same):
    """Rows of x times W^T, W stored [out, in]."""
    return rnd(x) @ rnd(w).T


# -- rotation -----------------------------------------------------------------------------------------------------------
def rotary_frequencies(rot: dict) -> np.ndarray:
    """Angle per position of each rotated pair: base^(-2i/dims), the slow pairs stretched where ``scaling`` says so."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = base ** (-2.0 * np.arange(dims // 2) / dims)
    scaling = rot.get("scaling")
    if scaling:
        factor, low, high, original = (float(scaling[key]) for key in ("factor", "low", "high", "original"))
        out = np.empty_like(f)
        for i, fi in enumerate(f):
            wavelength = 2.0 * np.pi / fi
            if wavelength < original / high:
                out[i] = fi
            elif low > 0 and wavelength > original / low:
                out[i] = fi / factor
            else:
                s = (original / wavelength - low) / (high - low)
                out[i] = (1.0 - s) * fi / factor + s * fi
        f = out
    return f


def rotate_pairs(x, positions, rot: dict | None):
    """x: [tokens, heads, dim]; elements 2i and 2i+1 of the first rot.dims of every head turn by position * f_i."""
    if not rot or not int(rot["dims"]):
        return x
    dims = int(rot["dims"])
    angles = np.asarray(positions, dtype=np.float64)[:, None] * rotary_frequencies(rot)[None, :]   # [T, dims/2]
    c, s = np.cos(angles)[:, None, :], np.sin(angles)[:, None, :]
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# -- attention over a window, with the options the design's two attention mixers pick from -------------------------------
def windowed_attention(q, k, v, scale, window=None, softcap=None, sinks=None):
    """q: [T, H, dim], k: [T, G, dim], v: [T, G, vdim] -> [T, H, vdim]. Query i sees keys j with 0 <= i - j < window.
    ``softcap``: score <- cap * tanh(score / cap). ``sinks`` [H]: exp(sink_h) joins the softmax's denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if window is None else max(0, i - int(window) + 1)
            s = (k[lo : i + 1, g] @ q[i, h]) * scale
            if softcap:
                s = softcap * np.tanh(s / softcap)
            top = s.max() if sinks is None else max(s.max(), sinks[h])
            w = np.exp(s - top)
            total = w.sum() + (0.0 if sinks is None else np.exp(sinks[h] - top))
            out[i, h] = (w / total) @ v[lo : i + 1, g]
    return out


def short_convolution(u, w):
    """u: [T, channels], w: [channels, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], axis=0)
    return sum(padded[j : j + T] * w[:, j][None, :] for j in range(taps))


# -- the recurrent mixers, token by token -------------------------------------------------------------------------------
def mlstm_recurrence(q, k, v, log_in, log_forget):
    """q, k: [T, H, dim] (q already scaled), v: [T, H, vdim], the log gates [T, H] -> [T, H, vdim]. Matrix memory with a
    running maximum that starts at 0."""
    T, H, dim = q.shape
    vdim = v.shape[2]
    out = np.zeros((T, H, vdim))
    for h in range(H):
        S, n, m = np.zeros((dim, vdim)), np.zeros(dim), 0.0
        for t in range(T):
            m_new = max(log_forget[t, h] + m, log_in[t, h])
            keep, take = np.exp(log_forget[t, h] + m - m_new), np.exp(log_in[t, h] - m_new)
            S = keep * S + take * np.outer(k[t, h], v[t, h])
            n = keep * n + take * k[t, h]
            m = m_new
            out[t, h] = (S.T @ q[t, h]) / (max(abs(n @ q[t, h]), np.exp(-m)) + 1e-6)
    return out


def decayed_recurrence(q, k, v, decay):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t. q, k: [T, H, dim], v: [T, H, vdim], decay [H]."""
    T, H, dim = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        S = np.zeros((dim, v.shape[2]))
        for t in range(T):
            S = decay[h] * S + np.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


# -- mixers ---------------------------------------------------------------------------------------------------------------
def mlstm_mixer(h, w: dict, mixer: dict, eps: float, rnd=_same):
    """w: the layer's '.mix.' tensors by their names behind that prefix."""
    H, dim, vdim = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = product(h, w["q"], rnd).reshape(T, H, dim) * dim ** -0.5
    k = product(h, w["k"], rnd).reshape(T, H, dim)
    v = product(h, w["v"], rnd).reshape(T, H, vdim)
    cap = mixer.get("gate_cap")
    capped = (lambda z: cap * np.tanh(z / cap)) if cap else _same
    log_in = capped(product(h, w["i"], rnd) + w["i.b"])
    log_forget = log_sigmoid(capped(product(h, w["f"], rnd) + w["f.b"]))
    o = rms_unit(mlstm_recurrence(q, k, v, log_in, log_forget), eps).reshape(T, H * vdim)
    o = o * w["norm"] * sigmoid(product(h, w["g"], rnd))
    return product(o, w["o"], rnd)


def attention_mixer(h, w: dict, mixer: dict, eps: float, positions, v_first=None, rnd=_same):
    """Returns (output, the values as cached). ``v_first``: the values of the first value-mixing layer, None in that layer
    itself and in layers that do not mix."""
    H, G, dim, vdim = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = rms_unit(product(h, w["q"], rnd), eps) * w["q.norm"]
    k = rms_unit(product(h, w["k"], rnd), eps) * w["k.norm"]
    v = product(h, w["v"], rnd)
    q = rotate_pairs(q.reshape(T, H, dim), positions, mixer.get("rot"))
    k = rotate_pairs(k.reshape(T, G, dim), positions, mixer.get("rot"))
    if v_first is not None:
        lam = float(w["vmix"])
        v = (1.0 - lam) * v + lam * v_first
    window = (mixer.get("mask") or {}).get("size")
    o = windowed_attention(rnd(q), rnd(k), rnd(v).reshape(T, G, vdim), float(mixer["scale"]), window, mixer.get("softcap"), w.get("sink"))
    return product(o.reshape(T, H * vdim), w["o"], rnd), v


def parallel_mixer(h, w: dict, mixer: dict, eps: float, positions, rnd=_same):
    """Two mixers side by side on the same input: attention whose values are its keys, and a decayed linear recurrence."""
    T = h.shape[0]
    left, right = mixer["left"], mixer["right"]
    # left
    H, G, dim = int(left["heads"]), int(left["kv_heads"]), int(left["dim"])
    q = product(h, w["left.q"], rnd) + w["left.q.b"]
    k = product(h, w["left.k"], rnd) + w["left.k.b"]
    if left.get("conv"):
        q, k = short_convolution(q, w["left.q.conv"]), short_convolution(k, w["left.k.conv"])
    v = k.reshape(T, G, dim)
    qn = rotate_pairs((rms_unit(q, eps) * w["left.q.norm"]).reshape(T, H, dim), positions, left.get("rot"))
    kn = rotate_pairs((rms_unit(k, eps) * w["left.k.norm"]).reshape(T, G, dim), positions, left.get("rot"))
    window = (left.get("mask") or {}).get("size")
    o = windowed_attention(rnd(qn), rnd(kn), rnd(v), float(left["scale"]), window)
    o = o * sigmoid(product(h, w["left.g"], rnd))[:, :, None]
    out_left = product(o.reshape(T, -1), w["left.o"], rnd) + w["left.o.b"]
    # right
    Hr, dr, vr = int(right["heads"]), int(right["dim"]), int(right["vdim"])
    qr = silu(product(h, w["right.q"], rnd)).reshape(T, Hr, dr)
    kr = silu(product(h, w["right.k"], rnd)).reshape(T, Hr, dr)
    vr_ = silu(product(h, w["right.v"], rnd)).reshape(T, Hr, vr)
    o = decayed_recurrence(qr, kr, vr_, np.asarray(right["decay"], dtype=np.float64)).reshape(T, Hr * vr)
    o = rms_unit(o, eps) * w["right.norm"] * sigmoid(product(h, w["right.g"], rnd))
    out_right = product(o, w["right.o"], rnd)
    return float(mixer["left_scale"]) * out_left + float(mixer["right_scale"]) * out_right


def dense_feed_forward(h, w: dict, rnd=_same):
    return product(silu(product(h, w["gate"], rnd)) * product(h, w["up"], rnd), w["down"], rnd)


# -- the model ------------------------------------------------------------------------------------------------------------
def _under(tensors: dict, prefix: str) -> dict:
    return {name[len(prefix):]: value for name, value in tensors.items() if name.startswith(prefix)}


def forward(config: dict, tensors: dict, tokens, round_to=None, layers_out: list | None = None) -> np.ndarray:
    """Logits [tokens, vocab] of one whole sequence. ``layers_out``: a list that receives the stream after every layer."""
    rnd = round_to or _same
    eps = float(config["norm"]["eps"])
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x = tensors["embed"][tokens].astype(np.float64)
    v_first = None
    for index, layer in enumerate(config["layers"]):
        prefix = f"l{index}."
        w = _under(tensors, prefix + "mix.")
        kind, mixer = layer["type"], layer["mixer"]
        if kind == "mlstm":
            branch = mlstm_mixer(x, w, mixer, eps, rnd)
        elif kind == "attention":
            mixes = bool(mixer.get("v_mix"))
            branch, v = attention_mixer(x, w, mixer, eps, positions, v_first if mixes else None, rnd)
            if mixes and v_first is None:
                v_first = v
        elif kind == "parallel":
            branch = parallel_mixer(x, w, mixer, eps, positions, rnd)
        else:
            raise ValueError(f"unknown layer type {kind!r}")
        x = x + rms_unit(branch, eps) * tensors[prefix + "norm1"]
        if layer.get("mlp"):
            x = x + rms_unit(dense_feed_forward(x, _under(tensors, prefix + "mlp."), rnd), eps) * tensors[prefix + "norm2"]
        if layers_out is not None:
            layers_out.append(x.copy())
    x = rms_unit(x, eps) * tensors["final.norm"]
    return product(x, tensors["embed"], rnd)


def greedy(config: dict, tensors: dict, prompt, n_new: int, round_to=None) -> list:
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(config, tensors, tokens, round_to)[-1].argmax()))
    return tokens[len(prompt):]


# -- random models for the tests ------------------------------------------------------------------------------------------
def tensor_shapes(config: dict) -> dict:
    """name -> shape of every tensor a model of this configuration has."""
    width = int(config["width"])
    shapes = {"embed": (int(config["vocab"]), width), "final.norm": (width,)}
    for index, layer in enumerate(config["layers"]):
        p, m = f"l{index}.", layer["mixer"]
        shapes[p + "norm1"] = (width,)
        if layer["type"] == "mlstm":
            H, d, e = m["heads"], m["dim"], m["vdim"]
            shapes.update({p + "mix.q": (H * d, width), p + "mix.k": (H * d, width), p + "mix.v": (H * e, width), p + "mix.g": (H * e, width),
                           p + "mix.o": (width, H * e), p + "mix.norm": (H * e,), p + "mix.i": (H, width), p + "mix.i.b": (H,),
                           p + "mix.f": (H, width), p + "mix.f.b": (H,)})
        elif layer["type"] == "attention":
            H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            shapes.update({p + "mix.q": (H * d, width), p + "mix.k": (G * d, width), p + "mix.v": (G * e, width), p + "mix.q.norm": (H * d,),
                           p + "mix.k.norm": (G * d,), p + "mix.sink": (H,), p + "mix.o": (width, H * e)})
            if m.get("v_mix"):
                shapes[p + "mix.vmix"] = ()
        elif layer["type"] == "parallel":
            left, right = m["left"], m["right"]
            H, G, d = left["heads"], left["kv_heads"], left["dim"]
            shapes.update({p + "mix.left.q": (H * d, width), p + "mix.left.q.b": (H * d,), p + "mix.left.k": (G * d, width), p + "mix.left.k.b": (G * d,),
                           p + "mix.left.q.norm": (H * d,), p + "mix.left.k.norm": (G * d,), p + "mix.left.g": (H, width),
                           p + "mix.left.o": (width, H * d), p + "mix.left.o.b": (width,)})
            if left.get("conv"):
                shapes.update({p + "mix.left.q.conv": (H * d, left["conv"]), p + "mix.left.k.conv": (G * d, left["conv"])})
            H, d, e = right["heads"], right["dim"], right["vdim"]
            shapes.update({p + "mix.right.q": (H * d, width), p + "mix.right.k": (H * d, width), p + "mix.right.v": (H * e, width),
                           p + "mix.right.g": (H * e, width), p + "mix.right.o": (width, H * e), p + "mix.right.norm": (H * e,)})
        if layer.get("mlp"):
            ff = layer["mlp"]["ff"]
            shapes.update({p + "norm2": (width,), p + "mlp.gate": (ff, width), p + "mlp.up": (ff, width), p + "mlp.down": (width, ff)})
    return shapes


def random_weights(config: dict, seed: int) -> dict:
    """Weights whose activations stay of order one: matrices ~ N(0, 1/in), gains around one, biases and sinks of order one, forget
    biases well above zero. float32 arrays holding bfloat16 values (as files hold them)."""
    import plain_gpt2

    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith(".sink"):
            value = rng.normal(0.0, 1.0, shape)
        elif name.endswith(".vmix"):
            value = rng.uniform(0.2, 0.8, shape)
        elif name.endswith(".f.b"):
            value = rng.normal(3.0, 0.5, shape)
        elif name.endswith(".conv"):
            value = rng.normal(0.0, shape[1] ** -0.5, shape)
        elif last in ("norm", "norm1", "norm2"):
            value = 1.0 + rng.normal(0.0, 0.1, shape)
        elif last == "b":
            value = rng.normal(0.0, 0.3, shape)
        elif name == "embed":
            value = rng.normal(0.0, 1.0, shape)
        else:
            value = rng.normal(0.0, shape[1] ** -0.5, shape)
        out[name] = plain_gpt2.round_to_bf16(np.asarray(value, dtype=np.float32))
    return out


def as_float64(weights: dict) -> dict:
    return {name: np.asarray(value, dtype=np.float64) for name, value in weights.items()}


def write_model_dir(path, config: dict, weights: dict):
    import json
    from pathlib import Path

    import plain_gpt2

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(config, indent=1))
    plain_gpt2.write_safetensors(path / "model.safetensors", {k: np.asarray(v, dtype=np.float32) for k, v in weights.items()}, bf16=True)
    return path
