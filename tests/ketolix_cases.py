"""Small Ketolix configurations for the tests: sizes, options and orders of layers that differ in every way the design allows."""


def mlp(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def rot(dims, base=10000.0, scaling=None):
    out = {"dims": dims, "base": base}
    if scaling:
        out["scaling"] = {"factor": scaling[0], "low": scaling[1], "high": scaling[2], "original": scaling[3]}
    return out


def mlstm_layer(heads=2, dim=16, vdim=24, cap=8.0, ff=48):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim}
    if cap is not None:
        mixer["gate_cap"] = cap
    return {"type": "mlstm", "mixer": mixer, "mlp": mlp(ff)}


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.25, softcap=15.0, window=40, rotation=None, v_mix=False, ff=48):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap is not None:
        mixer["softcap"] = softcap
    if window is not None:
        mixer["mask"] = {"size": window}
    if rotation is not None:
        mixer["rot"] = rotation
    if v_mix:
        mixer["v_mix"] = True
    return {"type": "attention", "mixer": mixer, "mlp": mlp(ff)}


def parallel_layer(heads=4, kv_heads=2, dim=24, scale=0.2, conv=3, window=33, rotation=None, right_heads=3, right_dim=8, right_vdim=40,
                   decay=(0.6, 0.9, 0.995), left_scale=0.7, right_scale=0.4, ff=48):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if conv is not None:
        left["conv"] = conv
    if window is not None:
        left["mask"] = {"size": window}
    if rotation is not None:
        left["rot"] = rotation
    right = {"heads": right_heads, "dim": right_dim, "vdim": right_vdim, "decay": list(decay)}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp(ff)}


def model(layers, width=64, vocab=97, eps=1e-5):
    return {"architecture": "Ketolix", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


CASES = {
    # every kind of layer, two of each; values mixed over three attention layers with different heads; grouped heads; a rotation of a
    # part of the heads with stretched wavelengths, one of whole heads without; windows shorter and longer than a page, and none
    "mixed": model([
        attention_layer(v_mix=True, rotation=rot(8, 500.0, (4.0, 1.0, 4.0, 32))),
        mlstm_layer(),
        attention_layer(heads=2, kv_heads=1, dim=16, vdim=32, softcap=None, window=None, v_mix=True),
        parallel_layer(rotation=rot(24, 2000.0)),
        attention_layer(heads=2, kv_heads=2, dim=24, vdim=16, window=70, v_mix=True, rotation=rot(24, 100.0, (8.0, 0.0, 2.0, 16)), ff=None),
        mlstm_layer(heads=3, dim=8, vdim=8, cap=None, ff=None),
        parallel_layer(heads=2, kv_heads=2, dim=16, conv=None, window=None, right_heads=1, right_dim=16, right_vdim=16, decay=(0.97,), ff=None),
    ]),
    # sizes that are no multiples of anything a kernel would like; a parallel layer first; one key/value head; a window of five
    "odd": model([
        parallel_layer(heads=5, kv_heads=1, dim=20, conv=2, window=5, rotation=rot(6, 777.0), right_heads=2, right_dim=12, right_vdim=20,
                       decay=(0.5, 0.999), left_scale=1.3, right_scale=1.0, ff=90),
        mlstm_layer(heads=5, dim=20, vdim=12, cap=3.0, ff=None),
        attention_layer(heads=5, kv_heads=1, dim=20, vdim=12, scale=0.3, softcap=4.0, window=5, rotation=rot(20, 50.0), ff=90),
    ], width=100, vocab=77, eps=1e-6),
    # heads of powers of two (the split-key kernel decodes them), matrices of several rows a thread and of several tiles of columns,
    # a window of exactly one page, five taps
    "wide": model([
        mlstm_layer(heads=2, dim=64, vdim=64, cap=12.0, ff=96),
        attention_layer(heads=2, kv_heads=1, dim=32, vdim=64, scale=0.18, softcap=30.0, window=64, rotation=rot(32, 10000.0)),
        parallel_layer(heads=2, kv_heads=1, dim=32, conv=5, window=64, rotation=rot(16, 300.0), right_heads=2, right_dim=16, right_vdim=130,
                       decay=(0.8, 0.99)),
    ], width=96, vocab=130),
    # heads of 80 to 128 (pages of 96 and 128 elements a head: other attention kernels than heads of 64 take), matrices of 96 x 128
    # and 128 x 96 (chunks of 32 rows), no softcap beside a softcap, a convolution of three taps on heads of 96
    "large": model([
        attention_layer(heads=4, kv_heads=2, dim=80, vdim=96, scale=80 ** -0.5, softcap=25.0, window=100, rotation=rot(40, 20000.0, (8.0, 1.0, 4.0, 64)), v_mix=True),
        mlstm_layer(heads=2, dim=96, vdim=128, cap=10.0, ff=None),
        attention_layer(heads=2, kv_heads=1, dim=128, vdim=192, scale=128 ** -0.5, softcap=None, window=None, rotation=rot(128, 300.0), v_mix=True, ff=None),
        parallel_layer(heads=2, kv_heads=2, dim=96, scale=96 ** -0.5, conv=3, window=72, rotation=rot(24, 5000.0), right_heads=2, right_dim=64, right_vdim=32,
                       decay=(0.9, 0.99), ff=200),
        mlstm_layer(heads=1, dim=128, vdim=96, cap=None, ff=None),
    ], width=160, vocab=211),
}
