"""Each mechanism of the Ketolix design alone: the kernel against the plain function of tests/plain_ketolix.py."""

import numpy as np
import pytest
import torch

import plain_ketolix as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def kernels():
    from mini_llm_amd.ops import kernels

    return kernels


def gpu(array, dtype=torch.float32):
    return torch.tensor(np.asarray(array), dtype=torch.float32).to(dtype).cuda().contiguous()


def ints(values):
    return torch.tensor(np.asarray(values), dtype=torch.int32).cuda()


def rounded(array, dtype):
    return torch.tensor(np.asarray(array), dtype=torch.float32).to(dtype).to(torch.float32).numpy().astype(np.float64)


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("width", [5, 64, 300, 2500])
def test_norm_of_a_branch_joins_the_stream(width):
    rng = np.random.default_rng(width)
    stream, branch, w = rng.normal(0, 2, (7, width)), rng.normal(0, 3, (7, width)), rng.normal(1, 0.3, width)
    k = kernels()
    want = stream + plain.rms_unit(branch, 1e-5) * w
    total, rows = k.rms_norm(gpu(branch), gpu(w), 1e-5, residual=gpu(stream), out_dtype=torch.bfloat16, with_stream=True)
    np.testing.assert_allclose(total.cpu().numpy(), want, atol=2e-5, rtol=2e-5)
    assert torch.equal(rows, total.to(torch.bfloat16))
    # the branch as the partial products of a product cut along K
    parts = rng.normal(0, 1, (4, 7, width))
    got = k.rms_norm(gpu(parts[0]), gpu(w), 1e-5, addend=gpu(parts[1:]), residual=gpu(stream))
    np.testing.assert_allclose(got.cpu().numpy(), stream + plain.rms_unit(parts.sum(axis=0), 1e-5) * w, atol=2e-5, rtol=2e-5)


def test_wavelength_scaling_of_the_rotation():
    from mini_llm_amd.parts import RotaryEncoding

    # wavelengths on both sides of both borders: kept, blended, divided
    for scaling in ((8.0, 1.0, 4.0, 64), (3.0, 0.0, 2.0, 16), (2.0, 2.0, 16.0, 4096)):
        rot = {"dims": 32, "base": 5000.0, "scaling": dict(zip(("factor", "low", "high", "original"), scaling))}
        part = RotaryEncoding(32, 5000.0, {"kind": "wavelength", **rot["scaling"]}, pairing="neighbours")
        want = plain.rotary_frequencies(rot)
        plain_f = 5000.0 ** (-2.0 * np.arange(16) / 32)
        np.testing.assert_allclose(part.values, want, rtol=1e-13)
        if scaling[1] > 0:
            assert (want == plain_f).any() and np.isclose(want, plain_f / scaling[0]).any()
        assert (~np.isclose(want, plain_f) & ~np.isclose(want, plain_f / scaling[0])).any()   # some pair lies between


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,vdim,heads,kv_heads,rot_dims", [(16, 16, 4, 2, 8), (24, 8, 3, 3, 24), (8, 40, 2, 1, 0), (64, 64, 6, 2, 64), (10, 6, 3, 3, 4)])
def test_projection_rows_norm_rotate_blend_and_store(dtype, dim, vdim, heads, kv_heads, rot_dims):
    k = kernels()
    rng = np.random.default_rng(dim + vdim)
    rows, page_size, n_pages, eps = 9, 4, 8, 1e-5
    head_size = -(-max(dim, vdim) // 16) * 16
    qw, kw, vw = heads * dim, kv_heads * dim, kv_heads * vdim
    fused = rng.normal(0, 2, (rows, qw + kw + vw + 3)).astype(np.float32).astype(np.float64)
    other = rng.normal(0, 2, (rows, vw)).astype(np.float32).astype(np.float64)
    qg, kg = rng.normal(1, 0.2, qw), rng.normal(1, 0.2, kw)
    positions = np.array([0, 1, 2, 63, 64, 65, 500, 1100, 7])
    slots = np.array([5, 4, 31, -1, 0, 1, 2, 3, 17])
    rot = {"dims": rot_dims, "base": 300.0}
    frequencies = torch.tensor(plain.rotary_frequencies(rot), dtype=torch.float64).cuda() if rot_dims else None
    k_pages = torch.full((n_pages, kv_heads, page_size, head_size), 7.0, dtype=dtype).cuda()
    v_pages = torch.full_like(k_pages, 7.0)
    f = gpu(fused)
    for blend in (None, 0.3):
        q = k.projection_rows(f[:, :qw], f[:, qw : qw + kw], f[:, qw + kw : qw + kw + vw], gpu(qg), gpu(kg), eps, frequencies, rot_dims, ints(positions),
                              ints(slots), k_pages, v_pages, heads, kv_heads, dim, vdim, v_other=None if blend is None else gpu(other),
                              mix=None if blend is None else gpu([blend]))
        want_q = plain.rotate_pairs((plain.rms_unit(fused[:, :qw], eps) * qg).reshape(rows, heads, dim), positions, rot)
        want_k = plain.rotate_pairs((plain.rms_unit(fused[:, qw : qw + kw], eps) * kg).reshape(rows, kv_heads, dim), positions, rot)
        want_v = fused[:, qw + kw : qw + kw + vw]
        if blend is not None:
            want_v = (1 - blend) * want_v + blend * other
        want_v = want_v.reshape(rows, kv_heads, vdim)
        got_q = q.float().cpu().numpy().reshape(rows, heads, head_size)
        loose = tol(dtype)   # (angles are taken in 64-bit: position 1,100 is as good as position 1)
        np.testing.assert_allclose(got_q[:, :, :dim], want_q, **loose)
        assert (got_q[:, :, dim:] == 0).all()
        kp, vp = k_pages.float().cpu().numpy(), v_pages.float().cpu().numpy()
        for row, slot in enumerate(slots):
            if slot < 0:
                continue
            page, offset = divmod(int(slot), page_size)
            np.testing.assert_allclose(kp[page, :, offset, :dim], want_k[row], **loose)
            np.testing.assert_allclose(vp[page, :, offset, :vdim], want_v[row], **tol(dtype))
            assert (kp[page, :, offset, dim:] == 0).all() and (vp[page, :, offset, vdim:] == 0).all()
        assert (kp[6] == 7).all() and (vp[5] == 7).all()   # pages no slot names are left alone


def test_projection_rows_norms_the_whole_projection_not_each_head():
    # one head far larger than the other: normed together, the small head stays small
    k = kernels()
    q = np.concatenate([np.full((1, 8), 10.0), np.full((1, 8), 0.1)], axis=1)
    pages = torch.zeros((1, 1, 4, 16)).cuda()
    got = k.projection_rows(gpu(q), gpu(q[:, :8]), gpu(q[:, :8]), gpu(np.ones(16)), gpu(np.ones(8)), 1e-6, None, 0, ints([0]), ints([0]), pages, pages.clone(),
                            2, 1, 8, 8).cpu().numpy()
    got = got.reshape(2, 16)   # heads of 8 in places of 16
    np.testing.assert_allclose(got[:, :8].reshape(1, 16), plain.rms_unit(q, 1e-6), rtol=1e-5)
    assert got[1, 0] < 0.02 < 1.0 < got[0, 0] and (got[:, 8:] == 0).all()


def batch_of(portions, slots):
    """q_starts, token_request and state_slots of a step whose requests bring ``portions`` rows each."""
    starts = np.concatenate([[0], np.cumsum(portions)])
    request = np.concatenate([np.full(n, i) for i, n in enumerate(portions)]) if sum(portions) else np.zeros(0)
    return ints(starts), ints(request), ints(slots)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_short_convolution_carries_its_last_inputs_from_step_to_step(taps):
    k = kernels()
    rng = np.random.default_rng(taps)
    channels, lengths = 37, [23, 9]
    u = [rng.normal(0, 1, (n, channels)) for n in lengths]
    w = rng.normal(0, 1, (channels, taps))
    want = [plain.short_convolution(x, w) for x in u]
    kept = torch.full((5, max(taps - 1, 1) * channels + 3), 0.0).cuda()
    kept[2] = 9.0   # a slot nobody holds
    view = kept[:, : (taps - 1) * channels] if taps > 1 else None
    # portions of 1, 2, 3, ... rows of request 0 beside single rows of request 1 (slots 3 and 0), a padding request between them
    fed, got, size = [0, 0], [[], []], 1
    while fed[0] < lengths[0] or fed[1] < lengths[1]:
        portions = [min(size, lengths[0] - fed[0]), 0, min(1, lengths[1] - fed[1])]
        rows = np.concatenate([u[0][fed[0] : fed[0] + portions[0]], u[1][fed[1] : fed[1] + portions[2]]])
        starts, request, slots = batch_of(portions, [3, -1, 0])
        y = k.short_conv(gpu(rows), gpu(w), view, request, starts, slots).cpu().numpy()
        got[0].append(y[: portions[0]])
        got[1].append(y[portions[0] :])
        fed = [fed[0] + portions[0], fed[1] + portions[2]]
        size += 1
    for i in range(2):
        np.testing.assert_allclose(np.concatenate(got[i]), want[i], atol=1e-5, rtol=1e-5)
    if taps > 1:
        np.testing.assert_allclose(kept[3, : (taps - 1) * channels].cpu().numpy().reshape(taps - 1, channels), u[0][-(taps - 1):], rtol=1e-6)
    assert (kept[2] == 9.0).all() and (kept[:, (taps - 1) * channels :][[0, 1, 3, 4]] == 0).all()


def test_gates_of_heads_and_of_elements():
    k = kernels()
    rng = np.random.default_rng(2)
    for dtype in DTYPES:
        x = rounded(rng.normal(0, 2, (6, 3 * 16 + 5)), dtype)
        gate = rng.normal(0, 2, (6, 3 + 2))
        out = torch.zeros((6, 3 * 16 + 9), dtype=dtype).cuda()
        k.head_gate(gpu(x, dtype), gpu(gate)[:, 1:4], out, 3, 16, scale=0.8)
        want = (x[:, :48].reshape(6, 3, 16) * plain.sigmoid(gate[:, 1:4])[:, :, None] * 0.8).reshape(6, 48)
        np.testing.assert_allclose(out.float().cpu().numpy()[:, :48], want, **tol(dtype))
        assert (out[:, 48:] == 0).all()
    x, w, gate = rng.normal(0, 3, (5, 90)), rng.normal(1, 0.2, 90), rng.normal(0, 2, (5, 90))
    for group in (None, 30, 5, 90):
        out = torch.zeros((5, 96)).cuda()
        k.gated_norm(gpu(x), gpu(w), gpu(gate), 1e-5, out, group=group, scale=0.5)
        unit = plain.rms_unit(x.reshape(5, -1, group or 90), 1e-5).reshape(5, 90)
        np.testing.assert_allclose(out.cpu().numpy()[:, :90], unit * w * plain.sigmoid(gate) * 0.5, atol=2e-5, rtol=2e-5)
    # wide groups (a block each): in registers up to 2,048 elements, read twice beyond
    wide, gains, gates = rng.normal(0, 3, (3, 5200)), rng.normal(1, 0.2, 5200), rng.normal(0, 2, (3, 5200))
    for group in (None, 2600, 1300, 650, 260):
        out = torch.zeros((3, 5200), dtype=torch.bfloat16).cuda()
        k.gated_norm(gpu(wide), gpu(gains), gpu(gates), 1e-5, out, group=group, scale=0.5)
        unit = plain.rms_unit(wide.reshape(3, -1, group or 5200), 1e-5).reshape(3, 5200)
        np.testing.assert_allclose(out.float().cpu().numpy(), unit * gains * plain.sigmoid(gates) * 0.5, atol=2e-2, rtol=2e-2)
    out = torch.zeros((5, 90)).cuda()
    k.gated_norm(gpu(x), None, None, 1e-5, out, group=45)
    np.testing.assert_allclose(out.cpu().numpy(), plain.rms_unit(x.reshape(5, 2, 45), 1e-5).reshape(5, 90), atol=2e-5, rtol=2e-5)


SIZES = [(2, 16, 24), (3, 8, 8), (1, 64, 64), (2, 48, 48), (2, 16, 130), (1, 128, 128), (4, 20, 12), (1, 256, 64), (2, 1, 1), (1, 384, 70)]


def step_through(run, lengths, sizes, n_slots=6):
    """Feeds several sequences through ``run(rows of each live request, q_starts, state_slots)`` in portions of changing size,
    one request decoding token by token beside the others, a padding request among them; returns each request's rows."""
    fed, got = [0] * len(lengths), [[] for _ in lengths]
    slots = [4, 1, 3, 0][: len(lengths)]
    turn = 0
    while any(f < n for f, n in zip(fed, lengths)):
        portions = []
        for i, n in enumerate(lengths):
            size = 1 if i == 1 else sizes[(turn + i) % len(sizes)]
            portions.append(min(size, n - fed[i]))
        starts = np.concatenate([[0], np.cumsum(portions[:1] + [0] + portions[1:])])   # a padding request behind the first
        out = run([(i, fed[i], portions[i]) for i in range(len(lengths))], ints(starts), ints(slots[:1] + [-1] + slots[1:]))
        at = 0
        for i, n in enumerate(portions):
            got[i].append(out[at : at + n])
            at += n
            fed[i] += n
        turn += 1
    return [np.concatenate(g) for g in got]


@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("heads,dim,vdim", SIZES)
def test_matrix_memory_in_portions_against_token_by_token(heads, dim, vdim, chunked):
    k = kernels()
    assert k.recurrence_supported(dim, vdim)
    rng = np.random.default_rng(dim * vdim)
    lengths, cap = [70, 19, 33], 6.0
    data = []
    for n in lengths:
        q, kk, v = rng.normal(0, 1, (n, heads * dim)), rng.normal(0, 1, (n, heads * dim)), rng.normal(0, 1, (n, heads * vdim))
        gi, gf = rng.normal(0, 4, (n, heads)), rng.normal(2, 4, (n, heads))
        data.append([np.float32(a).astype(np.float64) for a in (q, kk, v, gi, gf)])
    want = []
    for q, kk, v, gi, gf in data:
        n = len(q)
        capped = lambda z: cap * np.tanh(z / cap)
        want.append(plain.mlstm_recurrence(q.reshape(n, heads, dim) * dim ** -0.5, kk.reshape(n, heads, dim), v.reshape(n, heads, vdim), capped(gi),
                                           plain.log_sigmoid(capped(gf))).reshape(n, heads * vdim))
    size = heads * dim * vdim + heads * dim + heads
    state = torch.zeros((6, size + 2)).cuda()
    state[2] = 5.0   # a slot nobody holds

    def run(parts, starts, slots):
        rows = [np.concatenate([data[i][j][at : at + n] for i, at, n in parts]) for j in range(5)]
        fused = gpu(np.concatenate(rows, axis=1))
        qw, vw = heads * dim, heads * vdim
        return k.recurrence(fused[:, :qw], fused[:, qw : 2 * qw], fused[:, 2 * qw : 2 * qw + vw], state[:, :size], starts, slots, heads, dim, vdim,
                            gate_in=fused[:, 2 * qw + vw : 2 * qw + vw + heads], gate_forget=fused[:, 2 * qw + vw + heads :], cap=cap,
                            q_scale=dim ** -0.5, max_q_len=max(n for _, _, n in parts) + 8 if chunked else None).cpu().numpy()

    got = step_through(run, lengths, sizes=(7, 2, 16, 3, 9, 64))
    for a, b in zip(got, want):
        np.testing.assert_allclose(a, b, atol=2e-4, rtol=2e-4)
    assert (state[2] == 5.0).all() and (state[5] == 0).all() and (state[:, size:][[0, 1, 3, 4]] == 0).all()


@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("heads,dim,vdim", SIZES)
def test_decayed_recurrence_in_portions_against_token_by_token(heads, dim, vdim, chunked):
    k = kernels()
    rng = np.random.default_rng(dim + vdim)
    lengths = [70, 19, 33]
    decay = rng.uniform(0.5, 0.999, heads)
    decay32 = np.float32(decay).astype(np.float64)
    data = [[np.float32(rng.normal(0, 1, (n, heads * d))).astype(np.float64) for d in (dim, dim, vdim)] for n in lengths]
    want = [plain.decayed_recurrence(plain.silu(q).reshape(len(q), heads, dim), plain.silu(kk).reshape(len(q), heads, dim),
                                     plain.silu(v).reshape(len(q), heads, vdim), decay32).reshape(len(q), heads * vdim) for q, kk, v in data]
    state = torch.zeros((6, heads * dim * vdim)).cuda()

    def run(parts, starts, slots):
        rows = [gpu(np.concatenate([data[i][j][at : at + n] for i, at, n in parts])) for j in range(3)]
        return k.recurrence(rows[0], rows[1], rows[2], state, starts, slots, heads, dim, vdim, decay=gpu(decay),
                            max_q_len=max(n for _, _, n in parts) + 8 if chunked else None).cpu().numpy()

    got = step_through(run, lengths, sizes=(5, 2, 31, 8, 70))
    for a, b in zip(got, want):
        np.testing.assert_allclose(a, b, atol=2e-4, rtol=2e-4)


def test_matrix_memory_keeps_a_token_from_hundreds_of_steps_back():
    # one early token is written with an open input gate; every later one with a closed input gate and an open forget gate: the
    # output hundreds of tokens later is still that token's value, whether the rows come at once or one by one
    k = kernels()
    n, dim, vdim = 600, 16, 16
    rng = np.random.default_rng(0)
    key = rng.normal(0, 1, dim)
    q, kk, v = np.tile(key, (n, 1)), rng.normal(0, 1, (n, dim)), rng.normal(0, 1, (n, vdim))
    kk[3] = key
    gi, gf = np.full((n, 1), -30.0), np.full((n, 1), 30.0)
    gi[3] = 5.0
    want = plain.mlstm_recurrence(q.reshape(n, 1, dim), kk.reshape(n, 1, dim), v.reshape(n, 1, vdim), gi, plain.log_sigmoid(gf)).reshape(n, vdim)
    assert np.allclose(want[-1], v[3] * np.sign(key @ key), atol=1e-3)
    for cut in (n, 1, 64, -n, -100):   # (negative: chunk by chunk)
        state = torch.zeros((1, dim * vdim + dim + 1)).cuda()
        got = []
        chunked, cut = cut < 0, abs(cut)
        for at in range(0, n, cut):
            m = min(cut, n - at)
            got.append(k.recurrence(gpu(q[at : at + m]), gpu(kk[at : at + m]), gpu(v[at : at + m]), state, ints([0, m]), ints([0]), 1, dim, vdim,
                                    gate_in=gpu(gi[at : at + m]), gate_forget=gpu(gf[at : at + m]), max_q_len=m if chunked else None).cpu().numpy())
            if cut == 1 and at > 40:
                break
        got = np.concatenate(got)
        np.testing.assert_allclose(got, want[: len(got)], atol=1e-4, rtol=1e-4)


def paged(keys, values, page_size, head_size, dtype, order):
    """Keys and values [T, G, d] of one request in pages taken in ``order``; returns (k_pages, v_pages, block table)."""
    T, G, _ = keys.shape
    n_blocks = -(-T // page_size)
    k_pages = torch.zeros((max(order) + 1, G, page_size, head_size), dtype=dtype).cuda()
    v_pages = torch.zeros_like(k_pages)
    for b in range(n_blocks):
        rows = slice(b * page_size, min(T, (b + 1) * page_size))
        n = rows.stop - rows.start
        k_pages[order[b], :, :n, : keys.shape[2]] = gpu(keys[rows], dtype).transpose(0, 1)
        v_pages[order[b], :, :n, : values.shape[2]] = gpu(values[rows], dtype).transpose(0, 1)
    return k_pages, v_pages, ints([order[:n_blocks]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_size,heads,kv_heads,window,softcap", [(64, 4, 2, 40, 15.0), (32, 2, 1, None, 5.0), (48, 3, 3, 70, None), (16, 2, 2, 5, 2.0),
                                                                     (128, 2, 1, 64, 30.0), (160, 1, 1, 33, 8.0)])
def test_attention_with_a_softcap_and_a_sink_in_prompts_and_in_decoding(dtype, head_size, heads, kv_heads, window, softcap):
    k = kernels()
    rng = np.random.default_rng(head_size)
    T, page_size = 150, 16
    q = rounded(rng.normal(0, 1.5, (T, heads, head_size)), dtype)
    keys = rounded(rng.normal(0, 1.5, (T, kv_heads, head_size)), dtype)
    values = rounded(rng.normal(0, 1, (T, kv_heads, head_size)), dtype)
    sinks = rng.normal(1.0, 2.0, heads)
    scale = head_size ** -0.5 * 2.0
    want = plain.windowed_attention(q, keys, values, scale, window, softcap, sinks).reshape(T, heads * head_size)
    without = plain.windowed_attention(q, keys, values, scale, window, softcap, None).reshape(T, heads * head_size)
    assert np.abs(want - without).max() > 0.05   # the sink shows
    order = list(rng.permutation(12))
    k_pages, v_pages, table = paged(keys, values, page_size, head_size, dtype, order)
    rows = gpu(q.reshape(T, heads * head_size), dtype)
    common = dict(n_heads=heads, n_kv_heads=kv_heads, head_size=head_size, scale=scale, window=window or 0, softcap=softcap or 0.0, sinks=gpu(sinks))
    # the whole prompt at once, then a portion over cached keys, then the last rows one by one and in short portions
    got = k.paged_attention(rows, k_pages, v_pages, ints(np.zeros(T)), ints(np.arange(T)), table, max_q_len=T, max_len=T, q_starts=ints([0, T]),
                            context_lens=ints([0]), **common)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, **tol(dtype))
    got = k.paged_attention(rows[90:], k_pages, v_pages, ints(np.zeros(60)), ints(np.arange(90, T)), table, max_q_len=60, max_len=T, q_starts=ints([0, 60]),
                            context_lens=ints([90]), **common)
    np.testing.assert_allclose(got.float().cpu().numpy(), want[90:], **tol(dtype))
    for at, n in ((T - 1, 1), (T - 5, 5), (3, 1), (64, 2)):
        got = k.paged_attention(rows[at : at + n], k_pages, v_pages, ints(np.zeros(n)), ints(np.arange(at, at + n)), table, max_q_len=n, max_len=T,
                                q_starts=ints([0, n]), context_lens=ints([at]), **common)
        np.testing.assert_allclose(got.float().cpu().numpy(), want[at : at + n], **tol(dtype))


@pytest.mark.parametrize("head_size", [64, 48])
def test_a_long_context_in_runs_of_keys_counts_the_sink_once(head_size):
    # one row over 3,000 keys: the split-key kernel cuts them into runs whose last block merges them, the sink joining there
    k = kernels()
    rng = np.random.default_rng(1)
    T, page_size, heads = 3000, 64, 2
    keys, values = rng.normal(0, 1, (T, 1, head_size)), rng.normal(0, 1, (T, 1, head_size))
    q = rng.normal(0, 1, (1, heads, head_size))
    sinks = np.array([4.0, -1.0])
    k_pages, v_pages, table = paged(keys, values, page_size, head_size, torch.float32, list(range(47)))
    scores = 10.0 * np.tanh(np.einsum("hd,td->ht", q[0], np.float32(keys[:, 0]).astype(np.float64)) * 0.2 / 10.0)
    top = np.maximum(scores.max(axis=1), sinks)
    w = np.exp(scores - top[:, None])
    want = (w @ np.float32(values[:, 0]).astype(np.float64)) / (w.sum(axis=1) + np.exp(sinks - top))[:, None]
    got = k.paged_attention(gpu(q.reshape(1, -1)), k_pages, v_pages, ints([0]), ints([T - 1]), table, heads, 1, head_size, 0.2, max_q_len=1, max_len=T,
                            q_starts=ints([0, 1]), context_lens=ints([T - 1]), softcap=10.0, sinks=gpu(sinks))
    np.testing.assert_allclose(got.cpu().numpy().reshape(heads, head_size), want, atol=2e-5, rtol=2e-4)
