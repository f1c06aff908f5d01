"""Each mechanism of the Gimozen design alone: the kernel against the plain function of tests/plain_gimozen.py."""

import math

import numpy as np
import pytest
import torch

import plain_gimozen as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def kernels():
    from mini_llm_amd.ops import kernels

    return kernels


def gpu(array, dtype=torch.float32):
    return torch.tensor(np.asarray(array), dtype=torch.float32).to(dtype).cuda().contiguous()


def rounded(array, dtype):
    return torch.tensor(np.asarray(array), dtype=torch.float32).to(dtype).to(torch.float32).numpy().astype(np.float64)


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("width", [5, 64, 192, 300, 1030, 2500])
@pytest.mark.parametrize("one_plus", [False, True])
def test_rms_norm_with_the_scaled_sum(width, one_plus):
    rng = np.random.default_rng(width)
    x, y, w = rng.normal(0, 2, (7, width)), rng.normal(0, 1, (7, width)), rng.normal(0, 0.3, width)
    k = kernels()
    want = plain.rms_norm(1.5 * x + y, w, 1e-5, one_plus)
    stream, rows = k.rms_norm(gpu(x), gpu(w), 1e-5, addend=gpu(y), alpha=1.5, one_plus=one_plus, out_dtype=torch.bfloat16, with_stream=True)
    np.testing.assert_allclose(stream.cpu().numpy(), want, atol=2e-5, rtol=2e-5)
    assert torch.equal(rows, stream.to(torch.bfloat16))
    # an addend in bfloat16, and no addend with gathered rows
    y16 = rounded(y, torch.bfloat16)
    got = k.rms_norm(gpu(x), gpu(w), 1e-5, addend=gpu(y, torch.bfloat16), alpha=1.5, one_plus=one_plus)
    np.testing.assert_allclose(got.cpu().numpy(), plain.rms_norm(1.5 * x + y16, w, 1e-5, one_plus), atol=2e-5, rtol=2e-5)
    # the addend as the partial products of a product cut along K: the norm takes their sum
    parts = rng.normal(0, 1, (3, 7, width))
    got = k.rms_norm(gpu(x), gpu(w), 1e-5, addend=gpu(parts), alpha=1.5, one_plus=one_plus)
    np.testing.assert_allclose(got.cpu().numpy(), plain.rms_norm(1.5 * x + parts.sum(axis=0), w, 1e-5, one_plus), atol=2e-5, rtol=2e-5)
    index = torch.tensor([6, 0, 3], dtype=torch.int32).cuda()
    got = k.rms_norm(gpu(x), gpu(w), 1e-5, one_plus=one_plus, out_dtype=torch.float32, row_index=index)
    np.testing.assert_allclose(got.cpu().numpy(), plain.rms_norm(x[[6, 0, 3]], w, 1e-5, one_plus), atol=2e-5, rtol=2e-5)


def test_rms_norm_keeps_eps_inside_the_root():
    x = np.full((1, 8), 1e-3)
    got = kernels().rms_norm(gpu(x), gpu(np.ones(8)), 1e-2)
    np.testing.assert_allclose(got.cpu().numpy(), x / math.sqrt(1e-6 + 1e-2), rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    rng = np.random.default_rng(1)
    both = rounded(rng.normal(0, 3, (9, 2 * 37)), dtype)
    got = kernels().silu_mul(gpu(both, dtype)).float().cpu().numpy()
    np.testing.assert_allclose(got, plain.silu(both[:, :37]) * both[:, 37:], **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,vdim,heads,kv_heads", [(16, 16, 4, 2), (24, 8, 3, 3), (8, 40, 2, 1), (80, 80, 1, 1), (64, 64, 12, 4), (12, 20, 2, 1), (10, 6, 3, 3)])
def test_head_norm_writes_queries_keys_and_values(dtype, dim, vdim, heads, kv_heads):
    k = kernels()
    rng = np.random.default_rng(dim)
    rows, page_size, n_pages, eps = 11, 4, 8, 1e-5
    head_size = -(-max(dim, vdim) // 16) * 16
    width = (heads + kv_heads) * dim + kv_heads * vdim
    qkv = rounded(rng.normal(0, 2, (rows, width)), dtype)
    qg, kg = rng.normal(1, 0.2, dim), rng.normal(1, 0.2, dim)
    positions = np.array([0, 1, 2, 6, 7, 8, 13, 14, 15, 70, 200])
    slots = np.array([5, 4, 31, -1, 0, 1, 2, 3, 17, 9, 12])
    k_pages = torch.full((n_pages, kv_heads, page_size, head_size), 7.0, dtype=dtype).cuda()
    v_pages = torch.full_like(k_pages, 7.0)
    q = k.head_norm(gpu(qkv, dtype), gpu(qg), gpu(kg), eps, torch.tensor(positions, dtype=torch.int32).cuda(), torch.tensor(slots, dtype=torch.int32).cuda(),
                    k_pages, v_pages, heads, kv_heads, dim, vdim, temp_coef=0.3, temp_every=7)
    temp = plain.query_temperature(positions, 0.3, 7)
    assert temp[2] == 1.0 < temp[3] == temp[4] == temp[5] < temp[6] == temp[7]   # the steps lie where floor((p + 1) / 7) changes: at 6 and at 13
    want_q = plain.rms_norm(qkv[:, : heads * dim].reshape(rows, heads, dim), qg, eps) * temp[:, None, None]
    got_q = q.float().cpu().numpy().reshape(rows, heads, head_size)
    np.testing.assert_allclose(got_q[:, :, :dim], want_q, **tol(dtype))
    assert (got_q[:, :, dim:] == 0).all()
    want_k = plain.rms_norm(qkv[:, heads * dim : (heads + kv_heads) * dim].reshape(rows, kv_heads, dim), kg, eps)
    want_v = qkv[:, (heads + kv_heads) * dim :].reshape(rows, kv_heads, vdim)
    kp, vp = k_pages.float().cpu().numpy(), v_pages.float().cpu().numpy()
    written = set()
    for row, slot in enumerate(slots):
        if slot < 0:
            continue
        page, offset = divmod(int(slot), page_size)
        written.add((page, offset))
        np.testing.assert_allclose(kp[page, :, offset, :dim], want_k[row], **tol(dtype))
        np.testing.assert_array_equal(vp[page, :, offset, :vdim], want_v[row])
        assert (kp[page, :, offset, dim:] == 0).all() and (vp[page, :, offset, vdim:] == 0).all()
    for page in range(n_pages):
        for offset in range(page_size):
            if (page, offset) not in written:
                assert (kp[page, :, offset] == 7).all() and (vp[page, :, offset] == 7).all()


def test_rotary_frequencies_follow_the_scaling():
    from mini_llm_amd.parts import RotaryEncoding

    for rot in ({"dims": 32, "base": 10000.0}, {"dims": 16, "base": 500000.0, "scaling": {"factor": 8.0, "original": 128, "fast": 32.0, "slow": 1.0}},
                {"dims": 64, "base": 1000.0, "scaling": {"factor": 2.5, "original": 4096, "fast": 4.0, "slow": 0.5}}):
        part = RotaryEncoding(rot["dims"], rot["base"], rot.get("scaling"))
        freq, magnitude = plain.rotary_frequencies(rot)
        np.testing.assert_allclose(part.values, freq, rtol=1e-12)
        assert abs(part.magnitude - magnitude) < 1e-12
    # the ramp has both ends: the fastest pair keeps its frequency, the slowest is divided by the factor
    rot = {"dims": 16, "base": 500000.0, "scaling": {"factor": 8.0, "original": 128, "fast": 32.0, "slow": 1.0}}
    freq, magnitude = plain.rotary_frequencies(rot)
    assert freq[0] == 1.0 and abs(freq[-1] - 500000.0 ** (-14 / 16) / 8.0) < 1e-15 and magnitude == 0.1 * math.log(8.0) + 1.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,rot_dims,rank", [(3, 16, 8, 8, 40), (1, 8, 16, 8, 21), (2, 24, 4, 4, 64), (2, 8, 6, 0, 10)])
def test_latent_rows_rotate_and_keep(dtype, heads, dim, rot, rot_dims, rank):
    from mini_llm_amd.parts import RotaryEncoding

    k = kernels()
    rng = np.random.default_rng(rank)
    rot_config = {"dims": rot_dims, "base": 100.0, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    part = RotaryEncoding(rot_dims, 100.0, rot_config["scaling"])
    rows, page_size, n_pages, eps = 6, 4, 4, 1e-5
    row_size = k.latent_row_size(rank + rot)
    positions = np.array([0, 1, 5, 37, 300, 1021])
    slots = np.array([3, -1, 0, 9, 14, 6])
    q = rounded(rng.normal(0, 1, (rows, heads * (dim + rot))), dtype)
    dkv = rounded(rng.normal(0, 1, (rows, rank + rot)), dtype)
    gain = rng.normal(1, 0.2, rank)
    pages = torch.full((n_pages, 1, page_size, row_size), 7.0, dtype=dtype).cuda()
    q_full = k.latent_rows(gpu(q, dtype), gpu(dkv, dtype), gpu(gain), eps, part.frequencies("cuda"), part.magnitude, rot_dims,
                           torch.tensor(positions, dtype=torch.int32).cuda(), torch.tensor(slots, dtype=torch.int32).cuda(), pages, heads, dim, rot, rank)
    rotate = (lambda x: plain.rotate_half(x, positions, rot_config)) if rot_dims else (lambda x: x)
    want_q = rotate(q.reshape(rows, heads, dim + rot)[:, :, dim:])
    got = q_full.cpu().numpy()
    # angles are 32-bit products: at position p they are off by up to p * 6e-8
    np.testing.assert_allclose(got[:, :, rank : rank + rot], want_q, atol=2e-4, rtol=1e-5)
    assert (got[:, :, rank + rot :] == 0).all()
    kept = pages.float().cpu().numpy().reshape(n_pages * page_size, row_size)
    want_c, want_r = plain.rms_norm(dkv[:, :rank], gain, eps), rotate(dkv[:, rank:])
    for row, slot in enumerate(slots):
        if slot < 0:
            continue
        np.testing.assert_allclose(kept[slot, :rank], want_c[row], **tol(dtype))
        np.testing.assert_allclose(kept[slot, rank : rank + rot], want_r[row], **(tol(dtype) if dtype == torch.bfloat16 else dict(atol=2e-4, rtol=1e-5)))
        assert (kept[slot, rank + rot :] == 0).all()
    assert (np.delete(kept, [s for s in slots if s >= 0], axis=0) == 7).all()
    # a layer that borrows another's rows stores nothing
    before = pages.clone()
    k.latent_rows(gpu(q, dtype), None, None, eps, part.frequencies("cuda"), part.magnitude, rot_dims, torch.tensor(positions, dtype=torch.int32).cuda(),
                  torch.tensor(slots, dtype=torch.int32).cuda(), pages, heads, dim, rot, rank)
    assert torch.equal(before, pages)


@pytest.mark.parametrize("w_dtype", DTYPES)
@pytest.mark.parametrize("gap", [3, 16])
@pytest.mark.parametrize("rows,heads,n,k_size", [(1, 3, 40, 16), (17, 2, 24, 64), (33, 1, 300, 21), (5, 5, 7, 512), (70, 3, 130, 32)])
def test_heads_linear(w_dtype, rows, heads, n, k_size, gap):
    # gap: how far the heads of x lie apart beyond their K elements. With a gap of 16 the rows start on 16-byte boundaries, and
    # bfloat16 matrices with K a multiple of 16 then run on the matrix cores, where x is rounded to bfloat16 on its way in
    k = kernels()
    rng = np.random.default_rng(rows)
    x = rng.normal(0, 1, (rows, heads, k_size + gap))
    w = rounded(rng.normal(0, 1, (heads, n, k_size)), w_dtype)
    gate = rng.normal(0, 2, (rows, heads * n))
    rounds_x = w_dtype == torch.bfloat16 and gap == 16 and k_size % 16 == 0
    bound = dict(atol=0.02 * k_size ** 0.5, rtol=2e-2) if rounds_x else dict(atol=1e-4, rtol=1e-4)
    out = torch.full((rows, heads, n + 2), 5.0, dtype=torch.float32).cuda()
    k.heads_linear(gpu(x).view(rows, -1), gpu(w, w_dtype), out, n_heads=heads, k=k_size, x_head_stride=k_size + gap, gate=gpu(gate))
    want = np.einsum("rhk,hnk->rhn", x[:, :, :k_size], w) * plain.sigmoid(gate.reshape(rows, heads, n))
    got = out.cpu().numpy()
    np.testing.assert_allclose(got[:, :, :n], want, **bound)
    assert (got[:, :, n:] == 5).all()
    # x in bfloat16 (exact on either path), the result in bfloat16
    x16 = rounded(x, torch.bfloat16)
    out16 = torch.zeros((rows, heads, n), dtype=torch.bfloat16).cuda()
    k.heads_linear(gpu(x16, torch.bfloat16).view(rows, -1), gpu(w, w_dtype), out16, n_heads=heads, k=k_size, x_head_stride=k_size + gap)
    np.testing.assert_allclose(out16.float().cpu().numpy(), np.einsum("rhk,hnk->rhn", x16[:, :, :k_size], w), atol=0.1, rtol=1e-2)


def latent_case(rng, dtype, lengths, heads, rank, rot, page_size, sharp=None):
    """Requests of the given lengths, their cached rows spread over shuffled pages; one query row per request at its last
    position (decode) and, for the first request, a query at every position (a portion)."""
    row_size = kernels().latent_row_size(rank + rot)
    n_blocks = [-(-n // page_size) for n in lengths]
    order = rng.permutation(sum(n_blocks) + 3)
    pages = torch.zeros((len(order), 1, page_size, row_size), dtype=dtype)
    tables = np.full((len(lengths), max(n_blocks) + 2), -1, dtype=np.int32)
    cached, at = [], 0
    for r, n in enumerate(lengths):
        rows = rounded(rng.normal(0, 1, (n, row_size)), dtype)
        rows[:, rank + rot :] = 0
        cached.append(rows)
        for b in range(n_blocks[r]):
            tables[r, b] = order[at]
            chunk = rows[b * page_size : (b + 1) * page_size]
            pages[order[at], 0, : len(chunk)] = torch.tensor(chunk).to(dtype)
            at += 1
    return pages.cuda(), tables, cached, row_size


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("by_request", [False, True])
@pytest.mark.parametrize("heads,rank,rot,page_size,lengths", [(3, 40, 8, 16, [70, 1, 33, 16, 17]), (17, 64, 32, 64, [200, 64, 65]), (1, 21, 16, 4, [9, 700]),
                                                             (2, 300, 20, 32, [130, 31]), (12, 256, 32, 64, [100, 300]), (5, 130, 8, 32, [40, 41, 90])])
def test_latent_attention_with_a_sink(dtype, heads, rank, rot, page_size, lengths, by_request):
    # by_request: the batch's requests are named too (first rows, stored lengths), which lets a bfloat16 cache of a fitting row
    # size run on the matrix cores (queries and weights rounded to bfloat16 there)
    k = kernels()
    rng = np.random.default_rng(rank + heads)
    pages, tables, cached, row_size = latent_case(rng, dtype, lengths, heads, rank, rot, page_size)
    extra = {}
    if by_request:
        starts = [0, lengths[0]] + [lengths[0] + i for i in range(1, len(lengths))]
        extra = dict(q_starts=torch.tensor(starts, dtype=torch.int32).cuda(), context_lens=torch.tensor([0] + [n - 1 for n in lengths[1:]], dtype=torch.int32).cuda(),
                     max_q_len=lengths[0])
    on_matrix_cores = by_request and dtype == torch.bfloat16 and bool(k.library().mllm_latent_attention_mfma_supported(rank, row_size, 1))
    bound = dict(atol=3e-2, rtol=3e-2) if on_matrix_cores else dict(atol=2e-5, rtol=2e-4)
    # rows: every position of request 0 (a whole prompt), then the last position of the others
    token_request = [0] * lengths[0] + list(range(1, len(lengths)))
    positions = list(range(lengths[0])) + [n - 1 for n in lengths[1:]]
    q = rng.normal(0, 1, (len(positions), heads, row_size))
    q[:, :, rank + rot :] = 0
    sinks = rng.normal(0, 2, heads)
    scale = 0.3
    for use_sink in (True, False):
        for max_len in (None, max(lengths)):
            got = k.latent_attention(gpu(q), pages, gpu(sinks) if use_sink else None, torch.tensor(token_request, dtype=torch.int32).cuda(),
                                     torch.tensor(positions, dtype=torch.int32).cuda(), torch.tensor(tables).cuda(), rank, scale, max_len=max_len, **extra).cpu().numpy()
            for row, (request, position) in enumerate(zip(token_request, positions)):
                keys = cached[request][: position + 1]
                for head in range(heads):
                    scores = (keys @ q[row, head])[None, :] * scale
                    weights = plain.softmax_rows(scores, np.ones_like(scores, dtype=bool), sink=float(sinks[head]) if use_sink else None)
                    np.testing.assert_allclose(got[row, head], (weights @ keys[:, :rank])[0], **bound,
                                               err_msg=f"row {row} (request {request}, position {position}) head {head} sink {use_sink}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_attention_finds_one_far_key_and_never_a_later_one(dtype):
    # a long request in runs of keys: one cached row stands out; queries just before it must not see it, queries at and
    # behind it must put all their weight on it (up to what the sink takes); a padding row gives zeros
    k = kernels()
    rng = np.random.default_rng(5)
    heads, rank, rot, page_size, length = 4, 32, 8, 16, 1500
    pages, tables, cached, row_size = latent_case(rng, dtype, [length], heads, rank, rot, page_size)
    for hot in (0, 15, 16, 511, 512, 1023, 1499):
        direction = cached[0][hot] / np.linalg.norm(cached[0][hot])
        q = np.tile(direction * 60.0, (heads, 1))
        rows = [p for p in (hot - 1, hot, hot + 1, hot + 16, length - 1) if 0 <= p < length]
        token_request = [0] * len(rows) + [-1]
        got = k.latent_attention(gpu(np.tile(q, (len(rows) + 1, 1, 1))), pages, gpu(np.zeros(heads)), torch.tensor(token_request, dtype=torch.int32).cuda(),
                                 torch.tensor(rows + [0], dtype=torch.int32).cuda(), torch.tensor(tables).cuda(), rank, 1.0, max_len=length).cpu().numpy()
        assert (got[-1] == 0).all()
        for row, position in enumerate(rows):
            keys = cached[0][: position + 1]
            scores = (keys @ q[0])[None, :]
            want = (plain.softmax_rows(scores, np.ones_like(scores, dtype=bool), sink=0.0) @ keys[:, :rank])[0]
            np.testing.assert_allclose(got[row, 0], want, atol=1e-4, rtol=1e-3, err_msg=f"hot key {hot}, query at {position}")
            if position >= hot:
                np.testing.assert_allclose(got[row, 0], cached[0][hot, :rank], atol=2e-2)
            else:
                assert np.abs(got[row, 0] - cached[0][hot, :rank]).max() > 0.1
