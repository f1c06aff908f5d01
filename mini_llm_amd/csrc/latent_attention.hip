// Attention over a cache that holds one shared row per token (a latent and a rotated key part) instead of keys and values
// per head, and the per-head products on either side of it.
//
// A head's key is W_uk c (+ the shared rotated part) and its value W_uv c. Neither is ever formed: the key expansion is folded
// into the query, q' = W_uk^T q, so that a score is q' . c + q_rot . k_rot, a dot product with the cached row as it lies; the
// weighted sum is taken over the latents, o' = sum_j p_j c_j, and expanded once per query, o = W_uv o'. All heads of a token
// read the same rows, so a block takes a token and a wave a head, and a tile of rows is staged in LDS once for all of them.
// The softmax may hold a sink: a per-head number whose exponential joins the denominator without a value.
// Scores, weights and sums are 32-bit whatever the cache holds.
#include "common.h"

namespace {

__device__ __forceinline__ float load_as_float(const void* base, size_t index, int code) {
    return code == MLLM_F32 ? reinterpret_cast<const float*>(base)[index] : to_float(reinterpret_cast<const bf16_t*>(base)[index]);
}
__device__ __forceinline__ void store_from_float(void* base, size_t index, int code, float value) {
    if (code == MLLM_F32) reinterpret_cast<float*>(base)[index] = value;
    else reinterpret_cast<bf16_t*>(base)[index] = static_cast<bf16_t>(value);
}

// out[row, head, n] = sum_k x[row, head, k] * w[head, n, k] (* sigmoid(gate[row, head * N + n]), the gate's rows gate_row_stride apart):
// one small product per head.
// A block takes HEADS_ROWS rows of one head: their x in LDS (32-bit), a thread an output column at a time, its W row read in
// 16-byte pieces where K allows.
constexpr int HEADS_ROWS = 16;

template <typename WT>
__global__ __launch_bounds__(256) void heads_linear_kernel(const void* __restrict__ x, int x_code, int x_row_stride, int x_head_stride,
                                                           const WT* __restrict__ w, const void* __restrict__ gate, int gate_code, int gate_row_stride,
                                                           void* __restrict__ out, int out_code, int out_row_stride, int out_head_stride,
                                                           int n_rows, int N, int K) {
    extern __shared__ float x_tile[];   // [HEADS_ROWS][K]
    const int head = blockIdx.y, row0 = blockIdx.x * HEADS_ROWS;
    const int rows = min(HEADS_ROWS, n_rows - row0);
    for (int i = threadIdx.x; i < HEADS_ROWS * K; i += blockDim.x) {
        const int r = i / K, k = i % K;
        x_tile[i] = r < rows ? load_as_float(x, (size_t)(row0 + r) * x_row_stride + (size_t)head * x_head_stride + k, x_code) : 0.0f;
    }
    __syncthreads();
    constexpr int VEC = 16 / (int)sizeof(WT);
    const bool pieces = K % VEC == 0;
    for (int n = threadIdx.x; n < N; n += blockDim.x) {
        const WT* w_row = w + ((size_t)head * N + n) * K;
        float acc[HEADS_ROWS];
#pragma unroll
        for (int r = 0; r < HEADS_ROWS; r++) acc[r] = 0.0f;
        if (pieces) {
            for (int k = 0; k < K; k += VEC) {
                Vec16 piece = *reinterpret_cast<const Vec16*>(w_row + k);
                const WT* e = reinterpret_cast<const WT*>(&piece);
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    const float wv = to_float(e[j]);
#pragma unroll
                    for (int r = 0; r < HEADS_ROWS; r++) acc[r] += wv * x_tile[r * K + k + j];
                }
            }
        } else {
            for (int k = 0; k < K; k++) {
                const float wv = to_float(w_row[k]);
#pragma unroll
                for (int r = 0; r < HEADS_ROWS; r++) acc[r] += wv * x_tile[r * K + k];
            }
        }
        for (int r = 0; r < rows; r++) {
            float value = acc[r];
            if (gate) {
                const float g = load_as_float(gate, (size_t)(row0 + r) * gate_row_stride + (size_t)head * N + n, gate_code);
                value *= 1.0f / (1.0f + expf(-g));
            }
            store_from_float(out, (size_t)(row0 + r) * out_row_stride + (size_t)head * out_head_stride + n, out_code, value);
        }
    }
}

constexpr int LATENT_WAVES = 16;      // heads a block takes
constexpr int LATENT_TILE = 32;       // cached rows a tile holds
constexpr int LATENT_VALUE_REGS = 8;  // a lane's share of the latent: ranks up to 512

// A block per (row of the batch, run of its keys, 16 heads). q [rows, n_heads, D] (32-bit: the folded query, the rotated
// part, zeros), pages [num_pages, page_size, D], D a multiple of 16 bytes. The first R elements of a cached row are the
// latent (also the value). gridDim.y = 1: out [rows, n_heads, R] (32-bit) holds the finished sums, sink included. More runs:
// every run leaves its unnormalised sums, maximum and weight in parts [rows, n_heads, runs, R + 2], which latent_merge_kernel puts together.
template <typename T>
__global__ __launch_bounds__(64 * LATENT_WAVES) void latent_attention_kernel(
    const float* __restrict__ q, const T* __restrict__ pages, const float* __restrict__ sinks, float* __restrict__ out, float* __restrict__ parts,
    const int* __restrict__ token_request, const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks,
    int n_heads, int R, int D, int page_size, float scale, int run_length) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int token = blockIdx.x, run = blockIdx.y, n_runs = gridDim.y;
    const int head = blockIdx.z * LATENT_WAVES + wave;
    const int request = token_request[token];
    const bool live_head = head < n_heads;
    const int row_dwords = D * (int)sizeof(T) / 4 + 1;   // an odd stride: a lane per cached row reads without bank conflicts
    float* q_lds = lds;                                                  // [LATENT_WAVES][D]
    uint32_t* tile = reinterpret_cast<uint32_t*>(lds + LATENT_WAVES * D);   // [LATENT_TILE][row_dwords]
    float* weights = reinterpret_cast<float*>(tile + LATENT_TILE * row_dwords);   // [LATENT_WAVES][LATENT_TILE]

    float o[LATENT_VALUE_REGS];
#pragma unroll
    for (int r = 0; r < LATENT_VALUE_REGS; r++) o[r] = 0.0f;
    float running_max = -INFINITY, running_sum = 0.0f;

    if (request >= 0) {   // uniform over the block
        const int position = positions[token];
        const int first_key = run * run_length, last_key = min(position, first_key + run_length - 1);
        const int* table = block_tables + (size_t)request * max_blocks;
        if (live_head)
            for (int d = lane; d < D; d += WAVE) q_lds[wave * D + d] = q[((size_t)token * n_heads + head) * D + d] * scale;
        constexpr int VEC = 16 / (int)sizeof(T);
        const int pieces_per_row = D / VEC;
        for (int tile0 = first_key; tile0 <= last_key; tile0 += LATENT_TILE) {
            __syncthreads();   // the tile before has been read by every wave (and q_lds is written)
            for (int i = threadIdx.x; i < LATENT_TILE * pieces_per_row; i += blockDim.x) {
                const int j = i / pieces_per_row, piece = i % pieces_per_row;
                const int key = min(tile0 + j, last_key);
                const int page = table[key / page_size];
                const Vec16 v = *reinterpret_cast<const Vec16*>(pages + ((size_t)page * page_size + key % page_size) * D + piece * VEC);
                uint32_t* at = tile + j * row_dwords + piece * 4;
                at[0] = v.w[0]; at[1] = v.w[1]; at[2] = v.w[2]; at[3] = v.w[3];
            }
            __syncthreads();
            if (!live_head) continue;
            // scores: two lanes a cached row, each half of the elements
            const int j = lane % LATENT_TILE, part = lane / LATENT_TILE;
            const T* row = reinterpret_cast<const T*>(tile + j * row_dwords);
            const int half = (D / 2 + 1) & ~1;   // an even split, so that pairs of bfloat16 stay whole
            const int d_lo = part * half, d_hi = min(D, d_lo + half);
            float dot = 0.0f;
            const float* my_q = q_lds + wave * D;
            if constexpr (sizeof(T) == 2) {
                for (int d = d_lo; d < d_hi; d += 2) {
                    const uint32_t pair = *reinterpret_cast<const uint32_t*>(row + d);
                    dot += my_q[d] * __builtin_bit_cast(float, pair << 16) + my_q[d + 1] * __builtin_bit_cast(float, pair & 0xffff0000u);
                }
            } else {
                for (int d = d_lo; d < d_hi; d++) dot += my_q[d] * to_float(row[d]);
            }
            dot += __shfl_xor(dot, LATENT_TILE, WAVE);
            const bool valid = tile0 + j <= last_key;
            const float score = valid ? dot : -INFINITY;
            const float new_max = fmaxf(running_max, wave_max(score));
            const float p = valid ? expf(score - new_max) : 0.0f;
            const float rescale = expf(running_max - new_max);   // the first tile of a run always holds a key: new_max is finite
            running_sum = running_sum * rescale + wave_sum(part == 0 ? p : 0.0f);
            running_max = new_max;
            if (part == 0) weights[wave * LATENT_TILE + j] = p;
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const int in_tile = min(LATENT_TILE, last_key - tile0 + 1);
#pragma unroll
            for (int r = 0; r < LATENT_VALUE_REGS; r++) {
                const int d = lane + r * WAVE;
                if (d < R) {
                    float sum = o[r] * rescale;
                    for (int k = 0; k < in_tile; k++)
                        sum += weights[wave * LATENT_TILE + k] * to_float(reinterpret_cast<const T*>(tile + k * row_dwords)[d]);
                    o[r] = sum;
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
    if (!live_head) return;
    if (n_runs == 1) {
        float inverse = 0.0f;
        if (request >= 0) {
            float total = running_sum;
            if (sinks) {   // the sink joins the denominator once: measured from the larger of the two
                const float sink = sinks[head], top = fmaxf(running_max, sink);
                const float shrink = expf(running_max - top);
                total = running_sum * shrink + expf(sink - top);
                inverse = shrink / total;
            } else {
                inverse = 1.0f / total;
            }
        }
        float* out_row = out + ((size_t)token * n_heads + head) * R;
#pragma unroll
        for (int r = 0; r < LATENT_VALUE_REGS; r++) {
            const int d = lane + r * WAVE;
            if (d < R) out_row[d] = o[r] * inverse;
        }
        return;
    }
    float* mine = parts + (((size_t)token * n_heads + head) * n_runs + run) * (R + 2);
#pragma unroll
    for (int r = 0; r < LATENT_VALUE_REGS; r++) {
        const int d = lane + r * WAVE;
        if (d < R) mine[d] = o[r];
    }
    if (lane == 0) {
        mine[R] = running_max;   // -inf and 0 for a run without keys
        mine[R + 1] = running_sum;
    }
}

// out[row, head] = sum_p o_p e^(m_p - M) / (sum_p l_p e^(m_p - M) + e^(sink - M)) over the runs of a (row, head); a wave each.
__global__ __launch_bounds__(256) void latent_merge_kernel(const float* __restrict__ parts, const float* __restrict__ sinks,
                                                           const int* __restrict__ token_request, float* __restrict__ out, int n_rows,
                                                           int n_heads, int n_runs, int R) {
    const int lane = threadIdx.x % WAVE;
    const long long item = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (item >= (long long)n_rows * n_heads) return;
    const int token = (int)(item / n_heads), head = (int)(item % n_heads);
    float* out_row = out + (size_t)item * R;
    if (token_request[token] < 0) {
        for (int d = lane; d < R; d += WAVE) out_row[d] = 0.0f;
        return;
    }
    const float* runs = parts + (size_t)item * n_runs * (R + 2);
    float top = sinks ? sinks[head] : -INFINITY;
    for (int p = 0; p < n_runs; p++) top = fmaxf(top, runs[p * (R + 2) + R]);
    float total = sinks ? expf(sinks[head] - top) : 0.0f;
    for (int p = 0; p < n_runs; p++) {
        const float m = runs[p * (R + 2) + R];
        total += m == -INFINITY ? 0.0f : runs[p * (R + 2) + R + 1] * expf(m - top);
    }
    const float inverse = 1.0f / total;
    for (int d = lane; d < R; d += WAVE) {
        float sum = 0.0f;
        for (int p = 0; p < n_runs; p++) {
            const float m = runs[p * (R + 2) + R];
            sum += m == -INFINITY ? 0.0f : runs[p * (R + 2) + d] * expf(m - top);
        }
        out_row[d] = sum * inverse;
    }
}

size_t latent_lds_bytes(int D, int element) {
    const int row_dwords = D * element / 4 + 1;
    return (size_t)LATENT_WAVES * D * 4 + (size_t)LATENT_TILE * row_dwords * 4 + (size_t)LATENT_WAVES * LATENT_TILE * 4;
}

template <typename KernelT>
int allow_lds(KernelT kernel, size_t bytes, const char* what) {
    if (bytes <= 48 * 1024) return 0;
    hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (status != hipSuccess) {
        mllm_set_error("%s: %zu bytes of LDS were refused: %s", what, bytes, hipGetErrorString(status));
        return 1;
    }
    return 0;
}

}  // namespace

MLLM_API int mllm_heads_linear(const void* x, int x_dtype, int x_row_stride, int x_head_stride, const void* w, int w_dtype, const void* gate,
                               int gate_dtype, int gate_row_stride, void* out, int out_dtype, int out_row_stride, int out_head_stride, int n_rows, int n_heads,
                               int N, int K, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && N > 0 && K > 0, "heads_linear: bad sizes");
    MLLM_REQUIRE(x_head_stride >= 0 && out_head_stride >= N, "heads_linear: heads overlap");
    MLLM_REQUIRE(x_row_stride >= (n_heads - 1) * x_head_stride + K && out_row_stride >= (n_heads - 1) * out_head_stride + N,
                 "heads_linear: rows are too short for the heads");
    for (int code : {x_dtype, w_dtype, out_dtype}) MLLM_REQUIRE(code == MLLM_F32 || code == MLLM_BF16, "heads_linear: unknown dtype %d", code);
    MLLM_REQUIRE(gate == nullptr || ((gate_dtype == MLLM_F32 || gate_dtype == MLLM_BF16) && gate_row_stride >= n_heads * N), "heads_linear: a gate of unknown element type or with rows too short");
    const size_t lds = (size_t)HEADS_ROWS * K * sizeof(float);
    MLLM_REQUIRE(lds <= 64 * 1024, "heads_linear: K = %d is more than a block holds in LDS", K);
    if (n_rows == 0) return 0;
    dim3 grid(ceil_div(n_rows, HEADS_ROWS), n_heads);
    const int threads = N >= 256 ? 256 : (N > 64 ? 128 : 64);
    mllm_count_kernel(MLLM_K_HEADS_LINEAR);
    if (w_dtype == MLLM_F32) {
        if (allow_lds(heads_linear_kernel<float>, lds, "heads_linear")) return 1;
        heads_linear_kernel<float><<<grid, threads, lds, stream>>>(x, x_dtype, x_row_stride, x_head_stride, (const float*)w, gate, gate_dtype, gate_row_stride, out, out_dtype,
                                                                   out_row_stride, out_head_stride, n_rows, N, K);
    } else {
        if (allow_lds(heads_linear_kernel<bf16_t>, lds, "heads_linear")) return 1;
        heads_linear_kernel<bf16_t><<<grid, threads, lds, stream>>>(x, x_dtype, x_row_stride, x_head_stride, (const bf16_t*)w, gate, gate_dtype, gate_row_stride, out, out_dtype,
                                                                    out_row_stride, out_head_stride, n_rows, N, K);
    }
    return mllm_check_launch("heads_linear");
}

// Whether the latent attention kernel takes rows of D elements of which R are the latent.
MLLM_API int mllm_latent_attention_supported(int R, int D, int dtype) {
    const int element = dtype == MLLM_F32 ? 4 : 2;
    return R > 0 && R <= D && R <= WAVE * LATENT_VALUE_REGS && (D * element) % 16 == 0 && latent_lds_bytes(D, element) <= 160 * 1024 - 1024;
}

MLLM_API int mllm_latent_attention(const float* q, const void* pages, const float* sinks, float* out, float* parts, const int* token_request,
                                   const int* positions, const int* block_tables, int max_blocks, int n_rows, int n_heads, int R, int D,
                                   int page_size, float scale, int n_runs, int run_length, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && max_blocks > 0 && page_size > 0, "latent_attention: bad sizes");
    MLLM_REQUIRE(dtype == MLLM_F32 || dtype == MLLM_BF16, "latent_attention: unknown dtype %d", dtype);
    MLLM_REQUIRE(mllm_latent_attention_supported(R, D, dtype), "latent_attention: no kernel for rows of %d elements with a latent of %d", D, R);
    MLLM_REQUIRE(n_runs >= 1 && n_runs <= 65535 && run_length >= 1, "latent_attention: bad runs");
    MLLM_REQUIRE(n_runs == 1 || parts != nullptr, "latent_attention: runs need room for their sums");
    MLLM_REQUIRE(n_runs == 1 || (long long)n_runs * run_length >= (long long)max_blocks * page_size, "latent_attention: the runs do not cover the longest sequence");
    if (n_rows == 0) return 0;
    const size_t lds = latent_lds_bytes(D, dtype == MLLM_F32 ? 4 : 2);
    dim3 grid(n_rows, n_runs, ceil_div(n_heads, LATENT_WAVES));
    const int threads = 64 * (n_heads < LATENT_WAVES ? n_heads : LATENT_WAVES);
    if (n_runs == 1) run_length = 1 << 30;
    mllm_count_kernel(MLLM_K_LATENT_ATTENTION);
    if (dtype == MLLM_F32) {
        if (allow_lds(latent_attention_kernel<float>, lds, "latent_attention")) return 1;
        latent_attention_kernel<float><<<grid, threads, lds, stream>>>(q, (const float*)pages, sinks, out, parts, token_request, positions, block_tables,
                                                                       max_blocks, n_heads, R, D, page_size, scale, run_length);
    } else {
        if (allow_lds(latent_attention_kernel<bf16_t>, lds, "latent_attention")) return 1;
        latent_attention_kernel<bf16_t><<<grid, threads, lds, stream>>>(q, (const bf16_t*)pages, sinks, out, parts, token_request, positions, block_tables,
                                                                        max_blocks, n_heads, R, D, page_size, scale, run_length);
    }
    int status = mllm_check_launch("latent_attention");
    if (status || n_runs == 1) return status;
    const long long items = (long long)n_rows * n_heads;
    mllm_count_kernel(MLLM_K_LATENT_MERGE);
    latent_merge_kernel<<<(int)((items + 3) / 4), 256, 0, stream>>>(parts, sinks, token_request, out, n_rows, n_heads, n_runs, R);
    return mllm_check_launch("latent_merge");
}
