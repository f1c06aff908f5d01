// Attention over a cache that holds one shared row per token (a latent and a rotated key part) instead of keys and values
// per head, and the per-head products on either side of it.
//
// A head's key is W_uk c (+ the shared rotated part) and its value W_uv c. Neither is ever formed: the key expansion is folded
// into the query, q' = W_uk^T q, so that a score is q' . c + q_rot . k_rot, a dot product with the cached row as it lies; the
// weighted sum is taken over the latents, o' = sum_j p_j c_j, and expanded once per query, o = W_uv o'. All heads of a token
// read the same rows, so a wave takes several heads of a token at once and every cached element it loads serves them all.
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
// 16-byte pieces where K allows; with fewer columns than threads the threads cut K among themselves and add up through LDS.
constexpr int HEADS_ROWS = 16;

template <typename WT>
__global__ __launch_bounds__(256) void heads_linear_kernel(const void* __restrict__ x, int x_code, int x_row_stride, int x_head_stride,
                                                           const WT* __restrict__ w, const void* __restrict__ gate, int gate_code, int gate_row_stride,
                                                           void* __restrict__ out, int out_code, int out_row_stride, int out_head_stride,
                                                           int n_rows, int N, int K, int cols) {
    extern __shared__ float heads_lds[];   // x_tile [HEADS_ROWS][K], then the partial sums [slices - 1][cols][HEADS_ROWS]
    float* x_tile = heads_lds;
    float* partial = heads_lds + HEADS_ROWS * K;
    const int head = blockIdx.y, row0 = blockIdx.x * HEADS_ROWS;
    const int rows = min(HEADS_ROWS, n_rows - row0);
    for (int i = threadIdx.x; i < HEADS_ROWS * K; i += blockDim.x) {
        const int r = i / K, k = i % K;
        x_tile[i] = r < rows ? load_as_float(x, (size_t)(row0 + r) * x_row_stride + (size_t)head * x_head_stride + k, x_code) : 0.0f;
    }
    __syncthreads();
    constexpr int VEC = 16 / (int)sizeof(WT);
    const bool pieces = K % VEC == 0;
    // `cols` threads take a column each; where the block has more threads than that, they cut K into slices
    const int slices = blockDim.x / cols, column = threadIdx.x % cols, slice = threadIdx.x / cols;
    const int per_slice = ceil_div(ceil_div(K, slices), VEC) * VEC;
    const int k_lo = min(K, slice * per_slice), k_hi = min(K, k_lo + per_slice);
    for (int n0 = 0; n0 < N; n0 += cols) {
        const int n = n0 + column;
        float acc[HEADS_ROWS];
#pragma unroll
        for (int r = 0; r < HEADS_ROWS; r++) acc[r] = 0.0f;
        if (n < N) {
            const WT* w_row = w + ((size_t)head * N + n) * K;
            if (pieces) {
                for (int k = k_lo; k < k_hi; k += VEC) {
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
                for (int k = k_lo; k < k_hi; k++) {
                    const float wv = to_float(w_row[k]);
#pragma unroll
                    for (int r = 0; r < HEADS_ROWS; r++) acc[r] += wv * x_tile[r * K + k];
                }
            }
        }
        if (slices > 1) {   // uniform over the block
            if (slice > 0)
#pragma unroll
                for (int r = 0; r < HEADS_ROWS; r++) partial[((slice - 1) * cols + column) * HEADS_ROWS + r] = acc[r];
            __syncthreads();
            if (slice == 0)
                for (int other = 1; other < slices; other++)
#pragma unroll
                    for (int r = 0; r < HEADS_ROWS; r++) acc[r] += partial[((other - 1) * cols + column) * HEADS_ROWS + r];
            __syncthreads();
        }
        if (slice == 0 && n < N) {
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
}

// The same products on the matrix cores, for bfloat16 matrices with K a multiple of 16 and x rows that start on 16-byte
// boundaries: out^T tile [32 columns, 32 rows] = W_h tile . x_h tile^T, a wave a tile, both operands as they lie in memory (a
// lane's 16-byte piece of its W row, and of its x row: eight bfloat16, or eight floats rounded to bfloat16 on the way).
// The four waves of a block take four neighbouring column tiles of the same rows.
template <typename XT>
__global__ __launch_bounds__(256) void heads_linear_mfma_kernel(const XT* __restrict__ x, int x_row_stride, int x_head_stride,
                                                                const bf16_t* __restrict__ w, const void* __restrict__ gate, int gate_code,
                                                                int gate_row_stride, void* __restrict__ out, int out_code, int out_row_stride,
                                                                int out_head_stride, int n_rows, int N, int K) {
    const int lane = threadIdx.x % WAVE, lane32 = lane % 32, half = lane / 32;
    const int head = blockIdx.y, row0 = blockIdx.x * 32;
    const int n0 = (blockIdx.z * 4 + threadIdx.x / WAVE) * 32;
    if (n0 >= N) return;
    const bf16_t* w_row = w + ((size_t)head * N + min(n0 + lane32, N - 1)) * K + 8 * half;
    const XT* x_row = x + (size_t)min(row0 + lane32, n_rows - 1) * x_row_stride + (size_t)head * x_head_stride + 8 * half;
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;
#pragma unroll 4
    for (int k = 0; k < K; k += 16) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(w_row + k);
        bf16x8 b;
        if constexpr (sizeof(XT) == 2) {
            b = *reinterpret_cast<const bf16x8*>(x_row + k);
        } else {
            const f32x4 lo = *reinterpret_cast<const f32x4*>(x_row + k), hi = *reinterpret_cast<const f32x4*>(x_row + k + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                b[e] = static_cast<bf16_t>(lo[e]);
                b[4 + e] = static_cast<bf16_t>(hi[e]);
            }
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
    }
    const int row = row0 + lane32;
    if (row >= n_rows) return;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int n = n0 + 8 * (v / 4) + 4 * half + (v % 4);
        if (n >= N) continue;
        float value = acc[v];
        if (gate) {
            const float g = load_as_float(gate, (size_t)row * gate_row_stride + (size_t)head * N + n, gate_code);
            value *= 1.0f / (1.0f + expf(-g));
        }
        store_from_float(out, (size_t)row * out_row_stride + (size_t)head * out_head_stride + n, out_code, value);
    }
}

constexpr int LATENT_ROWS = 4;   // rows of the batch a block takes, a wave each

template <typename T>
__device__ __forceinline__ float piece_element(const Vec16& piece, int e) {
    if constexpr (sizeof(T) == 2) {
        const uint32_t word = piece.w[e / 2];
        return __builtin_bit_cast(float, (e & 1) ? (word & 0xffff0000u) : (word << 16));
    } else {
        return __builtin_bit_cast(float, piece.w[e]);
    }
}

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// A wave per (row of the batch, run of its keys, HG heads). q [rows, n_heads, D] (32-bit: the folded query, the rotated part,
// zeros), pages [num_pages, page_size, D], D a multiple of 16 bytes; the first R elements of a cached row are the latent
// (also the value), R <= 64 * RV.
//
// All heads of a row read the same cached rows, so a wave takes HG heads at once: for the scores a lane takes a key and
// reads its row in 16-byte pieces, each element of which meets the HG queries' elements, which are the same for every lane
// (they come through the scalar unit); for the weighted sum a lane takes pairs of latent elements, and a key's weight for
// each head is read out of the lane that holds it. So a cached element costs one load and HG multiply-adds. Keys in
// tiles of 64 with online softmax statistics per head. n_runs = 1: out [rows, n_heads, R] holds the finished sums, sink
// included. More runs: every run leaves its unnormalised sums, maximum and weight in parts [rows, n_heads, runs, R + 2].
template <typename T, int HG, int RV>
__global__ __launch_bounds__(64 * LATENT_ROWS) void latent_attention_kernel(
    const float* __restrict__ q, const T* __restrict__ pages, const float* __restrict__ sinks, float* __restrict__ out, float* __restrict__ parts,
    const int* __restrict__ token_request, const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks,
    int n_rows, int n_heads, int R, int D, int page_size, float scale, int run_length) {
    const int lane = threadIdx.x % WAVE;
    const int token = blockIdx.x * LATENT_ROWS + __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    if (token >= n_rows) return;
    const int run = blockIdx.y, n_runs = gridDim.y, head0 = blockIdx.z * HG;
    const int request = token_request[token];

    float o[HG][RV], top[HG], weight[HG];
#pragma unroll
    for (int h = 0; h < HG; h++) {
        top[h] = -INFINITY;
        weight[h] = 0.0f;
#pragma unroll
        for (int r = 0; r < RV; r++) o[h][r] = 0.0f;
    }

    if (request >= 0) {
        const int position = positions[token];
        const int first_key = run * run_length;
        const int last_key = run == n_runs - 1 ? position : min(position, first_key + run_length - 1);   // the last run is open-ended
        const int* table = block_tables + (size_t)request * max_blocks;
        const float* q_head[HG];   // the same for every lane
#pragma unroll
        for (int h = 0; h < HG; h++) q_head[h] = q + ((size_t)token * n_heads + min(head0 + h, n_heads - 1)) * D;
        constexpr int VEC = 16 / (int)sizeof(T);
        for (int tile0 = first_key; tile0 <= last_key; tile0 += WAVE) {
            const bool valid = tile0 + lane <= last_key;
            const int key = min(tile0 + lane, last_key);
            const int slot = table[key / page_size] * page_size + key % page_size;
            const T* row = pages + (size_t)slot * D;
            float s[HG];
#pragma unroll
            for (int h = 0; h < HG; h++) s[h] = 0.0f;
            // four pieces of the lane's row are asked for at a time, so that their ways from memory overlap
            int d0 = 0;
            for (; d0 + 4 * VEC <= D; d0 += 4 * VEC) {
                Vec16 pieces[4];
#pragma unroll
                for (int u = 0; u < 4; u++) pieces[u] = *reinterpret_cast<const Vec16*>(row + d0 + u * VEC);
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int e = 0; e < VEC; e++) {
                        const float k = piece_element<T>(pieces[u], e);
#pragma unroll
                        for (int h = 0; h < HG; h++) s[h] = __builtin_fmaf(q_head[h][d0 + u * VEC + e], k, s[h]);
                    }
            }
            for (; d0 < D; d0 += VEC) {
                const Vec16 piece = *reinterpret_cast<const Vec16*>(row + d0);
#pragma unroll
                for (int e = 0; e < VEC; e++) {
                    const float k = piece_element<T>(piece, e);
#pragma unroll
                    for (int h = 0; h < HG; h++) s[h] = __builtin_fmaf(q_head[h][d0 + e], k, s[h]);
                }
            }
            float p[HG];
#pragma unroll
            for (int h = 0; h < HG; h++) {
                const float score = valid ? s[h] * scale : -INFINITY;
                const float new_top = fmaxf(top[h], wave_max_total(score));   // finite: a tile holds at least one key
                p[h] = valid ? expf(score - new_top) : 0.0f;
                const float rescale = expf(top[h] - new_top);
                weight[h] = weight[h] * rescale + wave_total(p[h]);
                top[h] = new_top;
#pragma unroll
                for (int r = 0; r < RV; r++) o[h][r] *= rescale;
            }
            // the weighted sum: a lane takes elements 2 * lane + 128 * r2 and the one behind it. Eight keys' values are asked
            // for at a time; lanes beyond the tile's keys hold a weight of zero and the place of a key that exists
            const int in_tile = min(WAVE, last_key - tile0 + 1);
            constexpr int KEYS = 8;
            for (int j0 = 0; j0 < in_tile; j0 += KEYS) {
                float v[KEYS][RV];
#pragma unroll
                for (int u = 0; u < KEYS; u++) {
                    const T* value_row = pages + (size_t)__builtin_amdgcn_readlane(slot, j0 + u) * D;
#pragma unroll
                    for (int r2 = 0; r2 < RV / 2; r2++) {
                        const int d = min(2 * lane + 2 * WAVE * r2, D - 2);   // beyond R: read, and never stored
                        if constexpr (sizeof(T) == 2) {
                            const uint32_t pair = *reinterpret_cast<const uint32_t*>(value_row + d);
                            v[u][2 * r2] = __builtin_bit_cast(float, pair << 16);
                            v[u][2 * r2 + 1] = __builtin_bit_cast(float, pair & 0xffff0000u);
                        } else {
                            const float2 pair = *reinterpret_cast<const float2*>(value_row + d);
                            v[u][2 * r2] = pair.x;
                            v[u][2 * r2 + 1] = pair.y;
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < KEYS; u++)
#pragma unroll
                    for (int h = 0; h < HG; h++) {
                        const float pj = lane_value(p[h], j0 + u);
#pragma unroll
                        for (int r = 0; r < RV; r++) o[h][r] = __builtin_fmaf(pj, v[u][r], o[h][r]);
                    }
            }
        }
    }
#pragma unroll
    for (int h = 0; h < HG; h++) {
        const int head = head0 + h;
        if (head >= n_heads) break;
        if (n_runs == 1) {
            float inverse = 0.0f;
            if (request >= 0) {
                if (sinks) {   // the sink joins the denominator once: measured from the larger of the two
                    const float sink = sinks[head], highest = fmaxf(top[h], sink);
                    const float shrink = expf(top[h] - highest);
                    inverse = shrink / (weight[h] * shrink + expf(sink - highest));
                } else {
                    inverse = 1.0f / weight[h];
                }
            }
            float* out_row = out + ((size_t)token * n_heads + head) * R;
#pragma unroll
            for (int r = 0; r < RV; r++) {
                const int d = 2 * lane + 2 * WAVE * (r / 2) + (r & 1);
                if (d < R) out_row[d] = o[h][r] * inverse;
            }
        } else {
            float* mine = parts + (((size_t)token * n_heads + head) * n_runs + run) * (R + 2);
#pragma unroll
            for (int r = 0; r < RV; r++) {
                const int d = 2 * lane + 2 * WAVE * (r / 2) + (r & 1);
                if (d < R) mine[d] = o[h][r];
            }
            if (lane == 0) {
                mine[R] = top[h];   // -inf and 0 for a run without keys
                mine[R + 1] = weight[h];
            }
        }
    }
}

// out[row, head] = sum_p o_p e^(m_p - M) / (sum_p l_p e^(m_p - M) + e^(sink - M)) over the runs of a (row, head); a block each.
// Thread p takes run p's maximum and weight into LDS (one trip to memory for all of them), every thread then knows M and the
// denominator, takes an element of the latent and adds up its runs, eight loads under way at a time.
constexpr int MERGE_MAX_RUNS = 256;

__global__ __launch_bounds__(256) void latent_merge_kernel(const float* __restrict__ parts, const float* __restrict__ sinks,
                                                           const int* __restrict__ token_request, float* __restrict__ out, int n_rows,
                                                           int n_heads, int n_runs, int R) {
    __shared__ float factor[MERGE_MAX_RUNS];
    __shared__ float inverse_total;
    const int item = blockIdx.x, token = item / n_heads, head = item % n_heads;
    float* out_row = out + (size_t)item * R;
    if (token_request[token] < 0) {   // uniform over the block
        for (int d = threadIdx.x; d < R; d += blockDim.x) out_row[d] = 0.0f;
        return;
    }
    const float* runs = parts + (size_t)item * n_runs * (R + 2);
    const int p = threadIdx.x;
    const float my_top = p < n_runs ? runs[(size_t)p * (R + 2) + R] : -INFINITY;
    const float my_weight = p < n_runs ? runs[(size_t)p * (R + 2) + R + 1] : 0.0f;
    factor[p] = my_top;
    __syncthreads();
    const float sink = sinks ? sinks[head] : -INFINITY;
    float top = sink;
    for (int other = 0; other < n_runs; other++) top = fmaxf(top, factor[other]);   // finite: the first run always holds a key
    __syncthreads();
    const float mine = my_top == -INFINITY ? 0.0f : expf(my_top - top);
    factor[p] = mine;
    // the denominator: every wave adds up its runs' shares, the first wave the waves'
    __shared__ float wave_share[4];
    const float share = wave_total(mine * my_weight);
    if (threadIdx.x % WAVE == 0) wave_share[threadIdx.x / WAVE] = share;
    __syncthreads();
    if (threadIdx.x == 0) inverse_total = 1.0f / (wave_share[0] + wave_share[1] + wave_share[2] + wave_share[3] + (sinks ? expf(sink - top) : 0.0f));
    __syncthreads();
    const float inverse = inverse_total;
    for (int d = threadIdx.x; d < R; d += blockDim.x) {
        float sum = 0.0f;
        for (int p0 = 0; p0 < n_runs; p0 += 8) {
            float o[8];
#pragma unroll
            for (int u = 0; u < 8; u++) o[u] = runs[(size_t)min(p0 + u, n_runs - 1) * (R + 2) + d];
#pragma unroll
            for (int u = 0; u < 8; u++) sum += p0 + u < n_runs ? o[u] * factor[p0 + u] : 0.0f;
        }
        out_row[d] = sum * inverse;
    }
}

// The same attention on the matrix cores, for bfloat16 caches whose rows are DK x 16 elements with a latent of up to 32 x RT.
// A wave takes 32 (token, head) pairs of one request's portion, neighbours in (token, head) order: they all read the same cached
// rows, so a tile of 32 keys serves 32 pairs in one product. S^T = C Q'^T (a lane's 16-byte piece of its key's row is the
// operand as it lies in memory; the folded queries, rounded to bfloat16 with the scale folded in, stay in registers for the
// whole kernel), the statistics per pair in the lane that owns the pair's column, then O^T += C_latent^T P^T with the weights
// rounded to bfloat16 and the latent elements gathered two at a time (a lane's 32-bit load gives an element to each of two
// output tiles). Sums, scores and statistics are 32-bit. Runs of keys and the sink as in the kernel above.
template <int DK, int RT>
__global__ __launch_bounds__(64) void latent_attention_mfma_kernel(
    const float* __restrict__ q, const bf16_t* __restrict__ pages, const float* __restrict__ sinks, float* __restrict__ out, float* __restrict__ parts,
    const int* __restrict__ q_starts, const int* __restrict__ context_lens, const int* __restrict__ block_tables, int max_blocks,
    int n_heads, int R, int page_size, float scale, int run_length) {
    constexpr int D = 16 * DK;
    const int lane = threadIdx.x, lane32 = lane % 32, half = lane / 32;
    const int request = blockIdx.y, run = blockIdx.z, n_runs = gridDim.z;
    const int context = context_lens[request];
    if (context < 0) return;   // a padding request
    const int q_first = q_starts[request], q_len = q_starts[request + 1] - q_first;
    const int pair0 = blockIdx.x * 32, n_pairs = q_len * n_heads;
    if (pair0 >= n_pairs) return;
    const int pair = pair0 + lane32;
    const bool pair_valid = pair < n_pairs;
    const int token = min(pair / n_heads, q_len - 1), head = pair_valid ? pair % n_heads : 0;
    const int row = q_first + token, position = context + token;
    const int wave_last_position = context + min(q_len - 1, (pair0 + 31) / n_heads);
    const int* table = block_tables + (size_t)request * max_blocks;

    bf16x8 q_op[DK];
    {
        const float* q_row = q + ((size_t)row * n_heads + head) * D + 8 * half;
        const float factor = pair_valid ? scale : 0.0f;
#pragma unroll
        for (int ks = 0; ks < DK; ks++) {
            const f32x4 lo = *reinterpret_cast<const f32x4*>(q_row + 16 * ks), hi = *reinterpret_cast<const f32x4*>(q_row + 16 * ks + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                q_op[ks][e] = static_cast<bf16_t>(lo[e] * factor);
                q_op[ks][4 + e] = static_cast<bf16_t>(hi[e] * factor);
            }
        }
    }
    f32x16 o[RT];
#pragma unroll
    for (int i = 0; i < RT; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[i][v] = 0.0f;
    float top = -INFINITY, weight = 0.0f;

    const int first_key = run * run_length;
    const int last_key = run == n_runs - 1 ? wave_last_position : min(wave_last_position, first_key + run_length - 1);
    for (int kt = first_key; kt <= last_key; kt += 32) {
        const int key = min(kt + lane32, last_key);
        const int slot = table[key / page_size] * page_size + key % page_size;
        const bf16_t* k_row = pages + (size_t)slot * D + 8 * half;
        bf16x8 k_op[DK];
#pragma unroll
        for (int ks = 0; ks < DK; ks++) k_op[ks] = *reinterpret_cast<const bf16x8*>(k_row + 16 * ks);
        f32x16 s;
#pragma unroll
        for (int v = 0; v < 16; v++) s[v] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < DK; ks++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_op[ks], q_op[ks], s, 0, 0, 0);
        float tile_top = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int at = kt + 8 * (v / 4) + 4 * half + (v % 4);
            s[v] = pair_valid && at <= position && at <= last_key ? s[v] : -INFINITY;
            tile_top = fmaxf(tile_top, s[v]);
        }
        tile_top = fmaxf(tile_top, __shfl_xor(tile_top, 32, WAVE));
        const float new_top = fmaxf(top, tile_top);
        const float safe_top = new_top == -INFINITY ? 0.0f : new_top;   // a pair none of whose keys has come yet
        const float rescale = expf(top - safe_top);
        top = new_top;
        weight *= rescale;
#pragma unroll
        for (int i = 0; i < RT; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) o[i][v] *= rescale;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            s[v] = expf(s[v] - safe_top);
            weight += s[v];
        }
#pragma unroll
        for (int slab = 0; slab < 2; slab++) {   // 16 keys each: the lane's score registers 8 * slab .. + 7
            bf16x8 p;
#pragma unroll
            for (int e = 0; e < 8; e++) p[e] = static_cast<bf16_t>(s[8 * slab + e]);
            // the keys those registers belong to: 16 * slab + 4 * half + 0..3 and eight further on; their cached rows
            const bf16_t* rows_at[8];
#pragma unroll
            for (int e = 0; e < 8; e++) rows_at[e] = pages + (size_t)__shfl(slot, 16 * slab + 4 * half + (e % 4) + 8 * (e / 4), WAVE) * D;
#pragma unroll
            for (int t = 0; t < RT / 2; t++) {
                const int d = min(64 * t + 2 * lane32, D - 2);
                uint32_t word[8];
#pragma unroll
                for (int e = 0; e < 8; e++) word[e] = *reinterpret_cast<const uint32_t*>(rows_at[e] + d);
                Vec16 even, odd;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    even.w[j] = (word[2 * j] & 0xffffu) | (word[2 * j + 1] << 16);
                    odd.w[j] = (word[2 * j] >> 16) | (word[2 * j + 1] & 0xffff0000u);
                }
                o[2 * t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(&even), p, o[2 * t], 0, 0, 0);
                o[2 * t + 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(&odd), p, o[2 * t + 1], 0, 0, 0);
            }
        }
    }
    weight += __shfl_xor(weight, 32, WAVE);
    if (!pair_valid) return;
    const size_t item = (size_t)row * n_heads + head;
    if (n_runs == 1) {
        float inverse;
        if (sinks) {
            const float sink = sinks[head], highest = fmaxf(top, sink);
            const float shrink = expf(top - highest);
            inverse = shrink / (weight * shrink + expf(sink - highest));
        } else {
            inverse = 1.0f / weight;
        }
        float* out_row = out + item * R;
#pragma unroll
        for (int i = 0; i < RT; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int d = 64 * (i / 2) + 2 * (8 * (v / 4) + 4 * half + (v % 4)) + (i % 2);
                if (d < R) out_row[d] = o[i][v] * inverse;
            }
        return;
    }
    float* mine = parts + (item * n_runs + run) * (R + 2);
#pragma unroll
    for (int i = 0; i < RT; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int d = 64 * (i / 2) + 2 * (8 * (v / 4) + 4 * half + (v % 4)) + (i % 2);
            if (d < R) mine[d] = o[i][v];
        }
    if (half == 0) {
        mine[R] = top;
        mine[R + 1] = weight;
    }
}

struct LatentMfmaArgs {
    const float* q; const bf16_t* pages; const float* sinks; float* out; float* parts; const int* q_starts; const int* context_lens;
    const int* block_tables; int max_blocks, n_heads, R, page_size; float scale; int run_length; dim3 grid; hipStream_t stream;
};

template <int DK, int RT>
void launch_latent_mfma(const LatentMfmaArgs& a) {
    latent_attention_mfma_kernel<DK, RT><<<a.grid, 64, 0, a.stream>>>(a.q, a.pages, a.sinks, a.out, a.parts, a.q_starts, a.context_lens, a.block_tables,
                                                                      a.max_blocks, a.n_heads, a.R, a.page_size, a.scale, a.run_length);
}

template <int DK>
bool launch_latent_mfma_rt(const LatentMfmaArgs& a) {
    if (a.R <= 64) launch_latent_mfma<DK, 2>(a);
    else if constexpr (DK >= 6) {
        if (a.R <= 128) launch_latent_mfma<DK, 4>(a);
        else if constexpr (DK >= 12) launch_latent_mfma<DK, 8>(a);
        else return false;
    } else return false;
    return true;
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

// Heads a wave takes at once: all of them in equal groups where the count allows, else groups of which the last is not full.
int latent_head_group(int n_heads) {
    if (n_heads % 8 == 0) return 8;
    if (n_heads % 6 == 0) return 6;
    if (n_heads % 4 == 0) return 4;
    return n_heads <= 4 ? 4 : (n_heads <= 6 ? 6 : 8);
}

struct LatentArgs {
    const float* q; const void* pages; const float* sinks; float* out; float* parts; const int* token_request; const int* positions;
    const int* block_tables; int max_blocks, n_rows, n_heads, R, D, page_size; float scale; int n_runs, run_length; hipStream_t stream;
};

template <typename T, int HG, int RV>
void launch_latent(const LatentArgs& a) {
    dim3 grid(ceil_div(a.n_rows, LATENT_ROWS), a.n_runs, ceil_div(a.n_heads, HG));
    latent_attention_kernel<T, HG, RV><<<grid, 64 * LATENT_ROWS, 0, a.stream>>>(a.q, (const T*)a.pages, a.sinks, a.out, a.parts, a.token_request, a.positions,
                                                                                a.block_tables, a.max_blocks, a.n_rows, a.n_heads, a.R, a.D, a.page_size,
                                                                                a.scale, a.run_length);
}

template <typename T, int HG>
void launch_latent_rv(const LatentArgs& a) {
    if (a.R <= 2 * WAVE) launch_latent<T, HG, 2>(a);
    else if (a.R <= 4 * WAVE) launch_latent<T, HG, 4>(a);
    else launch_latent<T, HG, 8>(a);
}

template <typename T>
void launch_latent_hg(const LatentArgs& a) {
    switch (latent_head_group(a.n_heads)) {
        case 4: launch_latent_rv<T, 4>(a); break;
        case 6: launch_latent_rv<T, 6>(a); break;
        default: launch_latent_rv<T, 8>(a); break;
    }
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
    const int threads = 256, cols = N > 128 ? 256 : (N > 64 ? 128 : 64);
    const size_t lds = ((size_t)HEADS_ROWS * K + (size_t)(threads / cols - 1) * cols * HEADS_ROWS) * sizeof(float);
    MLLM_REQUIRE(lds <= 64 * 1024, "heads_linear: K = %d is more than a block holds in LDS", K);
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_HEADS_LINEAR);
    const size_t x_element = x_dtype == MLLM_F32 ? 4 : 2;
    if (w_dtype == MLLM_BF16 && K % 16 == 0 && (size_t)x % 16 == 0 && (x_row_stride * x_element) % 16 == 0 && (x_head_stride * x_element) % 16 == 0 &&
        (size_t)w % 16 == 0) {
        dim3 tiles(ceil_div(n_rows, 32), n_heads, ceil_div(N, 128));
        if (x_dtype == MLLM_F32)
            heads_linear_mfma_kernel<float><<<tiles, 256, 0, stream>>>((const float*)x, x_row_stride, x_head_stride, (const bf16_t*)w, gate, gate_dtype,
                                                                       gate_row_stride, out, out_dtype, out_row_stride, out_head_stride, n_rows, N, K);
        else
            heads_linear_mfma_kernel<bf16_t><<<tiles, 256, 0, stream>>>((const bf16_t*)x, x_row_stride, x_head_stride, (const bf16_t*)w, gate, gate_dtype,
                                                                        gate_row_stride, out, out_dtype, out_row_stride, out_head_stride, n_rows, N, K);
        return mllm_check_launch("heads_linear");
    }
    dim3 grid(ceil_div(n_rows, HEADS_ROWS), n_heads);
    if (w_dtype == MLLM_F32) {
        if (allow_lds(heads_linear_kernel<float>, lds, "heads_linear")) return 1;
        heads_linear_kernel<float><<<grid, threads, lds, stream>>>(x, x_dtype, x_row_stride, x_head_stride, (const float*)w, gate, gate_dtype, gate_row_stride, out, out_dtype,
                                                                   out_row_stride, out_head_stride, n_rows, N, K, cols);
    } else {
        if (allow_lds(heads_linear_kernel<bf16_t>, lds, "heads_linear")) return 1;
        heads_linear_kernel<bf16_t><<<grid, threads, lds, stream>>>(x, x_dtype, x_row_stride, x_head_stride, (const bf16_t*)w, gate, gate_dtype, gate_row_stride, out, out_dtype,
                                                                    out_row_stride, out_head_stride, n_rows, N, K, cols);
    }
    return mllm_check_launch("heads_linear");
}

// Whether the latent attention kernel takes rows of D elements of which R are the latent.
MLLM_API int mllm_latent_attention_supported(int R, int D, int dtype) {
    const int element = dtype == MLLM_F32 ? 4 : 2;
    return R > 0 && R <= D && R <= 8 * WAVE && (D * element) % 16 == 0;
}

// How many heads a wave of the latent attention kernel takes at once (its launches have rows / 4 x runs x heads / this many blocks).
MLLM_API int mllm_latent_attention_head_group(int n_heads) { return n_heads > 0 ? latent_head_group(n_heads) : 0; }

MLLM_API int mllm_latent_attention(const float* q, const void* pages, const float* sinks, float* out, float* parts, const int* token_request,
                                   const int* positions, const int* block_tables, int max_blocks, int n_rows, int n_heads, int R, int D,
                                   int page_size, float scale, int n_runs, int run_length, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && max_blocks > 0 && page_size > 0, "latent_attention: bad sizes");
    MLLM_REQUIRE(dtype == MLLM_F32 || dtype == MLLM_BF16, "latent_attention: unknown dtype %d", dtype);
    MLLM_REQUIRE(mllm_latent_attention_supported(R, D, dtype), "latent_attention: no kernel for rows of %d elements with a latent of %d", D, R);
    MLLM_REQUIRE(n_runs >= 1 && n_runs <= MERGE_MAX_RUNS && run_length >= 1, "latent_attention: bad runs");
    MLLM_REQUIRE(n_runs == 1 || parts != nullptr, "latent_attention: runs need room for their sums");
    if (n_rows == 0) return 0;
    if (n_runs == 1) run_length = 1 << 30;
    const LatentArgs args{q, pages, sinks, out, parts, token_request, positions, block_tables, max_blocks, n_rows, n_heads, R, D, page_size, scale, n_runs, run_length, stream};
    mllm_count_kernel(MLLM_K_LATENT_ATTENTION);
    if (dtype == MLLM_F32) launch_latent_hg<float>(args);
    else launch_latent_hg<bf16_t>(args);
    int status = mllm_check_launch("latent_attention");
    if (status || n_runs == 1) return status;
    const long long items = (long long)n_rows * n_heads;
    mllm_count_kernel(MLLM_K_LATENT_MERGE);
    latent_merge_kernel<<<(int)items, 256, 0, stream>>>(parts, sinks, token_request, out, n_rows, n_heads, n_runs, R);
    return mllm_check_launch("latent_merge");
}

// Rows of how many elements the matrix-core kernel takes: the smallest such size that holds `needed` elements (0: none does,
// and the rows are walked by the kernel above, which takes any multiple of 16 bytes).
MLLM_API int mllm_latent_mfma_row_size(int needed) {
    for (int size : {32, 64, 96, 128, 192, 288})
        if (needed <= size) return size;
    return 0;
}

MLLM_API int mllm_latent_attention_mfma_supported(int R, int D, int dtype) {
    return dtype == MLLM_BF16 && R > 0 && R <= D && R <= 256 && mllm_latent_mfma_row_size(D) == D;
}

// q_starts [requests + 1] and context_lens [requests] (negative: a padding request): each request's rows are consecutive, its
// first row's position is its stored length. max_pairs: the most (token, head) pairs any request brings.
MLLM_API int mllm_latent_attention_mfma(const float* q, const void* pages, const float* sinks, float* out, float* parts, const int* token_request,
                                        const int* q_starts, const int* context_lens, const int* block_tables, int max_blocks, int n_rows,
                                        int n_requests, int max_pairs, int n_heads, int R, int D, int page_size, float scale, int n_runs,
                                        int run_length, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_requests >= 0 && n_heads > 0 && max_blocks > 0 && page_size > 0 && max_pairs > 0, "latent_attention_mfma: bad sizes");
    MLLM_REQUIRE(mllm_latent_attention_mfma_supported(R, D, MLLM_BF16), "latent_attention_mfma: no kernel for rows of %d elements with a latent of %d", D, R);
    MLLM_REQUIRE(n_runs >= 1 && n_runs <= MERGE_MAX_RUNS && n_requests <= 65535 && run_length >= 1 && (n_runs == 1 || run_length % 32 == 0), "latent_attention_mfma: bad runs");
    MLLM_REQUIRE(n_runs == 1 || parts != nullptr, "latent_attention_mfma: runs need room for their sums");
    if (n_rows == 0 || n_requests == 0) return 0;
    if (n_runs == 1) run_length = 1 << 30;
    LatentMfmaArgs a{q, (const bf16_t*)pages, sinks, out, parts, q_starts, context_lens, block_tables, max_blocks, n_heads, R, page_size, scale, run_length,
                     dim3(ceil_div(max_pairs, 32), n_requests, n_runs), stream};
    mllm_count_kernel(MLLM_K_LATENT_ATTENTION);
    bool launched = false;
    switch (D / 16) {
        case 2: launched = launch_latent_mfma_rt<2>(a); break;
        case 4: launched = launch_latent_mfma_rt<4>(a); break;
        case 6: launched = launch_latent_mfma_rt<6>(a); break;
        case 8: launched = launch_latent_mfma_rt<8>(a); break;
        case 12: launched = launch_latent_mfma_rt<12>(a); break;
        case 18: launched = launch_latent_mfma_rt<18>(a); break;
    }
    MLLM_REQUIRE(launched, "latent_attention_mfma: no kernel for rows of %d elements with a latent of %d", D, R);
    int status = mllm_check_launch("latent_attention_mfma");
    if (status || n_runs == 1) return status;
    const long long items = (long long)n_rows * n_heads;
    mllm_count_kernel(MLLM_K_LATENT_MERGE);
    latent_merge_kernel<<<(int)items, 256, 0, stream>>>(parts, sinks, token_request, out, n_rows, n_heads, n_runs, R);
    return mllm_check_launch("latent_merge");
}
