// Mixers that keep a matrix per head and request instead of keys and values: S_t = a_t S_(t-1) + b_t k_t v_t^T, o_t = S_t^T q_t.
// Two kinds share the kernels of this file (one that walks a portion row by row, for decoding and short portions, and three
// further down that take long portions chunk by chunk):
//   GATED (the matrix memory of an mLSTM): log gates i_t and f_t per head and token, a running maximum m that starts at 0,
//     m_t = max(f_t + m_(t-1), i_t), a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t); a vector n that follows the same
//     recurrence with k alone; o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6). The gates arrive as the sums of their
//     projections (bias included): i = cap tanh(raw / cap), f = logsigmoid(cap tanh(raw / cap)); cap <= 0: no cap.
//   DECAYED (a linear attention with a fixed decay per head): a_t = decay_h, b_t = 1, q, k and v pass through silu first.
// State, gates, sums and outputs are 32-bit. The state of a request lies in its slot: S [heads, dim, vdim], then (GATED)
// n [heads, dim] and m [heads].
//
// Row by row: a block takes one (request, head, tile of VT value columns) and walks the request's rows of this step in order. Thread
// (part p, column j) keeps S[p R .. p R + R - 1, j] in registers across all rows. Rows are taken TB at a time: their q, k, v
// are staged in LDS while the first wave settles the gates of those rows (the scalar recurrence of m), then every thread
// moves its piece of S on row by row and leaves its share of each row's output, which are added up over the parts at the end.
#include "common.h"

namespace {

enum : int { GATED = 0, DECAYED = 1 };

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

template <int R, int MODE>
__global__ __launch_bounds__(512) void recurrence_kernel(const float* __restrict__ q, int q_stride, const float* __restrict__ k, int k_stride,
                                                         const float* __restrict__ v, int v_stride, const float* __restrict__ gate_in,
                                                         const float* __restrict__ gate_forget, int gate_stride, float cap,
                                                         const float* __restrict__ decay, float q_scale, float* __restrict__ state,
                                                         long long state_stride, long long n_at, long long m_at,
                                                         const int* __restrict__ q_starts, const int* __restrict__ state_slots,
                                                         float* __restrict__ out, int out_stride, int dim, int vdim, int P, int VT, int TB) {
    extern __shared__ float lds[];
    const int request = blockIdx.x, head = blockIdx.y;
    const int slot = state_slots[request];
    const int first_row = q_starts[request], rows = q_starts[request + 1] - first_row;
    if (slot < 0 || rows <= 0) return;   // the whole block: a padding request, or one that brings nothing

    const int dim_pad = P * R;
    float* sq = lds;                              // [TB][dim_pad]
    float* sk = sq + TB * dim_pad;                // [TB][dim_pad]
    float* sv = sk + TB * dim_pad;                // [TB][VT]
    float* keep = sv + TB * VT;                   // [TB] a_t
    float* take = keep + TB;                      // [TB] b_t
    float* floor_ = take + TB;                    // [TB] exp(-m_t)
    float* part = floor_ + TB;                    // [TB][P][VT]
    float* nq_part = part + TB * P * VT;          // [TB][P]

    const int tid = threadIdx.x;
    const int p = tid / VT, jt = tid % VT;
    const int j = blockIdx.z * VT + jt;
    const bool works = p < P;
    const bool column = works && j < vdim;
    const int i0 = p * R;
    float* mine = state + (size_t)slot * state_stride;
    float* S_at = mine + ((size_t)head * dim) * vdim;

    float S[R], n[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        S[r] = column && i0 + r < dim ? S_at[(size_t)(i0 + r) * vdim + j] : 0.0f;
        n[r] = 0.0f;
        if (MODE == GATED) n[r] = works && i0 + r < dim ? mine[n_at + (size_t)head * dim + i0 + r] : 0.0f;
    }
    float m = MODE == GATED ? mine[m_at + head] : 0.0f;   // every thread reads it; the first wave moves it on
    const float fixed_decay = MODE == DECAYED ? decay[head] : 0.0f;

    for (int t0 = 0; t0 < rows; t0 += TB) {
        const int n_valid = min(TB, rows - t0);
        // ---- staging: q and k of the head (zeros beyond dim), v of the tile ----
        for (int e = tid; e < n_valid * dim_pad; e += blockDim.x) {
            const int t = e / dim_pad, i = e % dim_pad;
            const size_t row = (size_t)(first_row + t0 + t);
            float qv = 0.0f, kv = 0.0f;
            if (i < dim) {
                qv = q[row * q_stride + head * dim + i];
                kv = k[row * k_stride + head * dim + i];
                if (MODE == DECAYED) qv = silu_f(qv), kv = silu_f(kv);
                qv *= q_scale;
            }
            sq[t * dim_pad + i] = qv;
            sk[t * dim_pad + i] = kv;
        }
        for (int e = tid; e < n_valid * VT; e += blockDim.x) {
            const int t = e / VT, c = blockIdx.z * VT + e % VT;
            float vv = 0.0f;
            if (c < vdim) {
                vv = v[(size_t)(first_row + t0 + t) * v_stride + head * vdim + c];
                if (MODE == DECAYED) vv = silu_f(vv);
            }
            sv[t * VT + e % VT] = vv;
        }
        if (tid < WAVE) {   // the first wave: lane t takes row t's gates, then all lanes walk the rows together
            if (MODE == GATED) {
                float gi = 0.0f, gf = 0.0f;
                if (tid < n_valid) {
                    const size_t row = (size_t)(first_row + t0 + tid);
                    gi = gate_in[row * gate_stride + head];
                    gf = gate_forget[row * gate_stride + head];
                    if (cap > 0.0f) gi = cap * tanhf(gi / cap), gf = cap * tanhf(gf / cap);
                    gf = log_sigmoid_f(gf);
                }
                for (int t = 0; t < n_valid; t++) {
                    const float it = __shfl(gi, t, WAVE), ft = __shfl(gf, t, WAVE);
                    const float m_new = fmaxf(ft + m, it);
                    if (tid == 0) {   // the differences in 64-bit: next to a large m, f + m - m' would lose what f holds
                        keep[t] = expf((float)((double)ft + (double)m - (double)m_new));
                        take[t] = expf((float)((double)it - (double)m_new));
                        floor_[t] = expf(-m_new);
                    }
                    m = m_new;
                }
            } else if (tid < n_valid) {
                keep[tid] = fixed_decay;
                take[tid] = 1.0f;
            }
        }
        __syncthreads();
        // ---- every thread moves its piece of S over the rows ----
        if (works) {
            for (int t = 0; t < n_valid; t++) {
                const float a = keep[t], b = take[t];
                const float bv = b * sv[t * VT + jt];
                const float* kt = sk + t * dim_pad + i0;
                const float* qt = sq + t * dim_pad + i0;
                float sum = 0.0f, nq = 0.0f;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    S[r] = a * S[r] + bv * kt[r];
                    sum += S[r] * qt[r];
                    if (MODE == GATED) {
                        n[r] = a * n[r] + b * kt[r];
                        nq += n[r] * qt[r];
                    }
                }
                part[(t * P + p) * VT + jt] = sum;
                if (MODE == GATED && jt == 0) nq_part[t * P + p] = nq;
            }
        }
        __syncthreads();
        // ---- the parts of each row's output added up ----
        for (int e = tid; e < n_valid * VT; e += blockDim.x) {
            const int t = e / VT, c = e % VT;
            if (blockIdx.z * VT + c >= vdim) continue;
            float sum = 0.0f;
            for (int pp = 0; pp < P; pp++) sum += part[(t * P + pp) * VT + c];
            if (MODE == GATED) {
                float nq = 0.0f;
                for (int pp = 0; pp < P; pp++) nq += nq_part[t * P + pp];
                sum /= fmaxf(fabsf(nq), floor_[t]) + 1e-6f;
            }
            out[(size_t)(first_row + t0 + t) * out_stride + head * vdim + blockIdx.z * VT + c] = sum;
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (column && i0 + r < dim) S_at[(size_t)(i0 + r) * vdim + j] = S[r];
        if (MODE == GATED && works && jt == 0 && blockIdx.z == 0 && i0 + r < dim) mine[n_at + (size_t)head * dim + i0 + r] = n[r];
    }
    if (MODE == GATED && tid == 0 && blockIdx.z == 0) mine[m_at + head] = m;
}

struct Plan {
    int R, P, VT, TB, threads, tiles;
    size_t lds_bytes;
};

// How a head of dim x vdim is laid over a block: tiles of up to 64 value columns, as many parts along dim as 512 threads
// allow, a power of two of rows of S a thread (up to 64: two waves a SIMD leave a thread 256 registers).
bool plan_for(int dim, int vdim, Plan& plan) {
    plan.VT = vdim <= 64 ? vdim : 64;
    plan.tiles = ceil_div(vdim, plan.VT);
    int most_parts = 512 / plan.VT;
    if (most_parts > dim) most_parts = dim;
    if (most_parts < 1) most_parts = 1;
    plan.R = 1;
    while (plan.R * most_parts < dim) plan.R *= 2;
    if (plan.R > 64) return false;
    plan.P = ceil_div(dim, plan.R);
    plan.threads = ceil_div(plan.P * plan.VT, 64) * 64;
    plan.TB = 8;
    for (;;) {
        plan.lds_bytes = (size_t)plan.TB * (2 * plan.P * plan.R + plan.VT + 3 + plan.P * plan.VT + plan.P) * sizeof(float);
        if (plan.lds_bytes <= 60 * 1024 || plan.TB == 1) break;
        plan.TB /= 2;
    }
    return plan.lds_bytes <= 64 * 1024;
}

}  // namespace

// 1 if a head of these sizes is taken.
MLLM_API int mllm_recurrence_supported(int dim, int vdim) {
    Plan plan;
    return dim > 0 && vdim > 0 && plan_for(dim, vdim, plan) ? 1 : 0;
}

// kind 0: gated (gate_in, gate_forget [rows, heads] strided, cap); kind 1: decayed (decay [heads]).
MLLM_API int mllm_recurrence(int kind, const float* q, int q_stride, const float* k, int k_stride, const float* v, int v_stride, const float* gate_in,
                             const float* gate_forget, int gate_stride, float cap, const float* decay, float q_scale, float* state,
                             long long state_stride, long long n_at, long long m_at, const int* q_starts, const int* state_slots, float* out,
                             int out_stride, int n_requests, int n_heads, int dim, int vdim, hipStream_t stream) {
    MLLM_REQUIRE(kind == GATED || kind == DECAYED, "recurrence: unknown kind %d", kind);
    MLLM_REQUIRE(n_requests >= 0 && n_heads > 0 && dim > 0 && vdim > 0, "recurrence: bad sizes");
    Plan plan;
    MLLM_REQUIRE(plan_for(dim, vdim, plan), "recurrence: heads of %d x %d are larger than the kernel takes", dim, vdim);
    MLLM_REQUIRE(q_stride >= n_heads * dim && k_stride >= n_heads * dim && v_stride >= n_heads * vdim && out_stride >= n_heads * vdim, "recurrence: rows are too short for the heads");
    MLLM_REQUIRE(q != nullptr && k != nullptr && v != nullptr && state != nullptr && q_starts != nullptr && state_slots != nullptr && out != nullptr, "recurrence: a missing operand");
    const long long matrices = (long long)n_heads * dim * vdim;
    if (kind == GATED) {
        MLLM_REQUIRE(gate_in != nullptr && gate_forget != nullptr && gate_stride >= n_heads, "recurrence: the gates are missing");
        MLLM_REQUIRE(n_at >= matrices && m_at >= n_at + (long long)n_heads * dim && state_stride >= m_at + n_heads, "recurrence: the state's parts overlap");
    } else {
        MLLM_REQUIRE(decay != nullptr && state_stride >= matrices, "recurrence: the decays are missing or the state is too small");
    }
    if (n_requests == 0) return 0;
    mllm_count_kernel(MLLM_K_RECURRENCE);
    dim3 grid(n_requests, n_heads, plan.tiles);
#define RECURRENCE_ARGS q, q_stride, k, k_stride, v, v_stride, gate_in, gate_forget, gate_stride, cap, decay, q_scale, state, state_stride, n_at, m_at, q_starts, \
                        state_slots, out, out_stride, dim, vdim, plan.P, plan.VT, plan.TB
#define LAUNCH(R)                                                                                                              \
    do {                                                                                                                       \
        if (kind == GATED) recurrence_kernel<R, GATED><<<grid, plan.threads, plan.lds_bytes, stream>>>(RECURRENCE_ARGS);       \
        else recurrence_kernel<R, DECAYED><<<grid, plan.threads, plan.lds_bytes, stream>>>(RECURRENCE_ARGS);                   \
    } while (0)
    switch (plan.R) {
        case 1: LAUNCH(1); break;
        case 2: LAUNCH(2); break;
        case 4: LAUNCH(4); break;
        case 8: LAUNCH(8); break;
        case 16: LAUNCH(16); break;
        case 32: LAUNCH(32); break;
        default: LAUNCH(64); break;
    }
#undef LAUNCH
#undef RECURRENCE_ARGS
    return mllm_check_launch("recurrence");
}

// ------------------------------------------------------------------------------------------------------------------------
// Long portions: the same recurrences chunk by chunk, so that the rows of a portion do not wait for each other.
//
// Inside a chunk of L rows (b_t the sum of the log decays up to row t, g_s the log input gate of row s, both 0-based inside the
// chunk; the state S0, n0, m0 at the chunk's start):
//     m_t = b_t + max(m0, max_{s<=t}(g_s - b_s))
//     o_t = [exp(b_t + m0 - m_t) q_t^T S0 + sum_{s<=t} exp(b_t - b_s + g_s - m_t) (q_t . k_s) v_s] / (max(|nq_t|, exp(-m_t)) + 1e-6)
//     nq_t = exp(b_t + m0 - m_t) q_t . n0 + sum_{s<=t} exp(b_t - b_s + g_s - m_t) (q_t . k_s)
// and over the whole chunk, with B = b_(L-1) and mu = max_s(B - b_s + g_s),
//     U = sum_s exp(B - b_s + g_s - mu) k_s v_s^T,  m' = max(B + m0, mu),  S' = exp(B + m0 - m') S0 + exp(mu - m') U   (n likewise),
// which is what the row-by-row recurrence gives, in another order of sums. Without gates (a fixed decay) g = 0, m = 0 throughout.
// Three kernels: (1) every chunk's U, its share of n, B and mu, all chunks at once; (2) per (request, head) the chunks in order,
// a few multiply-adds an element: each chunk's U is replaced by the state at its start, and the request's slot gets the state at
// the portion's end; (3) every chunk's outputs, all chunks at once. The sums b_t are taken in 64-bit, so that the difference of
// two of them is exact to 32 bits however far the gates have closed.
//
// Scratch: one record of dim * vdim + dim + 4 floats per (chunk, head). Chunk c of request r, whose first row in the batch is
// f, has the record f / L + r: no two chunks of a batch share one, and there are at most rows / L + requests of them.
// ------------------------------------------------------------------------------------------------------------------------
namespace {

constexpr int CHUNK_THREADS = 512, CHUNK_WAVES = CHUNK_THREADS / WAVE, CHUNK_VT = 64;

template <int L>
struct ChunkShape {
    static constexpr int DIM_MAX = 4096 / L;   // L = 64: heads up to 64 wide; 32: up to 128; 16: up to 256
    static constexpr int RPW = L / CHUNK_WAVES;
};

__device__ __forceinline__ size_t chunk_record(int first_row, int chunk_rows, int request) { return (size_t)(first_row / chunk_rows + request); }

__device__ __forceinline__ double lanes_prefix_sum(double v, int lane) {
#pragma unroll
    for (int offset = 1; offset < WAVE; offset <<= 1) {
        const double other = __shfl_up(v, offset, WAVE);
        if (lane >= offset) v += other;
    }
    return v;
}
__device__ __forceinline__ double lanes_prefix_max(double v, int lane) {
#pragma unroll
    for (int offset = 1; offset < WAVE; offset <<= 1) {
        const double other = __shfl_up(v, offset, WAVE);
        if (lane >= offset) v = fmax(v, other);
    }
    return v;
}

// The log decay and log input gate of a row (see the head of this file).
template <int MODE>
__device__ __forceinline__ void row_gates(const float* gate_in, const float* gate_forget, int gate_stride, float cap, float log_decay, size_t row,
                                          int head, float& log_keep, float& log_take) {
    if (MODE == GATED) {
        float gi = gate_in[row * gate_stride + head], gf = gate_forget[row * gate_stride + head];
        if (cap > 0.0f) gi = cap * tanhf(gi / cap), gf = cap * tanhf(gf / cap);
        log_take = gi;
        log_keep = log_sigmoid_f(gf);
    } else {
        log_take = 0.0f;
        log_keep = log_decay;
    }
}

template <int L, int MODE>
__global__ __launch_bounds__(CHUNK_THREADS) void chunk_sums_kernel(const float* __restrict__ k, int k_stride, const float* __restrict__ v, int v_stride,
                                                                   const float* __restrict__ gate_in, const float* __restrict__ gate_forget,
                                                                   int gate_stride, float cap, const float* __restrict__ decay,
                                                                   const int* __restrict__ q_starts, const int* __restrict__ state_slots,
                                                                   float* __restrict__ scratch, int dim, int vdim, int tiles) {
    constexpr int DIM_MAX = ChunkShape<L>::DIM_MAX;
    __shared__ float Ks[L][DIM_MAX];
    __shared__ float Vs[L][CHUNK_VT];
    __shared__ float weight[L];
    const int request = blockIdx.x, head = blockIdx.y, n_heads = gridDim.y, chunk = blockIdx.z / tiles, tile = blockIdx.z % tiles;
    const int first_row = q_starts[request], rows = q_starts[request + 1] - first_row;
    if (state_slots[request] < 0 || chunk * L >= rows) return;
    const int n_valid = min(L, rows - chunk * L), chunk_first = first_row + chunk * L;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const size_t record_floats = (size_t)dim * vdim + dim + 4;
    float* record = scratch + (chunk_record(chunk_first, L, request) * n_heads + head) * record_floats;

    for (int e = tid; e < L * dim; e += CHUNK_THREADS) {
        const int s = e / dim, i = e % dim;
        float value = 0.0f;
        if (s < n_valid) {
            value = k[(size_t)(chunk_first + s) * k_stride + head * dim + i];
            if (MODE == DECAYED) value = silu_f(value);
        }
        Ks[s][i] = value;
    }
    for (int e = tid; e < L * CHUNK_VT; e += CHUNK_THREADS) {
        const int s = e / CHUNK_VT, c = tile * CHUNK_VT + e % CHUNK_VT;
        float value = 0.0f;
        if (s < n_valid && c < vdim) {
            value = v[(size_t)(chunk_first + s) * v_stride + head * vdim + c];
            if (MODE == DECAYED) value = silu_f(value);
        }
        Vs[s][e % CHUNK_VT] = value;
    }
    if (wave == 0) {
        float log_keep = 0.0f, log_take = 0.0f;
        if (lane < n_valid) row_gates<MODE>(gate_in, gate_forget, gate_stride, cap, MODE == DECAYED ? logf(decay[head]) : 0.0f, (size_t)(chunk_first + lane), head, log_keep, log_take);
        const double b = lanes_prefix_sum((double)log_keep, lane);
        const double total = __shfl(b, n_valid - 1, WAVE);
        const double reach = lane < n_valid ? (total - b) + (double)log_take : -INFINITY;
        const float mu = MODE == GATED ? wave_max((float)reach) : 0.0f;
        if (lane < L) weight[lane] = lane < n_valid ? expf((float)(reach - (double)mu)) : 0.0f;
        if (lane == 0 && tile == 0) {
            record[record_floats - 4] = (float)total;
            record[record_floats - 3] = mu;
        }
    }
    __syncthreads();
    // U[i][j] = sum_s weight_s k_s[i] v_s[j]: a lane a column of the tile, a wave every eighth row i
    constexpr int ROWS = DIM_MAX / CHUNK_WAVES;
    float acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) acc[r] = 0.0f;
    for (int s = 0; s < n_valid; s++) {
        const float vv = Vs[s][lane] * weight[s];
#pragma unroll
        for (int r = 0; r < ROWS; r++) acc[r] += Ks[s][wave + r * CHUNK_WAVES] * vv;
    }
    const int j = tile * CHUNK_VT + lane;
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
        const int i = wave + r * CHUNK_WAVES;
        if (i < dim && j < vdim) record[(size_t)i * vdim + j] = acc[r];
    }
    if (MODE == GATED && tile == 0 && tid < dim) {
        float sum = 0.0f;
        for (int s = 0; s < n_valid; s++) sum += weight[s] * Ks[s][tid];
        record[(size_t)dim * vdim + tid] = sum;
    }
}

// The chunks of one (request, head) in order. A block takes up to 4,096 elements of the matrix (16 a thread); the block of the
// first elements also moves n and m on. Each chunk's record gets the state at the chunk's start (matrix, n, and m in its last
// place but two), and the request's slot the state at the portion's end.
template <int MODE>
__global__ __launch_bounds__(256) void chunk_scan_kernel(const int* __restrict__ q_starts, const int* __restrict__ state_slots, float* __restrict__ scratch,
                                                         float* __restrict__ state, long long state_stride, long long n_at, long long m_at, int dim, int vdim,
                                                         int chunk_rows) {
    constexpr int PER = 16;
    const int request = blockIdx.x, head = blockIdx.y, n_heads = gridDim.y;
    const int slot = state_slots[request];
    const int first_row = q_starts[request], rows = q_starts[request + 1] - first_row;
    if (slot < 0 || rows <= 0) return;
    const int n_chunks = (rows + chunk_rows - 1) / chunk_rows;
    const size_t elements = (size_t)dim * vdim, record_floats = elements + dim + 4;
    const size_t base = (size_t)blockIdx.z * 256 * PER;
    float* mine = state + (size_t)slot * state_stride;
    float* S_at = mine + (size_t)head * elements;
    const bool first_block = blockIdx.z == 0;
    const int tid = threadIdx.x;
    float S[PER], n = 0.0f;
#pragma unroll
    for (int u = 0; u < PER; u++) {
        const size_t e = base + (size_t)u * 256 + tid;
        S[u] = e < elements ? S_at[e] : 0.0f;
    }
    if (MODE == GATED && first_block && tid < dim) n = mine[n_at + (size_t)head * dim + tid];
    float m = MODE == GATED ? mine[m_at + head] : 0.0f;
    auto record_of = [&](int c) { return scratch + (chunk_record(first_row + c * chunk_rows, chunk_rows, request) * n_heads + head) * record_floats; };
    // the numbers of four chunks are asked for at once (a pass over the chunks one by one waits for memory at every chunk)
    constexpr int AHEAD = 4;
    for (int c0 = 0; c0 < n_chunks; c0 += AHEAD) {
        float sums[AHEAD][PER], sum_n[AHEAD], total[AHEAD], mu[AHEAD];
#pragma unroll
        for (int d = 0; d < AHEAD; d++) {
            const float* record = record_of(min(c0 + d, n_chunks - 1));
#pragma unroll
            for (int u = 0; u < PER; u++) {
                const size_t e = base + (size_t)u * 256 + tid;
                sums[d][u] = record[min(e, elements - 1)];
            }
            sum_n[d] = MODE == GATED && first_block ? record[elements + min(tid, dim - 1)] : 0.0f;
            total[d] = record[record_floats - 4];
            mu[d] = record[record_floats - 3];
        }
#pragma unroll
        for (int d = 0; d < AHEAD; d++) {
            if (c0 + d >= n_chunks) break;
            float* record = record_of(c0 + d);
            float keep, take, m_new = 0.0f;
            if (MODE == GATED) {
                m_new = fmaxf(total[d] + m, mu[d]);
                keep = expf((float)((double)total[d] + (double)m - (double)m_new));
                take = expf((float)((double)mu[d] - (double)m_new));
            } else {
                keep = expf(total[d]);
                take = 1.0f;
            }
#pragma unroll
            for (int u = 0; u < PER; u++) {
                const size_t e = base + (size_t)u * 256 + tid;
                if (e < elements) record[e] = S[u];
                S[u] = keep * S[u] + take * sums[d][u];
            }
            if (MODE == GATED && first_block) {
                if (tid < dim) {
                    record[elements + tid] = n;
                    n = keep * n + take * sum_n[d];
                }
                if (tid == 0) record[record_floats - 2] = m;
            }
            m = m_new;
        }
    }
#pragma unroll
    for (int u = 0; u < PER; u++) {
        const size_t e = base + (size_t)u * 256 + tid;
        if (e < elements) S_at[e] = S[u];
    }
    if (MODE == GATED && first_block) {
        if (tid < dim) mine[n_at + (size_t)head * dim + tid] = n;
        if (tid == 0) mine[m_at + head] = m;
    }
}

template <int L, int MODE>
__global__ __launch_bounds__(CHUNK_THREADS) void chunk_output_kernel(const float* __restrict__ q, int q_stride, const float* __restrict__ k, int k_stride,
                                                                     const float* __restrict__ v, int v_stride, const float* __restrict__ gate_in,
                                                                     const float* __restrict__ gate_forget, int gate_stride, float cap,
                                                                     const float* __restrict__ decay, float q_scale, const int* __restrict__ q_starts,
                                                                     const int* __restrict__ state_slots, const float* __restrict__ scratch,
                                                                     float* __restrict__ out, int out_stride, int dim, int vdim, int tiles) {
    constexpr int DIM_MAX = ChunkShape<L>::DIM_MAX, RPW = ChunkShape<L>::RPW;
    __shared__ __align__(16) float Qs[L][DIM_MAX];
    __shared__ float Kt[DIM_MAX][L];       // transposed; once the scores are taken, its first L rows hold them: A[t][s]
    __shared__ float Vs[L][CHUNK_VT];
    __shared__ double b_of[L];
    __shared__ double m_of[L];
    __shared__ float take_of[L], start_weight[L], nq_of[L];
    const int request = blockIdx.x, head = blockIdx.y, n_heads = gridDim.y, chunk = blockIdx.z / tiles, tile = blockIdx.z % tiles;
    const int first_row = q_starts[request], rows = q_starts[request + 1] - first_row;
    if (state_slots[request] < 0 || chunk * L >= rows) return;
    const int n_valid = min(L, rows - chunk * L), chunk_first = first_row + chunk * L;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const size_t elements = (size_t)dim * vdim, record_floats = elements + dim + 4;
    const float* record = scratch + (chunk_record(chunk_first, L, request) * n_heads + head) * record_floats;

    for (int e = tid; e < L * dim; e += CHUNK_THREADS) {
        const int s = e / dim, i = e % dim;
        float qv = 0.0f, kv = 0.0f;
        if (s < n_valid) {
            qv = q[(size_t)(chunk_first + s) * q_stride + head * dim + i];
            kv = k[(size_t)(chunk_first + s) * k_stride + head * dim + i];
            if (MODE == DECAYED) qv = silu_f(qv), kv = silu_f(kv);
            qv *= q_scale;
        }
        Qs[s][i] = qv;
        Kt[i][s] = kv;
    }
    for (int e = tid; e < L * CHUNK_VT; e += CHUNK_THREADS) {
        const int s = e / CHUNK_VT, c = tile * CHUNK_VT + e % CHUNK_VT;
        float value = 0.0f;
        if (s < n_valid && c < vdim) {
            value = v[(size_t)(chunk_first + s) * v_stride + head * vdim + c];
            if (MODE == DECAYED) value = silu_f(value);
        }
        Vs[s][e % CHUNK_VT] = value;
    }
    if (wave == 0) {
        float log_keep = 0.0f, log_take = 0.0f;
        if (lane < n_valid) row_gates<MODE>(gate_in, gate_forget, gate_stride, cap, MODE == DECAYED ? logf(decay[head]) : 0.0f, (size_t)(chunk_first + lane), head, log_keep, log_take);
        const double b = lanes_prefix_sum((double)log_keep, lane);
        double m_row = 0.0, from_start = b;
        if (MODE == GATED) {
            const double m_start = (double)record[record_floats - 2];
            const double best = lanes_prefix_max(lane < n_valid ? (double)log_take - b : -INFINITY, lane);
            m_row = b + fmax(m_start, best);
            from_start = b + m_start - m_row;
        }
        if (lane < L) {
            b_of[lane] = b;
            m_of[lane] = m_row;
            take_of[lane] = log_take;
            start_weight[lane] = expf((float)from_start);
        }
    }
    __syncthreads();
    // ---- scores: a lane a key s, a wave every eighth query t ----
    float a[RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) a[r] = 0.0f;
    if (lane < L) {
        for (int i = 0; i < dim; i += 4) {
            const float k0 = Kt[i][lane], k1 = Kt[i + 1][lane], k2 = Kt[i + 2][lane], k3 = Kt[i + 3][lane];
#pragma unroll
            for (int r = 0; r < RPW; r++) {
                const f32x4 qq = *reinterpret_cast<const f32x4*>(&Qs[wave + r * CHUNK_WAVES][i]);
                a[r] += qq[0] * k0 + qq[1] * k1 + qq[2] * k2 + qq[3] * k3;
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; r++) {
            const int t = wave + r * CHUNK_WAVES;
            const bool sees = lane <= t && t < n_valid;
            a[r] = sees ? a[r] * expf((float)((b_of[t] - b_of[lane]) + (double)take_of[lane] - m_of[t])) : 0.0f;
        }
    }
    __syncthreads();   // everybody has read the keys
    float (*A)[L] = Kt;
    const float* n_start = record + elements;
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const int t = wave + r * CHUNK_WAVES;
        if (lane < L) A[t][lane] = a[r];
        if (MODE == GATED) {
            float with_start = 0.0f;
            for (int i = lane; i < dim; i += WAVE) with_start += Qs[t][i] * n_start[i];
            const float nq = wave_sum(lane < L ? a[r] : 0.0f) + start_weight[t] * wave_sum(with_start);
            if (lane == 0) nq_of[t] = nq;
        }
    }
    __syncthreads();
    // ---- outputs: a lane a column of the tile, a wave every eighth row ----
    const int j = tile * CHUNK_VT + lane;
    const int column = min(j, vdim - 1);
    float inside[RPW], before[RPW];
#pragma unroll
    for (int r = 0; r < RPW; r++) inside[r] = before[r] = 0.0f;
    for (int s = 0; s < n_valid; s++) {
        const float vv = Vs[s][lane];
#pragma unroll
        for (int r = 0; r < RPW; r++) inside[r] += A[wave + r * CHUNK_WAVES][s] * vv;
    }
    for (int i = 0; i < dim; i++) {
        const float sv = record[(size_t)i * vdim + column];
#pragma unroll
        for (int r = 0; r < RPW; r++) before[r] += Qs[wave + r * CHUNK_WAVES][i] * sv;
    }
#pragma unroll
    for (int r = 0; r < RPW; r++) {
        const int t = wave + r * CHUNK_WAVES;
        if (t >= n_valid || j >= vdim) continue;
        float value = inside[r] + start_weight[t] * before[r];
        if (MODE == GATED) value /= fmaxf(fabsf(nq_of[t]), expf((float)-m_of[t])) + 1e-6f;
        out[(size_t)(chunk_first + t) * out_stride + head * vdim + j] = value;
    }
}

// The same two kernels for chunks of 64 rows (heads up to 64 wide) with their products on the matrix cores, in 32-bit
// (v_mfma_f32_32x32x2_f32: the first operand's lane holds row l % 32 and k = l / 32, the second's column l % 32 and k = l / 32; a
// lane's sixteen sums are rows 8 (v / 4) + 4 (l / 32) + v % 4 of column l % 32). Operands lie in LDS so that a lane's row or column
// is a lane's bank: q and k transposed ([i][t], rows of 65), v and the weighted keys as they come.
constexpr int CHUNK_PAD = 65;

template <int MODE>
__global__ __launch_bounds__(CHUNK_THREADS) void chunk_sums_mfma_kernel(const float* __restrict__ k, int k_stride, const float* __restrict__ v, int v_stride,
                                                                        const float* __restrict__ gate_in, const float* __restrict__ gate_forget,
                                                                        int gate_stride, float cap, const float* __restrict__ decay,
                                                                        const int* __restrict__ q_starts, const int* __restrict__ state_slots,
                                                                        float* __restrict__ scratch, int dim, int vdim, int tiles) {
    constexpr int L = 64;
    __shared__ float Ks[L][64];          // [s][i], already times the row's weight
    __shared__ float Vs[L][CHUNK_VT];
    __shared__ float weight[L];
    const int request = blockIdx.x, head = blockIdx.y, n_heads = gridDim.y, chunk = blockIdx.z / tiles, tile = blockIdx.z % tiles;
    const int first_row = q_starts[request], rows = q_starts[request + 1] - first_row;
    if (state_slots[request] < 0 || chunk * L >= rows) return;
    const int n_valid = min(L, rows - chunk * L), chunk_first = first_row + chunk * L;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const size_t record_floats = (size_t)dim * vdim + dim + 4;
    float* record = scratch + (chunk_record(chunk_first, L, request) * n_heads + head) * record_floats;

    // a thread's eight elements of k and of v (column tid % 64 of rows tid / 64 + 8 u) are asked for at once, from clamped places,
    // before the first wave settles the gates: one wait for memory
    constexpr int PER = L * 64 / CHUNK_THREADS;
    const int my_column = tid % 64, my_row = tid / 64;
    float k_mine[PER], v_mine[PER];
#pragma unroll
    for (int u = 0; u < PER; u++) {
        const size_t row = (size_t)(chunk_first + min(my_row + u * (CHUNK_THREADS / 64), n_valid - 1));
        k_mine[u] = k[row * k_stride + head * dim + min(my_column, dim - 1)];
        v_mine[u] = v[row * v_stride + head * vdim + min(tile * CHUNK_VT + my_column, vdim - 1)];
    }
    if (wave == 0) {
        float log_keep = 0.0f, log_take = 0.0f;
        if (lane < n_valid) row_gates<MODE>(gate_in, gate_forget, gate_stride, cap, MODE == DECAYED ? logf(decay[head]) : 0.0f, (size_t)(chunk_first + lane), head, log_keep, log_take);
        const double b = lanes_prefix_sum((double)log_keep, lane);
        const double total = __shfl(b, n_valid - 1, WAVE);
        const double reach = lane < n_valid ? (total - b) + (double)log_take : -INFINITY;
        const float mu = MODE == GATED ? wave_max((float)reach) : 0.0f;
        weight[lane] = lane < n_valid ? expf((float)(reach - (double)mu)) : 0.0f;
        if (lane == 0 && tile == 0) {
            record[record_floats - 4] = (float)total;
            record[record_floats - 3] = mu;
        }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < PER; u++) {
        const int s = my_row + u * (CHUNK_THREADS / 64);
        float kv = k_mine[u], vv = v_mine[u];
        if (MODE == DECAYED) kv = silu_f(kv), vv = silu_f(vv);
        Ks[s][my_column] = s < n_valid && my_column < dim ? kv * weight[s] : 0.0f;
        Vs[s][my_column] = s < n_valid && tile * CHUNK_VT + my_column < vdim ? vv : 0.0f;
    }
    __syncthreads();
    const int half = lane / 32, l32 = lane % 32;
    if (wave < 4 && (wave / 2) * 32 < dim) {   // U = (weighted K)^T V: a wave a tile of 32 rows i x 32 columns j
        const int ib = wave / 2, jb = wave % 2;
        f32x16 acc;
#pragma unroll
        for (int u = 0; u < 16; u++) acc[u] = 0.0f;
        const int s_end = (n_valid + 1) & ~1;
        for (int s = 0; s < s_end; s += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(Ks[s + half][ib * 32 + l32], Vs[s + half][jb * 32 + l32], acc, 0, 0, 0);
        const int j = tile * CHUNK_VT + jb * 32 + l32;
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const int i = ib * 32 + 8 * (u / 4) + 4 * half + (u % 4);
            if (i < dim && j < vdim) record[(size_t)i * vdim + j] = acc[u];
        }
    }
    if (MODE == GATED && tile == 0 && wave >= 4 && tid - 4 * WAVE < dim) {   // the chunk's share of n
        const int i = tid - 4 * WAVE;
        float sum = 0.0f;
        for (int s = 0; s < n_valid; s++) sum += Ks[s][i];
        record[(size_t)dim * vdim + i] = sum;
    }
}

template <int MODE>
__global__ __launch_bounds__(CHUNK_THREADS) void chunk_output_mfma_kernel(const float* __restrict__ q, int q_stride, const float* __restrict__ k, int k_stride,
                                                                          const float* __restrict__ v, int v_stride, const float* __restrict__ gate_in,
                                                                          const float* __restrict__ gate_forget, int gate_stride, float cap,
                                                                          const float* __restrict__ decay, float q_scale, const int* __restrict__ q_starts,
                                                                          const int* __restrict__ state_slots, const float* __restrict__ scratch,
                                                                          float* __restrict__ out, int out_stride, int dim, int vdim, int tiles) {
    constexpr int L = 64, PAD = CHUNK_PAD;
    __shared__ float Qt[64 * PAD];        // [i][t]; behind the products: the outputs [t][j]
    __shared__ float Kt[64 * PAD];        // [i][s]; behind the scores: the weighted scores [s][t]
    __shared__ float Vs[L][CHUNK_VT];     // [s][j]
    __shared__ double b_of[L];
    __shared__ double m_of[L];
    __shared__ float take_of[L], start_weight[L], nq_inside[2][L], nq_before[L];
    const int request = blockIdx.x, head = blockIdx.y, n_heads = gridDim.y, chunk = blockIdx.z / tiles, tile = blockIdx.z % tiles;
    const int first_row = q_starts[request], rows = q_starts[request + 1] - first_row;
    if (state_slots[request] < 0 || chunk * L >= rows) return;
    const int n_valid = min(L, rows - chunk * L), chunk_first = first_row + chunk * L;
    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int half = lane / 32, l32 = lane % 32;
    const size_t elements = (size_t)dim * vdim, record_floats = elements + dim + 4;
    const float* record = scratch + (chunk_record(chunk_first, L, request) * n_heads + head) * record_floats;

    {   // a thread's eight elements of q, k and v (column tid % 64 of rows tid / 64 + 8 u), asked for at once from clamped places
        constexpr int PER = L * 64 / CHUNK_THREADS;
        const int my_column = tid % 64, my_row = tid / 64;
        float q_mine[PER], k_mine[PER], v_mine[PER];
#pragma unroll
        for (int u = 0; u < PER; u++) {
            const size_t row = (size_t)(chunk_first + min(my_row + u * (CHUNK_THREADS / 64), n_valid - 1));
            q_mine[u] = q[row * q_stride + head * dim + min(my_column, dim - 1)];
            k_mine[u] = k[row * k_stride + head * dim + min(my_column, dim - 1)];
            v_mine[u] = v[row * v_stride + head * vdim + min(tile * CHUNK_VT + my_column, vdim - 1)];
        }
#pragma unroll
        for (int u = 0; u < PER; u++) {
            const int s = my_row + u * (CHUNK_THREADS / 64);
            float qv = q_mine[u], kv = k_mine[u], vv = v_mine[u];
            if (MODE == DECAYED) qv = silu_f(qv), kv = silu_f(kv), vv = silu_f(vv);
            const bool row_counts = s < n_valid;
            if (my_column < dim) {
                Qt[my_column * PAD + s] = row_counts ? qv * q_scale : 0.0f;
                Kt[my_column * PAD + s] = row_counts ? kv : 0.0f;
            }
            Vs[s][my_column] = row_counts && tile * CHUNK_VT + my_column < vdim ? vv : 0.0f;
        }
    }
    if (wave == 0) {
        float log_keep = 0.0f, log_take = 0.0f;
        if (lane < n_valid) row_gates<MODE>(gate_in, gate_forget, gate_stride, cap, MODE == DECAYED ? logf(decay[head]) : 0.0f, (size_t)(chunk_first + lane), head, log_keep, log_take);
        const double b = lanes_prefix_sum((double)log_keep, lane);
        double m_row = 0.0, from_start = b;
        if (MODE == GATED) {
            const double m_start = (double)record[record_floats - 2];
            const double best = lanes_prefix_max(lane < n_valid ? (double)log_take - b : -INFINITY, lane);
            m_row = b + fmax(m_start, best);
            from_start = b + m_start - m_row;
        }
        b_of[lane] = b;
        m_of[lane] = m_row;
        take_of[lane] = log_take;
        start_weight[lane] = expf((float)from_start);
    }
    __syncthreads();
    // ---- scores, transposed: rows the keys s, columns the queries t; the three tiles that hold a visible pair, a wave each ----
    f32x16 acc;
#pragma unroll
    for (int u = 0; u < 16; u++) acc[u] = 0.0f;
    const int key_block = wave == 2 ? 1 : 0, query_block = wave == 0 ? 0 : 1;
    if (wave < 3) {
        for (int i = 0; i < dim; i += 2)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(Kt[(i + half) * PAD + key_block * 32 + l32], Qt[(i + half) * PAD + query_block * 32 + l32], acc, 0, 0, 0);
        const int t = query_block * 32 + l32;
        float column_sum = 0.0f;
#pragma unroll
        for (int u = 0; u < 16; u++) {
            const int s = key_block * 32 + 8 * (u / 4) + 4 * half + (u % 4);
            const bool sees = s <= t && t < n_valid;
            acc[u] = sees ? acc[u] * expf((float)((b_of[t] - b_of[s]) + (double)take_of[s] - m_of[t])) : 0.0f;
            column_sum += acc[u];
        }
        column_sum += __shfl_xor(column_sum, 32, WAVE);
        if (half == 0) nq_inside[key_block][t] = column_sum;
    } else if (wave == 3) {
        if (lane < 32) nq_inside[1][lane] = 0.0f;   // no key of the second block is seen by a query of the first
    } else if (wave == 4 && MODE == GATED) {
        const float* n_start = record + elements;
        float sum = 0.0f;
        for (int i = 0; i < dim; i++) sum += Qt[i * PAD + lane] * n_start[i];
        nq_before[lane] = sum;
    }
    __syncthreads();   // everybody has read the keys
    float* At = Kt;    // [s][t]
    if (wave < 3) {
#pragma unroll
        for (int u = 0; u < 16; u++) At[(key_block * 32 + 8 * (u / 4) + 4 * half + (u % 4)) * PAD + query_block * 32 + l32] = acc[u];
    } else if (wave == 3) {
#pragma unroll
        for (int u = 0; u < 16; u++) At[(32 + 8 * (u / 4) + 4 * half + (u % 4)) * PAD + l32] = 0.0f;
    }
    __syncthreads();
    // ---- outputs, transposed: rows the tile's columns j, columns the queries t; four tiles, a wave each ----
    float value[16];
    const int j_block = wave / 2, t_block = wave % 2;
    if (wave < 4) {
        f32x16 inside, before;
#pragma unroll
        for (int u = 0; u < 16; u++) inside[u] = before[u] = 0.0f;
        const int s_end = min(t_block == 0 ? 32 : 64, (n_valid + 1) & ~1);
        for (int s = 0; s < s_end; s += 2)
            inside = __builtin_amdgcn_mfma_f32_32x32x2f32(Vs[s + half][j_block * 32 + l32], At[(s + half) * PAD + t_block * 32 + l32], inside, 0, 0, 0);
        const int column = min(tile * CHUNK_VT + j_block * 32 + l32, vdim - 1);
        for (int i = 0; i < dim; i += 2)
            before = __builtin_amdgcn_mfma_f32_32x32x2f32(record[(size_t)(i + half) * vdim + column], Qt[(i + half) * PAD + t_block * 32 + l32], before, 0, 0, 0);
        const int t = t_block * 32 + l32;
        float divide = 1.0f;
        if (MODE == GATED) divide = 1.0f / (fmaxf(fabsf(nq_inside[0][t] + nq_inside[1][t] + start_weight[t] * nq_before[t]), expf((float)-m_of[t])) + 1e-6f);
#pragma unroll
        for (int u = 0; u < 16; u++) value[u] = (inside[u] + start_weight[t] * before[u]) * divide;
    }
    __syncthreads();   // everybody has read the queries
    float* Ot = Qt;    // [t][j]
    if (wave < 4) {
#pragma unroll
        for (int u = 0; u < 16; u++) Ot[(t_block * 32 + l32) * PAD + j_block * 32 + 8 * (u / 4) + 4 * half + (u % 4)] = value[u];
    }
    __syncthreads();
    for (int e = tid; e < n_valid * CHUNK_VT; e += CHUNK_THREADS) {
        const int t = e / CHUNK_VT, j = tile * CHUNK_VT + e % CHUNK_VT;
        if (j < vdim) out[(size_t)(chunk_first + t) * out_stride + head * vdim + j] = Ot[t * PAD + e % CHUNK_VT];
    }
}

int chunk_rows_for(int dim) { return dim <= 64 ? 64 : (dim <= 128 ? 32 : 16); }

}  // namespace

// The rows a chunk holds for heads of `dim` (0: the chunked kernels do not take such heads).
MLLM_API int mllm_recurrence_chunk_rows(int dim) { return dim >= 4 && dim <= 256 && dim % 4 == 0 ? chunk_rows_for(dim) : 0; }

// The same as mllm_recurrence for batches with long portions: max_rows is the longest portion of the batch (or a bound on it),
// scratch holds (n_rows / chunk rows + n_requests + 1) * n_heads * (dim * vdim + dim + 4) floats.
MLLM_API int mllm_recurrence_chunked(int kind, const float* q, int q_stride, const float* k, int k_stride, const float* v, int v_stride, const float* gate_in,
                                     const float* gate_forget, int gate_stride, float cap, const float* decay, float q_scale, float* state,
                                     long long state_stride, long long n_at, long long m_at, const int* q_starts, const int* state_slots, float* out,
                                     int out_stride, int n_requests, int n_heads, int dim, int vdim, int max_rows, float* scratch, long long scratch_floats,
                                     int n_rows, hipStream_t stream) {
    MLLM_REQUIRE(kind == GATED || kind == DECAYED, "recurrence_chunked: unknown kind %d", kind);
    MLLM_REQUIRE(n_requests >= 0 && n_heads > 0 && vdim > 0 && max_rows >= 0 && n_rows >= 0, "recurrence_chunked: bad sizes");
    MLLM_REQUIRE(mllm_recurrence_chunk_rows(dim) > 0, "recurrence_chunked: heads of %d are not taken (a multiple of 4 up to 256)", dim);
    MLLM_REQUIRE(q_stride >= n_heads * dim && k_stride >= n_heads * dim && v_stride >= n_heads * vdim && out_stride >= n_heads * vdim, "recurrence_chunked: rows are too short for the heads");
    MLLM_REQUIRE(q != nullptr && k != nullptr && v != nullptr && state != nullptr && q_starts != nullptr && state_slots != nullptr && out != nullptr && scratch != nullptr, "recurrence_chunked: a missing operand");
    const long long matrices = (long long)n_heads * dim * vdim;
    if (kind == GATED) {
        MLLM_REQUIRE(gate_in != nullptr && gate_forget != nullptr && gate_stride >= n_heads, "recurrence_chunked: the gates are missing");
        MLLM_REQUIRE(n_at >= matrices && m_at >= n_at + (long long)n_heads * dim && state_stride >= m_at + n_heads, "recurrence_chunked: the state's parts overlap");
    } else {
        MLLM_REQUIRE(decay != nullptr && state_stride >= matrices, "recurrence_chunked: the decays are missing or the state is too small");
    }
    const int L = chunk_rows_for(dim);
    MLLM_REQUIRE(scratch_floats >= ((long long)n_rows / L + n_requests + 1) * n_heads * ((long long)dim * vdim + dim + 4), "recurrence_chunked: the scratch memory is too small");
    if (n_requests == 0 || max_rows == 0) return 0;
    const int tiles = ceil_div(vdim, CHUNK_VT), chunks = ceil_div(max_rows, L);
    MLLM_REQUIRE((long long)chunks * tiles <= 65535, "recurrence_chunked: too many chunks for one launch");
    dim3 grid(n_requests, n_heads, chunks * tiles), scan_grid(n_requests, n_heads, ceil_div(dim * vdim, 4096));
#define CHUNKED(LL, MODE)                                                                                                                              \
    do {                                                                                                                                               \
        mllm_count_kernel(MLLM_K_RECURRENCE);                                                                                                          \
        chunk_sums_kernel<LL, MODE><<<grid, CHUNK_THREADS, 0, stream>>>(k, k_stride, v, v_stride, gate_in, gate_forget, gate_stride, cap, decay, q_starts, \
                                                                        state_slots, scratch, dim, vdim, tiles);                                       \
        mllm_count_kernel(MLLM_K_RECURRENCE);                                                                                                          \
        chunk_scan_kernel<MODE><<<scan_grid, 256, 0, stream>>>(q_starts, state_slots, scratch, state, state_stride, n_at, m_at, dim, vdim, LL);         \
        mllm_count_kernel(MLLM_K_RECURRENCE);                                                                                                          \
        chunk_output_kernel<LL, MODE><<<grid, CHUNK_THREADS, 0, stream>>>(q, q_stride, k, k_stride, v, v_stride, gate_in, gate_forget, gate_stride, cap, \
                                                                          decay, q_scale, q_starts, state_slots, scratch, out, out_stride, dim, vdim, tiles); \
    } while (0)
#define CHUNKED_MFMA(MODE)                                                                                                                         \
    do {                                                                                                                                           \
        mllm_count_kernel(MLLM_K_RECURRENCE);                                                                                                      \
        chunk_sums_mfma_kernel<MODE><<<grid, CHUNK_THREADS, 0, stream>>>(k, k_stride, v, v_stride, gate_in, gate_forget, gate_stride, cap, decay, q_starts, \
                                                                         state_slots, scratch, dim, vdim, tiles);                                  \
        mllm_count_kernel(MLLM_K_RECURRENCE);                                                                                                      \
        chunk_scan_kernel<MODE><<<scan_grid, 256, 0, stream>>>(q_starts, state_slots, scratch, state, state_stride, n_at, m_at, dim, vdim, 64);      \
        mllm_count_kernel(MLLM_K_RECURRENCE);                                                                                                      \
        chunk_output_mfma_kernel<MODE><<<grid, CHUNK_THREADS, 0, stream>>>(q, q_stride, k, k_stride, v, v_stride, gate_in, gate_forget, gate_stride, cap, \
                                                                           decay, q_scale, q_starts, state_slots, scratch, out, out_stride, dim, vdim, tiles); \
    } while (0)
    if (kind == GATED) {
        if (L == 64) CHUNKED_MFMA(GATED);
        else if (L == 32) CHUNKED(32, GATED);
        else CHUNKED(16, GATED);
    } else {
        if (L == 64) CHUNKED_MFMA(DECAYED);
        else if (L == 32) CHUNKED(32, DECAYED);
        else CHUNKED(16, DECAYED);
    }
#undef CHUNKED_MFMA
#undef CHUNKED
    return mllm_check_launch("recurrence_chunked");
}
