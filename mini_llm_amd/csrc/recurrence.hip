// Mixers that keep a matrix per head and request instead of keys and values: S_t = a_t S_(t-1) + b_t k_t v_t^T, o_t = S_t^T q_t.
// Two kinds share one kernel:
//   GATED (the matrix memory of an mLSTM): log gates i_t and f_t per head and token, a running maximum m that starts at 0,
//     m_t = max(f_t + m_(t-1), i_t), a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t); a vector n that follows the same
//     recurrence with k alone; o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6). The gates arrive as the sums of their
//     projections (bias included): i = cap tanh(raw / cap), f = logsigmoid(cap tanh(raw / cap)); cap <= 0: no cap.
//   DECAYED (a linear attention with a fixed decay per head): a_t = decay_h, b_t = 1, q, k and v pass through silu first.
// State, gates, sums and outputs are 32-bit. The state of a request lies in its slot: S [heads, dim, vdim], then (GATED)
// n [heads, dim] and m [heads].
//
// A block takes one (request, head, tile of VT value columns) and walks the request's rows of this step in order. Thread
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
    const int request = blockIdx.x, head = blockIdx.y, n_heads = gridDim.y;
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
                    if (tid == 0) {
                        keep[t] = expf(ft + m - m_new);
                        take[t] = expf(it - m_new);
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
    (void)n_heads;
}

struct Plan {
    int R, P, VT, TB, threads, tiles;
    size_t lds_bytes;
};

// How a head of dim x vdim is laid over a block: tiles of up to 64 value columns, as many parts along dim as 512 threads
// allow, a power of two of rows of S a thread.
bool plan_for(int dim, int vdim, Plan& plan) {
    plan.VT = vdim <= 64 ? vdim : 64;
    plan.tiles = ceil_div(vdim, plan.VT);
    int most_parts = 512 / plan.VT;
    if (most_parts > dim) most_parts = dim;
    if (most_parts < 1) most_parts = 1;
    plan.R = 1;
    while (plan.R * most_parts < dim) plan.R *= 2;
    if (plan.R > 32) return false;
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
        default: LAUNCH(32); break;
    }
#undef LAUNCH
#undef RECURRENCE_ARGS
    return mllm_check_launch("recurrence");
}
