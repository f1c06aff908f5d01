// Row-wise kernels of mixers that norm a whole projection, rotate neighbouring pairs, blend their values with an earlier
// layer's, run a short convolution over time with the last inputs kept per request, or gate and norm what a recurrence
// leaves. Everything is computed in 32-bit; the rows these kernels read (the sums of a fused product) are 32-bit too.
#include "common.h"

namespace {

__device__ __forceinline__ float block_sum(float v, float* scratch) {
    // every thread gets the sum over the block (blockDim a multiple of 64, at most 16 waves); scratch: 16 floats of LDS
    v = wave_sum(v);
    const int wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    __syncthreads();   // whoever still reads scratch from a call before
    if (threadIdx.x % WAVE == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < n_waves; w++) total += scratch[w];
    return total;
}

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

// A block per row. Queries [n_heads * dim] and keys [n_kv_heads * dim] are each RMS-normed over the WHOLE projection (all
// heads at once) with a gain vector of that length (null: the projection goes on as it is), then the first rot_dims
// elements of every head are rotated, element 2i with element 2i+1, by position * frequencies[i] (64-bit). Queries go to q_out
// [rows, n_heads * head_size]; keys to the key pages; values [n_kv_heads * vdim], blended with another layer's values of
// the same row where v_other is given (v <- (1 - mix) v + mix v_other, mix read from the device), to the value pages. The
// pages' heads hold head_size >= dim, vdim elements, zeros beyond a head's own. A negative slot stores nothing.
template <typename T>
__global__ __launch_bounds__(256) void projection_rows_kernel(const float* __restrict__ q, int q_stride, const float* __restrict__ k, int k_stride,
                                                              const float* __restrict__ v, int v_stride, const float* __restrict__ v_other,
                                                              int v_other_stride, const float* __restrict__ mix, const float* __restrict__ q_gain,
                                                              const float* __restrict__ k_gain, float eps, const double* __restrict__ frequencies,
                                                              int rot_dims, const int* __restrict__ positions, const int* __restrict__ slots,
                                                              T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages, int n_heads,
                                                              int n_kv_heads, int dim, int vdim, int head_size, int page_size, int write_cache) {
    __shared__ float scratch[2][16];
    const int row = blockIdx.x;
    const float* q_row = q + (size_t)row * q_stride;
    const float* k_row = k + (size_t)row * k_stride;
    const int q_width = n_heads * dim, k_width = n_kv_heads * dim;
    // the row's position and slot are asked for together with its first elements, and both sums of squares settle in one exchange
    const int position_of_row = positions[row];
    const int slot = write_cache ? slots[row] : -1;
    const float blend = v_other ? mix[0] : 0.0f;
    float q_squares = 0.0f, k_squares = 0.0f;
    if (q_gain)
        for (int i = threadIdx.x; i < q_width; i += blockDim.x) q_squares += q_row[i] * q_row[i];
    if (k_gain)
        for (int i = threadIdx.x; i < k_width; i += blockDim.x) k_squares += k_row[i] * k_row[i];
    q_squares = wave_sum(q_squares);
    k_squares = wave_sum(k_squares);
    if (threadIdx.x % WAVE == 0) {
        scratch[0][threadIdx.x / WAVE] = q_squares;
        scratch[1][threadIdx.x / WAVE] = k_squares;
    }
    __syncthreads();
    q_squares = k_squares = 0.0f;
    for (int w = 0; w < (int)blockDim.x / WAVE; w++) {
        q_squares += scratch[0][w];
        k_squares += scratch[1][w];
    }
    const float q_factor = q_gain ? 1.0f / sqrtf(q_squares / (float)q_width + eps) : 1.0f;
    const float k_factor = k_gain ? 1.0f / sqrtf(k_squares / (float)k_width + eps) : 1.0f;
    const double position = (double)position_of_row;
    // a pair of neighbouring elements of a normed head, rotated where it lies among the first rot_dims: d its first element's place
    // in the head (even), `at` the head's first element in the row; elements beyond the head's own are zero
    auto turned_pair = [&](const float* in, const float* gain, float factor, int at, int d, float& first, float& second) {
        first = d < dim ? in[at + d] * factor * (gain ? gain[at + d] : 1.0f) : 0.0f;
        second = d + 1 < dim ? in[at + d + 1] * factor * (gain ? gain[at + d + 1] : 1.0f) : 0.0f;
        if (d < rot_dims) {
            // the angle in 64-bit (a 32-bit product of a position in the thousands is good to 1e-4 only), brought into -pi .. pi,
            // where its sine and cosine are taken in 32-bit
            const double angle = position * frequencies[d >> 1];
            const double turns = rint(angle * 0.15915494309189535);
            float s, c;
            sincosf((float)(angle - turns * 6.283185307179586), &s, &c);
            const float u = first, w = second;
            first = u * c - w * s;
            second = w * c + u * s;
        }
    };
    const int half_head = head_size / 2;   // (heads in pages are multiples of 16 wide)
    for (int i = threadIdx.x; i < n_heads * half_head; i += blockDim.x) {
        const int head = i / half_head, d = 2 * (i % half_head);
        float first, second;
        turned_pair(q_row, q_gain, q_factor, head * dim, d, first, second);
        T* to = q_out + (size_t)row * n_heads * head_size + (size_t)head * head_size + d;
        to[0] = from_float<T>(first);
        to[1] = from_float<T>(second);
    }
    if (slot < 0) return;   // no cache write, or a padding row
    const int page = slot / page_size, offset = slot % page_size;
    for (int i = threadIdx.x; i < n_kv_heads * half_head; i += blockDim.x) {
        const int head = i / half_head, d = 2 * (i % half_head);
        const size_t at = (((size_t)page * n_kv_heads + head) * page_size + offset) * head_size + d;
        float first, second;
        turned_pair(k_row, k_gain, k_factor, head * dim, d, first, second);
        k_pages[at] = from_float<T>(first);
        k_pages[at + 1] = from_float<T>(second);
#pragma unroll
        for (int e = 0; e < 2; e++) {
            float value = 0.0f;
            if (d + e < vdim) {
                value = v[(size_t)row * v_stride + head * vdim + d + e];
                if (v_other) value = (1.0f - blend) * value + blend * v_other[(size_t)row * v_other_stride + head * vdim + d + e];
            }
            v_pages[at + e] = from_float<T>(value);
        }
    }
}

// out[row, h, :] = x[row, h, :] * sigmoid(gate[row, h]) * scale: one gate per head of head_size elements.
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(const T* __restrict__ x, int x_stride, const float* __restrict__ gate, int gate_stride,
                                                        float scale, T* __restrict__ out, int out_stride, int n_rows, int n_heads, int head_size) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int width = n_heads * head_size;
    if (i >= (long long)n_rows * width) return;
    const int row = (int)(i / width), col = (int)(i % width);
    const float g = sigmoid_f(gate[(size_t)row * gate_stride + col / head_size]) * scale;
    out[(size_t)row * out_stride + col] = from_float<T>(to_float(x[(size_t)row * x_stride + col]) * g);
}

// A wave per (row, group of `group` neighbouring elements): out = x / sqrt(mean over the group of x^2 + eps) * weight *
// sigmoid(gate) * scale. weight [width] and gate [rows, width] may each be null.
template <typename T>
__global__ __launch_bounds__(256) void gated_norm_kernel(const float* __restrict__ x, int x_stride, const float* __restrict__ weight,
                                                         const float* __restrict__ gate, int gate_stride, float eps, float scale,
                                                         T* __restrict__ out, int out_stride, int n_rows, int width, int group) {
    const int lane = threadIdx.x % WAVE;
    const int groups = width / group;
    const long long item = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (item >= (long long)n_rows * groups) return;
    const int row = (int)(item / groups), first = (int)(item % groups) * group;
    const float* in = x + (size_t)row * x_stride + first;
    if (group <= 4 * WAVE) {
        // everything the wave needs asked for at once, so that it waits for memory once
        float xs[4], ws[4], gs[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int d = min(lane + r * WAVE, group - 1);
            xs[r] = in[d];
            ws[r] = weight ? weight[first + d] : 1.0f;
            gs[r] = gate ? gate[(size_t)row * gate_stride + first + d] : 0.0f;
        }
        float squares = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; r++) squares += lane + r * WAVE < group ? xs[r] * xs[r] : 0.0f;
        const float factor = scale / sqrtf(wave_sum(squares) / (float)group + eps);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int d = lane + r * WAVE;
            if (d < group) out[(size_t)row * out_stride + first + d] = from_float<T>(xs[r] * factor * ws[r] * (gate ? sigmoid_f(gs[r]) : 1.0f));
        }
        return;
    }
    float squares = 0.0f;
    for (int d = lane; d < group; d += WAVE) squares += in[d] * in[d];
    const float factor = scale / sqrtf(wave_sum(squares) / (float)group + eps);
    for (int d = lane; d < group; d += WAVE) {
        float value = in[d] * factor;
        if (weight) value *= weight[first + d];
        if (gate) value *= sigmoid_f(gate[(size_t)row * gate_stride + first + d]);
        out[(size_t)row * out_stride + first + d] = from_float<T>(value);
    }
}

// The same for wide groups, a block per (row, group): up to eight elements a thread stay in registers between the sum of squares
// and the output, asked for at once with their gains and gates; wider groups are read again.
template <typename T>
__global__ __launch_bounds__(256) void gated_norm_wide_kernel(const float* __restrict__ x, int x_stride, const float* __restrict__ weight,
                                                              const float* __restrict__ gate, int gate_stride, float eps, float scale,
                                                              T* __restrict__ out, int out_stride, int width, int group) {
    __shared__ float scratch[16];
    const int groups = width / group;
    const int row = blockIdx.x / groups, first = (blockIdx.x % groups) * group;
    const float* in = x + (size_t)row * x_stride + first;
    constexpr int REGS = 8;
    if (group <= REGS * 256) {
        float xs[REGS], ws[REGS], gs[REGS];
#pragma unroll
        for (int r = 0; r < REGS; r++) {
            const int d = min((int)threadIdx.x + r * 256, group - 1);
            xs[r] = in[d];
            ws[r] = weight ? weight[first + d] : 1.0f;
            gs[r] = gate ? gate[(size_t)row * gate_stride + first + d] : 0.0f;
        }
        float squares = 0.0f;
#pragma unroll
        for (int r = 0; r < REGS; r++) squares += (int)threadIdx.x + r * 256 < group ? xs[r] * xs[r] : 0.0f;
        const float factor = scale / sqrtf(block_sum(squares, scratch) / (float)group + eps);
#pragma unroll
        for (int r = 0; r < REGS; r++) {
            const int d = threadIdx.x + r * 256;
            if (d < group) out[(size_t)row * out_stride + first + d] = from_float<T>(xs[r] * factor * ws[r] * (gate ? sigmoid_f(gs[r]) : 1.0f));
        }
        return;
    }
    float squares = 0.0f;
    for (int d = threadIdx.x; d < group; d += 256) squares += in[d] * in[d];
    const float factor = scale / sqrtf(block_sum(squares, scratch) / (float)group + eps);
    for (int d = threadIdx.x; d < group; d += 256) {
        float value = in[d] * factor;
        if (weight) value *= weight[first + d];
        if (gate) value *= sigmoid_f(gate[(size_t)row * gate_stride + first + d]);
        out[(size_t)row * out_stride + first + d] = from_float<T>(value);
    }
}

// A short causal convolution over time on every channel: y_t = sum_j w[c, j] u_(t - taps + 1 + j). The inputs before a
// portion's first row come from the request's kept inputs, `kept` [slots, kept_stride] holding [taps - 1, channels] in the
// order of time (zeros at a sequence's start). A thread per (row, channel).
__global__ __launch_bounds__(256) void short_conv_kernel(const float* __restrict__ u, int u_stride, const float* __restrict__ w, int taps,
                                                         const float* __restrict__ kept, long long kept_stride,
                                                         const int* __restrict__ token_request, const int* __restrict__ q_starts,
                                                         const int* __restrict__ state_slots, float* __restrict__ y, int y_stride, int n_rows,
                                                         int channels) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long long)n_rows * channels) return;
    const int row = (int)(i / channels), c = (int)(i % channels);
    const int request = token_request[row];
    if (request < 0) return;
    const int slot = state_slots[request];
    if (slot < 0) return;
    const int local = row - q_starts[request];
    const float* before = kept + (size_t)slot * kept_stride;
    float sum = 0.0f;
    for (int j = 0; j < taps; j++) {
        const int at = local - taps + 1 + j;   // among the portion's rows; negative: so many inputs before it
        const float value = at >= 0 ? u[(size_t)(row - local + at) * u_stride + c] : before[(size_t)(taps - 1 + at) * channels + c];
        sum += w[(size_t)c * taps + j] * value;
    }
    y[(size_t)row * y_stride + c] = sum;
}

// Behind the convolution: each request's kept inputs become the last taps - 1 inputs of its sequence as it now stands. A
// thread per (request, channel) reads all it needs before it writes.
constexpr int MAX_TAPS = 16;
__global__ __launch_bounds__(256) void short_conv_keep_kernel(const float* __restrict__ u, int u_stride, int taps, float* __restrict__ kept,
                                                              long long kept_stride, const int* __restrict__ q_starts,
                                                              const int* __restrict__ state_slots, int n_requests, int channels) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long long)n_requests * channels) return;
    const int request = (int)(i / channels), c = (int)(i % channels);
    const int slot = state_slots[request];
    if (slot < 0) return;
    const int start = q_starts[request], rows = q_starts[request + 1] - start;
    if (rows <= 0) return;
    float* mine = kept + (size_t)slot * kept_stride;
    float next[MAX_TAPS];
    for (int s = 0; s < taps - 1; s++) {
        const int at = rows - (taps - 1) + s;
        next[s] = at >= 0 ? u[(size_t)(start + at) * u_stride + c] : mine[(size_t)(s + rows) * channels + c];
    }
    for (int s = 0; s < taps - 1; s++) mine[(size_t)s * channels + c] = next[s];
}

}  // namespace

MLLM_API int mllm_projection_rows(const float* q, int q_stride, const float* k, int k_stride, const float* v, int v_stride, const float* v_other,
                                  int v_other_stride, const float* mix, const float* q_gain, const float* k_gain, float eps,
                                  const double* frequencies, int rot_dims, const int* positions, const int* slots, void* q_out, void* k_pages,
                                  void* v_pages, int n_rows, int n_heads, int n_kv_heads, int dim, int vdim, int head_size, int page_size,
                                  int write_cache, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && n_kv_heads > 0 && dim > 0 && vdim > 0 && page_size > 0, "projection_rows: bad sizes");
    MLLM_REQUIRE(head_size >= dim && head_size >= vdim, "projection_rows: heads of %d do not hold %d / %d elements", head_size, dim, vdim);
    MLLM_REQUIRE(q_stride >= n_heads * dim && k_stride >= n_kv_heads * dim && v_stride >= n_kv_heads * vdim, "projection_rows: rows are too short for the heads");
    MLLM_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dim && (rot_dims == 0 || frequencies != nullptr), "projection_rows: the rotation does not fit the heads");
    MLLM_REQUIRE(q != nullptr && k != nullptr && v != nullptr && positions != nullptr && q_out != nullptr, "projection_rows: a missing operand");
    MLLM_REQUIRE(v_other == nullptr || (mix != nullptr && v_other_stride >= n_kv_heads * vdim), "projection_rows: blended values need their weight");
    MLLM_REQUIRE(!write_cache || (slots != nullptr && k_pages != nullptr && v_pages != nullptr), "projection_rows: a cache write needs slots and pages");
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_PROJECTION_ROWS);
#define PROJECTION_ARGS(T) q, q_stride, k, k_stride, v, v_stride, v_other, v_other_stride, mix, q_gain, k_gain, eps, frequencies, rot_dims, positions, slots, \
                           (T*)q_out, (T*)k_pages, (T*)v_pages, n_heads, n_kv_heads, dim, vdim, head_size, page_size, write_cache
    if (dtype == MLLM_F32) projection_rows_kernel<float><<<n_rows, 256, 0, stream>>>(PROJECTION_ARGS(float));
    else if (dtype == MLLM_BF16) projection_rows_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(PROJECTION_ARGS(bf16_t));
    else MLLM_REQUIRE(false, "projection_rows: unknown dtype %d", dtype);
#undef PROJECTION_ARGS
    return mllm_check_launch("projection_rows");
}

MLLM_API int mllm_head_gate(const void* x, int x_stride, const float* gate, int gate_stride, float scale, void* out, int out_stride, int n_rows,
                            int n_heads, int head_size, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_heads > 0 && head_size > 0, "head_gate: bad sizes");
    MLLM_REQUIRE(x_stride >= n_heads * head_size && out_stride >= n_heads * head_size && gate_stride >= n_heads, "head_gate: rows are too short for the heads");
    MLLM_REQUIRE(x != nullptr && gate != nullptr && out != nullptr, "head_gate: a missing operand");
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * n_heads * head_size;
    const int blocks = (int)((items + 255) / 256);
    mllm_count_kernel(MLLM_K_HEAD_GATE);
    if (dtype == MLLM_F32) head_gate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, x_stride, gate, gate_stride, scale, (float*)out, out_stride, n_rows, n_heads, head_size);
    else if (dtype == MLLM_BF16) head_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)x, x_stride, gate, gate_stride, scale, (bf16_t*)out, out_stride, n_rows, n_heads, head_size);
    else MLLM_REQUIRE(false, "head_gate: unknown dtype %d", dtype);
    return mllm_check_launch("head_gate");
}

MLLM_API int mllm_gated_norm(const float* x, int x_stride, const float* weight, const float* gate, int gate_stride, float eps, float scale, void* out,
                             int out_stride, int n_rows, int width, int group, int dtype, hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && width > 0 && group > 0 && width % group == 0, "gated_norm: %d elements do not divide into groups of %d", width, group);
    MLLM_REQUIRE(x_stride >= width && out_stride >= width && (gate == nullptr || gate_stride >= width), "gated_norm: rows are too short");
    MLLM_REQUIRE(x != nullptr && out != nullptr, "gated_norm: a missing operand");
    if (n_rows == 0) return 0;
    const long long items = (long long)n_rows * (width / group);
    const int blocks = (int)((items + 3) / 4);
    mllm_count_kernel(MLLM_K_GATED_NORM);
    if (group > 4 * WAVE) {   // wide groups: a block each
        MLLM_REQUIRE(items <= 0x7fffffffLL, "gated_norm: too many groups for one launch");
        if (dtype == MLLM_F32) gated_norm_wide_kernel<float><<<(int)items, 256, 0, stream>>>(x, x_stride, weight, gate, gate_stride, eps, scale, (float*)out, out_stride, width, group);
        else if (dtype == MLLM_BF16) gated_norm_wide_kernel<bf16_t><<<(int)items, 256, 0, stream>>>(x, x_stride, weight, gate, gate_stride, eps, scale, (bf16_t*)out, out_stride, width, group);
        else MLLM_REQUIRE(false, "gated_norm: unknown dtype %d", dtype);
        return mllm_check_launch("gated_norm");
    }
    if (dtype == MLLM_F32) gated_norm_kernel<float><<<blocks, 256, 0, stream>>>(x, x_stride, weight, gate, gate_stride, eps, scale, (float*)out, out_stride, n_rows, width, group);
    else if (dtype == MLLM_BF16) gated_norm_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, x_stride, weight, gate, gate_stride, eps, scale, (bf16_t*)out, out_stride, n_rows, width, group);
    else MLLM_REQUIRE(false, "gated_norm: unknown dtype %d", dtype);
    return mllm_check_launch("gated_norm");
}

// The convolution, then (keep != 0) the requests' kept inputs moved on; the two are separate launches because the first
// reads what the second overwrites.
MLLM_API int mllm_short_conv(const float* u, int u_stride, const float* w, int taps, float* kept, long long kept_stride, const int* token_request,
                             const int* q_starts, const int* state_slots, float* y, int y_stride, int n_rows, int n_requests, int channels, int keep,
                             hipStream_t stream) {
    MLLM_REQUIRE(n_rows >= 0 && n_requests >= 0 && channels > 0, "short_conv: bad sizes");
    MLLM_REQUIRE(taps >= 1 && taps <= MAX_TAPS, "short_conv: %d taps (1 to %d are taken)", taps, MAX_TAPS);
    MLLM_REQUIRE(u_stride >= channels && y_stride >= channels && kept_stride >= (long long)(taps - 1) * channels, "short_conv: rows are too short");
    MLLM_REQUIRE(u != nullptr && w != nullptr && y != nullptr && (taps == 1 || kept != nullptr) && token_request != nullptr && q_starts != nullptr && state_slots != nullptr,
                 "short_conv: a missing operand");
    if (n_rows == 0) return 0;
    mllm_count_kernel(MLLM_K_SHORT_CONV);
    short_conv_kernel<<<(int)(((long long)n_rows * channels + 255) / 256), 256, 0, stream>>>(u, u_stride, w, taps, kept, kept_stride, token_request, q_starts,
                                                                                           state_slots, y, y_stride, n_rows, channels);
    int status = mllm_check_launch("short_conv");
    if (status != 0 || !keep || taps == 1 || n_requests == 0) return status;
    mllm_count_kernel(MLLM_K_SHORT_CONV);
    short_conv_keep_kernel<<<(int)(((long long)n_requests * channels + 255) / 256), 256, 0, stream>>>(u, u_stride, taps, kept, kept_stride, q_starts, state_slots,
                                                                                                    n_requests, channels);
    return mllm_check_launch("short_conv_keep");
}
