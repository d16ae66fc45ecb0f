// An fp32 residual stream with ONE grouped RMS norm per layer, parallel sublayers and a normalised side input.
//
// nv_stream_boundary       per row, in place on the fp32 stream r:
//                              r <- r + mult * (a + sum_j p_j)                 (a in the matmul dtype, p_j fp32 parts,
//                                                                               e.g. the weighted outputs of the
//                                                                               chosen experts; either may be absent)
//                              r <- r + mult * n / sqrt(mean(n^2) + eps) * wn  (a sublayer output that is RMS-normed
//                                                                               on its way in; may be absent)
//                              c <- r in the matmul dtype                      (may be absent)
//                              y <- grouped RMS norm of r: the row is cut into `groups` equal consecutive parts, each
//                                   divided by its own sqrt(mean(part^2) + eps), the whole times w (may be absent;
//                                   written in fp32, in the matmul dtype, or both)
//                          so the stream is read and written once per boundary.  All statistics are fp32.
// nv_rms_norm_rows         y = x / sqrt(mean(x^2) + eps) * w over rows of the matmul dtype (fp32 arithmetic).
// nv_causal_conv_add       y[t, c] = x[t, c] + sum_j w[c, j] * x[t - taps + 1 + j, c] over time per channel on fp32
//                          inputs, the last taps-1 inputs of every sequence carried in fp32 in conv_state[slot]; a
//                          sequence whose rows start at position 0 ignores what its slot holds.
// nv_token_gate            y[t, j] = gelu_tanh(z[t, j]) * table[ids[t], offset + j].
#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kSbThreads = 256;

__device__ __forceinline__ float sb_block_sum(float x, float* red) {
    x = wave_sum(x);
    const int w = threadIdx.x >> 6;
    __syncthreads();                       // red may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) red[w] = x;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kSbThreads / 64; ++i) t += red[i];
    return t;
}

template <typename T>
__global__ __launch_bounds__(kSbThreads) void stream_boundary_kernel(
    float* __restrict__ resid, const T* __restrict__ add, int64_t add_stride, const float* __restrict__ parts,
    int n_parts, const T* __restrict__ normed, int64_t normed_stride, const float* __restrict__ normed_w, float mult,
    const float* __restrict__ norm_w, int groups, float eps, float* __restrict__ y32, T* __restrict__ y,
    T* __restrict__ copy, int cols) {
    extern __shared__ float row[];                 // [cols] the row, then [groups] 1 / rms of every part
    __shared__ float red[kSbThreads / 64];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    float* rrow = resid + r * cols;
    for (int c = tid; c < cols; c += kSbThreads) row[c] = rrow[c];
    bool changed = false;
    if (add != nullptr || parts != nullptr) {
        for (int c = tid; c < cols; c += kSbThreads) {
            float s = add != nullptr ? (float)add[r * add_stride + c] : 0.f;
            for (int j = 0; j < n_parts; ++j) s += parts[(r * n_parts + j) * cols + c];
            row[c] += mult * s;
        }
        changed = true;
    }
    if (normed != nullptr) {
        float ss = 0.f;
        for (int c = tid; c < cols; c += kSbThreads) {
            const float v = (float)normed[r * normed_stride + c];
            ss += v * v;
        }
        ss = sb_block_sum(ss, red);
        const float rstd = 1.0f / sqrtf(ss / (float)cols + eps);
        for (int c = tid; c < cols; c += kSbThreads)
            row[c] += mult * ((float)normed[r * normed_stride + c] * rstd * normed_w[c]);
        changed = true;
    }
    if (changed)
        for (int c = tid; c < cols; c += kSbThreads) rrow[c] = row[c];
    if (copy != nullptr)
        for (int c = tid; c < cols; c += kSbThreads) copy[r * cols + c] = (T)row[c];
    if (norm_w == nullptr) return;
    float* rg = row + cols;
    const int gs = cols / groups;
    __syncthreads();                               // the parts are summed by other threads than wrote the row
    if (groups <= 8) {
        for (int g = 0; g < groups; ++g) {
            float ss = 0.f;
            for (int c = tid; c < gs; c += kSbThreads) ss += row[g * gs + c] * row[g * gs + c];
            ss = sb_block_sum(ss, red);
            if (tid == 0) rg[g] = 1.0f / sqrtf(ss / (float)gs + eps);
        }
    } else {                                       // many short parts: one wave per part
        const int lane = tid & 63;
        for (int g = tid >> 6; g < groups; g += kSbThreads / 64) {
            float ss = 0.f;
            for (int c = lane; c < gs; c += 64) ss += row[g * gs + c] * row[g * gs + c];
            ss = wave_sum(ss);
            if (lane == 0) rg[g] = 1.0f / sqrtf(ss / (float)gs + eps);
        }
    }
    __syncthreads();
    for (int c = tid; c < cols; c += kSbThreads) {
        const float v = row[c] * rg[c / gs] * norm_w[c];
        if (y32 != nullptr) y32[r * cols + c] = v;
        if (y != nullptr) y[r * cols + c] = (T)v;
    }
}

template <typename T>
__global__ __launch_bounds__(kSbThreads) void rms_norm_rows_kernel(const T* __restrict__ x, int64_t x_stride,
                                                                   const float* __restrict__ w, T* __restrict__ y,
                                                                   int cols, float eps) {
    __shared__ float red[kSbThreads / 64];
    const int64_t r = blockIdx.x;
    float ss = 0.f;
    for (int c = threadIdx.x; c < cols; c += kSbThreads) {
        const float v = (float)x[r * x_stride + c];
        ss += v * v;
    }
    ss = sb_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)cols + eps);
    for (int c = threadIdx.x; c < cols; c += kSbThreads) y[r * cols + c] = (T)((float)x[r * x_stride + c] * rstd * w[c]);
}

__device__ __forceinline__ int seq_of_row(const int* cu_q, int B, int t) {
    int lo = 0, hi = B;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_add_kernel(
    const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ conv_state, T* __restrict__ y,
    const int* __restrict__ cu_q, const int* __restrict__ cu_k, const int* __restrict__ state_slots, int B, int C,
    int taps) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int b = seq_of_row(cu_q, B, t);
    const int i = t - cu_q[b];
    const int start = (cu_k[b + 1] - cu_k[b]) - (cu_q[b + 1] - cu_q[b]);
    const float* st = conv_state + (int64_t)state_slots[b] * (taps - 1) * C;
    const float cur = x[(int64_t)t * C + c];
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {               // j tokens back
        const int src = i - j;
        float xv = 0.f;
        if (j == 0) xv = cur;
        else if (src >= 0) xv = x[(int64_t)(t - j) * C + c];
        else if (start + src >= 0) xv = st[(int64_t)(taps - 1 + src) * C + c];
        acc += w[(int64_t)c * taps + (taps - 1 - j)] * xv;
    }
    y[(int64_t)t * C + c] = (T)(cur + acc);
}

// After the step: state row s holds the input at position len_k - (taps - 1) + s.  One thread per channel walks the
// rows upwards, so a row is read (s + len_q) before it is overwritten.
__global__ __launch_bounds__(256) void causal_conv_carry_kernel(const float* __restrict__ x, float* __restrict__ conv_state,
                                                                const int* __restrict__ cu_q, const int* __restrict__ cu_k,
                                                                const int* __restrict__ state_slots, int C, int taps) {
    const int b = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int q0 = cu_q[b], nq = cu_q[b + 1] - q0, nk = cu_k[b + 1] - cu_k[b];
    if (nq <= 0) return;
    const int keep = taps - 1, start = nk - nq;
    float* st = conv_state + (int64_t)state_slots[b] * keep * C;
    for (int s = 0; s < keep; ++s) {
        const int p = nk - keep + s;               // position this row holds afterwards
        float v = 0.f;
        if (p >= start) v = x[(int64_t)(q0 + p - start) * C + c];
        else if (p >= 0) v = st[(int64_t)(s + nq) * C + c];
        st[(int64_t)s * C + c] = v;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void token_gate_kernel(const T* __restrict__ z, int64_t z_stride,
                                                         const T* __restrict__ table, int64_t table_stride,
                                                         const int64_t* __restrict__ ids, int offset, int dim,
                                                         T* __restrict__ y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t t = i / dim;
    const int j = (int)(i - t * dim);
    const float v = (float)z[t * z_stride + j];
    const float g = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    y[i] = (T)(g * (float)table[ids[t] * table_stride + offset + j]);
}

}  // namespace nv

extern "C" int nv_stream_boundary(void* resid, const void* add, int64_t add_stride, const void* parts, int n_parts,
                                  const void* normed, int64_t normed_stride, const float* normed_w, float mult,
                                  const float* norm_w, int groups, float eps, void* y32, void* y, void* copy,
                                  int dtype, int64_t rows, int cols, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0 && cols <= 16384, NV_ERR_INVALID_ARG, "nv_stream_boundary: bad sizes");
    if (rows == 0) return NV_OK;
    NV_REQUIRE(resid, NV_ERR_INVALID_ARG, "nv_stream_boundary: null stream");
    NV_REQUIRE(!parts || n_parts > 0, NV_ERR_INVALID_ARG, "nv_stream_boundary: parts without a count");
    NV_REQUIRE(!normed || normed_w, NV_ERR_INVALID_ARG, "nv_stream_boundary: a normed input needs its weight");
    NV_REQUIRE(!norm_w || (groups >= 1 && groups <= 1024 && cols % groups == 0 && (y || y32)), NV_ERR_INVALID_ARG,
               "nv_stream_boundary: groups=%d must divide cols=%d (at most 1024), and the norm needs an output", groups, cols);
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_stream_boundary: bad dtype");
    NV_REQUIRE(rows < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_stream_boundary: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const size_t smem = sizeof(float) * ((size_t)cols + (norm_w ? groups : 0));
    const int np = parts ? n_parts : 0;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(stream_boundary_kernel<__bf16>, dim3((unsigned)rows), dim3(kSbThreads), smem, s, (float*)resid,
                           (const __bf16*)add, add_stride, (const float*)parts, np, (const __bf16*)normed, normed_stride,
                           normed_w, mult, norm_w, groups, eps, (float*)y32, (__bf16*)y, (__bf16*)copy, cols);
    else
        hipLaunchKernelGGL(stream_boundary_kernel<float>, dim3((unsigned)rows), dim3(kSbThreads), smem, s, (float*)resid,
                           (const float*)add, add_stride, (const float*)parts, np, (const float*)normed, normed_stride,
                           normed_w, mult, norm_w, groups, eps, (float*)y32, (float*)y, (float*)copy, cols);
    return check_launch("nv_stream_boundary");
}

extern "C" int nv_rms_norm_rows(const void* x, int64_t x_stride, const float* w, void* y, int dtype, int64_t rows,
                                int cols, float eps, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0, NV_ERR_INVALID_ARG, "nv_rms_norm_rows: bad sizes");
    if (rows == 0) return NV_OK;
    NV_REQUIRE(x && w && y, NV_ERR_INVALID_ARG, "nv_rms_norm_rows: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_rms_norm_rows: bad dtype");
    NV_REQUIRE(rows < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_rms_norm_rows: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(rms_norm_rows_kernel<__bf16>, dim3((unsigned)rows), dim3(kSbThreads), 0, s, (const __bf16*)x,
                           x_stride, w, (__bf16*)y, cols, eps);
    else
        hipLaunchKernelGGL(rms_norm_rows_kernel<float>, dim3((unsigned)rows), dim3(kSbThreads), 0, s, (const float*)x,
                           x_stride, w, (float*)y, cols, eps);
    return check_launch("nv_rms_norm_rows");
}

extern "C" int nv_causal_conv_add(const float* x, const float* w, float* conv_state, void* y, int y_dtype,
                                  const int* cu_seqlens_q, const int* cu_seqlens_k, const int* state_slots,
                                  int num_seqs, int64_t T, int C, int taps, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && T >= 0 && C > 0 && taps >= 1 && taps <= 64, NV_ERR_INVALID_ARG,
               "nv_causal_conv_add: bad sizes");
    if (T == 0 || num_seqs == 0) return NV_OK;
    NV_REQUIRE(x && w && y && cu_seqlens_q && cu_seqlens_k && state_slots && (conv_state || taps == 1),
               NV_ERR_INVALID_ARG, "nv_causal_conv_add: null pointer");
    NV_REQUIRE(y_dtype == NV_DTYPE_BF16 || y_dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_causal_conv_add: bad dtype");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_causal_conv_add: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const unsigned cb = (unsigned)((C + 255) / 256);
    if (y_dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(causal_conv_add_kernel<__bf16>, dim3((unsigned)T, cb), dim3(256), 0, s, x, w, conv_state,
                           (__bf16*)y, cu_seqlens_q, cu_seqlens_k, state_slots, num_seqs, C, taps);
    else
        hipLaunchKernelGGL(causal_conv_add_kernel<float>, dim3((unsigned)T, cb), dim3(256), 0, s, x, w, conv_state,
                           (float*)y, cu_seqlens_q, cu_seqlens_k, state_slots, num_seqs, C, taps);
    if (taps > 1)
        hipLaunchKernelGGL(causal_conv_carry_kernel, dim3((unsigned)num_seqs, cb), dim3(256), 0, s, x, conv_state,
                           cu_seqlens_q, cu_seqlens_k, state_slots, C, taps);
    return check_launch("nv_causal_conv_add");
}

extern "C" int nv_token_gate(const void* z, int64_t z_stride, const void* table, int64_t table_stride,
                             const int64_t* ids, int offset, int dim, void* y, int dtype, int64_t T, void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && dim > 0 && offset >= 0, NV_ERR_INVALID_ARG, "nv_token_gate: bad sizes");
    if (T == 0) return NV_OK;
    NV_REQUIRE(z && table && ids && y, NV_ERR_INVALID_ARG, "nv_token_gate: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_token_gate: bad dtype");
    const int64_t n = T * dim;
    NV_REQUIRE((n + 255) / 256 < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_token_gate: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(token_gate_kernel<__bf16>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const __bf16*)z,
                           z_stride, (const __bf16*)table, table_stride, ids, offset, dim, (__bf16*)y, n);
    else
        hipLaunchKernelGGL(token_gate_kernel<float>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const float*)z,
                           z_stride, (const float*)table, table_stride, ids, offset, dim, (float*)y, n);
    return check_launch("nv_token_gate");
}
