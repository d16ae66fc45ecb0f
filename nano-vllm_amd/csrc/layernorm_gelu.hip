// LayerNorm on an fp32 residual stream, and the tanh-GELU gate.
//
// Models whose residual stream stays in fp32 (sandwich-normed designs: a norm before AND after every sublayer)
// run each token row through ONE launch per sublayer boundary:
//
//     r  <- r + LN(h; w1, b1) + extra        (post-norm of the sublayer that just produced h, added to the stream;
//                                             `extra` is a second fp32 stream added as is, e.g. an embedding
//                                             re-injection; either part may be absent)
//     y  <- LN(r; w2, b2)                    (pre-norm of the next sublayer, in the matmul dtype; may be absent)
//
// so the stream is read and written once per boundary instead of four times.  All statistics are fp32, two
// passes over a row held in registers (mean first, then squared deviations), eps inside the root.
// One workgroup of 256 threads per row; a thread holds up to kMaxPerThread elements.
#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kLnThreads = 256;
constexpr int kLnMaxPerThread = 64;   // cols <= 16384

template <typename T>
__device__ __forceinline__ float ld(const T* p, int64_t i) { return (float)p[i]; }
template <typename T>
__device__ __forceinline__ void st(T* p, int64_t i, float v) { p[i] = (T)v; }

__device__ __forceinline__ float block_sum(float x, float* red) {
    x = wave_sum(x);
    const int w = threadIdx.x >> 6;
    __syncthreads();                       // red may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) red[w] = x;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kLnThreads / 64; ++i) t += red[i];
    return t;
}

template <typename TH, typename TY, int PER>
__global__ __launch_bounds__(kLnThreads) void add_layernorm_kernel(
    float* __restrict__ resid, const TH* __restrict__ h, int64_t h_stride, const float* __restrict__ w1,
    const float* __restrict__ b1, const float* __restrict__ extra, const float* __restrict__ w2,
    const float* __restrict__ b2, TY* __restrict__ y, int cols, float eps) {
    __shared__ float red[kLnThreads / 64];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const float inv_n = 1.0f / (float)cols;
    float r[PER];
    float* rrow = resid + row * cols;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int c = tid + i * kLnThreads;
        r[i] = c < cols ? rrow[c] : 0.f;
    }
    bool changed = false;
    if (h != nullptr) {
        float x[PER];
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + i * kLnThreads;
            x[i] = c < cols ? ld(h, row * h_stride + c) : 0.f;
            s += x[i];
        }
        const float mean = block_sum(s, red) * inv_n;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + i * kLnThreads;
            const float d = c < cols ? x[i] - mean : 0.f;
            q += d * d;
        }
        const float rstd = 1.0f / sqrtf(block_sum(q, red) * inv_n + eps);
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + i * kLnThreads;
            if (c < cols) r[i] += (x[i] - mean) * rstd * w1[c] + b1[c];
        }
        changed = true;
    }
    if (extra != nullptr) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + i * kLnThreads;
            if (c < cols) r[i] += extra[row * cols + c];
        }
        changed = true;
    }
    if (changed) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + i * kLnThreads;
            if (c < cols) rrow[c] = r[i];
        }
    }
    if (y != nullptr) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) s += r[i];          // padding lanes hold 0
        const float mean = block_sum(s, red) * inv_n;
        float q = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + i * kLnThreads;
            const float d = c < cols ? r[i] - mean : 0.f;
            q += d * d;
        }
        const float rstd = 1.0f / sqrtf(block_sum(q, red) * inv_n + eps);
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + i * kLnThreads;
            if (c < cols) st(y, row * cols + c, (r[i] - mean) * rstd * w2[c] + b2[c]);
        }
    }
}

template <typename TH, typename TY>
static int launch_add_layernorm(float* resid, const void* h, int64_t h_stride, const float* w1, const float* b1,
                                const float* extra, const float* w2, const float* b2, void* y, int64_t rows,
                                int cols, float eps, hipStream_t stream) {
    const int per = (cols + kLnThreads - 1) / kLnThreads;
#define NV_LN_CASE(P)                                                                                         \
    if (per <= P) {                                                                                           \
        hipLaunchKernelGGL((add_layernorm_kernel<TH, TY, P>), dim3((unsigned)rows), dim3(kLnThreads), 0,      \
                           stream, resid, (const TH*)h, h_stride, w1, b1, extra, w2, b2, (TY*)y, cols, eps);  \
        return check_launch("nv_add_layernorm");                                                              \
    }
    NV_LN_CASE(1)
    NV_LN_CASE(2)
    NV_LN_CASE(4)
    NV_LN_CASE(8)
    NV_LN_CASE(16)
    NV_LN_CASE(32)
    NV_LN_CASE(64)
#undef NV_LN_CASE
    set_error("nv_add_layernorm: cols=%d exceeds %d", cols, kLnThreads * kLnMaxPerThread);
    return NV_ERR_UNSUPPORTED;
}

// y[r, j] = gelu_tanh(x[r, j]) * x[r, I + j], fp32 arithmetic, one rounding.
__device__ __forceinline__ float gelu_tanh_f(float z) {
    const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    return 0.5f * z * (1.0f + tanhf(u));
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_and_mul_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                int64_t rows, int inter, int64_t x_stride) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * inter) return;
    const int64_t row = idx / inter;
    const int col = (int)(idx - row * inter);
    const float g = (float)x[row * x_stride + col];
    const float u = (float)x[row * x_stride + inter + col];
    y[idx] = (T)(gelu_tanh_f(g) * u);
}

// bf16 rows in 16-byte pieces (8 elements per thread).  tanh through one exponential: its error (a few fp32 ulps of
// a value that is rounded to 8 bits next) cannot show in bf16.
__device__ __forceinline__ float gelu_tanh_fast(float z) {
    const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    const float t = 1.0f - 2.0f / (__expf(2.0f * u) + 1.0f);
    return 0.5f * z * (1.0f + t);
}

__global__ __launch_bounds__(256) void gelu_tanh_and_mul_bf16x8_kernel(const uint4* __restrict__ x, uint4* __restrict__ y,
                                                                       int64_t rows, int inter_vec, int64_t x_stride_vec) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * inter_vec) return;
    const int64_t row = idx / inter_vec;
    const int col = (int)(idx - row * inter_vec);
    const uint4 g = x[row * x_stride_vec + col];
    const uint4 u = x[row * x_stride_vec + inter_vec + col];
    uint4 o;
#define NV_GELU2(G, U) pack_bf16(gelu_tanh_fast(bf16_lo(G)) * bf16_lo(U), gelu_tanh_fast(bf16_hi(G)) * bf16_hi(U))
    o.x = NV_GELU2(g.x, u.x);
    o.y = NV_GELU2(g.y, u.y);
    o.z = NV_GELU2(g.z, u.z);
    o.w = NV_GELU2(g.w, u.w);
#undef NV_GELU2
    y[idx] = o;
}

}  // namespace nv

extern "C" int nv_add_layernorm(void* resid, const void* h, int h_dtype, int64_t h_stride, const void* w1,
                                const void* b1, const void* extra, const void* w2, const void* b2, void* y,
                                int y_dtype, int64_t rows, int cols, float eps, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0, NV_ERR_INVALID_ARG, "nv_add_layernorm: bad sizes rows=%lld cols=%d",
               (long long)rows, cols);
    if (rows == 0) return NV_OK;
    NV_REQUIRE(resid, NV_ERR_INVALID_ARG, "nv_add_layernorm: null residual stream");
    NV_REQUIRE(!h || (w1 && b1), NV_ERR_INVALID_ARG, "nv_add_layernorm: h needs w1 and b1");
    NV_REQUIRE(!y || (w2 && b2), NV_ERR_INVALID_ARG, "nv_add_layernorm: y needs w2 and b2");
    NV_REQUIRE(h || extra || y, NV_ERR_INVALID_ARG, "nv_add_layernorm: nothing to do");
    NV_REQUIRE((h_dtype == NV_DTYPE_BF16 || h_dtype == NV_DTYPE_F32) && (y_dtype == NV_DTYPE_BF16 || y_dtype == NV_DTYPE_F32),
               NV_ERR_INVALID_ARG, "nv_add_layernorm: dtype must be NV_DTYPE_BF16 or NV_DTYPE_F32");
    NV_REQUIRE(rows < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_add_layernorm: launch too large");
    hipStream_t s = (hipStream_t)stream;
    float* r = (float*)resid;
    const float *fw1 = (const float*)w1, *fb1 = (const float*)b1, *fe = (const float*)extra, *fw2 = (const float*)w2,
                *fb2 = (const float*)b2;
    if (h_dtype == NV_DTYPE_BF16 && y_dtype == NV_DTYPE_BF16)
        return launch_add_layernorm<__bf16, __bf16>(r, h, h_stride, fw1, fb1, fe, fw2, fb2, y, rows, cols, eps, s);
    if (h_dtype == NV_DTYPE_F32 && y_dtype == NV_DTYPE_F32)
        return launch_add_layernorm<float, float>(r, h, h_stride, fw1, fb1, fe, fw2, fb2, y, rows, cols, eps, s);
    if (h_dtype == NV_DTYPE_BF16)
        return launch_add_layernorm<__bf16, float>(r, h, h_stride, fw1, fb1, fe, fw2, fb2, y, rows, cols, eps, s);
    return launch_add_layernorm<float, __bf16>(r, h, h_stride, fw1, fb1, fe, fw2, fb2, y, rows, cols, eps, s);
}

extern "C" int nv_gelu_tanh_and_mul(const void* x, void* y, int dtype, int64_t rows, int inter, int64_t x_stride,
                                    void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && inter > 0 && x_stride >= 2 * (int64_t)inter, NV_ERR_INVALID_ARG,
               "nv_gelu_tanh_and_mul: bad sizes rows=%lld inter=%d stride=%lld", (long long)rows, inter,
               (long long)x_stride);
    if (rows == 0) return NV_OK;
    NV_REQUIRE(x && y, NV_ERR_INVALID_ARG, "nv_gelu_tanh_and_mul: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_gelu_tanh_and_mul: bad dtype");
    if (dtype == NV_DTYPE_BF16 && inter % 8 == 0 && x_stride % 8 == 0 && ((uintptr_t)x | (uintptr_t)y) % 16 == 0) {
        const int64_t vgrid = (rows * (inter / 8) + 255) / 256;
        NV_REQUIRE(vgrid < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_gelu_tanh_and_mul: launch too large");
        hipLaunchKernelGGL(gelu_tanh_and_mul_bf16x8_kernel, dim3((unsigned)vgrid), dim3(256), 0, (hipStream_t)stream,
                           (const uint4*)x, (uint4*)y, rows, inter / 8, x_stride / 8);
        return check_launch("nv_gelu_tanh_and_mul");
    }
    const int64_t grid = (rows * inter + 255) / 256;
    NV_REQUIRE(grid < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_gelu_tanh_and_mul: launch too large");
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(gelu_tanh_and_mul_kernel<__bf16>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                           (const __bf16*)x, (__bf16*)y, rows, inter, x_stride);
    else
        hipLaunchKernelGGL(gelu_tanh_and_mul_kernel<float>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                           (const float*)x, (float*)y, rows, inter, x_stride);
    return check_launch("nv_gelu_tanh_and_mul");
}
