// Latent attention: what goes in front of the paged attention launch when keys and values are cached as ONE
// normalised low-rank latent per token plus one rotated key part shared by all heads.
//
// Attention then runs in the latent space as multi-query attention: the key up-projection has been applied to the
// query (q_lat = Uk_h^T q_plain, a matrix product done by the caller), the cached "key" of a token is
// [c | rot(k_r)] (rank + R wide), its "value" is c, and the value up-projection is applied to the attention output.
//
// nv_latent_prep_store, per token t at position p:
//     c        = ckv[t, :rank] / sqrt(mean(ckv[t, :rank]^2) + eps) * latent_w          (fp32, then the cache dtype)
//     k_r      = rot_p(ckv[t, rank:])
//     q_full[t, h] = [q_lat[t, h] | rot_p(q[t, h, Dq - R:])]
//     k_cache[slot(t)] = [c | k_r],   v_cache[slot(t)] = c                             (slot < 0: not stored; v_cache
//                                                                                       absent: values alias the keys)
// rot_p turns pair i by the angle p * freq[i] (fp32 product) with cos and sin both times `mag`; the pair is
// (2i, 2i+1) when `interleaved`, else (i, i + R/2).  The frequencies are a table of the caller's (plain powers of a
// base, or blended for long contexts).
#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_store_kernel(
    const T* __restrict__ q, int64_t q_stride, int Dq, const T* __restrict__ q_lat, int64_t ql_stride_t,
    int64_t ql_stride_h, const T* __restrict__ ckv, int64_t ckv_stride, const float* __restrict__ latent_w,
    const float* __restrict__ freq, float mag, int interleaved, const int64_t* __restrict__ positions,
    const int* __restrict__ slot_mapping, T* __restrict__ q_full, T* __restrict__ k_cache, T* __restrict__ v_cache,
    int H, int rank, int R, float eps) {
    __shared__ float red[4];
    __shared__ float cs[2 * 512];                  // cos | sin of the token's angles, R / 2 <= 512 each
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x, half = R >> 1, Dk = rank + R;
    const float pos = (float)positions[t];
    for (int i = tid; i < half; i += 256) {
        const float ang = pos * freq[i];
        cs[i] = cosf(ang) * mag;
        cs[512 + i] = sinf(ang) * mag;
    }
    const T* crow = ckv + t * ckv_stride;
    float ss = 0.f;
    for (int c = tid; c < rank; c += 256) {
        const float v = (float)crow[c];
        ss += v * v;
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();                               // also publishes cs
    const float rstd = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)rank + eps);
    const int64_t slot = slot_mapping != nullptr ? slot_mapping[t] : -1;
    if (slot >= 0) {
        T* krow = k_cache + slot * Dk;
        for (int c = tid; c < rank; c += 256) {
            const T v = (T)((float)crow[c] * rstd * latent_w[c]);
            krow[c] = v;
            if (v_cache != nullptr) v_cache[slot * rank + c] = v;      // (absent when the values alias the key rows)
        }
        for (int i = tid; i < half; i += 256) {
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            const float a = (float)crow[rank + ia], b = (float)crow[rank + ib];
            krow[rank + ia] = (T)(a * cs[i] - b * cs[512 + i]);
            krow[rank + ib] = (T)(b * cs[i] + a * cs[512 + i]);
        }
    }
    for (int h = 0; h < H; ++h) {
        T* qo = q_full + (t * H + h) * Dk;
        const T* ql = q_lat + t * ql_stride_t + h * ql_stride_h;
        for (int c = tid; c < rank; c += 256) qo[c] = ql[c];
        const T* qr = q + t * q_stride + (int64_t)h * Dq + (Dq - R);
        for (int i = tid; i < half; i += 256) {
            const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
            const float a = (float)qr[ia], b = (float)qr[ib];
            qo[rank + ia] = (T)(a * cs[i] - b * cs[512 + i]);
            qo[rank + ib] = (T)(b * cs[i] + a * cs[512 + i]);
        }
    }
}

}  // namespace nv

extern "C" int nv_latent_prep_store(const void* q, int64_t q_stride, int Dq, const void* q_lat, int64_t ql_stride_t,
                                    int64_t ql_stride_h, const void* ckv, int64_t ckv_stride, const float* latent_w,
                                    const float* freq, float mag, int interleaved, const int64_t* positions,
                                    const int32_t* slot_mapping, void* q_full, void* k_cache, void* v_cache, int dtype,
                                    int64_t T, int H, int rank, int R, float eps, void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && H > 0 && rank > 0 && R >= 0 && Dq >= R, NV_ERR_INVALID_ARG, "nv_latent_prep_store: bad sizes");
    if (T == 0) return NV_OK;
    NV_REQUIRE(q && q_lat && ckv && latent_w && positions && q_full, NV_ERR_INVALID_ARG,
               "nv_latent_prep_store: null pointer");
    NV_REQUIRE(!slot_mapping || k_cache, NV_ERR_INVALID_ARG, "nv_latent_prep_store: scatter needs the key cache");
    NV_REQUIRE(R % 2 == 0 && R <= 1024 && (R == 0 || freq), NV_ERR_INVALID_ARG,
               "nv_latent_prep_store: the rotated part (%d) must be even, at most 1024, with its frequencies", R);
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_latent_prep_store: bad dtype");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_latent_prep_store: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(latent_prep_store_kernel<__bf16>, dim3((unsigned)T), dim3(256), 0, s, (const __bf16*)q, q_stride,
                           Dq, (const __bf16*)q_lat, ql_stride_t, ql_stride_h, (const __bf16*)ckv, ckv_stride, latent_w,
                           freq, mag, interleaved, positions, slot_mapping, (__bf16*)q_full, (__bf16*)k_cache,
                           (__bf16*)v_cache, H, rank, R, eps);
    else
        hipLaunchKernelGGL(latent_prep_store_kernel<float>, dim3((unsigned)T), dim3(256), 0, s, (const float*)q, q_stride,
                           Dq, (const float*)q_lat, ql_stride_t, ql_stride_h, (const float*)ckv, ckv_stride, latent_w,
                           freq, mag, interleaved, positions, slot_mapping, (float*)q_full, (float*)k_cache,
                           (float*)v_cache, H, rank, R, eps);
    return check_launch("nv_latent_prep_store");
}
