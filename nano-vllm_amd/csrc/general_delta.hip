// Generalized delta rule with one decay AND one removal rate per head and key channel, state [D, D] per head in fp32,
// carried per SEQUENCE in numbered slots (as the other recurrent kernels of this library: a sequence whose rows start
// at position 0 starts from a zero state whatever its slot holds).
//
//     u = k / sqrt(sum k^2 + key_eps)                                   unit key per head
//     w = exp(-decay_rate * sigmoid(w_raw + w_bias))                    decay per key channel, in (exp(-decay_rate), 1)
//     a = sigmoid(a_raw + a_bias)                                       removal rate per key channel
//     S <- diag(w) S - (a * u)(u^T S) + k v^T                           both terms read the old state
//     o = S^T r;   out = o / sqrt(mean(o^2) + eps) * norm_w * sigmoid(gate_raw)
//
// Everything after the raw projections is fp32.  Layout as in the gated delta rule next door: one workgroup per
// (sequence, head); a lane owns one value column and a quarter of the key rows (its quad index r owns rows
// r * RPL .. r * RPL + RPL - 1, read from LDS four at a time, the four runs RPL + 4 words apart so that a quad's 16-byte
// reads fall on different banks), so the state lives in registers and the token loop has no workgroup barrier: the
// vectors of up to 16 tokens are prepared into LDS by all waves together (every load of the tile issued at once, then the
// unit keys per token), each wave then runs those tokens for its 16
// columns (one pass for u^T S, one for the update and the read-out, a two-step quad reduction each), and the
// normalised, gated read-out of the tile is written by all waves together.
#include <algorithm>

#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kGdMaxTile = 16;
constexpr int kGdLdsBudget = 60 * 1024;

__device__ __forceinline__ float gd_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float gd_quad_sum(float x) {
    x += dpp_f32<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp_f32<0x4E>(x);   // quad_perm [2,3,0,1]
    return x;
}

template <typename T, int RPL>
__global__ void general_delta_rule_kernel(
    const T* __restrict__ r_in, const T* __restrict__ k, const T* __restrict__ v, int64_t r_stride, int64_t k_stride,
    int64_t v_stride, const T* __restrict__ w_raw, int64_t w_stride, const T* __restrict__ a_raw, int64_t a_stride,
    const T* __restrict__ gate_raw, int64_t gate_stride, const float* __restrict__ w_bias,
    const float* __restrict__ a_bias, const float* __restrict__ norm_w, float* __restrict__ state, T* __restrict__ out,
    int64_t out_stride, const int* __restrict__ cu_q, const int* __restrict__ cu_k, const int* __restrict__ state_slots,
    int H, int D, float eps, float decay_rate, float key_eps, int tile) {
    constexpr int DP = (RPL + 4) * 4;                 // LDS words per token and vector: four runs of RPL rows, padded
    extern __shared__ float smem[];
    float* us = smem;                                 // [tile][DP] unit key
    float* ws = us + tile * DP;                       // [tile][DP] decay
    float* as = ws + tile * DP;                       // [tile][DP] removal rate times unit key
    float* ks = as + tile * DP;                       // [tile][DP] key
    float* rs = ks + tile * DP;                       // [tile][DP] read-out vector
    float* vs = rs + tile * DP;                       // [tile][D]
    float* os = vs + tile * D;                        // [tile][D]
    const int b = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
    const int q0 = cu_q[b], len_q = cu_q[b + 1] - q0;
    if (len_q <= 0) return;
    const int start = (cu_k[b + 1] - cu_k[b]) - len_q;
    const int col = wave * 16 + (lane >> 2), q = lane & 3;
    const bool live = col < D;
    float* S_slot = state + ((int64_t)state_slots[b] * H + h) * (int64_t)D * D;
    float S[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int row = q * RPL + i;
        S[i] = (live && start > 0 && row < D) ? S_slot[(int64_t)row * D + col] : 0.f;
    }
    for (int t0 = 0; t0 < len_q; t0 += tile) {
        const int nt = min(tile, len_q - t0);
        __syncthreads();                              // the previous tile's epilogue has read os
        // ---- prepare the tile: all loads of the tile in flight at once, then the unit keys per token -------
        for (int i = tid; i < nt * 4 * RPL; i += blockDim.x) {
            const int tt = i / (4 * RPL), d = i % (4 * RPL);
            const int at = tt * DP + (d / RPL) * (RPL + 4) + (d % RPL);
            float wv = 1.f, av = 0.f, kv = 0.f, rv = 0.f;
            if (d < D) {
                const int64_t t = q0 + t0 + tt, hd = (int64_t)h * D + d;
                kv = (float)k[t * k_stride + hd];
                rv = (float)r_in[t * r_stride + hd];
                wv = expf(-decay_rate * gd_sigmoid((float)w_raw[t * w_stride + hd] + w_bias[hd]));
                av = gd_sigmoid((float)a_raw[t * a_stride + hd] + a_bias[hd]);
            }
            ws[at] = wv;
            as[at] = av;
            ks[at] = kv;
            rs[at] = rv;
        }
        for (int i = tid; i < nt * D; i += blockDim.x) {
            const int tt = i / D, c = i % D;
            vs[tt * D + c] = (float)v[(int64_t)(q0 + t0 + tt) * v_stride + (int64_t)h * D + c];
        }
        __syncthreads();
        for (int tt = wave; tt < nt; tt += n_waves) {
            float kk = 0.f;
            for (int d = lane; d < 4 * RPL; d += 64) {
                const float kv = ks[tt * DP + (d / RPL) * (RPL + 4) + (d % RPL)];     // (zeros past D)
                kk += kv * kv;
            }
            kk = wave_sum(kk);
            const float kn = 1.0f / sqrtf(kk + key_eps);
            for (int d = lane; d < 4 * RPL; d += 64) {
                const int at = tt * DP + (d / RPL) * (RPL + 4) + (d % RPL);
                const float uv = ks[at] * kn;
                us[at] = uv;
                as[at] *= uv;
            }
        }
        __syncthreads();
        // ---- the recurrence over the tile, no barrier inside ---------------------------------------------
        if (live) {
            for (int tt = 0; tt < nt; ++tt) {
                const int base = tt * DP + q * (RPL + 4);
                const float4* ut = (const float4*)(us + base);
                const float4* wt = (const float4*)(ws + base);
                const float4* at = (const float4*)(as + base);
                const float4* kt = (const float4*)(ks + base);
                const float4* rt = (const float4*)(rs + base);
                float sk = 0.f;
#pragma unroll
                for (int i = 0; i < RPL / 4; ++i) {
                    const float4 u4 = ut[i];
                    sk += S[4 * i] * u4.x + S[4 * i + 1] * u4.y + S[4 * i + 2] * u4.z + S[4 * i + 3] * u4.w;
                }
                sk = gd_quad_sum(sk);
                const float vc = vs[tt * D + col];
                float so = 0.f;
#pragma unroll
                for (int i = 0; i < RPL / 4; ++i) {
                    const float4 w4 = wt[i], a4 = at[i], k4 = kt[i], r4 = rt[i];
                    S[4 * i] = w4.x * S[4 * i] - a4.x * sk + k4.x * vc;
                    S[4 * i + 1] = w4.y * S[4 * i + 1] - a4.y * sk + k4.y * vc;
                    S[4 * i + 2] = w4.z * S[4 * i + 2] - a4.z * sk + k4.z * vc;
                    S[4 * i + 3] = w4.w * S[4 * i + 3] - a4.w * sk + k4.w * vc;
                    so += S[4 * i] * r4.x + S[4 * i + 1] * r4.y + S[4 * i + 2] * r4.z + S[4 * i + 3] * r4.w;
                }
                so = gd_quad_sum(so);
                if (q == 0) os[tt * D + col] = so;
            }
        }
        __syncthreads();
        // ---- normalised, gated read-out of the tile ----------------------------------------------------
        for (int tt = wave; tt < nt; tt += n_waves) {
            const int64_t t = q0 + t0 + tt;
            float ss = 0.f;
            for (int c = lane; c < D; c += 64) ss += os[tt * D + c] * os[tt * D + c];
            ss = wave_sum(ss);
            const float rstd = 1.0f / sqrtf(ss / (float)D + eps);
            for (int c = lane; c < D; c += 64) {
                const int64_t hc = (int64_t)h * D + c;
                const float gate = gd_sigmoid((float)gate_raw[t * gate_stride + hc]);
                out[t * out_stride + hc] = (T)(os[tt * D + c] * rstd * norm_w[hc] * gate);
            }
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            const int row = q * RPL + i;
            if (row < D) S_slot[(int64_t)row * D + col] = S[i];
        }
    }
}

template <typename T>
static int launch_general_delta(const void* r, const void* k, const void* v, int64_t r_stride, int64_t k_stride,
                                int64_t v_stride, const void* w_raw, int64_t w_stride, const void* a_raw,
                                int64_t a_stride, const void* gate_raw, int64_t gate_stride, const float* w_bias,
                                const float* a_bias, const float* norm_w, float* state, void* out, int64_t out_stride,
                                const int* cu_q, const int* cu_k, const int* state_slots, int B, int H, int D, float eps,
                                float decay_rate, float key_eps, hipStream_t s) {
    const int waves = (D + 15) / 16;
    const dim3 grid((unsigned)B, (unsigned)H), block((unsigned)waves * 64);
    const int rpl = D <= 32 ? 8 : D <= 64 ? 16 : D <= 128 ? 32 : 64;
    const size_t per_token = sizeof(float) * (size_t)(5 * (rpl + 4) * 4 + 2 * D);
    const int tile = (int)std::max<size_t>(1, std::min<size_t>(kGdMaxTile, kGdLdsBudget / per_token));
    const size_t smem = per_token * tile;
#define NV_GD_CASE(R)                                                                                                \
    case R:                                                                                                          \
        hipLaunchKernelGGL((general_delta_rule_kernel<T, R>), grid, block, smem, s, (const T*)r, (const T*)k,       \
                           (const T*)v, r_stride, k_stride, v_stride, (const T*)w_raw, w_stride, (const T*)a_raw,   \
                           a_stride, (const T*)gate_raw, gate_stride, w_bias, a_bias, norm_w, state, (T*)out,       \
                           out_stride, cu_q, cu_k, state_slots, H, D, eps, decay_rate, key_eps, tile);              \
        break;
    switch (rpl) {
        NV_GD_CASE(8)
        NV_GD_CASE(16)
        NV_GD_CASE(32)
        NV_GD_CASE(64)
    }
#undef NV_GD_CASE
    return check_launch("nv_general_delta_rule");
}

}  // namespace nv

extern "C" int nv_general_delta_rule(const void* r, const void* k, const void* v, int64_t r_stride, int64_t k_stride,
                                     int64_t v_stride, const void* w_raw, int64_t w_stride, const void* a_raw,
                                     int64_t a_stride, const void* gate_raw, int64_t gate_stride, const float* w_bias,
                                     const float* a_bias, const float* norm_w, float* state, void* out,
                                     int64_t out_stride, const int* cu_seqlens_q, const int* cu_seqlens_k,
                                     const int* state_slots, int num_seqs, int H, int D, float eps, float decay_rate,
                                     float key_eps, int dtype, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && H > 0 && D > 0, NV_ERR_INVALID_ARG, "nv_general_delta_rule: bad sizes");
    if (num_seqs == 0) return NV_OK;
    NV_REQUIRE(r && k && v && w_raw && a_raw && gate_raw && w_bias && a_bias && norm_w && state && out &&
                   cu_seqlens_q && cu_seqlens_k && state_slots,
               NV_ERR_INVALID_ARG, "nv_general_delta_rule: null pointer");
    NV_REQUIRE(D <= 256, NV_ERR_UNSUPPORTED, "nv_general_delta_rule: D=%d exceeds 256", D);
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_general_delta_rule: bad dtype");
    NV_REQUIRE(H < 65536, NV_ERR_UNSUPPORTED, "nv_general_delta_rule: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        return launch_general_delta<__bf16>(r, k, v, r_stride, k_stride, v_stride, w_raw, w_stride, a_raw, a_stride,
                                            gate_raw, gate_stride, w_bias, a_bias, norm_w, state, out, out_stride,
                                            cu_seqlens_q, cu_seqlens_k, state_slots, num_seqs, H, D, eps, decay_rate,
                                            key_eps, s);
    return launch_general_delta<float>(r, k, v, r_stride, k_stride, v_stride, w_raw, w_stride, a_raw, a_stride, gate_raw,
                                       gate_stride, w_bias, a_bias, norm_w, state, out, out_stride, cu_seqlens_q,
                                       cu_seqlens_k, state_slots, num_seqs, H, D, eps, decay_rate, key_eps, s);
}
