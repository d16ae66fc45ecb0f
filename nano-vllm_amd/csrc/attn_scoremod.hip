// Paged attention with score modifiers, for designs that the fixed softmax(q k^T / sqrt(d)) kernels do not cover:
//
//   s_ij = scale * q_i . k_j                       fp32, from bf16 or fp32 operands
//   s_ij = cap * tanh(s_ij / cap)                  if cap > 0            (logit soft-capping)
//   s_ij = s_ij + bias[h][min(i - j, n_dist-1)]    if bias given         (learned distance bias, one row per head;
//                                                                         the host expands bucketed tables)
//   p_ij = exp(s_ij) / (sum_j' exp(s_ij') + exp(sink_h))                 (sink: an extra term of the denominator
//                                                                         with no key and no value, if given)
//
// Causal (key position <= query position), grouped heads (query head h reads kv head h / (H / G)), any head size:
// the key size D and the value size Dv are runtime arguments and may differ.  K/V are read through the block table
// of a paged cache [num_blocks, block_size, G, D | Dv] with a runtime block size; a step's rows may be prompt
// portions and single decoded tokens side by side (cu_seqlens_q / cu_seqlens_k as in the other attention entry
// points, query i of a sequence sits at position len_k - len_q + i).
//
// nv_qk_prep_store runs in front of it: interleaved-pair rotary on the first rot_dims dimensions of q and k
// (angle = position * inv_freq[i] as an fp32 product, full-precision sincosf), an optional position-dependent
// query temperature q *= 1 + coef * ln(floor((p + 1) / every) + 1), and the scatter of the step's K/V rows into the
// cache.
#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

// ------------------------------------------------------------------------------------------------ prep
template <typename T>
__global__ __launch_bounds__(256) void qk_prep_store_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const int64_t* __restrict__ positions,
    const int* __restrict__ slot_mapping, const float* __restrict__ inv_freq, int rot_dims, float temp_coef,
    int temp_every, int H, int G, int D, int Dv, int64_t q_stride, int64_t k_stride, int64_t v_stride) {
    const int64_t t = blockIdx.x;
    const int64_t pos = positions[t];
    const int slot = slot_mapping ? slot_mapping[t] : -1;
    float temp = 1.0f;
    if (temp_every > 0) temp = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
    const int half = D / 2;            // pairs per head when D is even; an odd last dimension passes through below
    const int rot_pairs = rot_dims / 2;
    // q heads then k heads, one (head, pair) per thread iteration
    const int total_pairs = (H + G) * half;
    for (int idx = threadIdx.x; idx < total_pairs; idx += blockDim.x) {
        const int head = idx / half, pr = idx - head * half;
        const bool is_q = head < H;
        const T* src = is_q ? q + t * q_stride + (int64_t)head * D : k + t * k_stride + (int64_t)(head - H) * D;
        float a = (float)src[2 * pr], b = (float)src[2 * pr + 1];
        if (pr < rot_pairs) {
            const float ang = (float)pos * inv_freq[pr];
            float sn, cs;
            sincosf(ang, &sn, &cs);
            const float ra = a * cs - b * sn, rb = b * cs + a * sn;
            a = ra;
            b = rb;
        }
        if (is_q) {
            T* dst = q_out + (t * H + head) * (int64_t)D;
            dst[2 * pr] = (T)(a * temp);
            dst[2 * pr + 1] = (T)(b * temp);
        } else if (slot >= 0) {
            T* dst = k_cache + ((int64_t)slot * G + (head - H)) * D;
            dst[2 * pr] = (T)a;
            dst[2 * pr + 1] = (T)b;
        }
    }
    if (D & 1) {
        for (int head = threadIdx.x; head < H + G; head += blockDim.x) {
            const bool is_q = head < H;
            const T* src = is_q ? q + t * q_stride + (int64_t)head * D : k + t * k_stride + (int64_t)(head - H) * D;
            const float a = (float)src[D - 1];
            if (is_q) q_out[(t * H + head) * (int64_t)D + D - 1] = (T)(a * temp);
            else if (slot >= 0) k_cache[((int64_t)slot * G + (head - H)) * D + D - 1] = (T)a;
        }
    }
    if (slot >= 0) {
        for (int idx = threadIdx.x; idx < G * Dv; idx += blockDim.x)
            v_cache[(int64_t)slot * G * Dv + idx] = v[t * v_stride + idx];
    }
}

// ------------------------------------------------------------------------------------------------ attention
// One wave per (query token, query head).  Keys go by in tiles of 64: lane j scores key j of the tile (its own
// K row, q broadcast from LDS), the tile's weights go through LDS, then the lanes switch to value channels
// (lane c accumulates channels c, c + 64, ...) and stream the tile's V rows, which are contiguous per key.
constexpr int kSmMaxDvPerLane = 4;   // Dv <= 256

template <typename T>
__global__ __launch_bounds__(64) void attn_scoremod_rowwave_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    const int* __restrict__ cu_q, const int* __restrict__ cu_k, const int* __restrict__ block_tables, int B,
    int max_blocks, int H, int G, int D, int Dv, int block_size, float scale, float softcap,
    const float* __restrict__ sink, const float* __restrict__ dist_bias, int n_dist, int64_t q_stride,
    int64_t out_stride) {
    extern __shared__ float smem[];
    float* qs = smem;                      // [D]
    float* ps = smem + D;                  // [64]
    int64_t* rows = (int64_t*)(smem + D + 64 + ((D & 1) ? 1 : 0));   // [64] element offsets of the tile's cache rows
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    // sequence of this token: cu_q is sorted, B is small
    int lo = 0, hi = B;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid;
    }
    const int b = lo;
    const int len_q = cu_q[b + 1] - cu_q[b], len_k = cu_k[b + 1] - cu_k[b];
    const int pos = len_k - len_q + (t - cu_q[b]);      // this query's position; it sees keys 0 .. pos
    const int g = h / (H / G);
    for (int d = lane; d < D; d += 64) qs[d] = (float)q[(int64_t)t * q_stride + (int64_t)h * D + d];
    const int* table = block_tables + (int64_t)b * max_blocks;
    const float* bias_h = dist_bias ? dist_bias + (int64_t)h * n_dist : nullptr;
    float m = -INFINITY, l = 0.f;
    float acc[kSmMaxDvPerLane] = {0.f, 0.f, 0.f, 0.f};
    const int n_keys = pos + 1;
    __syncthreads();
    for (int base = 0; base < n_keys; base += 64) {
        const int j = base + lane;
        float s = -INFINITY;
        int64_t row = 0;
        if (j < n_keys) {
            const int blk = table[j / block_size];
            row = ((int64_t)blk * block_size + (j % block_size)) * G + g;
            const T* kr = k_cache + row * D;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot += qs[d] * (float)kr[d];
            s = dot * scale;
            if (softcap > 0.f) s = softcap * tanhf(s / softcap);
            if (bias_h) s += bias_h[min(pos - j, n_dist - 1)];
        }
        float tile_max = s;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, o));
        const float m_new = fmaxf(m, tile_max);              // finite: key `base` is visible
        const float p = j < n_keys ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);                  // exp(-inf) = 0 on the first tile
        l = l * corr + wave_sum(p);
        m = m_new;
        __syncthreads();                                     // previous tile's readers are done
        ps[lane] = p;
        rows[lane] = row;
        __syncthreads();
        const int n_tile = min(64, n_keys - base);
#pragma unroll
        for (int i = 0; i < kSmMaxDvPerLane; ++i) acc[i] *= corr;
        for (int jj = 0; jj < n_tile; ++jj) {
            const float pj = ps[jj];
            const T* vr = v_cache + rows[jj] * Dv;
#pragma unroll
            for (int i = 0; i < kSmMaxDvPerLane; ++i) {
                const int c = lane + 64 * i;
                if (c < Dv) acc[i] += pj * (float)vr[c];
            }
        }
    }
    if (sink) {
        const float sk = sink[h];
        const float m_new = fmaxf(m, sk);
        const float corr = expf(m - m_new);
        l = l * corr + expf(sk - m_new);
#pragma unroll
        for (int i = 0; i < kSmMaxDvPerLane; ++i) acc[i] *= corr;
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < kSmMaxDvPerLane; ++i) {
        const int c = lane + 64 * i;
        if (c < Dv) out[(int64_t)t * out_stride + (int64_t)h * Dv + c] = (T)(acc[i] * inv);
    }
}

}  // namespace nv

extern "C" int nv_qk_prep_store(const void* q, const void* k, const void* v, void* q_out, void* k_cache,
                                void* v_cache, const int64_t* positions, const int* slot_mapping,
                                const float* inv_freq, int rot_dims, float temp_coef, int temp_every, int dtype,
                                int64_t T, int H, int G, int D, int Dv, int64_t q_stride, int64_t k_stride,
                                int64_t v_stride, void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && H > 0 && G > 0 && D > 0 && Dv > 0, NV_ERR_INVALID_ARG, "nv_qk_prep_store: bad sizes");
    if (T == 0) return NV_OK;
    NV_REQUIRE(q && k && v && q_out && positions, NV_ERR_INVALID_ARG, "nv_qk_prep_store: null pointer");
    NV_REQUIRE(!slot_mapping || (k_cache && v_cache), NV_ERR_INVALID_ARG, "nv_qk_prep_store: scatter needs the caches");
    NV_REQUIRE(rot_dims >= 0 && rot_dims <= D && rot_dims % 2 == 0 && (rot_dims == 0 || inv_freq), NV_ERR_INVALID_ARG,
               "nv_qk_prep_store: rot_dims=%d must be even, at most D=%d, with a frequency table", rot_dims, D);
    NV_REQUIRE(temp_every >= 0, NV_ERR_INVALID_ARG, "nv_qk_prep_store: temp_every < 0");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_qk_prep_store: bad dtype");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_qk_prep_store: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(qk_prep_store_kernel<__bf16>, dim3((unsigned)T), dim3(256), 0, s, (const __bf16*)q,
                           (const __bf16*)k, (const __bf16*)v, (__bf16*)q_out, (__bf16*)k_cache, (__bf16*)v_cache,
                           positions, slot_mapping, inv_freq, rot_dims, temp_coef, temp_every, H, G, D, Dv, q_stride,
                           k_stride, v_stride);
    else
        hipLaunchKernelGGL(qk_prep_store_kernel<float>, dim3((unsigned)T), dim3(256), 0, s, (const float*)q,
                           (const float*)k, (const float*)v, (float*)q_out, (float*)k_cache, (float*)v_cache,
                           positions, slot_mapping, inv_freq, rot_dims, temp_coef, temp_every, H, G, D, Dv, q_stride,
                           k_stride, v_stride);
    return check_launch("nv_qk_prep_store");
}

extern "C" int nv_attn_scoremod_paged(const void* q, const void* k_cache, const void* v_cache, void* out,
                                      const int* cu_seqlens_q, const int* cu_seqlens_k, const int* block_tables,
                                      int num_seqs, int max_blocks_per_seq, int64_t T, int H, int G, int D, int Dv,
                                      int64_t num_blocks, int block_size, float scale, float softcap,
                                      const float* sink, const float* dist_bias, int n_dist, int dtype,
                                      int64_t q_stride, int64_t out_stride, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && T >= 0 && H > 0 && G > 0 && D > 0 && Dv > 0 && block_size > 0 && num_blocks > 0 &&
                   max_blocks_per_seq > 0,
               NV_ERR_INVALID_ARG, "nv_attn_scoremod_paged: bad sizes");
    if (T == 0 || num_seqs == 0) return NV_OK;
    NV_REQUIRE(q && k_cache && v_cache && out && cu_seqlens_q && cu_seqlens_k && block_tables, NV_ERR_INVALID_ARG,
               "nv_attn_scoremod_paged: null pointer");
    NV_REQUIRE(H % G == 0, NV_ERR_INVALID_ARG, "nv_attn_scoremod_paged: H=%d not a multiple of G=%d", H, G);
    NV_REQUIRE(Dv <= 64 * kSmMaxDvPerLane, NV_ERR_UNSUPPORTED, "nv_attn_scoremod_paged: Dv=%d exceeds %d", Dv,
               64 * kSmMaxDvPerLane);
    NV_REQUIRE(D <= 1024, NV_ERR_UNSUPPORTED, "nv_attn_scoremod_paged: D=%d exceeds 1024", D);
    NV_REQUIRE(!dist_bias || n_dist > 0, NV_ERR_INVALID_ARG, "nv_attn_scoremod_paged: bias without rows");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_attn_scoremod_paged: bad dtype");
    NV_REQUIRE(T < (1LL << 31) && H < 65536, NV_ERR_UNSUPPORTED, "nv_attn_scoremod_paged: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const size_t smem = sizeof(float) * (D + 64 + (D & 1)) + sizeof(int64_t) * 64;
    const dim3 grid((unsigned)T, (unsigned)H);
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(attn_scoremod_rowwave_kernel<__bf16>, grid, dim3(64), smem, s, (const __bf16*)q,
                           (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out, cu_seqlens_q, cu_seqlens_k,
                           block_tables, num_seqs, max_blocks_per_seq, H, G, D, Dv, block_size, scale, softcap, sink,
                           dist_bias, n_dist, q_stride, out_stride);
    else
        hipLaunchKernelGGL(attn_scoremod_rowwave_kernel<float>, grid, dim3(64), smem, s, (const float*)q,
                           (const float*)k_cache, (const float*)v_cache, (float*)out, cu_seqlens_q, cu_seqlens_k,
                           block_tables, num_seqs, max_blocks_per_seq, H, G, D, Dv, block_size, scale, softcap, sink,
                           dist_bias, n_dist, q_stride, out_stride);
    return check_launch("nv_attn_scoremod_paged");
}
