// Paged attention with score modifiers, for designs that the fixed softmax(q k^T / sqrt(d)) kernels do not cover:
//
//   s_ij = scale * q_i . k_j                       fp32, from bf16 or fp32 operands
//   s_ij = cap * tanh(s_ij / cap)                  if cap > 0            (logit soft-capping)
//   s_ij = s_ij + bias[h][min(i - j, n_dist-1)]    if bias given         (learned distance bias, one row per head;
//                                                                         the host expands bucketed tables)
//   p_ij = exp(s_ij) / (sum_j' exp(s_ij') + exp(sink_h))                 (sink: a learned per-head logit that joins
//                                                                         the normalisation only, if given)
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
#include <algorithm>

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
constexpr int kSmMaxDvPerLane = 8;   // Dv <= 512 (the tile and decode kernels take Dv <= 256, the row-per-wave kernel the rest)

template <typename T>
__global__ __launch_bounds__(64) void attn_scoremod_rowwave_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    const int* __restrict__ cu_q, const int* __restrict__ cu_k, const int* __restrict__ block_tables, int B,
    int max_blocks, int H, int G, int D, int Dv, int block_size, float scale, float softcap,
    const float* __restrict__ sink, const float* __restrict__ dist_bias, int n_dist, int64_t q_stride,
    int64_t out_stride, int64_t v_ld, int only_single_rows) {
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
    // only_single_rows: 0 = every row, 1 = sequences with one row only, 2 = sequences with several rows only
    if ((only_single_rows == 1 && len_q != 1) || (only_single_rows == 2 && len_q == 1)) return;
    const int pos = len_k - len_q + (t - cu_q[b]);      // this query's position; it sees keys 0 .. pos
    const int g = h / (H / G);
    for (int d = lane; d < D; d += 64) qs[d] = (float)q[(int64_t)t * q_stride + (int64_t)h * D + d];
    const int* table = block_tables + (int64_t)b * max_blocks;
    const float* bias_h = dist_bias ? dist_bias + (int64_t)h * n_dist : nullptr;
    float m = -INFINITY, l = 0.f;
    float acc[kSmMaxDvPerLane] = {};
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
            const T* vr = v_cache + rows[jj] * v_ld;
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


// ------------------------------------------------------------------------------------------------ prompt portions
// bf16 MFMA kernel for sequences with several query rows.  A workgroup of four waves takes 64 consecutive queries of
// one (sequence, head); a wave owns 16 of them.  Key tiles of 64 go through LDS once per workgroup: K as stored
// ([key][d]) and V transposed ([dv][key]).  Everything is computed transposed, so that one lane keeps one query:
//     S^T (keys x queries) = K Q^T        v_mfma_f32_16x16x16_bf16: A = K rows from LDS, B = Q^T held in registers
//     O^T (dv x queries)  += V^T P^T      A = V^T rows from LDS, B = P^T, which is the accumulator layout of S^T as is
// Lane l holds query l % 16 in every accumulator, so the running maximum, the rescale factor and the denominator are
// per-lane scalars (the maximum joins the four lane groups with two shuffles per tile, the denominator once at the end).
constexpr int kTileQ = 64, kTileK = 64, kTileThreads = 256;

__device__ __forceinline__ float fast_tanh(float x) {
    // 1 - 2 / (e^{2x} + 1) with the hardware exponential and reciprocal (about 1 ulp each; the result feeds a bf16
    // probability): exact limits at both ends (e^{2x} -> inf gives 1, -> 0 gives -1)
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(x * 2.885390081777927f) + 1.0f);
}

template <int DS, int DVS>     // D = 16 DS, Dv = 16 DVS: every loop below has a compile-time length
__global__ __launch_bounds__(kTileThreads, 2) void attn_scoremod_tile_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
    __bf16* __restrict__ out, const int* __restrict__ cu_q, const int* __restrict__ cu_k,
    const int* __restrict__ block_tables, int max_blocks, int tiles_per_seq, int H, int G, int D, int Dv,
    int block_size, float scale, float softcap, const float* __restrict__ sink, const float* __restrict__ dist_bias,
    int n_dist, int64_t q_stride, int64_t out_stride, int64_t v_rs) {      // v_rs: elements between value rows
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int b = blockIdx.x / tiles_per_seq, qt = blockIdx.x % tiles_per_seq, h = blockIdx.y;
    const int q0 = cu_q[b], len_q = cu_q[b + 1] - q0, len_k = cu_k[b + 1] - cu_k[b];
    if (len_q <= 1 || qt * kTileQ >= len_q) return;          // single rows belong to the row-wave kernel
    const int g = h / (H / G);
    // LDS row lengths in elements: 2 words more than a multiple of 32 words, so the 16 lanes that read 8 bytes of 16
    // different rows in one pass of an operand load fall on 16 different bank pairs
    const int k_ld = D + 4, v_ld = kTileK + 4;
    __bf16* ldsK = (__bf16*)lds_raw;                          // [64][D + 4]
    __bf16* ldsV = ldsK + kTileK * k_ld;                      // [Dv][64 + 4]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 15, lg = lane >> 4;
    const int start = len_k - len_q;                          // position of the sequence's first row in this step
    const int row0 = qt * kTileQ + wave * 16;                 // first query of this wave (index within the step's rows)
    const int my_row = min(row0 + lq, len_q - 1);             // rows past the end repeat the last one and are not stored
    const int my_pos = start + my_row;
    const int wave_last_pos = start + min(row0 + 15, len_q - 1);
    const bool wave_live = row0 < len_q;
    // Q^T fragments: lane holds q[my_row][16 s + 4 lg .. + 3]
    s16x4 qf[DS];
    {
        const __bf16* qr = q + (int64_t)(q0 + my_row) * q_stride + (int64_t)h * D;
#pragma unroll
        for (int s = 0; s < DS; ++s) qf[s] = *(const s16x4*)(qr + 16 * s + 4 * lg);
    }
    f32x4 oacc[DVS];
#pragma unroll
    for (int i = 0; i < DVS; ++i) oacc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const int* table = block_tables + (int64_t)b * max_blocks;
    const float* bias_h = dist_bias ? dist_bias + (int64_t)h * n_dist : nullptr;
    const int last_pos = start + min(qt * kTileQ + kTileQ, len_q) - 1;      // the tile's last query sees keys 0 .. last_pos
    // Loading a tile: thread (key = tid % 64, quarter = tid / 64) fetches 16-byte pieces quarter, quarter + 4, ... of
    // its key's K row and V row.  One block-table lookup per thread and tile, every load of a tile issued before
    // anything waits on one, and the next tile's loads are in flight while this tile is computed.
    const int my_key = tid & (kTileK - 1), my_quarter = tid >> 6;
    // 16-byte pieces per thread of a K row / a V row (a row has 2 DS / 2 DVS pieces; with an odd count the last round
    // is taken by the first two quarters only)
    constexpr int KP = (2 * DS + 3) / 4, VP = (2 * DVS + 3) / 4;
    uint4 kreg[KP], vreg[VP];
    auto fetch = [&](int base) {
        const int j = base + my_key;
        const bool in = j < len_k;
        int64_t row = 0;
        if (in) row = ((int64_t)table[j / block_size] * block_size + (j % block_size)) * G + g;
#pragma unroll
        for (int i = 0; i < KP; ++i)
            kreg[i] = (in && my_quarter + 4 * i < 2 * DS) ? *(const uint4*)(k_cache + row * D + 8 * (my_quarter + 4 * i))
                                                         : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < VP; ++i)
            vreg[i] = (in && my_quarter + 4 * i < 2 * DVS) ? *(const uint4*)(v_cache + row * v_rs + 8 * (my_quarter + 4 * i))
                                                          : make_uint4(0, 0, 0, 0);
    };
    fetch(0);
    for (int base = 0; base <= last_pos; base += kTileK) {
        __syncthreads();                                      // the previous tile has been consumed
#pragma unroll
        for (int i = 0; i < KP; ++i) {                        // rows are 8-byte aligned: two 8-byte stores
            if (my_quarter + 4 * i >= 2 * DS) continue;
            uint2* dst = (uint2*)(ldsK + my_key * k_ld + 8 * (my_quarter + 4 * i));
            dst[0] = make_uint2(kreg[i].x, kreg[i].y);
            dst[1] = make_uint2(kreg[i].z, kreg[i].w);
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            // V goes in transposed; consecutive lanes hold consecutive keys, so each of the eight 2-byte stores of a
            // wave lands in consecutive LDS words
            const int ch = my_quarter + 4 * i;
            if (ch >= 2 * DVS) continue;
            const uint32_t w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                ((unsigned short*)ldsV)[(8 * ch + 2 * e) * v_ld + my_key] = (unsigned short)(w[e] & 0xffffu);
                ((unsigned short*)ldsV)[(8 * ch + 2 * e + 1) * v_ld + my_key] = (unsigned short)(w[e] >> 16);
            }
        }
        __syncthreads();
        if (base + kTileK <= last_pos) fetch(base + kTileK);
        if (!wave_live || base > wave_last_pos) continue;     // (uniform per wave; the barriers above stay matched)
        // ---- S^T for four 16-key blocks -----------------------------------------------------------------------
        f32x4 sacc[4];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            sacc[kb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < DS; ++s) {
                const s16x4 a = *(const s16x4*)(ldsK + (kb * 16 + lq) * k_ld + 16 * s + 4 * lg);
                sacc[kb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, qf[s], sacc[kb], 0, 0, 0);
            }
        }
        // ---- modifiers, mask, running maximum -----------------------------------------------------------------
        float tmax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = base + kb * 16 + 4 * lg + i;
                float sc = sacc[kb][i] * scale;
                if (softcap > 0.f) sc = softcap * fast_tanh(sc / softcap);
                if (bias_h) sc += bias_h[min(max(my_pos - j, 0), n_dist - 1)];
                sc = j <= my_pos ? sc : -INFINITY;
                sacc[kb][i] = sc;
                tmax = fmaxf(tmax, sc);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m, tmax);                   // finite from the first tile on: key 0 is visible to all
        const float corr = __expf(m - m_new);
        m = m_new;
        l *= corr;
#pragma unroll
        for (int i = 0; i < DVS; ++i) oacc[i] *= corr;
        // ---- P^T, then O^T += V^T P^T ---------------------------------------------------------------------------
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            float p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                p[i] = __expf(sacc[kb][i] - m_new);
                l += p[i];
            }
            const uint32_t p01 = pack_bf16(p[0], p[1]), p23 = pack_bf16(p[2], p[3]);
            const s16x4 pb = __builtin_bit_cast(s16x4, make_uint2(p01, p23));
#pragma unroll
            for (int dv = 0; dv < DVS; ++dv) {
                const s16x4 a = *(const s16x4*)(ldsV + (dv * 16 + lq) * v_ld + kb * 16 + 4 * lg);
                oacc[dv] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pb, oacc[dv], 0, 0, 0);
            }
        }
    }
    if (!wave_live) return;
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (sink) {
        const float sk = sink[h];
        const float m_new = fmaxf(m, sk);
        const float corr = __expf(m - m_new);
        l = l * corr + __expf(sk - m_new);
#pragma unroll
        for (int i = 0; i < DVS; ++i) oacc[i] *= corr;
    }
    if (row0 + lq < len_q) {
        const float inv = 1.0f / l;
        __bf16* orow = out + (int64_t)(q0 + row0 + lq) * out_stride + (int64_t)h * Dv;
#pragma unroll
        for (int dv = 0; dv < DVS; ++dv) {
            const uint2 pk = make_uint2(pack_bf16(oacc[dv][0] * inv, oacc[dv][1] * inv),
                                        pack_bf16(oacc[dv][2] * inv, oacc[dv][3] * inv));
            *(uint2*)(orow + dv * 16 + 4 * lg) = pk;
        }
    }
}


// ------------------------------------------------------------------------------------------------ single rows
// Decode kernel: sequences with ONE row in the step.  A workgroup takes one (sequence, kv head) and one slice of
// the keys, for all H / G query heads of the group at once, so K and V are read once per group.  Its four waves
// split the slice; a wave walks its keys 64 at a time: lane j reads key j's row with 16-byte loads and scores it
// against every head (q sits in LDS, read as broadcasts), the weights go through LDS, then the lanes regroup for the
// value pass: a V row is cut into 16-byte pieces and the wave's load instruction covers several whole rows, each lane
// keeping one piece of every head's accumulator.  No barrier inside the loop.  The
// waves' running (max, sum, accumulator) are joined through LDS, and the slices through a workspace and a second
// small launch that also puts the sink into the denominator.
constexpr int kDecRep = 8;             // query heads per kv head handled at once (larger groups take further passes)
constexpr int kDecThreads = 256;

template <typename T> struct Vec16;
template <> struct Vec16<__bf16> { static constexpr int n = 8; };
template <> struct Vec16<float> { static constexpr int n = 4; };

template <typename T>
__device__ __forceinline__ void load16(const T* p, float* o);
template <>
__device__ __forceinline__ void load16<__bf16>(const __bf16* p, float* o) {
    const uint4 u = *(const uint4*)p;
    o[0] = bf16_lo(u.x); o[1] = bf16_hi(u.x); o[2] = bf16_lo(u.y); o[3] = bf16_hi(u.y);
    o[4] = bf16_lo(u.z); o[5] = bf16_hi(u.z); o[6] = bf16_lo(u.w); o[7] = bf16_hi(u.w);
}
template <>
__device__ __forceinline__ void load16<float>(const float* p, float* o) {
    const float4 u = *(const float4*)p;
    o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
}
// REP: query heads of a group taken per pass (1, 2, 4 or 8): the per-head registers are sized by it, so small groups
// run at high occupancy.
template <typename T, int REP>
__global__ __launch_bounds__(kDecThreads) void attn_scoremod_decode_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    float* __restrict__ ws, const int* __restrict__ cu_q, const int* __restrict__ cu_k,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int D, int Dv, int block_size, float scale,
    float softcap, const float* __restrict__ sink, const float* __restrict__ dist_bias, int n_dist, int64_t q_stride,
    int64_t out_stride, int64_t v_ld, int splits, int slice_keys, int64_t T_rows, int cpr_log2, int repm) {      // repm: heads per pass (= REP): sizes the LDS arrays
    extern __shared__ float dsm[];
    const int b = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
    const int t = cu_q[b];
    if (cu_q[b + 1] - t != 1) return;                        // rows of longer portions belong to the other kernels
    const int n_keys = cu_k[b + 1] - cu_k[b], pos = n_keys - 1;
    const int rep_all = H / G;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int VN = Vec16<T>::n;
    const int rs = 2 + Dv;
    float* qs = dsm;                                          // [repm][D]
    float* ps = qs + repm * D;                                // [4 waves][repm][64]
    float* red = ps + 4 * repm * 64;                          // [4 waves][repm][2 + Dv]
    int64_t* rws = (int64_t*)(red + 4 * repm * rs + ((4 * repm * rs + repm * D) & 1));   // [4 waves][64] rows
    const int* table = block_tables + (int64_t)b * max_blocks;
    const int k_lo = split * slice_keys, k_hi = min(n_keys, k_lo + slice_keys);
    // value pass: a V row is cut into 16-byte pieces; lane (sub, piece) = (lane >> cpr_log2, lane & (2^cpr_log2 - 1))
    // takes piece `piece` of every (64 >> cpr_log2)-th key, so one load instruction of the wave covers several whole rows
    const int piece = lane & ((1 << cpr_log2) - 1), sub = lane >> cpr_log2, rows_per_load = 64 >> cpr_log2;
    const bool piece_live = piece * VN < Dv;
    for (int h0 = 0; h0 < rep_all; h0 += REP) {
        const int rep = min(REP, rep_all - h0);
        const int head0 = g * rep_all + h0;
        __syncthreads();
        for (int i = tid; i < rep * D; i += kDecThreads)
            qs[i] = (float)q[(int64_t)t * q_stride + (int64_t)(head0 + i / D) * D + (i % D)];
        __syncthreads();
        float m[REP], l[REP], acc[REP][VN];
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            m[r] = -INFINITY;
            l[r] = 0.f;
#pragma unroll
            for (int i = 0; i < VN; ++i) acc[r][i] = 0.f;
        }
        float* pw = ps + (wave * repm) * 64;
        int64_t* rw = rws + wave * 64;
        // the slice's 64-key tiles are dealt to the four waves in turn
        for (int base = k_lo + wave * 64; base < k_hi; base += 4 * 64) {
            const int j = base + lane;
            const bool live = j < k_hi;
            float sc[REP];
#pragma unroll
            for (int r = 0; r < REP; ++r) sc[r] = 0.f;
            int64_t row = 0;
            if (live) {
                row = ((int64_t)table[j / block_size] * block_size + (j % block_size)) * G + g;
                const T* kr = k_cache + row * D;
#pragma unroll 8
                for (int d = 0; d < D; d += VN) {             // unrolled: eight 16-byte loads in flight per lane
                    float kv[VN];
                    load16<T>(kr + d, kv);
#pragma unroll
                    for (int r = 0; r < REP; ++r) {
                        if (r < rep) {
#pragma unroll
                            for (int e = 0; e < VN; ++e) sc[r] += qs[r * D + d + e] * kv[e];
                        }
                    }
                }
            }
            // a lane past the slice names the tile's first key (always live): its weight is 0, and 0 times a row that was
            // really written is 0, whatever unwritten cache memory holds
            rw[lane] = live ? row : __shfl(row, 0);
            float corr[REP];
#pragma unroll
            for (int r = 0; r < REP; ++r) {
                corr[r] = 1.f;
                if (r < rep) {
                    float x = -INFINITY;
                    if (live) {
                        x = sc[r] * scale;
                        if (softcap > 0.f) x = softcap * tanhf(x / softcap);
                        if (dist_bias) x += dist_bias[(int64_t)(head0 + r) * n_dist + min(pos - j, n_dist - 1)];
                    }
                    float tm = x;
#pragma unroll
                    for (int o = 32; o > 0; o >>= 1) tm = fmaxf(tm, __shfl_xor(tm, o));
                    const float m_new = fmaxf(m[r], tm);          // finite: the tile has at least one live key
                    const float p = live ? expf(x - m_new) : 0.f;
                    corr[r] = expf(m[r] - m_new);
                    l[r] = l[r] * corr[r] + wave_sum(p);
                    m[r] = m_new;
                    pw[r * 64 + lane] = p;
#pragma unroll
                    for (int i = 0; i < VN; ++i) acc[r][i] *= corr[r];
                }
            }
            // the tile's V rows (the wave reads its own LDS words: no workgroup barrier needed)
            if (piece_live) {
#pragma unroll 4
                for (int jj = sub; jj < 64; jj += rows_per_load) {
                    float vv[VN];
                    load16<T>(v_cache + rw[jj] * v_ld + piece * VN, vv);
#pragma unroll
                    for (int r = 0; r < REP; ++r) {
                        if (r < rep) {
                            const float pj = pw[r * 64 + jj];
#pragma unroll
                            for (int e = 0; e < VN; ++e) acc[r][e] += pj * vv[e];
                        }
                    }
                }
            }
        }
        // ---- join the lanes that share a piece, then the four waves ---------------------------------------------
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            if (r < rep) {
                for (int o = 1 << cpr_log2; o < 64; o <<= 1) {
#pragma unroll
                    for (int e = 0; e < VN; ++e) acc[r][e] += __shfl_xor(acc[r][e], o);
                }
                float* dst = red + ((wave * repm) + r) * rs;
                if (lane == 0) {
                    dst[0] = m[r];
                    dst[1] = l[r];
                }
                if (sub == 0 && piece_live) {
#pragma unroll
                    for (int e = 0; e < VN; ++e) dst[2 + piece * VN + e] = acc[r][e];
                }
            }
        }
        __syncthreads();
        for (int r = wave; r < rep; r += 4) {                 // wave w finishes heads w, w + 4, ...
            float mm = -INFINITY;
#pragma unroll
            for (int w = 0; w < 4; ++w) mm = fmaxf(mm, red[(w * repm + r) * rs]);
            float ll = 0.f, f[4];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float mw = red[(w * repm + r) * rs];
                f[w] = mw == -INFINITY ? 0.f : expf(mw - mm);  // a wave (or the whole slice) may have had no keys
                ll += f[w] * red[(w * repm + r) * rs + 1];
            }
            const int head = head0 + r;
            if (splits == 1) {
                float den = ll, osc = 1.f;
                if (sink) {
                    const float sk = sink[head], m2 = fmaxf(mm, sk);
                    osc = expf(mm - m2);
                    den = ll * osc + expf(sk - m2);
                }
                for (int c = lane; c < Dv; c += 64) {
                    float o = 0.f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) o += f[w] * red[(w * repm + r) * rs + 2 + c];
                    out[(int64_t)t * out_stride + (int64_t)head * Dv + c] = (T)(o * osc / den);
                }
            } else {
                float* wrow = ws + (((int64_t)split * T_rows + t) * H + head) * rs;
                if (lane == 0) {
                    wrow[0] = mm;
                    wrow[1] = ll;
                }
                for (int c = lane; c < Dv; c += 64) {
                    float o = 0.f;
#pragma unroll
                    for (int w = 0; w < 4; ++w) o += f[w] * red[(w * repm + r) * rs + 2 + c];
                    wrow[2 + c] = o;
                }
            }
        }
    }
}

// Joins the key slices of a single row: one wave per (sequence, head).
template <typename T>
__global__ __launch_bounds__(64) void attn_scoremod_decode_merge_kernel(
    const float* __restrict__ ws, T* __restrict__ out, const int* __restrict__ cu_q, const float* __restrict__ sink,
    int H, int Dv, int64_t out_stride, int splits, int64_t T_rows) {
    const int b = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int t = cu_q[b];
    if (cu_q[b + 1] - t != 1) return;
    const int rs = 2 + Dv;
    float mm = -INFINITY;
    for (int s = 0; s < splits; ++s) mm = fmaxf(mm, ws[(((int64_t)s * T_rows + t) * H + head) * rs]);
    float m2 = mm;
    if (sink) m2 = fmaxf(mm, sink[head]);
    float den = sink ? expf(sink[head] - m2) : 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* w = ws + (((int64_t)s * T_rows + t) * H + head) * rs;
        if (w[0] != -INFINITY) den += expf(w[0] - m2) * w[1];
    }
    for (int c = lane; c < Dv; c += 64) {
        float o = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* w = ws + (((int64_t)s * T_rows + t) * H + head) * rs;
            if (w[0] != -INFINITY) o += expf(w[0] - m2) * w[2 + c];
        }
        out[(int64_t)t * out_stride + (int64_t)head * Dv + c] = (T)(o / den);
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

namespace nv {
struct DecodePlan {
    int splits, slice_keys;
    int64_t ws_bytes;
};
// Key slices of the decode kernel: about four workgroups per CU, and never less than 64 keys per wave of a slice.
static DecodePlan decode_plan(int num_seqs, int64_t T, int H, int G, int Dv, int max_seqlen_k) {
    DecodePlan p{1, 0, 0};
    const int64_t blocks = (int64_t)num_seqs * G;
    if (max_seqlen_k > 0 && blocks > 0) {
        const int64_t want = (1024 + blocks - 1) / blocks, most = std::max(1, max_seqlen_k / 256);
        p.splits = (int)std::max<int64_t>(1, std::min<int64_t>(std::min(want, most), 64));
    }
    const int len = max_seqlen_k > 0 ? max_seqlen_k : (1 << 30);
    p.slice_keys = ((len + p.splits - 1) / p.splits + 63) / 64 * 64;
    p.ws_bytes = p.splits > 1 ? (int64_t)p.splits * T * H * (2 + Dv) * (int64_t)sizeof(float) : 0;
    return p;
}
}  // namespace nv

extern "C" int64_t nv_attn_scoremod_workspace_bytes(int num_seqs, int64_t T, int H, int G, int Dv, int max_seqlen_k) {
    if (num_seqs <= 0 || T <= 0 || H <= 0 || G <= 0 || Dv <= 0) return 0;
    return nv::decode_plan(num_seqs, T, H, G, Dv, max_seqlen_k).ws_bytes;
}

namespace nv {
// Head sizes the tile kernel is built for: every multiple of 16 up to 128, every multiple of 32 up to 320.
static bool tile_built(int n) { return n >= 32 && n % 16 == 0 && (n <= 128 || n % 32 == 0); }
struct TileArgs {
    const __bf16 *q, *k_cache, *v_cache;
    __bf16* out;
    const int *cu_q, *cu_k, *block_tables;
    int max_blocks, tiles, H, G, D, Dv, block_size;
    float scale, softcap;
    const float *sink, *dist_bias;
    int n_dist;
    int64_t q_stride, out_stride, v_ld;
};
template <int DS, int DVS>
static bool launch_tile_one(dim3 grid, size_t lds, hipStream_t s, const TileArgs& a) {
    if (lds > 64 * 1024) {      // more than the default limit of dynamic LDS: raise this instantiation's once
        static bool raised = false;
        if (!raised) {
            if (hipFuncSetAttribute((const void*)attn_scoremod_tile_kernel<DS, DVS>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    80 * 1024) != hipSuccess)
                return false;
            raised = true;
        }
    }
    hipLaunchKernelGGL((attn_scoremod_tile_kernel<DS, DVS>), grid, dim3(kTileThreads), lds, s, a.q, a.k_cache, a.v_cache, a.out,
                       a.cu_q, a.cu_k, a.block_tables, a.max_blocks, a.tiles, a.H, a.G, a.D, a.Dv, a.block_size, a.scale,
                       a.softcap, a.sink, a.dist_bias, a.n_dist, a.q_stride, a.out_stride, a.v_ld);
    return true;
}
template <int DS>
static bool launch_tile_dv(int dvs, dim3 grid, size_t lds, hipStream_t s, const TileArgs& a) {
    switch (dvs) {
#define NV_DV(N) case N: return launch_tile_one<DS, N>(grid, lds, s, a);
        NV_DV(2) NV_DV(3) NV_DV(4) NV_DV(5) NV_DV(6) NV_DV(7) NV_DV(8) NV_DV(10) NV_DV(12) NV_DV(14) NV_DV(16)
#undef NV_DV
    }
    return false;
}
static bool launch_tile(int ds, int dvs, dim3 grid, size_t lds, hipStream_t s, const TileArgs& a) {
    switch (ds) {
#define NV_D(N) case N: return launch_tile_dv<N>(dvs, grid, lds, s, a);
        NV_D(2) NV_D(3) NV_D(4) NV_D(5) NV_D(6) NV_D(7) NV_D(8) NV_D(10) NV_D(12) NV_D(14) NV_D(16) NV_D(18) NV_D(20)
#undef NV_D
    }
    return false;
}
}  // namespace nv

extern "C" int nv_attn_scoremod_paged(const void* q, const void* k_cache, const void* v_cache, void* out,
                                      const int* cu_seqlens_q, const int* cu_seqlens_k, const int* block_tables,
                                      int num_seqs, int max_blocks_per_seq, int64_t T, int H, int G, int D, int Dv,
                                      int64_t num_blocks, int block_size, float scale, float softcap,
                                      const float* sink, const float* dist_bias, int n_dist, int max_seqlen_q,
                                      int max_seqlen_k, int single_rows, int dtype, int64_t q_stride,
                                      int64_t out_stride, void* workspace, int64_t workspace_bytes, void* stream) {
    return nv_attn_scoremod_paged_vld(q, k_cache, v_cache, Dv, out, cu_seqlens_q, cu_seqlens_k, block_tables, num_seqs,
                                      max_blocks_per_seq, T, H, G, D, Dv, num_blocks, block_size, scale, softcap, sink,
                                      dist_bias, n_dist, max_seqlen_q, max_seqlen_k, single_rows, dtype, q_stride,
                                      out_stride, workspace, workspace_bytes, stream);
}

extern "C" int nv_attn_scoremod_paged_vld(const void* q, const void* k_cache, const void* v_cache, int64_t v_ld, void* out,
                                          const int* cu_seqlens_q, const int* cu_seqlens_k, const int* block_tables,
                                          int num_seqs, int max_blocks_per_seq, int64_t T, int H, int G, int D, int Dv,
                                          int64_t num_blocks, int block_size, float scale, float softcap,
                                          const float* sink, const float* dist_bias, int n_dist, int max_seqlen_q,
                                          int max_seqlen_k, int single_rows, int dtype, int64_t q_stride,
                                          int64_t out_stride, void* workspace, int64_t workspace_bytes, void* stream) {
    using namespace nv;
    NV_REQUIRE(v_ld >= Dv, NV_ERR_INVALID_ARG, "nv_attn_scoremod_paged: value row stride %lld below Dv=%d", (long long)v_ld, Dv);
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
    NV_REQUIRE(T < (1LL << 31) && H < 65536 && G < 65536, NV_ERR_UNSUPPORTED, "nv_attn_scoremod_paged: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const bool bf = dtype == NV_DTYPE_BF16;
    const bool several = max_seqlen_q != 1, singles = single_rows != 0;      // what the step may hold
    // Sequences with several rows: the MFMA tile kernel when the shapes allow (bf16, head sizes in built multiples of
    // 16, aligned rows), else the row-per-wave kernel.
    const size_t tile_lds = sizeof(__bf16) * ((size_t)kTileK * (D + 4) + (size_t)Dv * (kTileK + 4));
    const bool tile_ok = bf && max_seqlen_q > 1 && tile_built(D) && tile_built(Dv) && D <= 320 && Dv <= 256 && v_ld % 8 == 0 &&
                         tile_lds <= 80 * 1024 && q_stride % 4 == 0 && out_stride % 4 == 0 &&
                         ((uintptr_t)q | (uintptr_t)out) % 8 == 0 && ((uintptr_t)k_cache | (uintptr_t)v_cache) % 16 == 0;
    // Sequences with one row: the decode kernel (key slices, the query heads of a group together) when rows can be
    // read in 16-byte pieces, else the row-per-wave kernel.
    const int vn = bf ? 8 : 4;
    const int rep_group = std::min(kDecRep, H / G);
    const int repm = rep_group <= 2 ? rep_group : rep_group <= 4 ? 4 : 8;       // heads per pass: the kernel's REP
    const size_t dec_lds = sizeof(float) * ((size_t)repm * D + 4 * repm * 64 + 4 * repm * (2 + Dv) + 1) +
                           sizeof(int64_t) * 4 * 64;
    int cpr_log2 = 0;                                          // 16-byte pieces per V row, rounded up to a power of two
    while ((vn << cpr_log2) < Dv) ++cpr_log2;
    const bool dec_ok = singles && D % vn == 0 && Dv % vn == 0 && Dv <= 256 && v_ld % vn == 0 && cpr_log2 <= 6 && dec_lds <= 64 * 1024 &&
                        ((uintptr_t)k_cache | (uintptr_t)v_cache) % 16 == 0;
    if (several && tile_ok) {
        const int tiles = (max_seqlen_q + kTileQ - 1) / kTileQ;
        NV_REQUIRE((int64_t)num_seqs * tiles < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_attn_scoremod_paged: launch too large");
        const dim3 tgrid((unsigned)(num_seqs * tiles), (unsigned)H);
        const TileArgs ta{(const __bf16*)q, (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out, cu_seqlens_q,
                          cu_seqlens_k, block_tables, max_blocks_per_seq, tiles, H, G, D, Dv, block_size, scale, softcap,
                          sink, dist_bias, n_dist, q_stride, out_stride, v_ld};
        NV_REQUIRE(launch_tile(D / 16, Dv / 16, tgrid, tile_lds, s, ta), NV_ERR_LAUNCH,
                   "nv_attn_scoremod_paged: no tile kernel for D=%d, Dv=%d", D, Dv);
        const int rc = check_launch("nv_attn_scoremod_paged (tile kernel)");
        if (rc != NV_OK) return rc;
    }
    if (dec_ok) {
        const DecodePlan plan = decode_plan(num_seqs, T, H, G, Dv, max_seqlen_k);
        NV_REQUIRE(plan.ws_bytes == 0 || (workspace && workspace_bytes >= plan.ws_bytes), NV_ERR_WORKSPACE,
                   "nv_attn_scoremod_paged: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
                   (long long)plan.ws_bytes);
        const dim3 dgrid((unsigned)num_seqs, (unsigned)G, (unsigned)plan.splits);
#define NV_DEC_ARGS(TT)                                                                                              \
    (const TT*)q, (const TT*)k_cache, (const TT*)v_cache, (TT*)out, (float*)workspace, cu_seqlens_q, cu_seqlens_k, \
        block_tables, max_blocks_per_seq, H, G, D, Dv, block_size, scale, softcap, sink, dist_bias, n_dist,        \
        q_stride, out_stride, v_ld, plan.splits, plan.slice_keys, T, cpr_log2, repm
#define NV_DEC_LAUNCH(TT, R) \
    hipLaunchKernelGGL((attn_scoremod_decode_kernel<TT, R>), dgrid, dim3(kDecThreads), dec_lds, s, NV_DEC_ARGS(TT))
#define NV_DEC_BY_REP(TT)                     \
    if (repm == 1) NV_DEC_LAUNCH(TT, 1);      \
    else if (repm == 2) NV_DEC_LAUNCH(TT, 2); \
    else if (repm <= 4) NV_DEC_LAUNCH(TT, 4); \
    else NV_DEC_LAUNCH(TT, 8);
        if (bf) { NV_DEC_BY_REP(__bf16) } else { NV_DEC_BY_REP(float) }
#undef NV_DEC_BY_REP
#undef NV_DEC_LAUNCH
#undef NV_DEC_ARGS
        int rc = check_launch("nv_attn_scoremod_paged (decode kernel)");
        if (rc != NV_OK) return rc;
        if (plan.splits > 1) {
            const dim3 mgrid((unsigned)num_seqs, (unsigned)H);
            if (bf)
                hipLaunchKernelGGL(attn_scoremod_decode_merge_kernel<__bf16>, mgrid, dim3(64), 0, s, (const float*)workspace,
                                   (__bf16*)out, cu_seqlens_q, sink, H, Dv, out_stride, plan.splits, T);
            else
                hipLaunchKernelGGL(attn_scoremod_decode_merge_kernel<float>, mgrid, dim3(64), 0, s, (const float*)workspace,
                                   (float*)out, cu_seqlens_q, sink, H, Dv, out_stride, plan.splits, T);
            rc = check_launch("nv_attn_scoremod_paged (decode merge)");
            if (rc != NV_OK) return rc;
        }
    }
    // what is left for the row-per-wave kernel: 0 = every row, 1 = single rows only, 2 = longer portions only
    const bool rw_several = several && !tile_ok, rw_singles = singles && !dec_ok;
    if (!rw_several && !rw_singles) return NV_OK;
    const int only = rw_several && rw_singles ? 0 : rw_singles ? 1 : 2;
    const size_t smem = sizeof(float) * (D + 64 + (D & 1)) + sizeof(int64_t) * 64;
    const dim3 grid((unsigned)T, (unsigned)H);
    if (bf)
        hipLaunchKernelGGL(attn_scoremod_rowwave_kernel<__bf16>, grid, dim3(64), smem, s, (const __bf16*)q,
                           (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out, cu_seqlens_q, cu_seqlens_k,
                           block_tables, num_seqs, max_blocks_per_seq, H, G, D, Dv, block_size, scale, softcap, sink,
                           dist_bias, n_dist, q_stride, out_stride, v_ld, only);
    else
        hipLaunchKernelGGL(attn_scoremod_rowwave_kernel<float>, grid, dim3(64), smem, s, (const float*)q,
                           (const float*)k_cache, (const float*)v_cache, (float*)out, cu_seqlens_q, cu_seqlens_k,
                           block_tables, num_seqs, max_blocks_per_seq, H, G, D, Dv, block_size, scale, softcap, sink,
                           dist_bias, n_dist, q_stride, out_stride, v_ld, only);
    return check_launch("nv_attn_scoremod_paged");
}
