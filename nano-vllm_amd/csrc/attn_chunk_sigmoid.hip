// Sigmoid attention inside fixed chunks of positions, with rotated values, over the paged cache.
//
//   visible(i, j):  j <= i  and  floor(i / chunk) == floor(j / chunk)        (chunks counted from position 0; chunk = 0:
//                                                                             every earlier key is visible)
//   a_ij = sigmoid(scale * q_i . k_j + bias_h)                                one weight per visible key, not
//                                                                             normalised over the keys
//   o_i  = R(-i) sum_j a_ij R(j) v_j                                          R(p): every pair (m, m + Dv/2) of a value
//                                                                             turned by p * value_freq[m]
//
// Values are cached ROTATED (R(j) v_j); the kernel turns the sum back by the query's position.  Grouped heads (query
// head h reads kv head h / (H / G)), any head size; K/V are read through the block table of a paged cache
// [num_blocks, block_size, G, D | Dv] with a runtime block size; a step's rows may be prompt portions and single decoded
// tokens side by side (query i of a sequence sits at position len_k - len_q + i).
//
// nv_chunk_attn_prep_store runs in front of it: RMS norm over the WHOLE q row and the whole k row (all heads at once,
// one weight per column), rotate-half rotary on the first rot_dims dimensions of every q / k head (pair (i, i + rot_dims/2),
// angle = position * freq[i] as an fp32 product, full-precision sincosf), the value rotation, and the scatter of the
// step's K/V rows into the cache.
//
// Two attention kernels: one wave per (query, kv head) in fp32 arithmetic for any element type and size (single rows,
// float32 models; the heads of a group share every key and value read), and a bf16 MFMA tile kernel for prompt portions
// (64 queries of one head per workgroup).
#include <algorithm>

#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

__device__ __forceinline__ float cs_block_sum(float x, float* red, int n_waves) {
    x = wave_sum(x);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < n_waves; ++i) t += red[i];
    return t;
}

// ------------------------------------------------------------------------------------------------ prep
template <typename T>
__global__ __launch_bounds__(256) void chunk_attn_prep_store_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t q_stride, int64_t k_stride,
    int64_t v_stride, const float* __restrict__ q_norm, const float* __restrict__ k_norm, float eps,
    const float* __restrict__ freq, int rot_dims, const float* __restrict__ vfreq, const int64_t* __restrict__ positions,
    const int* __restrict__ slot_mapping, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int H,
    int G, int D, int Dv) {
    __shared__ float red[4];
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x;
    const float pos = (float)positions[t];
    const int slot = slot_mapping ? slot_mapping[t] : -1;
    const T* qr = q + t * q_stride;
    const T* kr = k + t * k_stride;
    float sq = 0.f, sk = 0.f;
    for (int c = tid; c < H * D; c += 256) {
        const float x = (float)qr[c];
        sq += x * x;
    }
    for (int c = tid; c < G * D; c += 256) {
        const float x = (float)kr[c];
        sk += x * x;
    }
    sq = cs_block_sum(sq, red, 4);
    sk = cs_block_sum(sk, red, 4);
    const float rq = 1.0f / sqrtf(sq / (float)(H * D) + eps), rk = 1.0f / sqrtf(sk / (float)(G * D) + eps);
    const int half = rot_dims / 2;
    // q heads then k heads; a thread takes one rotated pair, or one unrotated dimension behind the rotated part
    const int per_head = half + (D - rot_dims);
    for (int idx = tid; idx < (H + G) * per_head; idx += 256) {
        const int head = idx / per_head, e = idx - head * per_head;
        const bool is_q = head < H;
        const int hh = is_q ? head : head - H;
        const T* src = (is_q ? qr : kr) + (int64_t)hh * D;
        const float* nw = (is_q ? q_norm : k_norm) + (int64_t)hh * D;
        const float rs = is_q ? rq : rk;
        T* dst = is_q ? q_out + (t * H + hh) * (int64_t)D : (slot >= 0 ? k_cache + ((int64_t)slot * G + hh) * D : nullptr);
        if (dst == nullptr) continue;
        if (e < half) {
            const float a = (float)src[e] * rs * nw[e], b = (float)src[e + half] * rs * nw[e + half];
            float sn, cs;
            sincosf(pos * freq[e], &sn, &cs);
            dst[e] = (T)(a * cs - b * sn);
            dst[e + half] = (T)(b * cs + a * sn);
        } else {
            const int d = rot_dims + (e - half);
            dst[d] = (T)((float)src[d] * rs * nw[d]);
        }
    }
    if (slot >= 0) {
        const int vh = Dv / 2;
        for (int idx = tid; idx < G * vh; idx += 256) {
            const int g = idx / vh, m = idx - g * vh;
            const T* src = v + t * v_stride + (int64_t)g * Dv;
            T* dst = v_cache + ((int64_t)slot * G + g) * Dv;
            const float a = (float)src[m], b = (float)src[m + vh];
            float sn, cs;
            sincosf(pos * vfreq[m], &sn, &cs);
            dst[m] = (T)(a * cs - b * sn);
            dst[m + vh] = (T)(b * cs + a * sn);
        }
    }
}

// ------------------------------------------------------------------------------------------------ one wave per row
// One wave per (query token, kv head), for the REP query heads of the group at once (a group with more heads takes
// several passes), so a cached key or value is read once per group.  Keys go by in tiles of 64: lane j scores key j of
// the tile against every head (its own K row, the q rows broadcast from LDS), the tile's weights go through LDS, then the
// lanes switch to value channels (lane c accumulates channels c, c + 64, ... of every head) and stream the tile's V rows,
// which are contiguous per key.
constexpr int kCsMaxDvPerLane = 8;   // Dv <= 512

template <typename T, int REP>
__global__ __launch_bounds__(64) void attn_chunk_sigmoid_rowwave_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    const int* __restrict__ cu_q, const int* __restrict__ cu_k, const int* __restrict__ block_tables, int B,
    int max_blocks, int H, int G, int D, int Dv, int block_size, float scale, const float* __restrict__ head_bias,
    int chunk, const float* __restrict__ vfreq, int64_t q_stride, int64_t out_stride, int only_single_rows) {
    extern __shared__ float smem[];
    float* qs = smem;                      // [REP][D]
    float* ps = qs + REP * D;              // [REP][64]
    float* os = ps + REP * 64;             // [Dv]
    int64_t* rows = (int64_t*)(os + Dv + ((REP * D + Dv) & 1));   // [64] element offsets of the tile's cache rows
    const int t = blockIdx.x, g = blockIdx.y, lane = threadIdx.x;
    int lo = 0, hi = B;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid;
    }
    const int b = lo;
    const int len_q = cu_q[b + 1] - cu_q[b], len_k = cu_k[b + 1] - cu_k[b];
    // only_single_rows: 0 = every row, 1 = sequences with one row only, 2 = sequences with several rows only
    if ((only_single_rows == 1 && len_q != 1) || (only_single_rows == 2 && len_q == 1)) return;
    const int pos = len_k - len_q + (t - cu_q[b]);      // this query's position
    const int first = chunk > 0 ? (pos / chunk) * chunk : 0;     // it sees keys first .. pos
    const int per = H / G, vh = Dv / 2;
    const int* table = block_tables + (int64_t)b * max_blocks;
    for (int h0 = 0; h0 < per; h0 += REP) {
        const int n = min(REP, per - h0);                // heads of this pass: g * per + h0 .. + n - 1
        __syncthreads();                                 // the previous pass is done with qs, ps, os
        for (int i = lane; i < n * D; i += 64)
            qs[i] = (float)q[(int64_t)t * q_stride + (int64_t)(g * per + h0) * D + i];
        float hb[REP];
#pragma unroll
        for (int r = 0; r < REP; ++r) hb[r] = (head_bias && r < n) ? head_bias[g * per + h0 + r] : 0.f;
        float acc[REP][kCsMaxDvPerLane] = {};
        __syncthreads();
        for (int base = first; base <= pos; base += 64) {
            const int j = base + lane;
            float dot[REP] = {};
            int64_t row = 0;
            if (j <= pos) {
                const int blk = table[j / block_size];
                row = ((int64_t)blk * block_size + (j % block_size)) * G + g;
                const T* kr = k_cache + row * D;
                for (int d = 0; d < D; ++d) {
                    const float kd = (float)kr[d];
#pragma unroll
                    for (int r = 0; r < REP; ++r) dot[r] += qs[r * D + d] * kd;      // (rows past n hold stale, finite values)
                }
            }
            __syncthreads();                                     // previous tile's readers are done
#pragma unroll
            for (int r = 0; r < REP; ++r) ps[r * 64 + lane] = (j <= pos && r < n) ? 1.0f / (1.0f + expf(-(dot[r] * scale + hb[r]))) : 0.f;
            rows[lane] = row;
            __syncthreads();
            const int n_tile = min(64, pos + 1 - base);
            for (int jj = 0; jj < n_tile; ++jj) {
                const T* vr = v_cache + rows[jj] * Dv;
#pragma unroll
                for (int i = 0; i < kCsMaxDvPerLane; ++i) {
                    const int c = lane + 64 * i;
                    if (c < Dv) {
                        const float vv = (float)vr[c];
#pragma unroll
                        for (int r = 0; r < REP; ++r) acc[r][i] += ps[r * 64 + jj] * vv;
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < REP; ++r) {
            if (r >= n) break;
            __syncthreads();                                     // the previous head's pairs have been read
#pragma unroll
            for (int i = 0; i < kCsMaxDvPerLane; ++i) {
                const int c = lane + 64 * i;
                if (c < Dv) os[c] = acc[r][i];
            }
            __syncthreads();
            T* dst = out + (int64_t)t * out_stride + (int64_t)(g * per + h0 + r) * Dv;
            for (int m = lane; m < vh; m += 64) {
                const float a = os[m], bb = os[m + vh];
                float sn, cs;
                sincosf((float)pos * vfreq[m], &sn, &cs);        // turned back: angle -pos * f
                dst[m] = (T)(a * cs + bb * sn);
                dst[m + vh] = (T)(bb * cs - a * sn);
            }
        }
    }
}

template <typename T>
static void launch_cs_rowwave(int rep, dim3 grid, hipStream_t s, const T* q, const T* kc, const T* vc, T* out, const int* cu_q,
                              const int* cu_k, const int* bt, int B, int max_blocks, int H, int G, int D, int Dv, int block_size,
                              float scale, const float* hb, int chunk, const float* vfreq, int64_t q_stride, int64_t out_stride,
                              int mode) {
    const size_t smem = sizeof(float) * (size_t)(rep * D + rep * 64 + Dv + ((rep * D + Dv) & 1)) + sizeof(int64_t) * 64;
#define NV_CS_ROW(R)                                                                                                       \
    hipLaunchKernelGGL((attn_chunk_sigmoid_rowwave_kernel<T, R>), grid, dim3(64), smem, s, q, kc, vc, out, cu_q, cu_k, bt, B, \
                       max_blocks, H, G, D, Dv, block_size, scale, hb, chunk, vfreq, q_stride, out_stride, mode)
    if (rep == 1) NV_CS_ROW(1);
    else if (rep == 2) NV_CS_ROW(2);
    else if (rep == 4) NV_CS_ROW(4);
    else NV_CS_ROW(8);
#undef NV_CS_ROW
}

// ------------------------------------------------------------------------------------------------ prompt portions
// bf16 MFMA kernel for sequences with several query rows.  A workgroup of four waves takes 64 consecutive queries of
// one (sequence, head); a wave owns 16 of them.  Key tiles of 64 go through LDS once per workgroup: K as stored
// ([key][d]) and V transposed ([dv][key]).  Everything is computed transposed, so that one lane keeps one query:
//     S^T (keys x queries) = K Q^T        v_mfma_f32_16x16x16_bf16: A = K rows from LDS, B = Q^T held in registers
//     O^T (dv x queries)  += V^T P^T      A = V^T rows from LDS, B = P^T, which is the accumulator layout of S^T as is
// Lane l holds query l % 16 in every accumulator and the four consecutive keys 4 (l / 16) .. + 3 of each 16-key block.
// There is no running maximum and no denominator: a weight is a sigmoid of its own score.  A tile's keys start at the
// chunk start of the workgroup's first query; a query whose chunk starts later masks the keys in front of it.
constexpr int kCsTileQ = 64, kCsTileK = 64, kCsThreads = 256;

template <int DS, int DVS>     // D = 16 DS, Dv = 16 DVS
__global__ __launch_bounds__(kCsThreads, 2) void attn_chunk_sigmoid_tile_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k_cache, const __bf16* __restrict__ v_cache,
    __bf16* __restrict__ out, const int* __restrict__ cu_q, const int* __restrict__ cu_k,
    const int* __restrict__ block_tables, int B, int max_blocks, int H, int G, int block_size, float scale,
    const float* __restrict__ head_bias, int chunk, const float* __restrict__ vfreq, int64_t q_stride, int64_t out_stride,
    const int* __restrict__ tile_seq, const int* __restrict__ tile_q0) {
    constexpr int D = 16 * DS, Dv = 16 * DVS;
    constexpr int KLD = D + 8;             // bf16 elements per K row in LDS (16-byte rows, banks spread)
    constexpr int VLD = kCsTileK + 8;      // bf16 elements per V^T row
    extern __shared__ __attribute__((aligned(16))) unsigned char cs_smem[];
    __bf16* Ks = (__bf16*)cs_smem;                        // [64][KLD]
    __bf16* Vt = Ks + kCsTileK * KLD;                     // [Dv][VLD]
    const int tile = blockIdx.x, h = blockIdx.y;
    const int b = tile_seq[tile], qt0 = tile_q0[tile];    // sequence, first query row (within the sequence's portion)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int len_q = cu_q[b + 1] - cu_q[b], len_k = cu_k[b + 1] - cu_k[b];
    const int start = len_k - len_q;
    const int g = h / (H / G);
    const int l16 = lane & 15, lg = lane >> 4;
    const int qi = qt0 + wave * 16 + l16;                 // this lane's query row within the portion
    const bool q_live = qi < len_q;
    const int pos = start + min(qi, len_q - 1);
    const int first = chunk > 0 ? (pos / chunk) * chunk : 0;
    const int pos_lo = start + qt0, pos_hi = start + min(qt0 + kCsTileQ, len_q) - 1;
    const int key_lo = chunk > 0 ? (pos_lo / chunk) * chunk : 0;
    // Q^T as the B operand: lane holds q[query l16][d = 16 s + 4 lg .. + 3]
    s16x4 qb[DS];
    {
        const __bf16* qr = q + (int64_t)(cu_q[b] + min(qi, len_q - 1)) * q_stride + (int64_t)h * D;
#pragma unroll
        for (int s = 0; s < DS; ++s) qb[s] = *(const s16x4*)(qr + 16 * s + 4 * lg);
    }
    f32x4 oacc[DVS];
#pragma unroll
    for (int i = 0; i < DVS; ++i) oacc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    const float hb = head_bias ? head_bias[h] : 0.f;
    const int* table = block_tables + (int64_t)b * max_blocks;
    for (int kb = key_lo; kb <= pos_hi; kb += kCsTileK) {
        __syncthreads();                                  // the previous tile's readers are done
        // K rows as stored, 16 bytes at a time; V transposed
        for (int i = tid; i < kCsTileK * (D / 8); i += kCsThreads) {
            const int kk = i / (D / 8), c8 = i % (D / 8);
            const int j = kb + kk;
            uint4 val = make_uint4(0, 0, 0, 0);
            if (j <= pos_hi) {
                const int64_t row = ((int64_t)table[j / block_size] * block_size + (j % block_size)) * G + g;
                val = *(const uint4*)(k_cache + row * D + 8 * c8);
            }
            *(uint4*)(Ks + kk * KLD + 8 * c8) = val;
        }
        for (int i = tid; i < kCsTileK * (Dv / 8); i += kCsThreads) {
            const int kk = i % kCsTileK, c8 = i / kCsTileK;
            const int j = kb + kk;
            uint4 val = make_uint4(0, 0, 0, 0);
            if (j <= pos_hi) {
                const int64_t row = ((int64_t)table[j / block_size] * block_size + (j % block_size)) * G + g;
                val = *(const uint4*)(v_cache + row * Dv + 8 * c8);
            }
            const __bf16* e = (const __bf16*)&val;
#pragma unroll
            for (int x = 0; x < 8; ++x) Vt[(8 * c8 + x) * VLD + kk] = e[x];
        }
        __syncthreads();
#pragma unroll
        for (int kblk = 0; kblk < kCsTileK / 16; ++kblk) {
            // S^T block: keys 16 kblk .. + 15 (rows) x this wave's 16 queries (columns)
            f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < DS; ++s) {
                const s16x4 ka = *(const s16x4*)(Ks + (16 * kblk + l16) * KLD + 16 * s + 4 * lg);
                sacc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ka, qb[s], sacc, 0, 0, 0);
            }
            // lane holds keys 16 kblk + 4 lg + i (i = 0..3) of query l16
            s16x4 pb;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = kb + 16 * kblk + 4 * lg + i;
                const bool vis = q_live && j >= first && j <= pos;
                const float p = vis ? 1.0f / (1.0f + __expf(-(sacc[i] * scale + hb))) : 0.f;
                pb[i] = __builtin_bit_cast(short, (__bf16)p);
            }
#pragma unroll
            for (int dv = 0; dv < DVS; ++dv) {
                const s16x4 va = *(const s16x4*)(Vt + (16 * dv + l16) * VLD + 16 * kblk + 4 * lg);
                oacc[dv] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(va, pb, oacc[dv], 0, 0, 0);
            }
        }
    }
    // O^T: lane holds channels 16 dv + 4 lg + i of query l16.  The partner of channel c is c +- Dv / 2, i.e. the
    // accumulator DVS / 2 further (Dv / 2 is a multiple of 8 here, so the partner sits in the same lane when DVS is
    // even; else through LDS).
    if constexpr (DVS % 2 == 0) {
        if (q_live) {
            __bf16* dst = out + (int64_t)(cu_q[b] + qi) * out_stride + (int64_t)h * Dv;
#pragma unroll
            for (int dv = 0; dv < DVS / 2; ++dv) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int m = 16 * dv + 4 * lg + i;
                    float sn, cs;
                    sincosf((float)pos * vfreq[m], &sn, &cs);
                    const float a = oacc[dv][i], bb = oacc[dv + DVS / 2][i];
                    dst[m] = (__bf16)(a * cs + bb * sn);
                    dst[m + Dv / 2] = (__bf16)(bb * cs - a * sn);
                }
            }
        }
    } else {
        __syncthreads();
        float* ob = (float*)cs_smem + (wave * 16 + l16) * (Dv + 1);      // [64 queries][Dv + 1]
#pragma unroll
        for (int dv = 0; dv < DVS; ++dv)
#pragma unroll
            for (int i = 0; i < 4; ++i) ob[16 * dv + 4 * lg + i] = oacc[dv][i];
        __syncthreads();
        if (q_live) {
            __bf16* dst = out + (int64_t)(cu_q[b] + qi) * out_stride + (int64_t)h * Dv;
            for (int m = lg; m < Dv / 2; m += 4) {
                float sn, cs;
                sincosf((float)pos * vfreq[m], &sn, &cs);
                const float a = ob[m], bb = ob[m + Dv / 2];
                dst[m] = (__bf16)(a * cs + bb * sn);
                dst[m + Dv / 2] = (__bf16)(bb * cs - a * sn);
            }
        }
    }
}

template <int DS, int DVS>
static void launch_cs_tile(dim3 grid, size_t lds, hipStream_t s, const __bf16* q, const __bf16* kc, const __bf16* vc,
                           __bf16* out, const int* cu_q, const int* cu_k, const int* bt, int B, int max_blocks, int H, int G,
                           int block_size, float scale, const float* hb, int chunk, const float* vfreq, int64_t q_stride,
                           int64_t out_stride, const int* tile_seq, const int* tile_q0) {
    hipLaunchKernelGGL((attn_chunk_sigmoid_tile_kernel<DS, DVS>), grid, dim3(kCsThreads), lds, s, q, kc, vc, out, cu_q, cu_k,
                       bt, B, max_blocks, H, G, block_size, scale, hb, chunk, vfreq, q_stride, out_stride, tile_seq, tile_q0);
}

}  // namespace nv

extern "C" int nv_chunk_attn_prep_store(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                                        int64_t v_stride, const float* q_norm, const float* k_norm, float eps,
                                        const float* freq, int rot_dims, const float* value_freq,
                                        const int64_t* positions, const int32_t* slot_mapping, void* q_out,
                                        void* k_cache, void* v_cache, int dtype, int64_t T, int H, int G, int D, int Dv,
                                        void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && H > 0 && G > 0 && D > 0 && Dv > 0, NV_ERR_INVALID_ARG, "nv_chunk_attn_prep_store: bad sizes");
    if (T == 0) return NV_OK;
    NV_REQUIRE(q && k && v && q_norm && k_norm && value_freq && positions && q_out, NV_ERR_INVALID_ARG,
               "nv_chunk_attn_prep_store: null pointer");
    NV_REQUIRE(rot_dims >= 0 && rot_dims <= D && rot_dims % 2 == 0 && (rot_dims == 0 || freq), NV_ERR_INVALID_ARG,
               "nv_chunk_attn_prep_store: rot_dims=%d must be even and at most D=%d", rot_dims, D);
    NV_REQUIRE(Dv % 2 == 0, NV_ERR_INVALID_ARG, "nv_chunk_attn_prep_store: the value size %d must be even", Dv);
    NV_REQUIRE(!slot_mapping || (k_cache && v_cache), NV_ERR_INVALID_ARG, "nv_chunk_attn_prep_store: slots without caches");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_chunk_attn_prep_store: bad dtype");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_chunk_attn_prep_store: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(chunk_attn_prep_store_kernel<__bf16>, dim3((unsigned)T), dim3(256), 0, s, (const __bf16*)q,
                           (const __bf16*)k, (const __bf16*)v, q_stride, k_stride, v_stride, q_norm, k_norm, eps, freq,
                           rot_dims, value_freq, positions, slot_mapping, (__bf16*)q_out, (__bf16*)k_cache,
                           (__bf16*)v_cache, H, G, D, Dv);
    else
        hipLaunchKernelGGL(chunk_attn_prep_store_kernel<float>, dim3((unsigned)T), dim3(256), 0, s, (const float*)q,
                           (const float*)k, (const float*)v, q_stride, k_stride, v_stride, q_norm, k_norm, eps, freq,
                           rot_dims, value_freq, positions, slot_mapping, (float*)q_out, (float*)k_cache, (float*)v_cache,
                           H, G, D, Dv);
    return check_launch("nv_chunk_attn_prep_store");
}

extern "C" int nv_attn_chunk_sigmoid_tile_ok(int D, int Dv, int dtype) {
    return dtype == NV_DTYPE_BF16 && (D == 64 || D == 128) && (Dv == 64 || Dv == 128) ? 1 : 0;
}

extern "C" int nv_attn_chunk_sigmoid_paged(const void* q, const void* k_cache, const void* v_cache, void* out,
                                           const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                                           const int32_t* block_tables, int num_seqs, int max_blocks, int64_t T, int H,
                                           int G, int D, int Dv, int64_t num_blocks, int block_size, float scale,
                                           const float* head_bias, int chunk, const float* value_freq,
                                           const int32_t* tile_seq, const int32_t* tile_q0, int num_tiles,
                                           int single_rows, int dtype, int64_t q_stride, int64_t out_stride,
                                           void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && T >= 0 && H > 0 && G > 0 && D > 0 && Dv > 0 && block_size > 0 && num_blocks > 0,
               NV_ERR_INVALID_ARG, "nv_attn_chunk_sigmoid_paged: bad sizes");
    if (T == 0 || num_seqs == 0) return NV_OK;
    NV_REQUIRE(q && k_cache && v_cache && out && cu_seqlens_q && cu_seqlens_k && block_tables && value_freq,
               NV_ERR_INVALID_ARG, "nv_attn_chunk_sigmoid_paged: null pointer");
    NV_REQUIRE(H % G == 0, NV_ERR_INVALID_ARG, "nv_attn_chunk_sigmoid_paged: H=%d not a multiple of G=%d", H, G);
    NV_REQUIRE(Dv % 2 == 0 && Dv <= 64 * kCsMaxDvPerLane, NV_ERR_UNSUPPORTED,
               "nv_attn_chunk_sigmoid_paged: the value size %d must be even and at most %d", Dv, 64 * kCsMaxDvPerLane);
    NV_REQUIRE(chunk >= 0, NV_ERR_INVALID_ARG, "nv_attn_chunk_sigmoid_paged: negative chunk");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_attn_chunk_sigmoid_paged: bad dtype");
    NV_REQUIRE(T < (1LL << 31) && H < 65536, NV_ERR_UNSUPPORTED, "nv_attn_chunk_sigmoid_paged: launch too large");
    hipStream_t s = (hipStream_t)stream;
    // prompt portions on the MFMA tile kernel when it is built for the sizes and the host has laid out the tiles;
    // the one-wave-per-row kernel takes the rest (every row without tiles)
    int rowwave_mode = 0;
    if (num_tiles > 0) {
        NV_REQUIRE(tile_seq && tile_q0, NV_ERR_INVALID_ARG, "nv_attn_chunk_sigmoid_paged: tiles without their tables");
        NV_REQUIRE(nv_attn_chunk_sigmoid_tile_ok(D, Dv, dtype), NV_ERR_UNSUPPORTED,
                   "nv_attn_chunk_sigmoid_paged: no tile kernel for D=%d, Dv=%d", D, Dv);
        NV_REQUIRE(q_stride % 4 == 0 && ((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache) % 16 == 0,
                   NV_ERR_INVALID_ARG, "nv_attn_chunk_sigmoid_paged: the tile kernel needs 16-byte aligned rows");
        const dim3 grid((unsigned)num_tiles, (unsigned)H);
        const size_t lds_kv = sizeof(__bf16) * ((size_t)kCsTileK * (D + 8) + (size_t)Dv * (kCsTileK + 8));
        const size_t lds = std::max(lds_kv, sizeof(float) * (size_t)kCsTileQ * (Dv + 1));
#define NV_CS_TILE(DS, DVS)                                                                                                \
    launch_cs_tile<DS, DVS>(grid, lds, s, (const __bf16*)q, (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out, \
                            cu_seqlens_q, cu_seqlens_k, block_tables, num_seqs, max_blocks, H, G, block_size, scale,       \
                            head_bias, chunk, value_freq, q_stride, out_stride, tile_seq, tile_q0)
        if (D == 64 && Dv == 64) NV_CS_TILE(4, 4);
        else if (D == 64 && Dv == 128) NV_CS_TILE(4, 8);
        else if (D == 128 && Dv == 64) NV_CS_TILE(8, 4);
        else NV_CS_TILE(8, 8);
#undef NV_CS_TILE
        int rc = check_launch("nv_attn_chunk_sigmoid_paged (tiles)");
        if (rc != NV_OK) return rc;
        if (single_rows == 0) return NV_OK;                 // the step has no single rows
        rowwave_mode = 1;
    }
    // query heads taken per pass: the group's, rounded up to 1, 2, 4 or 8; fewer when the q rows would not fit into LDS
    const int per = H / G;
    int rep = per <= 1 ? 1 : per <= 2 ? 2 : per <= 4 ? 4 : 8;
    while (rep > 1 && sizeof(float) * (size_t)rep * (D + 64) > 40 * 1024) rep /= 2;
    NV_REQUIRE(sizeof(float) * (size_t)(D + 64 + Dv + 1) + 512 <= 60 * 1024, NV_ERR_UNSUPPORTED,
               "nv_attn_chunk_sigmoid_paged: key size %d too large", D);
    const dim3 grid((unsigned)T, (unsigned)G);
    if (dtype == NV_DTYPE_BF16)
        launch_cs_rowwave<__bf16>(rep, grid, s, (const __bf16*)q, (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out,
                                  cu_seqlens_q, cu_seqlens_k, block_tables, num_seqs, max_blocks, H, G, D, Dv, block_size, scale,
                                  head_bias, chunk, value_freq, q_stride, out_stride, rowwave_mode);
    else
        launch_cs_rowwave<float>(rep, grid, s, (const float*)q, (const float*)k_cache, (const float*)v_cache, (float*)out,
                                 cu_seqlens_q, cu_seqlens_k, block_tables, num_seqs, max_blocks, H, G, D, Dv, block_size, scale,
                                 head_bias, chunk, value_freq, q_stride, out_stride, rowwave_mode);
    return check_launch("nv_attn_chunk_sigmoid_paged");
}
