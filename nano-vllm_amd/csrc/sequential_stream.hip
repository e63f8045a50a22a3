// An fp32 residual stream whose sublayers run one after the other (pre-norm), each output scaled per column on its way
// in, and what stands around its attention and feed-forward sublayers.
//
// nv_stream_boundary_scaled  per row, in place on the fp32 stream r:
//                                r <- r + ls * (a1 + sigmoid(g) a2 + sum_j p_j)    (a1, a2 in the matmul dtype, g one raw
//                                                                                  gate per row for a2, p_j fp32 parts such
//                                                                                  as the weighted outputs of the chosen
//                                                                                  experts, ls a scale per column; each
//                                                                                  may be absent)
//                                y32 / y <- r / sqrt(mean(r^2) + eps) * w          (fp32 and / or the matmul dtype; may
//                                                                                  be absent)
//                            so the stream is read and written once per sublayer.
// nv_poly_norm               y = a z / rms(z) + b z^2 / rms(z^2) + c z^3 / rms(z^3) + e per row, powers element by element,
//                            rms(u) = sqrt(mean(u^2) + eps) over the row, everything in fp32.
// nv_head_norm_rope_store    in front of nv_attn_scoremod_paged when queries and keys are RMS-normed per head (one weight
//                            [D] for all heads) and then rotated on their first rot_dims dimensions (pair (i, i + rot_dims/2)
//                            by position * freq[i]): writes the prepared queries, scatters the prepared keys into the key
//                            cache and the UNPREPARED keys into the value cache (this attention reads its values from the
//                            keys as they come in).
#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kSsThreads = 256;

__device__ __forceinline__ float ss_block_sum(float x, float* red) {
    x = wave_sum(x);
    const int w = threadIdx.x >> 6;
    __syncthreads();                       // red may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) red[w] = x;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kSsThreads / 64; ++i) t += red[i];
    return t;
}

template <typename T>
__global__ __launch_bounds__(kSsThreads) void stream_boundary_scaled_kernel(
    float* __restrict__ resid, const T* __restrict__ add1, int64_t add1_stride, const T* __restrict__ add2,
    int64_t add2_stride, const T* __restrict__ gate2, int64_t gate2_stride, const float* __restrict__ parts, int n_parts,
    const float* __restrict__ col_scale, const float* __restrict__ norm_w, float eps, float* __restrict__ y32,
    T* __restrict__ y, int cols) {
    extern __shared__ float row[];
    __shared__ float red[kSsThreads / 64];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    float* rrow = resid + r * cols;
    const float g2 = (add2 != nullptr && gate2 != nullptr) ? 1.0f / (1.0f + expf(-(float)gate2[r * gate2_stride])) : 1.0f;
    float ss = 0.f;
    for (int c = tid; c < cols; c += kSsThreads) {
        float s = 0.f;
        if (add1 != nullptr) s += (float)add1[r * add1_stride + c];
        if (add2 != nullptr) s += g2 * (float)add2[r * add2_stride + c];
        for (int j = 0; j < n_parts; ++j) s += parts[(r * n_parts + j) * cols + c];
        if (col_scale != nullptr) s *= col_scale[c];
        const float v = rrow[c] + s;
        if (add1 != nullptr || add2 != nullptr || n_parts > 0) rrow[c] = v;
        row[c] = v;
        ss += v * v;
    }
    if (norm_w == nullptr) return;
    const float rstd = 1.0f / sqrtf(ss_block_sum(ss, red) / (float)cols + eps);
    for (int c = tid; c < cols; c += kSsThreads) {         // a thread reads back its own columns only
        const float u = row[c] * rstd * norm_w[c];
        if (y32 != nullptr) y32[r * cols + c] = u;
        if (y != nullptr) y[r * cols + c] = (T)u;
    }
}

// 16 bytes of a row as floats (8 bfloat16 or 4 float32).
template <typename T> struct SsPiece;
template <> struct SsPiece<__bf16> {
    static constexpr int n = 8;
    static __device__ __forceinline__ void load(const __bf16* p, float* o) {
        const uint4 u = *(const uint4*)p;
        o[0] = bf16_lo(u.x); o[1] = bf16_hi(u.x); o[2] = bf16_lo(u.y); o[3] = bf16_hi(u.y);
        o[4] = bf16_lo(u.z); o[5] = bf16_hi(u.z); o[6] = bf16_lo(u.w); o[7] = bf16_hi(u.w);
    }
    static __device__ __forceinline__ void store(__bf16* p, const float* o) {
        *(uint4*)p = make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]), pack_bf16(o[6], o[7]));
    }
};
template <> struct SsPiece<float> {
    static constexpr int n = 4;
    static __device__ __forceinline__ void load(const float* p, float* o) {
        const float4 u = *(const float4*)p;
        o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
    }
    static __device__ __forceinline__ void store(float* p, const float* o) { *(float4*)p = make_float4(o[0], o[1], o[2], o[3]); }
};

// The three sums of a row (z^2, z^4, z^6) are reduced together: one exchange through LDS.  VEC: the row is walked in
// 16-byte pieces (the host checks size, stride and alignment); the second walk finds the row in cache.
template <typename T, bool VEC>
__global__ __launch_bounds__(kSsThreads) void poly_norm_kernel(const T* __restrict__ x, int64_t x_stride,
                                                               const float* __restrict__ coef, float eps,
                                                               T* __restrict__ y, int cols) {
    constexpr int N = SsPiece<T>::n;
    __shared__ float red[3][kSsThreads / 64];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    const T* xr = x + r * x_stride;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
    if constexpr (VEC) {
        for (int c = tid * N; c < cols; c += kSsThreads * N) {
            float z[N];
            SsPiece<T>::load(xr + c, z);
#pragma unroll
            for (int e = 0; e < N; ++e) {
                const float z2 = z[e] * z[e];
                s2 += z2;
                s4 += z2 * z2;
                s6 += z2 * z2 * z2;
            }
        }
    } else {
        for (int c = tid; c < cols; c += kSsThreads) {
            const float z = (float)xr[c], z2 = z * z;
            s2 += z2;
            s4 += z2 * z2;
            s6 += z2 * z2 * z2;
        }
    }
    s2 = wave_sum(s2);
    s4 = wave_sum(s4);
    s6 = wave_sum(s6);
    if ((tid & 63) == 0) {
        red[0][tid >> 6] = s2;
        red[1][tid >> 6] = s4;
        red[2][tid >> 6] = s6;
    }
    __syncthreads();
    s2 = s4 = s6 = 0.f;
#pragma unroll
    for (int i = 0; i < kSsThreads / 64; ++i) {
        s2 += red[0][i];
        s4 += red[1][i];
        s6 += red[2][i];
    }
    const float n = (float)cols;
    const float r1 = coef[0] / sqrtf(s2 / n + eps);
    const float r2 = coef[1] / sqrtf(s4 / n + eps);
    const float r3 = coef[2] / sqrtf(s6 / n + eps);
    const float shift = coef[3];
    if constexpr (VEC) {
        for (int c = tid * N; c < cols; c += kSsThreads * N) {
            float z[N];
            SsPiece<T>::load(xr + c, z);
#pragma unroll
            for (int e = 0; e < N; ++e) {
                const float z2 = z[e] * z[e];
                z[e] = r1 * z[e] + r2 * z2 + r3 * (z2 * z[e]) + shift;
            }
            SsPiece<T>::store(y + r * cols + c, z);
        }
    } else {
        for (int c = tid; c < cols; c += kSsThreads) {
            const float z = (float)xr[c], z2 = z * z;
            y[r * cols + c] = (T)(r1 * z + r2 * z2 + r3 * (z2 * z) + shift);
        }
    }
}

// One wave per (token, head); heads 0 .. H-1 are the query's, H .. H+G-1 the key's.  A lane holds both halves of its
// rotary pairs, so the rotation needs no exchange; the head is read twice (sum of squares, then output), the second
// time from cache.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_rope_store_kernel(
    const T* __restrict__ q, const T* __restrict__ k, int64_t q_stride, int64_t k_stride, const float* __restrict__ q_norm,
    const float* __restrict__ k_norm, float eps, const float* __restrict__ freq, int rot_dims,
    const int64_t* __restrict__ positions, const int* __restrict__ slot_mapping, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int64_t items, int H, int G, int D) {
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= items) return;                         // (whole waves leave together)
    const int lane = threadIdx.x & 63;
    const int64_t t = item / (H + G);
    const int head = (int)(item - t * (H + G));
    const bool is_q = head < H;
    const T* src = is_q ? q + t * q_stride + (int64_t)head * D : k + t * k_stride + (int64_t)(head - H) * D;
    const float* w = is_q ? q_norm : k_norm;
    T* dst;
    T* raw = nullptr;
    if (is_q) {
        dst = q_out + (t * H + head) * D;
    } else {
        const int slot = slot_mapping != nullptr ? slot_mapping[t] : -1;
        if (slot < 0) return;
        dst = k_cache + ((int64_t)slot * G + (head - H)) * D;
        raw = v_cache + ((int64_t)slot * G + (head - H)) * D;
    }
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
        const float x = (float)src[d];
        ss += x * x;
        if (raw != nullptr) raw[d] = src[d];
    }
    const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
    const int half = rot_dims >> 1;
    const float p = (float)positions[t];
    for (int i = lane; i < half; i += 64) {
        const float u = (float)src[i] * rstd * w[i], v = (float)src[i + half] * rstd * w[i + half];
        const float ang = p * freq[i];
        const float c = cosf(ang), s = sinf(ang);
        dst[i] = (T)(u * c - v * s);
        dst[i + half] = (T)(v * c + u * s);
    }
    for (int d = rot_dims + lane; d < D; d += 64) dst[d] = (T)((float)src[d] * rstd * w[d]);
}

// The same for heads of at most 128 dimensions with even sizes: a lane keeps two neighbouring dimensions in registers (one
// 4- or 8-byte load), the rotary partner (half the rotated part away) comes from another lane by a shuffle, so the head
// is read once and nothing waits on a second trip to memory.
template <typename T> struct SsPair;
template <> struct SsPair<__bf16> {
    static __device__ __forceinline__ void load(const __bf16* p, float& a, float& b) {
        const uint32_t u = *(const uint32_t*)p;
        a = bf16_lo(u);
        b = bf16_hi(u);
    }
    static __device__ __forceinline__ void store(__bf16* p, float a, float b) { *(uint32_t*)p = pack_bf16(a, b); }
    static __device__ __forceinline__ void copy(__bf16* d, const __bf16* s) { *(uint32_t*)d = *(const uint32_t*)s; }
};
template <> struct SsPair<float> {
    static __device__ __forceinline__ void load(const float* p, float& a, float& b) {
        const float2 u = *(const float2*)p;
        a = u.x;
        b = u.y;
    }
    static __device__ __forceinline__ void store(float* p, float a, float b) { *(float2*)p = make_float2(a, b); }
    static __device__ __forceinline__ void copy(float* d, const float* s) { *(float2*)d = *(const float2*)s; }
};

template <typename T>
__global__ __launch_bounds__(256) void head_norm_rope_store_pairs_kernel(
    const T* __restrict__ q, const T* __restrict__ k, int64_t q_stride, int64_t k_stride, const float* __restrict__ q_norm,
    const float* __restrict__ k_norm, float eps, const float* __restrict__ freq, int rot_dims,
    const int64_t* __restrict__ positions, const int* __restrict__ slot_mapping, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int D) {
    // A workgroup per token: the token's cosines and sines are computed once (full-precision argument reduction is the
    // expensive part of this kernel) and shared by the waves, which take the token's heads in turn.
    __shared__ float cs[2][64];
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int half = rot_dims >> 1;
    if ((int)threadIdx.x < half) {
        const float ang = (float)positions[t] * freq[threadIdx.x];
        sincosf(ang, &cs[1][threadIdx.x], &cs[0][threadIdx.x]);
    }
    __syncthreads();
    const int slot = slot_mapping != nullptr ? slot_mapping[t] : -1;
    const int e0 = 2 * lane;
    const bool live = e0 < D;
    const bool turns = e0 < rot_dims, low = e0 < half;
    const int partner = turns ? (low ? lane + (half >> 1) : lane - (half >> 1)) : lane;
    const int pair = turns ? (low ? e0 : e0 - half) : 0;
    for (int head = wave; head < H + G; head += 4) {
        const bool is_q = head < H;
        if (!is_q && slot < 0) break;                  // (the wave's later heads are key heads too)
        const T* src = is_q ? q + t * q_stride + (int64_t)head * D : k + t * k_stride + (int64_t)(head - H) * D;
        const float* w = is_q ? q_norm : k_norm;
        T* dst = is_q ? q_out + (t * H + head) * D : k_cache + ((int64_t)slot * G + (head - H)) * D;
        float x0 = 0.f, x1 = 0.f;
        if (live) {
            SsPair<T>::load(src + e0, x0, x1);
            if (!is_q) SsPair<T>::copy(v_cache + ((int64_t)slot * G + (head - H)) * D + e0, src + e0);
        }
        const float rstd = 1.0f / sqrtf(wave_sum(x0 * x0 + x1 * x1) / (float)D + eps);
        float y0 = 0.f, y1 = 0.f;
        if (live) {
            y0 = x0 * rstd * w[e0];
            y1 = x1 * rstd * w[e0 + 1];
        }
        const float p0 = __shfl(y0, partner), p1 = __shfl(y1, partner);
        if (turns) {
            const float c0 = cs[0][pair], s0 = cs[1][pair], c1 = cs[0][pair + 1], s1 = cs[1][pair + 1];
            if (low) {
                y0 = y0 * c0 - p0 * s0;
                y1 = y1 * c1 - p1 * s1;
            } else {
                y0 = y0 * c0 + p0 * s0;
                y1 = y1 * c1 + p1 * s1;
            }
        }
        if (live) SsPair<T>::store(dst + e0, y0, y1);
    }
}

}  // namespace nv

extern "C" int nv_stream_boundary_scaled(void* resid, const void* add1, int64_t add1_stride, const void* add2,
                                         int64_t add2_stride, const void* gate2, int64_t gate2_stride, const float* parts,
                                         int n_parts, const float* col_scale, const float* norm_w, float eps, float* y32,
                                         void* y, int dtype, int64_t rows, int cols, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0 && cols <= 16384, NV_ERR_INVALID_ARG, "nv_stream_boundary_scaled: bad sizes");
    if (rows == 0) return NV_OK;
    NV_REQUIRE(resid, NV_ERR_INVALID_ARG, "nv_stream_boundary_scaled: null stream");
    NV_REQUIRE(!parts || n_parts > 0, NV_ERR_INVALID_ARG, "nv_stream_boundary_scaled: parts without a count");
    NV_REQUIRE(!gate2 || add2, NV_ERR_INVALID_ARG, "nv_stream_boundary_scaled: a gate without its input");
    NV_REQUIRE(!norm_w || y32 || y, NV_ERR_INVALID_ARG, "nv_stream_boundary_scaled: the norm needs an output");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_stream_boundary_scaled: bad dtype");
    NV_REQUIRE(rows < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_stream_boundary_scaled: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const size_t smem = sizeof(float) * (size_t)cols;
    const int np = parts ? n_parts : 0;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(stream_boundary_scaled_kernel<__bf16>, dim3((unsigned)rows), dim3(kSsThreads), smem, s,
                           (float*)resid, (const __bf16*)add1, add1_stride, (const __bf16*)add2, add2_stride,
                           (const __bf16*)gate2, gate2_stride, parts, np, col_scale, norm_w, eps, y32, (__bf16*)y, cols);
    else
        hipLaunchKernelGGL(stream_boundary_scaled_kernel<float>, dim3((unsigned)rows), dim3(kSsThreads), smem, s,
                           (float*)resid, (const float*)add1, add1_stride, (const float*)add2, add2_stride,
                           (const float*)gate2, gate2_stride, parts, np, col_scale, norm_w, eps, y32, (float*)y, cols);
    return check_launch("nv_stream_boundary_scaled");
}

extern "C" int nv_poly_norm(const void* x, int64_t x_stride, const float* coef, float eps, void* y, int dtype, int64_t rows,
                            int cols, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0 && x_stride >= cols, NV_ERR_INVALID_ARG, "nv_poly_norm: bad sizes");
    if (rows == 0) return NV_OK;
    NV_REQUIRE(x && coef && y, NV_ERR_INVALID_ARG, "nv_poly_norm: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_poly_norm: bad dtype");
    NV_REQUIRE(rows < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_poly_norm: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const int n = dtype == NV_DTYPE_BF16 ? 8 : 4;              // elements in a 16-byte piece
    const bool vec = cols % n == 0 && x_stride % n == 0 && ((uintptr_t)x | (uintptr_t)y) % 16 == 0;
#define NV_POLY(T, V)                                                                                                \
    hipLaunchKernelGGL((poly_norm_kernel<T, V>), dim3((unsigned)rows), dim3(kSsThreads), 0, s, (const T*)x, x_stride, coef, \
                       eps, (T*)y, cols)
    if (dtype == NV_DTYPE_BF16) {
        if (vec) NV_POLY(__bf16, true); else NV_POLY(__bf16, false);
    } else {
        if (vec) NV_POLY(float, true); else NV_POLY(float, false);
    }
#undef NV_POLY
    return check_launch("nv_poly_norm");
}

extern "C" int nv_head_norm_rope_store(const void* q, const void* k, int64_t q_stride, int64_t k_stride, const float* q_norm,
                                       const float* k_norm, float eps, const float* freq, int rot_dims,
                                       const int64_t* positions, const int32_t* slot_mapping, void* q_out, void* k_cache,
                                       void* v_cache, int dtype, int64_t T, int H, int G, int D, void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && H > 0 && G > 0 && D > 0, NV_ERR_INVALID_ARG, "nv_head_norm_rope_store: bad sizes");
    NV_REQUIRE(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= D, NV_ERR_INVALID_ARG,
               "nv_head_norm_rope_store: rot_dims=%d must be even and at most D=%d", rot_dims, D);
    if (T == 0) return NV_OK;
    NV_REQUIRE(q && k && q_norm && k_norm && positions && q_out && k_cache && v_cache && (freq || rot_dims == 0),
               NV_ERR_INVALID_ARG, "nv_head_norm_rope_store: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_head_norm_rope_store: bad dtype");
    const int64_t items = T * (H + G), grid = (items + 3) / 4;
    NV_REQUIRE(grid < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_head_norm_rope_store: launch too large");
    hipStream_t s = (hipStream_t)stream;
    // two dimensions per lane: even sizes that fit one wave, rotary halves of an even number of dimensions, and rows that
    // start on the pair's alignment
    const uintptr_t align = dtype == NV_DTYPE_BF16 ? 4 : 8;
    const bool pairs = D <= 128 && D % 2 == 0 && rot_dims % 4 == 0 && q_stride % 2 == 0 && k_stride % 2 == 0 &&
                       ((uintptr_t)q | (uintptr_t)k | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)v_cache) % align == 0;
#define NV_HNR(T)                                                                                                          \
    hipLaunchKernelGGL(head_norm_rope_store_kernel<T>, dim3((unsigned)grid), dim3(256), 0, s, (const T*)q, (const T*)k, q_stride, \
                       k_stride, q_norm, k_norm, eps, freq, rot_dims, positions, slot_mapping, (T*)q_out, (T*)k_cache,             \
                       (T*)v_cache, items, H, G, D)
#define NV_HNR_PAIRS(T)                                                                                                    \
    hipLaunchKernelGGL(head_norm_rope_store_pairs_kernel<T>, dim3((unsigned)T_rows), dim3(256), 0, s, (const T*)q, (const T*)k, \
                       q_stride, k_stride, q_norm, k_norm, eps, freq, rot_dims, positions, slot_mapping, (T*)q_out,             \
                       (T*)k_cache, (T*)v_cache, H, G, D)
    const int64_t T_rows = T;
    if (dtype == NV_DTYPE_BF16) {
        if (pairs) NV_HNR_PAIRS(__bf16); else NV_HNR(__bf16);
    } else {
        if (pairs) NV_HNR_PAIRS(float); else NV_HNR(float);
    }
#undef NV_HNR
#undef NV_HNR_PAIRS
    return check_launch("nv_head_norm_rope_store");
}
