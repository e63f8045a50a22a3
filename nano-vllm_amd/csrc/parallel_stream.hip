// An fp32 residual stream whose layers read it through TWO RMS norms at once (one per parallel sublayer), fed by an
// embedding with a hashed bigram table.
//
// nv_hashed_bigram_embed   x[t] = rmsnorm(embed[id_t] + bigram[row_t]) * w in fp32, where
//                              row_t = (id_{t-1} * mul_prev + id_t * mul_cur) mod buckets,  or row `buckets` (the last
//                              one) at position 0.  The previous id of a portion's first row is carried per sequence in
//                              prev_state[slot], which then takes the portion's last id.  Without a bigram table only
//                              the embedding row is normed.
// nv_stream_boundary_pair  per row, in place on the fp32 stream r:
//                              r <- r + a1 + a2 + scale * sum_j p_j                (a1, a2 in the matmul dtype, p_j fp32
//                                                                                   parts, e.g. the outputs of the
//                                                                                   chosen experts; each may be absent)
//                              r <- r + m * (n1 / rms(n1) * w1 + n2 / rms(n2) * w2)  (sublayer outputs that are RMS-normed
//                                                                                   on their way in; may be absent)
//                              y32[:, 0:W] <- r / rms(r) * wa;   y32[:, W:2W] <- r / rms(r) * wb     (fp32, side by side
//                                                                                   in one [rows, 2W] buffer; wb may be
//                                                                                   absent: then y32 is [rows, W])
//                              y <- r / rms(r) * wa in the matmul dtype            (may be absent)
//                          so the stream is read and written once per layer.  rms(x) = sqrt(mean(x^2) + eps), fp32.
// nv_relu_squared          y = max(x, 0)^2.
#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kPsThreads = 256;

__device__ __forceinline__ float ps_block_sum(float x, float* red) {
    x = wave_sum(x);
    const int w = threadIdx.x >> 6;
    __syncthreads();                       // red may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) red[w] = x;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kPsThreads / 64; ++i) t += red[i];
    return t;
}

template <typename T>
__global__ __launch_bounds__(kPsThreads) void hashed_bigram_embed_kernel(
    const int64_t* __restrict__ ids, const int64_t* __restrict__ positions, const T* __restrict__ embed,
    const T* __restrict__ bigram, int64_t buckets, int64_t mul_prev, int64_t mul_cur, const float* __restrict__ norm_w,
    float eps, int64_t* __restrict__ prev_state, float* __restrict__ x, const int* __restrict__ cu_q,
    const int* __restrict__ slots, int B, int cols) {
    extern __shared__ float row[];
    __shared__ float red[kPsThreads / 64];
    __shared__ int64_t bigram_row;
    const int t = blockIdx.x, tid = threadIdx.x;
    const int64_t id = ids[t];
    if (tid == 0) {
        int lo = 0, hi = B;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (cu_q[mid] <= t) lo = mid; else hi = mid;
        }
        const int b = lo, i = t - cu_q[b];
        int64_t prev = 0;
        if (i > 0) prev = ids[t - 1];
        else if (prev_state != nullptr) {
            prev = prev_state[slots[b]];
            prev_state[slots[b]] = ids[cu_q[b + 1] - 1];       // this thread alone touches the slot in this launch
        }
        bigram_row = positions[t] == 0 ? buckets : (prev * mul_prev + id * mul_cur) % buckets;
    }
    __syncthreads();
    const T* er = embed + id * cols;
    const T* br = bigram != nullptr ? bigram + bigram_row * cols : nullptr;
    float ss = 0.f;
    for (int c = tid; c < cols; c += kPsThreads) {
        const float v = (float)er[c] + (br != nullptr ? (float)br[c] : 0.f);
        row[c] = v;
        ss += v * v;
    }
    if (norm_w == nullptr) {                                   // no norm: a thread reads back its own columns
        for (int c = tid; c < cols; c += kPsThreads) x[(int64_t)t * cols + c] = row[c];
        return;
    }
    ss = ps_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)cols + eps);
    for (int c = tid; c < cols; c += kPsThreads) x[(int64_t)t * cols + c] = row[c] * rstd * norm_w[c];
}

template <typename T>
__global__ __launch_bounds__(kPsThreads) void stream_boundary_pair_kernel(
    float* __restrict__ resid, const T* __restrict__ add1, int64_t add1_stride, const T* __restrict__ add2,
    int64_t add2_stride, const float* __restrict__ parts, int n_parts, float parts_scale, const T* __restrict__ n1,
    int64_t n1_stride, const float* __restrict__ w1, const T* __restrict__ n2, int64_t n2_stride,
    const float* __restrict__ w2, float normed_mult, const float* __restrict__ wa, const float* __restrict__ wb, float eps,
    float* __restrict__ y32, T* __restrict__ y, int cols) {
    extern __shared__ float row[];
    __shared__ float red[kPsThreads / 64];
    const int64_t r = blockIdx.x;
    const int tid = threadIdx.x;
    float* rrow = resid + r * cols;
    float s1 = 0.f, s2 = 0.f;
    for (int c = tid; c < cols; c += kPsThreads) {
        float v = rrow[c];
        float s = 0.f;
        if (add1 != nullptr) s += (float)add1[r * add1_stride + c];
        if (add2 != nullptr) s += (float)add2[r * add2_stride + c];
        if (n_parts > 0) {
            float ps = 0.f;
            for (int j = 0; j < n_parts; ++j) ps += parts[(r * n_parts + j) * cols + c];
            s += parts_scale * ps;
        }
        row[c] = v + s;
        if (n1 != nullptr) {
            const float a = (float)n1[r * n1_stride + c];
            s1 += a * a;
        }
        if (n2 != nullptr) {
            const float a = (float)n2[r * n2_stride + c];
            s2 += a * a;
        }
    }
    if (n1 != nullptr || n2 != nullptr) {
        const float r1 = n1 != nullptr ? 1.0f / sqrtf(ps_block_sum(s1, red) / (float)cols + eps) : 0.f;
        const float r2 = n2 != nullptr ? 1.0f / sqrtf(ps_block_sum(s2, red) / (float)cols + eps) : 0.f;
        for (int c = tid; c < cols; c += kPsThreads) {
            float s = 0.f;
            if (n1 != nullptr) s += (float)n1[r * n1_stride + c] * r1 * w1[c];
            if (n2 != nullptr) s += (float)n2[r * n2_stride + c] * r2 * w2[c];
            row[c] += normed_mult * s;
        }
    }
    float ss = 0.f;
    for (int c = tid; c < cols; c += kPsThreads) {         // a thread reads back its own columns only
        const float v = row[c];
        rrow[c] = v;
        ss += v * v;
    }
    if (wa == nullptr) return;
    const float rstd = 1.0f / sqrtf(ps_block_sum(ss, red) / (float)cols + eps);
    const int ld = wb != nullptr ? 2 * cols : cols;
    for (int c = tid; c < cols; c += kPsThreads) {
        const float u = row[c] * rstd;
        if (y32 != nullptr) {
            y32[r * ld + c] = u * wa[c];
            if (wb != nullptr) y32[r * ld + cols + c] = u * wb[c];
        }
        if (y != nullptr) y[r * cols + c] = (T)(u * wa[c]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void relu_squared_kernel(const T* __restrict__ x, int64_t x_stride, T* __restrict__ y,
                                                           int cols, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int64_t r = i / cols;
    const float v = fmaxf((float)x[r * x_stride + (i - r * cols)], 0.f);
    y[i] = (T)(v * v);
}

}  // namespace nv

extern "C" int nv_hashed_bigram_embed(const int64_t* ids, const int64_t* positions, const void* embed, const void* bigram,
                                      int64_t buckets, int64_t mul_prev, int64_t mul_cur, const float* norm_w, float eps,
                                      int64_t* prev_state, float* x, const int32_t* cu_seqlens_q,
                                      const int32_t* state_slots, int num_seqs, int64_t T, int cols, int dtype,
                                      void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && num_seqs >= 0 && cols > 0 && cols <= 16384, NV_ERR_INVALID_ARG, "nv_hashed_bigram_embed: bad sizes");
    if (T == 0 || num_seqs == 0) return NV_OK;
    NV_REQUIRE(ids && positions && embed && x && cu_seqlens_q, NV_ERR_INVALID_ARG,
               "nv_hashed_bigram_embed: null pointer");
    NV_REQUIRE(!bigram || (buckets > 0 && prev_state && state_slots), NV_ERR_INVALID_ARG,
               "nv_hashed_bigram_embed: a bigram table needs its bucket count and the carried ids");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_hashed_bigram_embed: bad dtype");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_hashed_bigram_embed: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const size_t smem = sizeof(float) * (size_t)cols;
    if (!bigram) buckets = 1;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(hashed_bigram_embed_kernel<__bf16>, dim3((unsigned)T), dim3(kPsThreads), smem, s, ids, positions,
                           (const __bf16*)embed, (const __bf16*)bigram, buckets, mul_prev, mul_cur, norm_w, eps,
                           bigram ? prev_state : nullptr, x, cu_seqlens_q, state_slots, num_seqs, cols);
    else
        hipLaunchKernelGGL(hashed_bigram_embed_kernel<float>, dim3((unsigned)T), dim3(kPsThreads), smem, s, ids, positions,
                           (const float*)embed, (const float*)bigram, buckets, mul_prev, mul_cur, norm_w, eps,
                           bigram ? prev_state : nullptr, x, cu_seqlens_q, state_slots, num_seqs, cols);
    return check_launch("nv_hashed_bigram_embed");
}

extern "C" int nv_stream_boundary_pair(void* resid, const void* add1, int64_t add1_stride, const void* add2,
                                       int64_t add2_stride, const float* parts, int n_parts, float parts_scale,
                                       const void* normed1, int64_t normed1_stride, const float* normed1_w,
                                       const void* normed2, int64_t normed2_stride, const float* normed2_w,
                                       float normed_mult, const float* norm_a, const float* norm_b, float eps, float* y32,
                                       void* y, int dtype, int64_t rows, int cols, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0 && cols <= 16384, NV_ERR_INVALID_ARG, "nv_stream_boundary_pair: bad sizes");
    if (rows == 0) return NV_OK;
    NV_REQUIRE(resid, NV_ERR_INVALID_ARG, "nv_stream_boundary_pair: null stream");
    NV_REQUIRE(!parts || n_parts > 0, NV_ERR_INVALID_ARG, "nv_stream_boundary_pair: parts without a count");
    NV_REQUIRE((!normed1 || normed1_w) && (!normed2 || normed2_w), NV_ERR_INVALID_ARG,
               "nv_stream_boundary_pair: a normed input needs its weight");
    NV_REQUIRE(!norm_b || norm_a, NV_ERR_INVALID_ARG, "nv_stream_boundary_pair: a second norm needs the first");
    NV_REQUIRE(!norm_a || y32 || y, NV_ERR_INVALID_ARG, "nv_stream_boundary_pair: the norm needs an output");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_stream_boundary_pair: bad dtype");
    NV_REQUIRE(rows < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_stream_boundary_pair: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const size_t smem = sizeof(float) * (size_t)cols;
    const int np = parts ? n_parts : 0;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(stream_boundary_pair_kernel<__bf16>, dim3((unsigned)rows), dim3(kPsThreads), smem, s,
                           (float*)resid, (const __bf16*)add1, add1_stride, (const __bf16*)add2, add2_stride, parts, np,
                           parts_scale, (const __bf16*)normed1, normed1_stride, normed1_w, (const __bf16*)normed2,
                           normed2_stride, normed2_w, normed_mult, norm_a, norm_b, eps, y32, (__bf16*)y, cols);
    else
        hipLaunchKernelGGL(stream_boundary_pair_kernel<float>, dim3((unsigned)rows), dim3(kPsThreads), smem, s,
                           (float*)resid, (const float*)add1, add1_stride, (const float*)add2, add2_stride, parts, np,
                           parts_scale, (const float*)normed1, normed1_stride, normed1_w, (const float*)normed2,
                           normed2_stride, normed2_w, normed_mult, norm_a, norm_b, eps, y32, (float*)y, cols);
    return check_launch("nv_stream_boundary_pair");
}

extern "C" int nv_relu_squared(const void* x, int64_t x_stride, void* y, int dtype, int64_t rows, int cols, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0 && x_stride >= cols, NV_ERR_INVALID_ARG, "nv_relu_squared: bad sizes");
    if (rows == 0) return NV_OK;
    NV_REQUIRE(x && y, NV_ERR_INVALID_ARG, "nv_relu_squared: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_relu_squared: bad dtype");
    const int64_t n = rows * cols, grid = (n + 255) / 256;
    NV_REQUIRE(grid < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_relu_squared: launch too large");
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(relu_squared_kernel<__bf16>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                           (const __bf16*)x, x_stride, (__bf16*)y, cols, n);
    else
        hipLaunchKernelGGL(relu_squared_kernel<float>, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream,
                           (const float*)x, x_stride, (float*)y, cols, n);
    return check_launch("nv_relu_squared");
}
