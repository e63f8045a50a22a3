// Recurrent mixer kernels: short causal convolution with carried taps, and the gated delta rule with one decay per
// key channel.  Both keep their state per SEQUENCE in numbered slots (a slot is a row of the state tensors; the
// engine hands a slot to a request at admission and takes it back at the end), and both take a step's flat token
// rows with cu_seqlens_q / cu_seqlens_k: a sequence whose rows start at position 0 (len_k == len_q) starts from a
// zero state whatever its slot holds, any other continues from the slot.
//
// nv_causal_conv_silu      y[t, c] = silu(sum_j w[c, taps-1-j] * x[t - j, c]), inputs before the step's first row
//                          come from conv_state[slot] (the last taps-1 inputs of the sequence), zeros before position
//                          0; afterwards conv_state[slot] holds the last taps-1 inputs including this step's.
//
// nv_gated_delta_rule      per head, token by token, state S [D, Dv] in fp32:
//                              S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//                          with q, k made unit vectors per head (sum of squares + 1e-6 under the root; q also times
//                          D^-1/2), beta = sigmoid(b_raw), g = exp(-exp(A_log_h) * softplus(a_raw + dt_bias)) per key
//                          channel, and the read-out normalised: o / rms(o) * norm_w * sigmoid(gate_raw).
//                          Everything after the raw projections is fp32.
//
// Layout of the recurrence: one workgroup per (sequence, head).  A lane owns one value column and a quarter of the
// key rows (a contiguous run: its quad index r owns rows r * RPL .. r * RPL + RPL - 1, read from LDS four at a time; the
// four runs sit RPL + 4 words apart so that the quad's 16-byte reads fall on different banks), so the state lives in
// registers, both read-outs of a token
// (S^T k and S^T q) are one pass over them and a two-step quad reduction, and the token loop has no workgroup
// barrier: k, q, g, beta, v of 16 tokens are prepared into LDS by all waves together, each wave then runs the 16
// tokens for its 16 columns, and the normalised read-out of the tile is written by all waves together.
#include <algorithm>

#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kConvMaxTaps = 8;

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_silu_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ conv_state, T* __restrict__ y, int64_t y_stride, const int* __restrict__ cu_q,
    const int* __restrict__ cu_k, const int* __restrict__ state_slots, int B, int C, int taps, int act) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    int lo = 0, hi = B;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid;
    }
    const int b = lo;
    const int i = t - cu_q[b];
    const int start = (cu_k[b + 1] - cu_k[b]) - (cu_q[b + 1] - cu_q[b]);
    const T* st = conv_state + (int64_t)state_slots[b] * (taps - 1) * C;
    float acc = bias != nullptr ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = i - j;
        float xv = 0.f;
        if (src >= 0) xv = (float)x[(int64_t)(t - j) * x_stride + c];
        else if (start + src >= 0) xv = (float)st[(int64_t)(taps - 1 + src) * C + c];
        acc += w[(int64_t)c * taps + (taps - 1 - j)] * xv;
    }
    y[(int64_t)t * y_stride + c] = (T)(act ? silu_f(acc) : acc);
}

// The same in 16-byte pieces: a thread takes 8 (bf16) or 4 (fp32) neighbouring channels of one token.
template <typename T> struct Piece;
template <> struct Piece<__bf16> {
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
template <> struct Piece<float> {
    static constexpr int n = 4;
    static __device__ __forceinline__ void load(const float* p, float* o) {
        const float4 u = *(const float4*)p;
        o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
    }
    static __device__ __forceinline__ void store(float* p, const float* o) { *(float4*)p = make_float4(o[0], o[1], o[2], o[3]); }
};


// A thread keeps its channels' weights and the last `taps` inputs in registers and walks a run of tokens (16 in a large step, fewer when the step has too few rows to fill the chip that way): inside a
// sequence every token costs one new 16-byte load; at a sequence's first row of the step the window is filled from
// the carried state (or zeros before position 0).
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_silu_pieces_kernel(
    const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ conv_state, T* __restrict__ y, int64_t y_stride, const int* __restrict__ cu_q,
    const int* __restrict__ cu_k, const int* __restrict__ state_slots, int B, int C, int taps, int T_rows,
    int tokens_per_group, int act) {
    constexpr int N = Piece<T>::n;
    const int c = (blockIdx.y * 256 + threadIdx.x) * N;
    if (c >= C) return;
    float wt[kConvMaxTaps][N], win[kConvMaxTaps][N];        // wt[j], win[j]: weight of / input at the token j back
    float bs[N];
#pragma unroll
    for (int e = 0; e < N; ++e) bs[e] = bias != nullptr ? bias[c + e] : 0.f;
#pragma unroll
    for (int j = 0; j < kConvMaxTaps; ++j) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            wt[j][e] = j < taps ? w[(int64_t)(c + e) * taps + (taps - 1 - j)] : 0.f;
            win[j][e] = 0.f;
        }
    }
    const int t0 = blockIdx.x * tokens_per_group, t1 = min(T_rows, t0 + tokens_per_group);
    int b = 0;
    {
        int lo = 0, hi = B;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (cu_q[mid] <= t0) lo = mid; else hi = mid;
        }
        b = lo;
    }
    for (int t = t0; t < t1; ++t) {
        while (b + 1 < B && t >= cu_q[b + 1]) ++b;           // sequences without rows in this step are skipped
        const int i = t - cu_q[b];
        if (i == 0 || t == t0) {                             // fill the window's older entries
            const int start = (cu_k[b + 1] - cu_k[b]) - (cu_q[b + 1] - cu_q[b]);
            const T* st = conv_state + (int64_t)state_slots[b] * (taps - 1) * C;
#pragma unroll
            for (int j = 1; j < kConvMaxTaps; ++j) {
                if (j < taps) {
                    const int src = i - j;
                    if (src >= 0) Piece<T>::load(x + (int64_t)(t - j) * x_stride + c, win[j]);
                    else if (start + src >= 0) Piece<T>::load(st + (int64_t)(taps - 1 + src) * C + c, win[j]);
                    else {
#pragma unroll
                        for (int e = 0; e < N; ++e) win[j][e] = 0.f;
                    }
                }
            }
        }
        Piece<T>::load(x + (int64_t)t * x_stride + c, win[0]);
        float acc[N];
#pragma unroll
        for (int e = 0; e < N; ++e) acc[e] = bs[e];
#pragma unroll
        for (int j = 0; j < kConvMaxTaps; ++j) {
#pragma unroll
            for (int e = 0; e < N; ++e) acc[e] += wt[j][e] * win[j][e];       // wt[j] = 0 for j >= taps
        }
#pragma unroll
        for (int e = 0; e < N; ++e) acc[e] = act ? silu_f(acc[e]) : acc[e];
        Piece<T>::store(y + (int64_t)t * y_stride + c, acc);
#pragma unroll
        for (int j = kConvMaxTaps - 1; j > 0; --j) {
#pragma unroll
            for (int e = 0; e < N; ++e) win[j][e] = win[j - 1][e];
        }
    }
}

// More taps than the register window holds: one thread per channel walks the state rows upwards, so a row is read
// (row s + len_q) before it is overwritten.
template <typename T>
__global__ __launch_bounds__(256) void conv_state_walk_kernel(
    const T* __restrict__ x, int64_t x_stride, T* __restrict__ conv_state, const int* __restrict__ cu_q,
    const int* __restrict__ cu_k, const int* __restrict__ state_slots, int C, int taps) {
    const int b = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int q0 = cu_q[b], nq = cu_q[b + 1] - q0, nk = cu_k[b + 1] - cu_k[b];
    if (nq <= 0) return;
    const int keep = taps - 1, start = nk - nq;
    T* st = conv_state + (int64_t)state_slots[b] * keep * C;
    for (int s = 0; s < keep; ++s) {
        const int p = nk - keep + s;               // position this row holds afterwards
        T v = (T)0.f;
        if (p >= start) v = x[(int64_t)(q0 + p - start) * x_stride + c];
        else if (p >= 0) v = st[(int64_t)(s + nq) * C + c];
        st[(int64_t)s * C + c] = v;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    const T* __restrict__ x, int64_t x_stride, T* __restrict__ conv_state, const int* __restrict__ cu_q,
    const int* __restrict__ cu_k, const int* __restrict__ state_slots, int C, int taps) {
    const int b = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int len_q = cu_q[b + 1] - cu_q[b];
    if (len_q <= 0) return;
    const int end = cu_k[b + 1] - cu_k[b], start = end - len_q;
    T* st = conv_state + (int64_t)state_slots[b] * (taps - 1) * C;
    T keep[kConvMaxTaps - 1];
#pragma unroll
    for (int s = 0; s < kConvMaxTaps - 1; ++s) {
        if (s < taps - 1) {
            const int pos = end - (taps - 1) + s;
            T val = (T)0.f;
            if (pos >= start) val = x[(int64_t)(cu_q[b] + pos - start) * x_stride + c];
            else if (pos >= 0) val = st[(int64_t)(pos - start + taps - 1) * C + c];
            keep[s] = val;
        }
    }
#pragma unroll
    for (int s = 0; s < kConvMaxTaps - 1; ++s)
        if (s < taps - 1) st[(int64_t)s * C + c] = keep[s];
}

// ------------------------------------------------------------------------------------------------ delta rule
constexpr int kDrMaxTile = 16;     // tokens prepared at a time, fewer when LDS is short
constexpr int kDrLdsBudget = 60 * 1024;

template <int CTRL>
__device__ __forceinline__ float quad_xchg(float x) { return dpp_f32<CTRL>(x); }
__device__ __forceinline__ float quad_sum(float x) {
    x += quad_xchg<0xB1>(x);   // quad_perm [1,0,3,2]
    x += quad_xchg<0x4E>(x);   // quad_perm [2,3,0,1]
    return x;
}

template <typename T, int RPL>
__global__ void gated_delta_rule_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t q_stride, int64_t k_stride,
    int64_t v_stride, const T* __restrict__ a_raw, int64_t a_stride, const T* __restrict__ b_raw, int64_t b_stride,
    const T* __restrict__ gate_raw, int64_t gate_stride, const float* __restrict__ A_log,
    const float* __restrict__ dt_bias, const float* __restrict__ norm_w, float* __restrict__ state,
    T* __restrict__ out, int64_t out_stride, const int* __restrict__ cu_q, const int* __restrict__ cu_k,
    const int* __restrict__ state_slots, int H, int G, int D, int Dv, float eps, int kDrTile) {
    constexpr int DP = (RPL + 4) * 4;                 // LDS words per token and vector: four runs of RPL rows, padded
    extern __shared__ float smem[];
    float* ks = smem;                                 // [tile][DP]
    float* qs = ks + kDrTile * DP;                    // [tile][DP]
    float* gs = qs + kDrTile * DP;                    // [tile][DP]
    float* vs = gs + kDrTile * DP;                    // [tile][Dv]
    float* os = vs + kDrTile * Dv;                    // [tile][Dv]
    float* bs = os + kDrTile * Dv;                    // [tile] beta, then [tile] k.q
    const int b = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
    const int q0 = cu_q[b], len_q = cu_q[b + 1] - q0;
    if (len_q <= 0) return;
    const int start = (cu_k[b + 1] - cu_k[b]) - len_q;
    const int hk = h / (H / G);                       // q/k head of this value head
    const int col = wave * 16 + (lane >> 2), r = lane & 3;
    const bool live = col < Dv;
    float* S_slot = state + ((int64_t)state_slots[b] * H + h) * (int64_t)D * Dv;
    float S[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int row = r * RPL + i;
        S[i] = (live && start > 0 && row < D) ? S_slot[(int64_t)row * Dv + col] : 0.f;
    }
    const float rate = expf(A_log[h]);
    const float q_scale = 1.0f / sqrtf((float)D);
    for (int t0 = 0; t0 < len_q; t0 += kDrTile) {
        const int nt = min(kDrTile, len_q - t0);
        __syncthreads();                              // the previous tile's epilogue has read os
        // ---- prepare the tile: unit q / k, decays, beta, v --------------------------------------------
        for (int tt = wave; tt < nt; tt += n_waves) {
            const int64_t t = q0 + t0 + tt;
            const T* kr = k + t * k_stride + (int64_t)hk * D;
            const T* qr = q + t * q_stride + (int64_t)hk * D;
            float kk = 0.f, qq = 0.f;
            for (int d = lane; d < D; d += 64) {
                const float kv = (float)kr[d], qv = (float)qr[d];
                kk += kv * kv;
                qq += qv * qv;
            }
            kk = wave_sum(kk);
            qq = wave_sum(qq);
            const float kn = 1.0f / sqrtf(kk + 1e-6f), qn = q_scale / sqrtf(qq + 1e-6f);
            float kq = 0.f;
            for (int d = lane; d < 4 * RPL; d += 64) {
                const int at = tt * DP + (d / RPL) * (RPL + 4) + (d % RPL);
                float kv = 0.f, qv = 0.f, gv = 1.f;
                if (d < D) {
                    kv = (float)kr[d] * kn;
                    qv = (float)qr[d] * qn;
                    const float a = (float)a_raw[t * a_stride + (int64_t)h * D + d] + dt_bias[(int64_t)h * D + d];
                    gv = expf(-rate * softplus_f(a));
                }
                ks[at] = kv;
                qs[at] = qv;
                gs[at] = gv;
                kq += kv * qv;
            }
            kq = wave_sum(kq);
            if (lane == 0) {
                bs[tt] = sigmoid_f((float)b_raw[t * b_stride + h]);
                bs[kDrTile + tt] = kq;
            }
            for (int c = lane; c < Dv; c += 64) vs[tt * Dv + c] = (float)v[t * v_stride + (int64_t)h * Dv + c];
        }
        __syncthreads();
        // ---- the recurrence over the tile, no barrier inside ---------------------------------------------
        if (live) {
            for (int tt = 0; tt < nt; ++tt) {
                const float4* kt = (const float4*)(ks + tt * DP + r * (RPL + 4));
                const float4* qt = (const float4*)(qs + tt * DP + r * (RPL + 4));
                const float4* gt = (const float4*)(gs + tt * DP + r * (RPL + 4));
                float sk = 0.f, sq = 0.f;
                float4 kk[RPL / 4];
#pragma unroll
                for (int i = 0; i < RPL / 4; ++i) {
                    const float4 g4 = gt[i], q4 = qt[i];
                    kk[i] = kt[i];
                    S[4 * i] *= g4.x; S[4 * i + 1] *= g4.y; S[4 * i + 2] *= g4.z; S[4 * i + 3] *= g4.w;
                    sk += S[4 * i] * kk[i].x + S[4 * i + 1] * kk[i].y + S[4 * i + 2] * kk[i].z + S[4 * i + 3] * kk[i].w;
                    sq += S[4 * i] * q4.x + S[4 * i + 1] * q4.y + S[4 * i + 2] * q4.z + S[4 * i + 3] * q4.w;
                }
                sk = quad_sum(sk);
                sq = quad_sum(sq);
                const float u = bs[tt] * (vs[tt * Dv + col] - sk);
#pragma unroll
                for (int i = 0; i < RPL / 4; ++i) {
                    S[4 * i] += kk[i].x * u; S[4 * i + 1] += kk[i].y * u; S[4 * i + 2] += kk[i].z * u; S[4 * i + 3] += kk[i].w * u;
                }
                if (r == 0) os[tt * Dv + col] = sq + u * bs[kDrTile + tt];     // (S + k u^T)^T q
            }
        }
        __syncthreads();
        // ---- normalised, gated read-out of the tile ----------------------------------------------------
        for (int tt = wave; tt < nt; tt += n_waves) {
            const int64_t t = q0 + t0 + tt;
            float ss = 0.f;
            for (int c = lane; c < Dv; c += 64) ss += os[tt * Dv + c] * os[tt * Dv + c];
            ss = wave_sum(ss);
            const float rstd = 1.0f / sqrtf(ss / (float)Dv + eps);
            for (int c = lane; c < Dv; c += 64) {
                const float gate = sigmoid_f((float)gate_raw[t * gate_stride + (int64_t)h * Dv + c]);
                out[t * out_stride + (int64_t)h * Dv + c] = (T)(os[tt * Dv + c] * rstd * norm_w[c] * gate);
            }
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            const int row = r * RPL + i;
            if (row < D) S_slot[(int64_t)row * Dv + col] = S[i];
        }
    }
}

template <typename T>
static int launch_delta(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                        int64_t v_stride, const void* a_raw, int64_t a_stride, const void* b_raw, int64_t b_stride,
                        const void* gate_raw, int64_t gate_stride, const float* A_log, const float* dt_bias,
                        const float* norm_w, float* state, void* out, int64_t out_stride, const int* cu_q,
                        const int* cu_k, const int* state_slots, int B, int H, int G, int D, int Dv, float eps,
                        hipStream_t s) {
    const int waves = (Dv + 15) / 16;
    const dim3 grid((unsigned)B, (unsigned)H), block((unsigned)waves * 64);
    const int rpl = D <= 32 ? 8 : D <= 64 ? 16 : D <= 128 ? 32 : 64;
    const size_t per_token = sizeof(float) * (size_t)(3 * (rpl + 4) * 4 + 2 * Dv + 2);
    const int tile = (int)std::max<size_t>(1, std::min<size_t>(kDrMaxTile, kDrLdsBudget / per_token));
    const size_t smem = per_token * tile;
#define NV_DR_CASE(R)                                                                                              \
    case R:                                                                                                        \
        hipLaunchKernelGGL((gated_delta_rule_kernel<T, R>), grid, block, smem, s, (const T*)q, (const T*)k,       \
                           (const T*)v, q_stride, k_stride, v_stride, (const T*)a_raw, a_stride, (const T*)b_raw, \
                           b_stride, (const T*)gate_raw, gate_stride, A_log, dt_bias, norm_w, state, (T*)out,     \
                           out_stride, cu_q, cu_k, state_slots, H, G, D, Dv, eps, tile);                          \
        break;
    switch (rpl) {
        NV_DR_CASE(8)
        NV_DR_CASE(16)
        NV_DR_CASE(32)
        NV_DR_CASE(64)
    }
#undef NV_DR_CASE
    return check_launch("nv_gated_delta_rule");
}

}  // namespace nv

extern "C" int nv_causal_conv_silu(const void* x, int64_t x_stride, const float* w, void* conv_state, void* y,
                                   int64_t y_stride, const int* cu_seqlens_q, const int* cu_seqlens_k,
                                   const int* state_slots, int num_seqs, int64_t T, int C, int taps, int dtype,
                                   void* stream) {
    return nv_causal_conv_bias_silu(x, x_stride, w, nullptr, conv_state, y, y_stride, cu_seqlens_q, cu_seqlens_k,
                                    state_slots, num_seqs, T, C, taps, dtype, stream);
}

extern "C" int nv_causal_conv_bias_silu(const void* x, int64_t x_stride, const float* w, const float* bias,
                                        void* conv_state, void* y, int64_t y_stride, const int* cu_seqlens_q,
                                        const int* cu_seqlens_k, const int* state_slots, int num_seqs, int64_t T, int C,
                                        int taps, int dtype, void* stream) {
    return nv_causal_conv_act(x, x_stride, w, bias, conv_state, y, y_stride, cu_seqlens_q, cu_seqlens_k, state_slots,
                              num_seqs, T, C, taps, NV_CONV_ACT_SILU, dtype, stream);
}

extern "C" int nv_causal_conv_act(const void* x, int64_t x_stride, const float* w, const float* bias, void* conv_state,
                                  void* y, int64_t y_stride, const int* cu_seqlens_q, const int* cu_seqlens_k,
                                  const int* state_slots, int num_seqs, int64_t T, int C, int taps, int act, int dtype,
                                  void* stream) {
    using namespace nv;
    NV_REQUIRE(act == NV_CONV_ACT_NONE || act == NV_CONV_ACT_SILU, NV_ERR_INVALID_ARG, "nv_causal_conv_act: bad activation");
    NV_REQUIRE(num_seqs >= 0 && T >= 0 && C > 0, NV_ERR_INVALID_ARG, "nv_causal_conv_silu: bad sizes");
    NV_REQUIRE(taps >= 1 && taps <= 64, NV_ERR_UNSUPPORTED, "nv_causal_conv_silu: taps=%d not in 1..64", taps);
    const bool wide = taps > kConvMaxTaps;                     // beyond the register window: the plain kernels
    if (T == 0 || num_seqs == 0) return NV_OK;
    NV_REQUIRE(x && w && y && cu_seqlens_q && cu_seqlens_k && state_slots && (conv_state || taps == 1),
               NV_ERR_INVALID_ARG, "nv_causal_conv_silu: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_causal_conv_silu: bad dtype");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_causal_conv_silu: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const unsigned cb = (unsigned)((C + 255) / 256);
    const int n = dtype == NV_DTYPE_BF16 ? 8 : 4;              // channels in a 16-byte piece
    const bool pieces = !wide && C % n == 0 && x_stride % n == 0 && y_stride % n == 0 &&
                        ((uintptr_t)x | (uintptr_t)y | (uintptr_t)conv_state) % 16 == 0;
    const unsigned pb = (unsigned)((C / n + 255) / 256);
    const int tpg = T * pb >= 8192 ? 16 : T * pb >= 2048 ? 4 : 1;      // tokens per workgroup: at least 512 workgroups
    if (dtype == NV_DTYPE_BF16) {
        if (pieces)
            hipLaunchKernelGGL(causal_conv_silu_pieces_kernel<__bf16>, dim3((unsigned)((T + tpg - 1) / tpg), pb), dim3(256), 0, s,
                               (const __bf16*)x, x_stride, w, bias, (const __bf16*)conv_state, (__bf16*)y, y_stride,
                               cu_seqlens_q, cu_seqlens_k, state_slots, num_seqs, C, taps, (int)T, tpg, act);
        else
        hipLaunchKernelGGL(causal_conv_silu_kernel<__bf16>, dim3((unsigned)T, cb), dim3(256), 0, s, (const __bf16*)x,
                           x_stride, w, bias, (const __bf16*)conv_state, (__bf16*)y, y_stride, cu_seqlens_q, cu_seqlens_k,
                           state_slots, num_seqs, C, taps, act);
        if (wide)
            hipLaunchKernelGGL(conv_state_walk_kernel<__bf16>, dim3((unsigned)num_seqs, cb), dim3(256), 0, s,
                               (const __bf16*)x, x_stride, (__bf16*)conv_state, cu_seqlens_q, cu_seqlens_k,
                               state_slots, C, taps);
        else if (taps > 1)
            hipLaunchKernelGGL(conv_state_update_kernel<__bf16>, dim3((unsigned)num_seqs, cb), dim3(256), 0, s,
                               (const __bf16*)x, x_stride, (__bf16*)conv_state, cu_seqlens_q, cu_seqlens_k,
                               state_slots, C, taps);
    } else {
        if (pieces)
            hipLaunchKernelGGL(causal_conv_silu_pieces_kernel<float>, dim3((unsigned)((T + tpg - 1) / tpg), pb), dim3(256), 0, s,
                               (const float*)x, x_stride, w, bias, (const float*)conv_state, (float*)y, y_stride,
                               cu_seqlens_q, cu_seqlens_k, state_slots, num_seqs, C, taps, (int)T, tpg, act);
        else
        hipLaunchKernelGGL(causal_conv_silu_kernel<float>, dim3((unsigned)T, cb), dim3(256), 0, s, (const float*)x,
                           x_stride, w, bias, (const float*)conv_state, (float*)y, y_stride, cu_seqlens_q, cu_seqlens_k,
                           state_slots, num_seqs, C, taps, act);
        if (wide)
            hipLaunchKernelGGL(conv_state_walk_kernel<float>, dim3((unsigned)num_seqs, cb), dim3(256), 0, s,
                               (const float*)x, x_stride, (float*)conv_state, cu_seqlens_q, cu_seqlens_k, state_slots,
                               C, taps);
        else if (taps > 1)
            hipLaunchKernelGGL(conv_state_update_kernel<float>, dim3((unsigned)num_seqs, cb), dim3(256), 0, s,
                               (const float*)x, x_stride, (float*)conv_state, cu_seqlens_q, cu_seqlens_k, state_slots,
                               C, taps);
    }
    return check_launch("nv_causal_conv_silu");
}

extern "C" int nv_gated_delta_rule(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                                   int64_t v_stride, const void* a_raw, int64_t a_stride, const void* b_raw,
                                   int64_t b_stride, const void* gate_raw, int64_t gate_stride, const float* A_log,
                                   const float* dt_bias, const float* norm_w, float* state, void* out,
                                   int64_t out_stride, const int* cu_seqlens_q, const int* cu_seqlens_k,
                                   const int* state_slots, int num_seqs, int H, int G, int D, int Dv, float eps,
                                   int dtype, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && H > 0 && G > 0 && D > 0 && Dv > 0, NV_ERR_INVALID_ARG, "nv_gated_delta_rule: bad sizes");
    if (num_seqs == 0) return NV_OK;
    NV_REQUIRE(q && k && v && a_raw && b_raw && gate_raw && A_log && dt_bias && norm_w && state && out &&
                   cu_seqlens_q && cu_seqlens_k && state_slots,
               NV_ERR_INVALID_ARG, "nv_gated_delta_rule: null pointer");
    NV_REQUIRE(H % G == 0, NV_ERR_INVALID_ARG, "nv_gated_delta_rule: H=%d not a multiple of G=%d", H, G);
    NV_REQUIRE(D <= 256 && Dv <= 256, NV_ERR_UNSUPPORTED, "nv_gated_delta_rule: D=%d, Dv=%d exceed 256", D, Dv);
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_gated_delta_rule: bad dtype");
    NV_REQUIRE(H < 65536, NV_ERR_UNSUPPORTED, "nv_gated_delta_rule: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        return launch_delta<__bf16>(q, k, v, q_stride, k_stride, v_stride, a_raw, a_stride, b_raw, b_stride, gate_raw,
                                    gate_stride, A_log, dt_bias, norm_w, state, out, out_stride, cu_seqlens_q,
                                    cu_seqlens_k, state_slots, num_seqs, H, G, D, Dv, eps, s);
    return launch_delta<float>(q, k, v, q_stride, k_stride, v_stride, a_raw, a_stride, b_raw, b_stride, gate_raw,
                               gate_stride, A_log, dt_bias, norm_w, state, out, out_stride, cu_seqlens_q, cu_seqlens_k,
                               state_slots, num_seqs, H, G, D, Dv, eps, s);
}
