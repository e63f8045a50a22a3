// Linear recurrences whose memory is written BEFORE it is read, state [Dk, Dv] (key channel x value channel) in fp32
// per head, carried per SEQUENCE in numbered slots (a sequence whose rows start at position 0 starts from a zero state
// whatever its slot holds).  Two forms share one kernel; both are  S <- diag(w) S + k v^T,  o = S^T r  with per-token
// vectors w, k, r [Dk] made from the raw projections in fp32:
//
//   nv_mlstm_memory        (matrix memory with exponential gates and a running maximum that keeps them bounded)
//       i = cap tanh((i_raw + b_i) / cap);   f = logsigmoid(cap tanh((f_raw + b_f) / cap))         per head
//       m_t = max(f + m_(t-1), i);   w = exp(f + m_(t-1) - m_t) (one number per head);   k = exp(i - m_t) k_t
//       r = q_t * q_scale;   n_t = w n_(t-1) + k   (a vector [Dk] carried beside S, as is m; m starts at 0)
//       o <- o / (max(|n_t . r|, exp(-m_t)) + 1e-6)
//       out = o / sqrt(mean(o^2) + eps) * norm_w[h] * sigmoid(gate_raw)                            per head
//
//   nv_gated_write_memory  (keyless: what is written is one minus the forget gate)
//       f = lower + (1 - lower) sigmoid(f_raw + b_f)   per head and key channel;   w = f;   k = 1 - f;   r = silu(q_raw)
//       out = o / sqrt(mean(o^2) + eps) * norm_w        (one weight [Dv] for all heads)
//
// Layout as in the decayed-memory kernel next door: one workgroup per (sequence, head); a lane owns one value column
// and a quarter of the key rows (its quad index q owns rows q * RPL .. q * RPL + RPL - 1, read from LDS four at a time,
// the four runs RPL + 4 words apart so that a quad's 16-byte reads fall on different banks), so the state lives in
// registers and the token loop has no workgroup barrier: the vectors of up to 16 tokens are prepared into LDS by all
// waves together (the running maximum of those tokens is a short serial chain of additions and maxima on one thread,
// every exponential around it is taken in parallel), each wave then runs those tokens for its 16 columns, and the
// tile's output is normalised and written by all waves.
#include <algorithm>

#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kGmMaxTile = 16;
constexpr int kGmLdsBudget = 60 * 1024;

__device__ __forceinline__ float gm_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float gm_logsigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float gm_quad_sum(float x) {
    x += dpp_f32<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp_f32<0x4E>(x);   // quad_perm [2,3,0,1]
    return x;
}

template <typename T>
struct GmArgs {
    const T *q, *k, *v;                    // q: [T, H * Dk]; k: [T, H * Dk] (matrix form); v: [T, H * Dv]
    int64_t q_stride, k_stride, v_stride;
    const T* f_raw;                        // gated-write form: [T, H * Dk]
    int64_t f_stride;
    const float *i_pre, *f_pre;            // matrix form: [T, H] fp32 gate pre-activations (without bias)
    int64_t gate_pre_stride;
    const T* gate_raw;                     // output gate [T, H * Dv] or NULL
    int64_t gate_stride;
    const float *i_bias, *f_bias;          // matrix form: [H], [H]; gated-write form: f_bias [H * Dk]
    const float* lower;                    // gated-write form: [H * Dk]
    const float* norm_w;                   // [H * Dv] (norm_head_stride = Dv) or [Dv] (0)
    int norm_head_stride;
    float *state, *nstate, *mstate;        // [slots, H, Dk, Dv], [slots, H, Dk], [slots, H]
    T* out;                                // [T, H * Dv]
    int64_t out_stride;
    const int *cu_q, *cu_k, *slots;
    int H, Dk, Dv;
    float eps, cap, q_scale;
    int tile;
};

template <typename T, int RPL, bool MATRIX, int MAXT>
__global__ __launch_bounds__(MAXT) void gated_memory_kernel(const GmArgs<T> a) {
    constexpr int DP = (RPL + 4) * 4;                 // LDS words per token and vector: four runs of RPL rows, padded
    constexpr int NPL = (4 * RPL + 63) / 64;          // key channels a lane of wave 0 owns for the vector n
    extern __shared__ float smem[];
    const int tile = a.tile, Dk = a.Dk, Dv = a.Dv, H = a.H;
    float* ws = smem;                                 // [tile][DP] decay
    float* ks = ws + tile * DP;                       // [tile][DP] what is written
    float* rs = ks + tile * DP;                       // [tile][DP] read-out vector
    float* vs = rs + tile * DP;                       // [tile][Dv]
    float* os = vs + tile * Dv;                       // [tile][Dv]
    float* gi = os + tile * Dv;                       // [tile] log input gate, then exp(i - m_t)
    float* gf = gi + tile;                            // [tile] log forget gate, then exp(f + m_(t-1) - m_t)
    float* gm = gf + tile;                            // [tile] m_t, then the denominator of the token
    const int b = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
    const int q0 = a.cu_q[b], len_q = a.cu_q[b + 1] - q0;
    if (len_q <= 0) return;
    const int start = (a.cu_k[b + 1] - a.cu_k[b]) - len_q;
    const int col = wave * 16 + (lane >> 2), q = lane & 3;
    const bool live = col < Dv;
    const int64_t slot_head = (int64_t)a.slots[b] * H + h;
    float* S_slot = a.state + slot_head * (int64_t)Dk * Dv;
    float S[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int row = q * RPL + i;
        S[i] = (live && start > 0 && row < Dk) ? S_slot[(int64_t)row * Dv + col] : 0.f;
    }
    float nvec[NPL];                                  // wave 0: n of the channels lane, lane + 64, ...
    float m_run = 0.f;                                // thread 0: the running maximum
    if constexpr (MATRIX) {
#pragma unroll
        for (int j = 0; j < NPL; ++j) {
            const int d = lane + 64 * j;
            nvec[j] = (wave == 0 && start > 0 && d < Dk) ? a.nstate[slot_head * Dk + d] : 0.f;
        }
        if (tid == 0 && start > 0) m_run = a.mstate[slot_head];
    }
    for (int t0 = 0; t0 < len_q; t0 += tile) {
        const int nt = min(tile, len_q - t0);
        __syncthreads();                              // the previous tile's epilogue has read os and gm
        if constexpr (MATRIX) {
            if (tid < nt) {
                const int64_t t = q0 + t0 + tid;
                const float ip = a.i_pre[t * a.gate_pre_stride + h] + a.i_bias[h];
                const float fp = a.f_pre[t * a.gate_pre_stride + h] + a.f_bias[h];
                gi[tid] = a.cap * tanhf(ip / a.cap);
                gf[tid] = gm_logsigmoid(a.cap * tanhf(fp / a.cap));
            }
            __syncthreads();
            if (tid == 0) {
                for (int tt = 0; tt < nt; ++tt) {
                    const float carried = gf[tt] + m_run;
                    m_run = fmaxf(carried, gi[tt]);
                    gf[tt] = carried;                 // f + m_(t-1)
                    gm[tt] = m_run;
                }
            }
            __syncthreads();
            if (tid < nt) {
                gi[tid] = expf(gi[tid] - gm[tid]);
                gf[tid] = expf(gf[tid] - gm[tid]);
            }
            __syncthreads();
        }
        for (int i = tid; i < nt * 4 * RPL; i += blockDim.x) {
            const int tt = i / (4 * RPL), d = i % (4 * RPL);
            const int at = tt * DP + (d / RPL) * (RPL + 4) + (d % RPL);
            float wv = 1.f, kv = 0.f, rv = 0.f;
            if (d < Dk) {
                const int64_t t = q0 + t0 + tt, hd = (int64_t)h * Dk + d;
                const float qv = (float)a.q[t * a.q_stride + hd];
                if constexpr (MATRIX) {
                    wv = gf[tt];
                    kv = gi[tt] * (float)a.k[t * a.k_stride + hd];
                    rv = qv * a.q_scale;
                } else {
                    const float lo = a.lower[hd];
                    wv = lo + (1.0f - lo) * gm_sigmoid((float)a.f_raw[t * a.f_stride + hd] + a.f_bias[hd]);
                    kv = 1.0f - wv;
                    rv = qv / (1.0f + expf(-qv));
                }
            }
            ws[at] = wv;
            ks[at] = kv;
            rs[at] = rv;
        }
        for (int i = tid; i < nt * Dv; i += blockDim.x) {
            const int tt = i / Dv, c = i % Dv;
            vs[tt * Dv + c] = (float)a.v[(int64_t)(q0 + t0 + tt) * a.v_stride + (int64_t)h * Dv + c];
        }
        __syncthreads();
        if constexpr (MATRIX) {
            // the normaliser n and every token's denominator, on wave 0 while the others start on the state
            if (wave == 0) {
                for (int tt = 0; tt < nt; ++tt) {
                    float dot = 0.f;
#pragma unroll
                    for (int j = 0; j < NPL; ++j) {
                        const int d = lane + 64 * j;
                        if (d < 4 * RPL) {
                            const int at = tt * DP + (d / RPL) * (RPL + 4) + (d % RPL);
                            nvec[j] = gf[tt] * nvec[j] + ks[at];
                            dot += nvec[j] * rs[at];
                        }
                    }
                    dot = wave_sum(dot);
                    if (lane == 0) gm[tt] = fmaxf(fabsf(dot), expf(-gm[tt])) + 1e-6f;
                }
            }
        }
        // ---- the recurrence over the tile, no barrier inside ---------------------------------------------
        if (live) {
            for (int tt = 0; tt < nt; ++tt) {
                const int base = tt * DP + q * (RPL + 4);
                const float4* wt = (const float4*)(ws + base);
                const float4* kt = (const float4*)(ks + base);
                const float4* rt = (const float4*)(rs + base);
                const float vc = vs[tt * Dv + col];
                float so = 0.f;
#pragma unroll
                for (int i = 0; i < RPL / 4; ++i) {
                    const float4 w4 = wt[i], k4 = kt[i], r4 = rt[i];
                    S[4 * i] = w4.x * S[4 * i] + k4.x * vc;
                    S[4 * i + 1] = w4.y * S[4 * i + 1] + k4.y * vc;
                    S[4 * i + 2] = w4.z * S[4 * i + 2] + k4.z * vc;
                    S[4 * i + 3] = w4.w * S[4 * i + 3] + k4.w * vc;
                    so += S[4 * i] * r4.x + S[4 * i + 1] * r4.y + S[4 * i + 2] * r4.z + S[4 * i + 3] * r4.w;
                }
                so = gm_quad_sum(so);
                if (q == 0) os[tt * Dv + col] = so;
            }
        }
        __syncthreads();
        // ---- the tile's output ---------------------------------------------------------------------------
        for (int tt = wave; tt < nt; tt += n_waves) {
            const int64_t t = q0 + t0 + tt;
            const float inv_den = MATRIX ? 1.0f / gm[tt] : 1.0f;
            float ss = 0.f;
            for (int c = lane; c < Dv; c += 64) {
                const float o = os[tt * Dv + c] * inv_den;
                ss += o * o;
            }
            ss = wave_sum(ss);
            const float rstd = inv_den / sqrtf(ss / (float)Dv + a.eps);
            for (int c = lane; c < Dv; c += 64) {
                const int64_t hc = (int64_t)h * Dv + c;
                float o = os[tt * Dv + c] * rstd * a.norm_w[(int64_t)h * a.norm_head_stride + c];
                if (a.gate_raw != nullptr) o *= gm_sigmoid((float)a.gate_raw[t * a.gate_stride + hc]);
                a.out[t * a.out_stride + hc] = (T)o;
            }
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            const int row = q * RPL + i;
            if (row < Dk) S_slot[(int64_t)row * Dv + col] = S[i];
        }
    }
    if constexpr (MATRIX) {
        if (wave == 0) {
#pragma unroll
            for (int j = 0; j < NPL; ++j) {
                const int d = lane + 64 * j;
                if (d < Dk) a.nstate[slot_head * Dk + d] = nvec[j];
            }
        }
        if (tid == 0) a.mstate[slot_head] = m_run;
    }
}

template <typename T, bool MATRIX>
static int launch_gated_memory(GmArgs<T> a, int B, hipStream_t s, const char* what) {
    const int waves = (a.Dv + 15) / 16;
    const dim3 grid((unsigned)B, (unsigned)a.H), block((unsigned)waves * 64);
    const int rpl = a.Dk <= 32 ? 8 : a.Dk <= 64 ? 16 : a.Dk <= 128 ? 32 : 64;
    const size_t per_token = sizeof(float) * (size_t)(3 * (rpl + 4) * 4 + 2 * a.Dv + 3);
    a.tile = (int)std::max<size_t>(1, std::min<size_t>(kGmMaxTile, kGmLdsBudget / per_token));
    const size_t smem = per_token * a.tile;
#define NV_GM_CASE(R)                                                                                            \
    case R:                                                                                                      \
        if (waves <= 4) hipLaunchKernelGGL((gated_memory_kernel<T, R, MATRIX, 256>), grid, block, smem, s, a);       \
        else if (waves <= 8) hipLaunchKernelGGL((gated_memory_kernel<T, R, MATRIX, 512>), grid, block, smem, s, a);  \
        else hipLaunchKernelGGL((gated_memory_kernel<T, R, MATRIX, 1024>), grid, block, smem, s, a);                 \
        break;
    switch (rpl) {
        NV_GM_CASE(8)
        NV_GM_CASE(16)
        NV_GM_CASE(32)
        default:
        NV_GM_CASE(64)
    }
#undef NV_GM_CASE
    return check_launch(what);
}

}  // namespace nv

extern "C" int nv_mlstm_memory(const void* q, const void* k, const void* v, int64_t q_stride, int64_t k_stride,
                               int64_t v_stride, const float* i_pre, const float* f_pre, int64_t gate_pre_stride,
                               const void* gate_raw, int64_t gate_stride, const float* i_bias, const float* f_bias,
                               const float* norm_w, float* state, float* norm_state, float* max_state, void* out,
                               int64_t out_stride, const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                               const int32_t* state_slots, int num_seqs, int H, int Dk, int Dv, float eps, float gate_cap,
                               float q_scale, int dtype, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && H > 0 && Dk > 0 && Dv > 0, NV_ERR_INVALID_ARG, "nv_mlstm_memory: bad sizes");
    if (num_seqs == 0) return NV_OK;
    NV_REQUIRE(q && k && v && i_pre && f_pre && gate_raw && i_bias && f_bias && norm_w && state && norm_state &&
                   max_state && out && cu_seqlens_q && cu_seqlens_k && state_slots,
               NV_ERR_INVALID_ARG, "nv_mlstm_memory: null pointer");
    NV_REQUIRE(Dk <= 256 && Dv <= 256, NV_ERR_UNSUPPORTED, "nv_mlstm_memory: Dk=%d, Dv=%d exceed 256", Dk, Dv);
    NV_REQUIRE(gate_cap > 0.f, NV_ERR_INVALID_ARG, "nv_mlstm_memory: the gate cap must be positive");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_mlstm_memory: bad dtype");
    NV_REQUIRE(H < 65536, NV_ERR_UNSUPPORTED, "nv_mlstm_memory: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16) {
        GmArgs<__bf16> a{(const __bf16*)q, (const __bf16*)k, (const __bf16*)v, q_stride, k_stride, v_stride, nullptr, 0,
                         i_pre, f_pre, gate_pre_stride, (const __bf16*)gate_raw, gate_stride, i_bias, f_bias, nullptr,
                         norm_w, Dv, state, norm_state, max_state, (__bf16*)out, out_stride, cu_seqlens_q, cu_seqlens_k,
                         state_slots, H, Dk, Dv, eps, gate_cap, q_scale, 0};
        return launch_gated_memory<__bf16, true>(a, num_seqs, s, "nv_mlstm_memory");
    }
    GmArgs<float> a{(const float*)q, (const float*)k, (const float*)v, q_stride, k_stride, v_stride, nullptr, 0, i_pre,
                    f_pre, gate_pre_stride, (const float*)gate_raw, gate_stride, i_bias, f_bias, nullptr, norm_w, Dv,
                    state, norm_state, max_state, (float*)out, out_stride, cu_seqlens_q, cu_seqlens_k, state_slots, H, Dk,
                    Dv, eps, gate_cap, q_scale, 0};
    return launch_gated_memory<float, true>(a, num_seqs, s, "nv_mlstm_memory");
}

extern "C" int nv_gated_write_memory(const void* q, const void* f_raw, const void* v, int64_t q_stride, int64_t f_stride,
                                     int64_t v_stride, const float* f_bias, const float* lower, const float* norm_w,
                                     float* state, void* out, int64_t out_stride, const int32_t* cu_seqlens_q,
                                     const int32_t* cu_seqlens_k, const int32_t* state_slots, int num_seqs, int H, int Dk,
                                     int Dv, float eps, int dtype, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && H > 0 && Dk > 0 && Dv > 0, NV_ERR_INVALID_ARG, "nv_gated_write_memory: bad sizes");
    if (num_seqs == 0) return NV_OK;
    NV_REQUIRE(q && f_raw && v && f_bias && lower && norm_w && state && out && cu_seqlens_q && cu_seqlens_k && state_slots,
               NV_ERR_INVALID_ARG, "nv_gated_write_memory: null pointer");
    NV_REQUIRE(Dk <= 256 && Dv <= 256, NV_ERR_UNSUPPORTED, "nv_gated_write_memory: Dk=%d, Dv=%d exceed 256", Dk, Dv);
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_gated_write_memory: bad dtype");
    NV_REQUIRE(H < 65536, NV_ERR_UNSUPPORTED, "nv_gated_write_memory: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16) {
        GmArgs<__bf16> a{(const __bf16*)q, nullptr, (const __bf16*)v, q_stride, 0, v_stride, (const __bf16*)f_raw, f_stride,
                         nullptr, nullptr, 0, nullptr, 0, nullptr, f_bias, lower, norm_w, 0, state, nullptr, nullptr,
                         (__bf16*)out, out_stride, cu_seqlens_q, cu_seqlens_k, state_slots, H, Dk, Dv, eps, 0.f, 1.f, 0};
        return launch_gated_memory<__bf16, false>(a, num_seqs, s, "nv_gated_write_memory");
    }
    GmArgs<float> a{(const float*)q, nullptr, (const float*)v, q_stride, 0, v_stride, (const float*)f_raw, f_stride, nullptr,
                    nullptr, 0, nullptr, 0, nullptr, f_bias, lower, norm_w, 0, state, nullptr, nullptr, (float*)out,
                    out_stride, cu_seqlens_q, cu_seqlens_k, state_slots, H, Dk, Dv, eps, 0.f, 1.f, 0};
    return launch_gated_memory<float, false>(a, num_seqs, s, "nv_gated_write_memory");
}
