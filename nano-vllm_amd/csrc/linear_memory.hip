// Linear recurrences with a decayed outer-product memory per head, state [Dk, Dv] (key channel x value channel) in
// fp32, carried per SEQUENCE in numbered slots (as the other recurrent kernels of this library: a sequence whose rows
// start at position 0 starts from a zero state whatever its slot holds).  Two forms share one kernel:
//
//   nv_decay_memory     (read before write, with a bonus for the current token; RWKV-style time mixing)
//       w = exp(-exp(w_raw + w_bias))                      decay per head and key channel
//       o = (S + diag(u) k v^T)^T r;   S <- diag(w) S + k v^T
//       out = o / sqrt(mean(o^2) + eps) * norm_w * silu(gate_raw)                  per head
//
//   nv_state_space_scan (write before read, one scalar decay per head and step; state-space duality)
//       dt = softplus(dt_raw + dt_bias);   a = exp(-exp(A_log) dt)
//       S <- a S + dt B x^T;   y = S^T C + D x;   out = y * silu(z)                (fp32; a grouped norm follows)
//
// Both reduce to  o = S_old^T r' + c v,  S <- diag(w) S_old + k v^T  with per-token vectors w, k, r' [Dk] and a scalar c:
// (r' = r, c = r . (u * k)) in the first form, (w = a, k = dt B, r' = a C, c = C . k + D) in the second.  Everything
// after the raw projections is fp32.
//
// nv_token_shift_mix    m_s[t] = h[t] + (h[t-1] - h[t]) * mu_s for several mixes s at once, the previous row of a
//                       sequence's first row carried in state[slot] (zeros at position 0).
// nv_group_rms_norm     y = x / sqrt(mean(part^2) + eps) * w over `groups` equal consecutive parts of fp32 rows.
//
// Layout as in the delta-rule kernels next door: one workgroup per (sequence, head); a lane owns one value column and
// a quarter of the key rows (its quad index q owns rows q * RPL .. q * RPL + RPL - 1, read from LDS four at a time,
// the four runs RPL + 4 words apart so that a quad's 16-byte reads fall on different banks), so the state lives in
// registers and the token loop has no workgroup barrier: the vectors of up to 16 tokens are prepared into LDS by all
// waves together, each wave then runs those tokens for its 16 columns, and the tile's output is written by all waves.
#include <algorithm>

#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kDmMaxTile = 16;
constexpr int kDmLdsBudget = 60 * 1024;

__device__ __forceinline__ float dm_silu(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float dm_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float dm_quad_sum(float x) {
    x += dpp_f32<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp_f32<0x4E>(x);   // quad_perm [2,3,0,1]
    return x;
}

template <typename T>
struct DmArgs {
    const T *r, *k, *v;                    // r, k: [T, G, Dk]; v: [T, H, Dv] (token strides below)
    int64_t r_stride, k_stride, v_stride;
    const T* w_raw;                        // bonus form: [T, H * Dk]; scan form: dt_raw [T, H]
    int64_t w_stride;
    const T* gate_raw;                     // [T, H * Dv]
    int64_t gate_stride;
    const float* w_bias;                   // bonus form: [H * Dk]; scan form: dt_bias [H]
    const float* bonus;                    // bonus form: u [H * Dk]; scan form: D [H]
    const float* rate;                     // scan form: A_log [H]
    const float* norm_w;                   // bonus form: [H * Dv]
    float* state;                          // [slots, H, Dk, Dv]
    void* out;                             // bonus form: T [T, H * Dv]; scan form: float [T, H * Dv]
    int64_t out_stride;
    const int *cu_q, *cu_k, *slots;
    int H, G, Dk, Dv;
    float eps;
    int tile;
};

// MAXT: the most threads a launch of this instantiation has (16 value columns per wave): the register budget of the state
// rows follows from it, so that the usual sizes (up to 128 value columns) keep the state in registers.
template <typename T, int RPL, bool SCAN, int MAXT>
__global__ __launch_bounds__(MAXT) void decay_memory_kernel(const DmArgs<T> a) {
    constexpr int DP = (RPL + 4) * 4;                 // LDS words per token and vector: four runs of RPL rows, padded
    extern __shared__ float smem[];
    const int tile = a.tile, Dk = a.Dk, Dv = a.Dv, H = a.H;
    float* ws = smem;                                 // [tile][DP] decay
    float* ks = ws + tile * DP;                       // [tile][DP] key
    float* rs = ks + tile * DP;                       // [tile][DP] read-out vector
    float* vs = rs + tile * DP;                       // [tile][Dv]
    float* os = vs + tile * Dv;                       // [tile][Dv]
    float* cs = os + tile * Dv;                       // [tile] weight of the current token's own value
    float* dts = cs + tile;                           // [tile] step size (scan form)
    float* decs = dts + tile;                         // [tile] scalar decay (scan form)
    const int b = blockIdx.x, h = blockIdx.y;
    const int g = h / (H / a.G);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n_waves = blockDim.x >> 6;
    const int q0 = a.cu_q[b], len_q = a.cu_q[b + 1] - q0;
    if (len_q <= 0) return;
    const int start = (a.cu_k[b + 1] - a.cu_k[b]) - len_q;
    const int col = wave * 16 + (lane >> 2), q = lane & 3;
    const bool live = col < Dv;
    float* S_slot = a.state + ((int64_t)a.slots[b] * H + h) * (int64_t)Dk * Dv;
    float S[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int row = q * RPL + i;
        S[i] = (live && start > 0 && row < Dk) ? S_slot[(int64_t)row * Dv + col] : 0.f;
    }
    for (int t0 = 0; t0 < len_q; t0 += tile) {
        const int nt = min(tile, len_q - t0);
        __syncthreads();                              // the previous tile's epilogue has read os
        if constexpr (SCAN) {
            if (tid < nt) {
                const int64_t t = q0 + t0 + tid;
                const float dt = dm_softplus((float)a.w_raw[t * a.w_stride + h] + a.w_bias[h]);
                dts[tid] = dt;
                decs[tid] = expf(-expf(a.rate[h]) * dt);
            }
            __syncthreads();
        }
        for (int i = tid; i < nt * 4 * RPL; i += blockDim.x) {
            const int tt = i / (4 * RPL), d = i % (4 * RPL);
            const int at = tt * DP + (d / RPL) * (RPL + 4) + (d % RPL);
            float wv = 1.f, kv = 0.f, rv = 0.f;
            if (d < Dk) {
                const int64_t t = q0 + t0 + tt, gd = (int64_t)g * Dk + d;
                kv = (float)a.k[t * a.k_stride + gd];
                rv = (float)a.r[t * a.r_stride + gd];
                if constexpr (SCAN) {
                    wv = decs[tt];
                    kv *= dts[tt];
                } else {
                    const int64_t hd = (int64_t)h * Dk + d;
                    wv = expf(-expf((float)a.w_raw[t * a.w_stride + hd] + a.w_bias[hd]));
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
        // the current token's own weight c, and (scan form) the read-out vector times the decay
        for (int tt = wave; tt < nt; tt += n_waves) {
            float cc = 0.f;
            for (int d = lane; d < 4 * RPL; d += 64) {
                const int at = tt * DP + (d / RPL) * (RPL + 4) + (d % RPL);
                if constexpr (SCAN) {
                    cc += rs[at] * ks[at];
                    rs[at] *= decs[tt];
                } else if (d < Dk) {
                    cc += rs[at] * a.bonus[(int64_t)h * Dk + d] * ks[at];
                }
            }
            cc = wave_sum(cc);
            if (lane == 0) cs[tt] = SCAN ? cc + a.bonus[h] : cc;
        }
        __syncthreads();
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
                    so += S[4 * i] * r4.x + S[4 * i + 1] * r4.y + S[4 * i + 2] * r4.z + S[4 * i + 3] * r4.w;
                    S[4 * i] = w4.x * S[4 * i] + k4.x * vc;
                    S[4 * i + 1] = w4.y * S[4 * i + 1] + k4.y * vc;
                    S[4 * i + 2] = w4.z * S[4 * i + 2] + k4.z * vc;
                    S[4 * i + 3] = w4.w * S[4 * i + 3] + k4.w * vc;
                }
                so = dm_quad_sum(so);
                if (q == 0) os[tt * Dv + col] = so + cs[tt] * vc;
            }
        }
        __syncthreads();
        // ---- the tile's output ---------------------------------------------------------------------------
        if constexpr (SCAN) {
            float* out = (float*)a.out;
            for (int i = tid; i < nt * Dv; i += blockDim.x) {
                const int tt = i / Dv, c = i % Dv;
                const int64_t t = q0 + t0 + tt, hc = (int64_t)h * Dv + c;
                out[t * a.out_stride + hc] = os[i] * dm_silu((float)a.gate_raw[t * a.gate_stride + hc]);
            }
        } else {
            T* out = (T*)a.out;
            for (int tt = wave; tt < nt; tt += n_waves) {
                const int64_t t = q0 + t0 + tt;
                float ss = 0.f;
                for (int c = lane; c < Dv; c += 64) ss += os[tt * Dv + c] * os[tt * Dv + c];
                ss = wave_sum(ss);
                const float rstd = 1.0f / sqrtf(ss / (float)Dv + a.eps);
                for (int c = lane; c < Dv; c += 64) {
                    const int64_t hc = (int64_t)h * Dv + c;
                    const float gate = dm_silu((float)a.gate_raw[t * a.gate_stride + hc]);
                    out[t * a.out_stride + hc] = (T)(os[tt * Dv + c] * rstd * a.norm_w[hc] * gate);
                }
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
}

template <typename T, bool SCAN>
static int launch_decay_memory(DmArgs<T> a, int B, hipStream_t s, const char* what) {
    const int waves = (a.Dv + 15) / 16;
    const dim3 grid((unsigned)B, (unsigned)a.H), block((unsigned)waves * 64);
    const int rpl = a.Dk <= 32 ? 8 : a.Dk <= 64 ? 16 : a.Dk <= 128 ? 32 : 64;
    const size_t per_token = sizeof(float) * (size_t)(3 * (rpl + 4) * 4 + 2 * a.Dv + 3);
    a.tile = (int)std::max<size_t>(1, std::min<size_t>(kDmMaxTile, kDmLdsBudget / per_token));
    const size_t smem = per_token * a.tile;
#define NV_DM_CASE(R)                                                                                           \
    case R:                                                                                                     \
        if (waves <= 4) hipLaunchKernelGGL((decay_memory_kernel<T, R, SCAN, 256>), grid, block, smem, s, a);        \
        else if (waves <= 8) hipLaunchKernelGGL((decay_memory_kernel<T, R, SCAN, 512>), grid, block, smem, s, a);   \
        else hipLaunchKernelGGL((decay_memory_kernel<T, R, SCAN, 1024>), grid, block, smem, s, a);                  \
        break;
    switch (rpl) {
        NV_DM_CASE(8)
        NV_DM_CASE(16)
        NV_DM_CASE(32)
        default:
        NV_DM_CASE(64)
    }
#undef NV_DM_CASE
    return check_launch(what);
}

// ------------------------------------------------------------------------------------------------ token shift
// One workgroup per token; a thread owns its channels, so the first row of a sequence's portion can read the carried
// row and then replace it with the portion's last row without a second launch.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(const T* __restrict__ h, int64_t h_stride,
                                                              const float* __restrict__ mu, int n_mix,
                                                              T* __restrict__ state, T* __restrict__ out,
                                                              const int* __restrict__ cu_q, const int* __restrict__ cu_k,
                                                              const int* __restrict__ slots, int B, int64_t T_rows, int C) {
    const int t = blockIdx.x;
    int lo = 0, hi = B;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid;
    }
    const int b = lo, i = t - cu_q[b];
    const int len_q = cu_q[b + 1] - cu_q[b];
    const int start = (cu_k[b + 1] - cu_k[b]) - len_q;
    T* st = state + (int64_t)slots[b] * C;
    const T* last = h + (int64_t)(cu_q[b + 1] - 1) * h_stride;
    for (int c = threadIdx.x; c < C; c += 256) {
        const float cur = (float)h[(int64_t)t * h_stride + c];
        float prev = 0.f;
        if (i > 0) prev = (float)h[(int64_t)(t - 1) * h_stride + c];
        else if (start > 0) prev = (float)st[c];
        if (i == 0) st[c] = last[c];
        for (int s = 0; s < n_mix; ++s)
            out[((int64_t)s * T_rows + t) * C + c] = (T)(cur + (prev - cur) * mu[(int64_t)s * C + c]);
    }
}

// ------------------------------------------------------------------------------------------------ grouped norm
template <typename T>
__global__ __launch_bounds__(64) void group_rms_norm_kernel(const float* __restrict__ x, int64_t x_stride,
                                                            const float* __restrict__ w, T* __restrict__ y,
                                                            int64_t y_stride, int groups, int gs, float eps) {
    const int64_t r = blockIdx.x;
    const int g = blockIdx.y, lane = threadIdx.x;
    const float* xr = x + r * x_stride + (int64_t)g * gs;
    float ss = 0.f;
    for (int c = lane; c < gs; c += 64) ss += xr[c] * xr[c];
    ss = wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int c = lane; c < gs; c += 64) y[r * y_stride + (int64_t)g * gs + c] = (T)(xr[c] * rstd * w[(int64_t)g * gs + c]);
}

}  // namespace nv

extern "C" int nv_decay_memory(const void* r, const void* k, const void* v, int64_t r_stride, int64_t k_stride,
                               int64_t v_stride, const void* w_raw, int64_t w_stride, const void* gate_raw,
                               int64_t gate_stride, const float* w_bias, const float* bonus, const float* norm_w,
                               float* state, void* out, int64_t out_stride, const int* cu_seqlens_q,
                               const int* cu_seqlens_k, const int* state_slots, int num_seqs, int H, int Dk, int Dv,
                               float eps, int dtype, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && H > 0 && Dk > 0 && Dv > 0, NV_ERR_INVALID_ARG, "nv_decay_memory: bad sizes");
    if (num_seqs == 0) return NV_OK;
    NV_REQUIRE(r && k && v && w_raw && gate_raw && w_bias && bonus && norm_w && state && out && cu_seqlens_q &&
                   cu_seqlens_k && state_slots,
               NV_ERR_INVALID_ARG, "nv_decay_memory: null pointer");
    NV_REQUIRE(Dk <= 256 && Dv <= 256, NV_ERR_UNSUPPORTED, "nv_decay_memory: Dk=%d, Dv=%d exceed 256", Dk, Dv);
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_decay_memory: bad dtype");
    NV_REQUIRE(H < 65536, NV_ERR_UNSUPPORTED, "nv_decay_memory: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16) {
        DmArgs<__bf16> a{(const __bf16*)r, (const __bf16*)k, (const __bf16*)v, r_stride, k_stride, v_stride,
                         (const __bf16*)w_raw, w_stride, (const __bf16*)gate_raw, gate_stride, w_bias, bonus, nullptr,
                         norm_w, state, out, out_stride, cu_seqlens_q, cu_seqlens_k, state_slots, H, H, Dk, Dv, eps, 0};
        return launch_decay_memory<__bf16, false>(a, num_seqs, s, "nv_decay_memory");
    }
    DmArgs<float> a{(const float*)r, (const float*)k, (const float*)v, r_stride, k_stride, v_stride, (const float*)w_raw,
                    w_stride, (const float*)gate_raw, gate_stride, w_bias, bonus, nullptr, norm_w, state, out, out_stride,
                    cu_seqlens_q, cu_seqlens_k, state_slots, H, H, Dk, Dv, eps, 0};
    return launch_decay_memory<float, false>(a, num_seqs, s, "nv_decay_memory");
}

extern "C" int nv_state_space_scan(const void* x, const void* Bm, const void* Cm, int64_t x_stride, int64_t b_stride,
                                   int64_t c_stride, const void* dt_raw, int64_t dt_stride, const void* z,
                                   int64_t z_stride, const float* dt_bias, const float* A_log, const float* D_skip,
                                   float* state, float* out, int64_t out_stride, const int* cu_seqlens_q,
                                   const int* cu_seqlens_k, const int* state_slots, int num_seqs, int H, int G, int N,
                                   int P, int dtype, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && H > 0 && G > 0 && N > 0 && P > 0, NV_ERR_INVALID_ARG, "nv_state_space_scan: bad sizes");
    if (num_seqs == 0) return NV_OK;
    NV_REQUIRE(x && Bm && Cm && dt_raw && z && dt_bias && A_log && D_skip && state && out && cu_seqlens_q &&
                   cu_seqlens_k && state_slots,
               NV_ERR_INVALID_ARG, "nv_state_space_scan: null pointer");
    NV_REQUIRE(H % G == 0, NV_ERR_INVALID_ARG, "nv_state_space_scan: H=%d not a multiple of G=%d", H, G);
    NV_REQUIRE(N <= 256 && P <= 256, NV_ERR_UNSUPPORTED, "nv_state_space_scan: N=%d, P=%d exceed 256", N, P);
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_state_space_scan: bad dtype");
    NV_REQUIRE(H < 65536, NV_ERR_UNSUPPORTED, "nv_state_space_scan: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16) {
        DmArgs<__bf16> a{(const __bf16*)Cm, (const __bf16*)Bm, (const __bf16*)x, c_stride, b_stride, x_stride,
                         (const __bf16*)dt_raw, dt_stride, (const __bf16*)z, z_stride, dt_bias, D_skip, A_log, nullptr,
                         state, out, out_stride, cu_seqlens_q, cu_seqlens_k, state_slots, H, G, N, P, 0.f, 0};
        return launch_decay_memory<__bf16, true>(a, num_seqs, s, "nv_state_space_scan");
    }
    DmArgs<float> a{(const float*)Cm, (const float*)Bm, (const float*)x, c_stride, b_stride, x_stride, (const float*)dt_raw,
                    dt_stride, (const float*)z, z_stride, dt_bias, D_skip, A_log, nullptr, state, out, out_stride,
                    cu_seqlens_q, cu_seqlens_k, state_slots, H, G, N, P, 0.f, 0};
    return launch_decay_memory<float, true>(a, num_seqs, s, "nv_state_space_scan");
}

extern "C" int nv_token_shift_mix(const void* h, int64_t h_stride, const float* mu, int n_mix, void* state, void* out,
                                  const int* cu_seqlens_q, const int* cu_seqlens_k, const int* state_slots,
                                  int num_seqs, int64_t T, int C, int dtype, void* stream) {
    using namespace nv;
    NV_REQUIRE(num_seqs >= 0 && T >= 0 && C > 0 && n_mix > 0, NV_ERR_INVALID_ARG, "nv_token_shift_mix: bad sizes");
    if (T == 0 || num_seqs == 0) return NV_OK;
    NV_REQUIRE(h && mu && state && out && cu_seqlens_q && cu_seqlens_k && state_slots, NV_ERR_INVALID_ARG,
               "nv_token_shift_mix: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_token_shift_mix: bad dtype");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_token_shift_mix: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(token_shift_mix_kernel<__bf16>, dim3((unsigned)T), dim3(256), 0, s, (const __bf16*)h, h_stride, mu,
                           n_mix, (__bf16*)state, (__bf16*)out, cu_seqlens_q, cu_seqlens_k, state_slots, num_seqs, T, C);
    else
        hipLaunchKernelGGL(token_shift_mix_kernel<float>, dim3((unsigned)T), dim3(256), 0, s, (const float*)h, h_stride, mu,
                           n_mix, (float*)state, (float*)out, cu_seqlens_q, cu_seqlens_k, state_slots, num_seqs, T, C);
    return check_launch("nv_token_shift_mix");
}

extern "C" int nv_group_rms_norm(const float* x, int64_t x_stride, const float* w, void* y, int64_t y_stride,
                                 int y_dtype, int64_t rows, int cols, int groups, float eps, void* stream) {
    using namespace nv;
    NV_REQUIRE(rows >= 0 && cols > 0 && groups > 0 && groups < 65536 && cols % groups == 0, NV_ERR_INVALID_ARG,
               "nv_group_rms_norm: groups=%d must divide cols=%d", groups, cols);
    if (rows == 0) return NV_OK;
    NV_REQUIRE(x && w && y, NV_ERR_INVALID_ARG, "nv_group_rms_norm: null pointer");
    NV_REQUIRE(y_dtype == NV_DTYPE_BF16 || y_dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_group_rms_norm: bad dtype");
    NV_REQUIRE(rows < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_group_rms_norm: launch too large");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)rows, (unsigned)groups);
    if (y_dtype == NV_DTYPE_BF16)
        hipLaunchKernelGGL(group_rms_norm_kernel<__bf16>, grid, dim3(64), 0, s, x, x_stride, w, (__bf16*)y, y_stride, groups,
                           cols / groups, eps);
    else
        hipLaunchKernelGGL(group_rms_norm_kernel<float>, grid, dim3(64), 0, s, x, x_stride, w, (float*)y, y_stride, groups,
                           cols / groups, eps);
    return check_launch("nv_group_rms_norm");
}
