// Routed experts (mixture of experts with small clamped-GLU experts), without a host round trip:
//
// nv_moe_route          per token, from fp32 router logits [T, E]: the `top` largest (lowest index first among equals),
//                       their weights = softmax over the chosen logits only.  ids [T, top] int32, weights [T, top] fp32.
// nv_moe_align          sorts the T * top (token, choice) pairs by expert: sorted_pairs[position] = pair index, and a
//                       table of row tiles (expert, first position, rows) of at most `tile_rows` rows that never
//                       straddle two experts, plus their count, all on the device.
// nv_moe_gate_up        y[position, :] = act(G_e h, U_e h) for every sorted position (expert e, token of the pair):
//                       g = min(G_e h, limit), u = clamp(U_e h, -limit, limit), act = g * sigmoid(alpha g) * (u + 1).
// nv_moe_down           out[pair, :] = weight[pair] * (D_e y[position, :]), fp32, at the pair's own row: the caller sums
//                       the `top` rows of a token in a fixed order (no atomics, bitwise reproducible).
//
// Both products are one grouped matrix product on the matrix cores: a workgroup of four waves takes one row tile
// (16 or 64 rows of ONE expert) and 64 or 128 output columns, stages 64-deep (fp32: 32-deep) slices of the rows and of the
// expert's weight rows through LDS, the next slices already on their way into registers, and issues v_mfma_f32_16x16x32_bf16 (bfloat16) or v_mfma_f32_16x16x4_f32 (true fp32) on them; a
// wave owns 16 or 32 columns and all row sub-tiles.  Weights are
// [E, rows_out, rows_in] with the contraction index contiguous, as stored.  The launch is sized for the most tiles any
// routing can produce; workgroups beyond the table's count return at once.
#include <algorithm>

#include "nv_common.h"
#include "../../include/nanovllm_hip_mixers.h"

namespace nv {

constexpr int kMoeMaxTop = 16;
constexpr int kMoeBN = 64;

// One wave per token: a lane keeps the logits e = lane, lane + 64, ... in registers (up to kMoeRoutePerLane of them;
// more experts than that are re-read from memory), and every choice is a wave-wide arg-max (larger value, then lower
// index) after which the winner's lane strikes its element out.
constexpr int kMoeRoutePerLane = 8;            // experts <= 512 stay in registers
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int* __restrict__ ids,
                                                        float* __restrict__ wgt, int64_t T, int E, int top) {
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;                                // (whole waves leave together)
    const int lane = threadIdx.x & 63;
    const float* z = logits + t * E;
    float reg[kMoeRoutePerLane];
#pragma unroll
    for (int i = 0; i < kMoeRoutePerLane; ++i) {
        const int e = lane + 64 * i;
        reg[i] = e < E ? z[e] : -INFINITY;
    }
    unsigned taken = 0;                                // bit i: this lane's element i (of the first 32) is chosen
    int chosen[kMoeMaxTop];
    float val[kMoeMaxTop];
    for (int j = 0; j < top; ++j) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < kMoeRoutePerLane; ++i) {
            const int e = lane + 64 * i;
            if (e < E && !((taken >> i) & 1u) && (be == 0x7fffffff || reg[i] > bv)) { bv = reg[i]; be = e; }
        }
        for (int e = lane + 64 * kMoeRoutePerLane; e < E; e += 64) {      // the part that is not in registers
            bool gone = false;
            for (int i = 0; i < j; ++i) gone |= chosen[i] == e;
            const float v = z[e];
            if (!gone && (be == 0x7fffffff || v > bv)) { bv = v; be = e; }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(bv, off);
            const int oe = __shfl_xor(be, off);
            const bool mine_valid = be != 0x7fffffff, other_valid = oe != 0x7fffffff;
            if (other_valid && (!mine_valid || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
        }
        chosen[j] = be;
        val[j] = bv;
        if ((be & 63) == lane && be < 64 * kMoeRoutePerLane) taken |= 1u << (be >> 6);
    }
    if (lane == 0) {
        float sum = 0.f;
        const float top_logit = val[0];
        for (int j = 0; j < top; ++j) {
            val[j] = expf(val[j] - top_logit);
            sum += val[j];
        }
        for (int j = 0; j < top; ++j) {
            ids[t * top + j] = chosen[j];
            wgt[t * top + j] = val[j] / sum;
        }
    }
}

// Sigmoid scores with a selection bias and a choice limited to the best consecutive blocks of experts.  One wave per
// token: the biased scores go to LDS, a lane adds up the top two of its block, every group counts how many
// groups beat it (larger merit, then lower index) and is open when fewer than `keep` do; the choice is the wave-wide
// arg-max of nv_moe_route over the experts of open groups, and the weights are the plain sigmoids of the chosen.
constexpr int kMoeGroupedMaxE = 512;
__global__ __launch_bounds__(64) void moe_route_grouped_kernel(const float* __restrict__ logits, const float* __restrict__ corr,
                                                               int* __restrict__ ids, float* __restrict__ wgt, int E, int top,
                                                               int n_groups, int keep) {
    __shared__ float choice[kMoeGroupedMaxE];
    __shared__ float merit[kMoeGroupedMaxE];
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x;
    const float* z = logits + t * E;
    const int gs = E / n_groups;
    for (int e = lane; e < E; e += 64) {
        const float s = 1.0f / (1.0f + expf(-z[e]));
        choice[e] = corr != nullptr ? s + corr[e] : s;
    }
    __syncthreads();
    if (n_groups > 1) {
        for (int g = lane; g < n_groups; g += 64) {
            float a = -INFINITY, b = -INFINITY;                // the largest and the second largest of the group
            for (int i = 0; i < gs; ++i) {
                const float c = choice[g * gs + i];
                if (c > a) { b = a; a = c; } else if (c > b) b = c;
            }
            merit[g] = gs > 1 ? a + b : a;
        }
        __syncthreads();
        for (int g = lane; g < n_groups; g += 64) {
            const float mine = merit[g];
            int ahead = 0;
            for (int o = 0; o < n_groups; ++o) ahead += (merit[o] > mine || (merit[o] == mine && o < g)) ? 1 : 0;
            if (ahead >= keep)
                for (int i = 0; i < gs; ++i) choice[g * gs + i] = -INFINITY;
        }
        __syncthreads();
    }
    unsigned taken = 0;
    for (int j = 0; j < top; ++j) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
        for (int i = 0; i < kMoeGroupedMaxE / 64; ++i) {
            const int e = lane + 64 * i;
            if (e < E && !((taken >> i) & 1u) && (be == 0x7fffffff || choice[e] > bv)) { bv = choice[e]; be = e; }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(bv, off);
            const int oe = __shfl_xor(be, off);
            const bool mine_valid = be != 0x7fffffff, other_valid = oe != 0x7fffffff;
            if (other_valid && (!mine_valid || ov > bv || (ov == bv && oe < be))) { bv = ov; be = oe; }
        }
        if ((be & 63) == lane) taken |= 1u << (be >> 6);
        if (lane == 0) {
            ids[t * top + j] = be;
            wgt[t * top + j] = 1.0f / (1.0f + expf(-z[be]));
        }
    }
}

// One workgroup.  meta: [0] = number of tiles, then (expert, first position, rows) per tile.
__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, int* __restrict__ sorted_pairs,
                                                         int* __restrict__ meta, int64_t P, int E, int tile_rows) {
    extern __shared__ int sm[];                    // [E] counts, [E] cursors
    int* count = sm;
    int* cursor = sm + E;
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += 1024) count[e] = 0;
    __syncthreads();
    for (int64_t p = tid; p < P; p += 1024) atomicAdd(&count[ids[p]], 1);
    __syncthreads();
    if (tid == 0) {
        int off = 0, n = 0;
        for (int e = 0; e < E; ++e) {
            const int c = count[e];
            cursor[e] = off;
            for (int m = 0; m < c; m += tile_rows) {
                meta[1 + 3 * n] = e;
                meta[2 + 3 * n] = off + m;
                meta[3 + 3 * n] = min(tile_rows, c - m);
                ++n;
            }
            off += c;
        }
        meta[0] = n;
    }
    __syncthreads();
    for (int64_t p = tid; p < P; p += 1024) sorted_pairs[atomicAdd(&cursor[ids[p]], 1)] = (int)p;
}

template <typename T> struct MoeMma;
template <> struct MoeMma<__bf16> {
    static constexpr int kVec = 8, kPad = 8, kStep = 32, kBK = 64;
    // the 32-deep product of gfx950: a lane holds 8 consecutive k of its row (16-byte LDS reads)
    static __device__ __forceinline__ f32x4 run(const __bf16* a, const __bf16* b, int lg, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(*(const bf16x8*)(a + 8 * lg), *(const bf16x8*)(b + 8 * lg), c, 0, 0, 0);
    }
};
template <> struct MoeMma<float> {
    static constexpr int kVec = 4, kPad = 4, kStep = 4, kBK = 32;
    static __device__ __forceinline__ f32x4 run(const float* a, const float* b, int lg, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a[lg], b[lg], c, 0, 0, 0);
    }
};

// 16 bytes (kVec elements) of a row starting at k0, zeros past K or for a missing row
template <typename T>
__device__ __forceinline__ uint4 moe_fetch(const T* row, int k0, int K, bool vec_ok) {
    constexpr int V = MoeMma<T>::kVec;
    if (row == nullptr || k0 >= K) return make_uint4(0, 0, 0, 0);
    if (vec_ok && k0 + V <= K) return *(const uint4*)(row + k0);
    __attribute__((aligned(16))) T tmp[V];
#pragma unroll
    for (int i = 0; i < V; ++i) tmp[i] = k0 + i < K ? row[k0 + i] : (T)0.f;
    return *(const uint4*)tmp;
}

// MODE 1 (gate and up): A rows are gathered token rows, B holds the expert's gate rows and up rows, the epilogue is the
//         gated activation.
// MODE 2 (up alone):   A rows are gathered token rows, B the expert's up rows, the epilogue is max(x, 0)^2.
// MODE 0 (down):       A rows are the sorted activation rows, B the expert's down rows, the epilogue weights and scatters.
// The slices of the next step are fetched into registers while the current ones are multiplied out of LDS.
template <typename T, int MT, int NT, int MODE>
__global__ __launch_bounds__(256) void moe_grouped_kernel(
    const T* __restrict__ a, int64_t a_stride, const T* __restrict__ w, const int* __restrict__ sorted_pairs,
    const int* __restrict__ meta, const float* __restrict__ pair_w, T* __restrict__ y, float* __restrict__ out, int top,
    int N, int K, float limit, float alpha, float up_shift, int vec_ok, int max_tiles) {
    using M = MoeMma<T>;
    constexpr bool GATE_UP = MODE == 1, GATHER = MODE != 0;
    constexpr int BK = M::kBK, BM = 16 * MT, BN = 64 * NT, NB = GATE_UP ? 2 : 1, LD = BK + M::kPad, KV = BK / M::kVec;
    constexpr int A_IT = (BM * KV + 255) / 256, B_IT = (NB * BN * KV + 255) / 256;
    __shared__ __attribute__((aligned(16))) T As[BM * LD];
    __shared__ __attribute__((aligned(16))) T Bs[NB * BN * LD];
    __shared__ int src_row[BM];                    // gathered rows: token of the row; else the pair of the row; -1 past the tile
    // Workgroups go to the chip's 8 XCDs (each with its own L2) round robin by their index: index i runs item
    // (i % 8) * (items / 8) + i / 8, so one XCD works through neighbouring row tiles -- the tiles of one expert, which
    // share their weight slices in that L2.  Items: row tile fastest, then the column block.
    const int items = gridDim.x, per_xcd = items / 8;
    int item = blockIdx.x;
    if (item < per_xcd * 8) item = (item % 8) * per_xcd + item / 8;
    const int tile = item % max_tiles, n0 = (item / max_tiles) * BN;
    if (tile >= meta[0]) return;
    const int e = meta[1 + 3 * tile], row0 = meta[2 + 3 * tile], rows = meta[3 + 3 * tile];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lq = lane & 15, lg = lane >> 4;
    for (int i = tid; i < BM; i += 256) {
        const int pair = i < rows ? sorted_pairs[row0 + i] : -1;
        src_row[i] = pair < 0 ? -1 : (GATHER ? pair / top : pair);
    }
    __syncthreads();
    const T* we = w + (int64_t)e * (NB * (int64_t)N) * K;     // [NB * N, K] of this expert
    // what this thread stages: row pointers are fixed over the K loop
    const T* a_row[A_IT];
    const T* b_row[B_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
        const int it = tid + 256 * i, r = it / KV;
        a_row[i] = nullptr;
        if (it < BM * KV && r < rows) a_row[i] = GATHER ? a + (int64_t)src_row[r] * a_stride : a + (int64_t)(row0 + r) * a_stride;
    }
#pragma unroll
    for (int i = 0; i < B_IT; ++i) {
        const int it = tid + 256 * i, r = it / KV, n = n0 + (r % BN);
        b_row[i] = (it < NB * BN * KV && n < N) ? we + ((int64_t)(r / BN) * N + n) * K : nullptr;
    }
    uint4 a_reg[A_IT], b_reg[B_IT];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_IT; ++i) a_reg[i] = moe_fetch<T>(a_row[i], k0 + ((tid + 256 * i) % KV) * M::kVec, K, vec_ok != 0);
#pragma unroll
        for (int i = 0; i < B_IT; ++i) b_reg[i] = moe_fetch<T>(b_row[i], k0 + ((tid + 256 * i) % KV) * M::kVec, K, vec_ok != 0);
    };
    f32x4 acc[NB * NT][MT];
#pragma unroll
    for (int b = 0; b < NB * NT; ++b)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[b][m] = f32x4{0.f, 0.f, 0.f, 0.f};
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();                               // the previous slices have been consumed
#pragma unroll
        for (int i = 0; i < A_IT; ++i) {
            const int it = tid + 256 * i;
            if (it < BM * KV) *(uint4*)(As + (it / KV) * LD + (it % KV) * M::kVec) = a_reg[i];
        }
#pragma unroll
        for (int i = 0; i < B_IT; ++i) {
            const int it = tid + 256 * i;
            if (it < NB * BN * KV) *(uint4*)(Bs + (it / KV) * LD + (it % KV) * M::kVec) = b_reg[i];
        }
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += M::kStep) {
#pragma unroll
            for (int b = 0; b < NB * NT; ++b) {      // b = (gate | up) * NT + column sub-tile of this wave
                const T* brow = Bs + ((b / NT) * BN + (wave * NT + b % NT) * 16 + lq) * LD + kk;
#pragma unroll
                for (int m = 0; m < MT; ++m) acc[b][m] = M::run(As + (m * 16 + lq) * LD + kk, brow, lg, acc[b][m]);
            }
        }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int n = n0 + (wave * NT + nt) * 16 + lq;
        if (n >= N) continue;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = m * 16 + 4 * lg + i;
                if (r >= rows) continue;
                if constexpr (GATE_UP) {
                    const float g = fminf(acc[nt][m][i], limit);
                    const float u = fminf(fmaxf(acc[NT + nt][m][i], -limit), limit);
                    y[(int64_t)(row0 + r) * N + n] = (T)(g / (1.0f + expf(-alpha * g)) * (u + up_shift));
                } else if constexpr (MODE == 2) {
                    const float u = fmaxf(acc[nt][m][i], 0.f);
                    y[(int64_t)(row0 + r) * N + n] = (T)(u * u);
                } else {
                    const int pair = src_row[r];
                    out[(int64_t)pair * N + n] = acc[nt][m][i] * pair_w[pair];
                }
            }
        }
    }
}

template <typename T, int MODE>
static void launch_grouped(const void* a, int64_t a_stride, const void* w, const int* sorted_pairs, const int* meta,
                           const float* pair_w, void* y, float* out, int top, int N, int K, float limit, float alpha,
                           float up_shift, int max_tiles, int tile_rows, hipStream_t s) {
    const int vec = MoeMma<T>::kVec;
    const int vec_ok = K % vec == 0 && a_stride % vec == 0 && ((uintptr_t)a | (uintptr_t)w) % 16 == 0;
    // many rows per expert: 64 x 128 tiles (a wave owns 32 columns; 128-row tiles measured slower: one workgroup per CU);
    // few: 16 x 64 tiles, more workgroups per weight byte
#define NV_MOE_LAUNCH(MT, NT)                                                                                          \
    hipLaunchKernelGGL((moe_grouped_kernel<T, MT, NT, MODE>), dim3((unsigned)(max_tiles * ((N + 64 * NT - 1) / (64 * NT)))), \
                       dim3(256), 0, s, (const T*)a, a_stride, (const T*)w, sorted_pairs, meta, pair_w, (T*)y, out, top, N, K,  \
                       limit, alpha, up_shift, vec_ok, max_tiles)
    if (tile_rows == 64 && sizeof(T) == 2) NV_MOE_LAUNCH(4, 2);
    else if (tile_rows == 64) NV_MOE_LAUNCH(4, 1);
    else NV_MOE_LAUNCH(1, 1);
#undef NV_MOE_LAUNCH
}

}  // namespace nv

extern "C" int nv_moe_route(const float* logits, int32_t* ids, float* weights, int64_t T, int E, int top, void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && E > 0 && top >= 1 && top <= E && top <= kMoeMaxTop, NV_ERR_INVALID_ARG,
               "nv_moe_route: top=%d must lie in 1 .. min(E=%d, %d)", top, E, kMoeMaxTop);
    if (T == 0) return NV_OK;
    NV_REQUIRE(logits && ids && weights, NV_ERR_INVALID_ARG, "nv_moe_route: null pointer");
    NV_REQUIRE((T + 3) / 4 < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_moe_route: launch too large");
    hipLaunchKernelGGL(moe_route_kernel, dim3((unsigned)((T + 3) / 4)), dim3(256), 0, (hipStream_t)stream, logits, ids,
                       weights, T, E, top);
    return check_launch("nv_moe_route");
}

extern "C" int nv_moe_tile_rows(int64_t pairs, int E) { return pairs >= 32 * (int64_t)E ? 64 : 16; }

extern "C" int64_t nv_moe_max_tiles(int64_t pairs, int E, int tile_rows) {
    return pairs / tile_rows + std::min<int64_t>(pairs, E);
}

extern "C" int nv_moe_align(const int32_t* ids, int32_t* sorted_pairs, int32_t* meta, int64_t pairs, int E,
                            int tile_rows, void* stream) {
    using namespace nv;
    NV_REQUIRE(pairs >= 0 && E > 0 && E <= 4096 && (tile_rows == 16 || tile_rows == 64), NV_ERR_INVALID_ARG,
               "nv_moe_align: bad sizes");
    NV_REQUIRE(ids && sorted_pairs && meta, NV_ERR_INVALID_ARG, "nv_moe_align: null pointer");
    NV_REQUIRE(pairs < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_moe_align: too many pairs");
    hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), sizeof(int) * 2 * (size_t)E, (hipStream_t)stream, ids,
                       sorted_pairs, meta, pairs, E, tile_rows);
    return check_launch("nv_moe_align");
}

extern "C" int nv_moe_gate_up(const void* h, int64_t h_stride, const void* gate_up, const int32_t* sorted_pairs,
                              const int32_t* meta, void* y, int dtype, int64_t pairs, int E, int top, int width, int ff,
                              float limit, float alpha, int tile_rows, void* stream) {
    return nv_moe_gate_up_act(h, h_stride, gate_up, sorted_pairs, meta, y, dtype, pairs, E, top, width, ff, limit, alpha,
                              1.0f, tile_rows, stream);
}

extern "C" int nv_moe_gate_up_act(const void* h, int64_t h_stride, const void* gate_up, const int32_t* sorted_pairs,
                                  const int32_t* meta, void* y, int dtype, int64_t pairs, int E, int top, int width,
                                  int ff, float limit, float alpha, float up_shift, int tile_rows, void* stream) {
    using namespace nv;
    NV_REQUIRE(pairs >= 0 && E > 0 && top > 0 && width > 0 && ff > 0 && (tile_rows == 16 || tile_rows == 64),
               NV_ERR_INVALID_ARG, "nv_moe_gate_up: bad sizes");
    if (pairs == 0) return NV_OK;
    NV_REQUIRE(h && gate_up && sorted_pairs && meta && y, NV_ERR_INVALID_ARG, "nv_moe_gate_up: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_moe_gate_up: bad dtype");
    const int64_t tiles = nv_moe_max_tiles(pairs, E, tile_rows);
    NV_REQUIRE(tiles * ((ff + kMoeBN - 1) / kMoeBN) < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_moe_gate_up: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        launch_grouped<__bf16, 1>(h, h_stride, gate_up, sorted_pairs, meta, nullptr, y, nullptr, top, ff, width, limit,
                                     alpha, up_shift, (int)tiles, tile_rows, s);
    else
        launch_grouped<float, 1>(h, h_stride, gate_up, sorted_pairs, meta, nullptr, y, nullptr, top, ff, width, limit,
                                    alpha, up_shift, (int)tiles, tile_rows, s);
    return check_launch("nv_moe_gate_up");
}

extern "C" int nv_moe_down(const void* y, const void* down, const int32_t* sorted_pairs, const int32_t* meta,
                           const float* pair_weights, float* out, int dtype, int64_t pairs, int E, int width, int ff,
                           int tile_rows, void* stream) {
    using namespace nv;
    NV_REQUIRE(pairs >= 0 && E > 0 && width > 0 && ff > 0 && (tile_rows == 16 || tile_rows == 64), NV_ERR_INVALID_ARG,
               "nv_moe_down: bad sizes");
    if (pairs == 0) return NV_OK;
    NV_REQUIRE(y && down && sorted_pairs && meta && pair_weights && out, NV_ERR_INVALID_ARG, "nv_moe_down: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_moe_down: bad dtype");
    const int64_t tiles = nv_moe_max_tiles(pairs, E, tile_rows);
    NV_REQUIRE(tiles * ((width + kMoeBN - 1) / kMoeBN) < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_moe_down: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        launch_grouped<__bf16, 0>(y, ff, down, sorted_pairs, meta, pair_weights, nullptr, out, 1, width, ff, 0.f, 0.f, 0.f,
                                      (int)tiles, tile_rows, s);
    else
        launch_grouped<float, 0>(y, ff, down, sorted_pairs, meta, pair_weights, nullptr, out, 1, width, ff, 0.f, 0.f, 0.f,
                                     (int)tiles, tile_rows, s);
    return check_launch("nv_moe_down");
}

extern "C" int nv_moe_route_grouped(const float* logits, const float* correction, int32_t* ids, float* weights, int64_t T,
                                    int E, int top, int n_groups, int keep_groups, void* stream) {
    using namespace nv;
    NV_REQUIRE(T >= 0 && E > 0 && E <= kMoeGroupedMaxE && top >= 1, NV_ERR_INVALID_ARG,
               "nv_moe_route_grouped: E=%d must lie in 1 .. %d", E, kMoeGroupedMaxE);
    NV_REQUIRE(n_groups >= 1 && E % n_groups == 0 && keep_groups >= 1 && keep_groups <= n_groups, NV_ERR_INVALID_ARG,
               "nv_moe_route_grouped: %d groups must divide E=%d and hold the %d kept", n_groups, E, keep_groups);
    NV_REQUIRE(top <= keep_groups * (E / n_groups), NV_ERR_INVALID_ARG,
               "nv_moe_route_grouped: top=%d exceeds the %d experts of the kept groups", top, keep_groups * (E / n_groups));
    if (T == 0) return NV_OK;
    NV_REQUIRE(logits && ids && weights, NV_ERR_INVALID_ARG, "nv_moe_route_grouped: null pointer");
    NV_REQUIRE(T < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_moe_route_grouped: launch too large");
    hipLaunchKernelGGL(moe_route_grouped_kernel, dim3((unsigned)T), dim3(64), 0, (hipStream_t)stream, logits, correction, ids,
                       weights, E, top, n_groups, keep_groups);
    return check_launch("nv_moe_route_grouped");
}

extern "C" int nv_moe_up_relu2(const void* h, int64_t h_stride, const void* up, const int32_t* sorted_pairs,
                               const int32_t* meta, void* y, int dtype, int64_t pairs, int E, int top, int width, int ff,
                               int tile_rows, void* stream) {
    using namespace nv;
    NV_REQUIRE(pairs >= 0 && E > 0 && top > 0 && width > 0 && ff > 0 && (tile_rows == 16 || tile_rows == 64),
               NV_ERR_INVALID_ARG, "nv_moe_up_relu2: bad sizes");
    if (pairs == 0) return NV_OK;
    NV_REQUIRE(h && up && sorted_pairs && meta && y, NV_ERR_INVALID_ARG, "nv_moe_up_relu2: null pointer");
    NV_REQUIRE(dtype == NV_DTYPE_BF16 || dtype == NV_DTYPE_F32, NV_ERR_INVALID_ARG, "nv_moe_up_relu2: bad dtype");
    const int64_t tiles = nv_moe_max_tiles(pairs, E, tile_rows);
    NV_REQUIRE(tiles * ((ff + kMoeBN - 1) / kMoeBN) < (1LL << 31), NV_ERR_UNSUPPORTED, "nv_moe_up_relu2: launch too large");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == NV_DTYPE_BF16)
        launch_grouped<__bf16, 2>(h, h_stride, up, sorted_pairs, meta, nullptr, y, nullptr, top, ff, width, 0.f, 0.f, 0.f,
                                  (int)tiles, tile_rows, s);
    else
        launch_grouped<float, 2>(h, h_stride, up, sorted_pairs, meta, nullptr, y, nullptr, top, ff, width, 0.f, 0.f, 0.f,
                                 (int)tiles, tile_rows, s);
    return check_launch("nv_moe_up_relu2");
}
