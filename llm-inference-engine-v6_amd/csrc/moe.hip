// Mixture of experts: every token runs `top` of E small gated feed-forward layers.
//
//   moe_route    logits [T, E] (32-bit) -> per token the `top` experts with the largest scores (softmax over
//                the experts, or a sigmoid of each logit on its own; the lower index wins a tie) and their
//                weights = score * scale, renormalised over the chosen ones or not; pairs are numbered t * top + k
//   moe_plan     the pairs grouped by expert: every expert's pairs take a run of places padded to whole
//                tiles of `tile` rows; place -> pair (-1: padding), pair -> place, tile -> expert, number
//                of tiles. One workgroup; which place of its expert's run a pair takes depends on the
//                order of atomics, which no result depends on (every place is computed on its own).
//   moe_gemm     per tile of places: rows gathered (token = pair / top, or the place itself) times the
//                tile's expert's matrix [N, K]; plain or gated (act(gate) * up, gate and up rows in one matrix);
//                the plain-precision kernel; bfloat16 steps take the grouped instances of the matrix-core tile kernel
//   moe_combine  out[t] (+)= sum_k weight[t, k] * y[place of (t, k)], k in order (no weights: each counts once)
//
// Everything that depends on the routing is read from device memory: a step's launches are the same
// whatever the tokens choose (grids are sized for the most tiles there can be; workgroups beyond the
// number of tiles leave at once).
#include "common.h"
#include <math.h>

namespace llme {

__device__ __forceinline__ float moe_act(float g, int act) {
    if (act == 0) return g / (1.0f + expf(-g));
    if (act == 1) return fmaxf(g, 0.f);
    return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
}

constexpr int kMoeMaxPerLane = 16;      // experts per lane: up to 1024 experts

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int T, int E, int top,
                                                        float scale, int renorm, int sigmoid, int* __restrict__ ids,
                                                        float* __restrict__ wts) {
    const int lane = threadIdx.x & (kWave - 1);
    const int t = blockIdx.x * 4 + threadIdx.x / kWave;
    if (t >= T) return;
    const float* z = logits + static_cast<size_t>(t) * E;
    float v[kMoeMaxPerLane];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < kMoeMaxPerLane; ++i) {
        const int e = lane + i * kWave;
        v[i] = e < E ? z[e] : -INFINITY;
        mx = fmaxf(mx, v[i]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    if (!sigmoid) {
#pragma unroll
        for (int i = 0; i < kMoeMaxPerLane; ++i) {
            v[i] = expf(v[i] - mx);                 // 0 beyond E
            sum += v[i];
        }
    }
    // (sigmoid scores: the experts are chosen by their logits, which order them as the scores do and still tell
    // experts apart where the 32-bit sigmoid has run into 1 or 0; a chosen expert's score is made from its logit)
    const float inv = sigmoid ? 1.0f : 1.0f / wave_sum(sum);
    const float none = sigmoid ? -INFINITY : -1.f;
    float chosen_sum = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = none;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < kMoeMaxPerLane; ++i) {
            const int e = lane + i * kWave;
            if (e < E && v[i] > best) {         // (within a lane the experts rise: the first maximum stays)
                best = v[i];
                at = e;
            }
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, kWave);
            const int oa = __shfl_xor(at, off, kWave);
            if (ob > best || (ob == best && oa < at)) {
                best = ob;
                at = oa;
            }
        }
        const float s = sigmoid ? 1.0f / (1.0f + expf(-best)) : best * inv;
        chosen_sum += s;
        if (lane == 0) {
            ids[static_cast<size_t>(t) * top + k] = at;
            wts[static_cast<size_t>(t) * top + k] = s;
        }
#pragma unroll
        for (int i = 0; i < kMoeMaxPerLane; ++i)
            if (lane + i * kWave == at) v[i] = sigmoid ? -INFINITY : -2.f;        // taken
    }
    if (lane == 0) {
        const float f = renorm ? scale / chosen_sum : scale;
        for (int k = 0; k < top; ++k) wts[static_cast<size_t>(t) * top + k] *= f;
    }
}

// counts -> padded offsets -> places. E <= 1024.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int pairs, int E, int tile,
                                                        int cap, int* __restrict__ place_pair, int* __restrict__ pair_place,
                                                        int* __restrict__ tile_expert, int* __restrict__ n_tiles) {
    __shared__ int count[1024];
    __shared__ int offset[1025];
    __shared__ int fill[1024];
    for (int e = threadIdx.x; e < E; e += 1024) {
        count[e] = 0;
        fill[e] = 0;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += 1024) atomicAdd(&count[ids[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < E; ++e) {
            offset[e] = at;
            at += (count[e] + tile - 1) / tile * tile;
        }
        offset[E] = at;
        n_tiles[0] = at / tile;
    }
    __syncthreads();
    const int used = offset[E];
    for (int i = threadIdx.x; i < cap; i += 1024) place_pair[i] = -1;
    for (int e = threadIdx.x; e < E; e += 1024)
        for (int i = offset[e] / tile; i < offset[e + 1] / tile; ++i) tile_expert[i] = e;
    __syncthreads();
    for (int i = threadIdx.x; i < pairs; i += 1024) {
        const int e = ids[i];
        const int at = offset[e] + atomicAdd(&fill[e], 1);
        place_pair[at] = i;
        pair_place[i] = at;
    }
    (void)used;
}

// Pieces of 16 places x 64 columns (a tile of `tile` places is tile / 16 pieces), k in slabs of 32 through LDS, 32-bit
// sums. GATED: out = act(a . gate) * (a . up), the expert's matrix holding gate and up rows in alternating groups of
// `group` rows (2 N rows in all). gather_div > 0: row of `a` = pair / gather_div (the token); 0: the place itself.
// Rows of padding give zeros.
template <typename TA, typename TW, typename TO, bool GATED>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const TA* __restrict__ a, const TW* __restrict__ w, TO* __restrict__ out,
                                                       const int* __restrict__ place_pair, const int* __restrict__ tile_expert,
                                                       const int* __restrict__ n_tiles, int tile, int gather_div, int N, int K,
                                                       int group, int act) {
    __shared__ float As[16][33];
    __shared__ float Ws[64][33];
    __shared__ float Us[GATED ? 64 : 1][33];
    __shared__ int rows[16];
    const int piece = blockIdx.y;
    const int big = piece * 16 / tile;
    if (big >= n_tiles[0]) return;
    const int n0 = blockIdx.x * 64;
    const int e = tile_expert[big];
    if (threadIdx.x < 16) {
        const int pair = place_pair[piece * 16 + threadIdx.x];
        rows[threadIdx.x] = pair < 0 ? -1 : (gather_div > 0 ? pair / gather_div : piece * 16 + threadIdx.x);
    }
    __syncthreads();
    const int tr = threadIdx.x / 16, tc = threadIdx.x % 16;
    const TW* we = w + static_cast<size_t>(e) * (GATED ? 2 : 1) * N * K;
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, acu[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        for (int i = threadIdx.x; i < 16 * 32; i += 256) {
            const int rr = i / 32, kk = i % 32;
            const int row = rows[rr], k = k0 + kk;
            As[rr][kk] = (row >= 0 && k < K) ? to_float(a[static_cast<size_t>(row) * K + k]) : 0.f;
        }
        for (int i = threadIdx.x; i < 64 * 32; i += 256) {
            const int nn = i / 32, kk = i % 32;
            const int n = n0 + nn, k = k0 + kk;
            const bool in = n < N && k < K;
            const size_t row = GATED ? static_cast<size_t>(n / group) * 2 * group + n % group : n;      // the gate's row; up: group further
            Ws[nn][kk] = in ? to_float(we[row * K + k]) : 0.f;
            if (GATED) Us[nn][kk] = in ? to_float(we[(row + group) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < 32; ++kk) {
            const float av = As[tr][kk];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] = fmaf(av, Ws[tc + 16 * j][kk], acc[j]);
                if (GATED) acu[j] = fmaf(av, Us[tc + 16 * j][kk], acu[j]);
            }
        }
        __syncthreads();
    }
    TO* orow = out + (static_cast<size_t>(piece) * 16 + tr) * N;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + tc + 16 * j;
        if (n < N) orow[n] = from_float<TO>(GATED ? moe_act(acc[j], act) * acu[j] : acc[j]);
    }
}

__global__ void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ pair_place,
                                   const float* __restrict__ wts, float* __restrict__ out, int top, int H, int accumulate,
                                   size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / H;
    const int c = static_cast<int>(idx % H);
    float s = accumulate ? out[idx] : 0.f;
    for (int k = 0; k < top; ++k)
        s = fmaf(wts != nullptr ? wts[t * top + k] : 1.0f, y[static_cast<size_t>(pair_place[t * top + k]) * H + c], s);
    out[idx] = s;
}

}  // namespace llme

using namespace llme;

extern "C" int llme_moe_route(const float* logits, int T, int E, int top, float scale, int renorm, int sigmoid, int* ids,
                              float* wts, hipStream_t stream) {
    if (T <= 0) return 0;
    if (E <= 0 || top <= 0 || top > E) return kErrBadArgument;
    if (E > kMoeMaxPerLane * kWave) return kErrUnsupported;
    hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), 0, stream, logits, T, E, top, scale, renorm, sigmoid, ids, wts);
    return launch_status();
}

extern "C" int llme_moe_plan(const int* ids, int pairs, int E, int tile, int cap, int* place_pair, int* pair_place,
                             int* tile_expert, int* n_tiles, hipStream_t stream) {
    if (pairs <= 0) return 0;
    if (E <= 0 || tile <= 0) return kErrBadArgument;
    if (E > 1024) return kErrUnsupported;
    // room for every expert's run rounded up to whole tiles
    if (cap % tile || cap < (pairs + E * (tile - 1)) / tile * tile) return kErrBadArgument;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, E, tile, cap, place_pair, pair_place,
                       tile_expert, n_tiles);
    return launch_status();
}

// gated: w [experts, 2 N, K] with gate and up rows in alternating groups of `group`; else w [experts, N, K].
extern "C" int llme_moe_gemm(const void* a, int a_dtype, const void* w, int gated, int w_dtype, void* out,
                             int out_dtype, const int* place_pair, const int* tile_expert, const int* n_tiles, int tile,
                             int max_tiles, int gather_div, int N, int K, int group, int act, hipStream_t stream) {
    if (max_tiles <= 0 || N <= 0) return 0;
    if (tile <= 0 || tile % 16 || (gated && (group <= 0 || N % group))) return kErrBadArgument;
    if (K <= 0 || static_cast<long>(max_tiles) * (tile / 16) > 65535) return kErrUnsupported;
    const dim3 grid((N + 63) / 64, max_tiles * (tile / 16));
#define LLME_MG(TA, TW, TO)                                                                                      \
    do {                                                                                                         \
        if (gated)                                                                                               \
            hipLaunchKernelGGL((moe_gemm_kernel<TA, TW, TO, true>), grid, dim3(256), 0, stream,                  \
                               static_cast<const TA*>(a), static_cast<const TW*>(w), static_cast<TO*>(out),      \
                               place_pair, tile_expert, n_tiles, tile, gather_div, N, K, group, act);            \
        else                                                                                                     \
            hipLaunchKernelGGL((moe_gemm_kernel<TA, TW, TO, false>), grid, dim3(256), 0, stream,                 \
                               static_cast<const TA*>(a), static_cast<const TW*>(w), static_cast<TO*>(out),      \
                               place_pair, tile_expert, n_tiles, tile, gather_div, N, K, group, act);            \
    } while (0)
    if (a_dtype == kF32 && w_dtype == kF32 && out_dtype == kF32) LLME_MG(float, float, float);
    else if (a_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kBF16) LLME_MG(bf16, bf16, bf16);
    else if (a_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kF32) LLME_MG(bf16, bf16, float);
    else if (a_dtype == kBF16 && w_dtype == kF32 && out_dtype == kBF16) LLME_MG(bf16, float, bf16);
    else if (a_dtype == kBF16 && w_dtype == kF32 && out_dtype == kF32) LLME_MG(bf16, float, float);
    else return kErrBadArgument;
#undef LLME_MG
    return launch_status();
}

extern "C" int llme_moe_combine(const float* y, const int* pair_place, const float* wts, float* out, int T, int top,
                                int H, int accumulate, hipStream_t stream) {
    if (T <= 0) return 0;
    const size_t total = static_cast<size_t>(T) * H;
    hipLaunchKernelGGL(moe_combine_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream, y,
                       pair_place, wts, out, top, H, accumulate, total);
    return launch_status();
}

LLME_LOAD_ENTRY(moe)
