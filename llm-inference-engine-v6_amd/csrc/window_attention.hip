// Softmax attention over paged keys and values for mixers whose heads are more than the plain kind:
//
//   * keys of `dk` and values of `dv` entries (the two sizes may differ), `nk` key heads and `nv` value heads with
//     nk = nv * maps: a value head is shared by `maps` score maps, each with a key head of its own. Query head
//     qh = (head, map) reads key head (head / (heads / nv)) * maps + map and value head head / (heads / nv);
//   * a score is scale * q . k, then softcap * tanh(score / softcap) where softcap > 0;
//   * a query at position p sees key j <= p with p - j < window (window 0: every j <= p) or j < keep_first (the first
//     tokens of a sequence stay visible behind a sliding window, at their true positions);
//   * `slopes` (one number a head): a score loses slope_h (p - j), a bias that grows with the distance;
//   * `sinks` (one number a head): the softmax's denominator also holds e^(sink_h), a key without a value.
//
// Three steps: `qk_prepare` turns the input product's 32-bit rows into queries and cache entries (an RMS norm per
// head with a weight over the head's entries where given, a rotation of the first `rot` entries by position x
// frequency, entry i with entry i + rot / 2 or, `pairs` = 1, entry 2 i with entry 2 i + 1; queries times a temperature
// 1 + coef ln(floor((p + 1) / every) + 1) where `every` > 0; nk = 0: the layer reads another layer's keys and values
// and only its queries are made), an attention kernel leaves per run of keys the maximum, the sum and the unscaled weighted values of
// every (token, query head), and `window_attention_finish` joins the runs in a fixed order and applies what a mixer
// does to a head's result before its output product: nothing, an element-wise sigmoid gate, a sigmoid gate of one
// number a head, or the difference of a head's two maps, o = a_1 - lambda a_2, divided by its root mean square; all
// times a constant.
//
// Scores, weights, norms, angles and sums over keys are 32-bit; q, k and v are read in their storage type.
// The kernel in this file is the plain-precision one (any sizes, both types); the matrix-core one is in
// window_attention_mfma.hip and leaves its results in the same form.
//
//   q          [T, nq * dk]                 nq = heads * maps
//   k_cache    [pages, nk, page, dk]        v_cache [pages, nv, dv, page]
//   part_o     [runs, T, nq, dv] 32-bit     part_ml [runs, T, nq, 2] (maximum, sum)
#include "common.h"
#include <math.h>

namespace llme {

constexpr int kMaxHeadEntries = 256;

// A workgroup per (token, group of heads): its four wavefronts take the group's heads in turn (queries first, then
// keys); gridDim.y groups share a token's heads. The angles of the token's position are made once per workgroup.
// Rows of p: queries at column 0, keys at k_col, values at v_col (v_col < 0: a value head is the key head as
// projected, before norm and rotation).
template <typename TQ, typename TC, typename TW>
__global__ __launch_bounds__(256) void qk_prepare_kernel(const float* __restrict__ p, int ld, int nq, int nk, int nv, int dk, int dv,
                                                         int k_col, int v_col, const TW* __restrict__ wq, const TW* __restrict__ wk,
                                                         float eps, const float* __restrict__ inv_freq, int rot, int pairs,
                                                         float qt_coef, int qt_every,
                                                         const int* __restrict__ positions, const int* __restrict__ seq_idx,
                                                         const int* __restrict__ block_table, int max_blocks,
                                                         TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                                         int page) {
    __shared__ float cs_t[kMaxHeadEntries / 2], sn_t[kMaxHeadEntries / 2];
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pos = positions[t];
    const float fpos = static_cast<float>(pos);
    const float* row = p + static_cast<size_t>(t) * ld;
    const int pg = nk > 0 ? block_table[static_cast<size_t>(seq_idx[t]) * max_blocks + pos / page] : 0;
    const int in_page = pos % page;
    const int half = rot / 2;
    // the queries' temperature at this position (32-bit)
    const float q_temp = qt_every > 0 ? 1.0f + qt_coef * logf(static_cast<float>((pos + 1) / qt_every + 1)) : 1.0f;
    for (int f = threadIdx.x; f < half; f += 256) {
        float sn, cs;
        sincosf(fpos * inv_freq[f], &sn, &cs);
        sn_t[f] = sn;
        cs_t[f] = cs;
    }
    __syncthreads();
    for (int u = blockIdx.y * 4 + wave; u < nq + nk; u += 4 * gridDim.y) {
        const bool is_q = u < nq;
        const int head = is_q ? u : u - nq;
        const float* hp = row + (is_q ? head * dk : k_col + head * dk);
        const TW* w = is_q ? wq : wk;
        float r = 1.f;
        if (w != nullptr) {
            float ss = 0.f;
            for (int e = lane; e < dk; e += 64) ss = fmaf(hp[e], hp[e], ss);
            r = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(dk) + eps);
        }
        for (int e = lane; e < dk; e += 64) {
            const float raw = hp[e];
            float v = w != nullptr ? raw * r * to_float(w[e]) : raw;
            if (e < rot) {
                const bool first = pairs ? (e & 1) == 0 : e < half;
                const int f = pairs ? e >> 1 : (e < half ? e : e - half);
                const int pe = pairs ? e ^ 1 : (e < half ? e + half : e - half);
                const float other = w != nullptr ? hp[pe] * r * to_float(w[pe]) : hp[pe];
                const float sn = sn_t[f], cs = cs_t[f];
                v = first ? v * cs - other * sn : v * cs + other * sn;
            }
            if (is_q) {
                q_out[(static_cast<size_t>(t) * nq + head) * dk + e] = from_float<TQ>(v * q_temp);
            } else {
                k_cache[((static_cast<size_t>(pg) * nk + head) * page + in_page) * dk + e] = from_float<TC>(v);
                if (v_col < 0) v_cache[((static_cast<size_t>(pg) * nv + head) * dv + e) * page + in_page] = from_float<TC>(raw);
            }
        }
    }
    if (v_col >= 0 && nv > 0) {
        const float* vp = row + v_col;
        for (int e = blockIdx.y * 256 + threadIdx.x; e < nv * dv; e += 256 * gridDim.y)
            v_cache[((static_cast<size_t>(pg) * nv + e / dv) * dv + e % dv) * page + in_page] = from_float<TC>(vp[e]);
    }
}

__device__ __forceinline__ bool key_visible(int key, int pos, int window, int keep_first) {
    return key <= pos && (window <= 0 || pos - key < window || key < keep_first);
}

// One workgroup per (token, query head): NW wavefronts take every NW-th chunk of 64 keys and join through LDS.
template <typename TQ, typename TC, int NW>
__global__ __launch_bounds__(NW * 64) void window_attention_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache, float* __restrict__ part_o,
    float* __restrict__ part_ml, const int* __restrict__ positions, const int* __restrict__ seq_idx,
    const int* __restrict__ block_table, int max_blocks, int nq, int nk, int nv, int maps, int dk, int dv, int page, float scale,
    float softcap, int window, int keep_first, const float* __restrict__ slopes) {
    constexpr int PER_LANE = kMaxHeadEntries / kWave;
    __shared__ float qs[kMaxHeadEntries];
    __shared__ float join_m[NW], join_l[NW];
    __shared__ float join_acc[NW > 1 ? NW : 1][NW > 1 ? kMaxHeadEntries : 1];
    const int t = blockIdx.x, qh = blockIdx.y;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int head = qh / maps, map = qh % maps;
    const int vh = head / (nq / maps / nv);
    const int kh = vh * maps + map;
    const int pos = positions[t];
    const int* table = block_table + static_cast<size_t>(seq_idx[t]) * max_blocks;
    const int hi = pos + 1;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int kept = keep_first < lo ? keep_first : lo;        // the first tokens that lie in front of the window
    const float slope = slopes != nullptr ? slopes[head] : 0.f;

    const TQ* qrow = q + (static_cast<size_t>(t) * nq + qh) * dk;
    for (int d = threadIdx.x; d < dk; d += NW * kWave) qs[d] = to_float(qrow[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[PER_LANE] = {0.f, 0.f, 0.f, 0.f};
    // the window's keys first (the first wavefront then always sees a key), then the kept ones
    for (int range = 0; range < 2; ++range) {
        const int r0 = range == 0 ? lo : 0, r1 = range == 0 ? hi : kept;
        for (int t0 = r0 + wave * kWave; t0 < r1; t0 += NW * kWave) {
            const int key = t0 + lane;
            float sc = -INFINITY;
            if (key < r1) {
                const int pg = table[key / page];
                const TC* kr = k_cache + ((static_cast<size_t>(pg) * nk + kh) * page + key % page) * dk;
                float dot = 0.f;
                for (int d = 0; d < dk; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
                sc = dot * scale;
                if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
                sc -= slope * static_cast<float>(pos - key);
            }
            const float m_new = fmaxf(m, wave_max(sc));
            const float alpha = expf(m - m_new);
            const float pr = (key < r1) ? expf(sc - m_new) : 0.f;
            l = l * alpha + wave_sum(pr);
            m = m_new;
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) acc[i] *= alpha;
            const int n = (r1 - t0 < kWave) ? r1 - t0 : kWave;
            for (int j = 0; j < n; ++j) {
                const int kj = t0 + j;
                const int pg = table[kj / page];
                const TC* vb = v_cache + (static_cast<size_t>(pg) * nv + vh) * dv * page + kj % page;
                const float pj = __shfl(pr, j, kWave);
#pragma unroll
                for (int i = 0; i < PER_LANE; ++i) {
                    const int d = lane + i * kWave;
                    if (d < dv) acc[i] = fmaf(pj, to_float(vb[static_cast<size_t>(d) * page]), acc[i]);
                }
            }
        }
    }
    if (NW > 1) {
        if (lane == 0) {
            join_m[wave] = m;
            join_l[wave] = l;
        }
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) join_acc[wave][lane + i * kWave] = acc[i];
        __syncthreads();
        if (wave != 0) return;
        float mx = -INFINITY;
        for (int w = 0; w < NW; ++w) mx = fmaxf(mx, join_m[w]);
        l = 0.f;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) acc[i] = 0.f;
        for (int w = 0; w < NW; ++w) {
            const float f = join_m[w] == -INFINITY ? 0.f : expf(join_m[w] - mx);
            l += f * join_l[w];
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) acc[i] += f * join_acc[w][lane + i * kWave];
        }
        m = mx;
    }
    const size_t at = static_cast<size_t>(t) * nq + qh;
    if (lane == 0) {
        part_ml[at * 2] = m;
        part_ml[at * 2 + 1] = l;
    }
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int d = lane + i * kWave;
        if (d < dv) part_o[at * dv + d] = acc[i];
    }
}

enum FinishMode : int { kFinishPlain = 0, kFinishGate = 1, kFinishDifference = 2, kFinishHeadGate = 3 };

// One wavefront per (token, head): the runs of each of the head's maps joined in the order of the runs, then the
// mixer's last step. gate [T, ld_gate] 32-bit, one entry per output entry (kFinishGate) or one per head
// (kFinishHeadGate). kFinishDifference: o = a_1 - lambda a_2 over the head's two maps, o / sqrt(mean(o^2) + eps).
// sinks [heads] (32-bit, or null; one map a head): the joined sum also holds e^(sink - maximum). All times out_scale.
template <typename TO, int MODE>
__global__ __launch_bounds__(256) void window_attention_finish_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                                      int runs, int T, int heads, int maps, int dv,
                                                                      const float* __restrict__ gate, int ld_gate, float lambda,
                                                                      float eps, float out_scale, const float* __restrict__ sinks,
                                                                      TO* __restrict__ out, int ld_out) {
    constexpr int PER_LANE = kMaxHeadEntries / kWave;
    const int lane = threadIdx.x & 63;
    const size_t item = static_cast<size_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (item >= static_cast<size_t>(T) * heads) return;
    const int t = static_cast<int>(item / heads), head = static_cast<int>(item % heads);
    const int nq = heads * maps;
    constexpr int MAPS = MODE == kFinishDifference ? 2 : 1;
    constexpr int CHUNK = 8;                // runs whose values are asked for together
    const size_t stride = static_cast<size_t>(T) * nq;
    const size_t at0 = static_cast<size_t>(t) * nq + head * MAPS;
    float a[MAPS][PER_LANE], l[MAPS];
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
        l[mp] = 0.f;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) a[mp][i] = 0.f;
    }
    // lane r holds run r's maximum and sum (64 runs at a time); the runs' values are then added in the order of the
    // runs, eight runs of every map of the head asked for before the first is used
    float mx[MAPS];
#pragma unroll
    for (int mp = 0; mp < MAPS; ++mp) {
        float v = -INFINITY;
        for (int r = lane; r < (runs == 1 ? 0 : runs); r += kWave) v = fmaxf(v, part_ml[(r * stride + at0 + mp) * 2]);
        mx[mp] = wave_max(v);
    }
    if (runs == 1) {                         // (prompts: one run, nothing to join)
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) {
            l[mp] = part_ml[(at0 + mp) * 2 + 1];
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) {
                const int d = lane + i * kWave;
                a[mp][i] = d < dv ? part_o[(at0 + mp) * dv + d] : 0.f;
            }
        }
    }
    for (int r0 = 0; r0 < (runs == 1 ? 0 : runs); r0 += kWave) {
        const int r = r0 + lane;
        float fr[MAPS], lr[MAPS];
#pragma unroll
        for (int mp = 0; mp < MAPS; ++mp) {
            fr[mp] = lr[mp] = 0.f;
            if (r < runs) {
                const float mr = part_ml[(r * stride + at0 + mp) * 2];
                fr[mp] = mr == -INFINITY ? 0.f : expf(mr - mx[mp]);            // (a run in which the row saw no key)
                lr[mp] = part_ml[(r * stride + at0 + mp) * 2 + 1];
            }
        }
        const int n = runs - r0 < kWave ? runs - r0 : kWave;
        for (int j0 = 0; j0 < n; j0 += CHUNK) {
            float v[CHUNK][MAPS][PER_LANE];
#pragma unroll
            for (int j = 0; j < CHUNK; ++j)
#pragma unroll
                for (int mp = 0; mp < MAPS; ++mp)
#pragma unroll
                    for (int i = 0; i < PER_LANE; ++i) {
                        const int d = lane + i * kWave;
                        v[j][mp][i] = (j0 + j < n && d < dv) ? part_o[((r0 + j0 + j) * stride + at0 + mp) * dv + d] : 0.f;
                    }
#pragma unroll
            for (int j = 0; j < CHUNK; ++j)
#pragma unroll
                for (int mp = 0; mp < MAPS; ++mp) {
                    const int jj = j0 + j < n ? j0 + j : 0;
                    const float f = j0 + j < n ? __shfl(fr[mp], jj, kWave) : 0.f;
                    l[mp] = fmaf(f, __shfl(lr[mp], jj, kWave), l[mp]);
#pragma unroll
                    for (int i = 0; i < PER_LANE; ++i) a[mp][i] = f != 0.f ? fmaf(f, v[j][mp][i], a[mp][i]) : a[mp][i];
                }
        }
    }
    if (MAPS == 1 && sinks != nullptr) {
        // the sink joins like a run that holds one weight and no value
        const float m0 = runs == 1 ? part_ml[at0 * 2] : mx[0];
        const float sk = sinks[head];
        const float top = fmaxf(m0, sk);
        const float f = m0 == -INFINITY ? 0.f : expf(m0 - top);
        l[0] = fmaf(l[0], f, expf(sk - top));
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) a[0][i] *= f;
    }
    float o[PER_LANE];
    {
        const float inv = 1.0f / l[0];
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) o[i] = a[0][i] * inv;
        if (MAPS == 2) {
            const float inv2 = 1.0f / l[MAPS - 1];
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) o[i] = fmaf(-lambda, a[MAPS - 1][i] * inv2, o[i]);
        }
    }
    float f = out_scale;
    if (MODE == kFinishDifference) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) ss = fmaf(o[i], o[i], ss);           // (entries beyond dv are zero)
        f = out_scale / sqrtf(wave_sum(ss) / static_cast<float>(dv) + eps);
    }
    if (MODE == kFinishHeadGate) f *= 1.0f / (1.0f + expf(-gate[static_cast<size_t>(t) * ld_gate + head]));
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int d = lane + i * kWave;
        if (d >= dv) continue;
        float v = o[i] * f;
        if (MODE == kFinishGate) {
            const float g = gate[static_cast<size_t>(t) * ld_gate + head * dv + d];
            v *= 1.0f / (1.0f + expf(-g));
        }
        out[static_cast<size_t>(t) * ld_out + head * dv + d] = from_float<TO>(v);
    }
}

}  // namespace llme

using namespace llme;

extern "C" int llme_qk_prepare(const float* p, int ld, int nq, int nk, int nv, int dk, int dv, int k_col, int v_col,
                               const void* wq, const void* wk, int w_dtype, float eps, const float* inv_freq, int rot,
                               int pairs, float qt_coef, int qt_every, const int* positions, const int* seq_idx, const int* block_table, int max_blocks, void* q_out,
                               int q_dtype, void* k_cache, void* v_cache, int cache_dtype, int page, int T, hipStream_t stream) {
    if (T <= 0) return 0;
    if (dk <= 0 || page <= 0 || rot < 0 || rot > dk || rot % 2 != 0 || qt_every < 0) return kErrBadArgument;
    if (nk > 0 && (dv <= 0 || nv <= 0 || nk % nv != 0 || k_cache == nullptr || v_cache == nullptr)) return kErrBadArgument;
    if (nk == 0) nv = 0;                    // (queries only: the keys and values are another layer's)
    if ((nk > 0 && (wq == nullptr) != (wk == nullptr)) || (rot > 0 && inv_freq == nullptr)) return kErrBadArgument;
    if (nk > 0 && v_col < 0 && (nk != nv || dk != dv)) return kErrBadArgument;
    if (dk > kMaxHeadEntries) return kErrBadArgument;
    // enough workgroups for the chip where the step has few tokens: up to a wavefront a head
    const int head_groups = (nq + nk + 3) / 4;
    const int want = (2048 + T - 1) / T;
    const dim3 grid(T, want < head_groups ? (want > 0 ? want : 1) : head_groups);
#define LLME_PREP(TQ, TC, TW)                                                                                              \
    hipLaunchKernelGGL((qk_prepare_kernel<TQ, TC, TW>), grid, dim3(256), 0, stream, p, ld, nq, nk, nv, dk, dv, k_col, v_col, \
                       static_cast<const TW*>(wq), static_cast<const TW*>(wk), eps, inv_freq, rot, pairs, qt_coef, qt_every, positions, seq_idx, \
                       block_table, max_blocks, static_cast<TQ*>(q_out), static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), page)
    if (q_dtype != cache_dtype) return kErrBadArgument;
    if (q_dtype == kF32 && w_dtype == kF32) LLME_PREP(float, float, float);
    else if (q_dtype == kBF16 && w_dtype == kF32) LLME_PREP(bf16, bf16, float);
    else if (q_dtype == kBF16 && w_dtype == kBF16) LLME_PREP(bf16, bf16, bf16);
    else return kErrBadArgument;
#undef LLME_PREP
    return launch_status();
}

extern "C" int llme_window_attention(const void* q, int q_dtype, const void* k_cache, const void* v_cache, int cache_dtype,
                                     float* part_o, float* part_ml, const int* positions, const int* seq_idx,
                                     const int* block_table, int max_blocks, int T, int nq, int nk, int nv, int dk, int dv, int page,
                                     float scale, float softcap, int window, int keep_first, const float* slopes,
                                     hipStream_t stream) {
    if (T <= 0) return 0;
    if (dk <= 0 || dk > kMaxHeadEntries || dv <= 0 || dv > kMaxHeadEntries || nv <= 0 || nk % nv != 0 || page <= 0) return kErrBadArgument;
    const int maps = nk / nv;
    if (nq % nk != 0 || window < 0 || keep_first < 0) return kErrBadArgument;
    const dim3 grid(T, nq);
    const bool few = static_cast<long>(T) * nq < 4096;
#define LLME_WATT(TQ, TC)                                                                                          \
    do {                                                                                                           \
        if (few)                                                                                                   \
            hipLaunchKernelGGL((window_attention_kernel<TQ, TC, 8>), grid, dim3(8 * 64), 0, stream,                \
                               static_cast<const TQ*>(q), static_cast<const TC*>(k_cache), static_cast<const TC*>(v_cache), \
                               part_o, part_ml, positions, seq_idx, block_table, max_blocks, nq, nk, nv, maps, dk, dv, page, \
                               scale, softcap, window, keep_first, slopes);                                              \
        else                                                                                                       \
            hipLaunchKernelGGL((window_attention_kernel<TQ, TC, 1>), grid, dim3(64), 0, stream,                    \
                               static_cast<const TQ*>(q), static_cast<const TC*>(k_cache), static_cast<const TC*>(v_cache), \
                               part_o, part_ml, positions, seq_idx, block_table, max_blocks, nq, nk, nv, maps, dk, dv, page, \
                               scale, softcap, window, keep_first, slopes);                                              \
    } while (0)
    if (q_dtype == kF32 && cache_dtype == kF32) LLME_WATT(float, float);
    else if (q_dtype == kBF16 && cache_dtype == kBF16) LLME_WATT(bf16, bf16);
    else return kErrBadArgument;
#undef LLME_WATT
    return launch_status();
}

extern "C" int llme_window_attention_finish(const float* part_o, const float* part_ml, int runs, int T, int heads, int maps, int dv,
                                            int mode, const float* gate, int ld_gate, float lambda, float eps, float out_scale,
                                            const float* sinks, void* out, int out_dtype, int ld_out, hipStream_t stream) {
    if (T <= 0) return 0;
    if (runs <= 0 || heads <= 0 || maps <= 0 || dv <= 0 || dv > kMaxHeadEntries) return kErrBadArgument;
    if ((mode == kFinishDifference && maps != 2) || (mode != kFinishDifference && maps != 1)) return kErrBadArgument;
    if ((mode == kFinishGate || mode == kFinishHeadGate) && gate == nullptr) return kErrBadArgument;
    if (sinks != nullptr && maps != 1) return kErrBadArgument;
    const dim3 grid(static_cast<unsigned>((static_cast<size_t>(T) * heads + 3) / 4));
#define LLME_FIN(TO, MODE)                                                                                            \
    hipLaunchKernelGGL((window_attention_finish_kernel<TO, MODE>), grid, dim3(256), 0, stream, part_o, part_ml, runs, T, heads, \
                       maps, dv, gate, ld_gate, lambda, eps, out_scale, sinks, static_cast<TO*>(out), ld_out)
#define LLME_FIN_T(TO)                                                     \
    do {                                                                   \
        if (mode == kFinishPlain) LLME_FIN(TO, kFinishPlain);              \
        else if (mode == kFinishGate) LLME_FIN(TO, kFinishGate);           \
        else if (mode == kFinishDifference) LLME_FIN(TO, kFinishDifference); \
        else if (mode == kFinishHeadGate) LLME_FIN(TO, kFinishHeadGate);   \
        else return kErrBadArgument;                                       \
    } while (0)
    if (out_dtype == kF32) LLME_FIN_T(float);
    else if (out_dtype == kBF16) LLME_FIN_T(bf16);
    else return kErrBadArgument;
#undef LLME_FIN_T
#undef LLME_FIN
    return launch_status();
}

LLME_LOAD_ENTRY(window_attention)
