// The attention of window_attention.hip on the matrix cores (v_mfma_f32_16x16x32_bf16), bfloat16 queries, keys and
// values; prompts, portions and single decoded tokens are the same case.
//
// A wavefront takes 16 consecutive (token, head) pairs of one request that read the same key head (the heads of a
// value head fastest, so with 16 heads on a value head a tile is one token, with one head 16 tokens); every row has
// its own position and so its own visible keys. Keys are walked in blocks of 32: the blocks that hold the first
// keep_first tokens where they lie in front of the window, then the blocks from the window's start of the tile's
// first row to the position of its last. The blocks of a tile are cut into `nsplit` runs (grid z); every run leaves
// its maximum, sum and unscaled weighted values, which window_attention_finish joins in the order of the runs.
//
//   S^T[key, row] = sum_d K[key, d] Q[row, d]     first operand: a key's entries as they lie in its page, 16 bytes a lane
//   O^T[c, row]  += sum_key V^T[c, key] P^T[key, row]
// Lane l holds, for query row l % 16, the scores of keys 4 (l / 16) + e of both 16-key halves of a block: exactly the 8
// keys it supplies as second operand of the second product, so weights never leave their registers. A weight is
// 32-bit; it enters the second product as the sum of two bfloat16 parts (16 bits of mantissa), and the row's sum adds
// the 32-bit weights. Operands come straight from the pages (no LDS): the four wavefronts of a workgroup take tiles
// next to each other and find each other's keys in the cache.
#include "common.h"
#include <math.h>

namespace llme {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

struct WindowArgs {
    const bf16* q;              // [T, nq, dk]
    const bf16* k_cache;        // [pages, nk, page, dk]
    const bf16* v_cache;        // [pages, nv, dv, page]
    float* part_o;              // [nsplit, T, nq, dv]
    float* part_ml;             // [nsplit, T, nq, 2]
    const int* positions;
    const int* q_start;
    const int* block_table;
    int max_blocks, T, nq, nk, nv, maps, per_value_head, dk, dv, page, window, keep_first, nsplit;
    float scale, softcap;
};

template <int DSM, int NVM>     // 32-entry slabs of a key, 16-entry tiles of a value: the most this instance holds
__global__ __launch_bounds__(256) void window_attention_mfma_kernel(WindowArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, qd = lane >> 4;
    const int s = blockIdx.y / a.nk, kh = blockIdx.y % a.nk;
    const int vh = kh / a.maps, map = kh % a.maps;
    const int row0 = a.q_start[s];
    const int rows_total = (a.q_start[s + 1] - row0) * a.per_value_head;
    const int R0 = (blockIdx.x * 4 + wave) * 16;
    if (R0 >= rows_total) return;
    const bool valid = R0 + r < rows_total;
    const int R = valid ? R0 + r : rows_total - 1;
    const int t = row0 + R / a.per_value_head;
    const int qh = (vh * a.per_value_head + R % a.per_value_head) * a.maps + map;
    const int pos = a.positions[t];
    const int pos_min = a.positions[row0 + R0 / a.per_value_head];
    const int last_row = R0 + 15 < rows_total ? R0 + 15 : rows_total - 1;
    const int pos_max = a.positions[row0 + last_row / a.per_value_head];
    const int* table = a.block_table + static_cast<size_t>(s) * a.max_blocks;
    const int ds = (a.dk + 31) >> 5, nvt = a.dv >> 4;

    bf16x8 qf[DSM];
    {
        const bf16* qrow = a.q + (static_cast<size_t>(t) * a.nq + qh) * a.dk;
#pragma unroll
        for (int c = 0; c < DSM; ++c) {
            const int d0 = c * 32 + qd * 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[c][e] = static_cast<bf16>(0.f);
            if (c < ds && d0 < a.dk) qf[c] = *reinterpret_cast<const bf16x8*>(qrow + d0);
        }
    }

    // the tile's blocks of 32 keys: [0, nb_kept) and [first_blk, last_blk]
    const int lo_min = (a.window > 0 && pos_min - a.window + 1 > 0) ? pos_min - a.window + 1 : 0;
    int first_blk = lo_min >> 5;
    const int last_blk = pos_max >> 5;
    int nb_kept = 0;
    if (a.window > 0 && a.keep_first > 0) {
        const int kept = a.keep_first < lo_min ? a.keep_first : lo_min;
        const int kb = (kept + 31) >> 5;
        if (kb >= first_blk) first_blk = 0;
        else nb_kept = kb;
    }
    const int nblk = nb_kept + last_blk - first_blk + 1;
    const int per = (nblk + a.nsplit - 1) / a.nsplit;
    const int b_begin = blockIdx.z * per;
    const int b_end = b_begin + per < nblk ? b_begin + per : nblk;

    float m = -INFINITY, l = 0.f;
    f32x4 acc[NVM];
#pragma unroll
    for (int c = 0; c < NVM; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int b = b_begin; b < b_end; ++b) {
        const int key0 = (b < nb_kept ? b : first_blk + b - nb_kept) << 5;
        f32x4 sc[2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            int key = key0 + sub * 16 + r;
            key = key < pos_max ? key : pos_max;               // (keys behind the tile's last are masked below)
            int pg = table[key / a.page];
            pg = pg < 0 ? 0 : pg;           // (a page that the window has left behind and given back: its keys are masked)
            const bf16* krow = a.k_cache + ((static_cast<size_t>(pg) * a.nk + kh) * a.page + key % a.page) * a.dk;
            sc[sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DSM; ++c) {
                const int d0 = c * 32 + qd * 8;
                if (c < ds) {
                    bf16x8 kf;
#pragma unroll
                    for (int e = 0; e < 8; ++e) kf[e] = static_cast<bf16>(0.f);
                    if (d0 < a.dk) kf = *reinterpret_cast<const bf16x8*>(krow + d0);
                    sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], sc[sub], 0, 0, 0);
                }
            }
        }
        // the values of this lane's 8 keys for every tile of value entries: asked for before the softmax
        bf16x8 vf[NVM];
        {
            int kq[2], pgs[2];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                kq[sub] = key0 + sub * 16 + qd * 4;
                const int kc = kq[sub] <= pos_max ? kq[sub] : (pos_max & ~3);
                pgs[sub] = table[kc / a.page];
                pgs[sub] = pgs[sub] < 0 ? 0 : pgs[sub];
                kq[sub] = kc;
            }
#pragma unroll
            for (int c = 0; c < NVM; ++c) {
                if (c < nvt) {
                    const int ch = c * 16 + r;
#pragma unroll
                    for (int sub = 0; sub < 2; ++sub) {
                        const bf16* vp = a.v_cache + ((static_cast<size_t>(pgs[sub]) * a.nv + vh) * a.dv + ch) * a.page + kq[sub] % a.page;
                        const bf16x4 v4 = *reinterpret_cast<const bf16x4*>(vp);
#pragma unroll
                        for (int e = 0; e < 4; ++e) vf[c][sub * 4 + e] = v4[e];
                    }
                }
            }
        }
        float p[8];
        float mx = -INFINITY;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = key0 + sub * 16 + qd * 4 + e;
                float v = sc[sub][e] * a.scale;
                if (a.softcap > 0.f) v = a.softcap * tanhf(v / a.softcap);
                const bool seen = valid && key <= pos && (a.window <= 0 || pos - key < a.window || key < a.keep_first);
                v = seen ? v : -INFINITY;
                p[sub * 4 + e] = v;
                mx = fmaxf(mx, v);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = expf(m - m_use);
        m = m_new;
        float sum = 0.f;
        bf16x8 ph, pl;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float w = expf(p[e] - m_use);
            sum += w;
            const bf16 hi = static_cast<bf16>(w);
            ph[e] = hi;
            pl[e] = static_cast<bf16>(w - static_cast<float>(hi));
        }
        l = l * alpha + sum;
#pragma unroll
        for (int c = 0; c < NVM; ++c) {
            if (c < nvt) {
                // a value behind the tile's last key may be anything that a freed page holds: its weight is zero, and
                // so is the value the product sees
                bf16x8 v = vf[c];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = key0 + (e >> 2) * 16 + qd * 4 + (e & 3);
                    if (key > pos_max) v[e] = static_cast<bf16>(0.f);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[c][e] *= alpha;
                acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, ph, acc[c], 0, 0, 0);
                acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pl, acc[c], 0, 0, 0);
            }
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!valid) return;
    const size_t at = (static_cast<size_t>(blockIdx.z) * a.T + t) * a.nq + qh;
    if (qd == 0) {
        a.part_ml[at * 2] = m;
        a.part_ml[at * 2 + 1] = l;
    }
#pragma unroll
    for (int c = 0; c < NVM; ++c)
        if (c < nvt) *reinterpret_cast<f32x4*>(a.part_o + at * a.dv + c * 16 + qd * 4) = acc[c];
}

}  // namespace llme

using namespace llme;

// max_new: the most tokens a request brings to the step (sizes the grid). Refuses (10002) what the kernel does not
// take: key entries no multiple of 8 or beyond 128, value entries no multiple of 16 or beyond 128, pages no multiple
// of 16.
extern "C" int llme_window_attention_mfma(const void* q, const void* k_cache, const void* v_cache, float* part_o, float* part_ml,
                                          const int* positions, const int* q_start, const int* block_table, int max_blocks, int T,
                                          int S, int max_new, int nq, int nk, int nv, int dk, int dv, int page, float scale,
                                          float softcap, int window, int keep_first, int nsplit, hipStream_t stream) {
    if (T <= 0 || S <= 0) return 0;
    if (nv <= 0 || nk % nv != 0 || nq % nk != 0 || max_new <= 0 || nsplit <= 0 || window < 0 || keep_first < 0) return kErrBadArgument;
    if (dk % 8 != 0 || dk > 128 || dv % 16 != 0 || dv > 128 || page % 16 != 0) return kErrUnsupported;
    WindowArgs a;
    a.q = static_cast<const bf16*>(q);
    a.k_cache = static_cast<const bf16*>(k_cache);
    a.v_cache = static_cast<const bf16*>(v_cache);
    a.part_o = part_o;
    a.part_ml = part_ml;
    a.positions = positions;
    a.q_start = q_start;
    a.block_table = block_table;
    a.max_blocks = max_blocks;
    a.T = T;
    a.nq = nq;
    a.nk = nk;
    a.nv = nv;
    a.maps = nk / nv;
    a.per_value_head = nq / nk;
    a.dk = dk;
    a.dv = dv;
    a.page = page;
    a.window = window;
    a.keep_first = keep_first;
    a.nsplit = nsplit;
    a.scale = scale;
    a.softcap = softcap;
    const int tiles = (max_new * a.per_value_head + 15) / 16;
    const dim3 grid((tiles + 3) / 4, S * nk, nsplit);
#define LLME_WMFMA(DSM, NVM) hipLaunchKernelGGL((window_attention_mfma_kernel<DSM, NVM>), grid, dim3(256), 0, stream, a)
    if (dk <= 64 && dv <= 64) LLME_WMFMA(2, 4);
    else if (dk <= 64) LLME_WMFMA(2, 8);
    else if (dv <= 64) LLME_WMFMA(4, 4);
    else LLME_WMFMA(4, 8);
#undef LLME_WMFMA
    return launch_status();
}

LLME_LOAD_ENTRY(window_attention_mfma)
