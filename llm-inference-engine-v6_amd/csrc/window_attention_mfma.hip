// The attention of window_attention.hip on the matrix cores (v_mfma_f32_16x16x32_bf16), bfloat16 queries, keys and
// values; prompts, portions and single decoded tokens are the same case.
//
// A wavefront takes 16 consecutive (token, head) pairs of one request that read the same key head (the heads of a
// value head fastest, so with 16 heads on a value head a tile is one token, with one head 16 tokens); every row has
// its own position and so its own visible keys. Keys are walked in blocks of 32: the blocks that hold the first
// keep_first tokens where they lie in front of the window, then the blocks from the window's start of the tile's
// first row to the position of its last. The blocks of a tile are cut into `nsplit` runs (grid z); every run leaves
// its maximum, sum and unscaled weighted values, which window_attention_finish joins in the order of the runs; where
// there is one run (prompts) and a head has one map, the kernel can finish its rows itself (sink, a gate per head, a
// scale) and write them in bfloat16.
//
//   S^T[key, row] = sum_d K[key, d] Q[row, d]     first operand: a key's entries as they lie in its page, 16 bytes a lane
//   O^T[c, row]  += sum_key V^T[c, key] P^T[key, row]
// The rows of a 16-key half are laid so that lane l ends up, for query row l % 16, with the scores of the 8 consecutive
// keys 8 (l / 16) .. of the block: exactly the keys it supplies as second operand of the second product (one 16-byte
// piece of a value row a tile), so weights never leave their registers. A weight is 32-bit; it enters the second
// product as the sum of two bfloat16 parts (16 bits of mantissa), and the row's sum adds the 32-bit weights. A score may
// be capped, or lose slope_h x (position - key) (`slopes`, one number a head). Blocks
// that every row of the tile sees whole (most of a window) skip the tests of visibility. Operands come straight from
// the pages (no LDS), the next block's keys asked for while this block's weights are made: the four wavefronts of a
// workgroup take tiles next to each other and find each other's keys in the cache.
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
    int max_blocks, T, nq, nk, nv, maps, per_value_head, dk, dv, page, page_shift, window, keep_first, nsplit;
    float scale, softcap;
    const float* slopes;        // [nq / maps] or null: a score loses slope (position - key)
    // Where the keys are in one run and a head has one map, the kernel may finish a row itself instead of leaving its
    // parts: out [T, ld_out] bfloat16 = acc / sum (the sum also holding e^(sink) where sinks [nq] are given), times
    // out_scale and, where head_gate [T, ld_gate] is given, times sigmoid(head_gate[t, head]). out null: the parts.
    bf16* out;
    const float* sinks;
    const float* head_gate;
    int ld_out, ld_gate;
    float out_scale;
};

// The end of a tile's walk: the row's parts into part_o / part_ml, or (a.out given) the finished row. l is the row's
// whole sum already.
template <int NVM>
__device__ __forceinline__ void window_store(const WindowArgs& a, const f32x4 (&acc)[NVM], float m, float l, int nvt, int t, int qh,
                                             int qd) {
    if (a.out != nullptr) {
        float f = 1.f, sum = l;
        if (a.sinks != nullptr) {               // the sink joins like a run that holds one weight and no value
            const float sk = a.sinks[qh];
            const float top = fmaxf(m, sk);
            f = m == -INFINITY ? 0.f : expf(m - top);
            sum = fmaf(l, f, expf(sk - top));
        }
        float mul = a.out_scale * f / sum;
        if (a.head_gate != nullptr) mul *= 1.0f / (1.0f + expf(-a.head_gate[static_cast<size_t>(t) * a.ld_gate + qh]));
        bf16* orow = a.out + static_cast<size_t>(t) * a.ld_out + qh * a.dv + qd * 4;
#pragma unroll
        for (int c = 0; c < NVM; ++c) {
            if (c < nvt) {
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = static_cast<__bf16>(acc[c][e] * mul);
                *reinterpret_cast<bf16x4*>(orow + c * 16) = o;
            }
        }
        return;
    }
    const size_t at = (static_cast<size_t>(blockIdx.z) * a.T + t) * a.nq + qh;
    if (qd == 0) {
        a.part_ml[at * 2] = m;
        a.part_ml[at * 2 + 1] = l;
    }
#pragma unroll
    for (int c = 0; c < NVM; ++c)
        if (c < nvt) *reinterpret_cast<f32x4*>(a.part_o + at * a.dv + c * 16 + qd * 4) = acc[c];
}

// What is done to a raw score besides the scale: nothing, a cap, or a bias that grows with the distance.
enum ScoreMode : int { kScorePlain = 0, kScoreCapped = 1, kScoreDistance = 2 };

// A capped score from the raw product: cap tanh(scale s / cap) = cap - 2 cap / (e^(2 scale s / cap) + 1), with the
// hardware's 32-bit power of two and reciprocal; `k` is 2 scale log2(e) / cap. (Where the score is near zero the
// result is exact to about cap x 1e-7.)
__device__ __forceinline__ float capped_score(float s, float k, float cap) {
    const float e = __builtin_amdgcn_exp2f(s * k);
    return fmaf(-2.f * cap, __builtin_amdgcn_rcpf(e + 1.f), cap);
}

// One block of 32 keys for a tile: scores in sc (this lane's row, keys key0 + 8 qd + j for j = 4 sub + e), values in vf.
// EDGE: some row of the tile does not see some key of the block (the window's start, the diagonal, kept tokens, rows
// beyond the request), or a key lies behind the tile's last; otherwise every weight counts and no test is made.
template <int NVM, bool EDGE, int CAP>
__device__ __forceinline__ void window_block(const WindowArgs& a, const f32x4 (&sc)[2], bf16x8 (&vf)[NVM], f32x4 (&acc)[NVM], float& m,
                                             float& l, int nvt, int key0, int qd, int pos, int pos_max, bool valid, float inv_cap, float slope) {
    float p[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float v0 = sc[j >> 2][j & 3];
        float v = CAP == kScoreCapped ? capped_score(v0, inv_cap, a.softcap) : v0 * a.scale;
        if (CAP == kScoreDistance) v = fmaf(slope, static_cast<float>(key0 + qd * 8 + j - pos), v);
        if (EDGE) {
            const int key = key0 + qd * 8 + j;
            const bool seen = valid && key <= pos && (a.window <= 0 || pos - key < a.window || key < a.keep_first);
            v = seen ? v : -INFINITY;
        }
        p[j] = v;
        mx = fmaxf(mx, v);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = (EDGE && m_new == -INFINITY) ? 0.f : m_new;
    // (where no row of the tile has a new maximum, which is the rule behind the first blocks, alpha is 1 for all)
    const bool rescale = __any(m_new != m);
    const float alpha = rescale ? __expf(m - m_use) : 1.f;
    m = m_new;
    float sum = 0.f;
    bf16x8 ph, pl;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float w = __expf(p[j] - m_use);
        sum += w;
        const bf16 hi = static_cast<bf16>(w);
        ph[j] = hi;
        pl[j] = static_cast<bf16>(w - static_cast<float>(hi));
    }
    l = rescale ? l * alpha + sum : l + sum;
#pragma unroll
    for (int c = 0; c < NVM; ++c) {
        if (c < nvt) {
            bf16x8 v = vf[c];
            if (EDGE) {
                // a value behind the tile's last key may be anything that a freed page holds: its weight is zero, and
                // so is the value the product sees
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (key0 + qd * 8 + j > pos_max) v[j] = static_cast<bf16>(0.f);
            }
            if (rescale) {
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[c][e] *= alpha;
            }
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, ph, acc[c], 0, 0, 0);
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pl, acc[c], 0, 0, 0);
        }
    }
}

// DSM, NVM: 32-entry slabs of a key, 16-entry tiles of a value: the most this instance holds. CAP: scores are capped.
template <int DSM, int NVM, int CAP>
__global__ __launch_bounds__(256, (DSM <= 2 && NVM <= 4) ? 4 : NVM <= 4 ? 3 : 2) void window_attention_mfma_kernel(WindowArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, qd = lane >> 4;
    const int s = blockIdx.y / a.nk, kh = blockIdx.y % a.nk;
    const int vh = kh / a.maps, map = kh % a.maps;
    const int row0 = a.q_start[s];
    const int rows_total = (a.q_start[s + 1] - row0) * a.per_value_head;
    const int R0 = (blockIdx.x * 4 + wave) * 16;
    if (R0 >= rows_total) return;
    const bool valid = R0 + r < rows_total;
    const bool all_valid = R0 + 15 < rows_total;
    const int R = valid ? R0 + r : rows_total - 1;
    const int t = row0 + R / a.per_value_head;
    const int qh = (vh * a.per_value_head + R % a.per_value_head) * a.maps + map;
    const int pos = a.positions[t];
    const int pos_min = a.positions[row0 + R0 / a.per_value_head];
    const int last_row = all_valid ? R0 + 15 : rows_total - 1;
    const int pos_max = a.positions[row0 + last_row / a.per_value_head];
    const int* table = a.block_table + static_cast<size_t>(s) * a.max_blocks;
    const int ds = (a.dk + 31) >> 5, nvt = a.dv >> 4;
    const int psh = a.page_shift, pmask = a.page - 1;
    const float inv_cap = a.softcap > 0.f ? 2.0f * 1.4426950408889634f * a.scale / a.softcap : 0.f;     // (capped_score's k)
    const float slope = CAP == kScoreDistance ? a.slopes[qh / a.maps] : 0.f;

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

    // Row i of a 16-key half `sub` of a block is key 8 (i / 4) + 4 sub + i % 4, so that the lane that ends up with rows
    // 4 qd .. 4 qd + 3 of both halves holds the 8 consecutive keys 8 qd .. 8 qd + 7: one 16-byte piece of a value row.
    const int k_in_block = 8 * (r >> 2) + (r & 3);
    bf16x8 kf[2][DSM];
    auto load_keys = [&](int b) {
        const int key0 = (b < nb_kept ? b : first_blk + b - nb_kept) << 5;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            int key = key0 + k_in_block + 4 * sub;
            key = key < pos_max ? key : pos_max;               // (keys behind the tile's last are masked below)
            int pg = table[key >> psh];
            pg = pg < 0 ? 0 : pg;           // (a page that the window has left behind and given back: its keys are masked)
            const bf16* krow = a.k_cache + (((static_cast<size_t>(pg) * a.nk + kh) << psh) + (key & pmask)) * a.dk;
#pragma unroll
            for (int c = 0; c < DSM; ++c) {
                const int d0 = c * 32 + qd * 8;
#pragma unroll
                for (int e = 0; e < 8; ++e) kf[sub][c][e] = static_cast<bf16>(0.f);
                if (c < ds && d0 < a.dk) kf[sub][c] = *reinterpret_cast<const bf16x8*>(krow + d0);
            }
        }
    };
    if (b_begin < b_end) load_keys(b_begin);

    for (int b = b_begin; b < b_end; ++b) {
        const int key0 = (b < nb_kept ? b : first_blk + b - nb_kept) << 5;
        // the values of this lane's 8 keys for every tile of value entries: asked for before the scores are made
        bf16x8 vf[NVM];
        {
            const int kq = key0 + qd * 8;
            const int kc = kq <= pos_max ? kq : (pos_max & ~7);
            int pg = table[kc >> psh];
            pg = pg < 0 ? 0 : pg;
            const bf16* vbase = a.v_cache + ((static_cast<size_t>(pg) * a.nv + vh) * a.dv << psh) + (kc & pmask);
#pragma unroll
            for (int c = 0; c < NVM; ++c)
                if (c < nvt) vf[c] = *reinterpret_cast<const bf16x8*>(vbase + (static_cast<size_t>(c * 16 + r) << psh));
        }
        f32x4 sc[2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            sc[sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DSM; ++c)
                if (c < ds) sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[sub][c], qf[c], sc[sub], 0, 0, 0);
        }
        if (b + 1 < b_end) load_keys(b + 1);                    // the next block's keys travel while this one's weights are made
        // every row sees every key of the block: behind the window's start of the tile's last row, up to the tile's
        // first position, not among the kept blocks (whose keys may lie beyond keep_first)
        const bool inner = all_valid && b >= nb_kept && key0 + 31 <= pos_min && (a.window <= 0 || pos_max - key0 < a.window);
        if (inner) window_block<NVM, false, CAP>(a, sc, vf, acc, m, l, nvt, key0, qd, pos, pos_max, valid, inv_cap, slope);
        else window_block<NVM, true, CAP>(a, sc, vf, acc, m, l, nvt, key0, qd, pos, pos_max, valid, inv_cap, slope);
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!valid) return;
    window_store<NVM>(a, acc, m, l, nvt, t, qh, qd);
}

// ---------------------------------------------------------------------------------------------------------------
// The same attention for steps in which a request brings many rows (prompts and their portions): the four wavefronts
// of a workgroup take tiles next to each other, so they walk nearly the same keys; the workgroup fetches every block
// of 32 keys once, through registers into LDS (two buffers: the next block travels while this one is used, one barrier
// a block), as keys [32][dk + 8] and values [dv][32], and each wavefront reads its operands from there just before the
// product that uses them, which leaves registers for four wavefronts a SIMD. Instances exist for values of up to 64 entries (wider ones
// measured slower than the kernel above). The workgroup walks
// the blocks that any of its tiles needs; a wavefront passes over a block behind its own last key, and tests visibility
// only in blocks that some row of its tile does not see whole. Values behind the workgroup's last key are zeroed as
// they are staged (their page may hold anything). Results are left as by the kernel above, block by block in the same
// order.
template <int NVM, bool EDGE, int CAP>
__device__ __forceinline__ void shared_block(const WindowArgs& a, const f32x4 (&sc)[2], const bf16* lds_v, f32x4 (&acc)[NVM], float& m,
                                             float& l, int nvt, int key0, int r, int qd, int pos, bool valid, float inv_cap, float slope) {
    float p[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float v0 = sc[j >> 2][j & 3];
        float v = CAP == kScoreCapped ? capped_score(v0, inv_cap, a.softcap) : v0 * a.scale;
        if (CAP == kScoreDistance) v = fmaf(slope, static_cast<float>(key0 + qd * 8 + j - pos), v);
        if (EDGE) {
            const int key = key0 + qd * 8 + j;
            const bool seen = valid && key <= pos && (a.window <= 0 || pos - key < a.window || key < a.keep_first);
            v = seen ? v : -INFINITY;
        }
        p[j] = v;
        mx = fmaxf(mx, v);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = (EDGE && m_new == -INFINITY) ? 0.f : m_new;
    const bool rescale = __any(m_new != m);
    const float alpha = rescale ? __expf(m - m_use) : 1.f;
    m = m_new;
    float sum = 0.f;
    bf16x8 ph, pl;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float w = __expf(p[j] - m_use);
        sum += w;
        const bf16 hi = static_cast<bf16>(w);
        ph[j] = hi;
        pl[j] = static_cast<bf16>(w - static_cast<float>(hi));
    }
    l = rescale ? l * alpha + sum : l + sum;
#pragma unroll
    for (int c = 0; c < NVM; ++c) {
        if (c < nvt) {
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(lds_v + (c * 16 + r) * 32 + qd * 8);
            if (rescale) {
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[c][e] *= alpha;
            }
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, ph, acc[c], 0, 0, 0);
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v, pl, acc[c], 0, 0, 0);
        }
    }
}

template <int DSM, int NVM, int CAP>
__global__ __launch_bounds__(256, 4) void window_attention_mfma_shared_kernel(WindowArgs a) {
    constexpr int DKP = DSM * 32 + 8;                       // a staged key's stride (entries): 16 bytes of padding
    constexpr int K_ELEMS = 32 * DKP, V_ELEMS = NVM * 16 * 32;
    constexpr int KL = DSM / 2, VL = NVM / 4;               // 16-byte pieces a thread stages of a block's keys and values
    __shared__ __align__(16) bf16 lds[2 * (K_ELEMS + V_ELEMS)];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, qd = lane >> 4;
    const int s = blockIdx.y / a.nk, kh = blockIdx.y % a.nk;
    const int vh = kh / a.maps, map = kh % a.maps;
    const int row0 = a.q_start[s];
    const int rows_total = (a.q_start[s + 1] - row0) * a.per_value_head;
    const int RW = blockIdx.x * 64;                         // the workgroup's first row
    if (RW >= rows_total) return;                           // (the whole workgroup)
    const int R0 = RW + wave * 16;
    const bool active = R0 < rows_total;
    const bool valid = R0 + r < rows_total;
    const bool all_valid = R0 + 15 < rows_total;
    const int R = valid ? R0 + r : rows_total - 1;
    const int t = row0 + R / a.per_value_head;
    const int qh = (vh * a.per_value_head + R % a.per_value_head) * a.maps + map;
    const int pos = a.positions[t];
    const int first_row = active ? R0 : rows_total - 1;
    const int pos_min = a.positions[row0 + first_row / a.per_value_head];
    const int last_row = all_valid ? R0 + 15 : rows_total - 1;
    const int pos_max = a.positions[row0 + last_row / a.per_value_head];
    // the workgroup's rows
    const int wg_pos_min = a.positions[row0 + RW / a.per_value_head];
    const int wg_last = RW + 63 < rows_total ? RW + 63 : rows_total - 1;
    const int wg_pos_max = a.positions[row0 + wg_last / a.per_value_head];
    const int* table = a.block_table + static_cast<size_t>(s) * a.max_blocks;
    const int ds = (a.dk + 31) >> 5, nvt = a.dv >> 4;
    const int psh = a.page_shift, pmask = a.page - 1;
    const float inv_cap = a.softcap > 0.f ? 2.0f * 1.4426950408889634f * a.scale / a.softcap : 0.f;     // (capped_score's k)
    const float slope = CAP == kScoreDistance ? a.slopes[qh / a.maps] : 0.f;

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

    // the workgroup's blocks of 32 keys: [0, nb_kept) and [first_blk, last_blk]
    const int lo_min = (a.window > 0 && wg_pos_min - a.window + 1 > 0) ? wg_pos_min - a.window + 1 : 0;
    int first_blk = lo_min >> 5;
    const int last_blk = wg_pos_max >> 5;
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

    // staging: piece i of a block's keys is entries 8 (i % cpk) .. of key i / cpk; piece i of its values the keys
    // 8 (i % 4) .. of value entry i / 4
    const int cpk = a.dk >> 3;
    bf16x8 k_st[KL], v_st[VL];
    auto fetch = [&](int b) {
        const int key0 = (b < nb_kept ? b : first_blk + b - nb_kept) << 5;
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int piece = tid + i * 256;
            if (piece < 32 * cpk) {
                int key = key0 + piece / cpk;
                key = key < wg_pos_max ? key : wg_pos_max;     // (keys behind the workgroup's last are masked by every row)
                int pg = table[key >> psh];
                pg = pg < 0 ? 0 : pg;       // (a page that the window has left behind and given back: its keys are masked)
                k_st[i] = *reinterpret_cast<const bf16x8*>(
                    a.k_cache + (((static_cast<size_t>(pg) * a.nk + kh) << psh) + (key & pmask)) * a.dk + (piece % cpk) * 8);
            }
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int piece = tid + i * 256;
            if (piece < a.dv * 4) {
                const int kq = key0 + (piece & 3) * 8;
                const int kc = kq <= wg_pos_max ? kq : (wg_pos_max & ~7);
                int pg = table[kc >> psh];
                pg = pg < 0 ? 0 : pg;
                bf16x8 v = *reinterpret_cast<const bf16x8*>(
                    a.v_cache + (((static_cast<size_t>(pg) * a.nv + vh) * a.dv + (piece >> 2)) << psh) + (kc & pmask));
                if (kq + 7 > wg_pos_max) {
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (kq + j > wg_pos_max) v[j] = static_cast<bf16>(0.f);
                }
                v_st[i] = v;
            }
        }
    };
    auto stage = [&](int buf) {
        bf16* lk = lds + buf * (K_ELEMS + V_ELEMS);
        bf16* lv = lk + K_ELEMS;
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const int piece = tid + i * 256;
            if (piece < 32 * cpk) *reinterpret_cast<bf16x8*>(lk + (piece / cpk) * DKP + (piece % cpk) * 8) = k_st[i];
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const int piece = tid + i * 256;
            if (piece < a.dv * 4) *reinterpret_cast<bf16x8*>(lv + (piece >> 2) * 32 + (piece & 3) * 8) = v_st[i];
        }
    };

    float m = -INFINITY, l = 0.f;
    f32x4 acc[NVM];
#pragma unroll
    for (int c = 0; c < NVM; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int k_in_block = 8 * (r >> 2) + (r & 3);          // (rows of a 16-key half, as in the kernel above)

    if (b_begin < b_end) {
        fetch(b_begin);
        stage(0);
    }
    __syncthreads();
    for (int b = b_begin; b < b_end; ++b) {
        const int buf = (b - b_begin) & 1;
        if (b + 1 < b_end) fetch(b + 1);
        const int key0 = (b < nb_kept ? b : first_blk + b - nb_kept) << 5;
        // (a block behind this tile's last key, or in front of the window's start of its first row and not among the
        // kept ones, has no key for it)
        const bool mine = active && key0 <= pos_max
                          && (a.window <= 0 || b < nb_kept || key0 + 31 >= pos_min - a.window + 1 || key0 < a.keep_first);
        if (mine) {
            const bf16* lk = lds + buf * (K_ELEMS + V_ELEMS);
            f32x4 sc[2];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                sc[sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < DSM; ++c) {
                    const int d0 = c * 32 + qd * 8;
                    if (c < ds) {
                        bf16x8 kf;
#pragma unroll
                        for (int e = 0; e < 8; ++e) kf[e] = static_cast<bf16>(0.f);
                        if (d0 < a.dk) kf = *reinterpret_cast<const bf16x8*>(lk + (k_in_block + 4 * sub) * DKP + d0);
                        sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], sc[sub], 0, 0, 0);
                    }
                }
            }
            const bool inner = all_valid && b >= nb_kept && key0 + 31 <= pos_min && (a.window <= 0 || pos_max - key0 < a.window);
            if (inner) shared_block<NVM, false, CAP>(a, sc, lk + K_ELEMS, acc, m, l, nvt, key0, r, qd, pos, valid, inv_cap, slope);
            else shared_block<NVM, true, CAP>(a, sc, lk + K_ELEMS, acc, m, l, nvt, key0, r, qd, pos, valid, inv_cap, slope);
        }
        if (b + 1 < b_end) stage(buf ^ 1);
        __syncthreads();
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!valid) return;
    window_store<NVM>(a, acc, m, l, nvt, t, qh, qd);
}

}  // namespace llme

using namespace llme;

// max_new: the most tokens a request brings to the step (sizes the grid). staged: 0 keeps every step on the kernel without LDS. Refuses (10002) what the kernel does not
// take: key entries no multiple of 8 or beyond 128, value entries no multiple of 16 or beyond 128, pages that are no
// power of two from 16 on.
extern "C" int llme_window_attention_mfma(const void* q, const void* k_cache, const void* v_cache, float* part_o, float* part_ml,
                                          const int* positions, const int* q_start, const int* block_table, int max_blocks, int T,
                                          int S, int max_new, int nq, int nk, int nv, int dk, int dv, int page, float scale,
                                          float softcap, int window, int keep_first, int nsplit, int staged, const float* slopes,
                                          void* out, int ld_out, const float* sinks, const float* head_gate, int ld_gate,
                                          float out_scale, hipStream_t stream) {
    if (T <= 0 || S <= 0) return 0;
    if (nv <= 0 || nk % nv != 0 || nq % nk != 0 || max_new <= 0 || nsplit <= 0 || window < 0 || keep_first < 0) return kErrBadArgument;
    if (dk % 8 != 0 || dk > 128 || dv % 16 != 0 || dv > 128 || page % 16 != 0 || (page & (page - 1)) != 0) return kErrUnsupported;
    if (softcap > 0.f && slopes != nullptr) return kErrUnsupported;         // (capped and biased scores: the plain kernel)
    // (finished rows: one run of keys, one map a head, rows of whole 8-byte pieces)
    if (out != nullptr && (nsplit != 1 || nk != nv || ld_out % 4 != 0 || reinterpret_cast<uintptr_t>(out) % 8 != 0)) return kErrBadArgument;
    WindowArgs a;
    a.slopes = slopes;
    a.out = static_cast<bf16*>(out);
    a.ld_out = ld_out;
    a.sinks = sinks;
    a.head_gate = head_gate;
    a.ld_gate = ld_gate;
    a.out_scale = out_scale;
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
    a.page_shift = __builtin_ctz(page);
    a.window = window;
    a.keep_first = keep_first;
    a.nsplit = nsplit;
    a.scale = scale;
    a.softcap = softcap;
    const int tiles = (max_new * a.per_value_head + 15) / 16;
    const dim3 grid((tiles + 3) / 4, S * nk, nsplit);
#define LLME_WMFMA(DSM, NVM)                                                                                     \
    do {                                                                                                         \
        if (softcap > 0.f) hipLaunchKernelGGL((window_attention_mfma_kernel<DSM, NVM, kScoreCapped>), grid, dim3(256), 0, stream, a); \
        else if (slopes != nullptr) hipLaunchKernelGGL((window_attention_mfma_kernel<DSM, NVM, kScoreDistance>), grid, dim3(256), 0, stream, a); \
        else hipLaunchKernelGGL((window_attention_mfma_kernel<DSM, NVM, kScorePlain>), grid, dim3(256), 0, stream, a);  \
    } while (0)
#define LLME_WSHARED(DSM, NVM)                                                                                          \
    do {                                                                                                                \
        if (softcap > 0.f) hipLaunchKernelGGL((window_attention_mfma_shared_kernel<DSM, NVM, kScoreCapped>), grid, dim3(256), 0, stream, a); \
        else if (slopes != nullptr) hipLaunchKernelGGL((window_attention_mfma_shared_kernel<DSM, NVM, kScoreDistance>), grid, dim3(256), 0, stream, a); \
        else hipLaunchKernelGGL((window_attention_mfma_shared_kernel<DSM, NVM, kScorePlain>), grid, dim3(256), 0, stream, a);  \
    } while (0)
    // a request that brings a workgroup's 64 rows or more, values of up to 64 entries: the blocks staged once a workgroup;
    // fewer rows (decoded tokens, short portions): a wavefront on its own
    // (with values beyond 64 entries the staged kernel measured slower: 170 against 156 us over a prompt of 2,048)
    const bool shared = staged != 0 && static_cast<long>(max_new) * a.per_value_head >= 64 && dv <= 64;
    if (shared) {
        if (dk <= 64) LLME_WSHARED(2, 4);
        else LLME_WSHARED(4, 4);
    } else if (dk <= 64 && dv <= 64) LLME_WMFMA(2, 4);
    else if (dk <= 64) LLME_WMFMA(2, 8);
    else if (dv <= 64) LLME_WMFMA(4, 4);
    else LLME_WMFMA(4, 8);
#undef LLME_WMFMA
#undef LLME_WSHARED
    return launch_status();
}

LLME_LOAD_ENTRY(window_attention_mfma)
