// Mixers that carry a state of fixed size from token to token: short causal convolutions, the gated
// diagonal recurrence (RG-LRU) and the gated delta rule. Everything that enters a recurrence, and the
// state itself, is 32-bit; only weights may be stored in bfloat16 (they are widened exactly).
//
// A step is a flat batch of rows; request s owns rows q_start[s] .. q_start[s + 1] - 1, which continue
// what its slot (slots[s]) of every state tensor holds. Inputs are column ranges of wider 32-bit
// buffers (a fused projection's output), so every matrix comes with its leading dimension.
#include "common.h"

namespace llme {

constexpr int kMaxTaps = 16;

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float gelu_tanhf_(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---------------------------------------------------------------------------------
// out[t, c] = act(bias[c] + sum_j w[c, j] * x[t - (K - 1 - j), c]) with x = in + in_bias (a bias of the product in
// front, null for none); rows before the request's first row of this step come from the slot's tail [K - 1, C]
// (oldest first; zero for a new request: what lies before a sequence's start counts as zero, bias and all).
__global__ __launch_bounds__(256) void short_conv_kernel(const float* __restrict__ in, int ld_in, const float* __restrict__ w,
                                                         const float* __restrict__ bias, const float* __restrict__ in_bias,
                                                         const float* __restrict__ tail, const int* __restrict__ seq_idx, const int* __restrict__ q_start,
                                                         const int* __restrict__ slots, float* __restrict__ out, int ld_out,
                                                         int C, int K, int act) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int s = seq_idx[t];
    const int first = q_start[s];
    const float* tl = tail + static_cast<size_t>(slots[s]) * (K - 1) * C;
    float acc = bias ? bias[c] : 0.f;
    const float ib = in_bias ? in_bias[c] : 0.f;
    for (int j = 0; j < K; ++j) {
        const int r = t - (K - 1 - j);
        const float x = r >= first ? in[static_cast<size_t>(r) * ld_in + c] + ib
                                   : tl[static_cast<size_t>(K - 1 + (r - first)) * C + c];
        acc += w[static_cast<size_t>(c) * K + j] * x;
    }
    out[static_cast<size_t>(t) * ld_out + c] = act == 1 ? siluf_(acc) : acc;
}

// A step in which every request brings one row (decoding): the convolution and the tail's move in one kernel. A thread
// reads its channel's tail, makes the row's output and stores the tail moved on by the row.
__global__ __launch_bounds__(256) void short_conv_single_kernel(const float* __restrict__ in, int ld_in, const float* __restrict__ w,
                                                                const float* __restrict__ bias, const float* __restrict__ in_bias,
                                                                float* __restrict__ tail, const int* __restrict__ seq_idx,
                                                                const int* __restrict__ slots, float* __restrict__ out, int ld_out,
                                                                int C, int K, int act) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    float* tl = tail + static_cast<size_t>(slots[seq_idx[t]]) * (K - 1) * C;
    const float x = in[static_cast<size_t>(t) * ld_in + c] + (in_bias ? in_bias[c] : 0.f);
    float keep[kMaxTaps];
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= K - 1) break;
        keep[i] = tl[static_cast<size_t>(i) * C + c];
    }
    float acc = bias ? bias[c] : 0.f;
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= K - 1) break;
        acc += w[static_cast<size_t>(c) * K + i] * keep[i];
    }
    acc += w[static_cast<size_t>(c) * K + K - 1] * x;
    out[static_cast<size_t>(t) * ld_out + c] = act == 1 ? siluf_(acc) : acc;
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= K - 1) break;
        tl[static_cast<size_t>(i) * C + c] = i + 1 < K - 1 ? keep[i + 1] : x;
    }
}

// The slot's tail after the step: the last K - 1 inputs of the request, from this step's rows and, where the
// step brought fewer, from the old tail.
__global__ __launch_bounds__(256) void conv_tail_kernel(const float* __restrict__ in, int ld_in,
                                                        const float* __restrict__ in_bias, float* __restrict__ tail,
                                                        const int* __restrict__ q_start, const int* __restrict__ slots,
                                                        int C, int K) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int first = q_start[s], n = q_start[s + 1] - first;
    float* tl = tail + static_cast<size_t>(slots[s]) * (K - 1) * C;
    float keep[kMaxTaps];
    const float ib = in_bias ? in_bias[c] : 0.f;
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= K - 1) break;
        const int rel = n - (K - 1) + i;            // row of the new tail's entry i, counted from the step's first
        keep[i] = rel >= 0 ? in[static_cast<size_t>(first + rel) * ld_in + c] + ib : tl[static_cast<size_t>(K - 1 + rel) * C + c];
    }
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i) {
        if (i >= K - 1) break;
        tl[static_cast<size_t>(i) * C + c] = keep[i];
    }
}

// ---------------------------------------------------------------------------------
// RG-LRU gates. u [T, width] in blocks of bw channels; per block b two maps [bw, bw] ([out, in]):
//   r = sigmoid(Ra_b u_b + ba), i = sigmoid(Ri_b u_b + bi), a = exp(-c r softplus(lam)),
//   decay[t, ch] = a,  drive[t, ch] = sqrt(1 - a^2) i u.
// A workgroup makes 16 rows x 64 channels of one block, stepping through the block's inputs in slabs of 32.
template <typename TW>
__global__ __launch_bounds__(256) void rglru_gates_kernel(const float* __restrict__ u, int ld_u, const TW* __restrict__ ra,
                                                          const float* __restrict__ rab, const TW* __restrict__ ri,
                                                          const float* __restrict__ rib, const float* __restrict__ lam,
                                                          float* __restrict__ decay, float* __restrict__ drive, int T,
                                                          int width, int bw, float c_rate) {
    constexpr int TM = 16, TN = 64, TK = 32;
    __shared__ float us[TM][TK + 1];
    __shared__ float was[TN][TK + 1];
    __shared__ float wis[TN][TK + 1];
    const int tiles_n = (bw + TN - 1) / TN;
    const int b = blockIdx.x / tiles_n;
    const int n0 = (blockIdx.x % tiles_n) * TN;
    const int t0 = blockIdx.y * TM;
    const int tid = threadIdx.x;
    const int tm = tid / 16;            // row of the tile
    const int tn = tid % 16;            // channels tn, tn + 16, tn + 32, tn + 48
    float accr[4] = {0.f, 0.f, 0.f, 0.f}, acci[4] = {0.f, 0.f, 0.f, 0.f};
    const TW* ra_b = ra + static_cast<size_t>(b) * bw * bw;
    const TW* ri_b = ri + static_cast<size_t>(b) * bw * bw;
    for (int k0 = 0; k0 < bw; k0 += TK) {
        for (int e = tid; e < TM * TK; e += 256) {
            const int r = e / TK, k = e % TK;
            us[r][k] = (t0 + r < T && k0 + k < bw) ? u[static_cast<size_t>(t0 + r) * ld_u + b * bw + k0 + k] : 0.f;
        }
        for (int e = tid; e < TN * TK; e += 256) {
            const int o = e / TK, k = e % TK;
            const bool ok = n0 + o < bw && k0 + k < bw;
            was[o][k] = ok ? to_float(ra_b[static_cast<size_t>(n0 + o) * bw + k0 + k]) : 0.f;
            wis[o][k] = ok ? to_float(ri_b[static_cast<size_t>(n0 + o) * bw + k0 + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < TK; ++k) {
            const float x = us[tm][k];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                accr[j] += was[tn + 16 * j][k] * x;
                acci[j] += wis[tn + 16 * j][k] * x;
            }
        }
        __syncthreads();
    }
    const int t = t0 + tm;
    if (t >= T) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int o = n0 + tn + 16 * j;
        if (o >= bw) continue;
        const int ch = b * bw + o;
        const float r = sigmoidf_(accr[j] + rab[ch]);
        const float g = sigmoidf_(acci[j] + rib[ch]);
        const float log_a = -c_rate * r * softplusf_(lam[ch]);
        const float a = expf(log_a);
        const float x = u[static_cast<size_t>(t) * ld_u + ch];
        decay[static_cast<size_t>(t) * width + ch] = a;
        drive[static_cast<size_t>(t) * width + ch] = sqrtf(-expm1f(2.0f * log_a)) * (g * x);
    }
}

// s_t = decay_t s_(t-1) + drive_t per request and channel, from the slot's state; out[t] = s_t * gelu_tanh(y[t] + yb)
// in the activation type. A thread walks one channel of one request through the step's rows.
template <typename TO>
__global__ __launch_bounds__(256) void rglru_scan_kernel(const float* __restrict__ decay, const float* __restrict__ drive,
                                                         const float* __restrict__ y, int ld_y, const float* __restrict__ yb,
                                                         float* __restrict__ state, const int* __restrict__ q_start,
                                                         const int* __restrict__ slots, TO* __restrict__ out, int ld_out,
                                                         int width) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= width) return;
    const int first = q_start[s], last = q_start[s + 1];
    float* st = state + static_cast<size_t>(slots[s]) * width + c;
    float h = *st;
    const float bias = yb ? yb[c] : 0.f;
    for (int t = first; t < last; ++t) {
        const size_t at = static_cast<size_t>(t) * width + c;
        h = decay[at] * h + drive[at];
        out[static_cast<size_t>(t) * ld_out + c] = from_float<TO>(h * gelu_tanhf_(y[static_cast<size_t>(t) * ld_y + c] + bias));
    }
    *st = h;
}

// The same recurrence for long runs of rows, in three passes over chunks of `chunk` rows of a request:
// (1) every chunk's product of decays P and its result from an empty state B; (2) per request and channel, the state in
// front of every chunk (carry_j+1 = P_j carry_j + B_j, from the slot's state, which becomes the last one); (3) every
// chunk again from its carry, with the outputs. part [n_seq, chunks, 2, width] holds (P, B), then (carry, -).
__global__ __launch_bounds__(256) void rglru_chunk_sums_kernel(const float* __restrict__ decay, const float* __restrict__ drive,
                                                               const int* __restrict__ q_start, float* __restrict__ part,
                                                               int width, int chunk, int chunks) {
    const int s = blockIdx.z, j = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    const int first = q_start[s] + j * chunk;
    const int last = min(q_start[s + 1], first + chunk);
    if (c >= width || first >= last) return;
    float p = 1.f, h = 0.f;
    for (int t = first; t < last; ++t) {
        const size_t at = static_cast<size_t>(t) * width + c;
        const float a = decay[at];
        p *= a;
        h = a * h + drive[at];
    }
    float* out = part + (static_cast<size_t>(s) * chunks + j) * 2 * width;
    out[c] = p;
    out[width + c] = h;
}

__global__ __launch_bounds__(256) void rglru_chunk_carry_kernel(float* __restrict__ part, float* __restrict__ state,
                                                                const int* __restrict__ q_start, const int* __restrict__ slots,
                                                                int width, int chunk, int chunks) {
    const int s = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= width) return;
    const int n = q_start[s + 1] - q_start[s];
    float* st = state + static_cast<size_t>(slots[s]) * width + c;
    float h = *st;
    for (int j = 0; j * chunk < n; ++j) {
        float* pb = part + (static_cast<size_t>(s) * chunks + j) * 2 * width;
        const float p = pb[c], b = pb[width + c];
        pb[c] = h;
        h = p * h + b;
    }
    *st = h;
}

template <typename TO>
__global__ __launch_bounds__(256) void rglru_chunk_scan_kernel(const float* __restrict__ decay, const float* __restrict__ drive,
                                                               const float* __restrict__ y, int ld_y, const float* __restrict__ yb,
                                                               const float* __restrict__ part, const int* __restrict__ q_start,
                                                               TO* __restrict__ out, int ld_out, int width, int chunk, int chunks) {
    const int s = blockIdx.z, j = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    const int first = q_start[s] + j * chunk;
    const int last = min(q_start[s + 1], first + chunk);
    if (c >= width || first >= last) return;
    float h = part[(static_cast<size_t>(s) * chunks + j) * 2 * width + c];
    const float bias = yb ? yb[c] : 0.f;
    for (int t = first; t < last; ++t) {
        const size_t at = static_cast<size_t>(t) * width + c;
        h = decay[at] * h + drive[at];
        out[static_cast<size_t>(t) * ld_out + c] = from_float<TO>(h * gelu_tanhf_(y[static_cast<size_t>(t) * ld_y + c] + bias));
    }
}

// dst [T, n] (contiguous) = src [T, n] with leading dimension ld: a few columns of a wide buffer made a matrix of their own.
template <typename TO>
__global__ __launch_bounds__(256) void copy_cols_kernel(const float* __restrict__ src, int ld, TO* __restrict__ dst, int n, size_t total) {
    const size_t e = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= total) return;
    dst[e] = from_float<TO>(src[(e / n) * ld + e % n]);
}

// ---------------------------------------------------------------------------------
// x <- x / sqrt(sum(x^2) + eps) * scale over every head of `dim` entries, in place; heads [0, n_a) scale by
// scale_a, heads [n_a, n_a + n_b) by scale_b (queries and keys lie side by side). One wavefront per (row, head).
__global__ __launch_bounds__(256) void unit_heads_kernel(float* __restrict__ x, int ld, int T, int n_a, int n_b, int dim,
                                                         float scale_a, float scale_b, float eps) {
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int item = blockIdx.x * 4 + wave;
    if (item >= T * (n_a + n_b)) return;
    const int t = item / (n_a + n_b), h = item % (n_a + n_b);
    float* p = x + static_cast<size_t>(t) * ld + static_cast<size_t>(h) * dim;
    float ss = 0.f;
    for (int i = lane; i < dim; i += kWave) ss += p[i] * p[i];
    ss = wave_sum(ss);
    const float f = (h < n_a ? scale_a : scale_b) / sqrtf(ss + eps);
    for (int i = lane; i < dim; i += kWave) p[i] *= f;
}

// beta[t, h] = sigmoid(b[t, h]);
// per channel: decay[t, h, d] = exp(-exp(A_log[h]) softplus(sum_r a2[h dim + d, r] a1[t, r] + dt_bias[h dim + d]))
//              (a2 null: a_in holds the sums already, [T, heads dim])
// per head:    decay[t, h]    = exp(-exp(A_log[h]) softplus(a[t, h] + dt_bias[h]))
template <typename TW>
__global__ __launch_bounds__(256) void delta_gates_kernel(const float* __restrict__ b_in, int ld_b, const float* __restrict__ a_in,
                                                          int ld_a, const TW* __restrict__ a2, int rank,
                                                          const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                          float* __restrict__ beta, float* __restrict__ decay, int T, int heads,
                                                          int dim, int per_channel) {
    const int t = blockIdx.y;
    const int n_dec = per_channel ? heads * dim : heads;
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e < heads) beta[static_cast<size_t>(t) * heads + e] = sigmoidf_(b_in[static_cast<size_t>(t) * ld_b + e]);
    if (e >= n_dec) return;
    const int h = per_channel ? e / dim : e;
    float z;
    if (per_channel && a2 != nullptr) {
        z = 0.f;
        const float* lo = a_in + static_cast<size_t>(t) * ld_a;
        const TW* row = a2 + static_cast<size_t>(e) * rank;
        for (int r = 0; r < rank; ++r) z += to_float(row[r]) * lo[r];
    } else {
        z = a_in[static_cast<size_t>(t) * ld_a + e];
    }
    z += dt_bias[e];
    decay[static_cast<size_t>(t) * n_dec + e] = expf(-expf(A_log[h]) * softplusf_(z));
}

// decay[t, e] = sigmoid(z[t, e] + bias[e])^(1 / tau) = exp(-softplus(-(z + bias)) / tau): a decay per channel from a
// logit, flattened by a temperature. z is a column range of a 32-bit buffer, or, where a2 [n, rank] is given, made here
// from the first stage of a two-stage map: z[t, e] = sum_r a2[e, r] low[t, r] (32-bit sums). bias (null: none) and a2
// in their stored type.
template <typename TW>
__global__ __launch_bounds__(256) void sigmoid_decay_kernel(const float* __restrict__ z, int ld, const TW* __restrict__ a2, int rank,
                                                            const TW* __restrict__ bias, float inv_tau, float* __restrict__ decay,
                                                            int n) {
    const int t = blockIdx.y;
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= n) return;
    const float* zr = z + static_cast<size_t>(t) * ld;
    float x;
    if (a2 != nullptr) {
        const TW* row = a2 + static_cast<size_t>(e) * rank;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        int r = 0;
        for (; r + 4 <= rank; r += 4) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = fmaf(to_float(row[r + i]), zr[r + i], acc[i]);
        }
        for (; r < rank; ++r) acc[0] = fmaf(to_float(row[r]), zr[r], acc[0]);
        x = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    } else {
        x = zr[e];
    }
    if (bias != nullptr) x += to_float(bias[e]);
    decay[static_cast<size_t>(t) * n + e] = expf(-softplusf_(-x) * inv_tau);
}

// The delta rule. State M per request and head (32-bit, in the request's slot), kept as [vdim][dim]: a column's key
// channels lie together. Per token:
//   M <- g * M (g per key channel or one per head);  w = beta (v - M^T k);  M <- M + k w^T;  o = M^T q.
// The columns of M do not depend on each other: LPC lanes (8, or 16 for keys of 64 and more) share a column (lane l holds
// the R key channels l R .. l R + R - 1), a workgroup of 256 threads owns 256 / LPC columns of one head of one request and
// walks the request's rows in order: the fewer channels a lane holds, the shorter a step, and a prompt's time is its steps'. The rows' k, q, decay, v and beta come through LDS in blocks of eight rows, the next block asked for from
// memory while the current one is worked through, so that a step waits for LDS only.
constexpr int kDeltaRows = 8, kDeltaFetch = 28;

// The sum over each group of 8 or 16 neighbouring lanes, in every lane of the group, by data-parallel-primitive moves
// inside the vector unit (a shuffle through LDS would put three trips to LDS into every step of the recurrence):
// neighbours in a quad, the quad's other pair, then the mirror image in the half row of 8.
template <int LANES>
__device__ __forceinline__ float sum_of_lanes(float v) {
    static_assert(LANES == 8 || LANES == 16, "groups of 8 or 16 lanes");
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));     // quad_perm [1, 0, 3, 2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));     // quad_perm [2, 3, 0, 1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));    // row_half_mirror
    if (LANES == 16)                                                                                                // and the row of 16's mirror image
        v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    return v;
}

// DELTA false is the plain linear rule (gated linear attention): nothing is read back before the write,
//   M <- g * M;  M <- M + k v^T;  o = M^T q,
// and beta is not looked at. Every read is multiplied by o_scale (a scale on the queries).
//
// The linear rule with a decay per channel is linear in M with a diagonal map, so long runs of rows can be cut into
// chunks of `chunk` rows that are walked side by side (grid z = request x chunk), in three launches:
//   phase 1: every chunk from an empty memory, no reads: what the chunk adds (B, into chunk_state) and the product
//            of its decays (P, into chunk_decay);
//   carry  : per request, chunk by chunk, M_start(c) = M; M <- P(c) M + B(c); chunk_state then holds M_start, the slot
//            the memory behind the last row;
//   phase 3: every chunk again from its M_start, with the reads.
// phase 0 is the walk over all rows of a request in one go.
template <int R, int LPC, bool PER_CHANNEL, bool DELTA>
__global__ __launch_bounds__(256) void delta_rule_kernel(const float* __restrict__ qkv, int ld, int q_col, int k_col, int v_col,
                                                         const float* __restrict__ beta, const float* __restrict__ decay,
                                                         float* __restrict__ state, const int* __restrict__ q_start,
 const int* __restrict__ slots, float* __restrict__ o, int heads,
                                                         int kv_heads, int dim, int vdim, float o_scale, int phase, int chunk,
                                                         int n_chunks, float* __restrict__ chunk_state,
                                                         float* __restrict__ chunk_decay) {
    constexpr int DP = LPC * R;                             // a row's k (q, decay) padded with zeros to this many
    constexpr int kDeltaCols = 256 / LPC;                   // columns of the state a workgroup owns
    constexpr int NV = PER_CHANNEL ? 3 : 2;
    constexpr int W = NV * DP + kDeltaCols + 4;             // floats of a row in LDS: k, q, (decay,) v, beta, the head's decay
    constexpr int BLOCK = kDeltaRows * W;
    constexpr int NF = (BLOCK + 255) / 256;
    static_assert(NF <= kDeltaFetch, "a block of rows is more than the threads fetch");
    __shared__ float lds[2 * BLOCK];
    const int s = phase == 0 ? blockIdx.z : blockIdx.z / n_chunks, h = blockIdx.y, col0 = blockIdx.x * kDeltaCols;
    const int tid = threadIdx.x;
    const int cl = tid / LPC, l = tid % LPC;
    const int col = col0 + cl;
    const bool live = col < vdim;
    const int kvh = h / (heads / kv_heads);
    int first = q_start[s], last = q_start[s + 1];
    if (phase != 0) {
        first += (blockIdx.z % n_chunks) * chunk;
        if (first >= last) return;                          // (the request has fewer chunks than the longest one)
        last = first + chunk < last ? first + chunk : last;
    }
    // where the memory comes from and where it goes: the request's slot, or this chunk's place in chunk_state
    float* M = phase == 0 ? state + ((static_cast<size_t>(slots[s]) * heads + h) * vdim + (live ? col : 0)) * dim
                          : chunk_state + ((static_cast<size_t>(blockIdx.z) * heads + h) * vdim + (live ? col : 0)) * dim;
    float m[R], pp[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int d = l * R + i;
        m[i] = (live && d < dim && phase != 1) ? M[d] : 0.f;
        pp[i] = 1.f;
    }
    const int n_dec = PER_CHANNEL ? heads * dim : heads;
    // Where each of a thread's NF values of a block of rows comes from is the same for every block: the address for the
    // first block and the distance to the next block's are worked out once (src null: padding, always zero).
    float pre[NF];
    const float* src[NF];
    int advance[NF], row_of[NF];
#pragma unroll
    for (int i = 0; i < NF; ++i) {
        const int e = tid + 256 * i;
        src[i] = nullptr;
        advance[i] = 0;
        row_of[i] = 0;
        if (e < BLOCK) {
            const int tt = e / W, x = e % W;
            const size_t t = static_cast<size_t>(first + tt);
            row_of[i] = tt;
            if (x < DP) {
                if (x < dim) { src[i] = qkv + t * ld + k_col + kvh * dim + x; advance[i] = kDeltaRows * ld; }
            } else if (x < 2 * DP) {
                if (x - DP < dim) { src[i] = qkv + t * ld + q_col + kvh * dim + x - DP; advance[i] = kDeltaRows * ld; }
            } else if (PER_CHANNEL && x < 3 * DP) {
                if (x - 2 * DP < dim) { src[i] = decay + t * n_dec + h * dim + x - 2 * DP; advance[i] = kDeltaRows * n_dec; }
            } else {
                const int y = x - NV * DP;
                if (y < kDeltaCols) {
                    if (col0 + y < vdim) { src[i] = qkv + t * ld + v_col + h * vdim + col0 + y; advance[i] = kDeltaRows * ld; }
                } else if (y == kDeltaCols && DELTA) {
                    src[i] = beta + t * heads + h;
                    advance[i] = kDeltaRows * heads;
                } else if (y == kDeltaCols + 1 && !PER_CHANNEL) {
                    src[i] = decay + t * heads + h;
                    advance[i] = kDeltaRows * heads;
                }
            }
        }
    }
    auto fetch = [&](int t0) {
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            pre[i] = (src[i] != nullptr && t0 + row_of[i] < last) ? *src[i] : 0.f;
            if (src[i] != nullptr) src[i] += advance[i];
        }
    };
    auto put = [&](int buf) {
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            const int e = tid + 256 * i;
            if (e < BLOCK) lds[buf * BLOCK + e] = pre[i];
        }
    };
    fetch(first);
    put(0);
    __syncthreads();
    int cur = 0;
    for (int t0 = first; t0 < last; t0 += kDeltaRows) {
        const bool more = t0 + kDeltaRows < last;
        if (more) fetch(t0 + kDeltaRows);
        const int nt = min(kDeltaRows, last - t0);
        auto one_row = [&](int tt) {
            const float* row = lds + cur * BLOCK + tt * W;
            const float vv = row[NV * DP + cl];
            const float bt = row[NV * DP + kDeltaCols];
            const float g_head = row[NV * DP + kDeltaCols + 1];
            float kk[R], qq[R], gg[R];
            // a lane's R channels of k, q and the decay lie together and aligned: whole vectors from LDS
            if constexpr (R % 4 == 0) {
#pragma unroll
                for (int i = 0; i < R; i += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(row + l * R + i);
                    const float4 q4v = *reinterpret_cast<const float4*>(row + DP + l * R + i);
                    kk[i] = k4.x; kk[i + 1] = k4.y; kk[i + 2] = k4.z; kk[i + 3] = k4.w;
                    qq[i] = q4v.x; qq[i + 1] = q4v.y; qq[i + 2] = q4v.z; qq[i + 3] = q4v.w;
                    if (PER_CHANNEL) {
                        const float4 g4 = *reinterpret_cast<const float4*>(row + 2 * DP + l * R + i);
                        gg[i] = g4.x; gg[i + 1] = g4.y; gg[i + 2] = g4.z; gg[i + 3] = g4.w;
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < R; i += 2) {
                    const float2 k2 = *reinterpret_cast<const float2*>(row + l * R + i);
                    const float2 q2 = *reinterpret_cast<const float2*>(row + DP + l * R + i);
                    kk[i] = k2.x; kk[i + 1] = k2.y;
                    qq[i] = q2.x; qq[i + 1] = q2.y;
                    if (PER_CHANNEL) {
                        const float2 g2 = *reinterpret_cast<const float2*>(row + 2 * DP + l * R + i);
                        gg[i] = g2.x; gg[i + 1] = g2.y;
                    }
                }
            }
            float dots[2] = {0.f, 0.f};
#pragma unroll
            for (int i = 0; i < R; ++i) {
                m[i] *= PER_CHANNEL ? gg[i] : g_head;
                if (PER_CHANNEL && !DELTA) pp[i] *= gg[i];
                dots[i % 2] += m[i] * kk[i];
            }
            const float w = DELTA ? bt * (vv - sum_of_lanes<LPC>(dots[0] + dots[1])) : vv;
            float reads[2] = {0.f, 0.f};
#pragma unroll
            for (int i = 0; i < R; ++i) {
                m[i] += kk[i] * w;
                reads[i % 2] += m[i] * qq[i];
            }
            const float read = sum_of_lanes<LPC>(reads[0] + reads[1]);
            if (live && l == 0 && phase != 1) o[static_cast<size_t>(t0 + tt) * heads * vdim + h * vdim + col] = read * o_scale;
        };
        if (nt == kDeltaRows) {             // a whole block: no test between its rows, so that the rows' loads from LDS run ahead
#pragma unroll
            for (int tt = 0; tt < kDeltaRows; ++tt) one_row(tt);
        } else {
            for (int tt = 0; tt < nt; ++tt) one_row(tt);
        }
        if (more) {
            put(cur ^ 1);
            __syncthreads();
            cur ^= 1;
        }
    }
    if (phase == 3) return;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int d = l * R + i;
        if (live && d < dim) M[d] = m[i];
        if (PER_CHANNEL && !DELTA && phase == 1 && col == 0 && d < dim)
            chunk_decay[(static_cast<size_t>(blockIdx.z) * heads + h) * dim + d] = pp[i];
    }
}

// The carry between the chunks of the linear rule: one thread per (request, head, column, key channel).
__global__ __launch_bounds__(256) void linear_rule_carry_kernel(float* __restrict__ state, const int* __restrict__ q_start,
                                                                const int* __restrict__ slots, float* __restrict__ chunk_state,
                                                                const float* __restrict__ chunk_decay, int heads, int dim, int vdim,
                                                                int chunk, int n_chunks) {
    const int s = blockIdx.y;
    const size_t per = static_cast<size_t>(heads) * vdim * dim;
    const size_t e = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= per) return;
    const int d = static_cast<int>(e % dim);
    const int h = static_cast<int>(e / (static_cast<size_t>(vdim) * dim));
    const int rows = q_start[s + 1] - q_start[s];
    const int nc = (rows + chunk - 1) / chunk;
    float* slot = state + static_cast<size_t>(slots[s]) * per + e;
    float m = *slot;
    for (int c = 0; c < nc; ++c) {
        const size_t z = static_cast<size_t>(s) * n_chunks + c;
        float* at = chunk_state + z * per + e;
        const float add = *at;
        *at = m;
        m = fmaf(chunk_decay[(z * heads + h) * dim + d], m, add);
    }
    if (nc > 0) *slot = m;
}

// out[t, h, j] = scale * o[t, h, j] / sqrt(mean_j o^2 + eps) * w[j] * gate, in the activation type.
//   gate 0: sigmoid(sum_r g2[h vdim + j, r] g1[t, r]);  gate 1: silu(g[t, h vdim + j]);  gate 2: sigmoid(g[t, h vdim + j])
// One wavefront per (row, head).
template <typename TW, typename TO>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                              const float* __restrict__ g_in, int ld_g, const TW* __restrict__ g2,
                                                              int rank, int gate, TO* __restrict__ out, int ld_out, int T, int heads,
                                                              int vdim, float eps, float scale) {
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int item = blockIdx.x * 4 + wave;
    if (item >= T * heads) return;
    const int t = item / heads, h = item % heads;
    const float* p = o + (static_cast<size_t>(t) * heads + h) * vdim;
    float ss = 0.f;
    for (int j = lane; j < vdim; j += kWave) ss += p[j] * p[j];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(vdim) + eps);
    const float* gi = g_in + static_cast<size_t>(t) * ld_g;
    for (int j = lane; j < vdim; j += kWave) {
        float z;
        if (gate == 2) {
            z = sigmoidf_(gi[h * vdim + j]);
        } else if (gate == 0) {
            z = 0.f;
            const TW* row = g2 + static_cast<size_t>(h * vdim + j) * rank;
            for (int r = 0; r < rank; ++r) z += to_float(row[r]) * gi[r];
            z = sigmoidf_(z);
        } else {
            z = siluf_(gi[h * vdim + j]);
        }
        out[static_cast<size_t>(t) * ld_out + h * vdim + j] = from_float<TO>(scale * ((p[j] * inv) * w[j] * z));
    }
}

}  // namespace llme

using namespace llme;

#define LLME_BY_W(dt, CALL)                                  \
    if ((dt) == kF32) { using TW = float; CALL; }            \
    else if ((dt) == kBF16) { using TW = bf16; CALL; }       \
    else return kErrBadArgument;

// in [T, ld_in] 32-bit; w [C, K], bias [C] or null (w_dtype); tail [slots, K - 1, C] 32-bit; out [T, ld_out] 32-bit.
// update_tail: after the convolution the slots' tails are moved on by the step's rows.
extern "C" int llme_short_conv(const void* in, int ld_in, const void* w, const void* bias, const void* in_bias, void* tail,
                               const void* seq_idx, const void* q_start, const void* slots, void* out, int ld_out, int T,
                               int n_seq, int C, int K, int act, int update_tail, hipStream_t stream) {
    if (T <= 0 || C <= 0) return 0;
    if (K < 1 || K > kMaxTaps) return kErrUnsupported;
    const dim3 grid((C + 255) / 256, T);
    if (update_tail && T == n_seq) {            // one row per request
        short_conv_single_kernel<<<grid, 256, 0, stream>>>(
            static_cast<const float*>(in), ld_in, static_cast<const float*>(w), static_cast<const float*>(bias),
            static_cast<const float*>(in_bias), static_cast<float*>(tail), static_cast<const int*>(seq_idx),
            static_cast<const int*>(slots), static_cast<float*>(out), ld_out, C, K, act);
        return launch_status();
    }
    short_conv_kernel<<<grid, 256, 0, stream>>>(
        static_cast<const float*>(in), ld_in, static_cast<const float*>(w), static_cast<const float*>(bias),
        static_cast<const float*>(in_bias), static_cast<const float*>(tail), static_cast<const int*>(seq_idx),
        static_cast<const int*>(q_start), static_cast<const int*>(slots), static_cast<float*>(out), ld_out, C, K, act);
    if (update_tail && K > 1)
        conv_tail_kernel<<<dim3((C + 255) / 256, n_seq), 256, 0, stream>>>(
            static_cast<const float*>(in), ld_in, static_cast<const float*>(in_bias), static_cast<float*>(tail),
            static_cast<const int*>(q_start),
            static_cast<const int*>(slots), C, K);
    return launch_status();
}

extern "C" int llme_rglru_gates(const void* u, int ld_u, const void* ra, const void* rab, const void* ri, const void* rib,
                                const void* lam, int w_dtype, void* decay, void* drive, int T, int width, int blocks,
                                float c_rate, hipStream_t stream) {
    if (T <= 0 || width <= 0) return 0;
    if (blocks <= 0 || width % blocks) return kErrBadArgument;
    const int bw = width / blocks;
    const dim3 grid(blocks * ((bw + 63) / 64), (T + 15) / 16);
    LLME_BY_W(w_dtype, (rglru_gates_kernel<TW><<<grid, 256, 0, stream>>>(
        static_cast<const float*>(u), ld_u, static_cast<const TW*>(ra), static_cast<const float*>(rab),
        static_cast<const TW*>(ri), static_cast<const float*>(rib), static_cast<const float*>(lam), static_cast<float*>(decay),
        static_cast<float*>(drive), T, width, bw, c_rate)));
    return launch_status();
}

extern "C" int llme_rglru_scan(const void* decay, const void* drive, const void* y, int ld_y, const void* yb,
                               void* state, const void* q_start, const void* slots, void* out, int out_dtype, int ld_out,
                               int n_seq, int width, hipStream_t stream) {
    if (n_seq <= 0 || width <= 0) return 0;
    const dim3 grid((width + 255) / 256, n_seq);
#define LLME_SCAN(TO_)                                                                                                   \
    rglru_scan_kernel<TO_><<<grid, 256, 0, stream>>>(                                                                    \
        static_cast<const float*>(decay), static_cast<const float*>(drive), static_cast<const float*>(y), ld_y,          \
        static_cast<const float*>(yb), static_cast<float*>(state), static_cast<const int*>(q_start),                     \
        static_cast<const int*>(slots), static_cast<TO_*>(out), ld_out, width)
    switch (out_dtype) {
        case kF32: LLME_SCAN(float); break;
        case kBF16: LLME_SCAN(bf16); break;
        default: return kErrBadArgument;
    }
#undef LLME_SCAN
    return launch_status();
}

// The chunked form: part is scratch of n_seq * chunks * 2 * width floats, chunks >= ceil(longest request's rows / chunk).
extern "C" int llme_rglru_scan_chunked(const void* decay, const void* drive, const void* y, int ld_y, const void* yb,
                                       void* state, const void* q_start, const void* slots, void* out, int out_dtype,
                                       int ld_out, int n_seq, int width, int chunk, int chunks, void* part,
                                       hipStream_t stream) {
    if (n_seq <= 0 || width <= 0) return 0;
    if (chunk <= 0 || chunks <= 0) return kErrBadArgument;
    const dim3 grid((width + 255) / 256, chunks, n_seq);
    const float* dp = static_cast<const float*>(decay);
    const float* vp = static_cast<const float*>(drive);
    const int* qs = static_cast<const int*>(q_start);
    float* pp = static_cast<float*>(part);
    rglru_chunk_sums_kernel<<<grid, 256, 0, stream>>>(dp, vp, qs, pp, width, chunk, chunks);
    rglru_chunk_carry_kernel<<<dim3((width + 255) / 256, n_seq), 256, 0, stream>>>(pp, static_cast<float*>(state), qs,
                                                                                   static_cast<const int*>(slots), width, chunk,
                                                                                   chunks);
    if (out_dtype == kF32)
        rglru_chunk_scan_kernel<float><<<grid, 256, 0, stream>>>(dp, vp, static_cast<const float*>(y), ld_y,
                                                                 static_cast<const float*>(yb), pp, qs,
                                                                 static_cast<float*>(out), ld_out, width, chunk, chunks);
    else if (out_dtype == kBF16)
        rglru_chunk_scan_kernel<bf16><<<grid, 256, 0, stream>>>(dp, vp, static_cast<const float*>(y), ld_y,
                                                                static_cast<const float*>(yb), pp, qs, static_cast<bf16*>(out),
                                                                ld_out, width, chunk, chunks);
    else
        return kErrBadArgument;
    return launch_status();
}

extern "C" int llme_copy_cols(const void* src, int ld, void* dst, int dst_dtype, int T, int n, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * n;
    if (total == 0) return 0;
    const int grid = static_cast<int>((total + 255) / 256);
    if (dst_dtype == kF32)
        copy_cols_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(src), ld, static_cast<float*>(dst), n, total);
    else if (dst_dtype == kBF16)
        copy_cols_kernel<bf16><<<grid, 256, 0, stream>>>(static_cast<const float*>(src), ld, static_cast<bf16*>(dst), n, total);
    else
        return kErrBadArgument;
    return launch_status();
}

extern "C" int llme_unit_heads(void* x, int ld, int T, int n_a, int n_b, int dim, float scale_a, float scale_b, float eps,
                               hipStream_t stream) {
    const long items = static_cast<long>(T) * (n_a + n_b);
    if (items <= 0 || dim <= 0) return 0;
    unit_heads_kernel<<<static_cast<int>((items + 3) / 4), 256, 0, stream>>>(static_cast<float*>(x), ld, T, n_a, n_b, dim,
                                                                            scale_a, scale_b, eps);
    return launch_status();
}

extern "C" int llme_delta_gates(const void* b_in, int ld_b, const void* a_in, int ld_a, const void* a2, int rank,
                                const void* A_log, const void* dt_bias, int w_dtype, void* beta, void* decay, int T, int heads,
                                int dim, int per_channel, hipStream_t stream) {
    if (T <= 0 || heads <= 0) return 0;
    const int n = per_channel ? heads * dim : heads;
    const dim3 grid(((n > heads ? n : heads) + 255) / 256, T);
    LLME_BY_W(w_dtype, (delta_gates_kernel<TW><<<grid, 256, 0, stream>>>(
        static_cast<const float*>(b_in), ld_b, static_cast<const float*>(a_in), ld_a, static_cast<const TW*>(a2), rank,
        static_cast<const float*>(A_log), static_cast<const float*>(dt_bias), static_cast<float*>(beta),
        static_cast<float*>(decay), T, heads, dim, per_channel)));
    return launch_status();
}

extern "C" int llme_sigmoid_decay(const void* z, int ld, const void* a2, int rank, const void* bias, int w_dtype, float tau,
                                  void* decay, int T, int n, hipStream_t stream) {
    if (T <= 0 || n <= 0) return 0;
    if (!(tau > 0.f) || ld < (a2 != nullptr ? rank : n) || (a2 != nullptr && rank <= 0)) return kErrBadArgument;
    const dim3 grid((n + 255) / 256, T);
    LLME_BY_W(w_dtype, (sigmoid_decay_kernel<TW><<<grid, 256, 0, stream>>>(static_cast<const float*>(z), ld, static_cast<const TW*>(a2),
                                                                       rank, static_cast<const TW*>(bias), 1.0f / tau,
                                                                       static_cast<float*>(decay), n)));
    return launch_status();
}

template <int R, int LPC>
static void launch_delta_rule(bool per_channel, int n_seq, hipStream_t stream, const float* qkv, int ld, int q_col, int k_col,
                              int v_col, const float* beta, const float* decay, float* state, const int* q_start,
                              const int* slots, float* o, int heads, int kv_heads, int dim, int vdim, float o_scale, int chunk,
                              int n_chunks, float* chunk_state, float* chunk_decay) {
    const dim3 grid((vdim + 256 / LPC - 1) / (256 / LPC), heads, n_seq);
#define LLME_DR(PC, DL)                                                                                                          \
    delta_rule_kernel<R, LPC, PC, DL><<<grid, 256, 0, stream>>>(qkv, ld, q_col, k_col, v_col, beta, decay, state, q_start, slots, o, \
                                                                 heads, kv_heads, dim, vdim, o_scale, 0, 0, 1, nullptr, nullptr)
    if (chunk > 0) {
        // (the linear rule with a decay per channel, in chunks walked side by side)
        const dim3 cgrid(grid.x, heads, n_seq * n_chunks);
        const size_t per = static_cast<size_t>(heads) * vdim * dim;
        delta_rule_kernel<R, LPC, true, false><<<cgrid, 256, 0, stream>>>(qkv, ld, q_col, k_col, v_col, beta, decay, state, q_start, slots,
                                                                         o, heads, kv_heads, dim, vdim, o_scale, 1, chunk, n_chunks,
                                                                         chunk_state, chunk_decay);
        linear_rule_carry_kernel<<<dim3(static_cast<unsigned>((per + 255) / 256), n_seq), 256, 0, stream>>>(
            state, q_start, slots, chunk_state, chunk_decay, heads, dim, vdim, chunk, n_chunks);
        delta_rule_kernel<R, LPC, true, false><<<cgrid, 256, 0, stream>>>(qkv, ld, q_col, k_col, v_col, beta, decay, state, q_start, slots,
                                                                         o, heads, kv_heads, dim, vdim, o_scale, 3, chunk, n_chunks,
                                                                         chunk_state, chunk_decay);
        return;
    }
    if (beta != nullptr) {
        if (per_channel) LLME_DR(true, true);
        else LLME_DR(false, true);
    } else {
        if (per_channel) LLME_DR(true, false);
        else LLME_DR(false, false);
    }
#undef LLME_DR
}

// qkv [T, ld] 32-bit with unit q at q_col, unit k at k_col (kv_heads x dim each) and v at v_col (heads x vdim);
// beta [T, heads], or null for the linear rule; decay [T, heads, dim] or [T, heads]; state [slots, heads, vdim, dim];
// o [T, heads, vdim] 32-bit, times o_scale. chunk > 0 (the linear rule with a decay per channel only): every request's
// rows in chunks of that many, walked side by side; n_chunks = the most chunks a request has; chunk_state
// [n_seq * n_chunks, heads, vdim, dim] and chunk_decay [n_seq * n_chunks, heads, dim] are scratch.
extern "C" int llme_delta_rule(const void* qkv, int ld, int q_col, int k_col, int v_col, const void* beta, const void* decay,
                               int per_channel, void* state, const void* q_start, const void* slots, void* o, int n_seq,
                               int heads, int kv_heads, int dim, int vdim, float o_scale, int chunk, int n_chunks,
                               void* chunk_state, void* chunk_decay, hipStream_t stream) {
    if (n_seq <= 0 || heads <= 0) return 0;
    if (kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0) return kErrBadArgument;
    if (dim > 256) return kErrUnsupported;
    if (chunk < 0 || (chunk > 0 && (beta != nullptr || !per_channel || n_chunks <= 0 || chunk_state == nullptr ||
                                    chunk_decay == nullptr || static_cast<long>(n_seq) * n_chunks > 65535)))
        return kErrBadArgument;
#define LLME_DELTA(R_, L_)                                                                                               \
    launch_delta_rule<R_, L_>(per_channel != 0, n_seq, stream, static_cast<const float*>(qkv), ld, q_col, k_col, v_col, \
                          static_cast<const float*>(beta), static_cast<const float*>(decay), static_cast<float*>(state), \
                          static_cast<const int*>(q_start), static_cast<const int*>(slots), static_cast<float*>(o), heads, \
                          kv_heads, dim, vdim, o_scale, chunk, n_chunks, static_cast<float*>(chunk_state),                 \
                          static_cast<float*>(chunk_decay))
    if (dim <= 16) LLME_DELTA(2, 8);
    else if (dim <= 32) LLME_DELTA(4, 8);
    else if (dim <= 64) LLME_DELTA(4, 16);
    else if (dim <= 128) LLME_DELTA(8, 16);
    else LLME_DELTA(16, 16);
#undef LLME_DELTA
    return launch_status();
}

extern "C" int llme_gated_head_norm(const void* o, const void* w, const void* g_in, int ld_g, const void* g2, int rank, int gate,
                                    int w_dtype, void* out, int out_dtype, int ld_out, int T, int heads, int vdim, float eps,
                                    float scale, hipStream_t stream) {
    const long items = static_cast<long>(T) * heads;
    if (items <= 0 || vdim <= 0) return 0;
    const int grid = static_cast<int>((items + 3) / 4);
#define LLME_GHN(TW_, TO_)                                                                                               \
    gated_head_norm_kernel<TW_, TO_><<<grid, 256, 0, stream>>>(                                                          \
        static_cast<const float*>(o), static_cast<const float*>(w), static_cast<const float*>(g_in), ld_g,               \
        static_cast<const TW_*>(g2), rank, gate, static_cast<TO_*>(out), ld_out, T, heads, vdim, eps, scale)
    switch (w_dtype * 2 + out_dtype) {
        case 0: LLME_GHN(float, float); break;
        case 1: LLME_GHN(float, bf16); break;
        case 2: LLME_GHN(bf16, float); break;
        case 3: LLME_GHN(bf16, bf16); break;
        default: return kErrBadArgument;
    }
#undef LLME_GHN
    return launch_status();
}

LLME_LOAD_ENTRY(recurrent)
