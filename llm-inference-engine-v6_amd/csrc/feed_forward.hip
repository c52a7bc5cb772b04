// Small kernels around feed-forward layers whose products carry more than a gate:
//
//   * gated_bias_act: out = act(gate + b_gate) * (up + b_up) from a product's 32-bit rows that hold gate and up columns in
//     alternating groups (biases in the same order, or none), with the activations
//       0 silu, 1 rectifier, 2 gelu (tanh form),
//       3 clamped swish: g = min(gate, limit), u = clamp(up, -limit, limit), out = g * sigmoid(alpha g) * (u + 1);
//     with `row_pair` and `pair_scale` the sums of row t are first multiplied by pair_scale[row_pair[t]] (0 where the row
//     holds no pair): an expert that runs on its weight times the input, the weight taken out of the two products;
//   * add_row_bias: every row of a 32-bit matrix gets the same row added (the bias of an output product that
//     accumulates into the residual stream);
//   * table_route: a token's experts read from a table by its id, each weighing 1 / top;
//   * concat_rows: [a | b] side by side in the activation type, the input of a product over both.
#include "common.h"
#include <math.h>

namespace llme {

template <typename TB, typename TO>
__global__ void gated_bias_act_kernel(const float* __restrict__ gu, int ld, const TB* __restrict__ bias, TO* __restrict__ out, int FF,
                                      int group, size_t total, int act, float limit, float alpha,
                                      const int* __restrict__ row_pair, const float* __restrict__ pair_scale) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / FF;
    const int j = static_cast<int>(idx % FF);
    const int col = (j / group) * 2 * group + (j % group);
    float g = gu[t * ld + col];
    float u = gu[t * ld + col + group];
    if (row_pair != nullptr) {
        const int pair = row_pair[t];
        const float sc = pair < 0 ? 0.f : pair_scale[pair];
        g *= sc;
        u *= sc;
    }
    if (bias != nullptr) {
        g += to_float(bias[col]);
        u += to_float(bias[col + group]);
    }
    float v;
    if (act == 1) {
        v = fmaxf(g, 0.f) * u;
    } else if (act == 2) {
        v = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
    } else if (act == 3) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        v = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    } else {
        v = g / (1.0f + expf(-g)) * u;
    }
    out[idx] = from_float<TO>(v);
}

template <typename TB>
__global__ void add_row_bias_kernel(float* __restrict__ x, const TB* __restrict__ bias, int H, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    x[idx] += to_float(bias[idx % H]);
}

__global__ void table_route_kernel(const int* __restrict__ table, const int* __restrict__ tokens, int* __restrict__ ids,
                                   float* __restrict__ wts, int top, int total, float weight) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    ids[idx] = table[static_cast<size_t>(tokens[idx / top]) * top + idx % top];
    wts[idx] = weight;
}

template <typename TO>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b, TO* __restrict__ out, int H, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / (2 * H);
    const int c = static_cast<int>(idx % (2 * H));
    out[idx] = from_float<TO>(c < H ? a[t * H + c] : b[t * H + c - H]);
}

}  // namespace llme

using namespace llme;

extern "C" int llme_gated_bias_act(const float* gu, int ld, const void* bias, int bias_dtype, void* out, int out_dtype, int T, int FF,
                                   int group, int act, float limit, float alpha, const int* row_pair, const float* pair_scale,
                                   hipStream_t stream) {
    if (T <= 0) return 0;
    if (group <= 0 || FF % group != 0 || act < 0 || act > 3 || ld < 2 * FF) return kErrBadArgument;
    if ((row_pair == nullptr) != (pair_scale == nullptr)) return kErrBadArgument;
    const size_t total = static_cast<size_t>(T) * FF;
    const dim3 grid(static_cast<unsigned>((total + 255) / 256));
#define LLME_GBA(TB, TO)                                                                                              \
    hipLaunchKernelGGL((gated_bias_act_kernel<TB, TO>), grid, dim3(256), 0, stream, gu, ld, static_cast<const TB*>(bias), \
                       static_cast<TO*>(out), FF, group, total, act, limit, alpha, row_pair, pair_scale)
    const bool bb = bias != nullptr && bias_dtype == kBF16;
    if (out_dtype == kF32 && !bb) LLME_GBA(float, float);
    else if (out_dtype == kF32 && bb) LLME_GBA(bf16, float);
    else if (out_dtype == kBF16 && !bb) LLME_GBA(float, bf16);
    else if (out_dtype == kBF16 && bb) LLME_GBA(bf16, bf16);
    else return kErrBadArgument;
#undef LLME_GBA
    return launch_status();
}

extern "C" int llme_add_row_bias(float* x, const void* bias, int bias_dtype, int T, int H, hipStream_t stream) {
    if (T <= 0) return 0;
    if (H <= 0) return kErrBadArgument;
    const size_t total = static_cast<size_t>(T) * H;
    const dim3 grid(static_cast<unsigned>((total + 255) / 256));
    if (bias_dtype == kF32)
        hipLaunchKernelGGL((add_row_bias_kernel<float>), grid, dim3(256), 0, stream, x, static_cast<const float*>(bias), H, total);
    else if (bias_dtype == kBF16)
        hipLaunchKernelGGL((add_row_bias_kernel<bf16>), grid, dim3(256), 0, stream, x, static_cast<const bf16*>(bias), H, total);
    else return kErrBadArgument;
    return launch_status();
}

extern "C" int llme_table_route(const int* table, const int* tokens, int* ids, float* wts, int T, int top, hipStream_t stream) {
    if (T <= 0) return 0;
    if (top <= 0) return kErrBadArgument;
    const int total = T * top;
    hipLaunchKernelGGL(table_route_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, table, tokens, ids, wts, top, total,
                       1.0f / static_cast<float>(top));
    return launch_status();
}

extern "C" int llme_concat_rows(const float* a, const float* b, void* out, int out_dtype, int T, int H, hipStream_t stream) {
    if (T <= 0) return 0;
    if (H <= 0) return kErrBadArgument;
    const size_t total = static_cast<size_t>(T) * 2 * H;
    const dim3 grid(static_cast<unsigned>((total + 255) / 256));
    if (out_dtype == kF32)
        hipLaunchKernelGGL((concat_rows_kernel<float>), grid, dim3(256), 0, stream, a, b, static_cast<float*>(out), H, total);
    else if (out_dtype == kBF16)
        hipLaunchKernelGGL((concat_rows_kernel<bf16>), grid, dim3(256), 0, stream, a, b, static_cast<bf16*>(out), H, total);
    else return kErrBadArgument;
    return launch_status();
}

LLME_LOAD_ENTRY(feed_forward)
