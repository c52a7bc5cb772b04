// A sublayer's result normed before it joins the residual stream ("sandwich" layers):
//   h[t] += w_post * y[t] / sqrt(mean(y[t]^2) + eps)
// and, in the same pass over the row, the norm in front of the next sublayer:
//   x[t] = w_next * h[t] / sqrt(mean(h[t]^2) + eps)      (h as just updated)
// or, where x is asked for without a weight, the updated row as it is in the activation type (x[t] = h[t]: layers
// whose sublayers read the stream itself and are normed behind).
// y and h are 32-bit; the weights multiply as given (a norm whose checkpoint stores the distance from one
// hands over 1 + w). The products are evaluated (w * v) * inv, as the norm kernel evaluates them, so that a
// row is rounded to the same values whichever kernel norms it. One workgroup a row; the row waits in LDS
// between the two passes. Also here: a stream scaled by a constant (an embedding's multiplier).
#include "common.h"

namespace llme {

template <typename TW, typename TN, typename TO>
__global__ __launch_bounds__(256) void norm_add_kernel(const float* __restrict__ y, const TW* __restrict__ w_post,
                                                       float* __restrict__ h, const TN* __restrict__ w_next,
                                                       TO* __restrict__ x_out, int H, float eps) {
    extern __shared__ float row[];
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const float* yr = y + static_cast<size_t>(t) * H;
    float* hr = h + static_cast<size_t>(t) * H;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = yr[i];
        row[i] = v;
        ss = fmaf(v, v, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch, 4) / static_cast<float>(H) + eps);
    float ss2 = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = hr[i] + (to_float(w_post[i]) * row[i]) * inv;
        hr[i] = v;
        row[i] = v;
        ss2 = fmaf(v, v, ss2);
    }
    if (x_out == nullptr) return;
    TO* xr = x_out + static_cast<size_t>(t) * H;
    if (w_next == nullptr) {
        for (int i = threadIdx.x; i < H; i += 256) xr[i] = from_float<TO>(row[i]);
        return;
    }
    const float inv2 = 1.0f / sqrtf(block_sum(ss2, scratch, 4) / static_cast<float>(H) + eps);
    for (int i = threadIdx.x; i < H; i += 256) xr[i] = from_float<TO>((to_float(w_next[i]) * row[i]) * inv2);
}

// The same for rows of up to 8,192 values that are a multiple of 4: a thread keeps its values in registers (NV groups of
// four), and everything a row needs from memory (y, h, both weights) is asked for before anything waits.
template <typename T> __device__ __forceinline__ void na_load4(const T* p, float (&v)[4]);
template <> __device__ __forceinline__ void na_load4<float>(const float* p, float (&v)[4]) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
template <> __device__ __forceinline__ void na_load4<bf16>(const bf16* p, float (&v)[4]) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    const bf16x4 x = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(x[i]);
}
template <typename T> __device__ __forceinline__ void na_store4(T* p, const float (&v)[4]);
template <> __device__ __forceinline__ void na_store4<float>(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
}
template <> __device__ __forceinline__ void na_store4<bf16>(bf16* p, const float (&v)[4]) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    bf16x4 x;
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = static_cast<__bf16>(v[i]);
    *reinterpret_cast<bf16x4*>(p) = x;
}

template <typename TW, typename TN, typename TO, int NV>
__global__ __launch_bounds__(256) void norm_add_vec_kernel(const float* __restrict__ y, const TW* __restrict__ w_post,
                                                           float* __restrict__ h, const TN* __restrict__ w_next,
                                                           TO* __restrict__ x_out, int H, float eps) {
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const float* yr = y + static_cast<size_t>(t) * H;
    float* hr = h + static_cast<size_t>(t) * H;
    float yv[NV][4], hv[NV][4], wv[NV][4], nv[NV][4];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int i = (threadIdx.x + 256 * k) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[k][e] = hv[k][e] = wv[k][e] = nv[k][e] = 0.f;
        if (i < H) {
            na_load4(yr + i, yv[k]);
            na_load4(hr + i, hv[k]);
            na_load4(w_post + i, wv[k]);
            if (w_next != nullptr) na_load4(w_next + i, nv[k]);
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
        for (int e = 0; e < 4; ++e) ss = fmaf(yv[k][e], yv[k][e], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch, 4) / static_cast<float>(H) + eps);
    float ss2 = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int i = (threadIdx.x + 256 * k) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            hv[k][e] += (wv[k][e] * yv[k][e]) * inv;
            ss2 = fmaf(hv[k][e], hv[k][e], ss2);
        }
        if (i < H) na_store4(hr + i, hv[k]);
    }
    if (x_out == nullptr) return;
    TO* xr = x_out + static_cast<size_t>(t) * H;
    if (w_next == nullptr) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int i = (threadIdx.x + 256 * k) * 4;
            if (i < H) na_store4(xr + i, hv[k]);
        }
        return;
    }
    const float inv2 = 1.0f / sqrtf(block_sum(ss2, scratch, 4) / static_cast<float>(H) + eps);
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const int i = (threadIdx.x + 256 * k) * 4;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (nv[k][e] * hv[k][e]) * inv2;
        if (i < H) na_store4(xr + i, o);
    }
}

__global__ void scale_kernel(float* __restrict__ x, size_t n, float s) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) x[i] *= s;
}

}  // namespace llme

using namespace llme;

extern "C" int llme_norm_add(const float* y, const void* w_post, int w_dtype, float* h, const void* w_next,
                             int wn_dtype, void* x_out, int xo_dtype, int T, int H, float eps, hipStream_t stream) {
    if (T <= 0) return 0;
    if (H <= 0 || H > 16000) return kErrUnsupported;
    const size_t lds = static_cast<size_t>(H) * sizeof(float);
    const bool vec = H % 4 == 0 && H <= 8192 && reinterpret_cast<uintptr_t>(y) % 16 == 0 && reinterpret_cast<uintptr_t>(h) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(w_post) % 16 == 0 && reinterpret_cast<uintptr_t>(w_next) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(x_out) % 16 == 0;
    const int nv = !vec ? 0 : H <= 2048 ? 2 : H <= 4096 ? 4 : 8;
#define LLME_NAV(TW, TN, TO, NV)                                                                          \
    hipLaunchKernelGGL((norm_add_vec_kernel<TW, TN, TO, NV>), dim3(T), dim3(256), 0, stream, y,           \
                       static_cast<const TW*>(w_post), h, static_cast<const TN*>(w_next), static_cast<TO*>(x_out), H, eps)
#define LLME_NA(TW, TN, TO)                                                                               \
    do {                                                                                                  \
        if (nv == 2) LLME_NAV(TW, TN, TO, 2);                                                             \
        else if (nv == 4) LLME_NAV(TW, TN, TO, 4);                                                        \
        else if (nv == 8) LLME_NAV(TW, TN, TO, 8);                                                        \
        else                                                                                              \
            hipLaunchKernelGGL((norm_add_kernel<TW, TN, TO>), dim3(T), dim3(256), lds, stream, y,         \
                               static_cast<const TW*>(w_post), h, static_cast<const TN*>(w_next),         \
                               static_cast<TO*>(x_out), H, eps);                                          \
    } while (0)
    if (w_next == nullptr) {
        // nothing more, or the updated rows as they are in x_out's type
        const bool xb = x_out != nullptr && xo_dtype == kBF16;
        if (x_out != nullptr && xo_dtype != kBF16 && xo_dtype != kF32) return kErrBadArgument;
        if (w_dtype == kF32 && !xb) LLME_NA(float, float, float);
        else if (w_dtype == kF32 && xb) LLME_NA(float, float, bf16);
        else if (w_dtype == kBF16 && !xb) LLME_NA(bf16, float, float);
        else if (w_dtype == kBF16 && xb) LLME_NA(bf16, float, bf16);
        else return kErrBadArgument;
        return launch_status();
    }
    if (w_dtype != wn_dtype) return kErrBadArgument;
    if (w_dtype == kF32 && xo_dtype == kF32) LLME_NA(float, float, float);
    else if (w_dtype == kF32 && xo_dtype == kBF16) LLME_NA(float, float, bf16);
    else if (w_dtype == kBF16 && xo_dtype == kF32) LLME_NA(bf16, bf16, float);
    else if (w_dtype == kBF16 && xo_dtype == kBF16) LLME_NA(bf16, bf16, bf16);
    else return kErrBadArgument;
#undef LLME_NA
#undef LLME_NAV
    return launch_status();
}

extern "C" int llme_scale_f32(float* x, size_t n, float s, hipStream_t stream) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(scale_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, stream, x, n, s);
    return launch_status();
}

LLME_LOAD_ENTRY(residual_norm)
