// A sublayer's result normed before it joins the residual stream ("sandwich" layers):
//   h[t] += w_post * y[t] / sqrt(mean(y[t]^2) + eps)
// and, in the same pass over the row, the norm in front of the next sublayer:
//   x[t] = w_next * h[t] / sqrt(mean(h[t]^2) + eps)      (h as just updated)
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
    if (w_next == nullptr) return;
    const float inv2 = 1.0f / sqrtf(block_sum(ss2, scratch, 4) / static_cast<float>(H) + eps);
    TO* xr = x_out + static_cast<size_t>(t) * H;
    for (int i = threadIdx.x; i < H; i += 256) xr[i] = from_float<TO>((to_float(w_next[i]) * row[i]) * inv2);
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
#define LLME_NA(TW, TN, TO)                                                                               \
    hipLaunchKernelGGL((norm_add_kernel<TW, TN, TO>), dim3(T), dim3(256), lds, stream, y,                 \
                       static_cast<const TW*>(w_post), h, static_cast<const TN*>(w_next), static_cast<TO*>(x_out), H, eps)
    if (w_next == nullptr) {
        if (w_dtype == kF32) LLME_NA(float, float, float);
        else if (w_dtype == kBF16) LLME_NA(bf16, float, float);
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
    return launch_status();
}

extern "C" int llme_scale_f32(float* x, size_t n, float s, hipStream_t stream) {
    if (n == 0) return 0;
    hipLaunchKernelGGL(scale_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, stream, x, n, s);
    return launch_status();
}

LLME_LOAD_ENTRY(residual_norm)
