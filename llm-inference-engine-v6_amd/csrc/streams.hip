// A residual kept as several streams (hyper-connections): x [S, T, H], 32-bit.
//
//   spread      x[s] = x[0] for every s                (all streams start as the embedding)
//   read_norm   u[t] = sum_s a[s] x[s][t];  out[r] = w * u[row(r)] / sqrt(mean(u^2) + eps)
//               (a null: plain sum; w null: u itself, 32-bit)
//   write       x'[j][t] = sum_s m[s][j] x[s][t] + b[j] * y[t]  for all j at once, in place
//
// Everything is summed in 32-bit; only read_norm's output may be a 16-bit type.
#include "common.h"

namespace llme {

constexpr int kMaxStreams = 8;

__global__ __launch_bounds__(256) void streams_spread_kernel(float4* __restrict__ x, int S, size_t n4) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n4; i += static_cast<size_t>(gridDim.x) * 256) {
        const float4 v = x[i];
        for (int s = 1; s < S; ++s) x[static_cast<size_t>(s) * n4 + i] = v;
    }
}

// (value by value, for sizes that are no multiple of 4)
__global__ __launch_bounds__(256) void streams_spread_scalar_kernel(float* __restrict__ x, int S, size_t n) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * 256) {
        const float v = x[i];
        for (int s = 1; s < S; ++s) x[static_cast<size_t>(s) * n + i] = v;
    }
}

// One workgroup per output row. The row's mixed value is kept in registers between the two passes
// (up to NV values per thread), or recomputed when the row is wider than that.
template <typename TW, typename TO, int NV>
__global__ __launch_bounds__(256) void streams_read_norm_kernel(const float* __restrict__ x, int S, size_t stream_stride,
                                                                 const float* __restrict__ a, const TW* __restrict__ w,
                                                                 TO* __restrict__ out, const int* __restrict__ rows,
                                                                 int H, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const float* xr = x + static_cast<size_t>(src) * H;
    float coef[kMaxStreams];
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s) coef[s] = s < S ? (a ? a[s] : 1.0f) : 0.f;
    float u[NV];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = threadIdx.x + j * 256;
        float v = 0.f;
        if (i < H)
            for (int s = 0; s < S; ++s) v += coef[s] * xr[static_cast<size_t>(s) * stream_stride + i];
        u[j] = v;
        ss += v * v;
    }
    for (int i = threadIdx.x + NV * 256; i < H; i += 256) {
        float v = 0.f;
        for (int s = 0; s < S; ++s) v += coef[s] * xr[static_cast<size_t>(s) * stream_stride + i];
        ss += v * v;
    }
    TO* o = out + static_cast<size_t>(r) * H;
    if (w == nullptr) {                     // the mixed value itself
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = threadIdx.x + j * 256;
            if (i < H) o[i] = from_float<TO>(u[j]);
        }
        for (int i = threadIdx.x + NV * 256; i < H; i += 256) {
            float v = 0.f;
            for (int s = 0; s < S; ++s) v += coef[s] * xr[static_cast<size_t>(s) * stream_stride + i];
            o[i] = from_float<TO>(v);
        }
        return;
    }
    ss = block_sum(ss, scratch, 4);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = threadIdx.x + j * 256;
        if (i < H) o[i] = from_float<TO>((to_float(w[i]) * u[j]) * inv);
    }
    for (int i = threadIdx.x + NV * 256; i < H; i += 256) {
        float v = 0.f;
        for (int s = 0; s < S; ++s) v += coef[s] * xr[static_cast<size_t>(s) * stream_stride + i];
        o[i] = from_float<TO>((to_float(w[i]) * v) * inv);
    }
}

// The same with a row's values four at a time (H a multiple of 4, at most 1024 NV4): every load of a thread is asked
// for before the first is used, so that a step of a few rows (decoding) does not wait for them one after the other.
constexpr int kVecStreams = 4;     // streams the vector form holds in registers
template <typename TW, typename TO, int NV4>
__global__ __launch_bounds__(256) void streams_read_norm_vec_kernel(const float* __restrict__ x, int S, size_t stream_stride,
                                                                     const float* __restrict__ a, const TW* __restrict__ w,
                                                                     TO* __restrict__ out, const int* __restrict__ rows,
                                                                     int H, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const float* xr = x + static_cast<size_t>(src) * H;
    float coef[kVecStreams];
#pragma unroll
    for (int s = 0; s < kVecStreams; ++s) coef[s] = s < S ? (a ? a[s] : 1.0f) : 0.f;
    float4 v[NV4][kVecStreams];
#pragma unroll
    for (int j = 0; j < NV4; ++j) {
        const int i = (threadIdx.x + j * 256) * 4;
#pragma unroll
        for (int s = 0; s < kVecStreams; ++s)
            v[j][s] = (i < H && s < S) ? *reinterpret_cast<const float4*>(xr + static_cast<size_t>(s) * stream_stride + i)
                                       : float4{0.f, 0.f, 0.f, 0.f};
    }
    float u[NV4][4];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV4; ++j) {
        u[j][0] = u[j][1] = u[j][2] = u[j][3] = 0.f;
#pragma unroll
        for (int s = 0; s < kVecStreams; ++s) {
            u[j][0] += coef[s] * v[j][s].x;
            u[j][1] += coef[s] * v[j][s].y;
            u[j][2] += coef[s] * v[j][s].z;
            u[j][3] += coef[s] * v[j][s].w;
        }
        ss += u[j][0] * u[j][0] + u[j][1] * u[j][1] + u[j][2] * u[j][2] + u[j][3] * u[j][3];
    }
    TO* o = out + static_cast<size_t>(r) * H;
    float inv = 1.f;
    if (w != nullptr) {
        ss = block_sum(ss, scratch, 4);
        inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps);
    }
#pragma unroll
    for (int j = 0; j < NV4; ++j) {
        const int i = (threadIdx.x + j * 256) * 4;
        if (i >= H) continue;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            o[i + e] = from_float<TO>(w != nullptr ? (to_float(w[i + e]) * u[j][e]) * inv : u[j][e]);
    }
}

// write and the next sublayer's read_norm in one pass over a row: the new streams are stored and, still in registers,
// mixed by the next sublayer's weights a2 and normed by w2 into out. Same limits as the vector form of read_norm.
template <typename TW, typename TO, int NV4>
__global__ __launch_bounds__(256) void streams_write_read_norm_kernel(float* __restrict__ x, int S, size_t stream_stride,
                                                                      const float* __restrict__ mix, const float* __restrict__ b,
                                                                      const float* __restrict__ y, const float* __restrict__ a2,
                                                                      const TW* __restrict__ w2, TO* __restrict__ out, int H, float eps) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    float* xr = x + static_cast<size_t>(r) * H;
    const float* yr = y + static_cast<size_t>(r) * H;
    float m[kVecStreams][kVecStreams], bo[kVecStreams], coef[kVecStreams];
#pragma unroll
    for (int s = 0; s < kVecStreams; ++s) {
        bo[s] = s < S ? b[s] : 0.f;
        coef[s] = s < S ? a2[s] : 0.f;
#pragma unroll
        for (int t = 0; t < kVecStreams; ++t) m[s][t] = (s < S && t < S) ? mix[s * S + t] : 0.f;
    }
    float4 v[NV4][kVecStreams], yv[NV4];
#pragma unroll
    for (int j = 0; j < NV4; ++j) {
        const int i = (threadIdx.x + j * 256) * 4;
        yv[j] = i < H ? *reinterpret_cast<const float4*>(yr + i) : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < kVecStreams; ++s)
            v[j][s] = (i < H && s < S) ? *reinterpret_cast<const float4*>(xr + static_cast<size_t>(s) * stream_stride + i)
                                       : float4{0.f, 0.f, 0.f, 0.f};
    }
    float u[NV4][4];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV4; ++j) {
        const int i = (threadIdx.x + j * 256) * 4;
        u[j][0] = u[j][1] = u[j][2] = u[j][3] = 0.f;
#pragma unroll
        for (int t = 0; t < kVecStreams; ++t) {
            if (t >= S) break;
            float n[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < kVecStreams; ++s) {
                n[0] += m[s][t] * v[j][s].x;
                n[1] += m[s][t] * v[j][s].y;
                n[2] += m[s][t] * v[j][s].z;
                n[3] += m[s][t] * v[j][s].w;
            }
            n[0] += bo[t] * yv[j].x;
            n[1] += bo[t] * yv[j].y;
            n[2] += bo[t] * yv[j].z;
            n[3] += bo[t] * yv[j].w;
            if (i < H) *reinterpret_cast<float4*>(xr + static_cast<size_t>(t) * stream_stride + i) = float4{n[0], n[1], n[2], n[3]};
#pragma unroll
            for (int e = 0; e < 4; ++e) u[j][e] += coef[t] * n[e];
        }
        ss += u[j][0] * u[j][0] + u[j][1] * u[j][1] + u[j][2] * u[j][2] + u[j][3] * u[j][3];
    }
    ss = block_sum(ss, scratch, 4);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps);
    TO* o = out + static_cast<size_t>(r) * H;
#pragma unroll
    for (int j = 0; j < NV4; ++j) {
        const int i = (threadIdx.x + j * 256) * 4;
        if (i >= H) continue;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[i + e] = from_float<TO>((to_float(w2[i + e]) * u[j][e]) * inv);
    }
}

__global__ __launch_bounds__(256) void streams_write_kernel(float* __restrict__ x, int S, size_t n, const float* __restrict__ mix,
                                                            const float* __restrict__ b, const float* __restrict__ y) {
    __shared__ float m[kMaxStreams * kMaxStreams];
    __shared__ float bo[kMaxStreams];
    if (threadIdx.x < S * S) m[threadIdx.x] = mix[threadIdx.x];
    if (threadIdx.x < S) bo[threadIdx.x] = b[threadIdx.x];
    __syncthreads();
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<size_t>(gridDim.x) * 256) {
        float old[kMaxStreams];
#pragma unroll
        for (int s = 0; s < kMaxStreams; ++s) old[s] = s < S ? x[static_cast<size_t>(s) * n + i] : 0.f;
        const float yv = y[i];
#pragma unroll
        for (int j = 0; j < kMaxStreams; ++j) {
            if (j >= S) break;
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < kMaxStreams; ++s)
                if (s < S) v += m[s * S + j] * old[s];
            x[static_cast<size_t>(j) * n + i] = v + bo[j] * yv;
        }
    }
}

template <typename TW, typename TO>
static int launch_read_norm(const float* x, int S, size_t stride, const float* a, const void* w, void* out, const int* rows,
                            int R, int H, float eps, hipStream_t stream) {
    const TW* wp = static_cast<const TW*>(w);
    TO* op = static_cast<TO*>(out);
    if (H % 4 == 0 && H <= 4096 && S <= kVecStreams && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        if (H <= 1024) streams_read_norm_vec_kernel<TW, TO, 1><<<R, 256, 0, stream>>>(x, S, stride, a, wp, op, rows, H, eps);
        else if (H <= 2048) streams_read_norm_vec_kernel<TW, TO, 2><<<R, 256, 0, stream>>>(x, S, stride, a, wp, op, rows, H, eps);
        else streams_read_norm_vec_kernel<TW, TO, 4><<<R, 256, 0, stream>>>(x, S, stride, a, wp, op, rows, H, eps);
        return launch_status();
    }
    if (H <= 1024)
        streams_read_norm_kernel<TW, TO, 4><<<R, 256, 0, stream>>>(x, S, stride, a, wp, op, rows, H, eps);
    else
        streams_read_norm_kernel<TW, TO, 16><<<R, 256, 0, stream>>>(x, S, stride, a, wp, op, rows, H, eps);
    return launch_status();
}

}  // namespace llme

using namespace llme;

extern "C" int llme_streams_spread(void* x, int S, size_t per_stream, hipStream_t stream) {
    if (S <= 1 || per_stream == 0) return 0;
    if (per_stream % 4 || reinterpret_cast<uintptr_t>(x) % 16) {
        const int blocks = static_cast<int>(per_stream / 256 + 1 < 4096 ? per_stream / 256 + 1 : 4096);
        streams_spread_scalar_kernel<<<blocks, 256, 0, stream>>>(static_cast<float*>(x), S, per_stream);
        return launch_status();
    }
    const size_t n4 = per_stream / 4;
    const int grid = static_cast<int>(n4 / 256 + 1 < 4096 ? n4 / 256 + 1 : 4096);
    streams_spread_kernel<<<grid, 256, 0, stream>>>(static_cast<float4*>(x), S, n4);
    return launch_status();
}

// x [S, T, H] 32-bit; a [S] 32-bit or null; w [H] (w_dtype) or null; out [R, H] (out_dtype; 32-bit when w is null);
// rows [R] or null (then R == T).
extern "C" int llme_streams_read_norm(const void* x, int S, int T, int H, const void* a, const void* w, int w_dtype,
                                      void* out, int out_dtype, const void* rows, int R, float eps, hipStream_t stream) {
    if (R <= 0 || H <= 0) return 0;
    if (S < 1 || S > kMaxStreams) return kErrUnsupported;
    const size_t stride = static_cast<size_t>(T) * H;
    const float* xp = static_cast<const float*>(x);
    const float* ap = static_cast<const float*>(a);
    const int* rp = static_cast<const int*>(rows);
    if (w == nullptr) {
        if (out_dtype != kF32) return kErrBadArgument;
        return launch_read_norm<float, float>(xp, S, stride, ap, nullptr, out, rp, R, H, eps, stream);
    }
    switch (w_dtype * 2 + out_dtype) {
        case 0: return launch_read_norm<float, float>(xp, S, stride, ap, w, out, rp, R, H, eps, stream);
        case 1: return launch_read_norm<float, bf16>(xp, S, stride, ap, w, out, rp, R, H, eps, stream);
        case 2: return launch_read_norm<bf16, float>(xp, S, stride, ap, w, out, rp, R, H, eps, stream);
        case 3: return launch_read_norm<bf16, bf16>(xp, S, stride, ap, w, out, rp, R, H, eps, stream);
    }
    return kErrBadArgument;
}

// write, then read_norm with the weights of the sublayer behind (a2 [S], w2 [H]) into out [T, H]: one kernel where the
// vector form fits (returns kErrUnsupported otherwise, having done nothing: the caller then launches the two).
extern "C" int llme_streams_write_read_norm(void* x, int S, int T, int H, const void* mix, const void* b, const void* y,
                                            const void* a2, const void* w2, int w_dtype, void* out, int out_dtype, float eps,
                                            hipStream_t stream) {
    if (T <= 0 || H <= 0) return 0;
    if (S < 1 || S > kVecStreams || H % 4 || H > 4096 || reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(y) % 16)
        return kErrUnsupported;
    const size_t stride = static_cast<size_t>(T) * H;
#define LLME_SWR(TW_, TO_, N_)                                                                                            \
    streams_write_read_norm_kernel<TW_, TO_, N_><<<T, 256, 0, stream>>>(                                                  \
        static_cast<float*>(x), S, stride, static_cast<const float*>(mix), static_cast<const float*>(b),                  \
        static_cast<const float*>(y), static_cast<const float*>(a2), static_cast<const TW_*>(w2), static_cast<TO_*>(out), H, eps)
#define LLME_SWR_N(TW_, TO_)                                                                                              \
    if (H <= 1024) LLME_SWR(TW_, TO_, 1); else if (H <= 2048) LLME_SWR(TW_, TO_, 2); else LLME_SWR(TW_, TO_, 4)
    switch (w_dtype * 2 + out_dtype) {
        case 0: LLME_SWR_N(float, float); break;
        case 1: LLME_SWR_N(float, bf16); break;
        case 2: LLME_SWR_N(bf16, float); break;
        case 3: LLME_SWR_N(bf16, bf16); break;
        default: return kErrBadArgument;
    }
#undef LLME_SWR_N
#undef LLME_SWR
    return launch_status();
}

// x [S, T, H] in place; mix [S, S] (from, to), b [S], y [T, H], all 32-bit.
extern "C" int llme_streams_write(void* x, int S, size_t per_stream, const void* mix, const void* b, const void* y,
                                  hipStream_t stream) {
    if (per_stream == 0) return 0;
    if (S < 1 || S > kMaxStreams) return kErrUnsupported;
    const int grid = static_cast<int>(per_stream / 256 + 1 < 8192 ? per_stream / 256 + 1 : 8192);
    streams_write_kernel<<<grid, 256, 0, stream>>>(static_cast<float*>(x), S, per_stream, static_cast<const float*>(mix),
                                                   static_cast<const float*>(b), static_cast<const float*>(y));
    return launch_status();
}

LLME_LOAD_ENTRY(streams)
