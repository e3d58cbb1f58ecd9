// Attention whose keys and values are expanded from one latent vector per token.
//
// Per token the cache keeps a row of D = R + r entries: the latent c [R] (RMS-normed) and, where the mixer
// rotates, r entries of a rotated key part that all heads share. A head's key would be [Wuk_h c | shared part]
// and its value Wuv_h c; neither is ever built. The query takes the key map onto itself,
//   q'_h = [Wuk_h^T q_h(unrotated) | q_h(rotated)]        (D entries),
// so that the score of head h with key j is q'_h . row_j, the same row for every head, and the weighted sum
// runs over the rows' first R entries: o'_h = sum_j p_hj c_j, the head's output being Wuv_h o'_h. Both maps
// are products batched over the heads (head_gemm).
//
// Kernels: latent_prepare (the two RMS norms behind the down maps, the rotation of the shared key part, the
// cache write), latent_q_rotate (the rotated part of the queries, into q'), head_gemm, and latent_attention
// (plain precision: scores, softmax statistics and sums in 32-bit; any sizes up to D = 1024, R = 512).
//
// Rotation: of a part's r entries the first rd are rotated, the rest pass unchanged; entries (2i, 2i + 1) turn by angle = position * freq[i], a 32-bit product; cos and sin are
// multiplied by `mag` (1 without frequency scaling). A token at position p sees keys lo .. p of its own
// request, lo = 0 or p - window + 1.
//
//   cache       [pages, page, D]; key t of request s lies in page block_table[s][t / page] at row t % page
#include "common.h"
#include <math.h>

namespace llme {

// ---------------------------------------------------------------------------------
// p [T, ldp] 32-bit, columns [0, Rq): the query latent, [Rq, Rq + R): the key/value latent, then r shared
// key entries. cq [T, Rq] = wq * rms-normed query latent; the cache row = [wc * rms-normed latent | rotated].
// R == 0: a layer that reads another layer's rows only norms its query latent.
template <typename TW, typename TO>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    const float* __restrict__ p, int ldp, int Rq, int R, int r, int rd, const TW* __restrict__ wq, const TW* __restrict__ wc,
    const float* __restrict__ freq, float mag, const int* __restrict__ positions, const int* __restrict__ seq_idx,
    const int* __restrict__ block_table, int max_blocks, TO* __restrict__ cq, TO* __restrict__ cache, int page, float eps) {
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const float* row = p + static_cast<size_t>(t) * ldp;
    float ss = 0.f;
    for (int i = threadIdx.x; i < Rq; i += 256) ss = fmaf(row[i], row[i], ss);
    const float inv_q = 1.0f / sqrtf(block_sum(ss, scratch, 4) / static_cast<float>(Rq) + eps);
    TO* cqr = cq + static_cast<size_t>(t) * Rq;
    for (int i = threadIdx.x; i < Rq; i += 256) cqr[i] = from_float<TO>((to_float(wq[i]) * row[i]) * inv_q);
    if (R == 0) return;
    const int pos = positions[t];
    const int pg = block_table[static_cast<size_t>(seq_idx[t]) * max_blocks + pos / page];
    TO* dst = cache + (static_cast<size_t>(pg) * page + pos % page) * (R + r);
    const float* c = row + Rq;
    ss = 0.f;
    for (int i = threadIdx.x; i < R; i += 256) ss = fmaf(c[i], c[i], ss);
    const float inv_c = 1.0f / sqrtf(block_sum(ss, scratch, 4) / static_cast<float>(R) + eps);
    for (int i = threadIdx.x; i < R; i += 256) dst[i] = from_float<TO>((to_float(wc[i]) * c[i]) * inv_c);
    const float* kr = c + R;
    for (int i = threadIdx.x; i < r / 2; i += 256) {
        float sn = 0.f, cs = 1.f;               // (entries beyond the first rd pass as they are)
        if (2 * i < rd) {
            sincosf(static_cast<float>(pos) * freq[i], &sn, &cs);
            sn *= mag;
            cs *= mag;
        }
        const float u = kr[2 * i], v = kr[2 * i + 1];
        dst[R + 2 * i] = from_float<TO>(u * cs - v * sn);
        dst[R + 2 * i + 1] = from_float<TO>(v * cs + u * sn);
    }
}

// q [T, n (d + r)] -> qp [T, n, R + r]: the last r entries of every head, rotated at the token's position.
template <typename TQ>
__global__ void latent_q_rotate_kernel(const TQ* __restrict__ q, const float* __restrict__ freq, float mag,
                                       const int* __restrict__ positions, TQ* __restrict__ qp, int n, int d, int r, int rd,
                                       int R, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;      // (t, head, pair)
    if (idx >= total) return;
    const int half = r / 2;
    const int i = static_cast<int>(idx % half);
    const size_t th = idx / half;                                               // t * n + head
    const int t = static_cast<int>(th / n);
    float sn = 0.f, cs = 1.f;
    if (2 * i < rd) {
        sincosf(static_cast<float>(positions[t]) * freq[i], &sn, &cs);
        sn *= mag;
        cs *= mag;
    }
    const TQ* src = q + th * (d + r) + d;
    TQ* dst = qp + th * (R + r) + R;
    const float u = to_float(src[2 * i]), v = to_float(src[2 * i + 1]);
    dst[2 * i] = from_float<TQ>(u * cs - v * sn);
    dst[2 * i + 1] = from_float<TQ>(v * cs + u * sn);
}

// ---------------------------------------------------------------------------------
// out[t, h, n] = sum_k a[t, h, k] w[h, n, k]; a and out are addressed by a row stride and a head stride
// (column ranges of wider rows), w is [heads, N, K] contiguous. Tiles of 16 rows x 64 columns, k in slabs
// of 32 through LDS, 32-bit sums.
template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void head_gemm_kernel(const TA* __restrict__ a, long lda, long sa,
                                                        const TW* __restrict__ w, TO* __restrict__ out, long ldo, long so,
                                                        int T, int N, int K) {
    __shared__ float As[16][33];
    __shared__ float Ws[64][33];
    const int h = blockIdx.z;
    const int t0 = blockIdx.y * 16, n0 = blockIdx.x * 64;
    const int tr = threadIdx.x / 16, tc = threadIdx.x % 16;         // row of the tile, group of 4 columns
    const TW* wh = w + static_cast<size_t>(h) * N * K;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += 32) {
        for (int i = threadIdx.x; i < 16 * 32; i += 256) {
            const int rr = i / 32, kk = i % 32;
            const int t = t0 + rr, k = k0 + kk;
            As[rr][kk] = (t < T && k < K) ? to_float(a[static_cast<size_t>(t) * lda + static_cast<size_t>(h) * sa + k]) : 0.f;
        }
        for (int i = threadIdx.x; i < 64 * 32; i += 256) {
            const int nn = i / 32, kk = i % 32;
            const int n = n0 + nn, k = k0 + kk;
            Ws[nn][kk] = (n < N && k < K) ? to_float(wh[static_cast<size_t>(n) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < 32; ++kk) {
            const float av = As[tr][kk];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fmaf(av, Ws[tc + 16 * j][kk], acc[j]);
        }
        __syncthreads();
    }
    const int t = t0 + tr;
    if (t >= T) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + tc + 16 * j;
        if (n < N) out[static_cast<size_t>(t) * ldo + static_cast<size_t>(h) * so + n] = from_float<TO>(acc[j]);
    }
}

// ---------------------------------------------------------------------------------
// Plain-precision attention over the latent rows: one wavefront per (token, head), or NW that take every
// NW-th chunk of 64 keys and join through LDS when a step has few such pairs. A lane scores one key of the
// chunk (q' waits in LDS), then the lanes share the rows' first R entries for the weighted sum.
constexpr int kLatMaxD = 1024;
constexpr int kLatMaxR = 512;

template <typename TQ, typename TC, int NW>
__global__ __launch_bounds__(NW * 64) void latent_attention_kernel(
    const TQ* __restrict__ qp, const TC* __restrict__ cache, TQ* __restrict__ out, const int* __restrict__ positions,
    const int* __restrict__ seq_idx, const int* __restrict__ block_table, int max_blocks, int n, int R, int D, int page,
    float scale, int window) {
    constexpr int PER_LANE = kLatMaxR / kWave;
    __shared__ float qs[kLatMaxD];
    __shared__ float join_m[NW], join_l[NW];
    __shared__ float join_acc[NW > 1 ? NW : 1][NW > 1 ? kLatMaxR : 1];
    const int t = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int pos = positions[t];
    const int* table = block_table + static_cast<size_t>(seq_idx[t]) * max_blocks;
    const int hi = pos + 1;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const TQ* qrow = qp + (static_cast<size_t>(t) * n + h) * D;
    for (int i = threadIdx.x; i < D; i += NW * kWave) qs[i] = to_float(qrow[i]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[PER_LANE];
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) acc[i] = 0.f;
    for (int t0 = lo + wave * kWave; t0 < hi; t0 += NW * kWave) {
        const int key = t0 + lane;
        float sc = -INFINITY;
        if (key < hi) {
            const TC* kr = cache + (static_cast<size_t>(table[key / page]) * page + key % page) * D;
            float dot = 0.f;
            for (int i = 0; i < D; ++i) dot = fmaf(qs[i], to_float(kr[i]), dot);
            sc = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(sc));
        const float alpha = expf(m - m_new);
        const float p = (key < hi) ? expf(sc - m_new) : 0.f;
        l = l * alpha + wave_sum(p);
        m = m_new;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) acc[i] *= alpha;
        const int cnt = (hi - t0 < kWave) ? hi - t0 : kWave;
        for (int j = 0; j < cnt; ++j) {
            const int kj = t0 + j;
            const TC* vr = cache + (static_cast<size_t>(table[kj / page]) * page + kj % page) * D;
            const float pj = __shfl(p, j, kWave);
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) {
                const int c = lane + i * kWave;
                if (c < R) acc[i] = fmaf(pj, to_float(vr[c]), acc[i]);
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
            const float f = expf(join_m[w] - mx);
            l += f * join_l[w];
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) acc[i] += f * join_acc[w][lane + i * kWave];
        }
    }
    const float inv = 1.0f / l;
    TQ* orow = out + (static_cast<size_t>(t) * n + h) * R;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int c = lane + i * kWave;
        if (c < R) orow[c] = from_float<TQ>(acc[i] * inv);
    }
}

}  // namespace llme

using namespace llme;

extern "C" int llme_latent_prepare(const float* p, int ldp, int Rq, int R, int r, int rd, const void* wq, const void* wc,
                                   int w_dtype, const float* freq, float mag, const int* positions, const int* seq_idx,
                                   const int* block_table, int max_blocks, void* cq, void* cache, int out_dtype,
                                   int page, int T, float eps, hipStream_t stream) {
    if (T <= 0) return 0;
    if (Rq <= 0 || R < 0 || r < 0 || r % 2 || ldp < Rq + R + r || (R > 0 && page <= 0)) return kErrBadArgument;
    if (rd < 0 || rd > r || rd % 2 || (rd > 0 && (freq == nullptr || R == 0))) return kErrBadArgument;
#define LLME_LP(TW, TO)                                                                                          \
    hipLaunchKernelGGL((latent_prepare_kernel<TW, TO>), dim3(T), dim3(256), 0, stream, p, ldp, Rq, R, r, rd,     \
                       static_cast<const TW*>(wq), static_cast<const TW*>(wc), freq, mag, positions, seq_idx,    \
                       block_table, max_blocks, static_cast<TO*>(cq), static_cast<TO*>(cache), page, eps)
    if (w_dtype == kF32 && out_dtype == kF32) LLME_LP(float, float);
    else if (w_dtype == kF32 && out_dtype == kBF16) LLME_LP(float, bf16);
    else if (w_dtype == kBF16 && out_dtype == kF32) LLME_LP(bf16, float);
    else if (w_dtype == kBF16 && out_dtype == kBF16) LLME_LP(bf16, bf16);
    else return kErrBadArgument;
#undef LLME_LP
    return launch_status();
}

extern "C" int llme_latent_q_rotate(const void* q, int dtype, const float* freq, float mag, const int* positions,
                                    void* qp, int T, int n, int d, int r, int rd, int R, hipStream_t stream) {
    if (T <= 0 || r == 0) return 0;
    if (r % 2 || rd < 0 || rd > r || rd % 2 || n <= 0 || d < 0 || R < 0 || (rd > 0 && freq == nullptr)) return kErrBadArgument;
    const size_t total = static_cast<size_t>(T) * n * (r / 2);
    const dim3 grid(static_cast<unsigned>((total + 255) / 256));
    if (dtype == kF32)
        hipLaunchKernelGGL(latent_q_rotate_kernel<float>, grid, dim3(256), 0, stream, static_cast<const float*>(q), freq,
                           mag, positions, static_cast<float*>(qp), n, d, r, rd, R, total);
    else if (dtype == kBF16)
        hipLaunchKernelGGL(latent_q_rotate_kernel<bf16>, grid, dim3(256), 0, stream, static_cast<const bf16*>(q), freq,
                           mag, positions, static_cast<bf16*>(qp), n, d, r, rd, R, total);
    else return kErrBadArgument;
    return launch_status();
}

extern "C" int llme_head_gemm(const void* a, int a_dtype, long lda, long sa, const void* w, int w_dtype, void* out,
                              int out_dtype, long ldo, long so, int T, int heads, int N, int K, hipStream_t stream) {
    if (T <= 0 || heads <= 0 || N <= 0) return 0;
    if (K <= 0 || heads > 65535) return kErrBadArgument;
    const dim3 grid((N + 63) / 64, (T + 15) / 16, heads);
    if (grid.y > 65535) return kErrUnsupported;
#define LLME_HG(TA, TW, TO)                                                                                   \
    hipLaunchKernelGGL((head_gemm_kernel<TA, TW, TO>), grid, dim3(256), 0, stream, static_cast<const TA*>(a), \
                       lda, sa, static_cast<const TW*>(w), static_cast<TO*>(out), ldo, so, T, N, K)
    if (a_dtype == kF32 && w_dtype == kF32 && out_dtype == kF32) LLME_HG(float, float, float);
    else if (a_dtype == kBF16 && w_dtype == kBF16 && out_dtype == kBF16) LLME_HG(bf16, bf16, bf16);
    else if (a_dtype == kBF16 && w_dtype == kF32 && out_dtype == kBF16) LLME_HG(bf16, float, bf16);
    else if (a_dtype == kF32 && w_dtype == kBF16 && out_dtype == kF32) LLME_HG(float, bf16, float);
    else return kErrBadArgument;
#undef LLME_HG
    return launch_status();
}

extern "C" int llme_latent_attention(const void* qp, int q_dtype, const void* cache, int cache_dtype, void* out,
                                     const int* positions, const int* seq_idx, const int* block_table, int max_blocks,
                                     int T, int n, int R, int D, int page, float scale, int window, hipStream_t stream) {
    if (T <= 0) return 0;
    if (n <= 0 || R <= 0 || D < R || page <= 0) return kErrBadArgument;
    if (D > kLatMaxD || R > kLatMaxR || n > 65535) return kErrUnsupported;
    const dim3 grid(T, n);
    const bool few = static_cast<long>(T) * n < 4096;
#define LLME_LA(TQ, TC)                                                                                       \
    do {                                                                                                      \
        if (few)                                                                                              \
            hipLaunchKernelGGL((latent_attention_kernel<TQ, TC, 8>), grid, dim3(8 * 64), 0, stream,           \
                               static_cast<const TQ*>(qp), static_cast<const TC*>(cache), static_cast<TQ*>(out), \
                               positions, seq_idx, block_table, max_blocks, n, R, D, page, scale, window);    \
        else                                                                                                  \
            hipLaunchKernelGGL((latent_attention_kernel<TQ, TC, 1>), grid, dim3(64), 0, stream,               \
                               static_cast<const TQ*>(qp), static_cast<const TC*>(cache), static_cast<TQ*>(out), \
                               positions, seq_idx, block_table, max_blocks, n, R, D, page, scale, window);    \
    } while (0)
    if (q_dtype == kF32 && cache_dtype == kF32) LLME_LA(float, float);
    else if (q_dtype == kBF16 && cache_dtype == kBF16) LLME_LA(bf16, bf16);
    else return kErrBadArgument;
#undef LLME_LA
    return launch_status();
}

LLME_LOAD_ENTRY(latent_attention)
