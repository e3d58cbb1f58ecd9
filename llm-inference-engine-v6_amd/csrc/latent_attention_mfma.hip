// Latent attention on the matrix cores (v_mfma_f32_16x16x32_bf16), bfloat16 queries and cache rows.
//
// Every head of a token is scored against the same cached rows (D = R + r entries: the latent and the shared
// rotated part), and the weighted sum runs over the rows' first R entries. So a block of 32 rows is fetched
// once into LDS by a workgroup and used by all of its 64 query rows (a row = one head of one token), first
// as the keys, then as the values:
//   S^T[key, row] = sum_d rows[key, d] q'[row, d]      first operand from LDS as the rows lie, 16 bytes a lane
//   O[row, c]    += sum_key P[row, key] rows[key, c]   second operand from a transposed copy of the rows'
//                                                      first R entries that the staging threads write
// Lane l of a wavefront holds, for query row l % 16, the scores of keys 4 (l / 16) + e of both 16-key halves,
// which are the 8 keys it must supply as first operand of the second product: weights never pass through LDS.
//
// A workgroup takes 64 consecutive (token, head) pairs of one request (heads fastest), a wavefront 16 of
// them; with 16 heads or more a wavefront's rows are heads of one token, so decoding and prompts are the same
// case. Every row has its own first and last visible key. The keys of a workgroup are cut into `nsplit` runs
// of whole blocks (grid z); with more than one run the partial sums (32-bit, not normalised), maxima and
// weights' sums go to a workspace and latent_join adds them in a fixed order.
//
// Softmax: running maximum m and sum l per row in units of log2; the sum adds the weights as rounded to
// bfloat16, which is what the second product sees.
//
//   qa [.., R], qr [.., r]   a pair's rows at (token * q_ts + head * q_hs) * R resp. * r
//   out [.., R]              at (token * o_ts + head * o_hs) * R
//   cache [pages, page, D]   page a multiple of 16; key t of request s in page block_table[s][t / page]
#include "common.h"
#include <math.h>

namespace llme {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

constexpr float kLatNoMax = -1.0e30f;
constexpr int kVtStride = 40;           // elements of a transposed row: 32 keys + 8 (80 bytes: 8-byte reads without conflicts)

__host__ __device__ inline int lat_k_stride(int D) {
    // elements of a staged row: its bytes are 32 more than a multiple of 128, so that 16-byte operand reads run at full rate
    const int bytes = D * 2;
    return (bytes + ((32 - bytes % 128) + 128) % 128) / 2;
}

struct LatentArgs {
    const bf16* qa;
    const bf16* qr;
    const bf16* cache;
    bf16* out;
    float* ws_o;                // [nsplit, pairs, R]
    float* ws_ml;               // [nsplit, pairs, 2]
    const int* positions;
    const int* q_start;
    const int* block_table;
    int max_blocks, T, n, R, r, page, window, nsplit;
    long q_ts, q_hs, o_ts, o_hs;
    float scale_log2;
};

template <int DC, int RC>       // 32-entry chunks of a row, 16-entry chunks of the latent: the most this instance holds
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(LatentArgs a) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int D = a.R + a.r, dc = D / 32, rc = a.R / 16;
    const int ks = lat_k_stride(D);
    bf16* Ks = reinterpret_cast<bf16*>(lds_raw);                    // [32][ks]
    bf16* Vt = Ks + 32 * ks;                                        // [R][kVtStride]
    const int s = blockIdx.y, z = blockIdx.z;
    const int first_tok = a.q_start[s], n_tok = a.q_start[s + 1] - first_tok;
    const int pairs = n_tok * a.n;
    const int p0 = blockIdx.x * 64;
    if (p0 >= pairs) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int* table = a.block_table + static_cast<size_t>(s) * a.max_blocks;

    // this lane's query row
    const int p = p0 + wave * 16 + r16;
    const bool row_ok = p < pairs;
    const int tl = row_ok ? p / a.n : 0, h = row_ok ? p % a.n : 0;
    const int tok = first_tok + tl;
    const int pos = a.positions[tok];
    const int row_hi = row_ok ? pos : -1;
    const int row_lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
    // the workgroup's keys: from the first row's first key to the last existing row's position
    const int last_p = (p0 + 63 < pairs ? p0 + 63 : pairs - 1);
    const int wg_hi = a.positions[first_tok + last_p / a.n];
    const int first_pos = a.positions[first_tok + p0 / a.n];
    const int wg_lo = (a.window > 0 && first_pos - a.window + 1 > 0) ? first_pos - a.window + 1 : 0;
    const int b_first = wg_lo / 32, b_all = wg_hi / 32 + 1 - b_first;
    const int b_per = (b_all + a.nsplit - 1) / a.nsplit;
    const int b_begin = b_first + z * b_per;
    const int b_end = (b_begin + b_per < b_first + b_all) ? b_begin + b_per : b_first + b_all;

    // q' of this lane's row as second operand: chunk c holds entries 32 c + 8 g .. + 7
    bf16x8 qf[DC];
    {
        const bf16* qa_row = a.qa + (static_cast<long>(tok) * a.q_ts + static_cast<long>(h) * a.q_hs) * a.R;
        const bf16* qr_row = a.r ? a.qr + (static_cast<long>(tok) * a.q_ts + static_cast<long>(h) * a.q_hs) * a.r : nullptr;
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            const int d = c * 32 + g * 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[c][e] = static_cast<__bf16>(0.f);
            if (c < dc && row_ok)
                qf[c] = d < a.R ? *reinterpret_cast<const bf16x8*>(qa_row + d) : *reinterpret_cast<const bf16x8*>(qr_row + d - a.R);
        }
    }
    f32x4 acc[RC];
#pragma unroll
    for (int c = 0; c < RC; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = kLatNoMax, l = 0.f;

    // staging: thread -> key tid % 32, 16-byte chunks tid / 32 + 8 i of its row
    const int skey = tid & 31, schunk = tid >> 5;
    const int chunks = D / 8;
    constexpr int SC = (DC * 4 + 7) / 8;
    u32x4 stage[SC];
    auto fetch = [&](int b) {
        const int key = b * 32 + skey;
        const bool ok = key >= wg_lo && key <= wg_hi;
        const bf16* src = a.cache;
        if (ok) src += (static_cast<size_t>(table[key / a.page]) * a.page + key % a.page) * D;
#pragma unroll
        for (int i = 0; i < SC; ++i) {
            const int c8 = schunk + 8 * i;
            stage[i] = (ok && c8 < chunks) ? *reinterpret_cast<const u32x4*>(src + c8 * 8) : u32x4{0u, 0u, 0u, 0u};
        }
    };
    auto put = [&]() {
#pragma unroll
        for (int i = 0; i < SC; ++i) {
            const int c8 = schunk + 8 * i;
            if (c8 >= chunks) continue;
            *reinterpret_cast<u32x4*>(Ks + skey * ks + c8 * 8) = stage[i];
            if (c8 * 8 < a.R) {
                const bf16x8 v = __builtin_bit_cast(bf16x8, stage[i]);
#pragma unroll
                for (int e = 0; e < 8; ++e) Vt[(c8 * 8 + e) * kVtStride + skey] = v[e];
            }
        }
    };

    if (b_begin < b_end) fetch(b_begin);
    for (int b = b_begin; b < b_end; ++b) {
        __syncthreads();                    // everybody has read the block before
        put();
        __syncthreads();
        if (b + 1 < b_end) fetch(b + 1);    // on its way while this block is computed
        // scores
        f32x4 sc[2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            sc[hf] = f32x4{0.f, 0.f, 0.f, 0.f};
            const bf16* krow = Ks + (hf * 16 + r16) * ks + g * 8;
#pragma unroll
            for (int c = 0; c < DC; ++c)
                if (c < dc)
                    sc[hf] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(krow + c * 32), qf[c],
                                                                     sc[hf], 0, 0, 0);
        }
        // weights of this lane's row for keys 32 b + 16 hf + 4 g + e
        float bm = kLatNoMax;
        bool vis[2][4];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int key = b * 32 + hf * 16 + g * 4 + e;
                vis[hf][e] = key >= row_lo && key <= row_hi;
                sc[hf][e] = vis[hf][e] ? sc[hf][e] * a.scale_log2 : kLatNoMax;
                bm = fmaxf(bm, sc[hf][e]);
            }
        bm = fmaxf(bm, __shfl_xor(bm, 16, 64));
        bm = fmaxf(bm, __shfl_xor(bm, 32, 64));
        const float m_new = fmaxf(m, bm);
        const float alpha = __builtin_amdgcn_exp2f(m - m_new);         // 1 where nothing moved; 0 or 1 for a row without keys so far
        m = m_new;
        float psum = 0.f;
        bf16x8 pf;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float pv = vis[hf][e] ? __builtin_amdgcn_exp2f(sc[hf][e] - m_new) : 0.f;
                const __bf16 pb = static_cast<__bf16>(pv);
                pf[hf * 4 + e] = pb;
                psum += static_cast<float>(pb);
            }
        l = l * alpha + psum;
        if (__any(alpha != 1.0f)) {
            float f[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) f[i] = __shfl(alpha, g * 4 + i, 64);      // rows 4 g + i of the accumulators
#pragma unroll
            for (int c = 0; c < RC; ++c)
                if (c < rc)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[c][i] *= f[i];
        }
        // weighted sum: second operand = transposed latent entries 16 c + r16, keys 4 g .. of both halves
#pragma unroll
        for (int c = 0; c < RC; ++c)
            if (c < rc) {
                const bf16* vrow = Vt + (c * 16 + r16) * kVtStride + g * 4;
                const bf16x4 lo4 = *reinterpret_cast<const bf16x4*>(vrow), hi4 = *reinterpret_cast<const bf16x4*>(vrow + 16);
                const bf16x8 vf = __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
                acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, acc[c], 0, 0, 0);
            }
    }
    // a row's sum over the four lanes that hold its keys
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    // the accumulators' rows are 4 g + i: their places and statistics come from the lanes that own those rows
    const long my_out = static_cast<long>(tok) * a.o_ts + static_cast<long>(h) * a.o_hs;
    const long my_pair = static_cast<long>(h) * a.T + tok;           // place in the workspace
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int src = g * 4 + i;
        const bool ok = __shfl(row_ok ? 1 : 0, src, 64) != 0;
        const float li = __shfl(l, src, 64), mi = __shfl(m, src, 64);
        const long oo = __shfl(static_cast<int>(my_out), src, 64);   // (pairs * strides stay below 2^31: checked by the entry point)
        const long pp = __shfl(static_cast<int>(my_pair), src, 64);
        if (!ok) continue;
        if (a.nsplit == 1) {
            const float inv = 1.0f / li;
#pragma unroll
            for (int c = 0; c < RC; ++c)
                if (c < rc) a.out[oo * a.R + c * 16 + r16] = static_cast<bf16>(acc[c][i] * inv);
        } else {
            const size_t at = static_cast<size_t>(z) * a.n * a.T + pp;
#pragma unroll
            for (int c = 0; c < RC; ++c)
                if (c < rc) a.ws_o[at * a.R + c * 16 + r16] = acc[c][i];
            if (r16 == 0) {
                a.ws_ml[at * 2] = mi;
                a.ws_ml[at * 2 + 1] = li;
            }
        }
    }
}

// out[pair] = sum_z 2^(m_z - M) O_z / sum_z 2^(m_z - M) l_z, z in order. One workgroup of 256 threads a pair: the first
// wavefront turns the runs' statistics into one factor per run (a lane a run, up to 64 runs), then every thread adds its
// entries of the runs' sums, eight loads asked for at a time.
__global__ __launch_bounds__(256) void latent_join_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                          bf16* __restrict__ out, int T, int n, int R, int nsplit, long o_ts,
                                                          long o_hs) {
    __shared__ float factor[64];
    const int tok = blockIdx.x, h = blockIdx.y;
    const size_t pairs = static_cast<size_t>(n) * T, pair = static_cast<size_t>(h) * T + tok;
    if (threadIdx.x < 64) {
        const int z = threadIdx.x;
        const float mz = z < nsplit ? ws_ml[(z * pairs + pair) * 2] : kLatNoMax;
        const float lz = z < nsplit ? ws_ml[(z * pairs + pair) * 2 + 1] : 0.f;
        const float M = wave_max(mz);
        const float f = __builtin_amdgcn_exp2f(mz - M);
        // (the sum over the runs in the order of the runs: lane 0 adds them up)
        float L = 0.f;
        for (int i = 0; i < nsplit; ++i) L += __shfl(f * lz, i, 64);
        factor[z] = f / L;
    }
    __syncthreads();
    bf16* o = out + (static_cast<long>(tok) * o_ts + static_cast<long>(h) * o_hs) * R;
    for (int c = threadIdx.x; c < R; c += 256) {
        const float* src = ws_o + pair * R + c;
        float sum = 0.f;
        int z = 0;
        for (; z + 8 <= nsplit; z += 8) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = src[static_cast<size_t>(z + e) * pairs * R];
#pragma unroll
            for (int e = 0; e < 8; ++e) sum = fmaf(factor[z + e], v[e], sum);
        }
        for (; z < nsplit; ++z) sum = fmaf(factor[z], src[static_cast<size_t>(z) * pairs * R], sum);
        o[c] = static_cast<bf16>(sum);
    }
}

// q [T, n (d + r)] -> qn [n, T, d] (the unrotated entries as they are) and qr [n, T, r] (the rotated ones: the first rd of
// them turned by position * freq, pairs of neighbours, cos and sin times mag).
__global__ void latent_q_split_kernel(const bf16* __restrict__ q, const float* __restrict__ freq, float mag,
                                      const int* __restrict__ positions, bf16* __restrict__ qn, bf16* __restrict__ qr, int T,
                                      int n, int d, int r, int rd, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;      // (t, head, pair of entries)
    if (idx >= total) return;
    const int half = (d + r) / 2;
    const int i = static_cast<int>(idx % half);
    const size_t th = idx / half;
    const int t = static_cast<int>(th / n), h = static_cast<int>(th % n);
    const bf16* src = q + th * (d + r) + 2 * i;
    if (2 * i < d) {
        bf16* dst = qn + (static_cast<size_t>(h) * T + t) * d + 2 * i;
        dst[0] = src[0];
        dst[1] = src[1];
        return;
    }
    const int j = i - d / 2;
    float sn = 0.f, cs = 1.f;
    if (2 * j < rd) {
        sincosf(static_cast<float>(positions[t]) * freq[j], &sn, &cs);
        sn *= mag;
        cs *= mag;
    }
    const float u = static_cast<float>(src[0]), v = static_cast<float>(src[1]);
    bf16* dst = qr + (static_cast<size_t>(h) * T + t) * r + 2 * j;
    dst[0] = static_cast<bf16>(u * cs - v * sn);
    dst[1] = static_cast<bf16>(v * cs + u * sn);
}

// o [n, T, c] -> out [T, n c]
__global__ void heads_to_rows_kernel(const bf16* __restrict__ o, bf16* __restrict__ out, int T, int n, int c, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int e = static_cast<int>(idx % c);
    const size_t th = idx / c;
    const int h = static_cast<int>(th % n), t = static_cast<int>(th / n);
    out[idx] = o[(static_cast<size_t>(h) * T + t) * c + e];
}

template <int DC, int RC>
static int launch_latent(const LatentArgs& a, int max_new, int n_seq, hipStream_t stream) {
    const int D = a.R + a.r;
    const int lds = (32 * lat_k_stride(D) + a.R * kVtStride) * 2;
    static int attr_lds = 0;
    if (lds > attr_lds) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attention_mfma_kernel<DC, RC>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return static_cast<int>(e);
        attr_lds = lds;
    }
    const dim3 grid((static_cast<long>(max_new) * a.n + 63) / 64, n_seq, a.nsplit);
    hipLaunchKernelGGL((latent_attention_mfma_kernel<DC, RC>), grid, dim3(256), lds, stream, a);
    return launch_status();
}

}  // namespace llme

using namespace llme;

// max_new: the most tokens a request brings in this step. ws_o / ws_ml: nsplit > 1 only.
extern "C" int llme_latent_attention_mfma(const void* qa, const void* qr, const void* cache, void* out, float* ws_o,
                                          float* ws_ml, const int* positions, const int* q_start, const int* block_table,
                                          int max_blocks, int T, int n_seq, int max_new, int n, int R, int r, int page,
                                          float scale, int window, int nsplit, long q_ts, long q_hs, long o_ts, long o_hs,
                                          hipStream_t stream) {
    if (T <= 0 || n_seq <= 0) return 0;
    const int D = R + r;
    if (n <= 0 || R <= 0 || r < 0 || max_new <= 0 || nsplit <= 0 || nsplit > 64 || n_seq > 65535) return kErrBadArgument;
    if (R % 16 || D % 32 || r % 8 || page % 16 || D > 576 || R > 512) return kErrUnsupported;
    if (static_cast<long>(T) * n * (R > 2 ? R : 2) >= (1l << 31)) return kErrUnsupported;
    if (nsplit > 1 && (ws_o == nullptr || ws_ml == nullptr)) return kErrBadArgument;
    LatentArgs a{static_cast<const bf16*>(qa), static_cast<const bf16*>(qr), static_cast<const bf16*>(cache),
                 static_cast<bf16*>(out), ws_o, ws_ml, positions, q_start, block_table, max_blocks, T, n, R, r, page, window,
                 nsplit, q_ts, q_hs, o_ts, o_hs, scale * 1.4426950408889634f};
    int rc;
    if (D <= 128 && R <= 128) rc = launch_latent<4, 8>(a, max_new, n_seq, stream);
    else if (D <= 320 && R <= 256) rc = launch_latent<10, 16>(a, max_new, n_seq, stream);
    else rc = launch_latent<18, 32>(a, max_new, n_seq, stream);
    if (rc != 0 || nsplit == 1) return rc;
    hipLaunchKernelGGL(latent_join_kernel, dim3(T, n), dim3(256), 0, stream, ws_o, ws_ml, static_cast<bf16*>(out), T, n, R, nsplit,
                       o_ts, o_hs);
    return launch_status();
}

extern "C" int llme_latent_q_split(const void* q, const float* freq, float mag, const int* positions, void* qn, void* qr,
                                   int T, int n, int d, int r, int rd, hipStream_t stream) {
    if (T <= 0) return 0;
    if (d % 2 || r % 2 || rd % 2 || rd > r || (rd > 0 && freq == nullptr)) return kErrBadArgument;
    const size_t total = static_cast<size_t>(T) * n * ((d + r) / 2);
    hipLaunchKernelGGL(latent_q_split_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const bf16*>(q), freq, mag, positions, static_cast<bf16*>(qn), static_cast<bf16*>(qr), T, n, d,
                       r, rd, total);
    return launch_status();
}

extern "C" int llme_heads_to_rows(const void* o, void* out, int T, int n, int c, hipStream_t stream) {
    if (T <= 0) return 0;
    const size_t total = static_cast<size_t>(T) * n * c;
    hipLaunchKernelGGL(heads_to_rows_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const bf16*>(o), static_cast<bf16*>(out), T, n, c, total);
    return launch_status();
}

LLME_LOAD_ENTRY(latent_attention_mfma)
