// Attention without a softmax over paged keys and values, with the heads' scores mixed before the
// weights are made ("talking heads"):
//
//   s[h, j]  = scale * q_h . k_(h / (H / G)), j          for every key j <= the row's position
//   s'[h, j] = sum_g mix[h, g] s[g, j]
//   w[h, j]  = sigmoid(s'[h, j] + bias[h])               (nothing is normalised over j)
//   o_h      = sum_j w[h, j] v_(h / (H / G)), j
//
// Scores, their mixing, the weights and the sums over keys are 32-bit; q, k and v are read in their
// storage type. Since nothing is normalised, a row's keys may be cut into runs whose partial sums add
// up: the first kernel writes one partial per run, the second adds them in a fixed order, multiplies
// head h by scale_out * sigmoid(gate[t, h]) and stores the activation type.
//
// Also here: the rotation of q and k by angles computed from the position (no table, so no longest
// position) and the write of k and v into pages whose key and value sizes differ.
#include "common.h"

namespace llme {

// q, k heads of qkvg [T, ld] (32-bit; q at column 0, k behind the q heads, v behind the k heads): entry i < rot / 2
// of a head turns with entry i + rot / 2 by the angle position * inv_freq[i] (a 32-bit product); q goes to q_out
// [T, H * dim], k and v into the row's page: k_cache [pages, G, page, dim], v_cache [pages, G, page, vdim].
template <typename TQ, typename TC>
__global__ __launch_bounds__(256) void rotate_write_kernel(const float* __restrict__ qkv, int ld, const float* __restrict__ inv_freq,
                                                           const int* __restrict__ positions, const int* __restrict__ seq_idx,
                                                           const int* __restrict__ block_table, int max_blocks,
                                                           TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                                           int H, int G, int dim, int vdim, int rot, int page) {
    const int t = blockIdx.x;
    const int pos = positions[t];
    const int half = rot / 2;
    const float* row = qkv + static_cast<size_t>(t) * ld;
    const int pg = block_table[static_cast<size_t>(seq_idx[t]) * max_blocks + pos / page];
    const int in_page = pos % page;
    const float fpos = static_cast<float>(pos);
    // q and k heads: H + G heads of dim entries
    for (int e = threadIdx.x; e < (H + G) * dim; e += 256) {
        const int head = e / dim, i = e % dim;
        const float* hp = row + static_cast<size_t>(head) * dim;
        float v = hp[i];
        if (i < rot) {
            const int f = i < half ? i : i - half;
            float sn, cs;
            sincosf(fpos * inv_freq[f], &sn, &cs);
            v = i < half ? hp[i] * cs - hp[i + half] * sn : hp[i] * cs + hp[i - half] * sn;
        }
        if (head < H)
            q_out[static_cast<size_t>(t) * H * dim + e] = from_float<TQ>(v);
        else
            k_cache[((static_cast<size_t>(pg) * G + (head - H)) * page + in_page) * dim + i] = from_float<TC>(v);
    }
    const float* vp = row + static_cast<size_t>(H + G) * dim;
    for (int e = threadIdx.x; e < G * vdim; e += 256) {
        const int head = e / vdim, i = e % vdim;
        v_cache[((static_cast<size_t>(pg) * G + head) * page + in_page) * vdim + i] = from_float<TC>(vp[e]);
    }
}

constexpr int kKeysPerTile = 32;

// One workgroup per (row, run of keys). Dynamic LDS: q [H dim], mix [H H], bias [H], scores [H KT], weights [H KT].
// NACC accumulators per thread cover the row's H * vdim outputs (element tid + 256 i).
template <typename TQ, typename TC, int NACC>
__global__ __launch_bounds__(256) void sigmoid_attention_kernel(const TQ* __restrict__ q, const TC* __restrict__ k_cache,
                                                                const TC* __restrict__ v_cache, const float* __restrict__ mix,
                                                                const float* __restrict__ bias, const int* __restrict__ positions,
                                                                const int* __restrict__ seq_idx, const int* __restrict__ block_table,
                                                                int max_blocks, float* __restrict__ partial, int T, int H, int G,
                                                                int dim, int vdim, int page, float scale, int run_len) {
    extern __shared__ float lds[];
    constexpr int KT = kKeysPerTile;
    float* qs = lds;
    float* ms = qs + H * dim;
    float* bs = ms + H * H;
    float* sc = bs + H;
    float* wt = sc + H * KT;
    const int t = blockIdx.x, run = blockIdx.y;
    const int tid = threadIdx.x;
    const int pos = positions[t];
    const int key0 = run * run_len;
    const int key1 = min(pos + 1, key0 + run_len);
    float acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    float* out = partial + (static_cast<size_t>(run) * T + t) * H * vdim;
    if (key0 < key1) {
        const int* table = block_table + static_cast<size_t>(seq_idx[t]) * max_blocks;
        for (int e = tid; e < H * dim; e += 256) qs[e] = to_float(q[static_cast<size_t>(t) * H * dim + e]);
        for (int e = tid; e < H * H; e += 256) ms[e] = mix[e];
        for (int e = tid; e < H; e += 256) bs[e] = bias[e];
        __syncthreads();
        const int per = H / G;
        for (int j0 = key0; j0 < key1; j0 += KT) {
            const int nk = min(KT, key1 - j0);
            // scores of every head for the tile's keys
            for (int e = tid; e < H * KT; e += 256) {
                const int h = e / KT, j = e % KT;
                float s = 0.f;
                if (j < nk) {
                    const int key = j0 + j;
                    const TC* kp = k_cache + ((static_cast<size_t>(table[key / page]) * G + h / per) * page + key % page) * dim;
                    const float* qp = qs + h * dim;
                    for (int d = 0; d < dim; ++d) s += qp[d] * to_float(kp[d]);
                }
                sc[e] = s * scale;
            }
            __syncthreads();
            // mixed over the heads, then the weight
            for (int e = tid; e < H * KT; e += 256) {
                const int h = e / KT, j = e % KT;
                float m = 0.f;
                for (int g = 0; g < H; ++g) m += ms[h * H + g] * sc[g * KT + j];
                wt[e] = j < nk ? 1.0f / (1.0f + expf(-(m + bs[h]))) : 0.f;
            }
            __syncthreads();
            // weighted values
#pragma unroll
            for (int i = 0; i < NACC; ++i) {
                const int e = tid + 256 * i;
                if (e < H * vdim) {
                    const int h = e / vdim, x = e % vdim;
                    const float* wp = wt + h * KT;
                    float a = acc[i];
                    for (int j = 0; j < nk; ++j) {
                        const int key = j0 + j;
                        a += wp[j] * to_float(v_cache[((static_cast<size_t>(table[key / page]) * G + h / per) * page + key % page) * vdim + x]);
                    }
                    acc[i] = a;
                }
            }
            __syncthreads();
        }
    }
#pragma unroll
    for (int i = 0; i < NACC; ++i) {
        const int e = tid + 256 * i;
        if (e < H * vdim) out[e] = acc[i];
    }
}

// out[t, h, :] = scale_out * sigmoid(gate[t, h]) * sum_runs partial[run, t, h, :]
template <typename TO>
__global__ __launch_bounds__(256) void sigmoid_attention_finish_kernel(const float* __restrict__ partial, int runs,
                                                                       const float* __restrict__ gate, int ld_gate,
                                                                       TO* __restrict__ out, int ld_out, int T, int H, int vdim,
                                                                       float scale_out) {
    const int t = blockIdx.x;
    const size_t per_run = static_cast<size_t>(T) * H * vdim;
    for (int e = threadIdx.x; e < H * vdim; e += 256) {
        float a = 0.f;
        for (int r = 0; r < runs; ++r) a += partial[r * per_run + static_cast<size_t>(t) * H * vdim + e];
        const float g = 1.0f / (1.0f + expf(-gate[static_cast<size_t>(t) * ld_gate + e / vdim]));
        out[static_cast<size_t>(t) * ld_out + e] = from_float<TO>(scale_out * (g * a));
    }
}

template <typename TQ, typename TC>
static int launch_sigmoid_attention(const void* q, const void* k_cache, const void* v_cache, const float* mix, const float* bias,
                                    const int* positions, const int* seq_idx, const int* block_table, int max_blocks,
                                    float* partial, int T, int H, int G, int dim, int vdim, int page, float scale, int run_len,
                                    int runs, hipStream_t stream) {
    const size_t lds = sizeof(float) * (static_cast<size_t>(H) * dim + static_cast<size_t>(H) * H + H + 2 * static_cast<size_t>(H) * kKeysPerTile);
    if (lds > 64 * 1024) return kErrUnsupported;
    const int outs = H * vdim;
    const dim3 grid(T, runs);
#define LLME_SA(N_)                                                                                                      \
    sigmoid_attention_kernel<TQ, TC, N_><<<grid, 256, lds, stream>>>(                                                    \
        static_cast<const TQ*>(q), static_cast<const TC*>(k_cache), static_cast<const TC*>(v_cache), mix, bias, positions, \
        seq_idx, block_table, max_blocks, partial, T, H, G, dim, vdim, page, scale, run_len)
    if (outs <= 256 * 2) LLME_SA(2);
    else if (outs <= 256 * 4) LLME_SA(4);
    else if (outs <= 256 * 8) LLME_SA(8);
    else if (outs <= 256 * 16) LLME_SA(16);
    else if (outs <= 256 * 32) LLME_SA(32);
    else return kErrUnsupported;
#undef LLME_SA
    return launch_status();
}

}  // namespace llme

using namespace llme;

extern "C" int llme_rotate_write(const void* qkv, int ld, const void* inv_freq, const void* positions, const void* seq_idx,
                                 const void* block_table, int max_blocks, void* q_out, int q_dtype, void* k_cache, void* v_cache,
                                 int c_dtype, int T, int H, int G, int dim, int vdim, int rot, int page, hipStream_t stream) {
    if (T <= 0) return 0;
    if (rot < 0 || rot > dim || rot % 2 || G <= 0 || H % G || page <= 0) return kErrBadArgument;
#define LLME_RW(TQ_, TC_)                                                                                                \
    rotate_write_kernel<TQ_, TC_><<<T, 256, 0, stream>>>(                                                                \
        static_cast<const float*>(qkv), ld, static_cast<const float*>(inv_freq), static_cast<const int*>(positions),    \
        static_cast<const int*>(seq_idx), static_cast<const int*>(block_table), max_blocks, static_cast<TQ_*>(q_out),   \
        static_cast<TC_*>(k_cache), static_cast<TC_*>(v_cache), H, G, dim, vdim, rot, page)
    switch (q_dtype * 2 + c_dtype) {
        case 0: LLME_RW(float, float); break;
        case 1: LLME_RW(float, bf16); break;
        case 2: LLME_RW(bf16, float); break;
        case 3: LLME_RW(bf16, bf16); break;
        default: return kErrBadArgument;
    }
#undef LLME_RW
    return launch_status();
}

// partial [runs, T, H, vdim] 32-bit scratch; run r of a row holds its keys r run_len .. (r + 1) run_len - 1.
extern "C" int llme_sigmoid_attention(const void* q, int q_dtype, const void* k_cache, const void* v_cache, int c_dtype,
                                      const void* mix, const void* bias, const void* positions, const void* seq_idx,
                                      const void* block_table, int max_blocks, void* partial, int T, int H, int G, int dim,
                                      int vdim, int page, float scale, int run_len, int runs, hipStream_t stream) {
    if (T <= 0) return 0;
    if (G <= 0 || H % G || run_len <= 0 || runs <= 0 || page <= 0) return kErrBadArgument;
    const float* mp = static_cast<const float*>(mix);
    const float* bp = static_cast<const float*>(bias);
    const int* pp = static_cast<const int*>(positions);
    const int* sp = static_cast<const int*>(seq_idx);
    const int* tp = static_cast<const int*>(block_table);
    float* part = static_cast<float*>(partial);
    switch (q_dtype * 2 + c_dtype) {
        case 0: return launch_sigmoid_attention<float, float>(q, k_cache, v_cache, mp, bp, pp, sp, tp, max_blocks, part, T, H, G,
                                                              dim, vdim, page, scale, run_len, runs, stream);
        case 3: return launch_sigmoid_attention<bf16, bf16>(q, k_cache, v_cache, mp, bp, pp, sp, tp, max_blocks, part, T, H, G,
                                                            dim, vdim, page, scale, run_len, runs, stream);
    }
    return kErrUnsupported;
}

extern "C" int llme_sigmoid_attention_finish(const void* partial, int runs, const void* gate, int ld_gate, void* out, int out_dtype,
                                             int ld_out, int T, int H, int vdim, float scale_out, hipStream_t stream) {
    if (T <= 0) return 0;
    if (out_dtype == kF32)
        sigmoid_attention_finish_kernel<float><<<T, 256, 0, stream>>>(static_cast<const float*>(partial), runs,
                                                                      static_cast<const float*>(gate), ld_gate,
                                                                      static_cast<float*>(out), ld_out, T, H, vdim, scale_out);
    else if (out_dtype == kBF16)
        sigmoid_attention_finish_kernel<bf16><<<T, 256, 0, stream>>>(static_cast<const float*>(partial), runs,
                                                                     static_cast<const float*>(gate), ld_gate,
                                                                     static_cast<bf16*>(out), ld_out, T, H, vdim, scale_out);
    else
        return kErrBadArgument;
    return launch_status();
}

LLME_LOAD_ENTRY(sigmoid_attention)
