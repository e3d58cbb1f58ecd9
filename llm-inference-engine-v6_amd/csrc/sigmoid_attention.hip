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
// [T, H * dim], k and v into the row's page: k_cache [pages, G, page, dim], v_cache [pages, G, vdim, page] (a value
// channel's tokens lie together, as the matrix instructions of the second product read them).
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
        v_cache[((static_cast<size_t>(pg) * G + head) * vdim + i) * page + in_page] = from_float<TC>(vp[e]);
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
                        a += wp[j] * to_float(v_cache[((static_cast<size_t>(table[key / page]) * G + h / per) * vdim + x) * page + key % page]);
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

// Eight neighbouring values of a row of keys, queries or values, widened to 32-bit, in one or two loads.
template <typename T> __device__ __forceinline__ void load8(const T* p, float (&v)[8]);
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <> __device__ __forceinline__ void load8<bf16>(const bf16* p, float (&v)[8]) {
    typedef __attribute__((ext_vector_type(8))) __bf16 v8;
    const v8 x = *reinterpret_cast<const v8*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = static_cast<float>(x[i]);
}

// For rows that come one or a few to a request (decoding): one workgroup per (row, run of keys) as in the plain kernel,
// but every thread reads whole lines. Per tile of 64 keys: (1) a thread takes a (key/value head, key) pair, reads the key's
// row 16 bytes at a time and makes the scores of all query heads of that group against q in LDS; (2) a thread mixes the
// heads' scores of eight (head, key) pairs and makes the weights; (3) a thread takes a (key/value head, value channel)
// pair, reads its 64 tokens (contiguous in a page) and adds the group's heads' weighted values. dim and the page size are
// multiples of 8, a group has at most PER query heads, G * 64 <= 256 NP and G * vdim <= 256 NP.
template <typename TQ, typename TC, int PER, int NP>
__global__ __launch_bounds__(256) void sigmoid_attention_rows_kernel(const TQ* __restrict__ q, const TC* __restrict__ k_cache,
                                                                     const TC* __restrict__ v_cache, const float* __restrict__ mix,
                                                                     const float* __restrict__ bias, const int* __restrict__ positions,
                                                                     const int* __restrict__ seq_idx, const int* __restrict__ block_table,
                                                                     int max_blocks, float* __restrict__ partial, int T, int H, int G,
                                                                     int dim, int vdim, int page, float scale, int run_len) {
    extern __shared__ float lds[];
    constexpr int KT = 64;
    float* qs = lds;                    // [H][dim]
    float* ms = qs + H * dim;           // [H][H]
    float* bs = ms + H * H;             // [H]
    float* sc = bs + H;                 // [H][KT + 1]
    float* wt = sc + H * (KT + 1);      // [H][KT]
    const int t = blockIdx.x, run = blockIdx.y, tid = threadIdx.x;
    const int pos = positions[t];
    const int key0 = run * run_len, key1 = min(pos + 1, key0 + run_len);
    const int per = H / G;
    float acc[NP][PER];
#pragma unroll
    for (int i = 0; i < NP; ++i)
#pragma unroll
        for (int u = 0; u < PER; ++u) acc[i][u] = 0.f;
    if (key0 < key1) {
        const int* table = block_table + static_cast<size_t>(seq_idx[t]) * max_blocks;
        for (int e = tid; e < H * dim; e += 256) qs[e] = to_float(q[static_cast<size_t>(t) * H * dim + e]);
        for (int e = tid; e < H * H; e += 256) ms[e] = mix[e];
        for (int e = tid; e < H; e += 256) bs[e] = bias[e];
        __syncthreads();
        for (int j0 = key0; j0 < key1; j0 += KT) {
            const int nk = min(KT, key1 - j0);
            // (1) scores: pair = (kv, key)
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int pair = tid + 256 * i;
                const int kv = pair / KT, j = pair % KT;
                if (kv >= G) break;
                float s[PER];
#pragma unroll
                for (int u = 0; u < PER; ++u) s[u] = 0.f;
                if (j < nk) {
                    const int key = j0 + j;
                    const TC* kp = k_cache + ((static_cast<size_t>(table[key / page]) * G + kv) * page + key % page) * dim;
                    for (int d = 0; d < dim; d += 8) {
                        float kk[8];
                        load8<TC>(kp + d, kk);
#pragma unroll
                        for (int u = 0; u < PER; ++u) {
                            if (u >= per) break;
                            const float* qp = qs + (kv * per + u) * dim + d;
#pragma unroll
                            for (int e = 0; e < 8; ++e) s[u] += qp[e] * kk[e];
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < PER; ++u)
                    if (u < per) sc[(kv * per + u) * (KT + 1) + j] = s[u] * scale;
            }
            __syncthreads();
            // (2) mixed over the heads, then the weight
            for (int e = tid; e < H * KT; e += 256) {
                const int h = e / KT, j = e % KT;
                float m = 0.f;
                for (int g = 0; g < H; ++g) m += ms[h * H + g] * sc[g * (KT + 1) + j];
                wt[e] = j < nk ? 1.0f / (1.0f + expf(-(m + bs[h]))) : 0.f;
            }
            __syncthreads();
            // (3) weighted values: pair = (kv, value channel), the tile's keys eight at a time
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const int pair = tid + 256 * i;
                const int kv = pair / vdim, x = pair % vdim;
                if (kv >= G) break;
                for (int c = 0; c < nk; c += 8) {
                    const int key = j0 + c;
                    float vv[8];
                    load8<TC>(v_cache + ((static_cast<size_t>(table[key / page]) * G + kv) * vdim + x) * page + key % page, vv);
#pragma unroll
                    for (int u = 0; u < PER; ++u) {
                        if (u >= per) break;
                        const float* wp = wt + (kv * per + u) * KT + c;
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc[i][u] += wp[e] * vv[e];
                    }
                }
            }
            __syncthreads();
        }
    }
    float* out = partial + (static_cast<size_t>(run) * T + t) * H * vdim;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int pair = tid + 256 * i;
        const int kv = pair / vdim, x = pair % vdim;
        if (kv >= G) break;
#pragma unroll
        for (int u = 0; u < PER; ++u)
            if (u < per) out[(kv * per + u) * vdim + x] = acc[i][u];
    }
}

// The same on the matrix cores, for bfloat16 rows that come at least 16 to a request (prompts and their portions).
// A workgroup owns 16 consecutive rows of one request and one run of its keys; each of its H / 4 wavefronts owns four
// heads. Per tile of 32 keys: (1) every wavefront makes the transposed scores K Q^T of its heads (so that a lane holds,
// for one query, the keys that the second product wants from it) and puts them, scaled, into LDS; (2) it mixes all
// heads' scores into its own heads' (32-bit FMAs against the mixing matrix, broadcast from LDS), makes the weights,
// splits each into two bfloat16 parts (w = hi + lo, 16 bits of mantissa) and adds both parts' products with V.
// Weights of keys behind a row's position are zero. Partial sums go where the finishing kernel adds the runs.
typedef __attribute__((ext_vector_type(8))) __bf16 sa_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 sa_bf16x4;
typedef __attribute__((ext_vector_type(4))) float sa_f32x4;

template <int DIM32, int VT>
__global__ __launch_bounds__(512) void sigmoid_attention_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const float* __restrict__ mix_t, const float* __restrict__ bias, const int* __restrict__ positions,
    const int* __restrict__ q_start, const int* __restrict__ block_table, int max_blocks, float* __restrict__ partial,
    int T, int n_seq, int H, int G, int page, float scale, int run_len) {
    constexpr int DIM = DIM32 * 32, VDIM = VT * 16, HPW = 4;
    extern __shared__ float lds[];
    float* sc = lds;                        // [H][64 lanes][8]
    float* mt = sc + H * 512;               // [H (from)][H (to)]
    float* bs = mt + H * H;
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int r16 = lane % 16, q4 = lane / 16;
    // which request and which 16 of its rows
    int item = gridDim.x - 1 - blockIdx.x, s = 0, row0 = 0, nrows = 0;       // (later rows have more keys: they start first)
    for (; s < n_seq; ++s) {
        const int n = q_start[s + 1] - q_start[s];
        const int tiles = (n + 15) / 16;
        if (item < tiles) {
            row0 = q_start[s] + item * 16;
            nrows = min(16, q_start[s + 1] - row0);
            break;
        }
        item -= tiles;
    }
    if (s >= n_seq) return;
    const int run = blockIdx.y;
    const int* table = block_table + static_cast<size_t>(s) * max_blocks;
    const int my_row = row0 + min(r16, nrows - 1);
    const int my_pos = positions[my_row];
    const int kmax = positions[row0 + nrows - 1];
    const int key_lo = run * run_len, key_hi = min(kmax + 1, key_lo + run_len);
    for (int e = threadIdx.x; e < H * H; e += blockDim.x) mt[e] = mix_t[e];
    for (int e = threadIdx.x; e < H; e += blockDim.x) bs[e] = bias[e];
    const int h0 = wave * HPW, per = H / G;
    sa_bf16x8 qf[HPW][DIM32];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int c = 0; c < DIM32; ++c)
            qf[hh][c] = *reinterpret_cast<const sa_bf16x8*>(q + (static_cast<size_t>(my_row) * H + h0 + hh) * DIM + c * 32 + q4 * 8);
    sa_f32x4 o[HPW][VT];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int dt = 0; dt < VT; ++dt) o[hh][dt] = sa_f32x4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    // The wavefront's four heads read one key/value head where the query heads come four or more to one (ONE_KV): its
    // keys for the next tile are then asked for as soon as this tile's scores are made, and its values ahead of the scores.
    const bool one_kv = (h0 / per) == ((h0 + HPW - 1) / per);
    sa_bf16x8 kf[2][DIM32], vf[VT];
    auto load_k = [&](int j, int kv) {
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const int key = min(j + rt * 16 + r16, kmax);
            const bf16* kp = k_cache + ((static_cast<size_t>(table[key / page]) * G + kv) * page + key % page) * DIM;
#pragma unroll
            for (int c = 0; c < DIM32; ++c) kf[rt][c] = *reinterpret_cast<const sa_bf16x8*>(kp + c * 32 + q4 * 8);
        }
    };
    auto load_v = [&](int j, int kv) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int key = min(j + half * 16 + 4 * q4, kmax & ~3);
            const bf16* vp = v_cache + (static_cast<size_t>(table[key / page]) * G + kv) * VDIM * page + key % page;
#pragma unroll
            for (int dt = 0; dt < VT; ++dt) {
                const sa_bf16x4 v4 = *reinterpret_cast<const sa_bf16x4*>(vp + static_cast<size_t>(dt * 16 + r16) * page);
#pragma unroll
                for (int e = 0; e < 4; ++e) vf[dt][half * 4 + e] = v4[e];
            }
        }
    };
    if (one_kv && key_lo < key_hi) load_k(key_lo, h0 / per);
    for (int j0 = key_lo; j0 < key_hi; j0 += 32) {
        // (1) transposed scores of this wavefront's heads
        {
            int have = one_kv ? h0 / per : -1;
            if (one_kv) load_v(j0, h0 / per);
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) {
                const int g = h0 + hh, kv = g / per;
                if (kv != have) {
                    load_k(j0, kv);
                    have = kv;
                }
                sa_f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < DIM32; ++c) {
                    a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[0][c], qf[hh][c], a0, 0, 0, 0);
                    a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[1][c], qf[hh][c], a1, 0, 0, 0);
                }
                float* dst = sc + (static_cast<size_t>(g) * 64 + lane) * 8;
                *reinterpret_cast<float4*>(dst) = float4{a0[0] * scale, a0[1] * scale, a0[2] * scale, a0[3] * scale};
                *reinterpret_cast<float4*>(dst + 4) = float4{a1[0] * scale, a1[1] * scale, a1[2] * scale, a1[3] * scale};
            }
            if (one_kv && j0 + 32 < key_hi) load_k(j0 + 32, h0 / per);
        }
        __syncthreads();
        // (2) all heads' scores mixed into this wavefront's heads
        float m[HPW][8];
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
            for (int e = 0; e < 8; ++e) m[hh][e] = 0.f;
        for (int g = 0; g < H; ++g) {
            const float4 s0 = *reinterpret_cast<const float4*>(sc + (static_cast<size_t>(g) * 64 + lane) * 8);
            const float4 s1 = *reinterpret_cast<const float4*>(sc + (static_cast<size_t>(g) * 64 + lane) * 8 + 4);
            const float4 tw = *reinterpret_cast<const float4*>(mt + g * H + h0);
            const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
            const float tv[4] = {tw.x, tw.y, tw.z, tw.w};
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
                for (int e = 0; e < 8; ++e) m[hh][e] += tv[hh] * sv[e];
        }
        {
            int have = one_kv ? h0 / per : -1;
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) {
                const int h = h0 + hh, kv = h / per;
                const float b = bs[h];
                sa_bf16x8 hi, lo;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = j0 + (e < 4 ? 4 * q4 + e : 16 + 4 * q4 + (e - 4));
                    const float w = (key <= my_pos && key < key_hi) ? 1.0f / (1.0f + expf(-(m[hh][e] + b))) : 0.f;
                    hi[e] = static_cast<__bf16>(w);
                    lo[e] = static_cast<__bf16>(w - static_cast<float>(hi[e]));
                }
                if (kv != have) {
                    load_v(j0, kv);
                    have = kv;
                }
#pragma unroll
                for (int dt = 0; dt < VT; ++dt) {
                    o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, vf[dt], o[hh][dt], 0, 0, 0);
                    o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lo, vf[dt], o[hh][dt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int dt = 0; dt < VT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * q4 + r;
                if (i < nrows)
                    partial[((static_cast<size_t>(run) * T) + row0 + i) * H * VDIM + (h0 + hh) * VDIM + dt * 16 + r16] = o[hh][dt][r];
            }
}

template <int DIM32, int VT>
static int launch_sigmoid_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const float* mix_t,
                                         const float* bias, const int* positions, const int* q_start, const int* block_table,
                                         int max_blocks, float* partial, int T, int n_seq, int H, int G, int page, float scale,
                                         int run_len, int runs, int tiles, hipStream_t stream) {
    const size_t lds = sizeof(float) * (static_cast<size_t>(H) * 512 + static_cast<size_t>(H) * H + H);
    auto kernel = sigmoid_attention_mfma_kernel<DIM32, VT>;
    static size_t allowed = 0;
    if (lds > 64 * 1024 && lds > allowed) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 static_cast<int>(lds));
        if (e != hipSuccess) return static_cast<int>(e);
        allowed = lds;
    }
    kernel<<<dim3(tiles, runs), (H / 4) * 64, lds, stream>>>(
        static_cast<const bf16*>(q), static_cast<const bf16*>(k_cache), static_cast<const bf16*>(v_cache), mix_t, bias, positions,
        q_start, block_table, max_blocks, partial, T, n_seq, H, G, page, scale, run_len);
    return launch_status();
}

// out[t, h, :] = scale_out * sigmoid(gate[t, h]) * sum_runs partial[run, t, h, :]
template <typename TO>
__global__ __launch_bounds__(256) void sigmoid_attention_finish_kernel(const float* __restrict__ partial, int runs,
                                                                       const float* __restrict__ gate, int ld_gate,
                                                                       TO* __restrict__ out, int ld_out, int T, int H, int vdim,
                                                                       float scale_out) {
    const int t = blockIdx.x;
    const size_t per_run = static_cast<size_t>(T) * H * vdim;
    for (int e = blockIdx.y * 256 + threadIdx.x; e < H * vdim; e += gridDim.y * 256) {
        float a = 0.f;
#pragma unroll 8
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
    const dim3 grid(T, runs);
    {
        // the kernel that reads whole lines, where the sizes let it
        const int per = H / G;
        const int np = (G * (64 > vdim ? 64 : vdim) + 255) / 256;
        const size_t lds_rows = sizeof(float) * (static_cast<size_t>(H) * dim + static_cast<size_t>(H) * H + H +
                                                 static_cast<size_t>(H) * 65 + static_cast<size_t>(H) * 64);
        if (dim % 8 == 0 && page % 8 == 0 && per <= 8 && np <= 4 && lds_rows <= 64 * 1024 &&
            reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0) {
#define LLME_SAR(P_, N_)                                                                                                 \
    sigmoid_attention_rows_kernel<TQ, TC, P_, N_><<<grid, 256, lds_rows, stream>>>(                                      \
        static_cast<const TQ*>(q), static_cast<const TC*>(k_cache), static_cast<const TC*>(v_cache), mix, bias, positions, \
        seq_idx, block_table, max_blocks, partial, T, H, G, dim, vdim, page, scale, run_len)
            const int pcode = per <= 1 ? 1 : per <= 2 ? 2 : per <= 4 ? 4 : 8;
            const int ncode = np <= 1 ? 1 : np <= 2 ? 2 : 4;
            switch (pcode * 10 + ncode) {
                case 11: LLME_SAR(1, 1); break; case 12: LLME_SAR(1, 2); break; case 14: LLME_SAR(1, 4); break;
                case 21: LLME_SAR(2, 1); break; case 22: LLME_SAR(2, 2); break; case 24: LLME_SAR(2, 4); break;
                case 41: LLME_SAR(4, 1); break; case 42: LLME_SAR(4, 2); break; case 44: LLME_SAR(4, 4); break;
                case 81: LLME_SAR(8, 1); break; case 82: LLME_SAR(8, 2); break; case 84: LLME_SAR(8, 4); break;
            }
#undef LLME_SAR
            return launch_status();
        }
    }
    const size_t lds = sizeof(float) * (static_cast<size_t>(H) * dim + static_cast<size_t>(H) * H + H + 2 * static_cast<size_t>(H) * kKeysPerTile);
    if (lds > 64 * 1024) return kErrUnsupported;
    const int outs = H * vdim;
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

// The matrix-core form: bfloat16 q and pages, H a multiple of 4 up to 32, dim a multiple of 32 up to 128, vdim a multiple
// of 16 up to 128, pages of a multiple of 16 tokens, run_len a multiple of 32. mix_t is the mixing matrix transposed
// ([from, to]). tiles = sum over the requests of ceil(rows / 16).
extern "C" int llme_sigmoid_attention_mfma(const void* q, const void* k_cache, const void* v_cache, const void* mix_t,
                                           const void* bias, const void* positions, const void* q_start,
                                           const void* block_table, int max_blocks, void* partial, int T, int n_seq, int H,
                                           int G, int dim, int vdim, int page, float scale, int run_len, int runs, int tiles,
                                           hipStream_t stream) {
    if (T <= 0 || tiles <= 0) return 0;
    if (G <= 0 || H % G || runs <= 0 || run_len <= 0 || run_len % 32) return kErrBadArgument;
    if (H % 4 || H > 32 || dim % 32 || dim > 128 || vdim % 16 || vdim > 128 || page % 16) return kErrUnsupported;
#define LLME_SAM(D_, V_)                                                                                                 \
    return launch_sigmoid_attention_mfma<D_, V_>(q, k_cache, v_cache, static_cast<const float*>(mix_t),                  \
                                                 static_cast<const float*>(bias), static_cast<const int*>(positions),   \
                                                 static_cast<const int*>(q_start), static_cast<const int*>(block_table), \
                                                 max_blocks, static_cast<float*>(partial), T, n_seq, H, G, page, scale,  \
                                                 run_len, runs, tiles, stream)
#define LLME_SAM_V(D_)                                                                                                   \
    switch (vdim / 16) {                                                                                                 \
        case 1: LLME_SAM(D_, 1); case 2: LLME_SAM(D_, 2); case 3: LLME_SAM(D_, 3); case 4: LLME_SAM(D_, 4);              \
        case 5: LLME_SAM(D_, 5); case 6: LLME_SAM(D_, 6); case 7: LLME_SAM(D_, 7); case 8: LLME_SAM(D_, 8);              \
    }
    switch (dim / 32) {
        case 1: LLME_SAM_V(1) break;
        case 2: LLME_SAM_V(2) break;
        case 3: LLME_SAM_V(3) break;
        case 4: LLME_SAM_V(4) break;
    }
#undef LLME_SAM_V
#undef LLME_SAM
    return kErrUnsupported;
}

extern "C" int llme_sigmoid_attention_finish(const void* partial, int runs, const void* gate, int ld_gate, void* out, int out_dtype,
                                             int ld_out, int T, int H, int vdim, float scale_out, hipStream_t stream) {
    if (T <= 0) return 0;
    if (out_dtype == kF32)
        sigmoid_attention_finish_kernel<float><<<dim3(T, (H * vdim + 255) / 256), 256, 0, stream>>>(static_cast<const float*>(partial), runs,
                                                                      static_cast<const float*>(gate), ld_gate,
                                                                      static_cast<float*>(out), ld_out, T, H, vdim, scale_out);
    else if (out_dtype == kBF16)
        sigmoid_attention_finish_kernel<bf16><<<dim3(T, (H * vdim + 255) / 256), 256, 0, stream>>>(static_cast<const float*>(partial), runs,
                                                                     static_cast<const float*>(gate), ld_gate,
                                                                     static_cast<bf16*>(out), ld_out, T, H, vdim, scale_out);
    else
        return kErrBadArgument;
    return launch_status();
}

LLME_LOAD_ENTRY(sigmoid_attention)
