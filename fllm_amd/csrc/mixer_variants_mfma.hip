// Windows with pooled blocks and sigmoid attention on the matrix cores (bfloat16 pages, float32 scores and weights).
//
// A workgroup of four waves takes one tile of up to 16 queries: 16 rows of one request and one head (prompt portions), or
// the heads of one key/value head of one row (steps of single rows).  The waves deal the tile's keys among themselves in
// pairs of blocks of 32 and meet in LDS at the end.  Nothing is staged: every operand is a 16-byte load straight from the pages, which
// hold 8 lanes of a key side by side and a value lane's tokens side by side.
//
//   S^T = K Q^T   v_mfma_f32_16x16x32_bf16, A = 16 keys x 32 lanes, B = Q^T: the result leaves lane l with its own query
//                 (l % 16) and four keys.  A's row c of tile j holds key (c / 4) * 8 + j * 4 + c % 4 of the block, so that
//                 the two tiles of a block leave lane group g = l / 16 with the keys g * 8 .. g * 8 + 7 in order,
//   O^T += V^T P^T  which is how the next product's B operand wants them (k = g * 8 + e) and how a value lane's tokens lie
//                 in a page (one 16-byte load).
// Weights stay float32: P goes into the product as the sum of two bfloat16 numbers (its rounding and what the rounding
// lost), two products a tile.  The means of blocks are float32 in memory and go in the same way, for keys and for values.
#include <algorithm>

#include "api.h"
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWavesM = kThreads / kWave;

struct TileParams {
    const bf16_t *q;
    int q_stride;
    const bf16_t *k_pages, *v_pages;
    const float *pool_k, *pool_v;
    const int32_t *tables;
    int table_stride;
    const int32_t *row_pos, *row_seg, *seg_start;
    int num_segs;
    bf16_t *out;
    int rows, heads, kv_heads, page_size;
    float scale;
    int window, pool, slots;                  // pooled windows
    float softcap, temp_coef;                 // sigmoid weights
    int temp_every;
    const float *r1, *r2, *pb;
    int by_heads;                             // 1: a tile is the heads of one key/value head of one row
    int splits;                               // workgroups that share a tile's keys (blockIdx.z); more than one: partial results
    float *parts;                             // [tile][split][16 * DV sums, 16 maxima, 16 denominators] for the merge kernel
};

// The hardware's exponential, logarithm and reciprocal (a unit or two in the last place of a float32): these kernels serve the
// bfloat16 path alone, whose operands are rounded to eight bits.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float fast_log(float x) { return __builtin_amdgcn_logf(x) * 0.6931471805599453f; }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ void split_bf16(const float (&x)[8], bf16x8_t &hi, bf16x8_t &lo) {
#pragma unroll
    for (int e = 0; e < 8; e++) {
        hi[e] = (bf16_t)x[e];
        lo[e] = (bf16_t)(x[e] - (float)hi[e]);
    }
}

// VARIANT 0: window + pooled blocks, softmax.  VARIANT 1: every key up to the row, sigmoid weights.
template <int KD, int VT, int VARIANT>
__global__ void __launch_bounds__(kThreads)
mixer_tile_kernel(const TileParams p) {
    constexpr int D = KD * 32, DV = VT * 16;
    __shared__ float sm_o[kWavesM][16][DV + 1];
    __shared__ float sm_m[kWavesM][16], sm_l[kWavesM][16];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int qi = lane & 15, g = lane >> 4;
    const int G = p.heads / p.kv_heads;
    // ---- which queries this tile holds
    int seg = -1, row0 = 0, count = 0, kvh = 0, head0 = 0;
    if (p.by_heads) {
        row0 = blockIdx.x;
        seg = p.row_seg[row0];
        kvh = blockIdx.y;
        head0 = kvh * G;
        count = G;
        if (seg < 0) {      // padding row: zeros
            if (blockIdx.z == 0)
                for (int i = threadIdx.x; i < G * DV; i += kThreads) p.out[((size_t)row0 * p.heads + head0) * DV + i] = (bf16_t)0.f;
            return;
        }
    } else {
        int tile = blockIdx.x;
        for (int s = 0; s < p.num_segs; s++) {
            const int first = p.seg_start[s], n = p.seg_start[s + 1] - first;
            const int tiles = (n + 15) >> 4;
            if (tile < tiles) {
                row0 = first + tile * 16;
                count = n - tile * 16 < 16 ? n - tile * 16 : 16;
                seg = p.row_seg[row0];
                break;
            }
            tile -= tiles;
        }
        if (seg < 0) return;      // no such tile, or rows of padding (their outputs are never read in a step of portions)
        head0 = blockIdx.y;
        kvh = head0 / G;
    }
    const bool valid = qi < count;
    const int my_row = p.by_heads ? row0 : row0 + (valid ? qi : 0);
    const int my_head = p.by_heads ? head0 + (valid ? qi : 0) : head0;
    const int my_pos = p.row_pos[my_row];
    const int pos_min = p.row_pos[row0], pos_max = p.by_heads ? pos_min : p.row_pos[row0 + count - 1];
    const int32_t *tbl = p.tables + (size_t)seg * p.table_stride;
    const int ps = p.page_size;
    // ---- Q^T as the B operand: column = the lane's query, k = g * 8 + e of every 32 lanes of a head
    bf16x8_t qf[KD];
    {
        const bf16_t *qrow = p.q + (size_t)my_row * p.q_stride + (size_t)my_head * D;
#pragma unroll
        for (int kk = 0; kk < KD; kk++) {
            qf[kk] = *(const bf16x8_t *)(qrow + kk * 32 + g * 8);
            if (!valid)
#pragma unroll
                for (int e = 0; e < 8; e++) qf[kk][e] = (bf16_t)0.f;
        }
    }
    f32x4_t o[VT];
#pragma unroll
    for (int t = 0; t < VT; t++) o[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    // what the lane's query sees
    int lo_q = 0, nb_q = 0;
    float temp = 1.f, a1 = 0.f, a2 = 0.f, bias = 0.f;
    if (VARIANT == 0) {
        lo_q = my_pos - p.window + 1 > 0 ? my_pos - p.window + 1 : 0;
        nb_q = lo_q / p.pool;
    } else {
        temp = 1.0f + p.temp_coef * logf((float)((my_pos + 1) / p.temp_every) + 1.0f);
        a1 = p.r1[my_head], a2 = p.r2[my_head], bias = p.pb[my_head];
    }
    const float sc = p.scale * temp;
    const float two_over_cap = VARIANT == 1 ? 2.0f / p.softcap : 0.f;
    int turn = 0;      // blocks are dealt to the waves in turn, over both kinds of keys

    // one block of 32 keys: scores in s[2], then weights, then the products with the values
    auto weigh_and_add = [&](f32x4_t (&s)[2], auto visible, auto distance, auto load_values) {
        float pvals[8];
        if (VARIANT == 0) {
            float m_blk = -INFINITY;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    s[j][i] = visible(g * 8 + j * 4 + i) ? s[j][i] * sc : -INFINITY;
                    m_blk = fmaxf(m_blk, s[j][i]);
                }
            m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16, kWave));
            m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, kWave));
            const float m_new = fmaxf(m_run, m_blk);
            const float alpha = m_run == -INFINITY ? 0.f : fast_exp(m_run - m_new);
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float pv = s[j][i] == -INFINITY ? 0.f : fast_exp(s[j][i] - m_new);
                    pvals[j * 4 + i] = pv;
                    sum += pv;
                }
            l_run = l_run * alpha + sum;      // the lane's own keys; the lane groups are added at the end
            m_run = m_new;
#pragma unroll
            for (int t = 0; t < VT; t++) o[t] *= alpha;
        } else {
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int slot = g * 8 + j * 4 + i;
                    // cap * tanh(x / cap) = cap - 2 cap / (exp(2 x / cap) + 1): an overflowing exponential gives cap, none -cap
                    float x = s[j][i] * sc;
                    x = p.softcap - 2.0f * p.softcap * fast_rcp(fast_exp(x * two_over_cap) + 1.0f);
                    x = x - a1 * fast_log(fmaf(a2, distance(slot), 1.0f)) + bias;
                    pvals[j * 4 + i] = visible(slot) ? fast_rcp(1.0f + fast_exp(-x)) : 0.f;
                }
        }
        bf16x8_t p_hi, p_lo;
        split_bf16(pvals, p_hi, p_lo);
        load_values(p_hi, p_lo);
    };

    // ---- the means of blocks behind the window (VARIANT 0)
    if constexpr (VARIANT == 0) {
        const int lo_max = pos_max - p.window + 1 > 0 ? pos_max - p.window + 1 : 0;
        const int nb_max = lo_max / p.pool;
        for (int base = 0; base < nb_max; base += 32, turn++) {
            if ((turn & (kWavesM - 1)) != wave || (turn / kWavesM) % p.splits != (int)blockIdx.z) continue;
            f32x4_t s[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                s[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                int b = base + (qi >> 2) * 8 + j * 4 + (qi & 3);
                b = b < nb_max ? b : nb_max - 1;
                const int end = b * p.pool + p.pool - 1;
                const float *kr = p.pool_k + (((size_t)tbl[end / ps] * p.kv_heads + kvh) * p.slots + (end % ps) / p.pool) * D;
#pragma unroll
                for (int kk = 0; kk < KD; kk++) {
                    float x[8];
                    *(f32x4_t *)x = *(const f32x4_t *)(kr + kk * 32 + g * 8);
                    *(f32x4_t *)(x + 4) = *(const f32x4_t *)(kr + kk * 32 + g * 8 + 4);
                    bf16x8_t hi, lo;
                    split_bf16(x, hi, lo);
                    s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, qf[kk], s[j], 0, 0, 0);
                    s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lo, qf[kk], s[j], 0, 0, 0);
                }
            }
            weigh_and_add(
                s, [&](int slot) { return valid && base + slot < nb_q; }, [&](int) { return 0.f; },
                [&](const bf16x8_t &p_hi, const bf16x8_t &p_lo) {
                    // A = V^T: row = a value lane, k = the blocks base + g * 8 + e, each in a page and slot of its own
                    size_t at[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        int b = base + g * 8 + e;
                        b = b < nb_max ? b : nb_max - 1;
                        const int end = b * p.pool + p.pool - 1;
                        at[e] = (((size_t)tbl[end / ps] * p.kv_heads + kvh) * p.slots + (end % ps) / p.pool) * DV;
                    }
#pragma unroll
                    for (int t = 0; t < VT; t++) {
                        float x[8];
#pragma unroll
                        for (int e = 0; e < 8; e++) x[e] = p.pool_v[at[e] + t * 16 + qi];
                        bf16x8_t hi, lo;
                        split_bf16(x, hi, lo);
                        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, p_hi, o[t], 0, 0, 0);
                        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hi, p_lo, o[t], 0, 0, 0);
                        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(lo, p_hi, o[t], 0, 0, 0);
                    }
                });
        }
    }
    // ---- the tokens: from the first one that the tile's first row sees, two blocks of 32 positions a turn.  All operands of a
    // turn are asked for before the first product, so that the second block's loads and both blocks' values travel while the
    // first block's scores are weighed.  Keys behind the tile's last row are read from an address that exists and masked.
    {
        const int first = VARIANT == 0 ? (pos_min - p.window + 1 > 0 ? pos_min - p.window + 1 : 0) : 0;
        for (int base0 = first & ~63; base0 <= pos_max; base0 += 64, turn++) {
            if ((turn & (kWavesM - 1)) != wave || (turn / kWavesM) % p.splits != (int)blockIdx.z) continue;
            bf16x8_t ka[2][2][KD], va[2][VT];
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const int base = base0 + half * 32;
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    int key = base + (qi >> 2) * 8 + j * 4 + (qi & 3);
                    key = key <= pos_max ? key : pos_max;
                    const bf16_t *kr = p.k_pages + key_offset(tbl[key / ps], p.kv_heads, kvh, ps, D, key % ps, g * 8);
#pragma unroll
                    for (int kk = 0; kk < KD; kk++) ka[half][j][kk] = *(const bf16x8_t *)(kr + (size_t)kk * 4 * ps * 8);      // 32 lanes on: four chunks of 8
                }
                int key = base + g * 8;                  // eight tokens side by side in one page (pages hold multiples of 16)
                key = key <= pos_max ? key : pos_max & ~7;
                const bf16_t *vr = p.v_pages + (((size_t)tbl[key / ps] * p.kv_heads + kvh) * DV + qi) * ps + key % ps;
#pragma unroll
                for (int t = 0; t < VT; t++) va[half][t] = *(const bf16x8_t *)(vr + (size_t)t * 16 * ps);
            }
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const int base = base0 + half * 32;
                f32x4_t s[2];
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    s[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kk = 0; kk < KD; kk++) s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[half][j][kk], qf[kk], s[j], 0, 0, 0);
                }
                weigh_and_add(
                    s, [&](int slot) { const int key = base + slot; return valid && key <= my_pos && key >= lo_q; },
                    [&](int slot) { const int dist = my_pos - (base + slot); return (float)(dist > 0 ? dist : 0); },
                    [&](const bf16x8_t &p_hi, const bf16x8_t &p_lo) {
#pragma unroll
                        for (int t = 0; t < VT; t++) {
                            o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[half][t], p_hi, o[t], 0, 0, 0);
                            o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[half][t], p_lo, o[t], 0, 0, 0);
                        }
                    });
            }
        }
    }
    // ---- the waves meet
    if (VARIANT == 0) {
        l_run += __shfl_xor(l_run, 16, kWave);
        l_run += __shfl_xor(l_run, 32, kWave);
        if (g == 0) sm_m[wave][qi] = m_run, sm_l[wave][qi] = l_run;
    }
#pragma unroll
    for (int t = 0; t < VT; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) sm_o[wave][qi][t * 16 + g * 4 + i] = o[t][i];
    __syncthreads();
    float *part = p.splits > 1 ? p.parts + ((size_t)(blockIdx.y * gridDim.x + blockIdx.x) * p.splits + blockIdx.z) * (16 * DV + 32) : nullptr;
    for (int idx = threadIdx.x; idx < count * DV; idx += kThreads) {
        const int q = idx / DV, d = idx - q * DV;
        float acc = 0.f, l = 0.f;
        if (VARIANT == 0) {
            float m = -INFINITY;
#pragma unroll
            for (int w = 0; w < kWavesM; w++) m = fmaxf(m, sm_m[w][q]);
#pragma unroll
            for (int w = 0; w < kWavesM; w++) {
                const float f = sm_m[w][q] == -INFINITY ? 0.f : expf(sm_m[w][q] - m);
                l += sm_l[w][q] * f;
                acc += sm_o[w][q][d] * f;
            }
            if (part != nullptr) {      // this workgroup's share of the keys: the sums as they are, against its own maximum
                part[q * DV + d] = acc;
                if (d == 0) part[16 * DV + q] = m, part[16 * DV + 16 + q] = l;
                continue;
            }
            acc = l > 0.f ? acc / l : 0.f;
        } else {
#pragma unroll
            for (int w = 0; w < kWavesM; w++) acc += sm_o[w][q][d];
            if (part != nullptr) {
                part[q * DV + d] = acc;
                continue;
            }
        }
        const int row = p.by_heads ? row0 : row0 + q, head = p.by_heads ? head0 + q : head0;
        p.out[((size_t)row * p.heads + head) * DV + d] = (bf16_t)acc;
    }
}

// The shares of a tile's keys put together in the order of the shares: grid (rows, kv_heads), tiles by heads.
template <int VARIANT>
__global__ void __launch_bounds__(kThreads)
mixer_merge_kernel(const float *__restrict__ parts, int splits, const int32_t *__restrict__ row_seg, bf16_t *__restrict__ out, int heads,
                   int kv_heads, int DV) {
    const int row = blockIdx.x, kvh = blockIdx.y, G = heads / kv_heads;
    if (row_seg[row] < 0) return;
    const int stride = 16 * DV + 32;
    const float *mine = parts + (size_t)(blockIdx.y * gridDim.x + blockIdx.x) * splits * stride;
    for (int idx = threadIdx.x; idx < G * DV; idx += kThreads) {
        const int q = idx / DV, d = idx - q * DV;
        float acc = 0.f;
        if (VARIANT == 0) {
            float m = -INFINITY, l = 0.f;
            for (int s = 0; s < splits; s++) m = fmaxf(m, mine[(size_t)s * stride + 16 * DV + q]);
            for (int s = 0; s < splits; s++) {
                const float ms = mine[(size_t)s * stride + 16 * DV + q];
                const float f = ms == -INFINITY ? 0.f : expf(ms - m);
                l += mine[(size_t)s * stride + 16 * DV + 16 + q] * f;
                acc += mine[(size_t)s * stride + q * DV + d] * f;
            }
            acc = l > 0.f ? acc / l : 0.f;
        } else {
            for (int s = 0; s < splits; s++) acc += mine[(size_t)s * stride + q * DV + d];
        }
        out[((size_t)row * heads + kvh * G + q) * DV + d] = (bf16_t)acc;
    }
}

template <int VARIANT, int KD>
int launch_vt(const TileParams &p, int vt, dim3 grid, hipStream_t stream) {
    switch (vt) {
    case 2: hipLaunchKernelGGL((mixer_tile_kernel<KD, 2, VARIANT>), grid, dim3(kThreads), 0, stream, p); return 0;
    case 4: hipLaunchKernelGGL((mixer_tile_kernel<KD, 4, VARIANT>), grid, dim3(kThreads), 0, stream, p); return 0;
    case 6: hipLaunchKernelGGL((mixer_tile_kernel<KD, 6, VARIANT>), grid, dim3(kThreads), 0, stream, p); return 0;
    case 8: hipLaunchKernelGGL((mixer_tile_kernel<KD, 8, VARIANT>), grid, dim3(kThreads), 0, stream, p); return 0;
    }
    return 1;
}

template <int VARIANT>
int launch_tiles(TileParams &p, int head_dim, int v_dim, int keys_bound, hipStream_t stream) {
    // takes: bfloat16, keys in chunks of 8 (checked by the caller), heads of 32, 64, 96 or 128 lanes, values of 32, 64, 96 or
    // 128, pages of a multiple of 16 tokens, and for steps of single rows at most 16 heads a key/value head
    if (head_dim % 32 != 0 || head_dim > 128 || v_dim % 32 != 0 || v_dim > 128 || p.page_size % 16 != 0) return 1;
    const int G = p.heads / p.kv_heads;
    p.by_heads = p.rows == p.num_segs ? 1 : 0;
    if (p.by_heads && G > 16) return 1;
    dim3 grid = p.by_heads ? dim3(p.rows, p.kv_heads) : dim3((p.rows + 15) / 16 + p.num_segs, p.heads);
    if (grid.y > 65535) return 1;
    // Steps of single rows have a tile a row and key/value head: with few of them, several workgroups share a tile's keys
    // (at least 256 keys each, two workgroups a compute unit at most) and a second kernel puts their shares together.
    p.splits = 1;
    p.parts = nullptr;
    if (p.by_heads) {
        const long tiles = (long)p.rows * p.kv_heads;
        long splits = std::min<long>(std::min<long>(512 / std::max<long>(tiles, 1), (keys_bound + 255) / 256), 32);
        void *base = nullptr;
        size_t bytes = 0;
        if (splits > 1 && fllm_device_workspace(&base, &bytes) && bytes > kWorkspaceCounterBytes) {
            const size_t room = (bytes - kWorkspaceCounterBytes) / sizeof(float), each = (size_t)tiles * (16 * v_dim + 32);
            splits = std::min<long>(splits, (long)(room / each));
            if (splits > 1) {
                p.splits = (int)splits;
                p.parts = (float *)((char *)base + kWorkspaceCounterBytes);
                grid.z = (unsigned)splits;
            }
        }
    }
    int declined = 1;
    switch (head_dim / 32) {
    case 1: declined = launch_vt<VARIANT, 1>(p, v_dim / 16, grid, stream); break;
    case 2: declined = launch_vt<VARIANT, 2>(p, v_dim / 16, grid, stream); break;
    case 3: declined = launch_vt<VARIANT, 3>(p, v_dim / 16, grid, stream); break;
    case 4: declined = launch_vt<VARIANT, 4>(p, v_dim / 16, grid, stream); break;
    }
    if (!declined && p.splits > 1)
        hipLaunchKernelGGL(mixer_merge_kernel<VARIANT>, dim3(p.rows, p.kv_heads), dim3(kThreads), 0, stream, p.parts, p.splits, p.row_seg, p.out,
                           p.heads, p.kv_heads, v_dim);
    return declined;
}

}  // namespace

// 0: launched; 1: the shape is not one these kernels take (the caller runs the plain kernel).
int fllm_pooled_window_attention_bf16_fast(const void *q, int q_stride, const void *k_pages, const void *v_pages, const float *pool_k,
                                           const float *pool_v, const int32_t *tables, int table_stride, const int32_t *row_pos,
                                           const int32_t *row_seg, const int32_t *seg_start, int num_segs, void *out, int rows,
                                           int heads, int kv_heads, int head_dim, int v_dim, int page_size, float scale, int window,
                                           int pool, int max_context, hipStream_t stream) {
    if (!fllm_fast_kernels_enabled() || seg_start == nullptr || num_segs <= 0) return 1;
    TileParams p = {};
    p.q = (const bf16_t *)q, p.q_stride = q_stride, p.k_pages = (const bf16_t *)k_pages, p.v_pages = (const bf16_t *)v_pages;
    p.pool_k = pool_k, p.pool_v = pool_v, p.tables = tables, p.table_stride = table_stride, p.row_pos = row_pos, p.row_seg = row_seg;
    p.seg_start = seg_start, p.num_segs = num_segs, p.out = (bf16_t *)out, p.rows = rows, p.heads = heads, p.kv_heads = kv_heads;
    p.page_size = page_size, p.scale = scale, p.window = window, p.pool = pool, p.slots = (page_size + pool - 1) / pool;
    const int span = max_context > 0 ? std::min(max_context, window + (max_context + pool - 1) / pool) : window;
    if (launch_tiles<0>(p, head_dim, v_dim, span, stream)) return 1;
    return fllm_check_launch("pooled_window_attention (matrix cores)");
}

int fllm_sigmoid_attention_bf16_fast(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                                     int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                                     int num_segs, void *out, int rows, int heads, int kv_heads, int head_dim, int v_dim, int page_size,
                                     float scale, float softcap, const float *r1, const float *r2, const float *pb, float temp_coef,
                                     int temp_every, int max_context, hipStream_t stream) {
    if (!fllm_fast_kernels_enabled() || seg_start == nullptr || num_segs <= 0) return 1;
    TileParams p = {};
    p.q = (const bf16_t *)q, p.q_stride = q_stride, p.k_pages = (const bf16_t *)k_pages, p.v_pages = (const bf16_t *)v_pages;
    p.tables = tables, p.table_stride = table_stride, p.row_pos = row_pos, p.row_seg = row_seg, p.seg_start = seg_start;
    p.num_segs = num_segs, p.out = (bf16_t *)out, p.rows = rows, p.heads = heads, p.kv_heads = kv_heads, p.page_size = page_size;
    p.scale = scale, p.softcap = softcap, p.temp_coef = temp_coef, p.temp_every = temp_every, p.r1 = r1, p.r2 = r2, p.pb = pb;
    p.window = 1, p.pool = 1, p.slots = 1;
    if (launch_tiles<1>(p, head_dim, v_dim, max_context, stream)) return 1;
    return fllm_check_launch("sigmoid_attention (matrix cores)");
}
