// Mixers beside the softmax attention over all keys, plain forms: float32 arithmetic, both element types, any sizes.
//
//   normed_rope_store        rows of a joint product [q | k | v | ..]: a weighted RMS norm of q and of k (a head at a time with
//                            one weight vector for all heads, or over the whole projection), rotary on the first lanes of every
//                            head (lane i with lane i + dims / 2), queries out, keys and values into the pages; the values may be
//                            the keys as projected.
//   pool_blocks              the float32 means of the keys and of the values of every block of `pool` positions whose last token
//                            is among the step's rows, kept beside the page that holds that token.
//   pooled_window_attention  a row sees its last `window` tokens and one mean key and value for every block that lies wholly
//                            before them; one softmax over both kinds.
//   sigmoid_attention        no softmax: key j weighs sigmoid(cap * tanh(s / cap) - r1 ln(1 + r2 (pos - j)) + pb) on its own.
//   rotate_scale             q and k of a linear attention rotated and k scaled, in float32, values beside them.
//   group_norm_gate          every group of lanes divided by its root mean square, times silu or sigmoid of a gate.
//   weighted_sum, stream_concat, activation: the small passes around them.
//
// A row's result depends on its own position, pages and slot alone, never on the rest of the batch.
#include "api.h"
#include "common.h"

// mixer_variants_mfma.hip; 1: the shape is not one the matrix-core kernels take
int fllm_pooled_window_attention_bf16_fast(const void *q, int q_stride, const void *k_pages, const void *v_pages, const float *pool_k,
                                           const float *pool_v, const int32_t *tables, int table_stride, const int32_t *row_pos,
                                           const int32_t *row_seg, const int32_t *seg_start, int num_segs, void *out, int rows,
                                           int heads, int kv_heads, int head_dim, int v_dim, int page_size, float scale, int window,
                                           int pool, int max_context, hipStream_t stream);
int fllm_sigmoid_attention_bf16_fast(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                                     int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                                     int num_segs, void *out, int rows, int heads, int kv_heads, int head_dim, int v_dim, int page_size,
                                     float scale, float softcap, const float *r1, const float *r2, const float *pb, float temp_coef,
                                     int temp_every, int max_context, hipStream_t stream);

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

__device__ __forceinline__ size_t key_at(size_t page, int kv_heads, int kvh, int page_size, int k_dim, int token, int d, int c) {
    return ((((size_t)page * kv_heads + kvh) * (k_dim / c) + d / c) * page_size + token) * c + d % c;
}

// ---- norm, rotation, store -----------------------------------------------------------------------------------------------
// norm_mode 0: none; 1: every head over its own lanes, weights [k_dim] shared by the heads; 2: the whole projection, weights
// [heads * k_dim] and [kv_heads * k_dim].  LDS: heads + kv_heads floats (the heads' factors).
template <typename T>
__global__ void __launch_bounds__(kBlock)
normed_rope_store_kernel(const T *__restrict__ qkv, int ld, int norm_mode, const float *__restrict__ q_weight,
                         const float *__restrict__ k_weight, float eps, T *__restrict__ q_out, const int32_t *__restrict__ row_pos,
                         const int32_t *__restrict__ row_seg, const int32_t *__restrict__ tables, int table_stride,
                         const float *__restrict__ cos_table, const float *__restrict__ sin_table, T *__restrict__ k_pages,
                         T *__restrict__ v_pages, int heads, int kv_heads, int k_dim, int v_dim, int rope_dims, int page_size,
                         int key_chunk, int store_kv, int values_from_keys) {
    extern __shared__ float inv_head[];   // heads + kv_heads
    __shared__ float scratch[kWaves];
    const size_t r = blockIdx.x;
    const int seg = row_seg[r];
    if (seg < 0) return;   // padding row: its queries are never read
    const int pos = row_pos[r];
    const int nq = heads * k_dim, nk = kv_heads * k_dim, nv = kv_heads * v_dim;
    const T *q = qkv + r * ld, *k = q + nq, *v = values_from_keys ? k : k + nk;
    const int page = store_kv ? tables[(size_t)seg * table_stride + pos / page_size] : 0, off = pos % page_size;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    float inv_q = 1.f, inv_k = 1.f;
    if (norm_mode == 2) {
        float sq = 0.f, sk = 0.f;
        for (int c = threadIdx.x; c < nq; c += kBlock) { const float a = to_f32<T>(q[c]); sq += a * a; }
        for (int c = threadIdx.x; c < nk; c += kBlock) { const float a = to_f32<T>(k[c]); sk += a * a; }
        sq = block_sum<kWaves>(sq, scratch);
        sk = block_sum<kWaves>(sk, scratch);
        inv_q = 1.0f / sqrtf(sq / (float)nq + eps);
        inv_k = 1.0f / sqrtf(sk / (float)nk + eps);
    } else if (norm_mode == 1) {
        for (int h = wave; h < heads + kv_heads; h += kWaves) {
            const T *head = q + (size_t)h * k_dim;      // the keys' heads follow the queries'
            float ss = 0.f;
            for (int c = lane; c < k_dim; c += kWave) { const float a = to_f32<T>(head[c]); ss = fmaf(a, a, ss); }
            ss = wave_sum(ss);
            if (lane == 0) inv_head[h] = 1.0f / sqrtf(ss / (float)k_dim + eps);
        }
        __syncthreads();
    }
    const int half = rope_dims / 2;
    const float *cs = cos_table + (size_t)pos * half, *sn = sin_table + (size_t)pos * half;
    for (int idx = threadIdx.x; idx < nq + (store_kv ? nk : 0); idx += kBlock) {
        const bool is_q = idx < nq;
        const int e = is_q ? idx : idx - nq;
        const T *src = is_q ? q : k;
        const float *w = is_q ? q_weight : k_weight;
        const int h = e / k_dim, c = e - h * k_dim;
        const float inv = norm_mode == 2 ? (is_q ? inv_q : inv_k) : (norm_mode == 1 ? inv_head[is_q ? h : heads + h] : 1.f);
        const float we = norm_mode == 2 ? w[e] : (norm_mode == 1 ? w[c] : 1.f);
        float val = to_f32<T>(src[e]) * inv * we;
        if (c < rope_dims) {
            const int i = c < half ? c : c - half;
            const int pe = c < half ? e + half : e - half, pc = c < half ? c + half : c - half;
            const float wp = norm_mode == 2 ? w[pe] : (norm_mode == 1 ? w[pc] : 1.f);
            const float other = to_f32<T>(src[pe]) * inv * wp;
            val = c < half ? val * cs[i] - other * sn[i] : val * cs[i] + other * sn[i];
        }
        if (is_q) q_out[r * nq + e] = from_f32<T>(val);
        else k_pages[key_at(page, kv_heads, h, page_size, k_dim, off, c, key_chunk)] = from_f32<T>(val);
    }
    if (!store_kv) return;
    for (int e = threadIdx.x; e < nv; e += kBlock) {
        const int h = e / v_dim, c = e - h * v_dim;
        v_pages[(((size_t)page * kv_heads + h) * v_dim + c) * page_size + off] = v[e];
    }
}

// ---- means of blocks -------------------------------------------------------------------------------------------------------
// grid (rows, kv_heads).  A row whose position ends a block of `pool` positions sums the block's keys and values from the pages
// in position order and stores the means: pool_k [page][kv_head][slot][k_dim], pool_v [page][kv_head][slot][v_dim], page the
// one of the block's last token, slot = (that token's place in the page) / pool.
template <typename T>
__global__ void __launch_bounds__(kBlock)
pool_blocks_kernel(const T *__restrict__ k_pages, const T *__restrict__ v_pages, float *__restrict__ pool_k, float *__restrict__ pool_v,
                   const int32_t *__restrict__ tables, int table_stride, const int32_t *__restrict__ row_pos,
                   const int32_t *__restrict__ row_seg, int kv_heads, int k_dim, int v_dim, int page_size, int key_chunk, int pool,
                   int slots) {
    const int r = blockIdx.x, kvh = blockIdx.y;
    const int seg = row_seg[r];
    if (seg < 0) return;
    const int pos = row_pos[r];
    if ((pos + 1) % pool != 0) return;
    const int32_t *tbl = tables + (size_t)seg * table_stride;
    const int first = pos - pool + 1;
    const size_t dst = (((size_t)tbl[pos / page_size] * kv_heads + kvh) * slots + (pos % page_size) / pool);
    for (int c = threadIdx.x; c < k_dim + v_dim; c += kBlock) {
        const bool is_key = c < k_dim;
        const int cv = c - k_dim;
        float sum = 0.f;
        for (int t0 = 0; t0 < pool; t0 += 8) {      // eight loads on their way at once, added in position order
            float vals[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int key = first + (t0 + j < pool ? t0 + j : pool - 1), page = tbl[key / page_size], off = key % page_size;
                const size_t at = is_key ? key_at(page, kv_heads, kvh, page_size, k_dim, off, c, key_chunk)
                                         : (((size_t)page * kv_heads + kvh) * v_dim + cv) * page_size + off;
                vals[j] = to_f32<T>((is_key ? k_pages : v_pages)[at]);
            }
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (t0 + j < pool) sum += vals[j];
        }
        if (is_key) pool_k[dst * k_dim + c] = sum / (float)pool;
        else pool_v[dst * v_dim + cv] = sum / (float)pool;
    }
}

// The same for bfloat16 pages with keys in chunks of 8, blocks of a multiple of 8 positions and pages of a multiple of 8
// tokens: every load takes 16 bytes (8 lanes of a key, or 8 tokens of a value lane), a thread sums eight positions in
// order, and the eights are added in order through LDS: two rounds of loads a block instead of one a position.
__global__ void __launch_bounds__(kBlock)
pool_blocks_vec_kernel(const bf16_t *__restrict__ k_pages, const bf16_t *__restrict__ v_pages, float *__restrict__ pool_k,
                       float *__restrict__ pool_v, const int32_t *__restrict__ tables, int table_stride,
                       const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seg, int kv_heads, int k_dim, int v_dim,
                       int page_size, int pool, int slots) {
    extern __shared__ float part[];      // [pool / 8][k_dim + v_dim]
    const int r = blockIdx.x, kvh = blockIdx.y;
    const int seg = row_seg[r];
    if (seg < 0) return;
    const int pos = row_pos[r];
    if ((pos + 1) % pool != 0) return;
    const int32_t *tbl = tables + (size_t)seg * table_stride;
    const int first = pos - pool + 1, eights = pool / 8, width = k_dim + v_dim;
    const size_t dst = (((size_t)tbl[pos / page_size] * kv_heads + kvh) * slots + (pos % page_size) / pool);
    // keys: an item is (eight positions, one chunk of 8 lanes)
    for (int item = threadIdx.x; item < eights * (k_dim / 8); item += kBlock) {
        const int tg = item / (k_dim / 8), ch = item - tg * (k_dim / 8);
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        bf16x8_t got[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int key = first + tg * 8 + j;
            got[j] = *(const bf16x8_t *)(k_pages + key_offset(tbl[key / page_size], kv_heads, kvh, page_size, k_dim, key % page_size, ch * 8));
        }
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] += (float)got[j][e];
#pragma unroll
        for (int e = 0; e < 8; e++) part[tg * width + ch * 8 + e] = acc[e];
    }
    // values: an item is (eight positions, one lane); the eight lie side by side in one page
    for (int item = threadIdx.x; item < eights * v_dim; item += kBlock) {
        const int tg = item / v_dim, c = item - tg * v_dim;
        const int key = first + tg * 8;
        const bf16x8_t got = *(const bf16x8_t *)(v_pages + (((size_t)tbl[key / page_size] * kv_heads + kvh) * v_dim + c) * page_size + key % page_size);
        float acc = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc += (float)got[e];
        part[tg * width + k_dim + c] = acc;
    }
    __syncthreads();
    for (int c = threadIdx.x; c < width; c += kBlock) {
        float sum = 0.f;
        for (int tg = 0; tg < eights; tg++) sum += part[tg * width + c];
        if (c < k_dim) pool_k[dst * k_dim + c] = sum / (float)pool;
        else pool_v[dst * v_dim + (c - k_dim)] = sum / (float)pool;
    }
}

// ---- what a thread's key contributes ---------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float key_dot(const float *__restrict__ qs, const T *__restrict__ kr, int head_dim, size_t chunk_step, int key_chunk) {
    float dot = 0.f;
    if (key_chunk == 8) {
        if constexpr (sizeof(T) == 2) {
            for (int ch = 0; ch < head_dim / 8; ch++) {
                const bf16x8_t k8 = *(const bf16x8_t *)(kr + (size_t)ch * chunk_step);
#pragma unroll
                for (int e = 0; e < 8; e++) dot = fmaf(qs[ch * 8 + e], (float)k8[e], dot);
            }
        } else {
            for (int ch = 0; ch < head_dim / 8; ch++) {
                const f32x4_t a = *(const f32x4_t *)(kr + (size_t)ch * chunk_step), b = *(const f32x4_t *)(kr + (size_t)ch * chunk_step + 4);
#pragma unroll
                for (int e = 0; e < 4; e++) dot = fmaf(qs[ch * 8 + e], to_f32<T>(a[e]), dot);
#pragma unroll
                for (int e = 0; e < 4; e++) dot = fmaf(qs[ch * 8 + 4 + e], to_f32<T>(b[e]), dot);
            }
        }
    } else {
        for (int c = 0; c < head_dim; c++) dot = fmaf(qs[c], to_f32<T>(kr[(size_t)(c / key_chunk) * chunk_step + c % key_chunk]), dot);
    }
    return dot;
}

// The weighted sum of values of one run of up to kBlock keys.  The workgroup's threads form groups of `vd_pad` lanes (a power
// of two of at least v_dim, at most kBlock); group g takes the keys g, g + groups, .. of the run, so all threads work whatever the
// head's width.  voff[j] is the address of key j's value lane 0 and vstep[j] the distance of its lanes (page_size: a token's
// values in the pages; 0: the float32 means of a block in `pool_v`, lane beside lane).
constexpr int kMaxLanes = 2;   // values of up to 2 * kBlock lanes a head
template <typename T, bool POOLED>
__device__ __forceinline__ void add_values(float (&acc)[kMaxLanes], const float *__restrict__ sc, const long long *__restrict__ voff,
                                           const int *__restrict__ vstep, int count, const T *__restrict__ v_pages,
                                           const float *__restrict__ pool_v, int v_dim, int vd_pad) {
    const int groups = kBlock / vd_pad, g = threadIdx.x / vd_pad, c0 = threadIdx.x % vd_pad;
#pragma unroll
    for (int t = 0; t < kMaxLanes; t++) {
        const int c = c0 + t * vd_pad;
        if (c >= v_dim) break;
        float a = acc[t];
        for (int j = g; j < count; j += groups) {
            const int step = vstep[j];
            float val;
            if constexpr (POOLED) val = step == 0 ? pool_v[voff[j] + c] : to_f32<T>(v_pages[voff[j] + (size_t)c * step]);
            else val = to_f32<T>(v_pages[voff[j] + (size_t)c * step]);
            a = fmaf(sc[j], val, a);
        }
        acc[t] = a;
    }
}

// The groups' partial sums added in group order; the result in the threads of group 0.
__device__ __forceinline__ void merge_groups(float (&acc)[kMaxLanes], float *__restrict__ buf /* kMaxLanes * kBlock */, int vd_pad) {
    const int groups = kBlock / vd_pad;
    if (groups == 1) return;
    __syncthreads();
#pragma unroll
    for (int t = 0; t < kMaxLanes; t++) buf[t * kBlock + threadIdx.x] = acc[t];
    __syncthreads();
    if (threadIdx.x < vd_pad) {
#pragma unroll
        for (int t = 0; t < kMaxLanes; t++) {
            float a = 0.f;
            for (int g = 0; g < groups; g++) a += buf[t * kBlock + g * vd_pad + threadIdx.x];
            acc[t] = a;
        }
    }
}

// ---- a window of tokens with pooled blocks behind it ------------------------------------------------------------------------
// grid (rows, heads).  The row's keys in one line: first the blocks 0 .. nb - 1 (means), then the tokens lo .. pos.
template <typename T>
__global__ void __launch_bounds__(kBlock)
pooled_window_attention_kernel(const T *__restrict__ q, int q_stride, const T *__restrict__ k_pages, const T *__restrict__ v_pages,
                               const float *__restrict__ pool_k, const float *__restrict__ pool_v, const int32_t *__restrict__ tables,
                               int table_stride, const int32_t *__restrict__ row_pos, const int32_t *__restrict__ row_seg,
                               T *__restrict__ out, int heads, int kv_heads, int head_dim, int v_dim, int page_size, float scale,
                               int window, int pool, int slots, int key_chunk, int vd_pad) {
    extern __shared__ float smem[];
    float *qs = smem;                                   // head_dim (rounded up to a multiple of 2)
    float *sc = qs + ((head_dim + 1) & ~1);             // kBlock
    float *scratch = sc + kBlock;                       // kWaves (+ padding to 8 bytes)
    long long *voff = (long long *)(scratch + 2 * ((kWaves + 1) / 2));   // kBlock
    int *vstep = (int *)(voff + kBlock);                // kBlock
    float *buf = (float *)(vstep + kBlock);             // kMaxLanes * kBlock
    const int r = blockIdx.x, h = blockIdx.y;
    const int seg = row_seg[r];
    T *dst = out + ((size_t)r * heads + h) * v_dim;
    if (seg < 0) {
        for (int c = threadIdx.x; c < v_dim; c += kBlock) dst[c] = from_f32<T>(0.f);
        return;
    }
    const int pos = row_pos[r];
    const int lo = pos - window + 1 > 0 ? pos - window + 1 : 0;
    const int nb = lo / pool;                            // blocks that end at or before pos - window
    const int n = nb + (pos - lo + 1);
    const int kvh = h / (heads / kv_heads);
    const int32_t *tbl = tables + (size_t)seg * table_stride;
    const T *qrow = q + (size_t)r * q_stride + (size_t)h * head_dim;
    for (int c = threadIdx.x; c < head_dim; c += kBlock) qs[c] = to_f32<T>(qrow[c]);
    __syncthreads();
    const size_t chunk_step = (size_t)page_size * key_chunk;
    float m = -INFINITY, l = 0.f;
    float acc[kMaxLanes] = {0.f, 0.f};
    for (int c0 = 0; c0 < n; c0 += kBlock) {
        const int t = c0 + threadIdx.x;
        float s = -INFINITY;
        if (t < nb) {
            const int end = t * pool + pool - 1, page = tbl[end / page_size], slot = (end % page_size) / pool;
            const size_t at = ((size_t)page * kv_heads + kvh) * slots + slot;
            const float *kr = pool_k + at * head_dim;
            float dot = 0.f;
            for (int c = 0; c < head_dim; c++) dot = fmaf(qs[c], kr[c], dot);
            s = dot * scale;
            voff[threadIdx.x] = (long long)(at * v_dim);
            vstep[threadIdx.x] = 0;
        } else if (t < n) {
            const int key = lo + (t - nb), page = tbl[key / page_size], off = key % page_size;
            const T *kr = k_pages + key_at(page, kv_heads, kvh, page_size, head_dim, off, 0, key_chunk);
            s = key_dot<T>(qs, kr, head_dim, chunk_step, key_chunk) * scale;
            voff[threadIdx.x] = (long long)(((size_t)page * kv_heads + kvh) * v_dim * page_size + off);
            vstep[threadIdx.x] = page_size;
        }
        const float m_new = fmaxf(m, block_max<kWaves>(s, scratch));
        const float alpha = expf(m - m_new);
        const float p = t < n ? expf(s - m_new) : 0.f;
        sc[threadIdx.x] = p;
        l = l * alpha + block_sum<kWaves>(p, scratch);   // the barriers inside also publish sc[], voff[] and vstep[]
        const int count = n - c0 < kBlock ? n - c0 : kBlock;
#pragma unroll
        for (int i = 0; i < kMaxLanes; i++) acc[i] *= alpha;
        add_values<T, true>(acc, sc, voff, vstep, count, v_pages, pool_v, v_dim, vd_pad);
        m = m_new;
        __syncthreads();
    }
    merge_groups(acc, buf, vd_pad);
    const float inv = 1.0f / l;
    if (threadIdx.x < vd_pad) {
#pragma unroll
        for (int i = 0; i < kMaxLanes; i++) {
            const int c = threadIdx.x + i * vd_pad;
            if (c < v_dim) dst[c] = from_f32<T>(acc[i] * inv);
        }
    }
}

// ---- sigmoid weights --------------------------------------------------------------------------------------------------------
// grid (rows, heads).  Every key 0 .. pos weighs on its own; the sum of weight * value is the output.
template <typename T>
__global__ void __launch_bounds__(kBlock)
sigmoid_attention_kernel(const T *__restrict__ q, int q_stride, const T *__restrict__ k_pages, const T *__restrict__ v_pages,
                         const int32_t *__restrict__ tables, int table_stride, const int32_t *__restrict__ row_pos,
                         const int32_t *__restrict__ row_seg, T *__restrict__ out, int heads, int kv_heads, int head_dim, int v_dim,
                         int page_size, float scale, float softcap, const float *__restrict__ r1, const float *__restrict__ r2,
                         const float *__restrict__ pb, float temp_coef, int temp_every, int key_chunk, int vd_pad) {
    extern __shared__ float smem[];
    float *qs = smem;
    float *sc = qs + ((head_dim + 1) & ~1);
    long long *voff = (long long *)(sc + kBlock);
    int *vstep = (int *)(voff + kBlock);
    float *buf = (float *)(vstep + kBlock);
    const int r = blockIdx.x, h = blockIdx.y;
    const int seg = row_seg[r];
    T *dst = out + ((size_t)r * heads + h) * v_dim;
    if (seg < 0) {
        for (int c = threadIdx.x; c < v_dim; c += kBlock) dst[c] = from_f32<T>(0.f);
        return;
    }
    const int pos = row_pos[r];
    const int n = pos + 1;
    const int kvh = h / (heads / kv_heads);
    const int32_t *tbl = tables + (size_t)seg * table_stride;
    const T *qrow = q + (size_t)r * q_stride + (size_t)h * head_dim;
    for (int c = threadIdx.x; c < head_dim; c += kBlock) qs[c] = to_f32<T>(qrow[c]);
    __syncthreads();
    // the query's temperature grows with its position; it multiplies the score, which is the product it would scale
    const float temp = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
    const float s_scale = scale * temp, a1 = r1[h], a2 = r2[h], bias = pb[h];
    const size_t chunk_step = (size_t)page_size * key_chunk;
    float acc[kMaxLanes] = {0.f, 0.f};
    for (int c0 = 0; c0 < n; c0 += kBlock) {
        const int key = c0 + threadIdx.x;
        float p = 0.f;
        if (key < n) {
            const int page = tbl[key / page_size], off = key % page_size;
            const T *kr = k_pages + key_at(page, kv_heads, kvh, page_size, head_dim, off, 0, key_chunk);
            float s = key_dot<T>(qs, kr, head_dim, chunk_step, key_chunk) * s_scale;
            s = softcap * tanhf(s / softcap) - a1 * log1pf(a2 * (float)(pos - key)) + bias;
            p = 1.0f / (1.0f + expf(-s));
            voff[threadIdx.x] = (long long)(((size_t)page * kv_heads + kvh) * v_dim * page_size + off);
            vstep[threadIdx.x] = page_size;
        }
        sc[threadIdx.x] = p;
        __syncthreads();
        const int count = n - c0 < kBlock ? n - c0 : kBlock;
        add_values<T, false>(acc, sc, voff, vstep, count, v_pages, nullptr, v_dim, vd_pad);
        __syncthreads();
    }
    merge_groups(acc, buf, vd_pad);
    if (threadIdx.x < vd_pad) {
#pragma unroll
        for (int i = 0; i < kMaxLanes; i++) {
            const int c = threadIdx.x + i * vd_pad;
            if (c < v_dim) dst[c] = from_f32<T>(acc[i]);
        }
    }
}

// ---- operands of a linear attention: rotated, scaled, float32 ----------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(kBlock)
rotate_scale_kernel(const T *__restrict__ qkv, int ld, float *__restrict__ out, const int32_t *__restrict__ row_pos,
                    const float *__restrict__ cos_table, const float *__restrict__ sin_table, int positions, int heads, int dim,
                    int vdim, int rope_dims, float key_scale) {
    const size_t r = blockIdx.x;
    int pos = row_pos[r];
    pos = pos < 0 ? 0 : (pos >= positions && positions > 0 ? positions - 1 : pos);   // padding rows carry any position
    const int nq = heads * dim, nv = heads * vdim, half = rope_dims / 2;
    const T *src = qkv + r * ld;
    float *dst = out + r * (size_t)(2 * nq + nv);
    const float *cs = cos_table + (size_t)pos * half, *sn = sin_table + (size_t)pos * half;
    for (int idx = threadIdx.x; idx < 2 * nq; idx += kBlock) {
        const int c = idx % dim;
        float val = to_f32<T>(src[idx]);
        if (c < rope_dims) {
            const int i = c < half ? c : c - half;
            const float other = to_f32<T>(src[c < half ? idx + half : idx - half]);
            val = c < half ? val * cs[i] - other * sn[i] : val * cs[i] + other * sn[i];
        }
        dst[idx] = idx < nq ? val : val * key_scale;
    }
    for (int idx = threadIdx.x; idx < nv; idx += kBlock) dst[2 * nq + idx] = to_f32<T>(src[2 * nq + idx]);
}

// ---- a norm a group of lanes, gated -----------------------------------------------------------------------------------------
template <typename X, typename T>
__global__ void __launch_bounds__(kBlock)
group_norm_gate_kernel(const X *__restrict__ x, float eps, int group, const T *__restrict__ gate, int gate_ld, T *__restrict__ out,
                       int width, int silu) {
    const size_t r = blockIdx.x;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    for (int g = wave; g < width / group; g += kWaves) {
        const X *src = x + r * width + (size_t)g * group;
        float ss = 0.f;
        for (int c = lane; c < group; c += kWave) { const float a = to_f32<X>(src[c]); ss = fmaf(a, a, ss); }
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)group + eps);
        for (int c = lane; c < group; c += kWave) {
            const float z = to_f32<T>(gate[r * gate_ld + (size_t)g * group + c]);
            const float sg = 1.0f / (1.0f + expf(-z));
            out[r * width + (size_t)g * group + c] = from_f32<T>(to_f32<X>(src[c]) * inv * (silu ? z * sg : sg));
        }
    }
}

__global__ void __launch_bounds__(kBlock)
weighted_sum_kernel(float *__restrict__ out, const float *__restrict__ x, float a, const float *__restrict__ y, float b, size_t total,
                    int accumulate) {
    for (size_t i = blockIdx.x * (size_t)kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock) {
        const float v = a * x[i] + b * y[i];
        out[i] = accumulate ? out[i] + v : v;
    }
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
stream_concat_kernel(const float *__restrict__ x, const int32_t *__restrict__ ids, const T *__restrict__ table, int vocab, float scale,
                     T *__restrict__ out, int width) {
    const size_t r = blockIdx.x;
    int id = ids[r];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int c = threadIdx.x; c < width; c += kBlock) {
        out[r * 2 * width + c] = from_f32<T>(x[r * width + c]);
        out[r * 2 * width + width + c] = from_f32<T>(to_f32<T>(table[(size_t)id * width + c]) * scale);
    }
}

template <typename T>
__global__ void __launch_bounds__(kBlock) relu_squared_kernel(const T *__restrict__ x, T *__restrict__ out, size_t total) {
    for (size_t i = blockIdx.x * (size_t)kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock) {
        const float a = fmaxf(to_f32<T>(x[i]), 0.f);
        out[i] = from_f32<T>(a * a);
    }
}

int pow2_lanes(int v_dim) {
    int p = 1;
    while (p < v_dim && p < kBlock) p *= 2;
    return p;
}
int small_grid(size_t total) {
    const size_t blocks = (total + kBlock - 1) / kBlock;
    return (int)(blocks < 4096 ? (blocks ? blocks : 1) : 4096);
}

}  // namespace

extern "C" int fllm_normed_rope_store(const void *qkv, int ld, int norm_mode, const float *q_weight, const float *k_weight, float eps,
                                      void *q_out, const int32_t *row_pos, const int32_t *row_seg, const int32_t *tables,
                                      int table_stride, const float *cos_table, const float *sin_table, int table_positions,
                                      void *k_pages, void *v_pages, int rows, int heads, int kv_heads, int k_dim, int v_dim,
                                      int rope_dims, int page_size, int key_chunk, int dtype, int store_kv, int values_from_keys,
                                      hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && kv_heads > 0 && k_dim > 0 && v_dim > 0 && page_size > 0 && table_stride > 0,
                 "normed_rope_store: bad sizes");
    FLLM_REQUIRE(norm_mode >= 0 && norm_mode <= 2, "normed_rope_store: unknown norm %d", norm_mode);
    FLLM_REQUIRE(!values_from_keys || v_dim == k_dim, "normed_rope_store: keys that double as values have one width");
    FLLM_REQUIRE(ld >= heads * k_dim + kv_heads * k_dim + (values_from_keys ? 0 : kv_heads * v_dim),
                 "normed_rope_store: rows of %d values cannot hold q, k and v", ld);
    FLLM_REQUIRE(rope_dims >= 0 && rope_dims <= k_dim && rope_dims % 2 == 0,
                 "normed_rope_store: rope_dims %d must be even and at most the head size %d", rope_dims, k_dim);
    FLLM_REQUIRE(rope_dims == 0 || (cos_table && sin_table && table_positions > 0), "normed_rope_store: rotary tables missing");
    FLLM_REQUIRE(key_chunk > 0 && k_dim % key_chunk == 0, "normed_rope_store: keys of %d values in chunks of %d", k_dim, key_chunk);
    FLLM_REQUIRE(!store_kv || (k_pages && v_pages), "normed_rope_store: pages missing");
    FLLM_REQUIRE(q_out && qkv && row_pos && row_seg && tables && (norm_mode == 0 || (q_weight && k_weight && eps > 0.f)),
                 "normed_rope_store: operands missing");
    if (rows == 0) return 0;
    const size_t smem = (size_t)(heads + kv_heads) * sizeof(float);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(normed_rope_store_kernel<float>, dim3(rows), dim3(kBlock), smem, stream, (const float *)qkv, ld, norm_mode,
                           q_weight, k_weight, eps, (float *)q_out, row_pos, row_seg, tables, table_stride, cos_table, sin_table,
                           (float *)k_pages, (float *)v_pages, heads, kv_heads, k_dim, v_dim, rope_dims, page_size, key_chunk, store_kv,
                           values_from_keys);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(normed_rope_store_kernel<bf16_t>, dim3(rows), dim3(kBlock), smem, stream, (const bf16_t *)qkv, ld, norm_mode,
                           q_weight, k_weight, eps, (bf16_t *)q_out, row_pos, row_seg, tables, table_stride, cos_table, sin_table,
                           (bf16_t *)k_pages, (bf16_t *)v_pages, heads, kv_heads, k_dim, v_dim, rope_dims, page_size, key_chunk,
                           store_kv, values_from_keys);
    else
        FLLM_REQUIRE(false, "normed_rope_store: unknown dtype %d", dtype);
    return fllm_check_launch("normed_rope_store");
}

extern "C" int fllm_pool_blocks(const void *k_pages, const void *v_pages, float *pool_k, float *pool_v, const int32_t *tables,
                                int table_stride, const int32_t *row_pos, const int32_t *row_seg, int rows, int kv_heads, int k_dim,
                                int v_dim, int page_size, int key_chunk, int pool, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && kv_heads > 0 && kv_heads <= 65535 && k_dim > 0 && v_dim > 0 && page_size > 0 && table_stride > 0 && pool > 0,
                 "pool_blocks: bad sizes");
    FLLM_REQUIRE(key_chunk > 0 && k_dim % key_chunk == 0, "pool_blocks: keys of %d values in chunks of %d", k_dim, key_chunk);
    FLLM_REQUIRE(k_pages && v_pages && pool_k && pool_v && tables && row_pos && row_seg, "pool_blocks: operands missing");
    if (rows == 0) return 0;
    const int slots = (page_size + pool - 1) / pool;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(pool_blocks_kernel<float>, dim3(rows, kv_heads), dim3(kBlock), 0, stream, (const float *)k_pages,
                           (const float *)v_pages, pool_k, pool_v, tables, table_stride, row_pos, row_seg, kv_heads, k_dim, v_dim,
                           page_size, key_chunk, pool, slots);
    else if (dtype == FLLM_BF16 && key_chunk == 8 && pool % 8 == 0 && page_size % 8 == 0 &&
             (size_t)(pool / 8) * (k_dim + v_dim) * sizeof(float) <= 48 * 1024)
        hipLaunchKernelGGL(pool_blocks_vec_kernel, dim3(rows, kv_heads), dim3(kBlock), (size_t)(pool / 8) * (k_dim + v_dim) * sizeof(float), stream,
                           (const bf16_t *)k_pages, (const bf16_t *)v_pages, pool_k, pool_v, tables, table_stride, row_pos, row_seg, kv_heads,
                           k_dim, v_dim, page_size, pool, slots);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(pool_blocks_kernel<bf16_t>, dim3(rows, kv_heads), dim3(kBlock), 0, stream, (const bf16_t *)k_pages,
                           (const bf16_t *)v_pages, pool_k, pool_v, tables, table_stride, row_pos, row_seg, kv_heads, k_dim, v_dim,
                           page_size, key_chunk, pool, slots);
    else
        FLLM_REQUIRE(false, "pool_blocks: unknown dtype %d", dtype);
    return fllm_check_launch("pool_blocks");
}

extern "C" int fllm_pooled_window_attention(const void *q, int q_stride, const void *k_pages, const void *v_pages, const float *pool_k,
                                            const float *pool_v, const int32_t *tables, int table_stride, const int32_t *row_pos,
                                            const int32_t *row_seg, const int32_t *seg_start, int num_segs, void *out, int rows,
                                            int heads, int kv_heads, int head_dim, int v_dim, int page_size, float scale, int window,
                                            int pool, int key_chunk, int dtype, int max_context, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && head_dim > 0 && v_dim > 0 && page_size > 0 && table_stride > 0,
                 "pooled_window_attention: bad sizes");
    FLLM_REQUIRE(window > 0 && pool > 0, "pooled_window_attention: a window of %d tokens, blocks of %d", window, pool);
    FLLM_REQUIRE(heads % kv_heads == 0, "pooled_window_attention: %d heads are not a multiple of %d key/value heads", heads, kv_heads);
    FLLM_REQUIRE(key_chunk > 0 && head_dim % key_chunk == 0, "pooled_window_attention: keys of %d lanes in chunks of %d", head_dim, key_chunk);
    FLLM_REQUIRE(v_dim <= kBlock * kMaxLanes, "pooled_window_attention: values of %d lanes a head are more than %d", v_dim, kBlock * kMaxLanes);
    FLLM_REQUIRE(q_stride >= heads * head_dim, "pooled_window_attention: q_stride %d is shorter than heads * head_dim", q_stride);
    FLLM_REQUIRE(q && k_pages && v_pages && pool_k && pool_v && tables && row_pos && row_seg && out, "pooled_window_attention: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_BF16 && key_chunk == 8) {
        const int fast = fllm_pooled_window_attention_bf16_fast(q, q_stride, k_pages, v_pages, pool_k, pool_v, tables, table_stride, row_pos,
                                                                row_seg, seg_start, num_segs, out, rows, heads, kv_heads, head_dim, v_dim,
                                                                page_size, scale, window, pool, max_context, stream);
        if (fast <= 0) return fast;
    }
    const int slots = (page_size + pool - 1) / pool, vd_pad = pow2_lanes(v_dim);
    const size_t smem = (size_t)(((head_dim + 1) & ~1) + kBlock + 2 * ((kWaves + 1) / 2)) * sizeof(float) + (size_t)kBlock * (sizeof(long long) + sizeof(int)) +
                        (size_t)kMaxLanes * kBlock * sizeof(float);
    FLLM_REQUIRE(smem <= 64 * 1024, "pooled_window_attention: heads of %d lanes do not fit into LDS", head_dim);
    const dim3 grid(rows, heads);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(pooled_window_attention_kernel<float>, grid, dim3(kBlock), smem, stream, (const float *)q, q_stride,
                           (const float *)k_pages, (const float *)v_pages, pool_k, pool_v, tables, table_stride, row_pos, row_seg,
                           (float *)out, heads, kv_heads, head_dim, v_dim, page_size, scale, window, pool, slots, key_chunk, vd_pad);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(pooled_window_attention_kernel<bf16_t>, grid, dim3(kBlock), smem, stream, (const bf16_t *)q, q_stride,
                           (const bf16_t *)k_pages, (const bf16_t *)v_pages, pool_k, pool_v, tables, table_stride, row_pos, row_seg,
                           (bf16_t *)out, heads, kv_heads, head_dim, v_dim, page_size, scale, window, pool, slots, key_chunk, vd_pad);
    else
        FLLM_REQUIRE(false, "pooled_window_attention: unknown dtype %d", dtype);
    return fllm_check_launch("pooled_window_attention");
}

extern "C" int fllm_sigmoid_attention(const void *q, int q_stride, const void *k_pages, const void *v_pages, const int32_t *tables,
                                      int table_stride, const int32_t *row_pos, const int32_t *row_seg, const int32_t *seg_start,
                                      int num_segs, void *out, int rows, int heads,
                                      int kv_heads, int head_dim, int v_dim, int page_size, float scale, float softcap, const float *r1,
                                      const float *r2, const float *pb, float temp_coef, int temp_every, int key_chunk, int dtype,
                                      int max_context, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && heads <= 65535 && kv_heads > 0 && head_dim > 0 && v_dim > 0 && page_size > 0 && table_stride > 0,
                 "sigmoid_attention: bad sizes");
    FLLM_REQUIRE(softcap > 0.f && temp_every > 0, "sigmoid_attention: a cap of %g, a temperature step every %d positions", softcap, temp_every);
    FLLM_REQUIRE(heads % kv_heads == 0, "sigmoid_attention: %d heads are not a multiple of %d key/value heads", heads, kv_heads);
    FLLM_REQUIRE(key_chunk > 0 && head_dim % key_chunk == 0, "sigmoid_attention: keys of %d lanes in chunks of %d", head_dim, key_chunk);
    FLLM_REQUIRE(v_dim <= kBlock * kMaxLanes, "sigmoid_attention: values of %d lanes a head are more than %d", v_dim, kBlock * kMaxLanes);
    FLLM_REQUIRE(q_stride >= heads * head_dim, "sigmoid_attention: q_stride %d is shorter than heads * head_dim", q_stride);
    FLLM_REQUIRE(q && k_pages && v_pages && tables && row_pos && row_seg && out && r1 && r2 && pb, "sigmoid_attention: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_BF16 && key_chunk == 8) {
        const int fast = fllm_sigmoid_attention_bf16_fast(q, q_stride, k_pages, v_pages, tables, table_stride, row_pos, row_seg, seg_start,
                                                          num_segs, out, rows, heads, kv_heads, head_dim, v_dim, page_size, scale, softcap,
                                                          r1, r2, pb, temp_coef, temp_every, max_context, stream);
        if (fast <= 0) return fast;
    }
    const int vd_pad = pow2_lanes(v_dim);
    const size_t smem = (size_t)(((head_dim + 1) & ~1) + kBlock) * sizeof(float) + (size_t)kBlock * (sizeof(long long) + sizeof(int)) +
                        (size_t)kMaxLanes * kBlock * sizeof(float);
    FLLM_REQUIRE(smem <= 64 * 1024, "sigmoid_attention: heads of %d lanes do not fit into LDS", head_dim);
    const dim3 grid(rows, heads);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(sigmoid_attention_kernel<float>, grid, dim3(kBlock), smem, stream, (const float *)q, q_stride,
                           (const float *)k_pages, (const float *)v_pages, tables, table_stride, row_pos, row_seg, (float *)out, heads,
                           kv_heads, head_dim, v_dim, page_size, scale, softcap, r1, r2, pb, temp_coef, temp_every, key_chunk, vd_pad);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(sigmoid_attention_kernel<bf16_t>, grid, dim3(kBlock), smem, stream, (const bf16_t *)q, q_stride,
                           (const bf16_t *)k_pages, (const bf16_t *)v_pages, tables, table_stride, row_pos, row_seg, (bf16_t *)out, heads,
                           kv_heads, head_dim, v_dim, page_size, scale, softcap, r1, r2, pb, temp_coef, temp_every, key_chunk, vd_pad);
    else
        FLLM_REQUIRE(false, "sigmoid_attention: unknown dtype %d", dtype);
    return fllm_check_launch("sigmoid_attention");
}

extern "C" int fllm_rotate_scale(const void *qkv, int ld, float *out, const int32_t *row_pos, const float *cos_table,
                                 const float *sin_table, int table_positions, int rows, int heads, int dim, int vdim, int rope_dims,
                                 float key_scale, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && dim > 0 && vdim > 0 && ld >= heads * (2 * dim + vdim), "rotate_scale: bad sizes");
    FLLM_REQUIRE(rope_dims >= 0 && rope_dims <= dim && rope_dims % 2 == 0, "rotate_scale: rope_dims %d must be even and at most %d", rope_dims, dim);
    FLLM_REQUIRE(rope_dims == 0 || (cos_table && sin_table && table_positions > 0), "rotate_scale: rotary tables missing");
    FLLM_REQUIRE(qkv && out && row_pos, "rotate_scale: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(rotate_scale_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, (const float *)qkv, ld, out, row_pos, cos_table,
                           sin_table, table_positions, heads, dim, vdim, rope_dims, key_scale);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(rotate_scale_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, (const bf16_t *)qkv, ld, out, row_pos, cos_table,
                           sin_table, table_positions, heads, dim, vdim, rope_dims, key_scale);
    else
        FLLM_REQUIRE(false, "rotate_scale: unknown dtype %d", dtype);
    return fllm_check_launch("rotate_scale");
}

extern "C" int fllm_group_norm_gate(const void *x, int x_dtype, float eps, int group, const void *gate, int gate_ld, void *out, int rows,
                                    int width, int silu, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && group > 0 && width % group == 0 && gate_ld >= width && eps > 0.f, "group_norm_gate: bad sizes");
    FLLM_REQUIRE(x && gate && out, "group_norm_gate: operands missing");
    if (rows == 0) return 0;
#define FLLM_GROUPED(X, T) hipLaunchKernelGGL((group_norm_gate_kernel<X, T>), dim3(rows), dim3(kBlock), 0, stream, (const X *)x, eps, group, \
                                              (const T *)gate, gate_ld, (T *)out, width, silu)
    if (x_dtype == FLLM_F32 && dtype == FLLM_F32) FLLM_GROUPED(float, float);
    else if (x_dtype == FLLM_F32 && dtype == FLLM_BF16) FLLM_GROUPED(float, bf16_t);
    else if (x_dtype == FLLM_BF16 && dtype == FLLM_BF16) FLLM_GROUPED(bf16_t, bf16_t);
    else FLLM_REQUIRE(false, "group_norm_gate: unknown dtypes %d, %d", x_dtype, dtype);
#undef FLLM_GROUPED
    return fllm_check_launch("group_norm_gate");
}

extern "C" int fllm_weighted_sum(float *out, const float *x, float a, const float *y, float b, size_t total, int accumulate,
                                 hipStream_t stream) {
    FLLM_REQUIRE(out && x && y, "weighted_sum: operands missing");
    if (total == 0) return 0;
    hipLaunchKernelGGL(weighted_sum_kernel, dim3(small_grid(total)), dim3(kBlock), 0, stream, out, x, a, y, b, total, accumulate);
    return fllm_check_launch("weighted_sum");
}

extern "C" int fllm_stream_concat(const float *x, const int32_t *ids, const void *table, int vocab, float scale, void *out, int rows,
                                  int width, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && vocab > 0, "stream_concat: bad sizes");
    FLLM_REQUIRE(x && ids && table && out, "stream_concat: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(stream_concat_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, x, ids, (const float *)table, vocab, scale,
                           (float *)out, width);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(stream_concat_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, x, ids, (const bf16_t *)table, vocab, scale,
                           (bf16_t *)out, width);
    else
        FLLM_REQUIRE(false, "stream_concat: unknown dtype %d", dtype);
    return fllm_check_launch("stream_concat");
}

extern "C" int fllm_relu_squared(const void *x, void *out, size_t total, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(x && out, "relu_squared: operands missing");
    if (total == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(relu_squared_kernel<float>, dim3(small_grid(total)), dim3(kBlock), 0, stream, (const float *)x, (float *)out, total);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(relu_squared_kernel<bf16_t>, dim3(small_grid(total)), dim3(kBlock), 0, stream, (const bf16_t *)x, (bf16_t *)out, total);
    else
        FLLM_REQUIRE(false, "relu_squared: unknown dtype %d", dtype);
    return fllm_check_launch("relu_squared");
}
