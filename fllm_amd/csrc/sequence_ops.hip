// Mechanisms that carry something from one token of a sequence to the next outside the pages, and the small kernels around
// them.  These are the plain kernels: float32 arithmetic in a fixed order, both element types, any sizes.  A row's result
// depends on its own sequence alone, never on the rest of the batch.
//
//   short_conv          y_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j): a causal convolution over time on every channel, the
//                       last taps - 1 inputs of a sequence kept in its state slot.
//   linear_attention    S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, S float32 [dim][vdim] in the sequence's
//                       state slot; q, k and v pass through an activation on the way in.  Token after token, the state in
//                       registers (values in groups of four lanes) or in LDS (any sizes).
//   gated_norm          out = x * rsqrt(mean x^2 + eps) * w * sigmoid(gate) (w absent: out = x * sigmoid(gate)).
//   polynorm            out = a N(z) + b N(z^2) + c N(z^3) + e, N the division by a row's root mean square.
//   head_norm_kv_store  q and k divided by their root mean square over a head's lanes, k and v stored into the pages.
#include "api.h"
#include "common.h"

int fllm_linear_attention_chunked(const void *q, const void *k, const void *v, int ld, const float *decay_hi, const float *decay_lo,
                                  float *state, const int32_t *row_seg, const int32_t *seg_start, const int32_t *slots, int num_segs,
                                  float *out, int rows, int heads, int dim, int vdim, int activation, int dtype, float *carried,
                                  hipStream_t stream);   // linear_attention_mfma.hip; 1: sizes declined

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float activate(float z, int activation) { return activation == 1 ? z * sigmoid_f(z) : z; }

// ---- short convolution ----------------------------------------------------------------------------------------------------
// One workgroup a row (a step of prompts has rows enough to fill the device; the loop takes any number of blocks of channels
// a row).  The input `d` tokens back is a row of this step while the step holds it, else an entry of the state:
// state[slot][i] is the input at position (tokens before this step) - (taps - 1) + i, zeros before the sequence's start.
template <typename T>
__global__ void __launch_bounds__(kBlock)
short_conv_kernel(const T *__restrict__ x, const float *__restrict__ w, const T *__restrict__ state, const int32_t *__restrict__ row_seg,
                  const int32_t *__restrict__ seg_start, const int32_t *__restrict__ slots, T *__restrict__ out, int width, int taps) {
    const int r = blockIdx.x;
    const int seg = row_seg[r];
    if (seg < 0) {   // padding row
        for (int c = blockIdx.y * kBlock + threadIdx.x; c < width; c += gridDim.y * kBlock) out[(size_t)r * width + c] = from_f32<T>(0.f);
        return;
    }
    const int t = r - seg_start[seg];
    const T *mine = state + (size_t)slots[seg] * (taps - 1) * width;
    for (int c = blockIdx.y * kBlock + threadIdx.x; c < width; c += gridDim.y * kBlock) {      // one channel a thread
        const float *wc = w + (size_t)c * taps;
        const float now = to_f32<T>(x[(size_t)r * width + c]);
        float acc = 0.f;
        for (int d = taps - 1; d >= 1; d--) {     // oldest input first
            const int at = t - d;
            const float v = at >= 0 ? to_f32<T>(x[(size_t)(r - d) * width + c]) : to_f32<T>(mine[(size_t)(taps - 1 + at) * width + c]);
            acc = fmaf(wc[taps - 1 - d], v, acc);
        }
        acc = fmaf(wc[taps - 1], now, acc);
        out[(size_t)r * width + c] = from_f32<T>(now + acc);
    }
}

// One workgroup a segment and block of channels, after the rows have been computed: the state becomes the last taps - 1 inputs of the sequence.
// A thread owns a channel: it reads what it keeps of the old entries before it writes any.
constexpr int kMaxKeep = 15;
template <typename T>
__global__ void __launch_bounds__(kBlock)
short_conv_state_kernel(const T *__restrict__ x, T *__restrict__ state, const int32_t *__restrict__ row_seg,
                        const int32_t *__restrict__ seg_start, const int32_t *__restrict__ slots, int width, int taps) {
    const int seg = blockIdx.x;
    const int r0 = seg_start[seg], n = seg_start[seg + 1] - r0;
    if (n <= 0 || row_seg[r0] < 0) return;   // nothing of this segment in the step, or padding rows
    const int keep = taps - 1;
    T *mine = state + (size_t)slots[seg] * keep * width;
    for (int c = blockIdx.y * kBlock + threadIdx.x; c < width; c += gridDim.y * kBlock) {      // one channel a thread
        T held[kMaxKeep];
#pragma unroll
        for (int i = 0; i < kMaxKeep; i++) {
            if (i >= keep) break;
            const int at = n - keep + i;      // index among the step's rows; negative: an old entry
            held[i] = at >= 0 ? x[(size_t)(r0 + at) * width + c] : mine[(size_t)(keep + at) * width + c];
        }
#pragma unroll
        for (int i = 0; i < kMaxKeep; i++) {
            if (i >= keep) break;
            mine[(size_t)i * width + c] = held[i];
        }
    }
}

// The norm before the convolution and the convolution in one pass, for steps of one row a segment: one workgroup a row and
// block of kBlock channels; every workgroup of a row sums the row's squares itself (in the norm kernel's order), so that no
// thread loops over channels and all it reads is on its way at once.  The normed value is rounded to T before it is used, as
// the norm kernel's output would be, so that a token gives the same bits whether it came alone or in a portion.  A thread
// owns a channel of the state: it reads the old entries before it writes any.
template <typename T>
__global__ void __launch_bounds__(kBlock)
norm_short_conv_kernel(const float *__restrict__ x, const float *__restrict__ norm_w, float eps, const float *__restrict__ w,
                       T *__restrict__ state, const int32_t *__restrict__ row_seg, const int32_t *__restrict__ slots,
                       T *__restrict__ out, int width, int taps) {
    __shared__ float scratch[kWaves];
    const int r = blockIdx.x;
    const int c = blockIdx.y * kBlock + threadIdx.x;
    const int seg = row_seg[r];
    if (seg < 0) {   // padding row
        if (c < width) out[(size_t)r * width + c] = from_f32<T>(0.f);
        return;
    }
    const float *src = x + (size_t)r * width;
    float ss = 0.f;
    for (int i0 = threadIdx.x; i0 < width; i0 += 4 * kBlock) {      // four loads on their way at once, summed in the row's order
        float a[4];
#pragma unroll
        for (int j = 0; j < 4; j++) a[j] = i0 + j * kBlock < width ? src[i0 + j * kBlock] : 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) ss = fmaf(a[j], a[j], ss);
    }
    ss = block_sum<kWaves>(ss, scratch);
    if (c >= width) return;
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    const int keep = taps - 1;
    T *mine = state + (size_t)slots[seg] * keep * width;
    const float *wc = w + (size_t)c * taps;
    T held[kMaxKeep];
#pragma unroll
    for (int i = 0; i < kMaxKeep; i++)
        if (i < keep) held[i] = mine[(size_t)i * width + c];
    const T h = from_f32<T>(src[c] * (inv * norm_w[c]));
    const float now = to_f32<T>(h);
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxKeep; i++) {      // oldest input first; entry i moves to i - 1
        if (i >= keep) break;
        acc = fmaf(wc[i], to_f32<T>(held[i]), acc);
        if (i > 0) mine[(size_t)(i - 1) * width + c] = held[i];
    }
    if (keep > 0) mine[(size_t)(keep - 1) * width + c] = h;
    acc = fmaf(wc[taps - 1], now, acc);
    out[(size_t)r * width + c] = from_f32<T>(now + acc);
}

// ---- linear attention, one token after the other ----------------------------------------------------------------------------
// One workgroup a (segment, head, slice of VB value lanes).  The slice of the state lives in LDS while the segment's tokens
// pass: thread (g, j) owns rows g, g + G, .. of column j.  The decay is given as a float pair (hi + lo) so that its
// power over a thousand tokens is that of the number the file gives, not of its rounding.
template <typename T>
__global__ void __launch_bounds__(kBlock)
linear_attention_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, int ld,
                        const float *__restrict__ decay_hi, const float *__restrict__ decay_lo, float *__restrict__ state,
                        const int32_t *__restrict__ row_seg, const int32_t *__restrict__ seg_start,
                        const int32_t *__restrict__ slots, float *__restrict__ out, int heads, int dim, int vdim, int VB,
                        int activation) {
    extern __shared__ float smem[];
    const int G = kBlock / VB;
    float *S = smem;                    // dim * VB
    float *qs = S + (size_t)dim * VB;   // dim
    float *ks = qs + dim;               // dim
    float *part = ks + dim;             // G * VB
    const int seg = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * VB;
    const int r0 = seg_start[seg], n = seg_start[seg + 1] - r0;
    if (n <= 0) return;
    const int j = threadIdx.x % VB, g = threadIdx.x / VB;
    const bool live = j0 + j < vdim;
    if (row_seg[r0] < 0) {   // padding rows: no state is touched
        if (g == 0 && live)
            for (int t = 0; t < n; t++) out[((size_t)(r0 + t) * heads + h) * vdim + j0 + j] = 0.f;
        return;
    }
    float *mine = state + ((size_t)slots[seg] * heads + h) * dim * vdim;
    for (int i = g; i < dim; i += G) S[i * VB + j] = live ? mine[(size_t)i * vdim + j0 + j] : 0.f;
    const float dh = decay_hi[h], dl = decay_lo[h];
    for (int t = 0; t < n; t++) {
        const size_t row = (size_t)(r0 + t) * ld;
        __syncthreads();      // the step before has read qs, ks and part
        for (int c = threadIdx.x; c < dim; c += kBlock) {
            qs[c] = activate(to_f32<T>(q[row + (size_t)h * dim + c]), activation);
            ks[c] = activate(to_f32<T>(k[row + (size_t)h * dim + c]), activation);
        }
        const float vj = live ? activate(to_f32<T>(v[row + (size_t)h * vdim + j0 + j]), activation) : 0.f;
        __syncthreads();
        float acc = 0.f;
        for (int i = g; i < dim; i += G) {
            float s = S[i * VB + j];
            s = fmaf(s, dh, fmaf(s, dl, ks[i] * vj));
            S[i * VB + j] = s;
            acc = fmaf(s, qs[i], acc);
        }
        part[g * VB + j] = acc;
        __syncthreads();
        if (g == 0 && live) {
            float o = part[j];
            for (int a = 1; a < G; a++) o += part[a * VB + j];
            out[((size_t)(r0 + t) * heads + h) * vdim + j0 + j] = o;
        }
    }
    if (live)
        for (int i = g; i < dim; i += G) mine[(size_t)i * vdim + j0 + j] = S[i * VB + j];
}

// The same recurrence with the state in registers, for values in groups of four lanes and keys of up to 32 * RP lanes: one
// workgroup a (segment, head, slice of 32 value lanes), thread (g, j4) owns rows g, g + 32, .. of the four columns at 4 * j4.
// The state is read once, 16 bytes a thread and 128 bytes a row, and written once behind the segment's last token, which is
// all a decode step does; the sum over the rows is taken over the lanes of a wave and then over the four waves, in an order
// that no size of the batch changes.
constexpr int kRowsVB = 32;
template <typename T, int RP>
__global__ void __launch_bounds__(kBlock)
linear_attention_rows_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, int ld,
                             const float *__restrict__ decay_hi, const float *__restrict__ decay_lo, float *__restrict__ state,
                             const int32_t *__restrict__ row_seg, const int32_t *__restrict__ seg_start,
                             const int32_t *__restrict__ slots, float *__restrict__ out, int heads, int dim, int vdim,
                             int activation) {
    constexpr int G = kBlock / (kRowsVB / 4);      // 32 groups of rows
    __shared__ float qs[G * RP], ks[G * RP];
    __shared__ f32x4_t part[kWaves][kRowsVB / 4];
    const int seg = blockIdx.x, h = blockIdx.y, j0 = blockIdx.z * kRowsVB;
    const int r0 = seg_start[seg], n = seg_start[seg + 1] - r0;
    if (n <= 0) return;
    const int tid = threadIdx.x, j4 = tid & 7, g = tid >> 3;
    const int col = j0 + 4 * j4;
    const bool live = col < vdim;
    const size_t out_ld = (size_t)heads * vdim;
    if (row_seg[r0] < 0) {   // padding rows: no state is touched
        if (g == 0 && live)
            for (int t = 0; t < n; t++) *(f32x4_t *)(out + (size_t)(r0 + t) * out_ld + (size_t)h * vdim + col) = f32x4_t{0.f, 0.f, 0.f, 0.f};
        return;
    }
    float *mine = state + ((size_t)slots[seg] * heads + h) * dim * vdim;
    f32x4_t S[RP];
#pragma unroll
    for (int p = 0; p < RP; p++) {
        const int i = g + G * p;
        S[p] = (live && i < dim) ? *(const f32x4_t *)(mine + (size_t)i * vdim + col) : f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    const float dh = decay_hi[h], dl = decay_lo[h];
    for (int t = 0; t < n; t++) {
        const size_t row = (size_t)(r0 + t) * ld;
        if (t > 0) __syncthreads();      // the token before has read qs, ks and part
        for (int c = tid; c < dim; c += kBlock) {
            qs[c] = activate(to_f32<T>(q[row + (size_t)h * dim + c]), activation);
            ks[c] = activate(to_f32<T>(k[row + (size_t)h * dim + c]), activation);
        }
        f32x4_t vv = {0.f, 0.f, 0.f, 0.f};
        if (live)
#pragma unroll
            for (int e = 0; e < 4; e++) vv[e] = activate(to_f32<T>(v[row + (size_t)h * vdim + col + e]), activation);
        __syncthreads();
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < RP; p++) {
            const int i = g + G * p;
            if (i < dim) {
                const float kk = ks[i], qq = qs[i];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float s = S[p][e];
                    s = fmaf(s, dh, fmaf(s, dl, kk * vv[e]));
                    S[p][e] = s;
                    acc[e] = fmaf(s, qq, acc[e]);
                }
            }
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {      // the eight row groups of a wave: lanes 8, 16 and 32 apart hold the same columns
            acc[e] += __shfl_xor(acc[e], 8, kWave);
            acc[e] += __shfl_xor(acc[e], 16, kWave);
            acc[e] += __shfl_xor(acc[e], 32, kWave);
        }
        if ((tid & (kWave - 1)) < 8) part[tid / kWave][j4] = acc;
        __syncthreads();
        if (tid < 8 && live) {
            f32x4_t o = part[0][tid];
#pragma unroll
            for (int a = 1; a < kWaves; a++) o += part[a][tid];
            *(f32x4_t *)(out + (size_t)(r0 + t) * out_ld + (size_t)h * vdim + col) = o;
        }
    }
    if (live)
#pragma unroll
        for (int p = 0; p < RP; p++) {
            const int i = g + G * p;
            if (i < dim) *(f32x4_t *)(mine + (size_t)i * vdim + col) = S[p];
        }
}

// ---- gated norm ---------------------------------------------------------------------------------------------------------------
template <typename X, typename T>
__global__ void __launch_bounds__(kBlock)
gated_norm_kernel(const X *__restrict__ x, const float *__restrict__ w, float eps, const T *__restrict__ gate, int gate_ld,
                  T *__restrict__ out, int width) {
    __shared__ float scratch[kWaves];
    const size_t r = blockIdx.x;
    const X *src = x + r * width;
    float inv = 1.0f;
    if (w != nullptr) {
        float ss = 0.f;
        // four loads on their way at once: a row is a few values a thread and waits for memory, not for arithmetic
        for (int c0 = threadIdx.x; c0 < width; c0 += 4 * kBlock) {
            float a[4];
#pragma unroll
            for (int j = 0; j < 4; j++) a[j] = c0 + j * kBlock < width ? to_f32<X>(src[c0 + j * kBlock]) : 0.f;
#pragma unroll
            for (int j = 0; j < 4; j++) ss = fmaf(a[j], a[j], ss);
        }
        ss = block_sum<kWaves>(ss, scratch);
        inv = 1.0f / sqrtf(ss / (float)width + eps);
    }
#pragma unroll 8
    for (int c = threadIdx.x; c < width; c += kBlock) {
        float a = to_f32<X>(src[c]) * inv;
        if (w != nullptr) a *= w[c];
        out[r * width + c] = from_f32<T>(a * sigmoid_f(to_f32<T>(gate[r * gate_ld + c])));
    }
}

// ---- polynomial activation with normed powers -----------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(kBlock)
polynorm_kernel(const T *__restrict__ z, int ld, const float *__restrict__ coeffs, float eps, T *__restrict__ out, int width) {
    __shared__ float scratch[kWaves];
    const size_t r = blockIdx.x;
    const T *src = z + r * ld;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll 8      // eight loads on their way at once
    for (int c = threadIdx.x; c < width; c += kBlock) {
        const float a = to_f32<T>(src[c]), a2 = a * a, a3 = a2 * a;
        s2 += a2;
        s4 = fmaf(a2, a2, s4);
        s6 = fmaf(a3, a3, s6);
    }
    s2 = block_sum<kWaves>(s2, scratch);
    s4 = block_sum<kWaves>(s4, scratch);
    s6 = block_sum<kWaves>(s6, scratch);
    const float n = (float)width;
    const float c1 = coeffs[0] / sqrtf(s2 / n + eps), c2 = coeffs[1] / sqrtf(s4 / n + eps), c3 = coeffs[2] / sqrtf(s6 / n + eps);
    const float c0 = coeffs[3];
#pragma unroll 8
    for (int c = threadIdx.x; c < width; c += kBlock) {
        const float a = to_f32<T>(src[c]);
        out[r * width + c] = from_f32<T>(fmaf(a, fmaf(a, fmaf(a, c3, c2), c1), c0));
    }
}

// ---- q and k normed a head, k and v into the pages ---------------------------------------------------------------------------------
// One workgroup a row of [q | k | v | ..] (row stride ld); a wave takes a head at a time.  The mean is over `norm_dim` lanes
// (heads widened with zero lanes keep the mean of their own lanes).
template <typename T>
__global__ void __launch_bounds__(kBlock)
head_norm_kv_store_kernel(T *__restrict__ qkv, int ld, float eps, int norm_dim, const int32_t *__restrict__ row_pos,
                          const int32_t *__restrict__ row_seg, const int32_t *__restrict__ tables, int table_stride,
                          T *__restrict__ k_pages, T *__restrict__ v_pages, int heads, int kv_heads, int head_dim, int v_dim,
                          int page_size, int key_chunk, int store_kv) {
    const int r = blockIdx.x;
    const int seg = row_seg[r];
    if (seg < 0) return;   // padding row
    const int pos = row_pos[r];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    T *row = qkv + (size_t)r * ld;
    int page = 0, off = 0;
    if (store_kv) {
        page = tables[(size_t)seg * table_stride + pos / page_size];
        off = pos % page_size;
    }
    const int normed = store_kv ? heads + kv_heads : heads;
    for (int h = wave; h < normed; h += kWaves) {
        T *head = row + (size_t)h * head_dim;
        float ss = 0.f;
        for (int c = lane; c < head_dim; c += kWave) {
            const float a = to_f32<T>(head[c]);
            ss = fmaf(a, a, ss);
        }
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)norm_dim + eps);
        for (int c = lane; c < head_dim; c += kWave) {
            const T y = from_f32<T>(to_f32<T>(head[c]) * inv);
            if (h < heads) head[c] = y;
            else k_pages[key_offset_chunked(page, kv_heads, h - heads, page_size, head_dim, off, c, key_chunk)] = y;
        }
    }
    if (!store_kv) return;
    const T *vrow = row + (size_t)(heads + kv_heads) * head_dim;
    for (int i = threadIdx.x; i < kv_heads * v_dim; i += kBlock) {
        const int h = i / v_dim, c = i - h * v_dim;
        v_pages[(((size_t)page * kv_heads + h) * v_dim + c) * page_size + off] = vrow[i];
    }
}

}  // namespace

extern "C" int fllm_short_conv(const void *x, const float *w, void *state, const int32_t *row_seg, const int32_t *seg_start,
                               const int32_t *slots, int num_segs, void *out, int rows, int width, int taps, int dtype,
                               hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && num_segs > 0, "short_conv: bad sizes");
    FLLM_REQUIRE(taps >= 1 && taps - 1 <= kMaxKeep, "short_conv: %d taps are outside 1..%d", taps, kMaxKeep + 1);
    FLLM_REQUIRE(x && w && out && row_seg && seg_start && slots && (state || taps == 1), "short_conv: operands missing");
    if (rows == 0) return 0;
    const int blocks = (width + kBlock - 1) / kBlock < 65535 ? (width + kBlock - 1) / kBlock : 65535;      // blocks of channels
    if (dtype == FLLM_F32) {
        hipLaunchKernelGGL(short_conv_kernel<float>, dim3(rows, 1), dim3(kBlock), 0, stream, (const float *)x, w, (const float *)state,
                           row_seg, seg_start, slots, (float *)out, width, taps);
        if (taps > 1)
            hipLaunchKernelGGL(short_conv_state_kernel<float>, dim3(num_segs, blocks), dim3(kBlock), 0, stream, (const float *)x,
                               (float *)state, row_seg, seg_start, slots, width, taps);
    } else if (dtype == FLLM_BF16) {
        hipLaunchKernelGGL(short_conv_kernel<bf16_t>, dim3(rows, 1), dim3(kBlock), 0, stream, (const bf16_t *)x, w, (const bf16_t *)state,
                           row_seg, seg_start, slots, (bf16_t *)out, width, taps);
        if (taps > 1)
            hipLaunchKernelGGL(short_conv_state_kernel<bf16_t>, dim3(num_segs, blocks), dim3(kBlock), 0, stream, (const bf16_t *)x,
                               (bf16_t *)state, row_seg, seg_start, slots, width, taps);
    } else
        FLLM_REQUIRE(false, "short_conv: unknown dtype %d", dtype);
    return fllm_check_launch("short_conv");
}

extern "C" int fllm_norm_short_conv(const float *x, const float *norm_w, float eps, const float *w, void *state, const int32_t *row_seg,
                                    const int32_t *slots, void *out, int rows, int width, int taps, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && taps >= 1 && taps - 1 <= kMaxKeep && eps > 0.f, "norm_short_conv: bad sizes");
    FLLM_REQUIRE(x && norm_w && w && out && row_seg && slots && (state || taps == 1), "norm_short_conv: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(norm_short_conv_kernel<float>, dim3(rows, (width + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, x, norm_w, eps, w, (float *)state, row_seg,
                           slots, (float *)out, width, taps);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(norm_short_conv_kernel<bf16_t>, dim3(rows, (width + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, x, norm_w, eps, w, (bf16_t *)state, row_seg,
                           slots, (bf16_t *)out, width, taps);
    else
        FLLM_REQUIRE(false, "norm_short_conv: unknown dtype %d", dtype);
    return fllm_check_launch("norm_short_conv");
}

extern "C" int fllm_linear_attention(const void *q, const void *k, const void *v, int ld, const float *decay_hi, const float *decay_lo,
                                     float *state, const int32_t *row_seg, const int32_t *seg_start, const int32_t *slots,
                                     int num_segs, float *out, int rows, int heads, int dim, int vdim, int activation, int form,
                                     int dtype, float *carried, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && dim > 0 && vdim > 0 && num_segs > 0 && ld > 0, "linear_attention: bad sizes");
    FLLM_REQUIRE(q && k && v && decay_hi && decay_lo && state && row_seg && seg_start && slots && out, "linear_attention: operands missing");
    FLLM_REQUIRE(activation == 0 || activation == 1, "linear_attention: unknown activation %d", activation);
    FLLM_REQUIRE(heads <= 65535, "linear_attention: too many heads");
    FLLM_REQUIRE(form >= 0 && form <= 2, "linear_attention: unknown form %d", form);
    FLLM_REQUIRE(dtype == FLLM_F32 || dtype == FLLM_BF16, "linear_attention: unknown dtype %d", dtype);
    if (rows == 0) return 0;
    // a step that holds more rows than segments holds portions of prompts: those go over the matrix cores a chunk at a time
    if (form == 2 || (form == 0 && rows > num_segs)) {
        const int declined = fllm_linear_attention_chunked(q, k, v, ld, decay_hi, decay_lo, state, row_seg, seg_start, slots, num_segs,
                                                           out, rows, heads, dim, vdim, activation, dtype, carried, stream);
        if (!declined) return fllm_check_launch("linear_attention_chunked");
        FLLM_REQUIRE(form != 2, "linear_attention: heads of %d and %d lanes are not the chunked kernel's", dim, vdim);
    }
    // values in groups of four lanes: the state passes through registers
    if (vdim % 4 == 0 && dim <= 256) {
        const dim3 grid(num_segs, heads, (vdim + kRowsVB - 1) / kRowsVB);
#define FLLM_ROWS(T, RP)                                                                                                          \
    hipLaunchKernelGGL((linear_attention_rows_kernel<T, RP>), grid, dim3(kBlock), 0, stream, (const T *)q, (const T *)k,          \
                       (const T *)v, ld, decay_hi, decay_lo, state, row_seg, seg_start, slots, out, heads, dim, vdim, activation)
#define FLLM_ROWS_OF(T)                                                                                                           \
    do {                                                                                                                          \
        if (dim <= 32) FLLM_ROWS(T, 1);                                                                                           \
        else if (dim <= 64) FLLM_ROWS(T, 2);                                                                                      \
        else if (dim <= 128) FLLM_ROWS(T, 4);                                                                                     \
        else FLLM_ROWS(T, 8);                                                                                                     \
    } while (0)
        if (dtype == FLLM_F32) FLLM_ROWS_OF(float);
        else FLLM_ROWS_OF(bf16_t);
#undef FLLM_ROWS_OF
#undef FLLM_ROWS
        return fllm_check_launch("linear_attention_rows");
    }
    // the widest slice of value lanes whose share of the state fits into LDS beside q, k and the partial sums
    int VB = 64;
    while (VB / 2 >= vdim && VB > 1) VB >>= 1;
    while (VB > 1 && ((size_t)dim * VB + 2 * (size_t)dim + kBlock) * sizeof(float) > 64 * 1024) VB >>= 1;
    const size_t smem = ((size_t)dim * VB + 2 * (size_t)dim + kBlock) * sizeof(float);
    FLLM_REQUIRE(smem <= 64 * 1024, "linear_attention: keys of %d lanes do not fit into LDS", dim);
    const int slices = (vdim + VB - 1) / VB;
    FLLM_REQUIRE(slices <= 65535, "linear_attention: values of %d lanes are too many", vdim);
    const dim3 grid(num_segs, heads, slices);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(linear_attention_kernel<float>, grid, dim3(kBlock), smem, stream, (const float *)q, (const float *)k,
                           (const float *)v, ld, decay_hi, decay_lo, state, row_seg, seg_start, slots, out, heads, dim, vdim, VB, activation);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(linear_attention_kernel<bf16_t>, grid, dim3(kBlock), smem, stream, (const bf16_t *)q, (const bf16_t *)k,
                           (const bf16_t *)v, ld, decay_hi, decay_lo, state, row_seg, seg_start, slots, out, heads, dim, vdim, VB, activation);
    else
        FLLM_REQUIRE(false, "linear_attention: unknown dtype %d", dtype);
    return fllm_check_launch("linear_attention");
}

extern "C" int fllm_gated_norm(const void *x, int x_dtype, const float *w, float eps, const void *gate, int gate_ld, void *out, int rows,
                               int width, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && gate_ld >= width, "gated_norm: bad sizes");
    FLLM_REQUIRE(x && gate && out, "gated_norm: operands missing");
    if (rows == 0) return 0;
#define FLLM_GATED(X, T) hipLaunchKernelGGL((gated_norm_kernel<X, T>), dim3(rows), dim3(kBlock), 0, stream, (const X *)x, w, eps, \
                                            (const T *)gate, gate_ld, (T *)out, width)
    if (x_dtype == FLLM_F32 && dtype == FLLM_F32) FLLM_GATED(float, float);
    else if (x_dtype == FLLM_F32 && dtype == FLLM_BF16) FLLM_GATED(float, bf16_t);
    else if (x_dtype == FLLM_BF16 && dtype == FLLM_BF16) FLLM_GATED(bf16_t, bf16_t);
    else FLLM_REQUIRE(false, "gated_norm: unknown dtypes %d, %d", x_dtype, dtype);
#undef FLLM_GATED
    return fllm_check_launch("gated_norm");
}

extern "C" int fllm_polynorm(const void *z, int ld, const float *coeffs, float eps, void *out, int rows, int width, int dtype,
                             hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && ld >= width, "polynorm: bad sizes");
    FLLM_REQUIRE(z && coeffs && out, "polynorm: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(polynorm_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, (const float *)z, ld, coeffs, eps, (float *)out, width);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(polynorm_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, (const bf16_t *)z, ld, coeffs, eps, (bf16_t *)out,
                           width);
    else
        FLLM_REQUIRE(false, "polynorm: unknown dtype %d", dtype);
    return fllm_check_launch("polynorm");
}

extern "C" int fllm_head_norm_kv_store(void *qkv, int ld, float eps, int norm_dim, const int32_t *row_pos, const int32_t *row_seg,
                                       const int32_t *tables, int table_stride, void *k_pages, void *v_pages, int rows, int heads,
                                       int kv_heads, int head_dim, int v_dim, int page_size, int key_chunk, int dtype, int store_kv,
                                       hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && v_dim > 0 && page_size > 0 && table_stride > 0,
                 "head_norm_kv_store: bad sizes");
    FLLM_REQUIRE(norm_dim > 0 && norm_dim <= head_dim && eps > 0.f, "head_norm_kv_store: a mean over %d of %d lanes", norm_dim, head_dim);
    FLLM_REQUIRE(ld >= (heads + kv_heads) * head_dim + kv_heads * v_dim, "head_norm_kv_store: rows of %d values are too short", ld);
    FLLM_REQUIRE(key_chunk > 0 && head_dim % key_chunk == 0, "head_norm_kv_store: keys of %d lanes cannot lie in chunks of %d", head_dim,
                 key_chunk);
    FLLM_REQUIRE(qkv && row_pos && row_seg && tables && (!store_kv || (k_pages && v_pages)), "head_norm_kv_store: operands missing");
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(head_norm_kv_store_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, (float *)qkv, ld, eps, norm_dim, row_pos,
                           row_seg, tables, table_stride, (float *)k_pages, (float *)v_pages, heads, kv_heads, head_dim, v_dim, page_size,
                           key_chunk, store_kv);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(head_norm_kv_store_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, (bf16_t *)qkv, ld, eps, norm_dim, row_pos,
                           row_seg, tables, table_stride, (bf16_t *)k_pages, (bf16_t *)v_pages, heads, kv_heads, head_dim, v_dim,
                           page_size, key_chunk, store_kv);
    else
        FLLM_REQUIRE(false, "head_norm_kv_store: unknown dtype %d", dtype);
    return fllm_check_launch("head_norm_kv_store");
}
