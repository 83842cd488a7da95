// Small kernels on the residual stream and around the feed-forward that the dense decoder's own kernels do not
// cover: two RMSNorms of one row in one pass (blocks whose branches read the same stream), a gated activation with
// clamped operands, a vector and the embedding added to the stream between passes of looped layers, and logits times
// a constant.  All arithmetic is float32; the element type only says how operands are stored.
#include "api.h"
#include "common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

// One workgroup a row.  The sum of squares is added in a fixed order (thread t its columns t, t + 256, ..., then
// lanes, then waves): a row gives the same bits whatever else is in the batch.  Both norms share the sum.
template <typename T>
__global__ void __launch_bounds__(kBlock)
rmsnorm_pair_kernel(const float *__restrict__ x, const float *__restrict__ w1, const float *__restrict__ w2,
                    T *__restrict__ out1, T *__restrict__ out2, int width, float eps1, float eps2) {
    __shared__ float scratch[kWaves];
    const size_t r = blockIdx.x;
    const float *src = x + r * width;
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += kBlock) ss += src[c] * src[c];
    ss = block_sum<kWaves>(ss, scratch);
    const float mean = ss / (float)width;
    const float inv1 = 1.0f / sqrtf(mean + eps1), inv2 = 1.0f / sqrtf(mean + eps2);
    for (int c = threadIdx.x; c < width; c += kBlock) {
        const float v = src[c];
        out1[r * width + c] = from_f32<T>(v * inv1 * w1[c]);
        if (out2 != nullptr) out2[r * width + c] = from_f32<T>(v * inv2 * w2[c]);
    }
}

// out = a(g) * (u + up_offset) with g = min(gate, limit), u = clamp(up, -limit, limit) (limit <= 0: neither is
// clamped) and a(g) = g * sigmoid(alpha * g)
template <typename T>
__global__ void __launch_bounds__(kBlock)
glu_clamped_kernel(const T *__restrict__ gu, T *__restrict__ out, int inter, float limit, float alpha, float up_offset) {
    const size_t r = blockIdx.y;
    const T *g = gu + r * 2 * inter, *u = g + inter;
    T *o = out + r * inter;
    const int c = blockIdx.x * kBlock + threadIdx.x;
    if (c >= inter) return;
    float gf = to_f32<T>(g[c]), uf = to_f32<T>(u[c]);
    if (limit > 0.f) {
        gf = fminf(gf, limit);
        uf = fminf(fmaxf(uf, -limit), limit);
    }
    o[c] = from_f32<T>(gf / (1.0f + expf(-alpha * gf)) * (uf + up_offset));
}

// the same for bfloat16 rows whose width is a multiple of 8: a thread takes 8 neighbours, 16 bytes of gate and of up
__global__ void __launch_bounds__(kBlock)
glu_clamped_vec_kernel(const bf16_t *__restrict__ gu, bf16_t *__restrict__ out, int inter, float limit, float alpha, float up_offset) {
    const size_t r = blockIdx.y;
    const int c = (blockIdx.x * kBlock + threadIdx.x) * 8;
    if (c >= inter) return;
    const bf16x8_t g8 = *(const bf16x8_t *)(gu + r * 2 * inter + c), u8 = *(const bf16x8_t *)(gu + r * 2 * inter + inter + c);
    bf16x8_t o8;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        float gf = (float)g8[e], uf = (float)u8[e];
        if (limit > 0.f) {
            gf = fminf(gf, limit);
            uf = fminf(fmaxf(uf, -limit), limit);
        }
        o8[e] = (bf16_t)(gf / (1.0f + expf(-alpha * gf)) * (uf + up_offset));
    }
    *(bf16x8_t *)(out + r * inter + c) = o8;
}

__global__ void __launch_bounds__(kBlock) scale_kernel(float *__restrict__ x, size_t total, float scale) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock) x[i] *= scale;
}

// x[r, :] = (x[r, :] + scale * table[ids[r], :]) + vec[:]; either addend may be absent
template <typename T>
__global__ void __launch_bounds__(kBlock)
stream_add_kernel(float *__restrict__ x, const int32_t *__restrict__ ids, const T *__restrict__ table, int vocab, float scale,
                  const float *__restrict__ vec, int width) {
    const size_t r = blockIdx.x;
    const T *src = nullptr;
    if (table != nullptr) {
        int id = ids[r];
        id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // ids are validated on the host; never read outside the table
        src = table + (size_t)id * width;
    }
    float *dst = x + r * width;
    for (int c = threadIdx.x; c < width; c += kBlock) {
        float v = dst[c];
        if (src != nullptr) v += to_f32<T>(src[c]) * scale;
        if (vec != nullptr) v += vec[c];
        dst[c] = v;
    }
}

// A branch that is normed on its way into the stream: v = sum of the row's `parts` partial branches (in index order),
// x[r] += v * rsqrt(mean(v^2) + eps) * gain (normalize 0: x[r] += v * gain).  `gain` is whatever multiplies the normed
// branch lane by lane: the norm's weight, a layer scale and the constant of the residual sum in one vector.  With
// `next_w`, the RMSNorm of the new row (its own eps) is written to `next_out` as well, the norm that reads the stream
// next.  One workgroup a row, sums in a fixed order: a row gives the same bits whatever else is in the batch.
template <typename B, typename T>
__global__ void __launch_bounds__(kBlock)
postnorm_add_kernel(float *__restrict__ x, const B *__restrict__ branch, int parts, const float *__restrict__ part_weights,
                    const float *__restrict__ gain, float eps, int normalize, const float *__restrict__ next_w, float next_eps, T *__restrict__ next_out, int width) {
    __shared__ float scratch[kWaves];
    const size_t r = blockIdx.x;
    const B *src = branch + r * parts * width;
    float *dst = x + r * width;
    const float *pw = part_weights == nullptr ? nullptr : part_weights + r * parts;      // a weight a partial row
    auto value = [&](int c) {
        if (pw != nullptr) {
            float v = to_f32<B>(src[c]) * pw[0];
            for (int k = 1; k < parts; k++) v = fmaf(to_f32<B>(src[(size_t)k * width + c]), pw[k], v);
            return v;
        }
        float v = to_f32<B>(src[c]);
        for (int k = 1; k < parts; k++) v += to_f32<B>(src[(size_t)k * width + c]);
        return v;
    };
    float inv = 1.0f;
    if (normalize) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < width; c += kBlock) {
            const float v = value(c);
            ss += v * v;
        }
        ss = block_sum<kWaves>(ss, scratch);
        inv = 1.0f / sqrtf(ss / (float)width + eps);
    }
    float ss2 = 0.f;
    for (int c = threadIdx.x; c < width; c += kBlock) {
        const float v = dst[c] + value(c) * inv * gain[c];
        dst[c] = v;
        ss2 += v * v;
    }
    if (next_w == nullptr) return;
    ss2 = block_sum<kWaves>(ss2, scratch);
    const float inv2 = 1.0f / sqrtf(ss2 / (float)width + next_eps);
    for (int c = threadIdx.x; c < width; c += kBlock) next_out[r * width + c] = from_f32<T>(dst[c] * inv2 * next_w[c]);   // the thread's own stores
}

}  // namespace

extern "C" int fllm_postnorm_add(float *x, const void *branch, int branch_dtype, int parts, const float *part_weights, const float *gain,
                                 float eps, int normalize,
                                 const float *next_w, float next_eps, void *next_out, int next_dtype, int rows, int width,
                                 hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0 && parts > 0, "postnorm_add: bad sizes");
    FLLM_REQUIRE(x && branch && gain && ((next_w == nullptr) == (next_out == nullptr)), "postnorm_add: operands missing");
    if (rows == 0) return 0;
#define FLLM_POSTNORM(B, T) hipLaunchKernelGGL((postnorm_add_kernel<B, T>), dim3(rows), dim3(kBlock), 0, stream, x, (const B *)branch, \
                                               parts, part_weights, gain, eps, normalize, next_w, next_eps, (T *)next_out, width)
    if (branch_dtype == FLLM_F32 && next_dtype == FLLM_F32) FLLM_POSTNORM(float, float);
    else if (branch_dtype == FLLM_F32 && next_dtype == FLLM_BF16) FLLM_POSTNORM(float, bf16_t);
    else if (branch_dtype == FLLM_BF16 && next_dtype == FLLM_F32) FLLM_POSTNORM(bf16_t, float);
    else if (branch_dtype == FLLM_BF16 && next_dtype == FLLM_BF16) FLLM_POSTNORM(bf16_t, bf16_t);
    else FLLM_REQUIRE(false, "postnorm_add: unknown dtypes %d, %d", branch_dtype, next_dtype);
#undef FLLM_POSTNORM
    return fllm_check_launch("postnorm_add");
}

extern "C" int fllm_rmsnorm_pair(const float *x, const float *w1, const float *w2, void *out1, void *out2, int rows, int width,
                                 float eps1, float eps2, int out_dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0, "rmsnorm_pair: bad sizes");
    FLLM_REQUIRE(x && w1 && out1 && ((w2 == nullptr) == (out2 == nullptr)), "rmsnorm_pair: operands missing");
    if (rows == 0) return 0;
    if (out_dtype == FLLM_F32)
        hipLaunchKernelGGL(rmsnorm_pair_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, x, w1, w2, (float *)out1, (float *)out2,
                           width, eps1, eps2);
    else if (out_dtype == FLLM_BF16)
        hipLaunchKernelGGL(rmsnorm_pair_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, x, w1, w2, (bf16_t *)out1,
                           (bf16_t *)out2, width, eps1, eps2);
    else
        FLLM_REQUIRE(false, "rmsnorm_pair: unknown dtype %d", out_dtype);
    return fllm_check_launch("rmsnorm_pair");
}

extern "C" int fllm_glu_clamped(const void *gate_up, void *out, int rows, int inter, float limit, float alpha, float up_offset,
                                int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && inter > 0 && rows <= 65535, "glu_clamped: bad sizes");
    if (rows == 0) return 0;
    const dim3 grid((inter + kBlock - 1) / kBlock, rows);
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(glu_clamped_kernel<float>, grid, dim3(kBlock), 0, stream, (const float *)gate_up, (float *)out, inter,
                           limit, alpha, up_offset);
    else if (dtype == FLLM_BF16 && inter % 8 == 0 && (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0)
        hipLaunchKernelGGL(glu_clamped_vec_kernel, dim3((inter / 8 + kBlock - 1) / kBlock, rows), dim3(kBlock), 0, stream,
                           (const bf16_t *)gate_up, (bf16_t *)out, inter, limit, alpha, up_offset);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(glu_clamped_kernel<bf16_t>, grid, dim3(kBlock), 0, stream, (const bf16_t *)gate_up, (bf16_t *)out, inter,
                           limit, alpha, up_offset);
    else
        FLLM_REQUIRE(false, "glu_clamped: unknown dtype %d", dtype);
    return fllm_check_launch("glu_clamped");
}

extern "C" int fllm_scale_f32(float *x, size_t total, float scale, hipStream_t stream) {
    if (total == 0) return 0;
    const size_t blocks = (total + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(kBlock), 0, stream, x, total, scale);
    return fllm_check_launch("scale_f32");
}

extern "C" int fllm_stream_add(float *x, const int32_t *ids, const void *table, int table_dtype, int vocab, float scale,
                               const float *vec, int rows, int width, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && width > 0, "stream_add: bad sizes");
    FLLM_REQUIRE(table == nullptr || (ids != nullptr && vocab > 0), "stream_add: a table needs ids");
    if (rows == 0 || (table == nullptr && vec == nullptr)) return 0;
    if (table_dtype == FLLM_F32)
        hipLaunchKernelGGL(stream_add_kernel<float>, dim3(rows), dim3(kBlock), 0, stream, x, ids, (const float *)table, vocab, scale,
                           vec, width);
    else if (table_dtype == FLLM_BF16)
        hipLaunchKernelGGL(stream_add_kernel<bf16_t>, dim3(rows), dim3(kBlock), 0, stream, x, ids, (const bf16_t *)table, vocab,
                           scale, vec, width);
    else
        FLLM_REQUIRE(false, "stream_add: unknown dtype %d", table_dtype);
    return fllm_check_launch("stream_add");
}
