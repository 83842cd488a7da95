// A feed-forward of many small gated layers ("experts") of which every row uses a few: the router that scores the
// experts and picks each row's best, and the products of the picked experts, one (row, pick) pair at a time.  These are
// the plain kernels: float32 sums in a fixed order, both element types, any sizes.  A pair's result depends on its own
// row alone, never on the rest of the batch.
#include "api.h"
#include "common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

// sum over the lanes' share of x . w for one weight row; x float32 in LDS, w in global memory
template <typename T>
__device__ __forceinline__ float lane_dot(const float *__restrict__ xs, const T *__restrict__ w, int K, int lane) {
    float acc = 0.f;
    for (int c = lane; c < K; c += kWave) acc = fmaf(xs[c], to_f32<T>(w[c]), acc);
    return acc;
}
// bfloat16 rows whose length is a multiple of 8 and that begin on 16 bytes: 8 neighbours a load
__device__ __forceinline__ float lane_dot8(const float *__restrict__ xs, const bf16_t *__restrict__ w, int K, int lane) {
    float acc = 0.f;
    for (int c = lane * 8; c < K; c += kWave * 8) {
        const bf16x8_t w8 = *(const bf16x8_t *)(w + c);
#pragma unroll
        for (int e = 0; e < 8; e++) acc = fmaf(xs[c + e], (float)w8[e], acc);
    }
    return acc;
}
// R weight rows against the same x at once, 8 neighbours a load and row: the loads of all rows are in flight together, which
// is what a workgroup that streams a few rows of a matrix is short of.  Row r's sum is added in the order lane_dot8 adds it.
template <int R>
__device__ __forceinline__ void lane_dots8(const float *__restrict__ xs, const bf16_t *const (&w)[R], int K, int lane, float (&acc)[R]) {
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;
    for (int c = lane * 8; c < K; c += kWave * 8) {
        bf16x8_t w8[R];
#pragma unroll
        for (int r = 0; r < R; r++) w8[r] = __builtin_nontemporal_load((const bf16x8_t *)(w[r] + c));
        float x8[8];
#pragma unroll
        for (int e = 0; e < 8; e++) x8[e] = xs[c + e];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int e = 0; e < 8; e++) acc[r] = fmaf(x8[e], (float)w8[r][e], acc[r]);
    }
}

template <typename T> __device__ __forceinline__ float row_dot(const float *xs, const T *w, int K, int lane, bool vec);
template <> __device__ __forceinline__ float row_dot<float>(const float *xs, const float *w, int K, int lane, bool) {
    return wave_sum(lane_dot<float>(xs, w, K, lane));
}
template <> __device__ __forceinline__ float row_dot<bf16_t>(const float *xs, const bf16_t *w, int K, int lane, bool vec) {
    return wave_sum(vec ? lane_dot8(xs, w, K, lane) : lane_dot<bf16_t>(xs, w, K, lane));
}

// Router: z = W h in float32, score = sigmoid(z) (score_mode 0) or the softmax of z over all experts (score_mode 1); the
// `top` largest scores of a row, ties to the lower index; weights[r, k] = the score of pick k, with `renormalize` divided by
// the sum of the picks' scores (+ 1e-20), times route_scale.  One workgroup a row; scores through LDS.
template <typename T>
__global__ void __launch_bounds__(kBlock)
route_kernel(const T *__restrict__ h, int ldh, const T *__restrict__ w, int K, int E, int top, int32_t *__restrict__ ids,
             float *__restrict__ weights, int score_mode, int renormalize, float route_scale) {
    extern __shared__ float smem[];
    float *xs = smem;          // K
    float *score = smem + K;   // E
    float *picks = score + E;  // top: the picks' scores, until their sum is known
    const size_t r = blockIdx.x;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    for (int c = threadIdx.x; c < K; c += kBlock) xs[c] = to_f32<T>(h[r * ldh + c]);
    __syncthreads();
    const bool vec = sizeof(T) == 2 && K % 8 == 0 && ((uintptr_t)w & 15) == 0;
    for (int e = wave; e < E; e += kWaves) {
        const float z = row_dot<T>(xs, w + (size_t)e * K, K, lane, vec);
        if (lane == 0) score[e] = score_mode == 0 ? 1.0f / (1.0f + expf(-z)) : z;
    }
    __syncthreads();
    if (wave != 0) return;
    if (score_mode == 1) {   // softmax over all experts: the largest logit, the sum in index order a lane, then across lanes
        float top_z = -INFINITY;
        for (int e = lane; e < E; e += kWave) top_z = fmaxf(top_z, score[e]);
        top_z = wave_max(top_z);
        float sum = 0.f;
        for (int e = lane; e < E; e += kWave) sum += expf(score[e] - top_z);
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += kWave) score[e] = expf(score[e] - top_z) / sum;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    float picked = 0.f;
    // one wave picks: every round the largest score not yet taken, the lowest index among equals
    for (int k = 0; k < top; k++) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < E; e += kWave) {
            const float s = score[e];
            if (s > best) best = s, at = e;      // ascending e: the first of equals stays
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float other = __shfl_xor(best, o, kWave);
            const int other_at = __shfl_xor(at, o, kWave);
            if (other > best || (other == best && other_at < at)) best = other, at = other_at;
        }
        if (at < 0 || at >= E) at = k;           // scores that compare with nothing (NaN rows): still an expert of the stack
        picked += best;
        if (lane == 0) {
            ids[r * top + k] = at;
            picks[k] = best;
            score[at] = -INFINITY;               // scores lie in [0, 1]: nothing real is that small
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    const float factor = renormalize ? route_scale / (picked + 1e-20f) : route_scale;
    for (int k = lane; k < top; k += kWave)
        weights[r * top + k] = (renormalize || route_scale != 1.0f) ? picks[k] * factor : picks[k];
}

// Router with corrections and groups: score = sigmoid(W h); the picks are made by choice = score + correction, and only among
// the experts of the `kept` groups (of `groups` equal groups of neighbours) whose two largest choices sum highest, the lower
// group among equals; weights[r, k] = the plain score of pick k divided by the sum of the picks' scores (+ 1e-20), times
// route_scale.  One workgroup a row; one wave chooses.
template <typename T>
__global__ void __launch_bounds__(kBlock)
route_grouped_kernel(const T *__restrict__ h, int ldh, const T *__restrict__ w, const float *__restrict__ correction, int K, int E,
                     int top, int groups, int kept, int32_t *__restrict__ ids, float *__restrict__ weights, float route_scale) {
    extern __shared__ float smem[];
    float *xs = smem;            // K
    float *score = smem + K;     // E
    float *choice = score + E;   // E
    float *gsum = choice + E;    // groups
    float *picks = gsum + groups;   // top
    const size_t r = blockIdx.x;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    for (int c = threadIdx.x; c < K; c += kBlock) xs[c] = to_f32<T>(h[r * ldh + c]);
    __syncthreads();
    const bool vec = sizeof(T) == 2 && K % 8 == 0 && ((uintptr_t)w & 15) == 0;
    for (int e = wave; e < E; e += kWaves) {
        const float z = row_dot<T>(xs, w + (size_t)e * K, K, lane, vec);
        if (lane == 0) {
            const float s = 1.0f / (1.0f + expf(-z));
            score[e] = s;
            choice[e] = s + correction[e];
        }
    }
    __syncthreads();
    if (wave != 0) return;
    const int per = E / groups;
    if (groups > 1) {
        for (int g = lane; g < groups; g += kWave) {      // a group counts the sum of its two largest choices (of its one, if it has one)
            float a = -INFINITY, b = -INFINITY;
            for (int e = g * per; e < (g + 1) * per; e++) {
                const float c = choice[e];
                if (c > a) b = a, a = c;
                else if (c > b) b = c;
            }
            gsum[g] = per > 1 ? a + b : a;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
        for (int k = 0; k < kept; k++) {                  // the best group not yet kept: marked with +inf
            float best = -INFINITY;
            int at = 0x7fffffff;
            for (int g = lane; g < groups; g += kWave) {
                const float s = gsum[g];
                if (s != INFINITY && s > best) best = s, at = g;
            }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float other = __shfl_xor(best, o, kWave);
                const int other_at = __shfl_xor(at, o, kWave);
                if (other > best || (other == best && other_at < at)) best = other, at = other_at;
            }
            if (at < 0 || at >= groups) {                 // sums that compare with nothing: the first group not yet kept
                at = 0;
                while (at < groups - 1 && gsum[at] == INFINITY) at++;
            }
            __builtin_amdgcn_wave_barrier();
            if (lane == 0) gsum[at] = INFINITY;
            __builtin_amdgcn_wave_barrier();
            __threadfence_block();
        }
        for (int e = lane; e < E; e += kWave)
            if (gsum[e / per] != INFINITY) choice[e] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    float picked = 0.f;
    for (int k = 0; k < top; k++) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < E; e += kWave) {
            const float s = choice[e];
            if (s > best) best = s, at = e;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float other = __shfl_xor(best, o, kWave);
            const int other_at = __shfl_xor(at, o, kWave);
            if (other > best || (other == best && other_at < at)) best = other, at = other_at;
        }
        if (at < 0 || at >= E) at = k;
        const float s = score[at];
        picked += s;
        __builtin_amdgcn_wave_barrier();
        if (lane == 0) {
            ids[r * top + k] = at;
            picks[k] = s;
            choice[at] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    const float factor = route_scale / (picked + 1e-20f);
    for (int k = lane; k < top; k += kWave) weights[r * top + k] = picks[k] * factor;
}

// One (row, pick) pair a workgroup row (blockIdx.y), kCols output columns a workgroup (blockIdx.x), two a wave.
// MODE 0: act[pair, c] = a(g) * (u + up_offset) with g, u = W_gate[e] x, W_up[e] x (clamped to `limit` when > 0),
//         a(g) = g * sigmoid(alpha g), x = the row times the pick's weight (rounded to the element type, as a stored
//         operand would be); w = [E][2 I][K], gate rows then up rows.
// MODE 1: out[pair, c] = W[e][c] . x, float32; w = [E][N][K]; x = act[pair].
// MODE 2: act[pair, c] = relu(W[e][c] . x)^2 with x = the pair's row as it is (an expert without a gate, its weight waits for
//         the output); w = [E][N][K].
constexpr int kColsPerWave = 2;
constexpr int kCols = kWaves * kColsPerWave;

template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock)
expert_rows_kernel(const T *__restrict__ x, int ldx, const int32_t *__restrict__ ids, const float *__restrict__ weights, int top,
                   const T *__restrict__ w, int E, int N, int K, T *__restrict__ act, float *__restrict__ out, float limit,
                   float alpha, float up_offset) {
    extern __shared__ float xs[];   // K
    const size_t pair = blockIdx.y;
    int e = ids[pair];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);     // never outside the stack of experts
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (MODE == 0) {
        const float scale = weights[pair];
        const T *src = x + (pair / top) * ldx;
        for (int c = threadIdx.x; c < K; c += kBlock) xs[c] = to_f32<T>(from_f32<T>(to_f32<T>(src[c]) * scale));
    } else if (MODE == 2) {
        const T *src = x + (pair / top) * ldx;
        for (int c = threadIdx.x; c < K; c += kBlock) xs[c] = to_f32<T>(src[c]);
    } else {
        const T *src = x + pair * ldx;
        for (int c = threadIdx.x; c < K; c += kBlock) xs[c] = to_f32<T>(src[c]);
    }
    __syncthreads();
    const bool vec = sizeof(T) == 2 && K % 8 == 0 && ((uintptr_t)w & 15) == 0;
    if constexpr (sizeof(T) == 2) {
        // bfloat16 rows of whole 16-byte pieces: the wave's columns at once (their sums are those of the loop below, bit for bit)
        const int c0 = blockIdx.x * kCols + wave * kColsPerWave;
        if (vec && c0 + kColsPerWave <= N) {
            if (MODE == 0) {
                const bf16_t *base = (const bf16_t *)w + ((size_t)e * 2 * N + c0) * K;
                const bf16_t *const rows[4] = {base, base + K, base + (size_t)N * K, base + (size_t)N * K + K};
                float acc[4];
                lane_dots8<4>(xs, rows, K, lane, acc);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    float g = wave_sum(acc[j]), u = wave_sum(acc[2 + j]);
                    if (limit > 0.f) {
                        g = fminf(g, limit);
                        u = fminf(fmaxf(u, -limit), limit);
                    }
                    if (lane == 0) act[pair * N + c0 + j] = from_f32<T>(g / (1.0f + expf(-alpha * g)) * (u + up_offset));
                }
            } else {
                const bf16_t *base = (const bf16_t *)w + ((size_t)e * N + c0) * K;
                const bf16_t *const rows[2] = {base, base + K};
                float acc[2];
                lane_dots8<2>(xs, rows, K, lane, acc);
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const float y = wave_sum(acc[j]);
                    if (MODE == 2) {
                        const float a = fmaxf(y, 0.f);
                        if (lane == 0) act[pair * N + c0 + j] = from_f32<T>(a * a);
                    } else if (lane == 0) out[pair * N + c0 + j] = y;
                }
            }
            return;
        }
    }
    static_assert(kColsPerWave == 2, "the wave's columns at once are two");
#pragma unroll
    for (int j = 0; j < kColsPerWave; j++) {
        const int c = blockIdx.x * kCols + wave * kColsPerWave + j;
        if (c >= N) break;
        if (MODE == 0) {
            const T *wg = w + ((size_t)e * 2 * N + c) * K, *wu = wg + (size_t)N * K;
            float g = row_dot<T>(xs, wg, K, lane, vec), u = row_dot<T>(xs, wu, K, lane, vec);
            if (limit > 0.f) {
                g = fminf(g, limit);
                u = fminf(fmaxf(u, -limit), limit);
            }
            if (lane == 0) act[pair * N + c] = from_f32<T>(g / (1.0f + expf(-alpha * g)) * (u + up_offset));
        } else {
            const float y = row_dot<T>(xs, w + ((size_t)e * N + c) * K, K, lane, vec);
            if (MODE == 2) {
                const float a = fmaxf(y, 0.f);
                if (lane == 0) act[pair * N + c] = from_f32<T>(a * a);
            } else if (lane == 0) out[pair * N + c] = y;
        }
    }
}

}  // namespace

extern "C" int fllm_route_topk(const void *h, int ldh, const void *w_router, int rows, int K, int E, int top, int32_t *ids,
                               float *weights, int score_mode, int renormalize, float route_scale, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(score_mode == 0 || score_mode == 1, "route_topk: unknown score %d", score_mode);
    FLLM_REQUIRE(rows >= 0 && K > 0 && E > 0 && top > 0 && top <= E && ldh >= K, "route_topk: bad sizes (rows %d, width %d, %d experts, %d picked)",
                 rows, K, E, top);
    FLLM_REQUIRE(h && w_router && ids && weights, "route_topk: operands missing");
    const size_t smem = (size_t)(K + E + top) * sizeof(float);
    FLLM_REQUIRE(smem <= 64 * 1024, "route_topk: a width of %d with %d experts does not fit into LDS", K, E);
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(route_kernel<float>, dim3(rows), dim3(kBlock), smem, stream, (const float *)h, ldh, (const float *)w_router, K, E,
                           top, ids, weights, score_mode, renormalize, route_scale);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(route_kernel<bf16_t>, dim3(rows), dim3(kBlock), smem, stream, (const bf16_t *)h, ldh, (const bf16_t *)w_router, K,
                           E, top, ids, weights, score_mode, renormalize, route_scale);
    else
        FLLM_REQUIRE(false, "route_topk: unknown dtype %d", dtype);
    return fllm_check_launch("route_topk");
}

extern "C" int fllm_experts_gate_up(const void *h, int ldh, const int32_t *ids, const float *weights, int rows, int top,
                                    const void *w_gate_up, int E, int inter, int K, void *act, float limit, float alpha, float up_offset,
                                    int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && top > 0 && E > 0 && inter > 0 && K > 0 && ldh >= K, "experts_gate_up: bad sizes");
    FLLM_REQUIRE(h && ids && weights && w_gate_up && act, "experts_gate_up: operands missing");
    FLLM_REQUIRE((size_t)K * sizeof(float) <= 64 * 1024, "experts_gate_up: a width of %d does not fit into LDS", K);
    const long pairs = (long)rows * top;
    FLLM_REQUIRE(pairs <= 65535 * 64L, "experts_gate_up: too many rows");
    if (pairs == 0) return 0;
    const size_t smem = (size_t)K * sizeof(float);
    // at most 65,535 pairs a launch (the grid's second dimension)
    for (long first = 0; first < pairs; first += 65535) {
        const int count = (int)(pairs - first < 65535 ? pairs - first : 65535);
        const dim3 grid((inter + kCols - 1) / kCols, count);
        FLLM_REQUIRE(first % top == 0 || top == 1 || pairs <= 65535, "experts_gate_up: a launch must begin on a row");
        if (dtype == FLLM_F32)
            hipLaunchKernelGGL((expert_rows_kernel<float, 0>), grid, dim3(kBlock), smem, stream, (const float *)h + (first / top) * ldh, ldh,
                               ids + first, weights + first, top, (const float *)w_gate_up, E, inter, K, (float *)act + first * inter, nullptr,
                               limit, alpha, up_offset);
        else if (dtype == FLLM_BF16)
            hipLaunchKernelGGL((expert_rows_kernel<bf16_t, 0>), grid, dim3(kBlock), smem, stream, (const bf16_t *)h + (first / top) * ldh, ldh,
                               ids + first, weights + first, top, (const bf16_t *)w_gate_up, E, inter, K, (bf16_t *)act + first * inter,
                               nullptr, limit, alpha, up_offset);
        else
            FLLM_REQUIRE(false, "experts_gate_up: unknown dtype %d", dtype);
    }
    return fllm_check_launch("experts_gate_up");
}

extern "C" int fllm_route_grouped(const void *h, int ldh, const void *w_router, const float *correction, int rows, int K, int E, int top,
                                  int groups, int kept, int32_t *ids, float *weights, float route_scale, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && K > 0 && E > 0 && top > 0 && ldh >= K, "route_grouped: bad sizes");
    FLLM_REQUIRE(groups > 0 && E % groups == 0 && kept > 0 && kept <= groups && top <= kept * (E / groups),
                 "route_grouped: %d experts in %d groups, %d kept, %d picked", E, groups, kept, top);
    FLLM_REQUIRE(h && w_router && correction && ids && weights, "route_grouped: operands missing");
    const size_t smem = (size_t)(K + 2 * E + groups + top) * sizeof(float);
    FLLM_REQUIRE(smem <= 64 * 1024, "route_grouped: a width of %d with %d experts does not fit into LDS", K, E);
    if (rows == 0) return 0;
    if (dtype == FLLM_F32)
        hipLaunchKernelGGL(route_grouped_kernel<float>, dim3(rows), dim3(kBlock), smem, stream, (const float *)h, ldh, (const float *)w_router,
                           correction, K, E, top, groups, kept, ids, weights, route_scale);
    else if (dtype == FLLM_BF16)
        hipLaunchKernelGGL(route_grouped_kernel<bf16_t>, dim3(rows), dim3(kBlock), smem, stream, (const bf16_t *)h, ldh,
                           (const bf16_t *)w_router, correction, K, E, top, groups, kept, ids, weights, route_scale);
    else
        FLLM_REQUIRE(false, "route_grouped: unknown dtype %d", dtype);
    return fllm_check_launch("route_grouped");
}

extern "C" int fllm_experts_up(const void *h, int ldh, const int32_t *ids, int rows, int top, const void *w_up, int E, int inter, int K,
                               void *act, int dtype, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && top > 0 && E > 0 && inter > 0 && K > 0 && ldh >= K, "experts_up: bad sizes");
    FLLM_REQUIRE(h && ids && w_up && act, "experts_up: operands missing");
    FLLM_REQUIRE((size_t)K * sizeof(float) <= 64 * 1024, "experts_up: a width of %d does not fit into LDS", K);
    const long pairs = (long)rows * top;
    FLLM_REQUIRE(pairs <= 65535 * 64L, "experts_up: too many rows");
    if (pairs == 0) return 0;
    const size_t smem = (size_t)K * sizeof(float);
    for (long first = 0; first < pairs; first += 65535) {
        const int count = (int)(pairs - first < 65535 ? pairs - first : 65535);
        const dim3 grid((inter + kCols - 1) / kCols, count);
        FLLM_REQUIRE(first % top == 0 || top == 1 || pairs <= 65535, "experts_up: a launch must begin on a row");
        if (dtype == FLLM_F32)
            hipLaunchKernelGGL((expert_rows_kernel<float, 2>), grid, dim3(kBlock), smem, stream, (const float *)h + (first / top) * ldh, ldh,
                               ids + first, nullptr, top, (const float *)w_up, E, inter, K, (float *)act + first * inter, nullptr, 0.f, 0.f, 0.f);
        else if (dtype == FLLM_BF16)
            hipLaunchKernelGGL((expert_rows_kernel<bf16_t, 2>), grid, dim3(kBlock), smem, stream, (const bf16_t *)h + (first / top) * ldh, ldh,
                               ids + first, nullptr, top, (const bf16_t *)w_up, E, inter, K, (bf16_t *)act + first * inter, nullptr, 0.f, 0.f,
                               0.f);
        else
            FLLM_REQUIRE(false, "experts_up: unknown dtype %d", dtype);
    }
    return fllm_check_launch("experts_up");
}

extern "C" int fllm_experts_down(const void *act, const int32_t *ids, int pairs, const void *w_down, int E, int N, int inter, float *out,
                                 int dtype, hipStream_t stream) {
    FLLM_REQUIRE(pairs >= 0 && E > 0 && N > 0 && inter > 0, "experts_down: bad sizes");
    FLLM_REQUIRE(act && ids && w_down && out, "experts_down: operands missing");
    FLLM_REQUIRE((size_t)inter * sizeof(float) <= 64 * 1024, "experts_down: experts of %d lanes do not fit into LDS", inter);
    if (pairs == 0) return 0;
    const size_t smem = (size_t)inter * sizeof(float);
    for (long first = 0; first < pairs; first += 65535) {
        const int count = (int)(pairs - first < 65535 ? pairs - first : 65535);
        const dim3 grid((N + kCols - 1) / kCols, count);
        if (dtype == FLLM_F32)
            hipLaunchKernelGGL((expert_rows_kernel<float, 1>), grid, dim3(kBlock), smem, stream, (const float *)act + first * inter, inter,
                               ids + first, nullptr, 1, (const float *)w_down, E, N, inter, nullptr, out + first * N, 0.f, 0.f, 0.f);
        else if (dtype == FLLM_BF16)
            hipLaunchKernelGGL((expert_rows_kernel<bf16_t, 1>), grid, dim3(kBlock), smem, stream, (const bf16_t *)act + first * inter, inter,
                               ids + first, nullptr, 1, (const bf16_t *)w_down, E, N, inter, nullptr, out + first * N, 0.f, 0.f, 0.f);
        else
            FLLM_REQUIRE(false, "experts_down: unknown dtype %d", dtype);
    }
    return fllm_check_launch("experts_down");
}
