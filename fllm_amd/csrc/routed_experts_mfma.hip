// Routed experts on the matrix cores (bfloat16, prompt portions): the (row, pick) pairs of a step are grouped by expert on
// the device, and every expert multiplies the rows that picked it as tiles of 64 or 128 rows, so that its matrices are read
// once a row tile instead of once a row.  Three launches: grouping, gate/up with the activation, down.  A pair's result does not
// depend on which rows share its tile (a row of a matrix-core product is a sum over K in an order of its own).
//
// MFMA operand layout used here (wave64, v_mfma_f32_32x32x16_bf16): A lane l holds A[m = l%32][k = 8*(l/32) .. +7]; B
// likewise with n = l%32; D lane l holds D[m = 8*(i/4) + 4*(l/32) + i%4][n = l%32], i = 0..15.
#include <algorithm>

#include "api.h"
#include "common.h"

namespace {

constexpr int GK = 64, LDT = GK + 8;
constexpr int kThreads = 256;

__device__ __forceinline__ bf16x8_t zero8() {
    bf16x8_t z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16_t)0.0f;
    return z;
}

// One workgroup.  counts -> first pair slot and first tile of every expert -> the pairs of an expert side by side in
// `order`, and a list of tiles (expert, first slot, pairs).  work: [0] number of tiles, then 3 ints a tile, then order.
__global__ void __launch_bounds__(1024)
group_pairs_kernel(const int32_t *__restrict__ ids, int pairs, int E, int max_tiles, int GM, int32_t *__restrict__ work) {
    extern __shared__ int lds[];      // count[E], slot[E], tile[E]
    int *count = lds, *slot = lds + E, *tile = lds + 2 * E;
    int32_t *tiles = work + 1, *order = work + 1 + 3 * max_tiles;
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        int e = ids[p];
        e = e < 0 ? 0 : (e >= E ? E - 1 : e);
        atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int s = 0, t = 0;
        for (int e = 0; e < E; e++) {
            slot[e] = s;
            tile[e] = t;
            s += count[e];
            t += (count[e] + GM - 1) / GM;
        }
        work[0] = t;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const int n = count[e];
        for (int i = 0, t = tile[e]; i < n; i += GM, t++) {
            tiles[3 * t] = e;
            tiles[3 * t + 1] = slot[e] + i;
            tiles[3 * t + 2] = n - i < GM ? n - i : GM;
        }
    }
    __syncthreads();       // slot[] becomes the cursor of its expert
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        int e = ids[p];
        e = e < 0 ? 0 : (e >= E ? E - 1 : e);
        order[atomicAdd(&slot[e], 1)] = p;
    }
}

// xs[slot] = h[pair / top] * weights[pair], rounded to bfloat16 as a stored operand is: the expert's input, once for all the
// column tiles that read it.  One workgroup a slot; K a multiple of 8.
__global__ void __launch_bounds__(256)
scaled_rows_kernel(const bf16_t *__restrict__ h, int ldh, const float *__restrict__ weights, int top, const int32_t *__restrict__ order,
                   bf16_t *__restrict__ xs, int K) {
    const int pair = order[blockIdx.x];
    const float s = weights[pair];
    const bf16_t *src = h + (size_t)(pair / top) * ldh;
    bf16_t *dst = xs + (size_t)blockIdx.x * K;
    for (int c = threadIdx.x * 8; c < K; c += 256 * 8) {
        bf16x8_t v = *(const bf16x8_t *)(src + c);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (bf16_t)((float)v[i] * s);
        *(bf16x8_t *)(dst + c) = v;
    }
}

// MODE 0: act[pair, c] = a(g) * (u + up_offset) for 64 columns c a workgroup; A rows = the scaled rows in slot order;
//         B = 64 gate rows and 64 up rows of the expert.  w: [E][2 N][K].
// MODE 1: out[pair, c] = w[e][c] . act[pair] for GN columns, float32.  w: [E][N][K].
// MODE 2: act[pair, c] = relu(w[e][c] . h[pair / top])^2 for GN columns: the up product of experts without a gate, whose rows
//         are read as they are (the picks' weights wait for the outputs).  w: [E][N][K]; x = h, row stride ldx.
// GN: weight rows a column tile, 128, or 64 (MODE 1 only) where a launch of 128-column tiles would leave most of the
// device without a workgroup (decode steps).
// GM: pairs a row tile, 64 (a wave 32 rows) or 128 (a wave 64 rows: an operand read from LDS serves twice the products).
template <int MODE, int GM, int GN>
__global__ void __launch_bounds__(kThreads)
grouped_tiles_kernel(const bf16_t *__restrict__ x, int ldx, const int32_t *__restrict__ work,
                     int max_tiles, const bf16_t *__restrict__ w, int N, int K, bf16_t *__restrict__ act, float *__restrict__ out,
                     float limit, float alpha, float up_offset, int k_per, size_t slice_stride, int top) {
    __shared__ __attribute__((aligned(16))) bf16_t As[GM * LDT];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[GN * LDT];
    __shared__ int s_pair[GM];
    static_assert(MODE != 0 || GN == 128, "gate and up rows come as 64 and 64");
    const int t = blockIdx.x % max_tiles, tn = blockIdx.x / max_tiles;     // neighbouring workgroups share a column tile
    if (t >= work[0]) return;
    const int32_t *tile = work + 1 + 3 * t, *order = work + 1 + 3 * max_tiles;
    const int e = tile[0], first = tile[1], count = tile[2];
    constexpr int COLS = MODE == 0 ? GN / 2 : GN;      // output columns a workgroup
    const int n0 = tn * COLS;
    if (threadIdx.x < GM) {
        const int pair = threadIdx.x < count ? order[first + threadIdx.x] : -1;
        s_pair[threadIdx.x] = pair;
    }
    __syncthreads();
    const bf16_t *wb = w + (size_t)e * (MODE == 0 ? 2 : 1) * N * K;
    // K slices (blockIdx.y) where a launch would otherwise leave most of the device idle: every slice leaves its sums in a
    // plane of its own, and a kernel behind this one adds the planes in slice order
    const int k_begin = blockIdx.y * k_per, k_end = min(K, k_begin + k_per);
    if (MODE == 1) out += blockIdx.y * slice_stride;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, lg = lane >> 5;

    constexpr int RI = GM / 64;       // 32-row product tiles a wave
    constexpr int CJ = MODE == 0 ? 2 : GN / 64;      // runs of 32 columns a wave
    f32x16_t acc[RI][CJ];
#pragma unroll
    for (int i = 0; i < RI; i++)
#pragma unroll
        for (int j = 0; j < CJ; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    constexpr int kA = (GM * GK / 8) / kThreads, kB = (GN * GK / 8) / kThreads;     // 16-byte chunks a thread
    bf16x8_t ra[kA], rb[kB];
    auto load_tile = [&](int k0) {
#pragma unroll
        for (int c = 0; c < kA; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            const int row = chunk / (GK / 8), k = k0 + (chunk % (GK / 8)) * 8;
            const int pair = s_pair[row];
            // MODE 0 reads the scaled rows, which lie in slot order; MODE 1 the activations, which lie in pair order
            const size_t from = MODE == 0 ? first + row : (MODE == 2 ? (pair < 0 ? 0 : pair / top) : pair);
            ra[c] = (pair >= 0 && k < k_end) ? *(const bf16x8_t *)(x + from * ldx + k) : zero8();
        }
#pragma unroll
        for (int c = 0; c < kB; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            const int row = chunk / (GK / 8), k = k0 + (chunk % (GK / 8)) * 8;
            // MODE 0: rows 0..63 are gate rows n0 .., rows 64..127 the up rows of the same columns
            const int col = MODE == 0 ? n0 + (row & (COLS - 1)) : n0 + row;
            const size_t wrow = MODE == 0 ? (size_t)(row >= COLS ? N : 0) + col : (size_t)col;
            rb[c] = (col < N && k < k_end) ? *(const bf16x8_t *)(wb + wrow * K + k) : zero8();
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int c = 0; c < kA; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            *(bf16x8_t *)(As + (chunk / (GK / 8)) * LDT + (chunk % (GK / 8)) * 8) = ra[c];
        }
#pragma unroll
        for (int c = 0; c < kB; c++) {
            const int chunk = threadIdx.x + c * kThreads;
            *(bf16x8_t *)(Bs + (chunk / (GK / 8)) * LDT + (chunk % (GK / 8)) * 8) = rb[c];
        }
    };
    // the wave's two product columns: MODE 0 the gate and the up rows of its 32 columns, MODE 1 two runs of 32 columns
    const int brow0 = MODE == 0 ? wn * 32 + l32 : wn * (GN / 2) + l32;
    const int brow1 = MODE == 0 ? COLS + wn * 32 + l32 : wn * (GN / 2) + 32 + l32;      // unused where a wave has one run

    load_tile(k_begin);
    for (int k0 = k_begin; k0 < k_end; k0 += GK) {
        store_tile();
        __syncthreads();
        if (k0 + GK < k_end) load_tile(k0 + GK);   // in flight while this tile is multiplied
#pragma unroll
        for (int kk = 0; kk < GK / 16; kk++) {
            const bf16x8_t b0 = *(const bf16x8_t *)(Bs + brow0 * LDT + kk * 16 + lg * 8);
            const bf16x8_t b1 = CJ > 1 ? *(const bf16x8_t *)(Bs + brow1 * LDT + kk * 16 + lg * 8) : b0;
#pragma unroll
            for (int i = 0; i < RI; i++) {
                const bf16x8_t a = *(const bf16x8_t *)(As + (wm * (GM / 2) + i * 32 + l32) * LDT + kk * 16 + lg * 8);
                acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[i][0], 0, 0, 0);
                if (CJ > 1) acc[i][CJ - 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[i][CJ - 1], 0, 0, 0);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < RI; i++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int pair = s_pair[wm * (GM / 2) + i * 32 + 8 * (v / 4) + 4 * lg + (v % 4)];
        if (pair < 0) continue;
        if (MODE == 0) {
            const int n = n0 + wn * 32 + l32;
            if (n >= N) continue;
            float g = acc[i][0][v], u = acc[i][CJ - 1][v];
            if (limit > 0.f) {
                g = fminf(g, limit);
                u = fminf(fmaxf(u, -limit), limit);
            }
            act[(size_t)pair * N + n] = (bf16_t)(g / (1.0f + expf(-alpha * g)) * (u + up_offset));
        } else if (MODE == 2) {
#pragma unroll
            for (int j = 0; j < CJ; j++) {
                const int n = n0 + wn * (GN / 2) + j * 32 + l32;
                const float a = fmaxf(acc[i][j][v], 0.f);
                if (n < N) act[(size_t)pair * N + n] = (bf16_t)(a * a);
            }
        } else {
#pragma unroll
            for (int j = 0; j < CJ; j++) {
                const int n = n0 + wn * (GN / 2) + j * 32 + l32;
                if (n < N) out[(size_t)pair * N + n] = acc[i][j][v];
            }
        }
    }
}

// out[i] = the sum of the K slices' planes, in slice order
__global__ void __launch_bounds__(256)
sum_planes_kernel(const float *__restrict__ planes, float *__restrict__ out, size_t count, int slices) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    float v = planes[i];
    for (int s = 1; s < slices; s++) v += planes[(size_t)s * count + i];
    out[i] = v;
}

// K slices of the down product: 1 unless 64-column tiles give the device fewer than two workgroups a compute unit
int down_slices(long pairs, int E, int N, int inter) {
    const long tiles = ((pairs + 63) / 64 + E) * ((N + 63) / 64);
    if (pairs / E >= 96 || tiles >= 512) return 1;
    const long want = (1024 + tiles - 1) / tiles, most = (inter + 255) / 256;
    return (int)std::max(1L, std::min(16L, std::min(want, most)));
}

}  // namespace

// floats of scratch that fllm_experts_grouped needs for the planes of a down product cut along K (0: it is not cut)
extern "C" size_t fllm_experts_grouped_plane_floats(int pairs, int E, int N, int inter) {
    const int slices = down_slices(pairs, E, N, inter);
    return slices > 1 ? (size_t)slices * pairs * N : 0;
}

// ints of scratch that fllm_experts_grouped needs for `pairs` (row, pick) pairs over E experts
extern "C" size_t fllm_experts_grouped_work_ints(int pairs, int E) {
    const size_t max_tiles = (size_t)(pairs + 63) / 64 + E;       // as many as the smaller row tile needs
    return 1 + 3 * max_tiles + pairs;
}

// 0: launched, negative: error, 1: shape declined (the caller runs the plain kernels).  h bfloat16 [rows, K] (row stride ldh);
// ids / weights [rows, top]; w_gate_up [E][2 inter][K]; w_down [E][N][inter]; act bfloat16 [rows * top, inter] and xs bfloat16
// [rows * top, K] (scratch); out float32 [rows * top, N]; work: fllm_experts_grouped_work_ints() int32.
extern "C" int fllm_experts_grouped(const void *h, int ldh, const int32_t *ids, const float *weights, int rows, int top,
                                    const void *w_gate_up, const void *w_down, int E, int inter, int K, int N, void *act, void *xs,
                                    float *out, int32_t *work, float *planes, float limit, float alpha, float up_offset, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && top > 0 && E > 0 && inter > 0 && K > 0 && N > 0 && ldh >= K, "experts_grouped: bad sizes");
    FLLM_REQUIRE(h && ids && weights && w_gate_up && w_down && act && xs && out && work, "experts_grouped: operands missing");
    if (!fllm_fast_kernels_enabled()) return 1;
    if (K % 8 != 0 || inter % 8 != 0 || ldh % 8 != 0 || E > 4096) return 1;
    if ((((uintptr_t)h | (uintptr_t)w_gate_up | (uintptr_t)w_down | (uintptr_t)act | (uintptr_t)xs) & 15) != 0) return 1;
    const long pairs = (long)rows * top;
    if (pairs == 0) return 0;
    // row tiles of 128 pairs where the experts' shares are large enough to fill them
    const int GM = pairs / E >= 96 ? 128 : 64;
    const long max_tiles = (pairs + GM - 1) / GM + E;
    // column tiles of 64 for the down product where 128 would give the device fewer workgroups than compute units, and
    // K slices where that is still too few (decode steps)
    const int GN_DOWN = max_tiles * ((N + 127) / 128) < 256 ? 64 : 128;
    const int slices = GN_DOWN == 64 ? down_slices(pairs, E, N, inter) : 1;
    FLLM_REQUIRE(slices == 1 || planes != nullptr, "experts_grouped: the planes of a down product cut along K are missing");
    const int k_per_down = slices > 1 ? ((inter + slices - 1) / slices + GK - 1) / GK * GK : inter;
    const long up_tiles = (inter + 63) / 64, down_tiles = (N + GN_DOWN - 1) / GN_DOWN;
    if (pairs > (1L << 24) || max_tiles * up_tiles > 0x7fffffffL || max_tiles * down_tiles > 0x7fffffffL) return 1;
    hipLaunchKernelGGL(group_pairs_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), stream, ids, (int)pairs, E, (int)max_tiles, GM, work);
    hipLaunchKernelGGL(scaled_rows_kernel, dim3((unsigned)pairs), dim3(256), 0, stream, (const bf16_t *)h, ldh, weights, top,
                       work + 1 + 3 * max_tiles, (bf16_t *)xs, K);
    float *down_out = slices > 1 ? planes : out;
#define FLLM_GROUPED(MODE, ROWS, COLS, X, LDX, W, NN, KK)                                                                                  \
    hipLaunchKernelGGL((grouped_tiles_kernel<MODE, ROWS, COLS>),                                                                           \
                       dim3((unsigned)(max_tiles * (MODE == 0 ? up_tiles : down_tiles)), MODE == 0 ? 1 : slices), dim3(kThreads), 0,        \
                       stream, (const bf16_t *)(X), LDX, work, (int)max_tiles, (const bf16_t *)(W), NN, KK, (bf16_t *)act, down_out, limit, \
                       alpha, up_offset, MODE == 0 ? KK : k_per_down, (size_t)pairs * N, top)
    if (GM == 128) FLLM_GROUPED(0, 128, 128, xs, K, w_gate_up, inter, K);
    else FLLM_GROUPED(0, 64, 128, xs, K, w_gate_up, inter, K);
    if (GM == 128 && GN_DOWN == 128) FLLM_GROUPED(1, 128, 128, act, inter, w_down, N, inter);
    else if (GM == 128) FLLM_GROUPED(1, 128, 64, act, inter, w_down, N, inter);
    else if (GN_DOWN == 128) FLLM_GROUPED(1, 64, 128, act, inter, w_down, N, inter);
    else FLLM_GROUPED(1, 64, 64, act, inter, w_down, N, inter);
#undef FLLM_GROUPED
    if (slices > 1) {
        const size_t count = (size_t)pairs * N;
        hipLaunchKernelGGL(sum_planes_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, planes, out, count, slices);
    }
    return fllm_check_launch("experts_grouped");
}

// The same for experts without a gate: act = relu(W_up[e] h)^2 on the rows as they are, then the down product.  w_up
// [E][inter][K]; no scaled copies of the rows are needed.  0: launched, negative: error, 1: shape declined.
extern "C" int fllm_experts_grouped_ungated(const void *h, int ldh, const int32_t *ids, int rows, int top, const void *w_up,
                                            const void *w_down, int E, int inter, int K, int N, void *act, float *out, int32_t *work,
                                            float *planes, hipStream_t stream) {
    FLLM_REQUIRE(rows >= 0 && top > 0 && E > 0 && inter > 0 && K > 0 && N > 0 && ldh >= K, "experts_grouped_ungated: bad sizes");
    FLLM_REQUIRE(h && ids && w_up && w_down && act && out && work, "experts_grouped_ungated: operands missing");
    if (!fllm_fast_kernels_enabled()) return 1;
    if (K % 8 != 0 || inter % 8 != 0 || ldh % 8 != 0 || E > 4096) return 1;
    if ((((uintptr_t)h | (uintptr_t)w_up | (uintptr_t)w_down | (uintptr_t)act) & 15) != 0) return 1;
    const long pairs = (long)rows * top;
    if (pairs == 0) return 0;
    const int GM = pairs / E >= 96 ? 128 : 64;
    const long max_tiles = (pairs + GM - 1) / GM + E;
    const int GN_UP = max_tiles * ((inter + 127) / 128) < 256 ? 64 : 128;
    const int GN_DOWN = max_tiles * ((N + 127) / 128) < 256 ? 64 : 128;
    const int slices = GN_DOWN == 64 ? down_slices(pairs, E, N, inter) : 1;
    FLLM_REQUIRE(slices == 1 || planes != nullptr, "experts_grouped_ungated: the planes of a down product cut along K are missing");
    const int k_per_down = slices > 1 ? ((inter + slices - 1) / slices + GK - 1) / GK * GK : inter;
    const long up_tiles = (inter + GN_UP - 1) / GN_UP, down_tiles = (N + GN_DOWN - 1) / GN_DOWN;
    if (pairs > (1L << 24) || max_tiles * up_tiles > 0x7fffffffL || max_tiles * down_tiles > 0x7fffffffL) return 1;
    hipLaunchKernelGGL(group_pairs_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), stream, ids, (int)pairs, E, (int)max_tiles, GM, work);
    float *down_out = slices > 1 ? planes : out;
#define FLLM_UNGATED(MODE, ROWS, COLS, X, LDX, W, NN, KK, TILES, SLICES, KPER)                                                          \
    hipLaunchKernelGGL((grouped_tiles_kernel<MODE, ROWS, COLS>), dim3((unsigned)(max_tiles * (TILES)), SLICES), dim3(kThreads), 0, stream, \
                       (const bf16_t *)(X), LDX, work, (int)max_tiles, (const bf16_t *)(W), NN, KK, (bf16_t *)act, down_out, 0.f, 0.f, 0.f, \
                       KPER, (size_t)pairs * N, top)
    if (GM == 128 && GN_UP == 128) FLLM_UNGATED(2, 128, 128, h, ldh, w_up, inter, K, up_tiles, 1, K);
    else if (GM == 128) FLLM_UNGATED(2, 128, 64, h, ldh, w_up, inter, K, up_tiles, 1, K);
    else if (GN_UP == 128) FLLM_UNGATED(2, 64, 128, h, ldh, w_up, inter, K, up_tiles, 1, K);
    else FLLM_UNGATED(2, 64, 64, h, ldh, w_up, inter, K, up_tiles, 1, K);
    if (GM == 128 && GN_DOWN == 128) FLLM_UNGATED(1, 128, 128, act, inter, w_down, N, inter, down_tiles, slices, k_per_down);
    else if (GM == 128) FLLM_UNGATED(1, 128, 64, act, inter, w_down, N, inter, down_tiles, slices, k_per_down);
    else if (GN_DOWN == 128) FLLM_UNGATED(1, 64, 128, act, inter, w_down, N, inter, down_tiles, slices, k_per_down);
    else FLLM_UNGATED(1, 64, 64, act, inter, w_down, N, inter, down_tiles, slices, k_per_down);
#undef FLLM_UNGATED
    if (slices > 1) {
        const size_t count = (size_t)pairs * N;
        hipLaunchKernelGGL(sum_planes_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, planes, out, count, slices);
    }
    return fllm_check_launch("experts_grouped_ungated");
}
