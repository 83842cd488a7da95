// Linear attention with a decay a head over portions of prompts, on the matrix cores in float32.
//
// The recurrence S_t = a S_(t-1) + k_t v_t^T, o_t = S_t^T q_t is taken kC = 32 tokens at a time.  With S the state before a
// chunk of n tokens (t, s count inside the chunk):
//     o_t = a^(t+1) S^T q_t + sum_{s <= t} a^(t-s) (q_t . k_s) v_s          S' = a^n S + sum_s a^(n-1-s) k_s v_s^T
// which are four matrix products: the scores Q K^T (masked and decayed into P), S^T Q^T, V^T P^T, and K~^T V.  Every product
// runs as v_mfma_f32_16x16x4_f32: the operands are float32 (the activations of q, k, v are not rounded, the scores, the
// weights and the state stay float32), so the kernel serves both element types of the projections.
//
// v_mfma_f32_16x16x4_f32: lane l gives A[m = l%16][k = l/16] and B[k = l/16][n = l%16] and receives
// D[m = 4*(l/16) + r][n = l%16] in register r.  A contraction may number its k's as it likes as long as A and B agree, so a
// result tile is at once the A operand of a later product over its rows: register r of lane l, D[4g + r][n] with g = l/16,
// is A[m = n][slot g] of step r, and B then brings row 4g + r of the other matrix into slot g.  The state lives in such
// tiles for the whole call: it is the accumulator of K~^T V and the A operand of S^T Q^T, and never passes through LDS.
//
// One workgroup of four waves a (segment, head, 32 value lanes).  Wave w holds the state's rows of the key blocks
// w, w + 4, .. (16 keys a block) for both 16-lane halves of the slice.  A chunk:
//   1. q, k (32 x dim) and v (32 x 32), loaded 16 bytes at a time while the chunk before was computed, pass the activation
//      into LDS; rows beyond the chunk's tokens are zeros.
//   2. waves 0..2 take the three 16 x 16 blocks of the scores on and under the diagonal, multiply by a^(t-s), zero what
//      lies above the diagonal and leave P in LDS; every wave multiplies its rows of the state with Q^T and leaves its
//      part of the 32 x 32 result in LDS (in register order, so that the sum needs no index).
//   3. wave w takes output block (w / 2, w % 2): the sum of the four parts times a^(t+1), then V^T P^T on top; the block
//      goes to `out`.  Then every wave multiplies its state by a^n and adds K~^T V.
// The powers a^0 .. a^32 come from the decay's float pair in double precision, once a workgroup.
#include "api.h"
#include "common.h"

namespace {

constexpr int kC = 32;            // tokens a chunk
constexpr int kVB = 32;           // value lanes a workgroup
constexpr int kLDV = 48;          // row stride of V in LDS: lane groups 16 banks apart
constexpr int kLDP = 33;
constexpr int kThreads = 256;
constexpr int kPart = 256;        // tokens a part, where a long segment is cut into parts that run side by side

// Where part `part` of the segment that begins at row seg_r0 keeps its state among the carried ones: no two parts of a step
// share an index, and the largest is below rows / kPart + segments.
__host__ __device__ inline int carried_index(int seg_r0, int seg, int part) { return seg_r0 / kPart + seg + part; }

// The grid of a step in parts has one workgroup (times heads and slices) an index that a part may have: workgroup w finds the
// last segment whose first index is not above w (the first indices grow with the segment) and is that segment's part
// w - first index, if the segment has so many.
__device__ inline void find_part(int w, const int32_t *seg_start, int num_segs, int &seg, int &part) {
    int lo = 0, hi = num_segs - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (carried_index(seg_start[mid], mid, 0) <= w) lo = mid;
        else hi = mid - 1;
    }
    seg = lo;
    part = w - carried_index(seg_start[lo], lo, 0);
}

// silu of a projection: float32 rows get the library's exponential and a division; bfloat16 rows, whose own rounding is
// 2^-9, the hardware's exponential and reciprocal (a few units in the last place of a float), a quarter of the instructions
template <typename T> __device__ __forceinline__ float act_f(float z, int activation);
template <> __device__ __forceinline__ float act_f<float>(float z, int activation) {
    return activation == 1 ? z / (1.0f + expf(-z)) : z;
}
template <> __device__ __forceinline__ float act_f<bf16_t>(float z, int activation) {
    return activation == 1 ? z * __frcp_rn(1.0f + __expf(-z)) : z;
}

__host__ __device__ constexpr size_t chunked_lds_floats(int dim) {
    return 2 * (size_t)kC * (dim + 4) + (size_t)kC * kLDV + (size_t)kC * kLDP + 4 * 4 * 4 * 64 + 40;
}

template <typename T, int NB>     // NB: key blocks a wave (dim <= 64 * NB)
__global__ void __launch_bounds__(kThreads)
linear_attention_chunked_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, int ld,
                                const float *__restrict__ decay_hi, const float *__restrict__ decay_lo, float *__restrict__ state,
                                const int32_t *__restrict__ row_seg, const int32_t *__restrict__ seg_start,
                                const int32_t *__restrict__ slots, float *__restrict__ out, int heads, int dim, int vdim,
                                int activation, float *__restrict__ carried, int in_parts, int num_segs) {
    extern __shared__ float smem[];
    const int LDQ = dim + 4;
    float *Qs = smem;                          // [kC][LDQ]
    float *Ks = Qs + kC * LDQ;                 // [kC][LDQ]
    float *Vs = Ks + kC * LDQ;                 // [kC][kLDV]
    float *Ps = Vs + kC * kLDV;                // [kC][kLDP]
    float *Part = Ps + kC * kLDP;              // [wave][block][register][lane]
    float *pw = Part + 4 * 4 * 4 * 64;         // a^0 .. a^kC

    // in_parts: a segment is cut into parts of kPart tokens, a workgroup a part; every part but the first starts from
    // zeros, and every part of a segment of several leaves its state in `carried` for the kernel that follows
    int seg = blockIdx.x, part = 0;
    if (in_parts) find_part(blockIdx.x, seg_start, num_segs, seg, part);
    const int h = blockIdx.y, j0 = blockIdx.z * kVB;
    const int seg_r0 = seg_start[seg], seg_n = seg_start[seg + 1] - seg_r0;
    if (part < 0 || seg_n <= part * kPart) return;
    const int parts = in_parts ? (seg_n + kPart - 1) / kPart : 1;
    const int r0 = seg_r0 + part * kPart, n = in_parts ? min(kPart, seg_n - part * kPart) : seg_n;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ln = lane & 15, g = lane >> 4;
    const int out_ld = heads * vdim;
    if (row_seg[r0] < 0) {   // padding rows: no state is touched
        for (int i = tid; i < n * kVB; i += kThreads) {
            const int t = i / kVB, c = j0 + i % kVB;
            if (c < vdim) out[(size_t)(r0 + t) * out_ld + (size_t)h * vdim + c] = 0.f;
        }
        return;
    }
    if (tid <= kC) pw[tid] = (float)pow((double)decay_hi[h] + (double)decay_lo[h], (double)tid);
    const int key_blocks = dim / 16;
    float *mine = state + ((size_t)slots[seg] * heads + h) * dim * vdim;

    f32x4_t S[NB][2];
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int vj = 0; vj < 2; vj++) {
            const int di = wave + 4 * b, col = j0 + 16 * vj + ln;
#pragma unroll
            for (int r = 0; r < 4; r++)
                S[b][vj][r] = (part == 0 && di < key_blocks && col < vdim) ? mine[(size_t)(16 * di + 4 * g + r) * vdim + col] : 0.f;
        }
    if (parts > 1) mine = carried + ((size_t)carried_index(seg_r0, seg, part) * heads + h) * dim * vdim;

    // 1. the chunk's q, k, v: 16 bytes a load, all of a thread's loads in flight at once, and the next chunk's loads issued
    // before this chunk's products, so that a chunk waits for memory once at most
    constexpr int EPV = 16 / (int)sizeof(T);                                  // elements a load
    constexpr int QV = (kC * 64 * NB / EPV + kThreads - 1) / kThreads;        // loads a thread for q, and for k
    constexpr int VV = (kC * kVB / EPV + kThreads - 1) / kThreads;
    const int dimv = dim / EPV;
    uint4 rq[QV], rk[QV], rv[VV];
    int tq[QV], cq[QV];                  // a load's token and first lane: the same in every chunk
#pragma unroll
    for (int it = 0; it < QV; it++) {
        const int i = tid + it * kThreads;
        tq[it] = i / dimv;
        cq[it] = (i - tq[it] * dimv) * EPV;
    }
    auto issue = [&](int c0) {
        const int nc = min(kC, n - c0);
#pragma unroll
        for (int it = 0; it < QV; it++) {
            rq[it] = rk[it] = uint4{0u, 0u, 0u, 0u};
            if (tq[it] < nc) {
                const size_t at = (size_t)(r0 + c0 + tq[it]) * ld + (size_t)h * dim + cq[it];
                rq[it] = *(const uint4 *)(q + at);
                rk[it] = *(const uint4 *)(k + at);
            }
        }
#pragma unroll
        for (int it = 0; it < VV; it++) {
            const int i = tid + it * kThreads, t = i / (kVB / EPV), cv = i % (kVB / EPV);
            rv[it] = uint4{0u, 0u, 0u, 0u};
            if (t < nc && j0 + cv * EPV < vdim)
                rv[it] = *(const uint4 *)(v + (size_t)(r0 + c0 + t) * ld + (size_t)h * vdim + j0 + cv * EPV);
        }
    };
    // through the activation into LDS, four lanes a store; rows beyond the chunk's tokens were loaded as zeros
    auto put = [&](float *dst, const uint4 &raw) {
        const T *e = (const T *)&raw;
#pragma unroll
        for (int e4 = 0; e4 < EPV; e4 += 4) {
            f32x4_t a;
#pragma unroll
            for (int x = 0; x < 4; x++) a[x] = act_f<T>(to_f32<T>(e[e4 + x]), activation);
            *(f32x4_t *)(dst + e4) = a;
        }
    };
    auto commit = [&]() {
#pragma unroll
        for (int it = 0; it < QV; it++)
            if (tq[it] < kC) {
                put(Qs + tq[it] * LDQ + cq[it], rq[it]);
                put(Ks + tq[it] * LDQ + cq[it], rk[it]);
            }
#pragma unroll
        for (int it = 0; it < VV; it++) {
            const int i = tid + it * kThreads, t = i / (kVB / EPV), cv = i % (kVB / EPV);
            if (t < kC) put(Vs + t * kLDV + cv * EPV, rv[it]);
        }
    };
    issue(0);
    for (int c0 = 0; c0 < n; c0 += kC) {
        const int nc = min(kC, n - c0);
        commit();
        if (c0 + kC < n) issue(c0 + kC);
        __syncthreads();

        // 2a. scores on and under the diagonal: block (ti, si) = (0, 0), (1, 0), (1, 1)
        if (wave < 3) {
            const int ti = wave == 0 ? 0 : 1, si = wave == 2 ? 1 : 0;
            f32x4_t acc = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};      // two chains: a product does not wait for the one before
            const float *qrow = Qs + (16 * ti + ln) * LDQ + 4 * g, *krow = Ks + (16 * si + ln) * LDQ + 4 * g;
            for (int j = 0; j < key_blocks; j++) {
                const f32x4_t qa = *(const f32x4_t *)(qrow + 16 * j), kb = *(const f32x4_t *)(krow + 16 * j);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[0], kb[0], acc, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[1], kb[1], acc1, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[2], kb[2], acc, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[3], kb[3], acc1, 0, 0, 0);
            }
            acc += acc1;
            const int s = 16 * si + ln;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int t = 16 * ti + 4 * g + r;
                Ps[t * kLDP + s] = s <= t ? acc[r] * pw[t - s] : 0.f;
            }
        } else {   // the block above the diagonal is never read: (0, 1) stays out of every sum below
        }
        // 2b. this wave's rows of the state times Q^T: four blocks (value half vj, token half nj)
        {
            f32x4_t part[2][2];
#pragma unroll
            for (int vj = 0; vj < 2; vj++)
#pragma unroll
                for (int nj = 0; nj < 2; nj++) part[vj][nj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const int di = wave + 4 * b;
                if (di < key_blocks) {
#pragma unroll
                    for (int nj = 0; nj < 2; nj++) {
                        const f32x4_t qb = *(const f32x4_t *)(Qs + (16 * nj + ln) * LDQ + 16 * di + 4 * g);
#pragma unroll
                        for (int vj = 0; vj < 2; vj++)
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                part[vj][nj] = __builtin_amdgcn_mfma_f32_16x16x4f32(S[b][vj][r], qb[r], part[vj][nj], 0, 0, 0);
                    }
                }
            }
#pragma unroll
            for (int vj = 0; vj < 2; vj++)
#pragma unroll
                for (int nj = 0; nj < 2; nj++)
#pragma unroll
                    for (int r = 0; r < 4; r++) Part[((wave * 4 + vj * 2 + nj) * 4 + r) * 64 + lane] = part[vj][nj][r];
        }
        __syncthreads();

        // 3a. output block (vj, nj) of this wave: lane (ln, g), register r is o[token 16 nj + ln][value 16 vj + 4 g + r]
        {
            const int vj = wave >> 1, nj = wave & 1;
            const int t = 16 * nj + ln;
            f32x4_t o;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < 4; w++) sum += Part[((w * 4 + vj * 2 + nj) * 4 + r) * 64 + lane];
                o[r] = sum * pw[t + 1];
            }
            const int steps = nj == 0 ? 4 : 8;       // keys of the first half alone reach tokens of the first half
            for (int s4 = 0; s4 < steps; s4++) {
                const int s = 4 * s4 + g;
                o = __builtin_amdgcn_mfma_f32_16x16x4f32(Vs[s * kLDV + 16 * vj + ln], Ps[t * kLDP + s], o, 0, 0, 0);
            }
            const int col = j0 + 16 * vj + 4 * g;
            if (t < nc && col < vdim) *(f32x4_t *)(out + (size_t)(r0 + c0 + t) * out_ld + (size_t)h * vdim + col) = o;
        }
        // 3b. the state behind the chunk
        {
            const float all = pw[nc];
            float wk[8];
#pragma unroll
            for (int s4 = 0; s4 < 8; s4++) {
                const int s = 4 * s4 + g;
                wk[s4] = s < nc ? pw[nc - 1 - s] : 0.f;
            }
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const int di = wave + 4 * b;
                if (di < key_blocks) {
#pragma unroll
                    for (int vj = 0; vj < 2; vj++) S[b][vj] *= all;
#pragma unroll
                    for (int s4 = 0; s4 < 8; s4++) {
                        const int s = 4 * s4 + g;
                        const float ka = Ks[s * LDQ + 16 * di + ln] * wk[s4];
#pragma unroll
                        for (int vj = 0; vj < 2; vj++)
                            S[b][vj] = __builtin_amdgcn_mfma_f32_16x16x4f32(ka, Vs[s * kLDV + 16 * vj + ln], S[b][vj], 0, 0, 0);
                    }
                }
            }
        }
        __syncthreads();      // the next chunk overwrites what this one read
    }

#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int vj = 0; vj < 2; vj++) {
            const int di = wave + 4 * b, col = j0 + 16 * vj + ln;
            if (di < key_blocks && col < vdim)
#pragma unroll
                for (int r = 0; r < 4; r++) mine[(size_t)(16 * di + 4 * g + r) * vdim + col] = S[b][vj][r];
        }
}

// The kernel behind the parts.  Part p > 0 of a segment ran from zeros; the state before it is
//     T_p = a^kPart T_(p-1) + U_(p-1),   T_1 = the state behind part 0,   U_i = what part i left in `carried`,
// and every token of the part lacks a^(t+1) T_p^T q_t (t counts inside the part).  One workgroup a (segment, part > 0, head,
// 32 value lanes): T_p in registers in the layout of the state above, the product as in step 2b, the sum added to `out`.
// The workgroup of the last part also leaves the segment's state: a^n T_p + U_p.
template <typename T, int NB>
__global__ void __launch_bounds__(kThreads)
linear_attention_carry_kernel(const T *__restrict__ q, int ld, const float *__restrict__ decay_hi, const float *__restrict__ decay_lo,
                              float *__restrict__ state, const int32_t *__restrict__ row_seg, const int32_t *__restrict__ seg_start,
                              const int32_t *__restrict__ slots, float *__restrict__ out, int heads, int dim, int vdim,
                              int activation, const float *__restrict__ carried, int num_segs) {
    extern __shared__ float smem[];
    const int LDQ = dim + 4;
    float *Qs = smem;                          // [kC][LDQ]
    float *Part = Qs + kC * LDQ;               // [wave][block][register][lane]
    float *pw = Part + 4 * 4 * 4 * 64;         // a^(c0 + 1) .. a^(c0 + kC)
    int seg, part;
    find_part(blockIdx.x, seg_start, num_segs, seg, part);
    const int h = blockIdx.y, j0 = blockIdx.z * kVB;
    const int seg_r0 = seg_start[seg], seg_n = seg_start[seg + 1] - seg_r0;
    if (part <= 0 || seg_n <= part * kPart || row_seg[seg_r0] < 0) return;
    const int parts = (seg_n + kPart - 1) / kPart;
    const int r0 = seg_r0 + part * kPart, n = min(kPart, seg_n - part * kPart);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ln = lane & 15, g = lane >> 4;
    const int out_ld = heads * vdim;
    const int key_blocks = dim / 16;
    const double a = (double)decay_hi[h] + (double)decay_lo[h];
    const float a_part = (float)pow(a, (double)kPart);

    f32x4_t S[NB][2];
    auto add_carried = [&](int i, float scale) {     // S = scale S + U_i
        const float *u = carried + ((size_t)carried_index(seg_r0, seg, i) * heads + h) * dim * vdim;
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int vj = 0; vj < 2; vj++) {
                const int di = wave + 4 * b, col = j0 + 16 * vj + ln;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float add = (di < key_blocks && col < vdim) ? u[(size_t)(16 * di + 4 * g + r) * vdim + col] : 0.f;
                    S[b][vj][r] = fmaf(S[b][vj][r], scale, add);
                }
            }
    };
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
        for (int vj = 0; vj < 2; vj++) S[b][vj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < part; i++) add_carried(i, a_part);

    constexpr int EPV = 16 / (int)sizeof(T);
    constexpr int QV = (kC * 64 * NB / EPV + kThreads - 1) / kThreads;
    const int dimv = dim / EPV;
    uint4 rq[QV];
    int tq[QV], cq[QV];
#pragma unroll
    for (int it = 0; it < QV; it++) {
        const int i = tid + it * kThreads;
        tq[it] = i / dimv;
        cq[it] = (i - tq[it] * dimv) * EPV;
    }
    auto issue = [&](int c0) {
        const int nc = min(kC, n - c0);
#pragma unroll
        for (int it = 0; it < QV; it++) {
            rq[it] = uint4{0u, 0u, 0u, 0u};
            if (tq[it] < nc) rq[it] = *(const uint4 *)(q + (size_t)(r0 + c0 + tq[it]) * ld + (size_t)h * dim + cq[it]);
        }
    };
    issue(0);
    for (int c0 = 0; c0 < n; c0 += kC) {
        const int nc = min(kC, n - c0);
#pragma unroll
        for (int it = 0; it < QV; it++)
            if (tq[it] < kC) {
                const T *e = (const T *)&rq[it];
#pragma unroll
                for (int e4 = 0; e4 < EPV; e4 += 4) {
                    f32x4_t x;
#pragma unroll
                    for (int i = 0; i < 4; i++) x[i] = act_f<T>(to_f32<T>(e[e4 + i]), activation);
                    *(f32x4_t *)(Qs + tq[it] * LDQ + cq[it] + e4) = x;
                }
            }
        if (tid < kC) pw[tid] = (float)pow(a, (double)(c0 + tid + 1));
        __syncthreads();
        if (c0 + kC < n) issue(c0 + kC);
        {
            f32x4_t part_sum[2][2];
#pragma unroll
            for (int vj = 0; vj < 2; vj++)
#pragma unroll
                for (int nj = 0; nj < 2; nj++) part_sum[vj][nj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int b = 0; b < NB; b++) {
                const int di = wave + 4 * b;
                if (di < key_blocks) {
#pragma unroll
                    for (int nj = 0; nj < 2; nj++) {
                        const f32x4_t qb = *(const f32x4_t *)(Qs + (16 * nj + ln) * LDQ + 16 * di + 4 * g);
#pragma unroll
                        for (int vj = 0; vj < 2; vj++)
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                part_sum[vj][nj] = __builtin_amdgcn_mfma_f32_16x16x4f32(S[b][vj][r], qb[r], part_sum[vj][nj], 0, 0, 0);
                    }
                }
            }
#pragma unroll
            for (int vj = 0; vj < 2; vj++)
#pragma unroll
                for (int nj = 0; nj < 2; nj++)
#pragma unroll
                    for (int r = 0; r < 4; r++) Part[((wave * 4 + vj * 2 + nj) * 4 + r) * 64 + lane] = part_sum[vj][nj][r];
        }
        __syncthreads();
        {   // output block (vj, nj) of this wave: lane (ln, g), register r is o[token 16 nj + ln][value 16 vj + 4 g + r]
            const int vj = wave >> 1, nj = wave & 1;
            const int t = 16 * nj + ln;
            const int col = j0 + 16 * vj + 4 * g;
            if (t < nc && col < vdim) {
                float *dst = out + (size_t)(r0 + c0 + t) * out_ld + (size_t)h * vdim + col;
                f32x4_t o = *(const f32x4_t *)dst;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float sum = 0.f;
#pragma unroll
                    for (int w = 0; w < 4; w++) sum += Part[((w * 4 + vj * 2 + nj) * 4 + r) * 64 + lane];
                    o[r] = fmaf(sum, pw[t], o[r]);
                }
                *(f32x4_t *)dst = o;
            }
        }
        __syncthreads();      // the next chunk overwrites what this one read
    }
    if (part == parts - 1) {
        add_carried(part, (float)pow(a, (double)n));
        float *mine = state + ((size_t)slots[seg] * heads + h) * dim * vdim;
#pragma unroll
        for (int b = 0; b < NB; b++)
#pragma unroll
            for (int vj = 0; vj < 2; vj++) {
                const int di = wave + 4 * b, col = j0 + 16 * vj + ln;
                if (di < key_blocks && col < vdim)
#pragma unroll
                    for (int r = 0; r < 4; r++) mine[(size_t)(16 * di + 4 * g + r) * vdim + col] = S[b][vj][r];
            }
    }
}

}  // namespace

// 0: launched; 1: the sizes are not this kernel's (keys in blocks of 16 up to 128 lanes, values in blocks of 16, rows that
// begin on 16 bytes).  `carried` (float32, carried_floats of them, or null): room for the states that the parts of long
// segments hand on; with it, a step of at least two parts' rows cuts every segment into parts of kPart tokens.
extern "C" size_t fllm_linear_attention_carried_floats(int rows, int num_segs, int heads, int dim, int vdim) {
    return ((size_t)rows / kPart + (size_t)num_segs + 1) * heads * dim * vdim;
}

int fllm_linear_attention_chunked(const void *q, const void *k, const void *v, int ld, const float *decay_hi, const float *decay_lo,
                                  float *state, const int32_t *row_seg, const int32_t *seg_start, const int32_t *slots, int num_segs,
                                  float *out, int rows, int heads, int dim, int vdim, int activation, int dtype, float *carried,
                                  hipStream_t stream) {
    if (dim % 16 != 0 || dim > 128 || vdim % 16 != 0) return 1;
    // rows are read 16 bytes at a time
    const int epv = dtype == FLLM_F32 ? 4 : 8;
    if (ld % epv != 0 || (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) != 0) return 1;
    const int slices = (vdim + kVB - 1) / kVB;
    if (slices > 65535 || heads > 65535) return 1;
    const size_t smem = chunked_lds_floats(dim) * sizeof(float);
    if (smem > 64 * 1024) return 1;
    const int in_parts = (carried != nullptr && rows >= 2 * kPart) ? 1 : 0;
    const dim3 grid(in_parts ? (unsigned)(rows / kPart + num_segs) : (unsigned)num_segs, heads, slices);
    const size_t smem_carry = ((size_t)kC * (dim + 4) + 4 * 4 * 4 * 64 + 40) * sizeof(float);
#define FLLM_CHUNKED(T, NB)                                                                                                       \
    do {                                                                                                                          \
        hipLaunchKernelGGL((linear_attention_chunked_kernel<T, NB>), grid, dim3(kThreads), smem, stream, (const T *)q,            \
                           (const T *)k, (const T *)v, ld, decay_hi, decay_lo, state, row_seg, seg_start, slots, out, heads, dim, \
                           vdim, activation, carried, in_parts, num_segs);                                                        \
        if (in_parts)                                                                                                             \
            hipLaunchKernelGGL((linear_attention_carry_kernel<T, NB>), grid, dim3(kThreads), smem_carry, stream, (const T *)q,    \
                               ld, decay_hi, decay_lo, state, row_seg, seg_start, slots, out, heads, dim, vdim, activation,       \
                               carried, num_segs);                                                                                \
    } while (0)
    if (dtype == FLLM_F32) {
        if (dim <= 64) FLLM_CHUNKED(float, 1);
        else FLLM_CHUNKED(float, 2);
    } else if (dtype == FLLM_BF16) {
        if (dim <= 64) FLLM_CHUNKED(bf16_t, 1);
        else FLLM_CHUNKED(bf16_t, 2);
    } else
        return 1;
#undef FLLM_CHUNKED
    return 0;
}
