// The any-shape product as device functions, shared by the plain entry point (one weight matrix, rows as they lie) and
// the grouped one (a weight matrix per tile, rows gathered through an index): a tile of the grid is handed the rows it
// covers through `RowMap`, everything else is the same code, so a row's result never depends on which entry point, tile
// or batch it travelled in.
#pragma once
#include "common.h"

namespace nvh_any {

// Which rows a 64-row tile covers: row r of the tile (r < rows) is read from x row `src(r)` and written to y row `dst(r)`.
struct RowMap {
    const int32_t* gather;     // source row per destination row (null: the destination row itself)
    int row0;                  // first destination row of the tile
    int rows;                  // real rows of the tile (<= 64)
    __device__ __forceinline__ int64_t dst(int r) const { return row0 + r; }
    __device__ __forceinline__ int64_t src(int r) const { return gather ? gather[row0 + r] : row0 + r; }
};

// ---------------------------------------------------------------------------------------------------------------
// y[M, N] = x[M, K] w[N, K]^T (+ bias[N]) for ANY M, N, K (ragged edges are zero-filled on the way into LDS and masked on
// the way out).  The order in which an output element sums over k depends on (N, K) only, never on M or on the row's
// place in the batch.  bf16: 64 x 64 tile per workgroup, four waves of 2 x 2 MFMA 16x16x32 tiles, fp32 accumulation.
// fp32: the same tile with 4 x 4 outputs per lane on the vector ALU (true fp32 products and sums).
constexpr int GT = 64, GK = 64, GLD = GK + 8;

template <bool OUT_F32>
__device__ __forceinline__ void gemm_any_bf16_tile(const bf16* __restrict__ x, int64_t ldx, const bf16* __restrict__ w, int64_t ldw,
                                                   const bf16* __restrict__ bias, void* __restrict__ yv, int64_t ldy, const RowMap rm, int n0, int N, int K,
                                                   int vec_ok) {
    __shared__ __attribute__((aligned(16))) bf16 xs[GT * GLD];
    __shared__ __attribute__((aligned(16))) bf16 ws[GT * GLD];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fq = lane >> 4;
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    f32x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int lr = tid >> 2, lc = (tid & 3) * 16;            // this thread's row and first column of the 64 x 64 tile
    const int64_t xrow = lr < rm.rows ? rm.src(lr) : 0;
    // This thread's four 16-byte pieces of the next k-step's tiles (x: 0, 1; w: 2, 3) are loaded while the current step's
    // products run: a step does not wait for its own loads.
    bf16x8 pre[4];
    auto gload = [&](int k0) {
#pragma unroll
        for (int which = 0; which < 2; ++which) {
            const bf16* src = which ? w : x;
            const int64_t ld = which ? ldw : ldx;
            const int64_t row = which ? n0 + lr : xrow;
            const bool row_ok = which ? n0 + lr < N : lr < rm.rows;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int kc = k0 + lc + half * 8;
                bf16x8 v;
                if (row_ok && vec_ok && kc + 8 <= K) {
                    v = *reinterpret_cast<const bf16x8*>(src + row * ld + kc);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = (row_ok && kc + e < K) ? src[row * ld + kc + e] : (bf16)0.f;
                }
                pre[which * 2 + half] = v;
            }
        }
    };
    gload(0);
    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int which = 0; which < 2; ++which)
#pragma unroll
            for (int half = 0; half < 2; ++half) *reinterpret_cast<bf16x8*>((which ? ws : xs) + lr * GLD + lc + half * 8) = pre[which * 2 + half];
        __syncthreads();
        if (k0 + GK < K) gload(k0 + GK);
#pragma unroll
        for (int ks = 0; ks < GK / 32; ++ks) {
            bf16x8 wf[2], xf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                wf[i] = *reinterpret_cast<const bf16x8*>(ws + (wn + i * 16 + fr) * GLD + ks * 32 + fq * 8);
                xf[i] = *reinterpret_cast<const bf16x8*>(xs + (wm + i * 16 + fr) * GLD + ks * 32 + fq * 8);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], xf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // lane holds, for weight tile i and row tile j: row m = wm + 16 j + fr, columns n = wn + 16 i + 4 fq + e
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int r = wm + j * 16 + fr;
            if (r >= rm.rows) continue;
            const int64_t m = rm.dst(r);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = n0 + wn + i * 16 + fq * 4 + e;
                if (n >= N) continue;
                float v = acc[i][j][e];
                if (bias) v += (float)bias[n];
                if constexpr (OUT_F32) ((float*)yv)[m * ldy + n] = v;
                else ((bf16*)yv)[m * ldy + n] = (bf16)v;
            }
        }
}

__device__ __forceinline__ void gemm_any_f32_tile(const float* __restrict__ x, int64_t ldx, const float* __restrict__ w, int64_t ldw,
                                                  const float* __restrict__ bias, float* __restrict__ y, int64_t ldy, const RowMap rm, int n0, int N, int K) {
    constexpr int BK = 16;
    __shared__ float xs[BK][GT + 4];
    __shared__ float ws[BK][GT + 4];
    const int tid = threadIdx.x;
    const int tm = (tid >> 4) * 4, tn = (tid & 15) * 4;
    float acc[4][4] = {};
    const int lr = tid >> 2, lc = (tid & 3) * 4;             // 64 rows x 16 columns per stage: 4 consecutive k per thread
    const int64_t xrow = lr < rm.rows ? rm.src(lr) : 0;
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lc + e;
            xs[lc + e][lr] = (lr < rm.rows && k < K) ? x[xrow * ldx + k] : 0.f;
            ws[lc + e][lr] = (n0 + lr < N && k < K) ? w[(int64_t)(n0 + lr) * ldw + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                a[e] = xs[k][tm + e];
                b[e] = ws[k][tn + e];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tn + j;
            if (tm + i < rm.rows && n < N) y[rm.dst(tm + i) * ldy + n] = acc[i][j] + (bias ? bias[n] : 0.f);
        }
}

}  // namespace nvh_any
