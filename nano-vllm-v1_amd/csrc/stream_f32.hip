// Row-wise operators around an fp32 residual stream, for designs whose residual sum, norms and softcap must stay in
// 32-bit while projections run in the activation type A (bf16, or fp32 for a model served in full precision):
//   embedding rows -> fp32 stream (+ a copy in A), Dynamic-Tanh norm fused with the residual add that precedes it,
//   tanh-GELU gate, [stream | first embedding] concatenation for a looped stack, row gather, logit softcap.
// Every kernel is one workgroup per row (or a flat element grid) with 16-byte accesses where the row allows.
#include "common.h"

namespace {

template <typename A>
__device__ __forceinline__ float ldf(const A* p, int64_t i) {
    return (float)p[i];
}

struct DytNorm {            // tanh(alpha * x) * w + b; all three in the activation type
    const void* alpha;
    const void* w;
    const void* b;
};

// tanh for the norm: the library's where everything is fp32; for bf16 results 1 - 2 / (e^2z + 1) on the hardware's 2^x and
// reciprocal (about 1e-6 absolute; the result is rounded to 8 bits of mantissa).
template <typename A>
__device__ __forceinline__ float dyt_tanh(float z) {
    if constexpr (sizeof(A) == 4) {
        return tanhf(z);
    } else {
        const float e = __builtin_amdgcn_exp2f(fminf(z, 20.f) * 2.8853900817779268f);        // e^(2z)
        return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
    }
}

// x[row] = (accumulate ? x[row] : 0) + post(y[row]) + bias;  h[row] = next(x[row]).
// y null: the stream is only normalised.  post / next with a null weight are skipped (next: no h written).
// VEC: dim % 4 == 0 and every row 16-byte (A: 8-byte) aligned: four consecutive elements per lane, one access each.
template <typename A, bool VEC>
__global__ __launch_bounds__(256) void residual_dyt_kernel(const A* __restrict__ y, int64_t y_stride, DytNorm post, const A* __restrict__ bias,
                                                           float* __restrict__ x, int accumulate, DytNorm next, A* __restrict__ h,
                                                           int64_t h_stride, int dim) {
    typedef A A4 __attribute__((ext_vector_type(4)));
    const int64_t row = blockIdx.x;
    const float pa = post.w ? ldf((const A*)post.alpha, 0) : 0.f;
    const float na = next.w ? ldf((const A*)next.alpha, 0) : 0.f;
    float* xr = x + row * dim;
    constexpr int W = VEC ? 4 : 1;
    for (int c = threadIdx.x * W; c < dim; c += 256 * W) {
        float s[W], t[W], bv[W], pw[W], pb[W], nw[W], nb[W];
        if constexpr (VEC) {
            const f32x4 xv = accumulate ? *reinterpret_cast<const f32x4*>(xr + c) : f32x4{0.f, 0.f, 0.f, 0.f};
            const A4 zero = {(A)0.f, (A)0.f, (A)0.f, (A)0.f};
            const A4 yv = y ? *reinterpret_cast<const A4*>(y + row * y_stride + c) : zero;
            const A4 b4 = bias ? *reinterpret_cast<const A4*>(bias + c) : zero;
            const A4 pw4 = post.w ? *reinterpret_cast<const A4*>((const A*)post.w + c) : zero, pb4 = post.w ? *reinterpret_cast<const A4*>((const A*)post.b + c) : zero;
            const A4 nw4 = next.w ? *reinterpret_cast<const A4*>((const A*)next.w + c) : zero, nb4 = next.w ? *reinterpret_cast<const A4*>((const A*)next.b + c) : zero;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                s[e] = xv[e];
                t[e] = (float)yv[e];
                bv[e] = (float)b4[e];
                pw[e] = (float)pw4[e];
                pb[e] = (float)pb4[e];
                nw[e] = (float)nw4[e];
                nb[e] = (float)nb4[e];
            }
        } else {
            s[0] = accumulate ? xr[c] : 0.f;
            t[0] = y ? ldf(y, row * y_stride + c) : 0.f;
            bv[0] = bias ? ldf(bias, c) : 0.f;
            pw[0] = post.w ? ldf((const A*)post.w, c) : 0.f;
            pb[0] = post.w ? ldf((const A*)post.b, c) : 0.f;
            nw[0] = next.w ? ldf((const A*)next.w, c) : 0.f;
            nb[0] = next.w ? ldf((const A*)next.b, c) : 0.f;
        }
        float hv[W];
#pragma unroll
        for (int e = 0; e < W; ++e) {
            if (y) s[e] += post.w ? dyt_tanh<A>(pa * t[e]) * pw[e] + pb[e] : t[e];
            s[e] += bv[e];
            hv[e] = next.w ? dyt_tanh<A>(na * s[e]) * nw[e] + nb[e] : 0.f;
        }
        if constexpr (VEC) {
            if (y || bias) *reinterpret_cast<f32x4*>(xr + c) = f32x4{s[0], s[1], s[2], s[3]};
            if (next.w) *reinterpret_cast<A4*>(h + row * h_stride + c) = A4{(A)hv[0], (A)hv[1], (A)hv[2], (A)hv[3]};
        } else {
            if (y || bias) xr[c] = s[0];
            if (next.w) h[row * h_stride + c] = (A)hv[0];
        }
    }
}

template <typename A>
__global__ __launch_bounds__(256) void embedding_stream_kernel(const int64_t* __restrict__ ids, const A* __restrict__ table, float* __restrict__ x,
                                                               A* __restrict__ x0, int64_t x0_stride, int dim, int64_t vocab) {
    const int64_t row = blockIdx.x;
    const int64_t id = ids[row];
    const bool ok = id >= 0 && id < vocab;
    for (int c = threadIdx.x; c < dim; c += 256) {
        const A v = ok ? table[id * dim + c] : (A)0.f;
        x[row * dim + c] = (float)v;
        if (x0) x0[row * x0_stride + c] = v;
    }
}

// out[row, :dim] = A(x[row]); the second half of the row (the first embedding) is already there.
template <typename A>
__global__ __launch_bounds__(256) void stream_cast_kernel(const float* __restrict__ x, A* __restrict__ out, int64_t out_stride, int dim) {
    const int64_t row = blockIdx.x;
    for (int c = threadIdx.x; c < dim; c += 256) out[row * out_stride + c] = (A)x[row * dim + c];
}

template <typename A>
__global__ __launch_bounds__(256) void gelu_tanh_mul_kernel(const A* __restrict__ gu, int64_t gu_stride, A* __restrict__ y, int64_t rows, int inter) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * inter) return;
    const int64_t row = i / inter;
    const int c = (int)(i - row * inter);
    const float g = ldf(gu, row * gu_stride + c), u = ldf(gu, row * gu_stride + inter + c);
    const float act = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    y[i] = (A)(act * u);
}

__global__ __launch_bounds__(256) void gather_rows_f32_kernel(const float* __restrict__ x, const int32_t* __restrict__ index, float* __restrict__ out, int dim) {
    const int64_t row = blockIdx.x;
    const int64_t src = index[row];
    for (int c = threadIdx.x; c < dim; c += 256) out[row * dim + c] = x[src * dim + c];
}

template <typename A>
__global__ __launch_bounds__(256) void softcap_kernel(const A* __restrict__ z, int64_t z_stride, float* __restrict__ out, int64_t rows, int vocab, float cap) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * vocab) return;
    const int64_t row = i / vocab;
    const float v = ldf(z, row * z_stride + (i - row * vocab));
    out[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

// ---------------------------------------------------------------------------------------------------------------
// y[M, N] = x[M, K] w[N, K]^T (+ bias[N]) for ANY M, N, K (ragged edges are zero-filled on the way into LDS and masked on
// the way out).  The order in which an output element sums over k depends on (N, K) only, never on M or on the row's
// place in the batch.  bf16: 64 x 64 tile per workgroup, four waves of 2 x 2 MFMA 16x16x32 tiles, fp32 accumulation.
// fp32: the same tile with 4 x 4 outputs per lane on the vector ALU (true fp32 products and sums).
constexpr int GT = 64, GK = 64, GLD = GK + 8;

template <bool OUT_F32>
__global__ __launch_bounds__(256) void gemm_any_bf16_kernel(const bf16* __restrict__ x, int64_t ldx, const bf16* __restrict__ w, int64_t ldw,
                                                            const bf16* __restrict__ bias, void* __restrict__ yv, int64_t ldy, int M, int N, int K,
                                                            int vec_ok) {
    __shared__ __attribute__((aligned(16))) bf16 xs[GT * GLD];
    __shared__ __attribute__((aligned(16))) bf16 ws[GT * GLD];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fq = lane >> 4;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
    f32x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int lr = tid >> 2, lc = (tid & 3) * 16;            // this thread's row and first column of the 64 x 64 tile
    for (int k0 = 0; k0 < K; k0 += GK) {
        // stage both tiles
#pragma unroll
        for (int which = 0; which < 2; ++which) {
            const bf16* src = which ? w : x;
            const int64_t ld = which ? ldw : ldx;
            const int row = (which ? n0 : m0) + lr, rows = which ? N : M;
            bf16* dst = (which ? ws : xs) + lr * GLD + lc;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int kc = k0 + lc + half * 8;
                bf16x8 v;
                if (row < rows && vec_ok && kc + 8 <= K) {
                    v = *reinterpret_cast<const bf16x8*>(src + (int64_t)row * ld + kc);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = (row < rows && kc + e < K) ? src[(int64_t)row * ld + kc + e] : (bf16)0.f;
                }
                *reinterpret_cast<bf16x8*>(dst + half * 8) = v;
            }
        }
        __syncthreads();
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
            const int m = m0 + wm + j * 16 + fr;
            if (m >= M) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = n0 + wn + i * 16 + fq * 4 + e;
                if (n >= N) continue;
                float v = acc[i][j][e];
                if (bias) v += (float)bias[n];
                if constexpr (OUT_F32) ((float*)yv)[(int64_t)m * ldy + n] = v;
                else ((bf16*)yv)[(int64_t)m * ldy + n] = (bf16)v;
            }
        }
}

__global__ __launch_bounds__(256) void gemm_any_f32_kernel(const float* __restrict__ x, int64_t ldx, const float* __restrict__ w, int64_t ldw,
                                                           const float* __restrict__ bias, float* __restrict__ y, int64_t ldy, int M, int N, int K) {
    constexpr int BK = 16;
    __shared__ float xs[BK][GT + 4];
    __shared__ float ws[BK][GT + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    const int tm = (tid >> 4) * 4, tn = (tid & 15) * 4;
    float acc[4][4] = {};
    const int lr = tid >> 2, lc = (tid & 3) * 4;             // 64 rows x 16 columns per stage: 4 consecutive k per thread
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lc + e;
            xs[lc + e][lr] = (m0 + lr < M && k < K) ? x[(int64_t)(m0 + lr) * ldx + k] : 0.f;
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
            const int m = m0 + tm + i, n = n0 + tn + j;
            if (m < M && n < N) y[(int64_t)m * ldy + n] = acc[i][j] + (bias ? bias[n] : 0.f);
        }
}

}  // namespace

#define NVH_STREAM_ARGS_OK(name, cond) NVH_REQUIRE(cond, NVH_EINVAL, name ": bad argument")

extern "C" int32_t nvh_embedding_stream(const int64_t* ids, const void* table, float* x, void* x0, int64_t x0_stride,
                                        int64_t num_tokens, int64_t dim, int64_t vocab, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_embedding_stream", ids && table && x && num_tokens >= 0 && dim > 0 && vocab > 0);
    if (num_tokens == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) embedding_stream_kernel<float><<<dim3((unsigned)num_tokens), 256, 0, st>>>(ids, (const float*)table, x, (float*)x0, x0_stride, (int)dim, vocab);
    else embedding_stream_kernel<bf16><<<dim3((unsigned)num_tokens), 256, 0, st>>>(ids, (const bf16*)table, x, (bf16*)x0, x0_stride, (int)dim, vocab);
    NVH_CHECK_LAUNCH("nvh_embedding_stream");
    return NVH_OK;
}

extern "C" int32_t nvh_residual_dyt(const void* y, int64_t y_stride, const void* post_alpha, const void* post_w, const void* post_b,
                                    const void* bias, float* x, int32_t accumulate, const void* next_alpha, const void* next_w,
                                    const void* next_b, void* h, int64_t h_stride, int64_t rows, int64_t dim, int32_t act_f32,
                                    nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_residual_dyt", x && rows >= 0 && dim > 0 && (!post_w || (post_alpha && post_b && y)) &&
                                               (!next_w || (next_alpha && next_b && h)) && (accumulate || y || bias));
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const DytNorm post{post_alpha, post_w, post_b}, next{next_alpha, next_w, next_b};
    const int esz = act_f32 ? 4 : 2;
    auto al = [&](const void* p, int bytes) { return p == nullptr || ((uintptr_t)p % bytes) == 0; };
    const bool vec = dim % 4 == 0 && al(x, 16) && al(y, 4 * esz) && y_stride % 4 == 0 && al(h, 4 * esz) && h_stride % 4 == 0 && al(bias, 4 * esz) &&
                     al(post_w, 4 * esz) && al(post_b, 4 * esz) && al(next_w, 4 * esz) && al(next_b, 4 * esz);
    const dim3 grid((unsigned)rows);
    if (act_f32) {
        if (vec) residual_dyt_kernel<float, true><<<grid, 256, 0, st>>>((const float*)y, y_stride, post, (const float*)bias, x, accumulate, next, (float*)h, h_stride, (int)dim);
        else residual_dyt_kernel<float, false><<<grid, 256, 0, st>>>((const float*)y, y_stride, post, (const float*)bias, x, accumulate, next, (float*)h, h_stride, (int)dim);
    } else {
        if (vec) residual_dyt_kernel<bf16, true><<<grid, 256, 0, st>>>((const bf16*)y, y_stride, post, (const bf16*)bias, x, accumulate, next, (bf16*)h, h_stride, (int)dim);
        else residual_dyt_kernel<bf16, false><<<grid, 256, 0, st>>>((const bf16*)y, y_stride, post, (const bf16*)bias, x, accumulate, next, (bf16*)h, h_stride, (int)dim);
    }
    NVH_CHECK_LAUNCH("nvh_residual_dyt");
    return NVH_OK;
}

extern "C" int32_t nvh_stream_cast(const float* x, void* out, int64_t out_stride, int64_t rows, int64_t dim, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_stream_cast", x && out && rows >= 0 && dim > 0 && out_stride >= dim);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    if (act_f32) stream_cast_kernel<float><<<dim3((unsigned)rows), 256, 0, st>>>(x, (float*)out, out_stride, (int)dim);
    else stream_cast_kernel<bf16><<<dim3((unsigned)rows), 256, 0, st>>>(x, (bf16*)out, out_stride, (int)dim);
    NVH_CHECK_LAUNCH("nvh_stream_cast");
    return NVH_OK;
}

extern "C" int32_t nvh_gelu_tanh_mul(const void* gate_up, int64_t row_stride, void* y, int64_t rows, int64_t inter, int32_t act_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_gelu_tanh_mul", gate_up && y && rows >= 0 && inter > 0 && row_stride >= 2 * inter);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)nvh_cdiv(rows * inter, 256);
    if (act_f32) gelu_tanh_mul_kernel<float><<<dim3(blocks), 256, 0, st>>>((const float*)gate_up, row_stride, (float*)y, rows, (int)inter);
    else gelu_tanh_mul_kernel<bf16><<<dim3(blocks), 256, 0, st>>>((const bf16*)gate_up, row_stride, (bf16*)y, rows, (int)inter);
    NVH_CHECK_LAUNCH("nvh_gelu_tanh_mul");
    return NVH_OK;
}

extern "C" int32_t nvh_gather_rows_f32(const float* x, const int32_t* index, float* out, int64_t rows, int64_t dim, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_gather_rows_f32", x && index && out && rows >= 0 && dim > 0);
    if (rows == 0) return NVH_OK;
    gather_rows_f32_kernel<<<dim3((unsigned)rows), 256, 0, (hipStream_t)stream>>>(x, index, out, (int)dim);
    NVH_CHECK_LAUNCH("nvh_gather_rows_f32");
    return NVH_OK;
}

extern "C" int32_t nvh_logit_softcap(const void* logits, int64_t row_stride, float* out, int64_t rows, int64_t vocab, float cap, int32_t act_f32,
                                     nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_logit_softcap", logits && out && rows >= 0 && vocab > 0 && row_stride >= vocab);
    if (rows == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const unsigned blocks = (unsigned)nvh_cdiv(rows * vocab, 256);
    if (act_f32) softcap_kernel<float><<<dim3(blocks), 256, 0, st>>>((const float*)logits, row_stride, out, rows, (int)vocab, cap);
    else softcap_kernel<bf16><<<dim3(blocks), 256, 0, st>>>((const bf16*)logits, row_stride, out, rows, (int)vocab, cap);
    NVH_CHECK_LAUNCH("nvh_logit_softcap");
    return NVH_OK;
}

extern "C" int32_t nvh_gemm_any_nt(const void* x, int64_t x_row_stride, const void* w, const void* bias, void* y, int64_t y_row_stride,
                                   int64_t M, int64_t N, int64_t K, int32_t in_f32, int32_t out_f32, nvh_stream_t stream) {
    NVH_STREAM_ARGS_OK("nvh_gemm_any_nt", x && w && y && M >= 0 && N > 0 && K > 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30) &&
                                              x_row_stride >= K && y_row_stride >= N);
    NVH_REQUIRE(!in_f32 || out_f32, NVH_ENOSYS, "nvh_gemm_any_nt: fp32 operands give an fp32 product");
    if (M == 0) return NVH_OK;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)nvh_cdiv(N, GT), (unsigned)nvh_cdiv(M, GT));
    if (in_f32) {
        gemm_any_f32_kernel<<<grid, 256, 0, st>>>((const float*)x, x_row_stride, (const float*)w, K, (const float*)bias, (float*)y, y_row_stride, (int)M, (int)N, (int)K);
    } else {
        const int vec_ok = K % 8 == 0 && x_row_stride % 8 == 0 && nvh_aligned16(x) && nvh_aligned16(w);
        if (out_f32) gemm_any_bf16_kernel<true><<<grid, 256, 0, st>>>((const bf16*)x, x_row_stride, (const bf16*)w, K, (const bf16*)bias, y, y_row_stride, (int)M, (int)N, (int)K, vec_ok);
        else gemm_any_bf16_kernel<false><<<grid, 256, 0, st>>>((const bf16*)x, x_row_stride, (const bf16*)w, K, (const bf16*)bias, y, y_row_stride, (int)M, (int)N, (int)K, vec_ok);
    }
    NVH_CHECK_LAUNCH("nvh_gemm_any_nt");
    return NVH_OK;
}
