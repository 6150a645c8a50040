// out[M, N] = x[M, K] . W[N, K]^T (+ bias), every multiply-add in IEEE 32-bit.
// Takes any M, N, K and every pairing of activation/weight/output element type
// that the engine uses.  This is the fallback of the bfloat16 mode for shapes the MFMA
// kernels refuse (the float32 mode's products go to gemm_f32.hip).
//
// 64x64 output tile per block of 256 threads, 4x4 outputs per thread, K in steps
// of 16 through shared memory.  Each output is summed over k in ascending order,
// whatever M is, so a row's result does not depend on what else is in the batch.
#include "common.h"

#define GT 64
#define GK 16

template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(
    const TA* __restrict__ x, const TW* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K) {
    __shared__ float xs[GK][GT + 4];
    __shared__ float ws[GK][GT + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    const int lr = tid >> 2;         // 0..63: row of the tile this thread loads
    const int lk = (tid & 3) * 4;    // 0,4,8,12: first k it loads
    const int ty = tid >> 4, tx = tid & 15;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int m = m0 + lr, n = n0 + lr;
            xs[lk + i][lr] = (m < M && k < K) ? Elem<TA>::load(x + (long)m * K + k) : 0.f;
            ws[lk + i][lr] = (n < N && k < K) ? Elem<TW>::load(w + (long)n * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += bias[n];
            Elem<TO>::store(out + (long)m * N + n, v);
        }
    }
}

template <typename TA, typename TW, typename TO>
static int launch_generic(const void* x, const void* w, const float* bias, void* out,
                          int M, int N, int K, hipStream_t stream) {
    dim3 grid(qe_cdiv(N, GT), qe_cdiv(M, GT));
    gemm_generic_kernel<TA, TW, TO><<<grid, 256, 0, stream>>>(
        (const TA*)x, (const TW*)w, bias, (TO*)out, M, N, K);
    QE_LAUNCH_CHECK();
    return 0;
}

int qe_gemm_f32(const float* x, const float* w, const float* bias, float* out, int M, int N, int K,
                hipStream_t stream);
extern int g_qe_matrix_f32;      // the all-float32 product goes to the matrix units (gemm_f32.hip) unless switched off

int qe_gemm_generic(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                    int dt_a, int dt_w, int dt_o, hipStream_t stream) {
    QE_REQUIRE(qe_cdiv(M, GT) <= 65535, "gemm: M=%d is too large for one launch", M);
    if (dt_a == QE_F32 && dt_w == QE_F32 && dt_o == QE_F32 && g_qe_matrix_f32)
        return qe_gemm_f32((const float*)x, (const float*)w, bias, (float*)out, M, N, K, stream);
    if (dt_a == QE_F32 && dt_w == QE_F32 && dt_o == QE_F32)
        return launch_generic<float, float, float>(x, w, bias, out, M, N, K, stream);
    if (dt_a == QE_BF16 && dt_w == QE_BF16 && dt_o == QE_BF16)
        return launch_generic<bf16_t, bf16_t, bf16_t>(x, w, bias, out, M, N, K, stream);
    if (dt_a == QE_BF16 && dt_w == QE_BF16 && dt_o == QE_F32)
        return launch_generic<bf16_t, bf16_t, float>(x, w, bias, out, M, N, K, stream);
    if (dt_a == QE_BF16 && dt_w == QE_F32 && dt_o == QE_BF16)
        return launch_generic<bf16_t, float, bf16_t>(x, w, bias, out, M, N, K, stream);
    if (dt_a == QE_BF16 && dt_w == QE_F32 && dt_o == QE_F32)
        return launch_generic<bf16_t, float, float>(x, w, bias, out, M, N, K, stream);
    QE_REQUIRE(false, "gemm: no kernel for element types x=%d w=%d out=%d", dt_a, dt_w, dt_o);
}
