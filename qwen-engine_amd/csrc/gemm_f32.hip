// out[M, N] = x[M, K] . W[N, K]^T (+ bias) with 32-bit operands on the matrix units: the product of
// the float32 mode.  v_mfma_f32_32x32x2_f32 multiplies 32-bit numbers and accumulates in 32-bit
// (no reduced-precision matrix mode), about ten times the rate of the vector units' multiply-adds.
//
// A block of four waves owns a 64 x 64 tile of the output, a wave a 32 x 32 quarter.  K goes in steps
// of 16 through shared memory; the next step's operands are asked for from global memory before
// the current step is computed.  For a step, lane (h, r), h = lane / 32, r = lane % 32, reads
// x[row r][8 h .. 8 h + 8] and W[row r][8 h .. 8 h + 8] as two 16-byte pieces each, and the j-th
// MFMA of the step takes element j of both (which k stands at which place of an MFMA's sum does
// not matter, as long as both operands have it at the same).  Every output is summed in the same
// order whatever M is, so a row's result does not depend on what else is in the batch.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(16))) float floatx16;

#define FT 64         // tile rows and columns
#define FK 16         // k step
#define FROW (FK + 4) // floats of a staged row: padded, so that the 32 rows a wave reads lie in different banks

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                       const float* __restrict__ bias, float* __restrict__ out,
                                                       int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) float xs[2][FT][FROW];
    __shared__ __attribute__((aligned(16))) float ws[2][FT][FROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int h = lane >> 5, r = lane & 31;
    const int m0 = blockIdx.y * FT, n0 = blockIdx.x * FT;
    // staging: thread tid brings four consecutive k of one row of each operand
    const int srow = tid >> 2, sk = (tid & 3) * 4;
    const bool xrow_ok = m0 + srow < M, wrow_ok = n0 + srow < N;
    const float* xsrc = x + (long)(xrow_ok ? m0 + srow : 0) * K + sk;
    const float* wsrc = w + (long)(wrow_ok ? n0 + srow : 0) * K + sk;
    const bool vec = (K & 3) == 0;

    auto fetch = [&](const float* src, bool row_ok, int k0, floatx4& v) {
        v = floatx4{0.f, 0.f, 0.f, 0.f};
        if (!row_ok) return;
        if (vec && k0 + sk + 3 < K) {
            v = *(const floatx4*)(src + k0);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (k0 + sk + e < K) v[e] = src[k0 + e];
        }
    };

    floatx16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    floatx4 xv, wv;
    fetch(xsrc, xrow_ok, 0, xv);
    fetch(wsrc, wrow_ok, 0, wv);
    *(floatx4*)&xs[0][srow][sk] = xv;
    *(floatx4*)&ws[0][srow][sk] = wv;
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += FK) {
        const bool more = k0 + FK < K;
        if (more) {
            fetch(xsrc, xrow_ok, k0 + FK, xv);
            fetch(wsrc, wrow_ok, k0 + FK, wv);
        }
        const float* xa = &xs[buf][wm * 32 + r][h * 8];
        const float* wa = &ws[buf][wn * 32 + r][h * 8];
        const floatx4 a0 = *(const floatx4*)xa, a1 = *(const floatx4*)(xa + 4);
        const floatx4 b0 = *(const floatx4*)wa, b1 = *(const floatx4*)(wa + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[j], b0[j], acc, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[j], b1[j], acc, 0, 0, 0);
        if (more) {
            *(floatx4*)&xs[buf ^ 1][srow][sk] = xv;     // (that buffer's readers passed the last barrier)
            *(floatx4*)&ws[buf ^ 1][srow][sk] = wv;
        }
        __syncthreads();
        buf ^= 1;
    }
    // lane (h, r) holds out[m0 + 32 wm + 8 b + 4 h + i][n0 + 32 wn + r] as element 4 b + i
    const int n = n0 + wn * 32 + r;
    if (n < N) {
        const float bv = bias ? bias[n] : 0.f;
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + wm * 32 + 8 * b + 4 * h + i;
                if (m < M) out[(long)m * N + n] = bias ? acc[4 * b + i] + bv : acc[4 * b + i];
            }
    }
}

int qe_gemm_f32(const float* x, const float* w, const float* bias, float* out, int M, int N, int K,
                hipStream_t stream) {
    QE_REQUIRE(qe_cdiv(M, FT) <= 65535, "gemm (32-bit): M=%d is too large for one launch", M);
    dim3 grid(qe_cdiv(N, FT), qe_cdiv(M, FT));
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(x, w, bias, out, M, N, K);
    QE_LAUNCH_CHECK();
    return 0;
}
