// A measurement, not part of a model step: what the matrix units reach when nothing feeds them
// but registers.  Every wave repeats v_mfma_f32_32x32x16_bf16 on operands it holds, with four
// accumulators in turn so that no instruction waits for the one before it; eight waves a compute
// unit.  The rate a step's matrix products reach is judged against this as well as against the
// published peak.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;

__global__ __launch_bounds__(256) void mfma_probe_kernel(float* __restrict__ out, int iters) {
    const int lane = threadIdx.x & 63;
    bf16x8 a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (__bf16)(0.001f * (float)((lane + e) % 7));
        b[e] = (__bf16)(0.002f * (float)((lane + 2 * e) % 5));
    }
    floatx16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) s += acc[j][i];
    out[(long)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Launches `blocks` blocks of four waves that each issue 4 * iters MFMAs of 32 x 32 x 16 (32768
// floating-point operations each); out holds blocks * 256 floats.  Returns the operations of the launch in *flops.
extern "C" int qe_mfma_probe(float* out, int blocks, int iters, double* flops, hipStream_t stream) {
    QE_REQUIRE(blocks > 0 && iters > 0 && out, "mfma probe: bad arguments");
    mfma_probe_kernel<<<blocks, 256, 0, stream>>>(out, iters);
    QE_LAUNCH_CHECK();
    if (flops) *flops = (double)blocks * 4.0 * (double)iters * 4.0 * 32768.0;
    return 0;
}
