// Entry point of all matrix products: picks a kernel for the shape and types.
#include "common.h"

int qe_gemm_generic(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                    int dt_a, int dt_w, int dt_o, hipStream_t stream);

// algo: 0 = choose, 1 = generic 32-bit kernel.
extern "C" int qe_gemm(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                       int dt_a, int dt_w, int dt_o, int algo, hipStream_t stream) {
    QE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    QE_REQUIRE(algo == 0 || algo == 1, "gemm: unknown algo %d", algo);
    return qe_gemm_generic(x, w, bias, out, M, N, K, dt_a, dt_w, dt_o, stream);
}
