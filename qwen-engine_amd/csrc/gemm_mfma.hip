// Matrix product for many rows of activations (prefill): out[M, N] = x[M, K] . W[N, K]^T (+ bias),
// bfloat16 in, 32-bit accumulation with v_mfma_f32_32x32x16_bf16, output bfloat16 or float32.
//
// A block of 256 threads (4 waves, 2 x 2) computes a TM x 128 tile of the output, TM = 128 or 64
// (the smaller one when the larger would leave compute units without a block); each wave
// a quarter as (TM / 64) x 2 MFMA tiles.  K is walked in steps of 64 through shared memory with
// two buffers: while the MFMAs of one step run, the 16-byte global loads of the next are in
// flight.  Both operands are K-contiguous in memory, so they are staged alike: a row of 64
// bfloat16 (128 bytes) is padded to 144 bytes, which makes the 16-byte fragment reads of the
// 32 rows of an MFMA operand fall into distinct banks.
//
// Rows of x beyond M and rows of W beyond N are read as zero and never stored; K must be a
// multiple of 8 (16-byte loads), a tail shorter than 64 is filled with zeros.
// blockIdx.x walks the tiles so that consecutive blocks share the same rows of W (one
// column of tiles after the other), which keeps an XCD's L2 on few weight rows at a time.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) unsigned int uint4_t;

#define BN 128
#define BK 64
#define ROWB 144   // bytes of a staged row: 128 of data + 16 of padding

template <typename TO, int BM>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int tiles_m) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // buffer b: A rows at smem + b * (BM + BN) * ROWB, then B rows
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    constexpr int WM = BM / 2;         // rows of a wave's part
    constexpr int MI = WM / 32;        // MFMA tiles along m per wave
    constexpr int LD = (BM + BN) / 32; // 16-byte pieces a thread stages per step
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * 64;

    // global -> shared: a step has (BM + BN) rows x 8 pieces of 16 bytes, LD per thread
    // piece q = tid + 256 * i: row = q / 8, piece-in-row = q % 8
    const int nk = (K + BK - 1) / BK;
    uint4_t stage[LD];

#define LOAD_GLOBAL(kt_)                                                                 \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                     \
        const int q = tid + 256 * i;                                                     \
        const int row = q >> 3, pc = q & 7;                                              \
        const int k = (kt_) * BK + pc * 8;                                               \
        const bool is_a = row < BM;                                                      \
        const int grow = is_a ? m0 + row : n0 + row - BM;                                \
        const bool ok = k < K && grow < (is_a ? M : N);                                  \
        const bf16_t* src = (is_a ? x : w) + (long)(ok ? grow : 0) * K + (ok ? k : 0);   \
        const uint4_t v = *(const uint4_t*)src;                                          \
        stage[i] = ok ? v : uint4_t{0u, 0u, 0u, 0u};                                     \
    }
#define STORE_SHARED(buf_)                                                               \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                      \
        const int q = tid + 256 * i;                                                     \
        const int row = q >> 3, pc = q & 7;                                              \
        *(uint4_t*)(smem + (buf_) * (BM + BN) * ROWB + row * ROWB + pc * 16) = stage[i]; \
    }

    floatx16 acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    LOAD_GLOBAL(0)
    STORE_SHARED(0)
    __syncthreads();
    const int fr = lane & 31;          // row of the fragment this lane holds
    const int fk = (lane >> 5) * 16;   // byte offset of its 8 k values within a 16-wide k step
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) { LOAD_GLOBAL(kt + 1) }
        const unsigned char* a_base = smem + buf * (BM + BN) * ROWB + (wm + fr) * ROWB + fk;
        const unsigned char* b_base = smem + buf * (BM + BN) * ROWB + (BM + wn + fr) * ROWB + fk;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 a[MI], b[2];
#pragma unroll
            for (int i = 0; i < MI; ++i) a[i] = *(const bf16x8*)(a_base + i * 32 * ROWB + ks * 32);
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = *(const bf16x8*)(b_base + j * 32 * ROWB + ks * 32);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) { STORE_SHARED(buf ^ 1) }   // the other buffer: its readers finished before the last barrier
        __syncthreads();
    }

    // C of a 32x32 MFMA: lane holds column (lane % 32), rows 8 * b + 4 * (lane / 32) + r for e = 4 * b + r.
    // With A = x rows and B = W rows that is: token row m, output column n = lane % 32.
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn + j * 32 + (lane & 31);
            if (n >= N) continue;
            const float bv = bias ? bias[n] : 0.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m < M) Elem<TO>::store(out + (long)m * N + n, acc[i][j][e] + bv);
            }
        }
}

bool qe_gemm_mfma_ok(int M, int N, int K, int dt_a, int dt_w) {
    return dt_a == QE_BF16 && dt_w == QE_BF16 && M > 64 && K % 8 == 0 && K >= 64;
}

template <typename TO, int BM>
static int launch_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                       hipStream_t stream) {
    const int tiles_m = qe_cdiv(M, BM), tiles_n = qe_cdiv(N, BN);
    const long blocks = (long)tiles_m * tiles_n;
    QE_REQUIRE(blocks <= 2147483647L, "mfma gemm: too many tiles");
    const size_t shmem = 2 * (BM + BN) * ROWB;
    static bool attr_set = false;   // one flag per instantiation
    if (!attr_set) {
        (void)hipFuncSetAttribute((const void*)gemm_mfma_kernel<TO, BM>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        attr_set = true;
    }
    gemm_mfma_kernel<TO, BM><<<(int)blocks, 256, shmem, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, (TO*)out, M, N, K, tiles_m);
    QE_LAUNCH_CHECK();
    return 0;
}

int qe_gemm_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int dt_o,
                 hipStream_t stream) {
    QE_REQUIRE(K % 8 == 0, "mfma gemm: K=%d is no multiple of 8", K);
    // 128-row tiles unless they give fewer than two blocks per compute unit (256 of them)
    const bool small = (long)qe_cdiv(M, 128) * qe_cdiv(N, BN) < 512;
    if (dt_o == QE_BF16)
        return small ? launch_mfma<bf16_t, 64>(x, w, bias, out, M, N, K, stream)
                     : launch_mfma<bf16_t, 128>(x, w, bias, out, M, N, K, stream);
    return small ? launch_mfma<float, 64>(x, w, bias, out, M, N, K, stream)
                 : launch_mfma<float, 128>(x, w, bias, out, M, N, K, stream);
}
