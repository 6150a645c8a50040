// Matrix product for many rows of activations (prefill): out[M, N] = x[M, K] . W[N, K]^T (+ bias),
// bfloat16 in, 32-bit accumulation with v_mfma_f32_32x32x16_bf16, output bfloat16 or float32.
//
// A block of 256 threads (4 waves, 2 x 2) computes a BM x BN tile of the output; each wave a
// quarter as (BM / 64) x (BN / 64) MFMA tiles.  K is walked in steps of BK through shared memory
// with two buffers: while the MFMAs of one step run, the 16-byte global loads of the next are in
// flight.  Both operands are K-contiguous in memory, so they are staged alike: a row of BK
// bfloat16 is padded by 16 bytes, which makes the 16-byte fragment reads of the 32 rows of an
// MFMA operand fall into distinct banks.
//
// The kernel is bound by shared-memory traffic rather than by the MFMA units unless a wave's
// part is large (an operand fragment read once serves several MFMAs): 256 x 128 tiles are used
// where they still give every compute unit a block, 128 x 128 and 64 x 128 for smaller products.
//
// Rows of x beyond M and rows of W beyond N are read as zero and never stored; K must be a
// multiple of 8 (16-byte loads), a tail shorter than BK is filled with zeros.
// blockIdx.x walks the tiles so that consecutive blocks share the same rows of W (one
// column of tiles after the other), which keeps an XCD's L2 on few weight rows at a time.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) unsigned int uint4_t;

template <typename TO, int BM, int BN, int BK, int MINB>
__global__ __launch_bounds__(256, MINB) void gemm_mfma_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int tiles_m) {
    constexpr int ROWB = BK * 2 + 16;       // bytes of a staged row
    constexpr int PPR = BK / 8;             // 16-byte pieces per row
    constexpr int WM = BM / 2, WN = BN / 2; // a wave's part
    constexpr int MI = WM / 32, NJ = WN / 32;
    constexpr int LD = (BM + BN) * PPR / 256;   // pieces a thread stages per step
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // buffer b: A rows at smem + b * (BM + BN) * ROWB, then B rows
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

    const int nk = (K + BK - 1) / BK;
    uint4_t stage[LD];

    // A piece outside the matrices is loaded from a valid address all the same and replaced by
    // zeros only when it is stored to shared memory: a select right after the load would make
    // the wave wait for the load before it computes.
#define LOAD_GLOBAL(kt_)                                                                 \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                     \
        const int q = tid + 256 * i;                                                     \
        const int row = q / PPR, pc = q % PPR;                                           \
        const int k = (kt_) * BK + pc * 8;                                               \
        const bool is_a = row < BM;                                                      \
        const int grow = is_a ? m0 + row : n0 + row - BM;                                \
        const bool ok = k < K && grow < (is_a ? M : N);                                  \
        const bf16_t* src = (is_a ? x : w) + (long)(ok ? grow : 0) * K + (ok ? k : 0);   \
        stage[i] = *(const uint4_t*)src;                                                 \
    }
#define STORE_SHARED(buf_, kt_)                                                          \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                     \
        const int q = tid + 256 * i;                                                     \
        const int row = q / PPR, pc = q % PPR;                                           \
        const int k = (kt_) * BK + pc * 8;                                               \
        const bool is_a = row < BM;                                                      \
        const int grow = is_a ? m0 + row : n0 + row - BM;                                \
        const bool ok = k < K && grow < (is_a ? M : N);                                  \
        *(uint4_t*)(smem + (buf_) * (BM + BN) * ROWB + row * ROWB + pc * 16) =           \
            ok ? stage[i] : uint4_t{0u, 0u, 0u, 0u};                                     \
    }

    floatx16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    LOAD_GLOBAL(0)
    STORE_SHARED(0, 0)
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
            bf16x8 a[MI], b[NJ];
#pragma unroll
            for (int i = 0; i < MI; ++i) a[i] = *(const bf16x8*)(a_base + i * 32 * ROWB + ks * 32);
#pragma unroll
            for (int j = 0; j < NJ; ++j) b[j] = *(const bf16x8*)(b_base + j * 32 * ROWB + ks * 32);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) { STORE_SHARED(buf ^ 1, kt + 1) }   // the other buffer: its readers finished before the last barrier
        __syncthreads();
    }
#undef LOAD_GLOBAL
#undef STORE_SHARED

    // C of a 32x32 MFMA: lane holds column (lane % 32), rows 8 * b + 4 * (lane / 32) + r for e = 4 * b + r.
    // With A = x rows and B = W rows that is: token row m, output column n = lane % 32.
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
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

template <typename TO, int BM, int BN, int BK, int MINB>
static int launch_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                       hipStream_t stream) {
    const int tiles_m = qe_cdiv(M, BM), tiles_n = qe_cdiv(N, BN);
    const long blocks = (long)tiles_m * tiles_n;
    QE_REQUIRE(blocks <= 2147483647L, "mfma gemm: too many tiles");
    const size_t shmem = 2 * (BM + BN) * (BK * 2 + 16);
    static bool attr_set = false;   // one flag per instantiation
    if (!attr_set) {
        (void)hipFuncSetAttribute((const void*)gemm_mfma_kernel<TO, BM, BN, BK, MINB>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        attr_set = true;
    }
    gemm_mfma_kernel<TO, BM, BN, BK, MINB><<<(int)blocks, 256, shmem, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, bias, (TO*)out, M, N, K, tiles_m);
    QE_LAUNCH_CHECK();
    return 0;
}

template <typename TO>
static int pick_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                     int tile, hipStream_t stream) {
    const long cus = 256;
    const long big = (long)qe_cdiv(M, 256) * qe_cdiv(N, 128), mid = (long)qe_cdiv(M, 128) * qe_cdiv(N, 128);
    // the largest tile that still gives every compute unit two blocks (one, for the middle size)
    if (tile == 0) tile = big >= 2 * cus ? 256 : (mid >= cus ? 128 : 64);
    if (tile == 256) return launch_mfma<TO, 256, 128, 32, 2>(x, w, bias, out, M, N, K, stream);
    if (tile == 128) return launch_mfma<TO, 128, 128, 64, 2>(x, w, bias, out, M, N, K, stream);
    return launch_mfma<TO, 64, 128, 64, 2>(x, w, bias, out, M, N, K, stream);
}

// tile: rows of the output tile (256, 128 or 64), 0 to choose by the shape
int qe_gemm_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int dt_o,
                 int tile, hipStream_t stream) {
    QE_REQUIRE(K % 8 == 0, "mfma gemm: K=%d is no multiple of 8", K);
    QE_REQUIRE(tile == 0 || tile == 256 || tile == 128 || tile == 64, "mfma gemm: tile of %d rows", tile);
    if (dt_o == QE_BF16) return pick_mfma<bf16_t>(x, w, bias, out, M, N, K, tile, stream);
    return pick_mfma<float>(x, w, bias, out, M, N, K, tile, stream);
}
