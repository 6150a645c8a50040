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

// SILU: W holds gate and up rows interleaved in blocks of 32 (gate 0..31, up 0..31, gate 32..63,
// ...), N counts all of them, and the result is silu(gate) * up, N / 2 wide: the two MFMA tiles a
// lane holds side by side are the gate and the up of the same outputs.
template <typename TO, int BM, int BN, int BK, int MINB, bool SILU>
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
    // the wave wait for the load before it computes.  Addresses are formed once; a step adds BK.
    const bf16_t* src[LD];
    bool row_ok[LD];
    int kofs[LD], dst[LD];
#pragma unroll
    for (int i = 0; i < LD; ++i) {
        const int q = tid + 256 * i;
        const int row = q / PPR, pc = q % PPR;
        const bool is_a = row < BM;
        const int grow = is_a ? m0 + row : n0 + row - BM;
        row_ok[i] = grow < (is_a ? M : N);
        kofs[i] = pc * 8;
        src[i] = (is_a ? x : w) + (long)(row_ok[i] ? grow : 0) * K + pc * 8;
        dst[i] = row * ROWB + pc * 16;
    }
#define LOAD_GLOBAL(kt_)                                                                 \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                     \
        const bool ok = (kt_) * BK + kofs[i] < K;                                        \
        stage[i] = *(const uint4_t*)(ok ? src[i] + (kt_) * BK : src[i]);                 \
    }
#define STORE_SHARED(buf_, kt_)                                                          \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                     \
        const bool ok = row_ok[i] && (kt_) * BK + kofs[i] < K;                           \
        *(uint4_t*)(smem + (buf_) * (BM + BN) * ROWB + dst[i]) =                         \
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
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) { STORE_SHARED(buf ^ 1, kt + 1) }   // the other buffer: its readers finished before the last barrier
        __syncthreads();
    }
#undef LOAD_GLOBAL
#undef STORE_SHARED

    // The MFMA is given the W rows as its first operand and the x rows as its second, so its
    // result is the tile transposed: a lane holds, for the token row m = lane % 32, the outputs
    // n = 8 b + 4 (lane / 32) + r (e = 4 b + r): four consecutive n at a time, one 8- or 16-byte store.
    const int NO = SILU ? N / 2 : N;             // width of the output
    const bool vec_ok = (NO % 4) == 0;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m0 + wm + i * 32 + (lane & 31);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < NJ; j += (SILU ? 2 : 1))
#pragma unroll
            for (int bq = 0; bq < 4; ++bq) {
                const int nw = n0 + wn + j * 32;                       // first weight row of the MFMA tile
                const int n = (SILU ? nw / 2 : nw) + 8 * bq + 4 * (lane >> 5);
                if (n >= NO) continue;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (SILU) {
                        const float gt = acc[i][j][4 * bq + r], up = acc[i][j + (SILU ? 1 : 0)][4 * bq + r];
                        v[r] = gt / (1.f + __expf(-gt)) * up;
                    } else {
                        v[r] = acc[i][j][4 * bq + r] + ((bias && n + r < NO) ? bias[n + r] : 0.f);
                    }
                }
                TO* o = out + (long)m * NO + n;
                if (vec_ok) {
                    Vec4<TO>::store(o, v);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) if (n + r < NO) Elem<TO>::store(o + r, v[r]);
                }
            }
    }
}

bool qe_gemm_mfma_ok(int M, int N, int K, int dt_a, int dt_w) {
    return dt_a == QE_BF16 && dt_w == QE_BF16 && M > 64 && K % 8 == 0 && K >= 64;
}

template <typename TO, int BM, int BN, int BK, int MINB, bool SILU>
static int launch_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                       hipStream_t stream) {
    const int tiles_m = qe_cdiv(M, BM), tiles_n = qe_cdiv(N, BN);
    const long blocks = (long)tiles_m * tiles_n;
    QE_REQUIRE(blocks <= 2147483647L, "mfma gemm: too many tiles");
    const size_t shmem = 2 * (BM + BN) * (BK * 2 + 16);
    static bool attr_set = false;   // one flag per instantiation
    if (!attr_set) {
        (void)hipFuncSetAttribute((const void*)gemm_mfma_kernel<TO, BM, BN, BK, MINB, SILU>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        attr_set = true;
    }
    gemm_mfma_kernel<TO, BM, BN, BK, MINB, SILU><<<(int)blocks, 256, shmem, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, bias, (TO*)out, M, N, K, tiles_m);
    QE_LAUNCH_CHECK();
    return 0;
}

template <typename TO, bool SILU>
static int pick_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                     int tile, hipStream_t stream) {
    const long cus = 256;
    const long big = (long)qe_cdiv(M, 256) * qe_cdiv(N, 128), mid = (long)qe_cdiv(M, 128) * qe_cdiv(N, 128);
    // the largest tile that still gives every compute unit two blocks (one, for the middle size)
    if (tile == 0) tile = big >= 2 * cus ? 256 : (mid >= cus ? 128 : 64);
    if (tile == 256) return launch_mfma<TO, 256, 128, 32, 2, SILU>(x, w, bias, out, M, N, K, stream);
    if (tile == 128) return launch_mfma<TO, 128, 128, 64, 2, SILU>(x, w, bias, out, M, N, K, stream);
    return launch_mfma<TO, 64, 128, 64, 2, SILU>(x, w, bias, out, M, N, K, stream);
}

// tile: rows of the output tile (256, 128 or 64), 0 to choose by the shape.  silu: w is [N, K] with
// gate and up rows interleaved in blocks of 32, out is [M, N / 2] = silu(gate) * up.
int qe_gemm_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int dt_o,
                 int tile, bool silu, hipStream_t stream) {
    QE_REQUIRE(K % 8 == 0, "mfma gemm: K=%d is no multiple of 8", K);
    QE_REQUIRE(tile == 0 || tile == 256 || tile == 128 || tile == 64, "mfma gemm: tile of %d rows", tile);
    if (silu) {
        QE_REQUIRE(!bias && N % 64 == 0, "mfma gemm: silu-mul takes no bias and gate|up rows in blocks of 32");
        if (dt_o == QE_BF16) return pick_mfma<bf16_t, true>(x, w, bias, out, M, N, K, tile, stream);
        return pick_mfma<float, true>(x, w, bias, out, M, N, K, tile, stream);
    }
    if (dt_o == QE_BF16) return pick_mfma<bf16_t, false>(x, w, bias, out, M, N, K, tile, stream);
    return pick_mfma<float, false>(x, w, bias, out, M, N, K, tile, stream);
}
