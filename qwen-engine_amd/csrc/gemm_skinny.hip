// Matrix product for few rows of activations (decode): out[M, N] = x[M, K] . W[N, K]^T, M <= 64,
// bfloat16 in, 32-bit accumulation on the MFMA units.  The weights are streamed from HBM
// exactly once; this kernel is bound by that stream.
//
// A block of 4 waves owns 16 rows of W (or two such tiles).  The rows are the M side of v_mfma_f32_16x16x32_bf16
// (lane (g, r), g = lane / 16, r = lane % 16, holds W[n0 + r][c * 32 + g * 8 .. + 8]: one 16-byte
// load), the tokens are the N side (lane (g, r) holds x[j * 16 + r][the same k]).  Wave w takes
// the 32-wide chunks c = w, w + 4, ... of K, so the four waves read neighbouring 64-byte pieces
// of the same rows at the same time; their partial tiles are summed through shared memory.
// The result tile has, per lane, 4 consecutive n for one token: one 8- or 16-byte store.
//
// Epilogues: store (+ bias); add into a 32-bit residual stream; silu(gate) * up, where W holds
// the gate rows followed by the up rows and a block owns 16 of each; 32-bit partial products
// of a product cut along K over several blocks (for matrices with few rows, to fill the chip).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SILU_MUL = 2, EPI_PARTIAL = 3, EPI_SILU_MUL_IL = 4 };

// grid (N / (16 NT), S): block (bx, s) sums the chunks [s * cps, (s + 1) * cps) of K.  With S > 1 the
// epilogue is EPI_PARTIAL: 32-bit partial products out[s][M][N] that the consumer adds up in the
// order of s (the fused residual-add + norm kernel does), so the sum has one fixed order.
// NT: tiles of 16 rows of W a block owns.  Every wave reads the activations of its chunks itself
// (M rows against the block's 16 NT rows of W), so with more than 16 rows of activations most of
// what a block reads is activations, from the L2; two tiles a block halve that.
template <int MT, int NT, int EPI, typename TO>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int cps) {
    constexpr bool SILU = EPI == EPI_SILU_MUL || EPI == EPI_SILU_MUL_IL;
    constexpr int NW = SILU ? 2 : 1;   // weight tiles per tile of outputs
    constexpr int U = (MT == 1 && !SILU && NT == 1) ? 8 : ((MT <= 2) ? 4 : 2);   // chunks whose loads are issued together
    __shared__ float red[4][NT][NW][MT][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, r = lane & 15;
    const int n0 = blockIdx.x * 16 * NT;
    const int nchunks = K / 32;
    const int c_begin = blockIdx.y * cps;
    const int c_end = min(nchunks, c_begin + cps);

    floatx4 acc[NT][NW][MT];
#pragma unroll
    for (int q = 0; q < NT; ++q)
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int j = 0; j < MT; ++j) acc[q][a][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    bool row_ok[NT];
    const bf16_t* wrow0[NT];
    const bf16_t* wrow1[NT];
#pragma unroll
    for (int q = 0; q < NT; ++q) {
        row_ok[q] = n0 + q * 16 + r < N;
        // gate row n and up row n: N rows apart, or, with the rows interleaved in blocks of 32
        // (gate 0..31, up 0..31, gate 32..63, ...), 32 rows apart inside the block of 64
        const int nrow = row_ok[q] ? n0 + q * 16 + r : 0;
        const long wr = (EPI == EPI_SILU_MUL_IL) ? (long)(nrow >> 5) * 64 + (nrow & 31) : nrow;
        wrow0[q] = w + wr * K + g * 8;
        wrow1[q] = (EPI == EPI_SILU_MUL_IL) ? wrow0[q] + 32L * K : (SILU ? wrow0[q] + (long)N * K : wrow0[q]);
    }
    const bf16_t* xrow[MT];
    bool tok_ok[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) {
        tok_ok[j] = j * 16 + r < M;
        xrow[j] = x + (long)(tok_ok[j] ? j * 16 + r : 0) * K + g * 8;
    }
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

    for (int c = c_begin + wave; c < c_end; c += 4 * U) {
        bf16x8 a0[U][NT], a1[U][NT], b[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int cc = c + 4 * u;
            const bool ok = cc < c_end;
#pragma unroll
            for (int q = 0; q < NT; ++q) {
                a0[u][q] = (ok && row_ok[q]) ? *(const bf16x8*)(wrow0[q] + cc * 32) : zero;
                if (SILU) a1[u][q] = (ok && row_ok[q]) ? *(const bf16x8*)(wrow1[q] + cc * 32) : zero;
            }
#pragma unroll
            for (int j = 0; j < MT; ++j) b[u][j] = (ok && tok_ok[j]) ? *(const bf16x8*)(xrow[j] + cc * 32) : zero;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int q = 0; q < NT; ++q)
#pragma unroll
                for (int j = 0; j < MT; ++j) {
                    acc[q][0][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[u][q], b[u][j], acc[q][0][j], 0, 0, 0);
                    if (SILU)
                        acc[q][1][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[u][q], b[u][j], acc[q][1][j], 0, 0, 0);
                }
    }
#pragma unroll
    for (int q = 0; q < NT; ++q)
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int j = 0; j < MT; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[wave][q][a][j][lane][i] = acc[q][a][j][i];
    __syncthreads();
    // wave w finishes the (output tile, token tile) pairs w, w + 4, ...
    for (int qj = wave; qj < NT * MT; qj += 4) {
        const int q = qj / MT, j = qj % MT;
        float v[NW][4];
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                v[a][i] = red[0][q][a][j][lane][i] + red[1][q][a][j][lane][i] + red[2][q][a][j][lane][i] +
                          red[3][q][a][j][lane][i];
        const int t = j * 16 + r;          // lane (g, r): token t, rows n0 + q * 16 + g * 4 + i
        if (t >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + q * 16 + g * 4 + i;
            if (n >= N) continue;
            float y = v[0][i];
            if (SILU) {
                y = y / (1.f + __expf(-y)) * v[1][i];
            } else if (bias && blockIdx.y == 0) {
                y += bias[n];
            }
            if (EPI == EPI_PARTIAL) {
                ((float*)out)[((long)blockIdx.y * M + t) * N + n] = y;
            } else if (EPI == EPI_RESIDUAL) {
                float* o = (float*)out + (long)t * N + n;
                *o = *o + y;
            } else {
                Elem<TO>::store(out + (long)t * N + n, y);
            }
        }
    }
}

template <int EPI, typename TO>
static int launch_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                         int splits, hipStream_t stream) {
    const int cps = qe_cdiv(K / 32, splits);
    const int mt = qe_cdiv(M, 16);
    constexpr bool SILU = EPI == EPI_SILU_MUL || EPI == EPI_SILU_MUL_IL;
    // two tiles of outputs a block where the activations have more than 16 rows and there are blocks
    // enough all the same (with silu.mul a tile of outputs is two tiles of W already: only up to 32 rows)
    const bool two = mt >= 2 && (!SILU || mt <= 2) && (long)qe_cdiv(N, 32) * splits >= 256;
    const dim3 grid(qe_cdiv(N, two ? 32 : 16), splits);
#define QE_SKINNY(MT_, NT_)                                                                            \
    gemm_skinny_kernel<MT_, NT_, EPI, TO><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, \
                                                                    (TO*)out, M, N, K, cps)
    if (two) {
        switch (mt) {
            case 2: QE_SKINNY(2, 2); break;
            case 3: if constexpr (!SILU) QE_SKINNY(3, 2); break;
            default: if constexpr (!SILU) QE_SKINNY(4, 2); break;
        }
    } else {
        switch (mt) {
            case 1: QE_SKINNY(1, 1); break;
            case 2: QE_SKINNY(2, 1); break;
            case 3: QE_SKINNY(3, 1); break;
            default: QE_SKINNY(4, 1); break;
        }
    }
#undef QE_SKINNY
    QE_LAUNCH_CHECK();
    return 0;
}

bool qe_gemm_skinny_ok(int M, int N, int K, int dt_a, int dt_w) {
    return dt_a == QE_BF16 && dt_w == QE_BF16 && M >= 1 && M <= 64 && K % 32 == 0 && K >= 32;
}

// How many partial products a [M, N] = [M, K] . [N, K]^T product is best cut into along K so that
// the launch has some 512 blocks, each wave still summing at least two chunks.
int qe_gemm_skinny_splits(int N, int K) {
    const int blocks = qe_cdiv(N, 16);
    int s = 512 / (blocks > 0 ? blocks : 1);
    const int most = (K / 32) / 8;
    if (s > most) s = most;
    if (s > 16) s = 16;
    return s < 1 ? 1 : s;
}

// epilogue EPI_STORE: out [M, N] in dt_o.  EPI_RESIDUAL: out is the 32-bit stream [M, N], added to.
// EPI_SILU_MUL: w is [2 N, K] (gate rows, then up rows), out [M, N] in dt_o.
// EPI_SILU_MUL_IL: the same with gate and up rows interleaved in blocks of 32.
// EPI_PARTIAL: out is float [splits, M, N]; the product is the sum over the first index.
int qe_gemm_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                   int dt_o, int epilogue, int splits, hipStream_t stream) {
    QE_REQUIRE(M >= 1 && M <= 64 && K % 32 == 0, "skinny gemm: M=%d K=%d not taken", M, K);
    QE_REQUIRE(splits >= 1 && splits <= 64 && (epilogue == EPI_PARTIAL || splits == 1),
               "skinny gemm: %d splits with epilogue %d", splits, epilogue);
    if (epilogue == EPI_PARTIAL) {
        QE_REQUIRE(dt_o == QE_F32, "skinny gemm: partial products are 32-bit");
        return launch_skinny<EPI_PARTIAL, float>(x, w, bias, out, M, N, K, splits, stream);
    }
    if (epilogue == EPI_RESIDUAL) {
        QE_REQUIRE(dt_o == QE_F32, "skinny gemm: the residual stream is 32-bit");
        return launch_skinny<EPI_RESIDUAL, float>(x, w, bias, out, M, N, K, 1, stream);
    }
    if (epilogue == EPI_SILU_MUL) {
        QE_REQUIRE(!bias, "skinny gemm: silu-mul takes no bias");
        if (dt_o == QE_BF16) return launch_skinny<EPI_SILU_MUL, bf16_t>(x, w, bias, out, M, N, K, 1, stream);
        return launch_skinny<EPI_SILU_MUL, float>(x, w, bias, out, M, N, K, 1, stream);
    }
    if (epilogue == EPI_SILU_MUL_IL) {
        QE_REQUIRE(!bias && N % 32 == 0, "skinny gemm: interleaved silu-mul takes no bias and N in blocks of 32");
        if (dt_o == QE_BF16) return launch_skinny<EPI_SILU_MUL_IL, bf16_t>(x, w, bias, out, M, N, K, 1, stream);
        return launch_skinny<EPI_SILU_MUL_IL, float>(x, w, bias, out, M, N, K, 1, stream);
    }
    QE_REQUIRE(epilogue == EPI_STORE, "skinny gemm: unknown epilogue %d", epilogue);
    if (dt_o == QE_BF16) return launch_skinny<EPI_STORE, bf16_t>(x, w, bias, out, M, N, K, 1, stream);
    return launch_skinny<EPI_STORE, float>(x, w, bias, out, M, N, K, 1, stream);
}
