// Matrix product for few rows of activations (decode): out[M, N] = x[M, K] . W[N, K]^T, M <= 64,
// bfloat16 in, 32-bit accumulation on the MFMA units.  The weights are streamed from HBM
// exactly once; this kernel is bound by that stream.
//
// A block of 4 waves owns 16 rows of W (or two such tiles).  The rows are the M side of v_mfma_f32_16x16x32_bf16
// (lane (g, r), g = lane / 16, r = lane % 16, holds W[n0 + r][c * 32 + g * 8 .. + 8]: one 16-byte
// load), the tokens are the N side (lane (g, r) holds x[j * 16 + r][the same k]).  The waves split
// the 32-wide chunks of K between them (in pairs: wave w takes the chunks 2 w, 2 w + 1, 2 w + 8, ...;
// see the kernel); their partial tiles are summed through shared memory.
// The result tile has, per lane, 4 consecutive n for one token: one 8- or 16-byte store.
//
// Against a large matrix with up to 16 rows of x the loads do not follow the operand layout (4 lanes
// and 64 bytes a row) but take whole 128-byte lines, 8 lanes a row, and the registers are turned into
// the operand layout through shared memory: the L1 serves half as many requests, which is what bounds
// the stream once rows of x are read beside the weights (see LN in the kernel).
//
// Epilogues: store (+ bias); add into a 32-bit residual stream; silu(gate) * up, where W holds
// the gate rows followed by the up rows and a block owns 16 of each; 32-bit partial products
// of a product cut along K over several blocks (for matrices with few rows, to fill the chip).
//
// Prologue (up to 16 rows): the RMSNorm that stands before the product.  x is then the 32-bit
// residual stream; every block norms the rows itself (sum of squares, rsqrt, weight: the same
// arithmetic in the same order as the norm kernel, so the same bits), leaves them as bfloat16 in
// shared memory and takes its operands from there.  A decode step is a chain of short dependent
// kernels, each of which costs a few microseconds whatever it does: the norm as a kernel of
// its own costs as much as the product behind it.
//
// WAVES: waves of a block, which split K between them: 4, or 8 for gate|up with up to 16 rows
// (a block then has all of its share of the weights in flight at once).  (A product that adds
// into the stream itself with 16 waves a block, instead of partial products over 256 blocks, was
// tried for o and down: its 64 blocks take 6.7 us where the partial products take 4.3.)
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SILU_MUL = 2, EPI_PARTIAL = 3, EPI_SILU_MUL_IL = 4 };

// The prologue of a product of few rows (M <= 16): the rows of the 32-bit stream hs [M][K], with the
// n_delta partial products delta[s][M][K] of the branch before added in the order of s (the residual
// sum), normed as rmsnorm_regs_kernel norms them and left as bfloat16 in xs [M][K + 8].  That kernel's
// block has tn = min(256, K / 4 rounded up to whole waves) threads, thread t owns the elements
// (t + i tn) 4 .. + 3, the sum of squares runs over i, then over the lanes of a wave, then over the
// waves in order; the same here (threads beyond tn add zeros), so the bits are the same.  If
// h_out is given, this block also writes the summed rows there (one block of the grid does).
//
// Rows of up to 1024 elements (one group of four a thread), MB >= M rows: everything is asked for in
// as few trips to memory as the registers allow (the rows and the first partial products
// together, then SB partial products of all rows at a time), with addresses that are always valid
// (a row or a partial product beyond the last reads the last again and is not used), so that no
// branch stands between the loads.  The rows stay in registers between the two passes.
template <int WAVES, int MB>
__device__ __forceinline__ void norm_short_rows(const float* __restrict__ hs, const float* __restrict__ delta,
                                                int n_delta, float* __restrict__ h_out, const float* __restrict__ norm_w,
                                                float norm_eps, bf16_t* xs, int M, int K, int KP, float (*ss_red)[16],
                                                bool mine) {
    constexpr int SB = MB <= 4 ? 8 : (MB <= 8 ? 4 : 2);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = (int)threadIdx.x * 4;
    const bool have = mine && c < K;                         // (threads beyond K / 4 have nothing)
    const int cc = have ? c : 0;
    const long dstride = (long)M * K;
    float v[MB][4];
#pragma unroll
    for (int m = 0; m < MB; ++m) Vec4<float>::load(hs + (long)min(m, M - 1) * K + cc, v[m]);
    float wv[4];
    Vec4<float>::load(norm_w + cc, wv);
    for (int s0 = 0; s0 < n_delta; s0 += SB) {
        float d[SB][MB][4];
#pragma unroll
        for (int j = 0; j < SB; ++j)
#pragma unroll
            for (int m = 0; m < MB; ++m)
                Vec4<float>::load(delta + min(s0 + j, n_delta - 1) * dstride + (long)min(m, M - 1) * K + cc, d[j][m]);
#pragma unroll
        for (int j = 0; j < SB; ++j)
            if (s0 + j < n_delta) {
#pragma unroll
                for (int m = 0; m < MB; ++m)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[m][e] += d[j][m][e];
            }
    }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) ss += v[m][e] * v[m][e];
        const float t = wave_sum(have ? ss : 0.f);
        if (lane == 0) ss_red[wave][m] = t;
    }
    __syncthreads();
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        if (m < M && have) {
            float tot = 0.f;
            for (int i = 0; i < WAVES; ++i) tot += ss_red[i][m];
            const float rstd = rsqrtf(tot / (float)K + norm_eps);
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = v[m][e] * rstd * wv[e];
            Vec4<bf16_t>::store(xs + (long)m * KP + c, o);
            if (h_out) Vec4<float>::store(h_out + (long)m * K + c, v[m]);
        }
    }
}

template <int WAVES>
__device__ __forceinline__ void norm_rows_into_lds(const float* __restrict__ hs, const float* __restrict__ delta,
                                                   int n_delta, float* __restrict__ h_out, const float* __restrict__ norm_w,
                                                   float norm_eps, bf16_t* xs, int M, int K, int KP) {
    __shared__ float ss_red[WAVES][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int tn = ((K / 4 + 63) / 64) * 64;
    if (tn > 256) tn = 256;
    const int nv = (K / 4 + tn - 1) / tn;
    const bool mine = (int)threadIdx.x < tn;
    const long dstride = (long)M * K;
    if (nv == 1) {
        // (every wave of the block goes through the same barriers; the waves beyond the norm's own
        // block have nothing: they read the first elements again and add zeros)
        if (M <= 1) norm_short_rows<WAVES, 1>(hs, delta, n_delta, h_out, norm_w, norm_eps, xs, M, K, KP, ss_red, mine);
        else if (M <= 2) norm_short_rows<WAVES, 2>(hs, delta, n_delta, h_out, norm_w, norm_eps, xs, M, K, KP, ss_red, mine);
        else if (M <= 4) norm_short_rows<WAVES, 4>(hs, delta, n_delta, h_out, norm_w, norm_eps, xs, M, K, KP, ss_red, mine);
        else if (M <= 8) norm_short_rows<WAVES, 8>(hs, delta, n_delta, h_out, norm_w, norm_eps, xs, M, K, KP, ss_red, mine);
        else norm_short_rows<WAVES, 16>(hs, delta, n_delta, h_out, norm_w, norm_eps, xs, M, K, KP, ss_red, mine);
    } else {
        // longer rows (up to 8 groups of four a thread): a row at a time, everything of the row asked
        // for at once (the row and four partial products at a time, with addresses that are always
        // valid), kept in registers from the sum of squares to the store
        for (int m = 0; m < M; ++m) {
            float v[8][4];
            int col[8];
            bool have[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = ((int)threadIdx.x + i * tn) * 4;
                have[i] = mine && i < nv && c < K;
                col[i] = have[i] ? c : 0;
                Vec4<float>::load(hs + (long)m * K + col[i], v[i]);
            }
            for (int s0 = 0; s0 < n_delta; s0 += 4) {
                float d[4][8][4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        Vec4<float>::load(delta + min(s0 + j, n_delta - 1) * dstride + (long)m * K + col[i], d[j][i]);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (s0 + j < n_delta) {
#pragma unroll
                        for (int i = 0; i < 8; ++i)
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[i][e] += d[j][i][e];
                    }
            }
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (have[i]) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) ss += v[i][e] * v[i][e];
                }
            const float t = wave_sum(ss);
            if (lane == 0) ss_red[wave][m] = t;
            __syncthreads();
            float tot = 0.f;
            for (int i = 0; i < WAVES; ++i) tot += ss_red[i][m];
            const float rstd = rsqrtf(tot / (float)K + norm_eps);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (have[i]) {
                    float wv[4], o[4];
                    Vec4<float>::load(norm_w + col[i], wv);
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = v[i][e] * rstd * wv[e];
                    Vec4<bf16_t>::store(xs + (long)m * KP + col[i], o);
                    if (h_out) Vec4<float>::store(h_out + (long)m * K + col[i], v[i]);
                }
        }
    }
    __syncthreads();
}

// grid (N / (16 NT), S): block (bx, s) sums the chunks [s * cps, (s + 1) * cps) of K.  With S > 1 the
// epilogue is EPI_PARTIAL: 32-bit partial products out[s][M][N] that the consumer adds up in the
// order of s (the fused residual-add + norm kernel does), so the sum has one fixed order.
// NT: tiles of 16 rows of W a block owns.  Every wave reads the activations of its chunks itself
// (M rows against the block's 16 NT rows of W), so with more than 16 rows of activations most of
// what a block reads is activations, from the L2; two tiles a block halve that, four quarter it.
// LN: whole lines a load (up to 16 rows, one tile a block); XH: more than 8 rows of x then.
template <int MT, int NT, int EPI, typename TO, int WAVES, bool NORM, bool LN = false, bool XH = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(
    const void* __restrict__ x_in, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int cps, const float* __restrict__ norm_w, float norm_eps,
    const float* __restrict__ delta, int n_delta, float* __restrict__ h_out) {
    constexpr bool SILU = EPI == EPI_SILU_MUL || EPI == EPI_SILU_MUL_IL;
    constexpr int NW = SILU ? 2 : 1;   // weight tiles per tile of outputs
    // chunks whose loads are issued together
    constexpr int U = (MT == 1 && WAVES >= 8) ? (SILU ? 4 : 8) : ((MT == 1 && !SILU && NT == 1) ? 8 : ((MT <= 2) ? 4 : 2));
    __shared__ float red[WAVES][NT][NW][MT][64][4];
    extern __shared__ __align__(16) unsigned char dyn_lds[];       // NORM: the normed rows, bfloat16 [M][K + 8]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, r = lane & 15;
    const int n0 = blockIdx.x * 16 * NT;
    const int nchunks = K / 32;
    const int c_begin = blockIdx.y * cps;
    const int c_end = min(nchunks, c_begin + cps);
    const bf16_t* x = (const bf16_t*)x_in;
    const int KP = K + 8;                                            // padded row of the normed copy

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
        xrow[j] = (NORM ? (const bf16_t*)dyn_lds : x) + (long)(tok_ok[j] ? j * 16 + r : 0) * (NORM ? KP : K) + g * 8;
    }
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    // How the chunks of K are dealt to the waves: in pairs (wave w takes the chunks 2 w and 2 w + 1, then those
    // 2 WAVES further on), so that a wave's two loads of a row are one line of 128 bytes: the q|k|v and down
    // products of the large models go 8 % faster than with single chunks dealt round the waves, where two
    // waves fetch a line's halves at different times.  With silu.mul (eight waves, two matrices) a block whose
    // waves have one round of chunks at most (the small model's) is faster with single chunks.  A wave's chunks
    // depend on the matrix and the cut of K alone, not on the rows of x or on the form of the loop below: a
    // row's sums are added in the same order whatever else is in the batch.
    static_assert(U % 2 == 0, "chunks are dealt in pairs");
    const bool pairs = !SILU || c_end - c_begin > WAVES * U;
#define QE_CHUNK(c_, u) (pairs ? (c_) + 2 * WAVES * ((u) >> 1) + ((u) & 1) : (c_) + WAVES * (u))
#define QE_MFMA(acc_, a0_, a1_, b_)                                                                    \
    _Pragma("unroll") for (int q = 0; q < NT; ++q) {                                                   \
        acc_[q][0][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0_[u][q], b_, acc_[q][0][j], 0, 0, 0); \
        if (SILU) acc_[q][1][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1_[u][q], b_, acc_[q][1][j], 0, 0, 0); \
    }
#define QE_KEEP(acc_)                                                                                  \
    _Pragma("unroll") for (int q = 0; q < NT; ++q)                                                     \
        _Pragma("unroll") for (int a = 0; a < NW; ++a)                                                 \
            _Pragma("unroll") for (int j = 0; j < MT; ++j)                                             \
                _Pragma("unroll") for (int i = 0; i < 4; ++i) red[wave][q][a][j][lane][i] = acc_[q][a][j][i];
#define QE_NORM_PROLOGUE()                                                                             \
    norm_rows_into_lds<WAVES>((const float*)x_in, delta, n_delta, (blockIdx.x == 0 && blockIdx.y == 0) ? h_out : nullptr, \
                              norm_w, norm_eps, (bf16_t*)dyn_lds, M, K, KP);
    const int last = c_end - 1;
    // Three forms of the main part: with the norm as prologue, for a block whose waves have one round of
    // chunks at most, and for several rounds.  Each leaves its sums in shared memory itself: the
    // accumulators of two forms never meet in one register.
#define QE_ZERO(acc_)                                                                                  \
    _Pragma("unroll") for (int q = 0; q < NT; ++q)                                                     \
        _Pragma("unroll") for (int a = 0; a < NW; ++a)                                                 \
            _Pragma("unroll") for (int j = 0; j < MT; ++j) acc_[q][a][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    // (loads that stand under their own conditions: a wave with few chunks asks for no more than it has)
#define QE_LOAD_W()                                                                                    \
    _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                    \
        const int cc = QE_CHUNK(c, u);                                                                 \
        const bool ok = cc <= last;                                                                    \
        _Pragma("unroll") for (int q = 0; q < NT; ++q) {                                               \
            a0[u][q] = (ok && row_ok[q]) ? *(const bf16x8*)(wrow0[q] + cc * 32) : zero;                \
            if (SILU) a1[u][q] = (ok && row_ok[q]) ? *(const bf16x8*)(wrow1[q] + cc * 32) : zero;      \
        }                                                                                              \
    }
#define QE_ROUND()                                                                                     \
    {                                                                                                  \
        bf16x8 b[U][MT];                                                                               \
        _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                \
            const int cc = QE_CHUNK(c, u);                                                             \
            const bool ok = cc <= last;                                                                \
            _Pragma("unroll") for (int j = 0; j < MT; ++j)                                             \
                b[u][j] = (ok && tok_ok[j]) ? *(const bf16x8*)(xrow[j] + cc * 32) : zero;              \
        }                                                                                              \
        _Pragma("unroll") for (int u = 0; u < U; ++u)                                                  \
            _Pragma("unroll") for (int j = 0; j < MT; ++j) { QE_MFMA(acc, a0, a1, b[u][j]) }           \
    }
    if (NORM || NT == 4) {
        // The norm as prologue (small matrices): the first round's weights travel while the rows are normed;
        // further rounds, if any, one after the other.  Four tiles of outputs a block (the logits' matrix) run
        // this way too: a round is 16 KB of weights a wave already, and the second set of registers only cost
        // (eight rows against the 8B sizes' logits: 241 us this way, 255 with two rounds in flight).
        floatx4 acc[NT][NW][MT];
        QE_ZERO(acc)
        bf16x8 a0[U][NT], a1[U][NT];
        int c = c_begin + (pairs ? 2 : 1) * wave_s;
        if (c <= last) { QE_LOAD_W() }
        if (NORM) { QE_NORM_PROLOGUE() }
        while (c <= last) {
            QE_ROUND()
            c += WAVES * U;
            if (c <= last) { QE_LOAD_W() }
        }
        QE_KEEP(acc)
    } else if (!LN && c_end - c_begin <= WAVES * U) {
        // One round at most a wave (the small model's products).
        floatx4 acc[NT][NW][MT];
        QE_ZERO(acc)
        bf16x8 a0[U][NT], a1[U][NT];
        const int c = c_begin + (pairs ? 2 : 1) * wave_s;
        QE_LOAD_W()
        QE_ROUND()
        QE_KEEP(acc)
        asm volatile("" ::: "memory");             // (so that this way does not end like the next: see there)
    } else {
        // Several rounds: the next round's weights and rows are asked for before the current round is
        // multiplied (two sets of registers used in turn), so a wave always has a round on its way.  No load
        // stands under a condition here (the compiler would wait for every load in flight behind one): a
        // chunk beyond the wave's last reads the last chunk's place instead, and its rows of x count as
        // zeros.
        //
        // LN (one tile of rows of x, one of outputs; K in whole lines of 128 bytes): a load instruction takes whole
        // lines, 8 lanes a row and 8 rows, of the weights and of x alike, instead of the 64 bytes a row that the
        // MFMA operand layout would have 4 lanes take: the L1 then serves half as many requests, and the weights
        // stream as fast beside 8 rows of x as beside one (a matrix of 1.2 GB: 6.3 TB/s where 64-byte pieces reach
        // 5.5 with 8 rows and 4.6 with 16).  The registers go through a piece of shared memory of the wave's own to
        // come out in the operand layout (written in the lanes' order, read by row and segment; the segments of a
        // row stand swapped about by the row, so that neither side meets a bank twice).  Chunk by chunk the same
        // products in the same order as without.
        floatx4 acc[NT][NW][MT];
        QE_ZERO(acc)
        bf16x8 a0[LN ? 1 : 2][LN ? 1 : U][NT], a1[LN ? 1 : 2][LN ? 1 : U][NT], b[LN ? 1 : 2][LN ? 1 : U][MT];
        constexpr int L = U / 2, XR = XH ? 2 : 1;                     // lines a round; load instructions a line of x
        constexpr int LINE_BYTES = NW * 2048 + XR * 1024;
        typedef __attribute__((ext_vector_type(4))) unsigned int u4;
        u4 wreg[LN ? 2 : 1][LN ? L : 1][NW][2], xreg[LN ? 2 : 1][LN ? L : 1][XR];
        unsigned char* scratch = dyn_lds + wave_s * LINE_BYTES;
        const bf16_t* wl[NW][2];
        const bf16_t* xlp[XR];
        if (LN) {
            static_assert(!LN || (MT == 1 && NT == 1 && !NORM), "whole lines: one tile of rows, one of outputs");
            const int row8 = lane >> 3, pos = lane & 7;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int row = h * 8 + row8;
                const int nrow = n0 + row < N ? n0 + row : 0;
                const long wr = (EPI == EPI_SILU_MUL_IL) ? (long)(nrow >> 5) * 64 + (nrow & 31) : nrow;
                wl[0][h] = w + wr * K + (pos ^ ((row >> 1) & 7)) * 8;
                if (SILU) wl[NW - 1][h] = (EPI == EPI_SILU_MUL_IL) ? wl[0][h] + 32L * K : wl[0][h] + (long)N * K;
            }
#pragma unroll
            for (int h = 0; h < XR; ++h) {
                const int row = h * 8 + row8;
                xlp[h] = x + (long)(row < M ? row : 0) * K + (pos ^ ((row >> 1) & 7)) * 8;
            }
        }
        int c = c_begin + 2 * wave_s;                                 // (several rounds: always pairs)
#define QE_LOAD(s_, c_)                                                                                \
    if (LN) {                                                                                          \
        _Pragma("unroll") for (int i = 0; i < L; ++i) {                                                \
            const int cc = min((c_) + 2 * WAVES * i, last & ~1);                                       \
            _Pragma("unroll") for (int a = 0; a < NW; ++a)                                             \
                _Pragma("unroll") for (int h = 0; h < 2; ++h)                                          \
                    wreg[s_][i][a][h] = *(const u4*)(wl[a][h] + cc * 32);                              \
        }                                                                                              \
    } else {                                                                                           \
        _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                \
            const int cc = min(QE_CHUNK(c_, u), last);                                                 \
            _Pragma("unroll") for (int q = 0; q < NT; ++q) {                                           \
                a0[s_][u][q] = *(const bf16x8*)(wrow0[q] + cc * 32);                                   \
                if (SILU) a1[s_][u][q] = *(const bf16x8*)(wrow1[q] + cc * 32);                         \
            }                                                                                          \
        }                                                                                              \
    }
#define QE_LOAD_X(s_, c_)                                                                              \
    if (LN) {                                                                                          \
        _Pragma("unroll") for (int i = 0; i < L; ++i) {                                                \
            const int cc = min((c_) + 2 * WAVES * i, last & ~1);                                       \
            _Pragma("unroll") for (int h = 0; h < XR; ++h) xreg[s_][i][h] = *(const u4*)(xlp[h] + cc * 32); \
        }                                                                                              \
    } else {                                                                                           \
        _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                \
            const int cc = min(QE_CHUNK(c_, u), last);                                                 \
            _Pragma("unroll") for (int j = 0; j < MT; ++j) b[s_][u][j] = *(const bf16x8*)(xrow[j] + cc * 32); \
        }                                                                                              \
    }
#define QE_MULTIPLY(s_, c_)                                                                            \
    if (LN) {                                                                                          \
        _Pragma("unroll") for (int i = 0; i < L; ++i) {                                                \
            const int cc = (c_) + 2 * WAVES * i;                                                       \
            _Pragma("unroll") for (int a = 0; a < NW; ++a)                                             \
                _Pragma("unroll") for (int h = 0; h < 2; ++h)                                          \
                    *(u4*)(scratch + (a * 2 + h) * 1024 + lane * 16) = wreg[s_][i][a][h];              \
            _Pragma("unroll") for (int h = 0; h < XR; ++h)                                             \
                *(u4*)(scratch + NW * 2048 + h * 1024 + lane * 16) = xreg[s_][i][h];                   \
            const int fr = (r >> 1) & 7, xr_ = XH ? r : (r & 7), fx = (xr_ >> 1) & 7;                  \
            const unsigned char* xs = scratch + NW * 2048 + xr_ * 128;                                 \
            const bf16x8 x0 = *(const bf16x8*)(xs + ((g ^ fx) * 16));                                  \
            const bf16x8 x1 = *(const bf16x8*)(xs + (((g + 4) ^ fx) * 16));                            \
            const bf16x8 b0 = cc <= last ? x0 : zero, b1 = cc + 1 <= last ? x1 : zero;                 \
            _Pragma("unroll") for (int a = 0; a < NW; ++a) {                                           \
                const bf16x8 w0 = *(const bf16x8*)(scratch + a * 2048 + r * 128 + ((g ^ fr) * 16));    \
                acc[0][a][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, b0, acc[0][a][0], 0, 0, 0); \
            }                                                                                          \
            _Pragma("unroll") for (int a = 0; a < NW; ++a) {                                           \
                const bf16x8 w1 = *(const bf16x8*)(scratch + a * 2048 + r * 128 + (((g + 4) ^ fr) * 16)); \
                acc[0][a][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, b1, acc[0][a][0], 0, 0, 0); \
            }                                                                                          \
        }                                                                                              \
    } else {                                                                                           \
        _Pragma("unroll") for (int u = 0; u < U; ++u) {                                                \
            const bool ok = QE_CHUNK(c_, u) <= last;                                                   \
            _Pragma("unroll") for (int j = 0; j < MT; ++j) {                                           \
                const bf16x8 bb = ok ? b[s_][u][j] : zero;                                             \
                QE_MFMA(acc, a0[s_], a1[s_], bb)                                                       \
            }                                                                                          \
        }                                                                                              \
    }
        const int rounds = c <= last ? (last - c) / (WAVES * U) + 1 : 1;     // of this wave: the same in all its lanes
        QE_LOAD(0, c)
        QE_LOAD_X(0, c)
        for (int p = (rounds - 1) >> 1; p > 0; --p) {          // while three rounds or more are left: two of them
            QE_LOAD(1, c + WAVES * U)
            QE_LOAD_X(1, c + WAVES * U)
            QE_MULTIPLY(0, c)
            c += WAVES * U;
            QE_LOAD(0, c + WAVES * U)
            QE_LOAD_X(0, c + WAVES * U)
            QE_MULTIPLY(1, c)
            c += WAVES * U;
        }
        // one round or two are left.  Each way leaves its sums in shared memory itself, and the two ways do not
        // end alike (the empty statement), so that the compiler does not join them behind the branch: joined,
        // the accumulators of the two ways would meet in one register, and this compiler's copies for that have
        // overwritten operands that were still to be multiplied (seen with two tiles of rows).
        if (rounds & 1) {
            QE_MULTIPLY(0, c)
            QE_KEEP(acc)
        } else {
            QE_LOAD(1, c + WAVES * U)
            QE_LOAD_X(1, c + WAVES * U)
            QE_MULTIPLY(0, c)
            c += WAVES * U;
            QE_MULTIPLY(1, c)
            QE_KEEP(acc)
            asm volatile("" ::: "memory");
        }
#undef QE_LOAD
#undef QE_LOAD_X
#undef QE_MULTIPLY
    }
#undef QE_MFMA
#undef QE_KEEP
#undef QE_ZERO
#undef QE_LOAD_W
#undef QE_ROUND
#undef QE_NORM_PROLOGUE
#undef QE_CHUNK
    __syncthreads();
    // wave w finishes the (output tile, token tile) pairs w, w + WAVES, ...: the waves' sums in their order
    for (int qj = wave; qj < NT * MT; qj += WAVES) {
        const int q = qj / MT, j = qj % MT;
        float v[NW][4];
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float t = red[0][q][a][j][lane][i] + red[1][q][a][j][lane][i] + red[2][q][a][j][lane][i] +
                          red[3][q][a][j][lane][i];
#pragma unroll
                for (int ww = 4; ww < WAVES; ++ww) t += red[ww][q][a][j][lane][i];
                v[a][i] = t;
            }
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

// Shared memory of the normed rows: M rows of K + 8 bfloat16.
static size_t norm_lds_bytes(int M, int K) { return (size_t)M * (K + 8) * 2; }
// (a compute unit of gfx950 has 160 KB of shared memory; the kernel's own arrays take up to 17 KB of it)
#define QE_SKINNY_MAX_NORM_LDS (136 * 1024)

// true if the product can take the norm before it as its prologue
bool qe_gemm_skinny_norm_ok(int M, int N, int K) {
    return M >= 1 && M <= 16 && K % 32 == 0 && K >= 32 && K <= 8192 && norm_lds_bytes(M, K) <= QE_SKINNY_MAX_NORM_LDS;
}

template <int EPI, typename TO>
static int launch_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                         int splits, const float* norm_w, float norm_eps, const float* delta, int n_delta, float* h_out,
                         hipStream_t stream) {
    const int cps = qe_cdiv(K / 32, splits);
    const int mt = qe_cdiv(M, 16);
    constexpr bool SILU = EPI == EPI_SILU_MUL || EPI == EPI_SILU_MUL_IL;
    // two tiles of outputs a block where the activations have more than 16 rows and there are blocks
    // enough all the same (with silu.mul a tile of outputs is two tiles of W already: only up to 32 rows)
    const bool two = mt >= 2 && (!SILU || mt <= 2) && (long)qe_cdiv(N, 32) * splits >= 256;
    // whole lines of K a load (see the kernel): up to 16 rows, one tile of outputs a block, several rounds of
    // chunks a wave (blocks of fewer chunks run the form for one round, but against a large matrix), every
    // block's chunks beginning at a line
    const bool lines = !norm_w && mt == 1 && K % 64 == 0 && (splits == 1 || cps % 2 == 0);
    // ... and four where 9 to 16 rows meet a matrix of very many rows (the logits') whose K is not in whole
    // lines: the activations are then a ninth of what a block reads instead of a third (16 rows against the 8B
    // sizes' logits: 266 us against 289; with whole lines a load, one tile a block: 234)
    const bool four = !lines && !SILU && mt == 1 && M > 8 && (long)qe_cdiv(N, 64) * splits >= 2048;
    const dim3 grid(qe_cdiv(N, four ? 64 : (two ? 32 : 16)), splits);
#define QE_SKINNY_W(MT_, NT_, WAVES_, NORM_) QE_SKINNY_K(MT_, NT_, WAVES_, NORM_, false, false)
#define QE_SKINNY_K(MT_, NT_, WAVES_, NORM_, LN_, XH_)                                                 \
    do {                                                                                               \
        auto kern = gemm_skinny_kernel<MT_, NT_, EPI, TO, WAVES_, NORM_, LN_, XH_>;                    \
        const size_t dyn = NORM_ ? norm_lds_bytes(M, K)                                                \
                                 : (LN_ ? (size_t)WAVES_ * ((SILU ? 2 : 1) * 2048 + ((XH_) ? 2 : 1) * 1024) : 0); \
        if (dyn > 32 * 1024) {                                                                         \
            static bool raised = false;   /* (once per kernel: the limit of dynamic shared memory) */ \
            if (!raised) {                                                                             \
                hipError_t e_ = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                                    QE_SKINNY_MAX_NORM_LDS);                           \
                if (e_ != hipSuccess) { qe_set_error("skinny gemm: %s", hipGetErrorString(e_)); return (int)e_; } \
                raised = true;                                                                         \
            }                                                                                          \
        }                                                                                              \
        kern<<<grid, WAVES_ * 64, dyn, stream>>>(x, (const bf16_t*)w, bias, (TO*)out, M, N, K, cps, norm_w, norm_eps, \
                                                 delta, n_delta, h_out);                               \
    } while (0)
#define QE_SKINNY(MT_, NT_) QE_SKINNY_W(MT_, NT_, 4, false)
    if (norm_w) {
        QE_REQUIRE(qe_gemm_skinny_norm_ok(M, N, K) && splits == 1, "skinny gemm: the norm prologue takes up to 16 rows, K <= 8192");
        if constexpr (SILU) QE_SKINNY_W(1, 1, 8, true);
        else if constexpr (EPI == EPI_STORE) QE_SKINNY_W(1, 1, 4, true);
        else QE_REQUIRE(false, "skinny gemm: the norm prologue goes with the store and silu-mul epilogues");
    } else if (mt == 1 && SILU) {
        if constexpr (SILU) {
            if (lines && cps > 8 * 4) {
                if (M > 8) QE_SKINNY_K(1, 1, 8, false, true, true);
                else QE_SKINNY_K(1, 1, 8, false, true, false);
            } else {
                QE_SKINNY_W(1, 1, 8, false);
            }
        }
    } else if (four) {
        if constexpr (!SILU) QE_SKINNY(1, 4);
    } else if (two) {
        switch (mt) {
            case 2: QE_SKINNY(2, 2); break;
            case 3: if constexpr (!SILU) QE_SKINNY(3, 2); break;
            default: if constexpr (!SILU) QE_SKINNY(4, 2); break;
        }
    } else {
        switch (mt) {
            case 1:
                if (lines && (cps > 4 * 8 || (long)N * K >= (16L << 20))) {      // (one round too, against a large matrix)
                    if (M > 8) QE_SKINNY_K(1, 1, 4, false, true, true);
                    else QE_SKINNY_K(1, 1, 4, false, true, false);
                } else {
                    QE_SKINNY(1, 1);
                }
                break;
            case 2: QE_SKINNY(2, 1); break;
            case 3: QE_SKINNY(3, 1); break;
            default: QE_SKINNY(4, 1); break;
        }
    }
#undef QE_SKINNY
#undef QE_SKINNY_W
#undef QE_SKINNY_K
    QE_LAUNCH_CHECK();
    return 0;
}

bool qe_gemm_skinny_ok(int M, int N, int K, int dt_a, int dt_w) {
    return dt_a == QE_BF16 && dt_w == QE_BF16 && M >= 1 && M <= 64 && K % 32 == 0 && K >= 32;
}

// How many partial products a [M, N] = [M, K] . [N, K]^T product is best cut into along K so that
// the launch has some 512 blocks (1024 against a matrix of 16 M elements or more: a wave has one round of
// loads in flight, and a large matrix is read at the memory's rate only with four waves a SIMD: the o and
// down products of eight rows at the 32B sizes take 22 and 64 us in four cuts where they took 31 and 98 in
// one), each wave still summing at least two chunks.
int qe_gemm_skinny_splits(int N, int K) {
    const int blocks = qe_cdiv(N, 16);
    const int want = (long)N * K >= (16L << 20) ? 1024 : 512;
    int s = qe_cdiv(want, blocks > 0 ? blocks : 1);
    if (want == 512) s = 512 / (blocks > 0 ? blocks : 1);
    const int most = (K / 32) / 8;
    if (s > most) s = most;
    if (s > 16) s = 16;
    return s < 1 ? 1 : s;
}

// epilogue EPI_STORE: out [M, N] in dt_o.  EPI_RESIDUAL: out is the 32-bit stream [M, N], added to.
// EPI_SILU_MUL: w is [2 N, K] (gate rows, then up rows), out [M, N] in dt_o.
// EPI_SILU_MUL_IL: the same with gate and up rows interleaved in blocks of 32.
// EPI_PARTIAL: out is float [splits, M, N]; the product is the sum over the first index.
// norm_w (or null): the weight of an RMSNorm that stands before the product; x is then the 32-bit
// stream [M, K] and the rows are normed (eps norm_eps) before they are multiplied.  delta (or null):
// n_delta partial products [n_delta][M][K] of the branch before, added to the stream's rows in
// order before the norm; the summed rows are written to h_out [M][K], which is not x (the blocks
// read x while one of them writes).
int qe_gemm_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                   int dt_o, int epilogue, int splits, const float* norm_w, float norm_eps,
                   const float* delta, int n_delta, float* h_out, hipStream_t stream) {
    QE_REQUIRE(norm_w || (!delta && !h_out), "skinny gemm: partial products to add go with the norm prologue");
    QE_REQUIRE(!delta || (n_delta >= 1 && h_out && h_out != x), "skinny gemm: %d partial products, and the summed stream needs a place of its own", n_delta);
    QE_REQUIRE(M >= 1 && M <= 64 && K % 32 == 0, "skinny gemm: M=%d K=%d not taken", M, K);
    QE_REQUIRE(splits >= 1 && splits <= 64 && (epilogue == EPI_PARTIAL || splits == 1),
               "skinny gemm: %d splits with epilogue %d", splits, epilogue);
    if (epilogue == EPI_PARTIAL) {
        QE_REQUIRE(dt_o == QE_F32, "skinny gemm: partial products are 32-bit");
        return launch_skinny<EPI_PARTIAL, float>(x, w, bias, out, M, N, K, splits, norm_w, norm_eps, delta, n_delta, h_out, stream);
    }
    if (epilogue == EPI_RESIDUAL) {
        QE_REQUIRE(dt_o == QE_F32, "skinny gemm: the residual stream is 32-bit");
        return launch_skinny<EPI_RESIDUAL, float>(x, w, bias, out, M, N, K, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
    }
    if (epilogue == EPI_SILU_MUL) {
        QE_REQUIRE(!bias, "skinny gemm: silu-mul takes no bias");
        if (dt_o == QE_BF16) return launch_skinny<EPI_SILU_MUL, bf16_t>(x, w, bias, out, M, N, K, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
        return launch_skinny<EPI_SILU_MUL, float>(x, w, bias, out, M, N, K, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
    }
    if (epilogue == EPI_SILU_MUL_IL) {
        QE_REQUIRE(!bias && N % 32 == 0, "skinny gemm: interleaved silu-mul takes no bias and N in blocks of 32");
        if (dt_o == QE_BF16) return launch_skinny<EPI_SILU_MUL_IL, bf16_t>(x, w, bias, out, M, N, K, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
        return launch_skinny<EPI_SILU_MUL_IL, float>(x, w, bias, out, M, N, K, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
    }
    QE_REQUIRE(epilogue == EPI_STORE, "skinny gemm: unknown epilogue %d", epilogue);
    if (dt_o == QE_BF16) return launch_skinny<EPI_STORE, bf16_t>(x, w, bias, out, M, N, K, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
    return launch_skinny<EPI_STORE, float>(x, w, bias, out, M, N, K, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
}
