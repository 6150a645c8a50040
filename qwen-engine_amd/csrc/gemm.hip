// Entry point of all matrix products: picks a kernel for the shape and types.
#include "common.h"

int qe_gemm_generic(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                    int dt_a, int dt_w, int dt_o, hipStream_t stream);
bool qe_gemm_skinny_ok(int M, int N, int K, int dt_a, int dt_w);
int qe_gemm_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                   int dt_o, int epilogue, int splits, const float* norm_w, float norm_eps,
                   const float* delta, int n_delta, float* h_out, hipStream_t stream);
bool qe_gemm_skinny_norm_ok(int M, int N, int K);
int qe_gemm_skinny_splits(int N, int K);
bool qe_gemm_mfma_ok(int M, int N, int K, int dt_a, int dt_w);
int qe_gemm_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int dt_o,
                 int tile, bool silu, int splits, hipStream_t stream);

int qe_gemm_qkv(const void* x, const void* w, const float* bias, int M, int K, int Hq, int Hkv, int P,
                const int* positions, const int* slots, const float* q_w, const float* k_w, float eps,
                const float* table, void* q_out, void* cache, int tile, hipStream_t stream);

enum { ALGO_AUTO = 0, ALGO_GENERIC = 1, ALGO_MFMA = 2, ALGO_TILE = 1000 };   // ALGO_TILE + rows: the tiled kernel with that tile
enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SILU_MUL = 2, EPI_PARTIAL = 3, EPI_SILU_MUL_IL = 4 };

// 1 if the fused epilogues (add into the 32-bit residual stream; silu(gate) * up) can be used
extern "C" int qe_gemm_fused_supported(int M, int N, int K, int dt_a, int dt_w) {
    return qe_gemm_skinny_ok(M, N, K, dt_a, dt_w) ? 1 : 0;
}

// 1 if the product can take the RMSNorm before it as its prologue (qe_gemm's norm_w): x is then the
// 32-bit stream; few rows, bfloat16 weights (N counts the weight rows)
extern "C" int qe_gemm_norm_supported(int M, int N, int K, int dt_w) {
    return (dt_w == QE_BF16 && qe_gemm_skinny_ok(M, N, K, QE_BF16, dt_w) && qe_gemm_skinny_norm_ok(M, N, K) &&
            !((long)N * K >= (16L << 20) && M > 16)) ? 1 : 0;
}

// Rows up to which a product may take the norm before it as its prologue at all.
extern "C" int qe_gemm_norm_max_rows() { return 16; }

// 1 if a product of M rows of the stream against w [N, K] should take the residual sum of n_delta partial
// products and the norm as its prologue rather than leave them to the norm's own kernel.  Beside what
// qe_gemm_norm_supported asks: a matrix of at most 8 M elements (a larger product is bound by the stream of
// its weights, which stands still while the prologue runs: at the 8B sizes a decode step of one request took
// 7 % longer with the prologue), and at most 192 KB of rows and partial products (every block reads all of
// them for all rows; beyond that the norm's kernel, which reads them once, is quicker).
extern "C" int qe_gemm_norm_preferred(int M, int N, int K, int dt_w, int n_delta) {
    return (qe_gemm_norm_supported(M, N, K, dt_w) && (long)N * K <= (8L << 20) &&
            (long)M * K * 4 * (1 + n_delta) <= 192L * 1024) ? 1 : 0;
}

// 1 if epilogue 4 (silu-mul over interleaved gate|up rows) can be used: N counts the outputs
extern "C" int qe_gemm_silu_supported(int M, int N, int K, int dt_a, int dt_w) {
    return (N % 32 == 0 && (qe_gemm_skinny_ok(M, N, K, dt_a, dt_w) || qe_gemm_mfma_ok(M, 2 * N, K, dt_a, dt_w))) ? 1 : 0;
}

// More than 16 rows against a large matrix: the kernel for few rows, in which every wave reads the
// activations of its chunks itself, reads several times more activations than weights there and
// falls well behind the memory; the tiled kernel shares them through shared memory and streams
// the weights at the memory's rate.  (Against a small matrix the tiled kernel has too few tiles.)
static bool tiled_for_few_rows(int M, int N, int K, int dt_a, int dt_w) {
    return M > 16 && (long)N * K >= (16L << 20) && qe_gemm_mfma_ok(M, N, K, dt_a, dt_w);
}

// 1 if a product of these sizes is quickest as partial products (epilogue 3) from the tiled kernel
extern "C" int qe_gemm_partial_preferred(int M, int N, int K, int dt_a, int dt_w) {
    return (M <= 64 && tiled_for_few_rows(M, N, K, dt_a, dt_w)) ? 1 : 0;
}

// number of partial products that epilogue 3 should be asked for
extern "C" int qe_gemm_partial_splits(int M, int N, int K) {
    if (tiled_for_few_rows(M, N, K, QE_BF16, QE_BF16)) {
        // (tiles of 64 rows: M <= 64 here)  As many cuts as still give every compute unit at most one block:
        // with a few blocks more than units, the units that get two take as long as if all had two
        // (10240 x 5120 against 64 rows: 240 blocks in 3 cuts 25.8 us, 320 in 4 cuts 31.4; 5120 x 25600: 240
        // blocks in 6 cuts 55.9 us, 280 in 7 cuts 70.4).
        const int tiles = qe_cdiv(N, 128);
        int s = 256 / tiles;
        const int most = K / 256;
        if (s > most) s = most;
        if (s > 16) s = 16;
        return s < 1 ? 1 : s;
    }
    return qe_gemm_skinny_splits(N, K);
}

// How the product of a layer's branch (its output goes to the norm that adds it to the stream)
// should be asked for: 0 = as a plain product; S >= 1 = as S partial products (epilogue 3), which
// that norm adds up.  Few rows: always, the cut fills the chip.  Many rows against a narrow matrix
// with a long K (at most one 64 x 128 tile a compute unit: a block then spends its time on the
// trips of its K loop): two to four cuts give every unit blocks to overlap (2048 x 1024 x 3072
// with the norm behind it: 27.7 us in two cuts against 30.8; 512 rows: 15.7 against 24.7).
extern "C" int qe_gemm_branch_splits(int M, int N, int K, int dt_a, int dt_w) {
    if (qe_gemm_skinny_ok(M, N, K, dt_a, dt_w) || (M <= 64 && tiled_for_few_rows(M, N, K, dt_a, dt_w))) {
        const int s = qe_gemm_partial_splits(M, N, K);
        // (rows few enough for the next product to add the parts up in its prologue: every block of that
        // product reads all of them for all rows, so at most four)
        return (M <= qe_gemm_norm_max_rows() && s > 4) ? 4 : s;
    }
    if (!qe_gemm_mfma_ok(M, N, K, dt_a, dt_w) || K < 2048) return 0;
    const long tiles = (long)qe_cdiv(M, 64) * qe_cdiv(N, 128);
    if (tiles > 256) return 0;
    int s = (int)qe_cdiv(512, tiles);
    s = s < 2 ? 2 : (s > 4 ? 4 : s);
    while (s > 1 && (long)(s - 1) * (qe_cdiv(qe_cdiv(K, s), 64) * 64) >= K) --s;   // every cut has some of K
    return s > 1 ? s : 0;
}

// out[M, N] = x[M, K] . w[N, K]^T (+ bias).  epilogue 0: store in dt_o.  1: add into out, the
// 32-bit stream.  2: w is [2 N, K], gate rows then up rows; out = silu(x.gate^T) * (x.up^T).
// 3: out is float [splits, M, N], partial products along K to be summed over the first index.
// 4: as 2 with the gate and up rows of w interleaved in blocks of 32 (gate 0..31, up 0..31, ...);
//    taken by the kernel for few rows and by the tiled one.
// norm_w (or null): the weight of an RMSNorm (eps norm_eps) that stands before the product: x is then the
// 32-bit stream [M, K]; needs qe_gemm_norm_supported and epilogue 0, 2 or 4.  With it, delta (or null):
// n_delta float tensors [M, K] one after the other that are added to the stream's rows, in order, before
// the norm (the partial products of the branch before); the sums are written to h_out [M, K] (not x).
// algo: 0 = choose, 1 = the generic 32-bit kernel, 2 = an MFMA kernel (the one for few rows up to
// 64 rows, except against a very wide matrix from 17 rows on; else the tiled one) or an error if
// neither takes the operands.
extern "C" int qe_gemm(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                       int dt_a, int dt_w, int dt_o, int algo, int epilogue, int splits,
                       const float* norm_w, float norm_eps, const float* delta, int n_delta, float* h_out,
                       hipStream_t stream) {
    QE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    if (M == 0) return 0;
    QE_REQUIRE(norm_w || (!delta && !h_out), "gemm: partial products to add go with the norm prologue");
    if (norm_w) {
        // x is the 32-bit stream; the kernel for few rows norms it itself
        const int n_rows = (epilogue == EPI_SILU_MUL || epilogue == EPI_SILU_MUL_IL) ? 2 * N : N;
        QE_REQUIRE(dt_a == QE_F32 && qe_gemm_norm_supported(M, n_rows, K, dt_w),
                   "gemm: M=%d N=%d K=%d is not taken with the norm as prologue", M, N, K);
        QE_REQUIRE(epilogue == EPI_STORE || epilogue == EPI_SILU_MUL || epilogue == EPI_SILU_MUL_IL,
                   "gemm: the norm prologue goes with the store and silu-mul epilogues");
        return qe_gemm_skinny(x, w, bias, out, M, N, K, dt_o, epilogue, 1, norm_w, norm_eps, delta, n_delta, h_out, stream);
    }
    const bool skinny = qe_gemm_skinny_ok(M, N, K, dt_a, dt_w);
    const bool tiled = qe_gemm_mfma_ok(M, N, K, dt_a, dt_w);
    if (epilogue == EPI_SILU_MUL_IL && (!skinny || tiled_for_few_rows(M, 2 * N, K, dt_a, dt_w))) {
        QE_REQUIRE(N % 32 == 0 && qe_gemm_mfma_ok(M, 2 * N, K, dt_a, dt_w),
                   "gemm: M=%d N=%d K=%d is not taken by a silu-mul kernel", M, N, K);
        return qe_gemm_mfma(x, w, bias, out, M, 2 * N, K, dt_o, algo > ALGO_TILE ? algo - ALGO_TILE : 0, true, 1, stream);
    }
    if (epilogue == EPI_PARTIAL && (tiled_for_few_rows(M, N, K, dt_a, dt_w) || (!skinny && tiled))) {
        QE_REQUIRE(dt_o == QE_F32, "gemm: partial products are 32-bit");
        return qe_gemm_mfma(x, w, bias, out, M, N, K, dt_o, algo > ALGO_TILE ? algo - ALGO_TILE : 0, false, splits, stream);
    }
    if (epilogue != EPI_STORE) {
        QE_REQUIRE(skinny, "gemm: M=%d N=%d K=%d with these element types is not taken by the kernel for few rows", M, N, K);
        return qe_gemm_skinny(x, w, bias, out, M, N, K, dt_o, epilogue, splits, nullptr, 0.f, nullptr, 0, nullptr, stream);
    }
    QE_REQUIRE(algo == ALGO_AUTO || algo == ALGO_GENERIC || algo == ALGO_MFMA || algo > ALGO_TILE, "gemm: unknown algo %d", algo);
    if (algo > ALGO_TILE) {
        QE_REQUIRE(tiled, "gemm: M=%d N=%d K=%d is not taken by the tiled MFMA kernel", M, N, K);
        return qe_gemm_mfma(x, w, bias, out, M, N, K, dt_o, algo - ALGO_TILE, false, 1, stream);
    }
    if (algo != ALGO_GENERIC) {
        if (skinny && !tiled_for_few_rows(M, N, K, dt_a, dt_w))
            return qe_gemm_skinny(x, w, bias, out, M, N, K, dt_o, EPI_STORE, 1, nullptr, 0.f, nullptr, 0, nullptr, stream);
        if (tiled) return qe_gemm_mfma(x, w, bias, out, M, N, K, dt_o, 0, false, 1, stream);
        QE_REQUIRE(algo == ALGO_AUTO, "gemm: M=%d N=%d K=%d with these element types is not taken by an MFMA kernel", M, N, K);
    }
    return qe_gemm_generic(x, w, bias, out, M, N, K, dt_a, dt_w, dt_o, stream);
}

// 1 if qe_gemm_qkv_run takes these sizes: bfloat16 operands, heads of 128, more rows than the
// kernel for few rows is made for (decode has the attention kernel that prepares its own inputs).
extern "C" int qe_gemm_qkv_supported(int M, int K, int Hq, int Hkv, int D, int P, int dt_a, int dt_w) {
    return (D == 128 && M > 64 && P >= 16 && (P & (P - 1)) == 0 &&
            qe_gemm_mfma_ok(M, (Hq + 2 * Hkv) * D, K, dt_a, dt_w)) ? 1 : 0;
}

// The q|k|v product with per-head q/k norm, rotation and the cache write in its epilogue: q_out
// [M, Hq, 128] bfloat16; k and v go to cache [pages, 2, Hkv, P, 128] at slots[m].  tile: 0 or the
// tile to use (64, 128, 256; 512 for 256 x 256).
extern "C" int qe_gemm_qkv_run(const void* x, const void* w, const float* bias, int M, int K, int Hq, int Hkv, int P,
                               const int* positions, const int* slots, const float* q_w, const float* k_w, float eps,
                               const float* table, void* q_out, void* cache, int tile, hipStream_t stream) {
    if (M == 0) return 0;
    return qe_gemm_qkv(x, w, bias, M, K, Hq, Hkv, P, positions, slots, q_w, k_w, eps, table, q_out, cache, tile, stream);
}
