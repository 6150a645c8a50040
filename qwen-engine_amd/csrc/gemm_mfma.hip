// Matrix product for many rows of activations (prefill): out[M, N] = x[M, K] . W[N, K]^T (+ bias),
// bfloat16 in, 32-bit accumulation with v_mfma_f32_32x32x16_bf16, output bfloat16 or float32.
//
// A block of NW waves (NW / 2 down, 2 across) computes a BM x BN tile of the output; each wave its
// part as MFMA tiles of 32 x 32.  K is walked in steps of BK through shared memory with two
// buffers.  Both operands are K-contiguous in memory, so they are staged alike: a row of BK
// bfloat16 is padded by 16 bytes, which makes the 16-byte fragment reads of the 32 rows of an
// MFMA operand fall into distinct banks.
//
// What the time of such a block goes to, as measured on this chip (cycle counters in a copy of
// the kernel, hardware counters): not to the MFMA units alone.  A compute unit takes 64 bytes a
// cycle from its L1, so a 128 x 128 x 64 step (32 KB) costs as many cycles to load as its MFMAs
// take; loads have to be in flight two steps ahead to arrive in time; and the result has to be
// stored as whole rows.  128 x 128 tiles (four waves, two blocks a compute unit) are the default,
// 64 x 128 where there would be too few blocks otherwise, 256 x 128 (eight waves) where even
// those give every compute unit two blocks, 256 x 256 (four waves, a wave's part 128 x 128) where
// even that shape gives every compute unit two blocks in turn: it reads half the bytes per MFMA
// from the L1 and from shared memory.
//
// Rows of x beyond M and rows of W beyond N are read as zero and never stored; K must be a
// multiple of 8 (16-byte loads), a tail shorter than BK is filled with zeros.
// The blocks of one XCD (every eighth block) take a compact part of the tiles, see the kernel.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) unsigned int uint4_t;
union Piece16 {   // 16 bytes, addressable by element
    uint4_t q;
    unsigned short e[8];
};

// SILU: W holds gate and up rows interleaved in blocks of 32 (gate 0..31, up 0..31, gate 32..63,
// ...), N counts all of them, and the result is silu(gate) * up, N / 2 wide: the two MFMA tiles a
// lane holds side by side are the gate and the up of the same outputs.
// What the q|k|v product of an attention layer does with its result instead of storing it (QKV):
// per-head RMSNorm of q and k (weights or null), half-split rotation from the table's row of the
// token's position (or null), then q to q_out [M, Hq, 128], k and v into the cache at the token's
// slot (negative: nowhere), exactly as the kernels of qk_rope_store.hip do on a stored product, in
// the same arithmetic: the product is rounded to bfloat16 first.  Heads are 128 wide, so that a
// tile's 128 columns are one head.
struct QkvTail {
    const int* positions;
    const int* slots;
    const float* q_w;
    const float* k_w;
    const float* table;
    bf16_t* q_out;
    bf16_t* cache;
    float eps;
    int Hq, Hkv, P;
    int lp;   // log2 P: the page size is a power of two, and a division by a number known only at run time costs dozens of instructions an item
};

// BIG (256 x 256 by four waves, one wave a SIMD, a wave's part 128 x 128): the accumulators fill the
// 256 AGPRs, so the staging registers are VGPRs.  Per MFMA this shape reads half the bytes from
// the L1 and from shared memory that 128 x 128 by four waves reads.
template <typename TO, int BM, int BN, int BK, int NW, int MINB, bool SILU, bool QKV = false>
__global__ __launch_bounds__(64 * NW, MINB) void gemm_mfma_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int tiles_m, int tiles_n, int k_per_split, int xcd_m, int xcd_n,
    int rotate, QkvTail tail) {
    constexpr int ROWB = BK * 2 + 16;       // bytes of a staged row
    constexpr int PPR = BK / 8;             // 16-byte pieces per row
    constexpr int RPI = 64 * NW / PPR;      // rows the block stages with one piece per thread
    constexpr int WM = BM / (NW / 2), WN = BN / 2;   // a wave's part: NW / 2 waves down, 2 across
    constexpr int MI = WM / 32, NJ = WN / 32;
    constexpr int LDA = BM / RPI, LD = (BM + BN) / RPI;   // pieces a thread stages per step: LDA of x, then of W
    constexpr bool BIG = BM == 256 && BN == 256 && NW == 4;
    static_assert((LD == 16 || LD == 12 || LD == 8 || LD == 6) && (LD == 16) == BIG && BM % RPI == 0 && BN % RPI == 0,
                  "tile rows must be a multiple of the rows staged at once");
    constexpr int BUF = (BM + BN) * ROWB;   // bytes of one buffer: the x rows, then the W rows
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Consecutive blocks go to the eight XCDs in turn, and each XCD has an L2 of its own: the blocks
    // of one XCD take a compact part of the tiles, xcd_m parts down by xcd_n across (the host picks
    // the cut that makes the XCDs read the fewest rows of x and W altogether; 0: no cut fits), so
    // that they share what they read through that L2.
    int tile_m, tile_n;
    if (xcd_m > 0) {
        const int xcd = blockIdx.x % 8, local = blockIdx.x / 8;
        const int per_m = tiles_m / xcd_m, per_n = tiles_n / xcd_n;
        // Inside the part the tiles go in bands of up to 8 tile rows, across the band column by
        // column: the 32 or 64 blocks that an XCD runs at a time are then a patch of 8 by 4 or 8
        // tiles, which reads 12 or 16 tiles' worth of rows where a column of 32 reads 33 (what
        // the XCDs fetch through the fabric is what bounds a large product).
        const int gm = per_m % 8 == 0 ? 8 : (per_m % 4 == 0 ? 4 : (per_m % 2 == 0 ? 2 : 1));
        const int band = local / (gm * per_n), within = local % (gm * per_n);
        tile_m = (xcd / xcd_n) * per_m + band * gm + within % gm;
        tile_n = (xcd % xcd_n) * per_n + within / gm;
    } else {
        tile_m = blockIdx.x % tiles_m;
        tile_n = blockIdx.x / tiles_m;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
    // (QKV: thread i fetches the position and the slot of the tile's row i now, for the end)
    int my_pos = 0, my_slot = -1;
    if constexpr (QKV) {
        static_assert(!QKV || BM <= 64 * NW, "a thread for every row of the tile");
        if (tid < BM && m0 + tid < M) {
            if (tail.table) my_pos = tail.positions[m0 + tid];
            if (tail.slots) my_slot = tail.slots[m0 + tid];
        }
    }

    // blockIdx.y cuts K: this block sums the k values [k0, k0 + klen) and writes the partial product
    // number blockIdx.y (out is then [splits][M][N]); without a cut k_per_split = K
    const int k0 = blockIdx.y * k_per_split;
    const int klen = K - k0 < k_per_split ? K - k0 : k_per_split;
    const int nk = (klen + BK - 1) / BK;
    // rotate: the block walks its k steps from another start than its neighbours (and wraps round).  Few rows
    // of x against a large matrix: the blocks stream their rows of W in step, and with a row stride that is a
    // power of two all their loads of a moment have the same address bits below the stride, which land on the
    // same few memory channels (the logits' matrix of 151936 x 4096 against 64 rows: 4.4 TB/s, and 5.1 with a
    // row of 4160; where the stride is no such power, walking in step is the quicker: the blocks then share
    // their rows of x through the caches).  The order of a tile's sum is then a function of its place, not of
    // the batch.
    const int rot = rotate ? (tile_n * 5 + (int)blockIdx.y * 3) % nk : 0;
#define QE_KK(kt_) ((kt_) < nk ? ((kt_) + rot < nk ? (kt_) + rot : (kt_) + rot - nk) : (kt_))
    // Two sets of staging registers in turn: a step's loads are issued two steps ahead and go to
    // shared memory one step ahead, so a load has a whole step of MFMAs to arrive.
    uint4_t stage[2][LD];

    // Piece i of a thread is row (tid / PPR) of the i-th group of RPI rows, 16 bytes at k = 8 (tid % PPR).
    // The loads are buffer loads: one descriptor for the tile's rows of x and one for its rows of W,
    // each ending with the last row that exists, so that a row beyond the matrix is "out of range"
    // and reads as zeros by itself.  The thread's byte offset never changes and the step's k offset
    // is a scalar.  A thread whose piece lies beyond K (in a last step shorter than BK) picks an
    // offset that is out of range.
    //
    // The loads and the waits for them are written as instructions: the compiler's own placing of
    // waits joins what it knows at the loop's top and so waits for the youngest loads as well,
    // which would undo the two steps of distance.  A set's registers pass through the wait
    // statement as operands, so nothing that uses them can move ahead of it.
    const int lrow = tid / PPR, pc = tid % PPR;
    const int a_rows = M - m0 < BM ? M - m0 : BM, b_rows = N - n0 < BN ? N - n0 : BN;
    const unsigned long a_addr = (unsigned long)(x + (long)m0 * K + k0), b_addr = (unsigned long)(w + (long)n0 * K + k0);
    uint4_t rsrc_a, rsrc_b;   // base, base high 16 bits (stride 0), bytes, format: 32-bit raw buffer
    rsrc_a[0] = (unsigned)a_addr; rsrc_a[1] = (unsigned)(a_addr >> 32) & 0xffffu;
    rsrc_a[2] = (unsigned)(((a_rows - 1) * K + klen) * 2); rsrc_a[3] = 0x00020000u;   // up to the last row's last k of this cut
    rsrc_b[0] = (unsigned)b_addr; rsrc_b[1] = (unsigned)(b_addr >> 32) & 0xffffu;
    rsrc_b[2] = (unsigned)(((b_rows - 1) * K + klen) * 2); rsrc_b[3] = 0x00020000u;
#pragma unroll
    for (int c = 0; c < 4; ++c) {   // the same in every lane: into scalar registers
        rsrc_a[c] = __builtin_amdgcn_readfirstlane(rsrc_a[c]);
        rsrc_b[c] = __builtin_amdgcn_readfirstlane(rsrc_b[c]);
    }
    int voff[LD];
#pragma unroll
    for (int i = 0; i < LD; ++i)
        voff[i] = ((i < LDA ? RPI * i : RPI * (i - LDA)) + lrow) * K * 2 + pc * 16;
    const int dst = lrow * ROWB + pc * 16;                 // where piece 0 goes in a buffer; piece i: + i RPI ROWB
#define LOAD_GLOBAL(set_, kt_)                                                           \
    {                                                                                    \
        const int kk = QE_KK(kt_);                                                       \
        const bool k_ok = kk * BK + pc * 8 < klen;                                       \
        const int soff = kk * BK * 2;                                                    \
        _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                 \
            const int vo = k_ok ? voff[i] : 0x7fffffff;                                  \
            if constexpr (BIG) {                                                         \
                if (i < LDA)                                                             \
                    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"              \
                                 : "=&v"(stage[set_][i]) : "v"(vo), "s"(rsrc_a), "s"(soff) : "memory"); \
                else                                                                     \
                    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"              \
                                 : "=&v"(stage[set_][i]) : "v"(vo), "s"(rsrc_b), "s"(soff) : "memory"); \
            } else if (i < LDA)                                                          \
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                  \
                             : "=&a"(stage[set_][i]) : "v"(vo), "s"(rsrc_a), "s"(soff) : "memory"); \
            else                                                                         \
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                  \
                             : "=&a"(stage[set_][i]) : "v"(vo), "s"(rsrc_b), "s"(soff) : "memory"); \
        }                                                                                \
    }
    // waits until at most `younger_` loads are in flight; the set's registers are valid afterwards
#define WAIT_LOADS(set_, younger_)                                                       \
    if constexpr (LD == 16)                                                              \
        asm volatile("s_waitcnt vmcnt(%16)"                                              \
                     : "+v"(stage[set_][0]), "+v"(stage[set_][1]), "+v"(stage[set_][2]), "+v"(stage[set_][3]), \
                       "+v"(stage[set_][4]), "+v"(stage[set_][5]), "+v"(stage[set_][6 % LD]), "+v"(stage[set_][7 % LD]), \
                       "+v"(stage[set_][8 % LD]), "+v"(stage[set_][9 % LD]), "+v"(stage[set_][10 % LD]),       \
                       "+v"(stage[set_][11 % LD]), "+v"(stage[set_][12 % LD]), "+v"(stage[set_][13 % LD]),     \
                       "+v"(stage[set_][14 % LD]), "+v"(stage[set_][15 % LD])                                  \
                     : "n"(younger_) : "memory");                                        \
    else if constexpr (LD == 12)                                                         \
        asm volatile("s_waitcnt vmcnt(%12)"                                              \
                     : "+a"(stage[set_][0]), "+a"(stage[set_][1]), "+a"(stage[set_][2]), "+a"(stage[set_][3]), \
                       "+a"(stage[set_][4]), "+a"(stage[set_][5]), "+a"(stage[set_][6]), "+a"(stage[set_][7]), \
                       "+a"(stage[set_][8 % LD]), "+a"(stage[set_][9 % LD]), "+a"(stage[set_][10 % LD]),       \
                       "+a"(stage[set_][11 % LD])                                        \
                     : "n"(younger_) : "memory");                                        \
    else if constexpr (LD == 8)                                                          \
        asm volatile("s_waitcnt vmcnt(%8)"                                               \
                     : "+a"(stage[set_][0]), "+a"(stage[set_][1]), "+a"(stage[set_][2]), "+a"(stage[set_][3]), \
                       "+a"(stage[set_][4]), "+a"(stage[set_][5]), "+a"(stage[set_][6 % LD]), "+a"(stage[set_][7 % LD]) \
                     : "n"(younger_) : "memory");                                        \
    else                                                                                 \
        asm volatile("s_waitcnt vmcnt(%6)"                                               \
                     : "+a"(stage[set_][0]), "+a"(stage[set_][1]), "+a"(stage[set_][2]), "+a"(stage[set_][3]), \
                       "+a"(stage[set_][4]), "+a"(stage[set_][5])                        \
                     : "n"(younger_) : "memory");
#define STORE_SHARED(buf_)                                                               \
    _Pragma("unroll") for (int i = 0; i < LD; ++i)                                       \
        *(uint4_t*)(smem + (buf_) * BUF + dst + i * RPI * ROWB) = stage[buf_][i];

    floatx16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int fr = lane & 31;          // row of the fragment this lane holds
    const int fk = (lane >> 5) * 16;   // byte offset of its 8 k values within a 16-wide k step
    const unsigned char* a_frag = smem + (wm + fr) * ROWB + fk;
    const unsigned char* b_frag = smem + (BM + wn + fr) * ROWB + fk;
    // One step on buffer buf_ (a constant, so every shared-memory address is base + immediate).
    // A wave issues in order, so whatever is not an MFMA stands between the MFMAs: the fragments of
    // k step ks + 1 are read before the MFMAs of ks; the loads of the step after the next go with
    // the MFMAs of the first k steps, the stores to shared memory of the next step's tile, loaded
    // a step ago, with those of the last.  Tiles of 128 rows or more spread the loads over all k
    // steps but the last and the stores over all but the first (the compute unit's L1 takes 64
    // bytes a cycle: the 64 KB a step of a 256 x 256 tile are half of the step's time, and as
    // much for the LDS; issued in a row they hold up the MFMAs behind them, which cost that
    // shape a third of the step).  The 64-row tile, whose steps are short, keeps the loads in
    // the first k step and the stores in the last: a load then has the longest time to arrive
    // (spread, its loads from HBM came late: 27 us against 24 for the o and down products of the
    // small model, though it was the faster on operands that lie in the L2).
    // (Passing the barrier before the last MFMAs and reading the next step's first fragments
    // under them was tried: 3 % faster with one wave a SIMD, 10 % slower with two.)
#define READ_FRAGS(buf_, ks_, a_, b_)                                                    \
    _Pragma("unroll") for (int i = 0; i < MI; ++i)                                       \
        a_[i] = *(const bf16x8*)(a_frag + (buf_) * BUF + i * 32 * ROWB + (ks_) * 32);    \
    _Pragma("unroll") for (int j = 0; j < NJ; ++j)                                       \
        b_[j] = *(const bf16x8*)(b_frag + (buf_) * BUF + j * 32 * ROWB + (ks_) * 32);
#define LOAD_PIECE(set_, kt_, i_)                                                        \
    {                                                                                    \
        const int kk = QE_KK(kt_);                                                       \
        const int vo = kk * BK + pc * 8 < klen ? voff[i_] : 0x7fffffff;                  \
        const int soff = kk * BK * 2;                                                    \
        if constexpr (BIG) {                                                             \
            if ((i_) < LDA)                                                              \
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                  \
                             : "=&v"(stage[set_][i_]) : "v"(vo), "s"(rsrc_a), "s"(soff) : "memory"); \
            else                                                                         \
                asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                  \
                             : "=&v"(stage[set_][i_]) : "v"(vo), "s"(rsrc_b), "s"(soff) : "memory"); \
        } else if ((i_) < LDA)                                                           \
            asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                      \
                         : "=&a"(stage[set_][i_]) : "v"(vo), "s"(rsrc_a), "s"(soff) : "memory"); \
        else                                                                             \
            asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                      \
                         : "=&a"(stage[set_][i_]) : "v"(vo), "s"(rsrc_b), "s"(soff) : "memory"); \
    }
    constexpr int NS = BK / 16, PER = MI * NJ;            // k steps; MFMAs of one
    constexpr bool SPREAD = BM >= 128;
    constexpr int LE = SPREAD ? NS - 1 : 1, SB = SPREAD ? 1 : NS - 1;   // loads go with the k steps [0, LE), stores with [SB, NS)
    constexpr int LSLOTS = LE * PER, SSLOTS = (NS - SB) * PER;    // places (MFMAs) for a load, for a store
    constexpr int EARLY = SB * PER * LD / LSLOTS < LD ? SB * PER * LD / LSLOTS : LD;   // this step's loads issued before k step SB
    static_assert(NS >= 2, "a step has two k steps or more");
    // the pieces that go with place s of n: [s LD / n, (s + 1) LD / n)
#define K_STEP(buf_, kt_)                                                                \
    {                                                                                    \
        bf16x8 fa[2][MI], fb[2][NJ];                                                     \
        READ_FRAGS(buf_, 0, fa[0], fb[0])                                                \
        _Pragma("unroll") for (int ks = 0; ks < NS; ++ks) {                              \
            if (ks + 1 < NS) { READ_FRAGS(buf_, ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1]) } \
            /* the other set, loaded a step ago; this step's own loads, issued so far, may stay in flight */ \
            if (ks == SB) { WAIT_LOADS((buf_) ^ 1, EARLY) }                              \
            __builtin_amdgcn_sched_barrier(0);                                           \
            _Pragma("unroll") for (int i = 0; i < MI; ++i)                               \
                _Pragma("unroll") for (int j = 0; j < NJ; ++j) {                         \
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ks & 1][j], fa[ks & 1][i], acc[i][j], 0, 0, 0); \
                    _Pragma("unroll") for (int p = 0; p < LD; ++p) {                     \
                        const int sl = ks * PER + i * NJ + j, ss = sl - SB * PER;   /* place of a load, of a store */ \
                        if (ks < LE && p >= sl * LD / LSLOTS && p < (sl + 1) * LD / LSLOTS) \
                            LOAD_PIECE(buf_, (kt_) + 2, p)   /* this set went to shared memory a step ago */ \
                        /* the other buffer: its readers finished before the last barrier (after the  \
                           last step this stores a step that does not exist, which nobody reads) */ \
                        if (ks >= SB && p >= ss * LD / SSLOTS && p < (ss + 1) * LD / SSLOTS) \
                            *(uint4_t*)(smem + ((buf_) ^ 1) * BUF + dst + p * RPI * ROWB) = stage[(buf_) ^ 1][p]; \
                    }                                                                    \
                    __builtin_amdgcn_sched_barrier(0);                                   \
                }                                                                        \
        }                                                                                \
        __syncthreads();                                                                 \
    }

    // step kt uses buffer and register set kt % 2
    LOAD_GLOBAL(0, 0)
    LOAD_GLOBAL(1, 1)
    WAIT_LOADS(0, LD)
    STORE_SHARED(0)
    __syncthreads();
    // (two steps in a body without branches, and an odd last step after the loop)
    int kt = 0;
    for (; kt + 1 < nk; kt += 2) {
        K_STEP(0, kt)
        K_STEP(1, kt + 1)
    }
    if (kt < nk) K_STEP(0, kt)
    // The loads past the end are still in flight and the compiler does not know of them: their
    // registers pass through a last wait, so that they stay reserved until the loads have landed
    // (a register whose value nobody uses would be handed out again at once).
    WAIT_LOADS(0, 0)
    WAIT_LOADS(1, 0)
#undef K_STEP
#undef QE_KK
#undef LOAD_PIECE
#undef READ_FRAGS
#undef LOAD_GLOBAL
#undef WAIT_LOADS
#undef STORE_SHARED

    // The MFMA is given the W rows as its first operand and the x rows as its second, so its
    // result is the tile transposed: a lane holds, for the token row m = lane % 32, the outputs
    // n = 8 b + 4 (lane / 32) + r (e = 4 b + r), four consecutive n at a time.  Stored from there,
    // one instruction would touch 32 rows with 16 bytes each.  So each wave turns its part round
    // in shared memory, a strip of 32 rows at a time (the staging buffers are free: every wave has
    // passed the loop's last barrier): it writes the strip as rows and reads it back 16 bytes a
    // lane, so that a store instruction covers whole rows of the strip.
    if constexpr (QKV) {
        // The whole tile goes to shared memory as bfloat16 rows (the staging buffers are free), then
        // 16 lanes take a row of a head each, as in qk_rope_store_vec_kernel: lane j has the features
        // 4 j .. 4 j + 3 and 64 + 4 j .. 64 + 4 j + 3, the two halves that rotate together.
        constexpr int TROW = BN * 2 + 16;                  // bytes of a row of the tile
        static_assert(BM * TROW <= 2 * BUF && BN % 128 == 0, "the tile must fit the staging buffers, in whole heads");
        // positions and slots of the tile's rows, once, into shared memory behind the tile
        int* pos_sh = (int*)(smem + BM * TROW);
        int* slot_sh = pos_sh + BM;
        static_assert(BM * TROW + 2 * BM * 4 <= 2 * BUF, "the rows' positions and slots must fit too");
        if (tid < BM) { pos_sh[tid] = my_pos; slot_sh[tid] = my_slot; }
        __syncthreads();
        const int D = 128, half = 64;
        const int j16 = tid % 16;
        const long page_stride = 2L * tail.Hkv * tail.P * D;
        constexpr int GROUPS = 64 * NW / 16, ITEMS = BM * (BN / 128);
        constexpr int NIT = (ITEMS + GROUPS - 1) / GROUPS;         // items a group of 16 lanes takes, one after the other
        constexpr int CHUNK = NIT < 8 ? NIT : 8;
        // The only loads from memory in the items' loop are the table's rows, and an item is short
        // beside a trip to memory: the rows of eight items are asked for at once, the first eight
        // before the tile is written to shared memory.
        float c[CHUNK][4], sn[CHUNK][4];
#define LOAD_TABLE_ROWS(it0_)                                                            \
        _Pragma("unroll") for (int k = 0; k < CHUNK; ++k) {                              \
            const int idx = tid / 16 + ((it0_) + k) * GROUPS;                            \
            _Pragma("unroll") for (int e = 0; e < 4; ++e) { c[k][e] = 1.f; sn[k][e] = 0.f; } \
            if (tail.table && idx < ITEMS && n0 / 128 + idx / BM < tail.Hq + tail.Hkv) {  \
                const float* cs = tail.table + (long)pos_sh[idx % BM] * D;               \
                Vec4<float>::load(cs + 4 * j16, c[k]);                                   \
                Vec4<float>::load(cs + half + 4 * j16, sn[k]);                           \
            }                                                                            \
        }
        LOAD_TABLE_ROWS(0)
        float wq_a[4], wq_b[4], wk_a[4], wk_b[4];
        if (tail.q_w) {
            Vec4<float>::load(tail.q_w + 4 * j16, wq_a);
            Vec4<float>::load(tail.q_w + half + 4 * j16, wq_b);
            Vec4<float>::load(tail.k_w + 4 * j16, wk_a);
            Vec4<float>::load(tail.k_w + half + 4 * j16, wk_b);
        }
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int bq = 0; bq < 4; ++bq) {
                    const int nl = wn + j * 32 + 8 * bq + 4 * (lane >> 5);
                    float v[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = acc[i][j][4 * bq + r];
                    if (bias) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) v[r] += bias[n0 + nl + r < N ? n0 + nl + r : N - 1];
                    }
                    Vec4<bf16_t>::store((bf16_t*)(smem + (wm + i * 32 + (lane & 31)) * TROW) + nl, v);
                }
        __syncthreads();
        for (int it0 = 0; it0 < NIT; it0 += CHUNK) {
            if (it0 > 0) { LOAD_TABLE_ROWS(it0) }
#pragma unroll
            for (int k = 0; k < CHUNK; ++k) {
                const int idx = tid / 16 + (it0 + k) * GROUPS;
                if (idx >= ITEMS) continue;
                const int hd = idx / BM, row = idx % BM;
                const int m = m0 + row, head = n0 / 128 + hd;
                if (m < M && head < tail.Hq + tail.Hkv) {                   // (values: below, by tiles)
                    const bool is_q = head < tail.Hq;
                    const bf16_t* src = (const bf16_t*)(smem + row * TROW) + hd * 128;
                    float a[4], b[4];
                    Vec4<bf16_t>::load(src + 4 * j16, a);
                    Vec4<bf16_t>::load(src + half + 4 * j16, b);
                    if (tail.q_w) {
                        float ss = 0.f;
#pragma unroll
                        for (int e = 0; e < 4; ++e) ss += a[e] * a[e] + b[e] * b[e];
                        ss = row16_sum(ss);                                  // (the item's 16 lanes are a row)
                        const float rstd = rsqrtf(ss / (float)D + tail.eps);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            a[e] = a[e] * rstd * (is_q ? wq_a[e] : wk_a[e]);
                            b[e] = b[e] * rstd * (is_q ? wq_b[e] : wk_b[e]);
                        }
                    }
                    if (tail.table) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) rotate_pair(c[k][e], sn[k][e], a[e], b[e]);
                    }
                    bf16_t* dst = nullptr;
                    if (is_q) {
                        dst = tail.q_out + ((long)m * tail.Hq + head) * D;
                    } else {
                        const int sl = slot_sh[row];
                        if (sl >= 0) dst = tail.cache + (long)(sl >> tail.lp) * page_stride + ((long)(head - tail.Hq) * tail.P + (sl & (tail.P - 1))) * D;
                    }
                    if (dst) {
                        Vec4<bf16_t>::store(dst + 4 * j16, a);
                        Vec4<bf16_t>::store(dst + half + 4 * j16, b);
                    }
                }
            }
        }
#undef LOAD_TABLE_ROWS
        // values: 16 tokens of a head at a time; where their slots lie side by side in one page,
        // 8 tokens of a feature are one 16-byte store into the transposed value tile [D][P].
        // Whether 16 rows lie so is found once, by one thread a group of rows (0: no, 1: yes).
        int* run_sh = slot_sh + BM;
        static_assert(BM * TROW + 2 * BM * 4 + (BM / 16) * 4 <= 2 * BUF, "the groups' flags must fit too");
        const bool has_values = tail.slots && n0 / 128 + BN / 128 > tail.Hq + tail.Hkv;   // the same for the whole block
        if (has_values && tid < BM / 16) {
            const int r0 = tid * 16, s0 = slot_sh[r0];
            bool run = m0 + r0 + 16 <= M && s0 >= 0 && (s0 & (tail.P - 1)) + 16 <= tail.P && (s0 & 7) == 0;
#pragma unroll
            for (int i = 1; i < 16; ++i) run = run && slot_sh[r0 + i] == s0 + i;
            run_sh[tid] = run ? 1 : 0;
        }
        if (has_values) __syncthreads();
        for (int hd = 0; hd < BN / 128; ++hd) {
            const int kh = n0 / 128 + hd - tail.Hq - tail.Hkv;
            if (!has_values || kh < 0 || kh >= tail.Hkv) continue;      // the same for the whole block
            // a thread: 16 rows from r0, the features d and d + 1, the tokens 8 h .. 8 h + 7 (two
            // features at a time: half the reads from shared memory)
            for (int idx = tid; idx < (BM / 16) * D; idx += 64 * NW) {
                const int r0 = idx / D * 16, d = idx % D / 2 * 2, h = idx % 2;
                if (m0 + r0 >= M) continue;
                if (run_sh[r0 / 16]) {
                    const int s0 = slot_sh[r0];
                    Piece16 lo, hi;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const unsigned two = *(const unsigned*)(smem + (r0 + 8 * h + e) * TROW + (hd * 128 + d) * 2);
                        lo.e[e] = (unsigned short)(two & 0xffffu);
                        hi.e[e] = (unsigned short)(two >> 16);
                    }
                    bf16_t* vt = tail.cache + (long)(s0 >> tail.lp) * page_stride + ((long)(tail.Hkv + kh) * tail.P) * D + (s0 & (tail.P - 1));
                    *(uint4_t*)(vt + (long)d * tail.P + 8 * h) = lo.q;
                    *(uint4_t*)(vt + (long)(d + 1) * tail.P + 8 * h) = hi.q;
                } else {
                    for (int e = 0; e < 8; ++e) {
                        const int i = 8 * h + e;
                        const int si = m0 + r0 + i < M ? slot_sh[r0 + i] : -1;
                        if (si >= 0) {
                            bf16_t* to = tail.cache + (long)(si >> tail.lp) * page_stride + ((long)(tail.Hkv + kh) * tail.P) * D + (si & (tail.P - 1));
                            const bf16_t* from = (const bf16_t*)(smem + (r0 + i) * TROW + (hd * 128 + d) * 2);
                            to[(long)d * tail.P] = from[0];
                            to[(long)(d + 1) * tail.P] = from[1];
                        }
                    }
                }
            }
        }
        return;
    }
    const int NO = SILU ? N / 2 : N;                       // width of the output
    constexpr int WNO = SILU ? WN / 2 : WN;                // output columns of a wave's strip
    constexpr int ESZ = (int)sizeof(TO);
    constexpr int CH = 16 / ESZ;                           // outputs in 16 bytes
    constexpr int CPR = WNO / CH;                          // 16-byte chunks in a row of the strip
    constexpr int SROW = WNO * ESZ + 16;                   // bytes of a staged row
    static_assert(NW * 32 * SROW <= 2 * BUF, "the strips of the waves must fit the staging buffers");
    unsigned char* strip = smem + wave * 32 * SROW;
    const int no0 = SILU ? (n0 + wn) / 2 : n0 + wn;        // first output column of the wave's strip
    const bool vec_ok = (NO % CH) == 0 && (((unsigned long)out) & 15) == 0;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        __builtin_amdgcn_sched_barrier(0);   // one strip after the other: nothing of the next is computed early
#pragma unroll
        for (int j = 0; j < NJ; j += (SILU ? 2 : 1))
#pragma unroll
            for (int bq = 0; bq < 4; ++bq) {
                const int nl = (SILU ? j * 16 : j * 32) + 8 * bq + 4 * (lane >> 5);   // column within the strip
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (SILU) {
                        const float gt = acc[i][j][4 * bq + r], up = acc[i][j + (SILU ? 1 : 0)][4 * bq + r];
                        v[r] = gt * __builtin_amdgcn_rcpf(1.f + __expf(-gt)) * up;   // rcp: within 1 ulp
                    } else {
                        v[r] = acc[i][j][4 * bq + r];
                    }
                }
                if (!SILU && bias && blockIdx.y == 0) {                       // (a column beyond the output is never stored: any bias does)
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] += bias[no0 + nl + r < NO ? no0 + nl + r : NO - 1];
                }
                Vec4<TO>::store((TO*)(strip + (lane & 31) * SROW) + nl, v);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the wave's writes before its reads
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int c = lane; c < 32 * CPR; c += 64) {
            const int row = c / CPR, col = (c % CPR) * CH;
            const int m = m0 + wm + i * 32 + row, n = no0 + col;
            if (m >= M || n >= NO) continue;
            const uint4_t piece = *(const uint4_t*)(strip + row * SROW + col * ESZ);
            TO* o = out + ((long)blockIdx.y * M + m) * NO + n;
            if (vec_ok) {
                *(uint4_t*)o = piece;                      // n + CH <= NO: both are multiples of CH
            } else {
                const TO* pv = (const TO*)&piece;
#pragma unroll
                for (int e = 0; e < CH; ++e) if (n + e < NO) o[e] = pv[e];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the reads before the next strip's writes
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

bool qe_gemm_mfma_ok(int M, int N, int K, int dt_a, int dt_w) {
    return dt_a == QE_BF16 && dt_w == QE_BF16 && M > 16 && K % 8 == 0 && K >= 64;
}

template <typename TO, int BM, int BN, int BK, int NW, int MINB, bool SILU, bool QKV = false>
static int launch_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                       int splits, hipStream_t stream, const QkvTail& tail = QkvTail{}) {
    const int tiles_m = qe_cdiv(M, BM), tiles_n = qe_cdiv(N, BN);
    const long blocks = (long)tiles_m * tiles_n;
    QE_REQUIRE(blocks <= 2147483647L, "mfma gemm: too many tiles");
    const size_t shmem = 2 * (BM + BN) * (BK * 2 + 16);
    static bool attr_set = false;   // one flag per instantiation
    if (!attr_set) {
        (void)hipFuncSetAttribute((const void*)gemm_mfma_kernel<TO, BM, BN, BK, NW, MINB, SILU, QKV>,
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        attr_set = true;
    }
    // a cut of K is a multiple of BK long (the last may be shorter)
    const int k_per_split = splits > 1 ? qe_cdiv(qe_cdiv(K, splits), BK) * BK : K;
    QE_REQUIRE(splits >= 1 && splits <= 65535 && (long)(splits - 1) * k_per_split < K,
               "mfma gemm: K=%d cannot be cut into %d parts", K, splits);
    // the eight XCDs as a by b parts of the tiles (a b = 8): every XCD reads M / a rows of x and
    // N / b rows of W, so all of them together b M + a N rows
    int xcd_m = 0, xcd_n = 0;
    long fewest = 0;
    for (int a = 1; a <= 8; a *= 2) {
        const int b = 8 / a;
        if (tiles_m % a || tiles_n % b) continue;
        const long rows = (long)b * M + (long)a * N;
        if (xcd_m == 0 || rows < fewest) { xcd_m = a; xcd_n = b; fewest = rows; }
    }
    gemm_mfma_kernel<TO, BM, BN, BK, NW, MINB, SILU, QKV><<<dim3((unsigned)blocks, (unsigned)splits), 64 * NW, shmem, stream>>>(
        (const bf16_t*)x, (const bf16_t*)w, bias, (TO*)out, M, N, K, tiles_m, tiles_n, k_per_split, xcd_m, xcd_n,
        (!QKV && M <= 64 && (K * 2) % 8192 == 0) ? 1 : 0, tail);
    QE_LAUNCH_CHECK();
    return 0;
}

static int choose_tile(int M, int N, int splits, bool with_256x256 = true) {
    // The shape is chosen by what the busiest compute unit gets: its number of tiles (they are dealt
    // out in turn) times a tile's area, over how well the shape uses the unit (measured on large
    // products: 256 x 256 reaches 1.30, 256 x 128 1.16, 128 x 128 1.07, 64 x 128 0.80 PFLOP/s).
    // A shape is never taller than the rows need.
    // The two smaller shapes reach their rate with two blocks on a compute unit: where the busiest
    // unit gets an odd number of them, three or more, the last runs alone at 0.7 of the rate
    // (5120 columns against 2048 rows: 640 tiles of 128 x 128 took 632 us where 160 of 256 x 256 took 513).
    const long cus = 256;
    struct Shape { int tile, bm, bn; float rate; bool pairs; };
    const Shape shapes[4] = {{64, 64, 128, 0.80f, true}, {128, 128, 128, 1.07f, true}, {256, 256, 128, 1.16f, false},
                             {512, 256, 256, 1.30f, false}};
    int tile = 0;
    float best = 0.f;
    for (const Shape& sh : shapes) {
        if (sh.tile != 64 && M <= sh.bm / 2) continue;
        if (sh.tile == 512 && !with_256x256) continue;
        const long blocks = (long)qe_cdiv(M, sh.bm) * qe_cdiv(N, sh.bn) * splits;
        const long turns = qe_cdiv(blocks, cus);
        const float alone = sh.pairs && turns >= 3 && turns % 2 ? 1.f / 0.7f - 1.f : 0.f;
        const float cost = ((float)turns + alone) * sh.bm * sh.bn / sh.rate;
        if (tile == 0 || cost < best) { tile = sh.tile; best = cost; }
    }
    return tile;
}

template <typename TO, bool SILU>
static int pick_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K,
                     int tile, int splits, hipStream_t stream) {
    // Up to 64 rows against a gate|up matrix of at most one tile column a compute unit (its K cannot be
    // cut): a block streams its weights alone on its unit, and what it has in flight bounds it.  A k step of
    // 128 doubles that (24576 x 4096 against 64 rows: 44.4 us against 49.2; with two blocks a unit, 51200 x
    // 5120, it gains nothing).
    if (tile == 0 && SILU && M <= 64 && qe_cdiv(N, 128) <= 256) tile = 65;
    if (tile == 0) tile = choose_tile(M, N, splits);
    if (tile == 65) return launch_mfma<TO, 64, 128, 128, 4, 1, SILU>(x, w, bias, out, M, N, K, splits, stream);
    if (tile == 512) return launch_mfma<TO, 256, 256, 64, 4, 1, SILU>(x, w, bias, out, M, N, K, splits, stream);
    if (tile == 256) return launch_mfma<TO, 256, 128, 64, 8, 1, SILU>(x, w, bias, out, M, N, K, splits, stream);
    if (tile == 128) return launch_mfma<TO, 128, 128, 64, 4, 2, SILU>(x, w, bias, out, M, N, K, splits, stream);
    return launch_mfma<TO, 64, 128, 64, 4, 2, SILU>(x, w, bias, out, M, N, K, splits, stream);
}

// tile: rows of the output tile (256, 128 or 64; 512 stands for 256 x 256, 65 for 64 x 128 with a k step of 128), 0 to choose
// by the shape.  silu: w is [N, K] with
// gate and up rows interleaved in blocks of 32, out is [M, N / 2] = silu(gate) * up.
// splits > 1: out is float [splits, M, N], partial products along K (no silu then).
int qe_gemm_mfma(const void* x, const void* w, const float* bias, void* out, int M, int N, int K, int dt_o,
                 int tile, bool silu, int splits, hipStream_t stream) {
    QE_REQUIRE(splits >= 1 && (splits == 1 || (!silu && dt_o == QE_F32)), "mfma gemm: partial products are 32-bit and plain");
    QE_REQUIRE(K % 8 == 0 && K >= 64 && K < (1 << 22), "mfma gemm: K=%d is no multiple of 8 in [64, 2^22)", K);
    QE_REQUIRE(tile == 0 || tile == 512 || tile == 256 || tile == 128 || tile == 64 || tile == 65, "mfma gemm: tile of %d rows", tile);
    if (silu) {
        QE_REQUIRE(!bias && N % 64 == 0, "mfma gemm: silu-mul takes no bias and gate|up rows in blocks of 32");
        if (dt_o == QE_BF16) return pick_mfma<bf16_t, true>(x, w, bias, out, M, N, K, tile, splits, stream);
        return pick_mfma<float, true>(x, w, bias, out, M, N, K, tile, splits, stream);
    }
    if (dt_o == QE_BF16) return pick_mfma<bf16_t, false>(x, w, bias, out, M, N, K, tile, splits, stream);
    return pick_mfma<float, false>(x, w, bias, out, M, N, K, tile, splits, stream);
}

// The q|k|v product of an attention layer with what follows it inside (see QkvTail): x [M, K] .
// w [(Hq + 2 Hkv) 128, K]^T (+ bias), then q to q_out [M, Hq, 128] and k, v into the cache
// [pages, 2, Hkv, P, 128] at slots[m] (negative or no slots: nowhere).  positions [M] index the
// table's rows [cos | sin] of 128 floats; q_w, k_w, table may be null.
int qe_gemm_qkv(const void* x, const void* w, const float* bias, int M, int K, int Hq, int Hkv, int P,
                const int* positions, const int* slots, const float* q_w, const float* k_w, float eps,
                const float* table, void* q_out, void* cache, int tile, hipStream_t stream) {
    const int N = (Hq + 2 * Hkv) * 128;
    QE_REQUIRE(K % 8 == 0 && K >= 64 && K < (1 << 22), "qkv gemm: K=%d is no multiple of 8 in [64, 2^22)", K);
    QE_REQUIRE(M > 16 && Hq > 0 && Hkv > 0 && P >= 16 && (P & (P - 1)) == 0, "qkv gemm: sizes not taken");
    QE_REQUIRE(tile == 0 || tile == 512 || tile == 256 || tile == 128 || tile == 64, "qkv gemm: tile of %d rows", tile);
    QE_REQUIRE(!table || positions, "qkv gemm: a rotation needs positions");
    int lp = 0;
    while ((1 << lp) < P) ++lp;
    QkvTail tail{positions, slots, q_w, k_w, table, (bf16_t*)q_out, (bf16_t*)cache, eps, Hq, Hkv, P, lp};
    // (the 256 x 256 shape has four waves for an epilogue over 65536 values: the others finish it sooner)
    if (tile == 0) tile = choose_tile(M, N, 1, false);
    if (tile == 512) return launch_mfma<bf16_t, 256, 256, 64, 4, 1, false, true>(x, w, bias, nullptr, M, N, K, 1, stream, tail);
    if (tile == 256) return launch_mfma<bf16_t, 256, 128, 64, 8, 1, false, true>(x, w, bias, nullptr, M, N, K, 1, stream, tail);
    if (tile == 128) return launch_mfma<bf16_t, 128, 128, 64, 4, 2, false, true>(x, w, bias, nullptr, M, N, K, 1, stream, tail);
    return launch_mfma<bf16_t, 64, 128, 64, 4, 2, false, true>(x, w, bias, nullptr, M, N, K, 1, stream, tail);
}
