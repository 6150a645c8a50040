// Attention of portions of prompts over the paged cache (prefill), bfloat16, on the MFMA units
// with 32 x 32 tiles.
//
// A wave owns 32 columns: R consecutive query rows of a request for each of GH = 32 / R query
// heads that share one key/value head (GH = the group size when that is a power of two up to 32,
// else 1), so one pass over the keys serves the whole group.  A block is four waves with four
// neighbouring row tiles of one request.  It walks the keys its rows see, 32 at a time, from the
// cache pages (keys written by this same step included): the 256 threads bring the next key
// tile and value tile into shared memory with contiguous 16-byte loads while the waves compute
// on the current one (two buffers, one barrier per tile); every wave then reads its MFMA
// operands from shared memory, whose rows are padded so that those reads do not collide.
//   S^T[key, col] = K[key, :] . Q[col, :]         v_mfma_f32_32x32x16_bf16, D / 16 of them;
//       lane (g, r), g = lane / 32, r = lane % 32, takes K[key r][ks * 16 + g * 8 .. + 8]
//       and ends up with 16 scores: keys 8 b + 4 g + j (b, j < 4) of column r
//   online softmax per column in 32-bit, in the base-2 domain (scores are scaled by
//       scale * log2 e once); the accumulator is rescaled only when a score exceeds the column's
//       reference by more than 8
//   O^T[d, col] += V^T[d, key] . P^T[key, col]    v_mfma_f32_32x32x16_bf16, 2 * D / 32 of them;
//       the 8 probabilities of a half tile that a lane holds are its B operand as they lie, and
//       because value tiles are stored transposed ([D][P]) the A operand is the same 8 keys of
//       one row of V^T: the staged rows hold the keys in the order 0-3, 8-11, 4-7, 12-15, so that
//       it is one 16-byte read
// The causal and window limits are applied per column, so the order of the sums for a row
// depends on its position and the window only.
//
// With NG = 2 a block has two such groups of four waves on the same four row tiles: group 0 takes
// the even key tiles and group 1 the odd ones, each through shared buffers of its own, and at the
// end group 0 merges the two partial results (maxima, sums, accumulators) through shared memory.
// That halves the length of the longest block, which is what the time of a causal prompt hangs on
// when there are no more blocks than compute units.  The longest blocks are started first.
//
// Key segments: with fewer blocks than compute units and many keys (a portion of a prompt far into
// its context) the keys are cut at absolute multiples of a segment length, and the blocks of the
// grid's second dimension walk one segment each.  A block whose rows' keys lie in one segment writes
// its result as before (the blocks of the other segments leave at once); else the blocks of the
// segments that hold keys of its rows leave their maxima, sums and accumulators, as the lanes hold
// them, in a workspace, and attention_prefill_merge_kernel, with the same lanes, weighs and adds them
// in the order of the segments.  The segment length comes from the host, or, where the host does not
// know the positions (a recorded step), from the position of the row that sees the most keys.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) unsigned int uint4_t;

union PackV {   // an MFMA operand, also addressable as two 8-byte pieces
    bf16x8 v;
    uint2 u[2];
};
union Piece {   // a staged 16-byte piece, addressable by element for masking
    uint4_t q;
    uint2 u[2];
    unsigned short e[8];
};

// Lane i and lane i ^ 32 exchange a value without a trip through shared memory.
__device__ __forceinline__ float max_of_both_halves(float v) {
    float a, b;
    pair_across_halves(v, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float sum_of_both_halves(float v) {
    float a, b;
    pair_across_halves(v, a, b);
    return a + b;
}

#define QE_PREFILL_UNCUT_KEYS 1024
#define QE_PREFILL_MIN_SEGMENT 512
#define VROW 48   // bytes of a staged value row: 16 keys = 32 bytes of data + 16 of padding

// The keys of a segment when ``keys`` keys are cut into ks segments: a multiple of 64, at least
// QE_PREFILL_MIN_SEGMENT; 0 (no cut) up to QE_PREFILL_UNCUT_KEYS keys.  One formula for the host's plan
// and for the kernels of a recorded step, which cut by a position they read on the device.
__host__ __device__ __forceinline__ int prefill_segment_length(int keys, int ks) {
    if (keys <= QE_PREFILL_UNCUT_KEYS || ks <= 1) return 0;
    const int seg = ((keys + ks - 1) / ks + 63) / 64 * 64;
    return seg < QE_PREFILL_MIN_SEGMENT ? QE_PREFILL_MIN_SEGMENT : seg;
}

// The keys of a segment when the host does not know the positions (a recorded step): seg_param < 0
// asks for -seg_param segments of the keys that row keys_row sees, each a multiple of 64 and at least
// QE_PREFILL_MIN_SEGMENT keys; up to QE_PREFILL_UNCUT_KEYS keys nothing is cut (0).  The same value
// in every block of the two kernels.
__device__ __forceinline__ int segment_keys(int seg_param, const int* __restrict__ positions, int keys_row) {
    if (seg_param >= 0) return seg_param;
    return prefill_segment_length(positions[keys_row] + 1, -seg_param);
}

// A lane's share of its column's result: the accumulators' element 4 b + j of block db is feature
// 32 db + 8 b + 4 g + j.
template <int D>
__device__ __forceinline__ void store_columns(bf16_t* __restrict__ out, const floatx16 (&acc)[D / 32], float inv,
                                              int row, int head, int Hq, int g) {
    bf16_t* orow = out + ((long)row * Hq + head) * D + 4 * g;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            bf16x4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = (__bf16)(acc[db][4 * b + j] * inv);
            *(bf16x4*)(orow + db * 32 + 8 * b) = o;
        }
}

// Two waves per SIMD (at most 256 registers a lane), as two blocks of one group or one block of
// two: while one wave waits for its next tile or at its barrier, the other computes.
template <int D, int NG>
__global__ __launch_bounds__(256 * NG, NG == 1 ? 2 : 1) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ tiles, const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks,
    int Hq, int Hkv, int P, int log2P, float scale_log2, int window, int R, int seg_param, int keys_row,
    float* __restrict__ part) {
    constexpr int KROW = D * 2 + 16;                 // bytes of a staged key row
    constexpr int KBYTES = 32 * KROW, VBYTES = 2 * D * VROW, BUF = KBYTES + VBYTES;
    constexpr int KP = 32 * (D / 8) / 256;           // 16-byte key pieces per thread (2 for D = 128)
    constexpr int VP = 2 * D * 2 / 256;              // 16-byte value pieces per thread
    __shared__ __attribute__((aligned(16))) unsigned char smem_all[NG * 2 * BUF];

    // (group and wave are the same for all lanes of a wave: kept in scalar registers, so that what
    // follows from them — tile keys, pages, addresses — is scalar arithmetic)
    const int grp = __builtin_amdgcn_readfirstlane(threadIdx.x / 256);   // which half of the key tiles (NG = 2)
    const int tid = threadIdx.x % 256, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned char* smem = smem_all + grp * 2 * BUF;
    const int g = lane >> 5, r = lane & 31;
    const int G = Hq / Hkv;
    const int GH = 32 / R;                                 // heads per wave
    // The grid is (head waves, segments, tile groups): blocks start in the order of the first
    // dimension first, so all heads and segments of the last rows (the longest walks) start before
    // anything of earlier rows, and a compute unit that is done takes the longest of what is left.
    const int bhead = blockIdx.x, bseg = blockIdx.y, bgroup = blockIdx.z;
    const int kvh = bhead / (G / GH);
    const int head = kvh * G + (bhead % (G / GH)) * GH + r / R;   // this lane's column: head and row

    // the block's four tiles belong to one request, in ascending rows; tiles of 0 rows pad the group
    const int* bt4 = tiles + 8 * (gridDim.z - 1 - bgroup);   // later rows see more keys: they start first
    if (bt4[1] <= 0) return;                               // a group without rows (a list filled up to a fixed length)
    const int row_first = bt4[0];
    int last = 0;
#pragma unroll
    for (int j = 1; j < 4; ++j) if (bt4[2 * j + 1] > 0) last = j;
    const int p_block = positions[row_first];
    int kmin = (window > 0 && p_block - window + 1 > 0) ? p_block - window + 1 : 0;
    int kmax = positions[bt4[2 * last]] + bt4[2 * last + 1];
    // key segments: this block walks the keys of segment bseg only
    bool partial = false;
    const int seg_keys = segment_keys(seg_param, positions, keys_row);
    if (seg_keys <= 0 && bseg > 0) return;                 // (asked for segments, but the keys are too few to cut)
    if (seg_keys > 0) {
        const int z = bseg, z_lo = kmin / seg_keys, z_hi = (kmax - 1) / seg_keys;
        if (z < z_lo || z > z_hi) return;                  // (the whole block: no barrier has been met yet)
        partial = z_hi > z_lo;
        if (partial) {
            kmin = max(kmin, z * seg_keys);
            kmax = min(kmax, (z + 1) * seg_keys);
        }
    }
    const int* bt = block_table + (long)tok_seq[row_first] * max_blocks;
    const long page_stride = 2L * Hkv * P * D;

    // this wave's tile
    const int row0 = bt4[2 * wave], cnt = bt4[2 * wave + 1];
    const bool wave_on = cnt > 0;
    const int rr = r % R;
    const bool col_ok = wave_on && rr < cnt;
    const int row = wave_on ? row0 + (rr < cnt ? rr : cnt - 1) : row_first;   // columns beyond the tile repeat its last row
    const int p = positions[row];
    const int hi = p + 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int p_first = positions[wave_on ? row0 : row_first];
    const int k_start = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int k_stop = wave_on ? p_first + cnt : 0;       // positions of a tile's rows are consecutive
    // keys every column of the wave sees without a limit: [all_lo, all_hi)
    const int p_last = p_first + cnt - 1;
    const int all_hi = p_first + 1;
    const int all_lo = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;

    bf16x8 qreg[D / 16];
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
        qreg[ks] = *(const bf16x8*)(q + ((long)row * Hq + head) * D + ks * 16 + g * 8);
    // Wait for q here, with an instruction the compiler sees: else it waits for these loads where q
    // is first used, inside the loop, where its count of loads in flight includes the loop's own,
    // and every round would end up waiting for the loads it has just issued.
    __builtin_amdgcn_s_waitcnt(0x0f70);                    // vmcnt(0)

    float m = -INFINITY, l = 0.f;
    floatx16 acc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;

    // ---- staging: global -> registers -> shared ------------------------------------------------
    // A 32-key tile has two halves of 16 keys with pages and offsets of their own.  A half that no
    // row of the block sees (beyond the request's keys, or wholly behind the window, where the page
    // may have been given back) reads the other half's memory again; what lies outside
    // [kmin, kmax) is zeroed in the value tile (it may be unwritten memory, and anything times a
    // weight of 0 must still be 0) and masked in the scores.
    // Two sets of staging registers in turn: the loads of a tile are issued two tiles ahead and
    // stored to shared memory one tile ahead, so a load has a whole tile's computation to arrive
    // (one tile of arithmetic is shorter than a trip to memory).
    // The loads are buffer loads: the page's address and the offset of the 16 keys in it are
    // scalar, and a thread adds bytes that are constant over the loop.  Which half of the tile a
    // piece belongs to is the same for a whole wave (256 pieces are 2 D / 8 rows of 8 pieces).
    Piece kst[2][KP], vst[2][VP];
    int kconst[KP], vconst[VP];                           // bytes from the page's start, without the keys' offset
    bool khalf[KP], vhalf[VP];
#pragma unroll
    for (int i = 0; i < KP; ++i) {
        const int id = tid + 256 * i;
        const int krow = id / (D / 8), col = id % (D / 8);
        khalf[i] = __builtin_amdgcn_readfirstlane(krow >= 16);
        kconst[i] = ((kvh * P + (krow & 15)) * D + col * 8) * 2;
    }
#pragma unroll
    for (int i = 0; i < VP; ++i) {
        const int id = tid + 256 * i;
        const int rem = id % (2 * D);
        vhalf[i] = __builtin_amdgcn_readfirstlane(id >= 2 * D);
        vconst[i] = (((Hkv + kvh) * P) * D + (rem >> 1) * P + (rem & 1) * 8) * 2;
    }
    const int pmask = P - 1;
    const int page_bytes = (int)page_stride * 2;
#define STAGE_LOAD(set_, kk_)                                                                       \
    {                                                                                               \
        const bool first_ = (kk_) + 16 > kmin, second_ = (kk_) + 16 < kmax;                         \
        const int ka_ = first_ ? (kk_) : (kk_) + 16;                                                \
        const int kb_ = second_ ? (kk_) + 16 : (kk_);                                               \
        const __amdgpu_buffer_rsrc_t ra_ = __builtin_amdgcn_make_buffer_rsrc(                       \
            (void*)(cache + (long)bt[ka_ >> log2P] * page_stride), 0, page_bytes, 0x00020000);      \
        const __amdgpu_buffer_rsrc_t rb_ = __builtin_amdgcn_make_buffer_rsrc(                       \
            (void*)(cache + (long)bt[kb_ >> log2P] * page_stride), 0, page_bytes, 0x00020000);      \
        const int oa_ = (ka_ & pmask) * 2, ob_ = (kb_ & pmask) * 2;   /* bytes in a row of V^T */   \
        _Pragma("unroll") for (int i = 0; i < KP; ++i)                                              \
            kst[set_][i].q = __builtin_amdgcn_raw_buffer_load_b128(khalf[i] ? rb_ : ra_, kconst[i], \
                                                                   (khalf[i] ? ob_ : oa_) * D, 0);  \
        _Pragma("unroll") for (int i = 0; i < VP; ++i)                                              \
            vst[set_][i].q = __builtin_amdgcn_raw_buffer_load_b128(vhalf[i] ? rb_ : ra_, vconst[i], \
                                                                   vhalf[i] ? ob_ : oa_, 0);        \
    }
#define STAGE_STORE(buf_, set_, kk_)                                                                \
    {                                                                                               \
        if ((kk_) + 32 > kmax || (kk_) < kmin) {                                                    \
            _Pragma("unroll") for (int i = 0; i < VP; ++i) {                                        \
                const int id = tid + 256 * i;                                                       \
                const int half = id / (2 * D), part = id & 1;                                       \
                _Pragma("unroll") for (int e = 0; e < 8; ++e) {                                     \
                    const int key = (kk_) + 16 * half + 8 * part + e;                               \
                    if (key < kmin || key >= kmax) vst[set_][i].e[e] = 0;                           \
                }                                                                                   \
            }                                                                                       \
        }                                                                                           \
        unsigned char* ks_ = smem + (buf_) * BUF;                                                   \
        unsigned char* vs_ = ks_ + KBYTES;                                                          \
        _Pragma("unroll") for (int i = 0; i < KP; ++i) {                                            \
            const int id = tid + 256 * i;                                                           \
            *(uint4_t*)(ks_ + (id / (D / 8)) * KROW + (id % (D / 8)) * 16) = kst[set_][i].q;        \
        }                                                                                           \
        _Pragma("unroll") for (int i = 0; i < VP; ++i) {                                            \
            const int id = tid + 256 * i;                                                           \
            unsigned char* dst = vs_ + (id >> 1) * VROW + (id & 1) * 8;                             \
            *(uint2*)dst = vst[set_][i].u[0];                                                       \
            *(uint2*)(dst + 16) = vst[set_][i].u[1];                                                \
        }                                                                                           \
    }

    // The group's i-th tile holds the keys from kk0 + 32 (NG i + grp) on and uses register set and
    // shared buffer i % 2.  All groups make the same number of rounds (the barriers are the
    // block's); a round whose tile lies beyond the keys brings and computes nothing.
    const int kk0 = (kmin / 32) * 32;
    const int rounds = ((kmax - kk0 + 31) / 32 + NG - 1) / NG;
#define TILE_KEY(i_) (kk0 + 32 * (NG * (i_) + grp))
    const int kk_first = TILE_KEY(0), kk_second = TILE_KEY(1);
    if (kk_first < kmax) {
        STAGE_LOAD(0, kk_first)
        STAGE_STORE(0, 0, kk_first)
    }
    // (From here on the loads are issued whether their tile exists or not, one that does not
    // exist reads the first tile again and is never stored: with loads under a condition the
    // compiler cannot count how many are in flight and waits for all of them before every store
    // to shared memory, the ones just issued included.)
#define EXISTING(kk_) ((kk_) < kmax ? (kk_) : kk0)
    STAGE_LOAD(1, EXISTING(kk_second))
    __syncthreads();
    for (int i2 = 0; i2 < rounds; i2 += 2) {
#pragma unroll
      for (int buf = 0; buf < 2; ++buf) {
        const int i = i2 + buf;
        if (i >= rounds) break;                           // the same for all threads of the block
        const int kk = TILE_KEY(i);
        const int kk_1 = TILE_KEY(i + 1), kk_2 = TILE_KEY(i + 2);   // (values, not expressions in i: the macros have loops over i)
        STAGE_LOAD(buf, EXISTING(kk_2))                   // this set's tile went to shared memory a round ago
        __builtin_amdgcn_sched_barrier(0);                // keep the loads ahead of the computation
        if (wave_on && kk < k_stop && kk + 32 > k_start && kk < kmax) {   // some row of the wave sees some key of the tile, and it is a tile of this block's keys
            const unsigned char* ks_ = smem + buf * BUF + r * KROW + g * 16;
            const unsigned char* vs_ = smem + buf * BUF + KBYTES + r * VROW + g * 16;
            // all key fragments are read before the first MFMA, all value fragments before the
            // softmax: shared-memory latency then passes under the arithmetic instead of before it
            bf16x8 kf[D / 16];
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks) kf[ks] = *(const bf16x8*)(ks_ + ks * 32);
            __builtin_amdgcn_sched_barrier(0);
            floatx16 s;
#pragma unroll
            for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks)
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qreg[ks], s, 0, 0, 0);
            PackV vf[D / 32][2];
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    vf[db][h].v = *(const bf16x8*)(vs_ + (h * D + db * 32) * VROW);
                }

            // (the scores stay unscaled: the scale is positive, so it is applied to the maximum, and
            // to each score by the multiply-add that also subtracts the maximum)
            float tmax = -INFINITY;
            if (kk >= all_lo && kk + 32 <= all_hi) {       // every column sees every key of the tile
#pragma unroll
                for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, s[e]);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = kk + 8 * (e >> 2) + 4 * g + (e & 3);
                    s[e] = (key >= lo && key < hi) ? s[e] : -INFINITY;
                    tmax = fmaxf(tmax, s[e]);
                }
            }
            tmax = max_of_both_halves(tmax) * scale_log2;
            // m is the reference the weights are taken against, not the exact maximum: a column moves
            // it only when a score exceeds it by more than 8 (a weight above 2^8), which after the
            // first tiles is rare, so that the accumulators are seldom rescaled.  The decision is the
            // column's own: its sums do not depend on the other columns of the wave.
            const bool moves = tmax > m + 8.f;                 // (never for a tile without a visible key)
            if (__any(moves)) {
                const float alpha = moves ? __builtin_amdgcn_exp2f(m - tmax) : 1.f;   // 0 from a column's first keys
                m = moves ? tmax : m;
                l *= alpha;
#pragma unroll
                for (int db = 0; db < D / 32; ++db) acc[db] *= alpha;
            }
            const float ref = (m == -INFINITY) ? 0.f : m;      // a column that has seen no key yet: all weights 0
            PackV pb[2];
            float psum = 0.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], scale_log2, -ref));   // 0 for keys that are not seen
                psum += pe;
                pb[e >> 3].v[e & 7] = (__bf16)pe;
            }
            l += psum;
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][h].v, pb[h].v, acc[db], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kk_1 < kmax) STAGE_STORE(buf ^ 1, buf ^ 1, kk_1)   // that buffer's readers finished before the last barrier
        __syncthreads();
      }
    }
#undef STAGE_LOAD
#undef EXISTING
#undef STAGE_STORE
#undef TILE_KEY
    l = sum_of_both_halves(l);
    if (NG == 2) {
        // group 1 hands its maxima, sums and accumulators to group 0, 16 values of every lane at a
        // time, through the staging memory (free after the loop's last barrier): [wave][value][lane]
        float* xch = (float*)smem_all + wave * 18 * 64 + lane;
        float a_own = 1.f, a_other = 0.f;
        if (grp == 1) { xch[0] = m; xch[64] = l; }
        __syncthreads();
        if (grp == 0) {
            const float m1 = xch[0], l1 = xch[64];
            const float mt = fmaxf(m, m1);
            const float ref = (mt == -INFINITY) ? 0.f : mt;
            a_own = __builtin_amdgcn_exp2f(m - ref);       // 0 for a side that has seen no key
            a_other = __builtin_amdgcn_exp2f(m1 - ref);
            l = l * a_own + l1 * a_other;
            m = mt;
        }
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
            if (grp == 1) {
#pragma unroll
                for (int e = 0; e < 16; ++e) xch[(2 + e) * 64] = acc[db][e];
            }
            __syncthreads();
            if (grp == 0) {
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[db][e] = acc[db][e] * a_own + xch[(2 + e) * 64] * a_other;
            }
            __syncthreads();
        }
        if (grp == 1) return;
    }
    if (partial) {
        // as the lanes hold them: [segment][block][wave][value][lane], value = m, l, then the accumulators
        constexpr int NV = 2 + (D / 32) * 16;
        float* dst = part + ((((long)bseg * gridDim.x + bhead) * gridDim.z + bgroup) * 4 + wave) * NV * 64 + lane;
        dst[0] = m;
        dst[64] = l;
        if (m != -INFINITY) {                              // (a column that saw no key of the segment: nothing else is read of it)
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int e = 0; e < 16; ++e) dst[(2 + db * 16 + e) * 64] = acc[db][e];
        }
        return;
    }
    if (col_ok) store_columns<D>(out, acc, 1.f / l, row, head, Hq, g);
}

// The segments' partial results of the blocks that left some: the same first two grid dimensions
// and the same lanes as the kernel above, the third dimension being the block of 32 features;
// lane by lane, in the order of the segments.
template <int D>
__global__ __launch_bounds__(256) void attention_prefill_merge_kernel(
    const float* __restrict__ part, bf16_t* __restrict__ out, const int* __restrict__ tiles,
    const int* __restrict__ positions, int Hq, int Hkv, int window, int R, int seg_param, int keys_row) {
    constexpr int NV = 2 + (D / 32) * 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 5, r = lane & 31;
    const int G = Hq / Hkv, GH = 32 / R;
    const int bhead = blockIdx.x, db = blockIdx.y, bgroup = blockIdx.z;     // (head waves, feature blocks, tile groups)
    const int kvh = bhead / (G / GH);
    const int head = kvh * G + (bhead % (G / GH)) * GH + r / R;
    const int* bt4 = tiles + 8 * (gridDim.z - 1 - bgroup);
    if (bt4[1] <= 0) return;
    const int row_first = bt4[0];
    int last = 0;
#pragma unroll
    for (int j = 1; j < 4; ++j) if (bt4[2 * j + 1] > 0) last = j;
    const int p_block = positions[row_first];
    const int kmin = (window > 0 && p_block - window + 1 > 0) ? p_block - window + 1 : 0;
    const int kmax = positions[bt4[2 * last]] + bt4[2 * last + 1];
    const int seg_keys = segment_keys(seg_param, positions, keys_row);
    if (seg_keys <= 0) return;                             // nothing was cut
    const int z_lo = kmin / seg_keys, z_hi = (kmax - 1) / seg_keys;
    if (z_hi <= z_lo) return;                              // the block wrote its result itself
    const int row0 = bt4[2 * wave], cnt = bt4[2 * wave + 1];
    const int rr = r % R;
    if (cnt <= 0 || rr >= cnt) return;
    const int row = row0 + rr;
    const long zstride = (long)gridDim.x * gridDim.z * 4 * NV * 64;
    const float* src = part + (((long)bhead * gridDim.z + bgroup) * 4 + wave) * NV * 64 + lane;
    float M = -INFINITY;
    for (int z = z_lo; z <= z_hi; ++z) M = fmaxf(M, src[z * zstride]);
    float l = 0.f;
    floatx16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    for (int z = z_lo; z <= z_hi; ++z) {
        const float mz = src[z * zstride];
        if (mz == -INFINITY) continue;                     // no key of this segment was seen by the column
        const float wgt = __builtin_amdgcn_exp2f(mz - M);
        l += wgt * src[z * zstride + 64];
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] += wgt * src[z * zstride + (2 + db * 16 + e) * 64];
    }
    const float inv = 1.f / l;
    bf16_t* orow = out + ((long)row * Hq + head) * D + 4 * g + db * 32;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        bf16x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = (__bf16)(acc[4 * b + j] * inv);
        *(bf16x4*)(orow + 8 * b) = o;
    }
}

// The tile list of qe_attention_prefill from the step's portions, made on the device (a recorded step
// does not know its portions' lengths on the host): portions [n_portions][2] = (first row, rows), each
// cut into tiles of at most `rows_per_tile` rows in groups of four, a group filled up with tiles of no
// rows; the list is filled up to max_groups groups with groups of no rows.  One thread per group.
__global__ void prefill_tiles_kernel(const int* __restrict__ portions, int n_portions, int rows_per_tile,
                                     int* __restrict__ tiles, int max_groups) {
    const int grp = blockIdx.x * blockDim.x + threadIdx.x;
    if (grp >= max_groups) return;
    int first = 0, start = 0, rows = 0, in_portion = -1;   // which portion the group lies in, and the group's place in it
    for (int i = 0; i < n_portions; ++i) {
        const int n = portions[2 * i + 1];
        const int groups = n > 0 ? (n + 4 * rows_per_tile - 1) / (4 * rows_per_tile) : 0;
        if (in_portion < 0 && grp < first + groups) {
            in_portion = grp - first;
            start = portions[2 * i];
            rows = n;
        }
        first += groups;
    }
    int* out = tiles + 8 * grp;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = in_portion < 0 ? rows : (4 * in_portion + j) * rows_per_tile;    // rows before this tile in its portion
        const int cnt = in_portion < 0 || r >= rows ? 0 : min(rows_per_tile, rows - r);
        out[2 * j] = cnt > 0 ? start + r : start;
        out[2 * j + 1] = cnt;
    }
}

int qe_attention_prefill_tiles(const int* portions, int n_portions, int rows_per_tile, int* tiles, int max_groups,
                               hipStream_t stream) {
    QE_REQUIRE(portions && tiles && n_portions >= 1 && n_portions <= 64 && rows_per_tile >= 1 && max_groups >= 1,
               "prefill tiles: %d portions, tiles of %d rows, %d groups", n_portions, rows_per_tile, max_groups);
    prefill_tiles_kernel<<<qe_cdiv(max_groups, 64), 64, 0, stream>>>(portions, n_portions, rows_per_tile, tiles, max_groups);
    QE_LAUNCH_CHECK();
    return 0;
}

// Rows per tile for a model's head counts: 32 / (heads that one wave serves).
int qe_attention_prefill_tile_rows(int Hq, int Hkv) {
    const int G = Hq / Hkv;
    const bool pow2 = G > 0 && (G & (G - 1)) == 0 && G <= 32;
    return 32 / (pow2 ? G : 1);
}

// How the keys of a call are best cut into segments: 0 (not at all) or the keys a segment (a multiple
// of 64).  blocks: blocks of the grid without segments; max_keys: the most keys a row of the call
// sees.  Every segment costs a trip of the partial results through memory, and more blocks than
// compute units gained nothing where it was measured (a whole prompt of 1536 or 2048 tokens took
// longer in two segments than in one), so there are only as many segments as fill the chip, of at
// least 512 keys; up to QE_PREFILL_UNCUT_KEYS keys a walk is too short to be worth one.
int qe_attention_prefill_uncut_keys() { return QE_PREFILL_UNCUT_KEYS; }

int qe_attention_prefill_segments(long blocks) {
    const int units = qe_compute_units();
    if (blocks <= 0 || blocks > units / 2) return 1;
    const long ks = units / blocks;                        // as many blocks as there are compute units, not more
    return ks > 8 ? 8 : (int)ks;
}

int qe_attention_prefill_segment_keys(long blocks, int max_keys) {
    const int ks = qe_attention_prefill_segments(blocks);
    const int seg = prefill_segment_length(max_keys, ks);
    return seg >= max_keys ? 0 : seg;
}

size_t qe_attention_prefill_workspace(int num_tiles, int Hq, int Hkv, int D, int segments) {
    const int R = qe_attention_prefill_tile_rows(Hq, Hkv);
    const long blocks = (long)(num_tiles / 4) * Hkv * ((Hq / Hkv) / (32 / R));
    return (size_t)segments * blocks * 4 * (2 + (D / 32) * 16) * 64 * sizeof(float);
}

// tiles: num_tiles pairs (first row of q, number of rows <= qe_attention_prefill_tile_rows), in
// groups of four that belong to one request, in ascending rows, with consecutive positions
// through the group; a group is filled up with pairs of 0 rows.  num_tiles is a multiple of 4.
// seg_keys: 0; or the keys of a segment (a multiple of 64) with max_keys, the most keys a row sees; or,
// for a caller that does not know the positions, minus the number of segments (at most 8) into which
// the keys of row keys_row, which sees the most, are to be cut.  The workspace has
// qe_attention_prefill_workspace(..., segments) bytes.
int qe_attention_prefill(const void* q, void* out, const void* cache, const int* tiles, int num_tiles,
                         const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                         int Hq, int Hkv, int D, int P, float scale, int window, int groups,
                         int seg_keys, int max_keys, int keys_row, void* workspace, size_t workspace_bytes,
                         hipStream_t stream) {
    QE_REQUIRE((D == 64 || D == 128) && P >= 16 && (P & (P - 1)) == 0 && Hq % Hkv == 0,
               "prefill attention: sizes not taken");
    int log2P = 0;
    while ((1 << log2P) < P) ++log2P;
    QE_REQUIRE(num_tiles % 4 == 0, "prefill attention: tiles come in groups of four");
    QE_REQUIRE(4L * Hkv * P * D < (1L << 31), "prefill attention: a page of %ld bytes is too large", 4L * Hkv * P * D);
    if (num_tiles == 0) return 0;
    const int R = qe_attention_prefill_tile_rows(Hq, Hkv);
    const int waves_per_kv = (Hq / Hkv) / (32 / R);
    int segments = 1;
    if (seg_keys > 0) {
        QE_REQUIRE(seg_keys % 64 == 0 && max_keys > 0, "prefill attention: segments of %d keys (a multiple of 64), %d keys", seg_keys, max_keys);
        segments = qe_cdiv(max_keys, seg_keys);
        QE_REQUIRE(segments <= 64, "prefill attention: %d segments", segments);
        if (segments <= 1) { seg_keys = 0; segments = 1; }
    } else if (seg_keys < 0) {
        segments = -seg_keys;
        QE_REQUIRE(segments <= 8 && keys_row >= 0, "prefill attention: %d segments of the keys of row %d", segments, keys_row);
        if (segments == 1) seg_keys = 0;
    }
    if (segments > 1)
        QE_REQUIRE(workspace && workspace_bytes >= qe_attention_prefill_workspace(num_tiles, Hq, Hkv, D, segments),
                   "prefill attention: workspace of %zu bytes is too small", workspace_bytes);
    QE_REQUIRE(num_tiles / 4 <= 65535, "prefill attention: %d tiles are too many for one launch", num_tiles);
    dim3 grid(Hkv * waves_per_kv, segments, num_tiles / 4);
    dim3 mgrid(Hkv * waves_per_kv, D / 32, num_tiles / 4);
    const float scale_log2 = scale * 1.4426950408889634f;
    // two groups a block where the blocks do not fill the compute units twice anyway
    // (groups: 0 = choose, 1 or 2)
    if (groups == 0) groups = (long)grid.x * grid.z <= qe_compute_units() ? 2 : 1;
    QE_REQUIRE(groups == 1 || groups == 2, "prefill attention: %d groups a block", groups);
#define QE_PREFILL(D_, NG_)                                                                         \
    attention_prefill_kernel<D_, NG_><<<grid, 256 * NG_, 0, stream>>>(                              \
        (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, tiles, positions, tok_seq, block_table, \
        max_blocks, Hq, Hkv, P, log2P, scale_log2, window, R, seg_keys, keys_row, (float*)workspace)
    if (D == 128) { if (groups == 2) QE_PREFILL(128, 2); else QE_PREFILL(128, 1); }
    else          { if (groups == 2) QE_PREFILL(64, 2); else QE_PREFILL(64, 1); }
#undef QE_PREFILL
    if (seg_keys != 0) {
        if (D == 128)
            attention_prefill_merge_kernel<128><<<mgrid, 256, 0, stream>>>((const float*)workspace, (bf16_t*)out, tiles,
                                                                           positions, Hq, Hkv, window, R, seg_keys, keys_row);
        else
            attention_prefill_merge_kernel<64><<<mgrid, 256, 0, stream>>>((const float*)workspace, (bf16_t*)out, tiles,
                                                                          positions, Hq, Hkv, window, R, seg_keys, keys_row);
    }
    QE_LAUNCH_CHECK();
    return 0;
}
