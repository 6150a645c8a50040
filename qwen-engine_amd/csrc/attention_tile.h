// The 16-key tile step shared by the MFMA attention kernels (bfloat16).
//
// A wave owns 16 columns (query heads of one token when decoding; consecutive query rows of one
// head when prefilling) against the keys of one key/value head.  For a tile of 16 keys:
//   S^T[key, col] = K[key, :] . Q[col, :]          v_mfma_f32_16x16x32_bf16, D / 32 of them;
//       lane (g, n), g = lane / 16, n = lane % 16, loads K[key n][c * 32 + g * 8 .. + 8] (16 bytes)
//       and ends up with the scores of keys g * 4 .. g * 4 + 3 for column n
//   online softmax per column in 32-bit (max over the lane's 4 keys and the 4 lanes of the column)
//   O^T[d, col] += V^T[d, key] . P^T[key, col]     v_mfma_f32_16x16x16_bf16, D / 16 of them;
//       the probabilities a lane holds are exactly its B operand, and because value tiles are
//       stored transposed ([D][P]) the A operand is one 8-byte load: V^T[d = db * 16 + n][keys g * 4 .. + 3]
// No shared memory and no shuffles apart from the two of the max.
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float floatx4;

__device__ __forceinline__ short bf16_bits(float f) { return (short)float_to_bf16(f).bits; }

// One tile of 16 keys in registers: the K rows as MFMA A operands, the V^T rows likewise.
template <int D>
struct KVTile {
    bf16x8 k[D / 32];
    short4_t v[D / 16];
};

// o: offset of the tile's first key inside its page (a multiple of 16)
// The loads are non-temporal: a decode step reads every key and value of the live requests once, far more
// than the caches hold, and a stream that is not kept goes faster (a wave with one tile in flight pulls 134 MB
// in 22.5 us where plain loads take 30.4; a decode step of 64 requests gains 4 %, one of 8 requests 1.3 %).
// Keys that other requests of the step read too (pages of a shared prefix) are asked for with plain loads
// (`stream` false, the same for the whole wave): the first request to read a line leaves it in the L2 for
// the others (32 requests with half of their 2300 keys shared: 48 us a layer against 55 with every load
// non-temporal).
template <int D>
__device__ __forceinline__ void load_tile(KVTile<D>& tile, const bf16_t* __restrict__ cache, long page,
                                          long page_stride, int kvh, int Hkv, int P, int o, int g, int n,
                                          bool stream) {
    const bf16_t* kbase = cache + page * page_stride + ((long)kvh * P + o) * D + (long)n * D + g * 8;
    const bf16_t* vbase = cache + page * page_stride + ((long)(Hkv + kvh) * P) * D + o + (long)n * P + g * 4;
    if (stream) {
#pragma unroll
        for (int c = 0; c < D / 32; ++c) tile.k[c] = __builtin_nontemporal_load((const bf16x8*)(kbase + c * 32));
#pragma unroll
        for (int db = 0; db < D / 16; ++db)
            tile.v[db] = __builtin_nontemporal_load((const short4_t*)(vbase + (long)db * 16 * P));
    } else {
#pragma unroll
        for (int c = 0; c < D / 32; ++c) tile.k[c] = *(const bf16x8*)(kbase + c * 32);
#pragma unroll
        for (int db = 0; db < D / 16; ++db) tile.v[db] = *(const short4_t*)(vbase + (long)db * 16 * P);
    }
}

// The largest of the four lanes n, n + 16, n + 32, n + 48 (the four rows of 16 lanes), in all of them:
// two swaps between vector registers (rows 1, 3 against rows 0, 2, then the halves of the wave)
// where `__shfl_xor` would go twice through the LDS crossbar, once per tile of every wave.
__device__ __forceinline__ float max_over_lane_rows(float v) {
    float a, b;
    pair_across_rows(v, a, b);
    v = fmaxf(a, b);
    pair_across_halves(v, a, b);
    return fmaxf(a, b);
}

template <int D>
struct AttnState {
    float m, l;              // running max and (this lane's share of the) running sum of column n
    floatx4 acc[D / 16];     // O^T rows d = db * 16 + g * 4 + j of column n
    __device__ __forceinline__ void init() {
        m = -INFINITY;
        l = 0.f;
#pragma unroll
        for (int db = 0; db < D / 16; ++db) acc[db] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
};

// The tile's keys are kk .. kk + 15; this lane's column sees the keys in [lo, hi); [vlo, vhi) is
// the range that any column of the wave sees (keys outside it may be unwritten memory).
template <int D>
__device__ __forceinline__ void attn_tile_step(AttnState<D>& st, const KVTile<D>& tile, const bf16x8 (&qreg)[D / 32],
                                               float scale, int kk, int g, int lo, int hi, int vlo, int vhi) {
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < D / 32; ++c) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tile.k[c], qreg[c], s, 0, 0, 0);
    float tmax = -INFINITY;
    bool ok[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int key = kk + g * 4 + j;
        ok[j] = key >= lo && key < hi;
        s[j] = ok[j] ? s[j] * scale : -INFINITY;
        tmax = fmaxf(tmax, s[j]);
    }
    tmax = max_over_lane_rows(tmax);
    const float mn = fmaxf(st.m, tmax);
    const float ref = (mn == -INFINITY) ? 0.f : mn;   // a column that has seen no key yet: all weights 0
    const float alpha = __expf(st.m - ref);
    short4_t pb;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float pj = __expf(s[j] - ref);           // 0 for keys that are not seen
        psum += pj;
        pb[j] = bf16_bits(pj);
    }
    st.l = st.l * alpha + psum;
    st.m = mn;
    // The value rows a lane holds serve every column, so they are masked by the wave's range only
    // (a key outside it may be an unwritten part of a page: anything, times a weight of 0);
    // what a single column does not see has weight 0 already.
    short4_t vmask;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int key = kk + g * 4 + j;
        vmask[j] = (short)((key >= vlo && key < vhi) ? -1 : 0);
    }
#pragma unroll
    for (int db = 0; db < D / 16; ++db) {
        st.acc[db] *= alpha;
        st.acc[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(tile.v[db] & vmask, pb, st.acc[db], 0, 0, 0);
    }
}
