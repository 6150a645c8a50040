// Attention of portions of prompts over the paged cache (prefill), bfloat16, on the MFMA units
// with 32 x 32 tiles.
//
// A wave owns 32 columns: R consecutive query rows of a request for each of GH = 32 / R query
// heads that share one key/value head (GH = the group size when that is a power of two up to 32,
// else 1), so one pass over the keys serves the whole group.  It walks the keys its rows see,
// 32 at a time, straight from the cache pages (keys written by this same step included):
//   S^T[key, col] = K[key, :] . Q[col, :]         v_mfma_f32_32x32x16_bf16, D / 16 of them;
//       lane (g, r), g = lane / 32, r = lane % 32, loads K[key r][ks * 16 + g * 8 .. + 8] (16 bytes)
//       and ends up with 16 scores: keys 8 b + 4 g + j (b, j < 4) of column r
//   online softmax per column in 32-bit, in the base-2 domain (scores are scaled by
//       scale * log2 e once); the accumulator is rescaled only when a maximum moved
//   O^T[d, col] += V^T[d, key] . P^T[key, col]    v_mfma_f32_32x32x16_bf16, 2 * D / 32 of them;
//       the 8 probabilities of a half tile that a lane holds are its B operand as they lie, and
//       because value tiles are stored transposed ([D][P]) the A operand is two 8-byte loads
// No shared memory; one shuffle per tile.  The causal and window limits are applied per
// column, so the order of the sums for a row depends on its position and the window only.
// A block holds four neighbouring row tiles, so that their key tiles meet in the CU's cache.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float floatx16;

union PackV {   // two 8-byte pieces of a value row as one MFMA operand
    bf16x8 v;
    bf16x4 h[2];
    uint2 u[2];
};

template <int D>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ tiles, int num_tiles,
    const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks,
    int Hq, int Hkv, int P, float scale_log2, int window, int R) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 5, r = lane & 31;
    const int ti = blockIdx.x * 4 + wave;
    if (ti >= num_tiles) return;
    const int G = Hq / Hkv;
    const int GH = 32 / R;                                 // heads per wave
    const int kvh = blockIdx.y / (G / GH);
    const int head = kvh * G + (blockIdx.y % (G / GH)) * GH + r / R;   // this lane's column: head and row
    const int row0 = tiles[2 * ti], cnt = tiles[2 * ti + 1];
    const int rr = r % R;
    const bool col_ok = rr < cnt;
    const int row = row0 + (col_ok ? rr : cnt - 1);        // columns beyond the tile repeat its last row
    const int p = positions[row];
    const int hi = p + 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int p_first = positions[row0];
    const int k_start = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int k_stop = p_first + cnt;                      // positions of a tile's rows are consecutive
    const int* bt = block_table + (long)tok_seq[row0] * max_blocks;
    const long page_stride = 2L * Hkv * P * D;

    bf16x8 qreg[D / 16];
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
        qreg[ks] = *(const bf16x8*)(q + ((long)row * Hq + head) * D + ks * 16 + g * 8);

    float m = -INFINITY, l = 0.f;
    floatx16 acc[D / 32];
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;

    // what a lane adds to a page's base to reach its piece of a key tile and of a value tile
    const long k_lane = ((long)kvh * P + (r & 15)) * D + g * 8;
    const long v_lane = ((long)(Hkv + kvh) * P) * D + (long)r * P + 4 * g;
    const long v_step = 32L * P;                          // from one block of 32 value rows to the next
    // keys every column sees without a limit: [all_lo, all_hi); a tile inside needs no masks
    const int p_last = p_first + cnt - 1;
    const int all_hi = p_first + 1;
    const int all_lo = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;

    // A 32-key tile has two halves of 16 keys with pages and offsets of their own.  A half that no
    // row sees (beyond the request's keys, or wholly behind the window, where the page may have
    // been given back) reads the other half's memory again and is masked out.
#define TILE_ADDR(kk_)                                                                              \
    const bool first_ = (kk_) + 16 > k_start, second_ = (kk_) + 16 < k_stop;                        \
    const int ka_ = first_ ? (kk_) : (kk_) + 16;                                                    \
    const int kb_ = second_ ? (kk_) + 16 : (kk_);                                                   \
    const long base_a = (long)bt[ka_ / P] * page_stride + (long)(ka_ % P) * D;                      \
    const long base_b = (long)bt[kb_ / P] * page_stride + (long)(kb_ % P) * D;                      \
    const long vbase_a = (long)bt[ka_ / P] * page_stride + (ka_ % P);                               \
    const long vbase_b = (long)bt[kb_ / P] * page_stride + (kb_ % P);
#define LOAD_K()                                                                                    \
    {                                                                                               \
        const bf16_t* kp = cache + ((r < 16) ? base_a : base_b) + k_lane;                           \
        _Pragma("unroll") for (int ks = 0; ks < D / 16; ++ks) kreg[ks] = *(const bf16x8*)(kp + ks * 16); \
    }

    bf16x8 kreg[D / 16];
    const int kk0 = (k_start / 32) * 32;
    {
        TILE_ADDR(kk0)
        LOAD_K()
        (void)vbase_a; (void)vbase_b;
    }
    for (int kk = kk0; kk < k_stop; kk += 32) {
        PackV vreg[D / 32][2];
        {
            TILE_ADDR(kk)
            const bf16_t* va = cache + vbase_a + v_lane;
            const bf16_t* vb = cache + vbase_b + v_lane;
            (void)base_a; (void)base_b;
#pragma unroll
            for (int db = 0; db < D / 32; ++db) {
                vreg[db][0].u[0] = *(const uint2*)(va + db * v_step);
                vreg[db][0].u[1] = *(const uint2*)(va + db * v_step + 8);
                vreg[db][1].u[0] = *(const uint2*)(vb + db * v_step);
                vreg[db][1].u[1] = *(const uint2*)(vb + db * v_step + 8);
            }
        }
        floatx16 s;
#pragma unroll
        for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks)
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kreg[ks], qreg[ks], s, 0, 0, 0);
        if (kk + 32 < k_stop) {   // the next tile's keys travel while this tile's softmax and values are computed
            TILE_ADDR(kk + 32)
            LOAD_K()
            (void)vbase_a; (void)vbase_b;
        }

        float tmax = -INFINITY;
        if (kk >= all_lo && kk + 32 <= all_hi) {           // every column sees every key of the tile
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                s[e] *= scale_log2;
                tmax = fmaxf(tmax, s[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int key = kk + 8 * (e >> 2) + 4 * g + (e & 3);
                s[e] = (key >= lo && key < hi) ? s[e] * scale_log2 : -INFINITY;
                tmax = fmaxf(tmax, s[e]);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float mn = fmaxf(m, tmax);
        const float ref = (mn == -INFINITY) ? 0.f : mn;    // a column that has seen no key yet: all weights 0
        if (__any(mn > m)) {                               // some column's maximum moved: rescale
            const float alpha = __builtin_amdgcn_exp2f(m - ref);
            l *= alpha;
#pragma unroll
            for (int db = 0; db < D / 32; ++db) acc[db] *= alpha;
        }
        m = mn;
        PackV pb[2];
        float psum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float pe = __builtin_amdgcn_exp2f(s[e] - ref);   // 0 for keys that are not seen
            psum += pe;
            pb[e >> 3].v[e & 7] = (__bf16)pe;
        }
        l += psum;
        if (kk + 32 > k_stop || kk < k_start) {
            // the tile reaches beyond what any row sees: such keys may be unwritten memory, and
            // anything times a weight of 0 must still be 0
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int key = kk + 16 * h + 8 * (e >> 2) + 4 * g + (e & 3);
                        if (key < k_start || key >= k_stop) vreg[db][h].v[e] = (__bf16)0.f;
                    }
        }
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vreg[db][h].v, pb[h].v, acc[db], 0, 0, 0);
    }
#undef TILE_ADDR
#undef LOAD_K
    l += __shfl_xor(l, 32, 64);
    if (col_ok) {
        const float inv = 1.f / l;
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
}

// Rows per tile for a model's head counts: 32 / (heads that one wave serves).
int qe_attention_prefill_tile_rows(int Hq, int Hkv) {
    const int G = Hq / Hkv;
    const bool pow2 = G > 0 && (G & (G - 1)) == 0 && G <= 32;
    return 32 / (pow2 ? G : 1);
}

// tiles: num_tiles pairs (first row of q, number of rows <= qe_attention_prefill_tile_rows);
// a tile's rows belong to one request and have consecutive positions.
int qe_attention_prefill(const void* q, void* out, const void* cache, const int* tiles, int num_tiles,
                         const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                         int Hq, int Hkv, int D, int P, float scale, int window, hipStream_t stream) {
    QE_REQUIRE((D == 64 || D == 128) && P % 16 == 0 && Hq % Hkv == 0, "prefill attention: sizes not taken");
    if (num_tiles == 0) return 0;
    const int R = qe_attention_prefill_tile_rows(Hq, Hkv);
    const int waves_per_kv = (Hq / Hkv) / (32 / R);
    QE_REQUIRE(Hkv * waves_per_kv <= 65535, "prefill attention: too many heads");
    dim3 grid(qe_cdiv(num_tiles, 4), Hkv * waves_per_kv);
    const float scale_log2 = scale * 1.4426950408889634f;
    if (D == 128)
        attention_prefill_kernel<128><<<grid, 256, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache,
                                                                tiles, num_tiles, positions, tok_seq, block_table,
                                                                max_blocks, Hq, Hkv, P, scale_log2, window, R);
    else
        attention_prefill_kernel<64><<<grid, 256, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache,
                                                               tiles, num_tiles, positions, tok_seq, block_table,
                                                               max_blocks, Hq, Hkv, P, scale_log2, window, R);
    QE_LAUNCH_CHECK();
    return 0;
}
