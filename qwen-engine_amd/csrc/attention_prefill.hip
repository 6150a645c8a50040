// Attention of portions of prompts over the paged cache (prefill), bfloat16, on the MFMA units.
//
// The new tokens of a request are cut into tiles of up to 16 consecutive query rows.  A wave
// takes one tile and one query head: its 16 columns (see attention_tile.h) are the tile's rows,
// and it walks the keys of the request from the first one its first row sees to the last one
// its last row sees, 16 at a time, straight from the cache pages (keys written by this same
// step included), with the causal and the window limits applied per column.  A block holds
// four neighbouring tiles of the same head, so that their key tiles meet in the cache of the CU.
// The order of the sums for a row depends on its position and the window only.
#include "attention_tile.h"

template <int D>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ cache,
    const int* __restrict__ tiles, int num_tiles,
    const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks,
    int Hq, int Hkv, int P, float scale, int window) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, n = lane & 15;
    const int ti = blockIdx.x * 4 + wave;
    if (ti >= num_tiles) return;
    const int head = blockIdx.y;
    const int kvh = head / (Hq / Hkv);
    const int row0 = tiles[2 * ti], cnt = tiles[2 * ti + 1];
    const int row = row0 + (n < cnt ? n : cnt - 1);       // columns beyond the tile repeat its last row
    const int p = positions[row];
    const int hi = p + 1;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int p_first = positions[row0];
    const int k_start = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int k_stop = p_first + cnt;                      // positions of a tile's rows are consecutive
    const int* bt = block_table + (long)tok_seq[row0] * max_blocks;
    const long page_stride = 2L * Hkv * P * D;

    bf16x8 qreg[D / 32];
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
        qreg[c] = *(const bf16x8*)(q + ((long)row * Hq + head) * D + c * 32 + g * 8);

    AttnState<D> st;
    st.init();
    KVTile<D> cur, nxt;
    int kk = (k_start / 16) * 16;
    load_tile<D>(cur, cache, bt[kk / P], page_stride, kvh, Hkv, P, kk % P, g, n);
    for (; kk < k_stop; kk += 16) {
        const int kn = kk + 16;
        if (kn < k_stop) load_tile<D>(nxt, cache, bt[kn / P], page_stride, kvh, Hkv, P, kn % P, g, n);
        attn_tile_step<D>(st, cur, qreg, scale, kk, g, lo, hi, k_start, k_stop);
        cur = nxt;
    }
    float l = st.l;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (n < cnt) {
        const float inv = 1.f / l;
        bf16_t* orow = out + ((long)row * Hq + head) * D + g * 4;
#pragma unroll
        for (int db = 0; db < D / 16; ++db) {
            short4_t o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = bf16_bits(st.acc[db][j] * inv);
            *(short4_t*)(orow + db * 16) = o;
        }
    }
}

// tiles: num_tiles pairs (first row of q, number of rows <= 16); a tile's rows belong to one
// request and have consecutive positions.
int qe_attention_prefill(const void* q, void* out, const void* cache, const int* tiles, int num_tiles,
                         const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                         int Hq, int Hkv, int D, int P, float scale, int window, hipStream_t stream) {
    QE_REQUIRE((D == 64 || D == 128) && P % 16 == 0 && Hq % Hkv == 0, "prefill attention: sizes not taken");
    QE_REQUIRE(Hq <= 65535, "prefill attention: too many heads");
    if (num_tiles == 0) return 0;
    dim3 grid(qe_cdiv(num_tiles, 4), Hq);
    if (D == 128)
        attention_prefill_kernel<128><<<grid, 256, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache,
                                                                tiles, num_tiles, positions, tok_seq, block_table,
                                                                max_blocks, Hq, Hkv, P, scale, window);
    else
        attention_prefill_kernel<64><<<grid, 256, 0, stream>>>((const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache,
                                                               tiles, num_tiles, positions, tok_seq, block_table,
                                                               max_blocks, Hq, Hkv, P, scale, window);
    QE_LAUNCH_CHECK();
    return 0;
}
