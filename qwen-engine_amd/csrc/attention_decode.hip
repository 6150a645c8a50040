// Attention of single new tokens over the paged cache (decode), bfloat16, split over the keys
// ("flash decoding"), on the MFMA units.  All query heads of a key/value group are the columns
// of one wave (see attention_tile.h), so the cache is read from HBM once; this kernel is bound
// by that read.  Heads beyond the group size (lanes n >= G) compute on zeros and are not stored.
//
// One wave per (split of the keys, key/value head, token).  The splits are cut at absolute key
// positions (multiples of SPLIT), so a token's result does not depend on what else is in the
// batch.  A second kernel merges the splits.
#include "attention_tile.h"

// SPLIT: keys per split (a multiple of 16, at most 64 tiles).  The next tile is loaded while the
// current one is computed, and the split's page ids are read before the loop.
// (Merging the splits in this same kernel, by the wave that finishes last, was tried: the
// device-wide fences it needs cost several times what the separate merge kernel costs.)
template <int D, int SPLIT>
__global__ __launch_bounds__(64) void attention_decode_split_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache,
    const int* __restrict__ dec_tokens, const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ shared_keys,
    float* __restrict__ part_acc, float* __restrict__ part_ml,
    int Hq, int Hkv, int P, float scale, int window, int num_splits) {
    constexpr int TILES = SPLIT / 16;
    const int lane = threadIdx.x, g = lane >> 4, n = lane & 15;
    const int split = blockIdx.x, kvh = blockIdx.y, di = blockIdx.z;
    const int G = Hq / Hkv;
    const int t = dec_tokens ? dec_tokens[di] : di;       // (no list: every row, in order)
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int k_begin = max(split * SPLIT, lo);
    const int k_end = min((split + 1) * SPLIT, p + 1);
    const int head = kvh * G + n;
    const bool head_ok = n < G;
    float* pacc = part_acc + (((long)di * Hq + head) * num_splits + split) * D;
    float* pml = part_ml + (((long)di * Hq + head) * num_splits + split) * 2;
    if (k_begin >= k_end) {   // nothing of this split is seen by the token
        if (head_ok && g == 0) { pml[0] = -INFINITY; pml[1] = 0.f; }
        return;
    }
    const int row = tok_seq[t];
    const int* bt = block_table + (long)row * max_blocks;
    // (keys that other requests read too are left in the caches, the others stream: see load_tile)
    const bool stream = !(shared_keys && split * SPLIT < shared_keys[row]);
    const long page_stride = 2L * Hkv * P * D;
    const int tile0 = (k_begin - split * SPLIT) / 16;                 // first and one-past-last tile of the split
    const int tile1 = (k_end - split * SPLIT + 15) / 16;
    // lane i holds the page of tile i (one vector load for the whole split); a tile's page is
    // then read from that lane
    int my_page = 0;
    if (lane >= tile0 && lane < tile1) my_page = bt[(split * SPLIT + lane * 16) / P];

    bf16x8 qreg[D / 32];
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
        qreg[c] = head_ok ? *(const bf16x8*)(q + ((long)t * Hq + head) * D + c * 32 + g * 8) : zero8;

    AttnState<D> st;
    st.init();

    // Two tile buffers used in turn: the loads of the next tile are issued before the current
    // one is computed, and nothing is copied from one buffer to the other.
#define LOAD(buf_, i_) load_tile<D>(buf_, cache, __builtin_amdgcn_readlane(my_page, (i_)), page_stride, kvh, Hkv, P, \
                                    (split * SPLIT + (i_) * 16) % P, g, n, stream)
#define STEP(buf_, i_) attn_tile_step<D>(st, buf_, qreg, scale, split * SPLIT + (i_) * 16, g, k_begin, k_end, k_begin, k_end)
    KVTile<D> ta, tb;
    int i = tile0;
    LOAD(ta, i);
    while (true) {
        if (i + 1 < tile1) LOAD(tb, i + 1);
        STEP(ta, i);
        if (++i >= tile1) break;
        if (i + 1 < tile1) LOAD(ta, i + 1);
        STEP(tb, i);
        if (++i >= tile1) break;
    }
#undef LOAD
#undef STEP
    float l = st.l;
    const float m = st.m;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (head_ok) {
#pragma unroll
        for (int db = 0; db < D / 16; ++db)
            *(floatx4*)(pacc + db * 16 + g * 4) = st.acc[db];    // O^T rows d = db * 16 + g * 4 + j of column head n
        if (g == 0) { pml[0] = m; pml[1] = l; }
    }
}

// ---- the same with the step before it folded in ---------------------------------------------
// (Folding the output projection into the merge kernel, a block per head and 128 output features
// that merges the head's splits for all tokens and multiplies with its part of W_o, was tried for
// few tokens: it takes as long as the two kernels it replaces.)
//
// The q/k norm, the rotation and the cache write of the new token cost a kernel of their own
// that runs a few microseconds for a few kilobytes.  Here every wave norms and rotates the query
// heads it needs itself, straight from the q|k|v rows (the pairs d, d + D/2 of the rotation lie in
// the same lane in the MFMA operand layout), and the wave whose split holds the token's own
// position also norms and rotates the new key, takes it and the new value into its softmax from
// registers (the cached keys it reads stop before that position), and writes both to the cache.
// Roundings are where the separate kernels have them: q and k to bfloat16 after the rotation,
// the probability to bfloat16 before it meets the value.

// One head's features c * 32 + g * 8 + e in the MFMA operand layout: fetch() issues the loads (the
// head, the norm's weights, the position's row [cos | sin] of the table), finish() does the
// RMSNorm (w) and the rotation (cs), each optional, and rounds to bfloat16.  Apart, so that the
// loads of the first key tiles can be issued between the two.
template <int D>
struct NormRotate {
    static constexpr int H = D / 64;                       // chunk c and chunk c + H rotate together
    bf16x8 raw[D / 32];
    float wv[D / 32][8], co[H][8], sn[H][8];
    __device__ __forceinline__ void fetch(const bf16_t* __restrict__ src, bool active, const float* __restrict__ w,
                                          const float* __restrict__ cs, int g) {
#pragma unroll
        for (int c = 0; c < D / 32; ++c) {
            raw[c] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (active) raw[c] = *(const bf16x8*)(src + c * 32 + g * 8);
        }
        if (w) {
#pragma unroll
            for (int c = 0; c < D / 32; ++c) {
                Vec4<float>::load(w + c * 32 + g * 8, *(float(*)[4])wv[c]);
                Vec4<float>::load(w + c * 32 + g * 8 + 4, *(float(*)[4])(wv[c] + 4));
            }
        }
        if (cs) {
#pragma unroll
            for (int c = 0; c < H; ++c) {
                Vec4<float>::load(cs + c * 32 + g * 8, *(float(*)[4])co[c]);
                Vec4<float>::load(cs + c * 32 + g * 8 + 4, *(float(*)[4])(co[c] + 4));
                Vec4<float>::load(cs + D / 2 + c * 32 + g * 8, *(float(*)[4])sn[c]);
                Vec4<float>::load(cs + D / 2 + c * 32 + g * 8 + 4, *(float(*)[4])(sn[c] + 4));
            }
        }
    }
    __device__ __forceinline__ void finish(bf16x8 (&out)[D / 32], bool has_w, float eps, bool has_cs) {
        float x[D / 32][8];
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) x[c][e] = (float)raw[c][e];
        if (has_w) {
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < D / 32; ++c)
#pragma unroll
                for (int e = 0; e < 8; ++e) ss += x[c][e] * x[c][e];
            ss += __shfl_xor(ss, 16, 64);
            ss += __shfl_xor(ss, 32, 64);
            const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
            for (int c = 0; c < D / 32; ++c)
#pragma unroll
                for (int e = 0; e < 8; ++e) x[c][e] = x[c][e] * rstd * wv[c][e];
        }
        if (has_cs) {
#pragma unroll
            for (int c = 0; c < H; ++c)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float x1 = x[c][e], x2 = x[c + H][e];
                    x[c][e] = co[c][e] * x1 - sn[c][e] * x2;
                    x[c + H][e] = sn[c][e] * x1 + co[c][e] * x2;
                }
        }
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) out[c][e] = (__bf16)x[c][e];
    }
};

// AHEAD: how many tiles the loads of a whole split run ahead of the computation.  A wave with one
// tile in flight gets 8 KB per trip to memory (about 0.7 us); that is enough when the chip holds
// two waves or more per SIMD, whose loads together keep the memory busy, and far too little for one
// token's 256 waves.  With 3 the code of a whole split is straight-line (waits are then exact) and
// takes 64 registers more, which with many waves costs more than it brings.  The order of the
// arithmetic is the same either way.
template <int D, int SPLIT, int AHEAD>
__global__ __launch_bounds__(64) void attention_decode_fused_split_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* cache,
    const int* __restrict__ dec_tokens, const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ shared_keys,
    const int* __restrict__ slots, const float* __restrict__ q_w, const float* __restrict__ k_w, float eps, const float* __restrict__ table,
    float* __restrict__ part_acc, float* __restrict__ part_ml,
    int Hq, int Hkv, int P, float scale, int window, int num_splits) {
    constexpr int TILES = SPLIT / 16;
    const int lane = threadIdx.x, g = lane >> 4, n = lane & 15;
    const int split = blockIdx.x, kvh = blockIdx.y, di = blockIdx.z;
    const int G = Hq / Hkv;
    const int t = dec_tokens ? dec_tokens[di] : di;       // (no list: every row, in order)
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const bool own = split == p / SPLIT;                   // this wave takes the token's own key and value
    const int k_begin = max(split * SPLIT, lo);
    const int k_end = min((split + 1) * SPLIT, p);         // cached keys: the token's own is not among them
    const int head = kvh * G + n;
    const bool head_ok = n < G;
    float* pacc = part_acc + (((long)di * Hq + head) * num_splits + split) * D;
    float* pml = part_ml + (((long)di * Hq + head) * num_splits + split) * 2;
    if (k_begin >= k_end && !own) {   // nothing of this split is seen by the token
        if (head_ok && g == 0) { pml[0] = -INFINITY; pml[1] = 0.f; }
        return;
    }
    const long width = (long)(Hq + 2 * Hkv) * D;
    const float* cs = table ? table + (long)p * D : nullptr;
    const long page_stride = 2L * Hkv * P * D;

    AttnState<D> st;
    st.init();
    bf16x8 qreg[D / 32];
    if (k_begin < k_end) {
        const int row = tok_seq[t];
        const int* bt = block_table + (long)row * max_blocks;
        const bool stream = !(shared_keys && split * SPLIT < shared_keys[row]);
        const int tile0 = (k_begin - split * SPLIT) / 16;
        const int tile1 = (k_end - split * SPLIT + 15) / 16;
        int my_page = 0;
        if (lane >= tile0 && lane < tile1) my_page = bt[(split * SPLIT + lane * 16) / P];
#define LOAD(buf_, i_) load_tile<D>(buf_, cache, __builtin_amdgcn_readlane(my_page, (i_)), page_stride, kvh, Hkv, P, \
                                    (split * SPLIT + (i_) * 16) % P, g, n, stream)
#define STEP(buf_, i_) attn_tile_step<D>(st, buf_, qreg, scale, split * SPLIT + (i_) * 16, g, k_begin, k_end, k_begin, k_end)
        NormRotate<D> nq;
        nq.fetch(qkv + t * width + (long)head * D, head_ok, q_w, cs, g);
        if (AHEAD > 1 && tile0 == 0 && tile1 == TILES) {
            KVTile<D> tl[AHEAD + 1];
#pragma unroll
            for (int j = 0; j < AHEAD; ++j) LOAD(tl[j], j);   // the first tiles travel while q is prepared
            nq.finish(qreg, q_w != nullptr, eps, cs != nullptr);
#pragma unroll
            for (int j = 0; j < TILES; ++j) {
                if (j + AHEAD < TILES) LOAD(tl[(j + AHEAD) % (AHEAD + 1)], j + AHEAD);
                __builtin_amdgcn_sched_barrier(0);         // (the scheduler would move the loads down to their uses)
                STEP(tl[j % (AHEAD + 1)], j);
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            KVTile<D> ta, tb;
            int i = tile0;
            LOAD(ta, i);                                   // the first tiles travel while q is prepared
            if (i + 1 < tile1) LOAD(tb, i + 1);
            nq.finish(qreg, q_w != nullptr, eps, cs != nullptr);
            while (true) {
                STEP(ta, i);
                if (++i >= tile1) break;
                if (i + 1 < tile1) LOAD(ta, i + 1);
                STEP(tb, i);
                if (++i >= tile1) break;
                if (i + 1 < tile1) LOAD(tb, i + 1);
            }
        }
#undef LOAD
#undef STEP
    } else {
        NormRotate<D> nq;
        nq.fetch(qkv + t * width + (long)head * D, head_ok, q_w, cs, g);
        nq.finish(qreg, q_w != nullptr, eps, cs != nullptr);
    }
    if (own) {
        bf16x8 kreg[D / 32];
        NormRotate<D> nk;
        nk.fetch(qkv + t * width + (long)(Hq + kvh) * D, true, k_w, cs, g);
        nk.finish(kreg, k_w != nullptr, eps, cs != nullptr);
        float dot = 0.f;
#pragma unroll
        for (int c = 0; c < D / 32; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) dot += (float)qreg[c][e] * (float)kreg[c][e];
        dot += __shfl_xor(dot, 16, 64);
        dot += __shfl_xor(dot, 32, 64);
        const float s_new = dot * scale;
        const float mn = fmaxf(st.m, s_new);
        const float alpha = __expf(st.m - mn);             // 0 when no cached key was seen
        const float pn = __expf(s_new - mn);
        const float pn_b = (float)(__bf16)pn;
        st.l = st.l * alpha + (g == 0 ? pn : 0.f);         // (a lane's share of the sum: once per column)
        st.m = mn;
        const bf16_t* vsrc = qkv + t * width + (long)(Hq + Hkv + kvh) * D;
#pragma unroll
        for (int db = 0; db < D / 16; ++db) {
            const short4_t vv = *(const short4_t*)(vsrc + db * 16 + g * 4);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                st.acc[db][j] = st.acc[db][j] * alpha + pn_b * bf16_bits_to_float((unsigned short)vv[j]);
        }
        const int slot = slots ? slots[t] : -1;
        if (slot >= 0) {
            const long page = slot / P;
            const int off = slot % P;
            if (n == 0) {
#pragma unroll
                for (int c = 0; c < D / 32; ++c)
                    *(bf16x8*)(cache + page * page_stride + ((long)kvh * P + off) * D + c * 32 + g * 8) = kreg[c];
            }
            if (n < D / 16) {                              // the value tile is [D][P]: a column of single elements
                bf16_t* vt = cache + page * page_stride + ((long)(Hkv + kvh) * P) * D + off;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int d = n * 16 + g * 4 + j;
                    vt[(long)d * P] = vsrc[d];
                }
            }
        }
    }
    float l = st.l;
    const float m = st.m;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (head_ok) {
#pragma unroll
        for (int db = 0; db < D / 16; ++db)
            *(floatx4*)(pacc + db * 16 + g * 4) = st.acc[db];
        if (g == 0) { pml[0] = m; pml[1] = l; }
    }
}

// out[t, head, :] = sum_s e^{m_s - M} acc_s / sum_s e^{m_s - M} l_s,  M = max_s m_s.
// One block of 256 threads per (token, head): wave w sums the splits w, w + 4, ... in ascending
// order, the four sums are added in the order of the waves.
template <int D>
__global__ __launch_bounds__(256) void attention_decode_merge_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, const int* __restrict__ dec_tokens,
    bf16_t* __restrict__ out, int Hq, int num_splits) {
    constexpr int PER = (D + 63) / 64;
    __shared__ float red_o[4][D];
    __shared__ float red_l[4];
    __shared__ float red_m[4];
    const int di = blockIdx.x, head = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* pml = part_ml + ((long)di * Hq + head) * num_splits * 2;
    const float* pacc = part_acc + ((long)di * Hq + head) * num_splits * D;
    // (the largest maximum is reduced only after the first eight splits' loads have been issued: its
    // own loads were issued before them, so waiting for those does not wait for these)
    float M = -INFINITY;
    for (int s = lane; s < num_splits; s += 64) M = fmaxf(M, pml[2 * s]);
    bool reduced = false;
    float denom = 0.f;
    float o[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) o[i] = 0.f;
    // eight of the wave's splits at a time: their maxima, sums and accumulator rows are all asked
    // for before the first is used (one trip to memory for eight); added in ascending order
    for (int s0 = wave; s0 < num_splits; s0 += 32) {
        float ms[8], ls[8], a[8][PER];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int s = s0 + 4 * k;
            ms[k] = s < num_splits ? pml[2 * s] : -INFINITY;
            ls[k] = s < num_splits ? pml[2 * s + 1] : 0.f;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int s = s0 + 4 * k;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const int d = lane + i * 64;
                // (asked for without waiting for the maxima: an empty split's accumulator was never
                // written, and what is read of it is not used below; a split beyond the last reads the last)
                a[k][i] = d < D ? pacc[(long)(s < num_splits ? s : num_splits - 1) * D + d] : 0.f;
            }
        }
        if (!reduced) { M = wave_max(M); reduced = true; }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            if (ms[k] == -INFINITY) continue;
            const float wgt = __expf(ms[k] - M);
            denom += wgt * ls[k];
#pragma unroll
            for (int i = 0; i < PER; ++i) o[i] += wgt * a[k][i];
        }
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int d = lane + i * 64;
        if (d < D) red_o[wave][d] = o[i];
    }
    if (lane == 0) red_l[wave] = denom;
    __syncthreads();
    if (wave == 0) {
        const float inv = 1.f / (red_l[0] + red_l[1] + red_l[2] + red_l[3]);
        bf16_t* orow = out + ((long)(dec_tokens ? dec_tokens[di] : di) * Hq + head) * D;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int d = lane + i * 64;
            if (d < D) orow[d] = float_to_bf16((red_o[0][d] + red_o[1][d] + red_o[2][d] + red_o[3][d]) * inv);
        }
    }
}

// also what the prefill kernel takes, but for the page size, which it wants to be a power of two
bool qe_attention_decode_ok(int Hq, int Hkv, int D, int P, int dt_a) {
    return dt_a == QE_BF16 && (D == 64 || D == 128) && P % 16 == 0 && Hq % Hkv == 0 && Hq / Hkv <= 16;
}

size_t qe_attention_decode_workspace(int n_dec, int Hq, int D, int num_splits) {
    return (size_t)n_dec * Hq * num_splits * (D + 2) * sizeof(float);
}

// dec_tokens: the rows of q that are single new tokens of their requests (null: the rows
// 0 .. n_dec - 1, which saves every wave a dependent load).  max_position: the
// largest of their positions (fixes the number of splits).  workspace: at least
// qe_attention_decode_workspace(...) bytes.  shared_keys: null, or for every row of the block table
// the number of the request's first keys that other requests of the step may read as well (pages they
// hold together): a hint for the caches, results do not depend on it.
int qe_attention_decode(const void* q, void* out, const void* cache, const int* dec_tokens, int n_dec,
                        const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                        const int* shared_keys, int Hq, int Hkv, int D, int P, float scale, int window, int max_position,
                        int split_keys, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    QE_REQUIRE(qe_attention_decode_ok(Hq, Hkv, D, P, QE_BF16), "decode attention: sizes not taken");
    QE_REQUIRE(split_keys == 128 || split_keys == 256, "decode attention: splits of 128 or 256 keys, not %d", split_keys);
    if (n_dec == 0) return 0;
    const int num_splits = max_position / split_keys + 1;
    QE_REQUIRE(num_splits <= 65535 && n_dec <= 65535, "decode attention: too many splits or tokens");
    QE_REQUIRE(workspace_bytes >= qe_attention_decode_workspace(n_dec, Hq, D, num_splits),
               "decode attention: workspace of %zu bytes is too small", workspace_bytes);
    float* part_acc = (float*)workspace;
    float* part_ml = part_acc + (size_t)n_dec * Hq * num_splits * D;
    (void)qe_cdiv;
    dim3 grid(num_splits, Hkv, n_dec);
    dim3 mgrid(n_dec, Hq);
#define QE_DECODE(D_, S_)                                                                               \
    do {                                                                                                \
        attention_decode_split_kernel<D_, S_><<<grid, 64, 0, stream>>>(                                 \
            (const bf16_t*)q, (const bf16_t*)cache, dec_tokens, positions, tok_seq, block_table,        \
            max_blocks, shared_keys, part_acc, part_ml, Hq, Hkv, P, scale, window, num_splits);         \
        attention_decode_merge_kernel<D_><<<mgrid, 256, 0, stream>>>(part_acc, part_ml, dec_tokens,     \
                                                                     (bf16_t*)out, Hq, num_splits);     \
    } while (0)
    if (D == 128 && split_keys == 128) QE_DECODE(128, 128);
    else if (D == 128) QE_DECODE(128, 256);
    else if (split_keys == 128) QE_DECODE(64, 128);
    else QE_DECODE(64, 256);
#undef QE_DECODE
    QE_LAUNCH_CHECK();
    return 0;
}

// The fused form: qkv [T, (Hq + 2 Hkv) D] as the projection left it; q_w, k_w (per-head norm weights)
// and table (rows [cos | sin] of D floats per position) may be null; slots: the cache slot of each
// row's own key and value (negative: not written).  Every row named in dec_tokens brings exactly
// its own new key; the cache holds the keys before it.
int qe_attention_decode_fused(const void* qkv, void* out, void* cache, const int* dec_tokens, int n_dec,
                              const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                              const int* shared_keys, const int* slots, const float* q_w, const float* k_w, float eps, const float* table,
                              int Hq, int Hkv, int D, int P, float scale, int window, int max_position,
                              int split_keys, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    QE_REQUIRE(qe_attention_decode_ok(Hq, Hkv, D, P, QE_BF16), "decode attention: sizes not taken");
    QE_REQUIRE(split_keys == 128 || split_keys == 256, "decode attention: splits of 128 or 256 keys, not %d", split_keys);
    if (n_dec == 0) return 0;
    const int num_splits = max_position / split_keys + 1;
    QE_REQUIRE(num_splits <= 65535 && n_dec <= 65535, "decode attention: too many splits or tokens");
    QE_REQUIRE(workspace_bytes >= qe_attention_decode_workspace(n_dec, Hq, D, num_splits),
               "decode attention: workspace of %zu bytes is too small", workspace_bytes);
    float* part_acc = (float*)workspace;
    float* part_ml = part_acc + (size_t)n_dec * Hq * num_splits * D;
    dim3 grid(num_splits, Hkv, n_dec);
    dim3 mgrid(n_dec, Hq);
    const bool few = (long)num_splits * Hkv * n_dec <= 1024;   // at most a wave per SIMD: loads further ahead
#define QE_DECODE_FUSED(D_, S_)                                                                         \
    do {                                                                                                \
        if (few)                                                                                        \
            attention_decode_fused_split_kernel<D_, S_, 3><<<grid, 64, 0, stream>>>(                    \
                (const bf16_t*)qkv, (bf16_t*)cache, dec_tokens, positions, tok_seq, block_table, max_blocks, \
                shared_keys, slots, q_w, k_w, eps, table, part_acc, part_ml, Hq, Hkv, P, scale, window, \
                num_splits);                                                                            \
        else                                                                                            \
        attention_decode_fused_split_kernel<D_, S_, 1><<<grid, 64, 0, stream>>>(                        \
            (const bf16_t*)qkv, (bf16_t*)cache, dec_tokens, positions, tok_seq, block_table, max_blocks, \
            shared_keys, slots, q_w, k_w, eps, table, part_acc, part_ml, Hq, Hkv, P, scale, window,     \
            num_splits);                                                                                \
        attention_decode_merge_kernel<D_><<<mgrid, 256, 0, stream>>>(part_acc, part_ml, dec_tokens,     \
                                                                     (bf16_t*)out, Hq, num_splits);     \
    } while (0)
    if (D == 128 && split_keys == 128) QE_DECODE_FUSED(128, 128);
    else if (D == 128) QE_DECODE_FUSED(128, 256);
    else if (split_keys == 128) QE_DECODE_FUSED(64, 128);
    else QE_DECODE_FUSED(64, 256);
#undef QE_DECODE_FUSED
    QE_LAUNCH_CHECK();
    return 0;
}
