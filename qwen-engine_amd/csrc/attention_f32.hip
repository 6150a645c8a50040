// Attention in 32-bit on the matrix units: the kernel of the float32 mode for head sizes in
// steps of 16.  Every product and sum is an IEEE 32-bit operation (v_mfma_f32_16x16x4_f32 takes
// 32-bit operands and accumulates in 32-bit; no reduced-precision matrix mode).
//
// One block of four waves per (token, key/value head, 16 query heads of its group): the heads are
// the 16 columns, so the keys and values of a key/value head are read once for all heads of the
// group.  The keys the token sees, lo .. p, are taken 16 at a time from absolute multiples of 16;
// wave w takes the tiles w, w + 4, ... and the four partial results are merged through shared
// memory in the order of the waves (a single new token over a long context would else be one
// wave's walk).  The order of the sums so depends on the position and the window only.  For a tile
// of 16 keys:
//   S^T[key, col] = K[key, :] . Q[col, :]       D / 4 MFMAs of 16 x 16 x 4;
//       lane (g, r), g = lane / 16, r = lane % 16, holds K[key r][16 c + 4 g .. + 4] of feature block
//       c as one 16-byte load, and its element j goes into the j-th MFMA of the block (which
//       feature stands at which place of the sum does not matter as long as Q has it at the same)
//   online softmax per column over the lanes (g, n) that share column n, in 32-bit
//   O^T[d, col] += V^T[d, key] . P^T[key, col]   4 MFMAs per 16 rows of d: the j-th takes, at place
//       g of its sum, key 4 g + j: that is the probability a lane already holds as its element j,
//       and of V^T the lane needs row d = 16 db + r at keys 4 g .. 4 g + 3
// Any page size: every lane looks its own keys' pages up.  Keys outside lo .. p are never read
// (their memory may be unwritten): they enter as zeros with a score of minus infinity.
#include "common.h"

typedef __attribute__((ext_vector_type(4))) float floatx4;

__device__ __forceinline__ float max_over_rows_of_lanes(float v) {
    float a, b;
    pair_across_rows(v, a, b);
    v = fmaxf(a, b);
    pair_across_halves(v, a, b);
    return fmaxf(a, b);
}

#define F32_WAVES 4

template <int DB>     // head size / 16
__global__ __launch_bounds__(64 * F32_WAVES) void attention_f32_kernel(
    const float* __restrict__ q, float* __restrict__ out, const float* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tokens,
    int Hq, int Hkv, int P, float scale, int window) {
    constexpr int D = DB * 16;
    extern __shared__ float merge_lds[];                  // [F32_WAVES][DB * 4 + 2][64]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, n = lane & 15;
    const long t = tokens ? tokens[blockIdx.x] : blockIdx.x;
    const int G = Hq / Hkv;
    const int groups16 = (G + 15) / 16;
    const int kvh = blockIdx.y / groups16, hg = blockIdx.y % groups16;
    const int head = kvh * G + hg * 16 + n;
    const bool head_ok = hg * 16 + n < G;
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int* bt = block_table + (long)tok_seq[t] * max_blocks;
    const long page_stride = 2L * Hkv * P * D;
    const bool vec_v = (P & 3) == 0;                      // four consecutive keys of a value row lie in one page, aligned

    floatx4 qv[DB];
#pragma unroll
    for (int c = 0; c < DB; ++c) {
        qv[c] = floatx4{0.f, 0.f, 0.f, 0.f};
        if (head_ok) qv[c] = *(const floatx4*)(q + (t * Hq + head) * D + c * 16 + g * 4);
    }
    float m = -INFINITY, l = 0.f;                         // l: this lane's share of the column's sum
    floatx4 acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int kk = (lo / 16) * 16 + 16 * wave; kk <= p; kk += 16 * F32_WAVES) {
        // S^T: this lane brings the key row kk + n
        const int key_r = kk + n;
        const bool row_ok = key_r >= lo && key_r <= p;
        floatx4 s = {0.f, 0.f, 0.f, 0.f};
        {
            const float* krow = cache;
            if (row_ok) krow = cache + (long)bt[key_r / P] * page_stride + ((long)kvh * P + key_r % P) * D + g * 4;
            floatx4 kf[DB];
#pragma unroll
            for (int c = 0; c < DB; ++c) kf[c] = row_ok ? *(const floatx4*)(krow + c * 16) : floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < DB; ++c)
#pragma unroll
                for (int j = 0; j < 4; ++j) s = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[c][j], qv[c][j], s, 0, 0, 0);
        }
        // the lane now holds the scores of keys kk + 4 g + i of column n
        float tmax = -INFINITY;
        bool ok[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kk + 4 * g + i;
            ok[i] = key >= lo && key <= p;
            s[i] = ok[i] ? s[i] * scale : -INFINITY;
            tmax = fmaxf(tmax, s[i]);
        }
        tmax = max_over_rows_of_lanes(tmax);
        const float mn = fmaxf(m, tmax);                   // finite: every tile of the walk holds a key that is seen
        const float alpha = expf(m - mn);                  // 0 on the first tile
        floatx4 pr;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            pr[i] = ok[i] ? expf(s[i] - mn) : 0.f;
            psum += pr[i];
        }
        l = l * alpha + psum;
        m = mn;
        // O^T: this lane brings, of the value rows d = 16 db + n, the keys kk + 4 g .. + 3
        const int key0 = kk + 4 * g;
        long voff[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = key0 + i;
            const int kc = ok[i] ? key : p;                // (an address that is valid; the value is not used)
            voff[i] = (long)bt[kc / P] * page_stride + ((long)(Hkv + kvh) * P) * D + kc % P;
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            floatx4 vf;
            const long drow = (long)(db * 16 + n) * P;
            if (vec_v && ok[0] && ok[3]) {
                vf = *(const floatx4*)(cache + voff[0] + drow);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) vf[i] = ok[i] ? cache[voff[i] + drow] : 0.f;
            }
            acc[db] *= alpha;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[db] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[j], pr[j], acc[db], 0, 0, 0);
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    // the four waves' results, merged by the first in the order of the waves (a wave without a tile
    // has m = -inf and weighs nothing)
    float* mine = merge_lds + (long)wave * (DB * 4 + 2) * 64 + lane;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) mine[(db * 4 + i) * 64] = acc[db][i];
    mine[(DB * 4) * 64] = m;
    mine[(DB * 4 + 1) * 64] = l;
    __syncthreads();
    if (wave != 0) return;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < F32_WAVES; ++w) M = fmaxf(M, merge_lds[((long)w * (DB * 4 + 2) + DB * 4) * 64 + lane]);
    float wgt[F32_WAVES], lsum = 0.f;
#pragma unroll
    for (int w = 0; w < F32_WAVES; ++w) {
        const float mw = merge_lds[((long)w * (DB * 4 + 2) + DB * 4) * 64 + lane];
        wgt[w] = (mw == -INFINITY) ? 0.f : expf(mw - M);
        lsum += wgt[w] * merge_lds[((long)w * (DB * 4 + 2) + DB * 4 + 1) * 64 + lane];
    }
    if (head_ok) {
        const float inv = 1.f / lsum;
        float* orow = out + (t * Hq + head) * D + g * 4;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            floatx4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float a = 0.f;
#pragma unroll
                for (int w = 0; w < F32_WAVES; ++w) a += wgt[w] * merge_lds[((long)w * (DB * 4 + 2) + db * 4 + i) * 64 + lane];
                o[i] = a * inv;
            }
            *(floatx4*)(orow + db * 16) = o;
        }
    }
}

bool qe_attention_f32_ok(int Hq, int Hkv, int D, int P) {
    return D % 16 == 0 && D >= 16 && D <= 256 && Hq % Hkv == 0 && P >= 1;
}

int qe_attention_f32(const float* q, float* out, const float* cache, const int* positions, const int* tok_seq,
                     const int* block_table, int max_blocks, const int* tokens, int T, int Hq, int Hkv, int D,
                     int P, float scale, int window, hipStream_t stream) {
    QE_REQUIRE(qe_attention_f32_ok(Hq, Hkv, D, P), "attention (32-bit): sizes not taken");
    const int groups16 = (Hq / Hkv + 15) / 16;
    QE_REQUIRE((long)Hkv * groups16 <= 65535, "attention (32-bit): too many heads");
    dim3 grid(T, Hkv * groups16);
#define QE_ATTN_F32(DB_)                                                                              \
    case DB_: {                                                                                       \
        const size_t lds = (size_t)F32_WAVES * (DB_ * 4 + 2) * 64 * sizeof(float);                    \
        if (lds > 48 * 1024) {                                                                        \
            static bool raised = false;                                                               \
            if (!raised) {                                                                            \
                hipError_t e_ = hipFuncSetAttribute((const void*)attention_f32_kernel<DB_>,           \
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
                if (e_ != hipSuccess) { qe_set_error("attention (32-bit): %s", hipGetErrorString(e_)); return (int)e_; } \
                raised = true;                                                                        \
            }                                                                                         \
        }                                                                                             \
        attention_f32_kernel<DB_><<<grid, 64 * F32_WAVES, lds, stream>>>(q, out, cache, positions, tok_seq, \
                                                    block_table, max_blocks, tokens, Hq, Hkv, P, scale, window); \
        break;                                                                                        \
    }
    switch (D / 16) {
        QE_ATTN_F32(1) QE_ATTN_F32(2) QE_ATTN_F32(3) QE_ATTN_F32(4) QE_ATTN_F32(5) QE_ATTN_F32(6)
        QE_ATTN_F32(7) QE_ATTN_F32(8) QE_ATTN_F32(9) QE_ATTN_F32(10) QE_ATTN_F32(11) QE_ATTN_F32(12)
        QE_ATTN_F32(13) QE_ATTN_F32(14) QE_ATTN_F32(15) QE_ATTN_F32(16)
    }
#undef QE_ATTN_F32
    QE_LAUNCH_CHECK();
    return 0;
}
