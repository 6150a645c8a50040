// Per-head q/k RMSNorm, half-split rotation and the write of keys and values
// into their cache pages, in one pass over the fused q|k|v projection.
//
//   qkv   [T, (Hq + 2 Hkv) D]   row = q heads, k heads, v heads
//   q_out [T, Hq, D]            normalised and rotated queries
//   cache of one layer: [page][2 (k, v)][Hkv][P * D]: key tiles [P][D], value tiles transposed [D][P];
//   slot[t] = page * P + offset, < 0: no write
//
// With packed_out [T, Hq + 2 Hkv, D] every head is written there instead (q and k
// after norm and rotation, v as it is) and neither q_out nor the cache is touched.
//
// Norm and rotation are computed in 32-bit from the stored projection and rounded
// once.  Each of the three steps can be switched off (no norm weights, no table,
// no slots), so that a mixer with another position encoding can run them apart.
#include "common.h"

template <typename TA>
__global__ __launch_bounds__(64) void qk_rope_store_kernel(
    const TA* __restrict__ qkv, const int* __restrict__ positions,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    const float* __restrict__ table, int rotary_dim,
    const int* __restrict__ slot, TA* __restrict__ cache, TA* __restrict__ q_out,
    TA* __restrict__ packed_out, int Hq, int Hkv, int D, int P) {
    extern __shared__ float row[];  // D floats
    const long t = blockIdx.x;
    const int head = blockIdx.y;  // 0..Hq-1 q, Hq..Hq+Hkv-1 k, then v
    const int lane = threadIdx.x;
    const int width = (Hq + 2 * Hkv) * D;
    const TA* src = qkv + t * width + (long)head * D;
    const bool is_q = head < Hq;
    const bool is_k = !is_q && head < Hq + Hkv;
    const bool is_v = !is_q && !is_k;

    TA* dst;
    if (packed_out) {
        dst = packed_out + t * width + (long)head * D;
    } else if (is_q) {
        dst = q_out + (t * Hq + head) * D;
    } else {
        if (!slot) return;
        const int s = slot[t];
        if (s < 0) return;
        const int kh = is_k ? head - Hq : head - Hq - Hkv;
        const long page = s / P, off = s % P;
        if (is_k) {
            dst = cache + page * (2L * Hkv * P * D) + ((long)kh * P + off) * D;
        } else {   // value tile is [D][P]
            TA* vt = cache + page * (2L * Hkv * P * D) + ((long)(Hkv + kh) * P) * D + off;
            for (int d = lane; d < D; d += 64) vt[(long)d * P] = src[d];
            return;
        }
    }
    if (is_v) {   // packed form
        for (int d = lane; d < D; d += 64) dst[d] = src[d];
        return;
    }
    const float* w = is_q ? q_w : k_w;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
        const float v = Elem<TA>::load(src + d);
        row[d] = v;
        ss += v * v;
    }
    if (w) {
        ss = wave_sum(ss);
        const float rstd = rsqrtf(ss / (float)D + eps);
        for (int d = lane; d < D; d += 64) row[d] = row[d] * rstd * w[d];
    }
    __syncthreads();
    if (table) {
        const int half = rotary_dim / 2;
        const float* cs = table + (long)positions[t] * rotary_dim;
        for (int i = lane; i < half; i += 64) {
            float x1 = row[i], x2 = row[half + i];
            rotate_pair(cs[i], cs[half + i], x1, x2);
            Elem<TA>::store(dst + i, x1);
            Elem<TA>::store(dst + half + i, x2);
        }
        for (int d = rotary_dim + lane; d < D; d += 64) Elem<TA>::store(dst + d, row[d]);
    } else {
        for (int d = lane; d < D; d += 64) Elem<TA>::store(dst + d, row[d]);
    }
}

// The same work for head sizes D = 8 * 2^k (and a rotation over the whole head): a head is
// taken by D / 8 lanes, each with 4 features of the first half and the 4 features 64... D / 2
// further that rotate with them, so a wave works on 512 / D heads at a time with 8-byte
// accesses and the norm's sum needs log2(D / 8) shuffles.  One block of 256 threads per token.
//
// Values go to the cache by tiles: a value tile is stored transposed, [D][P], so one token's
// values are a column of single elements.  The blocks of 16 consecutive tokens share the work
// on those tokens' values: each takes some of the key/value heads, reads the 16 tokens' values
// of that head, turns them round in shared memory and writes, per feature, the run of 16
// elements that are neighbours in the tile.  That needs the 16 tokens to lie side by side in
// one page (consecutive slots), which is how the tokens of a prompt lie; where they do not
// (single new tokens of several requests), every block writes its own token's values element by
// element.
//
// The projection can also come as 32-bit partial products [S][T][width] of a product that was cut
// along K (few rows against a large matrix: the cut fills the chip): they are added here in the
// order of S, with the bias if there is one, and rounded to the activation type first, as the
// product itself would have stored them.
template <typename TA>
struct QkvSource {
    const TA* qkv;          // [T][width], or null
    const float* parts;     // [S][T][width]
    const float* bias;      // [width] or null (with parts only)
    int S;
    long stride;            // T * width
    // four neighbouring elements from element index idx = t * width + col
    __device__ __forceinline__ void load4(long idx, int col, float (&v)[4]) const {
        if (qkv) {
            Vec4<TA>::load(qkv + idx, v);
            return;
        }
        // (eight parts are asked for before the first is used: one trip to memory for them all)
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = 0.f;
        for (int s0 = 0; s0 < S; s0 += 8) {
            float p[8][4];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int sk = s0 + k < S ? s0 + k : S - 1;
                Vec4<float>::load(parts + sk * stride + idx, p[k]);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (s0 + k < S) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += p[k][e];
                }
        }
        if (bias) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += bias[col + e];
        }
        TA r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) { Elem<TA>::store(r + e, v[e]); v[e] = Elem<TA>::load(r + e); }
    }
    // The same for two places of four elements at once (the two halves of a head that rotate together): the
    // parts of both are asked for together, and a part beyond the last is skipped by a select, not by a
    // branch, so that one trip to memory serves all of them.
    __device__ __forceinline__ void load4x2(long idx_a, int col_a, long idx_b, int col_b, float (&a)[4], float (&b)[4]) const {
        if (qkv) {
            Vec4<TA>::load(qkv + idx_a, a);
            Vec4<TA>::load(qkv + idx_b, b);
            return;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = b[e] = 0.f;
        for (int s0 = 0; s0 < S; s0 += 8) {
            float pa[8][4], pb[8][4];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int sk = s0 + k < S ? s0 + k : S - 1;
                Vec4<float>::load(parts + sk * stride + idx_a, pa[k]);
                Vec4<float>::load(parts + sk * stride + idx_b, pb[k]);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const bool on = s0 + k < S;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a[e] = on ? a[e] + pa[k][e] : a[e];
                    b[e] = on ? b[e] + pb[k][e] : b[e];
                }
            }
        }
        if (bias) {
#pragma unroll
            for (int e = 0; e < 4; ++e) { a[e] += bias[col_a + e]; b[e] += bias[col_b + e]; }
        }
        TA r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) { Elem<TA>::store(r + e, a[e]); a[e] = Elem<TA>::load(r + e); }
#pragma unroll
        for (int e = 0; e < 4; ++e) { Elem<TA>::store(r + e, b[e]); b[e] = Elem<TA>::load(r + e); }
    }
    __device__ __forceinline__ float load1(long idx, int col) const {
        if (qkv) return Elem<TA>::load(qkv + idx);
        float v = parts[idx];
        for (int s = 1; s < S; ++s) v += parts[s * stride + idx];
        if (bias) v += bias[col];
        TA r;
        Elem<TA>::store(&r, v);
        return Elem<TA>::load(&r);
    }
};

template <typename TA>
__global__ __launch_bounds__(256) void qk_rope_store_vec_kernel(
    const QkvSource<TA> in, const int* __restrict__ positions,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    const float* __restrict__ table, const int* __restrict__ slot, TA* __restrict__ cache,
    TA* __restrict__ q_out, TA* __restrict__ packed_out, int Hq, int Hkv, int D, int P, int value_blocks) {
    const long t = blockIdx.x;
    const int lph = D / 8;                     // lanes per head
    const int half = D / 2;
    const int j = threadIdx.x % lph;           // this lane's place in its head
    const int heads_per_pass = 256 / lph;
    const int nheads = Hq + 2 * Hkv;
    const int width = nheads * D;
    const int s = slot ? slot[t] : -1;
    const float* cs = table ? table + (long)positions[t] * D : nullptr;
    const int nloop = packed_out ? nheads : Hq + Hkv;   // (values go to the cache by tiles, further down)
    // (the blocks (t, 0 .. ny - 1) share the token's heads: more blocks where the tokens are few; with
    // value_blocks = 1 the last block of a token takes no heads but the values, further down, which block 0
    // does after its heads otherwise: a kernel for few tokens lasts as long as its longest chain of loads)
    const int ny = (int)gridDim.y - value_blocks;
    const int first = (int)blockIdx.y < ny ? (int)(threadIdx.x / lph + blockIdx.y * heads_per_pass) : nloop;
    for (int head = first; head < nloop; head += heads_per_pass * ny) {
        const bool is_q = head < Hq;
        const bool is_k = !is_q && head < Hq + Hkv;
        const long src = t * width + (long)head * D;   // element index of the head's first feature
        // the norm's weights and the table's row are asked for before the head, not after it has arrived
        const float* w = is_q ? q_w : k_w;
        float wa[4], wb[4], c[4], sn[4];
        if (w) {
            Vec4<float>::load(w + 4 * j, wa);
            Vec4<float>::load(w + half + 4 * j, wb);
        }
        if (cs) {
            Vec4<float>::load(cs + 4 * j, c);
            Vec4<float>::load(cs + half + 4 * j, sn);
        }
        float a[4], b[4];                      // features 4 j .. 4 j + 3 and half + 4 j .. half + 4 j + 3
        in.load4x2(src + 4 * j, head * D + 4 * j, src + half + 4 * j, head * D + half + 4 * j, a, b);
        TA* dst = nullptr;
        if (packed_out) {
            dst = packed_out + t * width + (long)head * D;
        } else if (is_q) {
            dst = q_out + (t * Hq + head) * D;
        } else if (s >= 0) {
            const long page = s / P, off = s % P;
            const int kh = is_k ? head - Hq : head - Hq - Hkv;
            if (is_k) {
                dst = cache + page * (2L * Hkv * P * D) + ((long)kh * P + off) * D;
            }                                               // (values: below, by tiles)
        }
        const bool is_v = !is_q && !is_k;
        if (is_v) {
            if (packed_out) {
                Vec4<TA>::store(dst + 4 * j, a);
                Vec4<TA>::store(dst + half + 4 * j, b);
            }
            continue;
        }
        if (w) {
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) ss += a[e] * a[e] + b[e] * b[e];
            if (lph == 16) ss = row16_sum(ss);             // (the same sum, without the LDS crossbar)
            else for (int o = lph >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
            const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
            for (int e = 0; e < 4; ++e) { a[e] = a[e] * rstd * wa[e]; b[e] = b[e] * rstd * wb[e]; }
        }
        if (cs) {
#pragma unroll
            for (int e = 0; e < 4; ++e) rotate_pair(c[e], sn[e], a[e], b[e]);
        }
        if (dst) {
            Vec4<TA>::store(dst + 4 * j, a);
            Vec4<TA>::store(dst + half + 4 * j, b);
        }
    }
    if (packed_out || !slot || (int)blockIdx.y != (value_blocks ? ny : 0)) return;

    // ---- values of the 16 tokens t0 .. t0 + n - 1, key/value heads t - t0, t - t0 + n, ... ----
    extern __shared__ __attribute__((aligned(16))) unsigned char vsh[];   // [D][16] elements + 16 bytes a row
    const int srow = 16 * (int)sizeof(TA) + 16;
    const long t0 = t / 16 * 16;
    const int n = (int)((long)gridDim.x - t0 < 16 ? (long)gridDim.x - t0 : 16);
    const int s0 = slot[t0];
    bool run = s0 >= 0 && s0 % P + n <= P;                 // side by side in one page?
    for (int i = 1; i < n; ++i) run = run && slot[t0 + i] == s0 + i;
    if (!run) {
        // not side by side (single new tokens of several requests): every block writes its own
        // token's values, four neighbouring features a thread, element by element into the tiles
        if (s < 0) return;
        TA* page = cache + (long)(s / P) * (2L * Hkv * P * D) + (long)Hkv * P * D + s % P;
        for (int idx = threadIdx.x; idx < Hkv * D / 4; idx += 256) {
            const int col = 4 * idx;                       // feature col % D of key/value head col / D
            float x[4];
            in.load4(t * width + (long)(Hq + Hkv) * D + col, (Hq + Hkv) * D + col, x);
#pragma unroll
            for (int e = 0; e < 4; ++e) Elem<TA>::store(page + (long)(col + e) * P, x[e]);
        }
        return;
    }
    const int cpr = D / 8;                                 // 8-element chunks in a head
    for (int kh = (int)(t - t0); kh < Hkv; kh += n) {
        const int col0 = (Hq + Hkv + kh) * D;
        const long src = t0 * width + col0;
        {
            __syncthreads();                               // the last head's readers are done
            for (int idx = threadIdx.x; idx < n * cpr; idx += 256) {
                const int i = idx / cpr, c = idx % cpr;
                float x[8];
                in.load4(src + (long)i * width + 8 * c, col0 + 8 * c, *(float(*)[4])x);
                in.load4(src + (long)i * width + 8 * c + 4, col0 + 8 * c + 4, *(float(*)[4])(x + 4));
#pragma unroll
                for (int e = 0; e < 8; ++e) Elem<TA>::store((TA*)(vsh + (8 * c + e) * srow) + i, x[e]);
            }
            __syncthreads();
            TA* vt = cache + (long)(s0 / P) * (2L * Hkv * P * D) + ((long)(Hkv + kh) * P) * D + s0 % P;
            const bool vec = n == 16 && P % 4 == 0 && (s0 % P) % 4 == 0;   // whole aligned groups of four
            for (int idx = threadIdx.x; idx < D * 4; idx += 256) {  // feature d, tokens 4 q .. 4 q + 3
                const int d = idx / 4, q4 = idx % 4;
                const TA* from = (const TA*)(vsh + d * srow) + 4 * q4;
                TA* to = vt + (long)d * P + 4 * q4;
                if (vec) {
                    float x[4];
                    Vec4<TA>::load(from, x);
                    Vec4<TA>::store(to, x);
                } else {
                    for (int e = 0; e < 4; ++e) if (4 * q4 + e < n) to[e] = from[e];
                }
            }
        }
    }
}

extern "C" int qe_qk_rope_store(const void* qkv, const int* positions, const float* q_w, const float* k_w,
                                float eps, const float* table, int rotary_dim, const int* slot,
                                void* cache, void* q_out, void* packed_out, int T, int Hq, int Hkv,
                                int D, int P, int dt_a, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && Hq > 0 && Hkv > 0 && D > 0 && P > 0, "qk_rope_store: bad sizes");
    QE_REQUIRE(!table || (rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= D),
               "qk_rope_store: rotary_dim=%d must be even and at most head_dim=%d", rotary_dim, D);
    QE_REQUIRE(!table || positions, "qk_rope_store: a rotation needs positions");
    QE_REQUIRE(!slot || cache, "qk_rope_store: slots without a cache");
    QE_REQUIRE(Hq + 2 * Hkv <= 65535, "qk_rope_store: too many heads");
    QE_REQUIRE(q_out || packed_out, "qk_rope_store: no output");
    if (T == 0) return 0;
    const int lph = D / 8;
    // (with few tokens the kernel with one wave per head has more waves in flight and is quicker)
    if ((long)T * (Hq + 2 * Hkv) > 2048 && D % 8 == 0 && lph >= 1 && lph <= 64 && (lph & (lph - 1)) == 0 &&
        (!table || rotary_dim == D)) {
        if (dt_a == QE_F32)
            qk_rope_store_vec_kernel<float><<<T, 256, (size_t)D * (16 * 4 + 16), stream>>>(
                QkvSource<float>{(const float*)qkv, nullptr, nullptr, 0, 0}, positions, q_w, k_w, eps, table, slot,
                (float*)cache, (float*)q_out, (float*)packed_out, Hq, Hkv, D, P, 0);
        else if (dt_a == QE_BF16)
            qk_rope_store_vec_kernel<bf16_t><<<T, 256, (size_t)D * (16 * 2 + 16), stream>>>(
                QkvSource<bf16_t>{(const bf16_t*)qkv, nullptr, nullptr, 0, 0}, positions, q_w, k_w, eps, table, slot,
                (bf16_t*)cache, (bf16_t*)q_out, (bf16_t*)packed_out, Hq, Hkv, D, P, 0);
        else
            QE_REQUIRE(false, "qk_rope_store: unknown dtype %d", dt_a);
        QE_LAUNCH_CHECK();
        return 0;
    }
    dim3 grid(T, Hq + 2 * Hkv);
    const size_t shmem = (size_t)D * sizeof(float);
    if (dt_a == QE_F32)
        qk_rope_store_kernel<float><<<grid, 64, shmem, stream>>>(
            (const float*)qkv, positions, q_w, k_w, eps, table, rotary_dim, slot, (float*)cache,
            (float*)q_out, (float*)packed_out, Hq, Hkv, D, P);
    else if (dt_a == QE_BF16)
        qk_rope_store_kernel<bf16_t><<<grid, 64, shmem, stream>>>(
            (const bf16_t*)qkv, positions, q_w, k_w, eps, table, rotary_dim, slot, (bf16_t*)cache,
            (bf16_t*)q_out, (bf16_t*)packed_out, Hq, Hkv, D, P);
    else
        QE_REQUIRE(false, "qk_rope_store: unknown dtype %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}

// 1 if qe_qk_rope_store_parts takes these sizes (the kernel with several lanes a head: a head size
// 8 * 2^k up to 512 and a rotation, if any, over the whole head)
extern "C" int qe_qk_rope_store_parts_supported(int D, int rotary_dim) {
    const int lph = D / 8;
    return (D % 8 == 0 && lph >= 1 && lph <= 64 && (lph & (lph - 1)) == 0 && (rotary_dim == 0 || rotary_dim == D)) ? 1 : 0;
}

// The same from 32-bit partial products parts [S, T, (Hq + 2 Hkv) D] (+ bias [width] or null) of
// the projection; q_out and cache are bfloat16.
extern "C" int qe_qk_rope_store_parts(const float* parts, int S, const float* bias, const int* positions,
                                      const float* q_w, const float* k_w, float eps, const float* table,
                                      int rotary_dim, const int* slot, void* cache, void* q_out, int T, int Hq,
                                      int Hkv, int D, int P, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && S >= 1 && Hq > 0 && Hkv > 0 && D > 0 && P > 0, "qk_rope_store: bad sizes");
    QE_REQUIRE(qe_qk_rope_store_parts_supported(D, table ? rotary_dim : 0),
               "qk_rope_store: partial products need a head size 8 * 2^k and a rotation over the whole head");
    QE_REQUIRE(!table || positions, "qk_rope_store: a rotation needs positions");
    QE_REQUIRE(!slot || cache, "qk_rope_store: slots without a cache");
    QE_REQUIRE(q_out, "qk_rope_store: no output");
    if (T == 0) return 0;
    const long stride = (long)T * (Hq + 2 * Hkv) * D;
    const int passes = qe_cdiv((Hq + Hkv) * (D / 8), 256);      // rounds of 256 lanes over the q and k heads of a token
    // (few tokens: a block of its own for each token's values)
    const int value_blocks = (slot && T <= 256) ? 1 : 0;
    const dim3 grid((unsigned)T, (unsigned)((passes < 4 ? passes : 4) + value_blocks));
    qk_rope_store_vec_kernel<bf16_t><<<grid, 256, (size_t)D * (16 * 2 + 16), stream>>>(
        QkvSource<bf16_t>{nullptr, parts, bias, S, stride}, positions, q_w, k_w, eps, table, slot,
        (bf16_t*)cache, (bf16_t*)q_out, nullptr, Hq, Hkv, D, P, value_blocks);
    QE_LAUNCH_CHECK();
    return 0;
}
