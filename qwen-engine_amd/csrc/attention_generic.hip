// Attention of a flat batch of new tokens over the paged cache, any sizes, all
// arithmetic in 32-bit.  One wave per (token, query head).  (The fallback of the bfloat16 mode for
// sizes the MFMA kernels refuse, and of the float32 mode for head sizes that are no multiple of 16;
// float32 otherwise goes to attention_f32.hip.)
//
// The query of token t at absolute position p = positions[t] of request
// s = tok_seq[t] sees the keys at positions lo..p of that request, read through
// block_table[s]; lo = 0, or p - window + 1 when a window is given.  Keys are
// taken 64 at a time from lo upwards with an online softmax, so the order of the
// sums depends on p and the window only: not on how the request's tokens were cut
// into steps, nor on what else is in the batch.
//
// cache of one layer: [page][2 (k, v)][Hkv][P * D]; a key tile is [P][D], a value tile is
// stored transposed, [D][P] (the layout the MFMA kernels read without a shuffle).
#include "common.h"

#define ATTN_MAX_D 256

template <typename TA>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const TA* __restrict__ q, TA* __restrict__ out, const TA* __restrict__ cache,
    const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks, const int* __restrict__ tokens,
    int Hq, int Hkv, int D, int P, float scale, int window) {
    extern __shared__ float smem[];
    float* qs = smem;            // D
    float* ps = smem + D;        // 64 probabilities of the current chunk
    long* voff = (long*)(smem + ((D + 64 + 1) & ~1));  // 64 offsets of the chunk's value rows
    const long t = tokens ? tokens[blockIdx.x] : blockIdx.x;   // a subset of the batch, or all of it
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int kvh = h / (Hq / Hkv);
    const int p = positions[t];
    const int* bt = block_table + (long)tok_seq[t] * max_blocks;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const long page_stride = 2L * Hkv * P * D;

    const TA* qrow = q + (t * Hq + h) * D;
    for (int d = lane; d < D; d += 64) qs[d] = Elem<TA>::load(qrow + d);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ATTN_MAX_D / 64];
#pragma unroll
    for (int i = 0; i < ATTN_MAX_D / 64; ++i) acc[i] = 0.f;

    for (int j0 = lo; j0 <= p; j0 += 64) {
        const int j = j0 + lane;
        float sc = -INFINITY;
        long vo = 0;
        if (j <= p) {
            const long page = bt[j / P];
            const int off = j % P;
            const long kbase = page * page_stride + ((long)kvh * P + off) * D;
            vo = page * page_stride + ((long)(Hkv + kvh) * P) * D + off;   // + d * P
            const TA* krow = cache + kbase;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], Elem<TA>::load(krow + d), dot);
            sc = dot * scale;
        }
        const float mn = fmaxf(m, wave_max(sc));   // finite: key j0 is always seen
        const float alpha = expf(m - mn);          // exp(-inf) = 0 on the first chunk
        const float pj = (j <= p) ? expf(sc - mn) : 0.f;
        l = l * alpha + wave_sum(pj);
        m = mn;
        ps[lane] = pj;
        voff[lane] = vo;
        __syncthreads();
        const int cnt = (p - j0 + 1 < 64) ? p - j0 + 1 : 64;
#pragma unroll
        for (int i = 0; i < ATTN_MAX_D / 64; ++i) {
            const int d = lane + i * 64;
            if (d < D) {
                float a = acc[i] * alpha;
                for (int jj = 0; jj < cnt; ++jj)
                    a = fmaf(ps[jj], Elem<TA>::load(cache + voff[jj] + (long)d * P), a);
                acc[i] = a;
            }
        }
        __syncthreads();
    }
    TA* orow = out + (t * Hq + h) * D;
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < ATTN_MAX_D / 64; ++i) {
        const int d = lane + i * 64;
        if (d < D) Elem<TA>::store(orow + d, acc[i] * inv);
    }
}

bool qe_attention_f32_ok(int Hq, int Hkv, int D, int P);
int qe_attention_f32(const float* q, float* out, const float* cache, const int* positions, const int* tok_seq,
                     const int* block_table, int max_blocks, const int* tokens, int T, int Hq, int Hkv, int D,
                     int P, float scale, int window, hipStream_t stream);

// 32-bit attention goes to the kernel on the matrix units (attention_f32.hip) where it takes the
// sizes, unless qe_use_matrix_f32(0) has switched that off.
extern int g_qe_matrix_f32;

int qe_attention_generic(const void* q, void* out, const void* cache, const int* positions,
                         const int* tok_seq, const int* block_table, int max_blocks, const int* tokens,
                         int T, int Hq, int Hkv, int D, int P, float scale, int window, int dt_a,
                         hipStream_t stream) {
    if (dt_a == QE_F32 && g_qe_matrix_f32 && qe_attention_f32_ok(Hq, Hkv, D, P))
        return qe_attention_f32((const float*)q, (float*)out, (const float*)cache, positions, tok_seq, block_table,
                                max_blocks, tokens, T, Hq, Hkv, D, P, scale, window, stream);
    QE_REQUIRE(D <= ATTN_MAX_D, "attention: head_dim=%d exceeds %d", D, ATTN_MAX_D);
    QE_REQUIRE(Hq <= 65535, "attention: too many heads");
    dim3 grid(T, Hq);
    const size_t shmem = (size_t)((D + 64 + 1) & ~1) * sizeof(float) + 64 * sizeof(long);
    if (dt_a == QE_F32)
        attention_generic_kernel<float><<<grid, 64, shmem, stream>>>(
            (const float*)q, (float*)out, (const float*)cache, positions, tok_seq, block_table,
            max_blocks, tokens, Hq, Hkv, D, P, scale, window);
    else if (dt_a == QE_BF16)
        attention_generic_kernel<bf16_t><<<grid, 64, shmem, stream>>>(
            (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)cache, positions, tok_seq, block_table,
            max_blocks, tokens, Hq, Hkv, D, P, scale, window);
    else
        QE_REQUIRE(false, "attention: unknown dtype %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}
