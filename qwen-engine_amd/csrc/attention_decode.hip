// Attention of single new tokens over the paged cache (decode), bfloat16, split over the keys
// ("flash decoding"), on the MFMA units.  All query heads of a key/value group are computed by
// one wave, so the cache is read from HBM once; this kernel is bound by that read.
//
// One wave per (split of the keys, key/value head, token).  For each tile of 16 keys (a page
// or a part of one; the page size is a multiple of 16):
//   S^T[key, head] = K[key, :] . Q[head, :]          v_mfma_f32_16x16x32_bf16, D / 32 of them;
//       lane (g, n), g = lane / 16, n = lane % 16, loads K[key n][c * 32 + g * 8 .. + 8] (16 bytes)
//       and ends up with the scores of keys g * 4 .. g * 4 + 3 for head n
//   online softmax per head n in 32-bit (max over the lane's 4 keys and the 4 lanes of the head)
//   O^T[d, head] += V^T[d, key] . P^T[key, head]     v_mfma_f32_16x16x16_bf16, D / 16 of them;
//       the probabilities a lane holds are exactly its B operand, and because value tiles are
//       stored transposed ([D][P]) the A operand is one 8-byte load: V^T[d = db * 16 + n][keys g * 4 .. + 3]
// No shared memory and no shuffles apart from the two of the max.  Heads beyond the group size
// (lanes n >= G) compute on zeros and are not stored.
//
// The splits are cut at absolute key positions (multiples of split_keys), so a token's result
// does not depend on what else is in the batch.  A second kernel merges the splits.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short short4_t;
typedef __attribute__((ext_vector_type(4))) float floatx4;

__device__ __forceinline__ short bf16_bits(float f) { return (short)float_to_bf16(f).bits; }

template <int D>
__global__ __launch_bounds__(64) void attention_decode_split_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache,
    const int* __restrict__ dec_tokens, const int* __restrict__ positions, const int* __restrict__ tok_seq,
    const int* __restrict__ block_table, int max_blocks,
    float* __restrict__ part_acc, float* __restrict__ part_ml,
    int Hq, int Hkv, int P, float scale, int window, int split_keys, int num_splits) {
    const int lane = threadIdx.x, g = lane >> 4, n = lane & 15;
    const int split = blockIdx.x, kvh = blockIdx.y, di = blockIdx.z;
    const int G = Hq / Hkv;
    const int t = dec_tokens[di];
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int k_begin = max(split * split_keys, lo);
    const int k_end = min((split + 1) * split_keys, p + 1);
    const int head = kvh * G + n;
    const bool head_ok = n < G;
    // partial results of this (token, head, split)
    float* pacc = part_acc + (((long)di * Hq + head) * num_splits + split) * D;
    float* pml = part_ml + (((long)di * Hq + head) * num_splits + split) * 2;
    if (k_begin >= k_end) {   // nothing of this split is seen by the token
        if (head_ok && g == 0) { pml[0] = -INFINITY; pml[1] = 0.f; }
        return;
    }
    const int* bt = block_table + (long)tok_seq[t] * max_blocks;
    const long page_stride = 2L * Hkv * P * D;

    bf16x8 qreg[D / 32];
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < D / 32; ++c)
        qreg[c] = head_ok ? *(const bf16x8*)(q + ((long)t * Hq + head) * D + c * 32 + g * 8) : zero8;

    float m = -INFINITY, l = 0.f;
    floatx4 acc[D / 16];
#pragma unroll
    for (int db = 0; db < D / 16; ++db) acc[db] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int kk = (k_begin / 16) * 16; kk < k_end; kk += 16) {
        const long page = bt[kk / P];
        const int o = kk % P;
        const bf16_t* kbase = cache + page * page_stride + ((long)kvh * P + o) * D;
        const bf16_t* vbase = cache + page * page_stride + ((long)(Hkv + kvh) * P) * D + o;
        bf16x8 kreg[D / 32];
#pragma unroll
        for (int c = 0; c < D / 32; ++c) kreg[c] = *(const bf16x8*)(kbase + (long)n * D + c * 32 + g * 8);
        short4_t vreg[D / 16];
#pragma unroll
        for (int db = 0; db < D / 16; ++db) vreg[db] = *(const short4_t*)(vbase + (long)(db * 16 + n) * P + g * 4);

        floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < D / 32; ++c) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[c], qreg[c], s, 0, 0, 0);
        float tmax = -INFINITY;
        bool ok[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = kk + g * 4 + i;
            ok[i] = key >= k_begin && key < k_end;
            s[i] = ok[i] ? s[i] * scale : -INFINITY;
            tmax = fmaxf(tmax, s[i]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float mn = fmaxf(m, tmax);        // finite: the tile holds at least one seen key
        const float alpha = __expf(m - mn);
        short4_t pb;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float pi = __expf(s[i] - mn);  // 0 for keys that are not seen
            psum += pi;
            pb[i] = bf16_bits(pi);
        }
        l = l * alpha + psum;
        m = mn;
        // values of unseen keys may be anything (an unwritten part of a page): keep them out
        const short4_t vmask = {(short)(ok[0] ? -1 : 0), (short)(ok[1] ? -1 : 0), (short)(ok[2] ? -1 : 0), (short)(ok[3] ? -1 : 0)};
#pragma unroll
        for (int db = 0; db < D / 16; ++db) {
            acc[db] *= alpha;
            acc[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vreg[db] & vmask, pb, acc[db], 0, 0, 0);
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (head_ok) {
#pragma unroll
        for (int db = 0; db < D / 16; ++db)
            *(floatx4*)(pacc + db * 16 + g * 4) = acc[db];    // O^T rows d = db * 16 + g * 4 + i of column head n
        if (g == 0) { pml[0] = m; pml[1] = l; }
    }
}

// out[t, head, :] = sum_s e^{m_s - M} acc_s / sum_s e^{m_s - M} l_s,  M = max_s m_s
template <int D>
__global__ __launch_bounds__(64) void attention_decode_merge_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, const int* __restrict__ dec_tokens,
    bf16_t* __restrict__ out, int Hq, int num_splits) {
    const int di = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* pml = part_ml + ((long)di * Hq + head) * num_splits * 2;
    const float* pacc = part_acc + ((long)di * Hq + head) * num_splits * D;
    float M = -INFINITY;
    for (int s = 0; s < num_splits; ++s) M = fmaxf(M, pml[2 * s]);
    float denom = 0.f;
    float o[(D + 63) / 64];
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) o[i] = 0.f;
    for (int s = 0; s < num_splits; ++s) {
        const float ms = pml[2 * s];
        if (ms == -INFINITY) continue;          // an empty split: its accumulator was never written
        const float wgt = __expf(ms - M);
        denom += wgt * pml[2 * s + 1];
#pragma unroll
        for (int i = 0; i < (D + 63) / 64; ++i) {
            const int d = lane + i * 64;
            if (d < D) o[i] += wgt * pacc[(long)s * D + d];
        }
    }
    bf16_t* orow = out + ((long)dec_tokens[di] * Hq + head) * D;
    const float inv = 1.f / denom;
#pragma unroll
    for (int i = 0; i < (D + 63) / 64; ++i) {
        const int d = lane + i * 64;
        if (d < D) orow[d] = float_to_bf16(o[i] * inv);
    }
}

bool qe_attention_decode_ok(int Hq, int Hkv, int D, int P, int dt_a) {
    return dt_a == QE_BF16 && (D == 64 || D == 128) && P % 16 == 0 && Hq % Hkv == 0 && Hq / Hkv <= 16;
}

size_t qe_attention_decode_workspace(int n_dec, int Hq, int D, int num_splits) {
    return (size_t)n_dec * Hq * num_splits * (D + 2) * sizeof(float);
}

// dec_tokens: the rows of q that are single new tokens of their requests.  max_position: the
// largest of their positions (fixes the number of splits).  workspace: at least
// qe_attention_decode_workspace(...) bytes.
int qe_attention_decode(const void* q, void* out, const void* cache, const int* dec_tokens, int n_dec,
                        const int* positions, const int* tok_seq, const int* block_table, int max_blocks,
                        int Hq, int Hkv, int D, int P, float scale, int window, int max_position,
                        int split_keys, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    QE_REQUIRE(qe_attention_decode_ok(Hq, Hkv, D, P, QE_BF16), "decode attention: sizes not taken");
    QE_REQUIRE(split_keys >= 16 && split_keys % 16 == 0, "decode attention: split of %d keys", split_keys);
    if (n_dec == 0) return 0;
    const int num_splits = max_position / split_keys + 1;
    QE_REQUIRE(num_splits <= 65535 && n_dec <= 65535, "decode attention: too many splits or tokens");
    QE_REQUIRE(workspace_bytes >= qe_attention_decode_workspace(n_dec, Hq, D, num_splits),
               "decode attention: workspace of %zu bytes is too small", workspace_bytes);
    float* part_acc = (float*)workspace;
    float* part_ml = part_acc + (size_t)n_dec * Hq * num_splits * D;
    dim3 grid(num_splits, Hkv, n_dec);
    dim3 mgrid(n_dec, Hq);
    if (D == 128) {
        attention_decode_split_kernel<128><<<grid, 64, 0, stream>>>(
            (const bf16_t*)q, (const bf16_t*)cache, dec_tokens, positions, tok_seq, block_table, max_blocks,
            part_acc, part_ml, Hq, Hkv, P, scale, window, split_keys, num_splits);
        attention_decode_merge_kernel<128><<<mgrid, 64, 0, stream>>>(part_acc, part_ml, dec_tokens, (bf16_t*)out, Hq, num_splits);
    } else {
        attention_decode_split_kernel<64><<<grid, 64, 0, stream>>>(
            (const bf16_t*)q, (const bf16_t*)cache, dec_tokens, positions, tok_seq, block_table, max_blocks,
            part_acc, part_ml, Hq, Hkv, P, scale, window, split_keys, num_splits);
        attention_decode_merge_kernel<64><<<mgrid, 64, 0, stream>>>(part_acc, part_ml, dec_tokens, (bf16_t*)out, Hq, num_splits);
    }
    QE_LAUNCH_CHECK();
    return 0;
}
