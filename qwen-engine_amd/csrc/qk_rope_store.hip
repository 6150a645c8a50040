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
            const float c = cs[i], s = cs[half + i];
            const float x1 = row[i], x2 = row[half + i];
            Elem<TA>::store(dst + i, c * x1 - s * x2);
            Elem<TA>::store(dst + half + i, s * x1 + c * x2);
        }
        for (int d = rotary_dim + lane; d < D; d += 64) Elem<TA>::store(dst + d, row[d]);
    } else {
        for (int d = lane; d < D; d += 64) Elem<TA>::store(dst + d, row[d]);
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
