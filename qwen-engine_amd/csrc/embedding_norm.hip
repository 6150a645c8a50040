// Embedding gather into the 32-bit residual stream, and RMSNorm with an optional
// fused residual add and an optional row gather.
#include "common.h"

// out[t, :] = float(table[ids[t], :]).  One block per token.
template <typename TW>
__global__ void embedding_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                                 float* __restrict__ out, int H) {
    const long t = blockIdx.x;
    const TW* row = table + (long)ids[t] * H;
    float* o = out + t * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) o[c] = Elem<TW>::load(row + c);
}

extern "C" int qe_embedding(const int* ids, const void* table, float* out, int T, int V, int H,
                            int dt_w, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && V > 0 && H > 0, "embedding: bad sizes T=%d V=%d H=%d", T, V, H);
    if (T == 0) return 0;
    const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
    if (dt_w == QE_F32)
        embedding_kernel<float><<<T, threads, 0, stream>>>(ids, (const float*)table, out, H);
    else if (dt_w == QE_BF16)
        embedding_kernel<bf16_t><<<T, threads, 0, stream>>>(ids, (const bf16_t*)table, out, H);
    else
        QE_REQUIRE(false, "embedding: unknown table dtype %d", dt_w);
    QE_LAUNCH_CHECK();
    return 0;
}

// One block per output row r.  src row = rows ? rows[r] : r.
//   v = h[src] (+ delta_0[src] + delta_1[src] + ...);  if delta and !rows: h[src] = v  (the residual sum, 32-bit)
//   out[r] = v * rsqrt(mean(v^2) + eps) * w        (all in 32-bit, one rounding at the store)
// delta holds n_delta tensors [T, H] one after the other (partial products of a matrix product cut
// along K, or one branch output); they are added in ascending order.
// Two passes over the row; the second re-reads h (and delta) instead of keeping the row in
// registers, so any H is taken.
template <typename TA, typename TD>
__global__ void rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_delta, long delta_stride,
                               const int* __restrict__ rows, const float* __restrict__ w,
                               TA* __restrict__ out, int H, float eps) {
    __shared__ float red[16];
    const long r = blockIdx.x;
    const long src = rows ? (long)rows[r] : r;
    float* hr = h + src * H;
    const TD* dr = delta ? delta + src * H : nullptr;
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = hr[c];
        if (dr)
            for (int s = 0; s < n_delta; ++s) v += Elem<TD>::load(dr + s * delta_stride + c);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float rstd = rsqrtf(ss / (float)H + eps);
    TA* o = out + r * H;
    const bool write_back = dr && !rows;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = hr[c];
        if (dr)
            for (int s = 0; s < n_delta; ++s) v += Elem<TD>::load(dr + s * delta_stride + c);
        if (write_back) hr[c] = v;
        Elem<TA>::store(o + c, v * rstd * w[c]);
    }
}

// The same for rows of up to NV * 4 * blockDim.x elements with H % 4 == 0: the row is read once
// (16-byte loads) and kept in registers.  This is the kernel of decode steps, where a launch has few
// rows and its time is the latency of its memory accesses: the row's pieces and the parts to add are
// asked for together, SB parts of all pieces at a time, before the first is added, from addresses that
// are always valid (a piece beyond the row or a part beyond the last reads another again and is not
// used), so that no branch stands between the loads and a trip to memory serves them all.  (With a
// trip per piece, a row of 4096 with eight parts took 6.8 us.)  The parts are added in ascending order.
// FEW: few rows, SB = 8 (or 4) parts at a time; many rows fill the chip anyway and are bound by the
// memory's rate, which more waves a compute unit (fewer registers: two parts at a time) serve better.
template <typename TA, typename TD, int NV, bool FEW>
__global__ __launch_bounds__(256) void rmsnorm_regs_kernel(float* __restrict__ h, const TD* __restrict__ delta, int n_delta, long delta_stride,
                                    const int* __restrict__ rows, const float* __restrict__ w,
                                    TA* __restrict__ out, int H, float eps) {
    constexpr int SB = !FEW ? 2 : (NV <= 4 ? 8 : 4);
    __shared__ float red[16];
    const long r = blockIdx.x;
    const long src = rows ? (long)rows[r] : r;
    float* hr = h + src * H;
    const TD* dr = delta ? delta + src * H : nullptr;
    int cs[NV];
    bool ok[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = (threadIdx.x + i * blockDim.x) * 4;
        ok[i] = c < H;
        cs[i] = ok[i] ? c : 0;
    }
    float v[NV][4];
#pragma unroll
    for (int i = 0; i < NV; ++i) Vec4<float>::load(hr + cs[i], v[i]);
    if (dr) {
        for (int s0 = 0; s0 < n_delta; s0 += SB) {
            float d[SB][NV][4];
#pragma unroll
            for (int s = 0; s < SB; ++s) {
                const TD* part = dr + (long)min(s0 + s, n_delta - 1) * delta_stride;
#pragma unroll
                for (int i = 0; i < NV; ++i) Vec4<TD>::load(part + cs[i], d[s][i]);
            }
#pragma unroll
            for (int s = 0; s < SB; ++s)
                if (s0 + s < n_delta) {
#pragma unroll
                    for (int i = 0; i < NV; ++i)
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[i][e] += d[s][i][e];
                }
        }
    }
    float wv[NV][4];                       // the weights are asked for before the sum is waited for
#pragma unroll
    for (int i = 0; i < NV; ++i) Vec4<float>::load(w + cs[i], wv[i]);
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
        if (ok[i]) {
#pragma unroll
            for (int e = 0; e < 4; ++e) ss += v[i][e] * v[i][e];
        }
    ss = block_sum(ss, red);
    const float rstd = rsqrtf(ss / (float)H + eps);
    const bool write_back = dr && !rows;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        if (ok[i]) {
            const int c = cs[i];
            if (write_back) Vec4<float>::store(hr + c, v[i]);
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = v[i][e] * rstd * wv[i][e];
            Vec4<TA>::store(out + r * H + c, o);
        }
    }
}

template <typename TA, typename TD>
static void launch_rmsnorm(float* h, const void* delta, int n_delta, long stride, const int* rows, const float* w,
                           void* out, int n_out_rows, int H, float eps, hipStream_t stream) {
    if (H % 4 == 0 && H <= 8192) {
        int threads = ((H / 4 + 63) / 64) * 64;
        if (threads > 256) threads = 256;
        const int nv = (H / 4 + threads - 1) / threads;
#define QE_NORM(NV_)                                                                                         \
    do {                                                                                                     \
        if (n_out_rows <= 512)                                                                               \
            rmsnorm_regs_kernel<TA, TD, NV_, true><<<n_out_rows, threads, 0, stream>>>(                      \
                h, (const TD*)delta, n_delta, stride, rows, w, (TA*)out, H, eps);                            \
        else                                                                                                 \
            rmsnorm_regs_kernel<TA, TD, NV_, false><<<n_out_rows, threads, 0, stream>>>(                     \
                h, (const TD*)delta, n_delta, stride, rows, w, (TA*)out, H, eps);                            \
    } while (0)
        if (nv <= 1) QE_NORM(1);
        else if (nv <= 2) QE_NORM(2);
        else if (nv <= 4) QE_NORM(4);
        else QE_NORM(8);
#undef QE_NORM
        return;
    }
    const int threads = H >= 2048 ? 512 : (H >= 512 ? 256 : 64);
    rmsnorm_kernel<TA, TD><<<n_out_rows, threads, 0, stream>>>(h, (const TD*)delta, n_delta, stride, rows, w, (TA*)out, H, eps);
}

// dt_d: element type of delta (that of the output, or float for partial products)
extern "C" int qe_rmsnorm(float* h, const void* delta, int n_delta, int dt_d, long n_rows_h, const int* rows,
                          const float* w, void* out, int n_out_rows, int H, float eps, int dt_a,
                          hipStream_t stream) {
    QE_REQUIRE(n_out_rows >= 0 && H > 0, "rmsnorm: bad sizes rows=%d H=%d", n_out_rows, H);
    QE_REQUIRE(!delta || n_delta >= 1, "rmsnorm: %d delta tensors", n_delta);
    if (n_out_rows == 0) return 0;
    const long stride = n_rows_h * H;
    if (dt_a == QE_F32 && (!delta || dt_d == QE_F32))
        launch_rmsnorm<float, float>(h, delta, n_delta, stride, rows, w, out, n_out_rows, H, eps, stream);
    else if (dt_a == QE_BF16 && (!delta || dt_d == QE_BF16))
        launch_rmsnorm<bf16_t, bf16_t>(h, delta, n_delta, stride, rows, w, out, n_out_rows, H, eps, stream);
    else if (dt_a == QE_BF16 && dt_d == QE_F32)
        launch_rmsnorm<bf16_t, float>(h, delta, n_delta, stride, rows, w, out, n_out_rows, H, eps, stream);
    else
        QE_REQUIRE(false, "rmsnorm: no kernel for output type %d with delta type %d", dt_a, dt_d);
    QE_LAUNCH_CHECK();
    return 0;
}

// h[t, :] += delta[t, :]  (for blocks whose norm does not fuse the residual sum)
template <typename TA>
__global__ void residual_add_kernel(float* __restrict__ h, const TA* __restrict__ delta, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        h[i] += Elem<TA>::load(delta + i);
}

extern "C" int qe_residual_add(float* h, const void* delta, long n, int dt_a, hipStream_t stream) {
    if (n <= 0) return 0;
    const int blocks = (int)((n + 255) / 256 > 4096 ? 4096 : (n + 255) / 256);
    if (dt_a == QE_F32)
        residual_add_kernel<float><<<blocks, 256, 0, stream>>>(h, (const float*)delta, n);
    else if (dt_a == QE_BF16)
        residual_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(h, (const bf16_t*)delta, n);
    else
        QE_REQUIRE(false, "residual_add: unknown dtype %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}

// out[t, i] = silu(gate[t, i]) * up[t, i], the product formed in 32-bit.  gu holds gate | up per
// row, or (interleave) gate and up in alternating blocks of 32: gate 0..31, up 0..31, gate 32..63, ...
template <typename TA>
__global__ void silu_mul_kernel(const TA* __restrict__ gu, TA* __restrict__ out, int T, int I, int interleave) {
    const long n = (long)T * I;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (long)gridDim.x * blockDim.x) {
        const long t = idx / I;
        const int i = (int)(idx - t * I);
        const long gi = interleave ? (long)(i >> 5) * 64 + (i & 31) : i;
        const float g = Elem<TA>::load(gu + t * 2 * I + gi);
        const float u = Elem<TA>::load(gu + t * 2 * I + gi + (interleave ? 32 : I));
        Elem<TA>::store(out + idx, g / (1.f + expf(-g)) * u);
    }
}

extern "C" int qe_silu_mul(const void* gu, void* out, int T, int I, int interleave, int dt_a, hipStream_t stream) {
    QE_REQUIRE(T >= 0 && I > 0, "silu_mul: bad sizes T=%d I=%d", T, I);
    QE_REQUIRE(!interleave || I % 32 == 0, "silu_mul: interleaved gate|up needs a width in blocks of 32, not %d", I);
    if (T == 0) return 0;
    const long n = (long)T * I;
    const int blocks = (int)((n + 255) / 256 > 8192 ? 8192 : (n + 255) / 256);
    if (dt_a == QE_F32)
        silu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, T, I, interleave);
    else if (dt_a == QE_BF16)
        silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, T, I, interleave);
    else
        QE_REQUIRE(false, "silu_mul: unknown dtype %d", dt_a);
    QE_LAUNCH_CHECK();
    return 0;
}

// table[idx[i]] = val[i] for idx[i] >= 0: keeps the device's copy of the block tables up to date.
__global__ void scatter_int_kernel(int* __restrict__ table, const int* __restrict__ idx,
                                   const int* __restrict__ val, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && idx[i] >= 0) table[idx[i]] = val[i];
}

extern "C" int qe_scatter_int(int* table, const int* idx, const int* val, int n, long table_size,
                              hipStream_t stream) {
    QE_REQUIRE(n >= 0 && table_size >= 0, "scatter: bad sizes");
    if (n == 0) return 0;
    scatter_int_kernel<<<qe_cdiv(n, 256), 256, 0, stream>>>(table, idx, val, n);
    QE_LAUNCH_CHECK();
    return 0;
}
