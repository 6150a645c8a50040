// Next-token choice on the device from 32-bit logits [R, V]: argmax (lowest index
// on ties) and temperature sampling by inverse CDF with one uniform per row.
#include "common.h"

// One block of 256 threads per row.
__global__ __launch_bounds__(256) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int V) {
    __shared__ float sv[256];
    __shared__ int si[256];
    const float* row = logits + (long)blockIdx.x * V;
    float best = -INFINITY;
    int bi = -1;
    for (int c = threadIdx.x; c < V; c += 256) {  // ascending c: a strict > keeps the lowest index
        const float v = row[c];
        if (bi < 0 || v > best) { best = v; bi = c; }
    }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            const float ov = sv[threadIdx.x + s];
            const int oi = si[threadIdx.x + s];
            const float mv = sv[threadIdx.x];
            const int mi = si[threadIdx.x];
            if (oi >= 0 && (mi < 0 || ov > mv || (ov == mv && oi < mi))) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = si[0];
}

extern "C" int qe_argmax(const float* logits, int* out, int R, int V, hipStream_t stream) {
    QE_REQUIRE(R >= 0 && V > 0, "argmax: bad sizes R=%d V=%d", R, V);
    if (R == 0) return 0;
    argmax_kernel<<<R, 256, 0, stream>>>(logits, out, V);
    QE_LAUNCH_CHECK();
    return 0;
}

// Row r: temperature[r] <= 0 -> argmax.  Else with z_i = logits_i / temperature,
// w_i = exp(z_i - max z): the token is the first i whose running sum of w (taken in
// index order) exceeds uniform[r] * sum w.  The vocabulary is cut into 256
// contiguous spans, one per thread, so the running sum is exact in its order:
// span sums first, then a scan inside the span that holds the target.
__global__ __launch_bounds__(256) void sample_kernel(const float* __restrict__ logits,
                                                     const float* __restrict__ temperature,
                                                     const float* __restrict__ uniform,
                                                     int* __restrict__ out, int V) {
    __shared__ float red[16];
    __shared__ float span_sum[256];
    __shared__ int chosen;
    const float* row = logits + (long)blockIdx.x * V;
    const float temp = temperature[blockIdx.x];
    const float inv_t = 1.f / temp;
    const int span = (V + 255) / 256;
    const int c0 = threadIdx.x * span;
    const int c1 = (c0 + span < V) ? c0 + span : V;
    float mx = -INFINITY;
    for (int c = c0; c < c1; ++c) mx = fmaxf(mx, row[c] * inv_t);
    mx = block_max(mx, red);
    float s = 0.f;
    for (int c = c0; c < c1; ++c) s += expf(row[c] * inv_t - mx);
    span_sum[threadIdx.x] = s;
    if (threadIdx.x == 0) chosen = -1;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int i = 0; i < 256; ++i) total += span_sum[i];
        const float target = uniform[blockIdx.x] * total;
        float run = 0.f;
        int pick = -1;
        for (int i = 0; i < 256 && pick < 0; ++i) {
            if (run + span_sum[i] > target) {
                const int b0 = i * span;
                const int b1 = (b0 + span < V) ? b0 + span : V;
                for (int c = b0; c < b1; ++c) {
                    run += expf(row[c] * inv_t - mx);
                    if (run > target) { pick = c; break; }
                }
                // not found after all (rounding): run now holds this span, go on to the next
            } else {
                run += span_sum[i];
            }
        }
        if (pick < 0) {  // target at or above the total after rounding: last token with weight
            pick = V - 1;
        }
        chosen = pick;
    }
    __syncthreads();
    if (threadIdx.x == 0) out[blockIdx.x] = chosen;
}

// Rows with temperature <= 0 must be given to qe_argmax by the caller.
extern "C" int qe_sample(const float* logits, const float* temperature, const float* uniform, int* out,
                         int R, int V, hipStream_t stream) {
    QE_REQUIRE(R >= 0 && V > 0, "sample: bad sizes R=%d V=%d", R, V);
    if (R == 0) return 0;
    sample_kernel<<<R, 256, 0, stream>>>(logits, temperature, uniform, out, V);
    QE_LAUNCH_CHECK();
    return 0;
}
