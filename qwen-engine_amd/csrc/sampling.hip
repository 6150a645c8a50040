// Next-token choice on the device from 32-bit logits [R, V]: argmax (lowest index
// on ties) and temperature sampling by inverse CDF with one uniform per row.
#include "common.h"
#include "no_alloc.h"
#include <mutex>

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

// Two stages for wide vocabularies: each block of the first takes a contiguous span of a row
// and leaves its best (value, index); the second picks among the spans, lowest index on ties.
__global__ __launch_bounds__(256) void argmax_span_kernel(const float* __restrict__ logits, float* __restrict__ pv,
                                                          int* __restrict__ pi, int V, int span) {
    __shared__ float sv[256];
    __shared__ int si[256];
    const float* row = logits + (long)blockIdx.x * V;
    const int c0 = blockIdx.y * span;
    const int c1 = min(V, c0 + span);
    float best = -INFINITY;
    int bi = -1;
    for (int c = c0 + threadIdx.x; c < c1; c += 256) {
        const float v = row[c];
        if (bi < 0 || v > best) { best = v; bi = c; }
    }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            const float ov = sv[threadIdx.x + s], mv = sv[threadIdx.x];
            const int oi = si[threadIdx.x + s], mi = si[threadIdx.x];
            if (oi >= 0 && (mi < 0 || ov > mv || (ov == mv && oi < mi))) { sv[threadIdx.x] = ov; si[threadIdx.x] = oi; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        pv[blockIdx.x * gridDim.y + blockIdx.y] = sv[0];
        pi[blockIdx.x * gridDim.y + blockIdx.y] = si[0];
    }
}

__global__ __launch_bounds__(64) void argmax_pick_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                         int* __restrict__ out, int spans) {
    float best = -INFINITY;
    int bi = -1;
    for (int s = threadIdx.x; s < spans; s += 64) {
        const float v = pv[blockIdx.x * spans + s];
        const int i = pi[blockIdx.x * spans + s];
        if (i >= 0 && (bi < 0 || v > best || (v == best && i < bi))) { best = v; bi = i; }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (oi >= 0 && (bi < 0 || ov > best || (ov == best && oi < bi))) { best = ov; bi = oi; }
    }
    if (threadIdx.x == 0) out[blockIdx.x] = bi;
}

#define ARGMAX_SPAN 2048

// bytes of workspace that qe_argmax needs for these sizes (0: none)
extern "C" long qe_argmax_workspace_bytes(int R, int V) {
    if (V <= 2 * ARGMAX_SPAN) return 0;
    return (long)R * qe_cdiv(V, ARGMAX_SPAN) * 8;
}

extern "C" int qe_argmax(const float* logits, int* out, int R, int V, void* workspace, long workspace_bytes,
                         hipStream_t stream) {
    QE_REQUIRE(R >= 0 && V > 0, "argmax: bad sizes R=%d V=%d", R, V);
    if (R == 0) return 0;
    if (V <= 2 * ARGMAX_SPAN) {
        argmax_kernel<<<R, 256, 0, stream>>>(logits, out, V);
    } else {
        const int spans = qe_cdiv(V, ARGMAX_SPAN);
        QE_REQUIRE(workspace && workspace_bytes >= (long)R * spans * 8, "argmax: workspace too small");
        QE_REQUIRE(spans <= 65535, "argmax: vocabulary too wide");
        float* pv = (float*)workspace;
        int* pi = (int*)(pv + (long)R * spans);
        argmax_span_kernel<<<dim3(R, spans), 256, 0, stream>>>(logits, pv, pi, V, ARGMAX_SPAN);
        argmax_pick_kernel<<<R, 64, 0, stream>>>(pv, pi, out, spans);
    }
    QE_LAUNCH_CHECK();
    return 0;
}

// ---- argmax for callers that cannot allocate ----------------------------------------------------
// The two-stage argmax keeps each span's best (value, index) in device memory between its two
// kernels.  qe_argmax takes that memory from the caller; qe_argmax_static keeps it in an array that
// is part of the loaded library, one copy on every GPU, so the call allocates nothing.  In host code
// the array's name is only a handle: the address the kernels get is asked for once per device
// with hipGetSymbolAddress and kept.
static __device__ __align__(256) unsigned char scratch[QE_ARGMAX_STATIC_BYTES];

#define QE_MAX_DEVICES 64
static void* g_scratch_ptr[QE_MAX_DEVICES];      // per device: the address of its copy of `scratch`
static std::mutex g_scratch_mutex;

// The current device's copy of the array (null and an error text if the runtime refuses).
static void* static_scratch_of_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= QE_MAX_DEVICES) {
        qe_set_error("argmax (static): no current device, or device %d beyond %d", dev, QE_MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            qe_set_error("argmax (static): hipGetSymbolAddress: %s", hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

extern "C" long qe_argmax_static_max_bytes() { return QE_ARGMAX_STATIC_BYTES; }

extern "C" int qe_argmax_static(const float* logits, int* out, int R, int V, hipStream_t stream) {
    QE_REQUIRE(R >= 0 && V > 0, "argmax (static): bad sizes R=%d V=%d", R, V);
    if (R == 0) return 0;
    const long need = qe_argmax_workspace_bytes(R, V);
    QE_REQUIRE(need <= (long)QE_ARGMAX_STATIC_BYTES,
               "argmax (static): R=%d rows of V=%d need %ld bytes between the two stages, the static buffer has %ld "
               "(use qe_argmax with a workspace)", R, V, need, (long)QE_ARGMAX_STATIC_BYTES);
    void* ws = nullptr;
    if (need > 0) {
        ws = static_scratch_of_current_device();
        if (!ws) return -1;
    }
    // (nothing has to start at zero: the first stage writes every entry that the second reads)
    return qe_argmax(logits, out, R, V, ws, need, stream);
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
        if (pick < 0) {  // target at or above the total after rounding: the last token with weight
            pick = V - 1;
            while (pick > 0 && !(expf(row[pick] * inv_t - mx) > 0.f)) --pick;
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
