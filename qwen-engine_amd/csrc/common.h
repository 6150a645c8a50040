// Shared device helpers for the gfx950 kernels: element types, conversions,
// wave64 reductions and the error convention of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define QE_WAVE 64

// Element type codes used across the C ABI.
enum QeDtype { QE_F32 = 0, QE_BF16 = 1 };

// bfloat16 held as its 16 bits; conversions are explicit so that every rounding
// point is visible in the kernels.
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
    return __uint_as_float(((uint32_t)v.bits) << 16);
}
// One pair of a half-split rotation: (a, b) <- (c a - s b, s a + c b), with the roundings fixed (a
// product, then one fused multiply-add), so that every kernel that rotates gives the same bits.
__device__ __forceinline__ void rotate_pair(float c, float s, float& a, float& b) {
#pragma clang fp contract(off)
    const float x1 = a, x2 = b;
    const float sx2 = s * x2, cx2 = c * x2;
    a = __builtin_fmaf(c, x1, -sx2);
    b = __builtin_fmaf(s, x1, cx2);
}

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}
// round to nearest even; NaN stays NaN (the hardware conversion of gfx950, v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
    bf16_t r;
    r.bits = __builtin_bit_cast(unsigned short, (__bf16)f);
    return r;
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<bf16_t> {
    static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_float(*p); }
    static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = float_to_bf16(v); }
};

// Four consecutive elements as one 16-byte (float) or 8-byte (bfloat16) access.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 t = *(const float4*)p;
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
        *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <> struct Vec4<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
        const uint2 t = *(const uint2*)p;
        v[0] = bf16_bits_to_float(t.x & 0xffffu); v[1] = bf16_bits_to_float(t.x >> 16);
        v[2] = bf16_bits_to_float(t.y & 0xffffu); v[3] = bf16_bits_to_float(t.y >> 16);
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
        typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
        typedef __attribute__((ext_vector_type(4))) float floatx4_t;
        const floatx4_t f = {v[0], v[1], v[2], v[3]};
        *(bf16x4_t*)p = __builtin_convertvector(f, bf16x4_t);
    }
};

// v of this lane and of its partner across the wave's halves (lane ^ 32) or across odd and even
// rows of 16 lanes (lane ^ 16), by a swap between two vector registers.  (The two results are
// taken out of the returned pair into plain integers first: a bit cast applied to an element of
// the pair gave the first element for both.)
__device__ __forceinline__ void pair_across_halves(float v, float& mine, float& other) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const unsigned r0 = r[0], r1 = r[1];
    mine = __uint_as_float(r0);
    other = __uint_as_float(r1);
}
__device__ __forceinline__ void pair_across_rows(float v, float& mine, float& other) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const unsigned r0 = r[0], r1 = r[1];
    mine = __uint_as_float(r0);
    other = __uint_as_float(r1);
}
// (mine and other are this lane's and its partner's value in one order or the other, depending on
// the lane's half or row: sums and maxima do not care)

// Sum over the 16 lanes of a row (lanes 16 r .. 16 r + 15), every lane getting it: the lane pairs and
// the order are those of the butterfly `v += __shfl_xor(v, o)` for o = 8, 4, 2, 1 (a rotation by o
// meets the same partner sums, which repeat with period 2 o), so the result is the same to the
// bit, by four vector instructions instead of four trips through the LDS crossbar.
__device__ __forceinline__ float row16_sum(float v) {
#define QE_ROW_ROR(n_) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + (n_), 0xf, 0xf, false))
    v += QE_ROW_ROR(8);
    v += QE_ROW_ROR(4);
    v += QE_ROW_ROR(2);
    v += QE_ROW_ROR(1);
#undef QE_ROW_ROR
    return v;
}
// Sum and maximum over the 64 lanes of a wave, in every lane.  The partners and the order are those
// of the butterfly `v += __shfl_xor(v, o)` for o = 32, 16, 8, 4, 2, 1, so the sum is the same to the
// bit; but the halves of the wave and the odd and even rows of 16 lanes are exchanged by register
// swaps and the lanes of a row by rotations, where each `__shfl_xor` is a trip through the LDS
// crossbar of about 120 cycles that the next has to wait for.
__device__ __forceinline__ float wave_sum(float v) {
    float a, b;
    pair_across_halves(v, a, b);
    v = a + b;
    pair_across_rows(v, a, b);
    v = a + b;
    return row16_sum(v);
}
__device__ __forceinline__ float wave_max(float v) {
    float a, b;
    pair_across_halves(v, a, b);
    v = fmaxf(a, b);
    pair_across_rows(v, a, b);
    v = fmaxf(a, b);
    // (a lane whose partner is switched off gets its own value back: neutral for a maximum, as the 0 above is for a sum)
#define QE_ROW_ROR(n_) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, v), __builtin_bit_cast(int, v), 0x120 + (n_), 0xf, 0xf, false))
    v = fmaxf(v, QE_ROW_ROR(8));
    v = fmaxf(v, QE_ROW_ROR(4));
    v = fmaxf(v, QE_ROW_ROR(2));
    v = fmaxf(v, QE_ROW_ROR(1));
#undef QE_ROW_ROR
    return v;
}

// Block-wide sum for blocks of up to 1024 threads (a multiple of 64).
// `scratch` holds at least 16 floats of shared memory.  All threads get the sum.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wid] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nw; ++i) r += scratch[i];
    return r;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wid] = v;
    __syncthreads();
    float r = scratch[0];
    for (int i = 1; i < nw; ++i) r = fmaxf(r, scratch[i]);
    return r;
}

// ---- host side ---------------------------------------------------------------
// Entry points return 0 on success, a positive hipError_t, or -1 for an argument
// the kernels do not take; qe_last_error() then holds the reason.
extern "C" const char* qe_last_error();
void qe_set_error(const char* fmt, ...);
extern "C" int qe_compute_units();

#define QE_REQUIRE(cond, ...)                         \
    do {                                              \
        if (!(cond)) { qe_set_error(__VA_ARGS__); return -1; } \
    } while (0)

#define QE_LAUNCH_CHECK()                             \
    do {                                              \
        hipError_t e_ = hipGetLastError();            \
        if (e_ != hipSuccess) { qe_set_error("%s: %s", __func__, hipGetErrorString(e_)); return (int)e_; } \
    } while (0)

static inline int qe_cdiv(long a, long b) { return (int)((a + b - 1) / b); }
