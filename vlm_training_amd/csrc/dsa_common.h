// Shared device helpers for the gfx950 DSA attention kernels (wave64, MFMA, LDS).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define DSA_WAVE 64
#define LOG2E_F 1.4426950408889634f
#define LN2_F 0.6931471805599453f

// MFMA operand layouts used throughout (wave64, lane l):
//   16x16x32 bf16:  A[i][k]: i = l%16, k = 8*(l/16)+e (e<8)   B[k][j]: j = l%16, k = 8*(l/16)+e
//                   C[i][j]: j = l%16, i = 4*(l/16)+v (v<4)
//   32x32x16 bf16:  A[i][k]: i = l%32, k = 8*(l/32)+e         B[k][j]: j = l%32, k = 8*(l/32)+e
//                   C[i][j]: j = l%32, i = 8*(v/4) + 4*(l/32) + v%4 (v<16)
__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 zero_bf16x8() {
    u32x4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8, z);
}
__device__ __forceinline__ bf16x8 load_bf16x8(const bf16_t *p) {   // 16-byte aligned global/LDS read
    return *reinterpret_cast<const bf16x8 *>(p);
}

// two fp32 -> packed bf16 pair, round-to-nearest-even (one v_cvt_pk_bf16_f32 on gfx950)
// acc + sum_e a[e] * b[e] over 8 bf16 pairs, one fused multiply-add per element in element order.  Every kernel that forms
// delta = rowsum(dO * O) goes through this one chain, so that they agree to the bit.
__device__ __forceinline__ float dot8_chain(bf16x8 a, bf16x8 b, float acc) {
    const u32x4 x = __builtin_bit_cast(u32x4, a), y = __builtin_bit_cast(u32x4, b);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        acc = __builtin_fmaf(__uint_as_float(x[e] << 16), __uint_as_float(y[e] << 16), acc);
        acc = __builtin_fmaf(__uint_as_float(x[e] & 0xffff0000u), __uint_as_float(y[e] & 0xffff0000u), acc);
    }
    return acc;
}

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2bf(float lo, float hi) {
    const f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// segment lookup: index i with cu[i] <= t < cu[i+1] (zero-length segments are stepped over)
__device__ __forceinline__ int find_segment(const int32_t *__restrict__ cu, int N, int t) {
    int lo = 0, hi = N;            // invariant: cu[lo] <= t < cu[hi]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if (cu[mid] <= t) lo = mid; else hi = mid;
    }
    return lo;
}

__device__ __forceinline__ float wave_xor_f(float v, int m) { return __shfl_xor(v, m, 64); }
// maximum / sum over the two lanes 32 apart, on every lane: v_permlane32_swap exchanges the wave's halves in
// the vector ALU (no LDS round trip, so LDS reads in flight are not waited for)
__device__ __forceinline__ float half_max_f(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum_f(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
