// Device-side building blocks shared by the gfx950 kernels: vector types, the bf16
// 16x16x32 MFMA wrapper with its register layout, 64-lane reductions, bf16 rounding.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace llsa {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int kWave = 64;        // CDNA wavefront
constexpr int kBlk = 16;         // tokens per block (block_size of the operator)
constexpr int kD = 64;           // head dimension the MFMA kernels are specialised for
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kScale = 0.125f;                          // 1/sqrt(kD)
constexpr float kScaleLog2e = 0.125f * 1.4426950408889634f;

// v_mfma_f32_16x16x32_bf16:  D(16x16) = A(16x32) * B(32x16) + C.
//   lane l supplies  A[row = l%16][k = 8*(l/16) + e]   e = 0..7
//                    B[k = 8*(l/16) + e][col = l%16]
//   and owns         D[row = 4*(l/16) + e][col = l%16] e = 0..3
// Both operands are "8 consecutive k for one row/column", i.e. a 16-byte load from a
// row-major matrix whose fast axis is the contraction axis.
__device__ __forceinline__ f32x4 mfma_bf16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 ld16(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 ld8(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }
__device__ __forceinline__ void st16(bf16* p, bf16x8 v) { *reinterpret_cast<bf16x8*>(p) = v; }
__device__ __forceinline__ void st8(bf16* p, bf16x4 v) { *reinterpret_cast<bf16x4*>(p) = v; }

__device__ __forceinline__ bf16x8 cat(bf16x4 lo, bf16x4 hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16)0.0f;
    return z;
}
__device__ __forceinline__ bf16x4 zero4() {
    bf16x4 z;
#pragma unroll
    for (int i = 0; i < 4; i++) z[i] = (bf16)0.0f;
    return z;
}
__device__ __forceinline__ bf16x4 cvt4(f32x4 v) {
    bf16x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = (bf16)v[i];
    return r;
}

// round-to-nearest-even through bf16, value kept in fp32
__device__ __forceinline__ float rn_bf16(float x) { return (float)(bf16)x; }

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// reductions over the four lanes {l, l^16, l^32, l^48} that share one MFMA column
__device__ __forceinline__ float quad_max(float v) {
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}
__device__ __forceinline__ float quad_sum(float v) {
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

}  // namespace llsa
