// Device-side building blocks for gfx950: vector types, bf16/f16 conversion,
// 64-lane wave reductions and the MFMA tile wrappers with their lane layouts.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

namespace fla {

typedef __bf16 bf16;
typedef _Float16 f16;
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

template <typename T> struct Vec8;
template <> struct Vec8<bf16> { typedef bf16x8 type; };
template <> struct Vec8<f16> { typedef f16x8 type; };

__device__ __forceinline__ float to_f32(bf16 x) { return (float)x; }
__device__ __forceinline__ float to_f32(f16 x) { return (float)x; }
__device__ __forceinline__ float to_f32(float x) { return x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }

// bits of a bf16 pair packed into one dword: lo in [15:0], hi in [31:16]
__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
    bf16x2 p;
    p[0] = (bf16)lo;
    p[1] = (bf16)hi;
    return __builtin_bit_cast(unsigned, p);
}

// ---- wave-level reductions (xor butterflies through ds_bpermute-free DPP where the
// compiler can, __shfl_xor otherwise) ---------------------------------------
template <int WIDTH> __device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int off = WIDTH / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ float wave_inclusive_scan(float v) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        float n = __shfl_up(v, off, kWave);
        if (lane >= off) v += n;
    }
    return v;
}

// ---- MFMA wrappers ---------------------------------------------------------
// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] * B[32x16].
//   A operand: lane l holds A[l%16][8*(l/16) + e], e = 0..7
//   B operand: lane l holds B[8*(l/16) + e][l%16]
//   D / C    : lane l holds D[4*(l/16) + i][l%16], i = 0..3
__device__ __forceinline__ f32x4 mfma16x32(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// v_mfma_f32_16x16x16_bf16: A lane l holds A[l%16][4*(l/16)+e], B lane l holds
// B[4*(l/16)+e][l%16], e = 0..3; D as above.  A D tile rounded to bf16 is
// therefore directly the B operand (rows = contraction) of a following MFMA.
__device__ __forceinline__ f32x4 mfma16x16(bf16x4 a, bf16x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c,
                                                     0, 0, 0);
}

__device__ __forceinline__ bf16x4 cvt4(f32x4 v) {
    bf16x4 r;
    r[0] = (bf16)v[0];
    r[1] = (bf16)v[1];
    r[2] = (bf16)v[2];
    r[3] = (bf16)v[3];
    return r;
}
__device__ __forceinline__ bf16x8 cat8(bf16x4 lo, bf16x4 hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

}  // namespace fla
