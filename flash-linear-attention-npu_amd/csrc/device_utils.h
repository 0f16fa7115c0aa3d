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
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
// Element type of the matrix operands of a translation unit: bf16, or f16 when the file is built with
// -DFLA_ELEM_F16 (the matrix-core kernels are compiled once per element type).
#ifdef FLA_ELEM_F16
typedef f16 elem;
#else
typedef bf16 elem;
#endif
typedef elem elemx2 __attribute__((ext_vector_type(2)));
typedef elem elemx4 __attribute__((ext_vector_type(4)));
typedef elem elemx8 __attribute__((ext_vector_type(8)));
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
// Sum over aligned groups of WIDTH lanes, result in every lane of the group.  Up to 16 lanes the
// butterfly runs on data-parallel-primitive adds (quad swaps, then the two mirrors, which pair every
// lane with one of the other half), 32 lanes add one LDS-crossbar swizzle (lane ^ 16); wider or odd
// widths fall back to generic shuffles.
#define FLA_DPP_XADD(v, ctrl) \
    ((v) + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xf, 0xf, true)))
template <int WIDTH> __device__ __forceinline__ float group_sum(float v) {
    if constexpr (WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16 || WIDTH == 32) {
        v = FLA_DPP_XADD(v, 0xB1);                          // quad_perm [1,0,3,2]
        if constexpr (WIDTH >= 4) v = FLA_DPP_XADD(v, 0x4E);   // quad_perm [2,3,0,1]
        if constexpr (WIDTH >= 8) v = FLA_DPP_XADD(v, 0x141);  // row_half_mirror
        if constexpr (WIDTH >= 16) v = FLA_DPP_XADD(v, 0x140); // row_mirror
        if constexpr (WIDTH == 32)
            v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
        return v;
    } else {
#pragma unroll
        for (int off = WIDTH / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
        return v;
    }
}
#undef FLA_DPP_XADD

// Inclusive prefix sum over the 64 lanes of a wave with data-parallel-primitive moves: four
// shifts inside each row of 16 lanes (sources outside the row read 0), then lane 15 of rows 0 / 2
// broadcast into rows 1 / 3 and lane 31 into rows 2 and 3.
#define FLA_DPP_ADD(v, ctrl, row_mask) \
    ((v) + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), (row_mask), 0xf, true)))
__device__ __forceinline__ float wave_inclusive_scan(float v) {
    v = FLA_DPP_ADD(v, 0x111, 0xf);  // row_shr:1
    v = FLA_DPP_ADD(v, 0x112, 0xf);  // row_shr:2
    v = FLA_DPP_ADD(v, 0x114, 0xf);  // row_shr:4
    v = FLA_DPP_ADD(v, 0x118, 0xf);  // row_shr:8
    v = FLA_DPP_ADD(v, 0x142, 0xa);  // row_bcast:15 into rows 1 and 3
    v = FLA_DPP_ADD(v, 0x143, 0xc);  // row_bcast:31 into rows 2 and 3
    return v;
}
#undef FLA_DPP_ADD
__device__ __forceinline__ float read_lane(float v, int lane) {  // lane must be wave-uniform
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// ---- MFMA wrappers ---------------------------------------------------------
// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] * B[32x16].
//   A operand: lane l holds A[l%16][8*(l/16) + e], e = 0..7
//   B operand: lane l holds B[8*(l/16) + e][l%16]
//   D / C    : lane l holds D[4*(l/16) + i][l%16], i = 0..3
__device__ __forceinline__ f32x4 mfma16x32(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16x32(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
// v_mfma_f32_16x16x16_bf16: A lane l holds A[l%16][4*(l/16)+e], B lane l holds
// B[4*(l/16)+e][l%16], e = 0..3; D as above.  A D tile rounded to the element type is
// therefore directly the B operand (rows = contraction) of a following MFMA.
__device__ __forceinline__ f32x4 mfma16x16(bf16x4 a, bf16x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c,
                                                     0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma16x16(f16x4 a, f16x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
}

// fp32 -> element type (round to nearest even), two values per packed conversion
__device__ __forceinline__ elemx2 cvt2(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_convertvector(v, elemx2);
}
// The two packed halves are joined as integers: joined as element vectors the optimiser folds them into
// one four-wide conversion, which the backend then splits into four scalar conversions plus permutes.
__device__ __forceinline__ elemx4 cvt4(f32x4 v) {
    u32x2 t;
    t[0] = __builtin_bit_cast(unsigned, cvt2(v[0], v[1]));
    t[1] = __builtin_bit_cast(unsigned, cvt2(v[2], v[3]));
    return __builtin_bit_cast(elemx4, t);
}
// x = hi + lo with hi = elem(x) and lo = elem(x - hi).
__device__ __forceinline__ void split_hilo(f32x4 x, elemx4 &hi, elemx4 &lo) {
#ifdef FLA_ELEM_F16
    hi = cvt4(x);
    f32x4 rem;
#pragma unroll
    for (int e = 0; e < 4; ++e) rem[e] = x[e] - (float)hi[e];
    lo = cvt4(rem);
#else
    // The remainder is formed from the packed conversion's bit pattern (a bf16 is the upper half of an
    // fp32), never by extracting vector elements: element extraction makes the optimiser split the packed
    // conversion into four scalar ones plus permutes.
    const elemx2 h01 = cvt2(x[0], x[1]), h23 = cvt2(x[2], x[3]);
    const unsigned u01 = __builtin_bit_cast(unsigned, h01), u23 = __builtin_bit_cast(unsigned, h23);
    f32x4 rem;
    rem[0] = x[0] - __builtin_bit_cast(float, u01 << 16);
    rem[1] = x[1] - __builtin_bit_cast(float, u01 & 0xffff0000u);
    rem[2] = x[2] - __builtin_bit_cast(float, u23 << 16);
    rem[3] = x[3] - __builtin_bit_cast(float, u23 & 0xffff0000u);
    u32x2 t;
    t[0] = u01;
    t[1] = u23;
    hi = __builtin_bit_cast(elemx4, t);
    lo = cvt4(rem);
#endif
}
// Persistent scans launch a (slabs, heads, sequences) grid: the `slabs` workgroups of one (sequence, head) chain read
// the same key-side operands.  Workgroups are handed to the eight XCDs in turn (linear id % 8), each XCD with an L2 of
// its own, so ids L, L + 8, ... go to one chain and its second and later reads of those operands hit that L2.
// For kernels whose LDS footprint or launch shape leaves two waves on a SIMD whatever their register count: tells the
// compiler that keeping registers low buys no occupancy, so that it schedules for latency instead.
#define FLA_TWO_WAVES_PER_SIMD __attribute__((amdgpu_waves_per_eu(2, 2)))

__device__ __forceinline__ void chain_of_block(int &slab, int &head, int &seq) {
    const int slabs = gridDim.x, heads = gridDim.y, total = slabs * heads * gridDim.z;
    const int lin = blockIdx.x + slabs * (blockIdx.y + heads * blockIdx.z);
    int chain;
    if (slabs > 1 && total % (8 * slabs) == 0) {
        chain = (lin / (8 * slabs)) * 8 + (lin & 7);
        slab = (lin >> 3) % slabs;
    } else {
        chain = lin / slabs;
        slab = lin % slabs;
    }
    head = chain % heads;
    seq = chain / heads;
}

// Workgroup barrier that orders LDS traffic only: the wave waits for its own LDS operations, not for its global loads
// and stores, which stay in flight across the barrier.  For data handed over through LDS while prefetches are pending.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ elemx8 cat8(elemx4 lo, elemx4 hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

}  // namespace fla
