// LDS-tile <-> MFMA-operand plumbing for the chunk kernels (gfx950).
//
// All matrix products use v_mfma_f32_16x16x32_bf16 with ONE fixed assignment of
// the 32 contraction indices of a step to the 8 operand slots of a lane
// ("split" mapping):
//     lane l = 16*g + i,  slot e:   c(g,e) = 4*g + e          for e < 4
//                                   c(g,e) = 16 + 4*g + e - 4  for e >= 4
// Any permutation works as long as both operands use the same one; this one is
// chosen because
//   * a pair of 16x16 accumulator tiles (lane holds rows 4g..4g+3 of column i)
//     rounded to bf16 IS an operand in this mapping (rows = contraction), so
//     products can be chained through registers;
//   * an LDS tile whose contraction index is the contiguous dimension is read
//     with two 8-byte loads (frag_kc);
//   * an LDS tile whose contraction index is the ROW dimension is read with two
//     ds_read_b64_tr_b16 transposing loads (frag_tr), so no tile is ever
//     transposed explicitly.
#pragma once

#include "device_utils.h"

namespace fla {

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
__device__ __forceinline__ int wave_id() { return threadIdx.x >> 6; }

// ds_read_b64_tr_b16: within each group of 16 lanes, lane s supplies the address
// of 4 consecutive 16-bit elements; lane i receives element (i % 4) of lanes
// i/4, i/4 + 4, i/4 + 8, i/4 + 12.
__device__ __forceinline__ elemx4 lds_tr4(const elem *p) {
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)p);
    return __builtin_bit_cast(elemx4, r);
}

// Operand with rows r0..r0+15 and contraction c0..c0+31 along the contiguous
// dimension of `tile` (pitch in elements).
// The two 8-byte halves stay separate LDS reads: fused into one two-address read (ds_read2_b64) the pair
// costs four times the LDS cycles on gfx950, which is why this library is built with the load/store
// merging pass of the backend switched off.
__device__ __forceinline__ elemx8 frag_kc(const elem *tile, int pitch, int r0, int c0) {
    const int l = lane_id(), i = l & 15, g = l >> 4;
    const int off = (r0 + i) * pitch + c0 + 4 * g;
    return cat8(*reinterpret_cast<const elemx4 *>(tile + off), *reinterpret_cast<const elemx4 *>(tile + off + 16));
}
// 16-wide contraction variant for v_mfma_f32_16x16x16_bf16.
__device__ __forceinline__ elemx4 frag_kc4(const elem *tile, int pitch, int r0, int c0) {
    const int l = lane_id(), i = l & 15, g = l >> 4;
    return *reinterpret_cast<const elemx4 *>(tile + (r0 + i) * pitch + c0 + 4 * g);
}

// Operand with index r0..r0+15 along the contiguous dimension and contraction
// c0..c0+31 along the rows of `tile`:  slot (g,e) = tile[c0 + c(g,e)][r0 + i].
__device__ __forceinline__ elemx8 frag_tr(const elem *tile, int pitch, int r0, int c0) {
    const int l = lane_id(), i = l & 15, g = l >> 4;
    const elem *p = tile + (c0 + 4 * g + (i >> 2)) * pitch + r0 + 4 * (i & 3);
    return cat8(lds_tr4(p), lds_tr4(p + 16 * pitch));
}
__device__ __forceinline__ elemx4 frag_tr4(const elem *tile, int pitch, int r0, int c0) {
    const int l = lane_id(), i = l & 15, g = l >> 4;
    return lds_tr4(tile + (c0 + 4 * g + (i >> 2)) * pitch + r0 + 4 * (i & 3));
}

// Two accumulator tiles (rows 0..15 and 16..31 of a 32-row block) as an operand
// whose contraction runs over those rows.
__device__ __forceinline__ elemx8 frag_from_acc(f32x4 lo, f32x4 hi) { return cat8(cvt4(lo), cvt4(hi)); }

// Accumulator tile element e of lane l sits at row 4*(l/16)+e, column l%16.
__device__ __forceinline__ int acc_row(int e) { return 4 * (lane_id() >> 4) + e; }
__device__ __forceinline__ int acc_col() { return lane_id() & 15; }

// ---- the hand-off type of the KDA forward ---------------------------------------------------------
// u = Akk (v beta) and kg = k 2^{g_last - g} pass from the chunk-parallel kernel to the state scan, and v_new enters
// the state update, as fp16 whatever the element type: with 8 significand bits (bf16) each of the three roundings
// alone moves the fp32 final state by about 2e-3 of its scale, with 11 bits all three together stay below 4e-4.
// Values beyond the fp16 range saturate instead of turning into infinities.
typedef f16 fine;
typedef f16 finex2 __attribute__((ext_vector_type(2)));
typedef f16x4 finex4;
typedef f16x8 finex8;
#ifdef FLA_ELEM_F16
constexpr bool kFineIsElem = true;
#else
constexpr bool kFineIsElem = false;
#endif
__device__ __forceinline__ unsigned cvt2_fine(float a, float b) {
    const f32x2 v = {__builtin_amdgcn_fmed3f(a, -65504.f, 65504.f), __builtin_amdgcn_fmed3f(b, -65504.f, 65504.f)};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, finex2));
}
// Without the saturation, for values bounded by an input of the caller: q and k times a decay factor <= 1 (the gated
// operands qg, kg).  |q|, |k| beyond 65504 would turn into infinities here.
__device__ __forceinline__ unsigned cvt2_fine_bounded(float a, float b) {
    const f32x2 v = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, finex2));
}
__device__ __forceinline__ finex4 cvt4_fine(f32x4 v) {
    u32x2 t;
    t[0] = cvt2_fine(v[0], v[1]);
    t[1] = cvt2_fine(v[2], v[3]);
    return __builtin_bit_cast(finex4, t);
}
__device__ __forceinline__ finex8 fine_from_acc(f32x4 lo, f32x4 hi) {
    return __builtin_shufflevector(cvt4_fine(lo), cvt4_fine(hi), 0, 1, 2, 3, 4, 5, 6, 7);
}
// tiles of `fine` values live in LDS behind elem pointers (both are 16 bits wide); these reinterpret what was read
__device__ __forceinline__ finex8 as_fine(elemx8 x) { return __builtin_bit_cast(finex8, x); }
__device__ __forceinline__ finex4 as_fine(elemx4 x) { return __builtin_bit_cast(finex4, x); }
__device__ __forceinline__ elemx8 fine_to_elem(finex8 x) {
    if constexpr (kFineIsElem) {
        return __builtin_bit_cast(elemx8, x);
    } else {
        f32x4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo[e] = (float)x[e];
            hi[e] = (float)x[4 + e];
        }
        return frag_from_acc(lo, hi);
    }
}
// Operand pairs that are `fine` values when F is set and elements otherwise, both carried as elemx8 bit patterns.
template <bool F> __device__ __forceinline__ elemx8 pack_operand(f32x4 lo, f32x4 hi) {
    if constexpr (F) return __builtin_bit_cast(elemx8, fine_from_acc(lo, hi));
    else return frag_from_acc(lo, hi);
}
template <bool F> __device__ __forceinline__ f32x4 mfma16x32_as(elemx8 a, elemx8 b, f32x4 c) {
    if constexpr (F) return mfma16x32(as_fine(a), as_fine(b), c);
    else return mfma16x32(a, b, c);
}

// ---- cooperative global <-> LDS tile copies (all threads of the block) -----------
// Copies rows [0, valid) x cols [0, ncols) of a row-major global matrix (row stride
// `gstride` elements, 16-byte aligned rows) into `tile`; rows [valid, nrows) are zeroed.
// A tile copy is split into fetch (global -> registers) and commit (registers -> LDS) so that a caller
// can issue the loads of all its tiles before the first commit waits for any of them.  Rows past
// `valid` re-read the last valid row and are zeroed by a select: a predicated load would be waited for
// inside its own branch, one memory round trip per piece.  `tid` is the thread's index among the
// THREADS threads that copy; NROWS x NCOLS must be a multiple of 8 * THREADS.
template <int THREADS, int NROWS, int NCOLS> struct TileCopy {
    static constexpr int CPR = NCOLS / 8;                    // 16-byte pieces per row
    static constexpr int N = NROWS * CPR / THREADS;          // pieces per thread
    static_assert(NROWS * CPR % THREADS == 0, "tile does not divide among the copying threads");
    u32x4 r[N];
    __device__ __forceinline__ void fetch(const elem *gsrc, int64_t gstride, int valid, int tid) {
        const int last = valid > 0 ? valid - 1 : 0;
#pragma unroll
        for (int m = 0; m < N; ++m) {
            const int idx = m * THREADS + tid;
            const int row = idx / CPR, c = (idx % CPR) << 3;
            // 32-bit element offset from the (uniform) tile base: a tile spans 64 rows of a stride the host
            // checks to be below 2^24 elements, and the load keeps its base in scalar registers
            const unsigned off = (unsigned)((row < valid ? row : last) * (int)gstride + c);
            r[m] = *reinterpret_cast<const u32x4 *>(gsrc + off);
        }
    }
    // the pieces were fetched from a tensor of `fine` values and are to be committed as elements
    __device__ __forceinline__ void to_elem() {
#pragma unroll
        for (int m = 0; m < N; ++m) r[m] = __builtin_bit_cast(u32x4, fine_to_elem(__builtin_bit_cast(finex8, r[m])));
    }
    __device__ __forceinline__ void commit(elem *tile, int pitch, int valid, int tid) const {
#pragma unroll
        for (int m = 0; m < N; ++m) {
            const int idx = m * THREADS + tid;
            const int row = idx / CPR, c = (idx % CPR) << 3;
            *reinterpret_cast<u32x4 *>(tile + row * pitch + c) = row < valid ? r[m] : u32x4{0u, 0u, 0u, 0u};
        }
    }
};
template <int THREADS>
__device__ __forceinline__ void load_tile(elem *tile, int pitch, const elem *gsrc, int64_t gstride, int nrows,
                                          int ncols, int valid, int tid) {
    const int cpr = ncols >> 3;  // 16-byte chunks per row
    const int total = nrows * cpr;
    const int last = valid > 0 ? valid - 1 : 0;
#pragma unroll
    for (int idx0 = 0; idx0 < total; idx0 += THREADS) {
        const int idx = idx0 + tid;
        if (idx < total) {
            const int r = idx / cpr, c = (idx % cpr) << 3;
            u32x4 v = *reinterpret_cast<const u32x4 *>(gsrc + (unsigned)((r < valid ? r : last) * (int)gstride + c));
            if (r >= valid) v = u32x4{0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4 *>(tile + r * pitch + c) = v;
        }
    }
}
template <int THREADS>
__device__ __forceinline__ void load_tile(elem *tile, int pitch, const elem *gsrc, int64_t gstride, int nrows,
                                          int ncols, int valid) {
    load_tile<THREADS>(tile, pitch, gsrc, gstride, nrows, ncols, valid, (int)threadIdx.x);
}
template <int THREADS>
__device__ __forceinline__ void store_tile(elem *gdst, int64_t gstride, const elem *tile, int pitch, int ncols,
                                           int valid) {
    const int cpr = ncols >> 3;
    for (int idx = threadIdx.x; idx < valid * cpr; idx += THREADS) {
        const int r = idx / cpr, c = (idx % cpr) << 3;
        *reinterpret_cast<u32x4 *>(gdst + (int64_t)r * gstride + c) = *reinterpret_cast<const u32x4 *>(tile + r * pitch + c);
    }
}

// Writes one accumulator tile, rounded to bf16, into a row-major LDS tile at (r0, c0).
// Neighbouring lanes hold neighbouring columns; they swap half of their values so that every
// lane writes two whole dwords (even lanes rows e = 0,1; odd lanes rows e = 2,3 of the column
// pair) instead of four 16-bit pieces, which also keeps the write free of bank conflicts.
// packed_to_tile takes the tile already rounded: p01 = rows 4lg, 4lg + 1 and p23 = rows 4lg + 2, 4lg + 3 of the lane's
// column, two elements per dword.
__device__ __forceinline__ void packed_to_tile(elem *tile, int pitch, int r0, int c0, unsigned p01, unsigned p23) {
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const bool odd = li & 1;
    const unsigned send = odd ? p01 : p23;
    const unsigned recv = (unsigned)__builtin_amdgcn_mov_dpp((int)send, 0xB1, 0xf, 0xf, true);  // lane ^ 1
    const unsigned left = odd ? recv : p01;    // column li & ~1
    const unsigned right = odd ? p23 : recv;   // column li | 1
    elem *dst = tile + (r0 + 4 * lg + (odd ? 2 : 0)) * pitch + c0 + (li & ~1);
    *reinterpret_cast<unsigned *>(dst) = __builtin_amdgcn_perm(right, left, 0x05040100u);          // low halves
    *reinterpret_cast<unsigned *>(dst + pitch) = __builtin_amdgcn_perm(right, left, 0x07060302u);  // high halves
}
__device__ __forceinline__ void acc_to_tile(elem *tile, int pitch, int r0, int c0, f32x4 acc) {
    packed_to_tile(tile, pitch, r0, c0, __builtin_bit_cast(unsigned, cvt2(acc[0], acc[1])),
                   __builtin_bit_cast(unsigned, cvt2(acc[2], acc[3])));
}

// One accumulator tile, rounded to bf16, straight to global memory (rows r0.. of a row-major matrix with
// `stride` bytes between rows; `base` points at column c0 of row 0).  Lane pairs exchange halves as in
// acc_to_tile so that every lane writes two whole dwords.  packed_to_global takes the tile already rounded:
// p01 = rows 4lg, 4lg + 1 and p23 = rows 4lg + 2, 4lg + 3 of the lane's column, two elements per dword.
__device__ __forceinline__ void packed_to_global(char *base, int64_t stride, int r0, int len, unsigned p01, unsigned p23) {
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const bool odd = li & 1;
    const unsigned send = odd ? p01 : p23;
    const unsigned recv = (unsigned)__builtin_amdgcn_mov_dpp((int)send, 0xB1, 0xf, 0xf, true);  // lane ^ 1
    const unsigned left = odd ? recv : p01, right = odd ? p23 : recv;
    const int row = r0 + 4 * lg + (odd ? 2 : 0);
    char *dst = base + row * stride + (li & ~1) * 2;
    if (row < len) *reinterpret_cast<unsigned *>(dst) = __builtin_amdgcn_perm(right, left, 0x05040100u);
    if (row + 1 < len) *reinterpret_cast<unsigned *>(dst + stride) = __builtin_amdgcn_perm(right, left, 0x07060302u);
}
__device__ __forceinline__ void acc_to_global(char *base, int64_t stride, int r0, int len, f32x4 acc) {
    packed_to_global(base, stride, r0, len, __builtin_bit_cast(unsigned, cvt2(acc[0], acc[1])),
                     __builtin_bit_cast(unsigned, cvt2(acc[2], acc[3])));
}

// ---- tiles of `fine` values ------------------------------------------------------------------------
__device__ __forceinline__ void acc_to_tile_fine(elem *tile, int pitch, int r0, int c0, f32x4 acc) {
    packed_to_tile(tile, pitch, r0, c0, cvt2_fine(acc[0], acc[1]), cvt2_fine(acc[2], acc[3]));
}
// store_tile for a tile of `fine` values that leaves as the element type
template <int THREADS>
__device__ __forceinline__ void store_tile_fine_as_elem(elem *gdst, int64_t gstride, const elem *tile, int pitch, int ncols,
                                                        int valid) {
    const int cpr = ncols >> 3;
    for (int idx = threadIdx.x; idx < valid * cpr; idx += THREADS) {
        const int r = idx / cpr, c = (idx % cpr) << 3;
        *reinterpret_cast<elemx8 *>(gdst + (int64_t)r * gstride + c) =
            fine_to_elem(*reinterpret_cast<const finex8 *>(tile + r * pitch + c));
    }
}

// ---- the k tile -------------------------------------------------------------------------------
// The k tile is read both ways (contraction along columns for k k^T and q k^T, along rows for
// k^T v and the right-hand sides).  No padding keeps both patterns conflict free, an XOR swizzle
// of the 16-byte column chunks does: chunk c of row r is stored at chunk c ^ f(r),
// f(r) = 2*(r % 8) + (r / 8) % 2.  Sixteen consecutive rows get sixteen different f (column-wise
// reads of one chunk hit 16 different bank groups); eight consecutive rows get eight different
// f >> 1 (row-wise reads of a chunk pair hit 8 different bank-group pairs).  K = 64 rows are too
// short for the swizzle and use a padded pitch instead.
template <int K> struct KTile {
    static constexpr int pitch = K == 128 ? 128 : K + 16;
    static __device__ __forceinline__ int f(int r) { return ((r & 7) << 1) | ((r >> 3) & 1); }
    static __device__ __forceinline__ int off(int r, int col) {  // element offset of (row r, column col)
        if (K == 128) return r * 128 + ((((col >> 3) ^ f(r)) << 3) | (col & 7));
        return r * pitch + col;
    }
    static __device__ __forceinline__ elemx8 kc(const elem *t, int r0, int c0) {
        const int l = lane_id(), i = l & 15, g = l >> 4;
        return cat8(*reinterpret_cast<const elemx4 *>(t + off(r0 + i, c0 + 4 * g)),
                    *reinterpret_cast<const elemx4 *>(t + off(r0 + i, c0 + 16 + 4 * g)));
    }
    static __device__ __forceinline__ elemx4 tr4(const elem *t, int r0, int c0) {
        const int l = lane_id(), i = l & 15, g = l >> 4;
        return lds_tr4(t + off(c0 + 4 * g + (i >> 2), r0 + 4 * (i & 3)));
    }
    static __device__ __forceinline__ elemx8 tr(const elem *t, int r0, int c0) {
        const int l = lane_id(), i = l & 15, g = l >> 4;
        return cat8(lds_tr4(t + off(c0 + 4 * g + (i >> 2), r0 + 4 * (i & 3))),
                    lds_tr4(t + off(c0 + 16 + 4 * g + (i >> 2), r0 + 4 * (i & 3))));
    }
};

}  // namespace fla
