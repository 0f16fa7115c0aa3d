// Inversion of I + A for a strictly lower 64 x 64 block on the matrix cores, shared by the kernels that form the
// block themselves (solve_tri, the fused kkt + inverse, and the WY backward that rebuilds A from k, g and beta).
#pragma once

#include "mfma_tiles.h"

namespace fla {

// 64 x 64 blocks on the matrix cores: four waves, wave R inverts diagonal block R and then fills column block R
// of the inverse.  (I + A)^-1 of a strictly lower 16 x 16 block is the finite product (I - A)(I + A^2)(I + A^4)
// (I + A^8); the blocks below the diagonal follow by block substitution, X_rc = -D_r sum_m A_rm X_mc, with both
// operands of those products carried as a 16-bit head plus remainder.
__device__ __forceinline__ f32x4 solve_lds4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
__device__ __forceinline__ f32x4 solve_mm3(f32x4 a, f32x4 b, f32x4 acc) {   // acc += a b without the lo * lo term
    elemx4 ah, al, bh, bl;
    split_hilo(a, ah, al);
    split_hilo(b, bh, bl);
    acc = mfma16x16(ah, bh, acc);
    acc = mfma16x16(al, bh, acc);
    acc = mfma16x16(ah, bl, acc);
    return acc;
}

// Column block R of the inverse below its diagonal block, top to bottom: X[k] = block (R + k, R).
template <int R>
__device__ __forceinline__ void invert64_column(const float *aS, elem *oS) {
    constexpr int pa = 68, pb = 72;
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 X[4 - R];
#pragma unroll
    for (int e = 0; e < 4; ++e) X[0][e] = aS[(16 * R + 4 * lg + e) * pa + 16 * R + li];
#pragma unroll
    for (int k = 1; k < 4 - R; ++k) {
        const int r = R + k;
        f32x4 sum = zero;
#pragma unroll
        for (int j = 0; j < k; ++j)
            sum = solve_mm3(solve_lds4(aS + (16 * r + li) * pa + 16 * (R + j) + 4 * lg), X[j], sum);
        const f32x4 dinv = solve_lds4(aS + (16 * r + li) * pa + 16 * r + 4 * lg);
        X[k] = solve_mm3(-dinv, sum, zero);
        acc_to_tile(oS, pb, 16 * r, 16 * R, X[k]);
    }
}

// Rows 16 W .. 16 W + 15 of strict_lower(beta_t e^{g_t - g_s} <k_t, k_s>), rounded to the element type as solve_tri
// rounds its input (chunk_scaled_dot_kkt/README.md:8-15): acc[J][e] is entry (t = 16 W + acc_col(), s = 16 J + acc_row(e)).
// W is the calling wave's index as a compile-time value, so its W + 1 column tiles advance together through the
// contraction instead of one branch per tile.
template <int W>
__device__ __forceinline__ void kkt_score_rows(const elem *kS, int pitch, int K, const float *gS, const float *bS, int len,
                                               f32x4 (&acc)[4]) {
    const int t = 16 * W + acc_col();
    const float gt = gS[t], bt = bS[t];
#pragma unroll
    for (int J = 0; J < 4; ++J) acc[J] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int kk = 0; kk < K; kk += 32) {
        const elemx8 own = frag_kc(kS, pitch, 16 * W, kk);
#pragma unroll
        for (int J = 0; J <= W; ++J) acc[J] = mfma16x32(frag_kc(kS, pitch, 16 * J, kk), own, acc[J]);
    }
#pragma unroll
    for (int J = 0; J <= W; ++J)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int s = 16 * J + acc_row(e);
            const float d = fminf(fmaxf(gt - gS[s], -50.f), 50.f);
            acc[J][e] = (s < t && t < len) ? (float)(elem)(bt * __expf(d) * acc[J][e]) : 0.f;
        }
}

// One 16 x 16 tile of the same scores, rows 16 I.., columns 16 J.. (J <= I), written to its place in the fp32 block sS
// (pitch 68), so that the ten tiles can be dealt over the waves by count instead of by row block.
template <int I, int J>
__device__ __forceinline__ void kkt_score_tile(const elem *kS, int pitch, int K, const float *gS, const float *bS, int len, float *sS) {
    const int t = 16 * I + acc_col();
    const float gt = gS[t], bt = bS[t];
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int kk = 0; kk < K; kk += 32) acc = mfma16x32(frag_kc(kS, pitch, 16 * J, kk), frag_kc(kS, pitch, 16 * I, kk), acc);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int s = 16 * J + acc_row(e);
        const float d = fminf(fmaxf(gt - gS[s], -50.f), 50.f);
        acc[e] = (s < t && t < len) ? (float)(elem)(bt * __expf(d) * acc[e]) : 0.f;
    }
    *reinterpret_cast<f32x4 *>(sS + t * 68 + 16 * J + 4 * (lane_id() >> 4)) = acc;
}

// (I + A)^-1 of the strictly lower 64 x 64 matrix in aS (fp32, pitch 68), written to oS (pitch 72) in the element
// type; called by all four waves of a 256-thread workgroup after a barrier that completes aS, ends with one.
__device__ __forceinline__ void invert64(float *aS, elem *oS) {
    constexpr int pa = 68, pb = 72;
    const int R = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    {   // diagonal block: a2 = A[4lg+e][li] and a1 = A[li][4lg+e] (both orientations feed the squarings)
        f32x4 a1, a2, Y;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int r = 4 * lg + e;
            a2[e] = aS[(16 * R + r) * pa + 16 * R + li];
            a1[e] = aS[(16 * R + li) * pa + 16 * R + r];
            Y[e] = (r == li ? 1.f : 0.f) - a1[e];
        }
        const elemx4 A1 = cvt4(a1), A2 = cvt4(a2);
        const f32x4 S1 = mfma16x16(A1, A2, zero);   // A^2
        const f32x4 T1 = mfma16x16(A2, A1, zero);   // (A^2)^T
        const elemx4 S1b = cvt4(S1), T1b = cvt4(T1);
        Y = mfma16x16(S1b, cvt4(Y), Y);
        const f32x4 S2 = mfma16x16(T1b, S1b, zero);  // A^4
        const f32x4 T2 = mfma16x16(S1b, T1b, zero);  // (A^4)^T
        const elemx4 S2b = cvt4(S2);
        Y = mfma16x16(S2b, cvt4(Y), Y);
        const f32x4 S3 = mfma16x16(cvt4(T2), S2b, zero);  // A^8
        Y = mfma16x16(cvt4(S3), cvt4(Y), Y);
        __syncthreads();   // every wave has read its block of A before the inverses replace the diagonal blocks
        // lane holds D[li][4lg+e]
        *reinterpret_cast<f32x4 *>(aS + (16 * R + li) * pa + 16 * R + 4 * lg) = Y;
        *reinterpret_cast<elemx4 *>(oS + (16 * R + li) * pb + 16 * R + 4 * lg) = cvt4(Y);
#pragma unroll
        for (int cb = R + 1; cb < 4; ++cb)
            *reinterpret_cast<elemx4 *>(oS + (16 * R + li) * pb + 16 * cb + 4 * lg) = elemx4{(elem)0.f, (elem)0.f, (elem)0.f, (elem)0.f};
    }
    __syncthreads();
    switch (R) {   // the wave's position as a compile-time value: straight-line code per wave, operands hoisted and split once
        case 0: invert64_column<0>(aS, oS); break;
        case 1: invert64_column<1>(aS, oS); break;
        case 2: invert64_column<2>(aS, oS); break;
        default: break;   // wave 3 owns the last diagonal block only
    }
    __syncthreads();
}

}  // namespace fla
