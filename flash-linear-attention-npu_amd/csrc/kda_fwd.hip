// chunk_kda_fwd: chunked forward of the per-channel gated delta rule (KDA).
//
// Two kernels (a third, kda_cross_kernel, couples the two 64-token halves of a 128-token chunk):
//   kda_intra_kernel  one workgroup per (64 tokens, value head): gate activation + chunk-local prefix
//                     sum (log2 units), the decayed scores Aqk = scale * tril(q k^T . 2^{g_i-g_j})
//                     and A0 = beta * stril(k k^T . 2^{g_i-g_j}), the explicit inverse
//                     Akk = (I + A0)^-1, and the WY factors  w = Akk (k beta 2^g),  u = Akk (v beta),
//                     plus the gated operands qg = q 2^g and kg = k 2^{g_last - g}.
//   kda_scan_kernel   one workgroup per (sequence, value head, 64-column slab of V) walks the chunks
//                     with the fp32 state in accumulator registers:
//                         v_new = u - w S ;  o = scale qg S + Aqk v_new ;  S <- 2^{g_last} S + kg^T v_new
//
// The pairwise decay 2^{g_i - g_j} is never formed from a quotient of two exponentials of the
// absolute gates (those under/overflow); every 16-row tile r is evaluated against the gate of its
// last row:  (x_i 2^{g_i - s_r}) . (k_j 2^{s_r - g_j}),  both factors rounded to bf16 before the MFMA.
// Math and tiling: tests/atk/chunk_kda_fwd/executor_chunk_kda_fwd.py:316-530,
// fla/ops/ascendc/kda/chunk_kda_fwd/docs/api.md:60-180; operand order of the launch:
// torch_custom/fla_npu/fla_npu/ops/ascendc/_aclnn_ctypes.py:1066-1265.
#include <cctype>
#include <mutex>

#include "gdn_common.h"
#include "kda_common.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;
constexpr int kIntraThreads = 512;   // kda_intra_kernel: two waves per SIMD share one set of LDS tiles

__device__ __forceinline__ f32x4 lds4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
__device__ __forceinline__ f32x4 zero4() { return f32x4{0.f, 0.f, 0.f, 0.f}; }
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }

struct KdaIntraParams {
    ChunkGeom geom;
    View4 q, k, v;       // bf16, strides of (batch, head, token) in the caller's layout
    const void *g;       // raw gate, f32 or bf16, same layout family
    int g_elem;
    int64_t g_sb, g_sh, g_st;
    View3 beta;
    const float *a_log, *dt_bias;
    int use_gate, safe_gate;
    float lower_bound;
    float scale;
    float *gk;                // [B,Hv,T,K] or null
    elem *aqk, *akk;          // [B,Hv,T,C], C = tokens per chunk
    elem *w, *qg;             // [B,Hv,T,K]
    // u [B,Hv,T,V] and kg [B,Hv,T,K] reach the scan as fp16 (u16, kg16: see `fine`); u and kg are the caller's
    // tensors of the element type, written as well when they are not null (never set when elem is fp16 itself)
    fine *u16, *kg16;
    elem *u, *kg;
    int qg_fine;              // qg is a tensor of `fine` values (the caller keeps it for a reverse scan that reads it so)
    float *dec;               // [B,NT,Hv,K]: 2^{g_last} of every chunk
    // 128-token chunks: a workgroup still owns 64 tokens (one half of a chunk); the operands of the block that
    // couples the halves go to x1 (first half: k 2^{G1 - g}; second half: q 2^{g - G1}) and x2 (second half:
    // beta k 2^{g - G1}), G1 = gate at the end of the first half.  Both [B,Hv,T,K].
    int c128;
    elem *x1, *x2;
};

// A operand of a 16x16x16 product from four fp32 values, split into a bf16 head and remainder.
struct HiLo {
    elemx4 hi, lo;
};
__device__ __forceinline__ HiLo split(f32x4 x) {
    HiLo r;
    split_hilo(x, r.hi, r.lo);
    return r;
}
// acc += a * b with both operands carried as head + remainder (the lo*lo term is dropped).
__device__ __forceinline__ f32x4 mm3(f32x4 a, f32x4 b, f32x4 acc) {
    const HiLo A = split(a), B = split(b);
    acc = mfma16x16(A.hi, B.hi, acc);
    acc = mfma16x16(A.lo, B.hi, acc);
    acc = mfma16x16(A.hi, B.lo, acc);
    return acc;
}

// rows row0..row0+15 of `tile` times 2^{+-(g_row - g_anchor)} as an MFMA operand (contraction
// slots 32j .. 32j+31 along the channels)
template <bool LEFT>
__device__ __forceinline__ elemx8 scaled_frag(const elem *tile, int pitch, const float *gS, int pg, int row0, int arow,
                                              int j) {
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const elemx8 raw = frag_kc(tile, pitch, row0, 32 * j);
    const float *gr = gS + (row0 + li) * pg + 32 * j + 4 * lg;
    const float *ga = gS + arow * pg + 32 * j + 4 * lg;
    const f32x4 g0 = lds4(gr), g1 = lds4(gr + 16), s0 = lds4(ga), s1 = lds4(ga + 16);
    f32x4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        lo[e] = (float)raw[e] * ex2(LEFT ? g0[e] - s0[e] : s0[e] - g0[e]);
        hi[e] = (float)raw[4 + e] * ex2(LEFT ? g1[e] - s1[e] : s1[e] - g1[e]);
    }
    return frag_from_acc(lo, hi);
}

template <int K, int V> struct IntraSmem {
    // WIDE (more than 128 channels): the tiles of the 128-channel form do not fit together.  The gate tile is dead
    // once the gated operands are formed, so v (times beta) and the Aqk staging tile take its place afterwards, and
    // the scratch of the gate scan lies over the fp32 score tile, which is first written after the scan.
    static constexpr bool WIDE = K > 128;
    static constexpr int pq = WIDE ? K + 8 : K + 16, pk = K + 8, pg = K + 4, pv = V + 16, pa = 68, pb = 72;
    static constexpr int SEG = kIntraThreads / K;  // token segments of the gate scan
    static constexpr size_t g_bytes = (size_t)(kChunk + 2) * pg * 4;
    // gate rows kChunk and kChunk + 1: the gate at the end of the chunk and the anchor of the coupling block
    static constexpr size_t q_off = 0;
    static constexpr size_t k_off = q_off + (size_t)kChunk * pq * 2;
    static constexpr size_t ak_off = k_off + (size_t)kChunk * pk * 2 + (WIDE ? 0 : (size_t)kChunk * pv * 2);
    static constexpr size_t g_off = ak_off + (size_t)kChunk * pb * 2 * (WIDE ? 1 : 2);
    static constexpr size_t v_off = WIDE ? g_off : k_off + (size_t)kChunk * pk * 2;
    static constexpr size_t aq_off = WIDE ? g_off + (size_t)kChunk * pv * 2 : ak_off + (size_t)kChunk * pb * 2;
    static constexpr size_t a_off = g_off + g_bytes;                       // fp32 scores [kChunk][pa], then beta [kChunk]
    static constexpr size_t t_off = a_off;                                 // scan scratch [2 SEG][K], dead before the scores
    // FACT: the right-hand score operand k_j 2^{s_R - g_j} (s_R = gate at the last row of row tile R) is formed as
    // (k_j 2^{s_c - g_j}) 2^{s_R - s_c}, c the 16-row tile of j: a tile computed once per chunk and a [6][K] table of the
    // tile-to-tile factors, instead of eight exponentials per operand fragment in every wave that needs it.
    static constexpr bool FACT = !WIDE;
    static constexpr size_t kh_off = a_off + (size_t)kChunk * (pa + 1) * 4;
    static constexpr size_t f_off = kh_off + (FACT ? (size_t)kChunk * pk * 2 : 0);
    static constexpr size_t bytes = f_off + (FACT ? (size_t)6 * K * 4 : 0);
    // w and u leave through LDS as whole rows.  Where the dead k 2^{s_c - g} tile and the dead gate tile can take them
    // (pitches pk and pv), the products are staged there at once; otherwise over their own operand tiles, behind a barrier.
    static constexpr bool FREE_STAGE = FACT && (size_t)kChunk * pv * 2 <= g_bytes;
    static_assert((size_t)2 * SEG * K <= (size_t)kChunk * pa, "the scan scratch must fit the score tile it lies over");
    static_assert(!WIDE || (size_t)kChunk * (pv + pb) * 2 <= g_bytes, "the tiles that replace the gate tile must fit it");
};

// rows 16c.. of the tile k 2^{s_c - g} times the factor 2^{s_R - s_c} of the row tile R > c it is paired with (none on
// the diagonal), as an MFMA operand with contraction slots 32j .. 32j+31 along the channels
template <int K>
__device__ __forceinline__ elemx8 paired_frag(const elem *khS, int pk, const float *fS, int R, int c, int j) {
    const elemx8 raw = frag_kc(khS, pk, 16 * c, 32 * j);
    if (c == R) return raw;
    const int lg = lane_id() >> 4;
    const float *f = fS + (R * (R - 1) / 2 + c) * K + 32 * j + 4 * lg;
    const f32x4 f0 = lds4(f), f1 = lds4(f + 16);
    f32x4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        lo[e] = (float)raw[e] * f0[e];
        hi[e] = (float)raw[4 + e] * f1[e];
    }
    return frag_from_acc(lo, hi);
}

// Everything a wave does after the gate scan.  Eight waves: wave W of role 0 owns row tile W of k k^T (with the
// diagonal block inverse and the off-diagonal solve of column block W) and later row tile W of w; wave W of role 1
// owns row tile 3 - W of q k^T and later row tile W of u.  The two waves of a SIMD (W and 4 + W) together carry five
// score tile products, as every other SIMD does.  W and ROLE are static so that the tile loops unroll.
template <int K, int V, int W, int ROLE, bool C128, bool QGF>
__device__ __forceinline__ void intra_wave(const KdaIntraParams &p, elem *qS, elem *kS, elem *vS, elem *akS, elem *aqS,
                                           float *gS, float *aS, const float *bS, int len, int64_t row_base,
                                           int64_t dec_base, int half, const elem *vg, const elem *khS, const float *fS) {
    using S = IntraSmem<K, V>;
    constexpr int pq = S::pq, pk = S::pk, pg = S::pg, pv = S::pv, pa = S::pa, pb = S::pb;
    constexpr int KS = K / 32, R1 = W, R2 = 3 - W;
    constexpr bool WIDE = S::WIDE;
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    f32x4 aqv[4];   // WIDE: the wave's Aqk tiles wait in registers until the gate tile has made room for them

    // ---- scores: k k^T row tile R1 (and its transposed diagonal tile) | q k^T row tile R2 ------------------
    f32x4 kacc[R1 + 1], kaccT = zero4(), qacc[R2 + 1];
#pragma unroll
    for (int c = 0; c <= R1; ++c) kacc[c] = zero4();
#pragma unroll
    for (int c = 0; c <= R2; ++c) qacc[c] = zero4();
    f32x4 brow = zero4();
    float bcol = 0.f;
    if constexpr (ROLE == 0) {
        if constexpr (WIDE) {   // rolled: with eight steps unrolled the scaled operands of all of them are formed up front
#pragma unroll 1
            for (int j = 0; j < KS; ++j) {
                const elemx8 lk = scaled_frag<true>(kS, pk, gS, pg, 16 * R1, 16 * R1 + 15, j);
#pragma unroll
                for (int c = 0; c <= R1; ++c) {
                    const elemx8 rk = scaled_frag<false>(kS, pk, gS, pg, 16 * c, 16 * R1 + 15, j);
                    kacc[c] = mfma16x32(lk, rk, kacc[c]);
                    if (c == R1) kaccT = mfma16x32(rk, lk, kaccT);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                const elemx8 lk = scaled_frag<true>(kS, pk, gS, pg, 16 * R1, 16 * R1 + 15, j);
#pragma unroll
                for (int c = 0; c <= R1; ++c) {
                    const elemx8 rk = paired_frag<K>(khS, pk, fS, R1, c, j);
                    kacc[c] = mfma16x32(lk, rk, kacc[c]);
                    if (c == R1) kaccT = mfma16x32(rk, lk, kaccT);
                }
            }
        }
        // lane holds (row 16R + 4lg + e, column 16c + li) of each tile
        brow = lds4(bS + 16 * R1 + 4 * lg);
        bcol = bS[16 * R1 + li];
#pragma unroll
        for (int c = 0; c < R1; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) aS[(16 * R1 + 4 * lg + e) * pa + 16 * c + li] = brow[e] * kacc[c][e];
    } else {
        if constexpr (WIDE) {
#pragma unroll 1
            for (int j = 0; j < KS; ++j) {
                const elemx8 lq = scaled_frag<true>(qS, pq, gS, pg, 16 * R2, 16 * R2 + 15, j);
#pragma unroll
                for (int c = 0; c <= R2; ++c) {
                    const elemx8 rk = scaled_frag<false>(kS, pk, gS, pg, 16 * c, 16 * R2 + 15, j);
                    qacc[c] = mfma16x32(lq, rk, qacc[c]);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                const elemx8 lq = scaled_frag<true>(qS, pq, gS, pg, 16 * R2, 16 * R2 + 15, j);
#pragma unroll
                for (int c = 0; c <= R2; ++c) {
                    const elemx8 rk = paired_frag<K>(khS, pk, fS, R2, c, j);
                    qacc[c] = mfma16x32(lq, rk, qacc[c]);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            f32x4 a = zero4();
            if (c <= R2) {
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = (c < R2 || li <= 4 * lg + e) ? p.scale * qacc[c <= R2 ? c : 0][e] : 0.f;
            }
            if constexpr (WIDE) aqv[c] = a;
            else acc_to_tile(aqS, pb, 16 * R2, 16 * c, a);
        }
    }

    if constexpr (ROLE == 0) {
        // ---- inverse of the diagonal block: (I + A)^-1 = (I - A)(I + A^2)(I + A^4)(I + A^8) ------------
        // a2 = A[4lg+e][li] (right operand of A, left operand of A^T); a1 = A[li][4lg+e] (the converse).
        f32x4 a1, a2, Y;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int r = 4 * lg + e;
            a2[e] = li < r ? brow[e] * kacc[R1][e] : 0.f;
            a1[e] = r < li ? bcol * kaccT[e] : 0.f;
            Y[e] = (r == li ? 1.f : 0.f) - a1[e];   // (I - A^T)[r][li]
        }
        {
            const elemx4 A1 = cvt4(a1), A2 = cvt4(a2);
            const f32x4 S1 = mfma16x16(A1, A2, zero4());   // A^2
            const f32x4 T1 = mfma16x16(A2, A1, zero4());   // (A^2)^T
            const elemx4 S1b = cvt4(S1), T1b = cvt4(T1);
            Y = mfma16x16(S1b, cvt4(Y), Y);
            const f32x4 S2 = mfma16x16(T1b, S1b, zero4());  // A^4
            const f32x4 T2 = mfma16x16(S1b, T1b, zero4());  // (A^4)^T
            const elemx4 S2b = cvt4(S2);
            Y = mfma16x16(S2b, cvt4(Y), Y);
            const f32x4 S3 = mfma16x16(cvt4(T2), S2b, zero4());  // A^8
            Y = mfma16x16(cvt4(S3), cvt4(Y), Y);
        }
        // lane holds Dinv[li][4lg+e]
        *reinterpret_cast<f32x4 *>(aS + (16 * R1 + li) * pa + 16 * R1 + 4 * lg) = Y;
        *reinterpret_cast<elemx4 *>(akS + (16 * R1 + li) * pb + 16 * R1 + 4 * lg) = cvt4(Y);
#pragma unroll
        for (int c = R1 + 1; c < 4; ++c)
            *reinterpret_cast<elemx4 *>(akS + (16 * R1 + li) * pb + 16 * c + 4 * lg) = elemx4{(elem)0.f, (elem)0.f, (elem)0.f, (elem)0.f};
    }
    __syncthreads();

    // ---- off-diagonal blocks of the inverse, column block W: X_rc = -Dinv_r sum_m A_rm X_mc --------
    if constexpr (ROLE == 0 && W < 3) {
        constexpr int C = W;
        f32x4 X[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) X[C][e] = aS[(16 * C + 4 * lg + e) * pa + 16 * C + li];
#pragma unroll
        for (int r = C + 1; r < 4; ++r) {
            f32x4 sum = zero4();
#pragma unroll
            for (int m = C; m < r; ++m) sum = mm3(lds4(aS + (16 * r + li) * pa + 16 * m + 4 * lg), X[m], sum);
            const f32x4 dinv = lds4(aS + (16 * r + li) * pa + 16 * r + 4 * lg);
            X[r] = mm3(-dinv, sum, zero4());
            acc_to_tile(akS, pb, 16 * r, 16 * C, X[r]);
        }
    }
    // ---- gated operands: qg, kg to memory; k beta 2^g over the q tile ----------------------------------
    // WIDE: one piece at a time (unrolled, the four pieces of a thread do not fit the registers together)
#pragma unroll(WIDE ? 1 : 2)
    for (int idx = threadIdx.x; idx < kChunk * (K / 8); idx += kIntraThreads) {
        const int r = idx / (K / 8), c8 = (idx % (K / 8)) * 8;
        const elemx8 q8 = *reinterpret_cast<const elemx8 *>(qS + r * pq + c8);
        const elemx8 k8 = *reinterpret_cast<const elemx8 *>(kS + r * pk + c8);
        const float br = bS[r];
        elemx8 qg8, kg8, kb8;
        u32x4 kgf, qgf = {};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const f32x4 gg = lds4(gS + r * pg + c8 + 4 * h), gl = lds4(gS + kChunk * pg + c8 + 4 * h);
            f32x4 a, b, c;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float eg = ex2(gg[e]), kk = (float)k8[4 * h + e];
                a[e] = (float)q8[4 * h + e] * eg;
                b[e] = kk * ex2(gl[e] - gg[e]);
                c[e] = kk * br * eg;
            }
            const elemx4 a4 = cvt4(a), b4 = cvt4(b), c4 = cvt4(c);
            kgf[2 * h] = cvt2_fine_bounded(b[0], b[1]);
            kgf[2 * h + 1] = cvt2_fine_bounded(b[2], b[3]);
            if constexpr (QGF) {
                qgf[2 * h] = cvt2_fine_bounded(a[0], a[1]);
                qgf[2 * h + 1] = cvt2_fine_bounded(a[2], a[3]);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                qg8[4 * h + e] = a4[e];
                kg8[4 * h + e] = b4[e];
                kb8[4 * h + e] = c4[e];
            }
        }
        if (r < len) {
            *reinterpret_cast<u32x4 *>(p.qg + (row_base + r) * K + c8) = QGF ? qgf : __builtin_bit_cast(u32x4, qg8);
            *reinterpret_cast<u32x4 *>(p.kg16 + (row_base + r) * K + c8) = kgf;
            if constexpr (!kFineIsElem) {
                if (p.kg != nullptr) *reinterpret_cast<elemx8 *>(p.kg + (row_base + r) * K + c8) = kg8;
            }
        }
        if constexpr (C128) {   // operands of the block that couples the two halves, both factors <= 1
            f32x4 x1lo, x1hi, x2lo, x2hi;
            const f32x4 g0 = lds4(gS + r * pg + c8), g1 = lds4(gS + r * pg + c8 + 4);
            const f32x4 a0 = lds4(gS + (kChunk + 1) * pg + c8), a1 = lds4(gS + (kChunk + 1) * pg + c8 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float d0 = half ? ex2(g0[e] - a0[e]) : ex2(a0[e] - g0[e]);
                const float d1 = half ? ex2(g1[e] - a1[e]) : ex2(a1[e] - g1[e]);
                x1lo[e] = (float)(half ? q8[e] : k8[e]) * d0;
                x1hi[e] = (float)(half ? q8[4 + e] : k8[4 + e]) * d1;
                x2lo[e] = (float)k8[e] * br * d0;
                x2hi[e] = (float)k8[4 + e] * br * d1;
            }
            if (r < len) {
                *reinterpret_cast<elemx8 *>(p.x1 + (row_base + r) * K + c8) = frag_from_acc(x1lo, x1hi);
                if (half) *reinterpret_cast<elemx8 *>(p.x2 + (row_base + r) * K + c8) = frag_from_acc(x2lo, x2hi);
            }
        }
        *reinterpret_cast<elemx8 *>(qS + r * pq + c8) = kb8;
    }
    if (threadIdx.x < K && dec_base >= 0) p.dec[dec_base + threadIdx.x] = ex2(gS[kChunk * pg + threadIdx.x]);
    if constexpr (WIDE) {
        __syncthreads();   // last read of the gate tile
        TileCopy<kIntraThreads, kChunk, V> tv;
        tv.fetch(vg, p.v.st, len, threadIdx.x);
        tv.commit(vS, pv, len, threadIdx.x);
        if constexpr (ROLE == 1) {
#pragma unroll
            for (int c = 0; c < 4; ++c) acc_to_tile(aqS, pb, 16 * R2, 16 * c, aqv[c]);
        }
    }
    __syncthreads();

    // ---- w = Akk (k beta 2^g) (role 0), u = Akk (v beta) (role 1): row tile W -----------------------------------
    // u is formed as (Akk diag(beta)) v from the v tile as it came from memory: the unit diagonal of Akk carries
    // beta_i v_i, the leading term of u_i, and its only rounding (beta_i to the element type in the left operand) is
    // made good below, so that u is accurate to fp32 products of the 16-bit Akk rather than to a rounded v beta.
    constexpr int NCT = ROLE == 0 ? K / 16 : V / 16;
    f32x4 oacc[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ++ct) oacc[ct] = zero4();
#pragma unroll
    for (int j = 0; j < (W < 2 ? 1 : 2); ++j) {   // Akk is lower triangular
        elemx8 a = frag_kc(akS, pb, 16 * W, 32 * j);
        if constexpr (ROLE == 1) {
            const f32x4 b0 = lds4(bS + 32 * j + 4 * lg), b1 = lds4(bS + 32 * j + 16 + 4 * lg);
            f32x4 lo, hi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[e] = (float)a[e] * b0[e];
                hi[e] = (float)a[4 + e] * b1[e];
            }
            a = frag_from_acc(lo, hi);
        }
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            oacc[ct] = mfma16x32(a, ROLE == 0 ? frag_tr(qS, pq, 16 * ct, 32 * j) : frag_tr(vS, pv, 16 * ct, 32 * j), oacc[ct]);
            if constexpr (WIDE) {
                if (ct % 4 == 3) __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    if constexpr (ROLE == 1) {   // u_i += (beta_i - rounded beta_i) v_i
        const f32x4 bw = lds4(bS + 16 * W + 4 * lg);
        f32x4 db;
#pragma unroll
        for (int e = 0; e < 4; ++e) db[e] = bw[e] - (float)(elem)bw[e];
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            const elemx4 vv = frag_tr4(vS, pv, 16 * ct, 16 * W);
#pragma unroll
            for (int e = 0; e < 4; ++e) oacc[ct][e] += db[e] * (float)vv[e];
        }
    }
    if constexpr (S::FREE_STAGE) {   // nobody reads the two dead tiles any more
        elem *wT = const_cast<elem *>(khS), *uT = reinterpret_cast<elem *>(gS);
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            if constexpr (ROLE == 0) acc_to_tile(wT, pk, 16 * W, 16 * ct, oacc[ct]);
            else acc_to_tile_fine(uT, pv, 16 * W, 16 * ct, oacc[ct]);
        }
    } else {
        __syncthreads();   // every wave has consumed the operand tiles; they become the output staging
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
            if constexpr (ROLE == 0) acc_to_tile(qS, pq, 16 * W, 16 * ct, oacc[ct]);
            else acc_to_tile_fine(vS, pv, 16 * W, 16 * ct, oacc[ct]);
        }
    }
    __syncthreads();
}

// C128: the workgroup owns one half of a 128-token chunk (a template flag, so that the 64-token form carries none of
// the second gate stream, the coupling operands or the zero fill).  QGF: qg is written as `fine` values (a template
// flag as well: as a run-time choice the second conversion cost the kernel 0.04 ms of 0.36 at B=2, T=8192, H=32).
template <int K, int V, bool C128, bool QGF>
__global__ void __launch_bounds__(kIntraThreads) FLA_TWO_WAVES_PER_SIMD kda_intra_kernel(const KdaIntraParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    using S = IntraSmem<K, V>;
    constexpr int pq = S::pq, pk = S::pk, pg = S::pg, pv = S::pv, pa = S::pa, pb = S::pb, SEG = S::SEG;
    elem *qS = reinterpret_cast<elem *>(smem + S::q_off);
    elem *kS = reinterpret_cast<elem *>(smem + S::k_off);
    elem *vS = reinterpret_cast<elem *>(smem + S::v_off);
    elem *akS = reinterpret_cast<elem *>(smem + S::ak_off);
    elem *aqS = reinterpret_cast<elem *>(smem + S::aq_off);
    float *gS = reinterpret_cast<float *>(smem + S::g_off);
    float *aS = reinterpret_cast<float *>(smem + S::a_off);
    float *bS = aS + kChunk * pa;
    float *tS = reinterpret_cast<float *>(smem + S::t_off);
    elem *khS = reinterpret_cast<elem *>(smem + S::kh_off);
    float *fS = reinterpret_cast<float *>(smem + S::f_off);

    int cx, hv;
    block_chunk_head(p.geom, cx, hv);
    const int half = C128 ? (cx & 1) : 0, c = C128 ? cx >> 1 : cx, b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    int ostart = start, olen = 0;   // the other half of a 128-token chunk: its gates enter this half's sums
    if constexpr (C128) {
        const int whole = len;
        olen = min(kChunk, max(0, whole - kChunk * (1 - half)));
        if (olen > 0) ostart = start + kChunk * (1 - half);
        start += kChunk * half;
        len = min(kChunk, whole - kChunk * half);
        if (len <= 0) return;
    }
    const int tid = threadIdx.x;

    const elem *qg = static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh + (int64_t)start * p.q.st;
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st;
    const elem *vg = static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st;
    // gate loads first (thread = (token segment, channel)); branch-free with a clamped token index so that
    // they are all in flight together with the tile loads below
    const int64_t row_base = ((int64_t)b * p.geom.Hv + hv) * p.geom.T + start;   // head-major row of token 0
    constexpr int TS = kChunk / SEG;
    const int ch = tid % K, sg = tid / K;
    float eig = 0.f, bias = 0.f;
    if (p.use_gate) {
        eig = __expf(p.a_log[hv]);
        if (p.dt_bias) bias = p.dt_bias[(int64_t)hv * K + ch];
    }
    float raw[TS], oraw[TS];
    {
        // one buffer resource per gate stream (the workgroup's first token of the head), 32-bit offsets per lane:
        // a clamped row index, one multiply and one add per load instead of 64-bit address arithmetic
        const int esz = p.g_elem ? 2 : 4, gst = (int)p.g_st;
        const char *gwg = static_cast<const char *>(p.g) + (b * p.g_sb + hv * p.g_sh) * esz;
        const __amdgpu_buffer_rsrc_t rg = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char *>(gwg + (int64_t)start * p.g_st * esz), 0, 0x7fffffff, 0x00020000);
        const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char *>(gwg + (int64_t)ostart * p.g_st * esz), 0, 0x7fffffff, 0x00020000);
        const int olast = max(olen, 1) - 1;
        auto gate_at = [&](const __amdgpu_buffer_rsrc_t &r, int row) -> float {
            const int off = (row * gst + ch) * esz;
            if (p.g_elem) {
                const unsigned short h = __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0);
                return (float)__builtin_bit_cast(elem, h);
            }
            return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
        };
#pragma unroll
        for (int j = 0; j < TS; ++j) raw[j] = gate_at(rg, min(sg * TS + j, len - 1));
        if constexpr (C128)
#pragma unroll
            for (int j = 0; j < TS; ++j) oraw[j] = gate_at(ro, min(sg * TS + j, olast));
    }
    {   // all loads of the chunk are issued before the first LDS write waits for one of them
        TileCopy<kIntraThreads, kChunk, K> tq, tk;
        TileCopy<kIntraThreads, kChunk, V> tv;
        tq.fetch(qg, p.q.st, len, tid);
        tk.fetch(kg, p.k.st, len, tid);
        if constexpr (!S::WIDE) tv.fetch(vg, p.v.st, len, tid);
        {   // segment sums of the gates (they were requested first) while the tiles are still on their way
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < TS; ++j) {
                const int t = sg * TS + j;
                if (t < len) {
                    const float a = p.use_gate ? kda_activate(raw[j], bias, eig, p.safe_gate, p.lower_bound) : raw[j];
                    acc += a * kRcpLn2;
                }
                raw[j] = acc;   // the running sum within the segment stays in the register of its gate
            }
            tS[sg * K + ch] = acc;
            float oacc = 0.f;
            if constexpr (C128) {
#pragma unroll
                for (int j = 0; j < TS; ++j)
                    if (sg * TS + j < olen)
                        oacc += (p.use_gate ? kda_activate(oraw[j], bias, eig, p.safe_gate, p.lower_bound) : oraw[j]) * kRcpLn2;
            }
            tS[(SEG + sg) * K + ch] = oacc;
        }
        tq.commit(qS, pq, len, tid);
        tk.commit(kS, pk, len, tid);
        if constexpr (!S::WIDE) tv.commit(vS, pv, len, tid);
    }
    if (tid < kChunk) bS[tid] = tid < len ? load_scalar(p.beta, b, hv, start + tid) : 0.f;

    {
        __syncthreads();
        float off = 0.f, own = 0.f, other = 0.f;
        float upto[SEG];   // gate at the end of every segment, relative to the start of this half
#pragma unroll
        for (int s = 0; s < SEG; ++s) {
            const float v = tS[s * K + ch];
            if (s < sg) off += v;
            own += v;
            upto[s] = own;
            other += tS[(SEG + s) * K + ch];
        }
        if (half) off += other;   // gates of the second half continue those of the first
        if (sg == 0) {
            gS[kChunk * pg + ch] = own + other;                 // gate at the end of the chunk
            gS[(kChunk + 1) * pg + ch] = half ? other : own;    // gate at the end of the first half
        }
        float *gkp = p.gk ? p.gk + row_base * K + ch : nullptr;
#pragma unroll
        for (int j = 0; j < TS; ++j) {
            const int t = sg * TS + j;
            const float v = raw[j] + off;
            gS[t * pg + ch] = v;
            if (gkp != nullptr && t < len) gkp[t * K] = v;
        }
        if constexpr (S::FACT) {
            // k 2^{s_c - g} for this thread's tokens (s_c: the gate at the last row of their 16-row tile) and, from the
            // first segment's threads, the tile-to-tile factors 2^{s_R - s_c} of the channel
            constexpr int SPT = 16 / TS;   // segments per 16-row tile
            static_assert(TS <= 16 && 16 % TS == 0, "a segment must not straddle two row tiles");
            float anchor = 0.f;
#pragma unroll
            for (int s = 0; s < SEG; ++s)
                if (s == (sg / SPT) * SPT + SPT - 1) anchor = upto[s];
            anchor += half ? other : 0.f;
#pragma unroll
            for (int j = 0; j < TS; ++j) {
                const int t = sg * TS + j;
                khS[t * pk + ch] = (elem)((float)kS[t * pk + ch] * ex2(anchor - (raw[j] + off)));
            }
            if (sg == 0) {
#pragma unroll
                for (int R = 1; R < 4; ++R)
#pragma unroll
                    for (int cc = 0; cc < R; ++cc)
                        fS[(R * (R - 1) / 2 + cc) * K + ch] = ex2(upto[R * SPT + SPT - 1] - upto[cc * SPT + SPT - 1]);
            }
        }
    }
    __syncthreads();

    const int64_t dec_base = half ? -1 : (((int64_t)b * p.geom.NT + c) * p.geom.Hv + hv) * K;
    switch (wave_id()) {
        case 0: intra_wave<K, V, 0, 0, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
        case 1: intra_wave<K, V, 1, 0, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
        case 2: intra_wave<K, V, 2, 0, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
        case 3: intra_wave<K, V, 3, 0, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
        case 4: intra_wave<K, V, 0, 1, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
        case 5: intra_wave<K, V, 1, 1, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
        case 6: intra_wave<K, V, 2, 1, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
        default: intra_wave<K, V, 3, 1, C128, QGF>(p, qS, kS, vS, akS, aqS, gS, aS, bS, len, row_base, dec_base, half, vg, khS, fS); break;
    }

    {
        const elem *wT = S::FREE_STAGE ? khS : qS, *uT = S::FREE_STAGE ? reinterpret_cast<const elem *>(gS) : vS;
        store_tile<kIntraThreads>(p.w + row_base * K, K, wT, S::FREE_STAGE ? pk : pq, K, len);
        store_tile<kIntraThreads>(reinterpret_cast<elem *>(p.u16) + row_base * V, V, uT, pv, V, len);
        if constexpr (!kFineIsElem) {
            if (p.u != nullptr) store_tile_fine_as_elem<kIntraThreads>(p.u + row_base * V, V, uT, pv, V, len);
        }
    }
    const int C = p.geom.C;
    store_tile<kIntraThreads>(p.aqk + row_base * C + kChunk * half, C, aqS, pb, kChunk, len);
    store_tile<kIntraThreads>(p.akk + row_base * C + kChunk * half, C, akS, pb, kChunk, len);
    if (C128 && half == 0) {   // nothing of the second half is visible to the first
        const elemx8 z = {};
        for (int idx = tid; idx < len * (kChunk / 8); idx += kIntraThreads) {
            const int64_t at = (row_base + idx / (kChunk / 8)) * C + kChunk + (idx % (kChunk / 8)) * 8;
            *reinterpret_cast<elemx8 *>(p.aqk + at) = z;
            *reinterpret_cast<elemx8 *>(p.akk + at) = z;
        }
    }
}


// =============================================================================================
// 128-token chunks: the block that couples the two 64-token halves
// =============================================================================================
// With A0 = [[A11, 0], [M21, A22]] the inverse is [[I11, 0], [-I22 M21 I11, I22]] (I11, I22 the inverses the
// intra kernel has written).  One workgroup per chunk with a second half:
//     Aqk21 = scale (q2 2^{g2-G1}) (k1 2^{G1-g1})^T          M21 = (beta2 k2 2^{g2-G1}) (k1 2^{G1-g1})^T
//     P = I22 M21 ;  Akk21 = -P I11 ;  w2 -= P w1 ;  u2 -= P u1
// (I21 (k beta 2^g)_1 = -P I11 (k beta 2^g)_1 = -P w1, likewise for u).  M21 and P pass between the products
// as a 16-bit head plus remainder.  Wave r owns rows 16r.. of the second half.
struct KdaCrossParams {
    ChunkGeom geom;
    const elem *x1, *x2;
    elem *w, *aqk, *akk;
    fine *u16;   // u as the scan reads it
    elem *u;     // the caller's u of the element type, or null
    float scale;
};

template <int K, int V> struct CrossSmem {
    // WIDE (more than 128 channels): w1 and u1 are staged after the scores, over the two operand tiles of the second half
    static constexpr bool WIDE = K > 128;
    static constexpr int pk = K + 8, pr = WIDE ? K + 8 : K + 16, pv = WIDE ? V + 8 : V + 16, pb = 72;
    static_assert(!WIDE || V <= K, "u1 takes the place of a K-wide tile");
    static constexpr size_t qa_off = 0;
    static constexpr size_t kb_off = qa_off + (size_t)kChunk * pk * 2;
    static constexpr size_t kc_off = kb_off + (size_t)kChunk * pk * 2;
    static constexpr size_t w_off = WIDE ? qa_off : kc_off + (size_t)kChunk * pk * 2;
    static constexpr size_t u_off = WIDE ? kb_off : w_off + (size_t)kChunk * pr * 2;
    static constexpr size_t a11_off = WIDE ? kc_off + (size_t)kChunk * pk * 2 : u_off + (size_t)kChunk * pv * 2;
    static constexpr size_t a22_off = a11_off + (size_t)kChunk * pb * 2;
    static constexpr size_t mhi_off = a22_off + (size_t)kChunk * pb * 2;
    static constexpr size_t mlo_off = mhi_off + (size_t)kChunk * pb * 2;
    static constexpr size_t bytes = mlo_off + (size_t)kChunk * pb * 2;
};

__device__ __forceinline__ void split8(f32x4 a, f32x4 b, elemx8 &hi, elemx8 &lo) {
    elemx4 ah, al, bh, bl;
    split_hilo(a, ah, al);
    split_hilo(b, bh, bl);
    hi = cat8(ah, bh);
    lo = cat8(al, bl);
}

template <int K, int V>
__global__ void __launch_bounds__(kThreads) kda_cross_kernel(const KdaCrossParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    typedef CrossSmem<K, V> L;
    constexpr int pk = L::pk, pr = L::pr, pv = L::pv, pb = L::pb, KS = K / 32, C = 2 * kChunk;
    elem *qaS = reinterpret_cast<elem *>(smem + L::qa_off), *kbS = reinterpret_cast<elem *>(smem + L::kb_off);
    elem *kcS = reinterpret_cast<elem *>(smem + L::kc_off), *wS = reinterpret_cast<elem *>(smem + L::w_off);
    elem *uS = reinterpret_cast<elem *>(smem + L::u_off), *a11S = reinterpret_cast<elem *>(smem + L::a11_off);
    elem *a22S = reinterpret_cast<elem *>(smem + L::a22_off), *mhiS = reinterpret_cast<elem *>(smem + L::mhi_off);
    elem *mloS = reinterpret_cast<elem *>(smem + L::mlo_off);

    const int c = blockIdx.x, hv = blockIdx.y, b = blockIdx.z;
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int len2 = len - kChunk;
    if (len2 <= 0) return;
    const int tid = threadIdx.x;
    const int64_t row1 = ((int64_t)b * p.geom.Hv + hv) * p.geom.T + start, row2 = row1 + kChunk;
    {
        TileCopy<kThreads, kChunk, K> tq, tb, tc, tw;
        TileCopy<kThreads, kChunk, V> tu;
        TileCopy<kThreads, kChunk, kChunk> t1, t2;
        tq.fetch(p.x1 + row2 * K, K, len2, tid);
        tb.fetch(p.x2 + row2 * K, K, len2, tid);
        tc.fetch(p.x1 + row1 * K, K, kChunk, tid);
        if constexpr (!L::WIDE) {
            tw.fetch(p.w + row1 * K, K, kChunk, tid);
            tu.fetch(reinterpret_cast<const elem *>(p.u16) + row1 * V, V, kChunk, tid);
        }
        t1.fetch(p.akk + row1 * C, C, kChunk, tid);
        t2.fetch(p.akk + row2 * C + kChunk, C, len2, tid);
        tq.commit(qaS, pk, len2, tid);
        tb.commit(kbS, pk, len2, tid);
        tc.commit(kcS, pk, kChunk, tid);
        if constexpr (!L::WIDE) {
            tw.commit(wS, pr, kChunk, tid);
            tu.to_elem();
            tu.commit(uS, pv, kChunk, tid);
        }
        t1.commit(a11S, pb, kChunk, tid);
        t2.commit(a22S, pb, len2, tid);
    }
    __syncthreads();

    const int r = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    {   // scores of the wave's rows against the first half
        f32x4 sq[4], sk[4];
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) sq[jt] = sk[jt] = zero4();
#pragma unroll
        for (int j = 0; j < KS; ++j) {
            const elemx8 lq = frag_kc(qaS, pk, 16 * r, 32 * j), lk = frag_kc(kbS, pk, 16 * r, 32 * j);
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                const elemx8 rk = frag_kc(kcS, pk, 16 * jt, 32 * j);
                sq[jt] = mfma16x32(lq, rk, sq[jt]);
                sk[jt] = mfma16x32(lk, rk, sk[jt]);
            }
        }
        char *ag = reinterpret_cast<char *>(p.aqk + row2 * C);
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) {
            acc_to_global(ag + 32 * jt, (int64_t)C * 2, 16 * r, len2, sq[jt] * p.scale);
            elemx4 hi, lo;
            split_hilo(sk[jt], hi, lo);
            acc_to_tile(mhiS, pb, 16 * r, 16 * jt, f32x4{(float)hi[0], (float)hi[1], (float)hi[2], (float)hi[3]});
            acc_to_tile(mloS, pb, 16 * r, 16 * jt, f32x4{(float)lo[0], (float)lo[1], (float)lo[2], (float)lo[3]});
        }
    }
    __syncthreads();
    if constexpr (L::WIDE) {   // the score operands are spent: w1 and u1 over the tiles of the second half
        TileCopy<kThreads, kChunk, K> tw;
        TileCopy<kThreads, kChunk, V> tu;
        tw.fetch(p.w + row1 * K, K, kChunk, tid);
        tu.fetch(reinterpret_cast<const elem *>(p.u16) + row1 * V, V, kChunk, tid);
        tw.commit(wS, pr, kChunk, tid);
        tu.to_elem();
        tu.commit(uS, pv, kChunk, tid);
        __syncthreads();
    }

    // P^T tiles (rows = first-half token j, columns = the wave's rows) as operands with contraction j
    elemx8 phi[2], plo[2];
    {
        f32x4 pt[4];
#pragma unroll
        for (int jt = 0; jt < 4; ++jt) pt[jt] = zero4();
        for (int ii = 0; ii <= (r >> 1); ++ii) {   // I22 is lower triangular
            const elemx8 a22 = frag_kc(a22S, pb, 16 * r, 32 * ii);
#pragma unroll
            for (int jt = 0; jt < 4; ++jt) {
                pt[jt] = mfma16x32(frag_tr(mhiS, pb, 16 * jt, 32 * ii), a22, pt[jt]);
                pt[jt] = mfma16x32(frag_tr(mloS, pb, 16 * jt, 32 * ii), a22, pt[jt]);
            }
        }
        split8(pt[0], pt[1], phi[0], plo[0]);
        split8(pt[2], pt[3], phi[1], plo[1]);
    }
    // (P R)^T tiles: rows = column of R, columns = the wave's rows; the lane's four values are adjacent in memory
    const bool live = 16 * r + li < len2;
    const int64_t orow = row2 + 16 * r + li;
    auto product = [&](const elem *R, int pitch, int ct) {
        f32x4 z = zero4();
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const elemx8 a = frag_tr(R, pitch, 16 * ct, 32 * jj);
            z = mfma16x32(a, phi[jj], z);
            z = mfma16x32(a, plo[jj], z);
        }
        return z;
    };
    auto minus = [&](elem *dst, f32x4 z) {   // *dst -= z
        if (!live) return;
        const elemx4 old = *reinterpret_cast<const elemx4 *>(dst);
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (float)old[e] - z[e];
        *reinterpret_cast<elemx4 *>(dst) = cvt4(v);
    };
#pragma unroll
    for (int ct = 0; ct < K / 16; ++ct) minus(p.w + orow * K + 16 * ct + 4 * lg, product(wS, pr, ct));
    auto minus_u = [&](int64_t at, f32x4 z) {   // u -= z, in the scan's copy and in the caller's
        if (!live) return;
        const finex4 old = *reinterpret_cast<const finex4 *>(p.u16 + at);
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (float)old[e] - z[e];
        *reinterpret_cast<finex4 *>(p.u16 + at) = cvt4_fine(v);
        if constexpr (!kFineIsElem) {
            if (p.u != nullptr) *reinterpret_cast<elemx4 *>(p.u + at) = cvt4(v);
        }
    };
#pragma unroll
    for (int ct = 0; ct < V / 16; ++ct) minus_u(orow * V + 16 * ct + 4 * lg, product(uS, pv, ct));
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        const f32x4 z = product(a11S, pb, ct);
        if (live) *reinterpret_cast<elemx4 *>(p.akk + orow * C + 16 * ct + 4 * lg) = cvt4(-z);
    }
}

// =============================================================================================
// inter-chunk scan
// =============================================================================================
struct KdaScanParams {
    ChunkGeom geom;
    const elem *w, *qg, *aqk;            // head-major [B,Hv,T,*]
    const fine *u, *kg;                  // fp16 whatever the element type (see `fine`)
    const float *dec;                    // [B,NT,Hv,K]
    View4 o;                             // attention output in the caller's layout
    elem *v_new;                         // [B,Hv,T,V] or null
    const float *h0;
    float *hT;
    elem *h;
    int64_t h_sb, h_sc, h_sh;            // strides of h over (batch, chunk, head)
    int64_t s_sn, s_sh;                  // strides of h0 / hT over (sequence, head)
    int v_first;
    float scale;
    int qg_fine;                         // qg holds `fine` values
};

template <int K> struct ScanSmem {
    static constexpr int pw = K + 8, pt = K + 16, pu = 64 + 8, pb = 72, ph = 64 + 8;
    static constexpr size_t w_off = 0;                                    // w
    static constexpr size_t q_off = w_off + (size_t)kChunk * pw * 2;      // qg
    static constexpr size_t k_off = q_off + (size_t)kChunk * pw * 2;      // kg (read transposed)
    static constexpr size_t u_off = k_off + (size_t)kChunk * pt * 2;      // u slab
    static constexpr size_t a_off = u_off + (size_t)kChunk * pu * 2;      // Aqk
    static constexpr size_t d_off = a_off + (size_t)kChunk * pb * 2;      // [K] decay of the chunk
    static constexpr size_t buf_bytes = d_off + (size_t)K * 4;
    static constexpr size_t h_off = 2 * buf_bytes;                        // [K][ph]: the state on its way to memory
    static constexpr size_t bytes = h_off + (size_t)K * ph * 2;
};

// 512 threads: waves 0-3 compute chunk c from LDS buffer c&1 while waves 4-7 copy the tiles of chunk
// c+1 from memory into the other buffer and have those of chunk c+2 in flight; the barriers wait for LDS traffic
// only, so that loads and stores stay in flight across them.  o leaves from registers.  The optional outputs
// for a backward pass leave through LDS as whole 128-byte rows, stored by the copying waves: v_new replaces the
// wave's own columns of the u tile and is written out one step later, before the tile is loaded again; h (default
// [K][V] blocks) goes through a tile of its own, written behind a second barrier in the middle of the step (the
// state changes only at the step's end) and written out one step later as well.
// SUB = 2: 128-token chunks walked as two 64-token steps.  Both steps see the state of the chunk's first token in
// w S and qg S (the operand copy of the state is refreshed on even steps only), the second step adds the
// coupling block Aqk21 times the first step's v_new, and the decay of the chunk is applied once, on the first step
// (kg already carries 2^{g_last - g} up to the end of the whole chunk).
// QF: qg holds `fine` values (the forward of a training step keeps it so for the reverse scan) and meets a `fine` copy
// of the state.
// VS: value columns per workgroup, 64 or 32 (VS / 16 compute waves in front of the four copying waves).  Every compute
// wave reads the whole w, qg and kg tiles for its 16 columns, so a workgroup's step is bound by its LDS traffic; when
// 64-column slabs leave compute units without a workgroup, 32-column slabs put half of that traffic on twice as many
// units (the slabs of a head share an XCD, so the tiles still come from memory once).
template <int K, int SUB, bool QF, int VS>
__global__ void __launch_bounds__((VS / 16 + 4) * 64) kda_scan_kernel(const KdaScanParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    typedef ScanSmem<K> L;
    constexpr int CW = VS / 16;   // compute waves
    constexpr int pw = L::pw, pt = L::pt, pu = L::pu, pb = L::pb, ph = L::ph;
    constexpr int KT = K / 16, KS = K / 32;

    int slab, hv, n;
    chain_of_block(slab, hv, n);
    const int V = p.geom.V;
    int b = n, bos = 0, eos = p.geom.T, chunk0 = 0;
    if (p.geom.cu != nullptr) {
        b = 0;
        bos = p.geom.cu[n];
        eos = p.geom.cu[n + 1];
        chunk0 = p.geom.choff[n];
    }
    const int nchunks = (eos - bos + kChunk - 1) / kChunk;
    const int64_t head_row = ((int64_t)b * p.geom.Hv + hv) * p.geom.T;

    elem *hS = reinterpret_cast<elem *>(smem + L::h_off);
    const bool stage_h = p.h != nullptr && !p.v_first;   // uniform: both groups run the second barrier or neither

    if (wave_id() >= CW) {
        // ------------------------------- loader waves -------------------------------------------
        const int tid = threadIdx.x - CW * 64;
        // The tiles of two steps are in flight at once: while step c is computed, those of step c + 1 are committed to
        // LDS and those of step c + 2 are on their way into the other register set, so that a load has two steps
        // to arrive.  Past the last step the loads re-read the last one (never committed), which keeps the number of
        // operations between a load and the commit that waits for it the same in every step.
        struct Tiles {
            TileCopy<kThreads, kChunk, K> tw, tq, tk;
            TileCopy<kThreads, kChunk, VS> tu;
            TileCopy<kThreads, kChunk, kChunk> ta;
            float dec;
        };
        Tiles t0, t1;
        auto fetch = [&](Tiles &t, int c) {
            c = min(c, nchunks - 1);
            const int start = bos + c * kChunk;
            const int len = min(kChunk, eos - start);
            const int64_t row = head_row + start;
            t.tw.fetch(p.w + row * K, K, len, tid);
            t.tq.fetch(p.qg + row * K, K, len, tid);
            t.tk.fetch(reinterpret_cast<const elem *>(p.kg) + row * K, K, len, tid);
            t.tu.fetch(reinterpret_cast<const elem *>(p.u) + row * V + slab * VS, V, len, tid);
            t.ta.fetch(p.aqk + row * (kChunk * SUB) + kChunk * (c % SUB), kChunk * SUB, len, tid);   // diagonal block
            t.dec = p.dec[(((int64_t)b * p.geom.NT + chunk0 + c / SUB) * p.geom.Hv + hv) * K + min(tid, K - 1)];
        };
        auto commit = [&](const Tiles &t, int c) {
            unsigned char *buf = smem + (c & 1) * L::buf_bytes;
            const int len = min(kChunk, eos - (bos + c * kChunk));
            t.tw.commit(reinterpret_cast<elem *>(buf + L::w_off), pw, len, tid);
            t.tq.commit(reinterpret_cast<elem *>(buf + L::q_off), pw, len, tid);
            t.tk.commit(reinterpret_cast<elem *>(buf + L::k_off), pt, len, tid);
            t.tu.commit(reinterpret_cast<elem *>(buf + L::u_off), pu, len, tid);
            t.ta.commit(reinterpret_cast<elem *>(buf + L::a_off), pb, len, tid);
            if (tid < K) reinterpret_cast<float *>(buf + L::d_off)[tid] = t.dec;
        };
        // v_new of step c sits in the u tile of buffer c & 1; a thread writes out exactly the pieces it later commits.
        // Both outputs are read from LDS before the barrier and stored after it, behind the loads of the next step.
        constexpr int NV = TileCopy<kThreads, kChunk, VS>::N, NH = K * (VS / 8) / kThreads;
        u32x4 vr[NV], hr[NH];
        auto read_vn = [&](int c) {
            const elem *uS = reinterpret_cast<const elem *>(smem + (c & 1) * L::buf_bytes + L::u_off);
#pragma unroll
            for (int m = 0; m < NV; ++m) {
                const int idx = m * kThreads + tid;
                vr[m] = *reinterpret_cast<const u32x4 *>(uS + (idx / (VS / 8)) * pu + (idx % (VS / 8)) * 8);
            }
        };
        auto store_vn = [&](int c) {
            const int start = bos + c * kChunk;
            const int len = min(kChunk, eos - start);
            elem *vg = p.v_new + (head_row + start) * V + slab * VS;
#pragma unroll
            for (int m = 0; m < NV; ++m) {
                const int idx = m * kThreads + tid;
                const int r = idx / (VS / 8), c8 = (idx % (VS / 8)) * 8;
                if (r < len) *reinterpret_cast<u32x4 *>(vg + (int64_t)r * V + c8) = vr[m];
            }
        };
        auto read_h = [&]() {
#pragma unroll
            for (int m = 0; m < NH; ++m) {
                const int idx = m * kThreads + tid;
                hr[m] = *reinterpret_cast<const u32x4 *>(hS + (idx / (VS / 8)) * ph + (idx % (VS / 8)) * 8);
            }
        };
        auto store_h = [&](int c) {   // the state at the start of step c, the first of its chunk
            elem *hg = p.h + b * p.h_sb + (int64_t)(chunk0 + c / SUB) * p.h_sc + hv * p.h_sh + slab * VS;
#pragma unroll
            for (int m = 0; m < NH; ++m) {
                const int idx = m * kThreads + tid;
                *reinterpret_cast<u32x4 *>(hg + (int64_t)(idx / (VS / 8)) * V + (idx % (VS / 8)) * 8) = hr[m];
            }
        };
        // one step: `ahead` takes the tiles of step c + 2, `next` holds those of step c + 1
        auto step = [&](Tiles &ahead, const Tiles &next, int c) {
            const bool with_h = stage_h && c > 0 && ((c - 1) % SUB) == 0, with_vn = p.v_new && c > 0;
            if (with_h) read_h();
            if (with_vn) read_vn(c - 1);
            if (stage_h) lds_barrier();   // the state tile of the step before has been read
            fetch(ahead, c + 2);
            if (c + 1 < nchunks) commit(next, c + 1);
            // the stores go last: the commit waits for everything issued before the loads it needs, and by the next
            // commit these stores are a whole step old
            if (with_h) store_h(c - 1);
            if (with_vn) store_vn(c - 1);
            lds_barrier();                // the loads of step c + 2 stay in flight
        };
        if (nchunks > 0) {
            fetch(t0, 0);
            commit(t0, 0);
            fetch(t1, 1);
        }
        lds_barrier();
        for (int c = 0; c < nchunks; c += 2) {
            step(t0, t1, c);
            if (c + 1 < nchunks) step(t1, t0, c + 1);
        }
        if (p.v_new && nchunks > 0) {
            read_vn(nchunks - 1);
            store_vn(nchunks - 1);
        }
        if (stage_h && nchunks > 0 && ((nchunks - 1) % SUB) == 0) {
            read_h();
            store_h(nchunks - 1);
        }
        return;
    }

    // --------------------------------- compute waves ---------------------------------------------
    const int wv = wave_id();
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const int vcol0 = slab * VS + wv * 16;
    f32x4 hacc[KT];
    auto state_off = [&](int kk, int v) -> int64_t { return p.v_first ? (int64_t)v * K + kk : (int64_t)kk * V + v; };
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        f32x4 a = zero4();
        if (p.h0) {
            const float *s = p.h0 + n * p.s_sn + hv * p.s_sh;
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = s[state_off(16 * kt + 4 * lg + e, vcol0 + li)];
        }
        hacc[kt] = a;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // initial state loaded before the loop (vmcnt(0))
    char *og = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.o.p)) + b * p.o.sb + hv * p.o.sh + vcol0);
    auto state_to_tile = [&]() {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) acc_to_tile(hS, ph, 16 * kt, wv * 16, hacc[kt]);
    };
    __syncthreads();

    elemx8 hB[KS], hQ[QF ? KS : 1], vprev[2] = {};
    for (int c = 0; c < nchunks; ++c) {
        const unsigned char *buf = smem + (c & 1) * L::buf_bytes;
        const elem *wS = reinterpret_cast<const elem *>(buf + L::w_off);
        const elem *qS = reinterpret_cast<const elem *>(buf + L::q_off);
        const elem *kS = reinterpret_cast<const elem *>(buf + L::k_off);
        elem *uS = const_cast<elem *>(reinterpret_cast<const elem *>(buf + L::u_off));
        const elem *aS = reinterpret_cast<const elem *>(buf + L::a_off);
        const float *dS = reinterpret_cast<const float *>(buf + L::d_off);
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
        const int64_t row = head_row + start;
        const bool first = SUB == 1 || (c % SUB) == 0;   // first step of a chunk

        if (first) {
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                hB[j] = frag_from_acc(hacc[2 * j], hacc[2 * j + 1]);
                if constexpr (QF) hQ[j] = pack_operand<true>(hacc[2 * j], hacc[2 * j + 1]);
            }
        }
        if (p.h && p.v_first && first) {   // [V][K] blocks: the lane's four K rows are contiguous
            elem *hg = p.h + b * p.h_sb + (int64_t)(chunk0 + c / SUB) * p.h_sc + hv * p.h_sh;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const elemx8 f = hB[kt >> 1];
                const elemx4 q4 = (kt & 1) ? elemx4{f[4], f[5], f[6], f[7]} : elemx4{f[0], f[1], f[2], f[3]};
                *reinterpret_cast<elemx4 *>(hg + (int64_t)(vcol0 + li) * K + 16 * kt + 4 * lg) = q4;
            }
        }

        // v_new = u - w S ;  o = scale qg S.  Every operand read is in flight before the first product, so the LDS
        // latency is paid once per chunk instead of once per contraction step.
        f32x4 vn[4], oacc[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) vn[rt] = oacc[rt] = zero4();
        {
            elemx8 wf[KS][4];
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) wf[j][rt] = frag_kc(wS, pw, rt * 16, 32 * j);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) vn[rt] = mfma16x32(wf[j][rt], hB[j], vn[rt]);
        }
        // second step of a 128-token chunk: rows of the coupling block Aqk21 straight from memory (rows past the
        // end re-read the last valid row; their outputs are never stored)
        elemx8 a21[4][2];
        if (SUB == 2 && !first) {
            const elem *ag = p.aqk + row * (kChunk * SUB) + 4 * lg;
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const elem *ar = ag + (int64_t)min(rt * 16 + li, len - 1) * (kChunk * SUB);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    a21[rt][j] = cat8(*reinterpret_cast<const elemx4 *>(ar + 32 * j), *reinterpret_cast<const elemx4 *>(ar + 32 * j + 16));
            }
        }
        {
            elemx8 qf[KS][4];
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) qf[j][rt] = frag_kc(qS, pw, rt * 16, 32 * j);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) oacc[rt] = mfma16x32_as<QF>(qf[j][rt], QF ? hQ[j] : hB[j], oacc[rt]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (stage_h) {   // the copying waves have read the state tile of the step before; the state is still that of
            lds_barrier();   // this step's start
            if (first) state_to_tile();
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const finex4 uu = as_fine(frag_tr4(uS, pu, wv * 16, rt * 16));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                vn[rt][e] = (float)uu[e] - vn[rt][e];
                oacc[rt][e] *= p.scale;
            }
        }
        if (p.v_new) {   // over the wave's own columns of u, which no other wave reads
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc_to_tile(uS, pu, rt * 16, wv * 16, vn[rt]);
        }
        // o += Aqk v_new ;  S <- 2^{g_last} S + kg^T v_new   (v_new as fp16 against the fp16 kg)
        elemx8 vB[2];
        finex8 vF[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            vB[j] = frag_from_acc(vn[2 * j], vn[2 * j + 1]);
            vF[j] = fine_from_acc(vn[2 * j], vn[2 * j + 1]);
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (2 * j <= rt) oacc[rt] = mfma16x32(frag_kc(aS, pb, rt * 16, 32 * j), vB[j], oacc[rt]);
        if (SUB == 2) {
            if (!first) {
#pragma unroll
                for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                    for (int j = 0; j < 2; ++j) oacc[rt] = mfma16x32(a21[rt][j], vprev[j], oacc[rt]);
            }
            vprev[0] = vB[0];
            vprev[1] = vB[1];
        }
        {
            f32x4 dk[KT];
            elemx8 kf[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) kf[kt] = frag_tr(kS, pt, kt * 16, 0);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) dk[kt] = lds4(dS + 16 * kt + 4 * lg);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                if (first) hacc[kt] *= dk[kt];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) hacc[kt] = mfma16x32(as_fine(kf[kt]), vF[0], hacc[kt]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) kf[kt] = frag_tr(kS, pt, kt * 16, 32);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) hacc[kt] = mfma16x32(as_fine(kf[kt]), vF[1], hacc[kt]);
        }
        char *ob = og + (int64_t)start * p.o.st * 2;
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) acc_to_global(ob, (int64_t)p.o.st * 2, rt * 16, len, oacc[rt]);
        lds_barrier();   // nothing waits for the stores of o
    }

    if (p.hT) {
        float *s = p.hT + n * p.s_sn + hv * p.s_sh;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) s[state_off(16 * kt + 4 * lg + e, vcol0 + li)] = hacc[kt][e];
    }
}

// More than 128 channels: the tiles of one step fill the LDS, so nothing is double-buffered.  256 threads, all four
// waves copy the tiles of a step, compute it (same products, operand fragments read as they are used so that the
// registers hold the 256 x 16 state of the wave and little else), and write the staged outputs.  Three barriers a step.
template <int K> struct WideScanSmem {
    static constexpr int pw = K + 8, pt = K + 16, pu = 64 + 8, pb = 72, ph = 64 + 8;
    static constexpr size_t w_off = 0;
    static constexpr size_t q_off = w_off + (size_t)kChunk * pw * 2;
    static constexpr size_t k_off = q_off + (size_t)kChunk * pw * 2;
    static constexpr size_t u_off = k_off + (size_t)kChunk * pt * 2;
    static constexpr size_t a_off = u_off + (size_t)kChunk * pu * 2;
    static constexpr size_t d_off = a_off + (size_t)kChunk * pb * 2;
    static constexpr size_t h_off = d_off + (size_t)K * 4;
    static constexpr size_t bytes = h_off + (size_t)K * ph * 2;
};

template <int K, int SUB>
__global__ void __launch_bounds__(kThreads) kda_scan_wide_kernel(const KdaScanParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    typedef WideScanSmem<K> L;
    constexpr int VS = 64;
    constexpr int pw = L::pw, pt = L::pt, pu = L::pu, pb = L::pb, ph = L::ph;
    constexpr int KT = K / 16, KS = K / 32;
    elem *wS = reinterpret_cast<elem *>(smem + L::w_off), *qS = reinterpret_cast<elem *>(smem + L::q_off);
    elem *kS = reinterpret_cast<elem *>(smem + L::k_off), *uS = reinterpret_cast<elem *>(smem + L::u_off);
    elem *aS = reinterpret_cast<elem *>(smem + L::a_off), *hS = reinterpret_cast<elem *>(smem + L::h_off);
    float *dS = reinterpret_cast<float *>(smem + L::d_off);

    int slab, hv, n;
    chain_of_block(slab, hv, n);
    const int V = p.geom.V;
    int b = n, bos = 0, eos = p.geom.T, chunk0 = 0;
    if (p.geom.cu != nullptr) {
        b = 0;
        bos = p.geom.cu[n];
        eos = p.geom.cu[n + 1];
        chunk0 = p.geom.choff[n];
    }
    const int nchunks = (eos - bos + kChunk - 1) / kChunk;
    const int64_t head_row = ((int64_t)b * p.geom.Hv + hv) * p.geom.T;
    const bool stage_h = p.h != nullptr && !p.v_first;
    const int tid = threadIdx.x, wv = wave_id();
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const int vcol0 = slab * VS + wv * 16;

    f32x4 hacc[KT];
    auto state_off = [&](int kk, int v) -> int64_t { return p.v_first ? (int64_t)v * K + kk : (int64_t)kk * V + v; };
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        f32x4 a = zero4();
        if (p.h0) {
            const float *s = p.h0 + n * p.s_sn + hv * p.s_sh;
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = s[state_off(16 * kt + 4 * lg + e, vcol0 + li)];
        }
        hacc[kt] = a;
    }
    char *og = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.o.p)) + b * p.o.sb + hv * p.o.sh + vcol0);

    elemx8 hB[KS], vprev[2] = {};
    for (int c = 0; c < nchunks; ++c) {
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
        const int64_t row = head_row + start;
        const bool first = SUB == 1 || (c % SUB) == 0;   // first step of a chunk
        const int chunk = chunk0 + c / SUB;

        load_tile<kThreads>(wS, pw, p.w + row * K, K, kChunk, K, len);
        load_tile<kThreads>(qS, pw, p.qg + row * K, K, kChunk, K, len);
        load_tile<kThreads>(kS, pt, reinterpret_cast<const elem *>(p.kg) + row * K, K, kChunk, K, len);
        load_tile<kThreads>(uS, pu, reinterpret_cast<const elem *>(p.u) + row * V + slab * VS, V, kChunk, VS, len);
        load_tile<kThreads>(aS, pb, p.aqk + row * (kChunk * SUB) + kChunk * (c % SUB), kChunk * SUB, kChunk, kChunk, len);
        for (int i = tid; i < K; i += kThreads) dS[i] = p.dec[(((int64_t)b * p.geom.NT + chunk) * p.geom.Hv + hv) * K + i];
        __syncthreads();   // tiles of this step in place

        if (first) {
#pragma unroll
            for (int j = 0; j < KS; ++j) hB[j] = frag_from_acc(hacc[2 * j], hacc[2 * j + 1]);
            if (p.h && p.v_first) {   // [V][K] blocks: the lane's four K rows are contiguous
                elem *hg = p.h + b * p.h_sb + (int64_t)chunk * p.h_sc + hv * p.h_sh;
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    const elemx8 f = hB[kt >> 1];
                    const elemx4 q4 = (kt & 1) ? elemx4{f[4], f[5], f[6], f[7]} : elemx4{f[0], f[1], f[2], f[3]};
                    *reinterpret_cast<elemx4 *>(hg + (int64_t)(vcol0 + li) * K + 16 * kt + 4 * lg) = q4;
                }
            }
            if (stage_h) {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) acc_to_tile(hS, ph, 16 * kt, wv * 16, hacc[kt]);
            }
        }

        // v_new = u - w S ;  o = scale qg S
        f32x4 vn[4], oacc[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) vn[rt] = oacc[rt] = zero4();
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) vn[rt] = mfma16x32(frag_kc(wS, pw, rt * 16, 32 * j), hB[j], vn[rt]);
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) oacc[rt] = mfma16x32(frag_kc(qS, pw, rt * 16, 32 * j), hB[j], oacc[rt]);
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const finex4 uu = as_fine(frag_tr4(uS, pu, wv * 16, rt * 16));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                vn[rt][e] = (float)uu[e] - vn[rt][e];
                oacc[rt][e] *= p.scale;
            }
        }
        if (p.v_new) {   // over the wave's own columns of u, which no other wave reads
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc_to_tile(uS, pu, rt * 16, wv * 16, vn[rt]);
        }
        // o += Aqk v_new ;  S <- 2^{g_last} S + kg^T v_new   (v_new as fp16 against the fp16 kg)
        elemx8 vB[2];
        finex8 vF[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            vB[j] = frag_from_acc(vn[2 * j], vn[2 * j + 1]);
            vF[j] = fine_from_acc(vn[2 * j], vn[2 * j + 1]);
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (2 * j <= rt) oacc[rt] = mfma16x32(frag_kc(aS, pb, rt * 16, 32 * j), vB[j], oacc[rt]);
        if (SUB == 2) {
            if (!first) {   // second step of a 128-token chunk: the coupling block Aqk21 times the first step's v_new,
                            // its rows straight from memory (rows past the end re-read the last valid row)
                const elem *ag = p.aqk + row * (kChunk * SUB) + 4 * lg;
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) {
                    const elem *ar = ag + (int64_t)min(rt * 16 + li, len - 1) * (kChunk * SUB);
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        oacc[rt] = mfma16x32(cat8(*reinterpret_cast<const elemx4 *>(ar + 32 * j),
                                                  *reinterpret_cast<const elemx4 *>(ar + 32 * j + 16)), vprev[j], oacc[rt]);
                }
            }
            vprev[0] = vB[0];
            vprev[1] = vB[1];
        }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            if (first) hacc[kt] *= lds4(dS + 16 * kt + 4 * lg);
            hacc[kt] = mfma16x32(as_fine(frag_tr(kS, pt, kt * 16, 0)), vF[0], hacc[kt]);
            hacc[kt] = mfma16x32(as_fine(frag_tr(kS, pt, kt * 16, 32)), vF[1], hacc[kt]);
        }
        char *ob = og + (int64_t)start * p.o.st * 2;
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) acc_to_global(ob, (int64_t)p.o.st * 2, rt * 16, len, oacc[rt]);
        __syncthreads();   // every tile has been read; v_new and the state tile are complete
        if (p.v_new) store_tile<kThreads>(p.v_new + row * V + slab * VS, V, uS, pu, VS, len);
        if (stage_h && first)
            store_tile<kThreads>(p.h + b * p.h_sb + (int64_t)chunk * p.h_sc + hv * p.h_sh + slab * VS, V, hS, ph, VS, K);
        __syncthreads();   // staged outputs read before the next step's tiles replace them
    }

    if (p.hT) {
        float *s = p.hT + n * p.s_sn + hv * p.s_sh;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) s[state_off(16 * kt + 4 * lg + e, vcol0 + li)] = hacc[kt][e];
    }
}

// =============================================================================================
// host side
// =============================================================================================
struct Layout {
    int ib, ih, it;   // dims of batch / head / token; ib < 0 when rank 3
    bool rank3() const { return ib < 0; }
};

int parse_layout(const char *op, const char *layout, Layout &L) {
    FLA_REQUIRE(layout != nullptr, FLA_ERR_NULL, "%s: layout must not be null.", op);
    if (!strcmp(layout, "BSND")) L = Layout{0, 2, 1};
    else if (!strcmp(layout, "BNSD")) L = Layout{0, 1, 2};
    else if (!strcmp(layout, "TND")) L = Layout{-1, 1, 0};
    else if (!strcmp(layout, "NTD")) L = Layout{-1, 0, 1};
    else return fail(FLA_ERR_UNSUPPORTED, "%s: layout must be uppercase and one of BSND, BNSD, TND, NTD.", op);
    return FLA_OK;
}

// [.., D] activation in layout L: checks rank, extents, alignment and returns the strided view
int layout_view(const char *op, const char *name, const fla_tensor *t, const Layout &L, int64_t B, int64_t H, int64_t T,
                int64_t D, int dtype_mask, int64_t &sb, int64_t &sh, int64_t &st) {
    int rc = check_tensor(t, op, name, L.rank3() ? 3 : 4, dtype_mask);
    if (rc) return rc;
    const int last = t->ndim - 1;
    FLA_REQUIRE((L.rank3() || t->shape[L.ib] == B) && t->shape[L.ih] == H && t->shape[L.it] == T && t->shape[last] == D,
                FLA_ERR_SHAPE, "%s: shape of %s does not match the selected layout.", op, name);
    FLA_REQUIRE(inner_unit(t), FLA_ERR_SHAPE, "%s: innermost stride of %s must be 1.", op, name);
    sb = L.rank3() ? 0 : t->stride[L.ib];
    sh = t->stride[L.ih];
    st = t->stride[L.it];
    const int64_t al = 16 / (int64_t)dtype_size(t->dtype);
    FLA_REQUIRE(sb % al == 0 && sh % al == 0 && st % al == 0 && reinterpret_cast<uintptr_t>(t->data) % 16 == 0, FLA_ERR_SHAPE,
                "%s: rows of %s must be 16-byte aligned.", op, name);
    FLA_REQUIRE(st >= 0 && st < (1 << 24), FLA_ERR_SHAPE, "%s: token stride of %s must be below 2^24 elements.", op, name);
    return FLA_OK;
}

// head-major output [B,Hv,T,D] (or [Hv,T,D]); contiguous
int head_major(const char *op, const char *name, const fla_tensor *t, bool rank3, int64_t B, int64_t H, int64_t T, int64_t D,
               int dtype, int also = -1) {
    int rc = check_tensor(t, op, name, rank3 ? 3 : 4, dt_bit(dtype) | (also < 0 ? 0 : dt_bit(also)));
    if (rc) return rc;
    const int o = rank3 ? 0 : 1;
    FLA_REQUIRE((rank3 || t->shape[0] == B) && t->shape[o] == H && t->shape[o + 1] == T && t->shape[o + 2] == D &&
                    is_contiguous(t) && reinterpret_cast<uintptr_t>(t->data) % 16 == 0,
                FLA_ERR_SHAPE, "%s: %s must be a contiguous head-major tensor [..,%lld,%lld,%lld].", op, name, (long long)H,
                (long long)T, (long long)D);
    return FLA_OK;
}

inline bool present(const fla_tensor *t) { return t != nullptr && t->data != nullptr; }
inline size_t align256(size_t x) { return (x + 255) / 256 * 256; }

template <int K, int V, bool C128, bool QGF>
int launch_intra_kernel(const KdaIntraParams &p, hipStream_t stream) {
    const size_t smem = IntraSmem<K, V>::bytes;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kda_intra_kernel<K, V, C128, QGF>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("kda_intra", stream, (kda_intra_kernel<K, V, C128, QGF>), chunk_head_grid(p.geom, p.geom.NT * (C128 ? 2 : 1), p.geom.Hv),
               dim3(kIntraThreads), smem, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

template <int K, int V>
int launch_intra(const KdaIntraParams &p, hipStream_t stream) {
    int rc;
    if (p.qg_fine) {
        if constexpr (K <= 128 && !kFineIsElem) {
            FLA_REQUIRE(!p.c128, FLA_ERR_UNSUPPORTED, "chunk_kda_fwd: a float16 qg beside other elements is built for chunk_size 64.");
            rc = launch_intra_kernel<K, V, false, true>(p, stream);
        } else {
            return fail(FLA_ERR_UNSUPPORTED, "chunk_kda_fwd: a float16 qg beside other elements is built for K <= 128.");
        }
    } else {
        rc = p.c128 ? launch_intra_kernel<K, V, true, false>(p, stream) : launch_intra_kernel<K, V, false, false>(p, stream);
    }
    if (rc) return rc;
    if (p.c128) {
        KdaCrossParams cp{p.geom, p.x1, p.x2, p.w, p.aqk, p.akk, p.u16, p.u, p.scale};
        const size_t csmem = CrossSmem<K, V>::bytes;
        FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kda_cross_kernel<K, V>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)csmem));
        FLA_LAUNCH("kda_cross", stream, (kda_cross_kernel<K, V>), dim3(p.geom.NT, p.geom.Hv, p.geom.B), dim3(kThreads), csmem,
                   stream, cp);
        FLA_HIP_CHECK(hipGetLastError());
    }
    return FLA_OK;
}

template <int K, int SUB, bool QF, int VS>
int launch_scan_as(const KdaScanParams &p, hipStream_t stream) {
    const size_t smem = ScanSmem<K>::bytes;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kda_scan_kernel<K, SUB, QF, VS>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("kda_scan", stream, (kda_scan_kernel<K, SUB, QF, VS>), dim3(p.geom.V / VS, p.geom.Hv, p.geom.N),
               dim3((VS / 16 + 4) * 64), smem, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}
template <int K, int SUB>
int launch_scan(const KdaScanParams &p, hipStream_t stream) {
    // 32-column slabs when 64-column ones leave compute units idle (see kda_scan_kernel)
    const bool narrow = (int64_t)p.geom.N * p.geom.Hv * (p.geom.V / 64) < (int64_t)num_cus();
    if constexpr (!kFineIsElem) {
        if (p.qg_fine) return narrow ? launch_scan_as<K, SUB, true, 32>(p, stream) : launch_scan_as<K, SUB, true, 64>(p, stream);
    }
    return narrow ? launch_scan_as<K, SUB, false, 32>(p, stream) : launch_scan_as<K, SUB, false, 64>(p, stream);
}

template <int K, int SUB>
int launch_scan_wide(const KdaScanParams &p, hipStream_t stream) {
    const size_t smem = WideScanSmem<K>::bytes;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kda_scan_wide_kernel<K, SUB>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("kda_scan", stream, (kda_scan_wide_kernel<K, SUB>), dim3(p.geom.V / 64, p.geom.Hv, p.geom.N), dim3(kThreads), smem,
               stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int kda_fwd_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
                 const fla_tensor *a_log, const fla_tensor *dt_bias, const fla_tensor *initial_state,
                 const fla_int_array *cu, const fla_int_array *ci, const char *layout, double scale, int64_t chunk_size,
                 bool safe_gate, double lower_bound, bool use_gate, bool state_v_first, const fla_tensor *attn_out,
                 const fla_tensor *final_state, const fla_tensor *gk, const fla_tensor *aqk, const fla_tensor *akk,
                 const fla_tensor *w, const fla_tensor *u, const fla_tensor *qg, const fla_tensor *kg,
                 const fla_tensor *v_new, const fla_tensor *h, void *ws, uint64_t ws_size, hipStream_t stream,
                 uint64_t *query) {
    const char *op = "chunk_kda_fwd";
    Layout L;
    int rc;
    if ((rc = parse_layout(op, layout, L))) return rc;
    FLA_REQUIRE(chunk_size == 64 || chunk_size == 128, FLA_ERR_SHAPE, "%s: chunk_size must be 64 or 128.", op);
    const int C = (int)chunk_size;
    if ((rc = check_tensor(q, op, "q", L.rank3() ? 3 : 4, dt_bit(kElemDtype)))) return rc;
    if ((rc = check_tensor(v, op, "v", L.rank3() ? 3 : 4, dt_bit(kElemDtype)))) return rc;
    const int last = q->ndim - 1;
    ChunkGeom geom{};
    geom.C = C;
    geom.B = L.rank3() ? 1 : (int)q->shape[L.ib];
    geom.T = (int)q->shape[L.it];
    geom.Hk = (int)q->shape[L.ih];
    geom.K = (int)q->shape[last];
    geom.Hv = (int)v->shape[L.ih];
    geom.V = (int)v->shape[last];
    FLA_REQUIRE(q->shape[L.it] < ((int64_t)1 << 31) && geom.B < 65536, FLA_ERR_SHAPE, "%s: extents too large.", op);
    FLA_REQUIRE(geom.Hk > 0 && geom.Hv >= geom.Hk && geom.Hv % geom.Hk == 0 && geom.Hv <= 128, FLA_ERR_SHAPE,
                "%s: H/HV must satisfy 0 < H <= HV <= 128 and HV %% H == 0.", op);
    FLA_REQUIRE(((geom.K == 64 || geom.K == 128) && (geom.V == geom.K || geom.V == 2 * geom.K)) || (geom.K == 256 && geom.V == 256),
                FLA_ERR_UNSUPPORTED, "%s: implemented head sizes are K in {64,128} with V in {K, 2K} and K = V = 256, got K=%d V=%d.",
                op, geom.K, geom.V);
    const int64_t B = geom.B, T = geom.T, Hk = geom.Hk, Hv = geom.Hv, K = geom.K, V = geom.V;
    const int bf = dt_bit(kElemDtype), f32 = dt_bit(FLA_F32);
    KdaIntraParams ip{};
    if ((rc = layout_view(op, "q", q, L, B, Hk, T, K, bf, ip.q.sb, ip.q.sh, ip.q.st))) return rc;
    if ((rc = layout_view(op, "k", k, L, B, Hk, T, K, bf, ip.k.sb, ip.k.sh, ip.k.st))) return rc;
    if ((rc = layout_view(op, "v", v, L, B, Hv, T, V, bf, ip.v.sb, ip.v.sh, ip.v.st))) return rc;
    ip.q.p = q->data;
    ip.k.p = k->data;
    ip.v.p = v->data;
    {   // g: scalar loads, no alignment requirement beyond the element
        if ((rc = check_tensor(g, op, "g", L.rank3() ? 3 : 4, bf | f32))) return rc;
        FLA_REQUIRE((L.rank3() || g->shape[L.ib] == B) && g->shape[L.ih] == Hv && g->shape[L.it] == T &&
                        g->shape[g->ndim - 1] == K && inner_unit(g),
                    FLA_ERR_SHAPE, "%s: v/g/beta shapes do not match the selected layout.", op);
        ip.g = g->data;
        ip.g_elem = g->dtype != FLA_F32;
        ip.g_sb = L.rank3() ? 0 : g->stride[L.ib];
        ip.g_sh = g->stride[L.ih];
        ip.g_st = g->stride[L.it];
        FLA_REQUIRE(ip.g_st >= 0 && ip.g_st < ((int64_t)1 << 23), FLA_ERR_SHAPE, "%s: token stride of g too large.", op);
    }
    {
        if ((rc = check_tensor(beta, op, "beta", L.rank3() ? 2 : 3, bf | f32))) return rc;
        FLA_REQUIRE((L.rank3() || beta->shape[L.ib] == B) && beta->shape[L.ih] == Hv && beta->shape[L.it] == T, FLA_ERR_SHAPE,
                    "%s: v/g/beta shapes do not match the selected layout.", op);
        ip.beta = View3{beta->data, L.rank3() ? 0 : beta->stride[L.ib], beta->stride[L.ih], beta->stride[L.it],
                        beta->dtype == FLA_F32 ? 0 : 1};
    }
    if (use_gate) {
        FLA_REQUIRE(present(a_log) && a_log->ndim == 1 && a_log->shape[0] == Hv && a_log->dtype == FLA_F32 &&
                        a_log->stride[0] == 1,
                    FLA_ERR_SHAPE, "%s: A_log must be float32 [HV] when use_gate_in_kernel=True.", op);
        if (present(dt_bias))
            FLA_REQUIRE(dt_bias->ndim == 1 && dt_bias->shape[0] == Hv * K && dt_bias->dtype == FLA_F32 && dt_bias->stride[0] == 1,
                        FLA_ERR_SHAPE, "%s: dt_bias must be float32 [HV*K].", op);
        FLA_REQUIRE(!safe_gate || (lower_bound >= -5.0 && lower_bound < 0.0), FLA_ERR_SHAPE,
                    "%s: lower_bound must be in [-5, 0) for safe gate.", op);
    }
    Varlen vl;
    if ((rc = build_varlen(vl, op, cu, ci, C, T))) return rc;
    FLA_REQUIRE(!vl.enabled || B == 1, FLA_ERR_SHAPE, "%s: rank4 varlen input requires B=1.", op);
    FLA_REQUIRE(!vl.enabled || vl.N <= 1024, FLA_ERR_SHAPE, "%s: varlen input supports at most 1024 sequences.", op);
    geom.NT = vl.enabled ? vl.NT : (int)((T + C - 1) / C);
    geom.N = vl.enabled ? vl.N : (int)B;
    const int64_t NT = geom.NT, N = geom.N;

    // outputs
    KdaScanParams sp{};
    if ((rc = layout_view(op, "attn_out", attn_out, L, B, Hv, T, V, bf, sp.o.sb, sp.o.sh, sp.o.st))) return rc;
    sp.o.p = attn_out->data;
    if ((rc = head_major(op, "Aqk", aqk, L.rank3(), B, Hv, T, C, kElemDtype))) return rc;
    if ((rc = head_major(op, "Akk", akk, L.rank3(), B, Hv, T, C, kElemDtype))) return rc;
    if (present(gk) && (rc = head_major(op, "gk", gk, L.rank3(), B, Hv, T, K, FLA_F32))) return rc;
    if (present(w) && (rc = head_major(op, "w", w, L.rank3(), B, Hv, T, K, kElemDtype))) return rc;
    if (present(u) && (rc = head_major(op, "u", u, L.rank3(), B, Hv, T, V, kElemDtype))) return rc;
    // qg and kg may be float16 tensors whatever the element type: the precision in which the scan reads kg anyway, and
    // in which a reverse scan (chunk_kda_bwd_dhu) wants both
    if (present(qg) && (rc = head_major(op, "qg", qg, L.rank3(), B, Hv, T, K, kElemDtype, FLA_F16))) return rc;
    if (present(kg) && (rc = head_major(op, "kg", kg, L.rank3(), B, Hv, T, K, kElemDtype, FLA_F16))) return rc;
    FLA_REQUIRE(geom.K <= 128 || ((!present(qg) || qg->dtype == kElemDtype) && (!present(kg) || kg->dtype == kElemDtype)),
                FLA_ERR_UNSUPPORTED, "%s: float16 qg / kg beside other elements are built for K <= 128.", op);
    if (present(v_new) && (rc = head_major(op, "v_new", v_new, L.rank3(), B, Hv, T, V, kElemDtype))) return rc;
    const int64_t d2 = state_v_first ? V : K, d3 = state_v_first ? K : V;
    auto check_state = [&](const fla_tensor *s, const char *name) -> int {
        int r = check_tensor(s, op, name, 4, f32);
        if (r) return r;
        FLA_REQUIRE(s->shape[0] == N && s->shape[1] == Hv && s->shape[2] == d2 && s->shape[3] == d3 && s->stride[3] == 1 &&
                        s->stride[2] == d3,
                    FLA_ERR_SHAPE, "%s: %s shape/dtype does not match state_v_first.", op, name);
        return FLA_OK;
    };
    if (present(initial_state) && (rc = check_state(initial_state, "initial_state"))) return rc;
    if (present(final_state) && (rc = check_state(final_state, "final_state"))) return rc;
    if (present(h)) {
        if ((rc = check_tensor(h, op, "h", L.rank3() ? 4 : 5, bf))) return rc;
        const int o = L.rank3() ? 0 : 1;
        FLA_REQUIRE((L.rank3() || h->shape[0] == B) && h->shape[o] == NT && h->shape[o + 1] == Hv && h->shape[o + 2] == d2 &&
                        h->shape[o + 3] == d3 && h->stride[o + 3] == 1 && h->stride[o + 2] == d3,
                    FLA_ERR_SHAPE, "%s: h must be [..,NT=%lld,HV,%lld,%lld].", op, (long long)NT, (long long)d2, (long long)d3);
        sp.h = static_cast<elem *>(h->data);
        sp.h_sb = L.rank3() ? 0 : h->stride[0];
        sp.h_sc = h->stride[o];
        sp.h_sh = h->stride[o + 1];
    }

    // workspace: varlen table | decay rows | the intermediates the caller did not ask for
    const size_t rows = (size_t)B * Hv * T;
    size_t off = vl.bytes();
    const size_t dec_off = off;
    off += align256((size_t)B * NT * Hv * K * 4);
    size_t w_off = 0, u_off = 0, qg_off = 0, kg_off = 0, x1_off = 0, x2_off = 0;
    // u and kg go to the scan as fp16 (`fine`): with fp16 elements the caller's tensors serve, otherwise the workspace
    // holds the fp16 copies whether or not the caller also takes u and kg
    const bool kg_is_fine = present(kg) && kg->dtype == FLA_F16;   // always so with fp16 elements
    const bool fine_u_ws = !kFineIsElem || !present(u), fine_kg_ws = !kg_is_fine;
    if (C == 128) {
        x1_off = off;
        off += align256(rows * K * 2);
        x2_off = off;
        off += align256(rows * K * 2);
    }
    if (!present(w)) { w_off = off; off += align256(rows * K * 2); }
    if (fine_u_ws) { u_off = off; off += align256(rows * V * 2); }
    if (!present(qg)) { qg_off = off; off += align256(rows * K * 2); }
    if (fine_kg_ws) { kg_off = off; off += align256(rows * K * 2); }
    if (query) {
        *query = off;
        return FLA_OK;
    }
    FLA_REQUIRE(off == 0 || (ws && ws_size >= off), FLA_ERR_WORKSPACE, "%s: workspace of %zu bytes required.", op, off);
    FLA_REQUIRE(reinterpret_cast<uintptr_t>(ws) % 256 == 0, FLA_ERR_WORKSPACE, "%s: workspace must be 256-byte aligned.", op);
    if ((rc = upload_varlen(vl, ws, stream))) return rc;
    geom.cu = vl.d_cu;
    geom.choff = vl.d_choff;
    geom.tab = vl.d_tab;
    if (B == 0 || T == 0 || NT == 0) return FLA_OK;
    unsigned char *wsb = static_cast<unsigned char *>(ws);

    ip.geom = geom;
    // token-major q, k, v, g (a token's row holds every head): neighbouring workgroups take the heads of one chunk
    ip.geom.head_fast = geom.Hv > 1 && ip.q.st > ip.q.sh && (int64_t)geom.NT * 2 <= 65535 ? 1 : 0;
    ip.a_log = use_gate ? static_cast<const float *>(a_log->data) : nullptr;
    ip.dt_bias = use_gate && present(dt_bias) ? static_cast<const float *>(dt_bias->data) : nullptr;
    ip.use_gate = use_gate;
    ip.safe_gate = safe_gate;
    ip.lower_bound = (float)lower_bound;
    ip.scale = (float)scale;
    ip.gk = present(gk) ? static_cast<float *>(gk->data) : nullptr;
    ip.aqk = static_cast<elem *>(aqk->data);
    ip.akk = static_cast<elem *>(akk->data);
    ip.w = present(w) ? static_cast<elem *>(w->data) : reinterpret_cast<elem *>(wsb + w_off);
    ip.u16 = fine_u_ws ? reinterpret_cast<fine *>(wsb + u_off) : static_cast<fine *>(u->data);
    ip.u = !kFineIsElem && present(u) ? static_cast<elem *>(u->data) : nullptr;
    ip.qg = present(qg) ? static_cast<elem *>(qg->data) : reinterpret_cast<elem *>(wsb + qg_off);
    ip.kg16 = fine_kg_ws ? reinterpret_cast<fine *>(wsb + kg_off) : static_cast<fine *>(kg->data);
    ip.kg = present(kg) && !kg_is_fine ? static_cast<elem *>(kg->data) : nullptr;
    ip.qg_fine = !kFineIsElem && present(qg) && qg->dtype == FLA_F16;
    ip.dec = reinterpret_cast<float *>(wsb + dec_off);
    ip.c128 = C == 128;
    ip.x1 = reinterpret_cast<elem *>(wsb + x1_off);
    ip.x2 = reinterpret_cast<elem *>(wsb + x2_off);
    if (K == 256) rc = launch_intra<256, 256>(ip, stream);
    else if (K == 128 && V == 128) rc = launch_intra<128, 128>(ip, stream);
    else if (K == 128 && V == 256) rc = launch_intra<128, 256>(ip, stream);
    else if (K == 64 && V == 64) rc = launch_intra<64, 64>(ip, stream);
    else rc = launch_intra<64, 128>(ip, stream);
    if (rc) return rc;

    sp.geom = geom;
    sp.w = ip.w;
    sp.u = ip.u16;
    sp.qg = ip.qg;
    sp.kg = ip.kg16;
    sp.aqk = ip.aqk;
    sp.dec = ip.dec;
    sp.v_new = present(v_new) ? static_cast<elem *>(v_new->data) : nullptr;
    if (present(initial_state)) {
        sp.h0 = static_cast<const float *>(initial_state->data);
        sp.s_sn = initial_state->stride[0];
        sp.s_sh = initial_state->stride[1];
    }
    if (present(final_state)) {
        sp.hT = static_cast<float *>(final_state->data);
        FLA_REQUIRE(!sp.h0 || (final_state->stride[0] == sp.s_sn && final_state->stride[1] == sp.s_sh), FLA_ERR_SHAPE,
                    "%s: initial_state and final_state must share strides.", op);
        sp.s_sn = final_state->stride[0];
        sp.s_sh = final_state->stride[1];
    }
    sp.v_first = state_v_first;
    sp.scale = (float)scale;
    sp.qg_fine = ip.qg_fine;
    if (N == 0) return FLA_OK;
    if (K == 256) return C == 128 ? launch_scan_wide<256, 2>(sp, stream) : launch_scan_wide<256, 1>(sp, stream);
    if (C == 128) return K == 128 ? launch_scan<128, 2>(sp, stream) : launch_scan<64, 2>(sp, stream);
    return K == 128 ? launch_scan<128, 1>(sp, stream) : launch_scan<64, 1>(sp, stream);
}

}  // namespace
}  // namespace fla

FLA_ENTRY(fla_chunk_kda_fwd_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
    const fla_tensor *A_log, const fla_tensor *dt_bias, const fla_tensor *initial_state, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const char *layout, double scale, int64_t chunk_size, bool safe_gate,
    double lower_bound, bool use_gate_in_kernel, bool state_v_first, const fla_tensor *attn_out,
    const fla_tensor *final_state, const fla_tensor *gk, const fla_tensor *Aqk, const fla_tensor *Akk, const fla_tensor *w,
    const fla_tensor *u, const fla_tensor *qg, const fla_tensor *kg, const fla_tensor *v_new, const fla_tensor *h,
    uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_kda_fwd_get_workspace_size, q, k, v, g, beta, A_log, dt_bias, initial_state, cu_seqlens, chunk_indices, layout, scale, chunk_size, safe_gate, lower_bound, use_gate_in_kernel, state_v_first, attn_out, final_state, gk, Aqk, Akk, w, u, qg, kg, v_new, h, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "chunk_kda_fwd: workspace_size must not be null.");
    return fla::guarded([&] { return fla::kda_fwd_impl(q, k, v, g, beta, A_log, dt_bias, initial_state, cu_seqlens, chunk_indices, layout, scale,
                             chunk_size, safe_gate, lower_bound, use_gate_in_kernel, state_v_first, attn_out, final_state, gk,
                             Aqk, Akk, w, u, qg, kg, v_new, h, nullptr, 0, nullptr, workspace_size); });
}

FLA_ENTRY(fla_chunk_kda_fwd)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
    const fla_tensor *A_log, const fla_tensor *dt_bias, const fla_tensor *initial_state, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const char *layout, double scale, int64_t chunk_size, bool safe_gate,
    double lower_bound, bool use_gate_in_kernel, bool state_v_first, const fla_tensor *attn_out,
    const fla_tensor *final_state, const fla_tensor *gk, const fla_tensor *Aqk, const fla_tensor *Akk, const fla_tensor *w,
    const fla_tensor *u, const fla_tensor *qg, const fla_tensor *kg, const fla_tensor *v_new, const fla_tensor *h,
    void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_kda_fwd, q, k, v, g, beta, A_log, dt_bias, initial_state, cu_seqlens, chunk_indices, layout, scale, chunk_size, safe_gate, lower_bound, use_gate_in_kernel, state_v_first, attn_out, final_state, gk, Aqk, Akk, w, u, qg, kg, v_new, h, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::kda_fwd_impl(q, k, v, g, beta, A_log, dt_bias, initial_state, cu_seqlens, chunk_indices, layout, scale,
                             chunk_size, safe_gate, lower_bound, use_gate_in_kernel, state_v_first, attn_out, final_state, gk,
                             Aqk, Akk, w, u, qg, kg, v_new, h, workspace, workspace_size, static_cast<hipStream_t>(stream),
                             nullptr); });
}

#ifndef FLA_ELEM_F16
// =============================================================================================
// chunk_kda_fwd for callers that cannot allocate (stream capture, serving loops that forbid hipMalloc)
// =============================================================================================
// Same kernels as fla_chunk_kda_fwd; the buffer that entry point takes as `workspace` (the per-chunk decay rows
// and the intermediates the caller did not ask for) is a fixed array in device memory instead.  Every call on a
// device uses that device's one array: calls that overlap in time on one device race.  Nothing in the array has
// to start at zero - the intra kernel writes every element the scan kernel reads.
namespace fla {
namespace {

static __device__ __align__(256) unsigned char scratch[FLA_CHUNK_KDA_FWD_NOALLOC_SCRATCH_BYTES];

std::mutex g_scratch_mu;
void *g_scratch_ptr[16] = {};   // device address of `scratch` per device, resolved on the first call there

// The address is resolved on the first call on a device.  That call must not come while `stream` is being captured
// (a symbol lookup is no stream operation; inside a capture it is refused here rather than tried): one call outside
// the capture - fla_chunk_kda_fwd_noalloc itself, or fla_chunk_kda_fwd_noalloc_init - comes first.
int scratch_address(void **out, hipStream_t stream) {
    int dev = 0;
    FLA_HIP_CHECK(hipGetDevice(&dev));
    FLA_REQUIRE(dev >= 0 && dev < 16, FLA_ERR_UNSUPPORTED, "chunk_kda_fwd_noalloc: device index %d out of range.", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (stream != nullptr && hipStreamIsCapturing(stream, &capturing) == hipSuccess)
            FLA_REQUIRE(capturing == hipStreamCaptureStatusNone, FLA_ERR_UNSUPPORTED,
                        "chunk_kda_fwd_noalloc: the first call on a device resolves the scratch array's address and must "
                        "come before stream capture (call fla_chunk_kda_fwd_noalloc_init once).");
        void *ptr = nullptr;
        FLA_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        FLA_REQUIRE(ptr != nullptr, FLA_ERR_LAUNCH, "chunk_kda_fwd_noalloc: the scratch array has no device address.");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return FLA_OK;
}

}  // namespace
}  // namespace fla

extern "C" int fla_chunk_kda_fwd_noalloc_init(void) {
    return fla::guarded([&] {
        void *ptr = nullptr;
        return fla::scratch_address(&ptr, nullptr);
    });
}

extern "C" int fla_chunk_kda_fwd_noalloc(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
    const fla_tensor *A_log, const fla_tensor *dt_bias, const fla_tensor *initial_state, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const char *layout, double scale, int64_t chunk_size, bool safe_gate,
    double lower_bound, bool use_gate_in_kernel, bool state_v_first, const fla_tensor *attn_out,
    const fla_tensor *final_state, const fla_tensor *gk, const fla_tensor *Aqk, const fla_tensor *Akk, const fla_tensor *w,
    const fla_tensor *u, const fla_tensor *qg, const fla_tensor *kg, const fla_tensor *v_new, const fla_tensor *h,
    void *stream) {
    return fla::guarded([&]() -> int {
        const char *op = "chunk_kda_fwd_noalloc";
        // packed batches upload their chunk table through a pinned staging ring that grows on demand
        if ((cu_seqlens && cu_seqlens->data && cu_seqlens->size) || (chunk_indices && chunk_indices->data && chunk_indices->size))
            return fla::fail(FLA_ERR_UNSUPPORTED, "%s: cu_seqlens / chunk_indices are not accepted (their upload allocates "
                             "pinned staging memory); use fla_chunk_kda_fwd.", op);
        const bool f16 = q != nullptr && q->dtype == FLA_F16;
        uint64_t need = 0;
        int rc = f16 ? fla_chunk_kda_fwd_get_workspace_size_f16(q, k, v, g, beta, A_log, dt_bias, initial_state, nullptr, nullptr,
                                                               layout, scale, chunk_size, safe_gate, lower_bound,
                                                               use_gate_in_kernel, state_v_first, attn_out, final_state, gk, Aqk,
                                                               Akk, w, u, qg, kg, v_new, h, &need)
                     : fla::kda_fwd_impl(q, k, v, g, beta, A_log, dt_bias, initial_state, nullptr, nullptr, layout, scale,
                                         chunk_size, safe_gate, lower_bound, use_gate_in_kernel, state_v_first, attn_out,
                                         final_state, gk, Aqk, Akk, w, u, qg, kg, v_new, h, nullptr, 0, nullptr, &need);
        if (rc) return rc;
        if (need > (uint64_t)FLA_CHUNK_KDA_FWD_NOALLOC_SCRATCH_BYTES)
            return fla::fail(FLA_ERR_WORKSPACE,
                             "%s: this call needs %llu bytes of scratch, the fixed array holds %llu; pass w, u, qg and kg "
                             "(1 KiB per token and head at K=V=128 otherwise; the fp16 copies of u and kg that the state "
                             "scan reads stay in the scratch with bf16 elements, 512 B) or use fla_chunk_kda_fwd with a "
                             "workspace.",
                             op, (unsigned long long)need, (unsigned long long)FLA_CHUNK_KDA_FWD_NOALLOC_SCRATCH_BYTES);
        void *ptr = nullptr;
        if ((rc = fla::scratch_address(&ptr, static_cast<hipStream_t>(stream)))) return rc;
        if (f16)
            return fla_chunk_kda_fwd_f16(q, k, v, g, beta, A_log, dt_bias, initial_state, nullptr, nullptr, layout, scale,
                                         chunk_size, safe_gate, lower_bound, use_gate_in_kernel, state_v_first, attn_out,
                                         final_state, gk, Aqk, Akk, w, u, qg, kg, v_new, h, ptr,
                                         FLA_CHUNK_KDA_FWD_NOALLOC_SCRATCH_BYTES, stream);
        return fla::kda_fwd_impl(q, k, v, g, beta, A_log, dt_bias, initial_state, nullptr, nullptr, layout, scale, chunk_size,
                                 safe_gate, lower_bound, use_gate_in_kernel, state_v_first, attn_out, final_state, gk, Aqk, Akk,
                                 w, u, qg, kg, v_new, h, ptr, FLA_CHUNK_KDA_FWD_NOALLOC_SCRATCH_BYTES,
                                 static_cast<hipStream_t>(stream), nullptr);
    });
}
#endif  // !FLA_ELEM_F16
