// gdn_chunk_fwd: the whole gated-delta-rule chunk forward in ONE persistent kernel.
//
// Replaces the six-operator composition of examples/flash_gated_delta_rule.py:796-881
// (cumsum -> kkt -> solve_tri -> recompute_w_u -> fwd_h -> fwd_o).  Only q, k, v, g, beta are
// read from HBM and only o (+ the cumulated gate and the final state) written; A, w, u, h and
// v_new never leave the chip.
//
// One 256-thread workgroup per (sequence, value head, 64*CT-column slab of V) walks the chunks
// of its sequence.  Wave w owns 16*CT columns of V for all K rows of the state, which stays in
// fp32 MFMA accumulators for the whole sequence.  Per chunk (C = 64 tokens):
//   A  scores      wave 0 : the four 16x16 diagonal blocks of beta_i e^{G_i-G_j} <k_i,k_j>, then
//                           their unit-lower inverses by fp32 forward substitution (lane = column)
//                  waves 1-3 : the six off-diagonal blocks (stored negated, bf16) and the masked,
//                           decayed q k^T tile P
//   B  WY solve    block forward substitution X_i = D_i^-1 (B_i - sum_{j<i} A_ij X_j) on the
//                  right-hand sides [k beta e^G | v beta]; X_j feeds the next block product
//                  straight from accumulator registers.  Wave w solves its own u columns (kept
//                  in registers, residuals as hi+lo bf16 pairs) and two 16-column tiles of w
//                  (rounded to bf16 into LDS, since w is an MFMA operand next)
//   C  scan        v_new = u - w h ; o = scale (e^G (q h) + P v_new) ;
//                  h <- e^{g_last} h + k^T (v_new e^{g_last - g})   (v_new e^.. as hi+lo bf16)
//   D  epilogue    o tile stored; the next chunk's q/k/v, prefetched into registers during A-C,
//                  are written to LDS
// Math and rounding points: SURVEY of the reference stages in chunk_scaled_dot_kkt/README.md:11-29,
// recompute_w_u_fwd/README.md:12-32, chunk_gated_delta_rule_fwd_h/README.md:16-30,
// chunk_fwd_o/README.md:6-15; acceptance oracle examples/flash_gated_delta_rule.py:1545-1571.
#include "gdn_common.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;

struct FusedParams {
    ChunkGeom geom;
    View4 q, k, v, o;   // o viewed as [B, Hv, T, V] through strides
    View3 g, beta;      // raw per-token log gate and beta, any layout through strides
    float *g_out;       // cumulated gate, or null
    int64_t go_sb, go_sh, go_st;
    const float *h0;
    float *hT;
    int64_t s_sn, s_sh;
    float scale;
    int slabs;
    int remap;          // 1: co-locate the slabs of one head on one XCD
};

template <int K, int CT> struct FusedSmem {
    static constexpr int VS = 64 * CT;
    static constexpr int pq = K + 8, pk = K + 16, pv = VS + 16, pa = kChunk + 8, pw = K + 8, pp = kChunk + 8,
                         po = VS + 8, pd = 24, a32_blk = 16 * 16 + 16;
    static constexpr size_t q_off = 0;
    static constexpr size_t k_off = q_off + (size_t)kChunk * pq * 2;
    static constexpr size_t v_off = k_off + (size_t)kChunk * pk * 2;
    static constexpr size_t a_off = v_off + (size_t)kChunk * pv * 2;
    static constexpr size_t w_off = a_off + (size_t)kChunk * pa * 2;
    static constexpr size_t p_off = w_off + (size_t)kChunk * pw * 2;
    static constexpr size_t o_off = p_off + (size_t)kChunk * pp * 2;
    static constexpr size_t d_off = o_off + (size_t)kChunk * po * 2;
    static constexpr size_t a32_off = d_off + (size_t)4 * 16 * pd * 2;
    static constexpr size_t tab_off = a32_off + (size_t)4 * a32_blk * 4;
    static constexpr size_t bytes = tab_off + 4 * kChunk * 4;
};

// D^-1 R for one 16x16 diagonal block; HILO feeds R as hi + lo bf16 pairs.
template <bool HILO>
__device__ __forceinline__ f32x4 diag_mul(const bf16 *dblk, int pd, f32x4 r) {
    const bf16x4 a = frag_kc4(dblk, pd, 0, 0);
    const bf16x4 hi = cvt4(r);
    f32x4 acc = mfma16x16(a, hi, f32x4{0.f, 0.f, 0.f, 0.f});
    if (HILO) {
        f32x4 rest;
#pragma unroll
        for (int e = 0; e < 4; ++e) rest[e] = r[e] - (float)hi[e];
        acc = mfma16x16(a, cvt4(rest), acc);
    }
    return acc;
}

// Block forward substitution for one 16-column tile.  In: r[i] = rows 16i..16i+15 of the
// right-hand side (accumulator layout).  Out: r[i] = the same rows of (I + A0)^-1 RHS.
// aS holds -A0 (bf16), dS the four inverted diagonal blocks.
template <bool HILO>
__device__ __forceinline__ void wy_solve_tile(const bf16 *aS, int pa, const bf16 *dS, int pd, f32x4 (&r)[4]) {
    r[0] = diag_mul<HILO>(dS, pd, r[0]);
    r[1] = mfma16x16(frag_kc4(aS, pa, 16, 0), cvt4(r[0]), r[1]);
    r[1] = diag_mul<HILO>(dS + 16 * pd, pd, r[1]);
    const bf16x8 x01 = frag_from_acc(r[0], r[1]);
    r[2] = mfma16x32(frag_kc(aS, pa, 32, 0), x01, r[2]);
    r[2] = diag_mul<HILO>(dS + 32 * pd, pd, r[2]);
    r[3] = mfma16x32(frag_kc(aS, pa, 48, 0), x01, r[3]);
    r[3] = mfma16x16(frag_kc4(aS, pa, 48, 32), cvt4(r[2]), r[3]);
    r[3] = diag_mul<HILO>(dS + 48 * pd, pd, r[3]);
}

template <int K, int CT>
__global__ void __launch_bounds__(kThreads) gdn_fused_kernel(const FusedParams p) {
    typedef FusedSmem<K, CT> L;
    constexpr int VS = L::VS, pq = L::pq, pk = L::pk, pv = L::pv, pa = L::pa, pw = L::pw, pp = L::pp, po = L::po,
                  pd = L::pd;
    constexpr int KT = K / 16, KS = K / 32;
    constexpr int QCH = kChunk * (K / 8) / kThreads;    // 16-byte chunks of a q/k tile per thread
    constexpr int VCH = kChunk * (VS / 8) / kThreads;   // ... of the v slab tile
    extern __shared__ __align__(16) unsigned char smem[];
    bf16 *qS = reinterpret_cast<bf16 *>(smem + L::q_off);
    bf16 *kS = reinterpret_cast<bf16 *>(smem + L::k_off);
    bf16 *vS = reinterpret_cast<bf16 *>(smem + L::v_off);
    bf16 *aS = reinterpret_cast<bf16 *>(smem + L::a_off);
    bf16 *wS = reinterpret_cast<bf16 *>(smem + L::w_off);
    bf16 *pS = reinterpret_cast<bf16 *>(smem + L::p_off);
    bf16 *oS = reinterpret_cast<bf16 *>(smem + L::o_off);
    bf16 *dS = reinterpret_cast<bf16 *>(smem + L::d_off);
    float *a32 = reinterpret_cast<float *>(smem + L::a32_off);
    float *GS = reinterpret_cast<float *>(smem + L::tab_off);  // cumulated gate G_t
    float *EG = GS + kChunk;                                    // e^{G_t}
    float *BS = EG + kChunk;                                    // beta_t
    float *BEG = BS + kChunk;                                   // beta_t e^{G_t}

    // ---- which (sequence, head, slab) ---------------------------------------------------
    int lin = blockIdx.x;
    int slab, hv, n;
    if (p.remap) {  // blocks L and L+8 run on the same XCD: make them the two slabs of one head
        const int pair = (lin >> 4) * 8 + (lin & 7);
        slab = (lin >> 3) & 1;
        hv = pair % p.geom.Hv;
        n = pair / p.geom.Hv;
    } else {
        slab = lin % p.slabs;
        hv = (lin / p.slabs) % p.geom.Hv;
        n = lin / (p.slabs * p.geom.Hv);
    }
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    const int V = p.geom.V;
    int b = n, bos = 0, eos = p.geom.T;
    if (p.geom.cu != nullptr) {
        b = 0;
        bos = p.geom.cu[n];
        eos = p.geom.cu[n + 1];
    }
    const int nchunks = (eos - bos + kChunk - 1) / kChunk;
    const int tid = threadIdx.x;
    const int wv = wave_id();
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const int vcol0 = slab * VS + wv * 16 * CT;  // first V column of this wave (global)
    const int vtile0 = wv * CT;                  // first 16-column tile of this wave inside the slab

    // ---- state ------------------------------------------------------------------------------
    f32x4 hacc[KT][CT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
            if (p.h0) {
                const float *s = p.h0 + n * p.s_sn + hv * p.s_sh;
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = s[(int64_t)(16 * kt + 4 * lg + e) * V + vcol0 + 16 * ct + li];
            }
            hacc[kt][ct] = a;
        }

    const bf16 *qg = static_cast<const bf16 *>(p.q.p) + b * p.q.sb + hk * p.q.sh;
    const bf16 *kg = static_cast<const bf16 *>(p.k.p) + b * p.k.sb + hk * p.k.sh;
    const bf16 *vg = static_cast<const bf16 *>(p.v.p) + b * p.v.sb + hv * p.v.sh + slab * VS;
    bf16 *og = static_cast<bf16 *>(const_cast<void *>(p.o.p)) + b * p.o.sb + hv * p.o.sh + slab * VS;

    // ---- register prefetch of one chunk's q, k, v rows and gates ------------------------------
    u32x4 pre_q[QCH], pre_k[QCH], pre_v[VCH];
    float pre_g = 0.f, pre_b = 0.f;
    auto prefetch = [&](int c) {
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
#pragma unroll
        for (int m = 0; m < QCH; ++m) {
            const int idx = tid + m * kThreads, r = idx / (K / 8), cc = (idx % (K / 8)) * 8;
            u32x4 zq = {0u, 0u, 0u, 0u}, zk = zq;
            if (r < len) {
                zq = *reinterpret_cast<const u32x4 *>(qg + (int64_t)(start + r) * p.q.st + cc);
                zk = *reinterpret_cast<const u32x4 *>(kg + (int64_t)(start + r) * p.k.st + cc);
            }
            pre_q[m] = zq;
            pre_k[m] = zk;
        }
#pragma unroll
        for (int m = 0; m < VCH; ++m) {
            const int idx = tid + m * kThreads, r = idx / (VS / 8), cc = (idx % (VS / 8)) * 8;
            u32x4 z = {0u, 0u, 0u, 0u};
            if (r < len) z = *reinterpret_cast<const u32x4 *>(vg + (int64_t)(start + r) * p.v.st + cc);
            pre_v[m] = z;
        }
        if (tid < kChunk) {
            pre_g = tid < len ? load_scalar(p.g, b, hv, start + tid) : 0.f;
            pre_b = tid < len ? load_scalar(p.beta, b, hv, start + tid) : 0.f;
        }
    };
    auto commit = [&](int c) {  // prefetched registers -> LDS tiles and gate tables of chunk c
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
#pragma unroll
        for (int m = 0; m < QCH; ++m) {
            const int idx = tid + m * kThreads, r = idx / (K / 8), cc = (idx % (K / 8)) * 8;
            *reinterpret_cast<u32x4 *>(qS + r * pq + cc) = pre_q[m];
            *reinterpret_cast<u32x4 *>(kS + r * pk + cc) = pre_k[m];
        }
#pragma unroll
        for (int m = 0; m < VCH; ++m) {
            const int idx = tid + m * kThreads, r = idx / (VS / 8), cc = (idx % (VS / 8)) * 8;
            *reinterpret_cast<u32x4 *>(vS + r * pv + cc) = pre_v[m];
        }
        if (wv == 0) {  // wave 0 holds token t = lane: chunk-local cumulative gate
            float G = wave_inclusive_scan(pre_g);
            const float g_end = __shfl(G, len - 1, kWave);
            if (l >= len) G = g_end;  // padded rows: finite, harmless (their q, k, v, beta are zero)
            const float eg = __expf(G);
            GS[l] = G;
            EG[l] = eg;
            BS[l] = pre_b;
            BEG[l] = pre_b * eg;
            if (p.g_out != nullptr && slab == 0 && l < len)
                p.g_out[b * p.go_sb + hv * p.go_sh + (int64_t)(start + l) * p.go_st] = G;
        }
    };

    if (nchunks > 0) {
        prefetch(0);
        commit(0);
    }
    __syncthreads();

    for (int c = 0; c < nchunks; ++c) {
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
        if (c + 1 < nchunks) prefetch(c + 1);

        // =========================== A: scores ===========================================
        if (wv == 0) {
            // diagonal blocks: fp32 into a32 (strictly lower part, rest zero)
#pragma unroll
            for (int I = 0; I < 4; ++I) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < K; kk += 32)
                    acc = mfma16x32(frag_kc(kS, pk, I * 16, kk), frag_kc(kS, pk, I * 16, kk), acc);
                // lane holds <k_s, k_t> for s = 16I + 4lg + e (row), t = 16I + li (column)
                const int t = I * 16 + li;
                const float gt = GS[t], bt = BS[t];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int s = I * 16 + 4 * lg + e;
                    acc[e] = s < t ? bt * __expf(fmaxf(gt - GS[s], -50.f)) * acc[e] : 0.f;
                }
                *reinterpret_cast<f32x4 *>(a32 + I * L::a32_blk + li * 16 + 4 * lg) = acc;
            }
            __builtin_amdgcn_wave_barrier();
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            // inverse of (I + A_II): lane = (block, column j); x[i] = row i of that column
            const int blk = lg, j = li;
            const float *ab = a32 + blk * L::a32_blk;
            float x[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) x[i] = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float acc = (i == j) ? 1.f : 0.f;
#pragma unroll
                for (int s4 = 0; s4 < (i + 3) / 4; ++s4) {
                    const f32x4 a = *reinterpret_cast<const f32x4 *>(ab + i * 16 + 4 * s4);
                    acc -= a[0] * x[4 * s4] + a[1] * x[4 * s4 + 1] + a[2] * x[4 * s4 + 2] + a[3] * x[4 * s4 + 3];
                }
                x[i] = acc;
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) dS[(blk * 16 + i) * pd + j] = (bf16)x[i];
        } else {
            // 6 off-diagonal score blocks + 16 tiles of P (10 computed, 6 zero) over waves 1..3
            for (int id = wv - 1; id < 22; id += 3) {
                if (id < 6) {
                    // (I, J): (1,0) (2,0) (2,1) (3,0) (3,1) (3,2)
                    const int I = id < 1 ? 1 : (id < 3 ? 2 : 3);
                    const int J = id < 1 ? 0 : (id < 3 ? id - 1 : id - 3);
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kk = 0; kk < K; kk += 32)
                        acc = mfma16x32(frag_kc(kS, pk, J * 16, kk), frag_kc(kS, pk, I * 16, kk), acc);
                    const int t = I * 16 + li;
                    const float gt = GS[t], bt = BS[t];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int s = J * 16 + 4 * lg + e;
                        acc[e] = -bt * __expf(fmaxf(gt - GS[s], -50.f)) * acc[e];
                    }
                    *reinterpret_cast<bf16x4 *>(aS + t * pa + J * 16 + 4 * lg) = cvt4(acc);
                } else {
                    const int pid = id - 6, I = pid >> 2, J = pid & 3;  // t block, s block
                    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
                    const int t = I * 16 + li;
                    if (J <= I) {
#pragma unroll
                        for (int kk = 0; kk < K; kk += 32)
                            acc = mfma16x32(frag_kc(kS, pk, J * 16, kk), frag_kc(qS, pq, I * 16, kk), acc);
                        const float gt = GS[t];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int s = J * 16 + 4 * lg + e;
                            acc[e] = s <= t ? acc[e] * __expf(fminf(gt - GS[s], 0.f)) : 0.f;
                        }
                    }
                    *reinterpret_cast<bf16x4 *>(pS + t * pp + J * 16 + 4 * lg) = cvt4(acc);
                }
            }
        }
        __syncthreads();  // #1: aS, dS, pS complete

        // =========================== B: WY solve =========================================
        f32x4 U[4][CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            f32x4 r[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bf16x4 vv = frag_tr4(vS, pv, (vtile0 + ct) * 16, 16 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) r[i][e] = (float)vv[e] * BS[16 * i + 4 * lg + e];
            }
            wy_solve_tile<true>(aS, pa, dS, pd, r);
#pragma unroll
            for (int i = 0; i < 4; ++i) U[i][ct] = r[i];
        }
#pragma unroll
        for (int m = 0; m < K / 64; ++m) {
            const int ctile = wv * (K / 64) + m;
            f32x4 r[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bf16x4 kv = frag_tr4(kS, pk, ctile * 16, 16 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) r[i][e] = (float)kv[e] * BEG[16 * i + 4 * lg + e];
            }
            wy_solve_tile<false>(aS, pa, dS, pd, r);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_to_tile(wS, pw, 16 * i, ctile * 16, r[i]);
        }
        __syncthreads();  // #2: wS complete

        // =========================== C: scan + output ====================================
        bf16x8 hB[KS][CT];
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) hB[j][ct] = frag_from_acc(hacc[2 * j][ct], hacc[2 * j + 1][ct]);

        f32x4 oacc[4][CT];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) oacc[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        // U <- v_new = u - w h (accumulated as -(w h - u)) ; oacc <- q h
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) U[rt][ct] *= -1.f;
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const bf16x8 wf = frag_kc(wS, pw, rt * 16, 32 * j);
                const bf16x8 qf = frag_kc(qS, pq, rt * 16, 32 * j);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    oacc[rt][ct] = mfma16x32(qf, hB[j][ct], oacc[rt][ct]);
                    U[rt][ct] = mfma16x32(wf, hB[j][ct], U[rt][ct]);
                }
            }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) U[rt][ct] *= -1.f;
        // o = scale (e^{G_t} q h + P v_new)
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float eg = EG[rt * 16 + 4 * lg + e];
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) oacc[rt][ct][e] *= eg;
            }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            bf16x8 vb[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) vb[ct] = frag_from_acc(U[2 * j][ct], U[2 * j + 1][ct]);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const bf16x8 pf = frag_kc(pS, pp, rt * 16, 32 * j);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) oacc[rt][ct] = mfma16x32(pf, vb[ct], oacc[rt][ct]);
            }
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc_to_tile(oS, po, rt * 16, (vtile0 + ct) * 16, oacc[rt][ct] * p.scale);

        // h <- e^{g_last} h + k^T (v_new e^{g_last - g}), the right operand as hi + lo bf16
        const float g_last = GS[len - 1];
        const float dec_all = __expf(g_last);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) hacc[kt][ct] *= dec_all;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            bf16x8 vhi[CT], vlo[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                f32x4 a0 = U[2 * j][ct], a1 = U[2 * j + 1][ct], r0, r1;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a0[e] *= __expf(g_last - GS[32 * j + 4 * lg + e]);
                    a1[e] *= __expf(g_last - GS[32 * j + 16 + 4 * lg + e]);
                }
                const bf16x4 h0 = cvt4(a0), h1 = cvt4(a1);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    r0[e] = a0[e] - (float)h0[e];
                    r1[e] = a1[e] - (float)h1[e];
                }
                vhi[ct] = cat8(h0, h1);
                vlo[ct] = frag_from_acc(r0, r1);
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const bf16x8 kf = frag_tr(kS, pk, kt * 16, 32 * j);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    hacc[kt][ct] = mfma16x32(kf, vhi[ct], hacc[kt][ct]);
                    hacc[kt][ct] = mfma16x32(kf, vlo[ct], hacc[kt][ct]);
                }
            }
        }
        __syncthreads();  // #3: every read of this chunk's tiles is done, oS complete

        // =========================== D: epilogue ==========================================
        store_tile<kThreads>(og + (int64_t)start * p.o.st, p.o.st, oS, po, VS, len);
        if (c + 1 < nchunks) commit(c + 1);
        __syncthreads();  // #4
    }

    if (p.hT) {
        float *s = p.hT + n * p.s_sn + hv * p.s_sh;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s[(int64_t)(16 * kt + 4 * lg + e) * V + vcol0 + 16 * ct + li] = hacc[kt][ct][e];
    }
}

template <int K, int CT>
int launch_fused(FusedParams &p, hipStream_t stream) {
    typedef FusedSmem<K, CT> L;
    const int64_t total = (int64_t)p.geom.N * p.geom.Hv * p.slabs;
    p.remap = (p.slabs == 2 && total % 16 == 0) ? 1 : 0;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(gdn_fused_kernel<K, CT>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)L::bytes));
    FLA_LAUNCH("gdn_fused", stream, (gdn_fused_kernel<K, CT>), dim3((unsigned)total), dim3(kThreads), L::bytes, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int fused_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
               double scale, const fla_tensor *initial_state, bool output_final_state, const fla_int_array *cu,
               int64_t chunk_size, const fla_tensor *o, const fla_tensor *g_cumsum, const fla_tensor *final_state,
               void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "gdn_chunk_fwd";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v, nullptr, chunk_size, geom))) return rc;
    const int bf = dt_bit(FLA_BF16);
    if ((rc = check_bhtd(op, "q", q, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    // g, beta: [B, T, Hv]
    auto check_bth = [&](const fla_tensor *t, const char *name, int mask) -> int {
        int r = check_tensor(t, op, name, 3, mask);
        if (r) return r;
        FLA_REQUIRE(t->shape[0] == geom.B && t->shape[1] == geom.T && t->shape[2] == geom.Hv, FLA_ERR_SHAPE,
                    "%s: %s must be [B,T,Hv] = [%d,%d,%d].", op, name, geom.B, geom.T, geom.Hv);
        return FLA_OK;
    };
    const int gmask = dt_bit(FLA_F32) | dt_bit(FLA_BF16);
    if ((rc = check_bth(g, "g", gmask))) return rc;
    if ((rc = check_bth(beta, "beta", gmask))) return rc;
    if ((rc = check_tensor(o, op, "o", 4, bf))) return rc;
    FLA_REQUIRE(o->shape[0] == geom.B && o->shape[1] == geom.T && o->shape[2] == geom.Hv && o->shape[3] == geom.V &&
                    inner_unit(o) && o->stride[0] % 8 == 0 && o->stride[1] % 8 == 0 && o->stride[2] % 8 == 0,
                FLA_ERR_SHAPE, "%s: o must be a 16-byte aligned [B,T,Hv,V].", op);
    const bool has_gout = g_cumsum && g_cumsum->data;
    if (has_gout && (rc = check_bth(g_cumsum, "g_cumsum", dt_bit(FLA_F32)))) return rc;
    Varlen vl;
    if ((rc = build_varlen(vl, op, cu, nullptr, kChunk, geom.T))) return rc;
    FLA_REQUIRE(!vl.enabled || geom.B == 1, FLA_ERR_SHAPE, "%s: batch must be 1 with cu_seqlens.", op);
    if (vl.enabled) {
        geom.NT = vl.NT;
        geom.N = vl.N;
    }
    auto check_state = [&](const fla_tensor *s, const char *name) -> int {
        int r = check_tensor(s, op, name, 4, dt_bit(FLA_F32));
        if (r) return r;
        FLA_REQUIRE(s->shape[0] == geom.N && s->shape[1] == geom.Hv && s->shape[2] == geom.K && s->shape[3] == geom.V &&
                        s->stride[3] == 1 && s->stride[2] == geom.V,
                    FLA_ERR_SHAPE, "%s: %s must be [N=%d,Hv,K,V] fp32 with contiguous K x V blocks.", op, name, geom.N);
        return FLA_OK;
    };
    const bool has_h0 = initial_state && initial_state->data;
    if (has_h0 && (rc = check_state(initial_state, "initial_state"))) return rc;
    if (output_final_state && (rc = check_state(final_state, "final_state"))) return rc;
    FLA_REQUIRE(geom.K == 128 || geom.K == 64, FLA_ERR_UNSUPPORTED, "%s: K must be 64 or 128, got %d.", op, geom.K);
    FLA_REQUIRE(geom.V % 64 == 0, FLA_ERR_UNSUPPORTED, "%s: V must be a multiple of 64, got %d.", op, geom.V);
    if (query) {
        *query = vl.bytes();
        return FLA_OK;
    }
    FLA_REQUIRE(vl.bytes() == 0 || (ws && ws_size >= vl.bytes()), FLA_ERR_WORKSPACE, "%s: workspace of %zu bytes required.",
                op, vl.bytes());
    if ((rc = upload_varlen(vl, ws, stream))) return rc;
    geom.cu = vl.d_cu;
    geom.choff = vl.d_choff;
    geom.tab = vl.d_tab;
    if (geom.N == 0 || geom.Hv == 0) return FLA_OK;

    FusedParams p{};
    p.geom = geom;
    p.q = view4(q);
    p.k = view4(k);
    p.v = view4(v);
    p.o = View4{o->data, o->stride[0], o->stride[2], o->stride[1]};  // [B,T,Hv,V] seen as [B,Hv,T,V]
    p.g = View3{g->data, g->stride[0], g->stride[2], g->stride[1], g->dtype == FLA_BF16 ? 1 : 0};
    p.beta = View3{beta->data, beta->stride[0], beta->stride[2], beta->stride[1], beta->dtype == FLA_BF16 ? 1 : 0};
    if (has_gout) {
        p.g_out = static_cast<float *>(g_cumsum->data);
        p.go_sb = g_cumsum->stride[0];
        p.go_sh = g_cumsum->stride[2];
        p.go_st = g_cumsum->stride[1];
    }
    p.h0 = has_h0 ? static_cast<const float *>(initial_state->data) : nullptr;
    p.hT = output_final_state ? static_cast<float *>(final_state->data) : nullptr;
    const fla_tensor *sref = has_h0 ? initial_state : (output_final_state ? final_state : nullptr);
    if (sref) {
        p.s_sn = sref->stride[0];
        p.s_sh = sref->stride[1];
    }
    if (has_h0 && output_final_state)
        FLA_REQUIRE(initial_state->stride[0] == final_state->stride[0] && initial_state->stride[1] == final_state->stride[1],
                    FLA_ERR_SHAPE, "%s: initial_state and final_state must share strides.", op);
    p.scale = (float)scale;

    // 128-column slabs (two 16-column tiles per wave) halve the per-FLOP LDS traffic and do the
    // score / w work once per head; 64-column slabs double the number of workgroups.  Use the
    // wide form once it alone fills the GPU.
    const int64_t chains = (int64_t)geom.N * geom.Hv;
    const bool wide = geom.V % 128 == 0 && chains * (geom.V / 128) >= (int64_t)num_cus();
    p.slabs = wide ? geom.V / 128 : geom.V / 64;
    if (geom.K == 128) return wide ? launch_fused<128, 2>(p, stream) : launch_fused<128, 1>(p, stream);
    return wide ? launch_fused<64, 2>(p, stream) : launch_fused<64, 1>(p, stream);
}

}  // namespace
}  // namespace fla

extern "C" int fla_gdn_chunk_fwd_get_workspace_size(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v,
                                                    const fla_tensor *g, const fla_tensor *beta, double scale,
                                                    const fla_tensor *initial_state, bool output_final_state,
                                                    const fla_int_array *cu_seqlens, int64_t chunk_size,
                                                    const fla_tensor *o, const fla_tensor *g_cumsum,
                                                    const fla_tensor *final_state, uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "gdn_chunk_fwd: workspace_size must not be null.");
    return fla::fused_impl(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, chunk_size, o,
                           g_cumsum, final_state, nullptr, 0, nullptr, workspace_size);
}

extern "C" int fla_gdn_chunk_fwd(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
                                 const fla_tensor *beta, double scale, const fla_tensor *initial_state,
                                 bool output_final_state, const fla_int_array *cu_seqlens, int64_t chunk_size,
                                 const fla_tensor *o, const fla_tensor *g_cumsum, const fla_tensor *final_state,
                                 void *workspace, uint64_t workspace_size, void *stream) {
    return fla::fused_impl(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, chunk_size, o,
                           g_cumsum, final_state, workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr);
}
