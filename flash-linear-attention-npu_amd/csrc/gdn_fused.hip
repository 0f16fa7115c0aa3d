// gdn_chunk_fwd: the whole gated-delta-rule chunk forward in ONE persistent kernel.
//
// Replaces the six-operator composition of examples/flash_gated_delta_rule.py:796-881
// (cumsum -> kkt -> solve_tri -> recompute_w_u -> fwd_h -> fwd_o).  Only q, k, v, g, beta are
// read from HBM and only o (+ the cumulated gate and the final state) written; A, w, u, h and
// v_new never leave the chip.
//
// One 256-thread workgroup per (sequence, value head, 64*CT-column slab of V) walks the chunks
// of its sequence.  Wave w owns 16*CT columns of V for all K rows of the state, which stays in
// fp32 MFMA accumulators for the whole sequence.  Per chunk (C = 64 tokens, 16-token blocks):
//   A  scores      wave w: row block w of  A0 = beta_i e^{G_i-G_j} <k_i,k_j>  (off-diagonal blocks
//                  stored negated as bf16; the diagonal block inverted in registers with the
//                  nilpotent product (I-A)(I+A^2)(I+A^4)(I+A^8), eight 16x16x16 MFMAs) and row
//                  block 3-w of the masked, decayed q k^T tile P  (5 tiles per wave)
//   B  WY solve    block forward substitution X_i = D_i^-1 (B_i - sum_{j<i} A_ij X_j) on the
//                  right-hand sides [k beta e^G | v beta]; X_j feeds the next block product
//                  straight from accumulator registers.  Wave w solves its own u columns (kept
//                  in fp32 registers, residuals fed as hi+lo bf16 pairs) and K/64 16-column
//                  tiles of w (rounded to bf16 into LDS, since w is an MFMA operand next)
//   C  scan        v_new = u - w h ; o = scale (e^G (q h) + P v_new) ;
//                  h <- e^{g_last} h + k^T (v_new e^{g_last - g})   (right operand as hi+lo bf16)
// The next chunk's q/k/v rows are prefetched into registers at the top of a chunk and written to
// the second LDS buffer between B and C, so HBM latency hides behind A and B.  LDS operand reads
// are software-pipelined by hand one k-step ahead of the MFMAs that consume them.
// Math and rounding points of the stages: chunk_scaled_dot_kkt/README.md:11-29,
// recompute_w_u_fwd/README.md:12-32, chunk_gated_delta_rule_fwd_h/README.md:16-30,
// chunk_fwd_o/README.md:6-15; acceptance oracle examples/flash_gated_delta_rule.py:1545-1571.
#include "gdn_common.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;

#define FLA_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

struct FusedParams {
    ChunkGeom geom;
    View4 q, k, v, o;   // o viewed as [B, Hv, T, V] through strides
    View3 g, beta;      // raw per-token log gate and beta, any layout through strides
    float *g_out;       // cumulated gate, or null
    int64_t go_sb, go_sh, go_st;
    const float *h0;
    float *hT;
    int64_t s_sn, s_sh, s_sk, s_sv;   // strides of (sequence or pool row, head, key channel, value channel)
    const int32_t *slot;               // per sequence: the pool row that holds its state; null: row n
    int pool_rows;
    float scale;
    int slabs;
    int remap;          // 1: co-locate the slabs of one head on one XCD
    int l2norm;         // 1: q and k rows are L2-normalised (rstd = 1/sqrt(sum x^2 + 1e-6)) while they are staged
    // what a backward pass needs from the forward, each or null (pipelined kernel only):
    elem *h_out;        // state at the start of every chunk [B,Hv,NT,K,V]
    int64_t h_sb, h_sh, h_sc;
    View4 vn_out, w_out;   // v_new [B,Hv,T,V], w [B,Hv,T,K]
    // with l2norm: the normalised q and k [B,Hk,T,K] and their rstd (fp32 [B,Hk,T], contiguous), all four or none
    View4 qn_out, kn_out;
    float *q_rstd, *k_rstd;
    int64_t rs_sb, rs_sh;
};

// Row of the state tensors that belongs to sequence n: n itself, or the pool row the caller names for it.  A negative
// index means no row (the sequence starts from zero and its final state is dropped); one past the pool is clamped
// into it, so that a wrong index reads and writes a wrong row, never outside the allocation.
__device__ __forceinline__ int64_t state_row(const FusedParams &p, int n) {
    return p.slot ? (int64_t)min(p.slot[n], p.pool_rows - 1) : (int64_t)n;
}

template <int K, int CT> struct FusedSmem {
    static constexpr int VS = 64 * CT;
    static constexpr bool DB = CT == 1;   // q/k/v tiles double-buffered in LDS
    static constexpr int NB = DB ? 2 : 1;
    static constexpr int pq = K + 8, pk = KTile<K>::pitch, pv = VS + 16, pa = kChunk + 8, pw = K + 8, pp = kChunk + 8,
                         po = VS + 8, pd = 24;
    static constexpr size_t q_bytes = (size_t)kChunk * pq * 2, k_bytes = (size_t)kChunk * pk * 2,
                            v_bytes = (size_t)kChunk * pv * 2, tab_bytes = (6 * kChunk + 16) * 4;
    static constexpr size_t buf_bytes = q_bytes + k_bytes + v_bytes + tab_bytes;
    static constexpr size_t a_off = NB * buf_bytes;
    static constexpr size_t w_off = a_off + (size_t)kChunk * pa * 2;
    static constexpr size_t p_off = w_off + (size_t)kChunk * pw * 2;
    static constexpr size_t o_off = p_off + (size_t)kChunk * pp * 2;
    static constexpr size_t d_off = o_off + (size_t)kChunk * po * 2;
    static constexpr size_t bytes = d_off + (size_t)kChunk * pd * 2;
};

struct Tiles {      // one LDS buffer of chunk inputs
    elem *q, *k, *v;
    // per token: cumulated gate G, scale e^G, beta, beta e^G, and the factors of
    //   e^{G_t - G_s} = ROWF[t] * BLKF[blk(t)][blk(s)] * COLF[s]   for blk(s) < blk(t)
    // with ROWF[t] = e^{G_t - G(first token of blk(t))}, COLF[s] = e^{G(last token of blk(s)) - G_s};
    // every factor is <= 1 for non-positive gates, so nothing overflows.
    float *G, *EGS, *B, *BEG, *ROWF, *COLF, *BLKF;
};
template <int K, int CT>
__device__ __forceinline__ Tiles tiles_at(unsigned char *smem, int buf) {
    typedef FusedSmem<K, CT> L;
    unsigned char *b = smem + buf * L::buf_bytes;
    Tiles t;
    t.q = reinterpret_cast<elem *>(b);
    t.k = reinterpret_cast<elem *>(b + L::q_bytes);
    t.v = reinterpret_cast<elem *>(b + L::q_bytes + L::k_bytes);
    t.G = reinterpret_cast<float *>(b + L::q_bytes + L::k_bytes + L::v_bytes);
    t.EGS = t.G + kChunk;
    t.B = t.EGS + kChunk;
    t.BEG = t.B + kChunk;
    t.ROWF = t.BEG + kChunk;
    t.COLF = t.ROWF + kChunk;
    t.BLKF = t.COLF + kChunk;
    return t;
}

__device__ __forceinline__ f32x4 zero4() { return f32x4{0.f, 0.f, 0.f, 0.f}; }
__device__ __forceinline__ f32x4 lds4(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }

// ---------------------------------------------------------------------------------------------
// Phase A for wave W: row block I1 = W of the score matrix, row block I2 = 3 - W of P.
// ---------------------------------------------------------------------------------------------
template <int K, int W>
__device__ __forceinline__ void phase_a(const Tiles &t, elem *aS, elem *pS, elem *dS, float scale) {
    constexpr int I1 = W, I2 = 3 - W, JM = I1 > I2 ? I1 : I2, KS = K / 32;
    constexpr int pq = K + 8, pa = kChunk + 8, pp = kChunk + 8, pd = 24;
    const int l = lane_id(), li = l & 15, lg = l >> 4;

    f32x4 kacc[I1 + 1], pacc[I2 + 1];
#pragma unroll
    for (int J = 0; J <= I1; ++J) kacc[J] = zero4();
#pragma unroll
    for (int J = 0; J <= I2; ++J) pacc[J] = zero4();
    elemx8 kf[2][JM + 1], qf[2];
#pragma unroll
    for (int J = 0; J <= JM; ++J) kf[0][J] = KTile<K>::kc(t.k, 16 * J, 0);
    qf[0] = frag_kc(t.q, pq, 16 * I2, 0);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int cb = s & 1, nb = cb ^ 1;
        if (s + 1 < KS) {
#pragma unroll
            for (int J = 0; J <= JM; ++J) kf[nb][J] = KTile<K>::kc(t.k, 16 * J, 32 * (s + 1));
            qf[nb] = frag_kc(t.q, pq, 16 * I2, 32 * (s + 1));
        }
        FLA_SCHED_FENCE();
        // rows of the tile = tokens s of block J (A operand), columns = tokens t of block I (B operand)
#pragma unroll
        for (int J = 0; J <= I1; ++J) kacc[J] = mfma16x32(kf[cb][J], kf[cb][I1], kacc[J]);
#pragma unroll
        for (int J = 0; J <= I2; ++J) pacc[J] = mfma16x32(kf[cb][J], qf[cb], pacc[J]);
        FLA_SCHED_FENCE();
    }

    // lane holds (row s = 16J + 4lg + e, column t = 16I + li) of each tile
    const int t1 = 16 * I1 + li, t2 = 16 * I2 + li;
    const float gt1 = t.G[t1], bt1 = t.B[t1], gt2 = t.G[t2];
    const float rf1 = -bt1 * t.ROWF[t1], rf2 = scale * t.ROWF[t2];
#pragma unroll
    for (int J = 0; J < I1; ++J) {  // off-diagonal score blocks, negated: -beta_t e^{G_t-G_s} <k_s,k_t>
        const f32x4 cf = lds4(t.COLF + 16 * J + 4 * lg);
        const float coef = rf1 * t.BLKF[4 * I1 + J];
        f32x4 a;
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = coef * cf[e] * kacc[J][e];
        *reinterpret_cast<elemx4 *>(aS + t1 * pa + 16 * J + 4 * lg) = cvt4(a);
    }
#pragma unroll
    for (int J = 0; J < 4; ++J) {  // scale * P[t][s] = scale q_t.k_s e^{min(G_t-G_s,0)} for s <= t
        f32x4 a = zero4();
        if (J < I2) {
            const f32x4 cf = lds4(t.COLF + 16 * J + 4 * lg);
            const float coef = rf2 * t.BLKF[4 * I2 + J];
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = coef * cf[e] * pacc[J < I2 ? J : 0][e];
        } else if (J == I2) {
            const f32x4 gs = lds4(t.G + 16 * J + 4 * lg);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                a[e] = 4 * lg + e <= li ? scale * __expf(fminf(gt2 - gs[e], 0.f)) * pacc[I2][e] : 0.f;
        }
        *reinterpret_cast<elemx4 *>(pS + t2 * pp + 16 * J + 4 * lg) = cvt4(a);
    }

    // diagonal block A (16x16, strictly lower): both operand views from the symmetric raw tile
    const f32x4 gs = lds4(t.G + 16 * I1 + 4 * lg), bs = lds4(t.B + 16 * I1 + 4 * lg);
    f32x4 a1, a2, Y;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int r = 4 * lg + e;
        const float raw = kacc[I1][e];
        a1[e] = r < li ? bt1 * __expf(fmaxf(gt1 - gs[e], -50.f)) * raw : 0.f;    // A[li][r]
        a2[e] = li < r ? bs[e] * __expf(fmaxf(gs[e] - gt1, -50.f)) * raw : 0.f;  // A[r][li]
        Y[e] = (r == li ? 1.f : 0.f) - a1[e];                                     // (I - A^T)[r][li]
    }
    // An accumulator tile of M is the right operand of M and the left operand of M^T, so the
    // chains S_k = A^(2^k) and T_k = S_k^T are advanced together and
    //   Y <- Y + T_k Y   accumulates   Y = ((I-A)(I+A^2)(I+A^4)(I+A^8))^T = ((I+A)^-1)^T.
    const elemx4 A1 = cvt4(a1), A2 = cvt4(a2);
    const f32x4 S1 = mfma16x16(A1, A2, zero4());
    const f32x4 T1 = mfma16x16(A2, A1, zero4());
    const elemx4 S1b = cvt4(S1), T1b = cvt4(T1);
    Y = mfma16x16(S1b, cvt4(Y), Y);
    const f32x4 S2 = mfma16x16(T1b, S1b, zero4());
    const f32x4 T2 = mfma16x16(S1b, T1b, zero4());
    const elemx4 S2b = cvt4(S2);
    Y = mfma16x16(S2b, cvt4(Y), Y);
    const f32x4 S3 = mfma16x16(cvt4(T2), S2b, zero4());
    Y = mfma16x16(cvt4(S3), cvt4(Y), Y);
    // lane holds Dinv^T[4lg+e][li] = Dinv[li][4lg+e]: the left-operand layout, 8 contiguous bytes
    *reinterpret_cast<elemx4 *>(dS + (16 * I1 + li) * pd + 4 * lg) = cvt4(Y);
}

// D^-1 R for one diagonal block; hilo feeds R as hi + lo bf16 pairs.
__device__ __forceinline__ f32x4 diag_mul(elemx4 d, f32x4 r, bool hilo) {
    if (!hilo) return mfma16x16(d, cvt4(r), zero4());
    elemx4 hi, lo;
    split_hilo(r, hi, lo);
    return mfma16x16(d, lo, mfma16x16(d, hi, zero4()));
}

template <int K, int CT>
__global__ void __launch_bounds__(kThreads) gdn_fused_kernel(const FusedParams p) {
    typedef FusedSmem<K, CT> L;
    constexpr int VS = L::VS, pq = L::pq, pv = L::pv, pa = L::pa, pw = L::pw, pp = L::pp, po = L::po,
                  pd = L::pd;
    constexpr bool DB = L::DB;
    constexpr int KT = K / 16, KS = K / 32;
    constexpr int QCH = kChunk * (K / 8) / kThreads;    // 16-byte pieces of a q/k tile per thread
    constexpr int VCH = kChunk * (VS / 8) / kThreads;   // ... of the v slab tile
    constexpr int QROWS = kThreads / (K / 8), VROWS = kThreads / (VS / 8);
    constexpr int NTW = K / 64, NT = NTW + CT;          // w tiles per wave, all solved tiles per wave
    extern __shared__ __align__(16) unsigned char smem[];
    elem *aS = reinterpret_cast<elem *>(smem + L::a_off);
    elem *wS = reinterpret_cast<elem *>(smem + L::w_off);
    elem *pS = reinterpret_cast<elem *>(smem + L::p_off);
    elem *oS = reinterpret_cast<elem *>(smem + L::o_off);
    elem *dS = reinterpret_cast<elem *>(smem + L::d_off);

    // ---- which (sequence, head, slab) ---------------------------------------------------
    const int lin = blockIdx.x;
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
            f32x4 a = zero4();
            if (p.h0 && state_row(p, n) >= 0) {
                const float *s = p.h0 + state_row(p, n) * p.s_sn + hv * p.s_sh;
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = s[(int64_t)(16 * kt + 4 * lg + e) * p.s_sk + (int64_t)(vcol0 + 16 * ct + li) * p.s_sv];
            }
            hacc[kt][ct] = a;
        }

    // ---- prefetch addressing: one uniform base per tensor and chunk, 32-bit per-lane byte offsets
    // (row r of the chunk, 8 columns from cq / cv) computed once ------------------------------------
    const int rq = tid / (K / 8), cq = (tid % (K / 8)) * 8;
    const int rv = tid / (VS / 8), cv = (tid % (VS / 8)) * 8;
    const char *qbase = reinterpret_cast<const char *>(static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh + (int64_t)bos * p.q.st);
    const char *kbase = reinterpret_cast<const char *>(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)bos * p.k.st);
    const char *vbase = reinterpret_cast<const char *>(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)bos * p.v.st + slab * VS);
    char *obase = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.o.p)) + b * p.o.sb + hv * p.o.sh + (int64_t)bos * p.o.st + slab * VS);
    unsigned qoff[QCH], koff[QCH], voff[VCH], ooff[VCH];
#pragma unroll
    for (int m = 0; m < QCH; ++m) {
        qoff[m] = (unsigned)(((rq + m * QROWS) * p.q.st + cq) * 2);
        koff[m] = (unsigned)(((rq + m * QROWS) * p.k.st + cq) * 2);
    }
#pragma unroll
    for (int m = 0; m < VCH; ++m) {
        voff[m] = (unsigned)(((rv + m * VROWS) * p.v.st + cv) * 2);
        ooff[m] = (unsigned)(((rv + m * VROWS) * p.o.st + cv) * 2);
    }

    const float *gptr = static_cast<const float *>(p.g.p) + b * p.g.sb + hv * p.g.sh;
    const float *bptr = static_cast<const float *>(p.beta.p) + b * p.beta.sb + hv * p.beta.sh;
    u32x4 pre_q[QCH], pre_k[QCH], pre_v[VCH];
    float pre_g = 0.f, pre_b = 0.f;
    auto prefetch = [&](int c) {  // global -> registers
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
        const char *qb = qbase + (int64_t)c * kChunk * p.q.st * 2, *kb = kbase + (int64_t)c * kChunk * p.k.st * 2,
                   *vb = vbase + (int64_t)c * kChunk * p.v.st * 2;
        if (len == kChunk) {
#pragma unroll
            for (int m = 0; m < QCH; ++m) {
                pre_q[m] = *reinterpret_cast<const u32x4 *>(qb + qoff[m]);
                pre_k[m] = *reinterpret_cast<const u32x4 *>(kb + koff[m]);
            }
#pragma unroll
            for (int m = 0; m < VCH; ++m) pre_v[m] = *reinterpret_cast<const u32x4 *>(vb + voff[m]);
        } else {
            const u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int m = 0; m < QCH; ++m) {
                const bool in = rq + m * QROWS < len;
                pre_q[m] = in ? *reinterpret_cast<const u32x4 *>(qb + qoff[m]) : z;
                pre_k[m] = in ? *reinterpret_cast<const u32x4 *>(kb + koff[m]) : z;
            }
#pragma unroll
            for (int m = 0; m < VCH; ++m)
                pre_v[m] = rv + m * VROWS < len ? *reinterpret_cast<const u32x4 *>(vb + voff[m]) : z;
        }
        if (tid < len) {  // fp32 gates: plain loads, no dtype branch whose join would wait for them
            pre_g = gptr[(int64_t)(start + tid) * p.g.st];
            pre_b = bptr[(int64_t)(start + tid) * p.beta.st];
        } else {
            pre_g = 0.f;
            pre_b = 0.f;
        }
    };
    auto commit = [&](int c, const Tiles &t) {  // registers -> LDS tiles and gate tables of chunk c
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
#pragma unroll
        for (int m = 0; m < QCH; ++m) {
            *reinterpret_cast<u32x4 *>(t.q + (rq + m * QROWS) * pq + cq) = pre_q[m];
            *reinterpret_cast<u32x4 *>(t.k + KTile<K>::off(rq + m * QROWS, cq)) = pre_k[m];
        }
#pragma unroll
        for (int m = 0; m < VCH; ++m) *reinterpret_cast<u32x4 *>(t.v + (rv + m * VROWS) * pv + cv) = pre_v[m];
        if (wv == 0) {  // wave 0 holds token t = lane: chunk-local cumulative gate
            float G = wave_inclusive_scan(pre_g);
            const float g_end = read_lane(G, len - 1);
            if (l >= len) G = g_end;  // padded rows: finite, harmless (their q, k, v, beta are zero)
            // gate at the first / last token of each 16-token block
            const float s0 = read_lane(G, 0), s1 = read_lane(G, 16), s2 = read_lane(G, 32), s3 = read_lane(G, 48);
            const float e0 = read_lane(G, 15), e1 = read_lane(G, 31), e2 = read_lane(G, 47), e3 = read_lane(G, 63);
            const int blk = l >> 4;
            const float Gs = blk == 0 ? s0 : (blk == 1 ? s1 : (blk == 2 ? s2 : s3));
            const float Ge = blk == 0 ? e0 : (blk == 1 ? e1 : (blk == 2 ? e2 : e3));
            const int bi = (l >> 2) & 3, bj = l & 3;
            const float gsI = bi == 0 ? s0 : (bi == 1 ? s1 : (bi == 2 ? s2 : s3));
            const float geJ = bj == 0 ? e0 : (bj == 1 ? e1 : (bj == 2 ? e2 : e3));
            const float eg = __expf(G);
            t.G[l] = G;
            t.EGS[l] = eg * p.scale;
            t.B[l] = pre_b;
            t.BEG[l] = pre_b * eg;
            t.ROWF[l] = __expf(G - Gs);
            t.COLF[l] = __expf(Ge - G);
            if (l < 16) t.BLKF[l] = bj < bi ? __expf(gsI - geJ) : 0.f;
            if (p.g_out != nullptr && slab == 0 && l < len)
                p.g_out[b * p.go_sb + hv * p.go_sh + (int64_t)(start + l) * p.go_st] = G;
        }
    };
    auto store_o = [&](int c) {  // staged o tile of chunk c -> HBM, 16 bytes per lane
        const int len = min(kChunk, eos - (bos + c * kChunk));
        char *ob = obase + (int64_t)c * kChunk * p.o.st * 2;
#pragma unroll
        for (int m = 0; m < VCH; ++m)
            if (rv + m * VROWS < len)
                *reinterpret_cast<u32x4 *>(ob + ooff[m]) = *reinterpret_cast<const u32x4 *>(oS + (rv + m * VROWS) * po + cv);
    };

    if (nchunks > 0) {
        prefetch(0);
        commit(0, tiles_at<K, CT>(smem, 0));
    }
    __syncthreads();

    for (int c = 0; c < nchunks; ++c) {
        const int len = min(kChunk, eos - (bos + c * kChunk));
        const Tiles t = tiles_at<K, CT>(smem, DB ? (c & 1) : 0);
        if (DB && c > 0) store_o(c - 1);
        if (c + 1 < nchunks) prefetch(c + 1);
        // =========================== A: scores ===========================================
        switch (wv) {
            case 0: phase_a<K, 0>(t, aS, pS, dS, p.scale); break;
            case 1: phase_a<K, 1>(t, aS, pS, dS, p.scale); break;
            case 2: phase_a<K, 2>(t, aS, pS, dS, p.scale); break;
            default: phase_a<K, 3>(t, aS, pS, dS, p.scale); break;
        }
        __syncthreads();  // #1: aS, dS, pS complete
        // =========================== B: WY solve =========================================
        // tiles 0..CT-1: this wave's u columns; tiles CT..NT-1: its w columns
        f32x4 r[NT][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f32x4 b4 = lds4(t.B + 16 * i + 4 * lg), be4 = lds4(t.BEG + 16 * i + 4 * lg);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const elemx4 vv = frag_tr4(t.v, pv, (vtile0 + ct) * 16, 16 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) r[ct][i][e] = (float)vv[e] * b4[e];
            }
#pragma unroll
            for (int m = 0; m < NTW; ++m) {
                const elemx4 kv = KTile<K>::tr4(t.k, (wv * NTW + m) * 16, 16 * i);
#pragma unroll
                for (int e = 0; e < 4; ++e) r[CT + m][i][e] = (float)kv[e] * be4[e];
            }
        }
        {
            const elemx4 d0 = frag_kc4(dS, pd, 0, 0), d1 = frag_kc4(dS, pd, 16, 0), d2 = frag_kc4(dS, pd, 32, 0),
                         d3 = frag_kc4(dS, pd, 48, 0);
            const elemx4 a10 = frag_kc4(aS, pa, 16, 0), a32 = frag_kc4(aS, pa, 48, 32);
            const elemx8 a2x = frag_kc(aS, pa, 32, 0), a3x = frag_kc(aS, pa, 48, 0);
            FLA_SCHED_FENCE();
            elemx8 x01[NT];
#pragma unroll
            for (int q = 0; q < NT; ++q) r[q][0] = diag_mul(d0, r[q][0], q < CT);
#pragma unroll
            for (int q = 0; q < NT; ++q) r[q][1] = mfma16x16(a10, cvt4(r[q][0]), r[q][1]);
#pragma unroll
            for (int q = 0; q < NT; ++q) r[q][1] = diag_mul(d1, r[q][1], q < CT);
#pragma unroll
            for (int q = 0; q < NT; ++q) {
                x01[q] = frag_from_acc(r[q][0], r[q][1]);
                r[q][2] = mfma16x32(a2x, x01[q], r[q][2]);
                r[q][3] = mfma16x32(a3x, x01[q], r[q][3]);
            }
#pragma unroll
            for (int q = 0; q < NT; ++q) r[q][2] = diag_mul(d2, r[q][2], q < CT);
#pragma unroll
            for (int q = 0; q < NT; ++q) r[q][3] = mfma16x16(a32, cvt4(r[q][2]), r[q][3]);
#pragma unroll
            for (int q = 0; q < NT; ++q) r[q][3] = diag_mul(d3, r[q][3], q < CT);
        }
#pragma unroll
        for (int m = 0; m < NTW; ++m)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_to_tile(wS, pw, 16 * i, (wv * NTW + m) * 16, -r[CT + m][i]);
        if (DB && c + 1 < nchunks) commit(c + 1, tiles_at<K, CT>(smem, (c + 1) & 1));
        __syncthreads();  // #2: wS complete (and, double-buffered, the next chunk's tiles)
        // =========================== C: scan + output ====================================
        elemx8 hB[KS][CT];
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) hB[j][ct] = frag_from_acc(hacc[2 * j][ct], hacc[2 * j + 1][ct]);

        // wS holds -w:  U = u + (-w) h = v_new ;  oacc = q h
        f32x4 U[4][CT], oacc[4][CT];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                U[rt][ct] = r[ct][rt];
                oacc[rt][ct] = zero4();
            }
        {
            elemx8 wf[2][4], qf[2][4];
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                wf[0][rt] = frag_kc(wS, pw, rt * 16, 0);
                qf[0][rt] = frag_kc(t.q, pq, rt * 16, 0);
            }
#pragma unroll
            for (int j = 0; j < KS; ++j) {
                const int cb = j & 1, nb = cb ^ 1;
                if (j + 1 < KS) {
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt) {
                        wf[nb][rt] = frag_kc(wS, pw, rt * 16, 32 * (j + 1));
                        qf[nb][rt] = frag_kc(t.q, pq, rt * 16, 32 * (j + 1));
                    }
                }
                FLA_SCHED_FENCE();
#pragma unroll
                for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        U[rt][ct] = mfma16x32(wf[cb][rt], hB[j][ct], U[rt][ct]);
                        oacc[rt][ct] = mfma16x32(qf[cb][rt], hB[j][ct], oacc[rt][ct]);
                    }
                FLA_SCHED_FENCE();
            }
        }
        // operands of the next two products, issued before the element-wise work below
        elemx8 pf[2][4], kfa[KT];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) pf[j][rt] = frag_kc(pS, pp, rt * 16, 32 * j);
        f32x4 eg4[4], dk4[4];
        const float g_last = t.G[len - 1];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            eg4[rt] = lds4(t.EGS + 16 * rt + 4 * lg);
            dk4[rt] = lds4(t.G + 16 * rt + 4 * lg);
        }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) kfa[kt] = KTile<K>::tr(t.k, kt * 16, 0);
        FLA_SCHED_FENCE();
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
            for (int e = 0; e < 4; ++e) dk4[rt][e] = __expf(g_last - dk4[rt][e]);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) oacc[rt][ct] *= eg4[rt];  // scale e^{G_t} (q h)
        }
        // o = scale (e^{G_t} q h + P v_new)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            elemx8 vb[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) vb[ct] = frag_from_acc(U[2 * j][ct], U[2 * j + 1][ct]);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) oacc[rt][ct] = mfma16x32(pf[j][rt], vb[ct], oacc[rt][ct]);
        }
        // h <- e^{g_last} h + k^T (v_new e^{g_last - g}), the right operand as hi + lo bf16
        const float dec_all = __expf(g_last);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) hacc[kt][ct] *= dec_all;
        elemx8 vhi[2][CT], vlo[2][CT];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const f32x4 a0 = U[2 * j][ct] * dk4[2 * j], a1 = U[2 * j + 1][ct] * dk4[2 * j + 1];
                elemx4 h0, h1, l0, l1;
                split_hilo(a0, h0, l0);
                split_hilo(a1, h1, l1);
                vhi[j][ct] = cat8(h0, h1);
                vlo[j][ct] = cat8(l0, l1);
            }
        {
            elemx8 kfb[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) kfb[kt] = KTile<K>::tr(t.k, kt * 16, 32);
            FLA_SCHED_FENCE();
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    hacc[kt][ct] = mfma16x32(kfa[kt], vhi[0][ct], hacc[kt][ct]);
                    hacc[kt][ct] = mfma16x32(kfa[kt], vlo[0][ct], hacc[kt][ct]);
                }
            FLA_SCHED_FENCE();
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    hacc[kt][ct] = mfma16x32(kfb[kt], vhi[1][ct], hacc[kt][ct]);
                    hacc[kt][ct] = mfma16x32(kfb[kt], vlo[1][ct], hacc[kt][ct]);
                }
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) acc_to_tile(oS, po, rt * 16, (vtile0 + ct) * 16, oacc[rt][ct]);
        __syncthreads();  // #3: every read of this chunk's tiles is done, oS complete
        if (!DB) {
            store_o(c);
            if (c + 1 < nchunks) commit(c + 1, tiles_at<K, CT>(smem, 0));
            __syncthreads();  // #4
        }
    }
    if (DB && nchunks > 0) store_o(nchunks - 1);

    if (p.hT && state_row(p, n) >= 0) {
        float *s = p.hT + state_row(p, n) * p.s_sn + hv * p.s_sh;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s[(int64_t)(16 * kt + 4 * lg + e) * p.s_sk + (int64_t)(vcol0 + 16 * ct + li) * p.s_sv] = hacc[kt][ct][e];
    }
}

// =============================================================================================
// Pipelined form for 64-column slabs: 512 threads, two groups of four waves that share the CU.
//   prep group  (waves 0-3)  chunk i  : scores (phase A), WY solve (phase B), tile prefetch
//   state group (waves 4-7)  chunk i-1: v_new, state update, output (phase C), gate tables
// Each SIMD holds one wave of each group, so the chunk-parallel work of the next chunk runs under
// the serial state update of the current one.  Two workgroup barriers per iteration i:
//   before `mid`  prep : o(i-2) LDS -> HBM, v(i) -> LDS, loads of chunk i+1 issued, A(i) -> aS, dS, pS[i&1]
//                 state: v_new = u - w h, state update, q h_old   (reads wS, uS, q, k and tables of i-1)
//   after  `mid`  prep : B(i) -> wS, uS; q, k of i+1 -> LDS
//                 state: o = scale e^G (q h_old) + P v_new -> oS  (reads pS[(i-1)&1]); tables of chunk i+1
// Every buffer written in one half was last read in the other half or earlier, which is what makes two
// barriers enough: q, k, the tables and P have two buffers, v, -w, u and o one.  The output leaves through an
// LDS tile because a state wave owns 16 columns: stored from its registers, o went out as 32-byte pieces of
// eight rows per instruction, which cost 14 % of the launch; the prep group writes whole 128-byte rows.
// =============================================================================================
template <int K> struct PipeSmem {
    static constexpr int pq = K + 8, pk = KTile<K>::pitch, pv = 64 + 8, pa = kChunk + 8, pw = K + 8, pp = kChunk + 8,
                         pd = 24;
    static constexpr size_t q_bytes = (size_t)kChunk * pq * 2, k_bytes = (size_t)kChunk * pk * 2,
                            v_bytes = (size_t)kChunk * pv * 2, tab_bytes = (7 * kChunk + 16) * 4;
    static constexpr size_t q_off = 0;                                         // two q tiles
    static constexpr size_t k_off = q_off + 2 * q_bytes;                       // two k tiles
    static constexpr size_t v_off = k_off + 2 * k_bytes;                       // one v tile
    static constexpr size_t t_off = v_off + v_bytes;                           // two sets of gate tables
    static constexpr size_t a_off = t_off + 2 * tab_bytes;
    static constexpr size_t w_off = a_off + (size_t)kChunk * pa * 2;
    static constexpr size_t p_off = w_off + (size_t)kChunk * pw * 2;           // two P tiles
    static constexpr size_t d_off = p_off + 2 * (size_t)kChunk * pp * 2;
    static constexpr size_t u_off = d_off + (size_t)kChunk * pd * 2;           // u as register images, fp32
    static constexpr int po = 64 + 8;                                          // pitch of the output staging tile
    static constexpr size_t o_off = u_off + (size_t)kChunk * 64 * 4;           // o of one chunk, [kChunk][po]
    static constexpr size_t bytes = o_off + (size_t)kChunk * po * 2;
};
// Tiles of chunk c: q, k and the tables cycle through two buffers, v has one.
template <int K>
__device__ __forceinline__ Tiles pipe_tiles_at(unsigned char *smem, int c) {
    typedef PipeSmem<K> L;
    const int c2 = c & 1;
    Tiles t;
    t.q = reinterpret_cast<elem *>(smem + L::q_off + c2 * L::q_bytes);
    t.k = reinterpret_cast<elem *>(smem + L::k_off + c2 * L::k_bytes);
    t.v = reinterpret_cast<elem *>(smem + L::v_off);
    t.G = reinterpret_cast<float *>(smem + L::t_off + c2 * L::tab_bytes);
    t.EGS = t.G + kChunk;
    t.B = t.EGS + kChunk;
    t.BEG = t.B + kChunk;
    t.ROWF = t.BEG + kChunk;
    t.COLF = t.ROWF + kChunk;
    t.BLKF = t.COLF + kChunk;
    return t;
}
// e^{G_last - G_t} per token (decay of v_new towards the chunk end), after the 16 block factors
__device__ __forceinline__ float *pipe_decay_table(const Tiles &t) { return t.BLKF + 16; }

// TRAIN: the state group also writes h, v_new and w (the operands the backward operators would otherwise recompute).
template <int K, bool TRAIN>
__global__ void __launch_bounds__(512) gdn_pipe_kernel(const FusedParams p) {
    typedef PipeSmem<K> L;
    constexpr int VS = 64, pq = L::pq, pv = L::pv, pa = L::pa, pw = L::pw, pp = L::pp, pd = L::pd;
    constexpr int KT = K / 16, KS = K / 32;
    constexpr int GT = 256;                              // threads of one group
    constexpr int QCH = kChunk * (K / 8) / GT, VCH = kChunk * (VS / 8) / GT;
    constexpr int QROWS = GT / (K / 8), VROWS = GT / (VS / 8);
    constexpr int NTW = K / 64, NT = NTW + 1;
    extern __shared__ __align__(16) unsigned char smem[];
    elem *aS = reinterpret_cast<elem *>(smem + L::a_off);
    elem *wS = reinterpret_cast<elem *>(smem + L::w_off);
    elem *pS0 = reinterpret_cast<elem *>(smem + L::p_off);
    elem *dS = reinterpret_cast<elem *>(smem + L::d_off);
    float *uS = reinterpret_cast<float *>(smem + L::u_off);
    elem *oS = reinterpret_cast<elem *>(smem + L::o_off);
    constexpr int po = L::po;

    const int lin = blockIdx.x;
    int slab, hv, n;
    if (p.remap) {
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
    const int wave = wave_id();
    const int l = lane_id(), li = l & 15, lg = l >> 4;

    if (wave < 4) {
        // ================================ prep group ==============================================
        const int wv = wave, tid = threadIdx.x;
        const int rq = tid / (K / 8), cq = (tid % (K / 8)) * 8;
        const int rv = tid / (VS / 8), cv = (tid % (VS / 8)) * 8;
        const char *qbase = reinterpret_cast<const char *>(static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh + (int64_t)bos * p.q.st);
        const char *kbase = reinterpret_cast<const char *>(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)bos * p.k.st);
        const char *vbase = reinterpret_cast<const char *>(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)bos * p.v.st + slab * VS);
        unsigned qoff[QCH], koff[QCH], voff[VCH];
#pragma unroll
        for (int m = 0; m < QCH; ++m) {
            qoff[m] = (unsigned)(((rq + m * QROWS) * p.q.st + cq) * 2);
            koff[m] = (unsigned)(((rq + m * QROWS) * p.k.st + cq) * 2);
        }
#pragma unroll
        for (int m = 0; m < VCH; ++m) voff[m] = (unsigned)(((rv + m * VROWS) * p.v.st + cv) * 2);
        u32x4 pre_q[QCH], pre_k[QCH], pre_v[VCH];
        // Rows past the end of the sequence must read as zero.  Buffer loads do that without a branch or
        // an exec mask: the resource of a chunk covers exactly its valid rows, anything beyond returns 0.
        auto prefetch = [&](int c) {
            const int len = min(kChunk, eos - (bos + c * kChunk));
            const __amdgpu_buffer_rsrc_t rq_ = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<char *>(qbase + (int64_t)c * kChunk * p.q.st * 2), 0, (int)((len - 1) * p.q.st * 2 + K * 2), 0x00020000);
            const __amdgpu_buffer_rsrc_t rk_ = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<char *>(kbase + (int64_t)c * kChunk * p.k.st * 2), 0, (int)((len - 1) * p.k.st * 2 + K * 2), 0x00020000);
            const __amdgpu_buffer_rsrc_t rv_ = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<char *>(vbase + (int64_t)c * kChunk * p.v.st * 2), 0, (int)((len - 1) * p.v.st * 2 + VS * 2), 0x00020000);
#pragma unroll
            for (int m = 0; m < QCH; ++m) {
                pre_q[m] = __builtin_amdgcn_raw_buffer_load_b128(rq_, (int)qoff[m], 0, 0);
                pre_k[m] = __builtin_amdgcn_raw_buffer_load_b128(rk_, (int)koff[m], 0, 0);
            }
#pragma unroll
            for (int m = 0; m < VCH; ++m) pre_v[m] = __builtin_amdgcn_raw_buffer_load_b128(rv_, (int)voff[m], 0, 0);
        };
        // A row is held by K/8 adjacent lanes, so its sum of squares is one DPP reduction; the normalised row is
        // rounded to bf16 exactly where the separate normalisation kernel would have rounded it.
        auto unit_row = [&](u32x4 raw, float &rstd) -> u32x4 {
            const elemx8 a = __builtin_bit_cast(elemx8, raw);
            f32x4 lo, hi;
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[e] = (float)a[e];
                hi[e] = (float)a[4 + e];
                ss += lo[e] * lo[e] + hi[e] * hi[e];
            }
            rstd = __builtin_amdgcn_rsqf(group_sum<K / 8>(ss) + 1e-6f);
            return __builtin_bit_cast(u32x4, frag_from_acc(lo * rstd, hi * rstd));
        };
        // For a backward pass the normalised rows and their rstd also go to memory, once per key head: from the first slab
        // of the first value head that shares it.  A row is a run of 16-byte pieces in neighbouring lanes.
        const bool emit_qk = TRAIN && p.qn_out.p != nullptr && slab == 0 && hv % (p.geom.Hv / p.geom.Hk) == 0;
        auto commit_qk = [&](const Tiles &t, int c) {
            const int len = min(kChunk, eos - (bos + c * kChunk));
#pragma unroll
            for (int m = 0; m < QCH; ++m) {
                const int row = rq + m * QROWS;
                u32x4 qv = pre_q[m], kv = pre_k[m];
                if (p.l2norm) {
                    float qr, kr;
                    qv = unit_row(qv, qr);
                    kv = unit_row(kv, kr);
                    if constexpr (TRAIN) {
                        if (emit_qk && row < len) {
                            const int64_t tok = bos + c * kChunk + row;
                            *reinterpret_cast<u32x4 *>(static_cast<elem *>(const_cast<void *>(p.qn_out.p)) + b * p.qn_out.sb + hk * p.qn_out.sh + tok * p.qn_out.st + cq) = qv;
                            *reinterpret_cast<u32x4 *>(static_cast<elem *>(const_cast<void *>(p.kn_out.p)) + b * p.kn_out.sb + hk * p.kn_out.sh + tok * p.kn_out.st + cq) = kv;
                            if (cq == 0) {
                                p.q_rstd[b * p.rs_sb + hk * p.rs_sh + tok] = qr;
                                p.k_rstd[b * p.rs_sb + hk * p.rs_sh + tok] = kr;
                            }
                        }
                    }
                }
                *reinterpret_cast<u32x4 *>(t.q + row * pq + cq) = qv;
                *reinterpret_cast<u32x4 *>(t.k + KTile<K>::off(row, cq)) = kv;
            }
        };
        elem *vS = reinterpret_cast<elem *>(smem + L::v_off);
        // The state group leaves o of a chunk in oS during the second half of an iteration; this group writes
        // it out in the first half of the next one, 16 bytes per lane, eight lanes per 128-byte row.
        char *og = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.o.p)) + b * p.o.sb + hv * p.o.sh +
                                            (int64_t)bos * p.o.st + slab * VS);
        auto store_o = [&](int c) {
            const int len = min(kChunk, eos - (bos + c * kChunk));
            char *dst = og + (int64_t)c * kChunk * p.o.st * 2;
#pragma unroll
            for (int m = 0; m < VCH; ++m) {
                const int row = rv + m * VROWS;
                if (row < len)
                    *reinterpret_cast<u32x4 *>(dst + ((int64_t)row * p.o.st + cv) * 2) = *reinterpret_cast<const u32x4 *>(oS + row * po + cv);
            }
        };
        if (nchunks > 0) {
            prefetch(0);
            commit_qk(pipe_tiles_at<K>(smem, 0), 0);
        }
        __syncthreads();   // start
        for (int i = 0; i <= nchunks; ++i) {
            const Tiles t = pipe_tiles_at<K>(smem, i);
            elem *pS = pS0 + (i & 1) * kChunk * pp;
            if (i >= 2) store_o(i - 2);
            if (i < nchunks) {
                // v of this chunk has waited in registers: its single LDS tile was read until the last barrier
#pragma unroll
                for (int m = 0; m < VCH; ++m) *reinterpret_cast<u32x4 *>(vS + (rv + m * VROWS) * pv + cv) = pre_v[m];
                if (i + 1 < nchunks) prefetch(i + 1);
                switch (wv) {
                    case 0: phase_a<K, 0>(t, aS, pS, dS, p.scale); break;
                    case 1: phase_a<K, 1>(t, aS, pS, dS, p.scale); break;
                    case 2: phase_a<K, 2>(t, aS, pS, dS, p.scale); break;
                    default: phase_a<K, 3>(t, aS, pS, dS, p.scale); break;
                }
            }
            __syncthreads();   // mid
            if (i < nchunks) {
                // tile 0: this wave's u columns; tiles 1..NTW: its w columns (the table holds -beta e^G, so
                // the solve yields -w, which is what the state group accumulates)
                f32x4 r[NT][4];
#pragma unroll
                for (int bi = 0; bi < 4; ++bi) {
                    const f32x4 b4 = lds4(t.B + 16 * bi + 4 * lg), be4 = lds4(t.BEG + 16 * bi + 4 * lg);
                    const elemx4 vv = frag_tr4(t.v, pv, wv * 16, 16 * bi);
#pragma unroll
                    for (int e = 0; e < 4; ++e) r[0][bi][e] = (float)vv[e] * b4[e];
#pragma unroll
                    for (int m = 0; m < NTW; ++m) {
                        const elemx4 kv = KTile<K>::tr4(t.k, (wv * NTW + m) * 16, 16 * bi);
#pragma unroll
                        for (int e = 0; e < 4; ++e) r[1 + m][bi][e] = (float)kv[e] * be4[e];
                    }
                }
                {
                    const elemx4 d0 = frag_kc4(dS, pd, 0, 0), d1 = frag_kc4(dS, pd, 16, 0), d2 = frag_kc4(dS, pd, 32, 0),
                                 d3 = frag_kc4(dS, pd, 48, 0);
                    const elemx4 a10 = frag_kc4(aS, pa, 16, 0), a32 = frag_kc4(aS, pa, 48, 32);
                    const elemx8 a2x = frag_kc(aS, pa, 32, 0), a3x = frag_kc(aS, pa, 48, 0);
                    elemx8 x01[NT];
#pragma unroll
                    for (int q = 0; q < NT; ++q) r[q][0] = diag_mul(d0, r[q][0], q == 0);
#pragma unroll
                    for (int q = 0; q < NT; ++q) r[q][1] = mfma16x16(a10, cvt4(r[q][0]), r[q][1]);
#pragma unroll
                    for (int q = 0; q < NT; ++q) r[q][1] = diag_mul(d1, r[q][1], q == 0);
#pragma unroll
                    for (int q = 0; q < NT; ++q) {
                        x01[q] = frag_from_acc(r[q][0], r[q][1]);
                        r[q][2] = mfma16x32(a2x, x01[q], r[q][2]);
                        r[q][3] = mfma16x32(a3x, x01[q], r[q][3]);
                    }
#pragma unroll
                    for (int q = 0; q < NT; ++q) r[q][2] = diag_mul(d2, r[q][2], q == 0);
#pragma unroll
                    for (int q = 0; q < NT; ++q) r[q][3] = mfma16x16(a32, cvt4(r[q][2]), r[q][3]);
#pragma unroll
                    for (int q = 0; q < NT; ++q) r[q][3] = diag_mul(d3, r[q][3], q == 0);
                }
#pragma unroll
                for (int m = 0; m < NTW; ++m)
#pragma unroll
                    for (int bi = 0; bi < 4; ++bi) acc_to_tile(wS, pw, 16 * bi, (wv * NTW + m) * 16, r[1 + m][bi]);
#pragma unroll
                for (int bi = 0; bi < 4; ++bi) *reinterpret_cast<f32x4 *>(uS + ((wv * 4 + bi) * 64 + l) * 4) = r[0][bi];
                if (i + 1 < nchunks) commit_qk(pipe_tiles_at<K>(smem, i + 1), i + 1);
            }
            __syncthreads();   // end
        }
        if (nchunks > 0) store_o(nchunks - 1);
        return;
    }

    // ================================== state group ===============================================
    const int wv = wave - 4;
    const int vcol0 = slab * VS + wv * 16;
    f32x4 hacc[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        f32x4 a = zero4();
        if (p.h0 && state_row(p, n) >= 0) {
            const float *s = p.h0 + state_row(p, n) * p.s_sn + hv * p.s_sh;
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = s[(int64_t)(16 * kt + 4 * lg + e) * p.s_sk + (int64_t)(vcol0 + li) * p.s_sv];
        }
        hacc[kt] = a;
    }
    // The initial-state loads must be complete before the loop: left pending, the compiler's wait-count
    // bookkeeping carries them around the loop and turns every first use of the state into a wait for
    // ALL outstanding memory operations, including the gate loads issued for the next chunk.
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    const float *gptr = static_cast<const float *>(p.g.p) + b * p.g.sb + hv * p.g.sh;
    const float *bptr = static_cast<const float *>(p.beta.p) + b * p.beta.sb + hv * p.beta.sh;
    float pre_g = 0.f, pre_b = 0.f;
    auto gate_fetch = [&](int c) {   // every wave of the group: lane = token
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
        const int tok = start + min(l, len - 1);   // clamped: no predicated load, padding is applied in gate_tables
        pre_g = gptr[(int64_t)tok * p.g.st];
        pre_b = bptr[(int64_t)tok * p.beta.st];
    };
    // Each wave scans the gates of the chunk itself and writes its share of the tables.
    auto gate_tables = [&](int c, const Tiles &t) {
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
        float G = wave_inclusive_scan(l < len ? pre_g : 0.f);
        const float g_end = read_lane(G, len - 1);
        if (l >= len) {
            G = g_end;
            pre_b = 0.f;
        }
        if (wv == 0) {
            t.G[l] = G;
            t.EGS[l] = __expf(G) * p.scale;
            pipe_decay_table(t)[l] = l < len ? __expf(g_end - G) : 0.f;
            if (p.g_out != nullptr && slab == 0 && l < len)
                p.g_out[b * p.go_sb + hv * p.go_sh + (int64_t)(start + l) * p.go_st] = G;
        } else if (wv == 1) {
            t.B[l] = pre_b;
            t.BEG[l] = -pre_b * __expf(G);
        } else if (wv == 2) {
            // gate at the first / last token of each 16-token block
            const float s0 = read_lane(G, 0), s1 = read_lane(G, 16), s2 = read_lane(G, 32), s3 = read_lane(G, 48);
            const float e0 = read_lane(G, 15), e1 = read_lane(G, 31), e2 = read_lane(G, 47), e3 = read_lane(G, 63);
            const int blk = l >> 4;
            const float Gs = blk == 0 ? s0 : (blk == 1 ? s1 : (blk == 2 ? s2 : s3));
            const float Ge = blk == 0 ? e0 : (blk == 1 ? e1 : (blk == 2 ? e2 : e3));
            t.ROWF[l] = __expf(G - Gs);
            t.COLF[l] = __expf(Ge - G);
        } else {
            const float s1 = read_lane(G, 16), s2 = read_lane(G, 32), s3 = read_lane(G, 48);
            const float e0 = read_lane(G, 15), e1 = read_lane(G, 31), e2 = read_lane(G, 47);
            const int bi = (l >> 2) & 3, bj = l & 3;
            const float gsI = bi == 1 ? s1 : (bi == 2 ? s2 : s3);
            const float geJ = bj == 0 ? e0 : (bj == 1 ? e1 : e2);
            if (l < 16) t.BLKF[l] = bj < bi ? __expf(gsI - geJ) : 0.f;
        }
    };
    if (nchunks > 0) {
        gate_fetch(0);
        gate_tables(0, pipe_tiles_at<K>(smem, 0));
        if (nchunks > 1) gate_fetch(1);
    }
    __syncthreads();   // start

    for (int i = 0; i <= nchunks; ++i) {
        const int c = i - 1;                               // chunk of this group
        const Tiles t = pipe_tiles_at<K>(smem, c);
        const elem *pS = pS0 + (c & 1) * kChunk * pp;
        const int len = c >= 0 ? min(kChunk, eos - (bos + c * kChunk)) : 0;
        f32x4 U[4], eg4[4];
        elemx8 hB[KS];
        if (c >= 0) {
            // state at chunk start as bf16 operand; it also serves q h after the update below
#pragma unroll
            for (int j = 0; j < KS; ++j) hB[j] = frag_from_acc(hacc[2 * j], hacc[2 * j + 1]);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) U[rt] = *reinterpret_cast<const f32x4 *>(uS + ((wv * 4 + rt) * 64 + l) * 4);
            {   // v_new = u + (-w) h
                // every operand read is in flight before the first product: their latency is paid once
                elemx8 wf[KS][4];
#pragma unroll
                for (int j = 0; j < KS; ++j)
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt) wf[j][rt] = frag_kc(wS, pw, rt * 16, 32 * j);
                FLA_SCHED_FENCE();
#pragma unroll
                for (int j = 0; j < KS; ++j)
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt) U[rt] = mfma16x32(wf[j][rt], hB[j], U[rt]);
                FLA_SCHED_FENCE();
            }
            if constexpr (TRAIN) {
                if (p.w_out.p != nullptr && slab == 0) {   // the tile holds -w: whole rows out, sign bits flipped
                    const int gt = threadIdx.x - GT, rw = gt / (K / 8), cw = (gt % (K / 8)) * 8;
                    char *wg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.w_out.p)) + b * p.w_out.sb +
                                                        hv * p.w_out.sh + (int64_t)(bos + c * kChunk) * p.w_out.st);
#pragma unroll
                    for (int m = 0; m < QCH; ++m) {
                        const int row = rw + m * QROWS;
                        u32x4 x = *reinterpret_cast<const u32x4 *>(wS + row * pw + cw);
#pragma unroll
                        for (int e = 0; e < 4; ++e) x[e] ^= 0x80008000u;
                        if (row < len) *reinterpret_cast<u32x4 *>(wg + ((int64_t)row * p.w_out.st + cw) * 2) = x;
                    }
                }
            }
            elemx8 kfa[KT], kfb[KT];
            f32x4 dk4[4];
            const float g_last = t.G[len - 1];
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                eg4[rt] = lds4(t.EGS + 16 * rt + 4 * lg);
                dk4[rt] = lds4(pipe_decay_table(t) + 16 * rt + 4 * lg);
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                kfa[kt] = KTile<K>::tr(t.k, kt * 16, 0);
            }
            FLA_SCHED_FENCE();
            // h <- e^{g_last} h + k^T (v_new e^{g_last - g}), the right operand as hi + lo bf16
            const float dec_all = __expf(g_last);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) hacc[kt] *= dec_all;
            elemx8 vhi[2], vlo[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const f32x4 a0 = U[2 * j] * dk4[2 * j], a1 = U[2 * j + 1] * dk4[2 * j + 1];
                elemx4 h0, h1, l0, l1;
                split_hilo(a0, h0, l0);
                split_hilo(a1, h1, l1);
                vhi[j] = cat8(h0, h1);
                vlo[j] = cat8(l0, l1);
            }
            {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) kfb[kt] = KTile<K>::tr(t.k, kt * 16, 32);
                FLA_SCHED_FENCE();
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    hacc[kt] = mfma16x32(kfa[kt], vhi[0], hacc[kt]);
                    hacc[kt] = mfma16x32(kfa[kt], vlo[0], hacc[kt]);
                }
                FLA_SCHED_FENCE();
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    hacc[kt] = mfma16x32(kfb[kt], vhi[1], hacc[kt]);
                    hacc[kt] = mfma16x32(kfb[kt], vlo[1], hacc[kt]);
                }
            }
        }
        // q h with the state at chunk start, here rather than after the barrier: q of this chunk is then read in
        // this half only, which is what lets q live in two buffers.  The P operands of the second half are
        // fetched before the barrier too, so their latency hides behind the wait.
        f32x4 oacc[4];
        elemx8 pf[6];
        if (c >= 0) {
            elemx8 qf[KS][4];
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) qf[j][rt] = frag_kc(t.q, pq, rt * 16, 32 * j);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) oacc[rt] = zero4();
            FLA_SCHED_FENCE();
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) oacc[rt] = mfma16x32(qf[j][rt], hB[j], oacc[rt]);
            FLA_SCHED_FENCE();
            pf[0] = frag_kc(pS, pp, 0, 0);
            pf[1] = frag_kc(pS, pp, 16, 0);
            pf[2] = frag_kc(pS, pp, 32, 0);
            pf[3] = frag_kc(pS, pp, 32, 32);
            pf[4] = frag_kc(pS, pp, 48, 0);
            pf[5] = frag_kc(pS, pp, 48, 32);
        }
        __syncthreads();   // mid
        if (c >= 0) {
            // o = scale (e^{G_t} q h + P v_new), h the state at chunk start
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) oacc[rt] *= eg4[rt];
            {
                const elemx8 vb0 = frag_from_acc(U[0], U[1]), vb1 = frag_from_acc(U[2], U[3]);
                oacc[0] = mfma16x32(pf[0], vb0, oacc[0]);
                oacc[1] = mfma16x32(pf[1], vb0, oacc[1]);
                oacc[2] = mfma16x32(pf[2], vb0, oacc[2]);
                oacc[3] = mfma16x32(pf[4], vb0, oacc[3]);
                oacc[2] = mfma16x32(pf[3], vb1, oacc[2]);
                oacc[3] = mfma16x32(pf[5], vb1, oacc[3]);
            }
            // tables of the next chunk, then the gate loads of the one after it
            if (i + 1 < nchunks) gate_tables(i + 1, pipe_tiles_at<K>(smem, i + 1));
            if (i + 2 < nchunks) gate_fetch(i + 2);
            // this wave's 16 columns of o into the staging tile; the prep group writes whole rows to memory
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc_to_tile(oS, po, 16 * rt, 16 * wv, oacc[rt]);
            if constexpr (TRAIN) {
                // this half leaves the state group waiting for the prep group: the stores ride in that slack
                if (p.h_out != nullptr) {   // the state the chunk started from, rounded as the products above used it
                    const int chunk = (p.geom.choff != nullptr ? p.geom.choff[n] : 0) + c;
                    char *hg = reinterpret_cast<char *>(p.h_out + b * p.h_sb + hv * p.h_sh + (int64_t)chunk * p.h_sc + vcol0);
#pragma unroll
                    for (int j = 0; j < KS; ++j) {
                        const u32x4 d = __builtin_bit_cast(u32x4, hB[j]);
                        packed_to_global(hg, (int64_t)V * 2, 32 * j, K, d[0], d[1]);
                        packed_to_global(hg, (int64_t)V * 2, 32 * j + 16, K, d[2], d[3]);
                    }
                }
                if (p.vn_out.p != nullptr) {
                    char *vg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.vn_out.p)) + b * p.vn_out.sb +
                                                        hv * p.vn_out.sh + (int64_t)(bos + c * kChunk) * p.vn_out.st + vcol0);
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt) acc_to_global(vg, p.vn_out.st * 2, 16 * rt, len, U[rt]);
                }
            }
        } else {
            if (i + 1 < nchunks) gate_tables(i + 1, pipe_tiles_at<K>(smem, i + 1));
            if (i + 2 < nchunks) gate_fetch(i + 2);
        }
        __syncthreads();   // end
    }
    if (p.hT && state_row(p, n) >= 0) {
        float *s = p.hT + state_row(p, n) * p.s_sn + hv * p.s_sh;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) s[(int64_t)(16 * kt + 4 * lg + e) * p.s_sk + (int64_t)(vcol0 + li) * p.s_sv] = hacc[kt][e];
    }
}

template <int K, bool TRAIN>
int launch_pipe(FusedParams &p, hipStream_t stream) {
    typedef PipeSmem<K> L;
    const int64_t total = (int64_t)p.geom.N * p.geom.Hv * p.slabs;
    p.remap = (p.slabs == 2 && total % 16 == 0) ? 1 : 0;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(gdn_pipe_kernel<K, TRAIN>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)L::bytes));
    FLA_LAUNCH(TRAIN ? "gdn_fused_train" : "gdn_fused", stream, (gdn_pipe_kernel<K, TRAIN>), dim3((unsigned)total), dim3(512),
               L::bytes, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
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
               int64_t chunk_size, bool use_qk_l2norm, const fla_tensor *o, const fla_tensor *g_cumsum, const fla_tensor *final_state,
               const fla_tensor *h, const fla_tensor *v_new, const fla_tensor *w, const fla_tensor *qn, const fla_tensor *kn,
               const fla_tensor *q_rstd, const fla_tensor *k_rstd,
               void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query, const fla_tensor *state_indices = nullptr) {
    const char *op = state_indices ? "gdn_chunk_fwd_state_pool" : "gdn_chunk_fwd";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v, nullptr, chunk_size, geom, kElemDtype))) return rc;
    const int bf = dt_bit(kElemDtype);
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
    const int gmask = dt_bit(FLA_F32);  // the Python front end casts gates to fp32
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
        if (state_indices) {   // rows of a pool, K x V blocks in either order
            FLA_REQUIRE(s->shape[0] >= 1 && s->shape[0] <= INT32_MAX && s->shape[1] == geom.Hv && s->shape[2] == geom.K &&
                            s->shape[3] == geom.V && s->stride[0] >= 0 && s->stride[1] >= 0 &&
                            ((s->stride[3] == 1 && s->stride[2] == geom.V) || (s->stride[2] == 1 && s->stride[3] == geom.K)),
                        FLA_ERR_SHAPE, "%s: %s must be [rows,Hv,K,V] fp32 with contiguous K x V or V x K blocks.", op, name);
            return FLA_OK;
        }
        FLA_REQUIRE(s->shape[0] == geom.N && s->shape[1] == geom.Hv && s->shape[2] == geom.K && s->shape[3] == geom.V &&
                        s->stride[3] == 1 && s->stride[2] == geom.V,
                    FLA_ERR_SHAPE, "%s: %s must be [N=%d,Hv,K,V] fp32 with contiguous K x V blocks.", op, name, geom.N);
        return FLA_OK;
    };
    if (state_indices) {
        if ((rc = check_tensor(state_indices, op, "state_indices", 1, dt_bit(FLA_I32)))) return rc;
        FLA_REQUIRE(state_indices->shape[0] == geom.N && (geom.N <= 1 || state_indices->stride[0] == 1), FLA_ERR_SHAPE,
                    "%s: state_indices must be a contiguous int32 [N=%d].", op, geom.N);
        FLA_REQUIRE(initial_state && initial_state->data && output_final_state && final_state &&
                        final_state->data == initial_state->data,
                    FLA_ERR_NULL, "%s: the state pool is both the initial and the final state.", op);
    }
    const bool has_h0 = initial_state && initial_state->data;
    if (has_h0 && (rc = check_state(initial_state, "initial_state"))) return rc;
    if (output_final_state && (rc = check_state(final_state, "final_state"))) return rc;
    FLA_REQUIRE(geom.K == 128 || geom.K == 64, FLA_ERR_UNSUPPORTED, "%s: K must be 64 or 128, got %d.", op, geom.K);
    FLA_REQUIRE(geom.V % 64 == 0, FLA_ERR_UNSUPPORTED, "%s: V must be a multiple of 64, got %d.", op, geom.V);
    // operands of the backward pass, each optional
    const bool has_h = h && h->data, has_vn = v_new && v_new->data, has_w = w && w->data;
    if (has_h) {
        if ((rc = check_tensor(h, op, "h", 5, bf))) return rc;
        FLA_REQUIRE(h->shape[0] == geom.B && h->shape[1] == geom.Hv && h->shape[2] == geom.NT && h->shape[3] == geom.K &&
                        h->shape[4] == geom.V && h->stride[4] == 1 && h->stride[3] == geom.V && h->stride[2] % 2 == 0 &&
                        h->stride[1] % 2 == 0 && h->stride[0] % 2 == 0 && reinterpret_cast<uintptr_t>(h->data) % 4 == 0,
                    FLA_ERR_SHAPE, "%s: h must be [B,Hv,NT=%d,K,V] with contiguous K x V blocks.", op, geom.NT);
    }
    if (has_vn && (rc = check_bhtd(op, "v_new", v_new, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if (has_w && (rc = check_bhtd(op, "w", w, geom.B, geom.Hv, geom.T, geom.K, bf))) return rc;
    const bool has_qn = qn && qn->data;
    if (has_qn) {
        FLA_REQUIRE(use_qk_l2norm && kn && kn->data && q_rstd && q_rstd->data && k_rstd && k_rstd->data, FLA_ERR_NULL,
                    "%s: q_normalised, k_normalised, q_rstd and k_rstd come together, with use_qk_l2norm_in_kernel.", op);
        if ((rc = check_bhtd(op, "q_normalised", qn, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
        if ((rc = check_bhtd(op, "k_normalised", kn, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
        const fla_tensor *rs[] = {q_rstd, k_rstd};
        for (int i = 0; i < 2; ++i) {
            if ((rc = check_tensor(rs[i], op, i ? "k_rstd" : "q_rstd", 3, dt_bit(FLA_F32)))) return rc;
            FLA_REQUIRE(rs[i]->shape[0] == geom.B && rs[i]->shape[1] == geom.Hk && rs[i]->shape[2] == geom.T && is_contiguous(rs[i]),
                        FLA_ERR_SHAPE, "%s: rstd must be contiguous fp32 [B,Hk,T].", op);
        }
    }
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
    p.g = View3{g->data, g->stride[0], g->stride[2], g->stride[1], g->dtype == FLA_F32 ? 0 : 1};
    p.beta = View3{beta->data, beta->stride[0], beta->stride[2], beta->stride[1], beta->dtype == FLA_F32 ? 0 : 1};
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
        p.s_sk = sref->stride[2];
        p.s_sv = sref->stride[3];
        p.pool_rows = (int)sref->shape[0];
    }
    if (state_indices) p.slot = static_cast<const int32_t *>(state_indices->data);
    if (has_h0 && output_final_state)
        FLA_REQUIRE(initial_state->stride[0] == final_state->stride[0] && initial_state->stride[1] == final_state->stride[1] &&
                        initial_state->stride[2] == final_state->stride[2] && initial_state->stride[3] == final_state->stride[3],
                    FLA_ERR_SHAPE, "%s: initial_state and final_state must share strides.", op);
    p.scale = (float)scale;
    p.l2norm = use_qk_l2norm ? 1 : 0;

    // 128-column slabs (two 16-column tiles per wave) halve the per-FLOP LDS traffic and do the score / w work once
    // per head; 64-column slabs double the number of workgroups and run as the two-group pipelined kernel.  The wide
    // form is used once it alone fills the GPU; the in-kernel normalisation lives in the pipelined kernel's tile commit.
    const int64_t chains = (int64_t)geom.N * geom.Hv;
    const bool train = has_h || has_vn || has_w || has_qn;
    if (has_qn) {
        p.qn_out = view4(qn);
        p.kn_out = view4(kn);
        p.q_rstd = static_cast<float *>(q_rstd->data);
        p.k_rstd = static_cast<float *>(k_rstd->data);
        p.rs_sb = q_rstd->stride[0];
        p.rs_sh = q_rstd->stride[1];
    }
    if (has_h) {
        p.h_out = static_cast<elem *>(h->data);
        p.h_sb = h->stride[0];
        p.h_sh = h->stride[1];
        p.h_sc = h->stride[2];
    }
    if (has_vn) p.vn_out = view4(v_new);
    if (has_w) p.w_out = view4(w);
    const bool wide = !train && !use_qk_l2norm && geom.V % 128 == 0 && chains * (geom.V / 128) >= (int64_t)num_cus();
    p.slabs = wide ? geom.V / 128 : geom.V / 64;
    if (train) return geom.K == 128 ? launch_pipe<128, true>(p, stream) : launch_pipe<64, true>(p, stream);
    if (!wide) return geom.K == 128 ? launch_pipe<128, false>(p, stream) : launch_pipe<64, false>(p, stream);
    return geom.K == 128 ? launch_fused<128, 2>(p, stream) : launch_fused<64, 2>(p, stream);
}

}  // namespace
}  // namespace fla

FLA_ENTRY(fla_gdn_chunk_fwd_get_workspace_size)(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v,
                                                    const fla_tensor *g, const fla_tensor *beta, double scale,
                                                    const fla_tensor *initial_state, bool output_final_state,
                                                    const fla_int_array *cu_seqlens, int64_t chunk_size,
                                                    bool use_qk_l2norm_in_kernel, const fla_tensor *o,
                                                    const fla_tensor *g_cumsum, const fla_tensor *final_state,
                                                    const fla_tensor *h, const fla_tensor *v_new, const fla_tensor *w,
                                                    const fla_tensor *q_normalised, const fla_tensor *k_normalised,
                                                    const fla_tensor *q_rstd, const fla_tensor *k_rstd,
                                                    uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_gdn_chunk_fwd_get_workspace_size, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, chunk_size, use_qk_l2norm_in_kernel, o, g_cumsum, final_state, h, v_new, w, q_normalised, k_normalised, q_rstd, k_rstd, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "gdn_chunk_fwd: workspace_size must not be null.");
    return fla::guarded([&] { return fla::fused_impl(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, chunk_size,
                           use_qk_l2norm_in_kernel, o, g_cumsum, final_state, h, v_new, w, q_normalised, k_normalised, q_rstd,
                           k_rstd, nullptr, 0, nullptr, workspace_size); });
}

FLA_ENTRY(fla_gdn_chunk_fwd)(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
                                 const fla_tensor *beta, double scale, const fla_tensor *initial_state,
                                 bool output_final_state, const fla_int_array *cu_seqlens, int64_t chunk_size,
                                 bool use_qk_l2norm_in_kernel, const fla_tensor *o, const fla_tensor *g_cumsum,
                                 const fla_tensor *final_state, const fla_tensor *h, const fla_tensor *v_new,
                                 const fla_tensor *w, const fla_tensor *q_normalised, const fla_tensor *k_normalised,
                                 const fla_tensor *q_rstd, const fla_tensor *k_rstd, void *workspace,
                                 uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_gdn_chunk_fwd, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, chunk_size, use_qk_l2norm_in_kernel, o, g_cumsum, final_state, h, v_new, w, q_normalised, k_normalised, q_rstd, k_rstd, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::fused_impl(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, chunk_size,
                           use_qk_l2norm_in_kernel, o, g_cumsum, final_state, h, v_new, w, q_normalised, k_normalised, q_rstd,
                           k_rstd, workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_gdn_chunk_fwd_state_pool_get_workspace_size)(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v,
                                                           const fla_tensor *g, const fla_tensor *beta, double scale,
                                                           const fla_tensor *state_pool, const fla_tensor *state_indices,
                                                           const fla_int_array *cu_seqlens, int64_t chunk_size,
                                                           bool use_qk_l2norm_in_kernel, const fla_tensor *o,
                                                           uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_gdn_chunk_fwd_state_pool_get_workspace_size, q, k, v, g, beta, scale, state_pool, state_indices, cu_seqlens, chunk_size, use_qk_l2norm_in_kernel, o, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "gdn_chunk_fwd_state_pool: workspace_size must not be null.");
    if (!state_indices) return fla::fail(FLA_ERR_NULL, "gdn_chunk_fwd_state_pool: state_indices must not be null.");
    return fla::guarded([&] { return fla::fused_impl(q, k, v, g, beta, scale, state_pool, true, cu_seqlens, chunk_size, use_qk_l2norm_in_kernel, o,
                           nullptr, state_pool, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr,
                           workspace_size, state_indices); });
}

FLA_ENTRY(fla_gdn_chunk_fwd_state_pool)(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
                                        const fla_tensor *beta, double scale, const fla_tensor *state_pool,
                                        const fla_tensor *state_indices, const fla_int_array *cu_seqlens, int64_t chunk_size,
                                        bool use_qk_l2norm_in_kernel, const fla_tensor *o, void *workspace,
                                        uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_gdn_chunk_fwd_state_pool, q, k, v, g, beta, scale, state_pool, state_indices, cu_seqlens, chunk_size, use_qk_l2norm_in_kernel, o, workspace, workspace_size, stream);
    if (!state_indices) return fla::fail(FLA_ERR_NULL, "gdn_chunk_fwd_state_pool: state_indices must not be null.");
    return fla::guarded([&] { return fla::fused_impl(q, k, v, g, beta, scale, state_pool, true, cu_seqlens, chunk_size, use_qk_l2norm_in_kernel, o,
                           nullptr, state_pool, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, workspace, workspace_size,
                           static_cast<hipStream_t>(stream), nullptr, state_indices); });
}
