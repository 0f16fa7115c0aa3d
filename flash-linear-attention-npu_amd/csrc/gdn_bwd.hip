// Chunk-parallel stages of the gated-delta-rule BACKWARD, bf16 MFMA with fp32 accumulation, one
// workgroup of four waves per chunk; wave w owns token rows 16w..16w+15 of every output:
//   chunk_bwd_dv_local        dv = triu(k q^T e^{G_j-G_i}) scale . do
//   chunk_bwd_dqkwg           dq, dk, dw and the gradient of the cumsummed gate from h, dh, v_new, do, dv
//   prepare_wy_repr_bwd_da    gradient of the strictly-lower chunk matrix (stored transposed)
//   prepare_wy_repr_bwd_full  dk, dv, dbeta, dg of w = A (k beta e^G), u = A (v beta)
// Stage math: torch_custom/fla_npu/test/golden.py:18-172 (dv_local),
// tests/atk/chunk_bwd_dqkwg/scripts/chunk_bwd_dqkwg_cpu.py:67-409 (dqkwg),
// torch_custom/fla_npu/test/test_npu_prepare_wy_repr_bwd_da.py:170-282 (bwd_da),
// torch_custom/fla_npu/test/test_npu_prepare_wy_repr_bwd_full.py:46-486 (bwd_full).
// Operators with key-head outputs (dq, dk) loop over the value heads that share a key head inside one
// workgroup, so grouped value heads need neither atomics nor a second pass.
#include "gdn_common.h"
#include "chunk_inverse.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ f32x4 zero4() { return f32x4{0.f, 0.f, 0.f, 0.f}; }

// Stages `len` gate values of a chunk (clamped: rows past the tail repeat the last one) into LDS.
__device__ __forceinline__ void stage_scalars(float *dst, const View3 &v, int b, int h, int start, int len) {
    if (threadIdx.x < kChunk) dst[threadIdx.x] = load_scalar(v, b, h, start + min((int)threadIdx.x, len - 1));
}

// =============================================================================
// chunk_bwd_dv_local
// =============================================================================
struct DvLocalParams {
    ChunkGeom geom;
    View4 q, k, d_o, dv;
    View3 g;
    float scale;
};

// C128: 128-token chunks, one workgroup per 64-row half.  The first half also receives the block that couples it to the
// second half (every column of it lies after every row, so it carries no mask); the gate is cumulated over the whole
// chunk, so the factors e^{G_j - G_i} need no re-basing.
template <int K, int V, bool C128>
__global__ void __launch_bounds__(kThreads) dv_local_kernel(const DvLocalParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pk = K + 8, pv = V + 16, pa = kChunk + 8;
    elem *qS = reinterpret_cast<elem *>(smem);
    elem *kS = qS + kChunk * pk;
    elem *oS = kS + kChunk * pk;
    elem *aS = oS + kChunk * pv;
    float *gS = reinterpret_cast<float *>(aS + kChunk * pa);   // gates of the rows
    float *cS = gS + kChunk;                                   // gates of the columns of the current tile

    int cx, hv;
    block_chunk_head(p.geom, cx, hv);
    const int c = C128 ? cx >> 1 : cx, half = C128 ? cx & 1 : 0, b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, cstart, clen;
    chunk_span(p.geom, b, c, seq, cstart, clen);
    const int start = cstart + kChunk * half, len = min(kChunk, clen - kChunk * half);
    if (len <= 0) return;
    const int tid = threadIdx.x, w = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    const elem *qg = static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh;
    const elem *og = static_cast<const elem *>(p.d_o.p) + b * p.d_o.sb + hv * p.d_o.sh;
    {   // the rows' k and gates together with the diagonal tile's q and do: one round trip to memory
        TileCopy<kThreads, kChunk, K> tk, tq;
        TileCopy<kThreads, kChunk, V> to;
        tk.fetch(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st, p.k.st, len, tid);
        tq.fetch(qg + (int64_t)start * p.q.st, p.q.st, len, tid);
        to.fetch(og + (int64_t)start * p.d_o.st, p.d_o.st, len, tid);
        if (tid < kChunk) gS[tid] = cS[tid] = load_scalar(p.g, b, hv, start + min(tid, len - 1));
        tk.commit(kS, pk, len, tid);
        tq.commit(qS, pk, len, tid);
        to.commit(oS, pv, len, tid);
    }
    char *dvg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dv.p)) + b * p.dv.sb + hv * p.dv.sh +
                                         (int64_t)start * p.dv.st);
    f32x4 dacc[C128 ? V / 16 : 1];
#pragma unroll
    for (int ct = 0; ct < (C128 ? V / 16 : 1); ++ct) dacc[ct] = zero4();
    for (int t = half; t < (C128 ? 2 : 1); ++t) {
        const int tstart = cstart + kChunk * t, tlen = min(kChunk, clen - kChunk * t);
        if (tlen <= 0) break;
        const bool diag = t == half;
        if (!diag) {
            __syncthreads();   // the products of the diagonal tile are done with qS, oS, aS
            TileCopy<kThreads, kChunk, K> tq;
            TileCopy<kThreads, kChunk, V> to;
            tq.fetch(qg + (int64_t)tstart * p.q.st, p.q.st, tlen, tid);
            to.fetch(og + (int64_t)tstart * p.d_o.st, p.d_o.st, tlen, tid);
            stage_scalars(cS, p.g, b, hv, tstart, tlen);
            tq.commit(qS, pk, tlen, tid);
            to.commit(oS, pv, tlen, tid);
        }
        __syncthreads();
        // A[i][j] = <k_i, q_j> e^{G_j - G_i} scale for j >= i: row tile w, column tiles w..3 (all four off the diagonal)
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            f32x4 acc = zero4();
            if (!diag || ct >= w) {
#pragma unroll
                for (int j = 0; j < K / 32; ++j) acc = mfma16x32(frag_kc(kS, pk, 16 * w, 32 * j), frag_kc(qS, pk, 16 * ct, 32 * j), acc);
                const int col = 16 * ct + li;
                const float gc = cS[col];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = 16 * w + 4 * lg + e;
                    const float f = __expf(fminf(gc - gS[row], 0.f)) * p.scale;
                    acc[e] = ((!diag || col >= row) && col < tlen) ? acc[e] * f : 0.f;
                }
            }
            acc_to_tile(aS, pa, 16 * w, 16 * ct, acc);
        }
        __syncthreads();
#pragma unroll
        for (int ct = 0; ct < V / 16; ++ct) {
            f32x4 acc = C128 ? dacc[ct] : zero4();
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (!diag || 32 * j + 31 >= 16 * w)
                    acc = mfma16x32(frag_kc(aS, pa, 16 * w, 32 * j), frag_tr(oS, pv, 16 * ct, 32 * j), acc);
            if constexpr (C128) dacc[ct] = acc;
            else acc_to_global(dvg + 32 * ct, p.dv.st * 2, 16 * w, len, acc);   // one tile: each store leaves under the next product
        }
    }
    if constexpr (C128) {
#pragma unroll
        for (int ct = 0; ct < V / 16; ++ct) acc_to_global(dvg + 32 * ct, p.dv.st * 2, 16 * w, len, dacc[ct]);
    }
}

// =============================================================================
// chunk_bwd_dqkwg
// =============================================================================
constexpr int kDqkwgThreads = 512;   // two waves per SIMD over one set of LDS tiles
constexpr int kMaxRep = 64;          // value heads per key head that the 128-token-chunk form can carry sums for
struct DqkwgParams {
    ChunkGeom geom;
    View4 q, k, v, d_o, dv, dq, dk, dw;
    View3 g;
    const elem *h, *dh;
    int64_t h_sb, h_sh, h_sc, dh_sb, dh_sh, dh_sc;
    float *dg;
    int64_t dg_sb, dg_sh, dg_st;
    float scale;
    int h_row = 0, dh_row = 0;   // row stride of the K x V blocks of h and dh (V, or more for a column slab of wider blocks)
    // q was l2-normalised by the caller: rstd [B,Hk,T] of that pass, and dq leaves as the gradient of the raw q
    const float *q_rstd = nullptr;
    int64_t r_sb = 0, r_sh = 0;
};

// V is the width of the value slab held in LDS; VSLABS slabs cover the value dimension (1: V itself, 2: V = 256 as
// two passes of 128 columns, every product over the value dimension accumulated across the passes).
// CH = 2: 128-token chunks.  The workgroup takes the two 64-token halves of its chunk one after the other: both read
// the chunk's one h / dh block and the gate cumulated over the whole chunk; a row of the second half also gets
// ds_21 k_1 in dq, a row of the first half ds_21^T q_2 in dk (ds_21 = do_2 v_1^T e^{G_i - G_j} scale, unmasked), and
// the sum that lands on the chunk's last token collects sum_t k_t . dk_state_t over both halves.
// QNORM: q is an l2-normalised tensor and dq leaves as the gradient of the raw one (p.q_rstd); an instance of its own,
// so that the plain operator carries none of it.
template <int K, int V, bool GVA, int VSLABS = 1, int CH = 1, bool QNORM = false>
__global__ void __launch_bounds__(kDqkwgThreads) dqkwg_kernel(const DqkwgParams p) {
    static_assert(CH == 1 || VSLABS == 1, "128-token chunks are built for one value slab");
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pk = K + 16, pv = V + 8, ps = kChunk + 8;
    constexpr int KT = K / 16, KTH = KT / 2;   // column tiles of q/k: all, and per wave
    elem *qS = reinterpret_cast<elem *>(smem);
    elem *kS = qS + kChunk * pk;
    elem *vS = kS + kChunk * pk;
    elem *oS = vS + kChunk * pv;       // do
    elem *dvS = oS + kChunk * pv;
    elem *hS = dvS + kChunk * pv;      // h, then dh
    elem *sS = hS + K * pv;            // ds
    float *gS = reinterpret_cast<float *>(sS + kChunk * ps);
    float *red = gS + kChunk;          // 16 partial sums
    float *dgp = red + 16;             // [2][kChunk] row sums of the two column halves
    float *goS = dgp + 2 * kChunk;     // gates of the other half (CH = 2)
    float *ksS = goS + kChunk;         // [kMaxRep] sum_t k_t . dk_state_t of the first half, per value head (CH = 2)

    int c, hk;
    block_chunk_head(p.geom, c, hk);
    const int b = blockIdx.z;
    const int rep = GVA ? p.geom.Hv / p.geom.Hk : 1;   // without grouping the head loop is a single pass
    int seq, cstart, clen;
    chunk_span(p.geom, b, c, seq, cstart, clen);
    for (int hh = 0; hh < CH; ++hh) {
    const int start = cstart + kChunk * hh, len = min(kChunk, clen - kChunk * hh);
    if (len <= 0) break;
    const int ostart = cstart + kChunk * (1 - hh), olen = CH > 1 ? min(kChunk, clen - kChunk * (1 - hh)) : 0;
    const bool last_half = kChunk * (hh + 1) >= clen;   // the chunk's last token is one of this half's rows
    if (hh > 0) __syncthreads();
    // eight waves: wave (w, half) owns token rows 16w.. and column tiles half*KTH .. half*KTH+KTH-1 of q/k;
    // waves w and 4 + w share a SIMD
    const int tid = threadIdx.x, w = wave_id() & 3, half = wave_id() >> 2, l = lane_id(), li = l & 15, lg = l >> 4;
    {
        TileCopy<kDqkwgThreads, kChunk, K> tq, tk;
        tq.fetch(static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh + (int64_t)start * p.q.st, p.q.st, len, tid);
        tk.fetch(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st, p.k.st, len, tid);
        tq.commit(qS, pk, len, tid);
        tk.commit(kS, pk, len, tid);
    }
    f32x4 dq_acc[KTH], dk_acc[KTH];
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) dq_acc[ct] = dk_acc[ct] = zero4();
    static_assert(!QNORM || CH == 1, "the de-normalising form is built for 64-token chunks");
    float qdot[4] = {0.f, 0.f, 0.f, 0.f};   // QNORM: <q, dq> of this lane's four rows, over every value head
    float q_rs[4] = {1.f, 1.f, 1.f, 1.f};   // QNORM: rstd of those rows, fetched ahead of everything else
    if constexpr (QNORM) {
#pragma unroll
        for (int e = 0; e < 4; ++e) q_rs[e] = p.q_rstd[b * p.r_sb + hk * p.r_sh + start + min(16 * w + 4 * lg + e, len - 1)];
    }

    for (int r = 0; r < rep; ++r) {
        const int hv = hk * rep + r;
        if (r > 0) __syncthreads();      // the previous head's tiles are no longer read
        float hd = 0.f;                  // this thread's share of sum(h . dh)
        f32x4 dqs[KTH], dsacc[2];
        f32x4 dwacc[VSLABS > 1 ? KTH : 1], dksacc[VSLABS > 1 ? KTH : 1];   // only carried across slabs
#pragma unroll
        for (int ct = 0; ct < KTH; ++ct) dqs[ct] = zero4();
        dsacc[0] = dsacc[1] = zero4();
        if constexpr (VSLABS > 1) {
#pragma unroll
            for (int ct = 0; ct < KTH; ++ct) dwacc[ct] = dksacc[ct] = zero4();
        }
        char *dwg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dw.p)) + b * p.dw.sb + hv * p.dw.sh +
                                             (int64_t)start * p.dw.st);
#pragma unroll
        for (int vs = 0; vs < VSLABS; ++vs) {
            if (vs > 0) __syncthreads();     // the previous slab's tiles are no longer read
            TileCopy<kDqkwgThreads, K, V> tdh;
            {
                TileCopy<kDqkwgThreads, kChunk, V> tv, to, tdv;
                TileCopy<kDqkwgThreads, K, V> th;
                tv.fetch(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st + vs * V, p.v.st, len, tid);
                to.fetch(static_cast<const elem *>(p.d_o.p) + b * p.d_o.sb + hv * p.d_o.sh + (int64_t)start * p.d_o.st + vs * V, p.d_o.st, len, tid);
                tdv.fetch(static_cast<const elem *>(p.dv.p) + b * p.dv.sb + hv * p.dv.sh + (int64_t)start * p.dv.st + vs * V, p.dv.st, len, tid);
                th.fetch(p.h + b * p.h_sb + hv * p.h_sh + (int64_t)c * p.h_sc + vs * V, p.h_row, K, tid);
                tdh.fetch(p.dh + b * p.dh_sb + hv * p.dh_sh + (int64_t)c * p.dh_sc + vs * V, p.dh_row, K, tid);
                if (vs == 0) stage_scalars(gS, p.g, b, hv, start, len);
                tv.commit(vS, pv, len, tid);
                to.commit(oS, pv, len, tid);
                tdv.commit(dvS, pv, len, tid);
                th.commit(hS, pv, K, tid);
#pragma unroll
                for (int m = 0; m < TileCopy<kDqkwgThreads, K, V>::N; ++m) {
                    const elemx8 a = __builtin_bit_cast(elemx8, th.r[m]), d = __builtin_bit_cast(elemx8, tdh.r[m]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) hd += (float)a[e] * (float)d[e];
                }
            }
            __syncthreads();
            // ---- products with the state at chunk start: dq (state part), dw; and the ds tile ---------
#pragma unroll
            for (int ct = 0; ct < KTH; ++ct) {
                const int cg = half * KTH + ct;
                f32x4 a = dqs[ct], d = VSLABS > 1 ? dwacc[ct] : zero4();
#pragma unroll
                for (int j = 0; j < V / 32; ++j) {
                    const elemx8 hf = frag_kc(hS, pv, 16 * cg, 32 * j);
                    a = mfma16x32(frag_kc(oS, pv, 16 * w, 32 * j), hf, a);
                    d = mfma16x32(frag_kc(dvS, pv, 16 * w, 32 * j), hf, d);
                }
                dqs[ct] = a;
                if constexpr (VSLABS > 1) dwacc[ct] = d;
                else acc_to_global(dwg + 32 * cg, p.dw.st * 2, 16 * w, len, -d);
            }
#pragma unroll
            for (int cc = 0; cc < 2; ++cc) {     // ds column tiles half and half + 2 of row tile w
                const int ct = half + 2 * cc;
                if (ct <= w) {
#pragma unroll
                    for (int j = 0; j < V / 32; ++j)
                        dsacc[cc] = mfma16x32(frag_kc(oS, pv, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), dsacc[cc]);
                }
                if (vs == VSLABS - 1) {      // complete: gate factors, causal mask, to LDS
                    f32x4 acc = zero4();
                    if (ct <= w) {
                        acc = dsacc[cc];
                        const int col = 16 * ct + li;
                        const float gc = gS[col];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int row = 16 * w + 4 * lg + e;
                            const float f = __expf(fminf(gS[row] - gc, 0.f)) * p.scale;
                            acc[e] = (col <= row && row < len) ? acc[e] * f : 0.f;
                        }
                    }
                    acc_to_tile(sS, ps, 16 * w, 16 * ct, acc);
                }
            }
            __syncthreads();                 // every wave is done with h; ds is complete after the last slab
            tdh.commit(hS, pv, K, tid);
            __syncthreads();
            if constexpr (VSLABS > 1) {      // dk (state part) of this slab; the single-slab form folds it into the loop below
#pragma unroll
                for (int ct = 0; ct < KTH; ++ct)
#pragma unroll
                    for (int j = 0; j < V / 32; ++j)
                        dksacc[ct] = mfma16x32(frag_kc(vS, pv, 16 * w, 32 * j), frag_kc(hS, pv, 16 * (half * KTH + ct), 32 * j), dksacc[ct]);
            }
        }
        if constexpr (VSLABS > 1) {
#pragma unroll
            for (int ct = 0; ct < KTH; ++ct) acc_to_global(dwg + 32 * (half * KTH + ct), p.dw.st * 2, 16 * w, len, -dwacc[ct]);
        }
        // ---- products with the state gradient, gate factors, intra-chunk parts -------------------------
        const float g_last = CH > 1 ? load_scalar(p.g, b, hv, cstart + clen - 1) : gS[len - 1];
        float grow[4], eq[4], ek[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            grow[e] = gS[16 * w + 4 * lg + e];
            eq[e] = __expf(grow[e]) * p.scale;
            ek[e] = __expf(g_last - grow[e]);
        }
        float dg_row[4] = {0.f, 0.f, 0.f, 0.f}, qdq[4] = {0.f, 0.f, 0.f, 0.f}, kdk_state = 0.f;
#pragma unroll
        for (int ct = 0; ct < KTH; ++ct) {
            const int cg = half * KTH + ct;
            f32x4 dks = zero4();
            if constexpr (VSLABS > 1) {
                dks = dksacc[ct];
            } else {
#pragma unroll
                for (int j = 0; j < V / 32; ++j) dks = mfma16x32(frag_kc(vS, pv, 16 * w, 32 * j), frag_kc(hS, pv, 16 * cg, 32 * j), dks);
            }
            f32x4 dq = dqs[ct], dk;
            float kv[4], qv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                kv[e] = (float)kS[row * pk + 16 * cg + li];
                qv[e] = (float)qS[row * pk + 16 * cg + li];
                dq[e] *= eq[e];
                dk[e] = dks[e] * ek[e];
                kdk_state += row < len ? dk[e] * kv[e] : 0.f;
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (32 * j <= 16 * w + 15) dq = mfma16x32(frag_kc(sS, ps, 16 * w, 32 * j), frag_tr(kS, pk, 16 * cg, 32 * j), dq);
                if (32 * j + 31 >= 16 * w) dk = mfma16x32(frag_tr(sS, ps, 16 * w, 32 * j), frag_tr(qS, pk, 16 * cg, 32 * j), dk);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                dg_row[e] += dq[e] * qv[e] - dk[e] * kv[e];
                if constexpr (QNORM) qdq[e] += dq[e] * qv[e];
            }
            dq_acc[ct] += dq;
            dk_acc[ct] += dk;
        }
        if constexpr (CH > 1) {
            if (olen > 0) {   // the block that couples the halves
                __syncthreads();   // dv, dh and ds are no longer read: their tiles take the other half's operands
                elem *xS = dvS;    // other half: v (hh = 1) or do (hh = 0)
                elem *yS = hS;     // other half: k (hh = 1) or q (hh = 0); the state tile is K x pv elements
                constexpr int py = K * pv >= kChunk * pk ? pk : K + 8;
                static_assert(K * pv >= kChunk * py, "the other half's k/q tile must fit the state tile");
                {
                    TileCopy<kDqkwgThreads, kChunk, V> tx;
                    TileCopy<kDqkwgThreads, kChunk, K> ty;
                    const View4 &xv = hh ? p.v : p.d_o, &yv = hh ? p.k : p.q;
                    tx.fetch(static_cast<const elem *>(xv.p) + b * xv.sb + hv * xv.sh + (int64_t)ostart * xv.st, xv.st, olen, tid);
                    ty.fetch(static_cast<const elem *>(yv.p) + b * yv.sb + hk * yv.sh + (int64_t)ostart * yv.st, yv.st, olen, tid);
                    stage_scalars(goS, p.g, b, hv, ostart, olen);
                    tx.commit(xS, pv, olen, tid);
                    ty.commit(yS, py, olen, tid);
                }
                __syncthreads();
                const elem *rowS = hh ? oS : vS;   // own do (second half) or own v (first half)
#pragma unroll
                for (int cc = 0; cc < 2; ++cc) {
                    const int ct = half + 2 * cc;
                    f32x4 acc = zero4();
#pragma unroll
                    for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(rowS, pv, 16 * w, 32 * j), frag_kc(xS, pv, 16 * ct, 32 * j), acc);
                    const int col = 16 * ct + li;
                    const float go = goS[col];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = 16 * w + 4 * lg + e;
                        const float d = hh ? gS[row] - go : go - gS[row];   // later token minus earlier token
                        acc[e] = (row < len && col < olen) ? acc[e] * __expf(fminf(d, 0.f)) * p.scale : 0.f;
                    }
                    acc_to_tile(sS, ps, 16 * w, 16 * ct, acc);
                }
                __syncthreads();
#pragma unroll
                for (int ct = 0; ct < KTH; ++ct) {
                    const int cg = half * KTH + ct;
                    f32x4 d = zero4();
#pragma unroll
                    for (int j = 0; j < 2; ++j) d = mfma16x32(frag_kc(sS, ps, 16 * w, 32 * j), frag_tr(yS, py, 16 * cg, 32 * j), d);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = 16 * w + 4 * lg + e;
                        const float own = (float)(hh ? qS : kS)[row * pk + 16 * cg + li];
                        dg_row[e] += hh ? d[e] * own : -d[e] * own;
                    }
                    if (hh) dq_acc[ct] += d;
                    else dk_acc[ct] += d;
                }
            }
        }
        // block sums for the gradient that lands on the last token of the chunk
        float s1 = hd, s2 = kdk_state;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            s1 += __shfl_xor(s1, off, kWave);
            s2 += __shfl_xor(s2, off, kWave);
        }
        if (l == 0) {
            red[wave_id()] = s1;
            red[8 + wave_id()] = s2;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float v = group_sum<16>(dg_row[e]);
            if (li == 0) dgp[half * kChunk + 16 * w + 4 * lg + e] = v;
            if constexpr (QNORM) {   // the two column halves of <q, dq> meet in the arrays the 128-token form uses
                const float u = group_sum<16>(qdq[e]);
                if (li == 0) goS[half * kChunk + 16 * w + 4 * lg + e] = u;
            }
        }
        __syncthreads();
        if constexpr (QNORM) {
#pragma unroll
            for (int e = 0; e < 4; ++e) qdot[e] += goS[16 * w + 4 * lg + e] + goS[kChunk + 16 * w + 4 * lg + e];
        }
        if (tid < kChunk && tid < len) {
            float hs = 0.f, ks = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                hs += red[i];
                ks += red[8 + i];
            }
            if (CH > 1 && hh > 0) ks += ksS[r];
            const float dg_last = hs * __expf(g_last) + ks;
            p.dg[b * p.dg_sb + hv * p.dg_sh + (int64_t)(start + tid) * p.dg_st] =
                dgp[tid] + dgp[kChunk + tid] + (last_half && tid == len - 1 ? dg_last : 0.f);
            if (CH > 1 && hh == 0 && tid == 0) ksS[r] = ks;
        }
    }
    if constexpr (QNORM) {
        // q is the l2-normalised tile y = x rstd: the gradient of x is (dq - y <y, dq>) rstd per row; <y, dq> was summed
        // with the gate gradient's row sums above
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
#pragma unroll
            for (int ct = 0; ct < KTH; ++ct)
                dq_acc[ct][e] = (dq_acc[ct][e] - (float)qS[row * pk + 16 * (half * KTH + ct) + li] * qdot[e]) * q_rs[e];
        }
    }
    char *dqg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dq.p)) + b * p.dq.sb + hk * p.dq.sh + (int64_t)start * p.dq.st);
    char *dkg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dk.p)) + b * p.dk.sb + hk * p.dk.sh + (int64_t)start * p.dk.st);
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {
        acc_to_global(dqg + 32 * (half * KTH + ct), p.dq.st * 2, 16 * w, len, dq_acc[ct]);
        acc_to_global(dkg + 32 * (half * KTH + ct), p.dk.st * 2, 16 * w, len, dk_acc[ct]);
    }
    }   // halves of the chunk
}

// =============================================================================
// prepare_wy_repr_bwd_da
// =============================================================================
struct WyBwdParams {
    ChunkGeom geom;
    View4 k, v, A, dA, dw, du, dk, dv;
    View3 g, beta;
    float *dbeta, *dg;
    int64_t db_sb, db_sh, db_st, dg_sb, dg_sh, dg_st;
    // accumulating form only: k was l2-normalised by the caller, rstd [B,Hk,T]; dk leaves as the gradient of the raw k
    const float *k_rstd = nullptr;
    int64_t r_sb = 0, r_sh = 0;
};

// Commits a fetched tile with every row scaled by f[row] (rows past `len` become zero).
template <int NCOLS>
__device__ __forceinline__ void commit_scaled(const TileCopy<kThreads, kChunk, NCOLS> &t, elem *dst, int pitch, int len,
                                              const float *f, int tid) {
#pragma unroll
    for (int m = 0; m < TileCopy<kThreads, kChunk, NCOLS>::N; ++m) {
        const int idx = m * kThreads + tid;
        const int r = idx / (NCOLS / 8), c8 = (idx % (NCOLS / 8)) << 3;
        const elemx8 a = __builtin_bit_cast(elemx8, t.r[m]);
        const float s = r < len ? f[r] : 0.f;
        f32x4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo[e] = (float)a[e] * s;
            hi[e] = (float)a[4 + e] * s;
        }
        *reinterpret_cast<elemx8 *>(dst + r * pitch + c8) = frag_from_acc(lo, hi);
    }
}
// Commits a 64 x 64 chunk matrix, zeroing rows and columns past the tail; with `colf` every column j is
// also scaled by colf[j].
__device__ __forceinline__ void commit_square(const TileCopy<kThreads, kChunk, kChunk> &t, elem *dst, int pitch, int len,
                                              const float *colf, int tid) {
#pragma unroll
    for (int m = 0; m < TileCopy<kThreads, kChunk, kChunk>::N; ++m) {
        const int idx = m * kThreads + tid;
        const int r = idx >> 3, c8 = (idx & 7) << 3;
        elemx8 a = __builtin_bit_cast(elemx8, t.r[m]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const bool in = r < len && c8 + e < len;
            a[e] = in ? (colf ? (elem)((float)a[e] * colf[c8 + e]) : a[e]) : (elem)0.f;
        }
        *reinterpret_cast<elemx8 *>(dst + r * pitch + c8) = a;
    }
}

template <int K, int V>
__global__ void __launch_bounds__(kThreads) wy_bwd_da_kernel(const WyBwdParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pk = K + 8, pv = V + 8, pa = kChunk + 8;
    elem *dwS = reinterpret_cast<elem *>(smem);
    elem *kS = dwS + kChunk * pk;
    elem *duS = kS + kChunk * pk;
    elem *vS = duS + kChunk * pv;
    elem *aS = vS + kChunk * pv;
    // the two intermediate 64 x 64 matrices reuse the dw and du tiles, which are dead by then: the kernel
    // stays under half of a compute unit's LDS, so two workgroups overlap their load and compute phases
    elem *m4S = dwS;
    elem *m5S = duS;
    float *gS = reinterpret_cast<float *>(aS + kChunk * pa);
    float *bS = gS + kChunk;
    float *fS = bS + kChunk;           // beta e^G

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x, w = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    {
        TileCopy<kThreads, kChunk, K> tdw, tk;
        TileCopy<kThreads, kChunk, V> tdu, tv;
        TileCopy<kThreads, kChunk, kChunk> ta;
        tdw.fetch(static_cast<const elem *>(p.dw.p) + b * p.dw.sb + hv * p.dw.sh + (int64_t)start * p.dw.st, p.dw.st, len, tid);
        tk.fetch(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st, p.k.st, len, tid);
        tdu.fetch(static_cast<const elem *>(p.du.p) + b * p.du.sb + hv * p.du.sh + (int64_t)start * p.du.st, p.du.st, len, tid);
        tv.fetch(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st, p.v.st, len, tid);
        ta.fetch(static_cast<const elem *>(p.A.p) + b * p.A.sb + hv * p.A.sh + (int64_t)start * p.A.st, p.A.st, len, tid);
        if (tid < kChunk) {
            const int t = start + min(tid, len - 1);
            const float gg = load_scalar(p.g, b, hv, t), bb = load_scalar(p.beta, b, hv, t);
            gS[tid] = gg;
            bS[tid] = bb;
            fS[tid] = bb * __expf(gg);
        }
        __syncthreads();
        tdw.commit(dwS, pk, len, tid);
        tdu.commit(duS, pv, len, tid);
        commit_scaled<K>(tk, kS, pk, len, fS, tid);
        commit_scaled<V>(tv, vS, pv, len, bS, tid);
        commit_square(ta, aS, pa, len, nullptr, tid);
    }
    __syncthreads();
    // M4 = strict_lower(dw (k beta e^G)^T + du (v beta)^T), row tile w
    f32x4 m4[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        f32x4 acc = zero4();
        if (ct <= w) {
#pragma unroll
            for (int j = 0; j < K / 32; ++j) acc = mfma16x32(frag_kc(dwS, pk, 16 * w, 32 * j), frag_kc(kS, pk, 16 * ct, 32 * j), acc);
#pragma unroll
            for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(duS, pv, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), acc);
            const int col = 16 * ct + li;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                acc[e] = (col < row && row < len) ? acc[e] : 0.f;
            }
        }
        m4[ct] = acc;
    }
    __syncthreads();   // every wave has read its dw / du rows: their tiles may be overwritten
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) acc_to_tile(m4S, pa, 16 * w, 16 * ct, m4[ct]);
    __syncthreads();
    // M5 = M4 A^T
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        f32x4 acc = zero4();
#pragma unroll
        for (int j = 0; j < 2; ++j) acc = mfma16x32(frag_kc(m4S, pa, 16 * w, 32 * j), frag_kc(aS, pa, 16 * ct, 32 * j), acc);
        acc_to_tile(m5S, pa, 16 * w, 16 * ct, acc);
    }
    __syncthreads();
    // (A^T M5)^T = M5^T A, gated, negated and masked; rows of this product are the stored rows
    char *dag = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dA.p)) + b * p.dA.sb + hv * p.dA.sh +
                                         (int64_t)start * p.dA.st);
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        f32x4 acc = zero4();
        if (ct >= w) {
#pragma unroll
            for (int j = 0; j < 2; ++j) acc = mfma16x32(frag_tr(m5S, pa, 16 * w, 32 * j), frag_tr(aS, pa, 16 * ct, 32 * j), acc);
            const int col = 16 * ct + li;     // i of the untransposed matrix
            const float gc = gS[col];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;   // j of the untransposed matrix
                acc[e] = (col > row && col < len) ? -acc[e] * __expf(fminf(gc - gS[row], 0.f)) : 0.f;
            }
        }
        acc_to_global(dag + 32 * ct, p.dA.st * 2, 16 * w, len, acc);
    }
}

// =============================================================================
// prepare_wy_repr_bwd_full
// =============================================================================
// GVA: several value heads share the key head, dk is accumulated over them in registers; otherwise every
// dk tile goes straight to memory and the column loop needs no accumulator array.
// ACC: dk and dg are added to what the caller's tensors hold.  The dk tiles then wait in registers like the GVA sums and
// leave through an fp32 LDS tile (the k and dw tiles, dead by then), so that memory is read and written in whole
// 16-byte row pieces: adding tile by tile from the accumulator layout, four bytes per lane, cost more than the separate
// elementwise pass it replaces.
// DA: dA is not an input.  prepare_wy_repr_bwd_da's result for the chunk is formed in place, from the tiles this kernel
// stages anyway (du v^T while du is in its tile, dw k^T once dw has taken it; the row scales beta and beta e^G of the
// second operands become column scales of the products), through the same two 64 x 64 intermediates, which pass through
// the tiles that then receive dA and its beta-scaled copy.
// AINV: A is not an input either.  The chunk's (I + strict_lower(beta k k^T e^{G_i - G_j}))^-1 is rebuilt from the k
// tile, g and beta that are staged anyway, with the arithmetic of the fused kkt + inverse kernel (scores rounded to
// the element type, the same block inversion), so the matrix equals the one that kernel would have stored; the fp32
// scores pass through the two tiles that later hold dA.
template <int K, int V, bool GVA, bool ACC = false, bool DA = false, bool AINV = false>
__global__ void __launch_bounds__(kThreads, GVA ? 1 : 2) wy_bwd_full_kernel(const WyBwdParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    // du and dw share one tile (du is dead once A^T du is formed) and v, which is only read element-wise,
    // is unpadded: the kernel stays under half of a compute unit's LDS and two workgroups share one
    constexpr int KV = K > V ? K : V;
    constexpr int pk = K + 16, px = KV + 16, pvv = V, pa = kChunk + 8;
    constexpr int KT = K / 16, VT = V / 16;
    elem *kS = reinterpret_cast<elem *>(smem);
    elem *xS = kS + kChunk * pk;        // du, then dw
    elem *vS = xS + kChunk * px;
    elem *aS = vS + kChunk * pvv;
    elem *dS = aS + kChunk * pa;        // dA as stored
    elem *dbS = dS + kChunk * pa;       // dA with column j scaled by beta_j
    float *gS = reinterpret_cast<float *>(dbS + kChunk * pa);
    float *bS = gS + kChunk;

    int c, hk;
    block_chunk_head(p.geom, c, hk);
    const int b = blockIdx.z;
    const int rep = GVA ? p.geom.Hv / p.geom.Hk : 1;   // without grouping the head loop is a single pass
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x, w = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    TileCopy<kThreads, kChunk, K> tk;
    tk.fetch(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st, p.k.st, len, tid);
    constexpr bool HOLD = GVA || ACC;   // dk tiles stay in registers until the head loop ends
    f32x4 dk_acc[HOLD ? KT : 1];
#pragma unroll
    for (int ct = 0; ct < (HOLD ? KT : 1); ++ct) dk_acc[ct] = zero4();
    char *dkg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dk.p)) + b * p.dk.sb + hk * p.dk.sh + (int64_t)start * p.dk.st);
    TileCopy<kThreads, kChunk, K> tdk;
    if constexpr (ACC && !AINV) tdk.fetch(reinterpret_cast<const elem *>(dkg), p.dk.st, len, tid);

    for (int r = 0; r < rep; ++r) {
        const int hv = hk * rep + r;
        if (r > 0) __syncthreads();
        TileCopy<kThreads, kChunk, K> tdw;
        {
            TileCopy<kThreads, kChunk, V> tdu, tv;
            TileCopy<kThreads, kChunk, kChunk> ta, td;
            // AINV: k, g and beta are asked for before everything else.  Loads return in order, so the scores and the
            // inversion can start as soon as these three are there and run while du and v are still on their way.
            float gv = 0.f, bv = 0.f;
            if constexpr (AINV) {
                if (tid < kChunk) {
                    const int t = start + min(tid, len - 1);
                    gv = load_scalar(p.g, b, hv, t);
                    bv = load_scalar(p.beta, b, hv, t);
                }
            }
            tdu.fetch(static_cast<const elem *>(p.du.p) + b * p.du.sb + hv * p.du.sh + (int64_t)start * p.du.st, p.du.st, len, tid);
            tv.fetch(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st, p.v.st, len, tid);
            if constexpr (!AINV) ta.fetch(static_cast<const elem *>(p.A.p) + b * p.A.sb + hv * p.A.sh + (int64_t)start * p.A.st, p.A.st, len, tid);
            if constexpr (!DA) td.fetch(static_cast<const elem *>(p.dA.p) + b * p.dA.sb + hv * p.dA.sh + (int64_t)start * p.dA.st, p.dA.st, len, tid);
            if (tid < kChunk) {
                if constexpr (AINV) {
                    gS[tid] = gv;
                    bS[tid] = bv;
                } else {
                    const int t = start + min(tid, len - 1);
                    gS[tid] = load_scalar(p.g, b, hv, t);
                    bS[tid] = load_scalar(p.beta, b, hv, t);
                }
            }
            if (r == 0) tk.commit(kS, pk, len, tid);
            __syncthreads();
            if constexpr (!AINV) {
                tdu.commit(xS, px, len, tid);
                tv.commit(vS, pvv, len, tid);
            }
            if constexpr (AINV) {
                static_assert(DA && pa == 72, "the fp32 score block lies over the two dA tiles; the inverse is written at pitch 72");
                static_assert(kChunk * 68 * 4 <= 2 * kChunk * pa * 2, "the fp32 score block must fit the two dA tiles");
                float *sS = reinterpret_cast<float *>(dS);
                // the ten tiles on and below the diagonal dealt 3, 3, 2, 2 (by row block it would be 1, 2, 3, 4)
                switch (w) {
                    case 0:
                        kkt_score_tile<0, 0>(kS, pk, K, gS, bS, len, sS);
                        kkt_score_tile<3, 0>(kS, pk, K, gS, bS, len, sS);
                        kkt_score_tile<3, 1>(kS, pk, K, gS, bS, len, sS);
                        break;
                    case 1:
                        kkt_score_tile<1, 0>(kS, pk, K, gS, bS, len, sS);
                        kkt_score_tile<1, 1>(kS, pk, K, gS, bS, len, sS);
                        kkt_score_tile<2, 0>(kS, pk, K, gS, bS, len, sS);
                        break;
                    case 2:
                        kkt_score_tile<2, 1>(kS, pk, K, gS, bS, len, sS);
                        kkt_score_tile<2, 2>(kS, pk, K, gS, bS, len, sS);
                        break;
                    default:
                        kkt_score_tile<3, 2>(kS, pk, K, gS, bS, len, sS);
                        kkt_score_tile<3, 3>(kS, pk, K, gS, bS, len, sS);
                        break;
                }
#pragma unroll
                for (int J = 1; J < 4; ++J)   // above the diagonal: zero
                    if (J > w) *reinterpret_cast<f32x4 *>(sS + (16 * w + li) * 68 + 16 * J + 4 * lg) = zero4();
                __syncthreads();
                invert64(sS, aS);
                if (tid < kChunk && tid >= len) aS[tid * pa + tid] = (elem)0.f;   // rows past the end hold nothing, as a staged A would
                tdu.commit(xS, px, len, tid);
                tv.commit(vS, pvv, len, tid);
            } else {
                commit_square(ta, aS, pa, len, nullptr, tid);
            }
            if constexpr (!DA) {
                commit_square(td, dS, pa, len, nullptr, tid);
                commit_square(td, dbS, pa, len, bS, tid);
            }
        }
        // dw is fetched only now, once the registers of the first batch are free; it lands during A^T du
        tdw.fetch(static_cast<const elem *>(p.dw.p) + b * p.dw.sb + hv * p.dw.sh + (int64_t)start * p.dw.st, p.dw.st, len, tid);
        if constexpr (ACC && AINV) {   // not needed before the end: asked for behind everything the products wait for
            if (r == 0) tdk.fetch(reinterpret_cast<const elem *>(dkg), p.dk.st, len, tid);
        }
        __syncthreads();
        float br[4], er[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            br[e] = bS[16 * w + 4 * lg + e];
            er[e] = __expf(gS[16 * w + 4 * lg + e]);
        }
        float db_row[4] = {0.f, 0.f, 0.f, 0.f}, dg_row[4] = {0.f, 0.f, 0.f, 0.f};
        const elemx8 at0 = frag_tr(aS, pa, 16 * w, 0), at1 = frag_tr(aS, pa, 16 * w, 32);
        char *dvg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dv.p)) + b * p.dv.sb + hv * p.dv.sh +
                                             (int64_t)start * p.dv.st);
#pragma unroll
        for (int ct = 0; ct < VT; ++ct) {      // A^T du
            f32x4 acc = mfma16x32(at0, frag_tr(xS, px, 16 * ct, 0), zero4());
            acc = mfma16x32(at1, frag_tr(xS, px, 16 * ct, 32), acc);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                db_row[e] += acc[e] * (float)vS[(16 * w + 4 * lg + e) * pvv + 16 * ct + li];
                acc[e] *= br[e];
            }
            acc_to_global(dvg + 32 * ct, p.dv.st * 2, 16 * w, len, acc);
            __builtin_amdgcn_sched_barrier(0);
        }
        f32x4 m4[4];                     // DA: row tile w of strict_lower(dw (k beta e^G)^T + du (v beta)^T)
        if constexpr (DA) {
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {
                f32x4 acc = zero4();
                if (ct <= w) {
#pragma unroll
                    for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(xS, px, 16 * w, 32 * j), frag_kc(vS, pvv, 16 * ct, 32 * j), acc);
                }
                m4[ct] = acc;
            }
        }
        __syncthreads();                 // du has been consumed by every wave
        tdw.commit(xS, px, len, tid);
        __syncthreads();
        if constexpr (DA) {
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {
                f32x4 acc = zero4();
                if (ct <= w) {
#pragma unroll
                    for (int j = 0; j < K / 32; ++j) acc = mfma16x32(frag_kc(xS, px, 16 * w, 32 * j), frag_kc(kS, pk, 16 * ct, 32 * j), acc);
                    const int col = 16 * ct + li;
                    const float bc = bS[col], fc = bc * __expf(gS[col]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = 16 * w + 4 * lg + e;
                        acc[e] = (col < row && row < len) ? acc[e] * fc + m4[ct][e] * bc : 0.f;
                    }
                }
                acc_to_tile(dS, pa, 16 * w, 16 * ct, acc);      // M4
            }
            __syncthreads();
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {                     // M5 = M4 A^T
                f32x4 acc = zero4();
#pragma unroll
                for (int j = 0; j < 2; ++j) acc = mfma16x32(frag_kc(dS, pa, 16 * w, 32 * j), frag_kc(aS, pa, 16 * ct, 32 * j), acc);
                acc_to_tile(dbS, pa, 16 * w, 16 * ct, acc);
            }
            __syncthreads();
            f32x4 da[4];                                         // rows 16 w.. of dA as stored: (A^T M5)^T, gated, negated, masked
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {
                f32x4 acc = zero4();
                if (ct >= w) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) acc = mfma16x32(frag_tr(dbS, pa, 16 * w, 32 * j), frag_tr(aS, pa, 16 * ct, 32 * j), acc);
                    const int col = 16 * ct + li;
                    const float gc = gS[col];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = 16 * w + 4 * lg + e;
                        acc[e] = (col > row && col < len) ? -acc[e] * __expf(fminf(gc - gS[row], 0.f)) : 0.f;
                    }
                }
                da[ct] = acc;
                acc_to_tile(dS, pa, 16 * w, 16 * ct, acc);      // M4 was last read before the barrier above
            }
            __syncthreads();                                     // every wave has read M5
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {
                // the stored value is the rounded one: the copy with column j scaled by beta_j starts from it, as a copy
                // made from memory would
                const elemx4 r4 = cvt4(da[ct]);
                const float bc = bS[16 * ct + li];
                acc_to_tile(dbS, pa, 16 * w, 16 * ct, f32x4{(float)r4[0] * bc, (float)r4[1] * bc, (float)r4[2] * bc, (float)r4[3] * bc});
            }
            __syncthreads();
        }
        const elemx8 dt0 = frag_tr(dS, pa, 16 * w, 0), dt1 = frag_tr(dS, pa, 16 * w, 32);
        const elemx8 db0 = frag_kc(dbS, pa, 16 * w, 0), db1 = frag_kc(dbS, pa, 16 * w, 32);
#pragma unroll
        for (int ct = 0; ct < KT; ++ct) {
            const elemx8 k0 = frag_tr(kS, pk, 16 * ct, 0), k1 = frag_tr(kS, pk, 16 * ct, 32);
            f32x4 p1 = mfma16x32(at0, frag_tr(xS, px, 16 * ct, 0), zero4());        // A^T dw
            p1 = mfma16x32(at1, frag_tr(xS, px, 16 * ct, 32), p1);
            f32x4 p2 = mfma16x32(dt0, k0, zero4());                                 // dA^T k
            p2 = mfma16x32(dt1, k1, p2);
            f32x4 q3 = mfma16x32(db0, k0, zero4());                                 // dA (k beta)
            q3 = mfma16x32(db1, k1, q3);
            f32x4 dk;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float kv = (float)kS[(16 * w + 4 * lg + e) * pk + 16 * ct + li];
                const float p1g = p1[e] * er[e];
                dk[e] = q3[e] + (p2[e] + p1g) * br[e];
                db_row[e] += (p2[e] + p1g) * kv;
                dg_row[e] += (p1g * br[e] + br[e] * p2[e] - q3[e]) * kv;
            }
            if constexpr (HOLD) dk_acc[ct] += dk;
            else acc_to_global(dkg + 32 * ct, p.dk.st * 2, 16 * w, len, dk);
            __builtin_amdgcn_sched_barrier(0);   // keeps the operand reads of later column tiles from piling up in registers
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float sb = group_sum<16>(db_row[e]), sg = group_sum<16>(dg_row[e]);
            const int row = 16 * w + 4 * lg + e;
            if (li == 0 && row < len) {
                p.dbeta[b * p.db_sb + hv * p.db_sh + (int64_t)(start + row) * p.db_st] = sb;
                float *dgp = p.dg + b * p.dg_sb + hv * p.dg_sh + (int64_t)(start + row) * p.dg_st;
                *dgp = ACC ? *dgp + sg : sg;
            }
        }
    }
    if constexpr (ACC) {
        constexpr int pf = K + 4;
        static_assert((size_t)kChunk * pf * 4 <= (size_t)kChunk * (pk + px) * 2, "the fp32 dk tile must fit the k and dw tiles");
        float *fS = reinterpret_cast<float *>(smem);
        __syncthreads();   // the last reads of k and dw are done
#pragma unroll
        for (int ct = 0; ct < KT; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) fS[(16 * w + 4 * lg + e) * pf + 16 * ct + li] = dk_acc[ct][e];
        __syncthreads();
#pragma unroll
        for (int m = 0; m < TileCopy<kThreads, kChunk, K>::N; ++m) {
            const int idx = m * kThreads + tid;
            const int r = idx / (K / 8), c8 = (idx % (K / 8)) << 3;
            const elemx8 in = __builtin_bit_cast(elemx8, tdk.r[m]);
            const f32x4 lo = *reinterpret_cast<const f32x4 *>(fS + r * pf + c8), hi = *reinterpret_cast<const f32x4 *>(fS + r * pf + c8 + 4);
            f32x4 a, c;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                a[e] = lo[e] + (float)in[e];
                c[e] = hi[e] + (float)in[4 + e];
            }
            if (p.k_rstd != nullptr) {   // k is the l2-normalised y = x rstd: dk of x is (dk - y <y, dk>) rstd per row
                const elemx8 y = __builtin_bit_cast(elemx8, tk.r[m]);   // the piece of k this thread fetched: same row, same columns
                float dot = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) dot += a[e] * (float)y[e] + c[e] * (float)y[4 + e];
                dot = group_sum<K / 8>(dot);                            // the K / 8 lanes that hold the row
                const float rs = p.k_rstd[b * p.r_sb + hk * p.r_sh + start + min(r, len - 1)];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a[e] = (a[e] - (float)y[e] * dot) * rs;
                    c[e] = (c[e] - (float)y[4 + e] * dot) * rs;
                }
            }
            if (r < len) *reinterpret_cast<elemx8 *>(dkg + ((int64_t)r * p.dk.st + c8) * 2) = frag_from_acc(a, c);
        }
    } else if constexpr (GVA) {
#pragma unroll
        for (int ct = 0; ct < KT; ++ct) acc_to_global(dkg + 32 * ct, p.dk.st * 2, 16 * w, len, dk_acc[ct]);
    }
}

// =============================================================================
// 128-token chunks in the two WY backward operators (prepare_wy_repr_bwd_full/README.md:74,101).  A and dA are
// 128 x 128 per chunk.  One workgroup per chunk; the products are the ones of the 64-token kernels with the
// contraction over 128 tokens, the operand tiles staged in 64-row pieces so that everything fits one CU's LDS.
// =============================================================================
// rows [0, valid) of a row-major source into an LDS tile of `nrows` rows, the rest zero; with `scale` every row r is
// multiplied by scale[r]; with `colf` every column c by colf[c]; columns >= `vcols` are zeroed.
template <int NCOLS>
__device__ __forceinline__ void stage_rows(elem *tile, int pitch, const elem *src, int64_t stride, int nrows, int valid,
                                           const float *scale, const float *colf = nullptr, int vcols = NCOLS) {
    constexpr int CPR = NCOLS / 8;
    for (int idx = threadIdx.x; idx < nrows * CPR; idx += kThreads) {
        const int r = idx / CPR, c8 = (idx % CPR) << 3;
        elemx8 a = {};
        if (r < valid) {
            a = *reinterpret_cast<const elemx8 *>(src + (int64_t)r * stride + c8);
            if (scale != nullptr || colf != nullptr || vcols < NCOLS) {
                const float sr = scale ? scale[r] : 1.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float f = c8 + e < vcols ? sr * (colf ? colf[c8 + e] : 1.f) : 0.f;
                    a[e] = (elem)((float)a[e] * f);
                }
            }
        }
        *reinterpret_cast<elemx8 *>(tile + r * pitch + c8) = a;
    }
}

template <int K, int V>
__global__ void __launch_bounds__(kThreads) wy_bwd_da128_kernel(const WyBwdParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int C = 128, pk = K + 8, pv = V + 8, pa = C + 8;
    elem *dwS = reinterpret_cast<elem *>(smem);      // 64 rows each: dw, k beta e^G, du, v beta of the block at hand
    elem *kS = dwS + kChunk * pk;
    elem *duS = kS + kChunk * pk;
    elem *vS = duS + kChunk * pv;
    elem *m4S = vS + kChunk * pv;                    // [128][pa]
    elem *aS = m4S + C * pa;                         // [128][pa]
    elem *m5S = dwS;                                 // [128][pa] over the operand tiles, dead by then
    static_assert((size_t)kChunk * (2 * pk + 2 * pv) >= (size_t)C * pa, "M5 must fit the operand tiles");
    float *gS = reinterpret_cast<float *>(aS + C * pa);
    float *bS = gS + C;
    float *fS = bS + C;                              // beta e^G

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x, w = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    if (tid < C) {
        const int t = start + min(tid, len - 1);
        const float gg = load_scalar(p.g, b, hv, t), bb = load_scalar(p.beta, b, hv, t);
        gS[tid] = gg;
        bS[tid] = bb;
        fS[tid] = bb * __expf(gg);
    }
    stage_rows<C>(aS, pa, static_cast<const elem *>(p.A.p) + b * p.A.sb + hv * p.A.sh + (int64_t)start * p.A.st, p.A.st, C, len,
                  nullptr, nullptr, len);
    __syncthreads();
    const elem *dwg = static_cast<const elem *>(p.dw.p) + b * p.dw.sb + hv * p.dw.sh + (int64_t)start * p.dw.st;
    const elem *dug = static_cast<const elem *>(p.du.p) + b * p.du.sb + hv * p.du.sh + (int64_t)start * p.du.st;
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st;
    const elem *vg = static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st;
    // M4 = strict_lower(dw (k beta e^G)^T + du (v beta)^T) in 64 x 64 blocks (0,0), (1,0), (1,1); block (0,1) is zero
    for (int blk = 0; blk < 3; ++blk) {
        const int rh = blk > 0, ch = blk > 1;
        if (blk > 0) __syncthreads();   // the previous block's products are done with the tiles that change
        if (blk != 2) {
            const int rv = max(0, min(kChunk, len - kChunk * rh));
            stage_rows<K>(dwS, pk, dwg + (int64_t)kChunk * rh * p.dw.st, p.dw.st, kChunk, rv, nullptr);
            stage_rows<V>(duS, pv, dug + (int64_t)kChunk * rh * p.du.st, p.du.st, kChunk, rv, nullptr);
        }
        if (blk != 1) {
            const int cv = max(0, min(kChunk, len - kChunk * ch));
            stage_rows<K>(kS, pk, kg + (int64_t)kChunk * ch * p.k.st, p.k.st, kChunk, cv, fS + kChunk * ch);
            stage_rows<V>(vS, pv, vg + (int64_t)kChunk * ch * p.v.st, p.v.st, kChunk, cv, bS + kChunk * ch);
        }
        __syncthreads();
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
            f32x4 acc = zero4();
            if (rh != ch || ct <= w) {
#pragma unroll
                for (int j = 0; j < K / 32; ++j) acc = mfma16x32(frag_kc(dwS, pk, 16 * w, 32 * j), frag_kc(kS, pk, 16 * ct, 32 * j), acc);
#pragma unroll
                for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(duS, pv, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), acc);
                const int col = kChunk * ch + 16 * ct + li;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = kChunk * rh + 16 * w + 4 * lg + e;
                    acc[e] = (col < row && row < len) ? acc[e] : 0.f;
                }
            }
            acc_to_tile(m4S, pa, kChunk * rh + 16 * w, kChunk * ch + 16 * ct, acc);
            if (blk == 0) acc_to_tile(m4S, pa, 16 * w, kChunk + 16 * ct, zero4());
        }
    }
    __syncthreads();
    // M5 = M4 A^T: wave w owns row tiles w and w + 4
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
        const int rt = w + 4 * rr;
#pragma unroll
        for (int ct = 0; ct < 8; ++ct) {
            f32x4 acc = zero4();
#pragma unroll
            for (int j = 0; j < 4; ++j) acc = mfma16x32(frag_kc(m4S, pa, 16 * rt, 32 * j), frag_kc(aS, pa, 16 * ct, 32 * j), acc);
            acc_to_tile(m5S, pa, 16 * rt, 16 * ct, acc);
        }
    }
    __syncthreads();
    // (A^T M5)^T = M5^T A, gated, negated and masked; rows of this product are the stored rows
    char *dag = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dA.p)) + b * p.dA.sb + hv * p.dA.sh +
                                         (int64_t)start * p.dA.st);
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
        const int rt = w + 4 * rr;
#pragma unroll
        for (int ct = 0; ct < 8; ++ct) {
            f32x4 acc = zero4();
            if (ct >= rt) {
#pragma unroll
                for (int j = 0; j < 4; ++j) acc = mfma16x32(frag_tr(m5S, pa, 16 * rt, 32 * j), frag_tr(aS, pa, 16 * ct, 32 * j), acc);
                const int col = 16 * ct + li;
                const float gc = gS[col];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = 16 * rt + 4 * lg + e;
                    acc[e] = (col > row && col < len) ? -acc[e] * __expf(fminf(gc - gS[row], 0.f)) : 0.f;
                }
            }
            acc_to_global(dag + 32 * ct, p.dA.st * 2, 16 * rt, len, acc);
        }
    }
}

// prepare_wy_repr_bwd_full on 128-token chunks: one workgroup per chunk and key head.  The 64 output rows of a half
// are produced in one pass: A^T and dA^T need the 64-column slab of A and dA that belongs to those rows (all 128 token
// rows of it), dA (k beta) the 64-row slab of dA; k of the whole chunk stays in LDS, du and dw take turns in one tile.
template <int K, int V>
__global__ void __launch_bounds__(kThreads) wy_bwd_full128_kernel(const WyBwdParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int C = 128, KV = K > V ? K : V;
    constexpr int pk = K + 16, px = KV + 16, pc = kChunk + 8, pa = C + 8, pvv = V;
    constexpr int KT = K / 16, VT = V / 16;
    elem *kS = reinterpret_cast<elem *>(smem);   // [128][pk]
    elem *xS = kS + C * pk;                      // [128][px] du, then dw
    elem *aS = xS + C * px;                      // [128][pc] columns of A for this half's rows
    elem *dS = aS + C * pc;                      // [128][pc] the same columns of dA as stored
    elem *dbS = dS + C * pc;                     // [64][pa] this half's rows of dA, column j scaled by beta_j
    elem *vS = dbS + kChunk * pa;                // [64][V]
    float *gS = reinterpret_cast<float *>(vS + kChunk * pvv);
    float *bS = gS + C;

    int c, hk;
    block_chunk_head(p.geom, c, hk);
    const int b = blockIdx.z;
    const int rep = p.geom.Hv / p.geom.Hk;
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x, w = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    stage_rows<K>(kS, pk, static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st, p.k.st, C, len, nullptr);

    for (int hh = 0; hh < 2; ++hh) {
        const int rlen = min(kChunk, len - kChunk * hh);   // rows of this half
        if (rlen <= 0) break;
        const int rstart = start + kChunk * hh, vcols = rlen;
        f32x4 dk_acc[KT];
#pragma unroll
        for (int ct = 0; ct < KT; ++ct) dk_acc[ct] = zero4();
        for (int r = 0; r < rep; ++r) {
            const int hv = hk * rep + r;
            __syncthreads();   // the previous pass is done with every tile
            if (tid < C) {
                const int t = start + min(tid, len - 1);
                gS[tid] = load_scalar(p.g, b, hv, t);
                bS[tid] = load_scalar(p.beta, b, hv, t);
            }
            __syncthreads();
            const elem *Ag = static_cast<const elem *>(p.A.p) + b * p.A.sb + hv * p.A.sh + (int64_t)start * p.A.st;
            const elem *dAg = static_cast<const elem *>(p.dA.p) + b * p.dA.sb + hv * p.dA.sh + (int64_t)start * p.dA.st;
            stage_rows<kChunk>(aS, pc, Ag + kChunk * hh, p.A.st, C, len, nullptr, nullptr, vcols);
            stage_rows<kChunk>(dS, pc, dAg + kChunk * hh, p.dA.st, C, len, nullptr, nullptr, vcols);
            stage_rows<C>(dbS, pa, dAg + (int64_t)kChunk * hh * p.dA.st, p.dA.st, kChunk, rlen, nullptr, bS, len);
            stage_rows<V>(vS, pvv, static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)rstart * p.v.st, p.v.st,
                          kChunk, rlen, nullptr);
            stage_rows<V>(xS, px, static_cast<const elem *>(p.du.p) + b * p.du.sb + hv * p.du.sh + (int64_t)start * p.du.st, p.du.st,
                          C, len, nullptr);
            __syncthreads();
            float br[4], er[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                br[e] = bS[kChunk * hh + 16 * w + 4 * lg + e];
                er[e] = __expf(gS[kChunk * hh + 16 * w + 4 * lg + e]);
            }
            float db_row[4] = {0.f, 0.f, 0.f, 0.f}, dg_row[4] = {0.f, 0.f, 0.f, 0.f};
            elemx8 at[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) at[j] = frag_tr(aS, pc, 16 * w, 32 * j);
            char *dvg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dv.p)) + b * p.dv.sb + hv * p.dv.sh +
                                                 (int64_t)rstart * p.dv.st);
#pragma unroll
            for (int ct = 0; ct < VT; ++ct) {      // A^T du
                f32x4 acc = zero4();
#pragma unroll
                for (int j = 0; j < 4; ++j) acc = mfma16x32(at[j], frag_tr(xS, px, 16 * ct, 32 * j), acc);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    db_row[e] += acc[e] * (float)vS[(16 * w + 4 * lg + e) * pvv + 16 * ct + li];
                    acc[e] *= br[e];
                }
                acc_to_global(dvg + 32 * ct, p.dv.st * 2, 16 * w, rlen, acc);
            }
            __syncthreads();                 // du has been consumed by every wave
            stage_rows<K>(xS, px, static_cast<const elem *>(p.dw.p) + b * p.dw.sb + hv * p.dw.sh + (int64_t)start * p.dw.st, p.dw.st,
                          C, len, nullptr);
            __syncthreads();
            elemx8 dt[4], db[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                dt[j] = frag_tr(dS, pc, 16 * w, 32 * j);
                db[j] = frag_kc(dbS, pa, 16 * w, 32 * j);
            }
#pragma unroll
            for (int ct = 0; ct < KT; ++ct) {
                f32x4 p1 = zero4(), p2 = zero4(), q3 = zero4();
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const elemx8 kf = frag_tr(kS, pk, 16 * ct, 32 * j);
                    p1 = mfma16x32(at[j], frag_tr(xS, px, 16 * ct, 32 * j), p1);   // A^T dw
                    p2 = mfma16x32(dt[j], kf, p2);                                  // dA^T k
                    q3 = mfma16x32(db[j], kf, q3);                                  // dA (k beta)
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float kv = (float)kS[(kChunk * hh + 16 * w + 4 * lg + e) * pk + 16 * ct + li];
                    const float p1g = p1[e] * er[e];
                    dk_acc[ct][e] += q3[e] + (p2[e] + p1g) * br[e];
                    db_row[e] += (p2[e] + p1g) * kv;
                    dg_row[e] += (p1g * br[e] + br[e] * p2[e] - q3[e]) * kv;
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float sb = group_sum<16>(db_row[e]), sg = group_sum<16>(dg_row[e]);
                const int row = 16 * w + 4 * lg + e;
                if (li == 0 && row < rlen) {
                    p.dbeta[b * p.db_sb + hv * p.db_sh + (int64_t)(rstart + row) * p.db_st] = sb;
                    p.dg[b * p.dg_sb + hv * p.dg_sh + (int64_t)(rstart + row) * p.dg_st] = sg;
                }
            }
        }
        char *dkg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dk.p)) + b * p.dk.sb + hk * p.dk.sh +
                                             (int64_t)rstart * p.dk.st);
#pragma unroll
        for (int ct = 0; ct < KT; ++ct) acc_to_global(dkg + 32 * ct, p.dk.st * 2, 16 * w, rlen, dk_acc[ct]);
    }
}

// ---- host side ------------------------------------------------------------------------------------
#define FLA_BWD_DISPATCH_T(KERNEL, NAME, GRID, SMEM_EXPR, P, THREADS)                                                   \
    do {                                                                                                               \
        const size_t smem__ = (SMEM_EXPR);                                                                             \
        FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(KERNEL), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                          (int)smem__));                                                               \
        FLA_LAUNCH(NAME, stream, KERNEL, GRID, dim3(THREADS), smem__, stream, P);                                       \
        FLA_HIP_CHECK(hipGetLastError());                                                                              \
        return FLA_OK;                                                                                                 \
    } while (0)
#define FLA_BWD_DISPATCH(KERNEL, NAME, GRID, SMEM_EXPR, P) FLA_BWD_DISPATCH_T(KERNEL, NAME, GRID, SMEM_EXPR, P, kThreads)

int check_f32_bht(const char *op, const char *name, const fla_tensor *t, const ChunkGeom &g) {
    int rc = check_tensor(t, op, name, 3, dt_bit(FLA_F32));
    if (rc) return rc;
    FLA_REQUIRE(t->shape[0] == g.B && t->shape[1] == g.Hv && t->shape[2] == g.T, FLA_ERR_SHAPE,
                "%s: %s must be [%d,%d,%d].", op, name, g.B, g.Hv, g.T);
    return FLA_OK;
}

int check_state5(const char *op, const char *name, const fla_tensor *h, const ChunkGeom &geom) {
    int rc = check_tensor(h, op, name, 5, dt_bit(kElemDtype));
    if (rc) return rc;
    FLA_REQUIRE(h->shape[0] == geom.B && h->shape[1] == geom.Hv && h->shape[2] == geom.NT && h->shape[3] == geom.K &&
                    h->shape[4] == geom.V && h->stride[4] == 1 && h->stride[3] >= geom.V && h->stride[3] % 8 == 0 &&
                    h->stride[3] < (1 << 16) && h->stride[2] % 8 == 0 && h->stride[1] % 8 == 0 && h->stride[0] % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(h->data) % 16 == 0,
                FLA_ERR_SHAPE, "%s: %s must be [B,Hv,NT=%d,K,V] with K x V blocks of 16-byte aligned rows.", op, name, geom.NT);
    return FLA_OK;
}

// ---- 128-token chunks with 256 value columns --------------------------------------------------------------------
// The 128-token kernels of chunk_bwd_dqkwg and of the two WY backward operators hold 128 value columns.  With 256 the
// launcher runs them twice, over 128 columns each: every result is either a per-column one (dv) or a sum over the value
// columns that is linear in the column-wise operands, so the second pass (which sees zeros for the operands that do not
// belong to the value dimension) lands in the workspace and is added to the first.  Each pass rounds its part to the
// element type, so a sum carries one more rounding than a single pass would, at the magnitude of the parts.
inline bool two_value_slabs(int64_t chunk_size, const fla_tensor *v) {
    return chunk_size == 128 && v != nullptr && v->ndim == 4 && v->shape[3] == 256;
}
inline size_t dtype_bytes(int dtype) { return dtype == FLA_F32 || dtype == FLA_I32 ? 4 : dtype == FLA_I64 ? 8 : 2; }
// columns [lo, lo + n) of the innermost dimension, as a view
inline fla_tensor column_slab(const fla_tensor *t, int64_t lo, int64_t n) {
    fla_tensor s = *t;
    s.shape[t->ndim - 1] = n;
    s.data = static_cast<char *>(t->data) + lo * t->stride[t->ndim - 1] * (int64_t)dtype_bytes(t->dtype);
    return s;
}
// a contiguous tensor shaped like `like` except for its innermost extent and dtype, at `data`
inline fla_tensor dense_like(const fla_tensor *like, int64_t inner, int dtype, void *data) {
    fla_tensor s = *like;
    s.dtype = dtype;
    s.data = data;
    if (inner > 0) s.shape[s.ndim - 1] = inner;
    int64_t st = 1;
    for (int d = s.ndim - 1; d >= 0; --d) {
        s.stride[d] = st;
        st *= s.shape[d];
    }
    return s;
}
inline uint64_t dense_bytes(const fla_tensor &t) {
    uint64_t n = dtype_bytes(t.dtype);
    for (int d = 0; d < t.ndim; ++d) n *= (uint64_t)t.shape[d];
    return (n + 255) & ~(uint64_t)255;
}

// out[b,h,t,:] = round(out + part) for a strided [B,H,T,D] element tensor and a contiguous part (D a multiple of 8)
__global__ void __launch_bounds__(256) add_part_kernel(View4 out, const elem *part, int H, int T, int D, int64_t rows) {
    const int per = D / 8;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < rows * per; i += (int64_t)gridDim.x * 256) {
        const int64_t row = i / per;
        const int c8 = (int)(i % per) * 8;
        const int t = (int)(row % T), h = (int)((row / T) % H);
        const int64_t b = row / ((int64_t)T * H);
        elem *o = static_cast<elem *>(const_cast<void *>(out.p)) + b * out.sb + h * out.sh + (int64_t)t * out.st + c8;
        const elemx8 a = *reinterpret_cast<const elemx8 *>(o), c = *reinterpret_cast<const elemx8 *>(part + row * D + c8);
        f32x4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo[e] = (float)a[e] + (float)c[e];
            hi[e] = (float)a[4 + e] + (float)c[4 + e];
        }
        *reinterpret_cast<elemx8 *>(o) = frag_from_acc(lo, hi);
    }
}
// out[b,h,t] += part for a strided fp32 [B,H,T] tensor and a contiguous part
__global__ void __launch_bounds__(256) add_scalars_kernel(float *out, int64_t sb, int64_t sh, int64_t st, const float *part, int H,
                                                          int T, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int t = (int)(i % T), h = (int)((i / T) % H);
        const int64_t b = i / ((int64_t)T * H);
        out[b * sb + h * sh + (int64_t)t * st] += part[i];
    }
}
__global__ void __launch_bounds__(256) zero_fill_kernel(u32x4 *dst, int64_t n16) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) dst[i] = u32x4{0u, 0u, 0u, 0u};
}
int add_part(const fla_tensor *out, const fla_tensor &part, hipStream_t stream) {
    const int64_t rows = out->shape[0] * out->shape[1] * out->shape[2];
    if (rows == 0) return FLA_OK;
    const unsigned blocks = (unsigned)std::min<int64_t>((rows * (out->shape[3] / 8) + 255) / 256, 8192);
    FLA_LAUNCH("add_part", stream, add_part_kernel, dim3(blocks), dim3(256), 0, stream, view4(out), static_cast<const elem *>(part.data),
               (int)out->shape[1], (int)out->shape[2], (int)out->shape[3], rows);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}
int add_scalars(const fla_tensor *out, const fla_tensor &part, hipStream_t stream) {
    const int64_t n = out->shape[0] * out->shape[1] * out->shape[2];
    if (n == 0) return FLA_OK;
    const unsigned blocks = (unsigned)std::min<int64_t>((n + 255) / 256, 4096);
    FLA_LAUNCH("add_scalars", stream, add_scalars_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<float *>(out->data), out->stride[0],
               out->stride[1], out->stride[2], static_cast<const float *>(part.data), (int)out->shape[1], (int)out->shape[2], n);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}
int zero_fill(void *dst, uint64_t bytes, hipStream_t stream) {   // bytes: a multiple of 256
    if (bytes == 0) return FLA_OK;
    const int64_t n16 = (int64_t)(bytes / 16);
    const unsigned blocks = (unsigned)std::min<int64_t>((n16 + 255) / 256, 8192);
    FLA_LAUNCH("zero_fill", stream, zero_fill_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<u32x4 *>(dst), n16);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}
// hands out 256-byte aligned pieces of the workspace behind the first `used` bytes
struct Carver {
    char *base;
    uint64_t used;
    void *take(uint64_t bytes) {
        void *ptr = base ? base + used : reinterpret_cast<void *>(uintptr_t(256));   // size queries get a non-null stand-in
        used += bytes;
        return ptr;
    }
};

int dv_local_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *d_o, const fla_tensor *g,
                  const fla_tensor *g_gamma, const fla_tensor *A, const fla_int_array *cu, const fla_int_array *ci,
                  double scale, int64_t chunk_size, const fla_tensor *out, void *ws, uint64_t ws_size, hipStream_t stream,
                  uint64_t *query) {
    const char *op = "chunk_bwd_dv_local";
    FLA_REQUIRE(g_gamma == nullptr || g_gamma->data == nullptr, FLA_ERR_UNSUPPORTED, "%s: g_gamma is not supported.", op);
    (void)A;   // accepted and unused, as in the reference kernel
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, d_o, nullptr, chunk_size, geom, kElemDtype, 128))) return rc;   // chunk_bwd_dv_local/README.md:114
    const int bf = dt_bit(kElemDtype);
    if ((rc = check_bhtd(op, "q", q, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "d_o", d_o, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bhtd(op, "out", out, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    FLA_REQUIRE(g != nullptr && g->data != nullptr, FLA_ERR_NULL, "%s: g must be provided.", op);
    if ((rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    DvLocalParams p{geom, view4(q), view4(k), view4(d_o), view4(out), view3(g), (float)scale};
    const bool c128 = geom.C == 128;
    const dim3 grid = chunk_head_grid(geom, geom.NT * (c128 ? 2 : 1), geom.Hv);
    const int K = geom.K, V = geom.V;
    const size_t smem = ((size_t)kChunk * (2 * (K + 8) + (V + 16) + kChunk + 8)) * 2 + 2 * kChunk * 4;
#define FLA_DV_LOCAL(KK, VV)                                                                                \
    do {                                                                                                    \
        if (c128) FLA_BWD_DISPATCH((dv_local_kernel<KK, VV, true>), "bwd_dv_local", grid, smem, p);         \
        FLA_BWD_DISPATCH((dv_local_kernel<KK, VV, false>), "bwd_dv_local", grid, smem, p);                  \
    } while (0)
    if (K == 128 && V == 128) FLA_DV_LOCAL(128, 128);
    if (K == 64 && V == 64) FLA_DV_LOCAL(64, 64);
    if (K == 64 && V == 128) FLA_DV_LOCAL(64, 128);
    if (K == 128 && V == 256) FLA_DV_LOCAL(128, 256);
#undef FLA_DV_LOCAL
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel; built: (128,128),(64,64),(64,128),(128,256).", op, K, V);
}

// rstd of an l2norm_fwd over [B,H,T,K]: contiguous fp32 [B,H,T]; null / no data = absent
int check_rstd(const char *op, const char *name, const fla_tensor *t, int64_t B, int64_t H, int64_t T, bool &present) {
    present = t != nullptr && t->data != nullptr;
    if (!present) return FLA_OK;
    int rc = check_tensor(t, op, name, 3, dt_bit(FLA_F32));
    if (rc) return rc;
    FLA_REQUIRE(t->shape[0] == B && t->shape[1] == H && t->shape[2] == T && is_contiguous(t), FLA_ERR_SHAPE,
                "%s: %s must be contiguous fp32 [%lld,%lld,%lld].", op, name, (long long)B, (long long)H, (long long)T);
    return FLA_OK;
}

int dqkwg_two_slabs(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
                    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu,
                    const fla_int_array *ci, float scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
                    const fla_tensor *dw, const fla_tensor *dg, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query);
int wy_bwd_da_two_slabs(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
                        const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu, const fla_int_array *ci,
                        int64_t chunk_size, const fla_tensor *dA, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query);
int wy_bwd_full_two_slabs(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
                          const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu,
                          const fla_int_array *ci, int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv,
                          const fla_tensor *dbeta, const fla_tensor *dg, void *ws, uint64_t ws_size, hipStream_t stream,
                          uint64_t *query);

int dqkwg_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
               const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu,
               const fla_int_array *ci, const fla_tensor *w, const fla_tensor *g_gamma, float scale, int64_t chunk_size,
               bool use_exp2, bool transpose_state_layout, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dw,
               const fla_tensor *dg, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query,
               const fla_tensor *q_rstd = nullptr) {
    const char *op = q_rstd ? "chunk_bwd_dqkwg_l2norm" : "chunk_bwd_dqkwg";
    FLA_REQUIRE(g_gamma == nullptr || g_gamma->data == nullptr, FLA_ERR_UNSUPPORTED, "%s: g_gamma is not supported.", op);
    FLA_REQUIRE(!use_exp2, FLA_ERR_UNSUPPORTED, "%s: use_exp2 is not supported with a scalar gate.", op);
    FLA_REQUIRE(!transpose_state_layout, FLA_ERR_UNSUPPORTED, "%s: transpose_state_layout is not supported.", op);
    (void)w;   // the reference accepts w and does not read it
    if (two_value_slabs(chunk_size, v) && !q_rstd)
        return dqkwg_two_slabs(q, k, v, g, h, d_o, dh, dv, cu, ci, scale, chunk_size, dq, dk, dw, dg, ws, ws_size, stream, query);
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v, nullptr, chunk_size, geom, kElemDtype, 128))) return rc;   // chunk_bwd_dqkwg/README.md:117
    const int bf = dt_bit(kElemDtype);
    if ((rc = check_bhtd(op, "q", q, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bhtd(op, "dox", d_o, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bhtd(op, "dv", dv, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bhtd(op, "dq", dq, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "dk", dk, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "dw", dw, geom.B, geom.Hv, geom.T, geom.K, bf))) return rc;
    FLA_REQUIRE(g != nullptr && g->data != nullptr, FLA_ERR_NULL, "%s: g must be provided.", op);
    if ((rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    if ((rc = check_f32_bht(op, "dg", dg, geom))) return rc;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query))) return rc;
    if ((rc = check_state5(op, "h", h, geom))) return rc;
    if ((rc = check_state5(op, "dh", dh, geom))) return rc;
    if (query) return FLA_OK;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    DqkwgParams p{geom, view4(q), view4(k), view4(v), view4(d_o), view4(dv), view4(dq), view4(dk), view4(dw), view3(g),
                  static_cast<const elem *>(h->data), static_cast<const elem *>(dh->data),
                  h->stride[0], h->stride[1], h->stride[2], dh->stride[0], dh->stride[1], dh->stride[2],
                  static_cast<float *>(dg->data), dg->stride[0], dg->stride[1], dg->stride[2], scale};
    p.h_row = (int)h->stride[3];
    p.dh_row = (int)dh->stride[3];
    bool has_rstd;
    if ((rc = check_rstd(op, "q_rstd", q_rstd, geom.B, geom.Hk, geom.T, has_rstd))) return rc;
    if (has_rstd) {
        p.q_rstd = static_cast<const float *>(q_rstd->data);
        p.r_sb = q_rstd->stride[0];
        p.r_sh = q_rstd->stride[1];
    }
    // token-major operands (the row of a token holds all heads): neighbouring workgroups take the heads of one chunk
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hk);
    const int K = geom.K, V = geom.V;
    const int VS = V == 256 ? 128 : V;   // value columns held in LDS at a time
    const size_t smem = ((size_t)kChunk * (2 * (K + 16) + 3 * (VS + 8) + kChunk + 8) + (size_t)K * (VS + 8)) * 2 +
                        (kChunk + 16 + 2 * kChunk + kChunk + kMaxRep) * 4;
    const bool gva = geom.Hv != geom.Hk;
    if (has_rstd) {   // dq de-normalised in the kernel: 64-token chunks
        FLA_REQUIRE(geom.C == kChunk, FLA_ERR_UNSUPPORTED, "%s: built for chunk_size 64.", op);
        if (K == 128 && V == 256) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, true, 2, 1, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        if (K == 128 && V == 128 && !gva) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, false, 1, 1, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        if (K == 128 && V == 128) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, true, 1, 1, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        if (K == 64 && V == 64) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 64, true, 1, 1, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        if (K == 64 && V == 128) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 128, true, 1, 1, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel; built: (128,128),(64,64),(64,128),(128,256).", op, K, V);
    }
    if (geom.C == 128) {   // one workgroup per chunk, its two halves in turn
        FLA_REQUIRE(geom.Hv / geom.Hk <= kMaxRep, FLA_ERR_UNSUPPORTED, "%s: at most %d value heads per key head with chunk_size 128.", op, kMaxRep);
        if (K == 128 && V == 128 && !gva) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, false, 1, 2>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        if (K == 128 && V == 128) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, true, 1, 2>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        if (K == 64 && V == 64) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 64, true, 1, 2>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        if (K == 64 && V == 128) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 128, true, 1, 2>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
        return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel for chunk_size 128; built: (128,128),(64,64),(64,128).", op, K, V);
    }
    if (K == 128 && V == 256) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, true, 2>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 128 && V == 128 && !gva) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, false>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 128 && V == 128) FLA_BWD_DISPATCH_T((dqkwg_kernel<128, 128, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 64 && V == 64 && !gva) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 64, false>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 64 && V == 64) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 64, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 64 && V == 128 && !gva) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 128, false>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 64 && V == 128) FLA_BWD_DISPATCH_T((dqkwg_kernel<64, 128, true>), "bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel; built: (128,128),(64,64),(64,128),(128,256).", op, K, V);
}

int wy_bwd_common(const char *op, const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A,
                  const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, int64_t chunk_size, ChunkGeom &geom) {
    int rc;
    if ((rc = gdn_geometry(op, k, v, nullptr, chunk_size, geom, kElemDtype, 128))) return rc;   // prepare_wy_repr_bwd_full/README.md:74
    const int bf = dt_bit(kElemDtype);
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if (A != nullptr && (rc = check_bhtd(op, "A", A, geom.B, geom.Hv, geom.T, geom.C, bf))) return rc;   // null: the caller has checked that the kernel can do without
    if ((rc = check_bhtd(op, "dw", dw, geom.B, geom.Hv, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "du", du, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    FLA_REQUIRE(g != nullptr && g->data != nullptr && beta != nullptr && beta->data != nullptr, FLA_ERR_NULL,
                "%s: g and beta must be provided.", op);
    if ((rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    if ((rc = check_bht(op, "beta", beta, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    return FLA_OK;
}

int wy_bwd_da_impl(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A,
                   const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu,
                   const fla_int_array *ci, int64_t chunk_size, const fla_tensor *dA, void *ws, uint64_t ws_size,
                   hipStream_t stream, uint64_t *query) {
    const char *op = "prepare_wy_repr_bwd_da";
    ChunkGeom geom;
    int rc;
    FLA_REQUIRE(A != nullptr && A->data != nullptr, FLA_ERR_NULL, "%s: A must not be null.", op);
    if (two_value_slabs(chunk_size, v)) return wy_bwd_da_two_slabs(k, v, beta, A, dw, du, g, cu, ci, chunk_size, dA, ws, ws_size, stream, query);
    if ((rc = wy_bwd_common(op, k, v, beta, A, dw, du, g, chunk_size, geom))) return rc;
    if ((rc = check_bhtd(op, "dA", dA, geom.B, geom.Hv, geom.T, geom.C, dt_bit(kElemDtype)))) return rc;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    WyBwdParams p{geom, view4(k), view4(v), view4(A), view4(dA), view4(dw), view4(du), View4{}, View4{}, view3(g),
                  view3(beta), nullptr, nullptr, 0, 0, 0, 0, 0, 0};
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hv);
    const int K = geom.K, V = geom.V;
    if (geom.C == 128) {
        const size_t smem128 = ((size_t)kChunk * (2 * (K + 8) + 2 * (V + 8)) + (size_t)2 * 128 * (128 + 8)) * 2 + 3 * 128 * 4;
        if (K == 128 && V == 128) FLA_BWD_DISPATCH((wy_bwd_da128_kernel<128, 128>), "wy_bwd_da", grid, smem128, p);
        if (K == 64 && V == 64) FLA_BWD_DISPATCH((wy_bwd_da128_kernel<64, 64>), "wy_bwd_da", grid, smem128, p);
        if (K == 64 && V == 128) FLA_BWD_DISPATCH((wy_bwd_da128_kernel<64, 128>), "wy_bwd_da", grid, smem128, p);
        return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel for chunk_size 128; built: (128,128),(64,64),(64,128).", op, K, V);
    }
    const size_t smem = ((size_t)kChunk * (2 * (K + 8) + 2 * (V + 8) + (kChunk + 8))) * 2 + 3 * kChunk * 4;
    if (K == 128 && V == 128) FLA_BWD_DISPATCH((wy_bwd_da_kernel<128, 128>), "wy_bwd_da", grid, smem, p);
    if (K == 64 && V == 64) FLA_BWD_DISPATCH((wy_bwd_da_kernel<64, 64>), "wy_bwd_da", grid, smem, p);
    if (K == 64 && V == 128) FLA_BWD_DISPATCH((wy_bwd_da_kernel<64, 128>), "wy_bwd_da", grid, smem, p);
    if (K == 128 && V == 256) FLA_BWD_DISPATCH((wy_bwd_da_kernel<128, 256>), "wy_bwd_da", grid, smem, p);
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel; built: (128,128),(64,64),(64,128),(128,256).", op, K, V);
}

int wy_bwd_full_impl(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A,
                     const fla_tensor *dA, const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g,
                     const fla_int_array *cu, const fla_int_array *ci, int64_t chunk_size, const fla_tensor *dk,
                     const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg, void *ws, uint64_t ws_size,
                     hipStream_t stream, uint64_t *query, bool accumulate = false, const fla_tensor *k_rstd = nullptr) {
    const char *op = accumulate ? "prepare_wy_repr_bwd_full_accumulate" : "prepare_wy_repr_bwd_full";
    ChunkGeom geom;
    int rc;
    // A absent (only together with dA, below): the kernel rebuilds the chunk's inverse from k, g and beta
    const bool has_a = A && A->data;
    FLA_REQUIRE(has_a || !(dA && dA->data), FLA_ERR_NULL, "%s: A must not be null when dA is given.", op);
    if (two_value_slabs(chunk_size, v) && !accumulate)
        return wy_bwd_full_two_slabs(k, v, beta, A, dA, dw, du, g, cu, ci, chunk_size, dk, dv, dbeta, dg, ws, ws_size, stream, query);
    if ((rc = wy_bwd_common(op, k, v, beta, has_a ? A : nullptr, dw, du, g, chunk_size, geom))) return rc;
    const int bf = dt_bit(kElemDtype);
    // dA absent (the accumulating form on 64-token chunks only): the kernel forms prepare_wy_repr_bwd_da's result itself
    const bool has_da = dA && dA->data;
    FLA_REQUIRE(has_da || (accumulate && geom.C == kChunk), FLA_ERR_NULL, "%s: dA must not be null.", op);
    if (has_da && (rc = check_bhtd(op, "dA", dA, geom.B, geom.Hv, geom.T, geom.C, bf))) return rc;
    if ((rc = check_bhtd(op, "dk", dk, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "dv", dv, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_f32_bht(op, "dbeta", dbeta, geom))) return rc;
    if ((rc = check_f32_bht(op, "dg", dg, geom))) return rc;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    WyBwdParams p{geom, view4(k), view4(v), has_a ? view4(A) : View4{nullptr, 0, 0, 0}, has_da ? view4(dA) : View4{nullptr, 0, 0, 0}, view4(dw), view4(du), view4(dk), view4(dv), view3(g),
                  view3(beta), static_cast<float *>(dbeta->data), static_cast<float *>(dg->data),
                  dbeta->stride[0], dbeta->stride[1], dbeta->stride[2], dg->stride[0], dg->stride[1], dg->stride[2]};
    bool has_rstd;
    if ((rc = check_rstd(op, "k_rstd", k_rstd, geom.B, geom.Hk, geom.T, has_rstd))) return rc;
    if (has_rstd) {
        p.k_rstd = static_cast<const float *>(k_rstd->data);
        p.r_sb = k_rstd->stride[0];
        p.r_sh = k_rstd->stride[1];
    }
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hk);
    const int K = geom.K, V = geom.V;
    if (geom.C == 128) {
        FLA_REQUIRE(!accumulate, FLA_ERR_UNSUPPORTED, "%s: the accumulating form is built for chunk_size 64.", op);
        const int KV = K > V ? K : V;
        const size_t smem128 = ((size_t)128 * ((K + 16) + (KV + 16) + 2 * (kChunk + 8)) + (size_t)kChunk * (128 + 8 + V)) * 2 + 2 * 128 * 4;
        if (K == 128 && V == 128) FLA_BWD_DISPATCH((wy_bwd_full128_kernel<128, 128>), "wy_bwd_full", grid, smem128, p);
        if (K == 64 && V == 64) FLA_BWD_DISPATCH((wy_bwd_full128_kernel<64, 64>), "wy_bwd_full", grid, smem128, p);
        if (K == 64 && V == 128) FLA_BWD_DISPATCH((wy_bwd_full128_kernel<64, 128>), "wy_bwd_full", grid, smem128, p);
        return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel for chunk_size 128; built: (128,128),(64,64),(64,128).", op, K, V);
    }
    const size_t smem = ((size_t)kChunk * ((K + 16) + ((K > V ? K : V) + 16) + V + 3 * (kChunk + 8))) * 2 + 2 * kChunk * 4;
    const bool gva = geom.Hv != geom.Hk;
#define FLA_WY_FULL(KK, VV, G)                                                                                      \
    do {                                                                                                            \
        if (accumulate && !has_da && !has_a) FLA_BWD_DISPATCH((wy_bwd_full_kernel<KK, VV, G, true, true, true>), "wy_bwd_full", grid, smem, p); \
        if (accumulate && !has_da) FLA_BWD_DISPATCH((wy_bwd_full_kernel<KK, VV, G, true, true>), "wy_bwd_full", grid, smem, p); \
        if (accumulate) FLA_BWD_DISPATCH((wy_bwd_full_kernel<KK, VV, G, true>), "wy_bwd_full", grid, smem, p);      \
        FLA_BWD_DISPATCH((wy_bwd_full_kernel<KK, VV, G, false>), "wy_bwd_full", grid, smem, p);                     \
    } while (0)
    if (K == 128 && V == 128 && !gva) FLA_WY_FULL(128, 128, false);
    if (K == 128 && V == 128) FLA_WY_FULL(128, 128, true);
    if (K == 64 && V == 64 && !gva) FLA_WY_FULL(64, 64, false);
    if (K == 64 && V == 64) FLA_WY_FULL(64, 64, true);
    if (K == 64 && V == 128 && !gva) FLA_WY_FULL(64, 128, false);
    if (K == 64 && V == 128) FLA_WY_FULL(64, 128, true);
    if (K == 128 && V == 256) FLA_WY_FULL(128, 256, true);
#undef FLA_WY_FULL
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel; built: (128,128),(64,64),(64,128),(128,256).", op, K, V);
}

int dqkwg_two_slabs(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
                    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu,
                    const fla_int_array *ci, float scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
                    const fla_tensor *dw, const fla_tensor *dg, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_bwd_dqkwg";
    const fla_tensor *need[] = {q, k, v, g, h, d_o, dh, dv, dq, dk, dw, dg};
    for (const fla_tensor *t : need) FLA_REQUIRE(t != nullptr && t->data != nullptr, FLA_ERR_NULL, "%s: an operand is null.", op);
    FLA_REQUIRE(d_o->ndim == 4 && dv->ndim == 4 && h->ndim == 5 && dh->ndim == 5 && d_o->shape[3] == 256 && dv->shape[3] == 256 &&
                    h->shape[4] == 256 && dh->shape[4] == 256 && dq->ndim == 4 && dk->ndim == 4 && dw->ndim == 4 && dg->ndim == 3,
                FLA_ERR_SHAPE, "%s: dox, dv, h and dh must carry the 256 value columns of v.", op);
    int rc;
    fla_tensor vs[2], os[2], dvs[2], hs[2], dhs[2];
    for (int i = 0; i < 2; ++i) {
        vs[i] = column_slab(v, 128 * i, 128);
        os[i] = column_slab(d_o, 128 * i, 128);
        dvs[i] = column_slab(dv, 128 * i, 128);
        hs[i] = column_slab(h, 128 * i, 128);
        dhs[i] = column_slab(dh, 128 * i, 128);
    }
    uint64_t meta = 0;
    if ((rc = dqkwg_impl(q, k, &vs[0], g, &hs[0], &os[0], &dhs[0], &dvs[0], cu, ci, nullptr, nullptr, scale, chunk_size, false, false,
                         dq, dk, dw, dg, nullptr, 0, nullptr, &meta)))
        return rc;
    Carver carve{static_cast<char *>(query ? nullptr : ws), (meta + 255) & ~(uint64_t)255};
    fla_tensor dq2 = dense_like(dq, 0, dq->dtype, nullptr), dk2 = dense_like(dk, 0, dk->dtype, nullptr),
               dw2 = dense_like(dw, 0, dw->dtype, nullptr), dg2 = dense_like(dg, 0, FLA_F32, nullptr);
    dq2.data = carve.take(dense_bytes(dq2));
    dk2.data = carve.take(dense_bytes(dk2));
    dw2.data = carve.take(dense_bytes(dw2));
    dg2.data = carve.take(dense_bytes(dg2));
    if (query) {
        *query = carve.used;
        return FLA_OK;
    }
    FLA_REQUIRE(ws && ws_size >= carve.used, FLA_ERR_WORKSPACE, "%s: workspace of %llu bytes required.", op, (unsigned long long)carve.used);
    if ((rc = dqkwg_impl(q, k, &vs[0], g, &hs[0], &os[0], &dhs[0], &dvs[0], cu, ci, nullptr, nullptr, scale, chunk_size, false, false, dq, dk,
                         dw, dg, ws, meta, stream, nullptr)))
        return rc;
    if ((rc = dqkwg_impl(q, k, &vs[1], g, &hs[1], &os[1], &dhs[1], &dvs[1], cu, ci, nullptr, nullptr, scale, chunk_size, false, false, &dq2,
                         &dk2, &dw2, &dg2, ws, meta, stream, nullptr)))
        return rc;
    if ((rc = add_part(dq, dq2, stream)) || (rc = add_part(dk, dk2, stream)) || (rc = add_part(dw, dw2, stream))) return rc;
    return add_scalars(dg, dg2, stream);
}

int wy_bwd_da_two_slabs(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
                        const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu, const fla_int_array *ci,
                        int64_t chunk_size, const fla_tensor *dA, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "prepare_wy_repr_bwd_da";
    const fla_tensor *need[] = {k, v, beta, A, dw, du, g, dA};
    for (const fla_tensor *t : need) FLA_REQUIRE(t != nullptr && t->data != nullptr, FLA_ERR_NULL, "%s: an operand is null.", op);
    FLA_REQUIRE(du->ndim == 4 && du->shape[3] == 256 && dw->ndim == 4 && dA->ndim == 4, FLA_ERR_SHAPE,
                "%s: du must carry the 256 value columns of v.", op);
    int rc;
    fla_tensor vs[2] = {column_slab(v, 0, 128), column_slab(v, 128, 128)}, dus[2] = {column_slab(du, 0, 128), column_slab(du, 128, 128)};
    uint64_t meta = 0;
    if ((rc = wy_bwd_da_impl(k, &vs[0], beta, A, dw, &dus[0], g, cu, ci, chunk_size, dA, nullptr, 0, nullptr, &meta))) return rc;
    Carver carve{static_cast<char *>(query ? nullptr : ws), (meta + 255) & ~(uint64_t)255};
    fla_tensor zero_dw = dense_like(dw, 0, dw->dtype, nullptr), part = dense_like(dA, 0, dA->dtype, nullptr);
    const uint64_t zero_bytes = dense_bytes(zero_dw);
    zero_dw.data = carve.take(zero_bytes);
    part.data = carve.take(dense_bytes(part));
    if (query) {
        *query = carve.used;
        return FLA_OK;
    }
    FLA_REQUIRE(ws && ws_size >= carve.used, FLA_ERR_WORKSPACE, "%s: workspace of %llu bytes required.", op, (unsigned long long)carve.used);
    if ((rc = zero_fill(zero_dw.data, zero_bytes, stream))) return rc;
    if ((rc = wy_bwd_da_impl(k, &vs[0], beta, A, dw, &dus[0], g, cu, ci, chunk_size, dA, ws, meta, stream, nullptr))) return rc;
    if ((rc = wy_bwd_da_impl(k, &vs[1], beta, A, &zero_dw, &dus[1], g, cu, ci, chunk_size, &part, ws, meta, stream, nullptr))) return rc;
    return add_part(dA, part, stream);
}

int wy_bwd_full_two_slabs(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
                          const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu,
                          const fla_int_array *ci, int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv,
                          const fla_tensor *dbeta, const fla_tensor *dg, void *ws, uint64_t ws_size, hipStream_t stream,
                          uint64_t *query) {
    const char *op = "prepare_wy_repr_bwd_full";
    const fla_tensor *need[] = {k, v, beta, A, dA, dw, du, g, dk, dv, dbeta, dg};
    for (const fla_tensor *t : need) FLA_REQUIRE(t != nullptr && t->data != nullptr, FLA_ERR_NULL, "%s: an operand is null.", op);
    FLA_REQUIRE(du->ndim == 4 && du->shape[3] == 256 && dv->ndim == 4 && dv->shape[3] == 256 && dw->ndim == 4 && dA->ndim == 4 &&
                    dk->ndim == 4 && dbeta->ndim == 3 && dg->ndim == 3,
                FLA_ERR_SHAPE, "%s: du and dv must carry the 256 value columns of v.", op);
    int rc;
    fla_tensor vs[2], dus[2], dvs[2];
    for (int i = 0; i < 2; ++i) {
        vs[i] = column_slab(v, 128 * i, 128);
        dus[i] = column_slab(du, 128 * i, 128);
        dvs[i] = column_slab(dv, 128 * i, 128);
    }
    uint64_t meta = 0;
    if ((rc = wy_bwd_full_impl(k, &vs[0], beta, A, dA, dw, &dus[0], g, cu, ci, chunk_size, dk, &dvs[0], dbeta, dg, nullptr, 0, nullptr, &meta)))
        return rc;
    Carver carve{static_cast<char *>(query ? nullptr : ws), (meta + 255) & ~(uint64_t)255};
    // the second pass reads zeros for dA and dw (one zeroed piece serves both) and drops its dk and dg
    fla_tensor zero_dw = dense_like(dw, 0, dw->dtype, nullptr), zero_da = dense_like(dA, 0, dA->dtype, nullptr);
    const uint64_t zero_bytes = std::max(dense_bytes(zero_dw), dense_bytes(zero_da));
    zero_dw.data = zero_da.data = carve.take(zero_bytes);
    fla_tensor dk2 = dense_like(dk, 0, dk->dtype, nullptr), db2 = dense_like(dbeta, 0, FLA_F32, nullptr), dg2 = dense_like(dg, 0, FLA_F32, nullptr);
    dk2.data = carve.take(dense_bytes(dk2));
    db2.data = carve.take(dense_bytes(db2));
    dg2.data = carve.take(dense_bytes(dg2));
    if (query) {
        *query = carve.used;
        return FLA_OK;
    }
    FLA_REQUIRE(ws && ws_size >= carve.used, FLA_ERR_WORKSPACE, "%s: workspace of %llu bytes required.", op, (unsigned long long)carve.used);
    if ((rc = zero_fill(zero_dw.data, zero_bytes, stream))) return rc;
    if ((rc = wy_bwd_full_impl(k, &vs[0], beta, A, dA, dw, &dus[0], g, cu, ci, chunk_size, dk, &dvs[0], dbeta, dg, ws, meta, stream, nullptr)))
        return rc;
    if ((rc = wy_bwd_full_impl(k, &vs[1], beta, A, &zero_da, &zero_dw, &dus[1], g, cu, ci, chunk_size, &dk2, &dvs[1], &db2, &dg2, ws, meta,
                               stream, nullptr)))
        return rc;
    return add_scalars(dbeta, db2, stream);
}

// da + full in one call: dA (bf16, transposed like the stand-alone operator writes it) lives in the caller's workspace
// behind the shared variable-length metadata.
int wy_bwd_impl(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A,
                const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu,
                const fla_int_array *ci, int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv,
                const fla_tensor *dbeta, const fla_tensor *dg, void *ws, uint64_t ws_size, hipStream_t stream,
                uint64_t *query) {
    const char *op = "prepare_wy_repr_bwd";
    if (!A) return fail(FLA_ERR_NULL, "%s: A must not be null.", op);
    fla_tensor dA = *A;     // same shape; contiguous [B,Hv,T,C] bf16
    dA.data = nullptr;
    int64_t st = 1;
    for (int d = dA.ndim - 1; d >= 0; --d) {
        dA.stride[d] = st;
        st *= dA.shape[d];
    }
    uint64_t meta_da = 0, meta_full = 0;
    int rc;
    dA.data = const_cast<void *>(A->data);  // a non-null stand-in for the size queries
    if ((rc = wy_bwd_da_impl(k, v, beta, A, dw, du, g, cu, ci, chunk_size, &dA, nullptr, 0, nullptr, &meta_da))) return rc;
    if ((rc = wy_bwd_full_impl(k, v, beta, A, &dA, dw, du, g, cu, ci, chunk_size, dk, dv, dbeta, dg, nullptr, 0, nullptr,
                               &meta_full)))
        return rc;
    const uint64_t meta = ((meta_da > meta_full ? meta_da : meta_full) + 255) & ~(uint64_t)255;
    const uint64_t need = meta + (uint64_t)st * 2;
    if (query) {
        *query = need;
        return FLA_OK;
    }
    if (st == 0) return FLA_OK;
    if (!ws || ws_size < need) return fail(FLA_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given.", op,
                                           (unsigned long long)need, (unsigned long long)ws_size);
    dA.data = static_cast<char *>(ws) + meta;
    if ((rc = wy_bwd_da_impl(k, v, beta, A, dw, du, g, cu, ci, chunk_size, &dA, ws, meta, stream, nullptr))) return rc;
    return wy_bwd_full_impl(k, v, beta, A, &dA, dw, du, g, cu, ci, chunk_size, dk, dv, dbeta, dg, ws, meta, stream, nullptr);
}

}  // namespace
}  // namespace fla

#define FLA_NULL_WS(op) \
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, op ": workspace_size must not be null.")

FLA_ENTRY(fla_chunk_bwd_dv_local_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *d_o, const fla_tensor *g, const fla_tensor *g_gamma,
    const fla_tensor *A, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *out, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_bwd_dv_local_get_workspace_size, q, k, d_o, g, g_gamma, A, cu_seqlens, chunk_indices, scale, chunk_size, out, workspace_size);
    FLA_NULL_WS("chunk_bwd_dv_local");
    return fla::guarded([&] { return fla::dv_local_impl(q, k, d_o, g, g_gamma, A, cu_seqlens, chunk_indices, scale, chunk_size, out, nullptr, 0,
                              nullptr, workspace_size); });
}
FLA_ENTRY(fla_chunk_bwd_dv_local)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *d_o, const fla_tensor *g, const fla_tensor *g_gamma,
    const fla_tensor *A, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *out, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_bwd_dv_local, q, k, d_o, g, g_gamma, A, cu_seqlens, chunk_indices, scale, chunk_size, out, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::dv_local_impl(q, k, d_o, g, g_gamma, A, cu_seqlens, chunk_indices, scale, chunk_size, out, workspace,
                              workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_bwd_dqkwg_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *w, const fla_tensor *g_gamma, float scale, int64_t chunk_size,
    bool use_exp2, bool transpose_state_layout, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dw,
    const fla_tensor *dg, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_bwd_dqkwg_get_workspace_size, q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, w, g_gamma, scale, chunk_size, use_exp2, transpose_state_layout, dq, dk, dw, dg, workspace_size);
    FLA_NULL_WS("chunk_bwd_dqkwg");
    return fla::guarded([&] { return fla::dqkwg_impl(q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, w, g_gamma, scale, chunk_size, use_exp2,
                           transpose_state_layout, dq, dk, dw, dg, nullptr, 0, nullptr, workspace_size); });
}
FLA_ENTRY(fla_chunk_bwd_dqkwg)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *w, const fla_tensor *g_gamma, float scale, int64_t chunk_size,
    bool use_exp2, bool transpose_state_layout, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dw,
    const fla_tensor *dg, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_bwd_dqkwg, q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, w, g_gamma, scale, chunk_size, use_exp2, transpose_state_layout, dq, dk, dw, dg, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::dqkwg_impl(q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, w, g_gamma, scale, chunk_size, use_exp2,
                           transpose_state_layout, dq, dk, dw, dg, workspace, workspace_size,
                           static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_bwd_dqkwg_l2norm_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *q_rstd, float scale, int64_t chunk_size, const fla_tensor *dq,
    const fla_tensor *dk, const fla_tensor *dw, const fla_tensor *dg, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_bwd_dqkwg_l2norm_get_workspace_size, q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, q_rstd, scale, chunk_size, dq, dk, dw, dg, workspace_size);
    FLA_NULL_WS("chunk_bwd_dqkwg_l2norm");
    if (!q_rstd || !q_rstd->data) return fla::fail(FLA_ERR_NULL, "chunk_bwd_dqkwg_l2norm: q_rstd must be provided.");
    return fla::guarded([&] { return fla::dqkwg_impl(q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, nullptr, nullptr, scale, chunk_size, false,
                           false, dq, dk, dw, dg, nullptr, 0, nullptr, workspace_size, q_rstd); });
}
FLA_ENTRY(fla_chunk_bwd_dqkwg_l2norm)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *q_rstd, float scale, int64_t chunk_size, const fla_tensor *dq,
    const fla_tensor *dk, const fla_tensor *dw, const fla_tensor *dg, void *workspace, uint64_t workspace_size,
    void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_bwd_dqkwg_l2norm, q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, q_rstd, scale, chunk_size, dq, dk, dw, dg, workspace, workspace_size, stream);
    if (!q_rstd || !q_rstd->data) return fla::fail(FLA_ERR_NULL, "chunk_bwd_dqkwg_l2norm: q_rstd must be provided.");
    return fla::guarded([&] { return fla::dqkwg_impl(q, k, v, g, h, dox, dh, dv, cu_seqlens, chunk_indices, nullptr, nullptr, scale, chunk_size, false,
                           false, dq, dk, dw, dg, workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr, q_rstd); });
}

FLA_ENTRY(fla_prepare_wy_repr_bwd_da_get_workspace_size)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dA, uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd_da_get_workspace_size, k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dA, workspace_size);
    FLA_NULL_WS("prepare_wy_repr_bwd_da");
    return fla::guarded([&] { return fla::wy_bwd_da_impl(k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dA, nullptr, 0, nullptr,
                               workspace_size); });
}
FLA_ENTRY(fla_prepare_wy_repr_bwd_da)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dA, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd_da, k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dA, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::wy_bwd_da_impl(k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dA, workspace,
                               workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_prepare_wy_repr_bwd_full_get_workspace_size)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv,
    const fla_tensor *dbeta, const fla_tensor *dg, uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd_full_get_workspace_size, k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg, workspace_size);
    FLA_NULL_WS("prepare_wy_repr_bwd_full");
    return fla::guarded([&] { return fla::wy_bwd_full_impl(k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg,
                                 nullptr, 0, nullptr, workspace_size); });
}
FLA_ENTRY(fla_prepare_wy_repr_bwd_full)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv,
    const fla_tensor *dbeta, const fla_tensor *dg, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd_full, k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::wy_bwd_full_impl(k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg,
                                 workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_prepare_wy_repr_bwd_full_accumulate_get_workspace_size)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *k_rstd, const fla_tensor *dk,
    const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg, uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd_full_accumulate_get_workspace_size, k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, k_rstd, dk, dv, dbeta, dg, workspace_size);
    FLA_NULL_WS("prepare_wy_repr_bwd_full_accumulate");
    return fla::guarded([&] { return fla::wy_bwd_full_impl(k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg,
                                 nullptr, 0, nullptr, workspace_size, true, k_rstd); });
}
FLA_ENTRY(fla_prepare_wy_repr_bwd_full_accumulate)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *k_rstd, const fla_tensor *dk,
    const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg, void *workspace, uint64_t workspace_size,
    void *stream) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd_full_accumulate, k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, k_rstd, dk, dv, dbeta, dg, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::wy_bwd_full_impl(k, v, beta, A, dA, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg,
                                 workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr, true, k_rstd); });
}

FLA_ENTRY(fla_prepare_wy_repr_bwd_get_workspace_size)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg,
    uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd_get_workspace_size, k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg, workspace_size);
    FLA_NULL_WS("prepare_wy_repr_bwd");
    return fla::guarded([&] { return fla::wy_bwd_impl(k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg, nullptr, 0,
                            nullptr, workspace_size); });
}
FLA_ENTRY(fla_prepare_wy_repr_bwd)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg,
    void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_prepare_wy_repr_bwd, k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::wy_bwd_impl(k, v, beta, A, dw, du, g, cu_seqlens, chunk_indices, chunk_size, dk, dv, dbeta, dg, workspace,
                            workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}
