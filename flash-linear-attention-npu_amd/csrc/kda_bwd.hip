// Chunk-parallel stages of the KDA (per-channel gated delta rule) BACKWARD around the reverse scan
// (chunk_gated_delta_rule_bwd_dhu with gK) and chunk_kda_bwd_intra:
//   chunk_kda_bwd_dav     dAqk = scale tril(do v_new^T),  dv = Aqk^T do
//   chunk_kda_bwd_dqkwg   dq, dk, dw and the gate gradient of the state-dependent parts of a chunk step
//   chunk_kda_bwd_wy      backward of  w = Akk (k beta 2^g),  u = Akk (v beta),  Akk = (I + M)^-1
// The reference has no kernels for these stages: its deployment leaves them to a third-party Triton package
// (torch_custom/fla_npu/fla_npu/adapters/triton_ascend_kda.py:1-8); the forward they differentiate is
// tests/atk/chunk_kda_fwd/executor_chunk_kda_fwd.py:459-484.  g is the chunk-local cumulated gate in log2
// units; "dg" is the gradient with respect to ln 2 * g, the convention of chunk_kda_bwd_intra
// (torch_custom/fla_npu/test/test_npu_chunk_kda_bwd_intra.py:7-91), so the stages add into one tensor.
// One workgroup per (chunk, value head); bf16 MFMA with fp32 accumulation; wave w owns token rows 16w..16w+15.
// dq, dk, dg are fp32 and per VALUE head (the gate is per value head); grouped heads are summed by the caller.
#include "gdn_common.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ f32x4 zero4() { return f32x4{0.f, 0.f, 0.f, 0.f}; }
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }

// fp32 [B,H,T,D] through strides, unit innermost stride
struct ViewF {
    float *p;
    int64_t sb, sh, st;
};
inline ViewF viewf(const fla_tensor *t) { return ViewF{static_cast<float *>(t->data), t->stride[0], t->stride[1], t->stride[2]}; }

// =============================================================================
// chunk_kda_bwd_dav
// =============================================================================
struct DavParams {
    ChunkGeom geom;
    View4 v_new, d_o, aqk, dv;
    ViewF daqk;
    float scale;
};

template <int V>
__global__ void __launch_bounds__(kThreads) kda_bwd_dav_kernel(const DavParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int po = V + 16, pv = V + 8, pa = kChunk + 16;
    elem *oS = reinterpret_cast<elem *>(smem);      // do: rows contracted over V (dAqk) and over tokens (dv)
    elem *vS = oS + kChunk * po;                    // v_new
    elem *aS = vS + kChunk * pv;                    // Aqk

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x, w = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    {
        TileCopy<kThreads, kChunk, V> to, tv;
        TileCopy<kThreads, kChunk, kChunk> ta;
        to.fetch(static_cast<const elem *>(p.d_o.p) + b * p.d_o.sb + hv * p.d_o.sh + (int64_t)start * p.d_o.st, p.d_o.st, len, tid);
        tv.fetch(static_cast<const elem *>(p.v_new.p) + b * p.v_new.sb + hv * p.v_new.sh + (int64_t)start * p.v_new.st, p.v_new.st, len, tid);
        ta.fetch(static_cast<const elem *>(p.aqk.p) + b * p.aqk.sb + hv * p.aqk.sh + (int64_t)start * p.aqk.st, p.aqk.st, len, tid);
        to.commit(oS, po, len, tid);
        tv.commit(vS, pv, len, tid);
        ta.commit(aS, pa, len, tid);
    }
    __syncthreads();
    // dAqk[i][j] = scale <do_i, v_new_j> for j <= i: row tile w, column tiles 0..w
    float *dag = p.daqk.p + b * p.daqk.sb + hv * p.daqk.sh + (int64_t)start * p.daqk.st;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        f32x4 acc = zero4();
        if (ct <= w) {
#pragma unroll
            for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(oS, po, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), acc);
        }
        const int col = 16 * ct + li;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
            if (row < len) dag[(int64_t)row * p.daqk.st + col] = (ct <= w && col <= row) ? acc[e] * p.scale : 0.f;
        }
    }
    // dv_j = sum_{i >= j} Aqk[i][j] do_i
    char *dvg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dv.p)) + b * p.dv.sb + hv * p.dv.sh +
                                         (int64_t)start * p.dv.st);
#pragma unroll
    for (int ct = 0; ct < V / 16; ++ct) {
        f32x4 acc = zero4();
#pragma unroll
        for (int j = 0; j < 2; ++j)
            if (32 * j + 31 >= 16 * w) acc = mfma16x32(frag_tr(aS, pa, 16 * w, 32 * j), frag_tr(oS, po, 16 * ct, 32 * j), acc);
        acc_to_global(dvg + 32 * ct, p.dv.st * 2, 16 * w, len, acc);
    }
}

// =============================================================================
// chunk_kda_bwd_dqkwg
// =============================================================================
constexpr int kDqkwgThreads = 512;   // two waves per SIMD over one set of LDS tiles
struct KdaDqkwgParams {
    ChunkGeom geom;
    View4 q, k, v, d_o, dv, dw;
    const float *gk;
    int64_t g_sb, g_sh, g_st;
    const elem *h, *dh;
    int64_t h_sb, h_sh, h_sc, dh_sb, dh_sh, dh_sc;
    ViewF dq, dk, dg;
    float scale;
    ViewF daqk;   // optional f32 [B,Hv,T,64]: dAqk = scale tril(d_o v_new^T), the first result of chunk_kda_bwd_dav
};

template <int K, int V>
__global__ void __launch_bounds__(kDqkwgThreads) kda_bwd_dqkwg_kernel(const KdaDqkwgParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pv = V + 8;
    constexpr int KT = K / 16, KTH = KT / 2;   // column tiles of the K-sized outputs: all, and per wave
    constexpr int CPR = V / 8;                 // 16-byte pieces per state row
    elem *vS = reinterpret_cast<elem *>(smem);  // v_new
    elem *oS = vS + kChunk * pv;                // do
    elem *dvS = oS + kChunk * pv;               // total dv_new
    elem *hS = dvS + kChunk * pv;               // h, then dh
    float *hdS = reinterpret_cast<float *>(hS + K * pv);   // [K]    sum_v h . dh per state row
    float *colS = hdS + K;                                  // [4][K] per row tile: sum_j k_j dk_j
    float *exS = colS + 4 * K;                              // [K]    what lands on the chunk's last token
    // q, k and the gate of the chunk as whole rows (the epilogue reads them element by element in the accumulator
    // layout; fetched that way from memory they came as 32- and 64-byte pieces)
    constexpr int pq = K + 8, pg = K + 4;
    elem *qS = reinterpret_cast<elem *>(exS + K);
    elem *kS = qS + kChunk * pq;
    float *gS = reinterpret_cast<float *>(kS + kChunk * pq);
    // the three fp32 results leave through tiles laid over everything above once the products are done
    float *outS = reinterpret_cast<float *>(smem);
    static_assert((size_t)3 * kChunk * pg * 4 <= ((size_t)3 * kChunk * pv + (size_t)K * pv) * 2 + (size_t)6 * K * 4 +
                                                     (size_t)2 * kChunk * pq * 2 + (size_t)kChunk * pg * 4,
                  "the result tiles must fit the operand tiles");

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    // eight waves: wave (w, half) owns token rows 16w.. and column tiles half*KTH .. half*KTH+KTH-1
    const int tid = threadIdx.x, w = wave_id() & 3, half = wave_id() >> 2, l = lane_id(), li = l & 15, lg = l >> 4;

    const float *gg = p.gk + b * p.g_sb + hv * p.g_sh + (int64_t)start * p.g_st;
    constexpr int GN = kChunk * (K / 4) / kDqkwgThreads;   // 16-byte pieces of the gate tile per thread
    f32x4 gpre[GN];
#pragma unroll
    for (int m = 0; m < GN; ++m) {
        const int idx = m * kDqkwgThreads + tid;
        const int r = min(idx / (K / 4), len - 1), c4 = (idx % (K / 4)) * 4;   // rows past the tail repeat the last valid row
        gpre[m] = *reinterpret_cast<const f32x4 *>(gg + (int64_t)r * p.g_st + c4);
    }
    TileCopy<kDqkwgThreads, kChunk, K> tq, tk;
    tq.fetch(static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh + (int64_t)start * p.q.st, p.q.st, len, tid);
    tk.fetch(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st, p.k.st, len, tid);
    TileCopy<kDqkwgThreads, K, V> tdh;
    {
        TileCopy<kDqkwgThreads, kChunk, V> tv, to, tdv;
        TileCopy<kDqkwgThreads, K, V> th;
        tv.fetch(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st, p.v.st, len, tid);
        to.fetch(static_cast<const elem *>(p.d_o.p) + b * p.d_o.sb + hv * p.d_o.sh + (int64_t)start * p.d_o.st, p.d_o.st, len, tid);
        tdv.fetch(static_cast<const elem *>(p.dv.p) + b * p.dv.sb + hv * p.dv.sh + (int64_t)start * p.dv.st, p.dv.st, len, tid);
        th.fetch(p.h + b * p.h_sb + hv * p.h_sh + (int64_t)c * p.h_sc, V, K, tid);
        tdh.fetch(p.dh + b * p.dh_sb + hv * p.dh_sh + (int64_t)c * p.dh_sc, V, K, tid);
#pragma unroll
        for (int m = 0; m < GN; ++m) {
            const int idx = m * kDqkwgThreads + tid;
            *reinterpret_cast<f32x4 *>(gS + (idx / (K / 4)) * pg + (idx % (K / 4)) * 4) = gpre[m];
        }
        tq.commit(qS, pq, len, tid);
        tk.commit(kS, pq, len, tid);
        tv.commit(vS, pv, len, tid);
        to.commit(oS, pv, len, tid);
        tdv.commit(dvS, pv, len, tid);
        th.commit(hS, pv, K, tid);
        // sum_v h[k][v] dh[k][v]: the CPR threads that hold the pieces of one state row add their shares
#pragma unroll
        for (int m = 0; m < TileCopy<kDqkwgThreads, K, V>::N; ++m) {
            const elemx8 a = __builtin_bit_cast(elemx8, th.r[m]), d = __builtin_bit_cast(elemx8, tdh.r[m]);
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) s += (float)a[e] * (float)d[e];
            s = group_sum<CPR>(s);
            const int idx = m * kDqkwgThreads + tid;
            if (idx % CPR == 0) hdS[idx / CPR] = s;
        }
    }
    __syncthreads();
    if (p.daqk.p != nullptr) {   // dAqk[i][j] = scale <do_i, v_new_j>, j <= i: row tile w, two column tiles per wave
        float *dag = p.daqk.p + b * p.daqk.sb + hv * p.daqk.sh + (int64_t)start * p.daqk.st;
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const int ct = 2 * half + cc;
            f32x4 acc = zero4();
            if (ct <= w) {
#pragma unroll
                for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(oS, pv, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), acc);
            }
            const int col = 16 * ct + li;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                if (row < len) dag[(int64_t)row * p.daqk.st + col] = (ct <= w && col <= row) ? acc[e] * p.scale : 0.f;
            }
        }
    }
    // ---- products with the state at chunk start: dq (do h^T) and dw (-dv h^T) ---------------------
    f32x4 dqa[KTH], dka[KTH];
    char *dwg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dw.p)) + b * p.dw.sb + hv * p.dw.sh +
                                         (int64_t)start * p.dw.st);
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {
        const int cg = half * KTH + ct;
        f32x4 a = zero4(), d = zero4();
#pragma unroll
        for (int j = 0; j < V / 32; ++j) {
            const elemx8 hf = frag_kc(hS, pv, 16 * cg, 32 * j);
            a = mfma16x32(frag_kc(oS, pv, 16 * w, 32 * j), hf, a);
            d = mfma16x32(frag_kc(dvS, pv, 16 * w, 32 * j), hf, d);
        }
        dqa[ct] = a;
        acc_to_global(dwg + 32 * cg, p.dw.st * 2, 16 * w, len, -d);
    }
    __syncthreads();                 // every wave is done with h
    tdh.commit(hS, pv, K, tid);
    __syncthreads();
    // ---- product with the state gradient: dk (v_new dh^T); gate factors; column sums of k . dk -----
    float qv[KTH][4], kv[KTH][4];
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {
        const int cg = half * KTH + ct, col = 16 * cg + li;
        f32x4 d = zero4();
#pragma unroll
        for (int j = 0; j < V / 32; ++j) d = mfma16x32(frag_kc(vS, pv, 16 * w, 32 * j), frag_kc(hS, pv, 16 * cg, 32 * j), d);
        const float gl = gS[(len - 1) * pg + col];
        float colsum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
            const float gv = gS[row * pg + col];
            qv[ct][e] = (float)qS[row * pq + col];
            kv[ct][e] = (float)kS[row * pq + col];
            dqa[ct][e] *= p.scale * ex2(gv);
            d[e] *= ex2(gl - gv);
            colsum += row < len ? kv[ct][e] * d[e] : 0.f;
        }
        dka[ct] = d;
        colsum += __shfl_xor(colsum, 16, kWave);
        colsum += __shfl_xor(colsum, 32, kWave);
        if (lg == 0) colS[w * K + col] = colsum;
    }
    __syncthreads();
    if (tid < K) exS[tid] = colS[tid] + colS[K + tid] + colS[2 * K + tid] + colS[3 * K + tid] + ex2(gS[(len - 1) * pg + tid]) * hdS[tid];
    __syncthreads();
    float extra[KTH];
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) extra[ct] = exS[16 * (half * KTH + ct) + li];
    __syncthreads();   // every operand tile is dead: the results take their place
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {
        const int col = 16 * (half * KTH + ct) + li;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
            outS[row * pg + col] = dqa[ct][e];
            outS[(kChunk + row) * pg + col] = dka[ct][e];
            outS[(2 * kChunk + row) * pg + col] = qv[ct][e] * dqa[ct][e] - kv[ct][e] * dka[ct][e] + (row == len - 1 ? extra[ct] : 0.f);
        }
    }
    __syncthreads();
    float *dst[3] = {p.dq.p + b * p.dq.sb + hv * p.dq.sh + (int64_t)start * p.dq.st,
                     p.dk.p + b * p.dk.sb + hv * p.dk.sh + (int64_t)start * p.dk.st,
                     p.dg.p + b * p.dg.sb + hv * p.dg.sh + (int64_t)start * p.dg.st};
    const int64_t dst_st[3] = {p.dq.st, p.dk.st, p.dg.st};
#pragma unroll
    for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int m = 0; m < GN; ++m) {
            const int idx = m * kDqkwgThreads + tid;
            const int r = idx / (K / 4), c4 = (idx % (K / 4)) * 4;
            if (r < len) *reinterpret_cast<f32x4 *>(dst[t] + (int64_t)r * dst_st[t] + c4) = *reinterpret_cast<const f32x4 *>(outS + (t * kChunk + r) * pg + c4);
        }
}

// =============================================================================
// chunk_kda_bwd_wy
// =============================================================================
struct KdaWyParams {
    ChunkGeom geom;
    View4 k, v, akk, dw, du, dv;
    View3 beta;
    const float *gk;
    int64_t g_sb, g_sh, g_st;
    ViewF dk, dg, dakk;         // dk and dg are added to
    float *db;
    int64_t db_sb, db_sh, db_st;
};

template <int K, int V>
__global__ void __launch_bounds__(kThreads, 2) kda_bwd_wy_kernel(const KdaWyParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pw = K + 16, pu = V + 16, pk = K + 8, pv = V + 8, pa = kChunk + 8;
    constexpr int KT = K / 16, VT = V / 16;
    elem *dwS = reinterpret_cast<elem *>(smem);   // contracted over K (dA) and over tokens (Akk^T dw)
    elem *duS = dwS + kChunk * pw;
    elem *kgS = duS + kChunk * pu;                // k 2^g
    elem *vS = kgS + kChunk * pk;
    elem *aS = vS + kChunk * pv;                  // Akk
    float *bS = reinterpret_cast<float *>(aS + kChunk * pa);
    // the two 64 x 64 intermediates of the chain through the inverse reuse the dw and du tiles once those are dead
    elem *m4S = dwS;
    elem *m5S = duS;

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x, w = wave_id(), l = lane_id(), li = l & 15, lg = l >> 4;
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st;
    const float *gg = p.gk + b * p.g_sb + hv * p.g_sh + (int64_t)start * p.g_st;
    {
        TileCopy<kThreads, kChunk, K> tdw, tk;
        TileCopy<kThreads, kChunk, V> tdu, tv;
        TileCopy<kThreads, kChunk, kChunk> ta;
        tdw.fetch(static_cast<const elem *>(p.dw.p) + b * p.dw.sb + hv * p.dw.sh + (int64_t)start * p.dw.st, p.dw.st, len, tid);
        tk.fetch(kg, p.k.st, len, tid);
        tdu.fetch(static_cast<const elem *>(p.du.p) + b * p.du.sb + hv * p.du.sh + (int64_t)start * p.du.st, p.du.st, len, tid);
        tv.fetch(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st, p.v.st, len, tid);
        ta.fetch(static_cast<const elem *>(p.akk.p) + b * p.akk.sb + hv * p.akk.sh + (int64_t)start * p.akk.st, p.akk.st, len, tid);
        // gate pieces that match the k pieces of this thread
        constexpr int NK = TileCopy<kThreads, kChunk, K>::N;
        f32x4 g0[NK], g1[NK];
#pragma unroll
        for (int m = 0; m < NK; ++m) {
            const int idx = m * kThreads + tid;
            const int r = min(idx / (K / 8), len - 1), c8 = (idx % (K / 8)) << 3;
            g0[m] = *reinterpret_cast<const f32x4 *>(gg + (int64_t)r * p.g_st + c8);
            g1[m] = *reinterpret_cast<const f32x4 *>(gg + (int64_t)r * p.g_st + c8 + 4);
        }
        if (tid < kChunk) bS[tid] = tid < len ? load_scalar(p.beta, b, hv, start + tid) : 0.f;
        tdw.commit(dwS, pw, len, tid);
        tdu.commit(duS, pu, len, tid);
        tv.commit(vS, pv, len, tid);
        ta.commit(aS, pa, len, tid);
#pragma unroll
        for (int m = 0; m < NK; ++m) {
            const int idx = m * kThreads + tid;
            const int r = idx / (K / 8), c8 = (idx % (K / 8)) << 3;
            const elemx8 a = __builtin_bit_cast(elemx8, tk.r[m]);
            f32x4 lo, hi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[e] = r < len ? (float)a[e] * ex2(g0[m][e]) : 0.f;
                hi[e] = r < len ? (float)a[4 + e] * ex2(g1[m][e]) : 0.f;
            }
            *reinterpret_cast<elemx8 *>(kgS + r * pk + c8) = frag_from_acc(lo, hi);
        }
    }
    __syncthreads();
    // ---- dA = strict_lower((dw (k 2^g)^T + du v^T) beta_col), row tile w --------------------------
    f32x4 m4[4];
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        f32x4 acc = zero4();
        if (ct <= w) {
#pragma unroll
            for (int j = 0; j < K / 32; ++j) acc = mfma16x32(frag_kc(dwS, pw, 16 * w, 32 * j), frag_kc(kgS, pk, 16 * ct, 32 * j), acc);
#pragma unroll
            for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(duS, pu, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), acc);
            const int col = 16 * ct + li;
            const float bc = bS[col];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                acc[e] = (col < row && row < len) ? acc[e] * bc : 0.f;
            }
        }
        m4[ct] = acc;
    }
    // ---- x = Akk^T dw, y = Akk^T du and everything element-wise in them ----------------------------
    float br[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) br[e] = bS[16 * w + 4 * lg + e];
    float db_row[4] = {0.f, 0.f, 0.f, 0.f};
    const elemx8 at0 = frag_tr(aS, pa, 16 * w, 0), at1 = frag_tr(aS, pa, 16 * w, 32);
    char *dvg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dv.p)) + b * p.dv.sb + hv * p.dv.sh +
                                         (int64_t)start * p.dv.st);
#pragma unroll
    for (int ct = 0; ct < VT; ++ct) {
        f32x4 acc = mfma16x32(at0, frag_tr(duS, pu, 16 * ct, 0), zero4());
        acc = mfma16x32(at1, frag_tr(duS, pu, 16 * ct, 32), acc);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            db_row[e] += acc[e] * (float)vS[(16 * w + 4 * lg + e) * pv + 16 * ct + li];
            acc[e] *= br[e];
        }
        acc_to_global(dvg + 32 * ct, p.dv.st * 2, 16 * w, len, acc);
    }
    // ---- x = Akk^T dw goes to an fp32 tile over the du, k 2^g and v tiles (dead by now); everything element-wise in
    // it (dk += x 2^g beta, dg += that k, dbeta += <x 2^g, k>) then runs over whole rows, 16 bytes per lane: read and
    // written from the accumulator layout the fp32 dk and dg moved as 64-byte pieces
    constexpr int px = K + 4;
    float *xS = reinterpret_cast<float *>(duS);
    static_assert((size_t)kChunk * px * 4 + kChunk * 4 <= (size_t)kChunk * (pu + pk + pv) * 2, "x must fit the dead tiles");
    float *dbS = xS + kChunk * px;   // [64] the <y, v> part of dbeta
    __syncthreads();
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float s_ = group_sum<16>(db_row[e]);
        if (li == 0) dbS[16 * w + 4 * lg + e] = s_;
    }
#pragma unroll
    for (int ct = 0; ct < KT; ++ct) {
        f32x4 x = mfma16x32(at0, frag_tr(dwS, pw, 16 * ct, 0), zero4());
        x = mfma16x32(at1, frag_tr(dwS, pw, 16 * ct, 32), x);
#pragma unroll
        for (int e = 0; e < 4; ++e) xS[(16 * w + 4 * lg + e) * px + 16 * ct + li] = x[e];
    }
    __syncthreads();
    {
        float *dkg = p.dk.p + b * p.dk.sb + hv * p.dk.sh + (int64_t)start * p.dk.st;
        float *dgg = p.dg.p + b * p.dg.sb + hv * p.dg.sh + (int64_t)start * p.dg.st;
        constexpr int PPR = K / 4;                        // 16-byte pieces per row: one row = PPR consecutive lanes
        constexpr int NP = kChunk * PPR / kThreads;
        static_assert(PPR <= kWave && kWave % PPR == 0, "a row's pieces must sit in one wave");
#pragma unroll
        for (int m = 0; m < NP; ++m) {
            const int idx = m * kThreads + tid;
            const int r = idx / PPR, c4 = (idx % PPR) * 4, rr = min(r, len - 1);
            const f32x4 x = *reinterpret_cast<const f32x4 *>(xS + r * px + c4);
            const f32x4 g4 = *reinterpret_cast<const f32x4 *>(gg + (int64_t)rr * p.g_st + c4);
            const elemx4 k4 = *reinterpret_cast<const elemx4 *>(kg + (int64_t)rr * p.k.st + c4);
            f32x4 dk4 = *reinterpret_cast<const f32x4 *>(dkg + (int64_t)rr * p.dk.st + c4);
            f32x4 dg4 = *reinterpret_cast<const f32x4 *>(dgg + (int64_t)rr * p.dg.st + c4);
            const float beta = bS[r];
            float dbp = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float xe = x[e] * ex2(g4[e]), kk = (float)k4[e];
                const float dk = xe * beta;
                dbp += xe * kk;
                dk4[e] += dk;
                dg4[e] += dk * kk;
            }
            dbp = group_sum<PPR>(dbp);
            if (r < len) {
                *reinterpret_cast<f32x4 *>(dkg + (int64_t)r * p.dk.st + c4) = dk4;
                *reinterpret_cast<f32x4 *>(dgg + (int64_t)r * p.dg.st + c4) = dg4;
                if (idx % PPR == 0) p.db[b * p.db_sb + hv * p.db_sh + (int64_t)(start + r) * p.db_st] = dbp + dbS[r];
            }
        }
    }
    __syncthreads();   // every wave has read its dw / du rows and columns: their tiles may be overwritten
    // ---- dM = -strict_lower(Akk^T dA Akk^T) ----------------------------------------------------
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) acc_to_tile(m4S, pa, 16 * w, 16 * ct, m4[ct]);
    __syncthreads();
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {   // M5 = dA Akk^T
        f32x4 acc = zero4();
#pragma unroll
        for (int j = 0; j < 2; ++j) acc = mfma16x32(frag_kc(m4S, pa, 16 * w, 32 * j), frag_kc(aS, pa, 16 * ct, 32 * j), acc);
        acc_to_tile(m5S, pa, 16 * w, 16 * ct, acc);
    }
    __syncthreads();
    float *dag = p.dakk.p + b * p.dakk.sb + hv * p.dakk.sh + (int64_t)start * p.dakk.st;
#pragma unroll
    for (int ct = 0; ct < 4; ++ct) {
        f32x4 acc = zero4();
        if (ct <= w) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if (32 * j + 31 >= 16 * w) acc = mfma16x32(frag_tr(aS, pa, 16 * w, 32 * j), frag_tr(m5S, pa, 16 * ct, 32 * j), acc);
        }
        const int col = 16 * ct + li;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
            if (row < len) dag[(int64_t)row * p.dakk.st + col] = (ct <= w && col < row) ? -acc[e] : 0.f;
        }
    }
}

// =============================================================================
// chunk_kda_bwd_dqkwg_wy: the two stages above for one (chunk, value head) in one workgroup
// =============================================================================
// Run one after the other, chunk_kda_bwd_dqkwg writes dk, dg (fp32) and dw, and chunk_kda_bwd_wy reads all three back,
// adds to dk and dg and writes them again: 4 KB of the 9.5 KB the pair moves per token and head.  Here dw passes through
// an LDS tile, and the x = Akk^T dw tiles land in the accumulator layout of the state part of dk (same row tile, same
// column tiles per wave), so dk and dg are completed in registers and written once.  Eight waves: wave (w, half) owns
// token rows 16w.. and one half of the column tiles of every result.  The tiles of the first stage make room for those of
// the second as they die: dw over d_o, v over v_new, Akk over dh, the two 64 x 64 intermediates of the chain through the
// inverse over q and the gate tile; k turns into k 2^g in place.
struct KdaDqkwgWyParams {
    ChunkGeom geom;
    View4 q, k, v_new, d_o, dv2, v, akk, dv;   // dv2: the total gradient of v_new (= du); dv: result, gradient of v
    View3 beta;
    const float *gk;
    int64_t g_sb, g_sh, g_st;
    const elem *h, *dh;
    int64_t h_sb, h_sh, h_sc, dh_sb, dh_sh, dh_sc;
    ViewF dq, dk, dg, daqk, dakk;
    float *db;
    int64_t db_sb, db_sh, db_st;
    float scale;
    int out16;   // with the intra-chunk stage: dq and dk point at 16-bit elements (strides in elements)
};

// Bytes of LDS of the kernel below.  The first two stages live in the tiles of the first; the intra-chunk stage keeps q, k
// and the gate to its end and needs the two masked 64 x 64 score gradients in fp32: with 128 channels they take the places
// of v and of the state tile, with 64 channels (smaller tiles) they get room of their own behind the others.
template <int K, int V, bool INTRA>
constexpr size_t kda_bwd_fused_smem() {
    const size_t base = ((size_t)3 * kChunk * (V + 8) + (size_t)K * (V + 8)) * 2 + (size_t)6 * K * 4 +
                        (size_t)2 * kChunk * (K + 8) * 2 + (size_t)kChunk * (K + 4) * 4;
    if (!INTRA) return base;
    const size_t tail = base + 2 * kChunk * 4;   // the two halves of dbeta
    const size_t pair = (size_t)2 * kChunk * (kChunk + 4) * 4;
    // the transposed copies of the score gradients take the dw and du tiles where those are large enough
    return (K == 128 ? tail : tail + (size_t)kChunk * (K + 8) * 2 + pair) + (V == 128 ? 0 : pair);
}

// D[16x16] += A[16x4] B[4x16] in fp32: lane l holds A[l%16][l/16], B[l/16][l%16], D[4*(l/16)+e][l%16]
__device__ __forceinline__ f32x4 mfma_f32(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// INTRA: chunk_kda_bwd_intra (with the reverse running sum of dg) follows in the same workgroup.  Its increments of dq, dk,
// dg have the accumulator layout of the first two stages (wave (w, half): row tile w, one half of the channel tiles), so
// they are added in registers; dAqk and dAkk stay on chip as fp32 tiles, and dq, dk, dg, dbeta are written once, final.
template <int K, int V, bool INTRA>
__global__ void __launch_bounds__(kDqkwgThreads) kda_bwd_dqkwg_wy_kernel(const KdaDqkwgWyParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pv = V + 8, pq = K + 8, pg = K + 4, pa = kChunk + 8, pf = kChunk + 4;
    constexpr bool BIG = K == 128;
    constexpr size_t kBase = kda_bwd_fused_smem<K, V, false>();
    constexpr int KT = K / 16, KTH = KT / 2, VTH = V / 32;   // column tiles per wave of the K- and V-sized results
    constexpr int CPR = V / 8;
    static_assert(K <= V, "the dw tile takes the place of the d_o tile");
    elem *vS = reinterpret_cast<elem *>(smem);  // v_new, then v
    elem *oS = vS + kChunk * pv;                // d_o, then dw [kChunk][pq]
    elem *dvS = oS + kChunk * pv;               // dv2 = du
    elem *hS = dvS + kChunk * pv;               // h, then dh, then Akk [kChunk][pa]
    float *hdS = reinterpret_cast<float *>(hS + K * pv);
    float *colS = hdS + K;                      // [4][K]; later beta [kChunk] and the two halves of dbeta [2][kChunk]
    float *exS = colS + 4 * K;
    elem *qS = reinterpret_cast<elem *>(exS + K);   // q, then the first intermediate of the chain through the inverse
    elem *kS = qS + kChunk * pq;                    // k, then k 2^g
    float *gS = reinterpret_cast<float *>(kS + kChunk * pq);   // gate, then the second intermediate
    float *outS = reinterpret_cast<float *>(smem);
    elem *dwS = oS, *aS = hS;
    // the intermediates of the chain through the inverse: over q and the gate, or (q, k, gate kept) over dw and du
    elem *m4S = INTRA ? oS : qS, *m5S = INTRA ? dvS : reinterpret_cast<elem *>(gS);
    elem *kgS = !INTRA ? kS : BIG ? hS + kChunk * pa : reinterpret_cast<elem *>(smem + kBase + 2 * kChunk * 4);   // k 2^g
    float *bS = colS, *dbS = INTRA ? reinterpret_cast<float *>(smem + kBase) : colS + kChunk;
    float *aqS = BIG ? reinterpret_cast<float *>(vS) : reinterpret_cast<float *>(kgS + kChunk * pq);   // tril(dAqk) [kChunk][pf]
    float *akS = BIG ? reinterpret_cast<float *>(hS) : aqS + kChunk * pf;                              // tril(dAkk)
    // their transposes, for the product that contracts over the rows
    float *aqT = V == 128 ? reinterpret_cast<float *>(oS) : reinterpret_cast<float *>(smem + kda_bwd_fused_smem<K, V, true>()) - 2 * kChunk * pf;
    float *akT = V == 128 ? reinterpret_cast<float *>(dvS) : aqT + kChunk * pf;
    static_assert(!INTRA || !BIG || ((size_t)kChunk * (pa + pq) * 2 <= (size_t)K * pv * 2 && (size_t)kChunk * pf * 4 <= (size_t)kChunk * pv * 2),
                  "k 2^g behind Akk in the state tile, a score gradient in the v tile");
    static_assert((size_t)kChunk * pa * 2 <= (size_t)kChunk * pv * 2, "an intermediate fits the dw and du tiles");
    static_assert((size_t)3 * kChunk * pg * 4 <= ((size_t)3 * kChunk * pv + (size_t)K * pv) * 2 + (size_t)6 * K * 4 + (size_t)2 * kChunk * pq * 2,
                  "the result tiles end before the gate tile, which holds the partial sums of the running sum of dg");
    static_assert((size_t)kChunk * pa * 2 <= (size_t)K * pv * 2 && (size_t)kChunk * pa * 2 <= (size_t)kChunk * pq * 2 &&
                      (size_t)kChunk * pa * 2 <= (size_t)kChunk * pg * 4 && 3 * kChunk <= 4 * K,
                  "the tiles of the second stage must fit the dead tiles of the first");
    static_assert((size_t)3 * kChunk * pg * 4 <= ((size_t)3 * kChunk * pv + (size_t)K * pv) * 2 + (size_t)6 * K * 4 +
                                                     (size_t)2 * kChunk * pq * 2 + (size_t)kChunk * pg * 4,
                  "the result tiles must fit the operand tiles");

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x, w = wave_id() & 3, half = wave_id() >> 2, l = lane_id(), li = l & 15, lg = l >> 4;

    // ---------------------------------- first stage: as kda_bwd_dqkwg_kernel -------------------------------------
    const float *gg = p.gk + b * p.g_sb + hv * p.g_sh + (int64_t)start * p.g_st;
    constexpr int GN = kChunk * (K / 4) / kDqkwgThreads;
    f32x4 gpre[GN];
#pragma unroll
    for (int m = 0; m < GN; ++m) {
        const int idx = m * kDqkwgThreads + tid;
        const int r = min(idx / (K / 4), len - 1), c4 = (idx % (K / 4)) * 4;
        gpre[m] = *reinterpret_cast<const f32x4 *>(gg + (int64_t)r * p.g_st + c4);
    }
    TileCopy<kDqkwgThreads, kChunk, K> tq, tk;
    tq.fetch(static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh + (int64_t)start * p.q.st, p.q.st, len, tid);
    tk.fetch(static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st, p.k.st, len, tid);
    TileCopy<kDqkwgThreads, K, V> tdh;
    {
        TileCopy<kDqkwgThreads, kChunk, V> tv, to, tdv;
        TileCopy<kDqkwgThreads, K, V> th;
        tv.fetch(static_cast<const elem *>(p.v_new.p) + b * p.v_new.sb + hv * p.v_new.sh + (int64_t)start * p.v_new.st, p.v_new.st, len, tid);
        to.fetch(static_cast<const elem *>(p.d_o.p) + b * p.d_o.sb + hv * p.d_o.sh + (int64_t)start * p.d_o.st, p.d_o.st, len, tid);
        tdv.fetch(static_cast<const elem *>(p.dv2.p) + b * p.dv2.sb + hv * p.dv2.sh + (int64_t)start * p.dv2.st, p.dv2.st, len, tid);
        th.fetch(p.h + b * p.h_sb + hv * p.h_sh + (int64_t)c * p.h_sc, V, K, tid);
        tdh.fetch(p.dh + b * p.dh_sb + hv * p.dh_sh + (int64_t)c * p.dh_sc, V, K, tid);
#pragma unroll
        for (int m = 0; m < GN; ++m) {
            const int idx = m * kDqkwgThreads + tid;
            *reinterpret_cast<f32x4 *>(gS + (idx / (K / 4)) * pg + (idx % (K / 4)) * 4) = gpre[m];
        }
        tq.commit(qS, pq, len, tid);
        tk.commit(kS, pq, len, tid);
        tv.commit(vS, pv, len, tid);
        to.commit(oS, pv, len, tid);
        tdv.commit(dvS, pv, len, tid);
        th.commit(hS, pv, K, tid);
#pragma unroll
        for (int m = 0; m < TileCopy<kDqkwgThreads, K, V>::N; ++m) {
            const elemx8 a = __builtin_bit_cast(elemx8, th.r[m]), d = __builtin_bit_cast(elemx8, tdh.r[m]);
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) s += (float)a[e] * (float)d[e];
            s = group_sum<CPR>(s);
            const int idx = m * kDqkwgThreads + tid;
            if (idx % CPR == 0) hdS[idx / CPR] = s;
        }
    }
    __syncthreads();
    f32x4 daq[2];   // INTRA: this wave's two tiles of the masked dAqk, kept until their LDS tile is free
    {   // dAqk[i][j] = scale <do_i, v_new_j>, j <= i
        float *dag = INTRA ? nullptr : p.daqk.p + b * p.daqk.sb + hv * p.daqk.sh + (int64_t)start * p.daqk.st;
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const int ct = 2 * half + cc;
            f32x4 acc = zero4();
            if (ct <= w) {
#pragma unroll
                for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(oS, pv, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), acc);
            }
            const int col = 16 * ct + li;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                const float val = (ct <= w && col <= row) ? acc[e] * p.scale : 0.f;
                if constexpr (INTRA) daq[cc][e] = row < len ? val : 0.f;
                else if (row < len) dag[(int64_t)row * p.daqk.st + col] = val;
            }
        }
    }
    f32x4 dqa[KTH], dka[KTH], dwa[KTH];
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {
        const int cg = half * KTH + ct;
        f32x4 a = zero4(), d = zero4();
#pragma unroll
        for (int j = 0; j < V / 32; ++j) {
            const elemx8 hf = frag_kc(hS, pv, 16 * cg, 32 * j);
            a = mfma16x32(frag_kc(oS, pv, 16 * w, 32 * j), hf, a);
            d = mfma16x32(frag_kc(dvS, pv, 16 * w, 32 * j), hf, d);
        }
        dqa[ct] = a;
        dwa[ct] = -d;
    }
    // the operands of the second stage are asked for now and land while the state-gradient product runs
    TileCopy<kDqkwgThreads, kChunk, V> tvv;
    TileCopy<kDqkwgThreads, kChunk, kChunk> ta;
    tvv.fetch(static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st, p.v.st, len, tid);
    ta.fetch(static_cast<const elem *>(p.akk.p) + b * p.akk.sb + hv * p.akk.sh + (int64_t)start * p.akk.st, p.akk.st, len, tid);
    const float beta_own = tid < kChunk ? (tid < len ? load_scalar(p.beta, b, hv, start + tid) : 0.f) : 0.f;
    __syncthreads();                 // every wave is done with h and d_o
    tdh.commit(hS, pv, K, tid);
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) acc_to_tile(dwS, pq, 16 * w, 16 * (half * KTH + ct), dwa[ct]);   // dw, rounded as it is stored
    __syncthreads();
    float qv[KTH][4], kv[KTH][4], eg[KTH][4];
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {
        const int cg = half * KTH + ct, col = 16 * cg + li;
        f32x4 d = zero4();
#pragma unroll
        for (int j = 0; j < V / 32; ++j) d = mfma16x32(frag_kc(vS, pv, 16 * w, 32 * j), frag_kc(hS, pv, 16 * cg, 32 * j), d);
        const float gl = gS[(len - 1) * pg + col];
        float colsum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
            const float gv = gS[row * pg + col];
            qv[ct][e] = (float)qS[row * pq + col];
            kv[ct][e] = (float)kS[row * pq + col];
            eg[ct][e] = ex2(gv);
            dqa[ct][e] *= p.scale * eg[ct][e];
            d[e] *= ex2(gl - gv);
            colsum += row < len ? kv[ct][e] * d[e] : 0.f;
        }
        dka[ct] = d;
        colsum += __shfl_xor(colsum, 16, kWave);
        colsum += __shfl_xor(colsum, 32, kWave);
        if (lg == 0) colS[w * K + col] = colsum;
    }
    __syncthreads();
    if (tid < K) exS[tid] = colS[tid] + colS[K + tid] + colS[2 * K + tid] + colS[3 * K + tid] + ex2(gS[(len - 1) * pg + tid]) * hdS[tid];
    __syncthreads();
    float extra[KTH];
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) extra[ct] = exS[16 * (half * KTH + ct) + li];
    // ---------------------------------- second stage: as kda_bwd_wy_kernel ----------------------------------------
    // v_new, dh, q and the column sums are dead (the barrier above came after their last reads; extra is in registers)
    tvv.commit(vS, pv, len, tid);
    ta.commit(aS, pa, len, tid);
    if (tid < kChunk) bS[tid] = beta_own;   // over the column sums, last read two barriers ago
#pragma unroll
    for (int m = 0; m < TileCopy<kDqkwgThreads, kChunk, K>::N; ++m) {   // k -> k 2^g, every thread its own pieces
        const int idx = m * kDqkwgThreads + tid;
        const int r = idx / (K / 8), c8 = (idx % (K / 8)) << 3;
        const elemx8 a = *reinterpret_cast<const elemx8 *>(kS + r * pq + c8);
        const f32x4 g0 = *reinterpret_cast<const f32x4 *>(gS + r * pg + c8), g1 = *reinterpret_cast<const f32x4 *>(gS + r * pg + c8 + 4);
        f32x4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo[e] = r < len ? (float)a[e] * ex2(g0[e]) : 0.f;
            hi[e] = r < len ? (float)a[4 + e] * ex2(g1[e]) : 0.f;
        }
        *reinterpret_cast<elemx8 *>(kgS + r * pq + c8) = frag_from_acc(lo, hi);
    }
    __syncthreads();
    // dA = strict_lower((dw (k 2^g)^T + du v^T) beta_col): row tile w, two column tiles per wave
    f32x4 m4[2];
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
        const int ct = 2 * half + cc;
        f32x4 acc = zero4();
        if (ct <= w) {
#pragma unroll
            for (int j = 0; j < K / 32; ++j) acc = mfma16x32(frag_kc(dwS, pq, 16 * w, 32 * j), frag_kc(kgS, pq, 16 * ct, 32 * j), acc);
#pragma unroll
            for (int j = 0; j < V / 32; ++j) acc = mfma16x32(frag_kc(dvS, pv, 16 * w, 32 * j), frag_kc(vS, pv, 16 * ct, 32 * j), acc);
            const int col = 16 * ct + li;
            const float bc = bS[col];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                acc[e] = (col < row && row < len) ? acc[e] * bc : 0.f;
            }
        }
        m4[cc] = acc;
    }
    float br[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) br[e] = bS[16 * w + 4 * lg + e];
    float db_row[4] = {0.f, 0.f, 0.f, 0.f};
    const elemx8 at0 = frag_tr(aS, pa, 16 * w, 0), at1 = frag_tr(aS, pa, 16 * w, 32);
    {   // y = Akk^T du: dv = y beta, dbeta += <y, v>
        char *dvg = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dv.p)) + b * p.dv.sb + hv * p.dv.sh +
                                             (int64_t)start * p.dv.st);
#pragma unroll
        for (int cc = 0; cc < VTH; ++cc) {
            const int ct = half * VTH + cc;
            f32x4 acc = mfma16x32(at0, frag_tr(dvS, pv, 16 * ct, 0), zero4());
            acc = mfma16x32(at1, frag_tr(dvS, pv, 16 * ct, 32), acc);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                db_row[e] += acc[e] * (float)vS[(16 * w + 4 * lg + e) * pv + 16 * ct + li];
                acc[e] *= br[e];
            }
            acc_to_global(dvg + 32 * ct, p.dv.st * 2, 16 * w, len, acc);
        }
    }
    f32x4 dga[KTH];
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {   // x = Akk^T dw in the layout of the state part of dk: dk += x 2^g beta, dg += that k
        const int cg = half * KTH + ct;
        f32x4 x = mfma16x32(at0, frag_tr(dwS, pq, 16 * cg, 0), zero4());
        x = mfma16x32(at1, frag_tr(dwS, pq, 16 * cg, 32), x);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
            const float xe = x[e] * eg[ct][e], add = xe * br[e];
            db_row[e] += xe * kv[ct][e];
            dga[ct][e] = qv[ct][e] * dqa[ct][e] - kv[ct][e] * dka[ct][e] + (row == len - 1 ? extra[ct] : 0.f) + add * kv[ct][e];
            dka[ct][e] += add;
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float s_ = group_sum<16>(db_row[e]);
        if (li == 0) dbS[half * kChunk + 16 * w + 4 * lg + e] = s_;
    }
    // dAkk = -strict_lower(Akk^T dA Akk^T) through two 64 x 64 tiles
    if constexpr (INTRA) __syncthreads();   // every wave is done with dw, du, v and k 2^g
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) acc_to_tile(m4S, pa, 16 * w, 16 * (2 * half + cc), m4[cc]);
    if constexpr (INTRA) {
#pragma unroll
        for (int cc = 0; cc < 2; ++cc)
#pragma unroll
            for (int e = 0; e < 4; ++e) aqS[(16 * w + 4 * lg + e) * pf + 16 * (2 * half + cc) + li] = daq[cc][e];
    }
    __syncthreads();                 // dA complete; every wave is past the tile that takes the second intermediate
    if constexpr (!INTRA)
        if (tid < len) p.db[b * p.db_sb + hv * p.db_sh + (int64_t)(start + tid) * p.db_st] = dbS[tid] + dbS[kChunk + tid];
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {   // M5 = dA Akk^T
        const int ct = 2 * half + cc;
        f32x4 acc = zero4();
#pragma unroll
        for (int j = 0; j < 2; ++j) acc = mfma16x32(frag_kc(m4S, pa, 16 * w, 32 * j), frag_kc(aS, pa, 16 * ct, 32 * j), acc);
        acc_to_tile(m5S, pa, 16 * w, 16 * ct, acc);
    }
    __syncthreads();
    // third stage: CPL neighbouring channels per lane; its increments of dq, dk, dg by row e of the lane's four rows
    constexpr int CPL = KTH;
    typedef float gvec __attribute__((ext_vector_type(CPL)));
    typedef elem kvec __attribute__((ext_vector_type(CPL)));
    gvec incq[4], inck[4], incg[4];
    if constexpr (INTRA) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int c_ = 0; c_ < CPL; ++c_) incq[e][c_] = inck[e][c_] = incg[e][c_] = 0.f;
    }
    f32x4 dak[2];
    {
        float *dag = INTRA ? nullptr : p.dakk.p + b * p.dakk.sb + hv * p.dakk.sh + (int64_t)start * p.dakk.st;
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const int ct = 2 * half + cc;
            f32x4 acc = zero4();
            if (ct <= w) {
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (32 * j + 31 >= 16 * w) acc = mfma16x32(frag_tr(aS, pa, 16 * w, 32 * j), frag_tr(m5S, pa, 16 * ct, 32 * j), acc);
            }
            const int col = 16 * ct + li;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                const float val = (ct <= w && col < row) ? -acc[e] : 0.f;
                if constexpr (INTRA) dak[cc][e] = row < len ? val : 0.f;
                else if (row < len) dag[(int64_t)row * p.dakk.st + col] = val;
            }
        }
    }
    if constexpr (INTRA) {
        // ------------------------- third stage: as kda_bwd_intra_kernel, for this wave's rows ----------------------
        // Wave (w, half): rows 16w.., one half of the channels; a lane's accumulator columns are CPL neighbouring channels
        // (cb + c in accumulator c), and step s of a 16-token tile contracts over tokens 4 lg + s, so that every operand
        // is one wide LDS read: four steps of a score-gradient row, CPL channels of a k, q or gate row.
        __syncthreads();             // every wave is done with Akk and both intermediates
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const int ct = 2 * half + cc;
#pragma unroll
            for (int e = 0; e < 4; ++e) akS[(16 * w + 4 * lg + e) * pf + 16 * ct + li] = dak[cc][e];
            *reinterpret_cast<f32x4 *>(aqT + (16 * ct + li) * pf + 16 * w + 4 * lg) = daq[cc];
            *reinterpret_cast<f32x4 *>(akT + (16 * ct + li) * pf + 16 * w + 4 * lg) = dak[cc];
        }
        __syncthreads();
        const int r0 = 16 * w, row_end = min(r0 + 16, len), anchor = min(r0 + 8, row_end - 1);
        const int cb = half * (K / 2) + CPL * li;
        if (r0 < len) {              // a row tile without a token (wave-uniform) adds nothing
            const gvec ca = *reinterpret_cast<const gvec *>(gS + anchor * pg + cb);
            f32x4 D1[CPL], D2[CPL], D3[CPL];
#pragma unroll
            for (int c_ = 0; c_ < CPL; ++c_) D1[c_] = D2[c_] = D3[c_] = zero4();
            // padded rows of the tiles hold k = 0, a score gradient of 0 and the gate of the chunk's last token
            for (int jt = 0; jt <= w; ++jt) {
                const f32x4 a1 = *reinterpret_cast<const f32x4 *>(aqS + (r0 + li) * pf + 16 * jt + 4 * lg);
                const f32x4 a2 = *reinterpret_cast<const f32x4 *>(akS + (r0 + li) * pf + 16 * jt + 4 * lg);
#pragma unroll
                for (int s_ = 0; s_ < 4; ++s_) {
                    const int j = 16 * jt + 4 * lg + s_;
                    const kvec kk = *reinterpret_cast<const kvec *>(kS + j * pq + cb);
                    const gvec gg = *reinterpret_cast<const gvec *>(gS + j * pg + cb);
#pragma unroll
                    for (int c_ = 0; c_ < CPL; ++c_) {
                        const float bval = (float)kk[c_] * ex2(ca[c_] - gg[c_]);
                        D1[c_] = mfma_f32(a1[s_], bval, D1[c_]);
                        D2[c_] = mfma_f32(a2[s_], bval, D2[c_]);
                    }
                }
            }
            for (int it = w; it < 4; ++it) {
                const f32x4 a1 = *reinterpret_cast<const f32x4 *>(aqT + (r0 + li) * pf + 16 * it + 4 * lg);
                const f32x4 a2 = *reinterpret_cast<const f32x4 *>(akT + (r0 + li) * pf + 16 * it + 4 * lg);
#pragma unroll
                for (int s_ = 0; s_ < 4; ++s_) {
                    const int i = 16 * it + 4 * lg + s_;
                    const kvec kk = *reinterpret_cast<const kvec *>(kS + i * pq + cb);
                    const kvec qq = *reinterpret_cast<const kvec *>(qS + i * pq + cb);
                    const gvec gg = *reinterpret_cast<const gvec *>(gS + i * pg + cb);
                    const float bi = bS[i];
#pragma unroll
                    for (int c_ = 0; c_ < CPL; ++c_) {
                        const float fw = ex2(gg[c_] - ca[c_]);
                        D3[c_] = mfma_f32(a1[s_], (float)qq[c_] * fw, D3[c_]);
                        D3[c_] = mfma_f32(a2[s_], (float)kk[c_] * bi * fw, D3[c_]);
                    }
                }
            }
            f32x4 dbacc = zero4();
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int i = r0 + 4 * lg + e;
                if (i < len) {
                    const kvec kk = *reinterpret_cast<const kvec *>(kS + i * pq + cb);
                    const kvec qq = *reinterpret_cast<const kvec *>(qS + i * pq + cb);
                    const gvec gg = *reinterpret_cast<const gvec *>(gS + i * pg + cb);
#pragma unroll
                    for (int c_ = 0; c_ < CPL; ++c_) {
                        const float up = ex2(gg[c_] - ca[c_]), down = ex2(ca[c_] - gg[c_]);
                        const float dqd = D1[c_][e] * up, dl = D2[c_][e] * up, du = D3[c_][e] * down;
                        const float qi = (float)qq[c_], ki = (float)kk[c_];
                        const float bdl = br[e] * dl;
                        incq[e][c_] = dqd;
                        inck[e][c_] = bdl + du;
                        incg[e][c_] = qi * dqd + ki * (bdl - du);
                        dbacc[e] += dl * ki;
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float s_ = group_sum<16>(dbacc[e]);
                if (li == 0) dbS[half * kChunk + r0 + 4 * lg + e] += s_;   // the lane that wrote the entry
            }
        }
    }
    __syncthreads();   // every operand tile is dead: the results take their place
#pragma unroll
    for (int ct = 0; ct < KTH; ++ct) {
        const int col = 16 * (half * KTH + ct) + li;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 16 * w + 4 * lg + e;
            outS[row * pg + col] = dqa[ct][e];
            outS[(kChunk + row) * pg + col] = dka[ct][e];
            outS[(2 * kChunk + row) * pg + col] = INTRA && row >= len ? 0.f : dga[ct][e];
        }
    }
    __syncthreads();
    if constexpr (INTRA) {
        {   // the increments of the third stage, in its own assignment of channels to lanes
            const int cb = half * (K / 2) + CPL * li;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * w + 4 * lg + e;
                *reinterpret_cast<gvec *>(outS + row * pg + cb) += incq[e];
                *reinterpret_cast<gvec *>(outS + (kChunk + row) * pg + cb) += inck[e];
                *reinterpret_cast<gvec *>(outS + (2 * kChunk + row) * pg + cb) += incg[e];
            }
        }
        __syncthreads();
        if (tid < len) p.db[b * p.db_sb + hv * p.db_sh + (int64_t)(start + tid) * p.db_st] = dbS[tid] + dbS[kChunk + tid];
        // dg is complete and a workgroup holds a whole chunk of it: the reverse running sum over the chunk's tokens is taken
        // in the tile, a thread per column and run of rows, the runs joined through their totals
        constexpr int SEGS = kDqkwgThreads / K, RS = kChunk / SEGS;
        const int col = tid % K, seg = tid / K;
        float *x0 = outS + 2 * kChunk * pg, *tot = gS;
        float run = 0.f;
#pragma unroll
        for (int j = RS - 1; j >= 0; --j) {
            float *x = x0 + (seg * RS + j) * pg + col;
            run += *x;
            *x = run;
        }
        tot[seg * K + col] = run;
        __syncthreads();
        float later = 0.f;
#pragma unroll
        for (int s2 = 1; s2 < SEGS; ++s2)
            if (seg + s2 < SEGS) later += tot[(seg + s2) * K + col];
#pragma unroll
        for (int j = 0; j < RS; ++j) x0[(seg * RS + j) * pg + col] += later;
        __syncthreads();
        char *d16[2] = {reinterpret_cast<char *>(p.dq.p), reinterpret_cast<char *>(p.dk.p)};
        const ViewF *vw[2] = {&p.dq, &p.dk};
        const int64_t esz = p.out16 ? 2 : 4;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int m = 0; m < GN; ++m) {
                const int idx = m * kDqkwgThreads + tid;
                const int r = idx / (K / 4), c4 = (idx % (K / 4)) * 4;
                if (r < len) {
                    const f32x4 val = *reinterpret_cast<const f32x4 *>(outS + (t * kChunk + r) * pg + c4);
                    char *at = d16[t] + (b * vw[t]->sb + hv * vw[t]->sh + (int64_t)(start + r) * vw[t]->st + c4) * esz;
                    if (p.out16) *reinterpret_cast<elemx4 *>(at) = cvt4(val);
                    else *reinterpret_cast<f32x4 *>(at) = val;
                }
            }
        float *dgd = p.dg.p + b * p.dg.sb + hv * p.dg.sh + (int64_t)start * p.dg.st;
#pragma unroll
        for (int m = 0; m < GN; ++m) {
            const int idx = m * kDqkwgThreads + tid;
            const int r = idx / (K / 4), c4 = (idx % (K / 4)) * 4;
            if (r < len) *reinterpret_cast<f32x4 *>(dgd + (int64_t)r * p.dg.st + c4) = *reinterpret_cast<const f32x4 *>(x0 + r * pg + c4);
        }
        return;
    }
    float *dst[3] = {p.dq.p + b * p.dq.sb + hv * p.dq.sh + (int64_t)start * p.dq.st,
                     p.dk.p + b * p.dk.sb + hv * p.dk.sh + (int64_t)start * p.dk.st,
                     p.dg.p + b * p.dg.sb + hv * p.dg.sh + (int64_t)start * p.dg.st};
    const int64_t dst_st[3] = {p.dq.st, p.dk.st, p.dg.st};
#pragma unroll
    for (int t = 0; t < 3; ++t)
#pragma unroll
        for (int m = 0; m < GN; ++m) {
            const int idx = m * kDqkwgThreads + tid;
            const int r = idx / (K / 4), c4 = (idx % (K / 4)) * 4;
            if (r < len) *reinterpret_cast<f32x4 *>(dst[t] + (int64_t)r * dst_st[t] + c4) = *reinterpret_cast<const f32x4 *>(outS + (t * kChunk + r) * pg + c4);
        }
}

// ---- host side ------------------------------------------------------------------------------------
#define FLA_KDA_BWD_LAUNCH(KERNEL, NAME, GRID, SMEM_EXPR, P, THREADS)                                                     \
    do {                                                                                                               \
        const size_t smem__ = (SMEM_EXPR);                                                                             \
        FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(KERNEL), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                          (int)smem__));                                                               \
        FLA_LAUNCH(NAME, stream, KERNEL, GRID, dim3(THREADS), smem__, stream, P);                                       \
        FLA_HIP_CHECK(hipGetLastError());                                                                              \
        return FLA_OK;                                                                                                 \
    } while (0)

// fp32 [B,H,T,D] with unit innermost stride and 16-byte aligned rows
int check_f32_bhtd(const char *op, const char *name, const fla_tensor *t, int64_t B, int64_t H, int64_t T, int64_t D) {
    int rc = check_tensor(t, op, name, 4, dt_bit(FLA_F32));
    if (rc) return rc;
    FLA_REQUIRE(t->shape[0] == B && t->shape[1] == H && t->shape[2] == T && t->shape[3] == D, FLA_ERR_SHAPE,
                "%s: %s must be [%lld,%lld,%lld,%lld].", op, name, (long long)B, (long long)H, (long long)T, (long long)D);
    FLA_REQUIRE(inner_unit(t) && t->stride[0] % 4 == 0 && t->stride[1] % 4 == 0 && t->stride[2] % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(t->data) % 16 == 0,
                FLA_ERR_SHAPE, "%s: %s needs a unit innermost stride and 16-byte aligned rows.", op, name);
    FLA_REQUIRE(t->stride[2] >= 0, FLA_ERR_SHAPE, "%s: %s has a negative token stride.", op, name);
    return FLA_OK;
}

int check_state_blocks(const char *op, const char *name, const fla_tensor *h, const ChunkGeom &geom) {
    int rc = check_tensor(h, op, name, 5, dt_bit(kElemDtype));
    if (rc) return rc;
    FLA_REQUIRE(h->shape[0] == geom.B && h->shape[1] == geom.Hv && h->shape[2] == geom.NT && h->shape[3] == geom.K &&
                    h->shape[4] == geom.V && h->stride[4] == 1 && h->stride[3] == geom.V && h->stride[2] % 8 == 0 &&
                    h->stride[1] % 8 == 0 && h->stride[0] % 8 == 0 && reinterpret_cast<uintptr_t>(h->data) % 16 == 0,
                FLA_ERR_SHAPE, "%s: %s must be [B,Hv,NT=%d,K,V] (any outer strides) with contiguous K x V blocks.", op, name,
                geom.NT);
    return FLA_OK;
}

int dav_impl(const fla_tensor *v_new, const fla_tensor *d_o, const fla_tensor *aqk, const fla_int_array *cu,
             const fla_int_array *ci, double scale, int64_t chunk_size, const fla_tensor *daqk, const fla_tensor *dv, void *ws,
             uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_kda_bwd_dav";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, v_new, nullptr, nullptr, chunk_size, geom, kElemDtype))) return rc;   // Hk=Hv, K=V here
    // v_new and Aqk are head-major whatever the caller's layout; d_o and dAqk follow it and carry more bytes
    geom.head_fast = d_o != nullptr && d_o->ndim == 4 && geom.Hv > 1 && d_o->stride[2] > d_o->stride[1] && geom.T <= (1 << 20) ? 1 : 0;
    const int bf = dt_bit(kElemDtype);
    const int64_t B = geom.B, H = geom.Hv, T = geom.T, V = geom.V;
    if ((rc = check_bhtd(op, "v_new", v_new, B, H, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "d_o", d_o, B, H, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "Aqk", aqk, B, H, T, kChunk, bf))) return rc;
    if ((rc = check_bhtd(op, "dv", dv, B, H, T, V, bf))) return rc;
    if ((rc = check_f32_bhtd(op, "dAqk", daqk, B, H, T, kChunk))) return rc;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    DavParams p{geom, view4(v_new), view4(d_o), view4(aqk), view4(dv), viewf(daqk), (float)scale};
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hv);
    const size_t smem = ((size_t)kChunk * ((V + 16) + (V + 8) + (kChunk + 16))) * 2;
    if (V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_dav_kernel<128>), "kda_bwd_dav", grid, smem, p, kThreads);
    if (V == 64) FLA_KDA_BWD_LAUNCH((kda_bwd_dav_kernel<64>), "kda_bwd_dav", grid, smem, p, kThreads);
    if (V == 256) FLA_KDA_BWD_LAUNCH((kda_bwd_dav_kernel<256>), "kda_bwd_dav", grid, smem, p, kThreads);
    return fail(FLA_ERR_UNSUPPORTED, "%s: V=%lld has no kernel; built: 64, 128, 256.", op, (long long)V);
}

int kda_dqkwg_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
                   const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu,
                   const fla_int_array *ci, double scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
                   const fla_tensor *dw, const fla_tensor *dg, const fla_tensor *daqk, void *ws, uint64_t ws_size, hipStream_t stream,
                   uint64_t *query) {
    const char *op = "chunk_kda_bwd_dqkwg";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v_new, nullptr, chunk_size, geom, kElemDtype))) return rc;
    const int bf = dt_bit(kElemDtype);
    const int64_t B = geom.B, Hk = geom.Hk, Hv = geom.Hv, T = geom.T, K = geom.K, V = geom.V;
    if ((rc = check_bhtd(op, "q", q, B, Hk, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, B, Hk, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "v_new", v_new, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "d_o", d_o, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "dv", dv, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "dw", dw, B, Hv, T, K, bf))) return rc;
    if ((rc = check_f32_bhtd(op, "gk", gk, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dq", dq, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dk", dk, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dg", dg, B, Hv, T, K))) return rc;
    const bool has_daqk = daqk && daqk->data;
    if (has_daqk && (rc = check_f32_bhtd(op, "dAqk", daqk, B, Hv, T, kChunk))) return rc;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query))) return rc;
    if ((rc = check_state_blocks(op, "h", h, geom))) return rc;
    if ((rc = check_state_blocks(op, "dh", dh, geom))) return rc;
    if (query) return FLA_OK;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    KdaDqkwgParams p{geom, view4(q), view4(k), view4(v_new), view4(d_o), view4(dv), view4(dw),
                     static_cast<const float *>(gk->data), gk->stride[0], gk->stride[1], gk->stride[2],
                     static_cast<const elem *>(h->data), static_cast<const elem *>(dh->data),
                     h->stride[0], h->stride[1], h->stride[2], dh->stride[0], dh->stride[1], dh->stride[2],
                     viewf(dq), viewf(dk), viewf(dg), (float)scale, has_daqk ? viewf(daqk) : ViewF{nullptr, 0, 0, 0}};
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hv);
    const size_t smem = ((size_t)3 * kChunk * (V + 8) + (size_t)K * (V + 8)) * 2 + (size_t)6 * K * 4 +
                        (size_t)2 * kChunk * (K + 8) * 2 + (size_t)kChunk * (K + 4) * 4;
    if (K == 128 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_kernel<128, 128>), "kda_bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 64 && V == 64) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_kernel<64, 64>), "kda_bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    if (K == 64 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_kernel<64, 128>), "kda_bwd_dqkwg", grid, smem, p, kDqkwgThreads);
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%lld,%lld) has no kernel; built: (128,128),(64,64),(64,128).", op, (long long)K,
                (long long)V);
}

int kda_wy_impl(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *gk, const fla_tensor *akk,
                const fla_tensor *dw, const fla_tensor *du, const fla_int_array *cu, const fla_int_array *ci, int64_t chunk_size,
                const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dg, const fla_tensor *dakk,
                void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_kda_bwd_wy";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v, nullptr, chunk_size, geom, kElemDtype))) return rc;
    const int bf = dt_bit(kElemDtype);
    const int64_t B = geom.B, Hk = geom.Hk, Hv = geom.Hv, T = geom.T, K = geom.K, V = geom.V;
    if ((rc = check_bhtd(op, "k", k, B, Hk, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "Akk", akk, B, Hv, T, kChunk, bf))) return rc;
    if ((rc = check_bhtd(op, "dw", dw, B, Hv, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "du", du, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "dv", dv, B, Hv, T, V, bf))) return rc;
    FLA_REQUIRE(beta != nullptr && beta->data != nullptr, FLA_ERR_NULL, "%s: beta must be provided.", op);
    if ((rc = check_bht(op, "beta", beta, B, Hv, T, kElemDtype))) return rc;
    if ((rc = check_f32_bhtd(op, "gk", gk, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dk", dk, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dg", dg, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dAkk", dakk, B, Hv, T, kChunk))) return rc;
    if ((rc = check_tensor(db, op, "db", 3, dt_bit(FLA_F32)))) return rc;
    FLA_REQUIRE(db->shape[0] == B && db->shape[1] == Hv && db->shape[2] == T, FLA_ERR_SHAPE, "%s: db must be [%lld,%lld,%lld].",
                op, (long long)B, (long long)Hv, (long long)T);
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    KdaWyParams p{geom, view4(k), view4(v), view4(akk), view4(dw), view4(du), view4(dv), view3(beta),
                  static_cast<const float *>(gk->data), gk->stride[0], gk->stride[1], gk->stride[2],
                  viewf(dk), viewf(dg), viewf(dakk), static_cast<float *>(db->data), db->stride[0], db->stride[1], db->stride[2]};
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hv);
    const size_t smem = ((size_t)kChunk * ((K + 16) + (V + 16) + (K + 8) + (V + 8) + (kChunk + 8))) * 2 + kChunk * 4;
    if (K == 128 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_wy_kernel<128, 128>), "kda_bwd_wy", grid, smem, p, kThreads);
    if (K == 64 && V == 64) FLA_KDA_BWD_LAUNCH((kda_bwd_wy_kernel<64, 64>), "kda_bwd_wy", grid, smem, p, kThreads);
    if (K == 64 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_wy_kernel<64, 128>), "kda_bwd_wy", grid, smem, p, kThreads);
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%lld,%lld) has no kernel; built: (128,128),(64,64),(64,128).", op, (long long)K,
                (long long)V);
}

int kda_dqkwg_wy_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
                      const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v,
                      const fla_tensor *beta, const fla_tensor *akk, const fla_int_array *cu, const fla_int_array *ci, double scale,
                      int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *daqk,
                      const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dakk, void *ws, uint64_t ws_size,
                      hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_kda_bwd_dqkwg_wy";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v_new, nullptr, chunk_size, geom, kElemDtype))) return rc;
    if (d_o != nullptr && d_o->ndim == 4 && geom.Hv > 1 && geom.T <= (1 << 20)) geom.head_fast = d_o->stride[2] > d_o->stride[1] ? 1 : 0;
    const int bf = dt_bit(kElemDtype);
    const int64_t B = geom.B, Hk = geom.Hk, Hv = geom.Hv, T = geom.T, K = geom.K, V = geom.V;
    if ((rc = check_bhtd(op, "q", q, B, Hk, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, B, Hk, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "v_new", v_new, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "d_o", d_o, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "dv2", dv2, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "Akk", akk, B, Hv, T, kChunk, bf))) return rc;
    if ((rc = check_bhtd(op, "dv", dv, B, Hv, T, V, bf))) return rc;
    FLA_REQUIRE(beta != nullptr && beta->data != nullptr, FLA_ERR_NULL, "%s: beta must be provided.", op);
    if ((rc = check_bht(op, "beta", beta, B, Hv, T, kElemDtype))) return rc;
    if ((rc = check_f32_bhtd(op, "gk", gk, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dq", dq, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dk", dk, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dg", dg, B, Hv, T, K))) return rc;
    if ((rc = check_f32_bhtd(op, "dAqk", daqk, B, Hv, T, kChunk))) return rc;
    if ((rc = check_f32_bhtd(op, "dAkk", dakk, B, Hv, T, kChunk))) return rc;
    if ((rc = check_tensor(db, op, "db", 3, dt_bit(FLA_F32)))) return rc;
    FLA_REQUIRE(db->shape[0] == B && db->shape[1] == Hv && db->shape[2] == T, FLA_ERR_SHAPE, "%s: db must be [%lld,%lld,%lld].",
                op, (long long)B, (long long)Hv, (long long)T);
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query))) return rc;
    if ((rc = check_state_blocks(op, "h", h, geom))) return rc;
    if ((rc = check_state_blocks(op, "dh", dh, geom))) return rc;
    if (query) return FLA_OK;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    KdaDqkwgWyParams p{geom, view4(q), view4(k), view4(v_new), view4(d_o), view4(dv2), view4(v), view4(akk), view4(dv), view3(beta),
                       static_cast<const float *>(gk->data), gk->stride[0], gk->stride[1], gk->stride[2],
                       static_cast<const elem *>(h->data), static_cast<const elem *>(dh->data),
                       h->stride[0], h->stride[1], h->stride[2], dh->stride[0], dh->stride[1], dh->stride[2],
                       viewf(dq), viewf(dk), viewf(dg), viewf(daqk), viewf(dakk),
                       static_cast<float *>(db->data), db->stride[0], db->stride[1], db->stride[2], (float)scale, 0};
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hv);
    if (K == 128 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_wy_kernel<128, 128, false>), "kda_bwd_dqkwg_wy", grid, (kda_bwd_fused_smem<128, 128, false>()), p, kDqkwgThreads);
    if (K == 64 && V == 64) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_wy_kernel<64, 64, false>), "kda_bwd_dqkwg_wy", grid, (kda_bwd_fused_smem<64, 64, false>()), p, kDqkwgThreads);
    if (K == 64 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_wy_kernel<64, 128, false>), "kda_bwd_dqkwg_wy", grid, (kda_bwd_fused_smem<64, 128, false>()), p, kDqkwgThreads);
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%lld,%lld) has no kernel; built: (128,128),(64,64),(64,128).", op, (long long)K,
                (long long)V);
}

// chunk_kda_bwd_dqkwg_wy_intra: the three stages after the reverse scan in one launch; dq, dk (fp32, or the element type
// when no two value heads share a key head), dg (reverse running sum taken), dv and dbeta leave final.
int kda_dqkwg_wy_intra_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk,
                            const fla_tensor *h, const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2,
                            const fla_tensor *v, const fla_tensor *beta, const fla_tensor *akk, const fla_int_array *cu,
                            const fla_int_array *ci, double scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
                            const fla_tensor *dg, const fla_tensor *dv, const fla_tensor *db, void *ws, uint64_t ws_size,
                            hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_kda_bwd_dqkwg_wy_intra";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v_new, nullptr, chunk_size, geom, kElemDtype))) return rc;
    if (d_o != nullptr && d_o->ndim == 4 && geom.Hv > 1 && geom.T <= (1 << 20)) geom.head_fast = d_o->stride[2] > d_o->stride[1] ? 1 : 0;
    const int bf = dt_bit(kElemDtype);
    const int64_t B = geom.B, Hk = geom.Hk, Hv = geom.Hv, T = geom.T, K = geom.K, V = geom.V;
    if ((rc = check_bhtd(op, "q", q, B, Hk, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, B, Hk, T, K, bf))) return rc;
    if ((rc = check_bhtd(op, "v_new", v_new, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "d_o", d_o, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "dv2", dv2, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, B, Hv, T, V, bf))) return rc;
    if ((rc = check_bhtd(op, "Akk", akk, B, Hv, T, kChunk, bf))) return rc;
    if ((rc = check_bhtd(op, "dv", dv, B, Hv, T, V, bf))) return rc;
    FLA_REQUIRE(beta != nullptr && beta->data != nullptr, FLA_ERR_NULL, "%s: beta must be provided.", op);
    if ((rc = check_bht(op, "beta", beta, B, Hv, T, kElemDtype))) return rc;
    if ((rc = check_f32_bhtd(op, "gk", gk, B, Hv, T, K))) return rc;
    FLA_REQUIRE(dq != nullptr && dk != nullptr, FLA_ERR_NULL, "%s: dq and dk must be provided.", op);
    FLA_REQUIRE(dq->dtype == dk->dtype, FLA_ERR_DTYPE, "%s: dq and dk must share one dtype.", op);
    const bool out16 = dq->dtype == kElemDtype;
    if (out16) {
        if ((rc = check_bhtd(op, "dq", dq, B, Hv, T, K, bf))) return rc;
        if ((rc = check_bhtd(op, "dk", dk, B, Hv, T, K, bf))) return rc;
    } else {
        if ((rc = check_f32_bhtd(op, "dq", dq, B, Hv, T, K))) return rc;
        if ((rc = check_f32_bhtd(op, "dk", dk, B, Hv, T, K))) return rc;
    }
    if ((rc = check_f32_bhtd(op, "dg", dg, B, Hv, T, K))) return rc;
    if ((rc = check_tensor(db, op, "db", 3, dt_bit(FLA_F32)))) return rc;
    FLA_REQUIRE(db->shape[0] == B && db->shape[1] == Hv && db->shape[2] == T, FLA_ERR_SHAPE, "%s: db must be [%lld,%lld,%lld].",
                op, (long long)B, (long long)Hv, (long long)T);
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query))) return rc;
    if ((rc = check_state_blocks(op, "h", h, geom))) return rc;
    if ((rc = check_state_blocks(op, "dh", dh, geom))) return rc;
    if (query) return FLA_OK;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    const ViewF none{nullptr, 0, 0, 0};
    auto any_view = [](const fla_tensor *t) { return ViewF{static_cast<float *>(t->data), t->stride[0], t->stride[1], t->stride[2]}; };
    KdaDqkwgWyParams p{geom, view4(q), view4(k), view4(v_new), view4(d_o), view4(dv2), view4(v), view4(akk), view4(dv), view3(beta),
                       static_cast<const float *>(gk->data), gk->stride[0], gk->stride[1], gk->stride[2],
                       static_cast<const elem *>(h->data), static_cast<const elem *>(dh->data),
                       h->stride[0], h->stride[1], h->stride[2], dh->stride[0], dh->stride[1], dh->stride[2],
                       any_view(dq), any_view(dk), viewf(dg), none, none,
                       static_cast<float *>(db->data), db->stride[0], db->stride[1], db->stride[2], (float)scale, out16 ? 1 : 0};
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hv);
    if (K == 128 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_wy_kernel<128, 128, true>), "kda_bwd_dqkwg_wy_intra", grid, (kda_bwd_fused_smem<128, 128, true>()), p, kDqkwgThreads);
    if (K == 64 && V == 64) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_wy_kernel<64, 64, true>), "kda_bwd_dqkwg_wy_intra", grid, (kda_bwd_fused_smem<64, 64, true>()), p, kDqkwgThreads);
    if (K == 64 && V == 128) FLA_KDA_BWD_LAUNCH((kda_bwd_dqkwg_wy_kernel<64, 128, true>), "kda_bwd_dqkwg_wy_intra", grid, (kda_bwd_fused_smem<64, 128, true>()), p, kDqkwgThreads);
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%lld,%lld) has no kernel; built: (128,128),(64,64),(64,128).", op, (long long)K,
                (long long)V);
}

}  // namespace
}  // namespace fla

#define FLA_NULL_WS(op) \
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, op ": workspace_size must not be null.")

FLA_ENTRY(fla_chunk_kda_bwd_dav_get_workspace_size)(
    const fla_tensor *v_new, const fla_tensor *d_o, const fla_tensor *Aqk, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dAqk, const fla_tensor *dv,
    uint64_t *workspace_size) {
    FLA_ROUTE_F16(v_new, fla_chunk_kda_bwd_dav_get_workspace_size, v_new, d_o, Aqk, cu_seqlens, chunk_indices, scale, chunk_size, dAqk, dv, workspace_size);
    FLA_NULL_WS("chunk_kda_bwd_dav");
    return fla::guarded([&] { return fla::dav_impl(v_new, d_o, Aqk, cu_seqlens, chunk_indices, scale, chunk_size, dAqk, dv, nullptr, 0, nullptr,
                         workspace_size); });
}
FLA_ENTRY(fla_chunk_kda_bwd_dav)(
    const fla_tensor *v_new, const fla_tensor *d_o, const fla_tensor *Aqk, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dAqk, const fla_tensor *dv,
    void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(v_new, fla_chunk_kda_bwd_dav, v_new, d_o, Aqk, cu_seqlens, chunk_indices, scale, chunk_size, dAqk, dv, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::dav_impl(v_new, d_o, Aqk, cu_seqlens, chunk_indices, scale, chunk_size, dAqk, dv, workspace, workspace_size,
                         static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_kda_bwd_dqkwg_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *dw, const fla_tensor *dg, const fla_tensor *dAqk, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_dqkwg_get_workspace_size, q, k, v_new, gk, h, d_o, dh, dv, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dw, dg, dAqk, workspace_size);
    FLA_NULL_WS("chunk_kda_bwd_dqkwg");
    return fla::guarded([&] { return fla::kda_dqkwg_impl(q, k, v_new, gk, h, d_o, dh, dv, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dw, dg,
                               dAqk, nullptr, 0, nullptr, workspace_size); });
}
FLA_ENTRY(fla_chunk_kda_bwd_dqkwg)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *dw, const fla_tensor *dg, const fla_tensor *dAqk, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_dqkwg, q, k, v_new, gk, h, d_o, dh, dv, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dw, dg, dAqk, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::kda_dqkwg_impl(q, k, v_new, gk, h, d_o, dh, dv, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dw, dg,
                               dAqk, workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_kda_bwd_wy_get_workspace_size)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *gk, const fla_tensor *Akk,
    const fla_tensor *dw, const fla_tensor *du, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dg,
    const fla_tensor *dAkk, uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_chunk_kda_bwd_wy_get_workspace_size, k, v, beta, gk, Akk, dw, du, cu_seqlens, chunk_indices, chunk_size, dk, dv, db, dg, dAkk, workspace_size);
    FLA_NULL_WS("chunk_kda_bwd_wy");
    return fla::guarded([&] { return fla::kda_wy_impl(k, v, beta, gk, Akk, dw, du, cu_seqlens, chunk_indices, chunk_size, dk, dv, db, dg, dAkk, nullptr, 0,
                            nullptr, workspace_size); });
}
FLA_ENTRY(fla_chunk_kda_bwd_wy)(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *gk, const fla_tensor *Akk,
    const fla_tensor *dw, const fla_tensor *du, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dg,
    const fla_tensor *dAkk, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_chunk_kda_bwd_wy, k, v, beta, gk, Akk, dw, du, cu_seqlens, chunk_indices, chunk_size, dk, dv, db, dg, dAkk, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::kda_wy_impl(k, v, beta, gk, Akk, dw, du, cu_seqlens, chunk_indices, chunk_size, dk, dv, db, dg, dAkk, workspace,
                            workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_kda_bwd_dqkwg_wy_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dAqk,
    const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dAkk, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_dqkwg_wy_get_workspace_size, q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dg, dAqk, dv, db, dAkk, workspace_size);
    FLA_NULL_WS("chunk_kda_bwd_dqkwg_wy");
    return fla::guarded([&] { return fla::kda_dqkwg_wy_impl(q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale,
                                  chunk_size, dq, dk, dg, dAqk, dv, db, dAkk, nullptr, 0, nullptr, workspace_size); });
}
FLA_ENTRY(fla_chunk_kda_bwd_dqkwg_wy)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dAqk,
    const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dAkk, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_dqkwg_wy, q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dg, dAqk, dv, db, dAkk, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::kda_dqkwg_wy_impl(q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale,
                                  chunk_size, dq, dk, dg, dAqk, dv, db, dAkk, workspace, workspace_size,
                                  static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_kda_bwd_dqkwg_wy_intra_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dv,
    const fla_tensor *db, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_dqkwg_wy_intra_get_workspace_size, q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dg, dv, db, workspace_size);
    FLA_NULL_WS("chunk_kda_bwd_dqkwg_wy_intra");
    return fla::guarded([&] { return fla::kda_dqkwg_wy_intra_impl(q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale,
                                        chunk_size, dq, dk, dg, dv, db, nullptr, 0, nullptr, workspace_size); });
}
FLA_ENTRY(fla_chunk_kda_bwd_dqkwg_wy_intra)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dv,
    const fla_tensor *db, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_dqkwg_wy_intra, q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale, chunk_size, dq, dk, dg, dv, db, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::kda_dqkwg_wy_intra_impl(q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, cu_seqlens, chunk_indices, scale,
                                        chunk_size, dq, dk, dg, dv, db, workspace, workspace_size,
                                        static_cast<hipStream_t>(stream), nullptr); });
}
