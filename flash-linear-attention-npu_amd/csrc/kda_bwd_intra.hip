// chunk_kda_bwd_intra: intra-chunk part of the KDA backward.
//
// For every chunk and head, with A = tril(dAqk), B = tril(dAkk) (64x64, fp32) and the chunk-local
// cumulated gate g (log2 units):
//     dq_i += sum_{j<=i} A_ij k_j 2^{g_i-g_j}
//     dl_i  = sum_{j<=i} B_ij k_j 2^{g_i-g_j}
//     du_j  = sum_{i>=j} (A_ij q_i + B_ij beta_i k_i) 2^{g_i-g_j}
//     dk_i += beta_i dl_i + du_i ;  db_i += <dl_i, k_i> ;  dg_i += q_i dq'_i + k_i (beta_i dl_i - du_i)
// Each 16-row tile is evaluated against an anchor gate c inside the tile (row 8, or the last valid
// row), 2^{g_i-g_j} = 2^{g_i-c} 2^{c-g_j}, so both factors stay finite for non-increasing gates.
// Golden: torch_custom/fla_npu/test/test_npu_chunk_kda_bwd_intra.py:7-91 (fp32 products, tolerance
// 2e-4), operand order: _aclnn_ctypes.py:1534-1768.
//
// The golden's tolerance rules out bf16 operands, so the products run on the fp32 matrix pipe
// (v_mfma_f32_16x16x4_f32).  One workgroup per (chunk, head); wave r owns row tile r: its "lower"
// products contract over (r+1) tiles and its "upper" product over (4-r) tiles, five in total for
// every wave.  Channels are processed in blocks of 64 so that two workgroups fit in a CU's LDS.
#include "gdn_common.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }
// D[16x16] += A[16x4] B[4x16]: lane l holds A[l%16][l/16], B[l/16][l%16], D[4*(l/16)+e][l%16]
__device__ __forceinline__ f32x4 mfma_f32(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

struct BwdIntraParams {
    ChunkGeom geom;              // Hv = heads, K = head size
    const elem *q, *k;
    const float *gk, *dq, *dk, *dg;
    float *dq_o, *dk_o, *dg_o;
    int64_t sb, sh, st;          // strides of (batch, head, token) of the six gradient tensors [..,K]
    int64_t q_sb, q_sh, q_st;    // of q and k, which may have fewer heads (head h reads key head h / rep)
    int64_t g_sb, g_sh, g_st;    // of gk
    int rep;
    View3 beta;
    const float *db;
    float *db_o;
    int64_t db_sb, db_sh, db_st;
    const float *daqk, *dakk;    // [..,64]
    int64_t m_sb, m_sh, m_st;
    int cumsum_dg;               // 1: dg leaves as its reverse running sum over the tokens of the chunk
    int out16;                   // 1: dq_o and dk_o point at 16-bit elements (same strides in elements)
};

template <int KC>
__global__ void __launch_bounds__(kThreads) kda_bwd_intra_kernel(const BwdIntraParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pa = 68, pg = KC + 4, pk = KC + 8;
    float *aqS = reinterpret_cast<float *>(smem);   // [64][pa] tril(dAqk)
    float *akS = aqS + kChunk * pa;                 // [64][pa] tril(dAkk)
    float *gS = akS + kChunk * pa;                  // [64][pg]
    float *bS = gS + kChunk * pg;                   // [64]
    elem *qS = reinterpret_cast<elem *>(bS + kChunk);
    elem *kS = qS + kChunk * pk;

    int c, h;
    block_chunk_head(p.geom, c, h);
    const int b = blockIdx.z;
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x;
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const int K = p.geom.K;

    {   // masked score gradients: branch-free loads (clamped row), all issued before the first LDS write
        const int64_t mbase = b * p.m_sb + h * p.m_sh + (int64_t)start * p.m_st;
        f32x4 a[4], k4[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const int idx = m * kThreads + tid;
            const int r = min(idx >> 4, len - 1), c4 = (idx & 15) << 2;
            a[m] = *reinterpret_cast<const f32x4 *>(p.daqk + mbase + (int64_t)r * p.m_st + c4);
            k4[m] = *reinterpret_cast<const f32x4 *>(p.dakk + mbase + (int64_t)r * p.m_st + c4);
        }
        const float bt = tid < kChunk ? load_scalar(p.beta, b, h, start + min(tid, len - 1)) : 0.f;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const int idx = m * kThreads + tid;
            const int r = idx >> 4, c4 = (idx & 15) << 2;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (c4 + e > r || r >= len) a[m][e] = k4[m][e] = 0.f;
            *reinterpret_cast<f32x4 *>(aqS + r * pa + c4) = a[m];
            *reinterpret_cast<f32x4 *>(akS + r * pa + c4) = k4[m];
        }
        if (tid < kChunk) bS[tid] = tid < len ? bt : 0.f;
    }

    const int r0 = 16 * wave_id();
    const int row_end = min(r0 + 16, len);
    const int anchor = min(r0 + 8, row_end - 1);
    const int64_t base = b * p.sb + h * p.sh + (int64_t)start * p.st;
    const int64_t qbase = b * p.q_sb + (h / p.rep) * p.q_sh + (int64_t)start * p.q_st;
    const int64_t gbase = b * p.g_sb + h * p.g_sh + (int64_t)start * p.g_st;
    f32x4 dbacc = {0.f, 0.f, 0.f, 0.f};

    for (int ch0 = 0; ch0 < K; ch0 += KC) {
        __syncthreads();
        f32x4 old[3][kChunk * (KC / 4) / kThreads];
        {
            TileCopy<kThreads, kChunk, KC> tq, tk;
            tq.fetch(p.q + qbase + ch0, p.q_st, len, tid);
            tk.fetch(p.k + qbase + ch0, p.q_st, len, tid);
            constexpr int GN = kChunk * (KC / 4) / kThreads;
            f32x4 gv[GN];
#pragma unroll
            for (int m = 0; m < GN; ++m) {   // padded rows repeat the last gate row
                const int idx = m * kThreads + tid;
                const int r = min(idx / (KC / 4), len - 1), c4 = (idx % (KC / 4)) * 4;
                gv[m] = *reinterpret_cast<const f32x4 *>(p.gk + gbase + (int64_t)r * p.g_st + ch0 + c4);
            }
#pragma unroll
            for (int t = 0; t < 3; ++t)
#pragma unroll
                for (int m = 0; m < GN; ++m) {   // the incoming gradients of the block, consumed after the products
                    const int idx = m * kThreads + tid;
                    const int r = min(idx / (KC / 4), len - 1), c4 = (idx % (KC / 4)) * 4;
                    old[t][m] = *reinterpret_cast<const f32x4 *>((t == 0 ? p.dq : t == 1 ? p.dk : p.dg) + base + (int64_t)r * p.st + ch0 + c4);
                }
            tq.commit(qS, pk, len, tid);
            tk.commit(kS, pk, len, tid);
#pragma unroll
            for (int m = 0; m < GN; ++m) {
                const int idx = m * kThreads + tid;
                *reinterpret_cast<f32x4 *>(gS + (idx / (KC / 4)) * pg + (idx % (KC / 4)) * 4) = gv[m];
            }
        }
        __syncthreads();
        // what this wave adds to dq, dk, dg of its 16 rows x KC channels, kept in registers until the products of the
        // channel block are done; a row tile without a token (wave-uniform) adds nothing
        f32x4 inc[KC / 16][3];
#pragma unroll
        for (int nt = 0; nt < KC / 16; ++nt) inc[nt][0] = inc[nt][1] = inc[nt][2] = f32x4{0.f, 0.f, 0.f, 0.f};
        const int nsteps_lo = (row_end + 3) >> 2;   // contraction over tokens j < row_end, four at a time
        if (r0 < len) {
#pragma unroll
            for (int nt = 0; nt < KC / 16; ++nt) {
                const int ch = 16 * nt + li;
                const float ca = gS[anchor * pg + ch];
                f32x4 D1 = {0.f, 0.f, 0.f, 0.f}, D2 = D1, D3 = D1;
                for (int js = 0; js < nsteps_lo; ++js) {
                    const int j = 4 * js + lg;
                    const float bval = (float)kS[j * pk + ch] * ex2(ca - gS[j * pg + ch]);
                    D1 = mfma_f32(aqS[(r0 + li) * pa + j], bval, D1);
                    D2 = mfma_f32(akS[(r0 + li) * pa + j], bval, D2);
                }
                for (int is = r0 >> 2; is < 16; ++is) {
                    const int i = 4 * is + lg;
                    const float fw = ex2(gS[i * pg + ch] - ca);
                    const float kk = (float)kS[i * pk + ch];
                    D3 = mfma_f32(aqS[i * pa + r0 + li], (float)qS[i * pk + ch] * fw, D3);
                    D3 = mfma_f32(akS[i * pa + r0 + li], kk * bS[i] * fw, D3);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = r0 + 4 * lg + e;
                    if (i < len) {
                        const float gi = gS[i * pg + ch];
                        const float up = ex2(gi - ca), down = ex2(ca - gi);
                        const float dqd = D1[e] * up, dl = D2[e] * up, du = D3[e] * down;
                        const float qi = (float)qS[i * pk + ch], ki = (float)kS[i * pk + ch];
                        const float bdl = bS[i] * dl;
                        inc[nt][0][e] = dqd;
                        inc[nt][1][e] = bdl + du;
                        inc[nt][2][e] = qi * dqd + ki * (bdl - du);
                        dbacc[e] += dl * ki;
                    }
                }
            }
        }
        // The increments leave through an fp32 tile laid over the q and k tiles (dead once every wave is past its
        // products), one gradient at a time, and are added to memory over whole rows, 16 bytes per lane: from the
        // accumulator layout the fp32 gradients moved in and out as 64-byte pieces.
        float *xS = reinterpret_cast<float *>(qS);
        constexpr int px = KC + 4;
        static_assert((size_t)kChunk * px * 4 <= (size_t)2 * kChunk * pk * 2, "the staging tile must fit the q and k tiles");
        float *gout[3] = {p.dq_o, p.dk_o, p.dg_o};
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            __syncthreads();
#pragma unroll
            for (int nt = 0; nt < KC / 16; ++nt)
#pragma unroll
                for (int e = 0; e < 4; ++e) xS[(r0 + 4 * lg + e) * px + 16 * nt + li] = inc[nt][t][e];
            __syncthreads();
            constexpr int PN = kChunk * (KC / 4) / kThreads;
            if (t == 2 && p.cumsum_dg) {
                // The gate gradient is complete with this kernel's part, and a workgroup holds a whole chunk of it: the
                // reverse running sum over the chunk's tokens (what follows in the composition) is taken here, column by
                // column in the tile, instead of by a pass of its own over memory.
#pragma unroll
                for (int m = 0; m < PN; ++m) {
                    const int idx = m * kThreads + tid;
                    const int r = idx / (KC / 4), c4 = (idx % (KC / 4)) * 4;
                    f32x4 v = old[t][m] + *reinterpret_cast<const f32x4 *>(xS + r * px + c4);
                    if (r >= len) v = f32x4{0.f, 0.f, 0.f, 0.f};
                    *reinterpret_cast<f32x4 *>(xS + r * px + c4) = v;
                }
                __syncthreads();
                constexpr int SEGS = kThreads / KC, RS = kChunk / SEGS;   // a thread sums RS rows of one column
                const int col = tid % KC, seg = tid / KC;
                float *tot = gS;                                          // the gates of this block are no longer read
                float run = 0.f;
#pragma unroll
                for (int j = RS - 1; j >= 0; --j) {
                    float *x = xS + (seg * RS + j) * px + col;
                    run += *x;
                    *x = run;
                }
                tot[seg * KC + col] = run;
                __syncthreads();
                float later = 0.f;
#pragma unroll
                for (int s2 = 1; s2 < SEGS; ++s2)
                    if (seg + s2 < SEGS) later += tot[(seg + s2) * KC + col];
#pragma unroll
                for (int j = 0; j < RS; ++j) xS[(seg * RS + j) * px + col] += later;
                __syncthreads();
#pragma unroll
                for (int m = 0; m < PN; ++m) {
                    const int idx = m * kThreads + tid;
                    const int r = idx / (KC / 4), c4 = (idx % (KC / 4)) * 4;
                    if (r < len)
                        *reinterpret_cast<f32x4 *>(gout[t] + base + (int64_t)r * p.st + ch0 + c4) =
                            *reinterpret_cast<const f32x4 *>(xS + r * px + c4);
                }
                continue;
            }
#pragma unroll
            for (int m = 0; m < PN; ++m) {
                const int idx = m * kThreads + tid;
                const int r = idx / (KC / 4), c4 = (idx % (KC / 4)) * 4;
                if (r < len) {
                    const int64_t off = base + (int64_t)r * p.st + ch0 + c4;
                    const f32x4 sum = old[t][m] + *reinterpret_cast<const f32x4 *>(xS + r * px + c4);
                    if (t < 2 && p.out16) *reinterpret_cast<elemx4 *>(reinterpret_cast<elem *>(gout[t]) + off) = cvt4(sum);
                    else *reinterpret_cast<f32x4 *>(gout[t] + off) = sum;
                }
            }
        }
    }
    if (r0 < len) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float s = group_sum<16>(dbacc[e]);
            const int i = r0 + 4 * lg + e;
            if (li == 0 && i < len) {
                const int64_t off = b * p.db_sb + h * p.db_sh + (int64_t)(start + i) * p.db_st;
                p.db_o[off] = p.db[off] + s;
            }
        }
    }
}

template <int KC>
int launch_bwd_intra(const BwdIntraParams &p, hipStream_t stream) {
    const size_t smem = (size_t)kChunk * (2 * 68 + (KC + 4) + 1) * 4 + (size_t)2 * kChunk * (KC + 8) * 2;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kda_bwd_intra_kernel<KC>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("kda_bwd_intra", stream, (kda_bwd_intra_kernel<KC>), chunk_head_grid(p.geom, p.geom.NT, p.geom.Hv), dim3(kThreads), smem,
               stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int bwd_intra_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta,
                   const fla_tensor *daqk, const fla_tensor *dakk, const fla_tensor *dq, const fla_tensor *dk,
                   const fla_tensor *db, const fla_tensor *dg, const fla_int_array *cu, const fla_int_array *ci,
                   int64_t chunk_size, bool safe_gate, const char *layout, const fla_tensor *dq_o, const fla_tensor *dk_o,
                   const fla_tensor *db_o, const fla_tensor *dg_o, bool cumsum_dg, void *ws, uint64_t ws_size,
                   hipStream_t stream, uint64_t *query) {
    const char *op = cumsum_dg ? "chunk_kda_bwd_intra_cumsum" : "chunk_kda_bwd_intra";
    FLA_REQUIRE(layout != nullptr, FLA_ERR_NULL, "%s: layout must not be null.", op);
    int ib, ih, it;
    if (!strcmp(layout, "BSND")) { ib = 0; it = 1; ih = 2; }
    else if (!strcmp(layout, "BNSD")) { ib = 0; ih = 1; it = 2; }
    else if (!strcmp(layout, "TND")) { ib = -1; it = 0; ih = 1; }
    else return fail(FLA_ERR_UNSUPPORTED, "%s: supports dense BSND/BNSD or varlen TND.", op);
    FLA_REQUIRE(safe_gate, FLA_ERR_UNSUPPORTED, "%s: safe_gate=False is reserved but not supported in v1.", op);
    FLA_REQUIRE(chunk_size == kChunk, FLA_ERR_UNSUPPORTED, "%s: chunk_size must be 64.", op);
    const int rank = ib < 0 ? 3 : 4;
    int rc;
    if ((rc = check_tensor(q, op, "q", rank, dt_bit(kElemDtype)))) return rc;
    if ((rc = check_tensor(k, op, "k", rank, dt_bit(kElemDtype)))) return rc;
    // The reference demands contiguous tensors of one layout.  Here every [..,K] tensor may be any strided view of that
    // index order with a unit innermost stride and 16-byte aligned rows; q and k may carry fewer heads than the gate
    // (grouped value heads: head h of gk and of the gradients reads key head h / (H / Hq)); the six gradient tensors
    // share one set of strides, and each output may be its own input.
    const fla_tensor *grads[] = {dq, dk, dg, dq_o, dk_o, dg_o};
    const char *gradn[] = {"dq", "dk", "dg", "dq_out", "dk_out", "dg_out"};
    if ((rc = check_tensor(gk, op, "gk", rank, dt_bit(FLA_F32)))) return rc;
    const int64_t B = ib < 0 ? 1 : gk->shape[ib], H = gk->shape[ih], T = gk->shape[it], K = gk->shape[rank - 1];
    auto strided_ok = [&](const fla_tensor *t, int64_t heads, int64_t al) {
        return (ib < 0 || t->shape[ib] == B) && t->shape[ih] == heads && t->shape[it] == T && t->shape[rank - 1] == K &&
               inner_unit(t) && (ib < 0 || t->stride[ib] % al == 0) && t->stride[ih] % al == 0 && t->stride[it] % al == 0 &&
               t->stride[it] >= 0 && reinterpret_cast<uintptr_t>(t->data) % 16 == 0;
    };
    // The library-only form that also sums dg may hand dq_out and dk_out over in the element type of q: they are final
    // with this stage, and the conversion that follows in a training step would read and write them once more.
    const bool out16 = cumsum_dg && dq_o != nullptr && dk_o != nullptr && dq_o->dtype == kElemDtype && dk_o->dtype == kElemDtype;
    for (int i = 0; i < 6; ++i) {
        const bool narrow = out16 && (i == 3 || i == 4);
        if ((rc = check_tensor(grads[i], op, gradn[i], rank, dt_bit(narrow ? kElemDtype : FLA_F32)))) return rc;
        FLA_REQUIRE(strided_ok(grads[i], H, narrow ? 8 : 4), FLA_ERR_SHAPE,
                    "%s: %s must have the shape of gk, a unit innermost stride and 16-byte aligned rows.", op, gradn[i]);
        FLA_REQUIRE((ib < 0 || grads[i]->stride[ib] == dq->stride[ib]) && grads[i]->stride[ih] == dq->stride[ih] &&
                        grads[i]->stride[it] == dq->stride[it],
                    FLA_ERR_SHAPE, "%s: dq, dk, dg and their outputs must share one set of strides.", op);
    }
    FLA_REQUIRE(strided_ok(gk, H, 4), FLA_ERR_SHAPE, "%s: gk needs a unit innermost stride and 16-byte aligned rows.", op);
    const int64_t Hq = q->shape[ih];
    FLA_REQUIRE(Hq > 0 && H % Hq == 0, FLA_ERR_SHAPE, "%s: heads of gk (%lld) must be a multiple of the heads of q (%lld).", op,
                (long long)H, (long long)Hq);
    FLA_REQUIRE(strided_ok(q, Hq, 8) && strided_ok(k, Hq, 8), FLA_ERR_SHAPE,
                "%s: q and k must be [..,%lld heads,..,K] with a unit innermost stride and 16-byte aligned rows.", op, (long long)Hq);
    FLA_REQUIRE((ib < 0 || q->stride[ib] == k->stride[ib]) && q->stride[ih] == k->stride[ih] && q->stride[it] == k->stride[it],
                FLA_ERR_SHAPE, "%s: q and k must share one set of strides.", op);
    FLA_REQUIRE(B > 0 && H > 0 && T > 0, FLA_ERR_SHAPE, "%s: B/H/T must be positive.", op);
    FLA_REQUIRE(K == 64 || K == 128 || K == 256, FLA_ERR_UNSUPPORTED, "%s: K must be 64, 128 or 256.", op);
    FLA_REQUIRE(B < 65536 && H < 65536 && T < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents too large.", op);
    if ((rc = check_tensor(beta, op, "beta", rank - 1, dt_bit(kElemDtype) | dt_bit(FLA_F32)))) return rc;
    const fla_tensor *sc[] = {beta, db, db_o};
    const char *scn[] = {"beta", "db", "db_out"};
    for (int i = 0; i < 3; ++i) {
        if (i && (rc = check_tensor(sc[i], op, scn[i], rank - 1, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE((ib < 0 || sc[i]->shape[ib] == B) && sc[i]->shape[ih] == H && sc[i]->shape[it] == T, FLA_ERR_SHAPE,
                    "%s: beta/db shape must match the selected layout.", op);
    }
    FLA_REQUIRE((ib < 0 || db->stride[ib] == db_o->stride[ib]) && db->stride[ih] == db_o->stride[ih] &&
                    db->stride[it] == db_o->stride[it],
                FLA_ERR_SHAPE, "%s: db and db_out must share one set of strides.", op);
    const fla_tensor *mats[] = {daqk, dakk};
    for (int i = 0; i < 2; ++i) {
        if ((rc = check_tensor(mats[i], op, i ? "dAkk" : "dAqk", rank, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE((ib < 0 || mats[i]->shape[ib] == B) && mats[i]->shape[ih] == H && mats[i]->shape[it] == T &&
                        mats[i]->shape[rank - 1] == kChunk && inner_unit(mats[i]) && mats[i]->stride[it] % 4 == 0 &&
                        mats[i]->stride[ih] % 4 == 0 && (ib < 0 || mats[i]->stride[ib] % 4 == 0) &&
                        reinterpret_cast<uintptr_t>(mats[i]->data) % 16 == 0,
                    FLA_ERR_SHAPE, "%s: dAqk/dAkk shape must match the selected layout.", op);
        FLA_REQUIRE((ib < 0 || mats[i]->stride[ib] == daqk->stride[ib]) && mats[i]->stride[ih] == daqk->stride[ih] &&
                        mats[i]->stride[it] == daqk->stride[it],
                    FLA_ERR_SHAPE, "%s: dAqk and dAkk must share one set of strides.", op);
    }
    const bool varlen = cu && cu->data && cu->size;
    // (the reference rejects packed BNSD input; with strided views it is the same addressing as BSND with B = 1)
    FLA_REQUIRE(varlen || ib >= 0, FLA_ERR_SHAPE, "%s: TND requires cu_seqlens.", op);
    FLA_REQUIRE(varlen || !(ci && ci->data && ci->size), FLA_ERR_SHAPE, "%s: chunk_indices requires cu_seqlens.", op);

    ChunkGeom geom{};
    geom.B = (int)B;
    geom.T = (int)T;
    geom.Hk = geom.Hv = (int)H;
    geom.K = geom.V = (int)K;
    geom.NT = (int)((T + kChunk - 1) / kChunk);
    geom.N = (int)B;
    Varlen vl;
    if ((rc = build_varlen(vl, op, cu, ci, kChunk, T))) return rc;
    FLA_REQUIRE(!vl.enabled || B == 1, FLA_ERR_SHAPE, "%s: packed rank-4 input requires B=1.", op);
    if (vl.enabled) {
        geom.NT = vl.NT;
        geom.N = vl.N;
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
    if (geom.NT == 0) return FLA_OK;

    BwdIntraParams p{};
    p.geom = geom;
    p.q = static_cast<const elem *>(q->data);
    p.k = static_cast<const elem *>(k->data);
    p.gk = static_cast<const float *>(gk->data);
    p.dq = static_cast<const float *>(dq->data);
    p.dk = static_cast<const float *>(dk->data);
    p.dg = static_cast<const float *>(dg->data);
    p.dq_o = static_cast<float *>(dq_o->data);
    p.dk_o = static_cast<float *>(dk_o->data);
    p.dg_o = static_cast<float *>(dg_o->data);
    p.sb = ib < 0 ? 0 : dq->stride[ib];
    p.sh = dq->stride[ih];
    p.st = dq->stride[it];
    p.q_sb = ib < 0 ? 0 : q->stride[ib];
    p.q_sh = q->stride[ih];
    p.q_st = q->stride[it];
    p.g_sb = ib < 0 ? 0 : gk->stride[ib];
    p.g_sh = gk->stride[ih];
    p.g_st = gk->stride[it];
    p.rep = (int)(H / Hq);
    p.beta = View3{beta->data, ib < 0 ? 0 : beta->stride[ib], beta->stride[ih], beta->stride[it], beta->dtype == FLA_F32 ? 0 : 1};
    p.db = static_cast<const float *>(db->data);
    p.db_o = static_cast<float *>(db_o->data);
    p.db_sb = ib < 0 ? 0 : db->stride[ib];
    p.db_sh = db->stride[ih];
    p.db_st = db->stride[it];
    p.daqk = static_cast<const float *>(daqk->data);
    p.dakk = static_cast<const float *>(dakk->data);
    p.m_sb = ib < 0 ? 0 : daqk->stride[ib];
    p.m_sh = daqk->stride[ih];
    p.m_st = daqk->stride[it];
    FLA_REQUIRE(p.q_st < (1 << 24), FLA_ERR_SHAPE, "%s: token stride of q and k must be below 2^24 elements.", op);
    p.cumsum_dg = cumsum_dg ? 1 : 0;
    // gradients laid out token-major (a token's row holds every head): neighbouring workgroups take the heads of one chunk
    p.geom.head_fast = H > 1 && p.st > p.sh && p.geom.NT <= 65535 ? 1 : 0;
    p.out16 = out16 ? 1 : 0;
    return launch_bwd_intra<64>(p, stream);   // 64-channel blocks: two workgroups fit on a CU
}

}  // namespace
}  // namespace fla

FLA_ENTRY(fla_chunk_kda_bwd_intra_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta, const fla_tensor *dAqk,
    const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *db, const fla_tensor *dg,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate,
    const char *layout, const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_intra_get_workspace_size, q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate, layout, dq_out, dk_out, db_out, dg_out, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "chunk_kda_bwd_intra: workspace_size must not be null.");
    return fla::guarded([&] { return fla::bwd_intra_impl(q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate,
                               layout, dq_out, dk_out, db_out, dg_out, false, nullptr, 0, nullptr, workspace_size); });
}

FLA_ENTRY(fla_chunk_kda_bwd_intra)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta, const fla_tensor *dAqk,
    const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *db, const fla_tensor *dg,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate,
    const char *layout, const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_intra, q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate, layout, dq_out, dk_out, db_out, dg_out, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::bwd_intra_impl(q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate,
                               layout, dq_out, dk_out, db_out, dg_out, false, workspace, workspace_size,
                               static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_kda_bwd_intra_cumsum_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta, const fla_tensor *dAqk,
    const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *db, const fla_tensor *dg,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate,
    const char *layout, const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_intra_cumsum_get_workspace_size, q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate, layout, dq_out, dk_out, db_out, dg_out, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "chunk_kda_bwd_intra_cumsum: workspace_size must not be null.");
    return fla::guarded([&] { return fla::bwd_intra_impl(q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate,
                               layout, dq_out, dk_out, db_out, dg_out, true, nullptr, 0, nullptr, workspace_size); });
}

FLA_ENTRY(fla_chunk_kda_bwd_intra_cumsum)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta, const fla_tensor *dAqk,
    const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *db, const fla_tensor *dg,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate,
    const char *layout, const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_kda_bwd_intra_cumsum, q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate, layout, dq_out, dk_out, db_out, dg_out, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::bwd_intra_impl(q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, cu_seqlens, chunk_indices, chunk_size, safe_gate,
                               layout, dq_out, dk_out, db_out, dg_out, true, workspace, workspace_size,
                               static_cast<hipStream_t>(stream), nullptr); });
}
