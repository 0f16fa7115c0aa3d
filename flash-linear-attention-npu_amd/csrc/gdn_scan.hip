// chunk_gated_delta_rule_fwd_h: the sequential inter-chunk state scan.
//
// One 256-thread workgroup per (sequence, value head, 64*CT-column slab of V)
// walks the chunks of its sequence.  Wave w owns 16*CT columns of V for ALL K
// rows of the state, so the fp32 state lives in accumulator registers for the
// whole sequence and never touches LDS or HBM between chunks:
//     wh     = w_i . h          (A = w tile in LDS, B = state registers as bf16)
//     v_new  = u_i - wh
//     h     <- e^{g_last} h + k_i^T . (v_new * e^{g_last - g})
//              (A = k tile read with transposing LDS loads, B = v_new registers)
// Per chunk the workgroup stages w, k and its u slab once; h (state at chunk
// start) and v_new are emitted as bf16, the final state as fp32.
// Stage math: chunk_gated_delta_rule_fwd_h/README.md:16-30,52-61; kernel
// op_kernel/gemm/kernel/gdn_fwd_h_kernel.hpp:441-753.
#include "gdn_common.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;

struct ScanParams {
    ChunkGeom geom;
    View4 k, w, u, v_new;
    View3 g;             // scalar gate (natural log), or p == null
    const float *gk;     // per-channel gate [B,Hv,T,K] f32 (log2; k then already carries 2^{gk_last - gk}), or null
    int64_t gk_sb, gk_sh, gk_st;
    const void *h0;      // [N,Hv,K,V] or [N,Hv,V,K], fp32 or the element type, or null
    void *hT;            // final state, same layout and type, or null
    int state_elem;      // 1: h0 / hT hold the element type (the carry itself stays fp32)
    int sub;             // 64-token steps per chunk: 1, or 2 for 128-token chunks (g is cumulated over the whole chunk)
    elem *h;             // [B,Hv,NT,K,V] (or V,K) bf16, or null
    int64_t h_sb, h_sh, h_sc;
    int64_t s_sn, s_sh;  // strides of h0 / hT over (sequence, head)
    int v_first;         // state blocks are [V][K] instead of [K][V]
};

template <int K, int CT> struct FwdHSmem {
    static constexpr int VS = 64 * CT;
    static constexpr int pw = K + 8, pk = K + 16, pu = VS + 16;
    static constexpr size_t w_off = 0;
    static constexpr size_t k_off = w_off + (size_t)kChunk * pw * 2;
    static constexpr size_t u_off = k_off + (size_t)kChunk * pk * 2;
    static constexpr size_t g_off = u_off + (size_t)kChunk * pu * 2;
    static constexpr size_t d_off = g_off + (size_t)kChunk * 4;          // [K] per-channel decay 2^{gk_last} of the chunk
    static constexpr size_t buf_bytes = d_off + (size_t)K * 4;
    static constexpr bool kStage = CT == 1;                              // wider slabs leave no LDS for the staging
    static constexpr int ps = VS + 8;                                    // pitch of the h staging tiles
    static constexpr size_t stage_off = 2 * buf_bytes;                   // two [K][ps] tiles of the emitted h
    static constexpr size_t stage_bytes = kStage ? (size_t)K * ps * 2 : 0;
    static constexpr size_t vstage_off = stage_off + 2 * stage_bytes;    // two [kChunk][ps] tiles of v_new
    static constexpr size_t vstage_bytes = kStage ? (size_t)kChunk * ps * 2 : 0;
    static constexpr size_t bytes = vstage_off + 2 * vstage_bytes;
};

// 512 threads: waves 0-3 compute chunk c from LDS buffer c&1 while waves 4-7 copy the tiles of chunk
// c+1 into the other buffer and have those of chunk c+2 in flight; one barrier per chunk, which waits for LDS
// traffic only.  The final state leaves from registers; v_new and the per-chunk state h go through LDS tiles and are
// written out by the loader waves one chunk later, as whole 128-byte rows (written from the accumulator layout they
// would leave as 32-byte pieces of eight different rows per store, which cost 0.19 ms of a 0.48 ms launch at B=4,
// T=8192, H=32; the 128-column slab form has no LDS left for the tiles and stores from registers).
template <int K, int CT>
__global__ void __launch_bounds__(512) fwd_h_kernel(const ScanParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    typedef FwdHSmem<K, CT> L;
    constexpr int VS = L::VS, pw = L::pw, pk = L::pk, pu = L::pu;
    constexpr int KT = K / 16, KS = K / 32;

    int slab, hv, n;
    chain_of_block(slab, hv, n);
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    const int V = p.geom.V;
    int b = n, bos = 0, eos = p.geom.T, chunk0 = 0;
    if (p.geom.cu != nullptr) {
        b = 0;
        bos = p.geom.cu[n];
        eos = p.geom.cu[n + 1];
        chunk0 = p.geom.choff[n];
    }
    const int nchunks = (eos - bos + kChunk - 1) / kChunk;
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh;
    const elem *wg = static_cast<const elem *>(p.w.p) + b * p.w.sb + hv * p.w.sh;
    const elem *ug = static_cast<const elem *>(p.u.p) + b * p.u.sb + hv * p.u.sh + slab * VS;

    if (wave_id() >= 4) {
        // ------------------------------- loader waves -------------------------------------------
        const int tid = threadIdx.x - kThreads;
        // Two register sets: while step c is computed, the tiles of step c + 1 are committed to LDS and those of step
        // c + 2 are on their way.  Past the last step the loads re-read the last one (never committed), so that the same
        // number of operations lies between a load and the commit that waits for it in every step.
        struct Tiles {
            TileCopy<kThreads, kChunk, K> tw, tk;
            TileCopy<kThreads, kChunk, VS> tu;
            float gv, dk;
        };
        Tiles t0, t1;
        auto fetch = [&](Tiles &t, int c) {
            c = min(c, nchunks - 1);
            const int start = bos + c * kChunk;
            const int len = min(kChunk, eos - start);
            t.tw.fetch(wg + (int64_t)start * p.w.st, p.w.st, len, tid);
            t.tk.fetch(kg + (int64_t)start * p.k.st, p.k.st, len, tid);
            t.tu.fetch(ug + (int64_t)start * p.u.st, p.u.st, len, tid);
            t.gv = 0.f;
            t.dk = 1.f;
            if (p.g.p) t.gv = load_scalar(p.g, b, hv, start + min(tid, len - 1));
            if (p.gk) {   // the decay of the whole chunk, 2^{gk at its last token} (a 128-token chunk: of both steps)
                const int chunk_end = min(bos + (c / p.sub + 1) * p.sub * kChunk, eos);
                t.dk = __builtin_amdgcn_exp2f(p.gk[b * p.gk_sb + hv * p.gk_sh + (int64_t)(chunk_end - 1) * p.gk_st + min(tid, K - 1)]);
            }
        };
        auto commit = [&](const Tiles &t, int c) {
            unsigned char *buf = smem + (c & 1) * L::buf_bytes;
            const int len = min(kChunk, eos - (bos + c * kChunk));
            t.tw.commit(reinterpret_cast<elem *>(buf + L::w_off), pw, len, tid);
            t.tk.commit(reinterpret_cast<elem *>(buf + L::k_off), pk, len, tid);
            t.tu.commit(reinterpret_cast<elem *>(buf + L::u_off), pu, len, tid);
            if (tid < kChunk) reinterpret_cast<float *>(buf + L::g_off)[tid] = tid < len ? t.gv : 0.f;
            if (tid < K) reinterpret_cast<float *>(buf + L::d_off)[tid] = t.dk;
        };
        const bool stage_h = L::kStage && p.h != nullptr && !p.v_first;
        auto store_h = [&](int c) {   // staged state at the start of step c (a chunk start) -> h[.., chunk, :, slab columns]
            if (c % p.sub != 0) return;
            const int cc = c / p.sub;
            const elem *st = reinterpret_cast<const elem *>(smem + L::stage_off + (cc & 1) * L::stage_bytes);
            elem *hg = p.h + b * p.h_sb + hv * p.h_sh + (int64_t)(chunk0 + cc) * p.h_sc + slab * VS;
#pragma unroll
            for (int m = 0; m < K * (VS / 8) / kThreads; ++m) {
                const int idx = m * kThreads + tid;
                const int r = idx / (VS / 8), c8 = (idx % (VS / 8)) << 3;
                *reinterpret_cast<u32x4 *>(hg + (int64_t)r * V + c8) = *reinterpret_cast<const u32x4 *>(st + r * L::ps + c8);
            }
        };
        elem *vnew_g = static_cast<elem *>(const_cast<void *>(p.v_new.p)) + b * p.v_new.sb + hv * p.v_new.sh + slab * VS;
        auto store_v = [&](int c) {   // staged v_new of chunk c -> memory, rows of the valid tokens only
            const elem *st = reinterpret_cast<const elem *>(smem + L::vstage_off + (c & 1) * L::vstage_bytes);
            const int start = bos + c * kChunk;
            const int len = min(kChunk, eos - start);
#pragma unroll
            for (int m = 0; m < kChunk * (VS / 8) / kThreads; ++m) {
                const int idx = m * kThreads + tid;
                const int r = idx / (VS / 8), c8 = (idx % (VS / 8)) << 3;
                if (r < len)
                    *reinterpret_cast<u32x4 *>(vnew_g + (int64_t)(start + r) * p.v_new.st + c8) =
                        *reinterpret_cast<const u32x4 *>(st + r * L::ps + c8);
            }
        };
        // one step: `ahead` takes the tiles of step c + 2, `next` holds those of step c + 1.  The stores go last: a
        // commit waits for everything issued before the loads it needs, and by the next commit they are a step old.
        auto step = [&](Tiles &ahead, const Tiles &next, int c) {
            fetch(ahead, c + 2);
            if (c + 1 < nchunks) commit(next, c + 1);
            if (L::kStage && c > 0) store_v(c - 1);
            if (stage_h && c > 0) store_h(c - 1);
            lds_barrier();   // the loads of step c + 2 stay in flight
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
        if (L::kStage && nchunks > 0) store_v(nchunks - 1);
        if (stage_h && nchunks > 0) store_h(nchunks - 1);
        return;
    }

    // --------------------------------- compute waves ---------------------------------------------
    const int wv = wave_id();
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const int vcol0 = slab * VS + wv * 16 * CT;  // first V column of this wave

    // state element (kk = 16*kt + 4*lg + e, v = vcol0 + 16*ct + li)
    f32x4 hacc[KT][CT];
    auto state_off = [&](int kk, int v) -> int64_t { return p.v_first ? (int64_t)v * K + kk : (int64_t)kk * V + v; };
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
            if (p.h0) {
                const int64_t base = n * p.s_sn + hv * p.s_sh;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int64_t off = base + state_off(16 * kt + 4 * lg + e, vcol0 + 16 * ct + li);
                    a[e] = p.state_elem ? (float)static_cast<const elem *>(p.h0)[off] : static_cast<const float *>(p.h0)[off];
                }
            }
            hacc[kt][ct] = a;
        }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // initial state loaded before the loop (vmcnt(0))
    char *vng = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.v_new.p)) + b * p.v_new.sb + hv * p.v_new.sh + vcol0);
    elemx8 hB[KS][CT];
    float gbase = 0.f;
    __syncthreads();

    for (int c = 0; c < nchunks; ++c) {
        const unsigned char *buf = smem + (c & 1) * L::buf_bytes;
        const elem *wS = reinterpret_cast<const elem *>(buf + L::w_off);
        const elem *kS = reinterpret_cast<const elem *>(buf + L::k_off);
        const elem *uS = reinterpret_cast<const elem *>(buf + L::u_off);
        const float *gS = reinterpret_cast<const float *>(buf + L::g_off);
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);

        // state at chunk start as a bf16 operand (and as the emitted h).  With 128-token chunks a chunk takes two
        // 64-token steps: the second one still subtracts w times the state at the CHUNK start (w carries the gate
        // cumulated from there), while the state itself advances step by step with the gate re-based on the
        // previous step's last token.
        const bool chunk_start = (c % p.sub) == 0;
        if (chunk_start) {
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) hB[j][ct] = frag_from_acc(hacc[2 * j][ct], hacc[2 * j + 1][ct]);
            gbase = 0.f;
        }
        if (p.h && chunk_start) {
            const int cc = c / p.sub;
            elem *hg = p.h + b * p.h_sb + hv * p.h_sh + (int64_t)(chunk0 + cc) * p.h_sc;
            if (p.v_first) {   // [V][K] blocks: the lane's four K rows are contiguous
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        const elemx8 f = hB[kt >> 1][ct];
                        const elemx4 q4 = (kt & 1) ? elemx4{f[4], f[5], f[6], f[7]} : elemx4{f[0], f[1], f[2], f[3]};
                        *reinterpret_cast<elemx4 *>(hg + (int64_t)(vcol0 + 16 * ct + li) * K + 16 * kt + 4 * lg) = q4;
                    }
            } else if constexpr (L::kStage) {   // to the staging tile of this chunk; the loader waves write it out during the next one
                elem *st = reinterpret_cast<elem *>(smem + L::stage_off + (cc & 1) * L::stage_bytes);
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) acc_to_tile(st, L::ps, 16 * kt, (wv * CT + ct) * 16, hacc[kt][ct]);
            } else {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct)
                        acc_to_global(reinterpret_cast<char *>(hg + vcol0 + 16 * ct), (int64_t)V * 2, 16 * kt, K, hacc[kt][ct]);
            }
        }

        // v_new = u - w h   (rows = tokens, columns = this wave's V columns)
        f32x4 vn[4][CT];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) vn[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const elemx8 afrag = frag_kc(wS, pw, rt * 16, 32 * j);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) vn[rt][ct] = mfma16x32(afrag, hB[j][ct], vn[rt][ct]);
            }
        const float g_last = gS[len - 1];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const elemx4 uu = frag_tr4(uS, pu, (wv * CT + ct) * 16, rt * 16);  // u[16rt+4g+e][col]
#pragma unroll
                for (int e = 0; e < 4; ++e) vn[rt][ct][e] = (float)uu[e] - vn[rt][ct][e];
            }
        if constexpr (L::kStage) {   // through LDS: the loader waves write whole rows during the next chunk
            elem *st = reinterpret_cast<elem *>(smem + L::vstage_off + (c & 1) * L::vstage_bytes);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) acc_to_tile(st, L::ps, rt * 16, (wv * CT + ct) * 16, vn[rt][ct]);
        } else {
            char *dst = vng + (int64_t)start * p.v_new.st * 2;
#pragma unroll
            for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) acc_to_global(dst + ct * 32, (int64_t)p.v_new.st * 2, rt * 16, len, vn[rt][ct]);
        }

        // h <- e^{g_last} h + k^T (v_new e^{g_last - g}); padded rows carry zeros
        const float dec_all = __expf(g_last - gbase);
        gbase = g_last;
        elemx8 vB[2][CT];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                f32x4 lo = vn[2 * j][ct], hi = vn[2 * j + 1][ct];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int t0 = 32 * j + 4 * lg + e, t1 = t0 + 16;
                    lo[e] = t0 < len ? (float)(elem)lo[e] * __expf(g_last - gS[t0]) : 0.f;
                    hi[e] = t1 < len ? (float)(elem)hi[e] * __expf(g_last - gS[t1]) : 0.f;
                }
                vB[j][ct] = frag_from_acc(lo, hi);
            }
        if (p.gk && chunk_start) {   // per-channel decay: row kk of the state by 2^{gk_last[kk]} (times the scalar decay, if
            // any), once per chunk: k arrives gated up to the end of the whole chunk, in both steps of a 128-token one
            const float *dS = reinterpret_cast<const float *>(buf + L::d_off);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const f32x4 d = *reinterpret_cast<const f32x4 *>(dS + 16 * kt + 4 * lg) * dec_all;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) hacc[kt][ct] *= d;
            }
        } else {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) hacc[kt][ct] *= dec_all;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const elemx8 afrag = frag_tr(kS, pk, kt * 16, 32 * j);  // k^T: rows kk, contraction over tokens
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) hacc[kt][ct] = mfma16x32(afrag, vB[j][ct], hacc[kt][ct]);
            }
        lds_barrier();   // nothing waits for stores to memory
    }

    if (p.hT) {
        const int64_t base = n * p.s_sn + hv * p.s_sh;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int64_t off = base + state_off(16 * kt + 4 * lg + e, vcol0 + 16 * ct + li);
                    if (p.state_elem) static_cast<elem *>(p.hT)[off] = (elem)hacc[kt][ct][e];
                    else static_cast<float *>(p.hT)[off] = hacc[kt][ct][e];
                }
    }
}

template <int K, int CT>
int launch_fwd_h(const ScanParams &p, int slabs, hipStream_t stream) {
    const size_t smem = FwdHSmem<K, CT>::bytes;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(fwd_h_kernel<K, CT>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("fwd_h", stream, (fwd_h_kernel<K, CT>), dim3(slabs, p.geom.Hv, p.geom.N), dim3(512), smem, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int fwd_h_impl(const fla_tensor *k, const fla_tensor *w, const fla_tensor *u, const fla_tensor *g, const fla_tensor *gk,
               const fla_tensor *initial_state, bool output_final_state, int64_t chunk_size, const fla_int_array *cu,
               const fla_int_array *ci, bool state_v_first, const fla_tensor *h, const fla_tensor *v_new,
               const fla_tensor *final_state, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_gated_delta_rule_fwd_h";
    const bool has_g = g != nullptr && g->data != nullptr, has_gk = gk != nullptr && gk->data != nullptr;
    FLA_REQUIRE(has_g || has_gk, FLA_ERR_NULL, "%s: either g or gk must be provided.", op);
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, u, nullptr, chunk_size, geom, kElemDtype, 128))) return rc;
    const int bf = dt_bit(kElemDtype);
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "w", w, geom.B, geom.Hv, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "u", u, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bhtd(op, "v_new", v_new, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if (has_g && (rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    if (has_gk) {   // key-wise gate, log2 units (README.md:16-30): the state rows decay by 2^{gk_last}, k arrives gated
        if ((rc = check_tensor(gk, op, "gk", 4, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(gk->shape[0] == geom.B && gk->shape[1] == geom.Hv && gk->shape[2] == geom.T && gk->shape[3] == geom.K &&
                        inner_unit(gk),
                    FLA_ERR_SHAPE, "%s: gk must be float32 [B,Hv,T,K] with a unit innermost stride.", op);
        FLA_REQUIRE(geom.C == kChunk || geom.K <= 128, FLA_ERR_UNSUPPORTED, "%s: gk with 128-token chunks is built for K <= 128.", op);
    }
    Varlen vl;
    if ((rc = build_varlen(vl, op, cu, ci, geom.C, geom.T))) return rc;
    FLA_REQUIRE(!vl.enabled || geom.B == 1, FLA_ERR_SHAPE, "%s: batch must be 1 with cu_seqlens.", op);
    if (vl.enabled) {
        geom.NT = vl.NT;
        geom.N = vl.N;
    }
    const int64_t d2 = state_v_first ? geom.V : geom.K, d3 = state_v_first ? geom.K : geom.V;
    auto check_state = [&](const fla_tensor *s, const char *name) -> int {
        int r = check_tensor(s, op, name, 4, dt_bit(FLA_F32) | bf);
        if (r) return r;
        FLA_REQUIRE(s->shape[0] == geom.N && s->shape[1] == geom.Hv && s->shape[2] == d2 && s->shape[3] == d3 &&
                        s->stride[3] == 1 && s->stride[2] == d3,
                    FLA_ERR_SHAPE, "%s: %s must be [N=%d,Hv,%lld,%lld] with contiguous blocks.", op, name, geom.N,
                    (long long)d2, (long long)d3);
        return FLA_OK;
    };
    const bool has_h0 = initial_state && initial_state->data;
    if (has_h0 && (rc = check_state(initial_state, "initial_state"))) return rc;
    if (output_final_state && (rc = check_state(final_state, "final_state"))) return rc;
    if (has_h0 && output_final_state)
        FLA_REQUIRE(initial_state->stride[0] == final_state->stride[0] && initial_state->stride[1] == final_state->stride[1] &&
                        initial_state->dtype == final_state->dtype,
                    FLA_ERR_SHAPE, "%s: initial_state and final_state must share strides and dtype.", op);
    const bool has_h = h && h->data;
    if (has_h) {
        if ((rc = check_tensor(h, op, "h", 5, bf))) return rc;
        FLA_REQUIRE(h->shape[0] == geom.B && h->shape[1] == geom.Hv && h->shape[2] == geom.NT && h->shape[3] == d2 &&
                        h->shape[4] == d3 && h->stride[4] == 1 && h->stride[3] == d3,
                    FLA_ERR_SHAPE, "%s: h must be [B,Hv,NT=%d,%lld,%lld] with contiguous blocks.", op, geom.NT,
                    (long long)d2, (long long)d3);
    }
    FLA_REQUIRE(geom.V % 64 == 0, FLA_ERR_UNSUPPORTED, "%s: V must be a multiple of 64, got %d.", op, geom.V);
    FLA_REQUIRE(geom.K == 128 || geom.K == 64, FLA_ERR_UNSUPPORTED, "%s: K must be 64 or 128, got %d.", op, geom.K);
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

    ScanParams p{};
    p.geom = geom;
    p.k = view4(k);
    p.w = view4(w);
    p.u = view4(u);
    p.v_new = view4(v_new);
    p.g = has_g ? view3(g) : View3{nullptr, 0, 0, 0, 0};
    if (has_gk) {
        p.gk = static_cast<const float *>(gk->data);
        p.gk_sb = gk->stride[0];
        p.gk_sh = gk->stride[1];
        p.gk_st = gk->stride[2];
    }
    p.h0 = has_h0 ? initial_state->data : nullptr;
    p.hT = output_final_state ? final_state->data : nullptr;
    const fla_tensor *sref = has_h0 ? initial_state : (output_final_state ? final_state : nullptr);
    p.state_elem = sref != nullptr && sref->dtype != FLA_F32;
    p.sub = geom.C / kChunk;
    if (sref) {
        p.s_sn = sref->stride[0];
        p.s_sh = sref->stride[1];
    }
    p.h = has_h ? static_cast<elem *>(h->data) : nullptr;
    if (has_h) {
        p.h_sb = h->stride[0];
        p.h_sh = h->stride[1];
        p.h_sc = h->stride[2];
    }
    p.v_first = state_v_first ? 1 : 0;

    // Two 16-column tiles per wave (128-column slabs) halve the LDS operand traffic per
    // FLOP; fall back to 64-column slabs when that leaves compute units idle.
    const int64_t chains = (int64_t)geom.N * geom.Hv;
    const bool wide = geom.V % 128 == 0 && chains * (geom.V / 128) >= 2 * (int64_t)num_cus();
    if (geom.K == 128) return wide ? launch_fwd_h<128, 2>(p, geom.V / 128, stream) : launch_fwd_h<128, 1>(p, geom.V / 64, stream);
    return wide ? launch_fwd_h<64, 2>(p, geom.V / 128, stream) : launch_fwd_h<64, 1>(p, geom.V / 64, stream);
}


// =============================================================================================
// chunk_gated_delta_rule_bwd_dhu: reverse scan of the state gradient.
//   dh[c]   = gradient of the state entering from later chunks (emitted before the update)
//   dv2     = dv + (k . dh) * e^{g_last - g}                         (g variant; gK: no factor)
//   dh     <- decay * dh + scale * (q e^{g})^T . do - w^T . dv2      (gK: decay = 2^{gK_last} per K row,
//                                                                     q and k already carry their gates)
// Same ownership as the forward scan: wave w keeps 16*CT columns of V for all K rows of dh in
// fp32 accumulators.  q and w are read with transposing LDS loads (contraction over tokens).
// Math: chunk_gated_delta_rule_bwd_dhu/README.md:6-13, design note
// chunk_gated_delta_rule_bwd_dhu_design.md:81-182, golden torch_custom/fla_npu/test/test_bwd_dhu.py:61-290.
// Unlike the reference kernel the terminal gradient dht is consumed, and dh0 may be the fp32
// [N,Hv,K,V] tensor of the design note as well as the reference's [B,Hv,NT,K,V] form.
// =============================================================================================
struct DhuParams {
    ChunkGeom geom;
    View4 q, k, w, d_o, dv, dv2;
    View4 aqk;           // per-channel gate without dv: the chunk-diagonal blocks Aqk [B,Hv,T,64], dv = Aqk^T d_o per chunk
    View3 g;             // scalar gate [B,Hv,T] (natural log) or null
    const float *gK;     // per-channel gate [B,Hv,T,K] fp32 (log2) or null
    int64_t gk_sb, gk_sh, gk_st;
    const float *dht;    // [N,Hv,K,V] fp32 or null
    int64_t t_sn, t_sh;
    elem *dh;            // [B,Hv,NT,K,V]
    int64_t h_sb, h_sh, h_sc;
    float *dh0_f32;      // [N,Hv,K,V] fp32 or null
    int64_t z_sn, z_sh;
    elem *dh0_ref;       // [B,Hv,NT,K,V] bf16 (value stored at each sequence's first chunk) or null
    float scale;
    int sub;             // 64-token steps per chunk: 1, or 2 for 128-token chunks (scalar gate only)
};

template <int K> struct DhuSmem {
    static constexpr int pk = K + 8, pt = K + 16, pv = 64 + 16;
    static constexpr size_t k_off = 0;                                    // k (contraction along channels)
    static constexpr size_t q_off = k_off + (size_t)kChunk * pk * 2;      // q (read transposed)
    static constexpr size_t w_off = q_off + (size_t)kChunk * pt * 2;      // w (read transposed)
    static constexpr size_t o_off = w_off + (size_t)kChunk * pt * 2;      // d_o slab
    static constexpr size_t v_off = o_off + (size_t)kChunk * pv * 2;      // dv slab
    static constexpr size_t g_off = v_off + (size_t)kChunk * pv * 2;      // [max(K,64)] gate row, [64] factors
    static constexpr size_t buf_bytes = g_off + (size_t)((K > kChunk ? K : kChunk) + kChunk) * 4;
    static constexpr size_t bytes = 2 * buf_bytes;
    // the form that builds dv itself: one [64][ptl] tile behind the two buffers (T, or the chunk's score block)
    static constexpr int ptl = kChunk + 8;
    static constexpr size_t t_off = bytes;
    static constexpr size_t bytes_dvl = t_off + (size_t)4 * 16 * ptl * 2;
};

// 512 threads: waves 0-3 compute chunk c (walking backwards) from LDS buffer c&1 while waves 4-7 copy
// the tiles of chunk c-1 into the other buffer and have those of chunk c-2 in flight.  Both results leave through LDS
// as whole 128-byte rows, stored by the copying waves one step later: dv2 replaces the wave's own columns of the dv
// tile, dh goes over the k tile once every wave is past its k . dh products (the barrier in the middle of a step).
// Tile (R, CT) of T[j][i] = scale (k_j . q_i) e^{g_i - g_j}, i >= j (see bwd_dhu_kernel, DVL), into the chunk's 64 x 64
// tile tS, rounded to the element type: rows are the tokens j whose dv the tile feeds, columns the tokens i of do.
template <int K, int R, int CT>
__device__ __forceinline__ void t_tile(const elem *kS, const elem *qS, const float *gS, elem *tS, int len, float scale) {
    typedef DhuSmem<K> L;
    constexpr int pk = L::pk, pt = L::pt, ptl = L::ptl, KS = K / 32;
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    f32x4 t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < KS; ++j) t = mfma16x32(frag_kc(kS, pk, 16 * R, 32 * j), frag_kc(qS, pt, 16 * CT, 32 * j), t);
    const int i = 16 * CT + li;
    const float gi = gS[i];
    f32x4 x;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int j = 16 * R + 4 * lg + e;
        // the gates enter as a difference: e^{g_i} and e^{-g_j} on their own leave the fp32 range for strong decays
        x[e] = ((CT > R || i >= j) && i < len) ? t[e] * scale * __expf(gi - gS[j]) : 0.f;
    }
    acc_to_tile(tS, ptl, 16 * R, 16 * CT, x);
}

// The six tiles above the diagonal, dealt to the four copying waves (2, 2, 1, 1); the four diagonal tiles are taken by
// the compute waves, one each, which otherwise wait for the copying waves in that half of the step.
template <int K, int LW>
__device__ __forceinline__ void t_tiles(const elem *kS, const elem *qS, const float *gS, elem *tS, int len, float scale) {
    if constexpr (LW == 0) {
        t_tile<K, 0, 1>(kS, qS, gS, tS, len, scale);
        t_tile<K, 0, 2>(kS, qS, gS, tS, len, scale);
    } else if constexpr (LW == 1) {
        t_tile<K, 0, 3>(kS, qS, gS, tS, len, scale);
        t_tile<K, 1, 2>(kS, qS, gS, tS, len, scale);
    } else if constexpr (LW == 2) {
        t_tile<K, 1, 3>(kS, qS, gS, tS, len, scale);
    } else {
        t_tile<K, 2, 3>(kS, qS, gS, tS, len, scale);
    }
}

// DVL (64-token chunks): dv is not an input.  With the per-channel gate it is Aqk^T do per chunk, from the score blocks
// the forward kept (p.aqk): the copying waves stage the block with the other tiles and every compute wave takes
// Aqk^T do for its own 16 columns, in the order of the plain form otherwise.  With the scalar gate it is
// chunk_bwd_dv_local's result
//     dv_j = sum_{i >= j} scale (q_i . k_j) e^{g_i - g_j} do_i = (T do)_j :
// in the first half of the chunk's step T is formed from the k and q tiles of the chunk (ten 16 x 16 tiles: the six
// above the diagonal by the copying waves, the four on it by the compute waves), in the second half every compute wave
// takes T do for its own 16 columns, which lands in accumulators of the layout of dv2, so the intra-chunk dv is never
// rounded or stored.
// FQ (per-channel gate only): q and k hold `fine` values (chunk_kda_fwd keeps qg and kg so for a training step) and meet
// fp16 copies of d_o * scale and of the incoming gradient; the two products that carry the leading terms of dh then round
// their operands to 11 bits instead of 8.
// VS: value columns per workgroup, 64 or 32 (VS / 16 compute waves in front of the four copying waves; 32 when 64 leave
// compute units without a workgroup: every compute wave reads the whole k, q and w tiles for its 16 columns, so half the
// columns are half the LDS traffic of a step).  The form that builds T deals its diagonal tiles to four compute waves.
template <int K, bool GK, bool DVL = false, bool FQ = false, int VS = 64>
__global__ void __launch_bounds__((VS / 16 + 4) * 64) bwd_dhu_kernel(const DhuParams p) {
    static_assert(!FQ || (GK && DVL), "fp16 q and k are built for the KDA form");
    static_assert(VS == 64 || !(DVL && !GK), "the form that builds T itself needs four compute waves");
    extern __shared__ __align__(16) unsigned char smem[];
    typedef DhuSmem<K> L;
    constexpr int CT = 1, CW = VS / 16;
    constexpr int pk = L::pk, pt = L::pt, pv = L::pv;
    constexpr int KT = K / 16, KS = K / 32;
    constexpr int ph = VS + 4;   // pitch of dh [K][VS] laid over the k tile: rows are 8-byte aligned
    static_assert(K * ph <= kChunk * pk, "dh must fit the k tile");

    int slab, hv, n;
    chain_of_block(slab, hv, n);
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    const int V = p.geom.V;
    int b = n, bos = 0, eos = p.geom.T, chunk0 = 0;
    if (p.geom.cu != nullptr) {
        b = 0;
        bos = p.geom.cu[n];
        eos = p.geom.cu[n + 1];
        chunk0 = p.geom.choff[n];
    }
    const int nchunks = (eos - bos + kChunk - 1) / kChunk;
    const elem *qg = static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh;
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh;
    const elem *wg = static_cast<const elem *>(p.w.p) + b * p.w.sb + hv * p.w.sh;
    const elem *og = static_cast<const elem *>(p.d_o.p) + b * p.d_o.sb + hv * p.d_o.sh + slab * VS;
    const elem *vg = DVL ? nullptr : static_cast<const elem *>(p.dv.p) + b * p.dv.sb + hv * p.dv.sh + slab * VS;

    if (wave_id() >= CW) {
        // ------------------------------- loader waves -------------------------------------------
        const int tid = threadIdx.x - CW * 64;
        // Two register sets: while chunk c is computed, the tiles of chunk c - 1 are committed to LDS and those of
        // chunk c - 2 are on their way.  Before the first chunk the loads re-read it (never committed), so that the same
        // number of operations lies between a load and the commit that waits for it in every step.
        struct Tiles {
            TileCopy<kThreads, kChunk, K> tk, tq, tw;
            TileCopy<kThreads, kChunk, VS> to, tv;
            TileCopy<kThreads, kChunk, kChunk> ta;   // DVL with the per-channel gate only
            float gv;
        };
        Tiles t0, t1;
        const elem *ag = (DVL && GK) ? static_cast<const elem *>(p.aqk.p) + b * p.aqk.sb + hv * p.aqk.sh : nullptr;
        auto fetch = [&](Tiles &t, int c) {
            c = max(c, 0);
            const int start = bos + c * kChunk;
            const int len = min(kChunk, eos - start);
            t.tk.fetch(kg + (int64_t)start * p.k.st, p.k.st, len, tid);
            t.tq.fetch(qg + (int64_t)start * p.q.st, p.q.st, len, tid);
            t.tw.fetch(wg + (int64_t)start * p.w.st, p.w.st, len, tid);
            t.to.fetch(og + (int64_t)start * p.d_o.st, p.d_o.st, len, tid);
            if constexpr (!DVL) t.tv.fetch(vg + (int64_t)start * p.dv.st, p.dv.st, len, tid);
            if constexpr (DVL && GK) t.ta.fetch(ag + (int64_t)start * p.aqk.st, p.aqk.st, len, tid);
            if (GK) t.gv = p.gK[b * p.gk_sb + hv * p.gk_sh + (int64_t)(start + len - 1) * p.gk_st + min(tid, K - 1)];
            else t.gv = load_scalar(p.g, b, hv, start + min(tid, len - 1));
        };
        auto commit = [&](const Tiles &t, int c) {
            unsigned char *buf = smem + (c & 1) * L::buf_bytes;
            const int len = min(kChunk, eos - (bos + c * kChunk));
            float *gS = reinterpret_cast<float *>(buf + L::g_off);
            float *fS = gS + (K > kChunk ? K : kChunk);
            t.tk.commit(reinterpret_cast<elem *>(buf + L::k_off), pk, len, tid);
            t.tq.commit(reinterpret_cast<elem *>(buf + L::q_off), pt, len, tid);
            t.tw.commit(reinterpret_cast<elem *>(buf + L::w_off), pt, len, tid);
            t.to.commit(reinterpret_cast<elem *>(buf + L::o_off), pv, len, tid);
            if constexpr (!DVL) t.tv.commit(reinterpret_cast<elem *>(buf + L::v_off), pv, len, tid);
            // one score tile serves both buffers: it is written in the second half of a step and read in the first half
            // of the next one, by the copying waves only
            if constexpr (DVL && GK) t.ta.commit(reinterpret_cast<elem *>(smem + L::t_off), L::ptl, len, tid);
            if (GK) {
                if (tid < K) gS[tid] = exp2f(t.gv);
                if (tid < kChunk) fS[tid] = p.scale;
            } else if (tid < kChunk) {
                gS[tid] = tid < len ? t.gv : 0.f;
                fS[tid] = tid < len ? p.scale * __expf(t.gv) : 0.f;
            }
        };
        // results of the step before (chunk c): read from LDS ahead of the barrier, stored behind the commit
        constexpr int NV = TileCopy<kThreads, kChunk, VS>::N, NH = K * (VS / 8) / kThreads;
        u32x4 vr[NV];
        u32x2 hr[NH][2];
        auto chunk_end = [&](int c) { return (c % p.sub) == p.sub - 1 || c == nchunks - 1; };
        auto read_out = [&](int c) {
            const unsigned char *buf = smem + (c & 1) * L::buf_bytes;
            const elem *vS = reinterpret_cast<const elem *>(buf + L::v_off);
            const elem *hS = reinterpret_cast<const elem *>(buf + L::k_off);
#pragma unroll
            for (int m = 0; m < NV; ++m) {
                const int idx = m * kThreads + tid;
                vr[m] = *reinterpret_cast<const u32x4 *>(vS + (idx / (VS / 8)) * pv + (idx % (VS / 8)) * 8);
            }
            if (chunk_end(c)) {
#pragma unroll
                for (int m = 0; m < NH; ++m) {
                    const int idx = m * kThreads + tid;
                    const elem *src = hS + (idx / (VS / 8)) * ph + (idx % (VS / 8)) * 8;
                    hr[m][0] = *reinterpret_cast<const u32x2 *>(src);
                    hr[m][1] = *reinterpret_cast<const u32x2 *>(src + 4);
                }
            }
        };
        auto store_out = [&](int c) {
            const int start = bos + c * kChunk;
            const int len = min(kChunk, eos - start);
            elem *v2 = static_cast<elem *>(const_cast<void *>(p.dv2.p)) + b * p.dv2.sb + hv * p.dv2.sh + (int64_t)start * p.dv2.st + slab * VS;
#pragma unroll
            for (int m = 0; m < NV; ++m) {
                const int idx = m * kThreads + tid;
                const int r = idx / (VS / 8), c8 = (idx % (VS / 8)) * 8;
                if (r < len) *reinterpret_cast<u32x4 *>(v2 + (int64_t)r * p.dv2.st + c8) = vr[m];
            }
            if (chunk_end(c)) {
                elem *hg = p.dh + b * p.h_sb + hv * p.h_sh + (int64_t)(chunk0 + c / p.sub) * p.h_sc + slab * VS;
#pragma unroll
                for (int m = 0; m < NH; ++m) {
                    const int idx = m * kThreads + tid;
                    *reinterpret_cast<u32x4 *>(hg + (int64_t)(idx / (VS / 8)) * V + (idx % (VS / 8)) * 8) =
                        u32x4{hr[m][0][0], hr[m][0][1], hr[m][1][0], hr[m][1][1]};
                }
            }
        };
        // DVL, chunk c, from its tiles (visible since the last barrier).  Scalar gate: the tiles above the diagonal of
        // T[j][i] = scale (k_j . q_i) e^{g_i - g_j}, i >= j, dealt over the copying waves, into one 64 x 64 tile;
        // the compute waves take T do for their own columns behind the next barrier.  (Per-channel gate: nothing to build,
        // the staged score block is the operand.)
        auto build_dv = [&](int c) {
            const unsigned char *buf = smem + (c & 1) * L::buf_bytes;
            const elem *kS = reinterpret_cast<const elem *>(buf + L::k_off);
            const elem *qS = reinterpret_cast<const elem *>(buf + L::q_off);
            const float *gS = reinterpret_cast<const float *>(buf + L::g_off);
            const int len = min(kChunk, eos - (bos + c * kChunk));
            elem *tS = reinterpret_cast<elem *>(smem + L::t_off);
            switch (wave_id() - CW) {   // the wave's tiles as constants: every operand read of the wave is issued at once
                case 0: t_tiles<K, 0>(kS, qS, gS, tS, len, p.scale); break;
                case 1: t_tiles<K, 1>(kS, qS, gS, tS, len, p.scale); break;
                case 2: t_tiles<K, 2>(kS, qS, gS, tS, len, p.scale); break;
                default: t_tiles<K, 3>(kS, qS, gS, tS, len, p.scale); break;
            }
        };
        // one step: `ahead` takes the tiles of chunk c - 2, `next` holds those of chunk c - 1
        auto step = [&](Tiles &ahead, const Tiles &next, int c) {
            if constexpr (DVL && !GK) build_dv(c);     // read by the compute waves behind the next barrier
            if (c + 1 < nchunks) read_out(c + 1);
            lds_barrier();   // results of chunk c + 1 are in registers; the compute waves are past the k tile of chunk c
            // (issued at the top of the step instead, the loads made both DVL forms a third slower)
            fetch(ahead, c - 2);
            if (c > 0) commit(next, c - 1);
            // the stores go last: a commit waits for everything issued before the loads it needs, and by the next
            // commit these stores are a whole step old
            if (c + 1 < nchunks) store_out(c + 1);
            lds_barrier();   // the loads of chunk c - 2 stay in flight
        };
        if constexpr (DVL && !GK) {   // the tiles of T below the diagonal are never written: they read as zero
            u32x4 *z = reinterpret_cast<u32x4 *>(smem + L::t_off);
            for (int idx = tid; idx < kChunk * L::ptl * 2 / 16; idx += kThreads) z[idx] = u32x4{0u, 0u, 0u, 0u};
        }
        if (nchunks > 0) {
            fetch(t0, nchunks - 1);
            commit(t0, nchunks - 1);
            fetch(t1, nchunks - 2);
        }
        lds_barrier();
        for (int c = nchunks - 1; c >= 0; c -= 2) {
            step(t0, t1, c);
            if (c > 0) step(t1, t0, c - 1);
        }
        if (nchunks > 0) {
            read_out(0);
            store_out(0);
        }
        return;
    }

    // --------------------------------- compute waves ---------------------------------------------
    const int wv = wave_id();
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const int vcol0 = slab * VS + wv * 16;
    f32x4 dacc[KT][CT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            f32x4 a = {0.f, 0.f, 0.f, 0.f};
            if (p.dht) {
                const float *s = p.dht + n * p.t_sn + hv * p.t_sh;
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = s[(int64_t)(16 * kt + 4 * lg + e) * V + vcol0 + 16 * ct + li];
            }
            dacc[kt][ct] = a;
        }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // terminal gradient loaded before the loop (vmcnt(0))
    __syncthreads();

    // With 128-token chunks a chunk takes two 64-token steps, the later tokens first.  Every token of the chunk sees the
    // gradient that ENTERS the chunk (k . dh uses one 16-bit copy, refreshed and stored at the chunk's last step only) and
    // the gate of the chunk's last token; the decay of the carried gradient is applied once, at that step, and the two
    // steps' q^T do and w^T dv2 terms add up.
    elemx8 hB[KS][CT];
    float g_end = 0.f;
    for (int c = nchunks - 1; c >= 0; --c) {
        const bool chunk_end = (c % p.sub) == p.sub - 1 || c == nchunks - 1;
        const unsigned char *buf = smem + (c & 1) * L::buf_bytes;
        elem *kS = const_cast<elem *>(reinterpret_cast<const elem *>(buf + L::k_off));
        const elem *qS = reinterpret_cast<const elem *>(buf + L::q_off);
        const elem *wS = reinterpret_cast<const elem *>(buf + L::w_off);
        const elem *oS = reinterpret_cast<const elem *>(buf + L::o_off);
        elem *vS = const_cast<elem *>(reinterpret_cast<const elem *>(buf + L::v_off));
        const float *gS = reinterpret_cast<const float *>(buf + L::g_off);
        const float *fS = gS + (K > kChunk ? K : kChunk);
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);

        if (chunk_end) {   // dh of this chunk = the incoming gradient
#pragma unroll
            for (int j = 0; j < KS; ++j)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) hB[j][ct] = pack_operand<FQ>(dacc[2 * j][ct], dacc[2 * j + 1][ct]);
        }

        // dv2 = dv + (k . dh) * e^{g_last - g}
        f32x4 dv2[4][CT];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) dv2[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const elemx8 afrag = frag_kc(kS, pk, rt * 16, 32 * j);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) dv2[rt][ct] = mfma16x32_as<FQ>(afrag, hB[j][ct], dv2[rt][ct]);
            }
        if (chunk_end) g_end = GK ? 0.f : gS[len - 1];
        const float g_last = g_end;
        // decay of the carried gradient and the q^T do term
        auto decay_and_q_term = [&]() {
            if (chunk_end) {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    f32x4 dec;
                    if (GK) {
                        dec = *reinterpret_cast<const f32x4 *>(gS + 16 * kt + 4 * lg);
                    } else {
                        const float d = __expf(g_last);
                        dec = f32x4{d, d, d, d};
                    }
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) dacc[kt][ct] *= dec;
                }
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const f32x4 f0 = *reinterpret_cast<const f32x4 *>(fS + 32 * j + 4 * lg),
                            f1 = *reinterpret_cast<const f32x4 *>(fS + 32 * j + 16 + 4 * lg);
                const elemx8 raw = frag_tr(oS, pv, wv * 16, 32 * j);   // do[t][col], t = 32j + c(g,e)
                f32x4 lo, hi;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lo[e] = (float)raw[e] * f0[e];
                    hi[e] = (float)raw[4 + e] * f1[e];
                }
                const elemx8 ob = frag_from_acc(lo, hi);
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) dacc[kt][0] = mfma16x32(frag_tr(qS, pt, kt * 16, 32 * j), ob, dacc[kt][0]);
            }
        };
        // DVL with the scalar gate: the copying waves spend this half of the step on the dv tile, so the part of the update
        // that needs neither dv nor the place of the k tile moves in front of the barrier; dh then leaves from its 16-bit
        // copy.  (From score blocks the dv tile is two products per wave: the order of the plain form is kept.)
        constexpr bool EARLY = DVL && !GK;
        f32x4 dvl[4];   // DVL: the dv operand of the wave's 16 columns, in the layout of dv2
        if constexpr (DVL && GK) {
            // per-channel gate: dv_j = sum_{i >= j} Aqk[i][j] do_i (the dv of chunk_kda_bwd_dav) from the score block the
            // copying waves staged with the chunk's tiles; Aqk is zero above its diagonal and past the chunk's end.  Taken
            // in this half of the step: the block's place is written again behind the barrier.
            const elem *aS = reinterpret_cast<const elem *>(smem + L::t_off);
            const elemx8 ob0 = frag_tr(oS, pv, wv * 16, 0), ob1 = frag_tr(oS, pv, wv * 16, 32);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f};
                if (rt < 2) a = mfma16x32(frag_tr(aS, L::ptl, 16 * rt, 0), ob0, a);
                dvl[rt] = mfma16x32(frag_tr(aS, L::ptl, 16 * rt, 32), ob1, a);
            }
        }
        if constexpr (EARLY) {
            elem *tS = reinterpret_cast<elem *>(smem + L::t_off);
            switch (wv) {   // the wave's diagonal tile of T (see t_tiles)
                case 0: t_tile<K, 0, 0>(kS, qS, gS, tS, len, p.scale); break;
                case 1: t_tile<K, 1, 1>(kS, qS, gS, tS, len, p.scale); break;
                case 2: t_tile<K, 2, 2>(kS, qS, gS, tS, len, p.scale); break;
                default: t_tile<K, 3, 3>(kS, qS, gS, tS, len, p.scale); break;
            }
            decay_and_q_term();
        }
        lds_barrier();   // every wave is past the k tile, which now takes dh on its way to memory
        if (chunk_end) {
            if constexpr (EARLY) {
#pragma unroll
                for (int j = 0; j < KS; ++j) {
                    const u32x4 d = __builtin_bit_cast(u32x4, hB[j][0]);
                    packed_to_tile(kS, ph, 32 * j, wv * 16, d[0], d[1]);
                    packed_to_tile(kS, ph, 32 * j + 16, wv * 16, d[2], d[3]);
                }
            } else {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) acc_to_tile(kS, ph, 16 * kt, wv * 16, dacc[kt][0]);
            }
        }
        // DVL with the scalar gate: the intra-chunk dv of the wave's 16 columns, T do, straight into accumulators of the
        // layout of dv2 (T complete since the barrier; its tiles (1,0) and (3,2) were zeroed once, (2,0), (2,1), (3,0),
        // (3,1) are skipped with their contraction step)
        if constexpr (EARLY) {
            const elem *tS = reinterpret_cast<const elem *>(smem + L::t_off);
            const elemx8 ob0 = frag_tr(oS, pv, wv * 16, 0), ob1 = frag_tr(oS, pv, wv * 16, 32);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                f32x4 a = {0.f, 0.f, 0.f, 0.f};
                if (rt < 2) a = mfma16x32(frag_kc(tS, L::ptl, 16 * rt, 0), ob0, a);
                dvl[rt] = mfma16x32(frag_kc(tS, L::ptl, 16 * rt, 32), ob1, a);
            }
        }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                elemx4 old = {};
                if constexpr (!DVL) old = frag_tr4(vS, pv, (wv * CT + ct) * 16, rt * 16);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int t = rt * 16 + 4 * lg + e;
                    const float f = GK ? 1.f : __expf(g_last - gS[t]);
                    const float add = DVL ? dvl[rt][e] : (float)old[e];
                    dv2[rt][ct][e] = t < len ? dv2[rt][ct][e] * f + add : 0.f;
                }
            }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) acc_to_tile(vS, pv, rt * 16, wv * 16, dv2[rt][0]);   // over the wave's own columns of dv

        // dh <- decay * dh + scale (q e^g)^T do - w^T dv2
        if constexpr (EARLY) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const elemx8 nb = frag_from_acc(-dv2[2 * j][0], -dv2[2 * j + 1][0]);
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) dacc[kt][0] = mfma16x32(frag_tr(wS, pt, kt * 16, 32 * j), nb, dacc[kt][0]);
            }
        } else {
        if (chunk_end) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                f32x4 dec;
                if (GK) {
                    dec = *reinterpret_cast<const f32x4 *>(gS + 16 * kt + 4 * lg);
                } else {
                    const float d = __expf(g_last);
                    dec = f32x4{d, d, d, d};
                }
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) dacc[kt][ct] *= dec;
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            elemx8 ob[CT], nb[CT];
            const f32x4 f0 = *reinterpret_cast<const f32x4 *>(fS + 32 * j + 4 * lg),
                        f1 = *reinterpret_cast<const f32x4 *>(fS + 32 * j + 16 + 4 * lg);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const elemx8 raw = frag_tr(oS, pv, (wv * CT + ct) * 16, 32 * j);   // do[t][col], t = 32j + c(g,e)
                f32x4 lo, hi;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lo[e] = (float)raw[e] * f0[e];
                    hi[e] = (float)raw[4 + e] * f1[e];
                }
                ob[ct] = pack_operand<FQ>(lo, hi);
                nb[ct] = frag_from_acc(-dv2[2 * j][ct], -dv2[2 * j + 1][ct]);
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const elemx8 qf = frag_tr(qS, pt, kt * 16, 32 * j);
                const elemx8 wf = frag_tr(wS, pt, kt * 16, 32 * j);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    dacc[kt][ct] = mfma16x32_as<FQ>(qf, ob[ct], dacc[kt][ct]);
                    dacc[kt][ct] = mfma16x32(wf, nb[ct], dacc[kt][ct]);
                }
            }
        }
        }
        lds_barrier();
    }

    // gradient of the initial state
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t off = (int64_t)(16 * kt + 4 * lg + e) * V + vcol0 + 16 * ct + li;
                if (p.dh0_f32) p.dh0_f32[n * p.z_sn + hv * p.z_sh + off] = dacc[kt][ct][e];
                if (p.dh0_ref && nchunks > 0)
                    p.dh0_ref[b * p.h_sb + hv * p.h_sh + (int64_t)chunk0 * p.h_sc + off] = (elem)dacc[kt][ct][e];
            }
}

// More than 128 channels (per-channel gate only): the k, q and w tiles of one step fill the LDS, so nothing is
// double-buffered.  256 threads: all four waves copy the tiles of a step, then compute it with the 256 x 16 gradient of
// each wave in registers; dh and dv2 leave straight from the accumulators.  Two barriers a step.
template <int K> struct WideDhuSmem {
    static constexpr int pk = K + 8, pt = K + 16, pv = 64 + 16;
    static constexpr size_t k_off = 0;
    static constexpr size_t q_off = k_off + (size_t)kChunk * pk * 2;
    static constexpr size_t w_off = q_off + (size_t)kChunk * pt * 2;
    static constexpr size_t o_off = w_off + (size_t)kChunk * pt * 2;
    static constexpr size_t v_off = o_off + (size_t)kChunk * pv * 2;
    static constexpr size_t g_off = v_off + (size_t)kChunk * pv * 2;
    static constexpr size_t bytes = g_off + (size_t)K * 4;
};

template <int K>
__global__ void __launch_bounds__(kThreads) bwd_dhu_wide_kernel(const DhuParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    typedef WideDhuSmem<K> L;
    constexpr int VS = 64;
    constexpr int pk = L::pk, pt = L::pt, pv = L::pv;
    constexpr int KT = K / 16, KS = K / 32;
    elem *kS = reinterpret_cast<elem *>(smem + L::k_off), *qS = reinterpret_cast<elem *>(smem + L::q_off);
    elem *wS = reinterpret_cast<elem *>(smem + L::w_off), *oS = reinterpret_cast<elem *>(smem + L::o_off);
    elem *vS = reinterpret_cast<elem *>(smem + L::v_off);
    float *gS = reinterpret_cast<float *>(smem + L::g_off);

    int slab, hv, n;
    chain_of_block(slab, hv, n);
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    const int V = p.geom.V;
    int b = n, bos = 0, eos = p.geom.T, chunk0 = 0;
    if (p.geom.cu != nullptr) {
        b = 0;
        bos = p.geom.cu[n];
        eos = p.geom.cu[n + 1];
        chunk0 = p.geom.choff[n];
    }
    const int nchunks = (eos - bos + kChunk - 1) / kChunk;
    const elem *qg = static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh;
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh;
    const elem *wg = static_cast<const elem *>(p.w.p) + b * p.w.sb + hv * p.w.sh;
    const elem *og = static_cast<const elem *>(p.d_o.p) + b * p.d_o.sb + hv * p.d_o.sh + slab * VS;
    const elem *vg = static_cast<const elem *>(p.dv.p) + b * p.dv.sb + hv * p.dv.sh + slab * VS;
    const int tid = threadIdx.x, wv = wave_id();
    const int l = lane_id(), li = l & 15, lg = l >> 4;
    const int vcol0 = slab * VS + wv * 16;

    f32x4 dacc[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        f32x4 a = {0.f, 0.f, 0.f, 0.f};
        if (p.dht) {
            const float *s = p.dht + n * p.t_sn + hv * p.t_sh;
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = s[(int64_t)(16 * kt + 4 * lg + e) * V + vcol0 + li];
        }
        dacc[kt] = a;
    }

    for (int c = nchunks - 1; c >= 0; --c) {
        const int start = bos + c * kChunk;
        const int len = min(kChunk, eos - start);
        load_tile<kThreads>(kS, pk, kg + (int64_t)start * p.k.st, p.k.st, kChunk, K, len);
        load_tile<kThreads>(qS, pt, qg + (int64_t)start * p.q.st, p.q.st, kChunk, K, len);
        load_tile<kThreads>(wS, pt, wg + (int64_t)start * p.w.st, p.w.st, kChunk, K, len);
        load_tile<kThreads>(oS, pv, og + (int64_t)start * p.d_o.st, p.d_o.st, kChunk, VS, len);
        load_tile<kThreads>(vS, pv, vg + (int64_t)start * p.dv.st, p.dv.st, kChunk, VS, len);
        for (int i = tid; i < K; i += kThreads)
            gS[i] = exp2f(p.gK[b * p.gk_sb + hv * p.gk_sh + (int64_t)(start + len - 1) * p.gk_st + i]);
        __syncthreads();

        // dh of this chunk = the incoming gradient; k . dh uses its 16-bit copy
        elemx8 hB[KS];
#pragma unroll
        for (int j = 0; j < KS; ++j) hB[j] = frag_from_acc(dacc[2 * j], dacc[2 * j + 1]);
        {
            char *hg = reinterpret_cast<char *>(p.dh + b * p.h_sb + hv * p.h_sh + (int64_t)(chunk0 + c) * p.h_sc + vcol0);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) acc_to_global(hg, (int64_t)V * 2, 16 * kt, K, dacc[kt]);
        }
        // dv2 = dv + k . dh   (k arrives gated)
        f32x4 dv2[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) dv2[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < KS; ++j)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) dv2[rt] = mfma16x32(frag_kc(kS, pk, rt * 16, 32 * j), hB[j], dv2[rt]);
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const elemx4 old = frag_tr4(vS, pv, wv * 16, rt * 16);
#pragma unroll
            for (int e = 0; e < 4; ++e) dv2[rt][e] = rt * 16 + 4 * lg + e < len ? dv2[rt][e] + (float)old[e] : 0.f;
        }
        {
            char *v2 = reinterpret_cast<char *>(static_cast<elem *>(const_cast<void *>(p.dv2.p)) + b * p.dv2.sb + hv * p.dv2.sh +
                                                (int64_t)start * p.dv2.st + vcol0);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc_to_global(v2, p.dv2.st * 2, 16 * rt, len, dv2[rt]);
        }
        // dh <- 2^{gK_last} dh + scale q^T do - w^T dv2   (q arrives gated)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) dacc[kt] *= *reinterpret_cast<const f32x4 *>(gS + 16 * kt + 4 * lg);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const elemx8 raw = frag_tr(oS, pv, wv * 16, 32 * j);
            f32x4 lo, hi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[e] = (float)raw[e] * p.scale;
                hi[e] = (float)raw[4 + e] * p.scale;
            }
            const elemx8 ob = frag_from_acc(lo, hi), nb = frag_from_acc(-dv2[2 * j], -dv2[2 * j + 1]);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                dacc[kt] = mfma16x32(frag_tr(qS, pt, kt * 16, 32 * j), ob, dacc[kt]);
                dacc[kt] = mfma16x32(frag_tr(wS, pt, kt * 16, 32 * j), nb, dacc[kt]);
            }
        }
        __syncthreads();   // every tile has been read before the next step's tiles replace them
    }

#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int64_t off = (int64_t)(16 * kt + 4 * lg + e) * V + vcol0 + li;
            if (p.dh0_f32) p.dh0_f32[n * p.z_sn + hv * p.z_sh + off] = dacc[kt][e];
            if (p.dh0_ref && nchunks > 0) p.dh0_ref[b * p.h_sb + hv * p.h_sh + (int64_t)chunk0 * p.h_sc + off] = (elem)dacc[kt][e];
        }
}

template <int K>
int launch_bwd_dhu_wide(const DhuParams &p, int slabs, hipStream_t stream) {
    const size_t smem = WideDhuSmem<K>::bytes;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(bwd_dhu_wide_kernel<K>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("bwd_dhu", stream, (bwd_dhu_wide_kernel<K>), dim3(slabs, p.geom.Hv, p.geom.N), dim3(kThreads), smem, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

template <int K, bool GK, bool DVL, bool FQ, int VS>
int launch_bwd_dhu_as(const DhuParams &p, hipStream_t stream) {
    const size_t smem = DVL ? DhuSmem<K>::bytes_dvl : DhuSmem<K>::bytes;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(bwd_dhu_kernel<K, GK, DVL, FQ, VS>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("bwd_dhu", stream, (bwd_dhu_kernel<K, GK, DVL, FQ, VS>), dim3(p.geom.V / VS, p.geom.Hv, p.geom.N),
               dim3((VS / 16 + 4) * 64), smem, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}
template <int K, bool GK, bool DVL = false, bool FQ = false>
int launch_bwd_dhu(const DhuParams &p, int slabs, hipStream_t stream) {
    // per-channel gate (the KDA forms): 32-column slabs when 64-column ones leave compute units idle
    if constexpr (GK) {
        if ((int64_t)p.geom.N * p.geom.Hv * slabs < (int64_t)num_cus())
            return launch_bwd_dhu_as<K, GK, DVL, FQ, 32>(p, stream);
    }
    return launch_bwd_dhu_as<K, GK, DVL, FQ, 64>(p, stream);
}

int bwd_dhu_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o, const fla_tensor *dv,
                 const fla_tensor *g, const fla_tensor *gK, const fla_tensor *h0, const fla_tensor *dht,
                 const fla_int_array *cu, const fla_int_array *ci, double scale, int64_t chunk_size, bool use_exp2,
                 const fla_tensor *dh, const fla_tensor *dh0, const fla_tensor *dv2, void *ws, uint64_t ws_size,
                 hipStream_t stream, uint64_t *query, const fla_tensor *aqk = nullptr) {
    // with aqk: the form for the KDA backward, whose dv operand is Aqk^T d_o per chunk and is formed inside the scan
    const bool has_aqk = aqk && aqk->data;
    const char *op = has_aqk ? "chunk_kda_bwd_dhu" : "chunk_gated_delta_rule_bwd_dhu";
    (void)h0;  // only its presence matters to the caller (it decides whether dh0 is allocated)
    const bool has_g = g && g->data, has_gk = gK && gK->data;
    FLA_REQUIRE(has_g != has_gk, FLA_ERR_NULL, "%s: exactly one of g and gK must be provided.", op);
    FLA_REQUIRE(!has_gk || use_exp2, FLA_ERR_UNSUPPORTED, "%s: use_exp2 must be true when gK is provided.", op);
    FLA_REQUIRE(!has_g || !use_exp2, FLA_ERR_UNSUPPORTED, "%s: the scalar gate g is a natural-log gate (use_exp2=false).", op);
    ChunkGeom geom;
    int rc;
    // dv absent: the intra-chunk part of dv (chunk_bwd_dv_local's result) is formed inside the scan
    const bool has_dv = dv && dv->data;
    FLA_REQUIRE(has_dv || has_aqk || (has_g && chunk_size == kChunk), FLA_ERR_UNSUPPORTED,
                "%s: dv may be left out with the scalar gate g and chunk_size 64 only.", op);
    FLA_REQUIRE(!has_aqk || (has_gk && !has_dv && chunk_size == kChunk), FLA_ERR_UNSUPPORTED,
                "%s: Aqk takes the place of dv with the per-channel gate gK and chunk_size 64 only.", op);
    // The KDA form also takes q and k (qg and kg of chunk_kda_fwd) as float16 tensors beside bf16 w, d_o and Aqk.
    const bool fine_qk = has_aqk && !kFineIsElem && q && k && q->dtype == FLA_F16 && k->dtype == FLA_F16;
    fla_tensor q_as_elem, k_as_elem;
    if (fine_qk) {
        q_as_elem = *q;
        k_as_elem = *k;
        q_as_elem.dtype = k_as_elem.dtype = kElemDtype;
        q = &q_as_elem;
        k = &k_as_elem;
    }
    if ((rc = gdn_geometry(op, k, has_dv ? dv : d_o, nullptr, chunk_size, geom, kElemDtype, 128))) return rc;   // README.md:101-104: 64 or 128
    // gK with 128-token chunks (README.md:104): q and k carry their gates relative to the whole chunk, the decay
    // 2^{gK at the chunk's last token} is applied once, at the chunk's last step
    FLA_REQUIRE(geom.C == kChunk || !has_gk || geom.K <= 128, FLA_ERR_UNSUPPORTED,
                "%s: gK with 128-token chunks is built for K <= 128.", op);
    const int bf = dt_bit(kElemDtype);
    if ((rc = check_bhtd(op, "q", q, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "w", w, geom.B, geom.Hv, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "d_o", d_o, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if (has_dv && (rc = check_bhtd(op, "dv", dv, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if (has_aqk && (rc = check_bhtd(op, "Aqk", aqk, geom.B, geom.Hv, geom.T, kChunk, bf))) return rc;
    FLA_REQUIRE(!has_aqk || geom.K == 128 || geom.K == 64, FLA_ERR_UNSUPPORTED, "%s: K must be 64 or 128, got %d.", op, geom.K);
    if ((rc = check_bhtd(op, "dv2", dv2, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if (has_g && (rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    if (has_gk) {
        if ((rc = check_tensor(gK, op, "gK", 4, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(gK->shape[0] == geom.B && gK->shape[1] == geom.Hv && gK->shape[2] == geom.T && gK->shape[3] == geom.K &&
                        inner_unit(gK),
                    FLA_ERR_SHAPE, "%s: gK must be fp32 [B,Hv,T,K].", op);
    }
    Varlen vl;
    if ((rc = build_varlen(vl, op, cu, ci, geom.C, geom.T))) return rc;
    FLA_REQUIRE(!vl.enabled || geom.B == 1, FLA_ERR_SHAPE, "%s: batch must be 1 with cu_seqlens.", op);
    if (vl.enabled) {
        geom.NT = vl.NT;
        geom.N = vl.N;
    }
    if ((rc = check_tensor(dh, op, "dh", 5, bf))) return rc;
    FLA_REQUIRE(dh->shape[0] == geom.B && dh->shape[1] == geom.Hv && dh->shape[2] == geom.NT && dh->shape[3] == geom.K &&
                    dh->shape[4] == geom.V && dh->stride[4] == 1 && dh->stride[3] == geom.V,
                FLA_ERR_SHAPE, "%s: dh must be [B,Hv,NT=%d,K,V] with contiguous blocks.", op, geom.NT);
    const bool has_dh0 = dh0 && dh0->data;
    bool dh0_is_ref = false;
    if (has_dh0) {
        if (dh0->ndim == 5) {
            dh0_is_ref = true;
            if ((rc = check_tensor(dh0, op, "dh0", 5, bf))) return rc;
            FLA_REQUIRE(same_shape(dh0, dh) && dh0->stride[0] == dh->stride[0] && dh0->stride[1] == dh->stride[1] &&
                            dh0->stride[2] == dh->stride[2] && dh0->stride[3] == geom.V && dh0->stride[4] == 1,
                        FLA_ERR_SHAPE, "%s: a 5-D dh0 must have the shape and strides of dh.", op);
        } else {
            if ((rc = check_tensor(dh0, op, "dh0", 4, dt_bit(FLA_F32)))) return rc;
            FLA_REQUIRE(dh0->shape[0] == geom.N && dh0->shape[1] == geom.Hv && dh0->shape[2] == geom.K &&
                            dh0->shape[3] == geom.V && dh0->stride[3] == 1 && dh0->stride[2] == geom.V,
                        FLA_ERR_SHAPE, "%s: a 4-D dh0 must be fp32 [N=%d,Hv,K,V].", op, geom.N);
        }
    }
    const bool has_dht = dht && dht->data;
    if (has_dht) {
        if ((rc = check_tensor(dht, op, "dht", 4, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(dht->shape[0] == geom.N && dht->shape[1] == geom.Hv && dht->shape[2] == geom.K && dht->shape[3] == geom.V &&
                        dht->stride[3] == 1 && dht->stride[2] == geom.V,
                    FLA_ERR_SHAPE, "%s: dht must be fp32 [N=%d,Hv,K,V].", op, geom.N);
    }
    FLA_REQUIRE(geom.K == 128 || geom.K == 64 || (geom.K == 256 && has_gk), FLA_ERR_UNSUPPORTED,
                "%s: K must be 64 or 128 (256 with gK), got %d.", op, geom.K);
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

    DhuParams p{};
    p.geom = geom;
    p.q = view4(q);
    p.k = view4(k);
    p.w = view4(w);
    p.d_o = view4(d_o);
    if (has_dv) p.dv = view4(dv);
    if (has_aqk) p.aqk = view4(aqk);
    p.dv2 = view4(dv2);
    if (has_g) p.g = view3(g);
    if (has_gk) {
        p.gK = static_cast<const float *>(gK->data);
        p.gk_sb = gK->stride[0];
        p.gk_sh = gK->stride[1];
        p.gk_st = gK->stride[2];
    }
    if (has_dht) {
        p.dht = static_cast<const float *>(dht->data);
        p.t_sn = dht->stride[0];
        p.t_sh = dht->stride[1];
    }
    p.dh = static_cast<elem *>(dh->data);
    p.h_sb = dh->stride[0];
    p.h_sh = dh->stride[1];
    p.h_sc = dh->stride[2];
    if (has_dh0 && dh0_is_ref) p.dh0_ref = static_cast<elem *>(dh0->data);
    if (has_dh0 && !dh0_is_ref) {
        p.dh0_f32 = static_cast<float *>(dh0->data);
        p.z_sn = dh0->stride[0];
        p.z_sh = dh0->stride[1];
    }
    p.scale = (float)scale;
    p.sub = geom.C / kChunk;
    const int slabs = geom.V / 64;
    if constexpr (!kFineIsElem) {
        if (fine_qk)
            return geom.K == 128 ? launch_bwd_dhu<128, true, true, true>(p, slabs, stream)
                                 : launch_bwd_dhu<64, true, true, true>(p, slabs, stream);
    }
    if (has_aqk) return geom.K == 128 ? launch_bwd_dhu<128, true, true>(p, slabs, stream) : launch_bwd_dhu<64, true, true>(p, slabs, stream);
    if (!has_dv) return geom.K == 128 ? launch_bwd_dhu<128, false, true>(p, slabs, stream) : launch_bwd_dhu<64, false, true>(p, slabs, stream);
    if (geom.K == 256) return launch_bwd_dhu_wide<256>(p, slabs, stream);
    if (geom.K == 128) return has_gk ? launch_bwd_dhu<128, true>(p, slabs, stream) : launch_bwd_dhu<128, false>(p, slabs, stream);
    return has_gk ? launch_bwd_dhu<64, true>(p, slabs, stream) : launch_bwd_dhu<64, false>(p, slabs, stream);
}

}  // namespace
}  // namespace fla

FLA_ENTRY(fla_chunk_gated_delta_rule_fwd_h_get_workspace_size)(
    const fla_tensor *k, const fla_tensor *w, const fla_tensor *u, const fla_tensor *g, const fla_tensor *gk,
    const fla_tensor *initial_state, bool output_final_state, int64_t chunk_size, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, bool state_v_first, const fla_tensor *h, const fla_tensor *v_new,
    const fla_tensor *final_state, uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_chunk_gated_delta_rule_fwd_h_get_workspace_size, k, w, u, g, gk, initial_state, output_final_state, chunk_size, cu_seqlens, chunk_indices, state_v_first, h, v_new, final_state, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "chunk_gated_delta_rule_fwd_h: workspace_size must not be null.");
    return fla::guarded([&] { return fla::fwd_h_impl(k, w, u, g, gk, initial_state, output_final_state, chunk_size, cu_seqlens, chunk_indices,
                           state_v_first, h, v_new, final_state, nullptr, 0, nullptr, workspace_size); });
}

FLA_ENTRY(fla_chunk_gated_delta_rule_fwd_h)(
    const fla_tensor *k, const fla_tensor *w, const fla_tensor *u, const fla_tensor *g, const fla_tensor *gk,
    const fla_tensor *initial_state, bool output_final_state, int64_t chunk_size, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, bool state_v_first, const fla_tensor *h, const fla_tensor *v_new,
    const fla_tensor *final_state, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_chunk_gated_delta_rule_fwd_h, k, w, u, g, gk, initial_state, output_final_state, chunk_size, cu_seqlens, chunk_indices, state_v_first, h, v_new, final_state, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::fwd_h_impl(k, w, u, g, gk, initial_state, output_final_state, chunk_size, cu_seqlens, chunk_indices,
                           state_v_first, h, v_new, final_state, workspace, workspace_size,
                           static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_kda_bwd_dhu_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o, const fla_tensor *Aqk,
    const fla_tensor *gK, const fla_tensor *h0, const fla_tensor *dht, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dh, const fla_tensor *dh0,
    const fla_tensor *dv2, uint64_t *workspace_size) {
    FLA_ROUTE_F16(d_o, fla_chunk_kda_bwd_dhu_get_workspace_size, q, k, w, d_o, Aqk, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, dh, dh0, dv2, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "chunk_kda_bwd_dhu: workspace_size must not be null.");
    if (!Aqk || !Aqk->data) return fla::fail(FLA_ERR_NULL, "chunk_kda_bwd_dhu: Aqk must not be null.");
    return fla::guarded([&] { return fla::bwd_dhu_impl(q, k, w, d_o, nullptr, nullptr, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, true,
                             dh, dh0, dv2, nullptr, 0, nullptr, workspace_size, Aqk); });
}

FLA_ENTRY(fla_chunk_kda_bwd_dhu)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o, const fla_tensor *Aqk,
    const fla_tensor *gK, const fla_tensor *h0, const fla_tensor *dht, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dh, const fla_tensor *dh0,
    const fla_tensor *dv2, void *workspace, uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(d_o, fla_chunk_kda_bwd_dhu, q, k, w, d_o, Aqk, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, dh, dh0, dv2, workspace, workspace_size, stream);
    if (!Aqk || !Aqk->data) return fla::fail(FLA_ERR_NULL, "chunk_kda_bwd_dhu: Aqk must not be null.");
    return fla::guarded([&] { return fla::bwd_dhu_impl(q, k, w, d_o, nullptr, nullptr, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, true,
                             dh, dh0, dv2, workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr, Aqk); });
}

FLA_ENTRY(fla_chunk_gated_delta_rule_bwd_dhu_get_workspace_size)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o, const fla_tensor *dv,
    const fla_tensor *g, const fla_tensor *gK, const fla_tensor *h0, const fla_tensor *dht,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale, int64_t chunk_size, bool use_exp2,
    const fla_tensor *dh, const fla_tensor *dh0, const fla_tensor *dv2, uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_gated_delta_rule_bwd_dhu_get_workspace_size, q, k, w, d_o, dv, g, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, use_exp2, dh, dh0, dv2, workspace_size);
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "chunk_gated_delta_rule_bwd_dhu: workspace_size must not be null.");
    return fla::guarded([&] { return fla::bwd_dhu_impl(q, k, w, d_o, dv, g, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, use_exp2, dh, dh0,
                             dv2, nullptr, 0, nullptr, workspace_size); });
}

FLA_ENTRY(fla_chunk_gated_delta_rule_bwd_dhu)(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o, const fla_tensor *dv,
    const fla_tensor *g, const fla_tensor *gK, const fla_tensor *h0, const fla_tensor *dht,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale, int64_t chunk_size, bool use_exp2,
    const fla_tensor *dh, const fla_tensor *dh0, const fla_tensor *dv2, void *workspace, uint64_t workspace_size,
    void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_gated_delta_rule_bwd_dhu, q, k, w, d_o, dv, g, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, use_exp2, dh, dh0, dv2, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::bwd_dhu_impl(q, k, w, d_o, dv, g, gK, h0, dht, cu_seqlens, chunk_indices, scale, chunk_size, use_exp2, dh, dh0,
                             dv2, workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}
