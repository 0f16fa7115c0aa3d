// Chunk-parallel stages of the gated-delta-rule forward, one workgroup per
// (chunk, value head, batch row), bf16 MFMA with fp32 accumulation:
//   chunk_scaled_dot_kkt   A0 = strict_lower(beta_i e^{clip(G_i-G_j)} <k_i,k_j>)
//   solve_tri              (I + A0)^-1 by fp32 forward substitution
//   recompute_w_u_fwd      w = Ainv (k beta e^G), u = Ainv (v beta)
//   chunk_fwd_o            o = scale (e^G (q h) + tril(q k^T e^{min(G_i-G_j,0)}) v_new)
// Stage math and rounding points: chunk_scaled_dot_kkt/README.md:11-29,
// solve_tri/README.md:7-19, recompute_w_u_fwd/README.md:12-32,
// chunk_fwd_o/README.md:6-15 (+ qkmask epilogue, op_kernel/.../block_epilogue_gdn_fwdo_qkmask.hpp:210-262).
#include "gdn_common.h"
#include "chunk_inverse.h"
#include "mfma_tiles.h"

namespace fla {
namespace {

constexpr int kThreads = 256;

// =============================================================================
// chunk_scaled_dot_kkt
// =============================================================================
struct KktParams {
    ChunkGeom geom;
    View4 k;
    View3 g, beta;
    float *out;
    int64_t o_sb, o_sh, o_st;
};

// C = tokens per chunk (64 or 128): the k rows of one chunk sit in LDS, wave w owns the 16-row blocks w, w + 4, ...
template <int C>
__global__ void __launch_bounds__(kThreads) kkt_kernel(const KktParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int K = p.geom.K, pitch = K + 8;
    elem *kS = reinterpret_cast<elem *>(smem);
    float *gS = reinterpret_cast<float *>(kS + C * pitch);
    float *bS = gS + C;

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st;
    load_tile<kThreads>(kS, pitch, kg, p.k.st, C, K, len);
    if (threadIdx.x < C) {
        const int t = threadIdx.x;
        gS[t] = t < len ? load_scalar(p.g, b, hv, start + t) : 0.f;
        bS[t] = t < len ? load_scalar(p.beta, b, hv, start + t) : 0.f;
    }
    __syncthreads();

    for (int I = wave_id(); I < C / 16; I += kThreads / 64) {  // t block
        const int t = I * 16 + acc_col();
        float *orow = p.out + b * p.o_sb + hv * p.o_sh + (int64_t)(start + t) * p.o_st;
        const float gt = gS[t], bt = bS[t];
        for (int J = 0; J < C / 16; ++J) {  // s block
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            if (J <= I) {
                for (int kk = 0; kk < K; kk += 32) acc = mfma16x32(frag_kc(kS, pitch, J * 16, kk), frag_kc(kS, pitch, I * 16, kk), acc);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int s = J * 16 + acc_row(e);
                    const float d = fminf(fmaxf(gt - gS[s], -50.f), 50.f);
                    acc[e] = (s < t && t < len) ? bt * __expf(d) * acc[e] : 0.f;
                }
            }
            if (t < len) *reinterpret_cast<f32x4 *>(orow + J * 16 + 4 * (lane_id() >> 4)) = acc;
        }
    }
}

// =============================================================================
// solve_tri: one wave per 64x64 block, lane j owns column j of the inverse.
// =============================================================================
struct SolveParams {
    ChunkGeom geom;  // Hv = heads of x
    const void *x;   // element type, or fp32 (rounded to the element type on load: the cast the caller would do)
    elem *out;
    int64_t sb, sh, st;  // strides of (batch, head, token) in x and out
};

// BT x BT blocks, BT in {16, 32, 64, 128}; one thread per column of the inverse (at least one full wave).
template <int BT, bool F32IN>
__global__ void __launch_bounds__(BT < 64 ? 64 : BT) solve_tri_kernel(const SolveParams p) {
    constexpr int NTH = BT < 64 ? 64 : BT;       // threads
    constexpr int CPR = BT / 8;                  // 16-byte pieces per row
    constexpr int PO = BT + 8;                   // pitch of the 16-bit output staging
    constexpr int NP = (BT * CPR + NTH - 1) / NTH;
    __shared__ __align__(16) float A[BT][BT];
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    int start, len;
    if (p.geom.cu == nullptr) {
        start = c * BT;
        len = min(BT, p.geom.T - start);
    } else {
        const int seq = p.geom.tab[2 * c];
        start = p.geom.cu[seq] + p.geom.tab[2 * c + 1] * BT;
        len = min(BT, p.geom.cu[seq + 1] - start);
    }
    const int64_t base = b * p.sb + h * p.sh + (int64_t)start * p.st;
    const int lane = threadIdx.x;
    {   // branch-free loads (clamped row), all in flight before the first LDS write
        elemx8 v[NP];
#pragma unroll
        for (int m = 0; m < NP; ++m) {
            const int idx = min(m * NTH + lane, BT * CPR - 1);
            const int64_t off = base + (int64_t)min(idx / CPR, len - 1) * p.st + ((idx % CPR) << 3);
            if constexpr (F32IN) {
                const float *src = static_cast<const float *>(p.x) + off;
                v[m] = frag_from_acc(*reinterpret_cast<const f32x4 *>(src), *reinterpret_cast<const f32x4 *>(src + 4));
            } else {
                v[m] = *reinterpret_cast<const elemx8 *>(static_cast<const elem *>(p.x) + off);
            }
        }
#pragma unroll
        for (int m = 0; m < NP; ++m) {
            const int idx = m * NTH + lane;
            if (idx < BT * CPR) {
                const int r = idx / CPR, c8 = (idx % CPR) << 3;
#pragma unroll
                for (int e = 0; e < 8; ++e) A[r][c8 + e] = (r < len && c8 + e < r) ? (float)v[m][e] : 0.f;
            }
        }
    }
    __syncthreads();

    float x[BT];
#pragma unroll
    for (int i = 0; i < BT; ++i) x[i] = 0.f;
#pragma unroll
    for (int i = 0; i < BT; ++i) {
        float acc = (i == lane) ? 1.f : 0.f;
#pragma unroll
        for (int s4 = 0; s4 < (i + 3) / 4; ++s4) {
            const f32x4 a = *reinterpret_cast<const f32x4 *>(&A[i][4 * s4]);  // same address in every lane
            acc -= a[0] * x[4 * s4] + a[1] * x[4 * s4 + 1] + a[2] * x[4 * s4 + 2] + a[3] * x[4 * s4 + 3];
        }
        x[i] = acc;
    }
    __syncthreads();
    elem *O = reinterpret_cast<elem *>(&A[0][0]);  // [BT][BT + 8] 16-bit staging, fits in the fp32 tile
    const int ocol = lane < BT ? lane : BT;   // surplus lanes (BT < 64) land in the pad column, branch-free
#pragma unroll
    for (int i = 0; i < BT; ++i) O[i * PO + ocol] = (elem)x[i];
    __syncthreads();
    for (int idx = lane; idx < len * CPR; idx += NTH) {
        const int r = idx / CPR, c8 = (idx % CPR) << 3;
        *reinterpret_cast<u32x4 *>(p.out + base + (int64_t)r * p.st + c8) = *reinterpret_cast<const u32x4 *>(O + r * PO + c8);
    }
}

template <bool F32IN>
__global__ void __launch_bounds__(256) solve_tri64_kernel(const SolveParams p) {
    constexpr int BT = 64, pa = 68, pb = 72, NTH = 256;
    __shared__ __align__(16) float aS[BT * pa];
    __shared__ __align__(16) elem oS[BT * pb];
    const int c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    int start, len;
    if (p.geom.cu == nullptr) {
        start = c * BT;
        len = min(BT, p.geom.T - start);
    } else {
        const int seq = p.geom.tab[2 * c];
        start = p.geom.cu[seq] + p.geom.tab[2 * c + 1] * BT;
        len = min(BT, p.geom.cu[seq + 1] - start);
    }
    const int64_t base = b * p.sb + h * p.sh + (int64_t)start * p.st;
    const int tid = threadIdx.x;
    {   // two 8-element pieces per thread, rows past the end re-read the last valid row and are zeroed
        elemx8 v[2];
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            const int idx = m * NTH + tid;
            const int64_t off = base + (int64_t)min(idx >> 3, len - 1) * p.st + ((idx & 7) << 3);
            if constexpr (F32IN) {
                const float *src = static_cast<const float *>(p.x) + off;
                v[m] = frag_from_acc(*reinterpret_cast<const f32x4 *>(src), *reinterpret_cast<const f32x4 *>(src + 4));
            } else {
                v[m] = *reinterpret_cast<const elemx8 *>(static_cast<const elem *>(p.x) + off);
            }
        }
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            const int idx = m * NTH + tid;
            const int r = idx >> 3, c8 = (idx & 7) << 3;
            f32x4 lo, hi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[e] = (r < len && c8 + e < r) ? (float)v[m][e] : 0.f;
                hi[e] = (r < len && c8 + 4 + e < r) ? (float)v[m][4 + e] : 0.f;
            }
            *reinterpret_cast<f32x4 *>(aS + r * pa + c8) = lo;
            *reinterpret_cast<f32x4 *>(aS + r * pa + c8 + 4) = hi;
        }
    }
    __syncthreads();

    invert64(aS, oS);
    for (int idx = tid; idx < len * 8; idx += NTH) {
        const int r = idx >> 3, c8 = (idx & 7) << 3;
        *reinterpret_cast<u32x4 *>(p.out + base + (int64_t)r * p.st + c8) = *reinterpret_cast<const u32x4 *>(oS + r * pb + c8);
    }
}

// chunk_scaled_dot_kkt followed by the inversion, without the round trip of the fp32 matrix through memory: the
// scores are rounded to the element type as solve_tri rounds its input, so the result equals the two operators'.
__global__ void __launch_bounds__(kThreads) kkt_inverse_kernel(const KktParams p, elem *inv) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int C = kChunk, pa = 68, pb = 72;
    const int K = p.geom.K, pitch = K + 8;
    // the score tile and the result take the place of the k rows once every wave holds its scores in registers
    float *gS = reinterpret_cast<float *>(smem);
    float *bS = gS + C;
    elem *kS = reinterpret_cast<elem *>(bS + C);
    float *aS = reinterpret_cast<float *>(kS);
    elem *oS = reinterpret_cast<elem *>(aS + C * pa);

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st;
    load_tile<kThreads>(kS, pitch, kg, p.k.st, C, K, len);
    if (threadIdx.x < C) {
        const int t = threadIdx.x;
        gS[t] = t < len ? load_scalar(p.g, b, hv, start + t) : 0.f;
        bS[t] = t < len ? load_scalar(p.beta, b, hv, start + t) : 0.f;
    }
    __syncthreads();
    {
        const int t = wave_id() * 16 + acc_col();
        f32x4 acc[C / 16];
        switch (wave_id()) {
            case 0: kkt_score_rows<0>(kS, pitch, K, gS, bS, len, acc); break;
            case 1: kkt_score_rows<1>(kS, pitch, K, gS, bS, len, acc); break;
            case 2: kkt_score_rows<2>(kS, pitch, K, gS, bS, len, acc); break;
            default: kkt_score_rows<3>(kS, pitch, K, gS, bS, len, acc); break;
        }
        __syncthreads();   // the k rows have been read by every wave
#pragma unroll
        for (int J = 0; J < C / 16; ++J) *reinterpret_cast<f32x4 *>(aS + t * pa + J * 16 + 4 * (lane_id() >> 4)) = acc[J];
    }
    __syncthreads();
    invert64(aS, oS);
    elem *og = inv + ((int64_t)(b * p.geom.Hv + hv) * p.geom.T + start) * C;
    for (int idx = threadIdx.x; idx < len * 8; idx += kThreads) {
        const int r = idx >> 3, c8 = (idx & 7) << 3;
        *reinterpret_cast<u32x4 *>(og + (int64_t)r * C + c8) = *reinterpret_cast<const u32x4 *>(oS + r * pb + c8);
    }
}

// =============================================================================
// recompute_w_u_fwd
// =============================================================================
struct WuParams {
    ChunkGeom geom;
    View4 k, v, A, w, u;
    View3 g, beta;
};

__global__ void __launch_bounds__(kThreads) wu_kernel_generic(const WuParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int K = p.geom.K, V = p.geom.V;
    const int pa = kChunk + 8, pk = K + 16, pv = V + 16;
    elem *aS = reinterpret_cast<elem *>(smem);
    elem *kS = aS + kChunk * pa;
    elem *vS = kS + kChunk * pk;
    float *gS = reinterpret_cast<float *>(vS + kChunk * pv);
    float *bS = gS + kChunk;

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    if (threadIdx.x < kChunk) {
        const int t = threadIdx.x;
        gS[t] = t < len ? __expf(load_scalar(p.g, b, hv, start + t)) : 0.f;
        bS[t] = t < len ? load_scalar(p.beta, b, hv, start + t) : 0.f;
    }
    const elem *ag = static_cast<const elem *>(p.A.p) + b * p.A.sb + hv * p.A.sh + (int64_t)start * p.A.st;
    for (int idx = threadIdx.x; idx < kChunk * 8; idx += kThreads) {
        const int r = idx >> 3, c8 = (idx & 7) << 3;
        elemx8 a;
        if (r < len) a = *reinterpret_cast<const elemx8 *>(ag + (int64_t)r * p.A.st + c8);
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (!(r < len && c8 + e < len)) a[e] = (elem)0.f;  // columns past the tail are not part of the block
        *reinterpret_cast<elemx8 *>(aS + r * pa + c8) = a;
    }
    __syncthreads();  // gS, bS visible
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st;
    const elem *vg = static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st;
    for (int idx = threadIdx.x; idx < kChunk * (K >> 3); idx += kThreads) {
        const int r = idx / (K >> 3), c8 = (idx % (K >> 3)) << 3;
        elemx8 o;
        if (r < len) {
            const elemx8 a = *reinterpret_cast<const elemx8 *>(kg + (int64_t)r * p.k.st + c8);
            const float s = bS[r] * gS[r];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (elem)((float)a[e] * s);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (elem)0.f;
        }
        *reinterpret_cast<elemx8 *>(kS + r * pk + c8) = o;
    }
    for (int idx = threadIdx.x; idx < kChunk * (V >> 3); idx += kThreads) {
        const int r = idx / (V >> 3), c8 = (idx % (V >> 3)) << 3;
        elemx8 o;
        if (r < len) {
            const elemx8 a = *reinterpret_cast<const elemx8 *>(vg + (int64_t)r * p.v.st + c8);
            const float s = bS[r];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (elem)((float)a[e] * s);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (elem)0.f;
        }
        *reinterpret_cast<elemx8 *>(vS + r * pv + c8) = o;
    }
    __syncthreads();

    // Each wave owns a quarter of the output columns of w and of u and overwrites
    // exactly those columns of the staged operand once its products are done.
    const int w = wave_id();
    auto product = [&](elem *tile, int pitch, int ncols) {
        const int per_wave = ncols / 64;  // 16-column tiles per wave
        for (int m = 0; m < per_wave; ++m) {
            const int c0 = (w * per_wave + m) * 16;
            f32x4 acc[4];
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const elemx8 bfrag = frag_tr(tile, pitch, c0, 32 * j);
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) acc[rt] = mfma16x32(frag_kc(aS, pa, rt * 16, 32 * j), bfrag, acc[rt]);
            }
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) acc_to_tile(tile, pitch, rt * 16, c0, acc[rt]);
        }
    };
    product(kS, pk, K);
    product(vS, pv, V);
    __syncthreads();
    elem *wg = static_cast<elem *>(const_cast<void *>(p.w.p)) + b * p.w.sb + hv * p.w.sh + (int64_t)start * p.w.st;
    elem *ug = static_cast<elem *>(const_cast<void *>(p.u.p)) + b * p.u.sb + hv * p.u.sh + (int64_t)start * p.u.st;
    store_tile<kThreads>(wg, p.w.st, kS, pk, K, len);
    store_tile<kThreads>(ug, p.u.st, vS, pv, V, len);
}

// Compile-time head sizes: every load of the chunk (A, k, v tiles, gates) is issued before the first
// LDS write waits for one of them.
template <int K, int V, int C = kChunk>
__global__ void __launch_bounds__(kThreads) wu_kernel(const WuParams p) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pa = C + 8, pk = K + 16, pv = V + 16;   // C = tokens per chunk (64 or 128)
    elem *aS = reinterpret_cast<elem *>(smem);
    elem *kS = aS + C * pa;
    elem *vS = kS + C * pk;

    int c, hv;
    block_chunk_head(p.geom, c, hv);
    const int b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, start, len;
    chunk_span(p.geom, b, c, seq, start, len);
    const int tid = threadIdx.x;
    const elem *ag = static_cast<const elem *>(p.A.p) + b * p.A.sb + hv * p.A.sh + (int64_t)start * p.A.st;
    const elem *kg = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh + (int64_t)start * p.k.st;
    const elem *vg = static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh + (int64_t)start * p.v.st;
    {
        TileCopy<kThreads, C, C> ta;
        TileCopy<kThreads, C, K> tk;
        TileCopy<kThreads, C, V> tv;
        ta.fetch(ag, p.A.st, len, tid);
        tk.fetch(kg, p.k.st, len, tid);
        tv.fetch(vg, p.v.st, len, tid);
        // per-row scale factors of the pieces this thread holds
        float sk[TileCopy<kThreads, C, K>::N], sv[TileCopy<kThreads, C, V>::N];
#pragma unroll
        for (int m = 0; m < TileCopy<kThreads, C, K>::N; ++m) {
            const int r = min((m * kThreads + tid) / (K / 8), len - 1);
            sk[m] = load_scalar(p.beta, b, hv, start + r) * __expf(load_scalar(p.g, b, hv, start + r));
        }
#pragma unroll
        for (int m = 0; m < TileCopy<kThreads, C, V>::N; ++m)
            sv[m] = load_scalar(p.beta, b, hv, start + min((m * kThreads + tid) / (V / 8), len - 1));
#pragma unroll
        for (int m = 0; m < TileCopy<kThreads, C, C>::N; ++m) {   // columns past the tail are not part of the block
            const int idx = m * kThreads + tid;
            const int r = idx / (C / 8), c8 = (idx % (C / 8)) << 3;
            elemx8 a = __builtin_bit_cast(elemx8, ta.r[m]);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (!(r < len && c8 + e < len)) a[e] = (elem)0.f;
            *reinterpret_cast<elemx8 *>(aS + r * pa + c8) = a;
        }
        auto scaled = [&](elem *dst, int pitch, int cpr, int m, u32x4 raw, float sc) {
            const int idx = m * kThreads + tid;
            const int r = idx / cpr, c8 = (idx % cpr) << 3;
            const elemx8 a = __builtin_bit_cast(elemx8, raw);
            const float f = r < len ? sc : 0.f;
            f32x4 lo, hi;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                lo[e] = (float)a[e] * f;
                hi[e] = (float)a[4 + e] * f;
            }
            *reinterpret_cast<elemx8 *>(dst + r * pitch + c8) = frag_from_acc(lo, hi);
        };
#pragma unroll
        for (int m = 0; m < TileCopy<kThreads, C, K>::N; ++m) scaled(kS, pk, K / 8, m, tk.r[m], sk[m]);
#pragma unroll
        for (int m = 0; m < TileCopy<kThreads, C, V>::N; ++m) scaled(vS, pv, V / 8, m, tv.r[m], sv[m]);
    }
    __syncthreads();

    // Each wave owns a quarter of the output columns of w and of u and overwrites
    // exactly those columns of the staged operand once its products are done.
    const int w = wave_id();
    auto product = [&](elem *tile, int pitch, int ncols) {
        const int per_wave = ncols / 64;  // 16-column tiles per wave
        for (int m = 0; m < per_wave; ++m) {
            const int c0 = (w * per_wave + m) * 16;
            f32x4 acc[C / 16];
#pragma unroll
            for (int rt = 0; rt < C / 16; ++rt) acc[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < C / 32; ++j) {
                const elemx8 bfrag = frag_tr(tile, pitch, c0, 32 * j);
#pragma unroll
                for (int rt = 0; rt < C / 16; ++rt)
                    if (32 * j <= 16 * rt + 15) acc[rt] = mfma16x32(frag_kc(aS, pa, rt * 16, 32 * j), bfrag, acc[rt]);   // A is lower triangular
            }
#pragma unroll
            for (int rt = 0; rt < C / 16; ++rt) acc_to_tile(tile, pitch, rt * 16, c0, acc[rt]);
        }
    };
    product(kS, pk, K);
    product(vS, pv, V);
    __syncthreads();
    elem *wg = static_cast<elem *>(const_cast<void *>(p.w.p)) + b * p.w.sb + hv * p.w.sh + (int64_t)start * p.w.st;
    elem *ug = static_cast<elem *>(const_cast<void *>(p.u.p)) + b * p.u.sb + hv * p.u.sh + (int64_t)start * p.u.st;
    store_tile<kThreads>(wg, p.w.st, kS, pk, K, len);
    store_tile<kThreads>(ug, p.u.st, vS, pv, V, len);
}

// =============================================================================
// chunk_fwd_o
// =============================================================================
struct FwdOParams {
    ChunkGeom geom;
    View4 q, k, v, o;
    const elem *h;
    int64_t h_sb, h_sh, h_sc;  // h [B,Hv,NT,K,V]: batch, head, chunk strides (K,V contiguous)
    View3 g;
    float scale;
};

// Eight waves when the value dimension gives each of them a 16-column tile (V >= 128): the tiles of one chunk
// take 97 KB of LDS, so a compute unit holds one workgroup and needs the waves of that one to hide latency.
// SUB = 64-token row tiles per chunk (2 for 128-token chunks): a workgroup owns one row tile; the second tile of a
// chunk also contracts over the k / v_new rows of the first (whole block, no causal mask), one block at a time.
template <int K, int V, int SUB = 1>
__global__ void __launch_bounds__(V >= 128 ? 512 : 256) fwd_o_kernel(const FwdOParams p) {
    constexpr int NTH = V >= 128 ? 512 : 256, NW = NTH / 64;
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int pq = K + 8, pv = V + 16, pp = kChunk + 8;
    constexpr int CT = V / (16 * NW);  // 16-column tiles per wave
    elem *qS = reinterpret_cast<elem *>(smem);
    elem *kS = qS + kChunk * pq;
    elem *vS = kS + kChunk * pq;
    elem *hS = vS + kChunk * pv;
    elem *pS = hS + K * pv;
    float *gS = reinterpret_cast<float *>(pS + kChunk * pp);   // gates of the row tile
    float *gC = gS + kChunk;                                   // gates of the current column block

    int cx, hv;
    block_chunk_head(p.geom, cx, hv);
    const int c = cx / SUB, r = cx % SUB, b = blockIdx.z;
    const int hk = hv / (p.geom.Hv / p.geom.Hk);
    int seq, cstart, clen;
    chunk_span(p.geom, b, c, seq, cstart, clen);
    const int start = cstart + r * kChunk;          // first token of this row tile
    const int len = min(kChunk, clen - r * kChunk);
    if (len <= 0) return;
    const elem *qg = static_cast<const elem *>(p.q.p) + b * p.q.sb + hk * p.q.sh + (int64_t)start * p.q.st;
    const elem *kbase = static_cast<const elem *>(p.k.p) + b * p.k.sb + hk * p.k.sh;
    const elem *vbase = static_cast<const elem *>(p.v.p) + b * p.v.sb + hv * p.v.sh;
    const elem *hg = p.h + b * p.h_sb + hv * p.h_sh + (int64_t)c * p.h_sc;
    const int tid = threadIdx.x;
    const int w = wave_id();

    f32x4 acc[4][CT];
#pragma unroll
    for (int jb = 0; jb <= (SUB > 1 ? r : 0); ++jb) {
        const int bstart = cstart + jb * kChunk;                    // first token of the column block
        const int blen = jb == r ? len : kChunk;                    // earlier blocks of the chunk are complete
        if (jb > 0) __syncthreads();                                // the previous block's tiles are no longer read
        {   // every load of the pass is in flight before the first LDS write waits
            TileCopy<NTH, kChunk, K> tq, tk;
            TileCopy<NTH, kChunk, V> tv;
            TileCopy<NTH, K, V> th;
            if (jb == 0) {
                tq.fetch(qg, p.q.st, len, tid);
                th.fetch(hg, V, K, tid);
            }
            tk.fetch(kbase + (int64_t)bstart * p.k.st, p.k.st, blen, tid);
            tv.fetch(vbase + (int64_t)bstart * p.v.st, p.v.st, blen, tid);
            float gv = 0.f, gc = 0.f;
            if (tid < kChunk) {
                if (jb == 0) gv = load_scalar(p.g, b, hv, start + min(tid, len - 1));
                gc = load_scalar(p.g, b, hv, bstart + min(tid, blen - 1));
            }
            if (jb == 0) {
                tq.commit(qS, pq, len, tid);
                th.commit(hS, pv, K, tid);
            }
            tk.commit(kS, pq, blen, tid);
            tv.commit(vS, pv, blen, tid);
            if (tid < kChunk) {
                if (jb == 0) gS[tid] = tid < len ? gv : 0.f;
                gC[tid] = tid < blen ? gc : 0.f;
            }
        }
        __syncthreads();

        // decayed (and, on the diagonal block, causally masked) scores P[t][s], computed as the transposed tile so
        // that a lane holds four consecutive s of one row t
        const bool diag = jb == r;
        for (int m = 0; m < 16 / NW; ++m) {
            const int id = w + NW * m, I = id >> 2, J = id & 3;  // t block, s block
            f32x4 sc = {0.f, 0.f, 0.f, 0.f};
            const int t = I * 16 + acc_col();
            if (!diag || J <= I) {
#pragma unroll
                for (int kk = 0; kk < K; kk += 32) sc = mfma16x32(frag_kc(kS, pq, J * 16, kk), frag_kc(qS, pq, I * 16, kk), sc);
                const float gt = gS[t];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int s2 = J * 16 + acc_row(e);
                    sc[e] = (!diag || s2 <= t) ? sc[e] * __expf(fminf(gt - gC[s2], 0.f)) : 0.f;
                }
            }
            *reinterpret_cast<elemx4 *>(pS + t * pp + J * 16 + 4 * (lane_id() >> 4)) = cvt4(sc);
        }

        if (jb == 0) {   // inter-chunk term e^{G_t} (q h) for this wave's V columns
#pragma unroll
            for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) acc[rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < K / 32; ++j) {
                elemx8 bfrag[CT];
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) bfrag[ct] = frag_tr(hS, pv, (w * CT + ct) * 16, 32 * j);
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) {
                    const elemx8 afrag = frag_kc(qS, pq, rt * 16, 32 * j);
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) acc[rt][ct] = mfma16x32(afrag, bfrag[ct], acc[rt][ct]);
                }
            }
#pragma unroll
            for (int rt = 0; rt < 4; ++rt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float eg = __expf(gS[rt * 16 + acc_row(e)]);
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) acc[rt][ct][e] *= eg;
                }
        }
        __syncthreads();  // P complete

#pragma unroll
        for (int j = 0; j < 2; ++j) {
            elemx8 bfrag[CT];
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) bfrag[ct] = frag_tr(vS, pv, (w * CT + ct) * 16, 32 * j);
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const elemx8 afrag = frag_kc(pS, pp, rt * 16, 32 * j);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) acc[rt][ct] = mfma16x32(afrag, bfrag[ct], acc[rt][ct]);
            }
        }
    }
    // this wave's columns of the v tile are no longer needed: stage o there
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) acc_to_tile(vS, pv, rt * 16, (w * CT + ct) * 16, acc[rt][ct] * p.scale);
    __syncthreads();
    elem *og = static_cast<elem *>(const_cast<void *>(p.o.p)) + b * p.o.sb + hv * p.o.sh + (int64_t)start * p.o.st;
    store_tile<NTH>(og, p.o.st, vS, pv, V, len);
}

// ---- host side ------------------------------------------------------------------
int kkt_impl(const fla_tensor *k, const fla_tensor *g, const fla_tensor *beta, const fla_int_array *cu,
             const fla_int_array *ci, int64_t chunk_size, const fla_tensor *out, void *ws, uint64_t ws_size,
             hipStream_t stream, uint64_t *query, bool inverse = false) {
    const char *op = inverse ? "chunk_scaled_dot_kkt_inverse" : "chunk_scaled_dot_kkt";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, nullptr, g, chunk_size, geom, kElemDtype, 128))) return rc;
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, dt_bit(kElemDtype)))) return rc;
    if ((rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    if ((rc = check_bht(op, "beta", beta, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    if ((rc = check_tensor(out, op, "out", 4, dt_bit(inverse ? kElemDtype : FLA_F32)))) return rc;
    FLA_REQUIRE(!inverse || (geom.C == kChunk && is_contiguous(out)), FLA_ERR_UNSUPPORTED,
                "%s: built for 64-token chunks and a contiguous result.", op);
    FLA_REQUIRE(out->shape[0] == geom.B && out->shape[1] == geom.Hv && out->shape[2] == geom.T && out->shape[3] == geom.C &&
                    inner_unit(out) && out->stride[2] % 4 == 0 && out->stride[1] % 4 == 0 && out->stride[0] % 4 == 0,
                FLA_ERR_SHAPE, "%s: out must be a 16-byte aligned [B,Hv,T,%d].", op, geom.C);
    FLA_REQUIRE(geom.K % 32 == 0 && geom.K >= 32 && geom.K <= 256, FLA_ERR_UNSUPPORTED,
                "%s: K must be a multiple of 32 in [32,256], got %d.", op, geom.K);
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    KktParams p{geom, view4(k), view3(g), view3(beta), inverse ? nullptr : static_cast<float *>(out->data), out->stride[0],
                out->stride[1], out->stride[2]};
    const size_t smem = (size_t)geom.C * (geom.K + 8) * 2 + 2 * geom.C * 4;
    if (inverse) {
        const size_t tiles = (size_t)kChunk * 68 * 4 + (size_t)kChunk * 72 * 2, rows = (size_t)kChunk * (geom.K + 8) * 2;
        const size_t ismem = (tiles > rows ? tiles : rows) + 2 * kChunk * 4;
        FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kkt_inverse_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)ismem));
        FLA_LAUNCH("kkt_inverse", stream, kkt_inverse_kernel, chunk_head_grid(geom, geom.NT, geom.Hv), dim3(kThreads), ismem, stream, p,
                   static_cast<elem *>(out->data));
    } else if (geom.C == 128) {
        FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kkt_kernel<128>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                          (int)smem));
        FLA_LAUNCH("kkt", stream, kkt_kernel<128>, chunk_head_grid(geom, geom.NT, geom.Hv), dim3(kThreads), smem, stream, p);
    } else {
        FLA_LAUNCH("kkt", stream, kkt_kernel<64>, chunk_head_grid(geom, geom.NT, geom.Hv), dim3(kThreads), smem, stream, p);
    }
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int solve_impl(const fla_tensor *x, const fla_int_array *cu, const fla_int_array *ci, const char *layout,
               const fla_tensor *out, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "solve_tri";
    int rc;
    if ((rc = check_tensor(x, op, "x", -1, dt_bit(kElemDtype) | dt_bit(FLA_F32)))) return rc;
    if ((rc = check_tensor(out, op, "out", -1, dt_bit(kElemDtype)))) return rc;
    FLA_REQUIRE(layout != nullptr, FLA_ERR_NULL, "%s: layout must not be null.", op);
    FLA_REQUIRE(same_shape(x, out), FLA_ERR_SHAPE, "%s: out must have the shape of x.", op);
    FLA_REQUIRE(is_contiguous(x) && is_contiguous(out), FLA_ERR_SHAPE, "%s: x and out must be contiguous.", op);
    int ib, ih, it;  // dims of batch, head, token (-1: absent)
    char lay[8] = {0};
    for (int i = 0; i < 7 && layout[i]; ++i) lay[i] = (char)tolower(layout[i]);
    if (!strcmp(lay, "bnsd")) { ib = 0; ih = 1; it = 2; }
    else if (!strcmp(lay, "bsnd")) { ib = 0; it = 1; ih = 2; }
    else if (!strcmp(lay, "tnd")) { ib = -1; it = 0; ih = 1; }
    else if (!strcmp(lay, "ntd")) { ib = -1; ih = 0; it = 1; }
    else return fail(FLA_ERR_UNSUPPORTED, "%s: unknown layout '%s' (bsnd, bnsd, tnd, ntd).", op, layout);
    FLA_REQUIRE(x->ndim == (ib < 0 ? 3 : 4), FLA_ERR_SHAPE, "%s: rank does not match layout '%s'.", op, layout);
    const int BT = (int)x->shape[x->ndim - 1];
    FLA_REQUIRE(BT == 16 || BT == 32 || BT == 64 || BT == 128, FLA_ERR_UNSUPPORTED,
                "%s: block size (last dimension) must be 16, 32, 64 or 128, got %lld.", op, (long long)x->shape[x->ndim - 1]);
    ChunkGeom geom{};
    geom.B = ib < 0 ? 1 : (int)x->shape[ib];
    geom.Hv = geom.Hk = (int)x->shape[ih];
    geom.T = (int)x->shape[it];
    FLA_REQUIRE(x->shape[it] < ((int64_t)1 << 31) && x->shape[ih] < 65536 && geom.B < 65536, FLA_ERR_SHAPE,
                "%s: extents too large.", op);
    geom.NT = (geom.T + BT - 1) / BT;
    geom.N = geom.B;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query, BT)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0 || geom.Hv == 0) return FLA_OK;
    SolveParams p{geom, x->data, static_cast<elem *>(out->data), ib < 0 ? 0 : x->stride[ib], x->stride[ih], x->stride[it]};
    const dim3 grid(geom.NT, geom.Hv, geom.B);
#define FLA_LAUNCH_SOLVE(BTV, NTHV)                                                                          \
    if (x->dtype == FLA_F32) FLA_LAUNCH("solve_tri", stream, (solve_tri_kernel<BTV, true>), grid, dim3(NTHV), 0, stream, p); \
    else FLA_LAUNCH("solve_tri", stream, (solve_tri_kernel<BTV, false>), grid, dim3(NTHV), 0, stream, p)
    switch (BT) {
        case 16: FLA_LAUNCH_SOLVE(16, 64); break;
        case 32: FLA_LAUNCH_SOLVE(32, 64); break;
        case 64:
            if (x->dtype == FLA_F32) FLA_LAUNCH("solve_tri", stream, (solve_tri64_kernel<true>), grid, dim3(256), 0, stream, p);
            else FLA_LAUNCH("solve_tri", stream, (solve_tri64_kernel<false>), grid, dim3(256), 0, stream, p);
            break;
        default: FLA_LAUNCH_SOLVE(128, 128); break;
    }
#undef FLA_LAUNCH_SOLVE
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int wu_impl(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *g,
            const fla_tensor *gk, const fla_int_array *cu, const fla_int_array *ci, int64_t chunk_size,
            const fla_tensor *w, const fla_tensor *u, void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "recompute_w_u_fwd";
    FLA_REQUIRE(gk == nullptr || gk->data == nullptr, FLA_ERR_UNSUPPORTED, "%s: gk must be None.", op);
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v, nullptr, chunk_size, geom, kElemDtype, 128))) return rc;
    const int bf = dt_bit(kElemDtype);
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bhtd(op, "A", A, geom.B, geom.Hv, geom.T, geom.C, bf))) return rc;
    if ((rc = check_bhtd(op, "w", w, geom.B, geom.Hv, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "u", u, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bht(op, "beta", beta, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    FLA_REQUIRE(g != nullptr && g->data != nullptr, FLA_ERR_NULL, "%s: g must be provided.", op);
    FLA_REQUIRE(geom.C == kChunk || ((geom.K == 128 || geom.K == 64) && (geom.V == geom.K || geom.V == 2 * geom.K)),
                FLA_ERR_UNSUPPORTED, "%s: chunk_size 128 is built for (K,V) in (128,128),(128,256),(64,64),(64,128).", op);
    if ((rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    FLA_REQUIRE(geom.K % 64 == 0 && geom.V % 64 == 0 && geom.K <= 256 && geom.V <= 256, FLA_ERR_UNSUPPORTED,
                "%s: K and V must be multiples of 64 up to 256, got K=%d V=%d.", op, geom.K, geom.V);
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query)) || query) return rc;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    WuParams p{geom, view4(k), view4(v), view4(A), view4(w), view4(u), view3(g), view3(beta)};
    const size_t smem = (size_t)geom.C * ((geom.C + 8) + (geom.K + 16) + (geom.V + 16)) * 2 + 2 * kChunk * 4;
    const dim3 grid = chunk_head_grid(geom, geom.NT, geom.Hv);
#define FLA_LAUNCH_WU(KERNEL)                                                                                      \
    do {                                                                                                           \
        FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(KERNEL), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                          (int)smem));                                                             \
        FLA_LAUNCH("wu", stream, KERNEL, grid, dim3(kThreads), smem, stream, p);                                    \
    } while (0)
    if (geom.C == 128 && geom.K == 128 && geom.V == 128) FLA_LAUNCH_WU((wu_kernel<128, 128, 128>));
    else if (geom.C == 128 && geom.K == 128) FLA_LAUNCH_WU((wu_kernel<128, 256, 128>));
    else if (geom.C == 128 && geom.V == 64) FLA_LAUNCH_WU((wu_kernel<64, 64, 128>));
    else if (geom.C == 128) FLA_LAUNCH_WU((wu_kernel<64, 128, 128>));
    else if (geom.K == 128 && geom.V == 128) FLA_LAUNCH_WU((wu_kernel<128, 128>));
    else if (geom.K == 128 && geom.V == 256) FLA_LAUNCH_WU((wu_kernel<128, 256>));
    else if (geom.K == 64 && geom.V == 64) FLA_LAUNCH_WU((wu_kernel<64, 64>));
    else if (geom.K == 64 && geom.V == 128) FLA_LAUNCH_WU((wu_kernel<64, 128>));
    else FLA_LAUNCH_WU(wu_kernel_generic);
#undef FLA_LAUNCH_WU
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

template <int K, int V, int SUB = 1>
int launch_fwd_o(const FwdOParams &p, hipStream_t stream) {
    const size_t smem = ((size_t)2 * kChunk * (K + 8) + (size_t)(kChunk + K) * (V + 16) + kChunk * (kChunk + 8)) * 2 + 2 * kChunk * 4;
    FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(fwd_o_kernel<K, V, SUB>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    FLA_LAUNCH("fwd_o", stream, (fwd_o_kernel<K, V, SUB>), chunk_head_grid(p.geom, p.geom.NT * SUB, p.geom.Hv), dim3(V >= 128 ? 512 : 256),
               smem, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int fwd_o_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *h, const fla_tensor *g,
               const fla_int_array *cu, const fla_int_array *ci, double scale, int64_t chunk_size, const fla_tensor *out,
               void *ws, uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_fwd_o";
    ChunkGeom geom;
    int rc;
    if ((rc = gdn_geometry(op, k, v, nullptr, chunk_size, geom, kElemDtype, 128))) return rc;
    const int bf = dt_bit(kElemDtype);
    if ((rc = check_bhtd(op, "q", q, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "k", k, geom.B, geom.Hk, geom.T, geom.K, bf))) return rc;
    if ((rc = check_bhtd(op, "v", v, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    if ((rc = check_bhtd(op, "out", out, geom.B, geom.Hv, geom.T, geom.V, bf))) return rc;
    FLA_REQUIRE(g != nullptr && g->data != nullptr, FLA_ERR_NULL, "%s: g must be provided.", op);
    if ((rc = check_bht(op, "g", g, geom.B, geom.Hv, geom.T, kElemDtype))) return rc;
    Varlen vl;
    if ((rc = finish_varlen(op, vl, geom, cu, ci, ws, ws_size, stream, query))) return rc;
    if ((rc = check_tensor(h, op, "h", 5, bf))) return rc;
    FLA_REQUIRE(h->shape[0] == geom.B && h->shape[1] == geom.Hv && h->shape[2] == geom.NT && h->shape[3] == geom.K &&
                    h->shape[4] == geom.V && h->stride[4] == 1 && h->stride[3] == geom.V && h->stride[2] % 8 == 0 &&
                    h->stride[1] % 8 == 0 && h->stride[0] % 8 == 0,
                FLA_ERR_SHAPE, "%s: h must be [B,Hv,NT=%d,K,V] with contiguous K x V blocks.", op, geom.NT);
    if (query) return FLA_OK;
    if (geom.NT == 0 || geom.B == 0) return FLA_OK;
    FwdOParams p{geom, view4(q), view4(k), view4(v), view4(out), static_cast<const elem *>(h->data),
                 h->stride[0], h->stride[1], h->stride[2], view3(g), (float)scale};
    if (geom.C == 128) {
        if (geom.K == 128 && geom.V == 128) return launch_fwd_o<128, 128, 2>(p, stream);
        if (geom.K == 128 && geom.V == 256) return launch_fwd_o<128, 256, 2>(p, stream);
        if (geom.K == 64 && geom.V == 64) return launch_fwd_o<64, 64, 2>(p, stream);
        if (geom.K == 64 && geom.V == 128) return launch_fwd_o<64, 128, 2>(p, stream);
        return fail(FLA_ERR_UNSUPPORTED, "%s: chunk_size 128 is built for (K,V) in (128,128),(128,256),(64,64),(64,128).", op);
    }
    if (geom.K == 128 && geom.V == 128) return launch_fwd_o<128, 128>(p, stream);
    if (geom.K == 128 && geom.V == 256) return launch_fwd_o<128, 256>(p, stream);
    if (geom.K == 64 && geom.V == 64) return launch_fwd_o<64, 64>(p, stream);
    if (geom.K == 64 && geom.V == 128) return launch_fwd_o<64, 128>(p, stream);
    return fail(FLA_ERR_UNSUPPORTED, "%s: (K,V)=(%d,%d) has no kernel; built: (128,128),(128,256),(64,64),(64,128).", op,
                geom.K, geom.V);
}

}  // namespace
}  // namespace fla

#define FLA_NULL_WS(op) \
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, op ": workspace_size must not be null.")

FLA_ENTRY(fla_chunk_scaled_dot_kkt_get_workspace_size)(const fla_tensor *k, const fla_tensor *g,
                                                           const fla_tensor *beta, const fla_int_array *cu_seqlens,
                                                           const fla_int_array *chunk_indices, int64_t chunk_size,
                                                           const fla_tensor *out, uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_chunk_scaled_dot_kkt_get_workspace_size, k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, workspace_size);
    FLA_NULL_WS("chunk_scaled_dot_kkt");
    return fla::guarded([&] { return fla::kkt_impl(k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, nullptr, 0, nullptr, workspace_size); });
}
FLA_ENTRY(fla_chunk_scaled_dot_kkt)(const fla_tensor *k, const fla_tensor *g, const fla_tensor *beta,
                                        const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
                                        int64_t chunk_size, const fla_tensor *out, void *workspace,
                                        uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_chunk_scaled_dot_kkt, k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::kkt_impl(k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, workspace, workspace_size,
                         static_cast<hipStream_t>(stream), nullptr); });
}
FLA_ENTRY(fla_chunk_scaled_dot_kkt_inverse_get_workspace_size)(const fla_tensor *k, const fla_tensor *g,
                                                                   const fla_tensor *beta, const fla_int_array *cu_seqlens,
                                                                   const fla_int_array *chunk_indices, int64_t chunk_size,
                                                                   const fla_tensor *out, uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_chunk_scaled_dot_kkt_inverse_get_workspace_size, k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, workspace_size);
    FLA_NULL_WS("chunk_scaled_dot_kkt_inverse");
    return fla::guarded([&] { return fla::kkt_impl(k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, nullptr, 0, nullptr, workspace_size, true); });
}
FLA_ENTRY(fla_chunk_scaled_dot_kkt_inverse)(const fla_tensor *k, const fla_tensor *g, const fla_tensor *beta,
                                                const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
                                                int64_t chunk_size, const fla_tensor *out, void *workspace,
                                                uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_chunk_scaled_dot_kkt_inverse, k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::kkt_impl(k, g, beta, cu_seqlens, chunk_indices, chunk_size, out, workspace, workspace_size,
                         static_cast<hipStream_t>(stream), nullptr, true); });
}

FLA_ENTRY(fla_solve_tri_get_workspace_size)(const fla_tensor *x, const fla_int_array *cu_seqlens,
                                                const fla_int_array *chunk_indices, const char *layout,
                                                const fla_tensor *out, uint64_t *workspace_size) {
    FLA_ROUTE_F16(out, fla_solve_tri_get_workspace_size, x, cu_seqlens, chunk_indices, layout, out, workspace_size);
    FLA_NULL_WS("solve_tri");
    return fla::guarded([&] { return fla::solve_impl(x, cu_seqlens, chunk_indices, layout, out, nullptr, 0, nullptr, workspace_size); });
}
FLA_ENTRY(fla_solve_tri)(const fla_tensor *x, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
                             const char *layout, const fla_tensor *out, void *workspace, uint64_t workspace_size,
                             void *stream) {
    FLA_ROUTE_F16(out, fla_solve_tri, x, cu_seqlens, chunk_indices, layout, out, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::solve_impl(x, cu_seqlens, chunk_indices, layout, out, workspace, workspace_size,
                           static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_recompute_w_u_fwd_get_workspace_size)(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta,
                                                        const fla_tensor *A, const fla_tensor *g, const fla_tensor *gk,
                                                        const fla_int_array *cu_seqlens,
                                                        const fla_int_array *chunk_indices, int64_t chunk_size,
                                                        const fla_tensor *w, const fla_tensor *u,
                                                        uint64_t *workspace_size) {
    FLA_ROUTE_F16(k, fla_recompute_w_u_fwd_get_workspace_size, k, v, beta, A, g, gk, cu_seqlens, chunk_indices, chunk_size, w, u, workspace_size);
    FLA_NULL_WS("recompute_w_u_fwd");
    return fla::guarded([&] { return fla::wu_impl(k, v, beta, A, g, gk, cu_seqlens, chunk_indices, chunk_size, w, u, nullptr, 0, nullptr,
                        workspace_size); });
}
FLA_ENTRY(fla_recompute_w_u_fwd)(const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta,
                                     const fla_tensor *A, const fla_tensor *g, const fla_tensor *gk,
                                     const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
                                     int64_t chunk_size, const fla_tensor *w, const fla_tensor *u, void *workspace,
                                     uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(k, fla_recompute_w_u_fwd, k, v, beta, A, g, gk, cu_seqlens, chunk_indices, chunk_size, w, u, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::wu_impl(k, v, beta, A, g, gk, cu_seqlens, chunk_indices, chunk_size, w, u, workspace, workspace_size,
                        static_cast<hipStream_t>(stream), nullptr); });
}

FLA_ENTRY(fla_chunk_fwd_o_get_workspace_size)(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v,
                                                  const fla_tensor *h, const fla_tensor *g,
                                                  const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
                                                  double scale, int64_t chunk_size, const fla_tensor *out,
                                                  uint64_t *workspace_size) {
    FLA_ROUTE_F16(q, fla_chunk_fwd_o_get_workspace_size, q, k, v, h, g, cu_seqlens, chunk_indices, scale, chunk_size, out, workspace_size);
    FLA_NULL_WS("chunk_fwd_o");
    return fla::guarded([&] { return fla::fwd_o_impl(q, k, v, h, g, cu_seqlens, chunk_indices, scale, chunk_size, out, nullptr, 0, nullptr,
                           workspace_size); });
}
FLA_ENTRY(fla_chunk_fwd_o)(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *h,
                               const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
                               double scale, int64_t chunk_size, const fla_tensor *out, void *workspace,
                               uint64_t workspace_size, void *stream) {
    FLA_ROUTE_F16(q, fla_chunk_fwd_o, q, k, v, h, g, cu_seqlens, chunk_indices, scale, chunk_size, out, workspace, workspace_size, stream);
    return fla::guarded([&] { return fla::fwd_o_impl(q, k, v, h, g, cu_seqlens, chunk_indices, scale, chunk_size, out, workspace, workspace_size,
                           static_cast<hipStream_t>(stream), nullptr); });
}
