// kda_gate_cumsum: gate activation fused with the chunk-local prefix sum of the per-channel KDA
// gate, emitted in log2 units (gk = cumsum(gate) / ln 2).
// Semantics: fla/ops/ascendc/kda/kda_gate_cumsum/op_kernel/kda_gate_cumsum_kernel.h:374-419 (activation),
// :516-534 (scale then accumulate), fla/ops/ascendc/kda/chunk_kda_fwd/docs/api.md:103-113.
//
// Bandwidth-bound: every element is read once and written once.  A thread owns four neighbouring
// channels of one chunk and walks its tokens; eight token rows are in flight per thread so the
// serial dependence of the prefix sum does not serialise the loads.
#include "gdn_common.h"
#include "kda_common.h"

namespace fla {
namespace {

struct GateParams {
    const void *g;
    float *out;
    const float *a_log;    // [Hv] or null
    const float *dt_bias;  // [Hv*K] or null
    ChunkGeom geom;        // Hv, T, K, NT, cu / tab
    int chunk;
    int use_gate;
    int safe_gate;
    float lower_bound;
    int64_t items;         // B * Hv * NT
};

template <typename TI> __device__ __forceinline__ f32x4 load4(const void *p, int64_t i);
template <> __device__ __forceinline__ f32x4 load4<float>(const void *p, int64_t i) {
    return __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(static_cast<const float *>(p) + i));
}
template <> __device__ __forceinline__ f32x4 load4<bf16>(const void *p, int64_t i) {
    const bf16x4 v = *reinterpret_cast<const bf16x4 *>(static_cast<const bf16 *>(p) + i);
    return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

template <typename TI, int TPC>  // TPC = threads per chunk = K / 4
__global__ void __launch_bounds__(256) kda_gate_cumsum_kernel(const GateParams p) {
    constexpr int CPB = 256 / TPC;  // chunks per block
    const int64_t item = (int64_t)blockIdx.x * CPB + threadIdx.x / TPC;
    if (item >= p.items) return;
    const int f = (threadIdx.x % TPC) * 4;
    const int K = p.geom.K;
    const int c = (int)(item % p.geom.NT);
    const int h = (int)((item / p.geom.NT) % p.geom.Hv);
    const int b = (int)(item / ((int64_t)p.geom.NT * p.geom.Hv));
    int start, len;
    if (p.geom.cu == nullptr) {
        start = c * p.chunk;
        len = min(p.chunk, p.geom.T - start);
    } else {
        const int seq = p.geom.tab[2 * c];
        start = p.geom.cu[seq] + p.geom.tab[2 * c + 1] * p.chunk;
        len = min(p.chunk, p.geom.cu[seq + 1] - start);
    }
    const int64_t base = (((int64_t)b * p.geom.Hv + h) * p.geom.T + start) * K + f;
    f32x4 bias = {0.f, 0.f, 0.f, 0.f};
    float eig = 0.f;
    if (p.use_gate) {
        eig = __expf(p.a_log[h]);
        if (p.dt_bias) bias = *reinterpret_cast<const f32x4 *>(p.dt_bias + (int64_t)h * K + f);
    }
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int t0 = 0; t0 < len; t0 += 8) {
        f32x4 rows[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            rows[j] = t0 + j < len ? load4<TI>(p.g, base + (int64_t)(t0 + j) * K) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (t0 + j < len) {
                f32x4 v = rows[j];
                if (p.use_gate) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = kda_activate(v[e], bias[e], eig, p.safe_gate, p.lower_bound);
                }
                acc += v * kRcpLn2;
                __builtin_nontemporal_store(acc, reinterpret_cast<f32x4 *>(p.out + base + (int64_t)(t0 + j) * K));
            }
        }
    }
}

template <typename TI>
int launch_gate(const GateParams &p, hipStream_t stream) {
    const int tpc = p.geom.K / 4;
    const auto grid = [&](int t) { return dim3((unsigned)((p.items + 256 / t - 1) / (256 / t))); };
    switch (tpc) {
        case 8: FLA_LAUNCH("kda_gate_cumsum", stream, (kda_gate_cumsum_kernel<TI, 8>), grid(8), dim3(256), 0, stream, p); break;
        case 16: FLA_LAUNCH("kda_gate_cumsum", stream, (kda_gate_cumsum_kernel<TI, 16>), grid(16), dim3(256), 0, stream, p); break;
        case 32: FLA_LAUNCH("kda_gate_cumsum", stream, (kda_gate_cumsum_kernel<TI, 32>), grid(32), dim3(256), 0, stream, p); break;
        case 64: FLA_LAUNCH("kda_gate_cumsum", stream, (kda_gate_cumsum_kernel<TI, 64>), grid(64), dim3(256), 0, stream, p); break;
        default: return fail(FLA_ERR_UNSUPPORTED, "kda_gate_cumsum: K must be 32, 64, 128 or 256, got %d.", p.geom.K);
    }
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int gate_impl(const fla_tensor *g, const fla_tensor *a_log, const fla_tensor *dt_bias, const fla_int_array *cu,
              int64_t chunk_size, bool use_gate, bool safe_gate, double lower_bound, const fla_tensor *gk, void *ws,
              uint64_t ws_size, hipStream_t stream, uint64_t *query) {
    const char *op = "kda_gate_cumsum";
    int rc;
    if ((rc = check_tensor(g, op, "g", 4, dt_bit(FLA_F32) | dt_bit(FLA_BF16)))) return rc;
    if ((rc = check_tensor(gk, op, "gk", 4, dt_bit(FLA_F32)))) return rc;
    FLA_REQUIRE(same_shape(g, gk), FLA_ERR_SHAPE, "%s: gk must have the shape of g.", op);
    FLA_REQUIRE(is_contiguous(g) && is_contiguous(gk), FLA_ERR_SHAPE, "%s: g and gk must be contiguous.", op);
    FLA_REQUIRE(reinterpret_cast<uintptr_t>(g->data) % 16 == 0 && reinterpret_cast<uintptr_t>(gk->data) % 16 == 0,
                FLA_ERR_SHAPE, "%s: g and gk must be 16-byte aligned.", op);
    FLA_REQUIRE(chunk_size == 64 || chunk_size == 128, FLA_ERR_UNSUPPORTED, "%s: chunk_size must be 64 or 128.", op);
    const int64_t B = g->shape[0], H = g->shape[1], T = g->shape[2], K = g->shape[3];
    FLA_REQUIRE(B < 65536 && H < 65536 && T < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents too large.", op);
    const bool has_a = a_log && a_log->data, has_bias = dt_bias && dt_bias->data;
    if (use_gate) {
        FLA_REQUIRE(has_a, FLA_ERR_NULL, "%s: A_log is required when use_gate_in_kernel is set.", op);
        if ((rc = check_tensor(a_log, op, "A_log", 1, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(a_log->shape[0] == H && a_log->stride[0] == 1, FLA_ERR_SHAPE, "%s: A_log must be fp32 [Hv].", op);
        if (has_bias) {
            if ((rc = check_tensor(dt_bias, op, "dt_bias", 1, dt_bit(FLA_F32)))) return rc;
            FLA_REQUIRE(dt_bias->shape[0] == H * K && dt_bias->stride[0] == 1 &&
                            reinterpret_cast<uintptr_t>(dt_bias->data) % 16 == 0,
                        FLA_ERR_SHAPE, "%s: dt_bias must be fp32 [Hv*K].", op);
        }
        FLA_REQUIRE(!safe_gate || (lower_bound >= -5.0 && lower_bound < 0.0), FLA_ERR_UNSUPPORTED,
                    "%s: lower_bound must be in [-5, 0) for the safe gate.", op);
    }
    Varlen vl;
    if ((rc = build_varlen(vl, op, cu, nullptr, chunk_size, T))) return rc;
    FLA_REQUIRE(!vl.enabled || B == 1, FLA_ERR_SHAPE, "%s: batch must be 1 with cu_seqlens.", op);
    if (query) {
        *query = vl.bytes();
        return FLA_OK;
    }
    FLA_REQUIRE(vl.bytes() == 0 || (ws && ws_size >= vl.bytes()), FLA_ERR_WORKSPACE, "%s: workspace of %zu bytes required.",
                op, vl.bytes());
    if ((rc = upload_varlen(vl, ws, stream))) return rc;

    GateParams p{};
    p.g = g->data;
    p.out = static_cast<float *>(gk->data);
    p.a_log = use_gate ? static_cast<const float *>(a_log->data) : nullptr;
    p.dt_bias = use_gate && has_bias ? static_cast<const float *>(dt_bias->data) : nullptr;
    p.geom.B = (int)B;
    p.geom.Hv = (int)H;
    p.geom.T = (int)T;
    p.geom.K = (int)K;
    p.geom.NT = vl.enabled ? vl.NT : (int)((T + chunk_size - 1) / chunk_size);
    p.geom.cu = vl.d_cu;
    p.geom.tab = vl.d_tab;
    p.chunk = (int)chunk_size;
    p.use_gate = use_gate;
    p.safe_gate = safe_gate;
    p.lower_bound = (float)lower_bound;
    p.items = B * H * p.geom.NT;
    if (p.items == 0 || K == 0) return FLA_OK;
    return g->dtype == FLA_F32 ? launch_gate<float>(p, stream) : launch_gate<bf16>(p, stream);
}


// =============================================================================================
// kda_gate_bwd: gradient of the gate activation (no counterpart among the reference's kernels; its KDA backward is a
// third-party Triton package, adapters/triton_ascend_kda.py:141-242).  With x = g + dt_bias and a = exp(A_log):
//   gate = -a softplus(x)             d gate / dx = -a sigmoid(x)          d gate / dA_log = gate
//   gate = lb sigmoid(a x)  (safe)    d gate / dx = lb s (1 - s) a         d gate / dA_log = lb s (1 - s) a x
// dg_raw = dgate * d gate / dx;  ddt_bias[h,k] = sum over tokens of dg_raw;  dA_log[h] = sum of dgate * d gate / dA_log.
// One workgroup takes kGateTile tokens of one head and writes its partial sums; the caller adds the partials.
// =============================================================================================
constexpr int kGateTile = 256;

struct GateBwdParams {
    const void *g;
    const float *dgate;
    void *dg_raw;
    const float *a_log, *dt_bias;
    float *dbias_part, *da_part;   // [B * tiles, H, K] / [B * tiles, H]
    int64_t g_sb, g_sh, g_st, d_sb, d_sh, d_st, o_sb, o_sh, o_st;
    int T, H, K, tiles;
    int safe_gate;
    float lower_bound;
};

template <typename TI> __device__ __forceinline__ void store4(void *p, int64_t i, f32x4 v);
template <> __device__ __forceinline__ void store4<float>(void *p, int64_t i, f32x4 v) {
    *reinterpret_cast<f32x4 *>(static_cast<float *>(p) + i) = v;
}
template <> __device__ __forceinline__ void store4<bf16>(void *p, int64_t i, f32x4 v) {
    *reinterpret_cast<bf16x4 *>(static_cast<bf16 *>(p) + i) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
}

template <typename TI, int TPR>  // TPR = threads per token row = K / 4
__global__ void __launch_bounds__(256) kda_gate_bwd_kernel(const GateBwdParams p) {
    constexpr int RP = 256 / TPR;   // token rows per pass
    __shared__ float redS[RP][TPR * 4 + 4];
    __shared__ float daS[4];
    const int tile = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int tid = threadIdx.x, f = (tid % TPR) * 4, rs = tid / TPR;
    const int t_end = min(p.T, (tile + 1) * kGateTile);
    const float a = __expf(p.a_log[h]);
    f32x4 bias = {0.f, 0.f, 0.f, 0.f};
    if (p.dt_bias) bias = *reinterpret_cast<const f32x4 *>(p.dt_bias + (int64_t)h * p.K + f);
    const int64_t gb = b * p.g_sb + h * p.g_sh + f, db = b * p.d_sb + h * p.d_sh + f, ob = b * p.o_sb + h * p.o_sh + f;
    f32x4 dbias = {0.f, 0.f, 0.f, 0.f};
    float da = 0.f;
    for (int t0 = tile * kGateTile + rs; t0 < t_end; t0 += 4 * RP) {
        f32x4 gv[4], dv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {   // four rows in flight per thread
            const int t = min(t0 + j * RP, t_end - 1);
            gv[j] = load4<TI>(p.g, gb + (int64_t)t * p.g_st);
            dv[j] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p.dgate + db + (int64_t)t * p.d_st));
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int t = t0 + j * RP;
            if (t >= t_end) break;
            f32x4 out;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float x = gv[j][e] + bias[e];
                float dx, dA;
                if (p.safe_gate) {
                    const float z = a * x, s = __builtin_amdgcn_rcpf(1.f + __expf(-z)), w = p.lower_bound * s * (1.f - s);
                    dx = w * a;
                    dA = w * z;
                } else {
                    const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-x));
                    dx = -a * sg;
                    dA = -a * (fmaxf(x, 0.f) + __logf(1.f + __expf(-fabsf(x))));
                }
                out[e] = dv[j][e] * dx;
                da += dv[j][e] * dA;
            }
            dbias += out;
            store4<TI>(p.dg_raw, ob + (int64_t)t * p.o_st, out);
        }
    }
    *reinterpret_cast<f32x4 *>(&redS[rs][f]) = dbias;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) da += __shfl_xor(da, off, 64);
    if ((tid & 63) == 0) daS[tid >> 6] = da;
    __syncthreads();
    const int64_t part = (int64_t)b * p.tiles + tile;
    if (tid < TPR * 4 && p.dbias_part) {
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < RP; ++r) s += redS[r][tid];
        p.dbias_part[(part * p.H + h) * p.K + tid] = s;
    }
    if (tid == 0) p.da_part[part * p.H + h] = daS[0] + daS[1] + daS[2] + daS[3];
}

template <typename TI>
int launch_gate_bwd(const GateBwdParams &p, int B, hipStream_t stream) {
    const dim3 grid(p.tiles, p.H, B);
    switch (p.K / 4) {
        case 8: FLA_LAUNCH("kda_gate_bwd", stream, (kda_gate_bwd_kernel<TI, 8>), grid, dim3(256), 0, stream, p); break;
        case 16: FLA_LAUNCH("kda_gate_bwd", stream, (kda_gate_bwd_kernel<TI, 16>), grid, dim3(256), 0, stream, p); break;
        case 32: FLA_LAUNCH("kda_gate_bwd", stream, (kda_gate_bwd_kernel<TI, 32>), grid, dim3(256), 0, stream, p); break;
        case 64: FLA_LAUNCH("kda_gate_bwd", stream, (kda_gate_bwd_kernel<TI, 64>), grid, dim3(256), 0, stream, p); break;
        default: return fail(FLA_ERR_UNSUPPORTED, "kda_gate_bwd: K must be 32, 64, 128 or 256, got %d.", p.K);
    }
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int gate_bwd_impl(const fla_tensor *g, const fla_tensor *dgate, const fla_tensor *a_log, const fla_tensor *dt_bias,
                  const char *layout, bool safe_gate, double lower_bound, const fla_tensor *dg_raw, const fla_tensor *dbias_part,
                  const fla_tensor *da_part, hipStream_t stream, uint64_t *query) {
    const char *op = "kda_gate_bwd";
    FLA_REQUIRE(layout != nullptr, FLA_ERR_NULL, "%s: layout must not be null.", op);
    int ib, ih, it;
    if (!strcmp(layout, "BSND")) { ib = 0; it = 1; ih = 2; }
    else if (!strcmp(layout, "BNSD")) { ib = 0; ih = 1; it = 2; }
    else if (!strcmp(layout, "TND")) { ib = -1; it = 0; ih = 1; }
    else if (!strcmp(layout, "NTD")) { ib = -1; ih = 0; it = 1; }
    else return fail(FLA_ERR_UNSUPPORTED, "%s: layout must be one of BSND, BNSD, TND, NTD.", op);
    const int rank = ib < 0 ? 3 : 4;
    int rc;
    if ((rc = check_tensor(g, op, "g", rank, dt_bit(FLA_F32) | dt_bit(FLA_BF16)))) return rc;
    if ((rc = check_tensor(dgate, op, "dgate", rank, dt_bit(FLA_F32)))) return rc;
    if ((rc = check_tensor(dg_raw, op, "dg_raw", rank, dt_bit(g->dtype)))) return rc;
    FLA_REQUIRE(same_shape(g, dgate) && same_shape(g, dg_raw), FLA_ERR_SHAPE, "%s: g, dgate and dg_raw must have one shape.", op);
    const int64_t B = ib < 0 ? 1 : g->shape[ib], H = g->shape[ih], T = g->shape[it], K = g->shape[rank - 1];
    FLA_REQUIRE(B < 65536 && H < 65536 && T < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents too large.", op);
    const fla_tensor *ts[] = {g, dgate, dg_raw};
    const char *tn[] = {"g", "dgate", "dg_raw"};
    for (int i = 0; i < 3; ++i) {
        const int64_t al = 16 / (int64_t)dtype_size(ts[i]->dtype);
        FLA_REQUIRE(inner_unit(ts[i]) && (ib < 0 || ts[i]->stride[ib] % al == 0) && ts[i]->stride[ih] % al == 0 &&
                        ts[i]->stride[it] % al == 0 && ts[i]->stride[it] >= 0 &&
                        reinterpret_cast<uintptr_t>(ts[i]->data) % 16 == 0,
                    FLA_ERR_SHAPE, "%s: %s needs a unit innermost stride and 16-byte aligned rows.", op, tn[i]);
    }
    if ((rc = check_tensor(a_log, op, "A_log", 1, dt_bit(FLA_F32)))) return rc;
    FLA_REQUIRE(a_log->shape[0] == H && a_log->stride[0] == 1, FLA_ERR_SHAPE, "%s: A_log must be fp32 [Hv].", op);
    const bool has_bias = dt_bias && dt_bias->data;
    if (has_bias) {
        if ((rc = check_tensor(dt_bias, op, "dt_bias", 1, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(dt_bias->shape[0] == H * K && dt_bias->stride[0] == 1 && reinterpret_cast<uintptr_t>(dt_bias->data) % 16 == 0,
                    FLA_ERR_SHAPE, "%s: dt_bias must be fp32 [Hv*K].", op);
    }
    FLA_REQUIRE(!safe_gate || (lower_bound >= -5.0 && lower_bound < 0.0), FLA_ERR_UNSUPPORTED,
                "%s: lower_bound must be in [-5, 0) for the safe gate.", op);
    const int64_t tiles = (T + kGateTile - 1) / kGateTile;
    if ((rc = check_tensor(da_part, op, "dA_log_partial", 2, dt_bit(FLA_F32)))) return rc;
    FLA_REQUIRE(da_part->shape[0] == B * tiles && da_part->shape[1] == H && is_contiguous(da_part), FLA_ERR_SHAPE,
                "%s: dA_log_partial must be contiguous fp32 [B*ceil(T/%d)=%lld, Hv].", op, kGateTile, (long long)(B * tiles));
    if (has_bias) {
        if ((rc = check_tensor(dbias_part, op, "ddt_bias_partial", 3, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(dbias_part->shape[0] == B * tiles && dbias_part->shape[1] == H && dbias_part->shape[2] == K &&
                        is_contiguous(dbias_part),
                    FLA_ERR_SHAPE, "%s: ddt_bias_partial must be contiguous fp32 [B*ceil(T/%d), Hv, K].", op, kGateTile);
    }
    if (query) {
        *query = 0;
        return FLA_OK;
    }
    if (B == 0 || H == 0 || T == 0 || K == 0) return FLA_OK;
    GateBwdParams p{};
    p.g = g->data;
    p.dgate = static_cast<const float *>(dgate->data);
    p.dg_raw = dg_raw->data;
    p.a_log = static_cast<const float *>(a_log->data);
    p.dt_bias = has_bias ? static_cast<const float *>(dt_bias->data) : nullptr;
    p.dbias_part = has_bias ? static_cast<float *>(dbias_part->data) : nullptr;
    p.da_part = static_cast<float *>(da_part->data);
    p.g_sb = ib < 0 ? 0 : g->stride[ib]; p.g_sh = g->stride[ih]; p.g_st = g->stride[it];
    p.d_sb = ib < 0 ? 0 : dgate->stride[ib]; p.d_sh = dgate->stride[ih]; p.d_st = dgate->stride[it];
    p.o_sb = ib < 0 ? 0 : dg_raw->stride[ib]; p.o_sh = dg_raw->stride[ih]; p.o_st = dg_raw->stride[it];
    p.T = (int)T; p.H = (int)H; p.K = (int)K; p.tiles = (int)tiles;
    p.safe_gate = safe_gate;
    p.lower_bound = (float)lower_bound;
    return g->dtype == FLA_F32 ? launch_gate_bwd<float>(p, (int)B, stream) : launch_gate_bwd<bf16>(p, (int)B, stream);
}

}  // namespace
}  // namespace fla

extern "C" int fla_kda_gate_cumsum_get_workspace_size(const fla_tensor *g, const fla_tensor *A_log, const fla_tensor *dt_bias,
                                                      const fla_int_array *cu_seqlens, int64_t chunk_size,
                                                      bool use_gate_in_kernel, bool safe_gate, double lower_bound,
                                                      const fla_tensor *gk, uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "kda_gate_cumsum: workspace_size must not be null.");
    return fla::guarded([&] { return fla::gate_impl(g, A_log, dt_bias, cu_seqlens, chunk_size, use_gate_in_kernel, safe_gate, lower_bound, gk, nullptr, 0,
                          nullptr, workspace_size); });
}

extern "C" int fla_kda_gate_cumsum(const fla_tensor *g, const fla_tensor *A_log, const fla_tensor *dt_bias,
                                   const fla_int_array *cu_seqlens, int64_t chunk_size, bool use_gate_in_kernel,
                                   bool safe_gate, double lower_bound, const fla_tensor *gk, void *workspace,
                                   uint64_t workspace_size, void *stream) {
    return fla::guarded([&] { return fla::gate_impl(g, A_log, dt_bias, cu_seqlens, chunk_size, use_gate_in_kernel, safe_gate, lower_bound, gk, workspace,
                          workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}

extern "C" int fla_kda_gate_bwd_get_workspace_size(const fla_tensor *g, const fla_tensor *dgate, const fla_tensor *A_log,
                                                   const fla_tensor *dt_bias, const char *layout, bool safe_gate,
                                                   double lower_bound, const fla_tensor *dg_raw, const fla_tensor *ddt_bias_partial,
                                                   const fla_tensor *dA_log_partial, uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "kda_gate_bwd: workspace_size must not be null.");
    return fla::guarded([&] { return fla::gate_bwd_impl(g, dgate, A_log, dt_bias, layout, safe_gate, lower_bound, dg_raw, ddt_bias_partial,
                          dA_log_partial, nullptr, workspace_size); });
}

extern "C" int fla_kda_gate_bwd(const fla_tensor *g, const fla_tensor *dgate, const fla_tensor *A_log, const fla_tensor *dt_bias,
                                const char *layout, bool safe_gate, double lower_bound, const fla_tensor *dg_raw,
                                const fla_tensor *ddt_bias_partial, const fla_tensor *dA_log_partial, void *workspace,
                                uint64_t workspace_size, void *stream) {
    (void)workspace;
    (void)workspace_size;
    return fla::guarded([&] { return fla::gate_bwd_impl(g, dgate, A_log, dt_bias, layout, safe_gate, lower_bound, dg_raw, ddt_bias_partial,
                          dA_log_partial, static_cast<hipStream_t>(stream), nullptr); });
}
