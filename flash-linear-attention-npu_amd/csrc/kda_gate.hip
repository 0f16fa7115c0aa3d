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
