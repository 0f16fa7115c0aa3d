// chunk_local_cumsum (bandwidth-bound prefix sums inside each chunk) and the
// host-side operand checks shared by the chunk operators.
// Semantics: chunk_local_cumsum/README.md:7-24,73-79.
#include "gdn_common.h"

namespace fla {

int check_bhtd(const char *op, const char *name, const fla_tensor *t, int64_t B, int64_t H, int64_t T, int64_t D,
               int dtype_mask) {
    int rc = check_tensor(t, op, name, 4, dtype_mask);
    if (rc) return rc;
    FLA_REQUIRE(t->shape[0] == B && t->shape[1] == H && t->shape[2] == T && t->shape[3] == D, FLA_ERR_SHAPE,
                "%s: %s must be [%lld,%lld,%lld,%lld], got [%lld,%lld,%lld,%lld].", op, name, (long long)B,
                (long long)H, (long long)T, (long long)D, (long long)t->shape[0], (long long)t->shape[1],
                (long long)t->shape[2], (long long)t->shape[3]);
    FLA_REQUIRE(inner_unit(t), FLA_ERR_SHAPE, "%s: innermost stride of %s must be 1.", op, name);
    FLA_REQUIRE(t->stride[0] % 8 == 0 && t->stride[1] % 8 == 0 && t->stride[2] % 8 == 0 &&
                    reinterpret_cast<uintptr_t>(t->data) % 16 == 0,
                FLA_ERR_SHAPE, "%s: rows of %s must be 16-byte aligned.", op, name);
    FLA_REQUIRE(t->stride[2] >= 0 && t->stride[2] < (1 << 24), FLA_ERR_SHAPE,
                "%s: token stride of %s must be below 2^24 elements.", op, name);
    return FLA_OK;
}

int check_bht(const char *op, const char *name, const fla_tensor *t, int64_t B, int64_t H, int64_t T, int elem_dtype) {
    int rc = check_tensor(t, op, name, 3, dt_bit(FLA_F32) | dt_bit(elem_dtype));
    if (rc) return rc;
    FLA_REQUIRE(t->shape[0] == B && t->shape[1] == H && t->shape[2] == T, FLA_ERR_SHAPE,
                "%s: %s must be [%lld,%lld,%lld].", op, name, (long long)B, (long long)H, (long long)T);
    return FLA_OK;
}

int gdn_geometry(const char *op, const fla_tensor *k, const fla_tensor *v_like, const fla_tensor *g_like,
                 int64_t chunk_size, ChunkGeom &geom, int elem_dtype, int max_chunk) {
    if (max_chunk >= 128)
        FLA_REQUIRE(chunk_size == kChunk || chunk_size == 128, FLA_ERR_UNSUPPORTED,
                    "%s: chunk_size must be %d or 128, got %lld.", op, kChunk, (long long)chunk_size);
    else
        FLA_REQUIRE(chunk_size == kChunk, FLA_ERR_UNSUPPORTED, "%s: chunk_size must be %d, got %lld.", op, kChunk,
                    (long long)chunk_size);
    int rc = check_tensor(k, op, "k", 4, dt_bit(elem_dtype));
    if (rc) return rc;
    geom = ChunkGeom{};
    geom.B = (int)k->shape[0];
    geom.Hk = (int)k->shape[1];
    geom.T = (int)k->shape[2];
    geom.K = (int)k->shape[3];
    geom.Hv = geom.Hk;
    geom.V = geom.K;
    FLA_REQUIRE(k->shape[0] < (1 << 16) && k->shape[2] < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents too large.",
                op);
    if (v_like) {
        if ((rc = check_tensor(v_like, op, "v", 4, dt_bit(elem_dtype)))) return rc;
        geom.Hv = (int)v_like->shape[1];
        geom.V = (int)v_like->shape[3];
    } else if (g_like) {
        if ((rc = check_tensor(g_like, op, "g", 3, dt_bit(FLA_F32) | dt_bit(elem_dtype)))) return rc;
        geom.Hv = (int)g_like->shape[1];
    }
    FLA_REQUIRE(geom.Hk > 0 && geom.Hv % geom.Hk == 0, FLA_ERR_SHAPE, "%s: Hv (%d) must be a multiple of Hk (%d).", op,
                geom.Hv, geom.Hk);
    FLA_REQUIRE(geom.Hv < 65536, FLA_ERR_SHAPE, "%s: too many heads.", op);
    geom.C = (int)chunk_size;
    geom.NT = (geom.T + geom.C - 1) / geom.C;
    geom.N = geom.B;
    // token-major k (a token's row holds every head): chunk-parallel launches put the heads of a chunk next to each other.
    // The chunk index then sits in a grid dimension limited to 65535, hence the bound on T (varlen adds a chunk per sequence
    // at most, a kernel may pack two steps into the index).
    geom.head_fast = geom.Hk > 1 && k->stride[2] > k->stride[1] && geom.T <= (1 << 20) ? 1 : 0;
    return FLA_OK;
}

int finish_varlen(const char *op, Varlen &vl, ChunkGeom &geom, const fla_int_array *cu, const fla_int_array *ci,
                  void *workspace, uint64_t workspace_size, hipStream_t stream, uint64_t *query, int chunk) {
    if (chunk > 0) geom.C = chunk;   // operators without gdn_geometry pass their block size here
    int rc = build_varlen(vl, op, cu, ci, geom.C, geom.T);
    if (rc) return rc;
    FLA_REQUIRE(!vl.enabled || geom.B == 1, FLA_ERR_SHAPE, "%s: batch must be 1 with cu_seqlens.", op);
    if (vl.enabled) {
        geom.NT = vl.NT;
        geom.N = vl.N;
    }
    if (query) {
        *query = vl.bytes();
        return FLA_OK;
    }
    FLA_REQUIRE(vl.bytes() == 0 || (workspace && workspace_size >= vl.bytes()), FLA_ERR_WORKSPACE,
                "%s: workspace of %zu bytes required.", op, vl.bytes());
    if ((rc = upload_varlen(vl, workspace, stream))) return rc;
    geom.cu = vl.d_cu;
    geom.choff = vl.d_choff;
    geom.tab = vl.d_tab;
    return FLA_OK;
}

namespace {

template <typename T> __device__ __forceinline__ float ld(const void *p, int64_t i) {
    return (float)static_cast<const T *>(p)[i];
}
template <typename T> __device__ __forceinline__ void st(void *p, int64_t i, float v) {
    static_cast<T *>(p)[i] = (T)v;
}

struct CumsumParams {
    const void *g;
    void *out;
    ChunkGeom geom;
    int chunk;     // chunk size (power of two)
    int feat;      // trailing feature extent (1 for [B,H,T])
    int reverse;
    float scale;
    int64_t i_sb, i_sh, i_st, o_sb, o_sh, o_st;   // (batch, head, token) strides of g and out, in elements
};

// [B,H,T]: one wave per (chunk, head, batch row); lanes scan 64 tokens at a time.
template <typename TI, typename TO>
__global__ void __launch_bounds__(64) cumsum_tokens_kernel(const CumsumParams p) {
    const int b = blockIdx.z, h = blockIdx.y, c = blockIdx.x;
    int start, len;
    if (p.geom.cu == nullptr) {
        start = c * p.chunk;
        len = min(p.chunk, p.geom.T - start);
    } else {
        const int seq = p.geom.tab[2 * c];
        start = p.geom.cu[seq] + p.geom.tab[2 * c + 1] * p.chunk;
        len = min(p.chunk, p.geom.cu[seq + 1] - start);
    }
    const int64_t ibase = b * p.i_sb + h * p.i_sh + (int64_t)start * p.i_st;
    const int64_t obase = b * p.o_sb + h * p.o_sh + (int64_t)start * p.o_st;
    const int lane = threadIdx.x;
    float carry = 0.f;
    for (int off = 0; off < len; off += kWave) {
        const int j = off + lane;
        const int t = p.reverse ? len - 1 - j : j;
        float v = j < len ? ld<TI>(p.g, ibase + (int64_t)t * p.i_st) : 0.f;
        v = wave_inclusive_scan(v) + carry;
        if (j < len) st<TO>(p.out, obase + (int64_t)t * p.o_st, v * p.scale);
        carry = __shfl(v, kWave - 1, kWave);
    }
}

// [B,H,T,F]: one thread per feature column, sequential over the chunk's tokens.
template <typename TI, typename TO>
__global__ void cumsum_features_kernel(const CumsumParams p) {
    const int b = blockIdx.z, h = blockIdx.y, c = blockIdx.x;
    int start, len;
    if (p.geom.cu == nullptr) {
        start = c * p.chunk;
        len = min(p.chunk, p.geom.T - start);
    } else {
        const int seq = p.geom.tab[2 * c];
        start = p.geom.cu[seq] + p.geom.tab[2 * c + 1] * p.chunk;
        len = min(p.chunk, p.geom.cu[seq + 1] - start);
    }
    const int64_t ibase = b * p.i_sb + h * p.i_sh + (int64_t)start * p.i_st;
    const int64_t obase = b * p.o_sb + h * p.o_sh + (int64_t)start * p.o_st;
    for (int f = threadIdx.x; f < p.feat; f += blockDim.x) {
        float acc = 0.f;
        for (int j = 0; j < len; ++j) {
            const int t = p.reverse ? len - 1 - j : j;
            acc += ld<TI>(p.g, ibase + (int64_t)t * p.i_st + f);
            st<TO>(p.out, obase + (int64_t)t * p.o_st + f, acc * p.scale);
        }
    }
}

template <typename TI, typename TO>
void launch_cumsum(const CumsumParams &p, hipStream_t stream) {
    const dim3 grid(p.geom.NT, p.geom.Hv, p.geom.B);
    if (p.feat == 1) {
        FLA_LAUNCH("cumsum_tokens", stream, (cumsum_tokens_kernel<TI, TO>), grid, dim3(64), 0, stream, p);
    } else {
        const int threads = p.feat >= 256 ? 256 : ((p.feat + 63) / 64) * 64;
        FLA_LAUNCH("cumsum_features", stream, (cumsum_features_kernel<TI, TO>), grid, dim3(threads), 0, stream, p);
    }
}

int cumsum_impl(const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices_out,
                int64_t chunk_size, bool reverse, double scale, bool head_first, const char *output_dtype,
                const fla_tensor *out, void *workspace, uint64_t workspace_size, hipStream_t stream, uint64_t *query) {
    const char *op = "chunk_local_cumsum";
    const int fmask = dt_bit(FLA_F32) | dt_bit(FLA_F16) | dt_bit(FLA_BF16);
    int rc;
    if ((rc = check_tensor(g, op, "g", -1, fmask))) return rc;
    if ((rc = check_tensor(out, op, "out", -1, fmask))) return rc;
    FLA_REQUIRE(head_first, FLA_ERR_UNSUPPORTED, "%s: head_first must be true ([B,H,T] layout).", op);
    FLA_REQUIRE(g->ndim == 3 || g->ndim == 4, FLA_ERR_SHAPE, "%s: g must be [B,H,T] or [B,H,T,K].", op);
    FLA_REQUIRE(same_shape(g, out), FLA_ERR_SHAPE, "%s: out must have the shape of g.", op);
    // [B,H,T] and [B,H,T,K] are index orders: any strides are taken (a [B,T,H,..] tensor is passed as its transposed
    // view); only the feature dimension of a rank-4 operand must be dense
    FLA_REQUIRE(g->ndim == 3 || (inner_unit(g) && inner_unit(out)), FLA_ERR_SHAPE,
                "%s: the innermost stride of a rank-4 g / out must be 1.", op);
    FLA_REQUIRE(chunk_size > 0 && (chunk_size & (chunk_size - 1)) == 0, FLA_ERR_SHAPE,
                "%s: chunk_size must be a power of 2, got %lld.", op, (long long)chunk_size);
    if (output_dtype != nullptr) {
        int want = -1;
        if (!strcmp(output_dtype, "float32")) want = FLA_F32;
        else if (!strcmp(output_dtype, "float16")) want = FLA_F16;
        else if (!strcmp(output_dtype, "bfloat16")) want = FLA_BF16;
        else if (!strcmp(output_dtype, "same") || !strcmp(output_dtype, "input") || !strcmp(output_dtype, "none")) want = g->dtype;
        FLA_REQUIRE(want >= 0, FLA_ERR_DTYPE, "%s: unsupported output_dtype '%s'.", op, output_dtype);
        FLA_REQUIRE(want == out->dtype, FLA_ERR_DTYPE, "%s: out dtype does not match output_dtype '%s'.", op, output_dtype);
    }
    const int64_t B = g->shape[0], H = g->shape[1], T = g->shape[2];
    const int64_t F = g->ndim == 4 ? g->shape[3] : 1;
    FLA_REQUIRE(B < 65536 && H < 65536 && T < ((int64_t)1 << 31) && F < ((int64_t)1 << 31), FLA_ERR_SHAPE,
                "%s: extents too large.", op);
    Varlen vl;
    // chunk_indices_out may be built for a different block size than chunk_size
    // (examples/flash_gated_delta_rule.py:473-478), so only cu_seqlens is consumed.
    (void)chunk_indices_out;
    if ((rc = build_varlen(vl, op, cu_seqlens, nullptr, chunk_size, T))) return rc;
    FLA_REQUIRE(!vl.enabled || B == 1, FLA_ERR_SHAPE, "%s: batch must be 1 with cu_seqlens.", op);
    if (query) {
        *query = vl.bytes();
        return FLA_OK;
    }
    FLA_REQUIRE(vl.bytes() == 0 || (workspace && workspace_size >= vl.bytes()), FLA_ERR_WORKSPACE,
                "%s: workspace of %zu bytes required.", op, vl.bytes());
    if ((rc = upload_varlen(vl, workspace, stream))) return rc;

    CumsumParams p{};
    p.g = g->data;
    p.out = out->data;
    p.geom.B = (int)B;
    p.geom.Hv = (int)H;
    p.geom.T = (int)T;
    p.geom.NT = vl.enabled ? vl.NT : (int)((T + chunk_size - 1) / chunk_size);
    p.geom.cu = vl.d_cu;
    p.geom.tab = vl.d_tab;
    p.chunk = (int)chunk_size;
    p.feat = (int)F;
    p.reverse = reverse ? 1 : 0;
    p.scale = (float)scale;
    p.i_sb = g->stride[0]; p.i_sh = g->stride[1]; p.i_st = g->stride[2];
    p.o_sb = out->stride[0]; p.o_sh = out->stride[1]; p.o_st = out->stride[2];
    if (p.geom.NT == 0 || B == 0 || H == 0) return FLA_OK;

#define FLA_CS(TI, TO) launch_cumsum<TI, TO>(p, stream)
#define FLA_CS_OUT(TI)                                   \
    switch (out->dtype) {                                \
        case FLA_F32: FLA_CS(TI, float); break;          \
        case FLA_F16: FLA_CS(TI, f16); break;            \
        default: FLA_CS(TI, bf16); break;                \
    }
    switch (g->dtype) {
        case FLA_F32: FLA_CS_OUT(float); break;
        case FLA_F16: FLA_CS_OUT(f16); break;
        default: FLA_CS_OUT(bf16); break;
    }
#undef FLA_CS_OUT
#undef FLA_CS
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

}  // namespace
}  // namespace fla

extern "C" int fla_chunk_local_cumsum_get_workspace_size(const fla_tensor *g, const fla_int_array *cu_seqlens,
                                                         const fla_int_array *chunk_indices_out, int64_t chunk_size,
                                                         bool reverse, double scale, bool head_first,
                                                         const char *output_dtype, const fla_tensor *out,
                                                         uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "chunk_local_cumsum: workspace_size must not be null.");
    return fla::guarded([&] { return fla::cumsum_impl(g, cu_seqlens, chunk_indices_out, chunk_size, reverse, scale, head_first, output_dtype, out,
                            nullptr, 0, nullptr, workspace_size); });
}

extern "C" int fla_chunk_local_cumsum(const fla_tensor *g, const fla_int_array *cu_seqlens,
                                      const fla_int_array *chunk_indices_out, int64_t chunk_size, bool reverse,
                                      double scale, bool head_first, const char *output_dtype, const fla_tensor *out,
                                      void *workspace, uint64_t workspace_size, void *stream) {
    return fla::guarded([&] { return fla::cumsum_impl(g, cu_seqlens, chunk_indices_out, chunk_size, reverse, scale, head_first, output_dtype, out,
                            workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}
