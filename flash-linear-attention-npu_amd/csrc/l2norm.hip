// l2norm_fwd / l2norm_bwd over the last dimension (the q/k normalisation of the chunk pipelines):
//   y = x rstd,  rstd = 1 / sqrt(sum x^2 + eps)            (fla/ops/triton/triton_core/l2norm.py:16-30,131-178)
//   dx = (dy - sum(dy y) y) rstd                            (l2norm.py:93-128,181-224)
// Bandwidth-bound row operations: a row of D = 64 / 128 / 256 elements is held by D/8 adjacent lanes (one 16-byte
// piece each) and reduced with data-parallel-primitive adds; rows are addressed through the outer strides of a
// rank <= 4 tensor, so head-first and token-first views need no copy.
#include "common.h"
#include "device_utils.h"

namespace fla {
namespace {

struct L2Params {
    const void *x, *dy;     // fwd: x; bwd: x = y (normalised), dy
    void *y;                // fwd: y; bwd: dx
    float *rstd;            // fwd out / bwd in, contiguous [rows]
    int64_t x_s[3], y_s[3], d_s[3];   // strides of the three outer dims (elements)
    int n1, n2;             // extents of outer dims 1 and 2 (dim 0 is rows / (n1 n2))
    int64_t rows;
    float eps;
};

template <typename T, int D, bool BWD>
__global__ void __launch_bounds__(256) l2norm_kernel(const L2Params p) {
    constexpr int LPR = D / 8;                 // lanes per row
    typedef typename Vec8<T>::type V8;
    const int64_t row = (int64_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
    const int c = (threadIdx.x % LPR) * 8;
    const int64_t r = min(row, p.rows - 1);    // clamped: every lane takes part in the reduction
    const int i2 = (int)(r % p.n2), i1 = (int)((r / p.n2) % p.n1);
    const int64_t i0 = r / ((int64_t)p.n1 * p.n2);
    const V8 xv = *reinterpret_cast<const V8 *>(static_cast<const T *>(p.x) + i0 * p.x_s[0] + i1 * p.x_s[1] + i2 * p.x_s[2] + c);
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = (float)xv[e];
    V8 out;
    if (!BWD) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
        ss = group_sum<LPR>(ss);
        const float rstd = 1.f / sqrtf(ss + p.eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (T)(f[e] * rstd);
        if (row < p.rows && c == 0 && p.rstd) p.rstd[row] = rstd;
    } else {
        const V8 dv = *reinterpret_cast<const V8 *>(static_cast<const T *>(p.dy) + i0 * p.d_s[0] + i1 * p.d_s[1] + i2 * p.d_s[2] + c);
        float d[8], dot = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            d[e] = (float)dv[e];
            dot += d[e] * f[e];
        }
        dot = group_sum<LPR>(dot);
        const float rstd = p.rstd[r];
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (T)((d[e] - dot * f[e]) * rstd);
    }
    if (row < p.rows)
        *reinterpret_cast<V8 *>(static_cast<T *>(p.y) + i0 * p.y_s[0] + i1 * p.y_s[1] + i2 * p.y_s[2] + c) = out;
}

inline bool present(const fla_tensor *t) { return t != nullptr && t->data != nullptr; }

// outer strides of a rank 1..4 tensor padded to three outer dims
int outer(const char *op, const char *name, const fla_tensor *t, const fla_tensor *like, int64_t (&s)[3], int &n1, int &n2,
          int64_t &rows) {
    FLA_REQUIRE(t->ndim >= 2 && t->ndim <= 4 && inner_unit(t), FLA_ERR_SHAPE, "%s: %s must have rank 2..4 and unit innermost stride.", op, name);
    FLA_REQUIRE(like == nullptr || same_shape(t, like), FLA_ERR_SHAPE, "%s: %s shape mismatch.", op, name);
    int64_t ext[3] = {1, 1, 1};
    s[0] = s[1] = s[2] = 0;
    const int no = t->ndim - 1;
    for (int i = 0; i < no; ++i) {
        ext[3 - no + i] = t->shape[i];
        s[3 - no + i] = t->stride[i];
        FLA_REQUIRE(t->stride[i] % 8 == 0, FLA_ERR_SHAPE, "%s: rows of %s must be 16-byte aligned.", op, name);
    }
    FLA_REQUIRE(reinterpret_cast<uintptr_t>(t->data) % 16 == 0, FLA_ERR_SHAPE, "%s: %s must be 16-byte aligned.", op, name);
    n1 = (int)ext[1];
    n2 = (int)ext[2];
    rows = ext[0] * ext[1] * ext[2];
    return FLA_OK;
}

template <bool BWD>
int l2_impl(const char *op, const fla_tensor *x, const fla_tensor *dy, const fla_tensor *rstd, double eps, const fla_tensor *y,
            hipStream_t stream, uint64_t *query) {
    const int half = dt_bit(FLA_BF16) | dt_bit(FLA_F16);
    int rc;
    if ((rc = check_tensor(x, op, BWD ? "y" : "x", -1, half))) return rc;
    if ((rc = check_tensor(y, op, BWD ? "dx" : "y", -1, dt_bit(x->dtype)))) return rc;
    L2Params p{};
    int n1, n2;
    int64_t rows;
    if ((rc = outer(op, "input", x, nullptr, p.x_s, n1, n2, rows))) return rc;
    int a, b;
    int64_t r2;
    if ((rc = outer(op, "output", y, x, p.y_s, a, b, r2))) return rc;
    if (BWD) {
        if ((rc = check_tensor(dy, op, "dy", -1, dt_bit(x->dtype)))) return rc;
        if ((rc = outer(op, "dy", dy, x, p.d_s, a, b, r2))) return rc;
    }
    const int64_t D = x->shape[x->ndim - 1];
    FLA_REQUIRE(D == 64 || D == 128 || D == 256, FLA_ERR_UNSUPPORTED, "%s: the normalised dimension must be 64, 128 or 256, got %lld.", op, (long long)D);
    if (BWD || present(rstd)) {
        if ((rc = check_tensor(rstd, op, "rstd", -1, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(numel(rstd) == rows && is_contiguous(rstd), FLA_ERR_SHAPE, "%s: rstd must be a contiguous fp32 tensor with one value per row.", op);
    }
    if (query) {
        *query = 0;
        return FLA_OK;
    }
    if (rows == 0) return FLA_OK;
    p.x = x->data;
    p.dy = BWD ? dy->data : nullptr;
    p.y = y->data;
    p.rstd = present(rstd) ? static_cast<float *>(rstd->data) : nullptr;
    p.n1 = n1;
    p.n2 = n2;
    p.rows = rows;
    p.eps = (float)eps;
    const bool is_bf16 = x->dtype == FLA_BF16;
    const char *name = BWD ? "l2norm_bwd" : "l2norm_fwd";
#define FLA_L2(DD)                                                                                                  \
    do {                                                                                                            \
        const dim3 grid((unsigned)((rows + 256 / (DD / 8) - 1) / (256 / (DD / 8))));                                \
        if (is_bf16) FLA_LAUNCH(name, stream, (l2norm_kernel<bf16, DD, BWD>), grid, dim3(256), 0, stream, p);      \
        else FLA_LAUNCH(name, stream, (l2norm_kernel<f16, DD, BWD>), grid, dim3(256), 0, stream, p);               \
    } while (0)
    if (D == 64) FLA_L2(64);
    else if (D == 128) FLA_L2(128);
    else FLA_L2(256);
#undef FLA_L2
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

}  // namespace
}  // namespace fla

extern "C" int fla_l2norm_fwd_get_workspace_size(const fla_tensor *x, double eps, const fla_tensor *y, const fla_tensor *rstd,
                                                 uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "l2norm_fwd: workspace_size must not be null.");
    return fla::guarded([&] { return fla::l2_impl<false>("l2norm_fwd", x, nullptr, rstd, eps, y, nullptr, workspace_size); });
}
extern "C" int fla_l2norm_fwd(const fla_tensor *x, double eps, const fla_tensor *y, const fla_tensor *rstd, void *workspace,
                              uint64_t workspace_size, void *stream) {
    (void)workspace;
    (void)workspace_size;
    return fla::guarded([&] { return fla::l2_impl<false>("l2norm_fwd", x, nullptr, rstd, eps, y, static_cast<hipStream_t>(stream), nullptr); });
}
extern "C" int fla_l2norm_bwd_get_workspace_size(const fla_tensor *y, const fla_tensor *rstd, const fla_tensor *dy, double eps,
                                                 const fla_tensor *dx, uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "l2norm_bwd: workspace_size must not be null.");
    return fla::guarded([&] { return fla::l2_impl<true>("l2norm_bwd", y, dy, rstd, eps, dx, nullptr, workspace_size); });
}
extern "C" int fla_l2norm_bwd(const fla_tensor *y, const fla_tensor *rstd, const fla_tensor *dy, double eps, const fla_tensor *dx,
                              void *workspace, uint64_t workspace_size, void *stream) {
    (void)workspace;
    (void)workspace_size;
    return fla::guarded([&] { return fla::l2_impl<true>("l2norm_bwd", y, dy, rstd, eps, dx, static_cast<hipStream_t>(stream), nullptr); });
}
