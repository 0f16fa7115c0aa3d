// causal_conv1d backward: dx, dw, db and the gradient of the initial state.
//
//   g_t  = dy_t                                   (activation 0)
//        = dy_t s(y_t) (1 + y_t (1 - s(y_t)))     (SiLU / Swish, y = pre-activation output)
//   dx_t = sum_i g_{t+i} w_{W-1-i}  (+ the final-state gradient on the last W-1 tokens)
//   dw_r = sum_t g_t xpad_{t-(W-1-r)},  db = sum_t g_t,  dh0_slot = sum_{row < slot} g_row w_{slot-1-row}
// where xpad is the sequence preceded by rows 1..W-1 of its initial state (states have W rows, row 0 unused).
// Semantics: causal_conv1d_bwd/README.md:24-52 and the golden test_npu_causal_conv1d_bwd.py:59-127,145-182.
//
// Bandwidth-bound.  One thread owns 8 adjacent channels and walks a tile of tokens with two register
// windows (the next W gradients, the last W inputs).  The four waves of a workgroup take four consecutive tiles
// of the same channels and add their partial dw / db through LDS; one workspace row per workgroup is left for a
// second kernel, which sums the rows in a fixed order, so the reductions are deterministic.  x and dx are always in
// the logical layout; y and dy may be head-split (BNSD / NTD), which only changes their row addressing.
#include "common.h"
#include "device_utils.h"

namespace fla {
namespace {

constexpr int kTileWaves = 4;              // waves of a workgroup = consecutive token tiles of the same channels
constexpr int kThreads = 64 * kTileWaves;
constexpr int kMaxW = 4;
constexpr int kTok = 32;   // tokens per tile
constexpr int kBatch = 4;  // dense path: token rows loaded ahead of their use (8 would spill at W = 4)

struct ConvBwdParams {
    const void *x, *y, *weight, *dy, *h0, *dht;
    void *dx, *dh0;
    float *partial;               // [tile groups][W+1][D]
    const int32_t *qsl;           // [N+1] or null
    int64_t x_sb, x_st;           // x and dx share the logical layout
    int64_t dx_sb, dx_st;
    int64_t g_sb, g_sh, g_st;     // y and dy: batch, head, token strides
    int64_t w_sr, s_sn, s_sp;     // weight rows; states: sequence, position
    int64_t d_sn, d_sp, o_sn, o_sp;   // dht and dh0 strides
    int B, T, D, W, N, head_dim, tiles_per_seq, tiles, activation, varlen;
};

template <typename T> __device__ __forceinline__ void ld8(const T *p, float (&f)[8]) {
    const typename Vec8<T>::type v = *reinterpret_cast<const typename Vec8<T>::type *>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
}
template <typename T> __device__ __forceinline__ void st8(T *p, const float (&f)[8]) {
    typename Vec8<T>::type v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (T)f[i];
    *reinterpret_cast<typename Vec8<T>::type *>(p) = v;
}
__device__ __forceinline__ void zero8(float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = 0.f;
}
__device__ __forceinline__ int find_seq(const int32_t *qsl, int N, int t) {   // largest n with qsl[n] <= t
    int lo = 0, hi = N - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (qsl[mid] <= t) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

// effective gradient of token row t (address already resolved by the caller)
template <typename T>
__device__ __forceinline__ void load_g(const T *dyp, const T *yp, int activation, float (&g)[8]) {
    ld8(dyp, g);
    if (activation) {
        float yy[8];
        ld8(yp, yy);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float s = __builtin_amdgcn_rcpf(1.f + __expf(-yy[i]));
            g[i] *= s * (1.f + yy[i] * (1.f - s));
        }
    }
}

template <typename T, int W>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) conv1d_bwd_kernel(const ConvBwdParams p) {
    // lane -> 8 channels, wave -> token tile; the waves' dw / db sums are added through LDS so that one row of
    // partial sums leaves the workgroup instead of one per tile
    __shared__ float red[kTileWaves][64][(kMaxW + 1) * 8 + 1];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int d0 = (blockIdx.y * 64 + lane) * 8;
    const int tile = blockIdx.x * kTileWaves + wv;
    float dw[W][8], db[8];
#pragma unroll
    for (int r = 0; r < W; ++r) zero8(dw[r]);
    zero8(db);
    if (d0 < p.D && tile < p.tiles) {
    int b, t0, t_end, n, bos, eos;
    if (p.varlen) {
        b = 0;
        t0 = tile * kTok;
        t_end = min(t0 + kTok, p.T);
        n = find_seq(p.qsl, p.N, t0);
        bos = p.qsl[n];
        eos = p.qsl[n + 1];
    } else {
        b = tile / p.tiles_per_seq;
        t0 = (tile % p.tiles_per_seq) * kTok;
        t_end = min(t0 + kTok, p.T);
        n = b;
        bos = 0;
        eos = p.T;
    }
    const T *xb = static_cast<const T *>(p.x) + b * p.x_sb + d0;
    T *dxb = static_cast<T *>(p.dx) + b * p.dx_sb + d0;
    const int hd = d0 / p.head_dim, dd = d0 % p.head_dim;
    const T *dyb = static_cast<const T *>(p.dy) + b * p.g_sb + hd * p.g_sh + dd;
    const T *yb = p.y ? static_cast<const T *>(p.y) + b * p.g_sb + hd * p.g_sh + dd : nullptr;

    float w[W][8];
#pragma unroll
    for (int r = 0; r < W; ++r) ld8(static_cast<const T *>(p.weight) + r * p.w_sr + d0, w[r]);
    float gwin[W][8];       // gwin[i] = g_{t+i} (zero past the end of the sequence)
    float xwin[W - 1][8];   // xwin[j] = xpad_{t-1-j}
    auto seed = [&](int t, int seq, int seq_bos, int seq_eos) {
#pragma unroll
        for (int i = 0; i < W - 1; ++i) {
            if (t + i < seq_eos) load_g(dyb + (int64_t)(t + i) * p.g_st, yb ? yb + (int64_t)(t + i) * p.g_st : nullptr, p.activation, gwin[i]);
            else zero8(gwin[i]);
        }
#pragma unroll
        for (int j = 0; j < W - 1; ++j) {
            const int src = t - 1 - j;
            if (src >= seq_bos) ld8(xb + (int64_t)src * p.x_st, xwin[j]);
            else if (p.h0) ld8(static_cast<const T *>(p.h0) + seq * p.s_sn + (int64_t)(W + src - seq_bos) * p.s_sp + d0, xwin[j]);
            else zero8(xwin[j]);
        }
    };
    seed(t0, n, bos, eos);
    if (!p.varlen) {
        // dense rows: kBatch tokens per batch, all their loads (look-ahead gradient rows, input rows) issued
        // before the first use; rows past the end are read from a clamped address and zeroed by a select
        typedef typename Vec8<T>::type V8;
        for (int tb = t0; tb < t_end; tb += kBatch) {
            V8 rdy[kBatch], ry[kBatch], rx[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int u = min(tb + j + W - 1, p.T - 1), t = min(tb + j, p.T - 1);
                rdy[j] = *reinterpret_cast<const V8 *>(dyb + (int64_t)u * p.g_st);
                if (yb) ry[j] = *reinterpret_cast<const V8 *>(yb + (int64_t)u * p.g_st);
                rx[j] = *reinterpret_cast<const V8 *>(xb + (int64_t)t * p.x_st);
            }
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int t = tb + j;
                if (t >= t_end) break;
                const bool live = t + W - 1 < p.T;
                float cur[8], dx[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    float g = (float)rdy[j][c];
                    if (yb) {
                        const float yy = (float)ry[j][c];
                        const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-yy));
                        g *= sg * (1.f + yy * (1.f - sg));
                    }
                    gwin[W - 1][c] = live ? g : 0.f;
                    cur[c] = (float)rx[j][c];
                }
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    float a = 0.f;
#pragma unroll
                    for (int i = 0; i < W; ++i) a = fmaf(gwin[i][c], w[W - 1 - i][c], a);
                    dx[c] = a;
                    const float g = gwin[0][c];
                    db[c] += g;
                    dw[W - 1][c] = fmaf(g, cur[c], dw[W - 1][c]);
#pragma unroll
                    for (int j2 = 0; j2 < W - 1; ++j2) dw[W - 2 - j2][c] = fmaf(g, xwin[j2][c], dw[W - 2 - j2][c]);
                }
                if (p.dht) {
                    const int tail = max(0, p.T - (W - 1));
                    if (t >= tail) {
                        float e[8];
                        ld8(static_cast<const T *>(p.dht) + n * p.d_sn + (int64_t)(1 + t - tail) * p.d_sp + d0, e);
#pragma unroll
                        for (int c = 0; c < 8; ++c) dx[c] += e[c];
                    }
                }
                st8(dxb + (int64_t)t * p.dx_st, dx);
#pragma unroll
                for (int i = 0; i + 1 < W; ++i)
#pragma unroll
                    for (int c = 0; c < 8; ++c) gwin[i][c] = gwin[i + 1][c];
#pragma unroll
                for (int j2 = W - 2; j2 > 0; --j2)
#pragma unroll
                    for (int c = 0; c < 8; ++c) xwin[j2][c] = xwin[j2 - 1][c];
#pragma unroll
                for (int c = 0; c < 8; ++c) xwin[0][c] = cur[c];
            }
        }
    } else
    for (int t = t0; t < t_end; ++t) {
        if (p.varlen && t >= eos) {   // entered the next non-empty sequence
            do {
                ++n;
                bos = p.qsl[n];
                eos = p.qsl[n + 1];
            } while (t >= eos);
            seed(t, n, bos, eos);
        }
        if (t + W - 1 < eos) load_g(dyb + (int64_t)(t + W - 1) * p.g_st, yb ? yb + (int64_t)(t + W - 1) * p.g_st : nullptr, p.activation, gwin[W - 1]);
        else zero8(gwin[W - 1]);
        float cur[8], dx[8];
        ld8(xb + (int64_t)t * p.x_st, cur);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            float a = 0.f;
#pragma unroll
            for (int i = 0; i < W; ++i) a = fmaf(gwin[i][c], w[W - 1 - i][c], a);
            dx[c] = a;
            const float g = gwin[0][c];
            db[c] += g;
            dw[W - 1][c] = fmaf(g, cur[c], dw[W - 1][c]);
#pragma unroll
            for (int j = 0; j < W - 1; ++j) dw[W - 2 - j][c] = fmaf(g, xwin[j][c], dw[W - 2 - j][c]);
        }
        if (p.dht) {   // the final state holds the last W-1 inputs: its gradient lands on them
            const int len = eos - bos, tail = max(0, len - (W - 1));
            const int rel = t - bos;
            if (rel >= tail) {
                float e[8];
                ld8(static_cast<const T *>(p.dht) + n * p.d_sn + (int64_t)(1 + rel - tail) * p.d_sp + d0, e);
#pragma unroll
                for (int c = 0; c < 8; ++c) dx[c] += e[c];
            }
        }
        st8(dxb + (int64_t)t * p.dx_st, dx);
#pragma unroll
        for (int i = 0; i + 1 < W; ++i)
#pragma unroll
            for (int c = 0; c < 8; ++c) gwin[i][c] = gwin[i + 1][c];
#pragma unroll
        for (int j = W - 2; j > 0; --j)
#pragma unroll
            for (int c = 0; c < 8; ++c) xwin[j][c] = xwin[j - 1][c];
#pragma unroll
        for (int c = 0; c < 8; ++c) xwin[0][c] = cur[c];
    }
    }
#pragma unroll
    for (int r = 0; r < W; ++r)
#pragma unroll
        for (int c = 0; c < 8; ++c) red[wv][lane][r * 8 + c] = dw[r][c];
#pragma unroll
    for (int c = 0; c < 8; ++c) red[wv][lane][W * 8 + c] = db[c];
    __syncthreads();
    // (W+1) rows of 512 channels, four channels per thread and step; the waves are added in wave order
    float *part = p.partial + (int64_t)blockIdx.x * (W + 1) * p.D + (int64_t)blockIdx.y * 512;
    for (int idx = threadIdx.x; idx < (W + 1) * 128; idx += kThreads) {
        const int r = idx >> 7, ch = (idx & 127) * 4;
        if (blockIdx.y * 512 + ch >= p.D) continue;
        const float *src = &red[0][ch >> 3][r * 8 + (ch & 7)];
        f32x4 s;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float a = src[k];
#pragma unroll
            for (int ww = 1; ww < kTileWaves; ++ww) a += src[ww * 64 * ((kMaxW + 1) * 8 + 1) + k];
            s[k] = a;
        }
        *reinterpret_cast<f32x4 *>(part + (int64_t)r * p.D + ch) = s;
    }
}

// dw[r][d] (r < W) and db[d] (r == W) from the tiles' partial sums.  A block covers 64 channels; its four
// slices each add every fourth tile (four independent chains per thread keep loads in flight) and the slices
// are then added in slice order, so the summation order is fixed.
template <typename T>
__global__ void __launch_bounds__(256) conv1d_bwd_reduce_kernel(const float *partial, int tiles, int W, int D, T *dw,
                                                                int64_t dw_sr, T *db) {
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const int d = blockIdx.x * 64 + lane;
    const int r = blockIdx.y;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (d < D) {
        const float *src = partial + (int64_t)r * D + d;
        const int64_t step = (int64_t)(W + 1) * D;
        int t = slice;
        for (; t + 12 < tiles; t += 16) {
            s0 += src[t * step];
            s1 += src[(t + 4) * step];
            s2 += src[(t + 8) * step];
            s3 += src[(t + 12) * step];
        }
        for (; t < tiles; t += 4) s0 += src[t * step];
    }
    part[slice][lane] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (slice == 0 && d < D) {
        const float s = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
        if (r < W) {
            if (dw) dw[r * dw_sr + d] = (T)s;
        } else if (db) {
            db[d] = (T)s;
        }
    }
}

// dh0[n][slot] = sum_{row < min(len, slot)} g_row w_{slot-1-row}, slot = 1..W-1; row 0 and, without an
// initial state, the whole tensor are zero.
template <typename T>
__global__ void conv1d_bwd_dh0_kernel(const ConvBwdParams p) {
    const int d0 = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    const int n = blockIdx.y;
    if (d0 >= p.D) return;
    const int W = p.W;
    int b = n, bos = 0, len = p.T;
    if (p.varlen) {
        b = 0;
        bos = p.qsl[n];
        len = p.qsl[n + 1] - bos;
    }
    T *out = static_cast<T *>(p.dh0) + n * p.o_sn + d0;
    float acc[kMaxW][8];
    for (int s = 0; s < kMaxW; ++s) zero8(acc[s]);
    if (p.h0) {
        const int hd = d0 / p.head_dim, dd = d0 % p.head_dim;
        const T *dyb = static_cast<const T *>(p.dy) + b * p.g_sb + hd * p.g_sh + dd;
        const T *yb = p.y ? static_cast<const T *>(p.y) + b * p.g_sb + hd * p.g_sh + dd : nullptr;
        for (int row = 0; row < min(len, W - 1); ++row) {
            float g[8], wt[8];
            load_g(dyb + (int64_t)(bos + row) * p.g_st, yb ? yb + (int64_t)(bos + row) * p.g_st : nullptr, p.activation, g);
            for (int slot = row + 1; slot < W; ++slot) {
                ld8(static_cast<const T *>(p.weight) + (slot - 1 - row) * p.w_sr + d0, wt);
                for (int c = 0; c < 8; ++c) acc[slot][c] = fmaf(g[c], wt[c], acc[slot][c]);
            }
        }
    }
    for (int slot = 0; slot < W; ++slot) st8(out + (int64_t)slot * p.o_sp, acc[slot]);
}

bool rows_aligned(const fla_tensor *t) {
    for (int i = 0; i + 1 < t->ndim; ++i)
        if (t->stride[i] % 8 != 0) return false;
    return reinterpret_cast<uintptr_t>(t->data) % 16 == 0;
}
inline bool present(const fla_tensor *t) { return t != nullptr && t->data != nullptr; }

int conv_bwd_impl(const fla_tensor *x, const fla_tensor *y, const fla_tensor *weight, const fla_tensor *dy,
                  const fla_tensor *initial_state, const fla_tensor *dht, const fla_int_array *query_start_loc,
                  int64_t activation, const char *input_layout, const fla_tensor *dx, const fla_tensor *dw,
                  const fla_tensor *db, const fla_tensor *dh0, void *workspace, uint64_t workspace_size, hipStream_t stream,
                  uint64_t *query) {
    const char *op = "causal_conv1d_bwd";
    const int half_mask = dt_bit(FLA_BF16) | dt_bit(FLA_F16);
    int rc;
    if ((rc = check_tensor(x, op, "x", -1, half_mask))) return rc;
    const int dt = dt_bit(x->dtype);
    if ((rc = check_tensor(weight, op, "weight", 2, dt))) return rc;
    if ((rc = check_tensor(dy, op, "dy", -1, dt))) return rc;
    if ((rc = check_tensor(dx, op, "dx", -1, dt))) return rc;
    FLA_REQUIRE(activation >= 0 && activation <= 2, FLA_ERR_SHAPE, "%s: activation must be 0, 1 or 2.", op);
    FLA_REQUIRE(input_layout != nullptr, FLA_ERR_NULL, "%s: input_layout must not be null.", op);
    const bool bsnd = !strcmp(input_layout, "BSND") || !strcmp(input_layout, "BSH");
    const bool bnsd = !strcmp(input_layout, "BNSD"), tnd = !strcmp(input_layout, "TND"), ntd = !strcmp(input_layout, "NTD");
    FLA_REQUIRE(bsnd || bnsd || tnd || ntd, FLA_ERR_UNSUPPORTED, "%s: input_layout must be BSND, BSH, BNSD, TND or NTD.", op);
    const bool packed = tnd || ntd, split = bnsd || ntd;
    FLA_REQUIRE(x->ndim == (packed ? 2 : 3) && same_shape(dx, x), FLA_ERR_SHAPE,
                "%s: x and dx must be %s for layout %s.", op, packed ? "[T,D]" : "[B,T,D]", input_layout);
    const int64_t D = x->shape[x->ndim - 1], T = x->shape[x->ndim - 2], B = packed ? 1 : x->shape[0];
    const int64_t W = weight->shape[0];
    FLA_REQUIRE(W >= 2 && W <= kMaxW && weight->shape[1] == D, FLA_ERR_SHAPE, "%s: weight must be [W,D] with W in 2..4.", op);
    FLA_REQUIRE(B * T > 0, FLA_ERR_SHAPE, "%s: empty inputs are not supported.", op);
    FLA_REQUIRE(B * T < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents exceed int32.", op);
    int64_t head_dim = D, g_sb = 0, g_sh = 0, g_st = 0;
    if (split) {
        const int o = packed ? 0 : 1;
        FLA_REQUIRE(dy->ndim == (packed ? 3 : 4) && (packed || dy->shape[0] == B) && dy->shape[o + 1] == T &&
                        dy->shape[o] * dy->shape[o + 2] == D,
                    FLA_ERR_SHAPE, "%s: dy must be [%sN,T,D/N] for layout %s.", op, packed ? "" : "B,", input_layout);
        head_dim = dy->shape[o + 2];
        g_sb = packed ? 0 : dy->stride[0];
        g_sh = dy->stride[o];
        g_st = dy->stride[o + 1];
    } else {
        FLA_REQUIRE(same_shape(dy, x), FLA_ERR_SHAPE, "%s: dy must have the shape of x for layout %s.", op, input_layout);
        g_sb = packed ? 0 : dy->stride[0];
        g_st = dy->stride[dy->ndim - 2];
    }
    FLA_REQUIRE(head_dim % 16 == 0, FLA_ERR_SHAPE, "%s: the innermost extent (%lld) must be a multiple of 16.", op, (long long)head_dim);
    if (activation != 0) {
        FLA_REQUIRE(present(y), FLA_ERR_NULL, "%s: y is required when an activation is enabled.", op);
        if ((rc = check_tensor(y, op, "y", dy->ndim, dt))) return rc;
        FLA_REQUIRE(same_shape(y, dy), FLA_ERR_SHAPE, "%s: y and dy must have the same shape.", op);
        for (int i = 0; i < dy->ndim; ++i)
            FLA_REQUIRE(y->stride[i] == dy->stride[i] || dy->shape[i] == 1, FLA_ERR_SHAPE, "%s: y and dy must have the same strides.", op);
    }
    std::vector<int32_t> qsl;
    int64_t N = B;
    if (packed) {
        FLA_REQUIRE(query_start_loc && query_start_loc->data && query_start_loc->size >= 2, FLA_ERR_METADATA,
                    "%s: query_start_loc is required for %s input.", op, input_layout);
        qsl.resize(query_start_loc->size);
        for (uint64_t i = 0; i < query_start_loc->size; ++i) qsl[i] = (int32_t)query_start_loc->data[i];
        N = (int64_t)qsl.size() - 1;
        FLA_REQUIRE(qsl[0] == 0 && qsl[N] == T, FLA_ERR_METADATA, "%s: query_start_loc must span [0, T].", op);
        for (int64_t i = 0; i < N; ++i)
            FLA_REQUIRE(qsl[i] <= qsl[i + 1], FLA_ERR_METADATA, "%s: query_start_loc must be non-decreasing.", op);
    }
    const fla_tensor *states[3] = {initial_state, dht, dh0};
    const char *snames[3] = {"initial_state", "dht", "dh0"};
    for (int i = 0; i < 3; ++i)
        if (present(states[i])) {
            if ((rc = check_tensor(states[i], op, snames[i], 3, dt))) return rc;
            FLA_REQUIRE(states[i]->shape[0] == N && states[i]->shape[1] == W && states[i]->shape[2] == D && inner_unit(states[i]) &&
                            rows_aligned(states[i]),
                        FLA_ERR_SHAPE, "%s: %s must be [N=%lld, W, D] with aligned rows.", op, snames[i], (long long)N);
        }
    if (present(dw)) {
        if ((rc = check_tensor(dw, op, "dw", 2, dt))) return rc;
        FLA_REQUIRE(same_shape(dw, weight) && inner_unit(dw), FLA_ERR_SHAPE, "%s: dw must be [W,D].", op);
    }
    if (present(db)) {
        if ((rc = check_tensor(db, op, "db", 1, dt))) return rc;
        FLA_REQUIRE(db->shape[0] == D && inner_unit(db), FLA_ERR_SHAPE, "%s: db must be [D].", op);
    }
    FLA_REQUIRE(inner_unit(x) && inner_unit(dx) && inner_unit(dy) && inner_unit(weight) && rows_aligned(x) && rows_aligned(dx) &&
                    rows_aligned(dy) && rows_aligned(weight) && (!present(y) || rows_aligned(y)),
                FLA_ERR_SHAPE, "%s: innermost strides must be 1 and rows 16-byte aligned.", op);

    const int64_t tiles_per_seq = (T + kTok - 1) / kTok;
    const int64_t tiles = packed ? tiles_per_seq : tiles_per_seq * B;
    const uint64_t meta = ((qsl.size() * 4 + 255) / 256) * 256;
    const int64_t groups = (tiles + kTileWaves - 1) / kTileWaves;
    const uint64_t need = meta + (uint64_t)groups * (W + 1) * D * 4;
    if (query) {
        *query = need;
        return FLA_OK;
    }
    FLA_REQUIRE(workspace != nullptr && workspace_size >= need, FLA_ERR_WORKSPACE, "%s: workspace of %llu bytes required.", op,
                (unsigned long long)need);
    ConvBwdParams p{};
    p.x = x->data;
    p.y = activation != 0 ? y->data : nullptr;
    p.weight = weight->data;
    p.dy = dy->data;
    p.h0 = present(initial_state) ? initial_state->data : nullptr;
    p.dht = present(dht) ? dht->data : nullptr;
    p.dx = dx->data;
    p.dh0 = present(dh0) ? dh0->data : nullptr;
    if (!qsl.empty()) {
        if ((rc = stage_to_device(workspace, qsl.data(), qsl.size() * 4, stream))) return rc;
        p.qsl = static_cast<const int32_t *>(workspace);
    }
    p.partial = reinterpret_cast<float *>(static_cast<char *>(workspace) + meta);
    p.x_sb = packed ? 0 : x->stride[0];
    p.x_st = x->stride[x->ndim - 2];
    p.dx_sb = packed ? 0 : dx->stride[0];
    p.dx_st = dx->stride[dx->ndim - 2];
    p.g_sb = g_sb;
    p.g_sh = g_sh;
    p.g_st = g_st;
    p.w_sr = weight->stride[0];
    if (p.h0) { p.s_sn = initial_state->stride[0]; p.s_sp = initial_state->stride[1]; }
    if (p.dht) { p.d_sn = dht->stride[0]; p.d_sp = dht->stride[1]; }
    if (p.dh0) { p.o_sn = dh0->stride[0]; p.o_sp = dh0->stride[1]; }
    p.B = (int)B;
    p.T = (int)T;
    p.D = (int)D;
    p.W = (int)W;
    p.N = (int)N;
    p.head_dim = (int)head_dim;
    p.tiles_per_seq = (int)tiles_per_seq;
    p.tiles = (int)tiles;
    p.activation = (int)activation;
    p.varlen = packed ? 1 : 0;
    const bool is_bf16 = x->dtype == FLA_BF16;
    const dim3 grid((unsigned)groups, (unsigned)((D / 8 + 63) / 64));
#define FLA_LAUNCH_BWD(WW)                                                                                         \
    if (is_bf16) FLA_LAUNCH("conv1d_bwd", stream, (conv1d_bwd_kernel<bf16, WW>), grid, dim3(kThreads), 0, stream, p); \
    else FLA_LAUNCH("conv1d_bwd", stream, (conv1d_bwd_kernel<f16, WW>), grid, dim3(kThreads), 0, stream, p)
    switch (W) {
        case 2: FLA_LAUNCH_BWD(2); break;
        case 3: FLA_LAUNCH_BWD(3); break;
        default: FLA_LAUNCH_BWD(4); break;
    }
#undef FLA_LAUNCH_BWD
    FLA_HIP_CHECK(hipGetLastError());
    if (present(dw) || present(db)) {
        const dim3 rgrid((unsigned)((D + 63) / 64), (unsigned)(W + 1));
        if (is_bf16)
            FLA_LAUNCH("conv1d_bwd_reduce", stream, conv1d_bwd_reduce_kernel<bf16>, rgrid, dim3(256), 0, stream, p.partial, (int)groups,
                       (int)W, (int)D, present(dw) ? static_cast<bf16 *>(dw->data) : nullptr, present(dw) ? dw->stride[0] : 0,
                       present(db) ? static_cast<bf16 *>(db->data) : nullptr);
        else
            FLA_LAUNCH("conv1d_bwd_reduce", stream, conv1d_bwd_reduce_kernel<f16>, rgrid, dim3(256), 0, stream, p.partial, (int)groups,
                       (int)W, (int)D, present(dw) ? static_cast<f16 *>(dw->data) : nullptr, present(dw) ? dw->stride[0] : 0,
                       present(db) ? static_cast<f16 *>(db->data) : nullptr);
        FLA_HIP_CHECK(hipGetLastError());
    }
    if (p.dh0) {
        const dim3 hgrid((unsigned)((D / 8 + 63) / 64), (unsigned)N);
        if (is_bf16) FLA_LAUNCH("conv1d_bwd_dh0", stream, conv1d_bwd_dh0_kernel<bf16>, hgrid, dim3(64), 0, stream, p);
        else FLA_LAUNCH("conv1d_bwd_dh0", stream, conv1d_bwd_dh0_kernel<f16>, hgrid, dim3(64), 0, stream, p);
        FLA_HIP_CHECK(hipGetLastError());
    }
    return FLA_OK;
}

}  // namespace
}  // namespace fla

extern "C" int fla_causal_conv1d_bwd_get_workspace_size(
    const fla_tensor *x, const fla_tensor *y, const fla_tensor *weight, const fla_tensor *dy, const fla_tensor *initial_state,
    const fla_tensor *dht, const fla_int_array *query_start_loc, int64_t activation, const char *input_layout,
    const fla_tensor *dx, const fla_tensor *dw, const fla_tensor *db, const fla_tensor *dh0, uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "causal_conv1d_bwd: workspace_size must not be null.");
    return fla::guarded([&] { return fla::conv_bwd_impl(x, y, weight, dy, initial_state, dht, query_start_loc, activation, input_layout, dx, dw, db, dh0,
                              nullptr, 0, nullptr, workspace_size); });
}
extern "C" int fla_causal_conv1d_bwd(
    const fla_tensor *x, const fla_tensor *y, const fla_tensor *weight, const fla_tensor *dy, const fla_tensor *initial_state,
    const fla_tensor *dht, const fla_int_array *query_start_loc, int64_t activation, const char *input_layout,
    const fla_tensor *dx, const fla_tensor *dw, const fla_tensor *db, const fla_tensor *dh0, void *workspace,
    uint64_t workspace_size, void *stream) {
    return fla::guarded([&] { return fla::conv_bwd_impl(x, y, weight, dy, initial_state, dht, query_start_loc, activation, input_layout, dx, dw, db, dh0,
                              workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}
