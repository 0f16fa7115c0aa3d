// causal_conv1d prefill (depthwise causal convolution, width 2..4, optional bias,
// optional SiLU, optional initial state, final-state write-back).
//
// Bandwidth-bound: each element of x is read once (plus a W-1 row halo per
// token tile) and each element of y written once.  One thread owns 8 adjacent
// channels (one 16-byte access) and walks TOK_PER_THREAD consecutive tokens with
// the last W-1 inputs held in registers, so a wave reads and writes 1 KiB
// contiguous per token row.  Semantics: causal_conv1d/README.md:15-31 and
// op_kernel/causal_conv1d.h:424-498 (tap loop), :753-776 (state write-back).
#include "common.h"
#include "device_utils.h"

namespace fla {
namespace {

constexpr int kThreads = 128;
constexpr int kMaxW = 4;

struct ConvParams {
    const void *x;
    const void *weight;
    const void *bias;
    void *conv_states;
    void *out;
    const int32_t *qsl;    // [N+1] device, varlen only
    const int32_t *cache;  // [N] device or null
    const int32_t *init;   // [N] device or null
    int64_t x_sb, x_ss;            // batch / token strides of x (elements)
    int64_t o_sb, o_sh, o_ss;      // out strides: batch, head, token
    int64_t w_sr;                  // weight row stride
    int64_t cs_sn, cs_sp;          // conv_states strides: slot, position
    int B, S, D, W, N;
    int head_dim;                  // D / head_num, or D when no head split
    int tiles_per_seq;             // dense only
    int tok;                       // tokens per thread (tile height)
    int activation;
    int pad_slot;
    int varlen;
};

template <typename T> __device__ __forceinline__ void load8(const T *p, float (&f)[8]) {
    typename Vec8<T>::type v = *reinterpret_cast<const typename Vec8<T>::type *>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
}
template <typename T> __device__ __forceinline__ void load8_cached(const T *p, float (&f)[8]) {
    typename Vec8<T>::type v = *reinterpret_cast<const typename Vec8<T>::type *>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
}
template <typename T> __device__ __forceinline__ void store8(T *p, const float (&f)[8]) {
    typename Vec8<T>::type v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (T)f[i];
    *reinterpret_cast<typename Vec8<T>::type *>(p) = v;
}

__device__ __forceinline__ int find_seq(const int32_t *qsl, int N, int t) {
    // largest n with qsl[n] <= t, skipping empty sequences implicitly
    int lo = 0, hi = N - 1;
    while (lo < hi) {
        int mid = (lo + hi + 1) >> 1;
        if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
    }
    return lo;
}

template <typename T, int W, int kTok>
__global__ void __launch_bounds__(kThreads) conv1d_fwd_kernel(const ConvParams p) {
    const int d0 = (blockIdx.y * kThreads + threadIdx.x) * 8;
    if (d0 >= p.D) return;
    const T *x = static_cast<const T *>(p.x);
    T *out = static_cast<T *>(p.out);

    float w[W][8], bias[8];
#pragma unroll
    for (int r = 0; r < W; ++r) load8_cached(static_cast<const T *>(p.weight) + r * p.w_sr + d0, w[r]);
    if (p.bias) {
        load8_cached(static_cast<const T *>(p.bias) + d0, bias);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) bias[i] = 0.f;
    }

    // token range of this tile and the sequence it starts in
    int b, t0, t_end, n, bos, eos;
    if (p.varlen) {
        b = 0;
        t0 = blockIdx.x * kTok;
        t_end = min(t0 + kTok, p.S);
        n = find_seq(p.qsl, p.N, t0);
        bos = p.qsl[n];
        eos = p.qsl[n + 1];
    } else {
        b = blockIdx.x / p.tiles_per_seq;
        t0 = (blockIdx.x % p.tiles_per_seq) * kTok;
        t_end = min(t0 + kTok, p.S);
        n = b;
        bos = 0;
        eos = p.S;
    }
    const T *xb = x + b * p.x_sb + d0;
    const int hd = d0 / p.head_dim, dd = d0 % p.head_dim;
    T *ob = out + b * p.o_sb + hd * p.o_sh + dd;
    const T *cs = static_cast<const T *>(p.conv_states);

    float win[W - 1][8];  // win[r] = input row (t - (W-1) + r)
    auto seed_window = [&](int t, int seq, int seq_bos) {
        const int slot = p.cache ? p.cache[seq] : seq;
        const bool use_init = cs != nullptr && p.init != nullptr && p.init[seq] == 1 && slot != p.pad_slot;
#pragma unroll
        for (int r = 0; r < W - 1; ++r) {
            const int tt = t - (W - 1) + r;
            if (tt >= seq_bos) {
                load8_cached(xb + (int64_t)tt * p.x_ss, win[r]);
            } else if (use_init) {
                // row (W-1) + (tt - seq_bos) of the saved state (negative offset from its end)
                load8_cached(cs + slot * p.cs_sn + (int64_t)(W - 1 + tt - seq_bos) * p.cs_sp + d0, win[r]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) win[r][i] = 0.f;
            }
        }
    };
    seed_window(t0, n, bos);
    bool skip = p.varlen && p.cache && p.cache[n] == p.pad_slot;

    for (int tb = t0; tb < t_end; tb += 8) {
        float cur[8][8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (tb + j < t_end) load8(xb + (int64_t)(tb + j) * p.x_ss, cur[j]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int t = tb + j;
            if (t >= t_end) break;
            if (p.varlen && t >= eos) {  // entered the next non-empty sequence
                do {
                    ++n;
                    bos = p.qsl[n];
                    eos = p.qsl[n + 1];
                } while (t >= eos);
                seed_window(t, n, bos);
                skip = p.cache && p.cache[n] == p.pad_slot;
            }
            float acc[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float a = bias[i];
#pragma unroll
                for (int r = 0; r < W - 1; ++r) a = fmaf(w[r][i], win[r][i], a);
                a = fmaf(w[W - 1][i], cur[j][i], a);
                if (p.activation == 1) a = a * __builtin_amdgcn_rcpf(1.f + __expf(-a));  // SiLU; the 1-ulp hardware reciprocal is ample for a 16-bit result
                acc[i] = a;
            }
#pragma unroll
            for (int r = 0; r + 1 < W - 1; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) win[r][i] = win[r + 1][i];
#pragma unroll
            for (int i = 0; i < 8; ++i) win[W - 2][i] = cur[j][i];
            if (!skip) store8(ob + (int64_t)t * p.o_ss, acc);
        }
    }
}

// Dense fast path: no packed sequences, no cache indirection, no initial states.  The tile
// loop is fully unrolled so the W-1 row window rotates through register renaming and the only
// per-row scalar work is one pointer increment; rows past the end of a sequence are loaded
// from a clamped address and never stored.
template <typename T, int W, int TOK, bool ACT>
__global__ void __launch_bounds__(kThreads) conv1d_dense_kernel(const ConvParams p) {
    typedef typename Vec8<T>::type V8;
    const int d0 = (blockIdx.y * kThreads + threadIdx.x) * 8;
    if (d0 >= p.D) return;
    // Workgroup ids go round the eight XCDs; give each XCD a contiguous run of row tiles so that
    // the W-1 halo rows a tile re-reads were fetched into the same L2 by its predecessor.
    int tile = blockIdx.x;
    if ((gridDim.x & 7) == 0) tile = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int b = tile / p.tiles_per_seq;
    const int t0 = (tile % p.tiles_per_seq) * TOK;
    const int nvalid = min(TOK, p.S - t0);
    const T *xp = static_cast<const T *>(p.x) + b * p.x_sb + (int64_t)t0 * p.x_ss + d0;
    const int hd = d0 / p.head_dim, dd = d0 % p.head_dim;
    T *op = static_cast<T *>(p.out) + b * p.o_sb + hd * p.o_sh + (int64_t)t0 * p.o_ss + dd;

    float w[W][8], bias[8];
#pragma unroll
    for (int r = 0; r < W; ++r) load8_cached(static_cast<const T *>(p.weight) + r * p.w_sr + d0, w[r]);
    if (p.bias) {
        load8_cached(static_cast<const T *>(p.bias) + d0, bias);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) bias[i] = 0.f;
    }
    float win[W - 1][8];
#pragma unroll
    for (int r = 0; r < W - 1; ++r) {
        if (t0 - (W - 1) + r >= 0) {
            load8_cached(xp - (int64_t)(W - 1 - r) * p.x_ss, win[r]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) win[r][i] = 0.f;
        }
    }
#pragma unroll
    for (int j0 = 0; j0 < TOK; j0 += 8) {
        V8 raw[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) raw[j] = *reinterpret_cast<const V8 *>(xp + (int64_t)min(j0 + j, nvalid - 1) * p.x_ss);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float cur[8];
            V8 o;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                cur[i] = (float)raw[j][i];
                float a = bias[i];
#pragma unroll
                for (int r = 0; r < W - 1; ++r) a = fmaf(w[r][i], win[r][i], a);
                a = fmaf(w[W - 1][i], cur[i], a);
                if (ACT) a = a * __builtin_amdgcn_rcpf(1.f + __expf(-a));  // SiLU; the 1-ulp hardware reciprocal is ample for a 16-bit result
                o[i] = (T)a;
            }
#pragma unroll
            for (int r = 0; r + 1 < W - 1; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) win[r][i] = win[r + 1][i];
#pragma unroll
            for (int i = 0; i < 8; ++i) win[W - 2][i] = cur[i];
            if (j0 + j < nvalid) __builtin_nontemporal_store(o, reinterpret_cast<V8 *>(op + (int64_t)(j0 + j) * p.o_ss));
        }
    }
}

// Final-state write-back, one thread per (sequence, 8 channels): conv_states[slot, pos]
// = row (len + pos) of [head rows | x rows], pos = 0..W-2.  Runs after the main
// kernel on the same stream, so initial states have already been consumed.
template <typename T>
__global__ void conv1d_state_kernel(const ConvParams p) {
    const int d0 = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    const int n = blockIdx.y;
    if (d0 >= p.D) return;
    const int W = p.W;
    const int slot = p.cache ? p.cache[n] : n;
    if (slot == p.pad_slot) return;
    int b = 0, bos = 0, len = p.S;
    if (p.varlen) {
        bos = p.qsl[n];
        len = p.qsl[n + 1] - bos;
    } else {
        b = n;
    }
    T *cs = static_cast<T *>(p.conv_states) + slot * p.cs_sn + d0;
    const T *xb = static_cast<const T *>(p.x) + b * p.x_sb + d0;
    const bool use_init = p.init != nullptr && p.init[n] == 1;
    float rows[kMaxW - 1][8];
    for (int pos = 0; pos < W - 1; ++pos) {
        const int j = len + pos - (W - 1);  // index into x rows of this sequence
        if (j >= 0) {
            load8_cached(xb + (int64_t)(bos + j) * p.x_ss, rows[pos]);
        } else if (use_init) {
            load8_cached(cs + (int64_t)(len + pos) * p.cs_sp, rows[pos]);
        } else {
            for (int i = 0; i < 8; ++i) rows[pos][i] = 0.f;
        }
    }
    for (int pos = 0; pos < W - 1; ++pos) {
        typename Vec8<T>::type v;
        for (int i = 0; i < 8; ++i) v[i] = (T)rows[pos][i];
        *reinterpret_cast<typename Vec8<T>::type *>(cs + (int64_t)pos * p.cs_sp) = v;
    }
}

// State-update mode (run_mode = 1), one thread per (sequence, 8 channels): the W-1 history rows come from
// conv_states[slot] (rows offset .. offset+W-2; offset = accepted-1 under speculative decoding, else 0), the
// S new tokens are convolved in order, and the state is rewritten: the plain form keeps the last W-1 rows of
// [history | x] in rows 0..W-2; the speculative form (width 4) keeps old rows offset+1..offset+W-2 in rows
// 0..W-3 and appends all S new tokens, so that the next call can pick its history by its own accepted count.
// Semantics: op_kernel/causal_conv1d.h:753-860,955-1025; goldens test_npu_causal_conv1d.py:56-151.
struct ConvUpdateParams {
    const void *x;
    const void *weight;
    const void *bias;
    void *conv_states;
    void *out;
    const int32_t *qsl;    // [N+1] or null
    const int32_t *cache;  // [N] or null
    const int32_t *nat;    // [N] or null (speculative decoding)
    int64_t x_sb, x_ss, o_sb, o_ss, w_sr, cs_sn, cs_sp;
    int S, D, W, N, state_len, activation, pad_slot;
};

template <typename T>
__global__ void conv1d_update_kernel(const ConvUpdateParams p) {
    typedef typename Vec8<T>::type V8;
    const int d0 = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    const int n = blockIdx.y;
    if (d0 >= p.D) return;
    const int slot = p.cache ? p.cache[n] : n;
    if (slot == p.pad_slot) return;
    int64_t xoff, ooff;
    int len = p.S;
    if (p.qsl) {
        const int bos = p.qsl[n];
        len = p.qsl[n + 1] - bos;
        xoff = (int64_t)bos * p.x_ss;
        ooff = (int64_t)bos * p.o_ss;
    } else {
        xoff = n * p.x_sb;
        ooff = n * p.o_sb;
    }
    if (len <= 0) return;
    const int W = p.W, keep = W - 2;
    const bool spec = p.nat != nullptr && W == 4;
    int offset = 0;
    if (spec) offset = min(max(p.nat[n] - 1, 0), p.state_len - (W - 1));
    T *cs = static_cast<T *>(p.conv_states) + slot * p.cs_sn + d0;
    const T *xb = static_cast<const T *>(p.x) + xoff + d0;
    T *ob = static_cast<T *>(p.out) + ooff + d0;
    float win[kMaxW - 1][8], wt[kMaxW][8], bias[8];
#pragma unroll
    for (int i = 0; i < kMaxW - 1; ++i)
        if (i < W - 1) load8_cached(cs + (int64_t)(offset + i) * p.cs_sp, win[i]);
#pragma unroll
    for (int r = 0; r < kMaxW; ++r)
        if (r < W) load8_cached(static_cast<const T *>(p.weight) + r * p.w_sr + d0, wt[r]);
    if (p.bias) load8_cached(static_cast<const T *>(p.bias) + d0, bias);
    else
        for (int i = 0; i < 8; ++i) bias[i] = 0.f;
    const bool spec_write = spec && keep + len <= p.state_len;
    if (spec_write) {   // rows offset+1 .. offset+keep of the old state move to the front
#pragma unroll
        for (int i = 0; i < kMaxW - 2; ++i)
            if (i < keep) {
                V8 v;
                for (int c = 0; c < 8; ++c) v[c] = (T)win[i + 1][c];
                *reinterpret_cast<V8 *>(cs + (int64_t)i * p.cs_sp) = v;
            }
    }
    for (int t = 0; t < len; ++t) {
        const V8 raw = *reinterpret_cast<const V8 *>(xb + (int64_t)t * p.x_ss);
        float cur[8], acc[8];
        for (int c = 0; c < 8; ++c) cur[c] = (float)raw[c];
        for (int c = 0; c < 8; ++c) acc[c] = bias[c] + wt[W - 1][c] * cur[c];
#pragma unroll
        for (int i = 0; i < kMaxW - 1; ++i)
            if (i < W - 1)
                for (int c = 0; c < 8; ++c) acc[c] += wt[i][c] * win[i][c];
        if (p.activation)
            for (int c = 0; c < 8; ++c) acc[c] = acc[c] * __builtin_amdgcn_rcpf(1.f + __expf(-acc[c]));
        V8 o;
        for (int c = 0; c < 8; ++c) o[c] = (T)acc[c];
        *reinterpret_cast<V8 *>(ob + (int64_t)t * p.o_ss) = o;
        if (spec_write) *reinterpret_cast<V8 *>(cs + (int64_t)(keep + t) * p.cs_sp) = raw;
#pragma unroll
        for (int i = 0; i < kMaxW - 2; ++i)
            if (i < W - 2)
                for (int c = 0; c < 8; ++c) win[i][c] = win[i + 1][c];
        for (int c = 0; c < 8; ++c) win[W - 2][c] = cur[c];
    }
    if (!spec_write) {
#pragma unroll
        for (int i = 0; i < kMaxW - 1; ++i)
            if (i < W - 1) {
                V8 v;
                for (int c = 0; c < 8; ++c) v[c] = (T)win[i][c];
                *reinterpret_cast<V8 *>(cs + (int64_t)i * p.cs_sp) = v;
            }
    }
}

// The kernels move 16-byte pieces: every row must start on a 16-byte boundary.
bool aligned(const fla_tensor *t) {
    for (int i = 0; i + 1 < t->ndim; ++i)
        if (t->stride[i] % 8 != 0) return false;
    return reinterpret_cast<uintptr_t>(t->data) % 16 == 0;
}

int copy_int_array(std::vector<int32_t> &dst, const fla_int_array *a) {
    dst.clear();
    if (a == nullptr || a->data == nullptr) return 0;
    dst.resize(a->size);
    for (uint64_t i = 0; i < a->size; ++i) dst[i] = (int32_t)a->data[i];
    return (int)a->size;
}

// run_mode = 1: x [B,S,D], [B,D] (one token per sequence) or packed [T,D] with query_start_loc.
int conv_update_impl(const fla_tensor *x, const fla_tensor *weight, const fla_tensor *bias, const fla_tensor *conv_states,
                     const fla_int_array *query_start_loc, const fla_int_array *cache_indices,
                     const fla_int_array *initial_state_mode, const fla_int_array *num_accepted_tokens,
                     int64_t activation_mode, int64_t pad_slot_id, int64_t head_num, const fla_tensor *out, void *workspace,
                     uint64_t workspace_size, hipStream_t stream, uint64_t *query) {
    const char *op = "causal_conv1d";
    int rc;
    FLA_REQUIRE(initial_state_mode == nullptr || initial_state_mode->data == nullptr, FLA_ERR_UNSUPPORTED,
                "%s: initial_state_mode is only supported in run_mode=0.", op);
    FLA_REQUIRE(head_num == 0, FLA_ERR_UNSUPPORTED, "%s: run_mode=1 does not support a head-split output (head_num must be 0).", op);
    FLA_REQUIRE(activation_mode == 0 || activation_mode == 1, FLA_ERR_SHAPE, "%s: activation_mode must be 0 or 1.", op);
    FLA_REQUIRE(x->ndim == 2 || x->ndim == 3, FLA_ERR_SHAPE, "%s: x must be [B,S,D], [B,D] or packed [T,D].", op);
    const int64_t D = x->shape[x->ndim - 1];
    const int64_t W = weight->shape[0];
    FLA_REQUIRE(W >= 2 && W <= kMaxW, FLA_ERR_SHAPE, "%s: width must be 2, 3 or 4, got %lld.", op, (long long)W);
    FLA_REQUIRE(weight->shape[1] == D, FLA_ERR_SHAPE, "%s: weight must be [W,D].", op);
    FLA_REQUIRE(D % 16 == 0, FLA_ERR_SHAPE, "%s: D must be a multiple of 16, got %lld.", op, (long long)D);
    FLA_REQUIRE(inner_unit(x) && inner_unit(weight) && inner_unit(out) && same_shape(out, x), FLA_ERR_SHAPE,
                "%s: out must have the shape of x; innermost strides must be 1.", op);
    if (bias && bias->data) {
        if ((rc = check_tensor(bias, op, "bias", 1, dt_bit(x->dtype)))) return rc;
        FLA_REQUIRE(bias->shape[0] == D && inner_unit(bias), FLA_ERR_SHAPE, "%s: bias must be a contiguous [D].", op);
    }
    FLA_REQUIRE(conv_states && conv_states->data, FLA_ERR_NULL, "%s: run_mode=1 needs conv_states.", op);
    if ((rc = check_tensor(conv_states, op, "conv_states", 3, dt_bit(x->dtype)))) return rc;
    const int64_t state_len = conv_states->shape[1];
    FLA_REQUIRE(state_len >= W - 1 && conv_states->shape[2] == D && inner_unit(conv_states), FLA_ERR_SHAPE,
                "%s: conv_states must be [N, >=W-1, D] with unit channel stride.", op);

    FLA_REQUIRE(aligned(x) && aligned(out) && aligned(weight) && aligned(conv_states), FLA_ERR_SHAPE,
                "%s: rows of x, out, weight and conv_states must be 16-byte aligned.", op);
    std::vector<int32_t> qsl, cache, nat;
    const bool has_qsl = query_start_loc && query_start_loc->data;
    int64_t N, S;
    bool packed = false;
    if (x->ndim == 3) {
        N = x->shape[0];
        S = x->shape[1];
        FLA_REQUIRE(!has_qsl || (int64_t)query_start_loc->size == N + 1, FLA_ERR_METADATA,
                    "%s: query_start_loc.size must equal batch + 1.", op);
        if (has_qsl)   // a [B,S,D] batch has S tokens per sequence: any other segmentation would be silently ignored
            for (int64_t i = 0; i <= N; ++i)
                FLA_REQUIRE(query_start_loc->data[i] == i * S, FLA_ERR_METADATA,
                            "%s: with a rank-3 x, query_start_loc must be [0, S, 2S, ...]; pack the tokens as [T,D] for "
                            "ragged sequences.", op);
    } else if (has_qsl && (int64_t)query_start_loc->size - 1 != x->shape[0]) {
        packed = true;                     // 2-D varlen decode: segments of a packed token axis
        N = (int64_t)query_start_loc->size - 1;
        S = 0;
    } else {
        N = x->shape[0];                   // 2-D decode: one token per sequence
        S = 1;
    }
    if (packed) {
        copy_int_array(qsl, query_start_loc);
        FLA_REQUIRE(N >= 1 && qsl[0] == 0 && qsl[N] == x->shape[0], FLA_ERR_METADATA, "%s: query_start_loc must span [0, T].", op);
        for (int i = 0; i < N; ++i)
            FLA_REQUIRE(qsl[i] <= qsl[i + 1], FLA_ERR_METADATA, "%s: query_start_loc must be non-decreasing.", op);
    }
    if (copy_int_array(cache, cache_indices))
        FLA_REQUIRE((int64_t)cache.size() == N, FLA_ERR_METADATA, "%s: cache_indices must have one entry per sequence.", op);
    for (int64_t i = 0; i < N; ++i) {
        const int64_t slot = cache.empty() ? i : cache[i];
        FLA_REQUIRE(slot == pad_slot_id || (slot >= 0 && slot < conv_states->shape[0]), FLA_ERR_METADATA,
                    "%s: cache index %lld out of range.", op, (long long)slot);
    }
    if (copy_int_array(nat, num_accepted_tokens)) {
        FLA_REQUIRE(W == 4, FLA_ERR_UNSUPPORTED, "%s: num_accepted_tokens is only supported for width 4.", op);
        FLA_REQUIRE((int64_t)nat.size() == N, FLA_ERR_METADATA, "%s: num_accepted_tokens must have one entry per sequence.", op);
        if (x->ndim == 3)
            FLA_REQUIRE(state_len >= (W - 1) + (S - 1), FLA_ERR_SHAPE,
                        "%s: speculative decoding needs state_len >= (W-1) + (S-1) = %lld, got %lld.", op,
                        (long long)((W - 1) + (S - 1)), (long long)state_len);
        for (int64_t i = 0; i < N; ++i) {
            const int64_t limit = packed ? qsl[i + 1] - qsl[i] : S;
            FLA_REQUIRE(nat[i] >= 0 && nat[i] <= limit, FLA_ERR_METADATA,
                        "%s: num_accepted_tokens[%lld]=%d must lie in [0, %lld].", op, (long long)i, nat[i], (long long)limit);
        }
    }
    const size_t meta_ints = qsl.size() + cache.size() + nat.size();
    const uint64_t need = ((meta_ints * 4 + 255) / 256) * 256;
    if (query) {
        *query = need;
        return FLA_OK;
    }
    FLA_REQUIRE(need == 0 || (workspace != nullptr && workspace_size >= need), FLA_ERR_WORKSPACE,
                "%s: workspace of %llu bytes required.", op, (unsigned long long)need);
    if (N == 0 || x->shape[0] == 0) return FLA_OK;
    ConvUpdateParams p{};
    p.x = x->data;
    p.weight = weight->data;
    p.bias = (bias && bias->data) ? bias->data : nullptr;
    p.conv_states = conv_states->data;
    p.out = out->data;
    if (meta_ints) {
        std::vector<int32_t> meta;
        meta.insert(meta.end(), qsl.begin(), qsl.end());
        meta.insert(meta.end(), cache.begin(), cache.end());
        meta.insert(meta.end(), nat.begin(), nat.end());
        if ((rc = stage_to_device(workspace, meta.data(), meta.size() * 4, stream))) return rc;
        const int32_t *base = static_cast<const int32_t *>(workspace);
        p.qsl = qsl.empty() ? nullptr : base;
        p.cache = cache.empty() ? nullptr : base + qsl.size();
        p.nat = nat.empty() ? nullptr : base + qsl.size() + cache.size();
    }
    if (x->ndim == 3) {
        p.x_sb = x->stride[0];
        p.x_ss = x->stride[1];
        p.o_sb = out->stride[0];
        p.o_ss = out->stride[1];
    } else {   // rows of a 2-D x are sequences (S = 1) or packed tokens
        p.x_sb = p.x_ss = x->stride[0];
        p.o_sb = p.o_ss = out->stride[0];
    }
    p.w_sr = weight->stride[0];
    p.cs_sn = conv_states->stride[0];
    p.cs_sp = conv_states->stride[1];
    p.S = (int)S;
    p.D = (int)D;
    p.W = (int)W;
    p.N = (int)N;
    p.state_len = (int)state_len;
    p.activation = (int)activation_mode;
    p.pad_slot = (int)pad_slot_id;
    const dim3 block(64), grid((unsigned)((D / 8 + 63) / 64), (unsigned)N);
    if (x->dtype == FLA_BF16) FLA_LAUNCH("conv1d_update", stream, conv1d_update_kernel<bf16>, grid, block, 0, stream, p);
    else FLA_LAUNCH("conv1d_update", stream, conv1d_update_kernel<f16>, grid, block, 0, stream, p);
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

int conv_impl(const fla_tensor *x, const fla_tensor *weight, const fla_tensor *bias, const fla_tensor *conv_states,
              const fla_int_array *query_start_loc, const fla_int_array *cache_indices,
              const fla_int_array *initial_state_mode, const fla_int_array *num_accepted_tokens,
              int64_t activation_mode, int64_t pad_slot_id, int64_t run_mode, int64_t head_num, const fla_tensor *out,
              void *workspace, uint64_t workspace_size, hipStream_t stream, uint64_t *query) {
    const char *op = "causal_conv1d";
    const int half_mask = dt_bit(FLA_BF16) | dt_bit(FLA_F16);
    int rc;
    if ((rc = check_tensor(x, op, "x", -1, half_mask))) return rc;
    if ((rc = check_tensor(weight, op, "weight", 2, dt_bit(x->dtype)))) return rc;
    if ((rc = check_tensor(out, op, "out", -1, dt_bit(x->dtype)))) return rc;
    FLA_REQUIRE(run_mode == 0 || run_mode == 1, FLA_ERR_SHAPE, "%s: run_mode must be 0 (prefill) or 1 (update), got %lld.", op,
                (long long)run_mode);
    if (run_mode == 1)
        return conv_update_impl(x, weight, bias, conv_states, query_start_loc, cache_indices, initial_state_mode,
                                num_accepted_tokens, activation_mode, pad_slot_id, head_num, out, workspace, workspace_size,
                                stream, query);
    FLA_REQUIRE(num_accepted_tokens == nullptr || num_accepted_tokens->data == nullptr, FLA_ERR_UNSUPPORTED,
                "%s: num_accepted_tokens is only meaningful for run_mode=1.", op);
    FLA_REQUIRE(activation_mode == 0 || activation_mode == 1, FLA_ERR_SHAPE, "%s: activation_mode must be 0 or 1.", op);
    FLA_REQUIRE(x->ndim == 2 || x->ndim == 3, FLA_ERR_SHAPE, "%s: x must be [B,S,D] or [T,D].", op);
    const bool packed = x->ndim == 2;
    const int64_t D = x->shape[x->ndim - 1];
    const int64_t S = x->shape[x->ndim - 2];
    const int64_t B = packed ? 1 : x->shape[0];
    const int64_t W = weight->shape[0];
    FLA_REQUIRE(W >= 2 && W <= kMaxW, FLA_ERR_SHAPE, "%s: width must be 2, 3 or 4, got %lld.", op, (long long)W);
    FLA_REQUIRE(weight->shape[1] == D, FLA_ERR_SHAPE, "%s: weight must be [W,D].", op);
    FLA_REQUIRE(D % 16 == 0, FLA_ERR_SHAPE, "%s: D must be a multiple of 16, got %lld.", op, (long long)D);
    FLA_REQUIRE(inner_unit(x) && inner_unit(weight) && inner_unit(out), FLA_ERR_SHAPE,
                "%s: innermost stride of x, weight and out must be 1.", op);
    FLA_REQUIRE(B * S < ((int64_t)1 << 31) && D < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents exceed int32.", op);
    FLA_REQUIRE(aligned(x) && aligned(out) && aligned(weight), FLA_ERR_SHAPE,
                "%s: rows of x, out and weight must be 16-byte aligned.", op);
    if (bias && bias->data) {
        if ((rc = check_tensor(bias, op, "bias", 1, dt_bit(x->dtype)))) return rc;
        FLA_REQUIRE(bias->shape[0] == D && inner_unit(bias) && aligned(bias), FLA_ERR_SHAPE,
                    "%s: bias must be a contiguous, 16-byte aligned [D].", op);
    }
    FLA_REQUIRE(head_num >= 0, FLA_ERR_SHAPE, "%s: head_num must be >= 0.", op);
    int64_t head_dim = D;
    if (head_num > 0) {
        FLA_REQUIRE(D % head_num == 0 && (D / head_num) % 8 == 0, FLA_ERR_SHAPE,
                    "%s: D/head_num must be a multiple of 8.", op);
        head_dim = D / head_num;
    }

    std::vector<int32_t> qsl, cache, init;
    int N = (int)B;
    if (packed) {
        FLA_REQUIRE(query_start_loc && query_start_loc->data && query_start_loc->size >= 2, FLA_ERR_METADATA,
                    "%s: a packed [T,D] input needs query_start_loc.", op);
        copy_int_array(qsl, query_start_loc);
        N = (int)qsl.size() - 1;
        FLA_REQUIRE(qsl[0] == 0 && qsl[N] == S, FLA_ERR_METADATA, "%s: query_start_loc must span [0, T].", op);
        for (int i = 0; i < N; ++i)
            FLA_REQUIRE(qsl[i] <= qsl[i + 1], FLA_ERR_METADATA, "%s: query_start_loc must be non-decreasing.", op);
    } else {
        FLA_REQUIRE(query_start_loc == nullptr || query_start_loc->data == nullptr, FLA_ERR_METADATA,
                    "%s: query_start_loc requires a packed [T,D] input.", op);
    }
    if (copy_int_array(cache, cache_indices))
        FLA_REQUIRE((int)cache.size() == N, FLA_ERR_METADATA, "%s: cache_indices must have one entry per sequence.", op);
    if (copy_int_array(init, initial_state_mode))
        FLA_REQUIRE((int)init.size() == N, FLA_ERR_METADATA, "%s: initial_state_mode must have one entry per sequence.",
                    op);
    const bool has_states = conv_states && conv_states->data;
    if (has_states) {
        if ((rc = check_tensor(conv_states, op, "conv_states", 3, dt_bit(x->dtype)))) return rc;
        FLA_REQUIRE(conv_states->shape[1] >= W - 1 && conv_states->shape[2] == D && inner_unit(conv_states),
                    FLA_ERR_SHAPE, "%s: conv_states must be [N, >=W-1, D] with unit channel stride.", op);
        FLA_REQUIRE(aligned(conv_states), FLA_ERR_SHAPE, "%s: rows of conv_states must be 16-byte aligned.", op);
        for (int i = 0; i < N; ++i) {
            const int64_t slot = cache.empty() ? i : cache[i];
            FLA_REQUIRE(slot == pad_slot_id || (slot >= 0 && slot < conv_states->shape[0]), FLA_ERR_METADATA,
                        "%s: cache index %lld out of range.", op, (long long)slot);
        }
    }
    // output shape
    if (head_num > 0) {
        const int nd = packed ? 3 : 4;
        FLA_REQUIRE(out->ndim == nd, FLA_ERR_SHAPE, "%s: head-split out must be rank %d.", op, nd);
        const int o = packed ? 0 : 1;
        FLA_REQUIRE(out->shape[o] == head_num && out->shape[o + 1] == S && out->shape[o + 2] == head_dim &&
                        (packed || out->shape[0] == B),
                    FLA_ERR_SHAPE, "%s: out must be [B,head_num,S,D/head_num].", op);
    } else {
        FLA_REQUIRE(same_shape(out, x), FLA_ERR_SHAPE, "%s: out must have the shape of x.", op);
    }

    const size_t meta_ints = qsl.size() + cache.size() + init.size();
    const uint64_t need = ((meta_ints * 4 + 255) / 256) * 256;
    if (query) {
        *query = need;
        return FLA_OK;
    }
    FLA_REQUIRE(need == 0 || (workspace != nullptr && workspace_size >= need), FLA_ERR_WORKSPACE,
                "%s: workspace of %llu bytes required.", op, (unsigned long long)need);
    if (B * S == 0) return FLA_OK;

    ConvParams p{};
    p.x = x->data;
    p.weight = weight->data;
    p.bias = (bias && bias->data) ? bias->data : nullptr;
    p.conv_states = has_states ? conv_states->data : nullptr;
    p.out = out->data;
    if (meta_ints) {
        std::vector<int32_t> meta;
        meta.insert(meta.end(), qsl.begin(), qsl.end());
        meta.insert(meta.end(), cache.begin(), cache.end());
        meta.insert(meta.end(), init.begin(), init.end());
        if ((rc = stage_to_device(workspace, meta.data(), meta.size() * 4, stream))) return rc;
        const int32_t *base = static_cast<const int32_t *>(workspace);
        p.qsl = qsl.empty() ? nullptr : base;
        p.cache = cache.empty() ? nullptr : base + qsl.size();
        p.init = init.empty() ? nullptr : base + qsl.size() + cache.size();
    }
    p.x_sb = packed ? 0 : x->stride[0];
    p.x_ss = x->stride[x->ndim - 2];
    if (head_num > 0) {
        const int o = packed ? 0 : 1;
        p.o_sb = packed ? 0 : out->stride[0];
        p.o_sh = out->stride[o];
        p.o_ss = out->stride[o + 1];
    } else {
        p.o_sb = packed ? 0 : out->stride[0];
        p.o_sh = 0;
        p.o_ss = out->stride[out->ndim - 2];
    }
    p.w_sr = weight->stride[0];
    if (has_states) {
        p.cs_sn = conv_states->stride[0];
        p.cs_sp = conv_states->stride[1];
    }
    p.B = (int)B;
    p.S = (int)S;
    p.D = (int)D;
    p.W = (int)W;
    p.N = N;
    p.head_dim = (int)head_dim;
    // Tile height: tall tiles amortise the W-1 row halo, short tiles give the scheduler enough
    // workgroups to keep every CU busy through the tail of the launch.
    int tok = 32;
    {
        const int64_t col_blocks = (D / 8 + kThreads - 1) / kThreads;
        while (tok > 8 && ((B * S + tok - 1) / tok) * col_blocks < (int64_t)24 * num_cus()) tok >>= 1;
    }
    p.tok = tok;
    p.tiles_per_seq = (int)((S + tok - 1) / tok);
    p.activation = (int)activation_mode;
    p.pad_slot = (int)pad_slot_id;
    p.varlen = packed ? 1 : 0;

    const bool is_bf16 = x->dtype == FLA_BF16;
    const dim3 block(kThreads);
    const dim3 grid((unsigned)(p.tiles_per_seq * (packed ? 1 : B)), (unsigned)((D / 8 + kThreads - 1) / kThreads));
    const bool dense_fast = !packed && cache.empty() && init.empty();
    if (dense_fast) {
        // 32-row tiles while they still give every CU eight workgroups, 16-row tiles below that
        const int ft = (B * ((S + 31) / 32) * (int64_t)grid.y >= (int64_t)8 * num_cus()) ? 32 : 16;
        p.tok = ft;
        p.tiles_per_seq = (int)((S + ft - 1) / ft);
        const dim3 fgrid((unsigned)(p.tiles_per_seq * B), grid.y);
        const bool act = activation_mode == 1;
#define FLA_LAUNCH_DENSE(TT, WW, TK)                                                                              \
    if (act) FLA_LAUNCH("conv1d_fwd", stream, (conv1d_dense_kernel<TT, WW, TK, true>), fgrid, block, 0, stream, p); \
    else FLA_LAUNCH("conv1d_fwd", stream, (conv1d_dense_kernel<TT, WW, TK, false>), fgrid, block, 0, stream, p)
#define FLA_LAUNCH_DENSE_W(TT, TK)               \
    switch (W) {                                 \
        case 2: FLA_LAUNCH_DENSE(TT, 2, TK); break; \
        case 3: FLA_LAUNCH_DENSE(TT, 3, TK); break; \
        default: FLA_LAUNCH_DENSE(TT, 4, TK); break; \
    }
        if (is_bf16) {
            if (ft == 32) { FLA_LAUNCH_DENSE_W(bf16, 32) } else { FLA_LAUNCH_DENSE_W(bf16, 16) }
        } else {
            if (ft == 32) { FLA_LAUNCH_DENSE_W(f16, 32) } else { FLA_LAUNCH_DENSE_W(f16, 16) }
        }
#undef FLA_LAUNCH_DENSE_W
#undef FLA_LAUNCH_DENSE
    } else {
#define FLA_LAUNCH_CONV_T(WW, TT)                                                                      \
    if (is_bf16) FLA_LAUNCH("conv1d_fwd", stream, (conv1d_fwd_kernel<bf16, WW, TT>), grid, block, 0, stream, p); \
    else FLA_LAUNCH("conv1d_fwd", stream, (conv1d_fwd_kernel<f16, WW, TT>), grid, block, 0, stream, p)
#define FLA_LAUNCH_CONV(WW)                                      \
    switch (tok) {                                               \
        case 8: FLA_LAUNCH_CONV_T(WW, 8); break;                 \
        case 16: FLA_LAUNCH_CONV_T(WW, 16); break;               \
        case 64: FLA_LAUNCH_CONV_T(WW, 64); break;               \
        default: FLA_LAUNCH_CONV_T(WW, 32); break;               \
    }
    switch (W) {
        case 2: FLA_LAUNCH_CONV(2); break;
        case 3: FLA_LAUNCH_CONV(3); break;
        default: FLA_LAUNCH_CONV(4); break;
    }
#undef FLA_LAUNCH_CONV
#undef FLA_LAUNCH_CONV_T
    }
    FLA_HIP_CHECK(hipGetLastError());
    if (has_states && N > 0) {
        const dim3 sgrid((unsigned)((D / 8 + 63) / 64), (unsigned)N);
        if (is_bf16) FLA_LAUNCH("conv1d_state", stream, conv1d_state_kernel<bf16>, sgrid, dim3(64), 0, stream, p);
        else FLA_LAUNCH("conv1d_state", stream, conv1d_state_kernel<f16>, sgrid, dim3(64), 0, stream, p);
        FLA_HIP_CHECK(hipGetLastError());
    }
    return FLA_OK;
}

}  // namespace
}  // namespace fla

extern "C" int fla_causal_conv1d_get_workspace_size(
    const fla_tensor *x, const fla_tensor *weight, const fla_tensor *bias, const fla_tensor *conv_states,
    const fla_int_array *query_start_loc, const fla_int_array *cache_indices, const fla_int_array *initial_state_mode,
    const fla_int_array *num_accepted_tokens, int64_t activation_mode, int64_t pad_slot_id, int64_t run_mode,
    int64_t head_num, const fla_tensor *out, uint64_t *workspace_size) {
    if (workspace_size == nullptr) return fla::fail(FLA_ERR_NULL, "causal_conv1d: workspace_size must not be null.");
    return fla::guarded([&] { return fla::conv_impl(x, weight, bias, conv_states, query_start_loc, cache_indices, initial_state_mode,
                          num_accepted_tokens, activation_mode, pad_slot_id, run_mode, head_num, out, nullptr, 0,
                          nullptr, workspace_size); });
}

extern "C" int fla_causal_conv1d(const fla_tensor *x, const fla_tensor *weight, const fla_tensor *bias,
                                 const fla_tensor *conv_states, const fla_int_array *query_start_loc,
                                 const fla_int_array *cache_indices, const fla_int_array *initial_state_mode,
                                 const fla_int_array *num_accepted_tokens, int64_t activation_mode,
                                 int64_t pad_slot_id, int64_t run_mode, int64_t head_num, const fla_tensor *out,
                                 void *workspace, uint64_t workspace_size, void *stream) {
    return fla::guarded([&] { return fla::conv_impl(x, weight, bias, conv_states, query_start_loc, cache_indices, initial_state_mode,
                          num_accepted_tokens, activation_mode, pad_slot_id, run_mode, head_num, out, workspace,
                          workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}
