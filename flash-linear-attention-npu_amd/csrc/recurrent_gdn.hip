// recurrent_gated_delta_rule: token-by-token gated delta rule with an in-place,
// V-first state [Block, Nv, Dv, Dk].  Bandwidth-bound for decode: the state is
// streamed once in and once out per (sequence, head); all arithmetic is fp32
// vector work with wave-level reductions, no MFMA.
//
// One 256-thread workgroup owns one (sequence, value head).  A state row (fixed
// v, Dk contiguous floats) is spread over Dk/4 adjacent lanes, 4 floats each, so
// every wave load/store instruction touches whole 512-byte (Dk=128) row
// segments.  The tile stays in registers across the tokens of a sequence.
// Semantics: recurrent_gated_delta_rule/README.md:6-33, tests/pta/golden.py:14-99,
// kernel op_kernel/recurrent_gated_delta_rule.h:364-403.
#include "common.h"
#include "device_utils.h"

namespace fla {
namespace {

constexpr int kThreads = 256;
constexpr int kTokBatch = 8;  // tokens staged in LDS per synchronisation

struct RecParams {
    const bf16 *q, *k, *v, *beta;
    void *state;
    const int32_t *seq_lens;   // [B+1]
    const int32_t *slot_idx;   // [T]
    const int32_t *accepted;   // [B] or null
    const float *g;            // [T,Nv] or null
    const float *gk;           // [T,Nv,Dk] or null
    bf16 *out;
    int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh, b_st, b_sh, o_st, o_sh;
    int64_t g_st, g_sh, gk_st, gk_sh;
    int64_t s_sb, s_sh, s_sv;  // state strides: block, head, v-row (elements)
    int T, B, Nk, Nv, n_blocks;
    float scale;
};

template <typename ST> struct StateIO;
template <> struct StateIO<float> {
    // the state is streamed exactly once in and once out: keep it out of the caches
    static __device__ __forceinline__ f32x4 load(const float *p) {
        return __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
    }
    static __device__ __forceinline__ void store(float *p, f32x4 v) {
        __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p));
    }
};
template <> struct StateIO<bf16> {
    static __device__ __forceinline__ f32x4 load(const bf16 *p) {
        bf16x4 r = *reinterpret_cast<const bf16x4 *>(p);
        f32x4 v = {(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
        return v;
    }
    static __device__ __forceinline__ void store(bf16 *p, f32x4 v) { *reinterpret_cast<bf16x4 *>(p) = cvt4(v); }
};

template <typename ST, int DK, int DV>
__global__ void __launch_bounds__(kThreads) recurrent_gdn_kernel(const RecParams p) {
    constexpr int LPR = DK / 4;               // lanes per state row
    constexpr int RPW = kWave / LPR;          // rows per wave pass
    constexpr int RPP = RPW * (kThreads / kWave);  // rows per block pass
    constexpr int NP = DV / RPP;              // passes = rows per thread
    static_assert(DV % RPP == 0, "tile does not divide");

    __shared__ float s_k[kTokBatch][DK], s_q[kTokBatch][DK], s_gk[kTokBatch][DK];
    __shared__ float s_v[kTokBatch][DV], s_o[kTokBatch][DV];
    __shared__ float s_decay[kTokBatch], s_beta[kTokBatch];
    __shared__ int s_slot[kTokBatch + 1];
    __shared__ int s_red[kThreads / kWave];

    const int n = blockIdx.x / p.Nv;          // sequence
    const int h = blockIdx.x % p.Nv;          // value head
    const int hk = h / (p.Nv / p.Nk);
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int col = (lane % LPR) * 4;         // first of this lane's 4 Dk columns
    const int row0 = wave * RPW + lane / LPR; // row within a pass

    // first token of sequence n = skip count + lengths of the earlier sequences
    int part = 0;
    for (int j = tid; j <= n; j += kThreads) part += p.seq_lens[j];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
    if (lane == 0) s_red[wave] = part;
    __syncthreads();
    int tok0 = 0;
#pragma unroll
    for (int w = 0; w < kThreads / kWave; ++w) tok0 += s_red[w];
    const int len = p.seq_lens[n + 1];
    if (len <= 0 || tok0 + len > p.T) return;  // invalid metadata: leave untouched (kernel :168-173)

    int src_tok = tok0;
    if (p.accepted) src_tok = tok0 + p.accepted[n] - 1;
    if (src_tok < 0 || src_tok >= p.T) return;
    const int src_slot = p.slot_idx[src_tok];
    if (src_slot < 0 || src_slot >= p.n_blocks) return;

    ST *state = static_cast<ST *>(p.state);
    f32x4 S[NP];
    {
        const ST *sp = state + src_slot * p.s_sb + h * p.s_sh + col;
#pragma unroll
        for (int i = 0; i < NP; ++i) S[i] = StateIO<ST>::load(sp + (int64_t)(i * RPP + row0) * p.s_sv);
    }

    for (int tb = 0; tb < len; tb += kTokBatch) {
        const int nb = min(kTokBatch, len - tb);
        __syncthreads();  // previous batch fully consumed
        // ---- stage q, k, v, gates of up to kTokBatch tokens -------------------------
        for (int idx = tid; idx < nb * DK; idx += kThreads) {
            const int j = idx / DK, c = idx % DK;
            const int64_t t = tok0 + tb + j;
            s_k[j][c] = (float)p.k[t * p.k_st + hk * p.k_sh + c];
            s_q[j][c] = (float)p.q[t * p.q_st + hk * p.q_sh + c] * p.scale;
            if (p.gk) s_gk[j][c] = __expf(p.gk[t * p.gk_st + h * p.gk_sh + c]);
        }
        for (int idx = tid; idx < nb * DV; idx += kThreads) {
            const int j = idx / DV, c = idx % DV;
            const int64_t t = tok0 + tb + j;
            s_v[j][c] = (float)p.v[t * p.v_st + h * p.v_sh + c];
        }
        if (tid < nb) {
            const int64_t t = tok0 + tb + tid;
            s_decay[tid] = p.g ? __expf(p.g[t * p.g_st + h * p.g_sh]) : 1.f;
            s_beta[tid] = (float)p.beta[t * p.b_st + h * p.b_sh];
            s_slot[tid] = p.slot_idx[t];
        }
        if (tid == nb) s_slot[nb] = (tb + nb < len) ? p.slot_idx[tok0 + tb + nb] : -1;
        __syncthreads();

        for (int j = 0; j < nb; ++j) {
            const f32x4 kv = *reinterpret_cast<const f32x4 *>(&s_k[j][col]);
            const f32x4 qv = *reinterpret_cast<const f32x4 *>(&s_q[j][col]);
            f32x4 dec = {s_decay[j], s_decay[j], s_decay[j], s_decay[j]};
            if (p.gk) dec *= *reinterpret_cast<const f32x4 *>(&s_gk[j][col]);
            const float beta = s_beta[j];
            float sk[NP];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                S[i] *= dec;
                sk[i] = S[i][0] * kv[0] + S[i][1] * kv[1] + S[i][2] * kv[2] + S[i][3] * kv[3];
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) sk[i] = group_sum<LPR>(sk[i]);
            float so[NP];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const float delta = beta * (s_v[j][i * RPP + row0] - sk[i]);
                S[i] += delta * kv;
                so[i] = S[i][0] * qv[0] + S[i][1] * qv[1] + S[i][2] * qv[2] + S[i][3] * qv[3];
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) so[i] = group_sum<LPR>(so[i]);
            if (lane % LPR == 0) {
#pragma unroll
                for (int i = 0; i < NP; ++i) s_o[j][i * RPP + row0] = so[i];
            }
            // the state is visible after every token; a write is redundant only when the
            // next token of this sequence targets the same slot
            const int slot = s_slot[j];
            if (slot != s_slot[j + 1] && slot >= 0 && slot < p.n_blocks) {
                ST *dp = state + slot * p.s_sb + h * p.s_sh + col;
#pragma unroll
                for (int i = 0; i < NP; ++i) StateIO<ST>::store(dp + (int64_t)(i * RPP + row0) * p.s_sv, S[i]);
            }
        }
        __syncthreads();
        for (int idx = tid; idx < nb * DV; idx += kThreads) {
            const int j = idx / DV, c = idx % DV;
            const int64_t t = tok0 + tb + j;
            p.out[t * p.o_st + h * p.o_sh + c] = (bf16)s_o[j][c];
        }
    }
}

int rec_impl(const fla_tensor *query, const fla_tensor *key, const fla_tensor *value, const fla_tensor *beta,
             const fla_tensor *state, const fla_tensor *actual_seq_lengths, const fla_tensor *ssm_state_indices,
             const fla_tensor *g, const fla_tensor *gk, const fla_tensor *num_accepted_tokens, float scale,
             const fla_tensor *out, void *workspace, uint64_t workspace_size, hipStream_t stream, uint64_t *query_ws) {
    (void)workspace;
    (void)workspace_size;
    const char *op = "recurrent_gated_delta_rule";
    const int bf = dt_bit(FLA_BF16);
    int rc;
    if ((rc = check_tensor(query, op, "query", 3, bf))) return rc;
    if ((rc = check_tensor(key, op, "key", 3, bf))) return rc;
    if ((rc = check_tensor(value, op, "value", 3, bf))) return rc;
    if ((rc = check_tensor(beta, op, "beta", 2, bf))) return rc;
    if ((rc = check_tensor(state, op, "state", 4, bf | dt_bit(FLA_F32)))) return rc;
    if ((rc = check_tensor(actual_seq_lengths, op, "actual_seq_lengths", 1, dt_bit(FLA_I32)))) return rc;
    if ((rc = check_tensor(ssm_state_indices, op, "ssm_state_indices", 1, dt_bit(FLA_I32)))) return rc;
    if ((rc = check_tensor(out, op, "out", 3, bf))) return rc;
    const bool has_g = g && g->data, has_gk = gk && gk->data, has_acc = num_accepted_tokens && num_accepted_tokens->data;
    FLA_REQUIRE(has_g || has_gk, FLA_ERR_NULL, "%s: either g or gk must be provided.", op);
    if (has_g && (rc = check_tensor(g, op, "g", 2, dt_bit(FLA_F32)))) return rc;
    if (has_gk && (rc = check_tensor(gk, op, "gk", 3, dt_bit(FLA_F32)))) return rc;
    if (has_acc && (rc = check_tensor(num_accepted_tokens, op, "num_accepted_tokens", 1, dt_bit(FLA_I32)))) return rc;

    const int64_t T = query->shape[0], Nk = query->shape[1], Dk = query->shape[2];
    const int64_t Nv = value->shape[1], Dv = value->shape[2];
    FLA_REQUIRE(same_shape(query, key), FLA_ERR_SHAPE, "%s: key shape must equal query shape.", op);
    FLA_REQUIRE(value->shape[0] == T && same_shape(out, value), FLA_ERR_SHAPE, "%s: value/out must be [T,Nv,Dv].", op);
    FLA_REQUIRE(beta->shape[0] == T && beta->shape[1] == Nv, FLA_ERR_SHAPE, "%s: beta must be [T,Nv].", op);
    FLA_REQUIRE(Nk > 0 && Nv > 0 && Nv % Nk == 0, FLA_ERR_SHAPE, "%s: Nv must be a positive multiple of Nk.", op);
    FLA_REQUIRE(Nk <= 256 && Nv <= 256, FLA_ERR_SHAPE, "%s: Nk and Nv must be <= 256.", op);
    FLA_REQUIRE(state->shape[1] == Nv && state->shape[2] == Dv && state->shape[3] == Dk, FLA_ERR_SHAPE,
                "%s: state must be [Block,Nv,Dv,Dk].", op);
    FLA_REQUIRE(state->stride[3] == 1 && state->stride[2] % 4 == 0 && state->stride[1] % 4 == 0 &&
                    state->stride[0] % 4 == 0,
                FLA_ERR_SHAPE, "%s: state rows must be contiguous and 16-byte aligned.", op);
    FLA_REQUIRE(actual_seq_lengths->shape[0] >= 2, FLA_ERR_SHAPE,
                "%s: actual_seq_lengths needs the prefix entry and at least one length.", op);
    FLA_REQUIRE(ssm_state_indices->shape[0] == T, FLA_ERR_SHAPE, "%s: ssm_state_indices must be [T].", op);
    const int64_t B = actual_seq_lengths->shape[0] - 1;
    if (has_g) FLA_REQUIRE(g->shape[0] == T && g->shape[1] == Nv, FLA_ERR_SHAPE, "%s: g must be [T,Nv].", op);
    if (has_gk)
        FLA_REQUIRE(gk->shape[0] == T && gk->shape[1] == Nv && gk->shape[2] == Dk && inner_unit(gk), FLA_ERR_SHAPE,
                    "%s: gk must be [T,Nv,Dk].", op);
    if (has_acc) FLA_REQUIRE(num_accepted_tokens->shape[0] == B, FLA_ERR_SHAPE, "%s: num_accepted_tokens must be [B].", op);
    FLA_REQUIRE(inner_unit(query) && inner_unit(key) && inner_unit(value) && inner_unit(out), FLA_ERR_SHAPE,
                "%s: innermost stride of query/key/value/out must be 1.", op);
    FLA_REQUIRE(is_contiguous(actual_seq_lengths) && is_contiguous(ssm_state_indices) &&
                    (!has_acc || is_contiguous(num_accepted_tokens)),
                FLA_ERR_SHAPE, "%s: index tensors must be contiguous.", op);
    const bool ok_dims = (Dk == 128 && Dv == 128) || (Dk == 64 && Dv == 64) || (Dk == 128 && Dv == 256) ||
                         (Dk == 64 && Dv == 128);
    FLA_REQUIRE(ok_dims, FLA_ERR_UNSUPPORTED, "%s: (Dk,Dv)=(%lld,%lld) has no kernel; built: (128,128),(64,64),(128,256),(64,128).",
                op, (long long)Dk, (long long)Dv);
    FLA_REQUIRE(B * Nv < ((int64_t)1 << 31) && T < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents exceed int32.", op);
    if (query_ws) {
        *query_ws = 0;
        return FLA_OK;
    }
    if (T == 0 || B == 0) return FLA_OK;

    RecParams p{};
    p.q = static_cast<const bf16 *>(query->data);
    p.k = static_cast<const bf16 *>(key->data);
    p.v = static_cast<const bf16 *>(value->data);
    p.beta = static_cast<const bf16 *>(beta->data);
    p.state = state->data;
    p.seq_lens = static_cast<const int32_t *>(actual_seq_lengths->data);
    p.slot_idx = static_cast<const int32_t *>(ssm_state_indices->data);
    p.accepted = has_acc ? static_cast<const int32_t *>(num_accepted_tokens->data) : nullptr;
    p.g = has_g ? static_cast<const float *>(g->data) : nullptr;
    p.gk = has_gk ? static_cast<const float *>(gk->data) : nullptr;
    p.out = static_cast<bf16 *>(out->data);
    p.q_st = query->stride[0]; p.q_sh = query->stride[1];
    p.k_st = key->stride[0]; p.k_sh = key->stride[1];
    p.v_st = value->stride[0]; p.v_sh = value->stride[1];
    p.b_st = beta->stride[0]; p.b_sh = beta->stride[1];
    p.o_st = out->stride[0]; p.o_sh = out->stride[1];
    if (has_g) { p.g_st = g->stride[0]; p.g_sh = g->stride[1]; }
    if (has_gk) { p.gk_st = gk->stride[0]; p.gk_sh = gk->stride[1]; }
    p.s_sb = state->stride[0]; p.s_sh = state->stride[1]; p.s_sv = state->stride[2];
    p.T = (int)T; p.B = (int)B; p.Nk = (int)Nk; p.Nv = (int)Nv; p.n_blocks = (int)state->shape[0];
    p.scale = scale;

    const dim3 grid((unsigned)(B * Nv)), block(kThreads);
    const bool f32s = state->dtype == FLA_F32;
#define FLA_LAUNCH_REC(DK, DV)                                                                       \
    if (f32s) FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_kernel<float, DK, DV>), grid, block, 0, stream, p);   \
    else FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_kernel<bf16, DK, DV>), grid, block, 0, stream, p)
    if (Dk == 128 && Dv == 128) { FLA_LAUNCH_REC(128, 128); }
    else if (Dk == 64 && Dv == 64) { FLA_LAUNCH_REC(64, 64); }
    else if (Dk == 128 && Dv == 256) { FLA_LAUNCH_REC(128, 256); }
    else { FLA_LAUNCH_REC(64, 128); }
#undef FLA_LAUNCH_REC
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

}  // namespace
}  // namespace fla

extern "C" int fla_recurrent_gated_delta_rule_get_workspace_size(
    const fla_tensor *query, const fla_tensor *key, const fla_tensor *value, const fla_tensor *beta,
    const fla_tensor *state, const fla_tensor *actual_seq_lengths, const fla_tensor *ssm_state_indices,
    const fla_tensor *g, const fla_tensor *gk, const fla_tensor *num_accepted_tokens, float scale,
    const fla_tensor *out, uint64_t *workspace_size) {
    if (workspace_size == nullptr)
        return fla::fail(FLA_ERR_NULL, "recurrent_gated_delta_rule: workspace_size must not be null.");
    return fla::rec_impl(query, key, value, beta, state, actual_seq_lengths, ssm_state_indices, g, gk,
                         num_accepted_tokens, scale, out, nullptr, 0, nullptr, workspace_size);
}

extern "C" int fla_recurrent_gated_delta_rule(
    const fla_tensor *query, const fla_tensor *key, const fla_tensor *value, const fla_tensor *beta,
    const fla_tensor *state, const fla_tensor *actual_seq_lengths, const fla_tensor *ssm_state_indices,
    const fla_tensor *g, const fla_tensor *gk, const fla_tensor *num_accepted_tokens, float scale,
    const fla_tensor *out, void *workspace, uint64_t workspace_size, void *stream) {
    return fla::rec_impl(query, key, value, beta, state, actual_seq_lengths, ssm_state_indices, g, gk,
                         num_accepted_tokens, scale, out, workspace, workspace_size, static_cast<hipStream_t>(stream),
                         nullptr);
}
