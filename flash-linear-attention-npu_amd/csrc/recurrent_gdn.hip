// recurrent_gated_delta_rule: token-by-token gated delta rule with an in-place,
// V-first state [Block, Nv, Dv, Dk].  Bandwidth-bound for decode: the state is
// streamed once in and once out per (sequence, head); all arithmetic is fp32
// vector work with wave-level reductions, no MFMA.
//
// One 256-thread workgroup owns one (sequence, value head).  A state row (fixed v, Dk contiguous
// floats) is spread over the 16 lanes of one DPP row, Dk/16 floats each in 16-byte pieces 64 columns
// apart, so that every wave load/store instruction touches 256-byte row segments and the two
// reductions per token (S k and S q) are four data-parallel-primitive adds each, with no LDS traffic.
// The tile stays in registers across the tokens of a sequence; q/k/v of the next eight tokens are
// loaded while the current eight are processed.
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

template <typename ST, int DK, int DV, int LPR>
__global__ void __launch_bounds__(kThreads) recurrent_gdn_kernel(const RecParams p) {
    // LPR lanes per state row: 16 (one DPP row, reductions without LDS traffic) for multi-token sequences,
    // Dk/4 (one 16-byte piece per lane, whole 512-byte rows per load instruction) for single-token decode
    constexpr int SEGW = 4 * LPR;             // columns between the 16-byte pieces of a lane
    constexpr int NSEG = DK / SEGW;           // pieces of a row per lane
    constexpr int RPW = kWave / LPR;          // rows per wave pass
    constexpr int RPP = RPW * (kThreads / kWave);  // rows per block pass
    constexpr int NP = DV / RPP;              // passes = rows per thread
    static_assert(DV % RPP == 0 && DK % SEGW == 0 && NSEG >= 1, "tile does not divide");
    constexpr int EQ = kTokBatch * DK / kThreads, EV = kTokBatch * DV / kThreads;   // staged elements per thread
    static_assert(EQ >= 1 && EV >= 1 && DK % EQ == 0 && DV % EV == 0, "staging does not divide");
    typedef bf16 vq_t __attribute__((ext_vector_type(EQ)));
    typedef bf16 vv_t __attribute__((ext_vector_type(EV)));
    typedef float fq_t __attribute__((ext_vector_type(EQ)));

    // token batches are double-buffered: while batch b is consumed from one half, the loads of batch b+1
    // are in flight and land in the other half
    __shared__ __align__(16) float s_k[2][kTokBatch][DK], s_q[2][kTokBatch][DK], s_gk[2][kTokBatch][DK];
    __shared__ __align__(16) float s_v[2][kTokBatch][DV], s_o[kTokBatch][DV];
    __shared__ float s_decay[2][kTokBatch], s_beta[2][kTokBatch];
    __shared__ int s_slot[2][kTokBatch + 1];
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
    f32x4 S[NP][NSEG];
    {
        const ST *sp = state + src_slot * p.s_sb + h * p.s_sh + col;
#pragma unroll
        for (int i = 0; i < NP; ++i)
#pragma unroll
            for (int sg = 0; sg < NSEG; ++sg) S[i][sg] = StateIO<ST>::load(sp + (int64_t)(i * RPP + row0) * p.s_sv + SEGW * sg);
    }

    // ---- staging: thread -> (token jq, columns cq..) of q/k/gk and (token jv, columns cv..) of v ----------
    const int jq = tid * EQ / DK, cq = tid * EQ % DK;
    const int jv = tid * EV / DV, cv = tid * EV % DV;
    vq_t pre_q, pre_k;
    vv_t pre_v;
    fq_t pre_gk;
    float pre_g = 0.f, pre_b = 0.f;
    int pre_slot = -1;
    auto fetch = [&](int tb) {   // branch-free: tokens past the batch re-read its last token
        const int nb = min(kTokBatch, len - tb);
        const int64_t tq = tok0 + tb + min(jq, nb - 1), tv = tok0 + tb + min(jv, nb - 1);
        pre_q = *reinterpret_cast<const vq_t *>(p.q + tq * p.q_st + hk * p.q_sh + cq);
        pre_k = *reinterpret_cast<const vq_t *>(p.k + tq * p.k_st + hk * p.k_sh + cq);
        pre_v = *reinterpret_cast<const vv_t *>(p.v + tv * p.v_st + h * p.v_sh + cv);
        if (p.gk) pre_gk = *reinterpret_cast<const fq_t *>(p.gk + tq * p.gk_st + h * p.gk_sh + cq);
        if (tid <= kTokBatch) {
            // entry nb is the look-ahead slot of the token after the batch (or -1 at the end of the sequence)
            const int64_t t = tok0 + tb + min(tid, tb + nb < len ? nb : nb - 1);
            pre_slot = p.slot_idx[t];
            if (tid == nb && tb + nb >= len) pre_slot = -1;
            const int64_t tg = tok0 + tb + min(tid, nb - 1);
            if (p.g) pre_g = p.g[tg * p.g_st + h * p.g_sh];
            pre_b = (float)p.beta[tg * p.b_st + h * p.b_sh];
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int e = 0; e < EQ; ++e) {
            s_k[buf][jq][cq + e] = (float)pre_k[e];
            s_q[buf][jq][cq + e] = (float)pre_q[e] * p.scale;
            if (p.gk) s_gk[buf][jq][cq + e] = __expf(pre_gk[e]);
        }
#pragma unroll
        for (int e = 0; e < EV; ++e) s_v[buf][jv][cv + e] = (float)pre_v[e];
        if (tid <= kTokBatch) {
            s_slot[buf][tid] = pre_slot;
            if (tid < kTokBatch) {
                s_decay[buf][tid] = p.g ? __expf(pre_g) : 1.f;
                s_beta[buf][tid] = pre_b;
            }
        }
    };
    fetch(0);
    commit(0);
    __syncthreads();

    for (int tb = 0, buf = 0; tb < len; tb += kTokBatch, buf ^= 1) {
        const int nb = min(kTokBatch, len - tb);
        if (tb + kTokBatch < len) fetch(tb + kTokBatch);
        for (int j = 0; j < nb; ++j) {
            f32x4 kv[NSEG], qv[NSEG], dec[NSEG];
#pragma unroll
            for (int sg = 0; sg < NSEG; ++sg) {
                kv[sg] = *reinterpret_cast<const f32x4 *>(&s_k[buf][j][col + SEGW * sg]);
                qv[sg] = *reinterpret_cast<const f32x4 *>(&s_q[buf][j][col + SEGW * sg]);
                dec[sg] = f32x4{s_decay[buf][j], s_decay[buf][j], s_decay[buf][j], s_decay[buf][j]};
                if (p.gk) dec[sg] *= *reinterpret_cast<const f32x4 *>(&s_gk[buf][j][col + SEGW * sg]);
            }
            const float beta = s_beta[buf][j];
            float sk[NP];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                float a = 0.f;
#pragma unroll
                for (int sg = 0; sg < NSEG; ++sg) {
                    S[i][sg] *= dec[sg];
                    a += S[i][sg][0] * kv[sg][0] + S[i][sg][1] * kv[sg][1] + S[i][sg][2] * kv[sg][2] + S[i][sg][3] * kv[sg][3];
                }
                sk[i] = a;
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) sk[i] = group_sum<LPR>(sk[i]);
            float so[NP];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const float delta = beta * (s_v[buf][j][i * RPP + row0] - sk[i]);
                float a = 0.f;
#pragma unroll
                for (int sg = 0; sg < NSEG; ++sg) {
                    S[i][sg] += delta * kv[sg];
                    a += S[i][sg][0] * qv[sg][0] + S[i][sg][1] * qv[sg][1] + S[i][sg][2] * qv[sg][2] + S[i][sg][3] * qv[sg][3];
                }
                so[i] = a;
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) so[i] = group_sum<LPR>(so[i]);
            if (lane % LPR == 0) {
#pragma unroll
                for (int i = 0; i < NP; ++i) s_o[j][i * RPP + row0] = so[i];
            }
            // the state is visible after every token; a write is redundant only when the
            // next token of this sequence targets the same slot
            const int slot = s_slot[buf][j];
            if (slot != s_slot[buf][j + 1] && slot >= 0 && slot < p.n_blocks) {
                ST *dp = state + slot * p.s_sb + h * p.s_sh + col;
#pragma unroll
                for (int i = 0; i < NP; ++i)
#pragma unroll
                    for (int sg = 0; sg < NSEG; ++sg)
                        StateIO<ST>::store(dp + (int64_t)(i * RPP + row0) * p.s_sv + SEGW * sg, S[i][sg]);
            }
        }
        __syncthreads();   // s_o complete, this half fully consumed
        if (jv < nb) {
            vv_t ov;
#pragma unroll
            for (int e = 0; e < EV; ++e) ov[e] = (bf16)s_o[jv][cv + e];
            *reinterpret_cast<vv_t *>(p.out + (int64_t)(tok0 + tb + jv) * p.o_st + h * p.o_sh + cv) = ov;
        }
        if (tb + kTokBatch < len) commit(buf ^ 1);
        __syncthreads();   // next half staged, s_o free again
    }
}

// Any head size up to 512 x 512 with Dk a multiple of 4: the rows of the state are independent recurrences
// (row v needs only S[v,:], k_t, q_t, v_t[v]), so the workgroup takes 16 rows at a time through all tokens of the
// sequence, a row spread over one 16-lane DPP row in 16-byte pieces 64 columns apart, as in the sized kernel.
// The state still moves once in and out per slot change; q, k and the gates are re-read for every 16 rows.
template <typename ST>
__global__ void __launch_bounds__(kThreads) recurrent_gdn_anysize_kernel(const RecParams p, int Dk, int Dv) {
    constexpr int MAXSEG = 8;                 // 512 columns
    __shared__ int s_red[kThreads / kWave];
    const int n = blockIdx.x / p.Nv, h = blockIdx.x % p.Nv;
    const int hk = h / (p.Nv / p.Nk);
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int col = (lane % 16) * 4, rw = wave * 4 + lane / 16;

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
    if (len <= 0 || tok0 + len > p.T) return;
    int src_tok = tok0;
    if (p.accepted) src_tok = tok0 + p.accepted[n] - 1;
    if (src_tok < 0 || src_tok >= p.T) return;
    const int src_slot = p.slot_idx[src_tok];
    if (src_slot < 0 || src_slot >= p.n_blocks) return;

    ST *state = static_cast<ST *>(p.state);
    const int nseg = (Dk + 63) / 64;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    for (int r0 = 0; r0 < Dv; r0 += 16) {
        const int row = r0 + rw;
        const bool row_ok = row < Dv;
        f32x4 S[MAXSEG];
#pragma unroll
        for (int sg = 0; sg < MAXSEG; ++sg) {
            const int c = col + 64 * sg;
            S[sg] = zero;
            if (sg < nseg && row_ok && c < Dk) S[sg] = StateIO<ST>::load(state + src_slot * p.s_sb + h * p.s_sh + (int64_t)row * p.s_sv + c);
        }
        for (int j = 0; j < len; ++j) {
            const int64_t tok = tok0 + j;
            const float decay = p.g ? __expf(p.g[tok * p.g_st + h * p.g_sh]) : 1.f;
            const float beta = (float)p.beta[tok * p.b_st + h * p.b_sh];
            const float vt = row_ok ? (float)p.v[tok * p.v_st + h * p.v_sh + row] : 0.f;
            f32x4 kv[MAXSEG], qv[MAXSEG];
            float sk = 0.f;
#pragma unroll
            for (int sg = 0; sg < MAXSEG; ++sg) {
                const int c = col + 64 * sg;
                kv[sg] = zero;
                qv[sg] = zero;
                if (sg < nseg && c < Dk) {
                    const bf16x4 k4 = *reinterpret_cast<const bf16x4 *>(p.k + tok * p.k_st + hk * p.k_sh + c);
                    const bf16x4 q4 = *reinterpret_cast<const bf16x4 *>(p.q + tok * p.q_st + hk * p.q_sh + c);
                    f32x4 dec = {decay, decay, decay, decay};
                    if (p.gk) {
                        const f32x4 g4 = *reinterpret_cast<const f32x4 *>(p.gk + tok * p.gk_st + h * p.gk_sh + c);
#pragma unroll
                        for (int e = 0; e < 4; ++e) dec[e] *= __expf(g4[e]);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        kv[sg][e] = (float)k4[e];
                        qv[sg][e] = (float)q4[e] * p.scale;
                    }
                    S[sg] *= dec;
                    sk += S[sg][0] * kv[sg][0] + S[sg][1] * kv[sg][1] + S[sg][2] * kv[sg][2] + S[sg][3] * kv[sg][3];
                }
            }
            const float delta = beta * (vt - group_sum<16>(sk));
            float so = 0.f;
#pragma unroll
            for (int sg = 0; sg < MAXSEG; ++sg) {
                if (sg < nseg) {
                    S[sg] += delta * kv[sg];
                    so += S[sg][0] * qv[sg][0] + S[sg][1] * qv[sg][1] + S[sg][2] * qv[sg][2] + S[sg][3] * qv[sg][3];
                }
            }
            so = group_sum<16>(so);
            if (lane % 16 == 0 && row_ok) p.out[tok * p.o_st + h * p.o_sh + row] = (bf16)so;
            const int slot = p.slot_idx[tok];
            const int next = j + 1 < len ? p.slot_idx[tok + 1] : -1;
            if (slot != next && slot >= 0 && slot < p.n_blocks && row_ok) {
#pragma unroll
                for (int sg = 0; sg < MAXSEG; ++sg) {
                    const int c = col + 64 * sg;
                    if (sg < nseg && c < Dk) StateIO<ST>::store(state + slot * p.s_sb + h * p.s_sh + (int64_t)row * p.s_sv + c, S[sg]);
                }
            }
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
    // four head sizes have a kernel that keeps the whole state tile in registers; every other one up to the
    // reference's 512 x 512 (torch_custom/fla_npu/fla_npu/ops/ascendc/_aclnn_ctypes.py:813-817) takes the row-block kernel
    const bool sized = (Dk == 128 && Dv == 128) || (Dk == 64 && Dv == 64) || (Dk == 128 && Dv == 256) ||
                       (Dk == 64 && Dv == 128);
    FLA_REQUIRE(Dk >= 1 && Dv >= 1 && Dk <= 512 && Dv <= 512, FLA_ERR_SHAPE, "%s: Dk and Dv must be <= 512, got Dk=%lld, Dv=%lld.",
                op, (long long)Dk, (long long)Dv);
    FLA_REQUIRE(sized || Dk % 4 == 0, FLA_ERR_UNSUPPORTED, "%s: Dk must be a multiple of 4, got %lld.", op, (long long)Dk);
    FLA_REQUIRE(B * Nv < ((int64_t)1 << 31) && T < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents exceed int32.", op);
    if (query_ws) {
        *query_ws = 0;
        return FLA_OK;
    }
    if (T == 0 || B == 0) return FLA_OK;

    if (!sized) {   // 8-byte pieces of q and k, 16-byte pieces of gk, scalar v and out
        const fla_tensor *vec[] = {query, key};
        for (const fla_tensor *t : vec)
            FLA_REQUIRE(t->stride[0] % 4 == 0 && t->stride[1] % 4 == 0 && reinterpret_cast<uintptr_t>(t->data) % 8 == 0,
                        FLA_ERR_SHAPE, "%s: query/key rows must be 8-byte aligned.", op);
        if (has_gk)
            FLA_REQUIRE(gk->stride[0] % 4 == 0 && gk->stride[1] % 4 == 0 && reinterpret_cast<uintptr_t>(gk->data) % 16 == 0,
                        FLA_ERR_SHAPE, "%s: gk rows must be 16-byte aligned.", op);
    } else {
        // the per-batch staging reads q, k, v, gk and writes out in 16-byte pieces at most
        const fla_tensor *vec[] = {query, key, value, out};
        for (const fla_tensor *t : vec)
            FLA_REQUIRE(t->stride[2] == 1 && t->stride[0] % 8 == 0 && t->stride[1] % 8 == 0 &&
                            reinterpret_cast<uintptr_t>(t->data) % 16 == 0,
                        FLA_ERR_SHAPE, "%s: query/key/value/out rows must be contiguous and 16-byte aligned.", op);
        if (has_gk)
            FLA_REQUIRE(gk->stride[2] == 1 && gk->stride[0] % 4 == 0 && gk->stride[1] % 4 == 0 &&
                            reinterpret_cast<uintptr_t>(gk->data) % 16 == 0,
                        FLA_ERR_SHAPE, "%s: gk rows must be contiguous and 16-byte aligned.", op);
    }
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
    // single-token decode is a pure stream of the state: widest rows per load; longer sequences are bound by
    // the per-token reductions: 16-lane rows
    const bool one_token = T <= B;
#define FLA_LAUNCH_REC(DK, DV)                                                                                       \
    if (one_token) {                                                                                                 \
        if (f32s) FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_kernel<float, DK, DV, DK / 4>), grid, block, 0, stream, p); \
        else FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_kernel<bf16, DK, DV, DK / 4>), grid, block, 0, stream, p);       \
    } else {                                                                                                         \
        if (f32s) FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_kernel<float, DK, DV, 16>), grid, block, 0, stream, p);     \
        else FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_kernel<bf16, DK, DV, 16>), grid, block, 0, stream, p);           \
    }
    if (!sized) {
        if (f32s) FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_anysize_kernel<float>), grid, block, 0, stream, p, (int)Dk, (int)Dv);
        else FLA_LAUNCH("recurrent_gdn", stream, (recurrent_gdn_anysize_kernel<bf16>), grid, block, 0, stream, p, (int)Dk, (int)Dv);
    } else if (Dk == 128 && Dv == 128) { FLA_LAUNCH_REC(128, 128); }
    else if (Dk == 64 && Dv == 64) { FLA_LAUNCH_REC(64, 64); }
    else if (Dk == 128 && Dv == 256) { FLA_LAUNCH_REC(128, 256); }
    else { FLA_LAUNCH_REC(64, 128); }
#undef FLA_LAUNCH_REC
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

// -------------------------------------------------------------------------------------------------
// Plan for running the sequences of a call on the chunk kernels: whether every sequence keeps ONE pool row (the
// row its first token names) that no other sequence uses, which row that is, and the lengths for the host.
// One workgroup per sequence; every workgroup scans the (short) list of lengths for its own offsets.
// -------------------------------------------------------------------------------------------------
constexpr int kPlanMaxSeqs = 8192;

__global__ void __launch_bounds__(kThreads) prefill_plan_kernel(const int32_t *lens, const int32_t *idx, int batch, int64_t total,
                                                                int pool_rows, int32_t *slots, int32_t *report) {
    __shared__ int32_t startS[kPlanMaxSeqs + 1];   // token offset of every sequence (capped at total + 1), then the end of the last
    __shared__ int64_t partS[kThreads];
    __shared__ int badS;
    const int tid = threadIdx.x, i = blockIdx.x;
    const int per = (batch + kThreads - 1) / kThreads;
    int64_t sum = 0;
    bool negative = false;
    for (int j = tid * per; j < min(batch, (tid + 1) * per); ++j) {
        const int n = lens[1 + j];
        negative |= n < 0;
        sum += max(n, 0);
    }
    partS[tid] = sum;
    if (tid == 0) badS = 0;
    __syncthreads();
    int64_t off = lens[0];
    for (int t = 0; t < tid; ++t) off += partS[t];
    for (int j = tid * per; j < min(batch, (tid + 1) * per); ++j) {
        startS[j] = (int32_t)min(off, total + 1);
        off += max(lens[1 + j], 0);
    }
    if ((tid + 1) * per >= batch) startS[batch] = (int32_t)min(off, total + 1);   // every such thread holds the same end
    __syncthreads();
    const int64_t start = startS[i], end = startS[i + 1];
    const int len = lens[1 + i];
    bool bad = negative || lens[0] < 0 || startS[batch] > total;
    int slot = -1;
    if (!__syncthreads_or(bad) && len > 0) {
        slot = idx[start];
        if (slot < 0 || slot >= pool_rows) bad = true;
        for (int64_t t = start + tid; t < end; t += kThreads) bad |= idx[t] != slot;          // one row for the whole sequence
        for (int j = tid; j < batch; j += kThreads)                                            // and for no other one
            if (j != i && lens[1 + j] > 0 && idx[startS[j]] == slot) bad = true;
    }
    if (bad) badS = 1;
    __syncthreads();
    if (tid == 0) {
        slots[i] = badS ? -1 : slot;
        report[1 + i] = len;
        report[1 + batch + i] = badS;
        if (i == 0) report[0] = lens[0];
    }
}

int prefill_plan_impl(const fla_tensor *actual_seq_lengths, const fla_tensor *ssm_state_indices, int64_t pool_rows,
                      const fla_tensor *slots, const fla_tensor *report, hipStream_t stream) {
    const char *op = "recurrent_gdn_prefill_plan";
    int rc;
    const int i32 = dt_bit(FLA_I32);
    if ((rc = check_tensor(actual_seq_lengths, op, "actual_seq_lengths", 1, i32))) return rc;
    if ((rc = check_tensor(ssm_state_indices, op, "ssm_state_indices", 1, i32))) return rc;
    if ((rc = check_tensor(slots, op, "slots", 1, i32))) return rc;
    if ((rc = check_tensor(report, op, "report", 1, i32))) return rc;
    const int64_t batch = actual_seq_lengths->shape[0] - 1;
    FLA_REQUIRE(batch >= 1 && batch <= kPlanMaxSeqs, FLA_ERR_UNSUPPORTED, "%s: between 1 and %d sequences, got %lld.", op,
                kPlanMaxSeqs, (long long)batch);
    FLA_REQUIRE(pool_rows >= 1 && pool_rows <= INT32_MAX, FLA_ERR_SHAPE, "%s: pool_rows out of range.", op);
    FLA_REQUIRE(ssm_state_indices->shape[0] < INT32_MAX, FLA_ERR_SHAPE, "%s: too many tokens.", op);
    const fla_tensor *flat[] = {actual_seq_lengths, ssm_state_indices, slots, report};
    for (const fla_tensor *t : flat)
        FLA_REQUIRE(t->shape[0] <= 1 || t->stride[0] == 1, FLA_ERR_SHAPE, "%s: the index tensors must be contiguous.", op);
    FLA_REQUIRE(slots->shape[0] == batch && report->shape[0] == 2 * batch + 1, FLA_ERR_SHAPE,
                "%s: slots must be int32 [B] and report int32 [2B+1].", op);
    FLA_LAUNCH("recurrent_gdn_prefill_plan", stream, prefill_plan_kernel, dim3((unsigned)batch), dim3(kThreads), 0, stream,
               static_cast<const int32_t *>(actual_seq_lengths->data), static_cast<const int32_t *>(ssm_state_indices->data),
               (int)batch, ssm_state_indices->shape[0], (int)pool_rows, static_cast<int32_t *>(slots->data),
               static_cast<int32_t *>(report->data));
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
    return fla::guarded([&] { return fla::rec_impl(query, key, value, beta, state, actual_seq_lengths, ssm_state_indices, g, gk,
                         num_accepted_tokens, scale, out, nullptr, 0, nullptr, workspace_size); });
}

extern "C" int fla_recurrent_gated_delta_rule(
    const fla_tensor *query, const fla_tensor *key, const fla_tensor *value, const fla_tensor *beta,
    const fla_tensor *state, const fla_tensor *actual_seq_lengths, const fla_tensor *ssm_state_indices,
    const fla_tensor *g, const fla_tensor *gk, const fla_tensor *num_accepted_tokens, float scale,
    const fla_tensor *out, void *workspace, uint64_t workspace_size, void *stream) {
    return fla::guarded([&] { return fla::rec_impl(query, key, value, beta, state, actual_seq_lengths, ssm_state_indices, g, gk,
                         num_accepted_tokens, scale, out, workspace, workspace_size, static_cast<hipStream_t>(stream),
                         nullptr); });
}

extern "C" int fla_recurrent_gdn_prefill_plan(const fla_tensor *actual_seq_lengths, const fla_tensor *ssm_state_indices,
                                              int64_t pool_rows, const fla_tensor *slots, const fla_tensor *report, void *stream) {
    return fla::guarded([&] { return fla::prefill_plan_impl(actual_seq_lengths, ssm_state_indices, pool_rows, slots, report,
                                                            static_cast<hipStream_t>(stream)); });
}
