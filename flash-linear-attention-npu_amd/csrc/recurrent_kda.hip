// recurrent_kda: token-by-token KDA (per-channel gated delta rule) for decode and speculative decoding, with
// the gate activation, q/k L2 normalisation and beta sigmoid optionally done in the kernel.
//
//   S <- S diag(e^{gate_t}) ; delta = beta_t (v_t - S k_t) ; S <- S + delta k_t^T ; o_t = S (scale q_t)
//
// with S kept as [V, K] (one row per value channel).  Bandwidth-bound: the state tile of a (sequence, value
// head) is streamed in once, stays in registers over the tokens of the sequence, and is written to the slot of
// every token whose successor uses a different slot (speculative decoding keeps one state per draft token).
// One 256-thread workgroup owns one (sequence, value head); a state row is spread over the 16 lanes of one
// DPP row, so the two reductions per token are four data-parallel-primitive adds each.  A K-first state pool
// ([slot, Hv, K, V]) is transposed through LDS on the way in and out.
// Semantics: kda/recurrent_kda/docs/design.md:47-78,155-166; op_kernel/recurrent_kda.h:270-366 (sequence and slot
// resolution), :416-470 (normalisation, gate), :796-806 (beta), :836-870 (per-token state store).
#include "common.h"
#include "device_utils.h"
#include "kda_common.h"

namespace fla {
namespace {

constexpr int kThreads = 256;
constexpr int kTokBatch = 8;   // tokens staged per synchronisation
constexpr int kLPR = 16;       // lanes per state row

struct KdaRecParams {
    const bf16 *q, *k, *v;
    const void *g, *beta;
    const void *state_in;
    void *state_out;
    const void *cu, *slots, *accepted;   // device index tensors (int32 or int64) or null
    const float *A_log, *dt_bias;
    bf16 *out;
    int64_t q_st, q_sh, v_st, v_sh, g_st, g_sh, b_st, b_sh, o_st, o_sh;
    int64_t si_sb, si_sh, si_sr, so_sb, so_sh, so_sr;   // state strides: slot, head, row (elements)
    int g_dt, beta_dt, cu64, slots64, acc64;   // dtypes: 0 f32, 1 bf16, 2 f16; index width flags
    int slot_stride;                           // 0: packed per token; > 0: [sequence, step]
    int T, N, S_dense, Nk, Nv, capacity;
    int l2norm, use_gate, safe, beta_sigmoid, neg_eig, store_state;
    float scale, lower_bound;
};

__device__ __forceinline__ int64_t ld_index(const void *p, int is64, int64_t i) {
    return is64 ? static_cast<const int64_t *>(p)[i] : (int64_t) static_cast<const int32_t *>(p)[i];
}
__device__ __forceinline__ float ld_scalar(const void *p, int dt, int64_t i) {
    if (dt == 0) return static_cast<const float *>(p)[i];
    if (dt == 1) return (float)static_cast<const bf16 *>(p)[i];
    return (float)static_cast<const f16 *>(p)[i];
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

template <typename ST> __device__ __forceinline__ f32x4 ld_state4(const ST *p);
template <> __device__ __forceinline__ f32x4 ld_state4<float>(const float *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(p));
}
template <> __device__ __forceinline__ f32x4 ld_state4<bf16>(const bf16 *p) {
    const bf16x4 r = *reinterpret_cast<const bf16x4 *>(p);
    return f32x4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
}
template <typename ST> __device__ __forceinline__ void st_state4(ST *p, f32x4 v);
template <> __device__ __forceinline__ void st_state4<float>(float *p, f32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p));
}
template <> __device__ __forceinline__ void st_state4<bf16>(bf16 *p, f32x4 v) { *reinterpret_cast<bf16x4 *>(p) = cvt4(v); }

template <typename ST, int DK, int DV, bool VFIRST>
__global__ void __launch_bounds__(kThreads) recurrent_kda_kernel(const KdaRecParams p) {
    constexpr int SEGW = 4 * kLPR, NSEG = DK / SEGW, RPW = kWave / kLPR, RPP = RPW * (kThreads / kWave), NP = DV / RPP;
    constexpr int TP = DV + 4;   // pitch of the transposition tile (K-first pools only)
    static_assert(DK % SEGW == 0 && DV % RPP == 0, "tile does not divide");
    extern __shared__ __align__(16) float s_tile[];   // [DK][TP] when !VFIRST
    __shared__ __align__(16) float s_k[kTokBatch][DK], s_q[kTokBatch][DK], s_dec[kTokBatch][DK];
    __shared__ __align__(16) float s_v[kTokBatch][DV], s_o[kTokBatch][DV];
    __shared__ float s_beta[kTokBatch];
    __shared__ int s_slot[kTokBatch + 1];

    const int n = blockIdx.x / p.Nv, h = blockIdx.x % p.Nv;
    const int hk = h / (p.Nv / p.Nk);
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int col = (lane % kLPR) * 4, row0 = wave * RPW + lane / kLPR;

    int64_t seq0, seq1;
    if (p.cu) {
        seq0 = ld_index(p.cu, p.cu64, n);
        seq1 = ld_index(p.cu, p.cu64, n + 1);
    } else {
        seq0 = (int64_t)n * p.S_dense;
        seq1 = seq0 + p.S_dense;
    }
    const int len = (int)(seq1 - seq0);
    if (seq0 < 0 || len <= 0 || seq1 > p.T) return;   // empty sequence or invalid metadata: nothing is touched
    auto slot_of = [&](int64_t tok) -> int64_t {
        if (!p.slots) return n;
        const int64_t at = p.slot_stride ? (int64_t)n * p.slot_stride + (tok - seq0) : tok;
        return ld_index(p.slots, p.slots64, at);
    };
    if (p.slots && p.slot_stride && len > p.slot_stride) return;
    int64_t src_tok = seq0;
    if (p.slots && p.accepted) {
        const int64_t acc = ld_index(p.accepted, p.acc64, n);
        if (acc <= 0 || acc > len) return;
        src_tok = seq0 + acc - 1;
    }
    const int64_t src_slot = slot_of(src_tok);
    if (src_slot < 0 || src_slot >= p.capacity) return;

    f32x4 S[NP][NSEG];
    const ST *sin = static_cast<const ST *>(p.state_in) + src_slot * p.si_sb + h * p.si_sh;
    if (VFIRST) {
#pragma unroll
        for (int i = 0; i < NP; ++i)
#pragma unroll
            for (int sg = 0; sg < NSEG; ++sg) S[i][sg] = ld_state4<ST>(sin + (int64_t)(i * RPP + row0) * p.si_sr + col + SEGW * sg);
    } else {
        for (int idx = tid; idx < DK * DV / 4; idx += kThreads) {
            const int kk = idx / (DV / 4), v4 = (idx % (DV / 4)) * 4;
            *reinterpret_cast<f32x4 *>(&s_tile[kk * TP + v4]) = ld_state4<ST>(sin + (int64_t)kk * p.si_sr + v4);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NP; ++i)
#pragma unroll
            for (int sg = 0; sg < NSEG; ++sg)
#pragma unroll
                for (int e = 0; e < 4; ++e) S[i][sg][e] = s_tile[(col + SEGW * sg + e) * TP + i * RPP + row0];
        __syncthreads();
    }
    ST *sout = static_cast<ST *>(p.state_out);
    auto store_state = [&](int64_t slot) {   // called by every thread of the block (uniform slot)
        ST *dp = sout + slot * p.so_sb + h * p.so_sh;
        if (VFIRST) {
#pragma unroll
            for (int i = 0; i < NP; ++i)
#pragma unroll
                for (int sg = 0; sg < NSEG; ++sg) st_state4<ST>(dp + (int64_t)(i * RPP + row0) * p.so_sr + col + SEGW * sg, S[i][sg]);
        } else {
            __syncthreads();
#pragma unroll
            for (int i = 0; i < NP; ++i)
#pragma unroll
                for (int sg = 0; sg < NSEG; ++sg)
#pragma unroll
                    for (int e = 0; e < 4; ++e) s_tile[(col + SEGW * sg + e) * TP + i * RPP + row0] = S[i][sg][e];
            __syncthreads();
            for (int idx = tid; idx < DK * DV / 4; idx += kThreads) {
                const int kk = idx / (DV / 4), v4 = (idx % (DV / 4)) * 4;
                st_state4<ST>(dp + (int64_t)kk * p.so_sr + v4, *reinterpret_cast<const f32x4 *>(&s_tile[kk * TP + v4]));
            }
        }
    };

    const float eig = (p.use_gate && p.A_log) ? __expf(p.A_log[h]) : 1.f;
    for (int tb = 0; tb < len; tb += kTokBatch) {
        const int nb = min(kTokBatch, len - tb);
        // ---- stage the batch: wave w prepares tokens w and w + 4 ---------------------------------------
        for (int j = wave; j < nb; j += kThreads / kWave) {
            const int64_t t = seq0 + tb + j;
            float qv[DK / kWave], kv[DK / kWave], qq = 0.f, kk2 = 0.f;
#pragma unroll
            for (int e = 0; e < DK / kWave; ++e) {
                const int c = lane + kWave * e;
                qv[e] = (float)p.q[t * p.q_st + hk * p.q_sh + c];
                kv[e] = (float)p.k[t * p.q_st + hk * p.q_sh + c];
                qq += qv[e] * qv[e];
                kk2 += kv[e] * kv[e];
                float gate = ld_scalar(p.g, p.g_dt, t * p.g_st + h * p.g_sh + c);
                if (p.use_gate) gate = kda_activate(gate, p.dt_bias ? p.dt_bias[h * DK + c] : 0.f, eig, p.safe, p.lower_bound);
                s_dec[j][c] = __expf(gate);
            }
            float qs = p.scale, ks = 1.f;
            if (p.l2norm) {
                const float nq = sqrtf(wave_sum(qq)), nk = sqrtf(wave_sum(kk2));
                if (nq > 0.f) qs /= nq;
                if (nk > 0.f) ks /= nk;
            }
#pragma unroll
            for (int e = 0; e < DK / kWave; ++e) {
                s_q[j][lane + kWave * e] = qv[e] * qs;
                s_k[j][lane + kWave * e] = kv[e] * ks;
            }
#pragma unroll
            for (int e = 0; e < DV / kWave; ++e) s_v[j][lane + kWave * e] = (float)p.v[t * p.v_st + h * p.v_sh + lane + kWave * e];
            if (lane == 0) {
                float b = ld_scalar(p.beta, p.beta_dt, t * p.b_st + h * p.b_sh);
                if (p.beta_sigmoid) {
                    b = 1.f / (1.f + __expf(-b));
                    if (p.neg_eig) b *= 2.f;
                }
                s_beta[j] = b;
                s_slot[j] = (int)slot_of(t);
                if (j == nb - 1) s_slot[nb] = tb + nb < len ? (int)slot_of(t + 1) : -1;
            }
        }
        __syncthreads();
        for (int j = 0; j < nb; ++j) {
            f32x4 kv[NSEG], qv[NSEG];
#pragma unroll
            for (int sg = 0; sg < NSEG; ++sg) {
                kv[sg] = *reinterpret_cast<const f32x4 *>(&s_k[j][col + SEGW * sg]);
                qv[sg] = *reinterpret_cast<const f32x4 *>(&s_q[j][col + SEGW * sg]);
            }
            const float beta = s_beta[j];
            float sk[NP], so[NP];
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                float a = 0.f;
#pragma unroll
                for (int sg = 0; sg < NSEG; ++sg) {
                    S[i][sg] *= *reinterpret_cast<const f32x4 *>(&s_dec[j][col + SEGW * sg]);
                    a += S[i][sg][0] * kv[sg][0] + S[i][sg][1] * kv[sg][1] + S[i][sg][2] * kv[sg][2] + S[i][sg][3] * kv[sg][3];
                }
                sk[i] = a;
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) sk[i] = group_sum<kLPR>(sk[i]);
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                const float delta = beta * (s_v[j][i * RPP + row0] - sk[i]);
                float a = 0.f;
#pragma unroll
                for (int sg = 0; sg < NSEG; ++sg) {
                    S[i][sg] += delta * kv[sg];
                    a += S[i][sg][0] * qv[sg][0] + S[i][sg][1] * qv[sg][1] + S[i][sg][2] * qv[sg][2] + S[i][sg][3] * qv[sg][3];
                }
                so[i] = a;
            }
#pragma unroll
            for (int i = 0; i < NP; ++i) so[i] = group_sum<kLPR>(so[i]);
            if (lane % kLPR == 0) {
#pragma unroll
                for (int i = 0; i < NP; ++i) s_o[j][i * RPP + row0] = so[i];
            }
            // the state is visible after every token; a store is redundant only when the next token of this
            // sequence writes the same slot
            const int slot = s_slot[j];
            if (p.store_state && slot != s_slot[j + 1] && slot >= 0 && slot < p.capacity) store_state(slot);
        }
        __syncthreads();   // s_o complete
        for (int idx = tid; idx < nb * DV; idx += kThreads) {
            const int j = idx / DV, c = idx % DV;
            p.out[(seq0 + tb + j) * p.o_st + h * p.o_sh + c] = (bf16)s_o[j][c];
        }
        __syncthreads();   // staging buffers free again
    }
}

// Copies a state pool [capacity, HV, rows, cols] between two views with dense rows (16-byte pieces).
__global__ void pool_copy_kernel(const char *src, char *dst, int64_t s_sb, int64_t s_sh, int64_t s_sr, int64_t d_sb, int64_t d_sh,
                                 int64_t d_sr, int HV, int rows, int pieces) {
    const int slot = blockIdx.x / HV, h = blockIdx.x % HV;
    const char *sp = src + slot * s_sb + h * s_sh;
    char *dp = dst + slot * d_sb + h * d_sh;
    for (int i = threadIdx.x; i < rows * pieces; i += blockDim.x) {
        const int r = i / pieces, c = i % pieces;
        *reinterpret_cast<u32x4 *>(dp + r * d_sr + c * 16) = *reinterpret_cast<const u32x4 *>(sp + r * s_sr + c * 16);
    }
}

inline bool present(const fla_tensor *t) { return t != nullptr && t->data != nullptr; }
int scalar_dt(int dt) { return dt == FLA_F32 ? 0 : (dt == FLA_BF16 ? 1 : 2); }

int rkda_impl(const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
              const fla_tensor *initial_state, const fla_tensor *cu_seqlens, const fla_tensor *ssm_state_indices,
              const fla_tensor *A_log, const fla_tensor *dt_bias, const fla_tensor *num_accepted_tokens, const char *layout,
              double scale, bool output_final_state, bool inplace_final_state, bool use_qk_l2norm, bool use_gate,
              bool use_beta_sigmoid, bool allow_neg_eigval, bool safe_gate, double lower_bound, bool state_v_first,
              const fla_tensor *attn_out, const fla_tensor *final_state, void *workspace, uint64_t workspace_size,
              hipStream_t stream, uint64_t *query_ws) {
    (void)workspace;
    (void)workspace_size;
    const char *op = "recurrent_kda";
    FLA_REQUIRE(layout != nullptr, FLA_ERR_NULL, "%s: layout must not be null.", op);
    const bool tnd = !strcmp(layout, "TND");
    FLA_REQUIRE(tnd || !strcmp(layout, "BSND"), FLA_ERR_UNSUPPORTED, "%s: layout must be BSND or TND.", op);
    const int rank = tnd ? 3 : 4;
    const int bf = dt_bit(FLA_BF16), any_f = bf | dt_bit(FLA_F32) | dt_bit(FLA_F16), idx = dt_bit(FLA_I32) | dt_bit(FLA_I64);
    int rc;
    if ((rc = check_tensor(q, op, "q", rank, bf))) return rc;
    if ((rc = check_tensor(k, op, "k", rank, bf))) return rc;
    if ((rc = check_tensor(v, op, "v", rank, bf))) return rc;
    if ((rc = check_tensor(g, op, "g", rank, any_f))) return rc;
    if ((rc = check_tensor(beta, op, "beta", rank - 1, any_f))) return rc;
    if ((rc = check_tensor(attn_out, op, "attn_out", rank, bf))) return rc;
    if ((rc = check_tensor(initial_state, op, "initial_state", 4, bf | dt_bit(FLA_F32)))) return rc;
    const int o = tnd ? 0 : 1;   // index of the token axis
    const int64_t B = tnd ? 1 : q->shape[0], S = q->shape[o], Nk = q->shape[o + 1], Dk = q->shape[o + 2];
    const int64_t Nv = v->shape[o + 1], Dv = v->shape[o + 2], T = B * S;
    FLA_REQUIRE(same_shape(q, k), FLA_ERR_SHAPE, "%s: q and k must have identical shape.", op);
    FLA_REQUIRE((tnd || v->shape[0] == B) && v->shape[o] == S && same_shape(attn_out, v), FLA_ERR_SHAPE, "%s: v/out shape mismatch.", op);
    FLA_REQUIRE((tnd || g->shape[0] == B) && g->shape[o] == S && g->shape[o + 1] == Nv && g->shape[o + 2] == Dk, FLA_ERR_SHAPE,
                "%s: g must be [..,T,HV,K].", op);
    FLA_REQUIRE((tnd || beta->shape[0] == B) && beta->shape[o] == S && beta->shape[o + 1] == Nv, FLA_ERR_SHAPE, "%s: beta must be [..,T,HV].", op);
    FLA_REQUIRE(Nk > 0 && Nv % Nk == 0, FLA_ERR_SHAPE, "%s: HV must be divisible by H.", op);
    FLA_REQUIRE(Dk == 128 && (Dv == 128 || Dv == 256), FLA_ERR_UNSUPPORTED, "%s: K/V support only K=128,V=128 or K=128,V=256.", op);
    // tokens are addressed by one flat index: the batch and token axes of a BSND operand must merge
    const fla_tensor *flat[] = {q, k, v, g, beta, attn_out};
    for (const fla_tensor *t : flat)
        FLA_REQUIRE(inner_unit(t) && (tnd || B == 1 || t->stride[0] == S * t->stride[1]), FLA_ERR_SHAPE,
                    "%s: operands must have unit innermost stride and mergeable batch/token axes.", op);
    FLA_REQUIRE(q->stride[o] == k->stride[o] && q->stride[o + 1] == k->stride[o + 1], FLA_ERR_SHAPE, "%s: q and k must share strides.", op);

    int64_t N = tnd ? 1 : B;
    if (present(cu_seqlens)) {
        if ((rc = check_tensor(cu_seqlens, op, "cu_seqlens", 1, idx))) return rc;
        FLA_REQUIRE(cu_seqlens->shape[0] >= 2 && is_contiguous(cu_seqlens), FLA_ERR_SHAPE, "%s: cu_seqlens must be a contiguous [seq_num+1].", op);
        N = cu_seqlens->shape[0] - 1;
    }
    const int64_t cap = initial_state->shape[0];
    const int64_t d2 = state_v_first ? Dv : Dk, d3 = state_v_first ? Dk : Dv;
    const fla_tensor *dst = inplace_final_state ? initial_state : final_state;
    const bool store = inplace_final_state || output_final_state;
    if (!inplace_final_state && store) {
        if ((rc = check_tensor(final_state, op, "final_state", 4, dt_bit(initial_state->dtype)))) return rc;
        FLA_REQUIRE(same_shape(final_state, initial_state), FLA_ERR_SHAPE, "%s: final_state must have the shape of initial_state.", op);
    }
    const fla_tensor *pools[] = {initial_state, store ? dst : initial_state};
    for (const fla_tensor *s : pools)
        FLA_REQUIRE(s->shape[1] == Nv && s->shape[2] == d2 && s->shape[3] == d3 && s->stride[3] == 1 && s->stride[2] % 4 == 0 &&
                        s->stride[1] % 4 == 0 && s->stride[0] % 4 == 0 && reinterpret_cast<uintptr_t>(s->data) % 16 == 0,
                    FLA_ERR_SHAPE, "%s: state must be %s with dense, 16-byte aligned rows.", op,
                    state_v_first ? "[state_capacity,HV,V,K]" : "[state_capacity,HV,K,V]");
    int slot_stride = 0;
    if (present(ssm_state_indices)) {
        if ((rc = check_tensor(ssm_state_indices, op, "ssm_state_indices", -1, idx))) return rc;
        const bool packed = ssm_state_indices->ndim == 1 && ssm_state_indices->shape[0] >= T;
        const bool spec = ssm_state_indices->ndim == 2 && ssm_state_indices->shape[0] == N && ssm_state_indices->shape[1] > 0;
        FLA_REQUIRE((packed || spec) && is_contiguous(ssm_state_indices), FLA_ERR_SHAPE,
                    "%s: ssm_state_indices must be packed [T] or speculative [seq_num,max_step].", op);
        slot_stride = spec ? (int)ssm_state_indices->shape[1] : 0;
    } else {
        FLA_REQUIRE(cap == N, FLA_ERR_SHAPE, "%s: without ssm_state_indices, state_capacity must equal seq_num.", op);
    }
    if (present(num_accepted_tokens)) {
        FLA_REQUIRE(present(ssm_state_indices), FLA_ERR_SHAPE, "%s: num_accepted_tokens requires ssm_state_indices.", op);
        if ((rc = check_tensor(num_accepted_tokens, op, "num_accepted_tokens", 1, idx))) return rc;
        FLA_REQUIRE(num_accepted_tokens->shape[0] == N && is_contiguous(num_accepted_tokens), FLA_ERR_SHAPE,
                    "%s: num_accepted_tokens must be [seq_num].", op);
    }
    if (use_gate) {
        if ((rc = check_tensor(A_log, op, "A_log", 1, dt_bit(FLA_F32)))) return rc;
        FLA_REQUIRE(A_log->shape[0] == Nv && is_contiguous(A_log), FLA_ERR_SHAPE, "%s: A_log must be FP32 [HV].", op);
        FLA_REQUIRE(!safe_gate || (lower_bound >= -5.0 && lower_bound < 0.0), FLA_ERR_SHAPE,
                    "%s: lower_bound must be in [-5,0) when safe_gate=True.", op);
        if (present(dt_bias)) {
            if ((rc = check_tensor(dt_bias, op, "dt_bias", -1, dt_bit(FLA_F32)))) return rc;
            FLA_REQUIRE(numel(dt_bias) == Nv * Dk && is_contiguous(dt_bias), FLA_ERR_SHAPE, "%s: dt_bias must be FP32 [HV*K] or [HV,K].", op);
        }
    } else {
        FLA_REQUIRE(!safe_gate && !present(A_log) && !present(dt_bias), FLA_ERR_SHAPE,
                    "%s: A_log, dt_bias and safe_gate require use_gate_in_kernel=True.", op);
    }
    FLA_REQUIRE(N * Nv < ((int64_t)1 << 31) && T < ((int64_t)1 << 31), FLA_ERR_SHAPE, "%s: extents exceed int32.", op);
    if (query_ws) {
        *query_ws = 0;
        return FLA_OK;
    }
    if (T == 0 || N == 0) return FLA_OK;

    KdaRecParams p{};
    p.q = static_cast<const bf16 *>(q->data);
    p.k = static_cast<const bf16 *>(k->data);
    p.v = static_cast<const bf16 *>(v->data);
    p.g = g->data;
    p.beta = beta->data;
    p.state_in = initial_state->data;
    p.state_out = store ? dst->data : nullptr;
    p.cu = present(cu_seqlens) ? cu_seqlens->data : nullptr;
    p.slots = present(ssm_state_indices) ? ssm_state_indices->data : nullptr;
    p.accepted = present(num_accepted_tokens) ? num_accepted_tokens->data : nullptr;
    p.A_log = use_gate ? static_cast<const float *>(A_log->data) : nullptr;
    p.dt_bias = (use_gate && present(dt_bias)) ? static_cast<const float *>(dt_bias->data) : nullptr;
    p.out = static_cast<bf16 *>(attn_out->data);
    p.q_st = q->stride[o]; p.q_sh = q->stride[o + 1];
    p.v_st = v->stride[o]; p.v_sh = v->stride[o + 1];
    p.g_st = g->stride[o]; p.g_sh = g->stride[o + 1];
    p.b_st = beta->stride[o]; p.b_sh = beta->stride[o + 1];
    p.o_st = attn_out->stride[o]; p.o_sh = attn_out->stride[o + 1];
    p.si_sb = initial_state->stride[0]; p.si_sh = initial_state->stride[1]; p.si_sr = initial_state->stride[2];
    if (store) { p.so_sb = dst->stride[0]; p.so_sh = dst->stride[1]; p.so_sr = dst->stride[2]; }
    p.g_dt = scalar_dt(g->dtype);
    p.beta_dt = scalar_dt(beta->dtype);
    p.cu64 = p.cu && cu_seqlens->dtype == FLA_I64;
    p.slots64 = p.slots && ssm_state_indices->dtype == FLA_I64;
    p.acc64 = p.accepted && num_accepted_tokens->dtype == FLA_I64;
    p.slot_stride = slot_stride;
    p.T = (int)T; p.N = (int)N; p.S_dense = (int)S; p.Nk = (int)Nk; p.Nv = (int)Nv; p.capacity = (int)cap;
    p.l2norm = use_qk_l2norm; p.use_gate = use_gate; p.safe = safe_gate; p.beta_sigmoid = use_beta_sigmoid;
    p.neg_eig = allow_neg_eigval; p.store_state = store;
    p.scale = (float)scale;
    p.lower_bound = (float)lower_bound;
    if (!inplace_final_state && store && final_state->data != initial_state->data) {
        // untouched slots of the separate output pool keep the input's contents
        const int64_t es = (int64_t)dtype_size(initial_state->dtype);
        FLA_REQUIRE((d3 * es) % 16 == 0, FLA_ERR_SHAPE, "%s: state rows must be a multiple of 16 bytes.", op);
        FLA_LAUNCH("recurrent_kda_pool_copy", stream, pool_copy_kernel, dim3((unsigned)(cap * Nv)), dim3(256), 0, stream,
                   static_cast<const char *>(initial_state->data), static_cast<char *>(final_state->data),
                   initial_state->stride[0] * es, initial_state->stride[1] * es, initial_state->stride[2] * es,
                   final_state->stride[0] * es, final_state->stride[1] * es, final_state->stride[2] * es, (int)Nv, (int)d2,
                   (int)(d3 * es / 16));
        FLA_HIP_CHECK(hipGetLastError());
    }
    const dim3 grid((unsigned)(N * Nv)), block(kThreads);
    const bool f32s = initial_state->dtype == FLA_F32;
#define FLA_LAUNCH_RKDA(DV_, VF)                                                                                                   \
    do {                                                                                                                           \
        const size_t smem = (VF) ? 0 : (size_t)128 * (DV_ + 4) * 4;                                                                \
        if (f32s) {                                                                                                                \
            if (smem) FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(recurrent_kda_kernel<float, 128, DV_, VF>), \
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));                   \
            FLA_LAUNCH("recurrent_kda", stream, (recurrent_kda_kernel<float, 128, DV_, VF>), grid, block, smem, stream, p);        \
        } else {                                                                                                                   \
            if (smem) FLA_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(recurrent_kda_kernel<bf16, 128, DV_, VF>),  \
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));                   \
            FLA_LAUNCH("recurrent_kda", stream, (recurrent_kda_kernel<bf16, 128, DV_, VF>), grid, block, smem, stream, p);         \
        }                                                                                                                          \
    } while (0)
    if (Dv == 128) {
        if (state_v_first) FLA_LAUNCH_RKDA(128, true);
        else FLA_LAUNCH_RKDA(128, false);
    } else {
        if (state_v_first) FLA_LAUNCH_RKDA(256, true);
        else FLA_LAUNCH_RKDA(256, false);
    }
#undef FLA_LAUNCH_RKDA
    FLA_HIP_CHECK(hipGetLastError());
    return FLA_OK;
}

}  // namespace
}  // namespace fla

extern "C" int fla_recurrent_kda_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
    const fla_tensor *initial_state, const fla_tensor *cu_seqlens, const fla_tensor *ssm_state_indices, const fla_tensor *A_log,
    const fla_tensor *dt_bias, const fla_tensor *num_accepted_tokens, const char *layout, double scale, bool output_final_state,
    bool inplace_final_state, bool use_qk_l2norm_in_kernel, bool use_gate_in_kernel, bool use_beta_sigmoid_in_kernel,
    bool allow_neg_eigval, bool safe_gate, double lower_bound, bool state_v_first, const fla_tensor *attn_out,
    const fla_tensor *final_state, uint64_t *workspace_size) {
    if (!workspace_size) return fla::fail(FLA_ERR_NULL, "recurrent_kda: workspace_size must not be null.");
    return fla::guarded([&] { return fla::rkda_impl(q, k, v, g, beta, initial_state, cu_seqlens, ssm_state_indices, A_log, dt_bias, num_accepted_tokens, layout,
                          scale, output_final_state, inplace_final_state, use_qk_l2norm_in_kernel, use_gate_in_kernel,
                          use_beta_sigmoid_in_kernel, allow_neg_eigval, safe_gate, lower_bound, state_v_first, attn_out,
                          final_state, nullptr, 0, nullptr, workspace_size); });
}
extern "C" int fla_recurrent_kda(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
    const fla_tensor *initial_state, const fla_tensor *cu_seqlens, const fla_tensor *ssm_state_indices, const fla_tensor *A_log,
    const fla_tensor *dt_bias, const fla_tensor *num_accepted_tokens, const char *layout, double scale, bool output_final_state,
    bool inplace_final_state, bool use_qk_l2norm_in_kernel, bool use_gate_in_kernel, bool use_beta_sigmoid_in_kernel,
    bool allow_neg_eigval, bool safe_gate, double lower_bound, bool state_v_first, const fla_tensor *attn_out,
    const fla_tensor *final_state, void *workspace, uint64_t workspace_size, void *stream) {
    return fla::guarded([&] { return fla::rkda_impl(q, k, v, g, beta, initial_state, cu_seqlens, ssm_state_indices, A_log, dt_bias, num_accepted_tokens, layout,
                          scale, output_final_state, inplace_final_state, use_qk_l2norm_in_kernel, use_gate_in_kernel,
                          use_beta_sigmoid_in_kernel, allow_neg_eigval, safe_gate, lower_bound, state_v_first, attn_out,
                          final_state, workspace, workspace_size, static_cast<hipStream_t>(stream), nullptr); });
}
