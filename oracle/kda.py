"""CPU oracle (test infrastructure) for the KDA (per-channel gated delta rule) path.

Head-major op layout: ``q, k [B,Hk,T,K]``, ``v [B,Hv,T,V]``, ``g / gk [B,Hv,T,K]``,
``beta [B,Hv,T]``.  ``gk`` is the chunk-local cumulative gate in log2 units
(``gk = chunk_cumsum(gate) / ln 2``), decays are ``2**gk``.

Reference statements followed:
  gate activation + cumsum   fla/ops/ascendc/kda/chunk_kda_fwd/docs/api.md:103-113,
                             kda_gate_cumsum/op_kernel/kda_gate_cumsum_kernel.h:384-419,516-534
  chunk forward              tests/atk/chunk_kda_fwd/executor_chunk_kda_fwd.py:316-530
  bwd_dhu                    torch_custom/fla_npu/test/test_bwd_dhu.py:61-290 and
                             chunk_gated_delta_rule_bwd_dhu_design.md:81-182 (terminal gradient dht and
                             the [N,Hv,K,V] dh0 follow the design note; the reference kernel drops dht)
  bwd_intra                  torch_custom/fla_npu/test/test_npu_chunk_kda_bwd_intra.py:7-91
The acceptance oracle for the forward is the per-token recurrence below; the chunked
restatement must agree with it (tests/test_oracle.py).
"""
from __future__ import annotations

import math

import torch

from .gdn import _cu_list, _round, chunk_spans, total_chunks

LN2 = math.log(2.0)
RCP_LN2 = 1.4426950408889634


def kda_gate(g, *, A_log=None, dt_bias=None, use_gate_in_kernel=False, safe_gate=False, lower_bound=-5.0):
    """Per-channel log decay (natural log) from the raw gate input ``g [B,Hv,T,K]``."""
    gf = g.float()
    if not use_gate_in_kernel:
        return gf
    Hv, K = g.shape[1], g.shape[3]
    eig = torch.exp(A_log.float()).view(1, Hv, 1, 1)
    raw = gf if dt_bias is None else gf + dt_bias.float().view(1, Hv, 1, K)
    if safe_gate:
        return float(lower_bound) * torch.sigmoid(eig * raw)
    sp = torch.clamp(raw, min=0.0) + torch.log1p(torch.exp(-raw.abs()))   # stable softplus
    return -eig * sp


def kda_gate_cumsum(g, chunk: int, *, A_log=None, dt_bias=None, cu_seqlens=None, use_gate_in_kernel=False,
                    safe_gate=False, lower_bound=-5.0):
    """gk [B,Hv,T,K] fp32 = chunk-local cumulative sum of the activated gate, in log2 units."""
    gate = kda_gate(g, A_log=A_log, dt_bias=dt_bias, use_gate_in_kernel=use_gate_in_kernel, safe_gate=safe_gate,
                    lower_bound=lower_bound)
    out = torch.empty_like(gate)
    B, T = g.shape[0], g.shape[2]
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        acc = torch.zeros_like(gate[b, :, 0])
        for t in range(s, e):
            acc = acc + gate[b, :, t]
            out[b, :, t] = acc * RCP_LN2
    return out


def naive_recurrent_kda(q, k, v, gate, beta, scale=None, *, initial_state=None, output_final_state=False,
                        cu_seqlens=None, compute_dtype=torch.float32):
    """Token-by-token KDA: S <- diag(e^{gate_t}) S ; delta = beta_t (v_t - S^T k_t) ; S <- S + k_t delta^T ;
    o_t = scale S^T q_t.   ``gate`` is the per-channel natural-log decay [B,Hv,T,K]."""
    B, Hk, T, K = q.shape
    Hv, V = v.shape[1], v.shape[3]
    rep = Hv // Hk
    if scale is None:
        scale = K ** -0.5
    cu = _cu_list(cu_seqlens)
    spans = [(b, b, 0, T) for b in range(B)] if cu is None else [(0, n, s, e) for n, (s, e) in enumerate(zip(cu, cu[1:]))]
    qf = q.to(compute_dtype).repeat_interleave(rep, dim=1)
    kf = k.to(compute_dtype).repeat_interleave(rep, dim=1)
    vf, gf, bf = v.to(compute_dtype), gate.to(compute_dtype), beta.to(compute_dtype)
    o = torch.zeros(B, Hv, T, V, dtype=compute_dtype)
    final = torch.zeros(len(spans), Hv, K, V, dtype=compute_dtype)
    for b, n, s, e in spans:
        S = torch.zeros(Hv, K, V, dtype=compute_dtype) if initial_state is None else \
            initial_state[n].to(compute_dtype).clone()
        for t in range(s, e):
            S = S * torch.exp(gf[b, :, t])[:, :, None]
            kt = kf[b, :, t]
            delta = (vf[b, :, t] - torch.einsum("hkv,hk->hv", S, kt)) * bf[b, :, t, None]
            S = S + kt[:, :, None] * delta[:, None, :]
            o[b, :, t] = torch.einsum("hkv,hk->hv", S, qf[b, :, t]) * scale
        final[n] = S
    return o, (final if output_final_state else None)


def chunk_kda_fwd(q, k, v, gk, beta, scale, chunk: int = 64, *, initial_state=None, output_final_state=False,
                  cu_seqlens=None, compute_dtype=torch.float32, lowp=None):
    """Chunked KDA forward from the cumulated log2 gate ``gk``.  Returns a dict with
    o [B,Hv,T,V], final_state, Aqk, Akk [B,Hv,T,C], w, u, qg, kg, v_new, h [B,Hv,NT,K,V]."""
    B, Hk, T, K = q.shape
    Hv, V = v.shape[1], v.shape[3]
    rep = Hv // Hk
    cu = _cu_list(cu_seqlens)
    N = B if cu is None else len(cu) - 1
    NT = total_chunks(B, T, chunk, cu)
    cd = compute_dtype
    qf, kf, vf, gf, bf = (x.to(cd) for x in (q, k, v, gk, beta))
    out = dict(o=torch.zeros(B, Hv, T, V, dtype=cd), Aqk=torch.zeros(B, Hv, T, chunk, dtype=cd),
               Akk=torch.zeros(B, Hv, T, chunk, dtype=cd), w=torch.zeros(B, Hv, T, K, dtype=cd),
               u=torch.zeros(B, Hv, T, V, dtype=cd), qg=torch.zeros(B, Hv, T, K, dtype=cd),
               kg=torch.zeros(B, Hv, T, K, dtype=cd), v_new=torch.zeros(B, Hv, T, V, dtype=cd),
               h=torch.zeros(B, Hv, NT, K, V, dtype=cd))
    state = torch.zeros(N, Hv, K, V, dtype=cd) if initial_state is None else initial_state.to(cd).clone()
    for b, n, ci, s, e in chunk_spans(B, T, chunk, cu):
        L = e - s
        qc = qf[b, :, s:e].repeat_interleave(rep, dim=0)
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        vc, gc, bc = vf[b, :, s:e], gf[b, :, s:e], bf[b, :, s:e]
        # scores with the pairwise decay 2^{gk_i - gk_j} per channel, evaluated through an anchor per
        # 16-row tile so that both factors stay finite (executor_chunk_kda_fwd.py:373-399)
        qk = torch.zeros(Hv, L, L, dtype=cd)
        kk = torch.zeros(Hv, L, L, dtype=cd)
        for r0 in range(0, L, 16):
            r1 = min(r0 + 16, L)
            shift = gc[:, r1 - 1:r1]
            left = torch.exp2(gc[:, r0:r1] - shift)
            right = _round(kc[:, :r1] * torch.exp2(shift - gc[:, :r1]), lowp)
            qk[:, r0:r1, :r1] = torch.matmul(_round(qc[:, r0:r1] * left, lowp), right.transpose(1, 2)) * scale
            kk[:, r0:r1, :r1] = torch.matmul(_round(kc[:, r0:r1] * left, lowp), right.transpose(1, 2))
        Aqk = torch.tril(qk)
        A0 = torch.tril(kk * bc[:, :, None], -1)
        eye = torch.eye(L, dtype=cd)
        Akk = torch.linalg.solve_triangular(A0 + eye, eye.expand(Hv, -1, -1), upper=False)
        eg = torch.exp2(gc)
        w = torch.matmul(_round(Akk, lowp), _round(kc * bc[..., None] * eg, lowp))
        u = torch.matmul(_round(Akk, lowp), _round(vc * bc[..., None], lowp))
        glast = gc[:, -1]
        kg = kc * torch.exp2(glast[:, None, :] - gc)
        qg = qc * eg
        S = state[n]
        vn = u - torch.matmul(_round(w, lowp), _round(S, lowp))
        o = torch.matmul(_round(qg, lowp), _round(S, lowp)) * scale + torch.matmul(_round(Aqk, lowp), _round(vn, lowp))
        out["h"][b, :, ci] = S
        state[n] = torch.exp2(glast)[:, :, None] * S + torch.matmul(_round(kg, lowp).transpose(1, 2), _round(vn, lowp))
        out["o"][b, :, s:e] = o
        out["Aqk"][b, :, s:e, :L] = Aqk
        out["Akk"][b, :, s:e, :L] = Akk
        for name, val in (("w", w), ("u", u), ("qg", qg), ("kg", kg), ("v_new", vn)):
            out[name][b, :, s:e] = val
    out["final_state"] = state.float() if output_final_state else None
    return out


def chunk_gated_delta_rule_bwd_dhu(q, k, w, do, dv, scale, chunk: int = 64, *, g=None, gK=None, dht=None,
                                   cu_seqlens=None, compute_dtype=torch.float32):
    """Reverse chunk scan.  Exactly one of g [B,Hv,T] (natural log, scalar gate) and gK [B,Hv,T,K]
    (log2, per-channel gate; q and k must then already carry their gates).  Returns
    (dh [B,Hv,NT,K,V] = gradient of the state at each chunk END seen from later chunks,
     dh0 [N,Hv,K,V] = gradient of the initial state, dv2 [B,Hv,T,V])."""
    assert (g is None) != (gK is None)
    B, Hk, T, K = q.shape
    Hv, V = do.shape[1], do.shape[3]
    rep = Hv // Hk
    cu = _cu_list(cu_seqlens)
    N = B if cu is None else len(cu) - 1
    NT = total_chunks(B, T, chunk, cu)
    cd = compute_dtype
    qf, kf, wf, dof, dvf = (x.to(cd) for x in (q, k, w, do, dv))
    dh = torch.zeros(B, Hv, NT, K, V, dtype=cd)
    dv2 = torch.zeros(B, Hv, T, V, dtype=cd)
    state = torch.zeros(N, Hv, K, V, dtype=cd) if dht is None else dht.to(cd).clone()
    for b, n, ci, s, e in reversed(list(chunk_spans(B, T, chunk, cu))):
        bdh = state[n]
        dh[b, :, ci] = bdh
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        qc = qf[b, :, s:e].repeat_interleave(rep, dim=0)
        bdv = torch.matmul(kc, bdh)                                     # [Hv, L, V]
        if g is not None:
            gc = g[b, :, s:e].to(cd)
            bdv = bdv * torch.exp(gc[:, -1:] - gc)[..., None]
            qc = qc * torch.exp(gc)[..., None]
            decay = torch.exp(gc[:, -1])[:, None, None]
        else:
            decay = torch.exp2(gK[b, :, e - 1].to(cd))[:, :, None]
        bdv = bdv + dvf[b, :, s:e]
        dv2[b, :, s:e] = bdv
        state[n] = bdh * decay + scale * torch.matmul(qc.transpose(1, 2), dof[b, :, s:e]) \
            - torch.matmul(wf[b, :, s:e].transpose(1, 2), bdv)
    return dh, state, dv2


def chunk_kda_bwd_intra(q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, *, chunk: int = 64, cu_seqlens=None,
                        compute_dtype=torch.float64):
    """Adds the intra-chunk terms to dq, dk, db, dg (head-major layouts [B,H,T,K] / [B,H,T]):
        dq_i += sum_{j<=i} dAqk_ij k_j 2^{g_i-g_j}
        dl_i  = sum_{j<=i} dAkk_ij k_j 2^{g_i-g_j}
        du_j  = sum_{i>=j} (dAqk_ij q_i + dAkk_ij beta_i k_i) 2^{g_i-g_j}
        dk_i += beta_i dl_i + du_i ; db_i += <dl_i, k_i> ; dg_i += q_i dq'_i + k_i (beta_i dl_i - du_i)
    evaluated directly (no anchors) in ``compute_dtype``; the reference's anchored 16-row tiling is the same
    sum reassociated."""
    cd = compute_dtype
    B, H, T, K = q.shape
    qf, kf, gf, bf = (x.to(cd) for x in (q, k, gk, beta))
    dq_o, dk_o, db_o, dg_o = (x.to(cd).clone() for x in (dq, dk, db, dg))
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        qc, kc, gc, bc = qf[b, :, s:e], kf[b, :, s:e], gf[b, :, s:e], bf[b, :, s:e]
        aq = torch.tril(dAqk[b, :, s:e, :L].to(cd))
        ak = torch.tril(dAkk[b, :, s:e, :L].to(cd))
        dec = torch.exp2(gc[:, :, None, :] - gc[:, None, :, :])          # [H, i, j, K] = 2^{g_i - g_j}
        mask = torch.tril(torch.ones(L, L, dtype=torch.bool))[None, :, :, None]
        dec = torch.where(mask, dec, torch.zeros((), dtype=cd))
        dq_delta = torch.einsum("hij,hijk,hjk->hik", aq, dec, kc)
        dl = torch.einsum("hij,hijk,hjk->hik", ak, dec, kc)
        du = torch.einsum("hij,hijk,hik->hjk", aq, dec, qc) + torch.einsum("hij,hijk,hik->hjk", ak, dec, kc * bc[..., None])
        bdl = bc[..., None] * dl
        dq_o[b, :, s:e] += dq_delta
        dk_o[b, :, s:e] += bdl + du
        db_o[b, :, s:e] += (dl * kc).sum(-1)
        dg_o[b, :, s:e] += qc * dq_delta + kc * (bdl - du)
    return dq_o, dk_o, db_o, dg_o


def recurrent_kda(q, k, v, g, beta, initial_state, *, cu_seqlens=None, ssm_state_indices=None, A_log=None, dt_bias=None,
                  num_accepted_tokens=None, layout="BSND", scale=None, use_qk_l2norm_in_kernel=False,
                  use_gate_in_kernel=False, use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, safe_gate=False,
                  lower_bound=-5.0, state_v_first=False, compute_dtype=torch.float32):
    """Decode / speculative-decode KDA over a state pool (kda/recurrent_kda/docs/design.md:47-78,155-166 and
    op_kernel/recurrent_kda.h:270-366,836-870).  Token-major operands: BSND ``q,k [B,T,H,K]``, ``v [B,T,HV,V]``,
    ``g [B,T,HV,K]``, ``beta [B,T,HV]`` (TND: without B).  ``initial_state`` is the pool ``[capacity,HV,V,K]``
    (``state_v_first``) or ``[capacity,HV,K,V]``.  Sequence i covers tokens cu[i]..cu[i+1]; it starts from the pool
    slot of its token ``accepted_i - 1`` (token 0 without ``num_accepted_tokens``; slot i without indices) and
    after every token the state is stored in that token's slot.  Returns (out, pool after the call)."""
    tnd = layout == "TND"
    flat = lambda t: t if tnd else t.reshape(-1, *t.shape[2:])
    qf, kf, vf, gf, bf = (flat(t).to(compute_dtype) for t in (q, k, v, g, beta))
    T, H, K = qf.shape
    HV, V = vf.shape[1], vf.shape[2]
    rep = HV // H
    if scale is None:
        scale = K ** -0.5
    if use_qk_l2norm_in_kernel:
        nq, nk = qf.norm(dim=-1, keepdim=True), kf.norm(dim=-1, keepdim=True)
        qf = torch.where(nq > 0, qf / nq, qf)
        kf = torch.where(nk > 0, kf / nk, kf)
    if use_gate_in_kernel:
        eig = torch.exp(A_log.to(compute_dtype)).view(1, HV, 1)
        raw = gf if dt_bias is None else gf + dt_bias.to(compute_dtype).reshape(1, HV, K)
        if safe_gate:
            gf = float(lower_bound) * torch.sigmoid(eig * raw)
        else:
            gf = -eig * torch.nn.functional.softplus(raw)
    if use_beta_sigmoid_in_kernel:
        bf = torch.sigmoid(bf)
        if allow_neg_eigval:
            bf = 2.0 * bf
    if cu_seqlens is None:
        S_len = T if tnd else q.shape[1]
        cu = list(range(0, T + 1, S_len))
    else:
        cu = [int(x) for x in cu_seqlens]
    pool = initial_state.clone()
    out = torch.zeros(T, HV, V, dtype=compute_dtype)
    idx = None if ssm_state_indices is None else ssm_state_indices
    for n, (s, e) in enumerate(zip(cu, cu[1:])):
        if e <= s:
            continue
        def slot_of(t):
            if idx is None:
                return n
            return int(idx[n, t - s]) if idx.dim() == 2 else int(idx[t])
        src = s if num_accepted_tokens is None else s + int(num_accepted_tokens[n]) - 1
        st = initial_state[slot_of(src)].to(compute_dtype)
        S = st.clone() if state_v_first else st.transpose(-1, -2).clone()          # [HV, V, K]
        for t in range(s, e):
            S = S * torch.exp(gf[t])[:, None, :]
            kt = kf[t].repeat_interleave(rep, dim=0)                               # [HV, K]
            delta = bf[t][:, None] * (vf[t] - torch.einsum("hvk,hk->hv", S, kt))
            S = S + delta[:, :, None] * kt[:, None, :]
            out[t] = torch.einsum("hvk,hk->hv", S, qf[t].repeat_interleave(rep, dim=0) * scale)
            pool[slot_of(t)] = (S if state_v_first else S.transpose(-1, -2)).to(pool.dtype)
    out = out.to(v.dtype)
    return (out if tnd else out.reshape(v.shape)), pool


# ---------------------------------------------------------------------------------------------
# KDA chunk backward.  The reference ships only two of its stages (bwd_dhu with gK and chunk_kda_bwd_intra); the
# rest of the chain lives in a third-party Triton package it patches around
# (torch_custom/fla_npu/fla_npu/adapters/triton_ascend_kda.py:1-8).  The three stages below are this build's own
# decomposition of the remaining work; each is the exact derivative of the forward stage it names and is pinned
# against torch autograd of that stage, the composition against autograd through naive_recurrent_kda
# (tests/test_oracle.py).  "dg" everywhere is the gradient with respect to the cumulated gate in natural-log
# units per step (dL/dgk / ln 2): a reverse chunk-local cumulative sum of it is the gradient of the per-token gate.
# ---------------------------------------------------------------------------------------------
def chunk_kda_bwd_dav(v_new, do, Aqk, scale, chunk: int = 64, *, cu_seqlens=None, compute_dtype=torch.float32):
    """Derivative of  o_intra = Aqk v_new,  Aqk = scale * tril(score):
        dAqk = scale * tril(do v_new^T)   (gradient of the unscaled score, what chunk_kda_bwd_intra consumes)
        dv   = Aqk^T do                   (first part of the gradient of v_new)."""
    cd = compute_dtype
    B, Hv, T, V = do.shape
    dA = torch.zeros(B, Hv, T, chunk, dtype=cd)
    dv = torch.zeros(B, Hv, T, V, dtype=cd)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        doc, vc = do[b, :, s:e].to(cd), v_new[b, :, s:e].to(cd)
        dA[b, :, s:e, :L] = torch.tril(torch.matmul(doc, vc.transpose(1, 2))) * scale
        dv[b, :, s:e] = torch.matmul(torch.tril(Aqk[b, :, s:e, :L].to(cd)).transpose(1, 2), doc)
    return dA, dv


def chunk_kda_bwd_dqkwg(q, k, v_new, gk, h, do, dh, dv, scale, chunk: int = 64, *, cu_seqlens=None,
                        compute_dtype=torch.float32):
    """Derivative of the parts of a chunk step that see the carried state:
        o_inter = scale (q 2^g) h ;  v_new = u - w h ;  h' = diag(2^{g_last}) h + (k 2^{g_last - g})^T v_new
    given do, dh = dL/dh' and dv = total dL/dv_new.  h, dh: [B,Hv,NT,K,V].  Returns per VALUE head
        dq = scale (do h^T) 2^g ;  dk = (v_new dh^T) 2^{g_last - g} ;  dw = -dv h^T ;
        dg = q dq - k dk, plus on the chunk's last token  sum_j k_j dk_j + 2^{g_last} rowsum(h . dh)."""
    cd = compute_dtype
    B, Hk, T, K = q.shape
    Hv = do.shape[1]
    rep = Hv // Hk
    dq = torch.zeros(B, Hv, T, K, dtype=cd)
    dk, dw, dg = torch.zeros_like(dq), torch.zeros_like(dq), torch.zeros_like(dq)
    for b, _, ci, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        qc = q[b, :, s:e].to(cd).repeat_interleave(rep, dim=0)
        kc = k[b, :, s:e].to(cd).repeat_interleave(rep, dim=0)
        gc = gk[b, :, s:e].to(cd)
        hc, dhc = h[b, :, ci].to(cd), dh[b, :, ci].to(cd)
        glast = gc[:, -1:]
        bdq = torch.matmul(do[b, :, s:e].to(cd), hc.transpose(1, 2)) * scale * torch.exp2(gc)
        bdk = torch.matmul(v_new[b, :, s:e].to(cd), dhc.transpose(1, 2)) * torch.exp2(glast - gc)
        bdg = qc * bdq - kc * bdk
        bdg[:, -1] += (kc * bdk).sum(1) + torch.exp2(glast[:, 0]) * (hc * dhc).sum(-1)
        dq[b, :, s:e], dk[b, :, s:e], dg[b, :, s:e] = bdq, bdk, bdg
        dw[b, :, s:e] = -torch.matmul(dv[b, :, s:e].to(cd), hc.transpose(1, 2))
    return dq, dk, dw, dg


def chunk_kda_bwd_wy(k, v, beta, gk, Akk, dw, du, chunk: int = 64, *, cu_seqlens=None, compute_dtype=torch.float32):
    """Derivative of  w = Akk (k beta 2^g),  u = Akk (v beta),  Akk = (I + M)^-1  (M strictly lower):
        dM  = -stril(Akk^T (dw (k beta 2^g)^T + du (v beta)^T) Akk^T)    [B,Hv,T,C]
        x   = Akk^T dw ;  y = Akk^T du
        dk  = x beta 2^g ;  dv = y beta ;  dbeta = <x, k 2^g> + <y, v> ;  dg = dk k.
    Returns (dk, dv, dbeta, dg, dM) per value head."""
    cd = compute_dtype
    B, Hk, T, K = k.shape
    Hv, V = v.shape[1], v.shape[3]
    rep = Hv // Hk
    dk = torch.zeros(B, Hv, T, K, dtype=cd)
    dg = torch.zeros_like(dk)
    dv = torch.zeros(B, Hv, T, V, dtype=cd)
    db = torch.zeros(B, Hv, T, dtype=cd)
    dM = torch.zeros(B, Hv, T, chunk, dtype=cd)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        kc = k[b, :, s:e].to(cd).repeat_interleave(rep, dim=0)
        vc, bc, gc = v[b, :, s:e].to(cd), beta[b, :, s:e].to(cd), gk[b, :, s:e].to(cd)
        A = torch.tril(Akk[b, :, s:e, :L].to(cd))
        dwc, duc = dw[b, :, s:e].to(cd), du[b, :, s:e].to(cd)
        eg = torch.exp2(gc)
        kbg, vb = kc * bc[..., None] * eg, vc * bc[..., None]
        dA = torch.tril(torch.matmul(dwc, kbg.transpose(1, 2)) + torch.matmul(duc, vb.transpose(1, 2)), -1)
        At = A.transpose(1, 2)
        dM[b, :, s:e, :L] = -torch.tril(torch.matmul(torch.matmul(At, dA), At), -1)
        x, y = torch.matmul(At, dwc), torch.matmul(At, duc)
        dk[b, :, s:e] = x * bc[..., None] * eg
        dg[b, :, s:e] = dk[b, :, s:e] * kc
        dv[b, :, s:e] = y * bc[..., None]
        db[b, :, s:e] = (x * kc * eg).sum(-1) + (y * vc).sum(-1)
    return dk, dv, db, dg, dM


def chunk_kda_bwd(q, k, v, gate, beta, scale, do, *, chunk: int = 64, initial_state=None, dht=None, cu_seqlens=None,
                  compute_dtype=torch.float32):
    """Whole KDA chunk backward from the per-token natural-log gate: forward intermediates recomputed with
    chunk_kda_fwd, then dav -> bwd_dhu (gK) -> dqkwg -> wy -> bwd_intra -> reverse chunk-local cumsum.
    Head-major operands; returns (dq, dk [B,Hk,T,K], dv [B,Hv,T,V], dg [B,Hv,T,K], dbeta [B,Hv,T], dh0 [N,Hv,K,V])."""
    cd = compute_dtype
    B, Hk, T, K = q.shape
    Hv = v.shape[1]
    rep = Hv // Hk
    gk = torch.empty(B, Hv, T, K, dtype=cd)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        gk[b, :, s:e] = torch.cumsum(gate[b, :, s:e].to(cd), dim=1) * RCP_LN2
    f = chunk_kda_fwd(q, k, v, gk, beta, scale, chunk, initial_state=initial_state, cu_seqlens=cu_seqlens,
                      compute_dtype=cd)
    dAqk, dv0 = chunk_kda_bwd_dav(f["v_new"], do, f["Aqk"], scale, chunk, cu_seqlens=cu_seqlens, compute_dtype=cd)
    dh, dh0, dv2 = chunk_gated_delta_rule_bwd_dhu(f["qg"], f["kg"], f["w"], do, dv0, scale, chunk, gK=gk, dht=dht,
                                                  cu_seqlens=cu_seqlens, compute_dtype=cd)
    dq, dk, dw, dg = chunk_kda_bwd_dqkwg(q, k, f["v_new"], gk, f["h"], do, dh, dv2, scale, chunk,
                                         cu_seqlens=cu_seqlens, compute_dtype=cd)
    dk2, dv, db, dg2, dM = chunk_kda_bwd_wy(k, v, beta, gk, f["Akk"], dw, dv2, chunk, cu_seqlens=cu_seqlens,
                                            compute_dtype=cd)
    qe = q.to(cd).repeat_interleave(rep, dim=1)
    ke = k.to(cd).repeat_interleave(rep, dim=1)
    dq, dk, db, dg = chunk_kda_bwd_intra(qe, ke, gk, beta, dAqk, dM, dq, dk + dk2, db, dg + dg2, chunk=chunk,
                                         cu_seqlens=cu_seqlens, compute_dtype=cd)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        dg[b, :, s:e] = torch.flip(torch.cumsum(torch.flip(dg[b, :, s:e], dims=[1]), dim=1), dims=[1])
    dq = dq.view(B, Hk, rep, T, K).sum(2)
    dk = dk.view(B, Hk, rep, T, K).sum(2)
    return dq, dk, dv, dg, db, dh0
