"""CPU oracle (test infrastructure) for the gated-delta-rule chunk BACKWARD chain.

Never imported by the shipped package: only tests, the smoke check and the CPU
leg of the benchmark may use it.

Layouts are head-first like the forward oracle: ``q, k [B, Hk, T, K]``,
``v, do, dv, du [B, Hv, T, V]``, ``w, dw [B, Hv, T, K]``, ``g, beta [B, Hv, T]``
(``g`` already chunk-cumsummed), chunk matrices ``A, dA [B, Hv, T, C]``, per-chunk
states ``h, dh [B, Hv, NT, K, V]``.

Reference statements followed:
  chunk_bwd_dv_local        torch_custom/fla_npu/test/golden.py:18-88 (dense), :90-172 (varlen)
  chunk_bwd_dqkwg           tests/atk/chunk_bwd_dqkwg/scripts/chunk_bwd_dqkwg_cpu.py:67-409
  prepare_wy_repr_bwd_da    torch_custom/fla_npu/test/test_npu_prepare_wy_repr_bwd_da.py:170-282
  prepare_wy_repr_bwd_full  torch_custom/fla_npu/test/test_npu_prepare_wy_repr_bwd_full.py:46-486
  composition               examples/flash_gated_delta_rule.py:884-1008

The exchanged ``dA`` follows the reference convention: it is the TRANSPOSE of the
gradient of the strictly-lower chunk matrix (bwd_da stores ``b_dA.T``, bwd_full reads
``dA_chunk.T`` wherever the upstream Triton kernel reads ``b_dA``).

Pins (tests/test_oracle.py): every function is checked against torch autograd of the
forward stage it differentiates, and the whole composition against autograd through
the per-token recurrence, all in fp64.
"""
from __future__ import annotations

import torch

from .gdn import (_cu_list, chunk_gated_delta_rule_fwd_h, chunk_local_cumsum, chunk_scaled_dot_kkt, chunk_spans,
                  recompute_w_u_fwd, solve_tri, total_chunks)
from .kda import chunk_gated_delta_rule_bwd_dhu


def chunk_bwd_dv_local(q, k, do, g, scale, chunk: int = 64, *, cu_seqlens=None, compute_dtype=torch.float32,
                       output_dtype=None):
    """dv[i] = sum_{j >= i} scale * <k_i, q_j> * exp(g_j - g_i) * do[j] within each chunk."""
    B, Hk, T, K = q.shape
    Hv = do.shape[1]
    rep = Hv // Hk
    cd = compute_dtype
    qf, kf, dof, gf = (x.to(cd) for x in (q, k, do, g))
    dv = torch.zeros_like(dof)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        qc = qf[b, :, s:e].repeat_interleave(rep, dim=0)
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        gc = gf[b, :, s:e]
        L = e - s
        upper = torch.triu(torch.ones(L, L, dtype=torch.bool))
        diff = torch.where(upper, gc[:, None, :] - gc[:, :, None], torch.zeros((), dtype=cd))   # g_j - g_i
        A = torch.where(upper, torch.matmul(kc, qc.transpose(-1, -2)) * torch.exp(diff) * scale,
                        torch.zeros((), dtype=cd))
        dv[b, :, s:e] = torch.matmul(A, dof[b, :, s:e])
    return dv.to(output_dtype if output_dtype is not None else do.dtype)


def chunk_bwd_dqkwg(q, k, v, g, h, do, dh, dv, scale, chunk: int = 64, *, cu_seqlens=None,
                    compute_dtype=torch.float32, output_dtype=None):
    """``v`` is v_new of the forward scan, ``h`` the state at each chunk start, ``dh`` the gradient of the
    state at each chunk end, ``dv`` the gradient of v_new.  Returns (dq, dk [B,Hk,T,K], dw [B,Hv,T,K],
    dg [B,Hv,T] fp32); dq and dk are summed over the value heads that share a key head."""
    B, Hk, T, K = q.shape
    Hv, V = v.shape[1], v.shape[3]
    rep = Hv // Hk
    cd = compute_dtype
    qf, kf, vf, gf, hf, dof, dhf, dvf = (x.to(cd) for x in (q, k, v, g, h, do, dh, dv))
    dq = torch.zeros(B, Hv, T, K, dtype=cd)
    dk = torch.zeros(B, Hv, T, K, dtype=cd)
    dw = torch.zeros(B, Hv, T, K, dtype=cd)
    dg = torch.zeros(B, Hv, T, dtype=cd)
    for b, _, ci, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        qc = qf[b, :, s:e].repeat_interleave(rep, dim=0)
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        vc, doc, dvc, gc = vf[b, :, s:e], dof[b, :, s:e], dvf[b, :, s:e], gf[b, :, s:e]
        hp, dhc = hf[b, :, ci], dhf[b, :, ci]                                   # [Hv, K, V]
        g_last = gc[:, -1]
        dq_state = torch.matmul(doc, hp.transpose(-1, -2)) * torch.exp(gc)[..., None] * scale
        dk_state = torch.matmul(vc, dhc.transpose(-1, -2)) * torch.exp(g_last[:, None] - gc)[..., None]
        dw[b, :, s:e] = -torch.matmul(dvc, hp.transpose(-1, -2))
        dg_last = (hp * dhc).sum(dim=(-1, -2)) * torch.exp(g_last) + (dk_state * kc).sum(dim=(-1, -2))
        dgc = (dq_state * qc).sum(-1) - (kc * dk_state).sum(-1)
        lower = torch.tril(torch.ones(L, L, dtype=torch.bool))
        diff = torch.where(lower, gc[:, :, None] - gc[:, None, :], torch.zeros((), dtype=cd))   # g_i - g_j
        ds = torch.where(lower, torch.matmul(doc, vc.transpose(-1, -2)) * torch.exp(diff), torch.zeros((), dtype=cd)) * scale
        ds2 = ds * torch.matmul(qc, kc.transpose(-1, -2))
        dgc = dgc + ds2.sum(-1) - ds2.sum(-2)
        dgc[:, L - 1] += dg_last
        dg[b, :, s:e] = dgc
        dq[b, :, s:e] = dq_state + torch.matmul(ds, kc)
        dk[b, :, s:e] = dk_state + torch.matmul(ds.transpose(-1, -2), qc)
    od = output_dtype if output_dtype is not None else q.dtype
    dq = dq.view(B, Hk, rep, T, K).sum(2)
    dk = dk.view(B, Hk, rep, T, K).sum(2)
    return dq.to(od), dk.to(od), dw.to(od), dg.float() if cd == torch.float32 else dg


def prepare_wy_repr_bwd_da(k, v, beta, A, dw, du, g, chunk: int = 64, *, cu_seqlens=None,
                           compute_dtype=torch.float32, output_dtype=None):
    """Gradient of the strictly-lower chunk matrix, stored transposed (reference convention)."""
    B, Hk, T, K = k.shape
    Hv = v.shape[1]
    rep = Hv // Hk
    cd = compute_dtype
    kf, vf, bf, Af, dwf, duf, gf = (x.to(cd) for x in (k, v, beta, A, dw, du, g))
    dA = torch.zeros(B, Hv, T, chunk, dtype=cd)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        gc, bc = gf[b, :, s:e], bf[b, :, s:e]
        a = Af[b, :, s:e, :L]
        strict = torch.tril(torch.ones(L, L, dtype=torch.bool), -1)
        m = torch.matmul(dwf[b, :, s:e], (kc * (bc * torch.exp(gc))[..., None]).transpose(-1, -2)) \
            + torch.matmul(duf[b, :, s:e], (vf[b, :, s:e] * bc[..., None]).transpose(-1, -2))
        m = torch.where(strict, m, torch.zeros((), dtype=cd))
        m = torch.matmul(a.transpose(-1, -2), torch.matmul(m, a.transpose(-1, -2)))
        diff = torch.where(strict, gc[:, :, None] - gc[:, None, :], torch.zeros((), dtype=cd))
        m = torch.where(strict, -m * torch.exp(diff), torch.zeros((), dtype=cd))
        dA[b, :, s:e, :L] = m.transpose(-1, -2)
    return dA.to(output_dtype if output_dtype is not None else A.dtype)


def prepare_wy_repr_bwd_full(k, v, beta, A, dA, dw, du, g, chunk: int = 64, *, cu_seqlens=None,
                             compute_dtype=torch.float32, output_dtype=None):
    """Returns (dk [B,Hk,T,K], dv [B,Hv,T,V], dbeta [B,Hv,T], dg [B,Hv,T]); ``dA`` as written by bwd_da."""
    B, Hk, T, K = k.shape
    Hv, V = v.shape[1], v.shape[3]
    rep = Hv // Hk
    cd = compute_dtype
    kf, vf, bf, Af, dAf, dwf, duf, gf = (x.to(cd) for x in (k, v, beta, A, dA, dw, du, g))
    dk = torch.zeros(B, Hv, T, K, dtype=cd)
    dv = torch.zeros(B, Hv, T, V, dtype=cd)
    db = torch.zeros(B, Hv, T, dtype=cd)
    dg = torch.zeros(B, Hv, T, dtype=cd)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        vc, gc, bc = vf[b, :, s:e], gf[b, :, s:e], bf[b, :, s:e]
        a, d = Af[b, :, s:e, :L], dAf[b, :, s:e, :L]
        eg = torch.exp(gc)
        dv_beta = torch.matmul(a.transpose(-1, -2), duf[b, :, s:e])            # A^T du
        dk_beta_g = torch.matmul(a.transpose(-1, -2), dwf[b, :, s:e])          # A^T dw
        dk_beta = torch.matmul(d.transpose(-1, -2), kc)                        # dA^T k
        dv[b, :, s:e] = dv_beta * bc[..., None]
        dk[b, :, s:e] = torch.matmul(d, kc * bc[..., None]) + dk_beta * bc[..., None] \
            + dk_beta_g * (bc * eg)[..., None]
        db[b, :, s:e] = (dk_beta * kc).sum(-1) + (dk_beta_g * kc * eg[..., None]).sum(-1) + (dv_beta * vc).sum(-1)
        bA = torch.matmul(kc, kc.transpose(-1, -2)) * bc[..., None]
        dA_A = d.transpose(-1, -2) * bA
        dg[b, :, s:e] = (dk_beta_g * kc * (bc * eg)[..., None]).sum(-1) + dA_A.sum(-1) - dA_A.sum(-2)
    od = output_dtype if output_dtype is not None else k.dtype
    dk = dk.view(B, Hk, rep, T, K).sum(2)
    return dk.to(od), dv.to(od), db.to(beta.dtype if cd == torch.float32 else cd), \
        dg.to(g.dtype if cd == torch.float32 else cd)


def chunk_gated_delta_rule_bwd(q, k, v, g, beta, scale, do, *, initial_state=None, dht=None, chunk: int = 64,
                               cu_seqlens=None, compute_dtype=torch.float32):
    """The reference's composition of the backward operators.  ``g`` is the RAW per-token log gate
    [B,Hv,T]; returns (dq, dk, dv, dbeta, dg, dh0) with dg the gradient of the raw gate and dh0
    [N,Hv,K,V] (None without an initial state)."""
    cd = compute_dtype
    kw = dict(cu_seqlens=cu_seqlens)
    G = chunk_local_cumsum(g, chunk, output_dtype=cd, **kw)
    A0 = chunk_scaled_dot_kkt(k, G, beta, chunk, compute_dtype=cd, **kw).to(cd)
    A = solve_tri(A0, compute_dtype=cd, output_dtype=cd, **kw)
    w, u = recompute_w_u_fwd(k, v, beta, A, chunk, g=G, compute_dtype=cd, output_dtype=cd, **kw)
    h, v_new, _ = chunk_gated_delta_rule_fwd_h(k, w, u, G, initial_state=initial_state, chunk=chunk,
                                               compute_dtype=cd, output_dtype=cd, **kw)
    dv = chunk_bwd_dv_local(q, k, do, G, scale, chunk, compute_dtype=cd, output_dtype=cd, **kw)
    dh, dh0, dv = chunk_gated_delta_rule_bwd_dhu(q, k, w, do, dv, scale, chunk, g=G, dht=dht, compute_dtype=cd, **kw)
    dq, dk, dw, dg = chunk_bwd_dqkwg(q, k, v_new, G, h, do, dh, dv, scale, chunk, compute_dtype=cd, output_dtype=cd, **kw)
    dA = prepare_wy_repr_bwd_da(k, v, beta, A, dw, dv, G, chunk, compute_dtype=cd, output_dtype=cd, **kw)
    dk2, dv, db, dg2 = prepare_wy_repr_bwd_full(k, v, beta, A, dA, dw, dv, G, chunk, compute_dtype=cd,
                                                output_dtype=cd, **kw)
    dg = chunk_local_cumsum((dg.to(cd) + dg2.to(cd)), chunk, reverse=True, output_dtype=cd, **kw)
    return dq, dk + dk2, dv, db, dg, (dh0 if initial_state is not None else None)
