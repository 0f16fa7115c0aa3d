"""CPU oracle (test infrastructure) for the gated-delta-rule chunk forward path.

Op-level layout is head-first, as in the reference operator API:
``q, k [B, Hk, T, K]``, ``v, u, v_new, o [B, Hv, T, V]``, ``g, beta [B, Hv, T]``,
chunk matrices ``[B, Hv, T, C]``, per-chunk states ``[B, Hv, NT, K, V]``.
With ``cu_seqlens`` the batch is 1 and ``T`` is the packed token count.

Every function computes in ``compute_dtype`` (fp32 by default, fp64 for truth
runs).  ``lowp`` (a torch dtype or None) reproduces the rounding points of the
reference kernels: operands are rounded to ``lowp`` before each matmul.

Reference statements followed:
  naive recurrence      examples/flash_gated_delta_rule.py:1545-1571
  pipeline order        examples/flash_gated_delta_rule.py:796-881
  chunk_local_cumsum    torch_custom/fla_npu/test/test_npu_chunk_local_cumsum.py:44-72
  chunk_scaled_dot_kkt  torch_custom/fla_npu/test/test_npu_chunk_scaled_dot_kkt.py:60-106
  solve_tri             torch_custom/fla_npu/test/test_npu_solve_tri_ascend910b.py:48-94
  recompute_w_u_fwd     torch_custom/fla_npu/test/test_npu_recompute_w_u_fwd.py:38-145
  chunk_fwd_h           torch_custom/fla_npu/test/test_fwd_h.py:35-124
  chunk_fwd_o           torch_custom/fla_npu/test/test_fwd_o.py:52-128
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch


def _cu_list(cu_seqlens) -> Optional[list]:
    if cu_seqlens is None:
        return None
    if isinstance(cu_seqlens, torch.Tensor):
        return [int(x) for x in cu_seqlens.detach().cpu().flatten().tolist()]
    return [int(x) for x in cu_seqlens]


def chunk_spans(batch: int, total_t: int, chunk: int, cu_seqlens=None):
    """Yield (batch_idx, seq_idx, global_chunk_idx_within_batch_row, start, end).

    Dense: every batch row is one sequence of ``total_t`` tokens.  Varlen: batch
    row 0 holds all sequences back to back; empty sequences own no chunk
    (examples/flash_gated_delta_rule.py:90-100).
    """
    cu = _cu_list(cu_seqlens)
    if cu is None:
        for b in range(batch):
            for ci, s in enumerate(range(0, total_t, chunk)):
                yield b, b, ci, s, min(s + chunk, total_t)
        return
    gi = 0
    for n, (bos, eos) in enumerate(zip(cu, cu[1:])):
        for s in range(bos, eos, chunk):
            yield 0, n, gi, s, min(s + chunk, eos)
            gi += 1


def total_chunks(batch: int, total_t: int, chunk: int, cu_seqlens=None) -> int:
    cu = _cu_list(cu_seqlens)
    if cu is None:
        return (total_t + chunk - 1) // chunk
    return sum((e - s + chunk - 1) // chunk for s, e in zip(cu, cu[1:]))


def prepare_chunk_indices(cu_seqlens, chunk: int) -> list:
    """Flat [seq0, chunk0, seq0, chunk1, ...] list (examples/...:82-100)."""
    cu = _cu_list(cu_seqlens)
    out = []
    for n, (bos, eos) in enumerate(zip(cu, cu[1:])):
        for c in range((eos - bos + chunk - 1) // chunk):
            out.extend([n, c])
    return out


def _round(x: torch.Tensor, lowp) -> torch.Tensor:
    return x if lowp is None else x.to(lowp).to(x.dtype)


# ----------------------------------------------------------------------------
# stage 1: chunk-local cumulative sum
# ----------------------------------------------------------------------------
def chunk_local_cumsum(g, chunk: int, *, cu_seqlens=None, reverse=False, scale=1.0,
                       output_dtype=torch.float32):
    """out[b,h,t] = scale * sum_{chunk_start <= s <= t} g[b,h,s] (suffix sum if reverse).

    ``g`` may have trailing feature dims ([B,H,T] or [B,H,T,K]); the scan runs
    over dim 2.  fp32 accumulation, then cast.
    """
    gf = g if g.dtype == torch.float64 else g.float()   # fp64 only for truth runs
    out = torch.empty_like(gf)
    B, T = g.shape[0], g.shape[2]
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        acc = torch.zeros_like(gf[b, :, 0])
        rng = range(e - 1, s - 1, -1) if reverse else range(s, e)
        for t in rng:                      # explicit running sum: not torch.cumsum
            acc = acc + gf[b, :, t]
            out[b, :, t] = acc
    return (out * scale).to(output_dtype)


# ----------------------------------------------------------------------------
# stage 2: A0 = strict_lower(beta_i * exp(clip(G_i - G_j)) * <k_i, k_j>)
# ----------------------------------------------------------------------------
def chunk_scaled_dot_kkt(k, g, beta, chunk: int = 64, *, cu_seqlens=None,
                         compute_dtype=torch.float32):
    """Returns A0 [B, Hv, T, C] fp32; row beta, clip +-50, zeros above/on the
    diagonal and in tail columns (chunk_scaled_dot_kkt/README.md:11-29)."""
    B, Hk, T, K = k.shape
    Hv = g.shape[1]
    rep = Hv // Hk
    kf = k.to(compute_dtype)
    gf = g.to(compute_dtype)
    bf = beta.to(compute_dtype)
    A = torch.zeros(B, Hv, T, chunk, dtype=compute_dtype)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)          # [Hv, L, K]
        gc = gf[b, :, s:e]                                        # [Hv, L]
        kk = torch.matmul(kc, kc.transpose(-1, -2))               # [Hv, L, L]
        dec = torch.exp(torch.clamp(gc[:, :, None] - gc[:, None, :], -50.0, 50.0))
        a = kk * dec * bf[b, :, s:e, None]
        A[b, :, s:e, :L] = torch.tril(a, -1)
    return A if compute_dtype == torch.float64 else A.float()


# ----------------------------------------------------------------------------
# stage 3: (I + A0)^-1 per chunk
# ----------------------------------------------------------------------------
def solve_tri(A, *, cu_seqlens=None, compute_dtype=torch.float32, output_dtype=None):
    """``A`` [B, H, T, C] strictly-lower chunk matrices -> (I + A)^-1, same shape.

    Forward substitution row by row (no library inverse): for row i,
    X[i,:] = e_i - sum_{s<i} A[i,s] X[s,:].
    """
    B, H, T, C = A.shape
    Af = A.to(compute_dtype)
    X = torch.zeros_like(Af)
    for b, _, _, s, e in chunk_spans(B, T, C, cu_seqlens):
        L = e - s
        a = Af[b, :, s:e, :L]                                     # [H, L, L]
        x = torch.zeros(H, L, L, dtype=compute_dtype)
        for i in range(L):
            row = -torch.einsum("hs,hsj->hj", a[:, i, :i], x[:, :i, :]) if i else \
                torch.zeros(H, L, dtype=compute_dtype)
            row[:, i] += 1.0
            x[:, i] = row
        X[b, :, s:e, :L] = x
    return X.to(output_dtype if output_dtype is not None else A.dtype)


# ----------------------------------------------------------------------------
# stage 4: w = Ainv (k beta e^G), u = Ainv (v beta)
# ----------------------------------------------------------------------------
def recompute_w_u_fwd(k, v, beta, A, chunk: int, *, g, cu_seqlens=None,
                      compute_dtype=torch.float32, lowp=None, output_dtype=None):
    B, Hk, T, K = k.shape
    Hv, V = v.shape[1], v.shape[3]
    rep = Hv // Hk
    kf, vf = k.to(compute_dtype), v.to(compute_dtype)
    bf, gf, Af = beta.to(compute_dtype), g.to(compute_dtype), A.to(compute_dtype)
    w = torch.zeros(B, Hv, T, K, dtype=compute_dtype)
    u = torch.zeros(B, Hv, T, V, dtype=compute_dtype)
    for b, _, _, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        L = e - s
        a = Af[b, :, s:e, :L]
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        kb = _round(kc * (bf[b, :, s:e] * torch.exp(gf[b, :, s:e]))[..., None], lowp)
        vb = _round(vf[b, :, s:e] * bf[b, :, s:e, None], lowp)
        w[b, :, s:e] = torch.matmul(a, kb)
        u[b, :, s:e] = torch.matmul(a, vb)
    od = output_dtype if output_dtype is not None else k.dtype
    return w.to(od), u.to(od)


# ----------------------------------------------------------------------------
# stage 5: sequential state scan
# ----------------------------------------------------------------------------
def chunk_gated_delta_rule_fwd_h(k, w, u, g=None, *, gk=None, initial_state=None, output_final_state=False,
                                 chunk: int = 64, cu_seqlens=None,
                                 compute_dtype=torch.float32, lowp=None, output_dtype=None):
    """Returns (h [B,Hv,NT,K,V] = state at each chunk start, v_new [B,Hv,T,V],
    final_state [N,Hv,K,V] fp32 or None).  ``g`` [B,Hv,T]: scalar gate (natural log); ``gk`` [B,Hv,T,K]:
    key-wise gate in log2 units, whose decay 2^{gk_last} multiplies the state rows while k arrives already gated
    (chunk_gated_delta_rule_fwd_h/README.md:16-30)."""
    if g is None:
        g = torch.zeros(u.shape[:3], dtype=compute_dtype)
    B, Hk, T, K = k.shape
    Hv, V = u.shape[1], u.shape[3]
    rep = Hv // Hk
    cu = _cu_list(cu_seqlens)
    N = B if cu is None else len(cu) - 1
    NT = total_chunks(B, T, chunk, cu)
    kf, wf, uf, gf = (x.to(compute_dtype) for x in (k, w, u, g))
    h = torch.zeros(B, Hv, NT, K, V, dtype=compute_dtype)
    v_new = torch.zeros(B, Hv, T, V, dtype=compute_dtype)
    state = torch.zeros(N, Hv, K, V, dtype=compute_dtype)
    if initial_state is not None:
        state = initial_state.to(compute_dtype).clone()
    for b, n, ci, s, e in chunk_spans(B, T, chunk, cu):
        S = state[n]
        h[b, :, ci] = S
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)          # [Hv, L, K]
        gc = gf[b, :, s:e]
        vn = uf[b, :, s:e] - torch.matmul(wf[b, :, s:e], _round(S, lowp))
        v_new[b, :, s:e] = vn
        glast = gc[:, -1]
        vdec = _round(_round(vn, lowp) * torch.exp(glast[:, None] - gc)[..., None], lowp)
        decay = torch.exp(glast)[:, None, None]
        if gk is not None:
            decay = decay * torch.exp2(gk[b, :, e - 1].to(compute_dtype))[:, :, None]
        state[n] = S * decay + torch.matmul(kc.transpose(-1, -2), vdec)
    od = output_dtype if output_dtype is not None else k.dtype
    return h.to(od), v_new.to(od), (state.float() if output_final_state else None)


# ----------------------------------------------------------------------------
# stage 6: output
# ----------------------------------------------------------------------------
def chunk_fwd_o(q, k, v_new, h, scale: float, *, g, chunk: int = 64, cu_seqlens=None,
                compute_dtype=torch.float32, lowp=None, output_dtype=None):
    B, Hk, T, K = q.shape
    Hv, V = v_new.shape[1], v_new.shape[3]
    rep = Hv // Hk
    qf, kf, vf, hf, gf = (x.to(compute_dtype) for x in (q, k, v_new, h, g))
    o = torch.zeros(B, Hv, T, V, dtype=compute_dtype)
    for b, _, ci, s, e in chunk_spans(B, T, chunk, cu_seqlens):
        qc = qf[b, :, s:e].repeat_interleave(rep, dim=0)
        kc = kf[b, :, s:e].repeat_interleave(rep, dim=0)
        gc = gf[b, :, s:e]
        dec = torch.exp(torch.clamp(gc[:, :, None] - gc[:, None, :], max=0.0))
        P = _round(torch.tril(torch.matmul(qc, kc.transpose(-1, -2)) * dec), lowp)
        inter = torch.matmul(qc, hf[b, :, ci]) * torch.exp(gc)[..., None]
        o[b, :, s:e] = (inter + torch.matmul(P, vf[b, :, s:e])) * scale
    return o.to(output_dtype if output_dtype is not None else q.dtype)


# ----------------------------------------------------------------------------
# composition (head-first op layout)
# ----------------------------------------------------------------------------
def chunk_gated_delta_rule_fwd(q, k, v, g, beta, scale=None, *, initial_state=None,
                               output_final_state=False, chunk: int = 64, cu_seqlens=None,
                               compute_dtype=torch.float32, lowp=None, return_intermediates=False):
    """g is the RAW per-token log gate [B,Hv,T]; stages as in the reference pipeline."""
    if scale is None:
        scale = k.shape[-1] ** -0.5
    kw = dict(cu_seqlens=cu_seqlens)
    G = chunk_local_cumsum(g, chunk, **kw).to(compute_dtype)
    A0 = chunk_scaled_dot_kkt(k, G, beta, chunk, compute_dtype=compute_dtype, **kw)
    Ainv = solve_tri(_round(A0.to(compute_dtype), lowp), compute_dtype=compute_dtype,
                     output_dtype=compute_dtype, **kw)
    Ainv = _round(Ainv, lowp)
    od = compute_dtype
    w, u = recompute_w_u_fwd(k, v, beta, Ainv, chunk, g=G, compute_dtype=compute_dtype,
                             lowp=lowp, output_dtype=od, **kw)
    w, u = _round(w, lowp), _round(u, lowp)
    h, v_new, final = chunk_gated_delta_rule_fwd_h(
        k, w, u, G, initial_state=initial_state, output_final_state=output_final_state,
        chunk=chunk, compute_dtype=compute_dtype, lowp=lowp, output_dtype=od, **kw)
    h, v_new = _round(h, lowp), _round(v_new, lowp)
    o = chunk_fwd_o(q, k, v_new, h, scale, g=G, chunk=chunk, compute_dtype=compute_dtype,
                    lowp=lowp, output_dtype=od, **kw)
    if return_intermediates:
        return o, final, dict(G=G, A0=A0, Ainv=Ainv, w=w, u=u, h=h, v_new=v_new)
    return o, final


def naive_recurrent_gated_delta_rule(q, k, v, g, beta, scale=None, *, initial_state=None,
                                     output_final_state=False, cu_seqlens=None,
                                     compute_dtype=torch.float32):
    """Token-by-token recurrence, the acceptance oracle
    (examples/flash_gated_delta_rule.py:1545-1571, extended with GVA, an initial
    state, the final state and packed variable-length batches).

    S <- e^{g_t} S ; delta = beta_t (v_t - S^T k_t) ; S <- S + k_t delta^T ; o_t = scale S^T q_t
    """
    B, Hk, T, K = q.shape
    Hv, V = v.shape[1], v.shape[3]
    rep = Hv // Hk
    if scale is None:
        scale = K ** -0.5
    cu = _cu_list(cu_seqlens)
    spans = [(b, b, 0, T) for b in range(B)] if cu is None else \
        [(0, n, s, e) for n, (s, e) in enumerate(zip(cu, cu[1:]))]
    N = len(spans)
    qf = q.to(compute_dtype).repeat_interleave(rep, dim=1)
    kf = k.to(compute_dtype).repeat_interleave(rep, dim=1)
    vf, gf, bf = v.to(compute_dtype), g.to(compute_dtype), beta.to(compute_dtype)
    o = torch.zeros(B, Hv, T, V, dtype=compute_dtype)
    final = torch.zeros(N, Hv, K, V, dtype=compute_dtype)
    for b, n, s, e in spans:
        S = torch.zeros(Hv, K, V, dtype=compute_dtype) if initial_state is None \
            else initial_state[n].to(compute_dtype).clone()
        for t in range(s, e):
            S = S * torch.exp(gf[b, :, t])[:, None, None]
            kt = kf[b, :, t]                                       # [Hv, K]
            delta = (vf[b, :, t] - torch.einsum("hkv,hk->hv", S, kt)) * bf[b, :, t, None]
            S = S + kt[:, :, None] * delta[:, None, :]
            o[b, :, t] = torch.einsum("hkv,hk->hv", S, qf[b, :, t]) * scale
        final[n] = S
    return o, (final if output_final_state else None)


# ----------------------------------------------------------------------------
# pipeline-level entry: reference layouts q,k,v [B,H,T,D]; g,beta [B,T,H]; o [B,T,H,V]
# ----------------------------------------------------------------------------
def flash_gated_delta_rule(q, k, v, g, beta, scale=None, initial_state=None,
                           output_final_state=False, cu_seqlens=None, chunk_size=64,
                           *, naive=True, compute_dtype=torch.float32, lowp=None):
    """Same argument / return layouts as examples/flash_gated_delta_rule.py:1126-1228."""
    gh = g.transpose(1, 2).contiguous()
    bh = beta.transpose(1, 2).contiguous()
    if naive:
        o, final = naive_recurrent_gated_delta_rule(
            q, k, v, gh, bh, scale, initial_state=initial_state,
            output_final_state=output_final_state, cu_seqlens=cu_seqlens,
            compute_dtype=compute_dtype)
    else:
        o, final = chunk_gated_delta_rule_fwd(
            q, k, v, gh, bh, scale, initial_state=initial_state,
            output_final_state=output_final_state, chunk=chunk_size, cu_seqlens=cu_seqlens,
            compute_dtype=compute_dtype, lowp=lowp)
    return o.transpose(1, 2).contiguous(), final


def make_gdn_inputs(B, T, H, K, V, *, dtype=torch.float32, seed=0, Hk=None, init_std=None,
                    head_first_gates=False):
    """Seeded synthetic inputs of the benchmark configurations: q,k ~ N(0,1)
    L2-normalised over K, v ~ N(0,1), beta = sigmoid(N(0,1)), g = logsigmoid(N(0,1))."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    Hk = H if Hk is None else Hk
    F = torch.nn.functional
    q = F.normalize(torch.randn(B, Hk, T, K, generator=gen), p=2, dim=-1).to(dtype)
    k = F.normalize(torch.randn(B, Hk, T, K, generator=gen), p=2, dim=-1).to(dtype)
    v = torch.randn(B, H, T, V, generator=gen).to(dtype)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen))
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen))
    h0 = None
    if init_std is not None:
        h0 = torch.randn(B, H, K, V, generator=gen) * init_std
    if head_first_gates:
        g, beta = g.transpose(1, 2).contiguous(), beta.transpose(1, 2).contiguous()
    return dict(q=q, k=k, v=v, g=g, beta=beta, initial_state=h0)


# ----------------------------------------------------------------------------
# q/k normalisation of the pipeline entry (fla/ops/triton/triton_core/l2norm.py:16-30,93-128)
# ----------------------------------------------------------------------------
def l2norm_fwd(x, eps: float = 1e-6, compute_dtype=torch.float32):
    """y = x * rstd with rstd = 1 / sqrt(sum x^2 + eps) over the last dimension; returns (y, rstd)."""
    xf = x.to(compute_dtype)
    ss = torch.zeros(xf.shape[:-1], dtype=compute_dtype)
    for i in range(xf.shape[-1]):                     # explicit accumulation: not torch.norm
        ss = ss + xf[..., i] * xf[..., i]
    rstd = 1.0 / torch.sqrt(ss + eps)
    return (xf * rstd[..., None]).to(x.dtype), rstd


def l2norm_bwd(y, rstd, dy, compute_dtype=torch.float32):
    """dx = (dy - sum(dy * y) * y) * rstd, y the normalised output."""
    yf, df = y.to(compute_dtype), dy.to(compute_dtype)
    dot = (df * yf).sum(-1, keepdim=True)
    return ((df - dot * yf) * rstd.to(compute_dtype)[..., None]).to(dy.dtype)
