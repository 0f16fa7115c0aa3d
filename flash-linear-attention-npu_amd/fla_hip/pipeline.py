"""Pipeline-level entry points: the gated-delta-rule chunk forward with the argument and
return layouts of examples/flash_gated_delta_rule.py:1126-1228 (``flash_gated_delta_rule``)
and :796-881 (``flash_chunk_gated_delta_rule_fwd``).

Two routes produce the same results:
* ``fused=True`` (default): one library call, ``fla_gdn_chunk_fwd``;
* ``fused=False``: the reference's own composition of the six operators
  (cumsum -> kkt -> solve_tri -> recompute_w_u -> fwd_h -> fwd_o), which also returns the
  inverted chunk matrix ``A``.
The backward (``flash_chunk_gated_delta_rule_bwd``, examples/flash_gated_delta_rule.py:884-1008) is the
reference's composition of the backward operators; ``flash_gated_delta_rule`` records it for autograd
(``ChunkGatedDeltaRuleFunction``, examples/flash_gated_delta_rule.py:1026-1123) when an input requires grad.
"""
from __future__ import annotations

import warnings
from typing import Optional

from . import ops as _ops
from .ops import _hip_ctypes as _raw


def _cu_list(cu_seqlens):
    if cu_seqlens is None:
        return None
    import torch

    if isinstance(cu_seqlens, torch.Tensor):
        return [int(x) for x in cu_seqlens.detach().cpu().flatten().tolist()]
    return [int(x) for x in cu_seqlens]


def flash_chunk_gated_delta_rule_fwd(q, k, v, g, beta, scale, initial_state, output_final_state,
                                     cu_seqlens=None, chunk_size: int = 64, *, fused: bool = True,
                                     use_qk_l2norm_in_kernel: bool = False, save_for_backward: bool = False):
    """q,k,v [B,H,T,D] bf16; g,beta [B,T,H].  Returns (g_cumsum [B,T,H] f32, o [B,T,H,V], A, final_state);
    ``A`` ([B,H,T,C] bf16, the inverted chunk matrices) is None on the fused route.  With
    ``use_qk_l2norm_in_kernel`` the fused route normalises q and k rows while it stages them; the composed
    route runs the two normalisation passes first (examples/flash_gated_delta_rule.py:1047-1049).
    ``save_for_backward`` appends a dict with h, v_new and w, which the backward then does not recompute
    (64-token chunks only); the fused route with ``use_qk_l2norm_in_kernel`` adds the normalised q and k and their
    q_rstd, k_rstd, written by the same kernel."""
    import torch

    cu = _cu_list(cu_seqlens)
    if fused:
        # the fused kernel carries and exchanges the state in fp32; a 16-bit state is widened here and the final
        # state returned in the caller's dtype (chunk_gated_delta_rule_fwd_h/README.md:85-91 allows both)
        h0 = initial_state
        if h0 is not None and h0.dtype != torch.float32:
            h0 = h0.float()
        res = _raw.gdn_chunk_fwd(q, k, v, g.float(), beta.float(), scale, h0, output_final_state, cu, chunk_size,
                                 use_qk_l2norm_in_kernel, save_for_backward=save_for_backward)
        gc, o, final = res[:3]
        if final is not None and initial_state is not None and final.dtype != initial_state.dtype:
            final = final.to(initial_state.dtype)
        if save_for_backward:
            return gc, o, None, final, dict(zip(("h", "v_new", "w", "q", "k", "q_rstd", "k_rstd"), res[3:]))
        return gc, o, None, final
    if use_qk_l2norm_in_kernel:
        q, _ = _raw.l2norm_fwd(q)
        k, _ = _raw.l2norm_fwd(k)
    # reference composition (examples/flash_gated_delta_rule.py:811-881)
    gh = _ops.chunk_local_cumsum(g.transpose(1, 2).contiguous(), chunk_size, cu_seqlens=cu,
                                 head_first=True, output_dtype=torch.float32)
    bh = beta.transpose(1, 2).contiguous().float()
    A = _ops.chunk_scaled_dot_kkt(k, gh, bh, cu_seqlens=cu, chunk_size=chunk_size)
    A = _ops.solve_tri(A, cu_seqlens=cu, layout="bnsd", output_dtype=k.dtype)   # rounds A to k.dtype on load
    w, u = _ops.recompute_w_u_fwd(k, v, bh, A, chunk_size, g=gh, cu_seqlens=cu)
    h, v_new, final = _ops.chunk_gated_delta_rule_fwd_h(
        k, w, u, g=gh, initial_state=initial_state, output_final_state=output_final_state,
        chunk_size=chunk_size, cu_seqlens=cu)
    o = _ops.chunk_fwd_o(q, k, v_new, h, scale, g=gh, cu_seqlens=cu, chunk_size=chunk_size, out_token_major=True)
    out = (gh.transpose(1, 2).contiguous(), o.transpose(1, 2).contiguous(), A, (final if output_final_state else None))
    if save_for_backward:
        return out + (dict(h=h, v_new=v_new, w=w),)
    return out


def flash_chunk_gated_delta_rule_bwd(q, k, v, g, beta, A, scale, initial_state, do, dht, cu_seqlens=None,
                                     chunk_size: int = 64, *, saved=None, qk_rstd=None):
    """q,k,v [B,H,T,D] bf16; ``g`` the chunk-cumsummed gate and beta [B,T,H] (as the forward returned /
    received them); ``A`` [B,H,T,C] the inverted chunk matrices or None (recomputed); do [B,T,H,V];
    dht [N,H,K,V] fp32 or None.  Returns (dq, dk, dv [B,H,T,D], dbeta, dg [B,T,H] fp32, dh0 [N,H,K,V] fp32 or
    None); dg is the gradient of the RAW gate.  Unlike the reference, the initial state and the final-state
    gradient take part (the reference passes neither to its reverse scan and returns dh0 = None).
    ``saved``: the dict of h, v_new and w the forward wrote with ``save_for_backward``; without it they are
    recomputed as the reference does (examples/flash_gated_delta_rule.py:913-951).  ``qk_rstd``: (q_rstd, k_rstd) of
    ``l2norm_fwd`` when q and k are the normalised tensors; dq and dk then come back as the gradients of the raw q and k
    (the reference runs ``l2norm_bwd`` over both afterwards, :1104-1106).  With 64-token chunks the two kernels that
    complete dq and dk do it themselves; otherwise two ``l2norm_bwd`` passes follow."""
    import torch

    cu = _cu_list(cu_seqlens)
    kw = dict(cu_seqlens=cu)
    # head-first VIEWS: every kernel takes the outer strides of its operands, nothing is copied
    gh = g.float().transpose(1, 2)
    bh = beta.float().transpose(1, 2)
    if A is None and chunk_size == 64 and saved is not None:
        pass   # nothing but the WY backward needs A then, and that kernel rebuilds it per chunk from k, g and beta
    elif A is None and chunk_size == 64:
        A = _ops.chunk_scaled_dot_kkt_inverse(k, gh, bh, chunk_size=chunk_size, **kw)   # the two operators below, fused
    elif A is None:
        A = _ops.chunk_scaled_dot_kkt(k, gh, bh, chunk_size=chunk_size, **kw)
        A = _ops.solve_tri(A, layout="bnsd", output_dtype=k.dtype, **kw)   # rounds A to k.dtype on load
    doh = do.transpose(1, 2) if do.stride(-1) == 1 else do.transpose(1, 2).contiguous()
    if saved is not None:
        h, v_new, w = saved["h"], saved["v_new"], saved["w"]
    else:
        w, u = _ops.recompute_w_u_fwd(k, v, bh, A, chunk_size, g=gh, **kw)
        h, v_new, _ = _ops.chunk_gated_delta_rule_fwd_h(k, w, u, g=gh, initial_state=initial_state,
                                                        output_final_state=False, chunk_size=chunk_size, **kw)
    # 64-token chunks: the reverse scan forms the intra-chunk part of dv from the tiles it holds; otherwise
    # chunk_bwd_dv_local runs first, as in the reference (examples/flash_gated_delta_rule.py:953-966)
    dv = None if chunk_size == 64 else _ops.chunk_bwd_dv_local(q, k, doh, gh, scale, chunk_size, **kw)
    dh, dh0, dv = _ops.chunk_gated_delta_rule_bwd_dhu(q, k, w, doh, dv, scale, chunk_size, g=gh, h0=initial_state,
                                                      dht=dht, dh0_per_sequence=True, **kw)
    in_kernel_norm = qk_rstd is not None and chunk_size == 64
    if in_kernel_norm:
        dq, dk, dw, dg = _raw.chunk_bwd_dqkwg_l2norm(q, k, v_new, gh, h, doh, dh, dv, qk_rstd[0], chunk_size, scale=scale, **kw)
    else:
        dq, dk, dw, dg = _ops.chunk_bwd_dqkwg(q, k, v_new, gh, h, doh, dh, dv, chunk_size, scale=scale, **kw)
    # the second part of dk and dg is added where it is produced (the reference adds with separate passes,
    # examples/flash_gated_delta_rule.py:994-1012), and on 64-token chunks dA is formed by the same kernel
    # (prepare_wy_repr_bwd_da, :985-992, as a pass of its own otherwise); A = None: see above
    if chunk_size == 64:
        dv, db = _raw.prepare_wy_repr_bwd_full_accumulate(k, v, bh, A, None, dw, dv, gh, dk, dg, chunk_size,
                                                          k_rstd=qk_rstd[1] if in_kernel_norm else None, **kw)
    else:   # 128-token chunks: the plain operators and the reference's two additions
        dA = _ops.prepare_wy_repr_bwd_da(k, v, bh, A, dw, dv, gh, chunk_size=chunk_size, **kw)
        dk2, dv, db, dg2 = _ops.prepare_wy_repr_bwd_full(k, v, bh, A, dA, dw, dv, gh, chunk_size, **kw)
        dk.add_(dk2)
        dg.add_(dg2)
    if qk_rstd is not None and not in_kernel_norm:
        dq = _raw.l2norm_bwd(q, qk_rstd[0], dq)
        dk = _raw.l2norm_bwd(k, qk_rstd[1], dk)
    dg = _ops.chunk_local_cumsum(dg, chunk_size, reverse=True, head_first=True, output_dtype=torch.float32, **kw)
    return dq, dk, dv, db.transpose(1, 2), dg.transpose(1, 2), dh0


def needs_grad_hint(*tensors) -> bool:
    """True when autograd will record the call."""
    import torch

    return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


def _autograd_function():
    """Built on first use so that importing this module does not import torch."""
    import torch

    class ChunkGatedDeltaRuleFunction(torch.autograd.Function):
        @staticmethod
        def forward(ctx, q, k, v, g, beta, scale, initial_state, output_final_state, cu, chunk_size, fused, l2norm,
                    save_intermediates=True):
            q_rstd = k_rstd = None
            if not save_intermediates:
                # the reference's memory profile (examples/flash_gated_delta_rule.py:1084): only q, k, v, the cumulated
                # gate, beta and the state are kept; w, u, h and v_new are recomputed by the backward (:913-951)
                if l2norm:
                    q, q_rstd = _raw.l2norm_fwd(q)
                    k, k_rstd = _raw.l2norm_fwd(k)
                gc, o, A, final = flash_chunk_gated_delta_rule_fwd(
                    q, k, v, g, beta, scale, initial_state, output_final_state, cu, chunk_size, fused=fused)
                ctx.save_for_backward(q, k, v, gc, beta, A, initial_state, q_rstd, k_rstd, None, None, None)
                ctx.scale, ctx.cu, ctx.chunk_size = scale, cu, chunk_size
                ctx.dtypes = (g.dtype, beta.dtype)
                return o, final
            # examples/flash_gated_delta_rule.py:1047-1049.  The fused forward normalises the rows itself and writes
            # them with their rstd; the composed route runs l2norm_fwd (y comes back in the memory order of x).
            in_kernel = bool(l2norm and fused)
            if l2norm and not in_kernel:
                q, q_rstd = _raw.l2norm_fwd(q)
                k, k_rstd = _raw.l2norm_fwd(k)
            gc, o, A, final, saved = flash_chunk_gated_delta_rule_fwd(
                q, k, v, g, beta, scale, initial_state, output_final_state, cu, chunk_size, fused=fused,
                use_qk_l2norm_in_kernel=in_kernel, save_for_backward=True)
            if in_kernel:
                q, k, q_rstd, k_rstd = saved["q"], saved["k"], saved["q_rstd"], saved["k_rstd"]
            ctx.save_for_backward(q, k, v, gc, beta, A, initial_state, q_rstd, k_rstd, saved["h"], saved["v_new"], saved["w"])
            ctx.scale, ctx.cu, ctx.chunk_size = scale, cu, chunk_size
            ctx.dtypes = (g.dtype, beta.dtype)
            return o, final

        @staticmethod
        def backward(ctx, do, dht):
            q, k, v, gc, beta, A, initial_state, q_rstd, k_rstd, h, v_new, w = ctx.saved_tensors
            dq, dk, dv, db, dg, dh0 = flash_chunk_gated_delta_rule_bwd(
                q, k, v, gc, beta, A, ctx.scale, initial_state, do.contiguous(),
                None if dht is None else dht.contiguous(), ctx.cu, ctx.chunk_size,
                saved=None if h is None else dict(h=h, v_new=v_new, w=w),
                qk_rstd=None if q_rstd is None else (q_rstd, k_rstd))
            return dq, dk, dv, dg.to(ctx.dtypes[0]), db.to(ctx.dtypes[1]), None, dh0, None, None, None, None, None, None

    return ChunkGatedDeltaRuleFunction


_FUNCTION = None


def flash_gated_delta_rule(q, k, v, g, beta, scale: Optional[float] = None, initial_state=None,
                           output_final_state: bool = False, use_qk_l2norm_in_kernel: bool = False,
                           cu_seqlens=None, cu_seqlens_list=None, chunk_indices=None, chunk_indices_list=None,
                           chunk_size: int = 64, head_first: bool = False, *, fused: bool = True,
                           save_intermediates: bool = True):
    """Same checks, defaults and layouts as the reference entry: q,k [B,H,T,K], v [B,H,T,V],
    g,beta [B,T,H]; returns (o [B,T,H,V], final_state [N,H,K,V] or None).

    ``save_intermediates`` (only matters when autograd records the call): True keeps h [B,H,NT,K,V], v_new and w of the
    forward for the backward, which then skips their recomputation (about 0.5 ms of a 2.8 ms training step at
    B=4, T=8192, H=32, d=128) at the price of roughly twice the activation memory per layer (h alone is 0.5 GB
    there); False keeps what the reference keeps (q, k, v, g, beta, the state) and recomputes the rest."""
    import torch

    del chunk_indices, chunk_indices_list  # derived from cu_seqlens inside the library
    if q.dtype != k.dtype or k.dtype != v.dtype:
        raise ValueError(
            f"q current type is {q.dtype}, k current type is {k.dtype}, "
            f"v current type is {v.dtype}; they should be equal")
    if q.dtype == torch.float32:
        raise ValueError("ChunkGatedDeltaRuleFunction does not support float32. Please use float16/bfloat16.")
    if beta.ndim != 3 or g.ndim != 3:
        raise ValueError("g and beta must be rank-3 tensors with shape [B, T, H].")
    if q.ndim != 4 or k.ndim != 4 or v.ndim != 4:
        raise ValueError("q, k and v must be rank-4 tensors with shape [B, H, T, D].")
    # the reference requires equal head counts here; grouped value heads (Hv a multiple of Hk) are
    # supported by every kernel of this library, so only batch and length must agree
    if q.shape[:3] != k.shape[:3] or (q.shape[0], q.shape[2]) != (v.shape[0], v.shape[2]) \
            or v.shape[1] % q.shape[1] != 0:
        raise ValueError(f"q/k/v shape prefixes must match, got {q.shape}, {k.shape}, {v.shape}.")
    if g.shape != beta.shape:
        raise ValueError(f"g and beta shapes must match, got {g.shape} and {beta.shape}.")
    if g.shape[0] != q.shape[0] or g.shape[1] != q.shape[2] or g.shape[2] != v.shape[1]:
        raise ValueError(
            "Expected q/k/v in [B, H, T, D] and g/beta in [B, T, H]; "
            f"got q={tuple(q.shape)}, g={tuple(g.shape)}.")
    if head_first:
        warnings.warn("head_first is kept only for API compatibility. q/k/v are always [B, H, T, D].", stacklevel=2)
    if chunk_size != 2 ** (chunk_size.bit_length() - 1):
        raise ValueError(f"chunk_size must be a power of 2, got {chunk_size}.")
    cu = _cu_list(cu_seqlens if cu_seqlens is not None else cu_seqlens_list)
    if cu is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f"The batch size is expected to be 1 rather than {q.shape[0]} when using cu_seqlens. "
                "Please flatten variable-length inputs before processing.")
        if initial_state is not None and initial_state.shape[0] != len(cu) - 1:
            raise ValueError(
                "The number of initial states is expected to match the number of input sequences, "
                f"got initial_state.shape[0]={initial_state.shape[0]} and sequences={len(cu) - 1}.")
    if scale is None:
        scale = k.shape[-1] ** -0.5
    # (o, final_state) do not depend on the chunk size: it only tiles the same recurrence.  The fused kernel tiles by
    # 64 tokens, so it serves every request on 64-token chunks; the operators, forward and backward, are built for 64
    # and 128.
    if chunk_size != 64 and (fused or chunk_size != 128):
        if not fused:
            raise NotImplementedError("the six-operator route is built for chunk_size 64 and 128; use fused=True.")
        chunk_size = 64
    needs_grad = needs_grad_hint(q, k, v, g, beta, initial_state)
    if not needs_grad:
        _, o, _, final = flash_chunk_gated_delta_rule_fwd(
            q, k, v, g, beta, float(scale), initial_state, output_final_state, cu, chunk_size, fused=fused,
            use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel)
        return o, final
    global _FUNCTION
    if _FUNCTION is None:
        _FUNCTION = _autograd_function()
    return _FUNCTION.apply(q, k, v, g, beta, float(scale), initial_state, output_final_state, cu, chunk_size, fused,
                           bool(use_qk_l2norm_in_kernel), bool(save_intermediates))


# =============================================================================================
# KDA (per-channel gated delta rule): chunk forward + backward as one differentiable call
# =============================================================================================
# The reference exposes the forward operator and two backward stages (bwd_dhu with gK, chunk_kda_bwd_intra) and
# leaves the composition to a third-party package it patches (adapters/triton_ascend_kda.py:141-242 hands that
# package the forward's saved tensors gk, Aqk, Akk, w, u, qg, kg, v_new, h).  Here the whole chain is the library's.
def _index_order(x, layout, *, scalar=False):
    """View of a tensor in ``layout`` (BSND / BNSD / TND / NTD) in [B,H,T,(D)] index order; nothing is copied."""
    if layout == "BSND":
        return x.transpose(1, 2)
    if layout == "BNSD":
        return x
    if layout == "TND":
        return x.transpose(0, 1)[None]
    if layout == "NTD":
        return x[None]
    raise ValueError(f"layout must be one of BSND, BNSD, TND, NTD, got {layout!r}.")


def _from_index_order(x, layout):
    if layout == "BSND":
        return x.transpose(1, 2)
    if layout == "BNSD":
        return x
    if layout == "TND":
        return x[0].transpose(0, 1)
    return x[0]


def chunk_kda_bwd(q, k, v, beta, gk, Aqk, Akk, w, qg, kg, v_new, h, scale, do, dht=None, *, initial_state=None,
                  layout="BSND", cu_seqlens=None, chunk_size: int = 64):
    """KDA chunk backward from the tensors the forward keeps (``chunk_kda_fwd(..., disable_recompute=True)``), on 64- or
    128-token chunks (with 128 only q, k, v, beta, gk and the initial state of what is passed are used, see below).

    q, k, v, beta, do in ``layout``; gk, Aqk, Akk, w, qg, kg, v_new head-major and h as the forward returned them;
    dht fp32 [N,Hv,K,V] or None.  Returns ``(dq, dk, dv, dg, dbeta, dh0)``: dq, dk, dv, dbeta in ``layout`` and the
    dtype of their inputs, dg fp32 in the layout of the gate = gradient of the per-token log decay (natural log),
    dh0 fp32 [N,Hv,K,V] or None.  Stages: reverse scan (bwd_dhu, gK; it forms dv = Aqk^T do itself) -> dq, dk, dw, dg of
    the state-dependent parts and dAqk -> backward of the WY factors (dv, dbeta, dAkk) -> chunk_kda_bwd_intra -> reverse
    chunk-local cumulative sum of dg; up to 128 channels the stages after the scan are one launch."""
    import torch

    cu = _cu_list(cu_seqlens)
    if chunk_size == 128:
        # The gradient kernels take 64-token tiles (as the reference's own backward kernel, _aclnn_ctypes.py:1582-1584).
        # What the forward kept on 128-token chunks (Aqk, Akk, w, qg, kg, v_new, h) tiles the same function differently,
        # so those intermediates are formed again on 64-token chunks from q, k, v, beta and the per-token gate, which the
        # cumulated gate determines: g_t = ln2 (gk_t - gk_{t-1}), and g_t = ln2 gk_t on the first token of a 128-token chunk.
        g_raw = _per_token_gate(gk, 128, cu, layout)
        f = _raw.chunk_kda_fwd_for_backward(q, k, v, g_raw, beta, float(scale), 64, layout=layout, initial_state=initial_state,
                                            cu_seqlens=cu)
        _, _, gk, Aqk, Akk, w, _, qg, kg, v_new, h, _ = f
        chunk_size = 64
    if chunk_size != 64:
        raise NotImplementedError("chunk_kda_bwd: chunk_size must be 64 or 128.")
    kw = dict(cu_seqlens=cu)
    rank3 = layout in ("TND", "NTD")
    hm = lambda t: _index_order(t, layout)
    lead = (lambda t: t[None]) if rank3 else (lambda t: t)
    qh, kh, vh, bh, doh = hm(q), hm(k), hm(v), hm(beta), hm(do)
    if doh.stride(-1) != 1:
        doh = hm(do.contiguous())
    gk4, Aqk4, Akk4, w4, qg4, kg4, vn4 = (lead(t) for t in (gk, Aqk, Akk, w, qg, kg, v_new))
    h5 = lead(h).transpose(1, 2)                                  # [B,NT,Hv,K,V] -> [B,Hv,NT,K,V] view
    Hk, Hv = qh.shape[1], vh.shape[1]
    # fp32 gradients per value head, laid out in memory like the caller's tensors (heads = Hv)
    layout_like = _index_order(_empty_in_layout(layout, gk4.shape), layout)
    if qh.shape[-1] > 128:
        dAqk, dv0 = _raw.chunk_kda_bwd_dav(vn4, doh, Aqk4, scale, chunk_size, layout_like=layout_like, **kw)
        dh, dh0, dv2 = _ops.chunk_gated_delta_rule_bwd_dhu(qg4, kg4, w4, doh, dv0, scale, chunk_size, gK=gk4,
                                                           h0=initial_state, dht=dht, use_exp2=True, dh0_per_sequence=True,
                                                           **kw)
        dq, dk, dg, dv, db, dAkk = _kda_bwd_state_stages_by_channel_halves(qh, kh, vh, bh, gk4, Akk4, vn4, h5, doh, dh, dv2, scale,
                                                                            chunk_size, layout_like, kw)
    else:
        # no pass for chunk_kda_bwd_dav: the reverse scan forms dv = Aqk^T do from the score blocks, the next stage writes
        # dAqk = scale tril(do v_new^T) from the do and v_new tiles it stages anyway
        dh, dh0, dv2 = _raw.chunk_kda_bwd_dhu(qg4, kg4, w4, doh, Aqk4, scale, chunk_size, gK=gk4, h0=initial_state, dht=dht, **kw)
        # everything after the reverse scan in one launch: the state-dependent stage, the backward of the WY factors and the
        # intra-chunk stage with the reverse running sum of dg (as operators of their own they pass dk, dg, dw, dq and the two
        # score gradients through memory between them)
        dq, dk, dg, dv, db = _raw.chunk_kda_bwd_dqkwg_wy_intra(qh, kh, vn4, gk4, h5, doh, dh, dv2, vh, bh, Akk4, scale, chunk_size,
                                                               layout_like=layout_like, grad_dtype=q.dtype if Hv == Hk else None,
                                                               **kw)
        if Hv != Hk:      # value heads that share a key head add their gradients
            dq = dq.unflatten(1, (Hk, Hv // Hk)).sum(2).to(q.dtype)
            dk = dk.unflatten(1, (Hk, Hv // Hk)).sum(2).to(k.dtype)
        back = lambda t: _from_index_order(t, layout)
        return (back(dq), back(dk), back(dv), back(dg), back(db[..., None])[..., 0].to(beta.dtype), dh0)
    # the last stage also takes the reverse chunk-local running sum of dg, which is complete with its own part
    back = lambda t: _from_index_order(t, layout)
    if Hv == Hk:          # dq, dk are final with the last stage: it writes them in the dtype of q and k
        dq16 = _raw._empty_strided_like(dq.shape, dq, q.dtype)
        dk16 = _raw._empty_strided_like(dk.shape, dk, k.dtype)
        _raw.chunk_kda_bwd_intra_inplace(qh, kh, gk4, bh, dAqk, dAkk, dq, dk, db, dg, cu_seqlens=cu, chunk_size=chunk_size,
                                         cumsum_dg=True, dq_out=dq16, dk_out=dk16)
        dq, dk = dq16, dk16
    else:                 # value heads that share a key head add their gradients
        _raw.chunk_kda_bwd_intra_inplace(qh, kh, gk4, bh, dAqk, dAkk, dq, dk, db, dg, cu_seqlens=cu, chunk_size=chunk_size,
                                         cumsum_dg=True)
        dq = dq.unflatten(1, (Hk, Hv // Hk)).sum(2).to(q.dtype)
        dk = dk.unflatten(1, (Hk, Hv // Hk)).sum(2).to(k.dtype)
    return (back(dq), back(dk), back(dv), back(dg), back(db[..., None])[..., 0].to(beta.dtype), dh0)


def _per_token_gate(gk, chunk_size, cu, layout):
    """The per-token log decay (natural log, in ``layout``) behind a chunk-local cumulated gate ``gk`` (head-major
    [..,Hv,T,K] fp32 in log2 units, cumulated over ``chunk_size``-token chunks that restart with every sequence)."""
    import math

    import torch

    g4 = gk if gk.dim() == 4 else gk[None]
    T = g4.shape[2]
    first = torch.zeros(T, dtype=torch.bool, device=gk.device)
    for bos, eos in ([(0, T)] if cu is None else zip(cu[:-1], cu[1:])):
        first[bos:eos:chunk_size] = True
    prev = torch.cat([torch.zeros_like(g4[:, :, :1]), g4[:, :, :-1]], dim=2)
    raw = (g4 - torch.where(first[None, None, :, None], torch.zeros_like(prev), prev)) * math.log(2.0)
    return _from_index_order(raw, layout).contiguous()


def _kda_bwd_state_stages_by_channel_halves(qh, kh, vh, bh, gk4, Akk4, vn4, h5, doh, dh, dv2, scale, chunk_size, layout_like, kw):
    """``chunk_kda_bwd_dqkwg`` and ``chunk_kda_bwd_wy`` for 256 channels on their 128-channel kernels.  Both stages are
    channel-wise except for sums over the channels that enter linearly: dq, dk, dw, dg of a channel need the state rows
    h[c,:], dh[c,:] of that channel only; in the WY backward dk and dg are channel-wise, while dAkk and dbeta add a part
    per channel half to the part of the value columns, which the first pass carries alone (the second one is given
    du = 0).  Returns (dq, dk, dg, dv, dbeta, dAkk) as the two stages leave them for 128 channels."""
    import torch

    K = qh.shape[-1]
    assert K == 256, K
    parts, dv, db, dAkk = [], None, None, None
    for lo in (0, 128):
        sl = slice(lo, lo + 128)
        q_, k_, g_ = qh[..., sl].contiguous(), kh[..., sl].contiguous(), gk4[..., sl].contiguous()
        h_, dh_ = h5[..., sl, :].contiguous(), dh[..., sl, :].contiguous()
        dq, dk, dw, dg = _raw.chunk_kda_bwd_dqkwg(q_, k_, vn4, g_, h_, doh, dh_, dv2, scale, chunk_size,
                                                  layout_like=None if layout_like is None else layout_like[..., sl], **kw)
        du = dv2 if lo == 0 else torch.zeros_like(dv2)
        dv_, db_, dA_ = _raw.chunk_kda_bwd_wy(k_, vh, bh, g_, Akk4, dw, du, dk, dg, chunk_size, **kw)
        parts.append((dq, dk, dg))
        if lo == 0:
            dv, db, dAkk = dv_, db_, dA_
        else:
            db, dAkk = db + db_, dAkk + dA_
    like = parts[0][0] if layout_like is None else layout_like

    def joined(i):
        out = _raw._empty_strided_like(tuple(parts[0][i].shape[:-1]) + (K,), like, torch.float32, parts[0][i].device)
        out[..., :128], out[..., 128:] = parts[0][i], parts[1][i]
        return out
    return joined(0), joined(1), joined(2), dv, db, dAkk


def _empty_in_layout(layout, index_shape):
    """A storage-less tensor in ``layout`` whose index-order shape is ``index_shape`` ([B,H,T,D]); only its strides are
    used (as the memory order of the gradients)."""
    import torch

    B, H, T, D = index_shape
    shape = {"BSND": (B, T, H, D), "BNSD": (B, H, T, D), "TND": (T, H, D), "NTD": (H, T, D)}[layout]
    return torch.empty(shape, dtype=torch.float32, device="meta")


_KDA_FUNCTION = None


def _kda_autograd_function():
    import torch

    class ChunkKdaFunction(torch.autograd.Function):
        # ``gate``: None (g is the log decay itself) or (A_log, dt_bias, safe_gate, lower_bound): g is the raw gate, the
        # forward kernel activates it, and the backward ends with the gradient of that activation (kda_gate_bwd).
        @staticmethod
        def forward(ctx, q, k, v, g, beta, scale, initial_state, output_final_state, cu, layout, chunk_size, A_log=None,
                    dt_bias=None, safe_gate=False, lower_bound=-5.0):
            in_kernel = A_log is not None
            out = _raw.chunk_kda_fwd_for_backward(q, k, v, g, beta, scale, chunk_size, layout=layout,
                                                  initial_state=initial_state, output_final_state=output_final_state,
                                                  cu_seqlens=cu, use_gate_in_kernel=in_kernel, A_log=A_log, dt_bias=dt_bias,
                                                  safe_gate=safe_gate, lower_bound=lower_bound)
            o, final, gk, Aqk, Akk, w, _u, qg, kg, v_new, h, _ = out
            ctx.save_for_backward(q, k, v, beta, gk, Aqk, Akk, w, qg, kg, v_new, h, initial_state,
                                  *((g, A_log, dt_bias) if in_kernel else ()))
            ctx.scale, ctx.cu, ctx.layout, ctx.chunk_size, ctx.g_dtype = scale, cu, layout, chunk_size, g.dtype
            ctx.gate = (safe_gate, lower_bound) if in_kernel else None
            return o, final

        @staticmethod
        def backward(ctx, do, dht):
            q, k, v, beta, gk, Aqk, Akk, w, qg, kg, v_new, h, initial_state = ctx.saved_tensors[:13]
            dht = None if dht is None else dht.contiguous()   # a view when the caller sliced or joined the final state
            dq, dk, dv, dg, db, dh0 = chunk_kda_bwd(q, k, v, beta, gk, Aqk, Akk, w, qg, kg, v_new, h, ctx.scale, do, dht,
                                                    initial_state=initial_state, layout=ctx.layout, cu_seqlens=ctx.cu,
                                                    chunk_size=ctx.chunk_size)
            if ctx.gate is None:
                return dq, dk, dv, dg.to(ctx.g_dtype), db, None, dh0, None, None, None, None, None, None, None, None
            g, A_log, dt_bias = ctx.saved_tensors[13:]
            dg_raw, dA, dbias = _raw.kda_gate_bwd(g, dg, A_log, dt_bias, layout=ctx.layout, safe_gate=ctx.gate[0],
                                                  lower_bound=ctx.gate[1])
            return dq, dk, dv, dg_raw, db, None, dh0, None, None, None, None, dA, dbias, None, None

    return ChunkKdaFunction


def _kda_gate_activation(g, A_log, dt_bias, layout, safe_gate, lower_bound):
    """The in-kernel gate of chunk_kda_fwd (fla/ops/ascendc/kda/chunk_kda_fwd/docs/api.md:103-113) as differentiable
    tensor operations: -exp(A_log) * softplus(g + dt_bias), or lower_bound * sigmoid(exp(A_log) * (g + dt_bias)) with
    ``safe_gate``; A_log [HV] and dt_bias [HV*K] broadcast along the head axis of ``layout``."""
    import torch

    HV, K = A_log.shape[0], g.shape[-1]
    head_axis = {"BSND": 2, "BNSD": 1, "TND": 1, "NTD": 0}[layout]
    shape = [1] * g.dim()
    shape[head_axis] = HV
    eig = torch.exp(A_log.float()).view(shape)
    raw = g.float()
    if dt_bias is not None:
        shape[-1] = K
        raw = raw + dt_bias.float().view(HV, K).view(shape)
    if safe_gate:
        return float(lower_bound) * torch.sigmoid(eig * raw)
    return -eig * torch.nn.functional.softplus(raw)


def chunk_kda(q, k, v, g, beta, scale: Optional[float] = None, initial_state=None, output_final_state: bool = False,
              cu_seqlens=None, *, layout: str = "BSND", chunk_size: int = 64, use_gate_in_kernel: bool = False,
              A_log=None, dt_bias=None, safe_gate: bool = False, lower_bound: Optional[float] = None):
    """KDA chunk attention, differentiable: ``(o, final_state)`` with q, k [..H,K], v [..HV,V], per-channel log decay
    g [..HV,K] (natural log, one value per token and channel), beta [..HV] in ``layout``; states fp32 [N,HV,K,V].
    The forward is ``chunk_kda_fwd``; when an input requires grad the forward keeps its intermediates and
    ``chunk_kda_bwd`` returns dq, dk, dv, dg, dbeta, dh0.  With ``use_gate_in_kernel`` g is the raw gate input and the
    forward kernel activates it; with gradients ``kda_gate_bwd`` ends the backward, so that autograd also reaches
    ``A_log`` and ``dt_bias`` (for a head size served by padding or by two value passes the activation runs as tensor
    operations ahead of the kernels instead).  Gradients cover every admitted head size (V above 128 as two passes over
    128 value columns; K above 128 on 256 channels, with the two state-dependent stages run per channel half) and run on
    64-token tiles whatever ``chunk_size``."""
    import torch

    if scale is None:
        scale = q.shape[-1] ** -0.5
    cu = _cu_list(cu_seqlens)
    lower_bound = -5.0 if lower_bound is None else float(lower_bound)
    if not needs_grad_hint(q, k, v, g, beta, initial_state, A_log, dt_bias):
        out = _ops.chunk_kda_fwd(q, k, v, g, beta, float(scale), chunk_size, layout=layout, initial_state=initial_state,
                                 output_final_state=output_final_state, cu_seqlens=cu,
                                 use_gate_in_kernel=use_gate_in_kernel, A_log=A_log, dt_bias=dt_bias, safe_gate=safe_gate,
                                 lower_bound=lower_bound)
        return out[0], out[1]
    if chunk_size not in (64, 128):
        raise RuntimeError("chunk_kda: chunk_size must be 64 or 128.")
    # The chunk size tiles the same function.  The gradient kernels are built for 64-token tiles, as the reference's own
    # backward kernel is (npu_chunk_kda_bwd_intra, _aclnn_ctypes.py:1582-1584), so a differentiated call runs on them.
    chunk_size = 64
    if layout not in ("BSND", "BNSD", "TND", "NTD"):
        raise RuntimeError("chunk_kda: layout must be uppercase and one of BSND, BNSD, TND, NTD.")
    K, V = q.shape[-1], v.shape[-1]
    if K < 16 or K > 256 or K % 16 or V < 16 or V > 256 or V % 16:      # _aclnn_ctypes.py:1141
        raise RuntimeError("chunk_kda: K/V must be multiples of 16 with K,V <= 256.")
    gate_args = ()
    if use_gate_in_kernel:
        # the operator's own checks (_aclnn_ctypes.py:1150-1165), ahead of the choice of route: a call is accepted or
        # rejected alike whether or not it asks for gradients and whatever its head size
        HV = v.shape[{"BSND": 2, "BNSD": 1, "TND": 1, "NTD": 0}[layout]]
        if A_log is None or tuple(A_log.shape) != (HV,) or A_log.dtype != torch.float32:
            raise RuntimeError("chunk_kda: A_log must be float32 [HV] when use_gate_in_kernel=True.")
        if dt_bias is not None and (tuple(dt_bias.shape) != (HV * K,) or dt_bias.dtype != torch.float32):
            raise RuntimeError("chunk_kda: dt_bias must be float32 [HV*K].")
        if safe_gate and not (-5.0 <= lower_bound < 0.0):
            raise RuntimeError("chunk_kda: lower_bound must be in [-5, 0) for safe gate.")
        if (K, V) in ((64, 64), (64, 128), (128, 128)):
            # a built head size: the forward kernel activates the gate, kda_gate_bwd differentiates the activation
            gate_args = (A_log, dt_bias, bool(safe_gate), lower_bound)
        else:   # the activation as tensor operations ahead of the padding and the split below
            g = _kda_gate_activation(g, A_log, dt_bias, layout, safe_gate, lower_bound)
    if V > 128:
        # Value columns never mix: o[.., c] and the state column c depend on v[.., c] only.  Two passes over 128 columns
        # each share q, k, g and beta, whose gradients autograd adds up.
        parts = []
        for lo in (0, 128):
            h0 = None if initial_state is None else initial_state[..., lo:lo + 128].contiguous()
            parts.append(chunk_kda(q, k, v[..., lo:lo + 128], g, beta, scale, h0, output_final_state, cu_seqlens,
                                   layout=layout, chunk_size=chunk_size))
        o = torch.cat([parts[0][0], parts[1][0]], dim=-1)
        final = None if parts[0][1] is None else torch.cat([parts[0][1], parts[1][1]], dim=-1)
        return o, final
    global _KDA_FUNCTION
    if _KDA_FUNCTION is None:
        _KDA_FUNCTION = _kda_autograd_function()
    # The backward kernels are built for (K, V) in {(64,64), (64,128), (128,128)}, and (256,128) is composed from them
    # (chunk_kda_bwd).  Other admitted head sizes run on the next of these with zero channels appended (a zero q/k channel adds nothing to any product, a
    # zero v column yields zero columns of o and of the state); the padding is itself differentiable, so autograd
    # returns the gradients of the unpadded tensors.
    Kp = 64 if K <= 64 else (128 if K <= 128 else 256)
    Vp = 128 if Kp == 256 else (Kp if V <= Kp else 128)
    if (Kp, Vp) != (K, V):
        F = torch.nn.functional
        h0 = None if initial_state is None else F.pad(initial_state, (0, Vp - V, 0, Kp - K))
        o, final = _KDA_FUNCTION.apply(F.pad(q, (0, Kp - K)), F.pad(k, (0, Kp - K)), F.pad(v, (0, Vp - V)),
                                       F.pad(g, (0, Kp - K)), beta, float(scale), h0, output_final_state, cu, layout,
                                       chunk_size)
        return o[..., :V], (None if final is None else final[..., :K, :V])
    return _KDA_FUNCTION.apply(q, k, v, g, beta, float(scale), initial_state, output_final_state, cu, layout, chunk_size,
                               *gate_args)
