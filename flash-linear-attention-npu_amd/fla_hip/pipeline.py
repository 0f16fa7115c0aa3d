"""Pipeline-level entry points: the gated-delta-rule chunk forward with the argument and
return layouts of examples/flash_gated_delta_rule.py:1126-1228 (``flash_gated_delta_rule``)
and :796-881 (``flash_chunk_gated_delta_rule_fwd``).

Two routes produce the same results:
* ``fused=True`` (default): one library call, ``fla_gdn_chunk_fwd``;
* ``fused=False``: the reference's own composition of the six operators
  (cumsum -> kkt -> solve_tri -> recompute_w_u -> fwd_h -> fwd_o), which also returns the
  inverted chunk matrix ``A``.
Forward only: inputs that require grad are rejected (the GDN backward operators are outside
this library).
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
                                     cu_seqlens=None, chunk_size: int = 64, *, fused: bool = True):
    """q,k,v [B,H,T,D] bf16; g,beta [B,T,H].  Returns (g_cumsum [B,T,H] f32, o [B,T,H,V], A, final_state);
    ``A`` ([B,H,T,C] bf16, the inverted chunk matrices) is None on the fused route."""
    import torch

    cu = _cu_list(cu_seqlens)
    if fused:
        gc, o, final = _raw.gdn_chunk_fwd(q, k, v, g.float(), beta.float(), scale, initial_state,
                                          output_final_state, cu, chunk_size)
        return gc, o, None, final
    # reference composition (examples/flash_gated_delta_rule.py:811-881)
    gh = _ops.chunk_local_cumsum(g.transpose(1, 2).contiguous(), chunk_size, cu_seqlens=cu,
                                 head_first=True, output_dtype=torch.float32)
    bh = beta.transpose(1, 2).contiguous().float()
    A = _ops.chunk_scaled_dot_kkt(k, gh, bh, cu_seqlens=cu, chunk_size=chunk_size)
    A = _ops.solve_tri(A.to(k.dtype), cu_seqlens=cu, layout="bnsd")
    w, u = _ops.recompute_w_u_fwd(k, v, bh, A, chunk_size, g=gh, cu_seqlens=cu)
    h, v_new, final = _ops.chunk_gated_delta_rule_fwd_h(
        k, w, u, g=gh, initial_state=initial_state, output_final_state=output_final_state,
        chunk_size=chunk_size, cu_seqlens=cu)
    o = _ops.chunk_fwd_o(q, k, v_new, h, scale, g=gh, cu_seqlens=cu, chunk_size=chunk_size)
    return gh.transpose(1, 2).contiguous(), o.transpose(1, 2).contiguous(), A, \
        (final if output_final_state else None)


def flash_gated_delta_rule(q, k, v, g, beta, scale: Optional[float] = None, initial_state=None,
                           output_final_state: bool = False, use_qk_l2norm_in_kernel: bool = False,
                           cu_seqlens=None, cu_seqlens_list=None, chunk_indices=None, chunk_indices_list=None,
                           chunk_size: int = 64, head_first: bool = False, *, fused: bool = True):
    """Same checks, defaults and layouts as the reference entry: q,k [B,H,T,K], v [B,H,T,V],
    g,beta [B,T,H]; returns (o [B,T,H,V], final_state [N,H,K,V] or None)."""
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
    if use_qk_l2norm_in_kernel:
        raise NotImplementedError("use_qk_l2norm_in_kernel is not implemented; pass normalised q and k.")
    if any(isinstance(t, torch.Tensor) and t.requires_grad for t in (q, k, v, g, beta)) and torch.is_grad_enabled():
        raise NotImplementedError("flash_gated_delta_rule: forward only; the GDN backward is not implemented.")
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
    _, o, _, final = flash_chunk_gated_delta_rule_fwd(
        q, k, v, g, beta, float(scale), initial_state, output_final_state, cu, chunk_size, fused=fused)
    return o, final
