"""Public operator namespace: the names of ``fla_npu.ops.ascendc`` backed by HIP kernels.

Every operator is exported twice, as ``npu_<op>`` and ``<op>``
(torch_custom/fla_npu/fla_npu/ops/ascendc/__init__.py:28-50,426-431).  Operators
that write into an argument declare it in ``MUTATED_ARGUMENTS``; their wrapper
rejects tensors that require grad and bumps the autograd version counter after
the launch (:61-71,146-185).  Names of reference operators that this library
does not implement raise ``NotImplementedError`` when called.
"""
from __future__ import annotations

import functools
import inspect
from typing import Callable

from ._hip_ctypes import HIP_CTYPES_OPS, chunk_kda_fwd_noalloc, gdn_chunk_fwd, l2norm_bwd, l2norm_fwd

_REFERENCE_OPS = (
    "npu_fast_gelu_custom",
    "npu_fast_gelu_custom_backward",
    "npu_causal_conv1d",
    "npu_causal_conv1d_bwd",
    "npu_prepare_wy_repr_bwd_full",
    "npu_prepare_wy_repr_bwd",
    "npu_chunk_gated_delta_rule_bwd_dhu",
    "npu_chunk_bwd_dv_local",
    "npu_prepare_wy_repr_bwd_da",
    "npu_chunk_bwd_dqkwg",
    "npu_chunk_fwd_o",
    "npu_chunk_gated_delta_rule_fwd_h",
    "npu_recompute_w_u_fwd",
    "npu_recurrent_gated_delta_rule",
    "npu_chunk_local_cumsum",
    "npu_chunk_scaled_dot_kkt",
    "npu_chunk_scaled_dot_kkt_inverse",
    "npu_solve_tri",
    "npu_chunk_kda_fwd",
    "npu_chunk_kda_bwd_intra",
    "npu_kda_gate_cumsum",
    "npu_recurrent_kda",
)

# Operators that write into one of their arguments through the library (invisible to autograd), and, where the write
# depends on a flag, the test that says whether this call writes (ops/ascendc/__init__.py:61-71).
MUTATED_ARGUMENTS = {
    "causal_conv1d": ("conv_states",),
    "npu_causal_conv1d": ("conv_states",),
    "npu_recurrent_kda": ("initial_state",),
    "recurrent_gated_delta_rule": ("state",),
    "npu_recurrent_gated_delta_rule": ("state",),
}

MUTATION_PREDICATES = {
    "npu_recurrent_kda": lambda arguments: bool(arguments["inplace_final_state"]),
}


def _strip_npu_prefix(name: str) -> str:
    return name[4:] if name.startswith("npu_") else name


def _wrap_mutable_op(name: str, op: Callable) -> Callable:
    """Guard for an operator that overwrites arguments in place (contract of ops/ascendc/__init__.py:146-185):
    a tensor about to be overwritten must not require grad, and after the launch its autograd version counter is
    bumped so that graphs which saved it notice.  ``MUTATION_PREDICATES`` can switch the guard off per call."""
    declared = MUTATED_ARGUMENTS.get(name, ())
    if not declared:
        return op
    parameters = inspect.signature(op)
    writes_this_call = MUTATION_PREDICATES.get(name)

    @functools.wraps(op)
    def guarded(*args, **kwargs):
        import torch

        call = parameters.bind(*args, **kwargs)
        call.apply_defaults()
        written = declared if writes_this_call is None or writes_this_call(call.arguments) else ()
        targets = {arg: call.arguments[arg] for arg in written}
        blocked = [arg for arg, value in targets.items() if getattr(value, "requires_grad", False)]
        if blocked:
            raise RuntimeError(
                f"{name} mutates {', '.join(blocked)} in place through ctypes. Mutable state tensors "
                "must not require gradients; use a functional state API for training."
            )
        result = op(*args, **kwargs)
        touched = [value for value in targets.values() if isinstance(value, torch.Tensor)]
        if touched:
            torch.autograd.graph.increment_version(touched)
        return result

    return guarded


def _missing_op(name: str) -> Callable:
    def op(*args, **kwargs):
        raise NotImplementedError(
            f"fla_hip.ops.{name} is not implemented by this library (outside the accelerated path)."
        )

    op.__name__ = name
    op.__qualname__ = name
    return op


for _name in _REFERENCE_OPS:
    _op = HIP_CTYPES_OPS.get(_name)
    _op = _missing_op(_name) if _op is None else _wrap_mutable_op(_name, _op)
    globals()[_name] = _op
    globals()[_strip_npu_prefix(_name)] = _op


def _has_tensor_requiring_grad(*tensors) -> bool:
    import torch

    return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


def causal_conv1d(x, weight, bias=None, conv_states=None, *, query_start_loc=None, cache_indices=None,
                  initial_state_mode=None, num_accepted_tokens=None, activation_mode=0, pad_slot_id=-1,
                  run_mode=0, head_num=0):
    """Causal conv1d with automatic backward binding for prefill mode (ops/ascendc/__init__.py:299-392).

    ``conv_states`` is mutable state in every mode and must not require gradients.  The update / speculative
    modes stay on the raw operator; a dense prefill without activation binds gradients for ``x``, ``weight`` and
    ``bias`` through ``causal_conv1d_bwd``.  Any other call with inputs that require grad is rejected rather than
    silently detached."""
    import torch

    direct = globals()["npu_causal_conv1d"]
    kwargs = dict(query_start_loc=query_start_loc, cache_indices=cache_indices, initial_state_mode=initial_state_mode,
                  num_accepted_tokens=num_accepted_tokens, activation_mode=activation_mode, pad_slot_id=pad_slot_id,
                  run_mode=run_mode, head_num=head_num)
    if not _has_tensor_requiring_grad(x, weight, bias):
        return direct(x=x, weight=weight, bias=bias, conv_states=conv_states, **kwargs)
    can_bind_backward = (run_mode == 0 and activation_mode == 0 and query_start_loc is None and cache_indices is None
                         and initial_state_mode is None and num_accepted_tokens is None)
    if not can_bind_backward:
        raise NotImplementedError(
            "fla_hip.ops.causal_conv1d: gradients are bound only for a dense prefill without activation "
            "(run_mode=0, activation_mode=0, no query_start_loc / cache_indices / initial_state_mode); pass detached inputs.")
    bwd = globals()["npu_causal_conv1d_bwd"]

    class Function(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x_, weight_, bias_, conv_states_):
            y = direct(x=x_, weight=weight_, bias=bias_, conv_states=conv_states_, **kwargs)
            ctx.has_bias = bias_ is not None
            ctx.save_for_backward(x_, weight_)
            return y

        @staticmethod
        def backward(ctx, grad):
            x_, weight_ = ctx.saved_tensors
            layout = "BSH"
            if head_num > 0:           # the forward returned [B, head_num, S, D/head_num]
                layout = "BNSD"
            dx, dw, db, _ = bwd(x_, None, weight_, grad.contiguous(), None, None, query_start_loc=None, activation=0,
                                input_layout=layout)
            return dx, dw, (db if ctx.has_bias else None), None

    return Function.apply(x, weight, bias, conv_states)


__all__ = [
    "MUTATED_ARGUMENTS",
    "MUTATION_PREDICATES",
    "chunk_kda_fwd_noalloc",
    "gdn_chunk_fwd",
    "l2norm_bwd",
    "l2norm_fwd",
    *sorted(set(_REFERENCE_OPS)),
    *sorted({_strip_npu_prefix(n) for n in _REFERENCE_OPS}),
]
