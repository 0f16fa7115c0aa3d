"""Per-operator ctypes wrappers over ``libfla_hip.so``.

Each function keeps the name, positional / keyword structure, defaults, output
allocation and error text of its counterpart in
torch_custom/fla_npu/fla_npu/ops/ascendc/_aclnn_ctypes.py (line numbers in the
docstrings); only the device type (ROCm ``cuda`` tensors) and the C symbol
differ.  Argument order of every C call equals the aclnn prototype's.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional

from . import _runtime
from ._runtime import INT_ARRAY_P, TENSOR_P

_call_op = _runtime.call_op
_empty = _runtime.empty
_empty_like = _runtime.empty_like


def _empty_ordered_like(like, *, dtype=None, shape=None, device=None):
    """An uninitialised tensor of ``shape`` (default: that of ``like``) whose dimensions sit in memory in the order of
    ``like``'s.  For a contiguous ``like`` this is a contiguous tensor, as the reference's operators return; for a
    token-major view [B,H,T,D] (what a caller holds after ``x.transpose(1, 2)``) the result is such a view too, so that
    a gradient flows back through the transpose without a copy.  The kernels take outer strides either way."""
    import torch

    shape = tuple(like.shape) if shape is None else tuple(int(d) for d in shape)
    order = sorted(range(len(shape)), key=lambda d: (-like.stride(d), d))
    base = torch.empty([shape[d] for d in order], dtype=dtype or like.dtype, device=like.device if device is None else device)
    return base.permute([order.index(d) for d in range(len(shape))])


_shape = _runtime.shape

_T, _IA = TENSOR_P, INT_ARRAY_P

# C operand types of each operator, in prototype order (workspace / stream tail excluded).
OP_ARGTYPES = {
    "chunk_local_cumsum": [_T, _IA, _IA, ctypes.c_int64, ctypes.c_bool, ctypes.c_double, ctypes.c_bool,
                           ctypes.c_char_p, _T],
    "chunk_scaled_dot_kkt": [_T, _T, _T, _IA, _IA, ctypes.c_int64, _T],
    "chunk_scaled_dot_kkt_inverse": [_T, _T, _T, _IA, _IA, ctypes.c_int64, _T],
    "solve_tri": [_T, _IA, _IA, ctypes.c_char_p, _T],
    "recompute_w_u_fwd": [_T, _T, _T, _T, _T, _T, _IA, _IA, ctypes.c_int64, _T, _T],
    "chunk_gated_delta_rule_fwd_h": [_T, _T, _T, _T, _T, _T, ctypes.c_bool, ctypes.c_int64, _IA, _IA,
                                     ctypes.c_bool, _T, _T, _T],
    "chunk_fwd_o": [_T, _T, _T, _T, _T, _IA, _IA, ctypes.c_double, ctypes.c_int64, _T],
    "gdn_chunk_fwd": [_T, _T, _T, _T, _T, ctypes.c_double, _T, ctypes.c_bool, _IA, ctypes.c_int64, ctypes.c_bool,
                      _T, _T, _T, _T, _T, _T, _T, _T, _T, _T],
    "gdn_chunk_fwd_state_pool": [_T, _T, _T, _T, _T, ctypes.c_double, _T, _T, _IA, ctypes.c_int64, ctypes.c_bool, _T],
    "recurrent_gated_delta_rule": [_T, _T, _T, _T, _T, _T, _T, _T, _T, _T, ctypes.c_float, _T],
    "recurrent_gdn_prefill_plan": [_T, _T, ctypes.c_int64, _T, _T],
    "causal_conv1d": [_T, _T, _T, _T, _IA, _IA, _IA, _IA, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                      ctypes.c_int64, _T],
    "kda_gate_cumsum": [_T, _T, _T, _IA, ctypes.c_int64, ctypes.c_bool, ctypes.c_bool, ctypes.c_double, _T],
    "chunk_kda_fwd": [_T, _T, _T, _T, _T, _T, _T, _T, _IA, _IA, ctypes.c_char_p, ctypes.c_double, ctypes.c_int64,
                      ctypes.c_bool, ctypes.c_double, ctypes.c_bool, ctypes.c_bool] + [_T] * 11,
    "kda_gate_bwd": [_T, _T, _T, _T, ctypes.c_char_p, ctypes.c_bool, ctypes.c_double, _T, _T, _T],
    "chunk_kda_bwd_intra": [_T] * 10 + [_IA, _IA, ctypes.c_int64, ctypes.c_bool, ctypes.c_char_p] + [_T] * 4,
    "chunk_kda_bwd_intra_cumsum": [_T] * 10 + [_IA, _IA, ctypes.c_int64, ctypes.c_bool, ctypes.c_char_p] + [_T] * 4,
    "chunk_gated_delta_rule_bwd_dhu": [_T, _T, _T, _T, _T, _T, _T, _T, _T, _IA, _IA, ctypes.c_double, ctypes.c_int64,
                                       ctypes.c_bool, _T, _T, _T],
    "l2norm_fwd": [_T, ctypes.c_double, _T, _T],
    "l2norm_bwd": [_T, _T, _T, ctypes.c_double, _T],
    "recurrent_kda": [_T] * 11 + [ctypes.c_char_p, ctypes.c_double] + [ctypes.c_bool] * 7 + [ctypes.c_double, ctypes.c_bool, _T, _T],
    "causal_conv1d_bwd": [_T, _T, _T, _T, _T, _T, _IA, ctypes.c_int64, ctypes.c_char_p, _T, _T, _T, _T],
    "chunk_bwd_dv_local": [_T, _T, _T, _T, _T, _T, _IA, _IA, ctypes.c_double, ctypes.c_int64, _T],
    "chunk_bwd_dqkwg": [_T] * 8 + [_IA, _IA, _T, _T, ctypes.c_float, ctypes.c_int64, ctypes.c_bool, ctypes.c_bool]
                       + [_T] * 4,
    "prepare_wy_repr_bwd_da": [_T] * 7 + [_IA, _IA, ctypes.c_int64, _T],
    "prepare_wy_repr_bwd_full": [_T] * 8 + [_IA, _IA, ctypes.c_int64] + [_T] * 4,
    "prepare_wy_repr_bwd_full_accumulate": [_T] * 8 + [_IA, _IA, ctypes.c_int64] + [_T] * 5,
    "chunk_bwd_dqkwg_l2norm": [_T] * 8 + [_IA, _IA, _T, ctypes.c_float, ctypes.c_int64] + [_T] * 4,
    "prepare_wy_repr_bwd": [_T] * 7 + [_IA, _IA, ctypes.c_int64] + [_T] * 4,
    "chunk_kda_bwd_dav": [_T, _T, _T, _IA, _IA, ctypes.c_double, ctypes.c_int64, _T, _T],
    "chunk_kda_bwd_dqkwg": [_T] * 8 + [_IA, _IA, ctypes.c_double, ctypes.c_int64] + [_T] * 5,
    "chunk_kda_bwd_dhu": [_T] * 8 + [_IA, _IA, ctypes.c_double, ctypes.c_int64] + [_T] * 3,
    "chunk_kda_bwd_wy": [_T] * 7 + [_IA, _IA, ctypes.c_int64] + [_T] * 5,
    "chunk_kda_bwd_dqkwg_wy": [_T] * 11 + [_IA, _IA, ctypes.c_double, ctypes.c_int64] + [_T] * 7,
    "chunk_kda_bwd_dqkwg_wy_intra": [_T] * 11 + [_IA, _IA, ctypes.c_double, ctypes.c_int64] + [_T] * 5,
}


def _optional_int(value, default: int) -> int:
    return default if value is None else int(value)


def _optional_bool(value, default: bool) -> bool:
    return default if value is None else bool(value)


def _optional_float(value, default: float) -> float:
    return default if value is None else float(value)


def _as_int_tuple(values) -> Optional[tuple]:
    if values is None:
        return None
    import torch

    if isinstance(values, torch.Tensor):
        values = values.detach().cpu().flatten().tolist()
    return tuple(int(v) for v in values)


def _build_chunk_indices(cu: tuple, chunk_size: int) -> tuple:
    """Canonical sequence-major (seq, chunk) list; empty sequences own no chunk."""
    out = []
    for n, (s, e) in enumerate(zip(cu, cu[1:])):
        for c in range((e - s + chunk_size - 1) // chunk_size):
            out.extend((n, c))
    return tuple(out)


def _total_chunks(B: int, T: int, chunk_size: int, cu: Optional[tuple]) -> int:
    if cu is None:
        return (T + chunk_size - 1) // chunk_size
    return sum((e - s + chunk_size - 1) // chunk_size for s, e in zip(cu, cu[1:]))


# ---------------------------------------------------------------------------------------------
def npu_chunk_fwd_o(q, k, v, h, scale, *, g=None, g_gamma=None, cu_seqlens=None, chunk_indices=None,
                    chunk_size=None, transpose_state_layout=False, out_token_major=False):
    """_aclnn_ctypes.py:517-549.  ``g_gamma`` and ``transpose_state_layout`` are ignored there too.
    ``out_token_major`` (not in the reference): the [B,H,T,V] result is a view of [B,T,H,V] storage, so that the
    caller's ``o.transpose(1, 2)`` is contiguous without a copy (the kernel takes the strides of its output)."""
    del g_gamma, transpose_state_layout
    chunk_size = _optional_int(chunk_size, 64)
    if out_token_major:
        B, H, T, V = _shape(v)
        out = _empty((B, T, H, V), v).transpose(1, 2)
    else:
        out = _empty_like(v)
    return _call_op(
        "chunk_fwd_o", OP_ARGTYPES["chunk_fwd_o"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(h, "h"), ctx.tensor(g, "g"),
            ctx.int_array(cu_seqlens), ctx.int_array(chunk_indices),
            ctypes.c_double(float(scale)), ctypes.c_int64(chunk_size), ctx.tensor(out, "out"),
        ],
        out,
    )


def npu_chunk_gated_delta_rule_fwd_h(k, w, u, g=None, *, gk=None, initial_state=None, output_final_state=False,
                                     chunk_size=None, cu_seqlens=None, chunk_indices=None, state_v_first=False):
    """_aclnn_ctypes.py:552-615."""
    import torch

    op = "npu_chunk_gated_delta_rule_fwd_h"
    if (g, gk) == (None, None):
        raise RuntimeError(f"{op}: either g or gk must be provided.")
    want_final = _optional_bool(output_final_state, False)
    v_first = _optional_bool(state_v_first, False)
    chunk_size = _optional_int(chunk_size, 64)
    (B, _, T, K), (_, HV, _, V) = _shape(k), _shape(u)
    cu, indices = _as_int_tuple(cu_seqlens), _as_int_tuple(chunk_indices)
    if cu is not None and indices is None:
        indices = _build_chunk_indices(cu, chunk_size)
    NT = _total_chunks(B, T, chunk_size, cu)
    N = B if cu is None else len(cu) - 1
    block = (V, K) if v_first else (K, V)
    if initial_state is not None and _shape(initial_state) != (N, HV, *block):
        raise RuntimeError(f"{op}: initial_state shape does not match state_v_first.")
    h_out = _empty((B, HV, NT, *block), k)
    v_new_out = _empty_like(u)
    final_state_out = None
    if want_final:   # the carried state keeps the dtype of the state the caller supplied, fp32 otherwise
        final_state_out = _empty((N, HV, *block), k, dtype=torch.float32 if initial_state is None else initial_state.dtype)
    output_final_state, state_v_first = want_final, v_first
    outputs = (h_out, v_new_out, final_state_out)
    return _call_op(
        "chunk_gated_delta_rule_fwd_h", OP_ARGTYPES["chunk_gated_delta_rule_fwd_h"],
        lambda ctx: [
            ctx.tensor(k, "k"), ctx.tensor(w, "w"), ctx.tensor(u, "u"), ctx.tensor(g, "g"), ctx.tensor(gk, "gk"),
            ctx.tensor(initial_state, "initial_state"),
            ctypes.c_bool(output_final_state), ctypes.c_int64(chunk_size),
            ctx.int_array(cu), ctx.int_array(indices), ctypes.c_bool(state_v_first),
            ctx.tensor(h_out, "h"), ctx.tensor(v_new_out, "v_new"), ctx.tensor(final_state_out, "final_state"),
        ],
        outputs,
    )


def npu_recompute_w_u_fwd(k, v, beta, A, chunk_size, *, g=None, gk=None, cu_seqlens=None, chunk_indices=None):
    """_aclnn_ctypes.py:618-651."""
    w_shape = list(_shape(v))
    w_shape[3] = int(k.shape[3])
    w_out = _empty(w_shape, v, dtype=k.dtype)
    u_out = _empty_like(v)
    outputs = (w_out, u_out)
    return _call_op(
        "recompute_w_u_fwd", OP_ARGTYPES["recompute_w_u_fwd"],
        lambda ctx: [
            ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"), ctx.tensor(A, "A"),
            ctx.tensor(g, "g"), ctx.tensor(gk, "gk"),
            ctx.int_array(cu_seqlens), ctx.int_array(chunk_indices), ctypes.c_int64(int(chunk_size)),
            ctx.tensor(w_out, "w"), ctx.tensor(u_out, "u"),
        ],
        outputs,
    )


def npu_recurrent_gated_delta_rule(query, key, value, state, *, beta, scale=1.0, actual_seq_lengths,
                                   ssm_state_indices, num_accepted_tokens=None, g=None, gk=None):
    """Run recurrent GDN and update ``state`` in place (_aclnn_ctypes.py:654-846).

    ``g`` and ``gk`` are independent optional gates; one of them must be given.
    """
    op_name = "npu_recurrent_gated_delta_rule"
    if g is None and gk is None:
        raise RuntimeError(f"{op_name}: either g or gk must be provided.")

    import torch

    bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32
    # operand -> (value, required, accepted dtypes, rank); checked in this order: presence and type, device, dtype, rank
    spec = {
        "query": (query, True, (bf,), 3), "key": (key, True, (bf,), 3), "value": (value, True, (bf,), 3),
        "state": (state, True, (bf, f32), 4), "beta": (beta, True, (bf,), 2),
        "actual_seq_lengths": (actual_seq_lengths, True, (i32,), 1),
        "ssm_state_indices": (ssm_state_indices, True, (i32,), 1),
        "g": (g, False, (f32,), 2), "gk": (gk, False, (f32,), 3),
        "num_accepted_tokens": (num_accepted_tokens, False, (i32,), 1),
    }
    for name, (tensor, required, _, _) in spec.items():
        if tensor is None and not required:
            continue
        if not isinstance(tensor, torch.Tensor):
            shown = "None" if tensor is None else repr(type(tensor))
            raise TypeError(f"{op_name}: {name} must be a torch.Tensor, got {shown}.")
        if tensor.device.type != "cuda":
            raise TypeError(f"{op_name}: {name} must be a torch GPU tensor, got device {tensor.device}.")
    present = {name: entry for name, entry in spec.items() if entry[0] is not None}
    for name, (tensor, _, accepted, _) in present.items():
        if tensor.dtype not in accepted:
            listed = ", ".join(str(d) for d in accepted)
            raise TypeError(f"{op_name}: {name} dtype must be one of ({listed}), got {tensor.dtype}.")
    shapes = {name: _shape(entry[0]) for name, entry in present.items()}
    for name, (_, _, _, rank) in present.items():
        if len(shapes[name]) != rank:
            raise RuntimeError(f"{op_name}: {name} must be rank {rank}, got shape {shapes[name]}.")

    if shapes["query"] != shapes["key"]:
        raise RuntimeError(
            f"{op_name}: key shape must equal query shape, got query={shapes['query']}, key={shapes['key']}.")
    total_tokens, key_heads, key_dim = shapes["query"]
    value_tokens, value_heads, value_dim = shapes["value"]
    state_blocks = shapes["state"][0]
    for name, size in {"T": total_tokens, "Nk": key_heads, "Nv": value_heads, "Dk": key_dim, "Dv": value_dim,
                       "state blocks": state_blocks}.items():
        if size <= 0:
            raise RuntimeError(f"{op_name}: {name} must be positive, got {size}.")
    if value_tokens != total_tokens:
        raise RuntimeError(f"{op_name}: value T dimension must be {total_tokens}, got {value_tokens}.")
    if shapes["beta"] != (total_tokens, value_heads):
        raise RuntimeError(f"{op_name}: beta shape must be {(total_tokens, value_heads)}, got {shapes['beta']}.")
    expected_state = (state_blocks, value_heads, value_dim, key_dim)
    if shapes["state"] != expected_state:
        raise RuntimeError(f"{op_name}: state shape must be {expected_state}, got {shapes['state']}.")
    if shapes["actual_seq_lengths"][0] < 2:
        raise RuntimeError(
            f"{op_name}: actual_seq_lengths must contain the prefix entry and at least one sequence length.")
    if shapes["ssm_state_indices"] != (total_tokens,):
        raise RuntimeError(
            f"{op_name}: ssm_state_indices shape must be ({total_tokens},), got {shapes['ssm_state_indices']}.")
    batch_size = shapes["actual_seq_lengths"][0] - 1
    for name, expected in {"g": (total_tokens, value_heads), "gk": (total_tokens, value_heads, key_dim),
                           "num_accepted_tokens": (batch_size,)}.items():
        shp = shapes.get(name)
        if shp is not None and shp != expected:
            raise RuntimeError(f"{op_name}: {name} shape must be {expected}, got {shp}.")
    if key_heads > 256 or value_heads > 256 or key_dim > 512 or value_dim > 512:
        raise RuntimeError(
            f"{op_name}: Nk and Nv must be <= 256 and Dk and Dv must be <= 512, "
            f"got Nk={key_heads}, Nv={value_heads}, Dk={key_dim}, Dv={value_dim}.")
    if value_heads % key_heads != 0:
        raise RuntimeError(
            f"{op_name}: Nv must be an integer multiple of Nk, got Nv={value_heads}, Nk={key_heads}.")
    scale = _optional_float(scale, 1.0)
    if not math.isfinite(scale):
        raise ValueError(f"{op_name}: scale must be finite, got {scale}.")

    routed = _recurrent_prefill_on_chunk_kernels(query, key, value, state, beta, scale, actual_seq_lengths,
                                                 ssm_state_indices, num_accepted_tokens, g, gk)
    if routed is not None:
        return routed
    out = _empty_like(value)
    return _call_op(
        "recurrent_gated_delta_rule", OP_ARGTYPES["recurrent_gated_delta_rule"],
        lambda ctx: [
            ctx.tensor(query, "query"), ctx.tensor(key, "key"), ctx.tensor(value, "value"),
            ctx.tensor(beta, "beta"), ctx.tensor(state, "state"),
            ctx.tensor(actual_seq_lengths, "actual_seq_lengths"),
            ctx.tensor(ssm_state_indices, "ssm_state_indices"),
            ctx.tensor(g, "g"), ctx.tensor(gk, "gk"), ctx.tensor(num_accepted_tokens, "num_accepted_tokens"),
            ctypes.c_float(scale), ctx.tensor(out, "out"),
        ],
        out,
    )


# A call of recurrent_gated_delta_rule with this many tokens per sequence on average is looked at as a prefill (the
# reference operator stops at 8 tokens per sequence, recurrent_gated_delta_rule.h:28,168-170); a prefill whose longest
# sequence has at least PREFILL_MIN_TOKENS tokens runs on the chunk kernels.
PREFILL_AVERAGE_TOKENS = 32
PREFILL_MIN_TOKENS = 64


def _recurrent_prefill_on_chunk_kernels(query, key, value, state, beta, scale, actual_seq_lengths, ssm_state_indices,
                                        num_accepted_tokens, g, gk):
    """Long sequences of ``recurrent_gated_delta_rule`` on the fused chunk forward (``gdn_chunk_fwd``) instead of the
    token-by-token kernel, whose time is the latency of the longest sequence.  Returns ``out`` with ``state`` updated
    in place, or None when the call stays on the token-by-token kernel: few tokens per sequence (decode and
    speculative decoding), a key-wise gate, accepted-token counts, a head size the chunk kernel is not built for,
    slots that change inside a sequence or are shared between sequences (then the state after EVERY token is part of
    the contract; here only the state after a sequence's last token is written, to that sequence's slot), or a stream
    under capture (the sequence lengths are read on the host, one synchronising copy)."""
    import torch

    total, nk, dk = _shape(query)
    _, nv, dv = _shape(value)
    batch = _shape(actual_seq_lengths)[0] - 1
    if g is None or gk is not None or num_accepted_tokens is not None:
        return None
    if total < PREFILL_AVERAGE_TOKENS * batch or dk not in (64, 128) or dv % 64 != 0 or dv > 256:
        return None
    if any(t.stride(-1) != 1 for t in (query, key, value)) or state.stride(-1) != 1 or torch.cuda.is_current_stream_capturing():
        return None
    # The plan is formed on the device by one launch and read with ONE synchronising copy: the sequence lengths and, per
    # sequence, a flag that says whether every token names the pool row of the first token, whether that row is valid
    # and whether no other sequence names it.
    dev, blocks = query.device, _shape(state)[0]
    if batch > 8192:
        return None
    lens_d = actual_seq_lengths.to(torch.int32).contiguous()
    idx_d = ssm_state_indices.to(torch.int32).contiguous()
    slots = torch.empty(batch, dtype=torch.int32, device=dev)
    report = torch.empty(2 * batch + 1, dtype=torch.int32, device=dev)
    _runtime.call_op_noalloc(
        "recurrent_gdn_prefill_plan", OP_ARGTYPES["recurrent_gdn_prefill_plan"],
        lambda ctx: [ctx.tensor(lens_d, "actual_seq_lengths"), ctx.tensor(idx_d, "ssm_state_indices"),
                     ctypes.c_int64(int(blocks)), ctx.tensor(slots, "slots"), ctx.tensor(report, "report")],
        (slots, report),
    )
    plan = report.tolist()
    skip, lens, flags = plan[0], plan[1:1 + batch], plan[1 + batch:]
    if any(flags) or skip < 0 or max(lens) < PREFILL_MIN_TOKENS:
        return None
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    at = skip + cu[-1]
    head_major = lambda t: t[skip:at].transpose(0, 1)[None]            # [T,H,D] -> [1,H,T,D] view, nothing copied
    qh, kh, vh = head_major(query), head_major(key), head_major(value)
    gate, bet = g[skip:at][None], beta[skip:at][None].float()
    if state.dtype == torch.float32 and state.stride(-2) == dk and state.stride(0) >= 0 and state.stride(1) >= 0:
        # the chunk forward reads each sequence's pool row before its first token and writes it after its last one
        o = gdn_chunk_fwd_state_pool(qh, kh, vh, gate, bet, scale, state.transpose(-1, -2), slots, cu, 64)
    else:
        rows = slots.to(torch.int64).clamp(min=0)
        h0 = state.transpose(-1, -2)[rows].float().contiguous()       # V-first pool rows -> [N,H,K,V] fp32
        _, o, final = gdn_chunk_fwd(qh, kh, vh, gate, bet, scale, h0, True, cu, 64)
        live = torch.tensor([i for i, n in enumerate(lens) if n > 0], dtype=torch.int64, device=dev)   # an empty sequence names no row
        state[rows[live]] = final[live].transpose(-1, -2).to(state.dtype)
    if skip == 0 and at == total:
        return o[0]
    out = torch.zeros_like(value)
    out[skip:at] = o[0]
    return out


def gdn_chunk_fwd_state_pool(q, k, v, g, beta, scale, state_pool, state_indices, cu_seqlens, chunk_size=64,
                             use_qk_l2norm_in_kernel=False):
    """``gdn_chunk_fwd`` whose initial and final states are rows of ``state_pool`` (fp32 [rows,H,K,V] as a view with
    contiguous K x V or V x K blocks), row ``state_indices[n]`` (int32, on the device) for sequence n: read before the
    sequence's first token, overwritten after its last one; a negative index means no row.  Returns o [B,T,H,V]."""
    B, _, T, _ = _shape(k)
    _, HV, _, V = _shape(v)
    o = _empty((B, T, HV, V), v)
    cu = _as_int_tuple(cu_seqlens)
    _call_op(
        "gdn_chunk_fwd_state_pool", OP_ARGTYPES["gdn_chunk_fwd_state_pool"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(g, "g"), ctx.tensor(beta, "beta"),
            ctypes.c_double(float(scale)), ctx.tensor(state_pool, "state_pool"), ctx.tensor(state_indices, "state_indices"),
            ctx.int_array(cu), ctypes.c_int64(int(chunk_size)), ctypes.c_bool(bool(use_qk_l2norm_in_kernel)), ctx.tensor(o, "o"),
        ],
        (o,),
    )
    return o


def _chunk_local_cumsum_output_dtype(g, output_dtype):
    """Name handed to the library and torch dtype of the output; accepted spellings as in _aclnn_ctypes.py:849-872
    (a torch dtype, its name with or without ``torch.``, the short forms, or same / input / none for g's dtype)."""
    import torch

    names = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}
    aliases = {"float": "float32", "half": "float16", "bf16": "bfloat16"}
    if output_dtype is None:
        return "float32", torch.float32
    key = str(output_dtype).removeprefix("torch.").lower()
    key = aliases.get(key, key)
    if key in names:
        return key, names[key]
    if key in ("same", "input", "none") and not isinstance(output_dtype, torch.dtype):
        return key, g.dtype
    raise TypeError(f"Unsupported chunk_local_cumsum output_dtype: {output_dtype}.")


def npu_chunk_local_cumsum(g, chunk_size, *, cu_seqlens=None, chunk_indices_out=None, reverse=False, scale=1.0,
                           head_first=True, output_dtype="float32"):
    """_aclnn_ctypes.py:875-904."""
    output_dtype_name, out_dtype = _chunk_local_cumsum_output_dtype(g, output_dtype)
    g_contig = g.contiguous()
    out = _empty(_shape(g_contig), g_contig, dtype=out_dtype)
    name_buf = ctypes.create_string_buffer(output_dtype_name.encode("utf-8"))
    return _call_op(
        "chunk_local_cumsum", OP_ARGTYPES["chunk_local_cumsum"],
        lambda ctx: [
            ctx.tensor(g_contig, "g"), ctx.int_array(cu_seqlens), ctx.int_array(chunk_indices_out),
            ctypes.c_int64(int(chunk_size)), ctypes.c_bool(bool(reverse)), ctypes.c_double(float(scale)),
            ctypes.c_bool(bool(head_first)), ctypes.cast(name_buf, ctypes.c_char_p), ctx.tensor(out, "out"),
        ],
        out,
    )


def npu_chunk_scaled_dot_kkt(k, g, beta, *, cu_seqlens=None, chunk_indices=None, chunk_size=64):
    """_aclnn_ctypes.py:907-936."""
    import torch

    k_contig, g_contig, beta_contig = k.contiguous(), g.contiguous(), beta.contiguous()
    B, _, T, _ = _shape(k_contig)
    _, Hv, _ = _shape(g_contig)
    out = _empty((B, Hv, T, int(chunk_size)), k_contig, dtype=torch.float32)
    return _call_op(
        "chunk_scaled_dot_kkt", OP_ARGTYPES["chunk_scaled_dot_kkt"],
        lambda ctx: [
            ctx.tensor(k_contig, "k"), ctx.tensor(g_contig, "g"), ctx.tensor(beta_contig, "beta"),
            ctx.int_array(cu_seqlens), ctx.int_array(chunk_indices), ctypes.c_int64(int(chunk_size)),
            ctx.tensor(out, "out"),
        ],
        out,
    )


def npu_chunk_scaled_dot_kkt_inverse(k, g, beta, *, cu_seqlens=None, chunk_indices=None, chunk_size=64):
    """``solve_tri(chunk_scaled_dot_kkt(k, g, beta), output_dtype=k.dtype)`` in one launch (no reference counterpart;
    the backward's recompute calls it).  Returns (I + A)^-1 as [B,Hv,T,64] in k's dtype; 64-token chunks only."""
    k_contig, g_contig, beta_contig = k, g, beta   # the library takes the outer strides of all three: no copies
    B, _, T, _ = _shape(k_contig)
    _, Hv, _ = _shape(g_contig)
    out = _empty((B, Hv, T, int(chunk_size)), k_contig)
    return _call_op(
        "chunk_scaled_dot_kkt_inverse", OP_ARGTYPES["chunk_scaled_dot_kkt_inverse"],
        lambda ctx: [
            ctx.tensor(k_contig, "k"), ctx.tensor(g_contig, "g"), ctx.tensor(beta_contig, "beta"),
            ctx.int_array(cu_seqlens), ctx.int_array(chunk_indices), ctypes.c_int64(int(chunk_size)),
            ctx.tensor(out, "out"),
        ],
        out,
    )


def _infer_causal_conv1d_y(x, head_num: int, run_mode: int):
    """_aclnn_ctypes.py:939-948."""
    if run_mode == 0 and head_num > 0:
        if x.dim() == 3:
            b, s, d_model = _shape(x)
            return _empty((b, head_num, s, d_model // head_num), x)
        if x.dim() == 2:
            s, d_model = _shape(x)
            return _empty((head_num, s, d_model // head_num), x)
    return _empty_like(x)


def npu_causal_conv1d(x, weight, bias=None, conv_states=None, *, query_start_loc=None, cache_indices=None,
                      initial_state_mode=None, num_accepted_tokens=None, activation_mode=0, pad_slot_id=-1,
                      run_mode=0, head_num=0):
    """_aclnn_ctypes.py:951-985."""
    out = _infer_causal_conv1d_y(x, int(head_num), int(run_mode))
    return _call_op(
        "causal_conv1d", OP_ARGTYPES["causal_conv1d"],
        lambda ctx: [
            ctx.tensor(x, "x"), ctx.tensor(weight, "weight"), ctx.tensor(bias, "bias"),
            ctx.tensor(conv_states, "conv_states"),
            ctx.int_array(query_start_loc), ctx.int_array(cache_indices), ctx.int_array(initial_state_mode),
            ctx.int_array(num_accepted_tokens),
            ctypes.c_int64(int(activation_mode)), ctypes.c_int64(int(pad_slot_id)), ctypes.c_int64(int(run_mode)),
            ctypes.c_int64(int(head_num)), ctx.tensor(out, "out"),
        ],
        out,
    )


def npu_solve_tri(x, *, cu_seqlens=None, chunk_indices=None, layout="bsnd", output_dtype=None):
    """_aclnn_ctypes.py:1786-1800.  Beyond the reference: ``x`` may be float32 with ``output_dtype`` bf16/fp16; the
    kernel then rounds x to that dtype as it loads it (the cast the caller would otherwise run as its own pass)."""
    x_contig = x.contiguous()
    out = _empty_like(x_contig) if output_dtype is None else _empty(_shape(x_contig), x_contig, dtype=output_dtype)
    layout_arg = ctypes.c_char_p(str(layout).encode("utf-8"))
    return _call_op(
        "solve_tri", OP_ARGTYPES["solve_tri"],
        lambda ctx: [
            ctx.tensor(x_contig, "x"), ctx.int_array(cu_seqlens), ctx.int_array(chunk_indices), layout_arg,
            ctx.tensor(out, "out"),
        ],
        out,
    )


def gdn_chunk_fwd(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, chunk_size,
                  use_qk_l2norm_in_kernel=False, *, save_for_backward=False):
    """Whole chunk forward in one library call (replaces the composition at
    examples/flash_gated_delta_rule.py:796-881).  q,k,v [B,H,T,D]; g,beta [B,T,H] f32.
    use_qk_l2norm_in_kernel normalises q and k rows inside the kernel (flash_gated_delta_rule.py:1047-1049).
    Returns (g_cumsum [B,T,H] f32, o [B,T,H,V], final_state or None); with ``save_for_backward`` also
    (h [B,HV,NT,K,V], v_new [B,HV,T,V], w [B,HV,T,K]), the operands the reference's backward recomputes
    (flash_gated_delta_rule.py:913-951), and with both flags further (q_normalised, k_normalised, q_rstd, k_rstd):
    what ``l2norm_fwd`` hands its backward (flash_gated_delta_rule.py:1086-1089), in the memory order of q and k."""
    import torch

    B, _, T, K = _shape(k)
    _, HV, _, V = _shape(v)
    cu = _as_int_tuple(cu_seqlens)
    N = len(cu) - 1 if cu is not None else B
    o = _empty((B, T, HV, V), v)
    g_out = _empty((B, T, HV), v, dtype=torch.float32)
    final = _empty((N, HV, K, V), v, dtype=torch.float32) if output_final_state else None
    h = v_new = w = qn = kn = q_rstd = k_rstd = None
    if save_for_backward:
        C = 64
        NT = -(-T // C) if cu is None else sum(-(-(cu[i + 1] - cu[i]) // C) for i in range(N))
        h = _empty((B, HV, NT, K, V), v)
        v_new = _empty((B, HV, T, V), v)
        w = _empty((B, HV, T, K), v)
        if use_qk_l2norm_in_kernel:
            qn, kn = _empty_ordered_like(q), _empty_ordered_like(k)
            q_rstd = _empty(_shape(q)[:-1], q, dtype=torch.float32)
            k_rstd = _empty(_shape(k)[:-1], k, dtype=torch.float32)
    _call_op(
        "gdn_chunk_fwd", OP_ARGTYPES["gdn_chunk_fwd"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(g, "g"),
            ctx.tensor(beta, "beta"), ctypes.c_double(float(scale)), ctx.tensor(initial_state, "initial_state"),
            ctypes.c_bool(bool(output_final_state)), ctx.int_array(cu), ctypes.c_int64(int(chunk_size)),
            ctypes.c_bool(bool(use_qk_l2norm_in_kernel)),
            ctx.tensor(o, "o"), ctx.tensor(g_out, "g_cumsum"), ctx.tensor(final, "final_state"),
            ctx.tensor(h, "h"), ctx.tensor(v_new, "v_new"), ctx.tensor(w, "w"),
            ctx.tensor(qn, "q_normalised"), ctx.tensor(kn, "k_normalised"),
            ctx.tensor(q_rstd, "q_rstd"), ctx.tensor(k_rstd, "k_rstd"),
        ],
        (o, g_out, final),
    )
    if save_for_backward and use_qk_l2norm_in_kernel:
        return g_out, o, final, h, v_new, w, qn, kn, q_rstd, k_rstd
    if save_for_backward:
        return g_out, o, final, h, v_new, w
    return g_out, o, final


def npu_kda_gate_cumsum(g, chunk_size, *, A_log=None, dt_bias=None, cu_seqlens=None, use_gate_in_kernel=False,
                        safe_gate=False, lower_bound=None):
    """_aclnn_ctypes.py:1268-1296.  ``g [B,Hv,T,K]`` -> ``gk`` fp32, chunk-local cumsum in log2 units."""
    import torch

    out = _empty(_shape(g), g, dtype=torch.float32)
    return _call_op(
        "kda_gate_cumsum", OP_ARGTYPES["kda_gate_cumsum"],
        lambda ctx: [
            ctx.tensor(g, "g"), ctx.tensor(A_log, "A_log"), ctx.tensor(dt_bias, "dt_bias"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctypes.c_int64(int(chunk_size)),
            ctypes.c_bool(_optional_bool(use_gate_in_kernel, False)), ctypes.c_bool(_optional_bool(safe_gate, False)),
            ctypes.c_double(_optional_float(lower_bound, -5.0)), ctx.tensor(out, "gk"),
        ],
        out,
    )


def npu_chunk_gated_delta_rule_bwd_dhu(q, k, w, d_o, dv, scale, chunk_size, *, g=None, gK=None, h0=None, dht=None,
                                       cu_seqlens=None, chunk_indices=None, use_exp2=False,
                                       transpose_state_layout=False, dh0_per_sequence=False):
    """_aclnn_ctypes.py:324-394.  Returns ``(dh, dh0, dv2)``; ``dh0`` is allocated only when ``h0`` is given.

    ``dh0_per_sequence=True`` (an extension) returns ``dh0`` as fp32 ``[N,Hv,K,V]`` instead of the
    reference's bf16 ``[B,Hv,NT,K,V]`` buffer whose first chunk of each sequence holds the value.
    ``dht`` (fp32 ``[N,Hv,K,V]``) seeds the scan; the reference accepts and ignores it.
    ``dv=None`` (an extension; scalar gate, 64-token chunks): the scan forms the intra-chunk part of dv itself, what
    ``chunk_bwd_dv_local`` would have been called for, from the q, k and d_o tiles it holds anyway.
    """
    import torch

    B, _, T, K = _shape(q)
    _, Hv, _, V = _shape(d_o)
    gates = {"g": (g, (B, Hv, T)), "gK": (gK, (B, Hv, T, K))}
    given = [name for name, (t, _) in gates.items() if t is not None]
    if len(given) != 1:
        raise ValueError("Exactly one of g and gK must be provided.")
    if given == ["gK"] and not _optional_bool(use_exp2, True):
        raise ValueError("use_exp2 must be true when gK is provided.")
    if {t.dtype for t in (k, w, d_o) + (() if dv is None else (dv,))} != {q.dtype}:
        raise ValueError("q, k, w, d_o and dv must have the same dtype.")
    gate, gate_shape = gates[given[0]]
    if gate.dtype not in (q.dtype, torch.float32):
        raise ValueError("g or gK must be float32 or have the same dtype as q and k.")
    if _shape(gate) != gate_shape:
        raise ValueError(f"{given[0]} must have shape {gate_shape}, got {_shape(gate)}.")
    chunk_size = int(chunk_size)
    cu = _as_int_tuple(cu_seqlens)
    indices = _as_int_tuple(chunk_indices)
    if indices is None and cu is not None:
        indices = _build_chunk_indices(cu, chunk_size)
    NT = _total_chunks(B, T, chunk_size, cu) if indices is None else len(indices) // 2
    N = len(cu) - 1 if cu is not None else B
    dh = _empty((B, Hv, NT, K, V), q)
    if h0 is None:
        dh0 = None
    elif dh0_per_sequence:
        dh0 = _empty((N, Hv, K, V), q, dtype=torch.float32)
    else:
        dh0 = _empty((B, Hv, NT, K, V), q)
    dv2 = _empty_ordered_like(d_o) if dv is None else _empty_like(dv)
    outputs = (dh, dh0, dv2)
    return _call_op(
        "chunk_gated_delta_rule_bwd_dhu", OP_ARGTYPES["chunk_gated_delta_rule_bwd_dhu"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(w, "w"), ctx.tensor(d_o, "d_o"), ctx.tensor(dv, "dv"),
            ctx.tensor(g, "g"), ctx.tensor(gK, "gK"), ctx.tensor(h0, "h0"), ctx.tensor(dht, "dht"),
            ctx.int_array(cu), ctx.int_array(indices), ctypes.c_double(float(scale)), ctypes.c_int64(chunk_size),
            ctypes.c_bool(_optional_bool(use_exp2, gK is not None)),
            ctx.tensor(dh, "dh"), ctx.tensor(dh0, "dh0"), ctx.tensor(dv2, "dv2"),
        ],
        outputs,
    )


def kda_fwd_optional_output_mask(*, output_final_state, use_gate_in_kernel, disable_recompute,
                                 return_intermediate_states):
    """Which of the 12 values of ``npu_chunk_kda_fwd`` are materialised
    (ops/ascendc/_kda_policy.py:16-39): o, final_state, gk, Aqk, Akk, w, u, qg, kg, v_new, h, initial_state."""
    keep = bool(disable_recompute)
    return (True, bool(output_final_state), (not use_gate_in_kernel) or keep, True, True, keep, keep, keep, keep, keep,
            keep or bool(return_intermediate_states), True)


def npu_chunk_kda_fwd(q, k, v, g, beta, scale, chunk_size=64, *, layout="BSND", initial_state=None,
                      output_final_state=False, cu_seqlens=None, chunk_indices=None, safe_gate=False, lower_bound=None,
                      use_gate_in_kernel=False, A_log=None, dt_bias=None, disable_recompute=False,
                      return_intermediate_states=False, state_v_first=False):
    """KDA chunk forward (_aclnn_ctypes.py:1066-1265).  Returns the 12-tuple
    ``(o, final_state, gk, Aqk, Akk, w, u, qg, kg, v_new, h, initial_state)``; entries the output policy
    hides are ``None``."""
    return _chunk_kda_fwd(False, q, k, v, g, beta, scale, chunk_size, layout, initial_state, output_final_state,
                          cu_seqlens, chunk_indices, safe_gate, lower_bound, use_gate_in_kernel, A_log, dt_bias,
                          disable_recompute, return_intermediate_states, state_v_first)


def chunk_kda_fwd_noalloc(q, k, v, g, beta, scale, chunk_size=64, *, layout="BSND", initial_state=None,
                          output_final_state=False, safe_gate=False, lower_bound=None, use_gate_in_kernel=False,
                          A_log=None, dt_bias=None, disable_recompute=False, return_intermediate_states=False,
                          state_v_first=False):
    """``npu_chunk_kda_fwd`` through ``fla_chunk_kda_fwd_noalloc``: the library call allocates nothing and takes
    no workspace (its scratch is a fixed array of 32 MiB per GPU; dense batches only).  This wrapper still
    allocates the OUTPUT tensors with torch, as every wrapper here does; a caller that must not allocate at all
    binds the C entry point with preallocated outputs.  Calls that overlap on one GPU race on the scratch array."""
    return _chunk_kda_fwd(True, q, k, v, g, beta, scale, chunk_size, layout, initial_state, output_final_state,
                          None, None, safe_gate, lower_bound, use_gate_in_kernel, A_log, dt_bias,
                          disable_recompute, return_intermediate_states, state_v_first)


def chunk_kda_fwd_for_backward(q, k, v, g, beta, scale, chunk_size=64, *, layout="BSND", initial_state=None,
                               output_final_state=False, cu_seqlens=None, safe_gate=False, lower_bound=None,
                               use_gate_in_kernel=False, A_log=None, dt_bias=None):
    """``npu_chunk_kda_fwd`` keeping every intermediate, as the forward of a training step: the same 12-tuple, except
    that ``u`` is None (no stage of the backward reads it) and that ``qg`` and ``kg`` are float16 tensors also when q is
    bfloat16 (head sizes up to 128 channels).  They only
    serve the reverse scan ``chunk_kda_bwd_dhu``, whose q^T d_o product carries the leading term of the state gradient:
    rounded to 8 significand bits they move dh0 by 3e-3 of its scale, to 11 bits by 5e-4.  No counterpart in the
    reference, whose backward is a third-party package."""
    return _chunk_kda_fwd(False, q, k, v, g, beta, scale, chunk_size, layout, initial_state, output_final_state,
                          cu_seqlens, None, safe_gate, lower_bound, use_gate_in_kernel, A_log, dt_bias, True, True, False,
                          fine_qk=True)


def _chunk_kda_fwd(noalloc, q, k, v, g, beta, scale, chunk_size, layout, initial_state, output_final_state, cu_seqlens,
                   chunk_indices, safe_gate, lower_bound, use_gate_in_kernel, A_log, dt_bias, disable_recompute,
                   return_intermediate_states, state_v_first, fine_qk=False):
    import torch

    op = "npu_chunk_kda_fwd"
    layout = str(layout)
    if layout not in {"BSND", "BNSD", "TND", "NTD"}:
        raise RuntimeError(f"{op}: layout must be uppercase and one of BSND, BNSD, TND, NTD.")
    chunk_size = int(chunk_size)
    if chunk_size not in {64, 128}:
        raise RuntimeError(f"{op}: chunk_size must be 64 or 128.")
    rank3 = layout in {"TND", "NTD"}
    shapes = [_shape(t) for t in (q, k, v, g, beta)]
    qs, ks, vs, gs, bs = shapes
    rank = 3 if rank3 else 4
    if any(len(s) != rank for s in (qs, ks, vs, gs)):
        raise RuntimeError(f"{op}: q/k/v/g rank does not match layout.")
    if len(bs) != rank - 1 or qs != ks:
        raise RuntimeError(f"{op}: beta rank must match layout and q/k shapes must be identical.")
    t_dim, h_dim = {"BSND": (1, 2), "BNSD": (2, 1), "TND": (0, 1), "NTD": (1, 0)}[layout]
    B = 1 if rank3 else qs[0]
    T, H, K = qs[t_dim], qs[h_dim], qs[-1]
    HV, V = vs[h_dim], vs[-1]

    def in_layout(heads, *tail):
        dims = [None] * (rank - 1)
        dims[t_dim], dims[h_dim] = T, heads
        if not rank3:
            dims[0] = B
        return (*dims, *tail)

    if vs != in_layout(HV, V) or gs != in_layout(HV, K) or bs != in_layout(HV):
        raise RuntimeError(f"{op}: v/g/beta shapes do not match the selected layout.")
    if H <= 0 or HV < H or HV % H != 0 or H > 128 or HV > 128:
        raise RuntimeError(f"{op}: H/HV must satisfy 0 < H <= HV <= 128 and HV % H == 0.")
    if q.dtype not in {torch.float16, torch.bfloat16} or k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError(f"{op}: q/k/v must use the same float16 or bfloat16 dtype.")
    if g.dtype not in {torch.float32, torch.bfloat16} or beta.dtype not in {torch.float32, torch.bfloat16}:
        raise RuntimeError(f"{op}: g and beta must be float32 or bfloat16.")
    if K < 16 or K > 256 or K % 16 or V < 16 or V > 256 or V % 16:
        raise RuntimeError(f"{op}: K/V must be multiples of 16 with K,V <= 256.")
    use_gate_in_kernel = _optional_bool(use_gate_in_kernel, False)
    safe_gate = _optional_bool(safe_gate, False)
    disable_recompute = _optional_bool(disable_recompute, False)
    return_intermediate_states = _optional_bool(return_intermediate_states, False)
    output_final_state = _optional_bool(output_final_state, False)
    state_v_first = _optional_bool(state_v_first, False)
    if use_gate_in_kernel:
        if A_log is None or _shape(A_log) != (HV,) or A_log.dtype != torch.float32:
            raise RuntimeError(f"{op}: A_log must be float32 [HV] when use_gate_in_kernel=True.")
        if dt_bias is not None and (_shape(dt_bias) != (HV * K,) or dt_bias.dtype != torch.float32):
            raise RuntimeError(f"{op}: dt_bias must be float32 [HV*K].")
    lower_bound = _optional_float(lower_bound, -5.0)
    if use_gate_in_kernel and safe_gate and not (-5.0 <= lower_bound < 0.0):
        raise RuntimeError(f"{op}: lower_bound must be in [-5, 0) for safe gate.")
    cu = _as_int_tuple(cu_seqlens)
    if cu is not None:
        if len(cu) < 2 or cu[0] != 0 or cu[-1] != T or any(a > b for a, b in zip(cu, cu[1:])):
            raise RuntimeError(f"{op}: cu_seqlens must be nondecreasing, start at 0 and end at T.")
        if len(cu) - 1 > 1024:
            raise RuntimeError(f"{op}: varlen input supports at most 1024 sequences.")
        if not rank3 and B != 1:
            raise RuntimeError(f"{op}: rank4 varlen input requires B=1.")
    N = len(cu) - 1 if cu is not None else B
    canonical = None if cu is None else _build_chunk_indices(cu, chunk_size)
    indices = canonical if chunk_indices is None else _as_int_tuple(chunk_indices)
    if indices is not None and indices != canonical:
        raise RuntimeError(f"{op}: chunk_indices must use canonical sequence-major order.")
    NT = _total_chunks(B, T, chunk_size, cu)
    state_shape = (N, HV, V, K) if state_v_first else (N, HV, K, V)
    if initial_state is not None and (_shape(initial_state) != state_shape or initial_state.dtype != torch.float32):
        raise RuntimeError(f"{op}: initial_state shape/dtype does not match state_v_first.")

    # The kernels are built for K in {64, 128} with V in {K, 2K} and for K = V = 256.  Every other admitted head size runs
    # on the next built size with zero channels appended: a zero q/k channel adds nothing to any product and a zero v
    # column yields zero u, v_new, o and state columns, so the leading K x V part of every result is unchanged.
    if K > 128:
        Kp = Vp = 256
    else:
        Kp = 64 if K <= 64 and V <= 128 else 128
        Vp = Kp if V <= Kp else 2 * Kp
    if (Kp, Vp) != (K, V):
        if noalloc:
            raise NotImplementedError(f"{op}: (K,V)=({K},{V}) needs padded copies; the no-allocation entry takes "
                                      "K in {64,128} with V in {K,2K} and K = V = 256 only.")
        F = torch.nn.functional
        padk = lambda t: F.pad(t, (0, Kp - K))
        padv = lambda t: F.pad(t, (0, Vp - V))
        state_pad = (0, Kp - K, 0, Vp - V) if state_v_first else (0, Vp - V, 0, Kp - K)
        bias = None if dt_bias is None else padk(dt_bias.view(HV, K)).reshape(-1)
        h0 = None if initial_state is None else F.pad(initial_state, state_pad)
        res = _chunk_kda_fwd(noalloc, padk(q), padk(k), padv(v), padk(g), beta, scale, chunk_size, layout, h0,
                             output_final_state, cu_seqlens, chunk_indices, safe_gate, lower_bound, use_gate_in_kernel, A_log,
                             bias, disable_recompute, return_intermediate_states, state_v_first, fine_qk=fine_qk)
        attn_out, final_state, gk, aqk, akk, w, u, qg, kg, v_new, h = res[:11]
        cut = lambda t, n: None if t is None else t[..., :n].contiguous()
        cut2 = lambda t: None if t is None else \
            (t[..., :V, :K] if state_v_first else t[..., :K, :V]).contiguous()
        return (cut(attn_out, V), cut2(final_state), cut(gk, K), aqk, akk, cut(w, K), cut(u, V), cut(qg, K), cut(kg, K),
                cut(v_new, V), cut2(h), initial_state)

    lead = () if rank3 else (B,)
    block = (V, K) if state_v_first else (K, V)
    mask = kda_fwd_optional_output_mask(output_final_state=output_final_state, use_gate_in_kernel=use_gate_in_kernel,
                                        disable_recompute=disable_recompute,
                                        return_intermediate_states=return_intermediate_states)
    attn_out = _empty(in_layout(HV, V), q)
    final_state = _empty(state_shape, q, dtype=torch.float32) if mask[1] else None
    gk = _empty((*lead, HV, T, K), q, dtype=torch.float32) if mask[2] else None
    aqk = _empty((*lead, HV, T, chunk_size), q)
    akk = _empty((*lead, HV, T, chunk_size), q)
    w = _empty((*lead, HV, T, K), q) if mask[5] else None
    u = _empty((*lead, HV, T, V), q) if mask[6] and not fine_qk else None   # no stage of the backward reads u
    qk_dtype = torch.float16 if fine_qk and K <= 128 else q.dtype
    qg = _empty((*lead, HV, T, K), q, dtype=qk_dtype) if mask[7] else None
    kg = _empty((*lead, HV, T, K), q, dtype=qk_dtype) if mask[8] else None
    v_new = _empty((*lead, HV, T, V), q) if mask[9] else None
    h = _empty((*lead, NT, HV, *block), q) if mask[10] else None
    outputs = (attn_out, final_state, gk, aqk, akk, w, u, qg, kg, v_new, h)
    names = ("attn_out", "final_state", "gk", "Aqk", "Akk", "w", "u", "qg", "kg", "v_new", "h")
    (_runtime.call_op_noalloc if noalloc else _call_op)(
        "chunk_kda_fwd_noalloc" if noalloc else "chunk_kda_fwd", OP_ARGTYPES["chunk_kda_fwd"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(g, "g"), ctx.tensor(beta, "beta"),
            ctx.tensor(A_log, "A_log"), ctx.tensor(dt_bias, "dt_bias"), ctx.tensor(initial_state, "initial_state"),
            ctx.int_array(cu), ctx.int_array(indices), ctypes.c_char_p(layout.encode("utf-8")),
            ctypes.c_double(float(scale)), ctypes.c_int64(chunk_size), ctypes.c_bool(safe_gate),
            ctypes.c_double(lower_bound), ctypes.c_bool(use_gate_in_kernel), ctypes.c_bool(state_v_first),
            *[ctx.tensor(t, n) for t, n in zip(outputs, names)],
        ],
        outputs,
    )
    return (*outputs, initial_state)


def npu_chunk_kda_bwd_intra(q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, *, cu_seqlens=None, chunk_indices=None,
                            chunk_size=64, safe_gate=True, layout="BSND"):
    """Intra-chunk KDA backward (_aclnn_ctypes.py:1534-1768).  Returns new ``(dq, dk, db, dg)`` = the inputs
    plus the intra-chunk terms; q/k bf16, beta bf16 or fp32, everything else fp32, all contiguous."""
    import torch

    op = "npu_chunk_kda_bwd_intra"
    tensors = {"q": q, "k": k, "gk": gk, "beta": beta, "dAqk": dAqk, "dAkk": dAkk, "dq": dq, "dk": dk, "db": db, "dg": dg}
    layout = str(layout)
    if layout not in {"BSND", "BNSD", "TND"}:
        raise RuntimeError(f"{op}: supports dense BSND/BNSD or varlen TND.")
    if not bool(safe_gate):
        raise RuntimeError(f"{op}: safe_gate=False is reserved but not supported in v1.")
    chunk_size = int(chunk_size)
    if chunk_size != 64:
        raise RuntimeError(f"{op}: chunk_size must be 64.")
    for name, tensor in tensors.items():
        if name == "beta":
            if tensor.dtype not in {torch.bfloat16, torch.float32}:
                raise RuntimeError(f"{op}: beta must be torch.bfloat16 or torch.float32.")
        else:
            want = torch.bfloat16 if name in ("q", "k") else torch.float32
            if tensor.dtype != want:
                raise RuntimeError(f"{op}: {name} must be {want}.")
        if tensor.device != q.device:
            raise RuntimeError(f"{op}: {name} must be on the same device as q.")
        if not tensor.is_contiguous():
            raise RuntimeError(f"{op}: {name} must be contiguous; implicit copies are disabled.")
    if chunk_indices is not None and cu_seqlens is None:
        raise RuntimeError(f"{op}: chunk_indices requires cu_seqlens.")
    varlen = cu_seqlens is not None
    if varlen and layout == "BNSD":
        raise RuntimeError(f"{op}: varlen supports TND or BSND, not BNSD.")
    if not varlen and layout == "TND":
        raise RuntimeError(f"{op}: TND requires cu_seqlens.")
    qs = _shape(q)
    if len(qs) != (3 if layout == "TND" else 4):
        raise RuntimeError(f"{op}: q rank does not match layout.")
    if layout == "TND":
        (T, H, K), B = qs, 1
        scalar_shape, matrix_shape = (T, H), (T, H, chunk_size)
    elif layout == "BSND":
        B, T, H, K = qs
        scalar_shape, matrix_shape = (B, T, H), (B, T, H, chunk_size)
    else:
        B, H, T, K = qs
        scalar_shape, matrix_shape = (B, H, T), (B, H, T, chunk_size)
    if B <= 0 or H <= 0 or T <= 0:
        raise RuntimeError(f"{op}: B/H/T must be positive.")
    if K not in {64, 128, 256}:
        raise RuntimeError(f"{op}: K must be 64, 128 or 256.")
    if varlen and layout == "BSND" and B != 1:
        raise RuntimeError(f"{op}: varlen BSND compatibility requires B=1.")
    for name in ("k", "gk", "dq", "dk", "dg"):
        if _shape(tensors[name]) != qs:
            raise RuntimeError(f"{op}: {name} must have the same shape as q.")
    if _shape(beta) != scalar_shape or _shape(db) != scalar_shape:
        raise RuntimeError(f"{op}: beta/db shape must match the selected layout.")
    if _shape(dAqk) != matrix_shape or _shape(dAkk) != matrix_shape:
        raise RuntimeError(f"{op}: dAqk/dAkk shape must match the selected layout.")
    cu = indices = None
    if varlen:
        cu = _as_int_tuple(cu_seqlens)
        if len(cu) < 2 or cu[0] != 0 or cu[-1] != T:
            raise RuntimeError(f"{op}: cu_seqlens must start at 0 and end at T.")
        if any(a > b for a, b in zip(cu, cu[1:])):
            raise RuntimeError(f"{op}: cu_seqlens must be nondecreasing.")
        canonical = _build_chunk_indices(cu, chunk_size)
        if not canonical:
            raise RuntimeError(f"{op}: varlen input has no non-empty sequence.")
        indices = canonical if chunk_indices is None else _as_int_tuple(chunk_indices)
        if indices != canonical:
            raise RuntimeError(f"{op}: chunk_indices must use canonical sequence-major order.")
    outputs = (_empty_like(dq), _empty_like(dk), _empty_like(db), _empty_like(dg))
    ins = (q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg)
    return _call_op(
        "chunk_kda_bwd_intra", OP_ARGTYPES["chunk_kda_bwd_intra"],
        lambda ctx: [
            *[ctx.tensor(t, n) for t, n in zip(ins, tensors)],
            ctx.int_array(cu), ctx.int_array(indices), ctypes.c_int64(chunk_size), ctypes.c_bool(True),
            ctypes.c_char_p(layout.encode("utf-8")),
            *[ctx.tensor(t, n) for t, n in zip(outputs, ("dq_out", "dk_out", "db_out", "dg_out"))],
        ],
        outputs,
    )


# ---------------------------------------------------------------------------------------------
# KDA chunk backward: the stages the reference leaves to a third-party package
# (torch_custom/fla_npu/fla_npu/adapters/triton_ascend_kda.py:1-8).  Operands are [B,H,T,D] index order; any
# strided view with a unit innermost stride is taken as is (pass ``x.transpose(1, 2)`` for a [B,T,H,D] tensor).
# ``out_like`` tensors let a caller choose the memory layout of the fp32 results.
def _empty_strided_like(shape, like, dtype, device=None):
    """A tensor of ``shape`` whose memory order follows ``like`` (same permutation of dimensions)."""
    import torch

    order = sorted(range(len(shape)), key=lambda d: (-like.stride(d), d))
    perm_shape = [shape[d] for d in order]
    base = torch.empty(perm_shape, dtype=dtype, device=like.device if device is None else device)
    inverse = [order.index(d) for d in range(len(shape))]
    return base.permute(inverse)


def chunk_kda_bwd_dav(v_new, d_o, Aqk, scale, chunk_size=64, *, cu_seqlens=None, chunk_indices=None, layout_like=None):
    """``dAqk = scale * tril(d_o v_new^T)`` (fp32 [B,Hv,T,64]) and ``dv = Aqk^T d_o`` ([B,Hv,T,V], dtype of v_new).
    ``layout_like`` ([B,Hv,T,*] view): dAqk is laid out in memory like it (default: like ``d_o``)."""
    import torch

    B, Hv, T, V = _shape(d_o)
    like = d_o if layout_like is None else layout_like
    dA = _empty_strided_like((B, Hv, T, int(chunk_size)), like, torch.float32, d_o.device)
    dv = _empty_strided_like((B, Hv, T, V), v_new, v_new.dtype)
    cu = _as_int_tuple(cu_seqlens)
    _call_op(
        "chunk_kda_bwd_dav", OP_ARGTYPES["chunk_kda_bwd_dav"],
        lambda ctx: [
            ctx.tensor(v_new, "v_new"), ctx.tensor(d_o, "d_o"), ctx.tensor(Aqk, "Aqk"), ctx.int_array(cu),
            ctx.int_array(_as_int_tuple(chunk_indices)), ctypes.c_double(float(scale)), ctypes.c_int64(int(chunk_size)),
            ctx.tensor(dA, "dAqk"), ctx.tensor(dv, "dv"),
        ],
        (dA, dv),
    )
    return dA, dv


def chunk_kda_bwd_dqkwg(q, k, v_new, gk, h, d_o, dh, dv, scale, chunk_size=64, *, cu_seqlens=None, chunk_indices=None,
                        layout_like=None, with_dAqk=False):
    """State-dependent part of the KDA backward: returns ``(dq, dk, dw, dg)``, dq / dk / dg fp32 [B,Hv,T,K] per value
    head laid out like ``layout_like`` (default: like ``gk``), dw [B,Hv,T,K] in the dtype of q.
    ``h`` and ``dh`` are [B,Hv,NT,K,V] views (any outer strides).  ``with_dAqk=True``: a fifth result, the dAqk of
    ``chunk_kda_bwd_dav`` (fp32 [B,Hv,T,64] laid out like the others), from the d_o and v_new tiles staged anyway."""
    import torch

    B, Hv, T, K = _shape(gk)
    like = gk if layout_like is None else layout_like
    dq = _empty_strided_like((B, Hv, T, K), like, torch.float32, q.device)
    dk = _empty_strided_like((B, Hv, T, K), like, torch.float32, q.device)
    dg = _empty_strided_like((B, Hv, T, K), like, torch.float32, q.device)
    dw = _empty((B, Hv, T, K), q)
    dAqk = _empty_strided_like((B, Hv, T, 64), like, torch.float32, q.device) if with_dAqk else None
    cu = _as_int_tuple(cu_seqlens)
    outs = (dq, dk, dw, dg) + ((dAqk,) if with_dAqk else ())
    _call_op(
        "chunk_kda_bwd_dqkwg", OP_ARGTYPES["chunk_kda_bwd_dqkwg"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v_new, "v_new"), ctx.tensor(gk, "gk"), ctx.tensor(h, "h"),
            ctx.tensor(d_o, "d_o"), ctx.tensor(dh, "dh"), ctx.tensor(dv, "dv"), ctx.int_array(cu),
            ctx.int_array(_as_int_tuple(chunk_indices)), ctypes.c_double(float(scale)), ctypes.c_int64(int(chunk_size)),
            *[ctx.tensor(t, n) for t, n in zip((dq, dk, dw, dg, dAqk), ("dq", "dk", "dw", "dg", "dAqk"))],
        ],
        outs,
    )
    return outs


def chunk_kda_bwd_dhu(qg, kg, w, d_o, Aqk, scale, chunk_size=64, *, gK, h0=None, dht=None, cu_seqlens=None, chunk_indices=None):
    """``npu_chunk_gated_delta_rule_bwd_dhu`` for the KDA backward (per-channel gate ``gK`` in log2 units, 64-token
    chunks) with its dv operand formed inside the scan: dv = Aqk^T d_o per chunk, the second result of
    ``chunk_kda_bwd_dav``, from the forward's score blocks ``Aqk`` [B,Hv,T,64] and the d_o tiles the scan stages anyway.
    ``qg`` and ``kg`` may be float16 tensors beside bfloat16 ``w``, ``d_o`` and ``Aqk`` (``chunk_kda_fwd_for_backward``).
    Returns ``(dh, dh0, dv2)`` with dh0 fp32 [N,Hv,K,V] (None without ``h0``).  No counterpart in the reference."""
    import torch

    B, _, T, K = _shape(qg)
    _, Hv, _, V = _shape(d_o)
    chunk_size = int(chunk_size)
    cu = _as_int_tuple(cu_seqlens)
    indices = _as_int_tuple(chunk_indices)
    if indices is None and cu is not None:
        indices = _build_chunk_indices(cu, chunk_size)
    NT = _total_chunks(B, T, chunk_size, cu) if indices is None else len(indices) // 2
    N = len(cu) - 1 if cu is not None else B
    dh = _empty((B, Hv, NT, K, V), w)
    dh0 = None if h0 is None else _empty((N, Hv, K, V), w, dtype=torch.float32)
    dv2 = _empty_ordered_like(d_o)
    outputs = (dh, dh0, dv2)
    return _call_op(
        "chunk_kda_bwd_dhu", OP_ARGTYPES["chunk_kda_bwd_dhu"],
        lambda ctx: [
            ctx.tensor(qg, "q"), ctx.tensor(kg, "k"), ctx.tensor(w, "w"), ctx.tensor(d_o, "d_o"), ctx.tensor(Aqk, "Aqk"),
            ctx.tensor(gK, "gK"), ctx.tensor(h0, "h0"), ctx.tensor(dht, "dht"),
            ctx.int_array(cu), ctx.int_array(indices), ctypes.c_double(float(scale)), ctypes.c_int64(chunk_size),
            ctx.tensor(dh, "dh"), ctx.tensor(dh0, "dh0"), ctx.tensor(dv2, "dv2"),
        ],
        outputs,
    )


def chunk_kda_bwd_wy(k, v, beta, gk, Akk, dw, du, dk, dg, chunk_size=64, *, cu_seqlens=None, chunk_indices=None):
    """Backward of ``w = Akk (k beta 2^g)``, ``u = Akk (v beta)``.  ``dk`` and ``dg`` (fp32 [B,Hv,T,K]) are ADDED TO in
    place; returns ``(dv, db, dAkk)``: dv like v, db fp32 [B,Hv,T], dAkk fp32 [B,Hv,T,64], both laid out like ``dk``."""
    import torch

    B, Hv, T, V = _shape(du)
    dv = _empty_strided_like((B, Hv, T, V), v, v.dtype)
    db = _empty_strided_like((B, Hv, T, 1), dk, torch.float32)[..., 0]
    dA = _empty_strided_like((B, Hv, T, int(chunk_size)), dk, torch.float32)
    cu = _as_int_tuple(cu_seqlens)
    outs = (dv, db, dA)
    _call_op(
        "chunk_kda_bwd_wy", OP_ARGTYPES["chunk_kda_bwd_wy"],
        lambda ctx: [
            ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"), ctx.tensor(gk, "gk"), ctx.tensor(Akk, "Akk"),
            ctx.tensor(dw, "dw"), ctx.tensor(du, "du"), ctx.int_array(cu), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_int64(int(chunk_size)), ctx.tensor(dk, "dk"), ctx.tensor(dv, "dv"), ctx.tensor(db, "db"),
            ctx.tensor(dg, "dg"), ctx.tensor(dA, "dAkk"),
        ],
        outs,
    )
    return outs


def chunk_kda_bwd_dqkwg_wy(q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, scale, chunk_size=64, *, cu_seqlens=None,
                           chunk_indices=None, layout_like=None):
    """``chunk_kda_bwd_dqkwg`` (with dAqk) followed by ``chunk_kda_bwd_wy`` in one launch: dw passes through on-chip memory
    and dk, dg are completed in registers, so neither is written, read back, added to and written again.  Returns
    ``(dq, dk, dg, dAqk, dv, db, dAkk)``: dq / dk / dg fp32 [B,Hv,T,K], dAqk / dAkk fp32 [B,Hv,T,64] and db fp32
    [B,Hv,T] laid out like ``layout_like`` (default: like ``gk``), dv like ``v``.  Head sizes (K,V) in (128,128),
    (64,64), (64,128), 64-token chunks."""
    import torch

    B, Hv, T, K = _shape(gk)
    V = _shape(v)[-1]
    like = gk if layout_like is None else layout_like
    f32 = lambda d: _empty_strided_like((B, Hv, T, d), like, torch.float32, q.device)
    dq, dk, dg, dAqk, dAkk = f32(K), f32(K), f32(K), f32(64), f32(64)
    db = f32(1)[..., 0]
    dv = _empty_strided_like((B, Hv, T, V), v, v.dtype)
    cu = _as_int_tuple(cu_seqlens)
    outs = (dq, dk, dg, dAqk, dv, db, dAkk)
    _call_op(
        "chunk_kda_bwd_dqkwg_wy", OP_ARGTYPES["chunk_kda_bwd_dqkwg_wy"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v_new, "v_new"), ctx.tensor(gk, "gk"), ctx.tensor(h, "h"),
            ctx.tensor(d_o, "d_o"), ctx.tensor(dh, "dh"), ctx.tensor(dv2, "dv2"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"),
            ctx.tensor(Akk, "Akk"), ctx.int_array(cu), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_double(float(scale)), ctypes.c_int64(int(chunk_size)),
            *[ctx.tensor(t, n) for t, n in zip(outs, ("dq", "dk", "dg", "dAqk", "dv", "db", "dAkk"))],
        ],
        outs,
    )
    return outs


def chunk_kda_bwd_dqkwg_wy_intra(q, k, v_new, gk, h, d_o, dh, dv2, v, beta, Akk, scale, chunk_size=64, *, cu_seqlens=None,
                                 chunk_indices=None, layout_like=None, grad_dtype=None):
    """Everything of the KDA chunk backward after the reverse scan in one launch: ``chunk_kda_bwd_dqkwg_wy`` followed by
    ``chunk_kda_bwd_intra`` with the reverse chunk-local running sum of dg.  dAqk and dAkk never leave the chip and dq,
    dk, dg, dbeta are written once, final.  Returns ``(dq, dk, dg, dv, db)``: dq / dk [B,Hv,T,K] in ``grad_dtype``
    (default fp32; q's dtype is meant for Hv == Hk, where no sum over the value heads of a key head follows), dg fp32
    [B,Hv,T,K] and db fp32 [B,Hv,T] laid out like ``layout_like`` (default: like ``gk``), dv like ``v``."""
    import torch

    B, Hv, T, K = _shape(gk)
    V = _shape(v)[-1]
    like = gk if layout_like is None else layout_like
    f32 = lambda d: _empty_strided_like((B, Hv, T, d), like, torch.float32, q.device)
    gdt = torch.float32 if grad_dtype is None else grad_dtype
    dq, dk = (_empty_strided_like((B, Hv, T, K), like, gdt, q.device) for _ in range(2))
    dg = f32(K)
    db = f32(1)[..., 0]
    dv = _empty_strided_like((B, Hv, T, V), v, v.dtype)
    cu = _as_int_tuple(cu_seqlens)
    outs = (dq, dk, dg, dv, db)
    _call_op(
        "chunk_kda_bwd_dqkwg_wy_intra", OP_ARGTYPES["chunk_kda_bwd_dqkwg_wy_intra"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v_new, "v_new"), ctx.tensor(gk, "gk"), ctx.tensor(h, "h"),
            ctx.tensor(d_o, "d_o"), ctx.tensor(dh, "dh"), ctx.tensor(dv2, "dv2"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"),
            ctx.tensor(Akk, "Akk"), ctx.int_array(cu), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_double(float(scale)), ctypes.c_int64(int(chunk_size)),
            *[ctx.tensor(t, n) for t, n in zip(outs, ("dq", "dk", "dg", "dv", "db"))],
        ],
        outs,
    )
    return outs


def chunk_kda_bwd_intra_inplace(q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg, *, cu_seqlens=None, chunk_size=64,
                                cumsum_dg=False, dq_out=None, dk_out=None):
    """``npu_chunk_kda_bwd_intra`` on [B,H,T,*] index-order views with the results written over ``dq, dk, db, dg``.
    The library accepts strided views, grouped heads (q, k with fewer heads than gk) and outputs that alias their
    inputs; the public operator keeps the reference's contiguous, allocate-new contract.  ``cumsum_dg``: dg leaves as
    its reverse chunk-local running sum, the pass that follows this operator in the KDA backward; with it, ``dq_out`` /
    ``dk_out`` may be tensors of q's dtype (same memory order as dq, dk) that take the final dq, dk instead."""
    cu = _as_int_tuple(cu_seqlens)
    indices = None if cu is None else _build_chunk_indices(cu, int(chunk_size))
    ins = (q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg)
    names = ("q", "k", "gk", "beta", "dAqk", "dAkk", "dq", "dk", "db", "dg")
    outs = (dq if dq_out is None else dq_out, dk if dk_out is None else dk_out, db, dg)
    name = "chunk_kda_bwd_intra_cumsum" if cumsum_dg else "chunk_kda_bwd_intra"
    _call_op(
        name, OP_ARGTYPES[name],
        lambda ctx: [
            *[ctx.tensor(t, n) for t, n in zip(ins, names)],
            ctx.int_array(cu), ctx.int_array(indices), ctypes.c_int64(int(chunk_size)), ctypes.c_bool(True),
            ctypes.c_char_p(b"BNSD"),
            *[ctx.tensor(t, n) for t, n in zip(outs, ("dq_out", "dk_out", "db_out", "dg_out"))],
        ],
        outs,
    )
    return outs


def kda_gate_bwd(g, dgate, A_log, dt_bias=None, *, layout="BSND", safe_gate=False, lower_bound=-5.0):
    """Gradient of the in-kernel KDA gate activation (fla/ops/ascendc/kda/chunk_kda_fwd/docs/api.md:103-113):
    ``(dg_raw, dA_log, ddt_bias)`` from the raw gate ``g`` and the gradient ``dgate`` (f32, shape of g) of the activated
    gate; dg_raw has the dtype and memory order of g, dA_log is f32 [HV], ddt_bias f32 [HV*K] or None."""
    import torch

    head_axis = {"BSND": 2, "BNSD": 1, "TND": 1, "NTD": 0}[layout]
    token_axis = {"BSND": 1, "BNSD": 2, "TND": 0, "NTD": 1}[layout]
    HV, K, T = int(g.shape[head_axis]), int(g.shape[-1]), int(g.shape[token_axis])
    B = int(g.shape[0]) if g.dim() == 4 else 1
    parts = B * ((T + 255) // 256)
    dg_raw = _empty_ordered_like(g)
    da_part = _empty((parts, HV), g, dtype=torch.float32)
    db_part = None if dt_bias is None else _empty((parts, HV, K), g, dtype=torch.float32)
    _call_op(
        "kda_gate_bwd", OP_ARGTYPES["kda_gate_bwd"],
        lambda ctx: [
            ctx.tensor(g, "g"), ctx.tensor(dgate, "dgate"), ctx.tensor(A_log, "A_log"), ctx.tensor(dt_bias, "dt_bias"),
            ctypes.c_char_p(layout.encode("utf-8")), ctypes.c_bool(bool(safe_gate)), ctypes.c_double(float(lower_bound)),
            ctx.tensor(dg_raw, "dg_raw"), ctx.tensor(db_part, "ddt_bias_partial"), ctx.tensor(da_part, "dA_log_partial"),
        ],
        (dg_raw, da_part),
    )
    return dg_raw, da_part.sum(0), (None if db_part is None else db_part.sum(0).reshape(HV * K))


def chunk_local_cumsum_into(g, out, chunk_size, *, cu_seqlens=None, reverse=False, scale=1.0):
    """``npu_chunk_local_cumsum`` on [B,H,T] / [B,H,T,K] index-order views, written into ``out`` (which may be ``g``)."""
    name_buf = ctypes.create_string_buffer(str(out.dtype).removeprefix("torch.").encode("utf-8"))
    _call_op(
        "chunk_local_cumsum", OP_ARGTYPES["chunk_local_cumsum"],
        lambda ctx: [
            ctx.tensor(g, "g"), ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(None),
            ctypes.c_int64(int(chunk_size)), ctypes.c_bool(bool(reverse)), ctypes.c_double(float(scale)),
            ctypes.c_bool(True), ctypes.cast(name_buf, ctypes.c_char_p), ctx.tensor(out, "out"),
        ],
        out,
    )
    return out


def _f32_like(t):
    import torch

    return _empty(_shape(t), t, dtype=torch.float32)


def _as_dtype(out, like):
    return out if out.dtype == like.dtype else out.to(like.dtype)


def npu_chunk_bwd_dv_local(q, k, d_o, g, scale, chunk_size, *, g_gamma=None, A=None, cu_seqlens=None,
                           chunk_indices=None):
    """_aclnn_ctypes.py:397-427.  q, k [B,Hk,T,K]; d_o [B,Hv,T,V]; g [B,Hv,T] chunk-cumsummed."""
    if g_gamma is not None:
        raise NotImplementedError("npu_chunk_bwd_dv_local: g_gamma is not supported.")
    out = _empty_ordered_like(d_o)
    return _call_op(
        "chunk_bwd_dv_local", OP_ARGTYPES["chunk_bwd_dv_local"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(d_o, "d_o"), ctx.tensor(g, "g"),
            ctx.tensor(g_gamma, "g_gamma"), ctx.tensor(A, "A"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_double(float(scale)), ctypes.c_int64(int(chunk_size)), ctx.tensor(out, "out"),
        ],
        out,
    )


def npu_prepare_wy_repr_bwd_da(k, v, beta, A, dw, du, g, *, chunk_size, cu_seqlens=None, chunk_indices=None):
    """_aclnn_ctypes.py:430-460.  Returns dA [B,Hv,T,C], stored transposed as the reference does."""
    out = _empty_like(A)
    return _call_op(
        "prepare_wy_repr_bwd_da", OP_ARGTYPES["prepare_wy_repr_bwd_da"],
        lambda ctx: [
            ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"), ctx.tensor(A, "A"),
            ctx.tensor(dw, "dw"), ctx.tensor(du, "du"), ctx.tensor(g, "g"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_int64(int(chunk_size)), ctx.tensor(out, "dA"),
        ],
        out,
    )


def npu_prepare_wy_repr_bwd_full(k, v, beta, A, dA, dw, du, g, chunk_size, *, cu_seqlens=None, chunk_indices=None):
    """_aclnn_ctypes.py:242-279.  Returns (dk, dv, dbeta, dg); dbeta and dg are computed in fp32 and
    returned in the dtype of beta and g."""
    dk = _empty_ordered_like(k)
    dv = _empty_ordered_like(v)
    dbeta = _f32_like(beta)
    dg = _f32_like(g)
    outputs = (dk, dv, dbeta, dg)
    dk, dv, dbeta, dg = _call_op(
        "prepare_wy_repr_bwd_full", OP_ARGTYPES["prepare_wy_repr_bwd_full"],
        lambda ctx: [
            ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"), ctx.tensor(A, "A"), ctx.tensor(dA, "dA"),
            ctx.tensor(dw, "dw"), ctx.tensor(du, "du"), ctx.tensor(g, "g"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_int64(int(chunk_size)),
            ctx.tensor(dk, "dk"), ctx.tensor(dv, "dv"), ctx.tensor(dbeta, "dbeta"), ctx.tensor(dg, "dg"),
        ],
        outputs,
    )
    return dk, dv, _as_dtype(dbeta, beta), _as_dtype(dg, g)


def prepare_wy_repr_bwd_full_accumulate(k, v, beta, A, dA, dw, du, g, dk, dg, chunk_size, *, cu_seqlens=None,
                                        chunk_indices=None, k_rstd=None):
    """npu_prepare_wy_repr_bwd_full with its key and gate gradients ADDED to ``dk`` ([B,Hk,T,K], dtype of k) and
    ``dg`` ([B,Hv,T] f32) in place: the reference's composition adds them with a separate pass
    (examples/flash_gated_delta_rule.py:994-1010).  Returns (dv, dbeta f32).  ``k_rstd`` (f32 [B,Hk,T], the second result
    of ``l2norm_fwd``): k is the normalised tensor and the completed dk leaves as the gradient of the raw k.
    ``dA=None`` (64-token chunks): the kernel forms ``npu_prepare_wy_repr_bwd_da``'s result itself, from the tiles it
    stages anyway, and dA never goes through memory.  Then ``A`` may be None as well: the kernel rebuilds each chunk's
    inverse from k, g and beta with the arithmetic of ``chunk_scaled_dot_kkt_inverse``, so neither matrix is read."""
    dv = _empty_ordered_like(v)
    dbeta = _f32_like(beta)
    dv, dbeta = _call_op(
        "prepare_wy_repr_bwd_full_accumulate", OP_ARGTYPES["prepare_wy_repr_bwd_full_accumulate"],
        lambda ctx: [
            ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"), ctx.tensor(A, "A"), ctx.tensor(dA, "dA"),
            ctx.tensor(dw, "dw"), ctx.tensor(du, "du"), ctx.tensor(g, "g"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_int64(int(chunk_size)), ctx.tensor(k_rstd, "k_rstd"),
            ctx.tensor(dk, "dk"), ctx.tensor(dv, "dv"), ctx.tensor(dbeta, "dbeta"), ctx.tensor(dg, "dg"),
        ],
        (dv, dbeta),
    )
    return dv, dbeta


def chunk_bwd_dqkwg_l2norm(q, k, v, g, h, dox, dh, dv, q_rstd, chunk_size, *, scale, cu_seqlens=None, chunk_indices=None):
    """``npu_chunk_bwd_dqkwg`` for an l2-normalised q: dq comes back as the gradient of the raw q (``q_rstd`` f32
    [B,Hk,T] from ``l2norm_fwd``), which replaces the ``l2norm_bwd`` pass over dq.  dk is the gradient of the normalised
    k (it is completed, and de-normalised, by ``prepare_wy_repr_bwd_full_accumulate(..., k_rstd=)``)."""
    q_shape = _shape(q)
    dq = _empty_ordered_like(q)
    dk = _empty_ordered_like(k)
    dw = _empty((q_shape[0], int(v.shape[1]), q_shape[2], q_shape[3]), q)
    dg = _f32_like(g)
    outputs = (dq, dk, dw, dg)
    return _call_op(
        "chunk_bwd_dqkwg_l2norm", OP_ARGTYPES["chunk_bwd_dqkwg_l2norm"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(g, "g"), ctx.tensor(h, "h"),
            ctx.tensor(dox, "dox"), ctx.tensor(dh, "dh"), ctx.tensor(dv, "dv"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctx.tensor(q_rstd, "q_rstd"), ctypes.c_float(float(scale)), ctypes.c_int64(int(chunk_size)),
            ctx.tensor(dq, "dq"), ctx.tensor(dk, "dk"), ctx.tensor(dw, "dw"), ctx.tensor(dg, "dg"),
        ],
        outputs,
    )


def npu_prepare_wy_repr_bwd(k, v, beta, A, dw, du, g, chunk_size, *, cu_seqlens=None, chunk_indices=None):
    """_aclnn_ctypes.py:284-321: bwd_da and bwd_full in one library call (dA stays in the workspace).
    Returns (dk, dv, dbeta, dg) like npu_prepare_wy_repr_bwd_full."""
    dk = _empty_ordered_like(k)
    dv = _empty_ordered_like(v)
    dbeta = _f32_like(beta)
    dg = _f32_like(g)
    outputs = (dk, dv, dbeta, dg)
    dk, dv, dbeta, dg = _call_op(
        "prepare_wy_repr_bwd", OP_ARGTYPES["prepare_wy_repr_bwd"],
        lambda ctx: [
            ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(beta, "beta"), ctx.tensor(A, "A"),
            ctx.tensor(dw, "dw"), ctx.tensor(du, "du"), ctx.tensor(g, "g"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctypes.c_int64(int(chunk_size)),
            ctx.tensor(dk, "dk"), ctx.tensor(dv, "dv"), ctx.tensor(dbeta, "dbeta"), ctx.tensor(dg, "dg"),
        ],
        outputs,
    )
    return dk, dv, _as_dtype(dbeta, beta), _as_dtype(dg, g)


def npu_chunk_bwd_dqkwg(q, k, v, g, h, dox, dh, dv, chunk_size, *, cu_seqlens=None, chunk_indices=None, w=None,
                        g_gamma=None, scale=None, use_exp2=None, transpose_state_layout=None):
    """_aclnn_ctypes.py:463-510.  Returns (dq, dk [B,Hk,T,K], dw [B,Hv,T,K], dg [B,Hv,T]); ``v`` is v_new."""
    if g_gamma is not None:
        raise NotImplementedError("npu_chunk_bwd_dqkwg: g_gamma is not supported.")
    q_shape = _shape(q)
    value_num_heads = int(v.shape[1])
    dq = _empty_ordered_like(q)
    dk = _empty_ordered_like(k)
    dw = _empty((q_shape[0], value_num_heads, q_shape[2], q_shape[3]), q)
    dg = _f32_like(g)
    outputs = (dq, dk, dw, dg)
    dq, dk, dw, dg = _call_op(
        "chunk_bwd_dqkwg", OP_ARGTYPES["chunk_bwd_dqkwg"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(g, "g"), ctx.tensor(h, "h"),
            ctx.tensor(dox, "dox"), ctx.tensor(dh, "dh"), ctx.tensor(dv, "dv"),
            ctx.int_array(_as_int_tuple(cu_seqlens)), ctx.int_array(_as_int_tuple(chunk_indices)),
            ctx.tensor(w, "w"), ctx.tensor(g_gamma, "g_gamma"),
            ctypes.c_float(_optional_float(scale, 1.0)), ctypes.c_int64(int(chunk_size)),
            ctypes.c_bool(_optional_bool(use_exp2, False)), ctypes.c_bool(_optional_bool(transpose_state_layout, False)),
            ctx.tensor(dq, "dq"), ctx.tensor(dk, "dk"), ctx.tensor(dw, "dw"), ctx.tensor(dg, "dg"),
        ],
        outputs,
    )
    return dq, dk, dw, _as_dtype(dg, g)


def npu_causal_conv1d_bwd(x, y, weight, dy, initial_state=None, dht=None, *, query_start_loc=None, activation=0,
                          input_layout="BSND"):
    """_aclnn_ctypes.py:988-1037.  Returns (dx, dw, db, dh0); ``y`` is the pre-activation output."""
    input_layout = str(input_layout)
    width, dim = int(weight.shape[0]), int(weight.shape[1])
    if input_layout in {"NTD", "TND"}:
        if query_start_loc is None:
            raise RuntimeError(f"query_start_loc is required for {input_layout} input.")
        batch = len(query_start_loc) - 1
    else:
        batch = int(x.shape[0])
    dx = _empty(_shape(x), x)
    dw = _empty((width, dim), weight)
    db = _empty((dim,), weight)
    dh0 = _empty((batch, width, dim), x)
    outputs = (dx, dw, db, dh0)
    return _call_op(
        "causal_conv1d_bwd", OP_ARGTYPES["causal_conv1d_bwd"],
        lambda ctx: [
            ctx.tensor(x, "x"), ctx.tensor(y, "y"), ctx.tensor(weight, "weight"), ctx.tensor(dy, "dy"),
            ctx.tensor(initial_state, "initial_state"), ctx.tensor(dht, "dht"),
            ctx.int_array(_as_int_tuple(query_start_loc)), ctypes.c_int64(int(activation)),
            ctypes.c_char_p(input_layout.encode("utf-8")),
            ctx.tensor(dx, "dx"), ctx.tensor(dw, "dw"), ctx.tensor(db, "db"), ctx.tensor(dh0, "dh0"),
        ],
        outputs,
    )


def npu_recurrent_kda(q, k, v, g, beta, initial_state=None, *, cu_seqlens=None, ssm_state_indices=None, A_log=None,
                      dt_bias=None, num_accepted_tokens=None, layout="BSND", scale=None, output_final_state=False,
                      inplace_final_state=True, use_qk_l2norm_in_kernel=False, use_gate_in_kernel=False,
                      use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, safe_gate=False, lower_bound=None,
                      state_v_first=False):
    """_aclnn_ctypes.py:1298-1503: same checks, defaults and error texts.  Returns (out, final_state or None)."""
    import torch

    def need(ok, text):
        if not ok:
            raise RuntimeError("npu_recurrent_kda: " + text)

    def on_q_device(t, name):
        need(t.device == q.device, f"{name} must be on the same device as q.")

    layout = str(layout)
    need(layout in ("BSND", "TND"), "layout must be BSND or TND.")
    is_tnd = layout == "TND"
    rank = 3 if is_tnd else 4
    shapes = [_shape(t) for t in (q, k, v, g, beta)]
    q_shape, k_shape, v_shape, g_shape, beta_shape = shapes
    need([len(x) for x in shapes] == [rank] * 4 + [rank - 1],
         "layout/rank mismatch. TND expects q/k [T,H,K], v [T,HV,V], g [T,HV,K], beta [T,HV]; "
         "BSND expects q/k [B,T,H,K], v [B,T,HV,V], g [B,T,HV,K], beta [B,T,HV].")
    need(q_shape == k_shape, "q and k must have identical shape.")
    need({q.dtype, k.dtype, v.dtype} == {torch.bfloat16}, "q/k/v currently support bfloat16 only.")
    need(all(t.device == q.device for t in (k, v, g, beta)), "q/k/v/g/beta must be on the same device.")
    floats = (torch.float16, torch.bfloat16, torch.float32)
    need(g.dtype in floats, "g must use FP16, BF16 or FP32.")
    need(beta.dtype in floats, "beta must use FP16, BF16 or FP32.")
    # token axes first, then (heads, width): the same test serves both layouts
    lead = q_shape[:-2]
    heads, key_dim = q_shape[-2:]
    value_heads, value_dim = v_shape[-2:]
    batch, dense_seq_len = (1, lead[0]) if is_tnd else lead
    total_tokens = batch * dense_seq_len
    need(v_shape[:-2] == lead and g_shape == (*lead, value_heads, key_dim) and beta_shape == (*lead, value_heads),
         "v/g/beta shape mismatch.")
    need(min(total_tokens, dense_seq_len, heads, value_heads, key_dim, value_dim) > 0, "all shape dimensions must be positive.")
    need(value_heads % heads == 0, "HV must be divisible by H.")
    need((key_dim, value_dim) in ((128, 128), (128, 256)), "K/V currently support only K=128,V=128 or K=128,V=256.")
    ints = (torch.int32, torch.int64)
    seq_num = 1 if is_tnd else batch
    if cu_seqlens is not None:
        need(isinstance(cu_seqlens, torch.Tensor) and cu_seqlens.dim() == 1 and cu_seqlens.numel() >= 2
             and cu_seqlens.dtype in ints, "cu_seqlens must be a 1D INT32 or INT64 tensor.")
        on_q_device(cu_seqlens, "cu_seqlens")
        seq_num = int(cu_seqlens.shape[0]) - 1
    state_v_first = _optional_bool(state_v_first, False)
    block = (value_dim, key_dim) if state_v_first else (key_dim, value_dim)
    expected_tail = (value_heads, *block)
    inplace = _optional_bool(inplace_final_state, True)
    if initial_state is None:
        need(not inplace, "inplace_final_state=True requires initial_state.")
        state_shape = (seq_num, *expected_tail)
        initial_state_work = torch.zeros(state_shape, device=q.device, dtype=torch.float32)
    else:
        need(initial_state.dtype in (torch.float32, torch.bfloat16), "initial_state must use FP32 or BF16.")
        on_q_device(initial_state, "initial_state")
        state_shape = _shape(initial_state)
        need(len(state_shape) == 4 and state_shape[0] > 0 and state_shape[1:] == expected_tail,
             "initial_state must be [state_capacity,HV,%s]." % ("V,K" if state_v_first else "K,V"))
        initial_state_work = initial_state
    if ssm_state_indices is None:
        need(state_shape[0] == seq_num, "without ssm_state_indices, state_capacity must equal seq_num.")
    else:
        idx_shape = _shape(ssm_state_indices)
        per_token = len(idx_shape) == 1 and idx_shape[0] >= total_tokens
        per_step = len(idx_shape) == 2 and idx_shape[0] == seq_num and idx_shape[1] > 0
        need(ssm_state_indices.dtype in ints and (per_token or per_step),
             "ssm_state_indices must be INT32/INT64 packed [T] or speculative [seq_num,max_step].")
        on_q_device(ssm_state_indices, "ssm_state_indices")
    if num_accepted_tokens is not None:
        need(ssm_state_indices is not None, "num_accepted_tokens requires ssm_state_indices.")
        need(num_accepted_tokens.dtype in ints and _shape(num_accepted_tokens) == (seq_num,),
             "num_accepted_tokens must be INT32/INT64 [seq_num].")
        on_q_device(num_accepted_tokens, "num_accepted_tokens")
    use_gate = _optional_bool(use_gate_in_kernel, False)
    safe = _optional_bool(safe_gate, False)
    lower = _optional_float(lower_bound, -5.0)
    if not use_gate:
        need(not safe and A_log is None and dt_bias is None, "A_log, dt_bias and safe_gate require use_gate_in_kernel=True.")
    else:
        need(A_log is not None and A_log.dtype == torch.float32 and _shape(A_log) == (value_heads,),
             "A_log must be FP32 [HV] when use_gate_in_kernel=True.")
        on_q_device(A_log, "A_log")
        need(not safe or -5.0 <= lower < 0.0, "lower_bound must be in [-5,0) when safe_gate=True.")
        if dt_bias is not None:
            need(dt_bias.dtype == torch.float32 and _shape(dt_bias) in ((value_heads * key_dim,), (value_heads, key_dim)),
                 "dt_bias must be FP32 [HV*K] or [HV,K].")
            on_q_device(dt_bias, "dt_bias")
    out = _empty_like(v)
    final_state_work = initial_state_work if inplace else _empty(state_shape, initial_state_work)
    output_final = _optional_bool(output_final_state, False)
    scale_value = _optional_float(scale, key_dim ** -0.5)
    _call_op(
        "recurrent_kda", OP_ARGTYPES["recurrent_kda"],
        lambda ctx: [
            ctx.tensor(q, "q"), ctx.tensor(k, "k"), ctx.tensor(v, "v"), ctx.tensor(g, "g"), ctx.tensor(beta, "beta"),
            ctx.tensor(initial_state_work, "initial_state"), ctx.tensor(cu_seqlens, "cu_seqlens"),
            ctx.tensor(ssm_state_indices, "ssm_state_indices"), ctx.tensor(A_log, "A_log"), ctx.tensor(dt_bias, "dt_bias"),
            ctx.tensor(num_accepted_tokens, "num_accepted_tokens"),
            ctypes.c_char_p(layout.encode("utf-8")), ctypes.c_double(float(scale_value)),
            ctypes.c_bool(output_final), ctypes.c_bool(inplace),
            ctypes.c_bool(_optional_bool(use_qk_l2norm_in_kernel, False)), ctypes.c_bool(use_gate),
            ctypes.c_bool(_optional_bool(use_beta_sigmoid_in_kernel, False)),
            ctypes.c_bool(_optional_bool(allow_neg_eigval, False)), ctypes.c_bool(safe), ctypes.c_double(lower),
            ctypes.c_bool(state_v_first), ctx.tensor(out, "attn_out"), ctx.tensor(final_state_work, "final_state"),
        ],
        (out, initial_state_work, final_state_work),
    )
    return out, (final_state_work if output_final else None)


def l2norm_fwd(x, eps: float = 1e-6, output_dtype=None):
    """fla/ops/triton/triton_core/l2norm.py:131-178: returns (y, rstd) with rstd fp32 of shape x.shape[:-1]."""
    import torch

    if output_dtype is not None and output_dtype != x.dtype:
        raise NotImplementedError("l2norm_fwd: output_dtype must equal the input dtype.")
    y = _empty_ordered_like(x)   # in the memory order of x, so that what is computed on y needs no layout copy back
    rstd = _empty(_shape(x)[:-1], x, dtype=torch.float32)
    _call_op("l2norm_fwd", OP_ARGTYPES["l2norm_fwd"],
             lambda ctx: [ctx.tensor(x, "x"), ctypes.c_double(float(eps)), ctx.tensor(y, "y"), ctx.tensor(rstd, "rstd")],
             (y, rstd))
    return y, rstd


def l2norm_bwd(y, rstd, dy, eps: float = 1e-6, *, like=None):
    """fla/ops/triton/triton_core/l2norm.py:181-224: dx from the normalised output, its rstd and dy.  ``like``: a tensor
    (it may be storage-less) whose memory order dx takes; default: that of y."""
    dx = _empty_ordered_like(y if like is None else like, dtype=y.dtype, shape=tuple(y.shape), device=y.device)
    return _call_op("l2norm_bwd", OP_ARGTYPES["l2norm_bwd"],
                    lambda ctx: [ctx.tensor(y, "y"), ctx.tensor(rstd.contiguous(), "rstd"), ctx.tensor(dy, "dy"),
                                 ctypes.c_double(float(eps)), ctx.tensor(dx, "dx")],
                    dx)


HIP_CTYPES_OPS = {name: value for name, value in globals().items() if name.startswith("npu_") and callable(value)}
