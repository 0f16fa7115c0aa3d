"""CPU oracle (test infrastructure) for recurrent_gated_delta_rule (decode).

Follows fla/ops/ascendc/gdn/recurrent_gdn/recurrent_gated_delta_rule/tests/pta/golden.py:14-99:
``query,key [T,Nk,Dk]``, ``value [T,Nv,Dv]``, ``beta [T,Nv]``,
``state [Block,Nv,Dv,Dk]`` (V-first), ``g [T,Nv]``, ``gk [T,Nv,Dk]``,
``actual_seq_lengths [B+1]`` (element 0 = leading tokens to skip, then one
length per sequence), ``ssm_state_indices [T]``.  Per token

    S <- e^{g} S (and column-wise e^{gk}) ; delta = beta (v - S k) ; S <- S + delta k^T ; o = S (scale q)

The state is read from slot ``ssm_state_indices[first token (+ accepted-1)]`` and
written after EVERY token to ``state[ssm_state_indices[t]]``.  Unlike the
reference golden this keeps fp32 throughout and returns fp32 tensors; the caller
casts as needed.  Sequences may be longer than the reference op's 8-token limit.
"""
from __future__ import annotations

import torch


def recurrent_gated_delta_rule(query, key, value, state, *, beta, scale=1.0,
                               actual_seq_lengths, ssm_state_indices,
                               num_accepted_tokens=None, g=None, gk=None,
                               compute_dtype=torch.float32):
    """Returns (out [T,Nv,Dv], new_state [Block,Nv,Dv,Dk]) in compute_dtype."""
    T, Nk, Dk = query.shape
    Nv, Dv = value.shape[1], value.shape[2]
    rep = Nv // Nk
    q = query.to(compute_dtype) * scale
    k = key.to(compute_dtype)
    v = value.to(compute_dtype)
    b = beta.to(compute_dtype)
    new_state = state.to(compute_dtype).clone()
    out = torch.zeros(T, Nv, Dv, dtype=compute_dtype)
    lens = [int(x) for x in actual_seq_lengths]
    idx = [int(x) for x in ssm_state_indices]
    ptr = lens[0]
    for n, L in enumerate(lens[1:]):
        s0, s1 = ptr, ptr + L
        ptr = s1
        if L <= 0:
            continue
        src_tok = s0
        if num_accepted_tokens is not None:
            src_tok = s0 + int(num_accepted_tokens[n]) - 1
        S = new_state[idx[src_tok]].clone()                       # [Nv, Dv, Dk]
        for t in range(s0, s1):
            kt = k[t].repeat_interleave(rep, dim=0)               # [Nv, Dk]
            qt = q[t].repeat_interleave(rep, dim=0)
            if g is not None:
                S = S * torch.exp(g[t].to(compute_dtype))[:, None, None]
            if gk is not None:
                S = S * torch.exp(gk[t].to(compute_dtype))[:, None, :]
            delta = (v[t] - torch.einsum("hvk,hk->hv", S, kt)) * b[t][:, None]
            S = S + delta[:, :, None] * kt[:, None, :]
            out[t] = torch.einsum("hvk,hk->hv", S, qt)
            new_state[idx[t]] = S
    return out, new_state
