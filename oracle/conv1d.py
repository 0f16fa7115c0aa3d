"""CPU oracle (test infrastructure) for causal_conv1d prefill.

Op-native layout (docs/aclnnCausalConv1d.md:57-66): ``x [B,S,D]`` or packed
``[T,D]`` with ``query_start_loc``; ``weight [W,D]``; ``bias [D]``;
``conv_states [N, W-1, D]``.  Semantics follow
torch_custom/fla_npu/test/test_npu_causal_conv1d.py:25-53 (the golden there is
phrased channel-first through F.conv1d; this restatement is an explicit tap
loop so that F.conv1d can serve as an independent pin in the tests):

    y[t,d] = act(bias[d] + sum_{r<W} weight[r,d] * xpad[t + r, d])

where ``xpad`` is the sequence with W-1 rows prepended: zeros, or the rows of
``conv_states[cache]`` when that sequence's ``initial_state_mode`` is 1.  After
the call ``conv_states[cache]`` holds the last W-1 rows of ``xpad``.
"""
from __future__ import annotations

import torch


def causal_conv1d(x, weight, bias=None, conv_states=None, *, query_start_loc=None,
                  cache_indices=None, initial_state_mode=None, activation_mode=0,
                  pad_slot_id=-1, head_num=0):
    """Returns (y, new_conv_states or None).  fp32 accumulate, cast to x.dtype."""
    W, D = weight.shape
    wf = weight.float()
    bf = None if bias is None else bias.float()
    packed = x.dim() == 2
    xs = x.unsqueeze(0) if packed else x
    y = torch.zeros(xs.shape, dtype=torch.float32)
    if packed:
        qsl = [int(v) for v in query_start_loc]
        seqs = [(0, s, e) for s, e in zip(qsl, qsl[1:])]
    else:
        seqs = [(b, 0, xs.shape[1]) for b in range(xs.shape[0])]
    new_states = None if conv_states is None else conv_states.clone()
    for n, (b, s, e) in enumerate(seqs):
        cache = n if cache_indices is None else int(cache_indices[n])
        if cache == pad_slot_id:
            continue
        use_init = (initial_state_mode is not None and int(initial_state_mode[n]) == 1
                    and conv_states is not None)
        head = conv_states[cache, :W - 1].float() if use_init else torch.zeros(W - 1, D)
        xpad = torch.cat([head, xs[b, s:e].float()], dim=0)        # [L + W - 1, D]
        L = e - s
        acc = torch.zeros(L, D)
        for r in range(W):
            acc = acc + wf[r][None, :] * xpad[r:r + L]
        if bf is not None:
            acc = acc + bf[None, :]
        if activation_mode == 1:
            acc = acc * torch.sigmoid(acc)
        y[b, s:e] = acc
        if new_states is not None:
            new_states[cache, :W - 1] = xpad[L:L + W - 1].to(conv_states.dtype)
    y = y.to(x.dtype)
    if head_num > 0:
        Bq, S, _ = y.shape
        y = y.view(Bq, S, head_num, D // head_num).permute(0, 2, 1, 3).contiguous()
    if packed:
        y = y.squeeze(0)
    return y, new_states
