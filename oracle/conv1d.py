"""CPU oracle (test infrastructure) for causal_conv1d: prefill, state update / speculative decode, backward.

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


def causal_conv1d_update(x, weight, bias=None, conv_states=None, *, query_start_loc=None, cache_indices=None,
                         num_accepted_tokens=None, activation_mode=0, pad_slot_id=-1):
    """State-update mode (run_mode=1).  ``x`` is ``[B,S,D]``, ``[B,D]`` (one token per sequence) or packed
    ``[T,D]`` with ``query_start_loc``; ``conv_states [slots, state_len >= W-1, D]`` always supplies the history.

    Without ``num_accepted_tokens`` (test_npu_causal_conv1d.py:56-95, op_kernel/causal_conv1d.h:753-776): history =
    state rows 0..W-2, afterwards those rows hold the last W-1 rows of [history | x].
    With it (speculative decoding, width 4; test_npu_causal_conv1d.py:98-151, causal_conv1d.h:778-860,995-1010):
    offset = clamp(accepted - 1, 0, state_len - (W-1)); history = state rows offset..offset+W-2; afterwards
    rows 0..W-3 = old rows offset+1..offset+W-2 and rows W-2..W-3+S = x, provided they fit (else the plain
    write-back).  Sequences whose cache index equals ``pad_slot_id`` are skipped: their y rows stay as allocated
    (returned as zeros here).  Returns (y, new_conv_states)."""
    W, D = weight.shape
    wf = weight.float()
    bf = None if bias is None else bias.float()
    if query_start_loc is not None:
        qsl = [int(v) for v in query_start_loc]
        xs = x.unsqueeze(0)
        seqs = [(0, s, e) for s, e in zip(qsl, qsl[1:])]
    elif x.dim() == 2:
        xs = x.unsqueeze(1)
        seqs = [(b, 0, 1) for b in range(x.shape[0])]
    else:
        xs = x
        seqs = [(b, 0, x.shape[1]) for b in range(x.shape[0])]
    y = torch.zeros(xs.shape, dtype=torch.float32)
    new_states = conv_states.clone()
    state_len = conv_states.shape[1]
    keep = W - 2
    for n, (b, s, e) in enumerate(seqs):
        slot = n if cache_indices is None else int(cache_indices[n])
        L = e - s
        if slot == pad_slot_id or L <= 0:
            continue
        spec = num_accepted_tokens is not None and W == 4
        offset = 0
        if spec:
            offset = min(max(int(num_accepted_tokens[n]) - 1, 0), state_len - (W - 1))
        hist = conv_states[slot, offset:offset + W - 1].float()
        xr = xs[b, s:e].float()
        xpad = torch.cat([hist, xr], dim=0)
        acc = torch.zeros(L, D)
        for r in range(W):
            acc = acc + wf[r][None, :] * xpad[r:r + L]
        if bf is not None:
            acc = acc + bf[None, :]
        if activation_mode == 1:
            acc = acc * torch.sigmoid(acc)
        y[b, s:e] = acc
        if spec and keep + L <= state_len:
            if keep > 0:
                new_states[slot, :keep] = conv_states[slot, offset + 1:offset + 1 + keep]
            new_states[slot, keep:keep + L] = xs[b, s:e].to(conv_states.dtype)
        else:
            new_states[slot, :W - 1] = xpad[L:L + W - 1].to(conv_states.dtype)
    y = y.to(x.dtype)
    if query_start_loc is not None:
        y = y.squeeze(0)
    elif x.dim() == 2:
        y = y.squeeze(1)
    return y, new_states


def causal_conv1d_bwd(x, y, weight, dy, initial_state=None, dht=None, *, query_start_loc=None, activation=0):
    """Backward of the prefill convolution in the logical layout (x, y, dy ``[B,T,D]`` or packed ``[T,D]``),
    following torch_custom/fla_npu/test/test_npu_causal_conv1d_bwd.py:59-127 (dense) and :145-182 (packed).
    ``y`` is the PRE-activation output (needed when activation is 1 or 2).  States have W rows of which rows
    1..W-1 hold the last W-1 inputs (row 0 is unused and its gradient is zero).  Returns (dx, dw, db, dh0)."""
    W, D = weight.shape
    wf = weight.float()
    packed = x.dim() == 2
    if packed:
        qsl = [int(v) for v in query_start_loc]
        spans = [(0, s, e) for s, e in zip(qsl, qsl[1:])]
        xs, dys = x.unsqueeze(0), dy.unsqueeze(0)
        ys = None if y is None else y.unsqueeze(0)
    else:
        spans = [(b, 0, x.shape[1]) for b in range(x.shape[0])]
        xs, dys, ys = x, dy, y
    N = len(spans)
    dx = torch.zeros(xs.shape, dtype=torch.float32)
    dw = torch.zeros(W, D)
    db = torch.zeros(D)
    dh0 = torch.zeros(N, W, D)
    for n, (b, s, e) in enumerate(spans):
        T = e - s
        g = dys[b, s:e].float()
        if activation != 0:
            yy = ys[b, s:e].float()
            sg = torch.sigmoid(yy)
            g = g * sg * (1.0 + yy * (1.0 - sg))
        xr = xs[b, s:e].float()
        db += g.sum(0)
        # token t of the output reads input row t - j with tap W-1-j; rows before the sequence come from the state
        for j in range(W):
            tap = W - 1 - j
            for t in range(T):
                src = t - j
                if src >= 0:
                    dx[b, s + src] += g[t] * wf[tap]
                    dw[tap] += g[t] * xr[src]
                elif initial_state is not None:
                    slot = W + src                       # src = -1 is the newest history row, row W-1
                    dw[tap] += g[t] * initial_state[n, slot].float()
                    dh0[n, slot] += g[t] * wf[tap]
        if dht is not None:
            tail_start = max(0, T - (W - 1))
            rows = T - tail_start
            dx[b, s + tail_start:e] += dht[n, 1:1 + rows].float()
    dx = dx.to(x.dtype)
    if packed:
        dx = dx.squeeze(0)
    return dx, dw.to(weight.dtype), db.to(weight.dtype), dh0.to(x.dtype)
