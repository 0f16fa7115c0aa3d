"""Parity of the KDA-side operators (through the C ABI) against the CPU oracle:
kda_gate_cumsum and chunk_gated_delta_rule_bwd_dhu (scalar-gate and per-channel-gate variants),
on dense, GVA, ragged-tail and packed variable-length cases."""
import math

import pytest
import torch

from oracle import gdn, kda
from util import assert_close, err_stats, TOL_BF16, TOL_STATE

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


# ---------------------------------------------------------------------------------------------
# kda_gate_cumsum
# ---------------------------------------------------------------------------------------------
GATE_CASES = [
    # B, Hv, T, K, chunk, cu, dtype, use_gate, safe, bias
    (2, 3, 200, 128, 64, None, torch.float32, False, False, False),
    (1, 2, 261, 128, 64, [0, 1, 16, 33, 33, 96, 160, 261], torch.float32, True, False, True),
    (1, 2, 300, 64, 128, None, BF, True, True, True),
    (2, 2, 65, 32, 64, None, BF, True, False, False),
    (1, 1, 1, 256, 64, None, torch.float32, True, True, False),
]


@pytest.mark.parametrize("case", GATE_CASES)
def test_kda_gate_cumsum(dev, case):
    from fla_hip import ops
    B, Hv, T, K, chunk, cu, dt, use_gate, safe, bias = case
    gen = torch.Generator().manual_seed(T + K)
    g = (torch.randn(B, Hv, T, K, generator=gen) * (1.5 if use_gate else 0.1) - (0.0 if use_gate else 0.05)).to(dt)
    A_log = torch.randn(Hv, generator=gen) * 0.5
    dt_bias = torch.randn(Hv * K, generator=gen) * 0.5 if bias else None
    out = ops.kda_gate_cumsum(g.to(dev), chunk, A_log=A_log.to(dev) if use_gate else None,
                              dt_bias=None if dt_bias is None else dt_bias.to(dev), cu_seqlens=cu,
                              use_gate_in_kernel=use_gate, safe_gate=safe, lower_bound=-3.0 if safe else None)
    ref = kda.kda_gate_cumsum(g, chunk, A_log=A_log, dt_bias=dt_bias, cu_seqlens=cu, use_gate_in_kernel=use_gate,
                              safe_gate=safe, lower_bound=-3.0)
    assert out.dtype == torch.float32 and out.shape == g.shape
    assert_close(out, ref, 1e-5, "gk")


def test_kda_gate_cumsum_errors(dev):
    from fla_hip import ops
    g = torch.zeros(1, 2, 64, 128, device=dev)
    with pytest.raises(RuntimeError, match="A_log"):
        ops.kda_gate_cumsum(g, 64, use_gate_in_kernel=True)
    with pytest.raises(RuntimeError, match="chunk_size"):
        ops.kda_gate_cumsum(g, 32)
    with pytest.raises(RuntimeError, match="lower_bound"):
        ops.kda_gate_cumsum(g, 64, A_log=torch.zeros(2, device=dev), use_gate_in_kernel=True, safe_gate=True,
                            lower_bound=-7.0)


# ---------------------------------------------------------------------------------------------
# chunk_gated_delta_rule_bwd_dhu
# ---------------------------------------------------------------------------------------------
def dhu_inputs(B, T, Hk, Hv, K, V, seed, per_channel):
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen)
    q = (rn(B, Hk, T, K) * K ** -0.5).to(BF)
    k = torch.nn.functional.normalize(rn(B, Hk, T, K), dim=-1).to(BF)
    w = (rn(B, Hv, T, K) * 0.1).to(BF)
    d_o = (rn(B, Hv, T, V) * 0.5).to(BF)
    dv = (rn(B, Hv, T, V) * 0.5).to(BF)
    if per_channel:
        gate = -torch.rand(B, Hv, T, K, generator=gen) * 0.1
    else:
        gate = -torch.rand(B, Hv, T, generator=gen) * 0.1
    return q, k, w, d_o, dv, gate


DHU_CASES = [
    # B, T, Hk, Hv, K, V, cu, per_channel, dht
    (2, 256, 2, 2, 128, 128, None, False, False),
    (1, 200, 2, 4, 128, 128, None, False, True),                      # GVA + ragged tail + terminal gradient
    (1, 261, 1, 2, 128, 128, [0, 1, 16, 33, 33, 96, 160, 261], False, True),
    (2, 192, 2, 2, 128, 128, None, True, False),
    (1, 261, 2, 2, 128, 128, [0, 1, 16, 33, 33, 96, 160, 261], True, True),
    (1, 130, 2, 2, 64, 64, None, False, False),
    (1, 130, 1, 2, 64, 128, None, True, True),
    (1, 96, 1, 1, 128, 256, None, False, False),
    (2, 200, 1, 2, 256, 128, None, True, True),                       # 256 channels: the unpipelined per-channel scan
    (1, 261, 2, 2, 256, 256, [0, 1, 16, 33, 33, 96, 160, 261], True, True),
]


# 128-token chunks (chunk_gated_delta_rule_bwd_dhu/README.md:101-104) with either gate (the per-channel one on the kernels
# for up to 128 channels): full chunks, a last chunk with only its first half, packed sequences of every remainder
DHU_CASES_128 = [c for c in DHU_CASES if not c[7] or c[4] <= 128] + [
    (1, 421, 2, 2, 128, 128, [0, 1, 66, 66, 194, 300, 421], False, True),
    (1, 192, 1, 2, 128, 128, None, False, True),
    (1, 421, 2, 2, 128, 128, [0, 1, 66, 66, 194, 300, 421], True, True),
    (1, 192, 1, 2, 128, 128, None, True, False),
]


@pytest.mark.parametrize("case", [(c, 64) for c in DHU_CASES] + [(c, 128) for c in DHU_CASES_128],
                         ids=lambda cc: f"T{cc[0][1]}-K{cc[0][4]}-V{cc[0][5]}-{'gK' if cc[0][7] else 'g'}-C{cc[1]}")
def test_bwd_dhu(dev, case):
    from fla_hip import ops
    (B, T, Hk, Hv, K, V, cu, per_channel, with_dht), C = case
    q, k, w, d_o, dv, gate = dhu_inputs(B, T, Hk, Hv, K, V, seed=T + V, per_channel=per_channel)
    scale = K ** -0.5
    # chunk-local cumulated gates, as the callers provide them
    if per_channel:
        gcum = kda.kda_gate_cumsum(gate, C, cu_seqlens=cu)        # log2 units
        # q and k carry their gates in this variant (they stay O(1): 2^{gk} <= 1, 2^{gk_last - gk} <= 1)
        qg = (q.float().repeat_interleave(Hv // Hk, 1) * torch.exp2(gcum)).to(BF)
        last = torch.zeros_like(gcum)
        for b, n, ci, s, e in gdn.chunk_spans(B, T, C, cu):
            last[b, :, s:e] = gcum[b, :, e - 1:e]
        kg = (k.float().repeat_interleave(Hv // Hk, 1) * torch.exp2(last - gcum)).to(BF)
        q_in, k_in = qg, kg
    else:
        gcum = gdn.chunk_local_cumsum(gate, C, cu_seqlens=cu)
        q_in, k_in = q, k
    N = B if cu is None else len(cu) - 1
    gen = torch.Generator().manual_seed(3)
    dht = torch.randn(N, Hv, K, V, generator=gen) * 0.1 if with_dht else None
    h0 = torch.zeros(N, Hv, K, V)

    kw = dict(gK=gcum.to(dev), use_exp2=True) if per_channel else dict(g=gcum.to(dev))
    args = [t.to(dev) for t in (q_in, k_in, w, d_o, dv)]
    dh, dh0, dv2 = ops.chunk_gated_delta_rule_bwd_dhu(*args, scale, C, h0=h0.to(dev),
                                                      dht=None if dht is None else dht.to(dev), cu_seqlens=cu,
                                                      dh0_per_sequence=True, **kw)
    okw = dict(gK=gcum) if per_channel else dict(g=gcum)
    dh_ref, dh0_ref, dv2_ref = kda.chunk_gated_delta_rule_bwd_dhu(q_in, k_in, w, d_o, dv, scale, C, dht=dht,
                                                                  cu_seqlens=cu, **okw)
    assert dh.dtype == BF and dv2.dtype == BF and dh0.dtype == torch.float32
    assert_close(dv2, dv2_ref, TOL_BF16, "dv2")
    assert_close(dh, dh_ref, TOL_BF16, "dh")
    assert_close(dh0, dh0_ref, TOL_BF16, "dh0")

    # reference-form dh0: bf16 buffer of dh's shape, written at the first chunk of each sequence
    dh_b, dh0_b, dv2_b = ops.chunk_gated_delta_rule_bwd_dhu(*args, scale, C, h0=h0.to(dev),
                                                            dht=None if dht is None else dht.to(dev), cu_seqlens=cu,
                                                            **kw)
    assert torch.equal(dh_b, dh) and torch.equal(dv2_b, dv2)
    assert dh0_b.shape == dh.shape and dh0_b.dtype == BF
    first = {}
    for b, n, ci, s, e in gdn.chunk_spans(B, T, C, cu):
        first.setdefault(n, (b, ci))
    for n, (b, ci) in first.items():
        assert torch.equal(dh0_b[b, :, ci].float(), dh0[n].to(BF).float())
    # without h0 no dh0 is produced
    out3 = ops.chunk_gated_delta_rule_bwd_dhu(*args, scale, C, cu_seqlens=cu, **kw)
    assert out3[1] is None


@pytest.mark.parametrize("case", [c for c in DHU_CASES if c[7] and c[4] <= 128],
                         ids=lambda c: f"T{c[1]}-K{c[4]}-V{c[5]}")
def test_kda_bwd_dhu_forms_dv_from_the_score_blocks(dev, case):
    """chunk_kda_bwd_dhu (no counterpart in the reference): the per-channel-gate scan with dv = Aqk^T d_o formed
    inside.  Against the oracle's two operators (chunk_kda_bwd_dav's dv, then the scan) and against the two-operator
    route on the device."""
    from fla_hip import ops
    from fla_hip.ops import _hip_ctypes as raw
    B, T, Hk, Hv, K, V, cu, _, with_dht = case
    q, k, w, d_o, _, gate = dhu_inputs(B, T, Hk, Hv, K, V, seed=T + V + 1, per_channel=True)
    scale = K ** -0.5
    gcum = kda.kda_gate_cumsum(gate, 64, cu_seqlens=cu)
    qg = (q.float().repeat_interleave(Hv // Hk, 1) * torch.exp2(gcum)).to(BF)
    last = torch.zeros_like(gcum)
    gen = torch.Generator().manual_seed(11)
    Aqk = torch.zeros(B, Hv, T, 64)
    for b, n, ci, s, e in gdn.chunk_spans(B, T, 64, cu):
        last[b, :, s:e] = gcum[b, :, e - 1:e]
        Aqk[b, :, s:e, :e - s] = torch.tril(torch.randn(Hv, e - s, e - s, generator=gen) * 0.3)
    Aqk = Aqk.to(BF)
    kg = (k.float().repeat_interleave(Hv // Hk, 1) * torch.exp2(last - gcum)).to(BF)
    N = B if cu is None else len(cu) - 1
    dht = torch.randn(N, Hv, K, V, generator=gen) * 0.1 if with_dht else None
    h0 = torch.zeros(N, Hv, K, V, device=dev)
    dht_d = None if dht is None else dht.to(dev)
    qd, kd, wd, od, ad, gd = (t.to(dev) for t in (qg, kg, w, d_o, Aqk, gcum))
    dh, dh0, dv2 = raw.chunk_kda_bwd_dhu(qd, kd, wd, od, ad, scale, 64, gK=gd, h0=h0, dht=dht_d, cu_seqlens=cu)
    assert dh.dtype == BF and dv2.dtype == BF and dh0.dtype == torch.float32 and dv2.shape == d_o.shape
    _, dv_ref = kda.chunk_kda_bwd_dav(d_o, d_o, Aqk, scale, cu_seqlens=cu)
    # dv enters the oracle's scan unrounded, as it stays in the kernel's accumulators
    dh_ref, dh0_ref, dv2_ref = kda.chunk_gated_delta_rule_bwd_dhu(qg, kg, w, d_o, dv_ref, scale, 64, dht=dht, cu_seqlens=cu,
                                                                  gK=gcum)
    assert_close(dv2, dv2_ref, TOL_BF16, "dv2")
    assert_close(dh, dh_ref, TOL_BF16, "dh")
    assert_close(dh0, dh0_ref, TOL_BF16, "dh0")
    _, dv_two = raw.chunk_kda_bwd_dav(od, od, ad, scale, cu_seqlens=cu)
    two = ops.chunk_gated_delta_rule_bwd_dhu(qd, kd, wd, od, dv_two, scale, 64, gK=gd, use_exp2=True, h0=h0, dht=dht_d,
                                             cu_seqlens=cu, dh0_per_sequence=True)
    # the two-operator route rounds dv to 16 bits on its way through memory, the scan takes it unrounded: a couple of
    # steps of the 16-bit results apart, inside the oracle's bound
    for name, a_, b_ in zip(("dh", "dh0", "dv2"), (dh, dh0, dv2), two):
        st = err_stats(a_, b_)
        assert st["rel_max"] <= 1e-2, f"{name} against the two-operator route: {st}"
    assert raw.chunk_kda_bwd_dhu(qd, kd, wd, od, ad, scale, 64, gK=gd, cu_seqlens=cu)[1] is None
    with pytest.raises(RuntimeError, match="Aqk"):
        raw.chunk_kda_bwd_dhu(qd, kd, wd, od, None, scale, 64, gK=gd, cu_seqlens=cu)


def test_bwd_dhu_first_chunk_is_terminal_gradient(dev):
    """dh of the last chunk is the terminal gradient itself (zero without dht)."""
    from fla_hip import ops
    q, k, w, d_o, dv, gate = dhu_inputs(1, 128, 1, 1, 128, 128, seed=1, per_channel=False)
    g = gdn.chunk_local_cumsum(gate, 64)
    dh, _, dv2 = ops.chunk_gated_delta_rule_bwd_dhu(*[t.to(dev) for t in (q, k, w, d_o, dv)], 0.1, 64, g=g.to(dev))
    assert float(dh[:, :, -1].abs().max()) == 0.0
    assert torch.equal(dv2[:, :, 64:].cpu(), dv[:, :, 64:])          # k . 0 adds nothing


def test_bwd_dhu_errors(dev):
    from fla_hip import ops
    q, k, w, d_o, dv, gate = dhu_inputs(1, 64, 1, 1, 128, 128, seed=1, per_channel=False)
    a = [t.to(dev) for t in (q, k, w, d_o, dv)]
    with pytest.raises(ValueError, match="Exactly one"):
        ops.chunk_gated_delta_rule_bwd_dhu(*a, 0.1, 64)
    with pytest.raises(ValueError, match="g must have shape"):
        ops.chunk_gated_delta_rule_bwd_dhu(*a, 0.1, 64, g=torch.zeros(1, 2, 64, device=dev))
    with pytest.raises(RuntimeError, match="chunk_size"):
        ops.chunk_gated_delta_rule_bwd_dhu(*a, 0.1, 32, g=gate.to(dev))


# ---------------------------------------------------------------------------------------------
# chunk_gated_delta_rule_fwd_h with the key-wise gate gk (README.md:16-30 of the operator): the KDA state scan
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("case", [(2, 200, 2, 2, 128, 128, None, False), (1, 261, 2, 4, 128, 128, [0, 1, 16, 33, 33, 96, 160, 261], False),
                                  (1, 130, 1, 2, 64, 64, None, True), (1, 96, 1, 1, 128, 256, None, False)])
def test_fwd_h_with_key_wise_gate(dev, case):
    from fla_hip import ops
    B, T, Hk, Hv, K, V, cu, v_first = case
    gen = torch.Generator().manual_seed(T + K)
    N = B if cu is None else len(cu) - 1
    kgt = (torch.randn(B, Hv, T, K, generator=gen) * 0.1).to(BF)           # k with its gate applied, per value head
    w = (torch.randn(B, Hv, T, K, generator=gen) * 0.1).to(BF)
    u = torch.randn(B, Hv, T, V, generator=gen).to(BF)
    gk = kda.kda_gate_cumsum(torch.nn.functional.logsigmoid(torch.randn(B, Hv, T, K, generator=gen)) * 0.3, 64, cu_seqlens=cu)
    h0 = torch.randn(N, Hv, K, V, generator=gen) * 0.1
    h_ref, vn_ref, f_ref = gdn.chunk_gated_delta_rule_fwd_h(kgt, w, u, gk=gk, initial_state=h0, output_final_state=True,
                                                            cu_seqlens=cu, lowp=BF, output_dtype=torch.float32)
    h0_d = (h0.transpose(-1, -2).contiguous() if v_first else h0).to(dev)
    h, v_new, final = ops.chunk_gated_delta_rule_fwd_h(kgt.to(dev), w.to(dev), u.to(dev), gk=gk.to(dev), initial_state=h0_d,
                                                       output_final_state=True, cu_seqlens=cu, state_v_first=v_first)
    if v_first:
        h, final = h.transpose(-1, -2), final.transpose(-1, -2)
    assert_close(v_new, vn_ref, TOL_BF16, "v_new")
    assert_close(h, h_ref, TOL_BF16, "h")
    assert_close(final, f_ref, 4e-3, "final_state")
    # both gates together: the scalar one multiplies the same rows
    g = gdn.chunk_local_cumsum(torch.nn.functional.logsigmoid(torch.randn(B, Hv, T, generator=gen)) * 0.2, 64, cu_seqlens=cu)
    if not v_first:
        ref2 = gdn.chunk_gated_delta_rule_fwd_h(kgt, w, u, g, gk=gk, initial_state=h0, output_final_state=True, cu_seqlens=cu,
                                                lowp=BF, output_dtype=torch.float32)
        got2 = ops.chunk_gated_delta_rule_fwd_h(kgt.to(dev), w.to(dev), u.to(dev), g.to(dev), gk=gk.to(dev), initial_state=h0_d,
                                                output_final_state=True, cu_seqlens=cu)
        assert_close(got2[1], ref2[1], TOL_BF16, "v_new (g and gk)")
        assert_close(got2[2], ref2[2], 4e-3, "final_state (g and gk)")
    # 128-token chunks (README.md:87): the gate cumulated over the whole chunk, its decay applied once per chunk
    gk128 = kda.kda_gate_cumsum(torch.nn.functional.logsigmoid(torch.randn(B, Hv, T, K, generator=gen)) * 0.3, 128, cu_seqlens=cu)
    ref3 = gdn.chunk_gated_delta_rule_fwd_h(kgt, w, u, gk=gk128, initial_state=h0, output_final_state=True, chunk=128,
                                            cu_seqlens=cu, lowp=BF, output_dtype=torch.float32)
    got3 = ops.chunk_gated_delta_rule_fwd_h(kgt.to(dev), w.to(dev), u.to(dev), gk=gk128.to(dev), initial_state=h0_d,
                                            output_final_state=True, chunk_size=128, cu_seqlens=cu, state_v_first=v_first)
    h3, f3 = (got3[0].transpose(-1, -2), got3[2].transpose(-1, -2)) if v_first else (got3[0], got3[2])
    assert_close(got3[1], ref3[1], TOL_BF16, "v_new (gk, 128-token chunks)")
    assert_close(h3, ref3[0], TOL_BF16, "h (gk, 128-token chunks)")
    assert_close(f3, ref3[2], 8e-3, "final_state (gk, 128-token chunks)")


# ---------------------------------------------------------------------------------------------
# chunk_kda_bwd_intra (fp32 products; the reference's own tolerance is 2e-4)
# ---------------------------------------------------------------------------------------------
def intra_inputs(B, T, H, K, seed, beta_dtype, cu=None, decay=0.05):
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen)
    q = (rn(B, H, T, K) * 0.1).to(BF)
    k = (rn(B, H, T, K) * 0.1).to(BF)
    inc = -torch.rand(B, H, T, K, generator=gen) * decay
    gk = torch.zeros_like(inc)
    for b, n, ci, s, e in gdn.chunk_spans(B, T, 64, cu):
        gk[b, :, s:e] = inc[b, :, s:e].cumsum(dim=1)
    beta = torch.rand(B, H, T, generator=gen).to(beta_dtype)
    dAqk, dAkk = rn(B, H, T, 64) * 0.1, rn(B, H, T, 64) * 0.1
    dq, dk, dg = rn(B, H, T, K) * 0.01, rn(B, H, T, K) * 0.01, rn(B, H, T, K) * 0.01
    db = rn(B, H, T) * 0.01
    return q, k, gk, beta, dAqk, dAkk, dq, dk, db, dg


def _lay(x, layout):   # head-major [B,H,T,..] -> layout
    if layout == "BNSD":
        return x.contiguous()
    if layout == "BSND":
        return x.transpose(1, 2).contiguous()
    return x[0].transpose(0, 1).contiguous()


def _unlay(x, layout):
    if layout == "BNSD":
        return x
    if layout == "BSND":
        return x.transpose(1, 2)
    return x.transpose(0, 1)[None]


INTRA_CASES = [(K, H, T, "BNSD", None, BF) for K in (64, 128, 256) for H, T in ((1, 1), (2, 15), (3, 16), (2, 17), (1, 63),
                                                                               (2, 64), (3, 65), (2, 129))]
INTRA_CASES += [
    (128, 2, 65, "BSND", None, BF),
    (128, 3, 63, "BNSD", None, torch.float32),
    (128, 3, 129, "TND", [0, 17, 64, 129], BF),
    (128, 2, 261, "TND", [0, 1, 16, 33, 33, 96, 160, 261], torch.float32),
    (128, 2, 130, "BSND", [0, 65, 130], BF),
    (128, 2, 128, "BNSD", None, BF, 2.0),     # strong decay: 2 bits per token and channel
]


@pytest.mark.parametrize("case", INTRA_CASES, ids=lambda c: f"K{c[0]}-H{c[1]}-T{c[2]}-{c[3]}")
def test_chunk_kda_bwd_intra(dev, case):
    from fla_hip import ops
    K, H, T, layout, cu, beta_dtype = case[:6]
    decay = case[6] if len(case) > 6 else 0.05
    B = 1 if layout == "TND" or cu is not None else 2
    x = intra_inputs(B, T, H, K, seed=K + T, beta_dtype=beta_dtype, cu=cu, decay=decay)
    ref = kda.chunk_kda_bwd_intra(*x, chunk=64, cu_seqlens=cu)                       # fp64
    got = ops.chunk_kda_bwd_intra(*[_lay(t, layout).to(dev) for t in x], cu_seqlens=cu, chunk_size=64, safe_gate=True,
                                  layout=layout)
    for name, a, e in zip(("dq", "dk", "db", "dg"), got, ref):
        assert a.dtype == torch.float32
        assert_close(_unlay(a, layout), e.float(), 2e-4, name)


@pytest.mark.parametrize("case", [(64, 2, 130, None), (128, 3, 200, None), (128, 2, 261, [0, 1, 16, 33, 33, 96, 160, 261]),
                                  (256, 1, 65, None)], ids=lambda c: f"K{c[0]}-H{c[1]}-T{c[2]}")
def test_chunk_kda_bwd_intra_with_the_reverse_running_sum(dev, case):
    """The library-only form that also takes the reverse chunk-local running sum of dg (the pass that follows the
    operator in the KDA backward): dq, dk, db equal the operator's bit for bit, dg equals the fp64 reference of the
    operator summed backwards over each chunk."""
    from fla_hip.ops import _hip_ctypes as raw
    K, H, T, cu = case
    x = intra_inputs(1, T, H, K, seed=K + T, beta_dtype=BF, cu=cu)
    ref = kda.chunk_kda_bwd_intra(*x, chunk=64, cu_seqlens=cu)
    dg_ref = ref[3].double().clone()
    for b, n, ci, s, e in gdn.chunk_spans(1, T, 64, cu):
        dg_ref[b, :, s:e] = torch.flip(torch.cumsum(torch.flip(dg_ref[b, :, s:e], dims=[1]), dim=1), dims=[1])
    xd = [t.to(dev) for t in x]
    plain = [t.clone() for t in xd]
    raw.chunk_kda_bwd_intra_inplace(*plain, cu_seqlens=cu)
    fused = [t.clone() for t in xd]
    raw.chunk_kda_bwd_intra_inplace(*fused, cu_seqlens=cu, cumsum_dg=True)
    for i in (6, 7, 8):
        assert torch.equal(plain[i], fused[i])
    assert_close(fused[9], dg_ref.float(), 2e-4, "dg, reverse running sum")
    again = [t.clone() for t in xd]
    raw.chunk_kda_bwd_intra_inplace(*again, cu_seqlens=cu, cumsum_dg=True)
    assert torch.equal(again[9], fused[9])
    # dq and dk handed over in the 16-bit type of q: the fp32 results rounded once
    narrow = [t.clone() for t in xd]
    dq16, dk16 = torch.empty_like(narrow[6], dtype=BF), torch.empty_like(narrow[7], dtype=BF)
    raw.chunk_kda_bwd_intra_inplace(*narrow, cu_seqlens=cu, cumsum_dg=True, dq_out=dq16, dk_out=dk16)
    assert torch.equal(dq16, fused[6].to(BF)) and torch.equal(dk16, fused[7].to(BF))
    assert torch.equal(narrow[9], fused[9]) and torch.equal(narrow[8], fused[8])


def test_chunk_kda_bwd_intra_errors(dev):
    from fla_hip import ops
    x = [t.to(dev) for t in intra_inputs(1, 64, 2, 128, seed=1, beta_dtype=BF)]
    with pytest.raises(RuntimeError, match="safe_gate=False"):
        ops.chunk_kda_bwd_intra(*x, safe_gate=False, layout="BNSD")
    with pytest.raises(RuntimeError, match="chunk_size must be 64"):
        ops.chunk_kda_bwd_intra(*x, chunk_size=128, layout="BNSD")
    with pytest.raises(RuntimeError, match="TND requires cu_seqlens"):
        ops.chunk_kda_bwd_intra(*[t[0] for t in x], layout="TND")
    with pytest.raises(RuntimeError, match="not BNSD"):
        ops.chunk_kda_bwd_intra(*x, cu_seqlens=[0, 64], layout="BNSD")
    bad = list(x)
    bad[4] = bad[4].to(BF)
    with pytest.raises(RuntimeError, match="dAqk must be"):
        ops.chunk_kda_bwd_intra(*bad, layout="BNSD")
    bad = list(x)
    bad[8] = torch.zeros(1, 2, 63, device=dev)
    with pytest.raises(RuntimeError, match="beta/db shape"):
        ops.chunk_kda_bwd_intra(*bad, layout="BNSD")
