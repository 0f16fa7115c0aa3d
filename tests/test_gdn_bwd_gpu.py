"""Parity of the GDN backward operators (through the C ABI) against the CPU oracle, operator by operator
on the same bf16 inputs, and of their composition against autograd through the per-token recurrence.
Cases follow the reference's sweeps: dense, grouped value heads, ragged tails, packed variable-length
batches with an empty sequence (test_npu_chunk_bwd_dv_local.py, test_npu_chunk_bwd_dqkwg.py,
test_npu_prepare_wy_repr_bwd_da.py, test_npu_prepare_wy_repr_bwd_full.py)."""
import pytest
import torch

from oracle import gdn, gdn_bwd
from oracle.kda import chunk_gated_delta_rule_bwd_dhu as dhu_oracle
from util import assert_close, err_stats, TOL_BF16

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
F = torch.nn.functional

CASES = [
    # B, T, Hv, Hk, K, V, cu_seqlens
    (2, 128, 2, 2, 128, 128, None),
    (1, 200, 4, 2, 128, 128, None),                     # grouped value heads + ragged tail
    (1, 1, 1, 1, 128, 128, None),
    (1, 65, 2, 2, 64, 64, None),
    (1, 130, 2, 1, 64, 128, None),
    (1, 261, 2, 1, 128, 128, [0, 1, 16, 33, 33, 96, 160, 261]),   # lengths 1,15,17,0,63,64,101
    (1, 150, 2, 1, 128, 256, None),                     # V = 256: two value slabs in chunk_bwd_dqkwg
    (1, 200, 2, 2, 128, 256, [0, 70, 200]),
]


def make(B, T, Hv, Hk, K, V, cu, seed, dtype=BF, C=64):
    """Forward quantities of one problem, every tensor rounded to the dtype the operators exchange."""
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen)
    q = F.normalize(rn(B, Hk, T, K), dim=-1).to(dtype)
    k = F.normalize(rn(B, Hk, T, K), dim=-1).to(dtype)
    v = rn(B, Hv, T, V).to(dtype)
    beta = torch.sigmoid(rn(B, Hv, T))
    g = F.logsigmoid(rn(B, Hv, T))
    N = B if cu is None else len(cu) - 1
    h0 = rn(N, Hv, K, V) * 0.1
    do = rn(B, Hv, T, V).to(dtype)
    dht = rn(N, Hv, K, V) * 0.1
    G = gdn.chunk_local_cumsum(g, C, cu_seqlens=cu)
    A0 = gdn.chunk_scaled_dot_kkt(k, G, beta, C, cu_seqlens=cu)
    A = gdn.solve_tri(A0, cu_seqlens=cu, output_dtype=dtype)
    w, u = gdn.recompute_w_u_fwd(k, v, beta, A, C, g=G, cu_seqlens=cu, output_dtype=dtype)
    h, v_new, _ = gdn.chunk_gated_delta_rule_fwd_h(k, w, u, G, initial_state=h0, chunk=C, cu_seqlens=cu, output_dtype=dtype)
    return dict(q=q, k=k, v=v, beta=beta, g=g, G=G, A=A, w=w, u=u, h=h, v_new=v_new, h0=h0, do=do, dht=dht)


def to_dev(d, dev):
    return {n: t.to(dev) for n, t in d.items()}


@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", CASES)
def test_backward_operators_against_oracle(dev, case, dtype):
    from fla_hip import ops
    B, T, Hv, Hk, K, V, cu = case
    scale = K ** -0.5
    d = make(B, T, Hv, Hk, K, V, cu, seed=T + K, dtype=dtype)
    BF = dtype                   # the dtype the operators exchange
    TOL_BF16 = 2e-2 if dtype == torch.bfloat16 else 5e-3
    x = to_dev(d, dev)
    kw = dict(cu_seqlens=cu)

    # chunk_bwd_dv_local
    dv_l = ops.chunk_bwd_dv_local(x["q"], x["k"], x["do"], x["G"], scale, 64, **kw)
    dv_l_ref = gdn_bwd.chunk_bwd_dv_local(d["q"], d["k"], d["do"], d["G"], scale, 64, output_dtype=torch.float32, **kw)
    assert dv_l.dtype == BF and dv_l.shape == d["do"].shape
    assert_close(dv_l, dv_l_ref, TOL_BF16, "dv_local")

    # the reverse scan feeds the remaining operators (oracle values, rounded as exchanged)
    dh_ref, dh0_ref, dv2_ref = dhu_oracle(d["q"], d["k"], d["w"], d["do"], dv_l_ref.to(BF), scale, 64, g=d["G"],
                                          dht=d["dht"], **kw)
    dh, dv2 = dh_ref.to(BF), dv2_ref.to(BF)

    # chunk_bwd_dqkwg
    dq, dk, dw, dg = ops.chunk_bwd_dqkwg(x["q"], x["k"], x["v_new"], x["G"], x["h"], x["do"], dh.to(dev), dv2.to(dev), 64,
                                         scale=scale, **kw)
    dq_r, dk_r, dw_r, dg_r = gdn_bwd.chunk_bwd_dqkwg(d["q"], d["k"], d["v_new"], d["G"], d["h"], d["do"], dh, dv2, scale, 64,
                                                     output_dtype=torch.float32, **kw)
    assert dq.shape == d["q"].shape and dk.shape == d["k"].shape and dw.shape == d["w"].shape and dg.shape == d["G"].shape
    assert dg.dtype == torch.float32
    assert_close(dq, dq_r, TOL_BF16, "dq")
    assert_close(dk, dk_r, TOL_BF16, "dk")
    assert_close(dw, dw_r, TOL_BF16, "dw")
    # dg sums hundreds of bf16-rounded products of both signs: bound the error against the gradient's scale
    st = err_stats(dg, dg_r)
    assert st["rel_max"] <= TOL_BF16, f"dg: {st}"

    # prepare_wy_repr_bwd_da: transposed (upper-triangular) storage, zero tail columns
    dwb = dw_r.to(BF)
    dA = ops.prepare_wy_repr_bwd_da(x["k"], x["v"], x["beta"], x["A"], dwb.to(dev), dv2.to(dev), x["G"], chunk_size=64, **kw)
    dA_ref = gdn_bwd.prepare_wy_repr_bwd_da(d["k"], d["v"], d["beta"], d["A"], dwb, dv2, d["G"], 64,
                                            output_dtype=torch.float32, **kw)
    st = err_stats(dA, dA_ref)
    assert st["rel_max"] <= TOL_BF16, f"dA: {st}"
    a = dA.float().cpu()
    for b, n, ci, s, e in gdn.chunk_spans(B, T, 64, cu):
        blk = a[b, :, s:e]
        assert float(torch.tril(blk[:, :, : e - s], 0).abs().max()) == 0.0
        if e - s < 64:
            assert float(blk[:, :, e - s:].abs().max()) == 0.0

    # prepare_wy_repr_bwd_full
    dAb = dA_ref.to(BF)
    dk2, dv3, db, dg2 = ops.prepare_wy_repr_bwd_full(x["k"], x["v"], x["beta"], x["A"], dAb.to(dev), dwb.to(dev),
                                                     dv2.to(dev), x["G"], 64, **kw)
    dk2_r, dv3_r, db_r, dg2_r = gdn_bwd.prepare_wy_repr_bwd_full(d["k"], d["v"], d["beta"], d["A"], dAb, dwb, dv2, d["G"], 64,
                                                                 output_dtype=torch.float32, **kw)
    assert db.dtype == torch.float32 and dg2.dtype == torch.float32
    assert_close(dv3, dv3_r, TOL_BF16, "dv")
    for name, got, ref in (("dk2", dk2, dk2_r), ("dbeta", db, db_r), ("dg2", dg2, dg2_r)):
        st = err_stats(got, ref)
        assert st["rel_max"] <= TOL_BF16, f"{name}: {st}"

    # prepare_wy_repr_bwd: one call == bwd_da followed by bwd_full, bit for bit
    one = ops.prepare_wy_repr_bwd(x["k"], x["v"], x["beta"], x["A"], dwb.to(dev), dv2.to(dev), x["G"], 64, **kw)
    two = ops.prepare_wy_repr_bwd_full(x["k"], x["v"], x["beta"], x["A"], dA, dwb.to(dev), dv2.to(dev), x["G"], 64, **kw)
    for name, a_, b_ in zip(("dk", "dv", "dbeta", "dg"), one, two):
        assert torch.equal(a_, b_), name

    # the accumulating form adds the same dk and dg (taken in fp32) to what the caller's tensors hold
    from fla_hip.ops import _hip_ctypes as raw
    torch.manual_seed(5)
    dk_acc = (torch.randn_like(two[0].float()) * two[0].float().abs().mean()).to(dtype)
    dg_acc = torch.randn_like(two[3]) * two[3].abs().mean()
    dk0, dg0 = dk_acc.clone(), dg_acc.clone()
    dv_a, db_a = raw.prepare_wy_repr_bwd_full_accumulate(x["k"], x["v"], x["beta"], x["A"], dA, dwb.to(dev), dv2.to(dev),
                                                         x["G"], dk_acc, dg_acc, 64, **kw)
    assert torch.equal(dv_a, two[1]) and torch.equal(db_a, two[2])
    assert_close(dk_acc, dk0.float() + dk2_r.to(dev), TOL_BF16, "dk accumulated")
    assert_close(dg_acc, dg0 + two[3], 1e-6, "dg accumulated")
    # without dA the same kernel forms prepare_wy_repr_bwd_da's result itself (dA never goes through memory)
    dk_f, dg_f = dk0.clone(), dg0.clone()
    dv_f, db_f = raw.prepare_wy_repr_bwd_full_accumulate(x["k"], x["v"], x["beta"], x["A"], None, dwb.to(dev), dv2.to(dev),
                                                         x["G"], dk_f, dg_f, 64, **kw)
    assert torch.equal(dv_f, two[1])
    assert_close(dk_f, dk0.float() + dk2_r.to(dev), TOL_BF16, "dk accumulated, dA formed in the kernel")
    for name, got, ref in (("dbeta", db_f, db_r), ("dg2", dg_f - dg0, dg2_r)):
        st = err_stats(got, ref)
        assert st["rel_max"] <= TOL_BF16, f"{name}, dA formed in the kernel: {st}"
    # without A as well the kernel rebuilds each chunk's inverse as chunk_scaled_dot_kkt_inverse does.  dv = (A^T du) beta
    # is one matrix product and one multiply per element, so it pins the rebuilt matrix bit for bit against a call that
    # is handed that operator's result; the sums behind dk, dg and dbeta may differ in their last fp32 bit (the two forms
    # are separate instances of the kernel, and the compiler is free to contract their multiply-adds differently), which
    # now and then rounds a 16-bit result to the other neighbour
    A_dev = ops.chunk_scaled_dot_kkt_inverse(x["k"], x["G"], x["beta"], chunk_size=64, **kw)
    outs = []
    for A_in in (A_dev, None):
        dk_i, dg_i = dk0.clone(), dg0.clone()
        dv_i, db_i = raw.prepare_wy_repr_bwd_full_accumulate(x["k"], x["v"], x["beta"], A_in, None, dwb.to(dev), dv2.to(dev),
                                                             x["G"], dk_i, dg_i, 64, **kw)
        outs.append((dk_i, dg_i, dv_i, db_i))
    assert torch.equal(outs[0][2], outs[1][2]), "dv: A rebuilt in the kernel"
    for name, a_, b_ in zip(("dk", "dg", "dv", "dbeta"), *outs):
        st = err_stats(a_, b_)
        # dg and dbeta are differences of sums that nearly cancel: their last-bit differences are larger relative to the result
        assert st["rel_max"] <= (1e-4 if a_.dtype == torch.float32 else 2.0 ** -7), f"{name}: A rebuilt in the kernel: {st}"
        if a_.dtype != torch.float32:
            assert int((a_ != b_).sum()) <= 2 + 1e-2 * a_.numel(), f"{name}: A rebuilt in the kernel"
    with pytest.raises(RuntimeError, match="A must not be null"):
        raw.prepare_wy_repr_bwd_full_accumulate(x["k"], x["v"], x["beta"], None, dA, dwb.to(dev), dv2.to(dev), x["G"],
                                                dk0.clone(), dg0.clone(), 64, **kw)


@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", CASES)
def test_reverse_scan_forms_the_local_dv_itself(dev, case, dtype):
    """chunk_gated_delta_rule_bwd_dhu without dv (an extension for 64-token chunks and the scalar gate): the scan forms
    chunk_bwd_dv_local's result from the q, k and d_o tiles it holds.  Against the oracle's two operators on the same
    inputs (the local part enters in fp32 there, unrounded as in the kernel), and against the two-operator route."""
    from fla_hip import ops
    B, T, Hv, Hk, K, V, cu = case
    scale = K ** -0.5
    d = make(B, T, Hv, Hk, K, V, cu, seed=T + V, dtype=dtype)
    tol = 2e-2 if dtype == torch.bfloat16 else 5e-3
    x = to_dev(d, dev)
    kw = dict(cu_seqlens=cu)
    dv_l_ref = gdn_bwd.chunk_bwd_dv_local(d["q"], d["k"], d["do"], d["G"], scale, 64, output_dtype=torch.float32, **kw)
    dh_ref, dh0_ref, dv2_ref = dhu_oracle(d["q"], d["k"], d["w"], d["do"], dv_l_ref, scale, 64, g=d["G"], dht=d["dht"], **kw)
    args = (x["q"], x["k"], x["w"], x["do"])
    okw = dict(g=x["G"], h0=x["h0"], dht=x["dht"], dh0_per_sequence=True, **kw)
    dh, dh0, dv2 = ops.chunk_gated_delta_rule_bwd_dhu(*args, None, scale, 64, **okw)
    assert dv2.shape == d["do"].shape and dv2.dtype == dtype and dh.dtype == dtype and dh0.dtype == torch.float32
    assert_close(dv2, dv2_ref, tol, "dv2")
    assert_close(dh, dh_ref, tol, "dh")
    assert_close(dh0, dh0_ref, tol, "dh0")
    dv_l = ops.chunk_bwd_dv_local(x["q"], x["k"], x["do"], x["G"], scale, 64, **kw)
    dh_b, dh0_b, dv2_b = ops.chunk_gated_delta_rule_bwd_dhu(*args, dv_l, scale, 64, **okw)
    assert_close(dv2, dv2_b.float(), tol, "dv2 against the two operators")
    assert_close(dh0, dh0_b, tol, "dh0 against the two operators")
    # The two routes are not bit-compatible: with dv given, the local part arrives rounded to 16 bits (as the reference
    # composes it); left out, it enters dv2 unrounded.  They stay a couple of steps of the 16-bit results apart.
    steps = 1e-2 if dtype == torch.bfloat16 else 1.5e-3
    for name, a_, b_ in (("dv2", dv2, dv2_b), ("dh", dh, dh_b), ("dh0", dh0, dh0_b)):
        st = err_stats(a_, b_)
        assert st["rel_max"] <= steps, f"{name}: dv=None against dv=chunk_bwd_dv_local: {st}"
    # 128-token chunks and the per-channel gate keep the operator's own signature
    with pytest.raises(RuntimeError, match="dv may be left out"):
        ops.chunk_gated_delta_rule_bwd_dhu(*args, None, scale, 128, g=x["G"], **kw)


CASES_128 = [
    # B, T, Hv, Hk, K, V, cu_seqlens: full chunks, a last chunk with only its first half, every remainder when packed
    (2, 256, 2, 2, 128, 128, None),
    (1, 200, 4, 2, 128, 128, None),
    (1, 192, 2, 1, 64, 128, None),
    (1, 421, 2, 1, 128, 128, [0, 1, 66, 66, 194, 300, 421]),
    (1, 330, 2, 2, 128, 256, None),
    (1, 130, 2, 2, 64, 64, None),
    (1, 1, 1, 1, 128, 128, None),
    (1, 65, 2, 2, 128, 128, None),
    (2, 129, 2, 1, 128, 128, None),
]


@pytest.mark.parametrize("case", CASES_128)
def test_dv_local_with_128_token_chunks(dev, case):
    """chunk_bwd_dv_local on 128-token chunks (chunk_bwd_dv_local/README.md:114): the gate is cumulated over the whole
    chunk and a row of the first half also sees the queries of the second."""
    from fla_hip import ops
    B, T, Hv, Hk, K, V, cu = case
    d = make(B, T, Hv, Hk, K, V, cu, seed=T + V)
    G = gdn.chunk_local_cumsum(d["g"], 128, cu_seqlens=cu)
    scale = K ** -0.5
    got = ops.chunk_bwd_dv_local(d["q"].to(dev), d["k"].to(dev), d["do"].to(dev), G.to(dev), scale, 128, cu_seqlens=cu)
    ref = gdn_bwd.chunk_bwd_dv_local(d["q"], d["k"], d["do"], G, scale, 128, output_dtype=torch.float32, cu_seqlens=cu)
    assert got.dtype == BF and got.shape == d["do"].shape
    assert_close(got, ref, TOL_BF16, "dv_local, 128-token chunks")


@pytest.mark.parametrize("case", CASES_128)
def test_backward_operators_with_128_token_chunks(dev, case):
    """The operators that follow dv_local, each on 128-token operands (A [T,128], one h / dh block per 128 tokens, the
    gate cumulated over the chunk) against the oracle on the same 16-bit inputs
    (chunk_gated_delta_rule_bwd_dhu/README.md:101-104, chunk_bwd_dqkwg/README.md:117)."""
    from fla_hip import ops
    B, T, Hv, Hk, K, V, cu = case
    C, scale = 128, K ** -0.5
    d = make(B, T, Hv, Hk, K, V, cu, seed=T + K, C=C)
    x = to_dev(d, dev)
    kw = dict(cu_seqlens=cu)
    dv_l = gdn_bwd.chunk_bwd_dv_local(d["q"], d["k"], d["do"], d["G"], scale, C, output_dtype=torch.float32, **kw).to(BF)
    dh_ref, _, dv2_ref = dhu_oracle(d["q"], d["k"], d["w"], d["do"], dv_l, scale, C, g=d["G"], dht=d["dht"], **kw)
    dh, dv2 = dh_ref.to(BF), dv2_ref.to(BF)

    dq, dk, dw, dg = ops.chunk_bwd_dqkwg(x["q"], x["k"], x["v_new"], x["G"], x["h"], x["do"], dh.to(dev), dv2.to(dev), C,
                                         scale=scale, **kw)
    dq_r, dk_r, dw_r, dg_r = gdn_bwd.chunk_bwd_dqkwg(d["q"], d["k"], d["v_new"], d["G"], d["h"], d["do"], dh, dv2, scale, C,
                                                     output_dtype=torch.float32, **kw)
    assert_close(dq, dq_r, TOL_BF16, "dq, 128-token chunks")
    assert_close(dk, dk_r, TOL_BF16, "dk, 128-token chunks")
    assert_close(dw, dw_r, TOL_BF16, "dw, 128-token chunks")
    st = err_stats(dg, dg_r)
    assert st["rel_max"] <= TOL_BF16, f"dg: {st}"

    # prepare_wy_repr_bwd_da / _full / both in one call, A and dA 128 wide
    dwb = dw_r.to(BF)
    dA = ops.prepare_wy_repr_bwd_da(x["k"], x["v"], x["beta"], x["A"], dwb.to(dev), dv2.to(dev), x["G"], chunk_size=C, **kw)
    dA_ref = gdn_bwd.prepare_wy_repr_bwd_da(d["k"], d["v"], d["beta"], d["A"], dwb, dv2, d["G"], C,
                                            output_dtype=torch.float32, **kw)
    assert dA.shape == d["A"].shape and dA.shape[-1] == C
    st = err_stats(dA, dA_ref)
    assert st["rel_max"] <= TOL_BF16, f"dA: {st}"
    a = dA.float().cpu()
    for b, n, ci, s0, e0 in gdn.chunk_spans(B, T, C, cu):
        blk = a[b, :, s0:e0]
        assert float(torch.tril(blk[:, :, : e0 - s0], 0).abs().max()) == 0.0
        if e0 - s0 < C:
            assert float(blk[:, :, e0 - s0:].abs().max()) == 0.0
    dAb = dA_ref.to(BF)
    dk2, dv3, db, dg2 = ops.prepare_wy_repr_bwd_full(x["k"], x["v"], x["beta"], x["A"], dAb.to(dev), dwb.to(dev),
                                                     dv2.to(dev), x["G"], C, **kw)
    dk2_r, dv3_r, db_r, dg2_r = gdn_bwd.prepare_wy_repr_bwd_full(d["k"], d["v"], d["beta"], d["A"], dAb, dwb, dv2, d["G"], C,
                                                                 output_dtype=torch.float32, **kw)
    assert_close(dv3, dv3_r, TOL_BF16, "dv, 128-token chunks")
    for name, got, ref in (("dk2", dk2, dk2_r), ("dbeta", db, db_r), ("dg2", dg2, dg2_r)):
        st = err_stats(got, ref)
        assert st["rel_max"] <= TOL_BF16, f"{name}: {st}"
    one = ops.prepare_wy_repr_bwd(x["k"], x["v"], x["beta"], x["A"], dwb.to(dev), dv2.to(dev), x["G"], C, **kw)
    two = ops.prepare_wy_repr_bwd_full(x["k"], x["v"], x["beta"], x["A"], dA, dwb.to(dev), dv2.to(dev), x["G"], C, **kw)
    for name, a_, b_ in zip(("dk", "dv", "dbeta", "dg"), one, two):
        assert torch.equal(a_, b_), name


@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", [(CASES[1], 64), (CASES[5], 64), (CASES[6], 64), (CASES_128[1], 128), (CASES_128[3], 128),
                                  (CASES_128[4], 128)],
                         ids=lambda cc: f"T{cc[0][1]}-V{cc[0][5]}-C{cc[1]}")
def test_backward_pipeline_against_recurrence_autograd(dev, case, dtype):
    """The composed GPU backward against autograd (fp64) through the per-token recurrence on the same bf16
    inputs: every gradient within 2e-2 of its own scale; on 64- and on 128-token chunks."""
    from fla_hip import pipeline
    (B, T, Hv, Hk, K, V, cu), C = case
    scale = K ** -0.5
    d = make(B, T, Hv, Hk, K, V, cu, seed=77, dtype=dtype, C=C)
    dd = torch.float64
    leaf = {n: d[n].to(dd).requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "h0")}
    o, final = gdn.naive_recurrent_gated_delta_rule(leaf["q"], leaf["k"], leaf["v"], leaf["g"], leaf["beta"], scale,
                                                    initial_state=leaf["h0"], output_final_state=True, cu_seqlens=cu,
                                                    compute_dtype=dd)
    ((o * d["do"].to(dd)).sum() + (final * d["dht"].to(dd)).sum()).backward()
    x = to_dev(d, dev)
    # pipeline layouts: g, beta [B,T,H]; do [B,T,H,V]
    got = pipeline.flash_chunk_gated_delta_rule_bwd(
        x["q"], x["k"], x["v"], x["G"].transpose(1, 2).contiguous(), x["beta"].transpose(1, 2).contiguous(), None, scale,
        x["h0"], x["do"].transpose(1, 2).contiguous(), x["dht"], cu_seqlens=cu, chunk_size=C)
    dq, dk, dv, db, dg, dh0 = got
    want = dict(dq=leaf["q"].grad, dk=leaf["k"].grad, dv=leaf["v"].grad, db=leaf["beta"].grad.transpose(1, 2),
                dg=leaf["g"].grad.transpose(1, 2), dh0=leaf["h0"].grad)
    for name, t in (("dq", dq), ("dk", dk), ("dv", dv), ("db", db), ("dg", dg), ("dh0", dh0)):
        st = err_stats(t, want[name])
        assert st["rel_max"] <= TOL_BF16, f"{name}: {st}"


def test_backward_linearity_at_full_head_size(dev):
    """Size-independent property at the benchmark's head shape (T shortened): the backward is linear in
    (do, dht), so gradients of a sum of two cotangents equal the sum of gradients up to bf16 rounding."""
    from fla_hip import pipeline
    B, T, H, K, V = 1, 1024, 4, 128, 128
    d = make(B, T, H, H, K, V, None, seed=3)
    x = to_dev(d, dev)
    gen = torch.Generator().manual_seed(9)
    do2 = torch.randn(B, T, H, V, generator=gen).to(BF).to(dev)
    do1 = x["do"].transpose(1, 2).contiguous()
    args = (x["q"], x["k"], x["v"], x["G"].transpose(1, 2).contiguous(), x["beta"].transpose(1, 2).contiguous(), None,
            K ** -0.5, x["h0"])
    r1 = pipeline.flash_chunk_gated_delta_rule_bwd(*args, do1, x["dht"])
    r2 = pipeline.flash_chunk_gated_delta_rule_bwd(*args, do2, None)
    r12 = pipeline.flash_chunk_gated_delta_rule_bwd(*args, (do1.float() + do2.float()).to(BF), x["dht"])
    for name, a, b2, c in zip(("dq", "dk", "dv", "db", "dg", "dh0"), r1, r2, r12):
        st = err_stats(c, a.float() + b2.float())
        assert st["rel_max"] <= TOL_BF16, f"{name}: {st}"


def test_autograd_through_flash_gated_delta_rule(dev):
    """loss.backward() through the pipeline entry (fused forward, composed backward) against fp64 autograd
    through the recurrence."""
    from fla_hip import pipeline
    B, T, H, K, V = 1, 150, 2, 128, 128
    d = make(B, T, H, H, K, V, None, seed=11)
    dd = torch.float64
    leaf = {n: d[n].to(dd).requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "h0")}
    o, final = gdn.naive_recurrent_gated_delta_rule(leaf["q"], leaf["k"], leaf["v"], leaf["g"], leaf["beta"], K ** -0.5,
                                                    initial_state=leaf["h0"], output_final_state=True, compute_dtype=dd)
    ((o * d["do"].to(dd)).sum() + (final * d["dht"].to(dd)).sum()).backward()
    x = to_dev(d, dev)
    q, k, v = (x[n].clone().requires_grad_(True) for n in ("q", "k", "v"))
    g = x["g"].transpose(1, 2).contiguous().requires_grad_(True)
    beta = x["beta"].transpose(1, 2).contiguous().requires_grad_(True)
    h0 = x["h0"].clone().requires_grad_(True)
    want = dict(q=leaf["q"].grad, k=leaf["k"].grad, v=leaf["v"].grad, g=leaf["g"].grad.transpose(1, 2),
                beta=leaf["beta"].grad.transpose(1, 2), h0=leaf["h0"].grad)
    # fused forward + backward on 64-token chunks; the six operators forward and backward on 64- and 128-token chunks
    # save_intermediates=False: the reference's memory profile, h, v_new and w recomputed by the backward
    for kwargs in (dict(), dict(fused=False), dict(fused=False, chunk_size=128), dict(save_intermediates=False)):
        for t in (q, k, v, g, beta, h0):
            t.grad = None
        o_g, fin_g = pipeline.flash_gated_delta_rule(q, k, v, g, beta, None, h0, True, **kwargs)
        ((o_g.float() * x["do"].transpose(1, 2).float()).sum() + (fin_g * x["dht"]).sum()).backward()
        for name, t in (("q", q), ("k", k), ("v", v), ("g", g), ("beta", beta), ("h0", h0)):
            st = err_stats(t.grad, want[name])
            assert st["rel_max"] <= TOL_BF16, f"d{name} with {kwargs}: {st}"


def test_autograd_with_token_major_operands(dev):
    """q, k, v as [B,H,T,D] views of token-major [B,T,H,D] tensors (what a model holds after its projections): the same
    gradients as for head-major operands, returned in the memory order of the inputs (no layout copy on the way back)."""
    from fla_hip import pipeline
    B, T, H, K, V = 2, 200, 2, 128, 128
    d = make(B, T, H, H, K, V, None, seed=5)
    x = to_dev(d, dev)
    g = x["g"].transpose(1, 2).contiguous()
    beta = x["beta"].transpose(1, 2).contiguous()
    for l2norm in (False, True):
        grads = []
        for token_major in (False, True):
            leaves = []
            for n in ("q", "k", "v"):
                t = x[n].transpose(1, 2).contiguous().transpose(1, 2) if token_major else x[n].clone()
                leaves.append(t.detach().requires_grad_(True))
            o, _ = pipeline.flash_gated_delta_rule(*leaves, g, beta, None, None, True, use_qk_l2norm_in_kernel=l2norm)
            (o.float() * x["do"].transpose(1, 2).float()).sum().backward()
            for t in leaves:
                assert t.grad.stride() == t.stride()
            grads.append([t.grad for t in leaves])
        for a, b_ in zip(*grads):
            assert torch.equal(a, b_)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_l2norm_kernels_against_oracle(dev, D):
    """Forward and backward of the q/k normalisation on contiguous and on transposed (strided) views."""
    from fla_hip import ops
    gen = torch.Generator().manual_seed(D)
    x = torch.randn(2, 37, 3, D, generator=gen).to(BF)
    dy = torch.randn(2, 37, 3, D, generator=gen).to(BF)
    for view in (lambda t: t, lambda t: t.transpose(1, 2)):
        xv, dv_ = view(x), view(dy)
        y_ref, r_ref = gdn.l2norm_fwd(xv)
        y, rstd = ops.l2norm_fwd(view(x.to(dev)))
        assert y.shape == xv.shape and rstd.shape == xv.shape[:-1] and rstd.dtype == torch.float32
        assert_close(y, y_ref, 1e-2, "y")
        assert_close(rstd, r_ref, 1e-5, "rstd")
        dx = ops.l2norm_bwd(y, rstd, view(dy.to(dev)))
        dx_ref = gdn.l2norm_bwd(y.cpu(), rstd.cpu(), dv_)
        assert_close(dx, dx_ref, 1e-2, "dx")
    h = x.to(torch.float16)
    y, rstd = ops.l2norm_fwd(h.to(dev))
    assert_close(y, gdn.l2norm_fwd(h)[0], 2e-3, "y f16")


@pytest.mark.parametrize("Hk,Hv,kwargs", [(2, 2, {}), (1, 2, {}), (2, 2, dict(fused=False, chunk_size=128)),
                                          (2, 2, dict(save_intermediates=False))],
                         ids=["64-token chunks", "grouped heads", "128-token chunks", "recomputing backward"])
def test_pipeline_with_in_kernel_l2norm(dev, Hk, Hv, kwargs):
    """use_qk_l2norm_in_kernel=True: forward equals the recurrence on normalised q, k; gradients reach the
    UN-normalised q and k (fp64 autograd through F.normalize and the recurrence).  With 64-token chunks the kernels
    that complete dq and dk de-normalise them (chunk_bwd_dqkwg_l2norm, prepare_wy_repr_bwd_full_accumulate with k_rstd);
    with 128-token chunks two l2norm_bwd passes do."""
    from fla_hip import pipeline
    B, T, K, V = 1, 150, 128, 128
    d = make(B, T, Hv, Hk, K, V, None, seed=21)
    gen = torch.Generator().manual_seed(22)
    qraw = (torch.randn(B, Hk, T, K, generator=gen) * 1.7).to(BF)
    kraw = (torch.randn(B, Hk, T, K, generator=gen) * 0.6).to(BF)
    dd = torch.float64
    leaf = {n: t.to(dd).requires_grad_(True) for n, t in (("q", qraw), ("k", kraw), ("v", d["v"]), ("g", d["g"]), ("beta", d["beta"]))}
    o, _ = gdn.naive_recurrent_gated_delta_rule(F.normalize(leaf["q"], dim=-1), F.normalize(leaf["k"], dim=-1), leaf["v"], leaf["g"],
                                                leaf["beta"], K ** -0.5, compute_dtype=dd)
    (o * d["do"].to(dd)).sum().backward()
    x = to_dev(d, dev)
    g = x["g"].transpose(1, 2).contiguous()
    beta = x["beta"].transpose(1, 2).contiguous()
    # inference path
    o_inf, _ = pipeline.flash_gated_delta_rule(qraw.to(dev), kraw.to(dev), x["v"], g, beta, use_qk_l2norm_in_kernel=True)
    assert_close(o_inf.transpose(1, 2), o.detach(), TOL_BF16, "o")
    # training path
    q, k, v = (t.to(dev).clone().requires_grad_(True) for t in (qraw, kraw, d["v"]))
    o_g, _ = pipeline.flash_gated_delta_rule(q, k, v, g, beta, use_qk_l2norm_in_kernel=True, **kwargs)
    (o_g.float() * x["do"].transpose(1, 2).float()).sum().backward()
    for name, t in (("q", q), ("k", k), ("v", v)):
        st = err_stats(t.grad, leaf[name].grad)
        assert st["rel_max"] <= TOL_BF16, f"d{name}: {st}"
