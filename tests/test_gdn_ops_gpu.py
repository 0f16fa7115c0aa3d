"""Per-operator parity of the GDN chunk-forward kernels (through the C ABI) against the CPU
oracle, on the cases the reference sweeps: dense, GVA (Hv = 2 Hk), ragged tails
(lengths 1, 15, 16, 17, 63, 64, 65), packed variable-length batches with an empty sequence."""
import pytest
import torch

from oracle import gdn
from util import assert_close, err_stats, TOL_BF16, TOL_STATE

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


F16 = torch.float16
# fp16 carries three more mantissa bits than bf16: its outputs are held to a 4x tighter bound
TOL_OF = {BF: TOL_BF16, F16: TOL_BF16 / 4}


def inputs(B, T, H, K, V, Hk=None, seed=0, init=False, dtype=BF):
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=dtype, seed=seed, Hk=Hk, init_std=0.01 if init else None,
                            head_first_gates=True)
    return d


CASES = [
    # B, T, H, Hk, K, V, cu_seqlens
    (2, 128, 2, 2, 128, 128, None),
    (1, 200, 4, 2, 128, 128, None),                     # GVA + ragged tail (200 = 3*64 + 8)
    (1, 1, 1, 1, 128, 128, None),
    (1, 65, 2, 2, 128, 128, None),
    (1, 261, 2, 1, 128, 128, [0, 1, 16, 33, 33, 96, 160, 261]),   # lengths 1,15,17,0,63,64,101
]


def dev_kw(d, dev):
    return {k: (None if v is None else v.to(dev)) for k, v in d.items()}


@pytest.mark.parametrize("dtype", [BF, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", CASES)
def test_stagewise_against_oracle(dev, case, dtype):
    from fla_hip import ops
    B, T, H, Hk, K, V, cu = case
    TOL = TOL_OF[dtype]
    d = inputs(B, T, H, K, V, Hk=Hk, seed=T, dtype=dtype)
    N = B if cu is None else len(cu) - 1
    gen = torch.Generator().manual_seed(5)
    h0 = torch.randn(N, H, K, V, generator=gen) * 0.01
    x = dev_kw(d, dev)

    # a1 cumsum
    G = ops.chunk_local_cumsum(x["g"], 64, cu_seqlens=cu)
    G_ref = gdn.chunk_local_cumsum(d["g"], 64, cu_seqlens=cu)
    assert_close(G, G_ref, 1e-5, "cumsum")

    # a2 kkt (fp32 out; inputs are bf16 k so the only difference is accumulation order)
    A0 = ops.chunk_scaled_dot_kkt(x["k"], G, x["beta"], cu_seqlens=cu, chunk_size=64)
    A0_ref = gdn.chunk_scaled_dot_kkt(d["k"], G_ref, d["beta"], 64, cu_seqlens=cu)
    assert_close(A0, A0_ref, 1e-4, "kkt")
    # structural zeros: on/above the diagonal and tail columns are exactly zero
    a0 = A0.cpu()
    for b, n, ci, s, e in gdn.chunk_spans(B, T, 64, cu):
        blk = a0[b, :, s:e]
        assert float(torch.triu(blk[:, :, : e - s], 0).abs().max()) == 0.0
        assert float(blk[:, :, e - s:].abs().max() if e - s < 64 else 0.0) == 0.0

    # a3 solve_tri on the bf16-rounded A0 (as the pipeline does); residual test of the reference
    A0b = A0.to(dtype)
    Ainv = ops.solve_tri(A0b, cu_seqlens=cu, layout="bnsd")
    Ainv_ref = gdn.solve_tri(A0b.cpu().float(), cu_seqlens=cu, output_dtype=torch.float32)
    assert_close(Ainv, Ainv_ref, TOL, "solve_tri")
    for b, n, ci, s, e in gdn.chunk_spans(B, T, 64, cu):
        L = e - s
        M = torch.eye(L) + A0b.cpu().float()[b, :, s:e, :L]
        res = torch.matmul(M, Ainv.cpu().float()[b, :, s:e, :L]) - torch.eye(L)
        assert float(res.abs().max()) < (2e-2 if dtype == BF else 1e-3)      # test_npu_solve_tri_ascend910b.py:39-41

    # a4 w, u
    w, u = ops.recompute_w_u_fwd(x["k"], x["v"], x["beta"], Ainv, 64, g=G, cu_seqlens=cu)
    w_ref, u_ref = gdn.recompute_w_u_fwd(d["k"], d["v"], d["beta"], Ainv.cpu(), 64, g=G_ref, cu_seqlens=cu,
                                         output_dtype=torch.float32)
    assert_close(w, w_ref, TOL, "w")
    assert_close(u, u_ref, TOL, "u")

    # a5 state scan
    h, v_new, final = ops.chunk_gated_delta_rule_fwd_h(x["k"], w, u, g=G, initial_state=h0.to(dev),
                                                       output_final_state=True, chunk_size=64, cu_seqlens=cu)
    h_ref, vn_ref, final_ref = gdn.chunk_gated_delta_rule_fwd_h(
        d["k"], w.cpu(), u.cpu(), G_ref, initial_state=h0, output_final_state=True, chunk=64, cu_seqlens=cu,
        output_dtype=torch.float32)
    assert_close(v_new, vn_ref, TOL, "v_new")
    assert_close(h, h_ref, TOL, "h")
    # The update multiplies k^T by v_new rounded to the matrices' 16-bit type, as the operator defines it
    # (chunk_gated_delta_rule_fwd_h/README.md:16-30): the restatement with the same roundings is the tight check, the
    # all-fp32 one bounds what they cost over the sequence.
    _, _, final_low = gdn.chunk_gated_delta_rule_fwd_h(
        d["k"], w.cpu(), u.cpu(), G_ref, initial_state=h0, output_final_state=True, chunk=64, cu_seqlens=cu,
        lowp=dtype, output_dtype=torch.float32)
    assert_close(final, final_low, TOL_STATE, "final_state")
    assert_close(final, final_ref, 4 * TOL_STATE, "final_state vs the fp32 update")
    assert final.dtype == torch.float32 and h.dtype == dtype

    # a6 output
    scale = K ** -0.5
    o = ops.chunk_fwd_o(x["q"], x["k"], v_new, h, scale, g=G, cu_seqlens=cu, chunk_size=64)
    o_ref = gdn.chunk_fwd_o(d["q"], d["k"], v_new.cpu(), h.cpu(), scale, g=G_ref, chunk=64, cu_seqlens=cu,
                            output_dtype=torch.float32)
    assert_close(o, o_ref, TOL, "o")

    # composition against the naive recurrence (the acceptance oracle)
    o_nv, final_nv = gdn.naive_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], scale,
                                                          initial_state=h0, output_final_state=True, cu_seqlens=cu)
    st = assert_close(o, o_nv, TOL, "o vs naive")
    assert st["rel_max"] < 2e-2, st
    assert_close(final, final_nv, TOL_STATE * 4, "final vs naive")   # unfused path rounds A, w, u to bf16


CASES_128 = [
    (2, 256, 2, 2, 128, 128, None),
    (1, 200, 4, 2, 128, 128, None),                     # GVA; last chunk holds 72 tokens (a full and a ragged row tile)
    (1, 130, 2, 2, 128, 256, None),                     # V = 256; last chunk holds 2 tokens
    (1, 389, 2, 1, 128, 128, [0, 1, 65, 193, 193, 389]),  # lengths 1, 64, 128, 0, 196
    (1, 330, 2, 1, 64, 64, None),                       # 64 key channels
    (1, 300, 4, 2, 64, 128, [0, 1, 130, 130, 300]),
]


@pytest.mark.parametrize("dtype", [BF, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", CASES_128)
def test_stagewise_chunk_128(dev, case, dtype):
    """The forward operators at chunk_size = 128 (chunk_gated_delta_rule_fwd_h/README.md:85-91, chunk_fwd_o/README.md:100):
    each stage against the oracle at that chunk size, and the composition against the per-token recurrence."""
    from fla_hip import ops
    C = 128
    B, T, H, Hk, K, V, cu = case
    TOL = TOL_OF[dtype]
    d = inputs(B, T, H, K, V, Hk=Hk, seed=T + 1, dtype=dtype)
    N = B if cu is None else len(cu) - 1
    h0 = torch.randn(N, H, K, V, generator=torch.Generator().manual_seed(5)) * 0.01
    x = dev_kw(d, dev)
    G = ops.chunk_local_cumsum(x["g"], C, cu_seqlens=cu)
    G_ref = gdn.chunk_local_cumsum(d["g"], C, cu_seqlens=cu)
    assert_close(G, G_ref, 1e-5, "cumsum")
    A0 = ops.chunk_scaled_dot_kkt(x["k"], G, x["beta"], cu_seqlens=cu, chunk_size=C)
    A0_ref = gdn.chunk_scaled_dot_kkt(d["k"], G_ref, d["beta"], C, cu_seqlens=cu)
    assert A0.shape == (B, H, T, C)
    assert_close(A0, A0_ref, 1e-4, "kkt")
    a0 = A0.cpu()
    for b, n, ci, s, e in gdn.chunk_spans(B, T, C, cu):
        blk = a0[b, :, s:e]
        assert float(torch.triu(blk[:, :, : e - s], 0).abs().max()) == 0.0
        assert float(blk[:, :, e - s:].abs().max() if e - s < C else 0.0) == 0.0
    Ainv = ops.solve_tri(A0, cu_seqlens=cu, layout="bnsd", output_dtype=dtype)
    Ainv_ref = gdn.solve_tri(A0.to(dtype).cpu().float(), cu_seqlens=cu, output_dtype=torch.float32)
    assert_close(Ainv, Ainv_ref, TOL, "solve_tri")
    w, u = ops.recompute_w_u_fwd(x["k"], x["v"], x["beta"], Ainv, C, g=G, cu_seqlens=cu)
    w_ref, u_ref = gdn.recompute_w_u_fwd(d["k"], d["v"], d["beta"], Ainv.cpu(), C, g=G_ref, cu_seqlens=cu,
                                         output_dtype=torch.float32)
    assert_close(w, w_ref, TOL, "w")
    assert_close(u, u_ref, TOL, "u")
    h, v_new, final = ops.chunk_gated_delta_rule_fwd_h(x["k"], w, u, g=G, initial_state=h0.to(dev),
                                                       output_final_state=True, chunk_size=C, cu_seqlens=cu)
    h_ref, vn_ref, final_ref = gdn.chunk_gated_delta_rule_fwd_h(
        d["k"], w.cpu(), u.cpu(), G_ref, initial_state=h0, output_final_state=True, chunk=C, cu_seqlens=cu,
        output_dtype=torch.float32)
    assert h.shape == h_ref.shape
    assert_close(v_new, vn_ref, TOL, "v_new")
    assert_close(h, h_ref, TOL, "h")
    # w of a 128-token chunk is larger than that of a 64-token one, and with it the effect of feeding w h with the
    # 16-bit state (the reference's rounding point, which the fp32 oracle does not have)
    assert_close(final, final_ref, 4 * TOL_STATE, "final_state")
    scale = K ** -0.5
    o = ops.chunk_fwd_o(x["q"], x["k"], v_new, h, scale, g=G, cu_seqlens=cu, chunk_size=C)
    o_ref = gdn.chunk_fwd_o(d["q"], d["k"], v_new.cpu(), h.cpu(), scale, g=G_ref, chunk=C, cu_seqlens=cu,
                            output_dtype=torch.float32)
    assert_close(o, o_ref, TOL, "o")
    o_nv, final_nv = gdn.naive_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], scale,
                                                          initial_state=h0, output_final_state=True, cu_seqlens=cu)
    assert_close(o, o_nv, TOL_BF16, "o vs naive")
    assert_close(final, final_nv, TOL_STATE * 8, "final vs naive")


def test_cumsum_variants(dev):
    from fla_hip import ops
    gen = torch.Generator().manual_seed(3)
    g = torch.randn(2, 3, 300, generator=gen)
    for chunk in (16, 64, 128):
        for rev in (False, True):
            out = ops.chunk_local_cumsum(g.to(dev), chunk, reverse=rev, scale=0.5)
            ref = gdn.chunk_local_cumsum(g, chunk, reverse=rev, scale=0.5)
            assert_close(out, ref, 1e-5, f"cumsum c={chunk} rev={rev}")
    g4 = torch.randn(1, 2, 130, 96, generator=gen)
    out = ops.chunk_local_cumsum(g4.to(dev), 64, cu_seqlens=[0, 70, 130])
    assert_close(out, gdn.chunk_local_cumsum(g4, 64, cu_seqlens=[0, 70, 130]), 1e-5, "cumsum 4d")
    out = ops.chunk_local_cumsum(g.bfloat16().to(dev), 64, output_dtype=torch.bfloat16)
    assert out.dtype == BF
    assert_close(out, gdn.chunk_local_cumsum(g.bfloat16(), 64), 2e-2, "cumsum bf16")


def test_solve_tri_layouts_and_inverse(dev):
    """Against numpy.linalg.inv and across the bsnd / bnsd / tnd / ntd layouts."""
    import numpy as np
    from fla_hip import ops
    gen = torch.Generator().manual_seed(9)
    B, H, T = 2, 3, 128
    A = torch.tril(torch.randn(B, H, T // 64, 64, 64, generator=gen) * 0.2, -1).reshape(B, H, T, 64).to(BF)
    ref = torch.from_numpy(np.linalg.inv(np.eye(64) + A.float().reshape(B, H, 2, 64, 64).numpy())).reshape(B, H, T, 64)
    out = ops.solve_tri(A.to(dev), layout="bnsd")
    assert_close(out, ref, TOL_BF16, "bnsd")
    out = ops.solve_tri(A.transpose(1, 2).contiguous().to(dev), layout="bsnd")
    assert_close(out.transpose(1, 2), ref, TOL_BF16, "bsnd")
    out = ops.solve_tri(A[0].contiguous().to(dev), layout="ntd")
    assert_close(out, ref[0], TOL_BF16, "ntd")
    out = ops.solve_tri(A[0].transpose(0, 1).contiguous().to(dev), layout="tnd")
    assert_close(out.transpose(0, 1), ref[0], TOL_BF16, "tnd")
    # fp32 input rounded on load == the caller's own cast followed by the 16-bit call, bit for bit
    Af = torch.tril(torch.randn(B, H, T // 64, 64, 64, generator=gen) * 0.2, -1).reshape(B, H, T, 64)
    for dt in (BF, F16):
        a = ops.solve_tri(Af.to(dev), layout="bnsd", output_dtype=dt)
        b2 = ops.solve_tri(Af.to(dt).to(dev), layout="bnsd")
        assert a.dtype == dt and torch.equal(a, b2)


@pytest.mark.parametrize("BT", [16, 32, 128])
@pytest.mark.parametrize("dtype", [BF, F16], ids=["bf16", "f16"])
def test_solve_tri_other_block_sizes(dev, BT, dtype):
    """The block size is the last dimension (16 / 32 / 64 / 128, solve_tri.cpp:47-62): numpy inverse per block,
    ragged tail blocks, a packed batch with an empty sequence, and the reference's residual bound."""
    import numpy as np
    from fla_hip import ops
    gen = torch.Generator().manual_seed(BT)
    H = 2
    for T, cu in ((3 * BT + 5, None), (4 * BT + 3, [0, BT - 1, BT - 1, 2 * BT + 1, 4 * BT + 3])):
        A = torch.tril(torch.randn(1, H, T, BT, generator=gen) * (2.0 / BT ** 0.5), -1)
        spans = list(gdn.chunk_spans(1, T, BT, cu))
        Ab = torch.zeros_like(A)
        for b, n, ci, s, e in spans:            # strictly lower inside each block
            Ab[b, :, s:e, : e - s] = torch.tril(A[b, :, s:e, : e - s], -1)
        Ab = Ab.to(dtype)
        out = ops.solve_tri(Ab.to(dev), cu_seqlens=cu, layout="bnsd").float().cpu()
        for b, n, ci, s, e in spans:
            L = e - s
            M = np.eye(L) + Ab[b, :, s:e, :L].float().numpy()
            ref = torch.from_numpy(np.linalg.inv(M)).float()
            assert_close(out[b, :, s:e, :L], ref, TOL_OF[dtype], f"block {s}:{e}")
            res = torch.from_numpy(M).float() @ out[b, :, s:e, :L] - torch.eye(L)
            assert float(res.abs().max()) < (2e-2 if dtype == BF else 2e-3) * max(1.0, float(ref.abs().max()))
            assert float(out[b, :, s:e, L:].abs().max() if L < BT else 0.0) == 0.0
    with pytest.raises(RuntimeError):
        ops.solve_tri(torch.zeros(1, 2, 48, 24, dtype=dtype, device=dev), layout="bnsd")


def test_state_v_first_and_no_final(dev):
    from fla_hip import ops
    d = inputs(1, 130, 2, 128, 128, seed=4)
    x = dev_kw(d, dev)
    G = ops.chunk_local_cumsum(x["g"], 64)
    gen = torch.Generator().manual_seed(1)
    w = (torch.randn(1, 2, 130, 128, generator=gen) * 0.1).to(BF)
    u = torch.randn(1, 2, 130, 128, generator=gen).to(BF)
    h0 = torch.randn(1, 2, 128, 128, generator=gen) * 0.01
    h_a, vn_a, f_a = ops.chunk_gated_delta_rule_fwd_h(x["k"], w.to(dev), u.to(dev), g=G, initial_state=h0.to(dev),
                                                      output_final_state=True)
    h_b, vn_b, f_b = ops.chunk_gated_delta_rule_fwd_h(
        x["k"], w.to(dev), u.to(dev), g=G, initial_state=h0.transpose(-1, -2).contiguous().to(dev),
        output_final_state=True, state_v_first=True)
    assert torch.equal(vn_a, vn_b)
    assert torch.equal(h_a, h_b.transpose(-1, -2))
    assert torch.equal(f_a, f_b.transpose(-1, -2))
    h_c, vn_c, f_c = ops.chunk_gated_delta_rule_fwd_h(x["k"], w.to(dev), u.to(dev), g=G, initial_state=h0.to(dev))
    assert f_c is None and torch.equal(vn_a, vn_c)


@pytest.mark.parametrize("dtype", [BF, F16], ids=["bf16", "f16"])
def test_fwd_h_sixteen_bit_state(dev, dtype):
    """initial_state / final_state in the dtype of the matrices (chunk_gated_delta_rule_fwd_h/README.md:85-91):
    same recurrence, the carry stays fp32 inside the kernel, the final state is rounded once on the way out."""
    from fla_hip import ops, pipeline
    B, T, H, K, V = 1, 200, 2, 128, 128
    d = inputs(B, T, H, K, V, seed=9, dtype=dtype)
    x = dev_kw(d, dev)
    gen = torch.Generator().manual_seed(4)
    h0 = (torch.randn(B, H, K, V, generator=gen) * 0.1).to(dtype)
    G_ref = gdn.chunk_local_cumsum(d["g"], 64)
    A = gdn.solve_tri(gdn.chunk_scaled_dot_kkt(d["k"], G_ref, d["beta"], 64), output_dtype=dtype)
    w, u = gdn.recompute_w_u_fwd(d["k"], d["v"], d["beta"], A, 64, g=G_ref, output_dtype=dtype)
    h, v_new, final = ops.chunk_gated_delta_rule_fwd_h(x["k"], w.to(dev), u.to(dev), g=G_ref.to(dev), initial_state=h0.to(dev),
                                                       output_final_state=True, chunk_size=64)
    h_ref, vn_ref, f_ref = gdn.chunk_gated_delta_rule_fwd_h(d["k"], w, u, G_ref, initial_state=h0.float(),
                                                            output_final_state=True, chunk=64, output_dtype=torch.float32)
    assert final.dtype == dtype and h.dtype == dtype
    assert_close(final, f_ref, TOL_OF[dtype], "final_state")
    assert_close(v_new, vn_ref, TOL_OF[dtype], "v_new")
    assert_close(h, h_ref, TOL_OF[dtype], "h")
    # pipeline entry: fp32 carry inside, caller's dtype outside
    o, fin = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"].transpose(1, 2).contiguous(),
                                             x["beta"].transpose(1, 2).contiguous(), None, h0.to(dev), True)
    o_ref, fin_ref = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"].transpose(1, 2), d["beta"].transpose(1, 2),
                                                None, h0.float(), True)
    assert fin.dtype == dtype
    assert_close(o, o_ref, TOL_OF[dtype], "o")
    assert_close(fin, fin_ref, TOL_OF[dtype], "final_state (pipeline)")


def test_rejects_bad_metadata(dev):
    from fla_hip import ops
    d = inputs(1, 128, 1, 128, 128)
    x = dev_kw(d, dev)
    G = ops.chunk_local_cumsum(x["g"], 64)
    with pytest.raises(RuntimeError, match="canonical"):
        ops.chunk_scaled_dot_kkt(x["k"], G, x["beta"], cu_seqlens=[0, 64, 128], chunk_indices=[0, 0, 0, 1])
    with pytest.raises(RuntimeError, match="chunk_size must be 64"):
        ops.chunk_scaled_dot_kkt(x["k"], G, x["beta"], chunk_size=32)
    with pytest.raises(RuntimeError, match="either g or gk"):
        ops.chunk_gated_delta_rule_fwd_h(x["k"], x["k"], x["v"])


@pytest.mark.parametrize("dtype", [BF, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("shape", [dict(B=2, T=256, Hk=2, Hv=2, K=128), dict(B=1, T=200, Hk=2, Hv=4, K=64),
                                   dict(B=1, T=261, Hk=1, Hv=2, K=128, cu=[0, 1, 16, 33, 33, 96, 160, 261])],
                         ids=["dense", "gva-ragged", "packed"])
def test_kkt_inverse_equals_the_two_operators(dev, shape, dtype):
    """chunk_scaled_dot_kkt_inverse is chunk_scaled_dot_kkt followed by solve_tri in one launch: same rounding
    points, same inversion code, so the results are compared for equality (and against the oracle's inverse)."""
    from fla_hip import ops
    B, T, Hk, Hv, K = (shape[x] for x in ("B", "T", "Hk", "Hv", "K"))
    cu = shape.get("cu")
    gen = torch.Generator().manual_seed(T + K)
    k = torch.nn.functional.normalize(torch.randn(B, Hk, T, K, generator=gen), dim=-1).to(dtype)
    g = gdn.chunk_local_cumsum(torch.nn.functional.logsigmoid(torch.randn(B, Hv, T, generator=gen)), 64, cu_seqlens=cu)
    beta = torch.sigmoid(torch.randn(B, Hv, T, generator=gen))
    kd, gd, bd = k.to(dev), g.to(dev), beta.to(dev)
    A0 = ops.chunk_scaled_dot_kkt(kd, gd, bd, cu_seqlens=cu, chunk_size=64)
    two = ops.solve_tri(A0, cu_seqlens=cu, layout="bnsd", output_dtype=dtype)
    one = ops.chunk_scaled_dot_kkt_inverse(kd, gd, bd, cu_seqlens=cu, chunk_size=64)
    assert one.dtype == dtype and one.shape == two.shape
    for b, n, ci, s, e in gdn.chunk_spans(B, T, 64, cu):
        assert torch.equal(one[b, :, s:e, : e - s], two[b, :, s:e, : e - s]), f"chunk {ci}"
    ref = gdn.solve_tri(gdn.chunk_scaled_dot_kkt(k, g, beta, 64, cu_seqlens=cu), cu_seqlens=cu)
    for b, n, ci, s, e in gdn.chunk_spans(B, T, 64, cu):
        assert_close(one[b, :, s:e, : e - s], ref[b, :, s:e, : e - s], TOL_BF16, f"inverse, chunk {ci}")
    with pytest.raises(RuntimeError, match="64-token chunks"):
        ops.chunk_scaled_dot_kkt_inverse(kd, gd, bd, chunk_size=128)
