"""End-to-end parity of the GDN chunk forward (fused library call and the six-operator route)
against the fp32 naive recurrence, with the pipeline-level layouts of
examples/flash_gated_delta_rule.py:1126-1228: q,k,v [B,H,T,D]; g,beta [B,T,H]; o [B,T,H,V];
final_state [N,H,K,V].  Tolerances: bf16 output 2e-2, fp32 state 1e-3 (fused route)."""
import pytest
import torch

from oracle import gdn
from util import assert_close, err_stats, TOL_BF16, TOL_STATE

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def run_both(dev, d, cu=None, scale=None, h0=None, fused=True):
    from fla_hip import pipeline
    to = lambda t: None if t is None else t.to(dev)
    o, final = pipeline.flash_gated_delta_rule(to(d["q"]), to(d["k"]), to(d["v"]), to(d["g"]), to(d["beta"]),
                                               scale, to(h0), True, cu_seqlens=cu, fused=fused)
    o_ref, f_ref = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], scale, h0, True,
                                              cu_seqlens=cu, naive=True)
    return o, final, o_ref, f_ref


CASES = [
    # B, T, H, Hk, K, V, cu
    (2, 256, 2, 2, 128, 128, None),
    (1, 200, 4, 2, 128, 128, None),                   # GVA, ragged tail
    (1, 1, 1, 1, 128, 128, None),
    (1, 63, 2, 2, 128, 128, None),
    (1, 65, 2, 2, 128, 128, None),
    (1, 130, 2, 2, 128, 256, None),                   # V = 256
    (1, 130, 2, 2, 64, 64, None),                     # K = V = 64
    (1, 192, 8, 8, 128, 128, None),
    (1, 261, 2, 1, 128, 128, [0, 1, 16, 33, 33, 96, 160, 261]),   # lengths 1,15,17,0,63,64,101
]


@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("case", CASES)
def test_against_naive_recurrence(dev, case, fused, dtype):
    B, T, H, Hk, K, V, cu = case
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=dtype, seed=T + H, Hk=Hk)
    N = B if cu is None else len(cu) - 1
    h0 = torch.randn(N, H, K, V, generator=torch.Generator().manual_seed(2)) * 0.01
    o, final, o_ref, f_ref = run_both(dev, d, cu=cu, h0=h0, fused=fused)
    assert o.shape == (B, T, H, V) and o.dtype == dtype and final.shape == (N, H, K, V) and final.dtype == torch.float32
    st = assert_close(o, o_ref, TOL_BF16 if dtype == BF else TOL_BF16 / 4, "o")
    assert st["rel_max"] < 2e-2, st
    assert_close(final, f_ref, TOL_STATE if fused else 4 * TOL_STATE, "final_state")


@pytest.mark.parametrize("fused", [True, False], ids=["fused", "operators"])
def test_cfg1_shape_and_seed_in_bf16(dev, fused):
    """The self-check configuration of the benchmark set on the GPU: B=1 T=256 H=2 K=V=64, chunk 64, seed 0, zero
    initial state (the CPU oracle runs it in fp32, tests/test_oracle.py); here the same tensors rounded to bf16 go
    through both routes of the pipeline entry and are held to the acceptance tolerances against the fp32 per-token
    recurrence on those bf16 inputs."""
    d = gdn.make_gdn_inputs(1, 256, 2, 64, 64, dtype=BF, seed=0)
    o, final, o_ref, f_ref = run_both(dev, d, fused=fused)
    assert o.shape == (1, 256, 2, 64) and o.dtype == BF and final.shape == (1, 2, 64, 64) and final.dtype == torch.float32
    st = assert_close(o, o_ref, TOL_BF16, "o")
    assert st["rel_max"] < 2e-2, st
    assert_close(final, f_ref, TOL_STATE if fused else 4 * TOL_STATE, "final_state")


@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", CASES)
def test_forward_writes_the_operands_of_the_backward(dev, case, dtype):
    """save_for_backward: h (state at every chunk start), v_new and w as the stage-by-stage fp32 restatement computes
    them (recompute_w_u_fwd/README.md:12-32, chunk_gated_delta_rule_fwd_h/README.md:16-30), while o, the final state
    and the cumulated gate stay bit-identical to the call without them."""
    from fla_hip.ops import _hip_ctypes as raw
    B, T, H, Hk, K, V, cu = case
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=dtype, seed=T + 2 * H, Hk=Hk)
    N = B if cu is None else len(cu) - 1
    h0 = torch.randn(N, H, K, V, generator=torch.Generator().manual_seed(4)) * 0.01
    x = {n: d[n].to(dev) for n in ("q", "k", "v", "g", "beta")}
    scale = K ** -0.5
    plain = raw.gdn_chunk_fwd(x["q"], x["k"], x["v"], x["g"], x["beta"], scale, h0.to(dev), True, cu, 64)
    gc, o, final, h, v_new, w = raw.gdn_chunk_fwd(x["q"], x["k"], x["v"], x["g"], x["beta"], scale, h0.to(dev), True,
                                                  cu, 64, save_for_backward=True)
    for name, a, b in zip(("g_cumsum", "o", "final_state"), (gc, o, final), plain):
        assert torch.equal(a, b), name
    _, _, mid = gdn.chunk_gated_delta_rule_fwd(d["q"], d["k"], d["v"], d["g"].transpose(1, 2), d["beta"].transpose(1, 2),
                                               scale, initial_state=h0, output_final_state=True, cu_seqlens=cu,
                                               return_intermediates=True)
    NT = gdn.total_chunks(B, T, 64, cu)
    assert h.shape == (B, H, NT, K, V) and v_new.shape == (B, H, T, V) and w.shape == (B, H, T, K)
    assert h.dtype == dtype and v_new.dtype == dtype and w.dtype == dtype
    tol = TOL_BF16 if dtype == BF else TOL_BF16 / 4
    assert_close(w, mid["w"], tol, "w")
    assert_close(v_new, mid["v_new"], tol, "v_new")
    assert_close(h, mid["h"], tol, "h")


# Batches large enough that the host picks the kernels with 128-column value slabs: the fused forward once
# sequences x heads x (V / 128) reaches the number of compute units (256), the stand-alone state scan at twice that.
WIDE_CASES = [
    (8, 200, 32, 32, 128, 128, None),                    # fused: 256 chains
    (4, 130, 32, 32, 128, 256, None),                    # fused: 128 chains x 2 slabs, V = 256
    (16, 130, 32, 16, 128, 128, None),                   # fused and the six-operator scan (512 chains), grouped heads
    (1, 8 * 70, 32, 32, 128, 128, [70 * i for i in range(9)]),   # packed: 8 sequences x 32 heads, initial states
    (1, 600, 32, 32, 64, 128, [0, 1, 65, 130, 130, 258, 300, 450, 600]),   # K = 64, ragged packed sequences
]


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("case", WIDE_CASES)
def test_large_batches_on_the_wide_slab_kernels(dev, case, fused):
    B, T, H, Hk, K, V, cu = case
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=BF, seed=T + H, Hk=Hk)
    N = B if cu is None else len(cu) - 1
    h0 = torch.randn(N, H, K, V, generator=torch.Generator().manual_seed(2)) * 0.01
    o, final, o_ref, f_ref = run_both(dev, d, cu=cu, h0=h0, fused=fused)
    st = assert_close(o, o_ref, TOL_BF16, "o")
    assert st["rel_max"] < 2e-2, st
    assert_close(final, f_ref, TOL_STATE if fused else 4 * TOL_STATE, "final_state")


def test_six_operator_route_with_k64_v128(dev):
    d = gdn.make_gdn_inputs(1, 130, 2, 64, 128, dtype=BF, seed=7, Hk=2)
    h0 = torch.randn(1, 2, 64, 128, generator=torch.Generator().manual_seed(2)) * 0.01
    o, final, o_ref, f_ref = run_both(dev, d, h0=h0, fused=False)
    assert_close(o, o_ref, TOL_BF16, "o")
    assert_close(final, f_ref, 4 * TOL_STATE, "final_state")


@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", CASES)
def test_in_kernel_l2norm_equals_separate_pass(dev, case, dtype):
    """use_qk_l2norm_in_kernel on the fused route: same result as normalising q and k with l2norm_fwd first (the
    rows are rounded to bf16 at the same point, so only the order of the fp32 sum of squares may differ), and
    the recurrence on F.normalize'd inputs within the bf16 tolerance."""
    from fla_hip import ops, pipeline
    B, T, H, Hk, K, V, cu = case
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=dtype, seed=T + 3 * H, Hk=Hk)
    gen = torch.Generator().manual_seed(T)
    q = (d["q"].float() * (0.3 + 3 * torch.rand(B, Hk, T, 1, generator=gen))).to(dtype).to(dev)
    k = (d["k"].float() * (0.3 + 3 * torch.rand(B, Hk, T, 1, generator=gen))).to(dtype).to(dev)
    v, g, beta = (d[n].to(dev) for n in ("v", "g", "beta"))
    N = B if cu is None else len(cu) - 1
    h0 = (torch.randn(N, H, K, V, generator=gen) * 0.01).to(dev)
    o, final = pipeline.flash_gated_delta_rule(q, k, v, g, beta, None, h0, True, use_qk_l2norm_in_kernel=True,
                                               cu_seqlens=cu)
    qn, kn = ops.l2norm_fwd(q)[0], ops.l2norm_fwd(k)[0]
    o2, final2 = pipeline.flash_gated_delta_rule(qn, kn, v, g, beta, None, h0, True, cu_seqlens=cu)
    assert_close(o, o2.float(), 1e-2 if dtype == BF else 2e-3, "o vs two-pass")     # a 1-ulp bf16 flip in a row is possible, no more
    assert_close(final, final2, TOL_STATE, "state vs two-pass")
    nrm = lambda t: torch.nn.functional.normalize(t.float().cpu(), dim=-1)
    o_ref, f_ref = gdn.flash_gated_delta_rule(nrm(q), nrm(k), d["v"], d["g"], d["beta"], None, h0.cpu(), True,
                                              cu_seqlens=cu, naive=True)
    assert_close(o, o_ref, TOL_BF16, "o")
    assert_close(final, f_ref, 2 * TOL_STATE, "final_state")


@pytest.mark.parametrize("token_major", [False, True], ids=["head_major", "token_major"])
@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", CASES)
def test_forward_writes_normalised_q_k_and_rstd(dev, case, dtype, token_major):
    """use_qk_l2norm_in_kernel with save_for_backward: the kernel also writes the normalised q, k and their rstd, what
    l2norm_fwd hands its backward (examples/flash_gated_delta_rule.py:1086-1089).  Checked against the oracle's
    l2norm_fwd (fla/ops/triton/triton_core/l2norm.py:131-178): rstd to fp32 rounding of the sum, the rows to one
    rounding of the element type; they come in the memory order of q and k, and o, the state and the gate are
    bit-identical to the call that does not ask for them."""
    from fla_hip.ops import _hip_ctypes as raw
    B, T, H, Hk, K, V, cu = case
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=dtype, seed=T + 5 * H, Hk=Hk)
    gen = torch.Generator().manual_seed(T + 1)
    q = (d["q"].float() * (0.3 + 3 * torch.rand(B, Hk, T, 1, generator=gen))).to(dtype)
    k = (d["k"].float() * (0.3 + 3 * torch.rand(B, Hk, T, 1, generator=gen))).to(dtype)
    place = (lambda t: t.transpose(1, 2).contiguous().to(dev).transpose(1, 2)) if token_major else (lambda t: t.to(dev))
    qd, kd = place(q), place(k)
    v, g, beta = (d[n].to(dev) for n in ("v", "g", "beta"))
    N = B if cu is None else len(cu) - 1
    h0 = (torch.randn(N, H, K, V, generator=gen) * 0.01).to(dev)
    scale = K ** -0.5
    plain = raw.gdn_chunk_fwd(qd, kd, v, g, beta, scale, h0, True, cu, 64, True)
    res = raw.gdn_chunk_fwd(qd, kd, v, g, beta, scale, h0, True, cu, 64, True, save_for_backward=True)
    assert len(res) == 10
    for name, a, b in zip(("g_cumsum", "o", "final_state"), res[:3], plain):
        assert torch.equal(a, b), name
    qn, kn, q_rstd, k_rstd = res[6:]
    for name, x, y, rstd in (("q", q, qn, q_rstd), ("k", k, kn, k_rstd)):
        y_ref, r_ref = gdn.l2norm_fwd(x)
        assert y.shape == x.shape and y.dtype == dtype and y.stride() == (qd if name == "q" else kd).stride(), name
        assert rstd.shape == x.shape[:-1] and rstd.dtype == torch.float32 and rstd.is_contiguous(), name
        assert_close(rstd, r_ref, 1e-5, name + "_rstd")
        assert_close(y, y_ref.float(), 4e-3 if dtype == BF else 5e-4, name + "_normalised")
    # the backward's operands are those of the normalised problem
    w_ref = raw.gdn_chunk_fwd(qn, kn, v, g, beta, scale, h0, True, cu, 64, save_for_backward=True)[5]
    assert_close(res[5], w_ref.float(), 1e-2 if dtype == BF else 2e-3, "w")


@pytest.mark.parametrize("chunk_size", [16, 128, 256])
def test_other_chunk_sizes_give_the_same_result(dev, chunk_size):
    """chunk_size only tiles the recurrence: the entry accepts any power of two and returns the result of the
    reference's chunked algorithm at that size (oracle run at that chunk size) within the usual tolerance."""
    from fla_hip import pipeline
    d = gdn.make_gdn_inputs(1, 300, 2, 128, 128, dtype=BF, seed=5, init_std=0.01)
    x = {k: v.to(dev) for k, v in d.items()}
    o, final = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["initial_state"], True,
                                               chunk_size=chunk_size)
    o_ref, f_ref = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], None, d["initial_state"], True,
                                              chunk_size=chunk_size, naive=False)
    assert_close(o, o_ref, TOL_BF16, "o")
    assert_close(final, f_ref, TOL_STATE, "final_state")
    with pytest.raises(ValueError, match="power of 2"):
        pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], chunk_size=96)
    if chunk_size == 128:      # the six-operator route runs 128-token chunks natively
        o2, f2 = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["initial_state"], True,
                                                 chunk_size=128, fused=False)
        assert_close(o2, o_ref, TOL_BF16, "o (operators, 128)")
        assert_close(f2, f_ref, 8 * TOL_STATE, "final_state (operators, 128)")


def test_no_initial_state_and_default_scale(dev):
    from fla_hip import pipeline
    d = gdn.make_gdn_inputs(2, 128, 2, 128, 128, dtype=BF, seed=3)
    to = lambda t: t.to(dev)
    o, final = pipeline.flash_gated_delta_rule(to(d["q"]), to(d["k"]), to(d["v"]), to(d["g"]), to(d["beta"]))
    assert final is None
    o_ref, _ = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"])
    assert_close(o, o_ref, TOL_BF16, "o")


def test_special_cases_fix_the_formula(dev):
    """beta = 0: the state only decays, o_t = scale * q_t . (prod decay) S0.  g = 0, beta = 1: plain delta rule."""
    from fla_hip import pipeline
    d = gdn.make_gdn_inputs(1, 128, 2, 128, 128, dtype=BF, seed=5)
    h0 = torch.randn(1, 2, 128, 128, generator=torch.Generator().manual_seed(1))
    to = lambda t: t.to(dev)
    beta0 = torch.zeros_like(d["beta"])
    o, final = pipeline.flash_gated_delta_rule(to(d["q"]), to(d["k"]), to(d["v"]), to(d["g"]), to(beta0), 0.5, to(h0), True)
    G = torch.cumsum(d["g"], 1)                                   # [B,T,H]
    expect = 0.5 * torch.einsum("bhtk,bhkv->bthv", d["q"].float(), h0) * torch.exp(G)[..., None]
    assert_close(o, expect, TOL_BF16, "o beta=0")
    assert_close(final, h0 * torch.exp(G[:, -1])[..., None, None], TOL_STATE, "state beta=0")
    g0, beta1 = torch.zeros_like(d["g"]), torch.ones_like(d["beta"])
    o, final = pipeline.flash_gated_delta_rule(to(d["q"]), to(d["k"]), to(d["v"]), to(g0), to(beta1), None, None, True)
    # delta rule with beta = 1 stores v_t exactly under key k_t: S_t^T k_t = v_t  =>  o_t(q = k_t) = scale v_t
    o2, _ = pipeline.flash_gated_delta_rule(to(d["k"]), to(d["k"]), to(d["v"]), to(g0), to(beta1), 1.0, None, False)
    assert_close(o2.transpose(1, 2), d["v"].float(), 3e-2, "delta-rule write/read identity")


def test_wrapper_errors(dev):
    from fla_hip import pipeline
    d = gdn.make_gdn_inputs(1, 64, 2, 128, 128, dtype=BF)
    to = lambda t: t.to(dev)
    with pytest.raises(ValueError, match="does not support float32"):
        pipeline.flash_gated_delta_rule(to(d["q"]).float(), to(d["k"]).float(), to(d["v"]).float(), to(d["g"]), to(d["beta"]))
    with pytest.raises(ValueError, match="g and beta must be rank-3"):
        pipeline.flash_gated_delta_rule(to(d["q"]), to(d["k"]), to(d["v"]), to(d["g"])[0], to(d["beta"])[0])
    with pytest.raises(ValueError, match="batch size is expected to be 1"):
        q2 = torch.cat([to(d["q"])] * 2)
        pipeline.flash_gated_delta_rule(q2, q2, q2, torch.cat([to(d["g"])] * 2), torch.cat([to(d["beta"])] * 2),
                                        cu_seqlens=[0, 32, 64])


def test_benchmark_shape(dev):
    """B=4, T=8192, H=32, K=V=128: oracle on two batch rows; hand-off, route agreement and determinism on all."""
    from fla_hip import pipeline
    B, T, H, K, V = 4, 8192, 32, 128, 128
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=BF, seed=0, init_std=0.01)
    x = {k: v.to(dev) for k, v in d.items()}
    o, final = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["initial_state"], True)
    # (1) fp32 chunked oracle == naive recurrence to 1e-5 is a CPU test; here the chunked fp32 oracle on rows 0, 3
    for b in (0, 3):
        sl = slice(b, b + 1)
        o_ref, f_ref = gdn.flash_gated_delta_rule(d["q"][sl], d["k"][sl], d["v"][sl], d["g"][sl], d["beta"][sl], None,
                                                  d["initial_state"][sl], True, naive=False)
        st = assert_close(o[sl], o_ref, TOL_BF16, f"o row {b}")
        assert st["rel_max"] < 2e-2, st
        assert_close(final[sl], f_ref, TOL_STATE, f"final_state row {b}")
    # (2) state hand-off at a chunk boundary reproduces the single call bit for bit
    half = T // 2
    o1, f1 = pipeline.flash_gated_delta_rule(x["q"][:, :, :half], x["k"][:, :, :half], x["v"][:, :, :half],
                                             x["g"][:, :half], x["beta"][:, :half], None, x["initial_state"], True)
    o2, f2 = pipeline.flash_gated_delta_rule(x["q"][:, :, half:], x["k"][:, :, half:], x["v"][:, :, half:],
                                             x["g"][:, half:], x["beta"][:, half:], None, f1, True)
    assert torch.equal(torch.cat([o1, o2], 1), o)
    assert torch.equal(f2, final)
    # (3) the six-operator route agrees within tolerance; (4) reruns are bit-identical
    o_ops, f_ops = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["initial_state"],
                                                   True, fused=False)
    assert_close(o_ops, o.float(), TOL_BF16, "ops vs fused o")
    assert_close(f_ops, final, 4 * TOL_STATE, "ops vs fused state")
    o_again, f_again = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], None,
                                                       x["initial_state"], True)
    assert torch.equal(o_again, o) and torch.equal(f_again, final)


def _rel_stats(x, truth):
    x, truth = x.double().cpu(), truth.double()
    err = (x - truth).abs()
    denom = truth.abs().clamp_min(1e-3 * float(truth.abs().max()))
    re = err / denom
    return dict(max_re=float(re.max()), avg_re=float(re.mean()),
                rmse=float(err.pow(2).mean().sqrt()))


@pytest.mark.parametrize("dtype", [BF, torch.float16], ids=["bf16", "f16"])
def test_dual_benchmark_against_fp64_truth(dev, dtype):
    """The reference's acceptance standard (tests/atk/*/atk_*.json "standard" blocks): the device result and a CPU
    control that rounds where the reference kernels round are both held against an fp64 truth; the device passes
    when its max / mean relative error and its RMSE stay within 10x / 3x / 3x of the control's."""
    from fla_hip import pipeline
    B, T, H, K, V = 2, 512, 4, 128, 128
    d = gdn.make_gdn_inputs(B, T, H, K, V, dtype=dtype, seed=101, init_std=0.05)
    dd = torch.float64
    truth_o, truth_f = gdn.flash_gated_delta_rule(d["q"].to(dd), d["k"].to(dd), d["v"].to(dd), d["g"].to(dd), d["beta"].to(dd),
                                                  None, d["initial_state"].to(dd), True, naive=True, compute_dtype=dd)
    ctrl_o, ctrl_f = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], None, d["initial_state"], True,
                                                naive=False, lowp=dtype)
    ctrl_o = ctrl_o.to(dtype)                          # the control's output leaves in the element type too
    x = {k: v.to(dev) for k, v in d.items()}
    for fused in (True, False):
        o, f = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["initial_state"], True,
                                               fused=fused)
        for name, dut, ctrl, truth in (("o", o, ctrl_o, truth_o), ("final_state", f, ctrl_f, truth_f)):
            a, c = _rel_stats(dut, truth), _rel_stats(ctrl, truth)
            assert a["max_re"] <= 10 * c["max_re"] + 1e-6, (fused, name, a, c)
            assert a["avg_re"] <= 3 * c["avg_re"] + 1e-7, (fused, name, a, c)
            assert a["rmse"] <= 3 * c["rmse"] + 1e-9, (fused, name, a, c)


def test_long_context_packed(dev):
    """T = 65536 in one packed row (the reference example's default length, examples/flash_gated_delta_rule.py:1863):
    a 40,000-token sequence between two shorter ones.  Chunked fp32 oracle on the whole row; the long sequence alone
    (dense call) must reproduce its slice of the packed result bit for bit."""
    from fla_hip import pipeline
    T, H, K, V = 65536, 2, 128, 128
    cu = [0, 12345, 52345, 65536]
    d = gdn.make_gdn_inputs(1, T, H, K, V, dtype=BF, seed=7)
    h0 = torch.randn(3, H, K, V, generator=torch.Generator().manual_seed(8)) * 0.01
    x = {k: (None if v is None else v.to(dev)) for k, v in d.items()}
    o, f = pipeline.flash_gated_delta_rule(x["q"], x["k"], x["v"], x["g"], x["beta"], None, h0.to(dev), True, cu_seqlens=cu)
    o_ref, f_ref = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], None, h0, True, cu_seqlens=cu,
                                              naive=False)
    st = assert_close(o, o_ref, TOL_BF16, "o")
    assert st["rel_max"] < 2e-2, st
    assert_close(f, f_ref, TOL_STATE, "final_state")
    s, e = cu[1], cu[2]
    o1, f1 = pipeline.flash_gated_delta_rule(x["q"][:, :, s:e], x["k"][:, :, s:e], x["v"][:, :, s:e], x["g"][:, s:e],
                                             x["beta"][:, s:e], None, h0[1:2].to(dev), True)
    assert torch.equal(o1, o[:, s:e]) and torch.equal(f1, f[1:2])
