"""Parity of chunk_kda_fwd (through the C ABI) against the CPU oracle.

Acceptance: attention output within 2e-2 and final state within 1e-3 (relative to the state's
scale) of the fp32 per-token recurrence; every intermediate of the 12-tuple within 2e-2 of the
chunked fp32 restatement.  Cases follow the reference sweep: the four layouts, GVA, ragged tails,
packed variable-length batches with an empty sequence, in-kernel gate activations, initial state,
V-first state blocks, and the optional-output policy."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn, kda
from util import assert_close, TOL_BF16, TOL_STATE

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def make_inputs(B, T, Hk, Hv, K, V, seed, *, raw_gate=False, gate_scale=0.3, g_dtype=torch.float32, beta_dtype=torch.float32,
                dtype=BF):
    gen = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, Hk, T, K, generator=gen), dim=-1).to(dtype)
    k = F.normalize(torch.randn(B, Hk, T, K, generator=gen), dim=-1).to(dtype)
    v = torch.randn(B, Hv, T, V, generator=gen).to(dtype)
    if raw_gate:
        g = torch.randn(B, Hv, T, K, generator=gen).to(g_dtype)
    else:
        g = (F.logsigmoid(torch.randn(B, Hv, T, K, generator=gen)) * gate_scale).to(g_dtype)
    beta = torch.sigmoid(torch.randn(B, Hv, T, generator=gen)).to(beta_dtype)
    return q, k, v, g, beta


def to_layout(x, layout, scalar=False):
    """head-major [B,H,T,(D)] -> the caller's layout"""
    if layout == "BNSD":
        return x.contiguous()
    if layout == "BSND":
        return x.transpose(1, 2).contiguous()
    if layout == "NTD":
        return x[0].contiguous()
    return x[0].transpose(0, 1).contiguous()   # TND


def from_layout(x, layout):
    if layout == "BNSD":
        return x
    if layout == "BSND":
        return x.transpose(1, 2)
    if layout == "NTD":
        return x[None]
    return x.transpose(0, 1)[None]


CASES = [
    # B, T, Hk, Hv, K, V, layout, cu, gate kwargs, h0, v_first
    dict(B=2, T=256, Hk=2, Hv=2, K=128, V=128, layout="BSND"),
    dict(B=1, T=200, Hk=2, Hv=4, K=128, V=128, layout="BNSD", h0=True),                       # GVA, ragged tail
    dict(B=1, T=261, Hk=2, Hv=2, K=128, V=128, layout="TND", cu=[0, 1, 16, 33, 33, 96, 160, 261], h0=True),
    dict(B=1, T=130, Hk=1, Hv=2, K=64, V=64, layout="NTD", cu=[0, 65, 130]),
    dict(B=1, T=192, Hk=2, Hv=2, K=128, V=256, layout="BSND", v_first=True, h0=True),
    dict(B=2, T=100, Hk=2, Hv=2, K=64, V=128, layout="BNSD"),
    dict(B=1, T=160, Hk=2, Hv=2, K=128, V=128, layout="BSND", gate=dict(use_gate_in_kernel=True, bias=True)),
    dict(B=1, T=160, Hk=2, Hv=2, K=128, V=128, layout="BSND",
         gate=dict(use_gate_in_kernel=True, safe_gate=True, lower_bound=-5.0, bias=True), g_dtype=BF, beta_dtype=BF),
    dict(B=1, T=1, Hk=1, Hv=1, K=128, V=128, layout="BSND"),
    dict(B=1, T=128, Hk=1, Hv=1, K=128, V=128, layout="BSND", gate_scale=3.0),             # strong decay
    # float16 q/k/v and outputs (gates mild enough for the anchored factors to stay inside float16's range)
    dict(B=2, T=200, Hk=2, Hv=4, K=128, V=128, layout="BSND", h0=True, dtype=torch.float16),
    dict(B=1, T=130, Hk=1, Hv=2, K=64, V=64, layout="NTD", cu=[0, 65, 130], dtype=torch.float16),
]


# 128-token chunks: full and ragged chunks, a chunk with an empty second half, packed sequences, both head sizes,
# both state layouts, the in-kernel gate, fp16
CASES += [
    dict(B=2, T=256, Hk=2, Hv=2, K=128, V=128, layout="BSND", chunk=128, h0=True),
    dict(B=1, T=330, Hk=2, Hv=4, K=128, V=128, layout="BNSD", chunk=128, h0=True),
    dict(B=1, T=192, Hk=1, Hv=2, K=128, V=128, layout="BSND", chunk=128),                    # last chunk: first half only
    dict(B=1, T=421, Hk=2, Hv=2, K=128, V=128, layout="TND", chunk=128, cu=[0, 1, 66, 66, 194, 300, 421], h0=True),
    dict(B=1, T=200, Hk=1, Hv=2, K=64, V=64, layout="NTD", chunk=128, cu=[0, 129, 200]),
    dict(B=1, T=256, Hk=2, Hv=2, K=128, V=256, layout="BSND", chunk=128, v_first=True, h0=True),
    dict(B=2, T=150, Hk=2, Hv=2, K=64, V=128, layout="BNSD", chunk=128),
    dict(B=1, T=256, Hk=2, Hv=2, K=128, V=128, layout="BSND", chunk=128,
         gate=dict(use_gate_in_kernel=True, bias=True, safe_gate=True, lower_bound=-5.0)),
    dict(B=1, T=256, Hk=1, Hv=1, K=128, V=128, layout="BSND", chunk=128, gate_scale=3.0),     # strong decay
    dict(B=1, T=300, Hk=2, Hv=4, K=128, V=128, layout="BSND", chunk=128, h0=True, dtype=torch.float16),
]


# head sizes between the built ones (the reference admits multiples of 16 up to 256, _aclnn_ctypes.py:1141): served by
# zero channels appended in the wrapper
CASES += [
    dict(B=1, T=150, Hk=2, Hv=2, K=96, V=80, layout="BSND", h0=True),
    dict(B=1, T=130, Hk=1, Hv=2, K=16, V=16, layout="TND", cu=[0, 65, 130], h0=True),
    dict(B=1, T=100, Hk=2, Hv=2, K=48, V=160, layout="BNSD", v_first=True, h0=True),
    dict(B=1, T=192, Hk=1, Hv=2, K=112, V=256, layout="BSND", chunk=128,
         gate=dict(use_gate_in_kernel=True, bias=True, safe_gate=True, lower_bound=-5.0)),
    dict(B=1, T=70, Hk=1, Hv=1, K=128, V=64, layout="NTD"),
]


# more than 128 channels (up to 256, _aclnn_ctypes.py:1141): kernels for K = V = 256, sizes between on zero channels
CASES += [
    dict(B=2, T=200, Hk=2, Hv=4, K=256, V=256, layout="BSND", h0=True),                       # GVA, ragged tail
    dict(B=1, T=261, Hk=2, Hv=2, K=256, V=256, layout="TND", cu=[0, 1, 16, 33, 33, 96, 160, 261], h0=True),
    dict(B=1, T=192, Hk=1, Hv=2, K=256, V=256, layout="BNSD", v_first=True, h0=True,
         gate=dict(use_gate_in_kernel=True, bias=True, safe_gate=True, lower_bound=-5.0), g_dtype=BF, beta_dtype=BF),
    dict(B=1, T=128, Hk=1, Hv=1, K=256, V=256, layout="BSND", gate_scale=3.0),              # strong decay
    dict(B=1, T=330, Hk=2, Hv=4, K=256, V=256, layout="BNSD", chunk=128, h0=True),
    dict(B=1, T=421, Hk=1, Hv=2, K=256, V=256, layout="TND", chunk=128, cu=[0, 1, 66, 66, 194, 300, 421], h0=True,
         v_first=True),
    dict(B=1, T=192, Hk=1, Hv=1, K=256, V=256, layout="NTD", chunk=128, gate=dict(use_gate_in_kernel=True, bias=True)),
    dict(B=1, T=150, Hk=1, Hv=2, K=192, V=96, layout="BSND", h0=True),                       # padded to 256 x 256
    dict(B=1, T=140, Hk=1, Hv=1, K=144, V=256, layout="BSND", chunk=128, dtype=torch.float16),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(f"{k}{v}" for k, v in c.items() if k in ("T", "K", "V", "layout", "chunk")))
def test_chunk_kda_fwd(dev, case):
    from fla_hip import ops
    B, T, Hk, Hv, K, V, layout = (case[x] for x in ("B", "T", "Hk", "Hv", "K", "V", "layout"))
    cu = case.get("cu")
    C = case.get("chunk", 64)
    gate = dict(case.get("gate", {}))
    use_gate = gate.get("use_gate_in_kernel", False)
    v_first = case.get("v_first", False)
    q, k, v, g, beta = make_inputs(B, T, Hk, Hv, K, V, seed=T + K + V, raw_gate=use_gate,
                                   gate_scale=case.get("gate_scale", 0.3), g_dtype=case.get("g_dtype", torch.float32),
                                   beta_dtype=case.get("beta_dtype", torch.float32), dtype=case.get("dtype", BF))
    assert q.dtype == case.get("dtype", BF)
    gen = torch.Generator().manual_seed(11)
    A_log = torch.randn(Hv, generator=gen) * 0.3 - 1.5 if use_gate else None
    dt_bias = torch.randn(Hv * K, generator=gen) * 0.3 if gate.pop("bias", False) else None
    N = B if cu is None else len(cu) - 1
    h0 = torch.randn(N, Hv, K, V, generator=gen) * 0.1 if case.get("h0") else None
    scale = K ** -0.5

    # oracle
    okw = dict(A_log=A_log, dt_bias=dt_bias, use_gate_in_kernel=use_gate, safe_gate=gate.get("safe_gate", False),
               lower_bound=gate.get("lower_bound", -5.0))
    nat = kda.kda_gate(g, **okw)
    gk_ref = kda.kda_gate_cumsum(g, C, cu_seqlens=cu, **okw)
    o_naive, f_naive = kda.naive_recurrent_kda(q, k, v, nat, beta, scale, initial_state=h0, output_final_state=True,
                                               cu_seqlens=cu)
    ref = kda.chunk_kda_fwd(q, k, v, gk_ref, beta, scale, C, initial_state=h0, output_final_state=True, cu_seqlens=cu)

    h0_dev = None
    if h0 is not None:
        h0_dev = (h0.transpose(-1, -2).contiguous() if v_first else h0).to(dev)
    out = ops.chunk_kda_fwd(
        to_layout(q, layout).to(dev), to_layout(k, layout).to(dev), to_layout(v, layout).to(dev),
        to_layout(g, layout).to(dev), to_layout(beta, layout).to(dev), scale, C, layout=layout, initial_state=h0_dev,
        output_final_state=True, cu_seqlens=cu, A_log=None if A_log is None else A_log.to(dev),
        dt_bias=None if dt_bias is None else dt_bias.to(dev), disable_recompute=True, state_v_first=v_first, **gate)
    assert len(out) == 12
    o, final, gk, Aqk, Akk, w, u, qg, kg, v_new, h, init_back = out
    assert init_back is h0_dev
    assert all(t.dtype == q.dtype for t in (o, Aqk, Akk, w, u, qg, kg, v_new, h))
    head = (lambda x: x[None]) if layout in ("TND", "NTD") else (lambda x: x)

    st = assert_close(from_layout(o, layout), o_naive, TOL_BF16, "o vs recurrence")
    assert st["rel_max"] < 2e-2, st
    fin = final.transpose(-1, -2) if v_first else final
    assert final.dtype == torch.float32
    # a 128-token chunk works against one 16-bit copy of the state for twice as many tokens
    assert_close(fin, f_naive, (1 if C == 64 else 2) * TOL_STATE, "final state vs recurrence")
    assert_close(fin, ref["final_state"], TOL_BF16, "final state vs chunked")

    assert gk.dtype == torch.float32
    assert_close(head(gk), gk_ref, 2e-5 if g.dtype == torch.float32 else 1e-4, "gk")
    assert_close(head(Aqk), ref["Aqk"], TOL_BF16, "Aqk")
    assert_close(head(Akk), ref["Akk"], TOL_BF16, "Akk")
    assert_close(head(w), ref["w"], TOL_BF16, "w")
    assert_close(head(u), ref["u"], TOL_BF16, "u")
    assert_close(head(qg), ref["qg"], TOL_BF16, "qg")
    assert_close(head(kg), ref["kg"], TOL_BF16, "kg")
    assert_close(head(v_new), ref["v_new"], TOL_BF16, "v_new")
    hh = head(h).transpose(1, 2)                      # [B,NT,Hv,..] -> [B,Hv,NT,..]
    hh = hh.transpose(-1, -2) if v_first else hh
    assert_close(hh, ref["h"], TOL_BF16, "h")
    # structure of the score matrices: upper triangles are exactly zero
    for b, n, ci, s, e in gdn.chunk_spans(B, T, C, cu):
        blk = head(Akk)[b, :, s:e, : e - s].float().cpu()
        assert float(torch.triu(blk, 1).abs().max()) == 0.0
        assert float(torch.triu(head(Aqk)[b, :, s:e, : e - s].float().cpu(), 1).abs().max()) == 0.0


def test_chunk_kda_fwd_output_policy(dev):
    """Hidden outputs are None and do not change the visible ones."""
    from fla_hip import ops
    q, k, v, g, beta = make_inputs(1, 128, 2, 2, 128, 128, seed=3)
    args = [to_layout(x, "BSND").to(dev) for x in (q, k, v, g, beta)]
    full = ops.chunk_kda_fwd(*args, 0.1, 64, output_final_state=True, disable_recompute=True)
    lean = ops.chunk_kda_fwd(*args, 0.1, 64)
    assert [x is None for x in lean] == [False, True, False, False, False, True, True, True, True, True, True, True]
    assert torch.equal(lean[0], full[0]) and torch.equal(lean[3], full[3]) and torch.equal(lean[4], full[4])
    mid = ops.chunk_kda_fwd(*args, 0.1, 64, return_intermediate_states=True, use_gate_in_kernel=True,
                            A_log=torch.zeros(2, device=dev))
    assert mid[2] is None and mid[10] is not None and mid[5] is None


def test_chunk_kda_fwd_errors(dev):
    from fla_hip import ops
    q, k, v, g, beta = make_inputs(1, 64, 2, 2, 128, 128, seed=3)
    a = [to_layout(x, "BSND").to(dev) for x in (q, k, v, g, beta)]
    with pytest.raises(RuntimeError, match="layout must be uppercase"):
        ops.chunk_kda_fwd(*a, 0.1, 64, layout="bsnd")
    with pytest.raises(RuntimeError, match="chunk_size must be 64 or 128"):
        ops.chunk_kda_fwd(*a, 0.1, 32)
    with pytest.raises(RuntimeError, match="rank does not match"):
        ops.chunk_kda_fwd(*a, 0.1, 64, layout="TND")
    with pytest.raises(RuntimeError, match="A_log must be float32"):
        ops.chunk_kda_fwd(*a, 0.1, 64, use_gate_in_kernel=True)
    with pytest.raises(RuntimeError, match="cu_seqlens must be nondecreasing"):
        ops.chunk_kda_fwd(*a, 0.1, 64, cu_seqlens=[0, 70, 60, 64])
    with pytest.raises(RuntimeError, match="canonical"):
        ops.chunk_kda_fwd(*a, 0.1, 64, cu_seqlens=[0, 64], chunk_indices=[0, 1])
    with pytest.raises(RuntimeError, match="initial_state shape"):
        ops.chunk_kda_fwd(*a, 0.1, 64, initial_state=torch.zeros(1, 2, 128, 64, device=dev))
    with pytest.raises(RuntimeError, match="same float16 or bfloat16 dtype"):
        ops.chunk_kda_fwd(a[0].half(), *a[1:], 0.1, 64)


def test_chunk_kda_fwd_state_handoff_and_determinism(dev):
    """A sequence processed in one call equals the same sequence cut at a chunk boundary with the final
    state handed over as initial state (bit for bit), and repeated calls are deterministic; the long
    case is also held against the fp32 recurrence."""
    from fla_hip import ops
    B, T, H, K, V = 1, 1024, 4, 128, 128
    q, k, v, g, beta = make_inputs(B, T, H, H, K, V, seed=21)
    scale = K ** -0.5
    x = [to_layout(t, "BSND").to(dev) for t in (q, k, v, g, beta)]
    o, final = ops.chunk_kda_fwd(*x, scale, 64, output_final_state=True)[:2]
    o_again, final_again = ops.chunk_kda_fwd(*x, scale, 64, output_final_state=True)[:2]
    assert torch.equal(o, o_again) and torch.equal(final, final_again)
    half = T // 2
    a = [t[:, :half].contiguous() for t in x]
    b = [t[:, half:].contiguous() for t in x]
    o1, f1 = ops.chunk_kda_fwd(*a, scale, 64, output_final_state=True)[:2]
    o2, f2 = ops.chunk_kda_fwd(*b, scale, 64, initial_state=f1, output_final_state=True)[:2]
    assert torch.equal(torch.cat([o1, o2], dim=1), o) and torch.equal(f2, final)
    nat = kda.kda_gate(g)
    o_naive, f_naive = kda.naive_recurrent_kda(q, k, v, nat, beta, scale, output_final_state=True)
    assert_close(from_layout(o, "BSND"), o_naive, TOL_BF16, "o vs recurrence, T=1024")
    assert_close(final, f_naive, TOL_STATE, "final state vs recurrence, T=1024")


def test_chunk_kda_fwd_packed_equals_separate(dev):
    """A packed variable-length batch gives, sequence by sequence, exactly what separate calls give."""
    from fla_hip import ops
    cu = [0, 100, 100, 361, 425]
    T, H, K, V = cu[-1], 2, 128, 128
    q, k, v, g, beta = make_inputs(1, T, H, H, K, V, seed=5)
    x = [to_layout(t, "TND").to(dev) for t in (q, k, v, g, beta)]
    gen = torch.Generator().manual_seed(2)
    h0 = (torch.randn(len(cu) - 1, H, K, V, generator=gen) * 0.1).to(dev)
    o, final = ops.chunk_kda_fwd(*x, 0.1, 64, layout="TND", initial_state=h0, output_final_state=True, cu_seqlens=cu)[:2]
    for n, (s, e) in enumerate(zip(cu, cu[1:])):
        if s == e:
            assert torch.equal(final[n], h0[n])          # an empty sequence hands its state through
            continue
        part = [t[s:e].contiguous() for t in x]
        o_n, f_n = ops.chunk_kda_fwd(*part, 0.1, 64, layout="TND", initial_state=h0[n:n + 1], output_final_state=True)[:2]
        assert torch.equal(o[s:e], o_n) and torch.equal(final[n], f_n[0])


def test_chunk_kda_fwd_dual_benchmark(dev):
    """The reference's acceptance standard for chunk_kda_fwd (tests/atk/chunk_kda_fwd/atk_chunk_kda_fwd.json): device
    and a CPU control that rounds to bf16 where the kernels round, both against the fp64 recurrence; the device's
    max / mean relative error and RMSE must stay within 5x / 1.5x / 1.5x of the control's."""
    from fla_hip import ops
    B, T, H, K, V = 2, 512, 4, 128, 128
    q, k, v, g, beta = make_inputs(B, T, H, H, K, V, seed=77)
    scale = K ** -0.5
    gen = torch.Generator().manual_seed(5)
    h0 = torch.randn(B, H, K, V, generator=gen) * 0.05
    dd = torch.float64
    t_o, t_f = kda.naive_recurrent_kda(q.to(dd), k.to(dd), v.to(dd), g.to(dd), beta.to(dd), scale, initial_state=h0.to(dd),
                                       output_final_state=True, compute_dtype=dd)
    gk = kda.kda_gate_cumsum(g, 64)
    ctrl = kda.chunk_kda_fwd(q, k, v, gk, beta, scale, 64, initial_state=h0, output_final_state=True, lowp=BF)
    out = ops.chunk_kda_fwd(*[to_layout(x, "BSND").to(dev) for x in (q, k, v, g, beta)], scale, 64, initial_state=h0.to(dev),
                            output_final_state=True)

    def stats(x, truth):
        x, truth = x.double().cpu(), truth.double()
        err = (x - truth).abs()
        re = err / truth.abs().clamp_min(1e-3 * float(truth.abs().max()))
        return float(re.max()), float(re.mean()), float(err.pow(2).mean().sqrt())

    for name, dut, c, truth in (("o", from_layout(out[0], "BSND"), ctrl["o"].to(BF), t_o), ("final_state", out[1], ctrl["final_state"], t_f)):
        a, cc = stats(dut, truth), stats(c, truth)
        assert a[0] <= 5 * cc[0] + 1e-6 and a[1] <= 1.5 * cc[1] + 1e-7 and a[2] <= 1.5 * cc[2] + 1e-9, (name, a, cc)


def test_chunk_kda_fwd_bench_shape_properties(dev):
    """B=2 T=8192 H=32 K=V=128, too large for the CPU oracle: the result must not depend on the chunk size (64 against
    128 tokens), a sequence cut at a chunk boundary with the state handed over must equal the uncut run, and the
    oracle's per-token recurrence is checked on one (batch row, head) slice."""
    from fla_hip import ops
    B, T, H, K, V = 2, 8192, 32, 128, 128
    gen = torch.Generator(device=dev).manual_seed(3)
    rn = lambda *s: torch.randn(*s, device=dev, generator=gen)
    q = torch.nn.functional.normalize(rn(B, T, H, K), dim=-1).to(BF)
    k = torch.nn.functional.normalize(rn(B, T, H, K), dim=-1).to(BF)
    v = rn(B, T, H, V).to(BF)
    g = torch.nn.functional.logsigmoid(rn(B, T, H, K)) * 0.3
    beta = torch.sigmoid(rn(B, T, H))
    h0 = rn(B, H, K, V) * 0.05
    scale = K ** -0.5
    o64, f64 = ops.chunk_kda_fwd(q, k, v, g, beta, scale, 64, initial_state=h0, output_final_state=True)[:2]
    o128, f128 = ops.chunk_kda_fwd(q, k, v, g, beta, scale, 128, initial_state=h0, output_final_state=True)[:2]
    assert_close(o128, o64, TOL_BF16, "o: 128- against 64-token chunks")
    assert_close(f128, f64, 2 * TOL_STATE, "final state: 128- against 64-token chunks")
    cut = 4096 + 128
    a = [x[:, :cut].contiguous() for x in (q, k, v, g, beta)]
    b = [x[:, cut:].contiguous() for x in (q, k, v, g, beta)]
    o1, f1 = ops.chunk_kda_fwd(*a, scale, 128, initial_state=h0, output_final_state=True)[:2]
    o2, f2 = ops.chunk_kda_fwd(*b, scale, 128, initial_state=f1, output_final_state=True)[:2]
    assert torch.equal(torch.cat([o1, o2], dim=1), o128) and torch.equal(f2, f128)
    # one slice against the per-token recurrence on the CPU
    bi, hi, Ts = 1, 17, 1024
    sl = lambda x: x[bi:bi + 1, :Ts, hi:hi + 1].transpose(1, 2).float().cpu()
    o_ref, _ = kda.naive_recurrent_kda(sl(q), sl(k), sl(v), sl(g), beta[bi:bi + 1, :Ts, hi:hi + 1].transpose(1, 2).cpu(), scale,
                                       initial_state=h0[bi:bi + 1, hi:hi + 1].cpu(), output_final_state=True)
    assert_close(o128[bi:bi + 1, :Ts, hi:hi + 1].transpose(1, 2), o_ref, TOL_BF16, "o slice vs recurrence")


def test_chunk_kda_fwd_bench_shape_unscaled_gate(dev):
    """B=2 T=8192 H=32 K=V=128 with the gate as the benchmark configuration draws it (logsigmoid of a standard normal,
    not scaled down): attention output and fp32 final state of one (batch row, head) slice over all 8192 tokens against
    the per-token recurrence on the CPU, at the acceptance tolerances."""
    from fla_hip import ops
    B, T, H, K, V = 2, 8192, 32, 128, 128
    gen = torch.Generator(device=dev).manual_seed(5)
    rn = lambda *s: torch.randn(*s, device=dev, generator=gen)
    q = torch.nn.functional.normalize(rn(B, T, H, K), dim=-1).to(BF)
    k = torch.nn.functional.normalize(rn(B, T, H, K), dim=-1).to(BF)
    v = rn(B, T, H, V).to(BF)
    g = torch.nn.functional.logsigmoid(rn(B, T, H, K))
    beta = torch.sigmoid(rn(B, T, H))
    h0 = rn(B, H, K, V) * 0.01
    scale = K ** -0.5
    o, final = ops.chunk_kda_fwd(q, k, v, g, beta, scale, 64, initial_state=h0, output_final_state=True)[:2]
    for bi, hi in ((1, 17), (0, 0)):
        sl = lambda x: x[bi:bi + 1, :, hi:hi + 1].transpose(1, 2).float().cpu()
        o_ref, f_ref = kda.naive_recurrent_kda(sl(q), sl(k), sl(v), sl(g), beta[bi:bi + 1, :, hi:hi + 1].transpose(1, 2).cpu(),
                                               scale, initial_state=h0[bi:bi + 1, hi:hi + 1].cpu(), output_final_state=True)
        st = assert_close(o[bi:bi + 1, :, hi:hi + 1].transpose(1, 2), o_ref, TOL_BF16, f"o of slice ({bi}, {hi})")
        assert st["rel_max"] < 2e-2, st
        assert_close(final[bi:bi + 1, hi:hi + 1], f_ref, TOL_STATE, f"final state of slice ({bi}, {hi})")
