"""Parity of the HIP recurrent_gated_delta_rule (through the C ABI) against the CPU oracle.

Shapes follow fla/ops/ascendc/gdn/recurrent_gdn/recurrent_gated_delta_rule/tests/pta
(T=2..., K=V=128) plus the decode benchmark layout; tolerance: bf16 out 2e-2, fp32 state 1e-3."""
import pytest
import torch

from oracle import decode as od
from util import assert_close, TOL_BF16, TOL_STATE

pytestmark = pytest.mark.gpu
F = torch.nn.functional


def make_inputs(lens, Nk, Nv, Dk, Dv, *, seed=0, skip=0, blocks=None, state_dtype=torch.float32, gk=False, g=True):
    gen = torch.Generator().manual_seed(seed)
    T = skip + sum(lens)
    q = F.normalize(torch.randn(T, Nk, Dk, generator=gen), dim=-1).bfloat16()
    k = F.normalize(torch.randn(T, Nk, Dk, generator=gen), dim=-1).bfloat16()
    v = torch.randn(T, Nv, Dv, generator=gen).bfloat16()
    beta = torch.sigmoid(torch.randn(T, Nv, generator=gen)).bfloat16()
    gate = F.logsigmoid(torch.randn(T, Nv, generator=gen)) if g else None
    gkk = F.logsigmoid(torch.randn(T, Nv, Dk, generator=gen)) * 0.1 if gk else None
    blocks = blocks or T
    state = (torch.randn(blocks, Nv, Dv, Dk, generator=gen) * 0.01).to(state_dtype)
    seq = torch.tensor([skip] + list(lens), dtype=torch.int32)
    idx = torch.randperm(blocks, generator=gen)[:T].to(torch.int32)
    return dict(q=q, k=k, v=v, beta=beta, g=gate, gk=gkk, state=state, lens=seq, idx=idx, scale=Dk ** -0.5)


def run(dev, d, accepted=None, idx=None):
    from fla_hip import ops
    idx = d["idx"] if idx is None else idx
    o_ref, s_ref = od.recurrent_gated_delta_rule(
        d["q"], d["k"], d["v"], d["state"], beta=d["beta"], scale=d["scale"], actual_seq_lengths=d["lens"],
        ssm_state_indices=idx, num_accepted_tokens=accepted, g=d["g"], gk=d["gk"])
    st = d["state"].to(dev)
    to = lambda t: None if t is None else t.to(dev)
    o = ops.recurrent_gated_delta_rule(
        to(d["q"]), to(d["k"]), to(d["v"]), st, beta=to(d["beta"]), scale=d["scale"],
        actual_seq_lengths=to(d["lens"]), ssm_state_indices=to(idx), num_accepted_tokens=to(accepted),
        g=to(d["g"]), gk=to(d["gk"]))
    return o, o_ref, st, s_ref


@pytest.mark.parametrize("dims", [(128, 128), (64, 64), (128, 256), (64, 128)])
def test_single_token_decode(dev, dims):
    Dk, Dv = dims
    d = make_inputs([1] * 6, 2, 4, Dk, Dv, seed=1)   # GVA: Nv = 2 * Nk; K != V cases check the V-first layout
    o, o_ref, st, s_ref = run(dev, d)
    assert_close(o, o_ref, TOL_BF16, "out")
    assert_close(st, s_ref, TOL_STATE, "state")


@pytest.mark.parametrize("dims", [(16, 16), (48, 80), (96, 32), (192, 160), (256, 256), (512, 512), (320, 24), (128, 64), (100, 36)])
def test_other_head_sizes(dev, dims):
    """Head sizes without a register-resident kernel (the reference admits any Dk, Dv <= 512,
    _aclnn_ctypes.py:813-817): multi-token sequences with slot changes, accepted-token source slots, both gates,
    fp32 and bf16 pools."""
    Dk, Dv = dims
    d = make_inputs([3, 1, 6, 2], 2, 4, Dk, Dv, seed=Dk + Dv, blocks=30, gk=True)
    acc = torch.tensor([2, 1, 4, 1], dtype=torch.int32)
    o, o_ref, st, s_ref = run(dev, d, accepted=acc)
    assert_close(o, o_ref, TOL_BF16, "out")
    assert_close(st, s_ref, TOL_STATE, "state")
    d = make_inputs([1] * 5, 2, 2, Dk, Dv, seed=Dk, state_dtype=torch.bfloat16)
    o, o_ref, st, s_ref = run(dev, d)
    assert_close(o, o_ref, TOL_BF16, "out")
    assert_close(st, s_ref.bfloat16(), TOL_BF16, "state")


def test_multi_token_and_skip_prefix(dev):
    d = make_inputs([3, 8, 1, 0, 5], 2, 2, 128, 128, seed=2, skip=2, blocks=40)
    o, o_ref, st, s_ref = run(dev, d)
    # skipped leading tokens are not produced by the op: compare from the prefix on
    assert_close(o[2:], o_ref[2:], TOL_BF16, "out")
    assert_close(st, s_ref, TOL_STATE, "state")


def test_accepted_tokens_select_source_slot(dev):
    d = make_inputs([4, 4], 1, 2, 128, 128, seed=3, blocks=16)
    acc = torch.tensor([2, 4], dtype=torch.int32)
    o, o_ref, st, s_ref = run(dev, d, accepted=acc)
    assert_close(o, o_ref, TOL_BF16, "out")
    assert_close(st, s_ref, TOL_STATE, "state")


def test_gk_only_and_both_gates(dev):
    for g, gk in ((False, True), (True, True)):
        d = make_inputs([2, 3], 2, 2, 128, 128, seed=4, g=g, gk=gk)
        o, o_ref, st, s_ref = run(dev, d)
        assert_close(o, o_ref, TOL_BF16, "out")
        assert_close(st, s_ref, TOL_STATE, "state")


def test_bf16_state(dev):
    d = make_inputs([1, 2, 1], 2, 2, 128, 128, seed=5, state_dtype=torch.bfloat16)
    o, o_ref, st, s_ref = run(dev, d)
    assert_close(o, o_ref, TOL_BF16, "out")
    assert_close(st, s_ref.bfloat16(), TOL_BF16, "state")


def test_long_sequence_same_slot(dev):
    """Prefill through the recurrent kernel: 300 tokens, every token mapped to one slot
    (beyond the reference op's 8-token limit; oracle = the same recurrence)."""
    d = make_inputs([300, 70], 1, 2, 128, 128, seed=6, blocks=4)
    idx = torch.cat([torch.full((300,), 2), torch.full((70,), 0)]).to(torch.int32)
    o, o_ref, st, s_ref = run(dev, d, idx=idx)
    assert_close(o, o_ref, TOL_BF16, "out")
    assert_close(st, s_ref, TOL_STATE, "state")


def test_strided_state_pool(dev):
    from fla_hip import ops
    d = make_inputs([1, 1, 1], 2, 2, 128, 128, seed=7, blocks=3)
    pool = torch.zeros(3, 4, 128, 128)
    pool[:, ::2] = d["state"]
    o_ref, s_ref = od.recurrent_gated_delta_rule(
        d["q"], d["k"], d["v"], d["state"], beta=d["beta"], scale=d["scale"], actual_seq_lengths=d["lens"],
        ssm_state_indices=d["idx"], g=d["g"])
    pool_d = pool.to(dev)
    o = ops.recurrent_gated_delta_rule(
        d["q"].to(dev), d["k"].to(dev), d["v"].to(dev), pool_d[:, ::2], beta=d["beta"].to(dev), scale=d["scale"],
        actual_seq_lengths=d["lens"].to(dev), ssm_state_indices=d["idx"].to(dev), g=d["g"].to(dev))
    assert_close(o, o_ref, TOL_BF16, "out")
    assert_close(pool_d[:, ::2], s_ref, TOL_STATE, "state")
    assert float(pool_d[:, 1::2].abs().max()) == 0.0


def test_decode_benchmark_shape_properties(dev):
    """256 sequences x 1 token, 32 heads, K=V=128: oracle on a subset of sequences."""
    from fla_hip import ops
    d = make_inputs([1] * 256, 32, 32, 128, 128, seed=0, blocks=256)
    d["idx"] = torch.arange(256, dtype=torch.int32)
    st = d["state"].to(dev)
    to = lambda t: t.to(dev)
    o = ops.recurrent_gated_delta_rule(to(d["q"]), to(d["k"]), to(d["v"]), st, beta=to(d["beta"]), scale=d["scale"],
                                       actual_seq_lengths=to(d["lens"]), ssm_state_indices=to(d["idx"]), g=to(d["g"]))
    sub = [0, 17, 255]
    for t in sub:
        o_ref, s_ref = od.recurrent_gated_delta_rule(
            d["q"][t:t + 1], d["k"][t:t + 1], d["v"][t:t + 1], d["state"][t:t + 1], beta=d["beta"][t:t + 1],
            scale=d["scale"], actual_seq_lengths=torch.tensor([0, 1], dtype=torch.int32),
            ssm_state_indices=torch.zeros(1, dtype=torch.int32), g=d["g"][t:t + 1])
        assert_close(o[t:t + 1], o_ref, TOL_BF16, "out")
        assert_close(st[t:t + 1], s_ref, TOL_STATE, "state")


def test_varlen_prefill_benchmark_shape(dev):
    """The variable-length prefill of the decode benchmark at full size: 64 sequences with lengths uniform in
    [128, 4096] (about 135 K tokens), 32 heads, K=V=128, one state slot per sequence.  (a) Every sequence run on its own
    gives the bits of the packed run (a sequence never sees its neighbours); (b) the shortest, the longest and a
    middle sequence equal the fp32 per-token recurrence.  Far beyond the reference operator's 8-token limit, so the
    recurrence is the only oracle."""
    from fla_hip import ops
    H, D, NSEQ = 32, 128, 64
    lens = torch.randint(128, 4097, (NSEQ,), generator=torch.Generator().manual_seed(0))
    T = int(lens.sum())
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).tolist()
    gen = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=gen)
    q = F.normalize(rn(T, H, D), dim=-1).bfloat16()
    k = F.normalize(rn(T, H, D), dim=-1).bfloat16()
    v = rn(T, H, D).bfloat16()
    beta = torch.sigmoid(rn(T, H)).bfloat16()
    gate = F.logsigmoid(rn(T, H))
    state0 = rn(NSEQ, H, D, D) * 0.01
    seq = torch.cat([torch.zeros(1, dtype=torch.int32), lens.to(torch.int32)]).to(dev)
    idx = torch.repeat_interleave(torch.arange(NSEQ, dtype=torch.int32), lens).to(dev)
    state = state0.clone()
    o = ops.recurrent_gated_delta_rule(q, k, v, state, beta=beta, scale=D ** -0.5, actual_seq_lengths=seq,
                                       ssm_state_indices=idx, g=gate)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o.float()).all()) and bool(torch.isfinite(state).all())
    one = torch.tensor([0, 0], dtype=torch.int32)
    for n in range(NSEQ):
        s, e = cu[n], cu[n + 1]
        st = state0[n:n + 1].clone()
        one[1] = e - s
        o_n = ops.recurrent_gated_delta_rule(q[s:e], k[s:e], v[s:e], st, beta=beta[s:e], scale=D ** -0.5,
                                             actual_seq_lengths=one.to(dev),
                                             ssm_state_indices=torch.zeros(e - s, dtype=torch.int32, device=dev), g=gate[s:e])
        assert torch.equal(o_n, o[s:e]) and torch.equal(st[0], state[n]), f"sequence {n} differs from the packed run"
    order = torch.argsort(lens).tolist()
    for n in (order[0], order[NSEQ // 2], order[-1]):
        s, e = cu[n], cu[n + 1]
        c = lambda t: t[s:e].cpu()
        o_ref, s_ref = od.recurrent_gated_delta_rule(
            c(q), c(k), c(v), state0[n:n + 1].cpu(), beta=c(beta), scale=D ** -0.5,
            actual_seq_lengths=torch.tensor([0, e - s], dtype=torch.int32),
            ssm_state_indices=torch.zeros(e - s, dtype=torch.int32), g=c(gate))
        assert_close(o[s:e], o_ref, TOL_BF16, f"out of sequence {n} ({e - s} tokens)")
        assert_close(state[n:n + 1], s_ref, TOL_STATE, f"state of sequence {n}")
    # (c) the chunked forward on the same packed tokens (strided head-major views, the pool rows transposed into its
    # [N,H,K,V] state) agrees with the token-by-token kernel on every sequence
    from fla_hip import pipeline
    hm = lambda t: t.transpose(0, 1)[None]
    o_c, fin = pipeline.flash_gated_delta_rule(hm(q), hm(k), hm(v), gate[None], beta[None].float(), D ** -0.5,
                                               state0.transpose(-1, -2).contiguous(), True, cu_seqlens=cu)
    assert_close(o_c[0], o.float(), TOL_BF16, "chunked forward vs recurrent kernel, out")
    assert_close(fin.transpose(-1, -2), state, 2 * TOL_STATE, "chunked forward vs recurrent kernel, state")


def test_wrapper_errors(dev):
    from fla_hip import ops
    with pytest.raises(RuntimeError, match=r"^npu_recurrent_gated_delta_rule: either g or gk must be provided\.$"):
        ops.npu_recurrent_gated_delta_rule(None, None, None, None, beta=None, actual_seq_lengths=None,
                                           ssm_state_indices=None)
