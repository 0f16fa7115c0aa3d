"""Parity of the HIP recurrent_gated_delta_rule (through the C ABI) against the CPU oracle.

Shapes follow fla/ops/ascendc/gdn/recurrent_gdn/recurrent_gated_delta_rule/tests/pta
(T=2..., K=V=128) plus the decode benchmark layout; tolerance: bf16 out 2e-2, fp32 state 1e-3."""
import pytest
import torch
import torch.nn.functional as F

from oracle import decode as od
from util import assert_close, TOL_BF16, TOL_STATE

pytestmark = pytest.mark.gpu
F = torch.nn.functional
BF = torch.bfloat16


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


def launches(kernel, call):
    """Runs ``call`` and checks through the library's own launch records that ``kernel`` ran."""
    import ctypes

    import fla_hip
    lib = fla_hip.load_library()
    lib.fla_profile_enable.argtypes = [ctypes.c_int]
    lib.fla_profile_report.argtypes = [ctypes.c_char_p, ctypes.c_uint64]
    lib.fla_profile_enable(1)
    try:
        out = call()
        torch.cuda.synchronize()
    finally:
        lib.fla_profile_enable(0)
    buf = ctypes.create_string_buffer(1 << 14)
    lib.fla_profile_report(buf, len(buf))
    names = [line.split()[0] for line in buf.value.decode().splitlines()]
    assert kernel in names, (kernel, names)
    return out


class token_by_token:
    """Keeps recurrent_gated_delta_rule on its token-by-token kernel whatever the sequence lengths."""

    def __enter__(self):
        from fla_hip.ops import _hip_ctypes as raw
        self.raw, self.saved = raw, raw.PREFILL_MIN_TOKENS
        raw.PREFILL_MIN_TOKENS = 1 << 62

    def __exit__(self, *exc):
        self.raw.PREFILL_MIN_TOKENS = self.saved


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
    [128, 4096] (about 135 K tokens), 32 heads, K=V=128, one state slot per sequence.  The operator runs it on the chunk
    kernels; the token-by-token kernel is run on the same call beside it.  (a) Every sequence run on its own gives what
    the packed run gives (a sequence never sees its neighbours); (b) the shortest, the longest and a middle sequence
    equal the fp32 per-token recurrence on both kernels.  Far beyond the reference operator's 8-token limit, so the
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
    o = launches("gdn_fused", lambda: ops.recurrent_gated_delta_rule(
        q, k, v, state, beta=beta, scale=D ** -0.5, actual_seq_lengths=seq, ssm_state_indices=idx, g=gate))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o.float()).all()) and bool(torch.isfinite(state).all())
    # the token-by-token kernel on the same call (what the operator runs for short sequences)
    state_tok = state0.clone()
    with token_by_token():
        o_tok = launches("recurrent_gdn", lambda: ops.recurrent_gated_delta_rule(
            q, k, v, state_tok, beta=beta, scale=D ** -0.5, actual_seq_lengths=seq, ssm_state_indices=idx, g=gate))
    assert_close(o, o_tok.float(), TOL_BF16, "chunk kernels vs token-by-token kernel, out")
    assert_close(state, state_tok, 2 * TOL_STATE, "chunk kernels vs token-by-token kernel, state")
    one = torch.tensor([0, 0], dtype=torch.int32)
    for n in range(NSEQ):
        s, e = cu[n], cu[n + 1]
        st = state0[n:n + 1].clone()
        one[1] = e - s
        o_n = ops.recurrent_gated_delta_rule(q[s:e], k[s:e], v[s:e], st, beta=beta[s:e], scale=D ** -0.5,
                                             actual_seq_lengths=one.to(dev),
                                             ssm_state_indices=torch.zeros(e - s, dtype=torch.int32, device=dev), g=gate[s:e])
        # (the chunk kernels pick their slab width by the size of the batch: the same products in another order)
        assert_close(o_n, o[s:e], 1e-2, f"sequence {n} on its own, out")
        assert_close(st[0], state[n], 1e-5, f"sequence {n} on its own, state")
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
        o_ref_t, s_ref_t = o_tok[s:e], state_tok[n:n + 1]
        assert_close(o_ref_t, o_ref, TOL_BF16, f"token-by-token kernel, out of sequence {n}")
        assert_close(s_ref_t, s_ref, TOL_STATE, f"token-by-token kernel, state of sequence {n}")


def test_prefill_route_keeps_the_operator_contract(dev):
    """Which calls leave the token-by-token kernel, and what they write: a skipped prefix, an empty sequence, a bf16
    pool, slots in arbitrary order and untouched slots of the pool; slots that change inside a sequence, slots shared by
    two sequences, a key-wise gate and accepted-token counts stay on the token-by-token kernel."""
    from fla_hip import ops
    lens = [100, 0, 333, 64]
    d = make_inputs(lens, 2, 4, 128, 128, seed=5, skip=3, blocks=9)
    slots = [7, 2, 0, 5]
    d["idx"] = torch.cat([torch.zeros(3, dtype=torch.int32)] +
                         [torch.full((n,), s, dtype=torch.int32) for n, s in zip(lens, slots)])
    to = lambda t: None if t is None else t.to(dev)
    for pool_dtype, tol in ((torch.float32, TOL_STATE), (BF, TOL_BF16)):
        pool = d["state"].to(pool_dtype)
        o_ref, s_ref = od.recurrent_gated_delta_rule(d["q"], d["k"], d["v"], pool.float(), beta=d["beta"], scale=d["scale"],
                                                     actual_seq_lengths=d["lens"], ssm_state_indices=d["idx"], g=d["g"])
        st = pool.to(dev)
        o = launches("gdn_fused", lambda: ops.recurrent_gated_delta_rule(
            to(d["q"]), to(d["k"]), to(d["v"]), st, beta=to(d["beta"]), scale=d["scale"], actual_seq_lengths=to(d["lens"]),
            ssm_state_indices=to(d["idx"]), g=to(d["g"])))
        assert_close(o[3:], o_ref[3:], TOL_BF16, "out")
        assert_close(st, s_ref.to(pool_dtype), tol, "pool")
        untouched = [b for b in range(9) if b not in (7, 0, 5)]
        assert torch.equal(st[untouched].cpu(), pool[untouched]), "slots of no sequence must keep their contents"
    # not a prefill in the sense of the route
    changing = d["idx"].clone()
    changing[50] = 8
    shared = d["idx"].clone()
    shared[d["idx"] == 5] = 7
    for what, idx, extra in (("changing", changing, {}), ("shared", shared, {}),
                             ("accepted", d["idx"], dict(num_accepted_tokens=torch.tensor([1, 1, 1, 1], dtype=torch.int32)))):
        st = d["state"].to(dev)
        launches("recurrent_gdn", lambda: ops.recurrent_gated_delta_rule(
            to(d["q"]), to(d["k"]), to(d["v"]), st, beta=to(d["beta"]), scale=d["scale"], actual_seq_lengths=to(d["lens"]),
            ssm_state_indices=to(idx), g=to(d["g"]), **{k_: to(v_) for k_, v_ in extra.items()}))


def test_prefill_plan_and_pooled_forward(dev):
    """The two entry points under the prefill route on their own: the plan's slots and flags for good and bad index
    lists, and the chunk forward on pool rows (K x V blocks here; the route passes V x K ones) against the same forward
    on gathered rows."""
    import ctypes
    from fla_hip.ops import _hip_ctypes as raw, _runtime

    def plan(lens, idx, blocks, skip=0):
        B = len(lens)
        lens_d = torch.tensor([skip] + lens, dtype=torch.int32, device=dev)
        idx_d = torch.tensor(idx, dtype=torch.int32, device=dev)
        slots = torch.full((B,), 99, dtype=torch.int32, device=dev)
        report = torch.full((2 * B + 1,), 99, dtype=torch.int32, device=dev)
        _runtime.call_op_noalloc("recurrent_gdn_prefill_plan", raw.OP_ARGTYPES["recurrent_gdn_prefill_plan"],
                                 lambda ctx: [ctx.tensor(lens_d), ctx.tensor(idx_d), ctypes.c_int64(blocks), ctx.tensor(slots),
                                              ctx.tensor(report)], (slots, report))
        r = report.tolist()
        assert r[0] == skip and r[1:1 + B] == lens
        return slots.tolist(), r[1 + B:]

    rows = lambda lens, slots: [s for n, s in zip(lens, slots) for _ in range(n)]
    lens = [3, 0, 5, 2]
    assert plan(lens, [4, 4] + rows(lens, [6, 1, 0, 2]), 7, skip=2) == ([6, -1, 0, 2], [0, 0, 0, 0])
    changing = rows(lens, [6, 1, 0, 2])
    changing[4] = 3
    assert plan(lens, changing, 7) == ([6, -1, -1, 2], [0, 0, 1, 0])
    assert plan(lens, rows(lens, [6, 1, 6, 2]), 7) == ([-1, -1, -1, 2], [1, 0, 1, 0])        # two sequences on one row
    assert plan(lens, rows(lens, [6, 1, 7, 2]), 7) == ([6, -1, -1, 2], [0, 0, 1, 0])         # a row outside the pool
    assert plan(lens, rows(lens, [6, 1, -1, 2]), 7) == ([6, -1, -1, 2], [0, 0, 1, 0])
    assert plan(lens, rows(lens, [6, 1, 0, 2])[:-1], 7)[1] == [1, 1, 1, 1]                   # lengths that overrun the token list
    assert plan([3, -1, 5, 2], rows(lens, [6, 1, 0, 2]), 7)[1] == [1, 1, 1, 1]
    big = list(range(300))
    assert plan([1] * 300, big, 300) == (big, [0] * 300)                                      # more sequences than threads

    gen = torch.Generator().manual_seed(3)
    H, K, V, seqs = 2, 128, 128, [70, 0, 130]
    T = sum(seqs)
    cu = [0, 70, 70, 200]
    q = F.normalize(torch.randn(1, H, T, K, generator=gen), dim=-1).to(BF).to(dev)
    k = F.normalize(torch.randn(1, H, T, K, generator=gen), dim=-1).to(BF).to(dev)
    v = torch.randn(1, H, T, V, generator=gen).to(BF).to(dev)
    g = F.logsigmoid(torch.randn(1, T, H, generator=gen)).to(dev)
    beta = torch.sigmoid(torch.randn(1, T, H, generator=gen)).to(dev)
    pool0 = (torch.randn(5, H, K, V, generator=gen) * 0.1).to(dev)
    slots = torch.tensor([3, -1, 1], dtype=torch.int32, device=dev)
    h0 = pool0[[3, 0, 1]].clone()
    h0[1] = 0
    _, o_ref, final = raw.gdn_chunk_fwd(q, k, v, g, beta, K ** -0.5, h0, True, cu, 64)
    for vfirst in (False, True):
        pool = pool0.transpose(-1, -2).contiguous().transpose(-1, -2) if vfirst else pool0.clone()
        o = raw.gdn_chunk_fwd_state_pool(q, k, v, g, beta, K ** -0.5, pool, slots, cu, 64)
        assert torch.equal(o, o_ref)
        assert torch.equal(pool[[3, 1]], final[[0, 2]]) and torch.equal(pool[[0, 2, 4]], pool0[[0, 2, 4]])
    # 64 channels, 128 value columns, rows normalised inside the kernel
    K2 = 64
    q2, k2 = (torch.randn(1, H, T, K2, generator=gen).to(BF).to(dev) for _ in range(2))
    pool2 = (torch.randn(5, H, K2, V, generator=gen) * 0.1).to(dev)
    h2 = pool2[[3, 0, 1]].clone()
    h2[1] = 0
    _, o_ref, final = raw.gdn_chunk_fwd(q2, k2, v, g, beta, K2 ** -0.5, h2, True, cu, 64, True)
    pool = pool2.clone()
    o = raw.gdn_chunk_fwd_state_pool(q2, k2, v, g, beta, K2 ** -0.5, pool, slots, cu, 64, use_qk_l2norm_in_kernel=True)
    assert torch.equal(o, o_ref) and torch.equal(pool[[3, 1]], final[[0, 2]]) and torch.equal(pool[[0, 2, 4]], pool2[[0, 2, 4]])


def test_wrapper_errors(dev):
    from fla_hip import ops
    with pytest.raises(RuntimeError, match=r"^npu_recurrent_gated_delta_rule: either g or gk must be provided\.$"):
        ops.npu_recurrent_gated_delta_rule(None, None, None, None, beta=None, actual_seq_lengths=None,
                                           ssm_state_indices=None)
