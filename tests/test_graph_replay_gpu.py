"""Serving loops replay the decode step (and a dense prefill) from a HIP graph.  Each operator here is captured once
and replayed several times with new contents in the same buffers, the program's own eager launches and
synchronisations in between; every replay must equal the eager result of the same inputs bit for bit (same kernels,
fixed summation order).  Sequence lengths, slot indices and accepted counts are device tensors read by the kernels,
so they may change between replays as well."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def capture(fn):
    """Warm up on a side stream (lazy initialisation must not land inside the capture), then capture one call."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


def test_gdn_decode_step_replays(dev):
    from fla_hip import ops
    B, Nk, Nv, D, slots = 16, 2, 4, 128, 40
    gen = torch.Generator().manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=gen)
    buf = dict(q=F.normalize(rn(B, Nk, D), dim=-1).to(BF), k=F.normalize(rn(B, Nk, D), dim=-1).to(BF), v=rn(B, Nv, D).to(BF),
               beta=torch.sigmoid(rn(B, Nv)).to(BF), g=F.logsigmoid(rn(B, Nv)),
               lens=torch.tensor([0] + [1] * B, dtype=torch.int32),   # leading entry: tokens skipped before the first sequence
                idx=torch.randperm(slots, generator=gen)[:B].to(torch.int32))
    buf = {n: t.to(dev) for n, t in buf.items()}
    pool = (rn(slots, Nv, D, D) * 0.01).to(dev)

    def step(state):
        return ops.recurrent_gated_delta_rule(buf["q"], buf["k"], buf["v"], state, beta=buf["beta"], scale=D ** -0.5,
                                              actual_seq_lengths=buf["lens"], ssm_state_indices=buf["idx"], g=buf["g"])

    static_pool = pool.clone()
    graph, out = capture(lambda: step(static_pool))
    for trial in range(4):
        gen.manual_seed(100 + trial)
        buf["q"].copy_(F.normalize(rn(B, Nk, D), dim=-1).to(BF))
        buf["v"].copy_(rn(B, Nv, D).to(BF))
        buf["idx"].copy_(torch.randperm(slots, generator=gen)[:B].to(torch.int32))   # other slots on every replay
        static_pool.copy_(pool)
        eager_pool = pool.clone()
        eager = step(eager_pool)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {trial}: output"
        assert torch.equal(static_pool, eager_pool), f"replay {trial}: state pool"
        assert not torch.equal(static_pool, pool)


def test_recurrent_kda_step_replays(dev):
    from fla_hip import ops
    B, H, HV, K, V, slots = 8, 2, 4, 128, 128, 12
    gen = torch.Generator().manual_seed(1)
    rn = lambda *s: torch.randn(*s, generator=gen)
    q, k, v = rn(B, 1, H, K).to(BF).to(dev), rn(B, 1, H, K).to(BF).to(dev), rn(B, 1, HV, V).to(BF).to(dev)
    g, beta = (F.logsigmoid(rn(B, 1, HV, K)) * 0.3).to(dev), torch.sigmoid(rn(B, 1, HV)).to(dev)
    idx = torch.randperm(slots, generator=gen)[:B].to(torch.int32).reshape(B, 1).to(dev)
    pool = (rn(slots, HV, K, V) * 0.1).to(dev)

    def step(state):
        return ops.recurrent_kda(q, k, v, g, beta, state, ssm_state_indices=idx, use_qk_l2norm_in_kernel=True)[0]

    static_pool = pool.clone()
    graph, out = capture(lambda: step(static_pool))
    for trial in range(3):
        gen.manual_seed(200 + trial)
        k.copy_(rn(B, 1, H, K).to(BF))
        g.copy_(F.logsigmoid(rn(B, 1, HV, K)) * 0.3)
        idx.copy_(torch.randperm(slots, generator=gen)[:B].to(torch.int32).reshape(B, 1))
        static_pool.copy_(pool)
        eager_pool = pool.clone()
        eager = step(eager_pool)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {trial}: output"
        assert torch.equal(static_pool, eager_pool), f"replay {trial}: state pool"


def test_conv1d_update_and_dense_prefill_replay(dev):
    from fla_hip import ops
    from fla_hip.pipeline import flash_gated_delta_rule
    gen = torch.Generator().manual_seed(2)
    rn = lambda *s: torch.randn(*s, generator=gen)
    # conv state update of one token per sequence
    N, D, W = 32, 512, 4
    x, weight, bias = rn(N, 1, D).to(BF).to(dev), rn(W, D).to(BF).to(dev), rn(D).to(BF).to(dev)
    states = rn(N, W - 1, D).to(BF).to(dev)
    static_states = states.clone()
    conv = lambda st: ops.causal_conv1d(x, weight, bias, st, activation_mode=1, run_mode=1)
    g1, y = capture(lambda: conv(static_states))
    # dense chunk forward
    B, T, H, K = 1, 512, 4, 128
    q, k, v = (F.normalize(rn(B, H, T, K), dim=-1).to(BF).to(dev) for _ in range(3))
    gg, beta = F.logsigmoid(rn(B, T, H)).to(dev), torch.sigmoid(rn(B, T, H)).to(dev)
    h0 = (rn(B, H, K, K) * 0.1).to(dev)
    prefill = lambda: flash_gated_delta_rule(q, k, v, gg, beta, initial_state=h0, output_final_state=True)
    g2, (o, hT) = capture(prefill)
    for trial in range(3):
        gen.manual_seed(300 + trial)
        x.copy_(rn(N, 1, D).to(BF))
        static_states.copy_(states)
        eager_states = states.clone()
        y_eager = conv(eager_states)
        v.copy_(rn(B, H, T, K).to(BF))
        h0.copy_(rn(B, H, K, K) * 0.1)
        o_eager, hT_eager = prefill()
        torch.cuda.synchronize()
        g1.replay()
        g2.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, y_eager) and torch.equal(static_states, eager_states), f"replay {trial}: conv1d update"
        assert torch.equal(o, o_eager) and torch.equal(hT, hT_eager), f"replay {trial}: chunk forward"


def test_calls_with_host_integer_arrays_refuse_stream_capture(dev):
    """A packed batch hands cu_seqlens over as a host array that the library uploads through a recycled pinned slot: a
    captured upload would replay other calls' metadata, so the call is refused while the stream is capturing (nothing is
    launched), and the same call works eagerly before and after."""
    from fla_hip import pipeline
    from oracle import gdn
    d = gdn.make_gdn_inputs(1, 130, 2, 128, 128, dtype=BF, seed=3)
    cu = [0, 65, 130]
    args = [d[n].to(dev) for n in ("q", "k", "v", "g", "beta")]
    call = lambda: pipeline.flash_gated_delta_rule(*args, None, None, True, cu_seqlens=cu)
    o_before, f_before = call()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="cannot be uploaded while the stream is being captured"):
        with torch.cuda.graph(graph):
            call()
    torch.cuda.synchronize()
    for _ in range(20):            # more calls than the staging ring has slots
        o_after, f_after = call()
    torch.cuda.synchronize()
    assert torch.equal(o_before, o_after) and torch.equal(f_before, f_after)
