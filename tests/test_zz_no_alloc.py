"""fla_chunk_kda_fwd_noalloc (the entry point that allocates nothing and keeps its scratch in a fixed device
array) against fla_chunk_kda_fwd, both called through the C ABI.

The two entry points launch the same kernels on the same operands, so every output must be bit-identical.
Two calls in a row, the second smaller than the first: the array still holds the first call's decay rows and
intermediates when the second call starts.  Then the limits: a call whose scratch need exceeds the array and a
packed batch are rejected with a status, before anything is launched."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
NAMES = ("o", "final_state", "gk", "Aqk", "Akk", "w", "u", "qg", "kg", "v_new", "h")


def make(B, T, Hk, Hv, K, V, seed, dev, dtype=BF):
    gen = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, T, Hk, K, generator=gen), dim=-1).to(dtype)
    k = F.normalize(torch.randn(B, T, Hk, K, generator=gen), dim=-1).to(dtype)
    v = torch.randn(B, T, Hv, V, generator=gen).to(dtype)
    g = F.logsigmoid(torch.randn(B, T, Hv, K, generator=gen)) * 0.3
    beta = torch.sigmoid(torch.randn(B, T, Hv, generator=gen))
    h0 = torch.randn(B, Hv, K, V, generator=gen) * 0.01
    return [t.to(dev) for t in (q, k, v, g, beta, h0)]


def run_pair(dev, B, T, Hk, Hv, K, V, seed, *, keep, dtype=BF):
    from fla_hip import ops

    q, k, v, g, beta, h0 = make(B, T, Hk, Hv, K, V, seed, dev, dtype)
    kw = dict(layout="BSND", initial_state=h0, output_final_state=True, disable_recompute=keep,
              return_intermediate_states=True)
    want = ops.chunk_kda_fwd(q, k, v, g, beta, K ** -0.5, 64, **kw)
    got = ops.chunk_kda_fwd_noalloc(q, k, v, g, beta, K ** -0.5, 64, **kw)
    torch.cuda.synchronize()
    for name, a, e in zip(NAMES, got, want):
        assert (a is None) == (e is None), name
        if a is not None:
            assert torch.equal(a, e), f"{name}: differs from fla_chunk_kda_fwd (B={B} T={T} keep={keep})"


def test_two_calls_in_a_row_second_smaller(dev):
    # first: w, u, qg, kg live in the array (2*300*4 rows x 1 KiB) next to the decay rows
    run_pair(dev, 2, 300, 2, 4, 128, 128, seed=1, keep=False)
    # second, smaller, with different data: stale contents of the first call must not show
    run_pair(dev, 1, 100, 2, 2, 128, 128, seed=2, keep=False)
    # the caller keeps the intermediates: only the decay rows use the array
    run_pair(dev, 1, 70, 1, 2, 64, 128, seed=3, keep=True)
    run_pair(dev, 1, 130, 2, 2, 128, 128, seed=4, keep=False, dtype=torch.float16)


def test_limits_are_reported_not_launched(dev):
    from fla_hip import ops

    # 40,000 token-heads x 1 KiB of intermediates > 32 MiB
    q, k, v, g, beta, h0 = make(1, 10000, 4, 4, 128, 128, 5, dev)
    with pytest.raises(RuntimeError, match="bytes of scratch"):
        ops.chunk_kda_fwd_noalloc(q, k, v, g, beta, 128 ** -0.5, 64, layout="BSND")
    # the same call fits once the caller owns the intermediates, and still equals the workspace entry point
    kw = dict(layout="BSND", initial_state=h0, output_final_state=True, disable_recompute=True)
    want = ops.chunk_kda_fwd(q, k, v, g, beta, 128 ** -0.5, 64, **kw)
    got = ops.chunk_kda_fwd_noalloc(q, k, v, g, beta, 128 ** -0.5, 64, **kw)
    torch.cuda.synchronize()
    for name, a, e in zip(NAMES, got, want):
        if a is not None:
            assert torch.equal(a, e), name


def test_packed_batches_are_rejected(dev):
    import ctypes

    from fla_hip.ops import _hip_ctypes as raw, _runtime

    q, k, v, g, beta, _ = make(1, 128, 1, 1, 128, 128, 6, dev)
    o = torch.empty_like(v)
    aqk = torch.empty(1, 1, 128, 64, dtype=BF, device=dev)
    akk = torch.empty_like(aqk)

    def build(ctx):
        none = ctx.tensor(None)
        return [ctx.tensor(q), ctx.tensor(k), ctx.tensor(v), ctx.tensor(g), ctx.tensor(beta), none, none, none,
                ctx.int_array((0, 64, 128)), ctx.int_array(None), ctypes.c_char_p(b"BSND"), ctypes.c_double(0.1),
                ctypes.c_int64(64), ctypes.c_bool(False), ctypes.c_double(-5.0), ctypes.c_bool(False), ctypes.c_bool(False),
                ctx.tensor(o), none, none, ctx.tensor(aqk), ctx.tensor(akk), none, none, none, none, none, none]

    with pytest.raises(RuntimeError, match="cu_seqlens"):
        _runtime.call_op_noalloc("chunk_kda_fwd_noalloc", raw.OP_ARGTYPES["chunk_kda_fwd"], build, o)


def test_capture_and_replay(dev):
    """The entry point under stream capture, which is what it is for: the scratch address is resolved ahead of the
    capture (fla_chunk_kda_fwd_noalloc_init), one call is captured and the graph replayed with new contents in the same
    input buffers, the program's own eager launches and synchronisations in between; every replay must equal the eager
    result of fla_chunk_kda_fwd on the same inputs bit for bit."""
    import fla_hip
    from fla_hip import ops

    assert fla_hip.load_library().fla_chunk_kda_fwd_noalloc_init() == 0
    B, T, Hk, Hv, K, V = 1, 200, 2, 2, 128, 128
    static = make(B, T, Hk, Hv, K, V, 11, dev)
    kw = dict(layout="BSND", output_final_state=True)
    run = lambda: ops.chunk_kda_fwd_noalloc(*static[:5], K ** -0.5, 64, initial_state=static[5], **kw)[:2]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_static, f_static = run()
    for trial in range(3):
        fresh = make(B, T, Hk, Hv, K, V, 20 + trial, dev)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        want_o, want_f = ops.chunk_kda_fwd(*fresh[:5], K ** -0.5, 64, initial_state=fresh[5], **kw)[:2]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o_static, want_o) and torch.equal(f_static, want_f), f"replay {trial}"
