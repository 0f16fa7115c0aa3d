"""Parity of the HIP causal_conv1d (through the C ABI) against the CPU oracle.

Cases follow torch_custom/fla_npu/test/test_npu_causal_conv1d.py: the deterministic
arange/128 known-answer inputs (:154-161, :208-211), batch / packed prefill, head-split
output, initial states, and the benchmark shape."""
import pytest
import torch

from oracle import conv1d as oc
from util import assert_close, err_stats, TOL_BF16

pytestmark = pytest.mark.gpu


def make_tensor(shape, *, dtype=torch.float16, start=1.0):
    numel = 1
    for d in shape:
        numel *= d
    return (torch.arange(start, start + numel, dtype=torch.float32).reshape(shape) / 128.0).to(dtype)


def run_case(dev, x, w, b, cs, **kw):
    from fla_hip import ops

    y_ref, cs_ref = oc.causal_conv1d(x, w, b, cs, **kw)
    cs_d = None if cs is None else cs.to(dev)
    y = ops.causal_conv1d(x.to(dev), w.to(dev), None if b is None else b.to(dev), cs_d, **kw)
    return y, y_ref, cs_d, cs_ref


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kat_batch_prefill(dev, dtype):
    x = make_tensor((2, 4, 16), dtype=dtype, start=1.0)
    w = make_tensor((4, 16), dtype=dtype, start=101.0)
    b = make_tensor((16,), dtype=dtype, start=201.0)
    cs = make_tensor((2, 3, 16), dtype=dtype, start=301.0)
    y, y_ref, cs_d, cs_ref = run_case(dev, x, w, b, cs, activation_mode=1)
    # same tolerances as the reference test (:246-253)
    assert torch.allclose(y.float().cpu(), y_ref.float(), rtol=1e-1, atol=2e-1)
    assert torch.equal(cs_d.cpu(), cs_ref)


def test_kat_head_split(dev):
    x = make_tensor((2, 4, 32), start=1.0)
    w = make_tensor((4, 32), start=101.0)
    b = make_tensor((32,), start=201.0)
    cs = make_tensor((2, 3, 32), start=301.0)
    y, y_ref, cs_d, cs_ref = run_case(dev, x, w, b, cs, activation_mode=1, head_num=2)
    assert y.shape == (2, 2, 4, 16)
    assert torch.allclose(y.float().cpu(), y_ref.float(), rtol=1e-1, atol=2e-1)
    assert torch.equal(cs_d.cpu(), cs_ref)


@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("S", [1, 2, 3, 31, 32, 33, 257])
def test_random_dense(dev, W, act, S):
    g = torch.Generator().manual_seed(S * 10 + W)
    D = 48
    x = torch.randn(3, S, D, generator=g).bfloat16()
    w = (torch.randn(W, D, generator=g) * 0.3).bfloat16()
    b = (torch.randn(D, generator=g) * 0.1).bfloat16()
    cs = torch.randn(3, W - 1, D, generator=g).bfloat16()
    y, y_ref, cs_d, cs_ref = run_case(dev, x, w, b, cs, activation_mode=act, initial_state_mode=[1, 0, 1])
    assert_close(y, y_ref, TOL_BF16, "y")
    assert torch.equal(cs_d.cpu(), cs_ref)


def test_packed_varlen_with_cache_and_pad(dev):
    g = torch.Generator().manual_seed(7)
    D, W = 64, 4
    lens = [5, 0, 1, 70, 2, 33]
    qsl = [0]
    for n in lens:
        qsl.append(qsl[-1] + n)
    T = qsl[-1]
    x = torch.randn(T, D, generator=g).bfloat16()
    w = (torch.randn(W, D, generator=g) * 0.3).bfloat16()
    cs = torch.randn(8, W - 1, D, generator=g).bfloat16()
    cache = [3, 1, 0, 7, -1, 5]
    init = [1, 1, 0, 1, 1, 0]
    kw = dict(query_start_loc=qsl, cache_indices=cache, initial_state_mode=init, activation_mode=1, pad_slot_id=-1)
    from fla_hip import ops
    y_ref, cs_ref = oc.causal_conv1d(x, w, None, cs, **kw)
    cs_d = cs.to(dev)
    y = torch.zeros(T, D, dtype=torch.bfloat16, device=dev)
    y_new = ops.causal_conv1d(x.to(dev), w.to(dev), None, cs_d, **kw)
    # tokens of the padded sequence are not written by the op: compare the rest
    keep = torch.ones(T, dtype=torch.bool)
    keep[qsl[4]:qsl[5]] = False
    assert_close(y_new[keep.to(dev)], y_ref[keep], TOL_BF16, "y")
    assert torch.equal(cs_d.cpu(), cs_ref)


def test_strided_input_and_state_pool(dev):
    g = torch.Generator().manual_seed(11)
    B, S, D, W = 2, 50, 32, 4
    big = torch.randn(B, S, 2 * D, generator=g).bfloat16()
    x = big[:, :, :D]                       # row stride 2D
    w = (torch.randn(W, D, generator=g) * 0.3).bfloat16()
    pool = torch.randn(B, 5, D, generator=g).bfloat16()
    cs = pool[:, :W - 1]                    # slot stride 5*D
    from fla_hip import ops
    y_ref, cs_ref = oc.causal_conv1d(x, w, None, cs.clone())
    big_d, pool_d = big.to(dev), pool.to(dev)
    y = ops.causal_conv1d(big_d[:, :, :D], w.to(dev), None, pool_d[:, :W - 1])
    assert_close(y, y_ref, TOL_BF16, "y")
    assert torch.equal(pool_d[:, :W - 1].cpu(), cs_ref)
    assert torch.equal(pool_d[:, W - 1:].cpu(), pool[:, W - 1:])   # rows beyond W-1 untouched


def test_benchmark_shape(dev):
    """B=4, T=4096, D=4096, W=4 + SiLU: oracle on a channel slice, linearity over the rest."""
    from fla_hip import ops
    g = torch.Generator().manual_seed(0)
    B, T, D, W = 4, 4096, 4096, 4
    x = torch.randn(B, T, D, generator=g).bfloat16()
    w = (torch.randn(W, D, generator=g) * 0.1).bfloat16()
    b = (torch.randn(D, generator=g) * 0.01).bfloat16()
    y = ops.causal_conv1d(x.to(dev), w.to(dev), b.to(dev), activation_mode=1).cpu()
    sl = slice(1024, 1024 + 128)
    y_ref, _ = oc.causal_conv1d(x[:, :, sl].contiguous(), w[:, sl].contiguous(), b[sl].contiguous(),
                                activation_mode=1)
    assert_close(y[:, :, sl], y_ref, TOL_BF16, "y slice")
    # shift equivariance away from the left edge (size-independent property)
    y2 = ops.causal_conv1d(x[:, 100:].contiguous().to(dev), w.to(dev), b.to(dev), activation_mode=1).cpu()
    assert torch.equal(y2[:, 3:], y[:, 103:])


def test_errors(dev):
    from fla_hip import ops
    x = torch.zeros(1, 4, 16, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(5, 16, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="width must be 2, 3 or 4"):
        ops.causal_conv1d(x, w)
    with pytest.raises(RuntimeError, match="run_mode"):
        ops.causal_conv1d(x, w[:4], run_mode=1)
    cs = torch.zeros(1, 3, 16, dtype=torch.bfloat16, device=dev, requires_grad=False)
    cs.requires_grad_(True)
    with pytest.raises(RuntimeError, match="mutates conv_states"):
        ops.causal_conv1d(x, w[:4], None, cs)


# ---------------------------------------------------------------------------------------------
# state-update mode (run_mode=1): the reference's update / speculative-decode cases
# (test_npu_causal_conv1d.py:386-520) and random sweeps against the oracle
# ---------------------------------------------------------------------------------------------
def run_update(dev, x, w, b, cs, **kw):
    from fla_hip import ops

    y_ref, cs_ref = oc.causal_conv1d_update(x, w, b, cs, **kw)
    cs_d = cs.to(dev)
    y = ops.causal_conv1d(x.to(dev), w.to(dev), None if b is None else b.to(dev), cs_d, run_mode=1, **kw)
    return y, y_ref, cs_d, cs_ref


def test_kat_update_one_token(dev):
    x = make_tensor((2, 16), start=1.0)
    w, b = make_tensor((4, 16), start=101.0), make_tensor((16,), start=201.0)
    cs = make_tensor((2, 3, 16), start=301.0)
    y, y_ref, cs_d, cs_ref = run_update(dev, x, w, b, cs, cache_indices=[0, 1], activation_mode=1)
    assert torch.allclose(y.float().cpu(), y_ref.float(), rtol=5e-2, atol=5e-2)      # the reference's tolerance (:186-187)
    assert torch.equal(cs_d.cpu(), cs_ref)


def test_kat_speculative_decode(dev):
    x = make_tensor((2, 4, 16), start=1.0)
    w, b = make_tensor((4, 16), start=101.0), make_tensor((16,), start=201.0)
    cs = make_tensor((2, 6, 16), start=301.0)
    y, y_ref, cs_d, cs_ref = run_update(dev, x, w, b, cs, cache_indices=[0, 1], num_accepted_tokens=[2, 4])
    assert torch.allclose(y.float().cpu(), y_ref.float(), rtol=5e-2, atol=5e-2)
    assert torch.equal(cs_d.cpu(), cs_ref)


def test_kat_update_width3_and_padded_batch(dev):
    x = make_tensor((3, 3, 16), start=1.0)
    w = make_tensor((3, 16), start=101.0)
    cs = make_tensor((3, 2, 16), start=301.0)
    y, y_ref, cs_d, cs_ref = run_update(dev, x, w, None, cs, cache_indices=[0, 1, 2])
    assert torch.allclose(y.float().cpu(), y_ref.float(), rtol=5e-2, atol=5e-2)
    assert torch.equal(cs_d.cpu(), cs_ref)
    # batch gather with padded rows: valid rows match, padded rows and untouched slots stay as they were
    x = make_tensor((5, 3, 16), start=1.0)
    w, b = make_tensor((4, 16), start=101.0), make_tensor((16,), start=201.0)
    cs = make_tensor((7, 3, 16), start=301.0)
    from fla_hip import ops
    cs_d = cs.to(dev)
    y = torch.full((5, 3, 16), 7.0, dtype=x.dtype, device=dev)
    y_ref, cs_ref = oc.causal_conv1d_update(x, w, b, cs, cache_indices=[1, 3, 5, -1, -1], activation_mode=1)
    y = ops.causal_conv1d(x.to(dev), w.to(dev), b.to(dev), cs_d, cache_indices=[1, 3, 5, -1, -1], activation_mode=1, run_mode=1)
    assert torch.allclose(y[:3].float().cpu(), y_ref[:3].float(), rtol=5e-2, atol=5e-2)
    assert torch.equal(cs_d.cpu(), cs_ref)


@pytest.mark.parametrize("W", [2, 3, 4])
@pytest.mark.parametrize("S", [1, 2, 5])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_random_update(dev, W, S, dtype):
    gen = torch.Generator().manual_seed(100 * W + S)
    B, D, slots = 9, 192, 12
    x = torch.randn(B, S, D, generator=gen).to(dtype)
    w = (torch.randn(W, D, generator=gen) * 0.3).to(dtype)
    b = (torch.randn(D, generator=gen) * 0.1).to(dtype)
    cs = torch.randn(slots, W - 1 + 2, D, generator=gen).to(dtype)          # longer than needed: only rows 0..W-2 take part
    cache = torch.randperm(slots, generator=gen)[:B].tolist()
    cache[4] = -1
    y, y_ref, cs_d, cs_ref = run_update(dev, x, w, b, cs, cache_indices=cache, activation_mode=1)
    keep = [i for i in range(B) if cache[i] != -1]
    assert_close(y[keep], y_ref[keep], TOL_BF16, "y")
    assert torch.equal(cs_d.cpu(), cs_ref)
    if S == 1:      # the 2-D one-token form gives the same rows
        y2, _, cs2, _ = run_update(dev, x[:, 0], w, b, cs, cache_indices=cache, activation_mode=1)
        assert torch.equal(y2[keep].cpu(), y[keep][:, 0].cpu()) and torch.equal(cs2.cpu(), cs_d.cpu())


def test_speculative_decode_loop_and_packed_update(dev):
    """A draft/accept loop on the GPU tracks the oracle step by step (outputs and the whole state pool), and the
    packed 2-D varlen form equals the per-sequence results."""
    from fla_hip import ops
    gen = torch.Generator().manual_seed(5)
    W, D, S, B = 4, 256, 4, 3
    w = (torch.randn(W, D, generator=gen) * 0.3).bfloat16()
    cs = torch.zeros(5, (W - 1) + (S - 1), D).bfloat16()
    cs_d = cs.to(dev)
    cache = [3, 0, 4]
    nat = [1, 1, 1]
    for step in range(5):
        x = torch.randn(B, S, D, generator=gen).bfloat16()
        y_ref, cs = oc.causal_conv1d_update(x, w, None, cs, cache_indices=cache, num_accepted_tokens=nat)
        y = ops.causal_conv1d(x.to(dev), w.to(dev), None, cs_d, cache_indices=cache, num_accepted_tokens=nat, run_mode=1)
        assert_close(y, y_ref, TOL_BF16, f"step {step}")
        assert torch.equal(cs_d.cpu(), cs)
        nat = [int(v) for v in torch.randint(1, S + 1, (B,), generator=gen)]
    # packed tokens with query_start_loc (segments of different length, one of them padded out)
    qsl = [0, 3, 4, 9]
    x = torch.randn(9, D, generator=gen).bfloat16()
    cs0 = torch.randn(4, 3, D, generator=gen).bfloat16()
    y_ref, cs_ref = oc.causal_conv1d_update(x, w, None, cs0, query_start_loc=qsl, cache_indices=[2, -1, 0])
    cs_d = cs0.to(dev)
    y = ops.causal_conv1d(x.to(dev), w.to(dev), None, cs_d, query_start_loc=qsl, cache_indices=[2, -1, 0], run_mode=1)
    rows = [0, 1, 2, 4, 5, 6, 7, 8]
    assert_close(y[rows], y_ref[rows], TOL_BF16, "packed")
    assert torch.equal(cs_d.cpu(), cs_ref)


def test_update_mode_errors(dev):
    from fla_hip import ops
    x = torch.zeros(2, 4, 16, dtype=torch.bfloat16, device=dev)
    w4, w3 = torch.zeros(4, 16, dtype=torch.bfloat16, device=dev), torch.zeros(3, 16, dtype=torch.bfloat16, device=dev)
    cs = torch.zeros(2, 6, 16, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="needs conv_states"):
        ops.causal_conv1d(x, w4, run_mode=1)
    with pytest.raises(RuntimeError, match="only supported for width 4"):
        ops.causal_conv1d(x, w3, None, cs, num_accepted_tokens=[1, 1], run_mode=1)
    with pytest.raises(RuntimeError, match="state_len >="):
        ops.causal_conv1d(x, w4, None, cs[:, :4], num_accepted_tokens=[1, 1], run_mode=1)
    with pytest.raises(RuntimeError, match=r"must lie in \[0, 4\]"):
        ops.causal_conv1d(x, w4, None, cs, num_accepted_tokens=[1, 5], run_mode=1)
    with pytest.raises(RuntimeError, match="initial_state_mode is only supported in run_mode=0"):
        ops.causal_conv1d(x, w4, None, cs, initial_state_mode=[1, 1], run_mode=1)
    with pytest.raises(RuntimeError, match="head_num must be 0"):
        ops.causal_conv1d(x, w4, None, cs, run_mode=1, head_num=2)


# ---------------------------------------------------------------------------------------------
# backward (test_npu_causal_conv1d_bwd.py: fixed BSH with every activation, BNSD, packed TND / NTD)
# ---------------------------------------------------------------------------------------------
def bwd_tensor(shape, *, dtype=torch.bfloat16, offset=0):       # the reference's deterministic inputs (:23-29)
    numel = 1
    for d in shape:
        numel *= d
    values = torch.arange(offset, offset + numel, dtype=torch.float32)
    return ((values.remainder(37) - 18.0) / 64.0).reshape(shape).to(dtype)


def preactivation(x, w, h0, qsl=None):
    """fp32 forward pre-activation in the logical layout (the forward oracle with the state's rows 1..W-1)."""
    W = w.shape[0]
    cs = None if h0 is None else h0[:, 1:].contiguous()
    N = (len(qsl) - 1) if qsl is not None else x.shape[0]
    y, _ = oc.causal_conv1d(x.float(), w.float(), None, cs if cs is None else cs.float(), query_start_loc=qsl,
                            initial_state_mode=None if cs is None else [1] * N)
    return y


def check_bwd(dev, x, w, dy, h0, dht, *, qsl=None, activation=0, layout="BSND", heads=1, tol=TOL_BF16):
    from fla_hip import ops
    y = preactivation(x, w, h0, qsl).to(x.dtype) if activation else None
    ref = oc.causal_conv1d_bwd(x, y, w, dy, h0, dht, query_start_loc=qsl, activation=activation)

    def phys(t):        # logical -> physical layout of y / dy
        if t is None or layout in ("BSND", "BSH", "TND"):
            return t
        if layout == "BNSD":
            B, T, D = t.shape
            return t.reshape(B, T, heads, D // heads).permute(0, 2, 1, 3).contiguous()
        T, D = t.shape
        return t.reshape(T, heads, D // heads).permute(1, 0, 2).contiguous()

    d = lambda t: None if t is None else t.to(dev)
    got = ops.causal_conv1d_bwd(d(x), d(phys(y)), d(w), d(phys(dy)), d(h0), d(dht), query_start_loc=qsl, activation=activation,
                                input_layout=layout)
    for name, a, e in zip(("dx", "dw", "db", "dh0"), got, ref):
        assert a.shape == e.shape and a.dtype == e.dtype, name
        st = err_stats(a, e)
        assert st["rel_max"] <= tol, f"{name} ({layout}, act={activation}): {st}"
    return got


@pytest.mark.parametrize("activation", [0, 1, 2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_bwd_kat_fixed_bsh(dev, activation, dtype):
    B, T, D, W = 2, 9, 32, 4
    x, w = bwd_tensor((B, T, D), dtype=dtype, offset=3), bwd_tensor((W, D), dtype=dtype, offset=11)
    dy = bwd_tensor((B, T, D), dtype=dtype, offset=23)
    h0, dht = bwd_tensor((B, W, D), dtype=dtype, offset=31), bwd_tensor((B, W, D), dtype=dtype, offset=41)
    got = check_bwd(dev, x, w, dy, h0, dht, activation=activation, layout="BSH")
    assert float(got[3][:, 0].abs().max()) == 0.0


def test_bwd_bnsd_and_packed_layouts(dev):
    gen = torch.Generator().manual_seed(17)
    B, T, D, H = 2, 70, 64, 2
    for W in (2, 3, 4):
        x = torch.randn(B, T, D, generator=gen).bfloat16()
        w = (torch.randn(W, D, generator=gen) * 0.3).bfloat16()
        dy = torch.randn(B, T, D, generator=gen).bfloat16()
        h0, dht = torch.randn(B, W, D, generator=gen).bfloat16(), torch.randn(B, W, D, generator=gen).bfloat16()
        check_bwd(dev, x, w, dy, h0, dht, activation=1, layout="BNSD", heads=H)
        check_bwd(dev, x, w, dy, None, None, activation=0, layout="BSND")
        qsl = [0, 1, 3, 3, 40, 41, 140]            # lengths 1, 2, 0, 37, 1, 99: shorter than the kernel, empty, across tiles
        xp, dyp = x.reshape(B * T, D), dy.reshape(B * T, D)
        N = len(qsl) - 1
        h0p, dhtp = torch.randn(N, W, D, generator=gen).bfloat16(), torch.randn(N, W, D, generator=gen).bfloat16()
        check_bwd(dev, xp, w, dyp, h0p, dhtp, qsl=qsl, activation=1, layout="TND")
        check_bwd(dev, xp, w, dyp, h0p, None, qsl=qsl, activation=2, layout="NTD", heads=H)


def test_bwd_benchmark_shape_and_autograd_binding(dev):
    """The conv1d benchmark shape: the reductions over 16384 tokens stay within tolerance, and loss.backward()
    through ops.causal_conv1d reaches the same gradients."""
    from fla_hip import ops
    gen = torch.Generator().manual_seed(2)
    B, T, D, W = 4, 4096, 4096, 4
    x = torch.randn(B, T, D, generator=gen).bfloat16()
    w = (torch.randn(W, D, generator=gen) * 0.1).bfloat16()
    b = (torch.randn(D, generator=gen) * 0.01).bfloat16()
    dy = torch.randn(B, T, D, generator=gen).bfloat16()
    xd, wd, bd = (t.to(dev).requires_grad_(True) for t in (x, w, b))
    y = ops.causal_conv1d(xd, wd, bd)
    (y.float() * dy.to(dev).float()).sum().backward()
    # fp32 reference on the GPU with torch ops (the CPU oracle's token loop is too slow at this size)
    xf, wf, dyf = x.to(dev).float(), w.to(dev).float(), dy.to(dev).float()
    dx_ref = torch.zeros_like(xf)
    dw_ref = torch.zeros(W, D, device=dev)
    for j in range(W):
        tap = W - 1 - j
        dx_ref[:, :T - j] += dyf[:, j:] * wf[tap]
        dw_ref[tap] = (dyf[:, j:] * xf[:, :T - j]).sum((0, 1))
    assert err_stats(xd.grad, dx_ref)["rel_max"] <= TOL_BF16
    assert err_stats(wd.grad, dw_ref)["rel_max"] <= TOL_BF16
    assert err_stats(bd.grad, dyf.sum((0, 1)))["rel_max"] <= TOL_BF16
    with pytest.raises(NotImplementedError, match="gradients are bound only"):
        ops.causal_conv1d(xd, wd, bd, activation_mode=1)


def test_bwd_errors(dev):
    from fla_hip import ops
    x = torch.zeros(2, 8, 32, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(4, 32, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="y is required"):
        ops.causal_conv1d_bwd(x, None, w, x, activation=1)
    with pytest.raises(RuntimeError, match="query_start_loc is required"):
        ops.causal_conv1d_bwd(x[0], None, w, x[0], input_layout="TND")
    with pytest.raises(RuntimeError, match="input_layout must be"):
        ops.causal_conv1d_bwd(x, None, w, x, input_layout="SBH")
    with pytest.raises(RuntimeError, match=r"must be \[N=2, W, D\]"):
        ops.causal_conv1d_bwd(x, None, w, x, torch.zeros(2, 3, 32, dtype=torch.bfloat16, device=dev))
