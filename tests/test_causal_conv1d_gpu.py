"""Parity of the HIP causal_conv1d (through the C ABI) against the CPU oracle.

Cases follow torch_custom/fla_npu/test/test_npu_causal_conv1d.py: the deterministic
arange/128 known-answer inputs (:154-161, :208-211), batch / packed prefill, head-split
output, initial states, and the benchmark shape."""
import pytest
import torch

from oracle import conv1d as oc
from util import assert_close, TOL_BF16

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
