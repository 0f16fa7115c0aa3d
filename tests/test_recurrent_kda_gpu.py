"""Parity of recurrent_kda (through the C ABI) against the CPU oracle on the reference's case matrix
(kda/recurrent_kda/docs/design.md:168-186): BSND raw gate with beta sigmoid, safe gate with allow_neg_eigval, TND
precomputed gate without an initial state, grouped value heads, K=128/V=256, uneven and empty sequences, 2-D slot
rows with a capacity pool, speculative decoding, strided state views, both state layouts and dtypes, in-place and
separate final states.  Tolerances: the reference's rtol 0.02 / atol 0.01 for bf16 outputs, 1e-3 for fp32 states."""
import pytest
import torch

from oracle import kda
from util import assert_close, err_stats, TOL_STATE

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def close_out(a, e, name="out"):
    a, e = a.float().cpu(), e.float()
    assert torch.allclose(a, e, rtol=0.02, atol=0.01), f"{name}: {err_stats(a, e)}"


def make(T_shape, H, HV, K, V, seed, raw_gate=False):
    gen = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen)
    q, k = rn(*T_shape, H, K).to(BF), rn(*T_shape, H, K).to(BF)
    v = rn(*T_shape, HV, V).to(BF)
    g = rn(*T_shape, HV, K) if raw_gate else -torch.rand(*T_shape, HV, K, generator=gen) * 0.5
    beta = rn(*T_shape, HV) if raw_gate else torch.rand(*T_shape, HV, generator=gen)
    return q, k, v, g, beta, gen


def dev_all(dev, *ts):
    return [None if t is None else t.to(dev) for t in ts]


@pytest.mark.parametrize("safe", [False, True])
@pytest.mark.parametrize("v_first", [True, False])
def test_bsnd_raw_gate_options(dev, safe, v_first):
    from fla_hip import ops
    B, T, H, HV, K, V = 2, 2, 2, 4, 128, 128
    q, k, v, g, beta, gen = make((B, T), H, HV, K, V, 1 + safe, raw_gate=True)
    A_log, dt = torch.randn(HV, generator=gen) * 0.3, torch.randn(HV, K, generator=gen) * 0.1
    tail = (V, K) if v_first else (K, V)
    state = torch.randn(B, HV, *tail, generator=gen) * 0.1
    cu = torch.arange(B + 1, dtype=torch.int32) * T
    kw = dict(A_log=A_log, dt_bias=dt, use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True,
              allow_neg_eigval=safe, safe_gate=safe, lower_bound=-4.0 if safe else None, state_v_first=v_first)
    okw = dict(kw, lower_bound=-4.0 if safe else -5.0)
    o_ref, pool_ref = kda.recurrent_kda(q, k, v, g, beta, state, cu_seqlens=cu, **okw)
    qd, kd, vd, gd, bd, sd, cud, Ad, dtd = dev_all(dev, q, k, v, g, beta, state, cu, A_log, dt)
    out, final = ops.recurrent_kda(qd, kd, vd, gd, bd, sd, cu_seqlens=cud, output_final_state=True, A_log=Ad, dt_bias=dtd,
                                   **{n: x for n, x in kw.items() if n not in ("A_log", "dt_bias")})
    close_out(out, o_ref)
    assert final.data_ptr() == sd.data_ptr()                       # in place
    assert_close(final, pool_ref, TOL_STATE, "state")


@pytest.mark.parametrize("V", [128, 256])
def test_tnd_precomputed_gate_without_initial_state(dev, V):
    from fla_hip import ops
    T, H, HV, K = 6, 2, 2, 128
    q, k, v, g, beta, gen = make((T,), H, HV, K, V, 3)
    cu = torch.tensor([0, 2, 6], dtype=torch.int64)
    zero = torch.zeros(2, HV, K, V)
    o_ref, pool_ref = kda.recurrent_kda(q, k, v, g, beta, zero, cu_seqlens=cu, layout="TND")
    out, final = ops.recurrent_kda(*dev_all(dev, q, k, v, g.to(BF), beta.to(torch.float16)), None, cu_seqlens=cu.to(dev),
                                   layout="TND", output_final_state=True, inplace_final_state=False)
    o_ref2, pool_ref2 = kda.recurrent_kda(q, k, v, g.to(BF).float(), beta.to(torch.float16).float(), zero, cu_seqlens=cu, layout="TND")
    close_out(out, o_ref2)
    assert_close(final, pool_ref2, TOL_STATE, "state")
    with pytest.raises(RuntimeError, match="inplace_final_state=True requires initial_state"):
        ops.recurrent_kda(*dev_all(dev, q, k, v, g, beta), None, cu_seqlens=cu.to(dev), layout="TND")


@pytest.mark.parametrize("state_dtype", [torch.float32, BF])
@pytest.mark.parametrize("v_first", [True, False])
def test_uneven_and_empty_sequences_slot_rows_and_strided_pool(dev, state_dtype, v_first):
    """cu [0,1,1,4,4,8] with 2-D slot rows into a pool of larger capacity that is a strided view (every other slot of
    a bigger allocation): hit slots match, all other memory is untouched, in place and with a separate output."""
    from fla_hip import ops
    H, HV, K, V = 3, 6, 128, 128
    cu = torch.tensor([0, 1, 1, 4, 4, 8], dtype=torch.int32)
    T, N, cap = 8, 5, 20
    q, k, v, g, beta, gen = make((T,), H, HV, K, V, 5)
    tail = (V, K) if v_first else (K, V)
    big = (torch.randn(2 * cap, HV, *tail, generator=gen) * 0.1).to(state_dtype)
    rows = torch.tensor([[3, 0, 0, 0], [9, 9, 9, 9], [17, 5, 11, 0], [2, 2, 2, 2], [7, 7, 12, 13]], dtype=torch.int64)
    pool_view = big[::2]
    o_ref, pool_ref = kda.recurrent_kda(q, k, v, g, beta, pool_view.float(), cu_seqlens=cu, ssm_state_indices=rows, layout="TND",
                                        state_v_first=v_first)
    for inplace in (True, False):
        big_d = big.to(dev)
        out, final = ops.recurrent_kda(*dev_all(dev, q, k, v, g, beta), big_d[::2], cu_seqlens=cu.to(dev),
                                       ssm_state_indices=rows.to(dev), layout="TND", output_final_state=True,
                                       inplace_final_state=inplace, state_v_first=v_first)
        close_out(out, o_ref)
        tol = TOL_STATE if state_dtype == torch.float32 else 2e-2
        hit = [3, 17, 5, 11, 7, 12, 13]
        assert_close(final[hit], pool_ref[hit], tol, "hit slots")
        miss = [i for i in range(cap) if i not in hit]
        assert torch.equal(final[miss].cpu(), pool_view[miss])
        if inplace:
            assert torch.equal(big_d[1::2].cpu(), big[1::2])       # the gaps of the strided view
        else:
            assert torch.equal(big_d.cpu(), big)                   # the input pool is unchanged


def test_speculative_decoding_loop(dev):
    """Draft / accept loop on the GPU against the oracle, call by call (outputs and the whole pool)."""
    from fla_hip import ops
    H, HV, K, V, S, N = 2, 4, 128, 128, 4, 3
    gen = torch.Generator().manual_seed(9)
    rows = torch.tensor([[0, 1, 2, 3], [8, 9, 10, 11], [4, 5, 6, 7]], dtype=torch.int32)
    pool = torch.zeros(12, HV, V, K)
    pool_d = pool.to(dev)
    accepted = torch.ones(N, dtype=torch.int32)
    for step in range(4):
        q, k, v, g, beta, _ = make((N, S), H, HV, K, V, 20 + step)
        o_ref, pool = kda.recurrent_kda(q, k, v, g, beta, pool, ssm_state_indices=rows, num_accepted_tokens=accepted,
                                        state_v_first=True, use_qk_l2norm_in_kernel=True)
        out, _ = ops.recurrent_kda(*dev_all(dev, q, k, v, g, beta), pool_d, ssm_state_indices=rows.to(dev),
                                   num_accepted_tokens=accepted.to(dev), state_v_first=True, use_qk_l2norm_in_kernel=True)
        close_out(out, o_ref, f"step {step}")
        assert_close(pool_d, pool, TOL_STATE, f"pool after step {step}")
        accepted = torch.randint(1, S + 1, (N,), generator=gen, dtype=torch.int32)


def test_long_sequence_and_packed_slots(dev):
    """Sequences longer than the staging batch (the reference stops at 8 tokens; this kernel does not) with packed
    per-token slots."""
    from fla_hip import ops
    H, HV, K, V = 1, 2, 128, 128
    cu = torch.tensor([0, 19, 30], dtype=torch.int32)
    T = 30
    q, k, v, g, beta, gen = make((T,), H, HV, K, V, 11)
    slots = torch.cat([torch.full((19,), 2), torch.full((11,), 0)]).to(torch.int32)
    slots[5] = 1                                                    # one detour: token 5 lands in slot 1
    pool = torch.randn(3, HV, K, V, generator=gen) * 0.1
    o_ref, pool_ref = kda.recurrent_kda(q, k, v, g, beta, pool, cu_seqlens=cu, ssm_state_indices=slots, layout="TND",
                                        use_qk_l2norm_in_kernel=True)
    pool_d = pool.to(dev)
    out, _ = ops.recurrent_kda(*dev_all(dev, q, k, v, g, beta), pool_d, cu_seqlens=cu.to(dev), ssm_state_indices=slots.to(dev),
                               layout="TND", use_qk_l2norm_in_kernel=True)
    close_out(out, o_ref)
    assert_close(pool_d, pool_ref, TOL_STATE, "pool")


def test_invalid_metadata_leaves_everything_untouched_and_errors(dev):
    from fla_hip import ops
    H, HV, K, V, T = 1, 1, 128, 128, 4
    q, k, v, g, beta, gen = make((T,), H, HV, K, V, 13)
    pool = torch.randn(2, HV, K, V, generator=gen)
    pool_d = pool.to(dev)
    args = dev_all(dev, q, k, v, g, beta)
    out = torch.full((T, HV, V), 3.0, dtype=BF, device=dev)
    # slot out of range for sequence 1: that sequence is skipped, sequence 0 is processed
    cu = torch.tensor([0, 2, 4], dtype=torch.int32)
    slots = torch.tensor([0, 0, 5, 5], dtype=torch.int32)
    o, _ = ops.recurrent_kda(*args, pool_d, cu_seqlens=cu.to(dev), ssm_state_indices=slots.to(dev), layout="TND")
    o_ref, pool_ref = kda.recurrent_kda(q[:2], k[:2], v[:2], g[:2], beta[:2], pool[:1], cu_seqlens=[0, 2], layout="TND")
    close_out(o[:2], o_ref)
    assert_close(pool_d[:1], pool_ref, TOL_STATE, "slot 0")
    assert torch.equal(pool_d[1:].cpu(), pool[1:])
    with pytest.raises(RuntimeError, match="layout must be BSND or TND"):
        ops.recurrent_kda(*args, pool_d, layout="BNSD")
    with pytest.raises(RuntimeError, match="state_capacity must equal seq_num"):
        ops.recurrent_kda(*args, pool_d, layout="TND")
    with pytest.raises(RuntimeError, match="num_accepted_tokens requires ssm_state_indices"):
        ops.recurrent_kda(*args, pool_d, cu_seqlens=cu.to(dev), num_accepted_tokens=torch.ones(2, dtype=torch.int32, device=dev), layout="TND")
    with pytest.raises(RuntimeError, match="require use_gate_in_kernel=True"):
        ops.recurrent_kda(*args, pool_d, cu_seqlens=cu.to(dev), safe_gate=True, layout="TND")
    with pytest.raises(RuntimeError, match="K/V currently support only"):
        ops.recurrent_kda(args[0][..., :64], args[1][..., :64], args[2], args[3][..., :64], args[4], pool_d, cu_seqlens=cu.to(dev), layout="TND")
