"""Seeded random shapes through the assertions of the other GPU tests.

The hand-picked case tables of the other files name the edges the reference tests (ragged tails, empty and one-token
sequences, grouped heads, every built head size).  Here a generator draws combinations nobody wrote down - batch, length,
head counts, packing, state options, element types - and hands each to the same checking function as the table cases, so
every drawn case is held to the same oracle and tolerance.  The seeds are fixed: the run is reproducible and its cost
bounded (a few hundred small problems)."""
import random

import pytest
import torch

import test_causal_conv1d_gpu as conv_tests
import test_gdn_bwd_gpu as bwd_tests
import test_gdn_ops_gpu as ops_tests
import test_gdn_pipeline_gpu as pipe_tests
import test_kda_bwd_gpu as kda_bwd_tests
import test_kda_fwd_gpu as kda_fwd_tests
import test_recurrent_gdn_gpu as decode_tests
from util import assert_close, TOL_BF16, TOL_STATE

pytestmark = pytest.mark.gpu
BF, F16 = torch.bfloat16, torch.float16
GDN_SIZES = ((128, 128), (64, 64), (128, 256), (64, 128))


def packed(rng, T):
    """cu_seqlens of 1-6 sequences over T tokens; equal cut points give empty sequences."""
    cuts = sorted(rng.randint(0, T) for _ in range(rng.randint(0, 5)))
    return [0] + cuts + [T]


def gdn_case(rng, tmax=330):
    """(B, T, Hv, Hk, K, V, cu) as the GDN case tables list them."""
    K, V = rng.choice(GDN_SIZES)
    Hk = rng.choice((1, 2, 3))
    Hv = Hk * rng.choice((1, 1, 2, 4))
    T = rng.choice((1, 2, 15, 63, 64, 65, 127, 128, 129, rng.randint(1, tmax), rng.randint(1, tmax)))
    cu = packed(rng, T) if rng.random() < 0.4 else None
    B = 1 if cu is not None else rng.choice((1, 1, 2, 3))
    return (B, T, Hv, Hk, K, V, cu)


def kda_case(rng, grad):
    sizes = ((128, 128), (64, 64), (64, 128), (128, 256), (96, 80), (16, 48), (128, 64), (256, 256), (192, 112), (144, 256))
    K, V = rng.choice(sizes)
    Hk = rng.choice((1, 2))
    c = dict(T=rng.choice((1, 17, 64, 65, 128, 129, 191, rng.randint(1, 300))), Hk=Hk, Hv=Hk * rng.choice((1, 2)), K=K, V=V,
             layout=rng.choice(("BSND", "BNSD", "TND", "NTD")))
    if c["layout"] in ("TND", "NTD"):
        c["B"], c["cu"] = 1, packed(rng, c["T"])
    else:
        c["B"] = rng.choice((1, 2))
    if rng.random() < 0.6:
        c["h0"] = True
    if rng.random() < 0.4:
        c["chunk"] = 128
    if rng.random() < 0.3:
        c["dtype"] = F16
    if grad:
        if rng.random() < 0.6:
            c["dht"] = True
        if c["T"] == 1:      # a single token on a zero state has dg = 0 exactly: nothing to compare a relative error with
            c["h0"] = True
    else:
        if rng.random() < 0.4:
            c["v_first"] = True
        if rng.random() < 0.3 and c.get("dtype") != F16:
            c["gate"] = dict(use_gate_in_kernel=True, bias=rng.random() < 0.5)
            if rng.random() < 0.5:
                c["gate"].update(safe_gate=True, lower_bound=-5.0)
    return c


def kda_stage_case(rng):
    B, T, Hv, Hk, _, _, cu = gdn_case(rng)
    K, V = rng.choice(((128, 128), (64, 64), (64, 128)))
    return (B, T, Hk, Hv, K, V, cu)


@pytest.mark.parametrize("seed", [11, 12])
def test_gdn_forward_routes(dev, seed):
    rng = random.Random(seed)
    for _ in range(20):
        pipe_tests.test_against_naive_recurrence(dev, gdn_case(rng), rng.random() < 0.6, rng.choice((BF, BF, F16)))
        pipe_tests.test_forward_writes_the_operands_of_the_backward(dev, gdn_case(rng), rng.choice((BF, F16)))
        pipe_tests.test_forward_writes_normalised_q_k_and_rstd(dev, gdn_case(rng), rng.choice((BF, F16)), rng.random() < 0.5)
        pipe_tests.test_in_kernel_l2norm_equals_separate_pass(dev, gdn_case(rng), rng.choice((BF, F16)))


@pytest.mark.parametrize("seed", [21, 22])
def test_gdn_forward_operators(dev, seed):
    rng = random.Random(seed)
    for _ in range(25):
        ops_tests.test_stagewise_against_oracle(dev, gdn_case(rng), rng.choice((BF, F16)))
        ops_tests.test_stagewise_chunk_128(dev, gdn_case(rng), rng.choice((BF, F16)))


@pytest.mark.parametrize("seed", [31, 32])
def test_gdn_backward(dev, seed):
    rng = random.Random(seed)
    for _ in range(20):
        bwd_tests.test_backward_operators_against_oracle(dev, gdn_case(rng), rng.choice((BF, F16)))
        # two value passes (V = 256 on 128-token chunks) add parts rounded to 16 bits: short chunks whose parts nearly
        # cancel miss the relative bound of the single-pass kernels, so the draw keeps to the single-pass sizes
        case = gdn_case(rng)
        if case[5] != 256:
            bwd_tests.test_backward_operators_with_128_token_chunks(dev, case)
        bwd_tests.test_backward_pipeline_against_recurrence_autograd(dev, (gdn_case(rng, tmax=200), rng.choice((64, 128))),
                                                                     rng.choice((BF, F16)))


@pytest.mark.parametrize("seed", [41, 42])
def test_kda_forward_and_backward(dev, seed):
    rng = random.Random(seed)
    for _ in range(20):
        kda_fwd_tests.test_chunk_kda_fwd(dev, kda_case(rng, grad=False))
        kda_bwd_tests.test_bwd_dav(dev, kda_stage_case(rng))
        kda_bwd_tests.test_bwd_dqkwg(dev, kda_stage_case(rng))
        kda_bwd_tests.test_bwd_wy(dev, kda_stage_case(rng))
        case = kda_case(rng, grad=True)
        if case.get("cu") is not None and case["T"] > 0 and len(set(case["cu"])) == 1:
            continue
        kda_bwd_tests.test_chunk_kda_backward_against_autograd_through_the_recurrence(dev, case)


@pytest.mark.parametrize("seed", [51, 52])
def test_recurrent_decode(dev, seed):
    """Any head size the reference admits (Dk a multiple of 4, both up to 512, _aclnn_ctypes.py:813-817), skipped
    prefixes, empty sequences, accepted-token source slots, both gates, fp32 and bf16 pools."""
    rng = random.Random(seed)
    for _ in range(40):
        Dk, Dv = rng.choice(GDN_SIZES + ((16, 16), (48, 80), (192, 160), (256, 256), (100, 36), (4 * rng.randint(1, 128), rng.randint(1, 512))))
        Nk = rng.choice((1, 2, 3))
        lens = [rng.choice((0, 1, 1, 1, 2, 3, 8, 9, 17, rng.randint(1, 40))) for _ in range(rng.randint(1, 6))]
        lens[0] = max(lens[0], 1)
        skip = rng.choice((0, 0, 1, 3))
        bf_state = rng.random() < 0.3
        g, gk = rng.choice(((True, False), (True, True), (False, True)))
        d = decode_tests.make_inputs(lens, Nk, Nk * rng.choice((1, 2, 4)), Dk, Dv, seed=rng.randint(0, 10 ** 6), skip=skip,
                                     blocks=skip + sum(lens) + rng.randint(0, 5),
                                     state_dtype=BF if bf_state else torch.float32, g=g, gk=gk)
        acc = torch.tensor([rng.randint(1, max(1, n)) for n in lens], dtype=torch.int32) if rng.random() < 0.4 else None
        o, o_ref, st, s_ref = decode_tests.run(dev, d, accepted=acc)
        what = f"Dk={Dk} Dv={Dv} lens={lens} skip={skip}"
        assert_close(o[skip:], o_ref[skip:], TOL_BF16, "out " + what)
        assert_close(st, s_ref.bfloat16() if bf_state else s_ref, TOL_BF16 if bf_state else TOL_STATE, "state " + what)


@pytest.mark.parametrize("seed", [61, 62])
def test_causal_conv1d(dev, seed):
    """Dense batches and packed sequences with cache slots, padded slots and per-sequence initial-state switches; the
    feature dimension a multiple of 16 as the reference requires (docs/aclnnCausalConv1d.md:62)."""
    from fla_hip import ops
    from oracle import conv1d as oc
    rng = random.Random(seed)
    for _ in range(40):
        W, D, act = rng.choice((2, 3, 4)), 16 * rng.randint(1, 40), rng.choice((0, 1))
        dtype = rng.choice((BF, F16))
        g = torch.Generator().manual_seed(rng.randint(0, 10 ** 6))
        w = (torch.randn(W, D, generator=g) * 0.3).to(dtype)
        if rng.random() < 0.5:
            B, S = rng.randint(1, 4), rng.choice((1, 2, 3, 31, 32, 33, rng.randint(1, 300)))
            x = torch.randn(B, S, D, generator=g).to(dtype)
            b = (torch.randn(D, generator=g) * 0.1).to(dtype) if rng.random() < 0.5 else None
            cs = torch.randn(B, W - 1, D, generator=g).to(dtype)
            y, y_ref, cs_d, cs_ref = conv_tests.run_case(dev, x, w, b, cs, activation_mode=act,
                                                         initial_state_mode=[rng.choice((0, 1)) for _ in range(B)])
            assert_close(y, y_ref, TOL_BF16, f"y W={W} D={D} B={B} S={S}")
            assert torch.equal(cs_d.cpu(), cs_ref)
            continue
        lens = [rng.choice((0, 1, 2, 5, 33, rng.randint(1, 90))) for _ in range(rng.randint(1, 6))]
        lens[0] = max(lens[0], 2)
        qsl = [0]
        for n in lens:
            qsl.append(qsl[-1] + n)
        x = torch.randn(qsl[-1], D, generator=g).to(dtype)
        cs = torch.randn(len(lens) + 2, W - 1, D, generator=g).to(dtype)
        cache = rng.sample(range(len(lens) + 2), len(lens))
        padded = [i for i in range(len(lens)) if rng.random() < 0.2]
        for i in padded:
            cache[i] = -1
        kw = dict(query_start_loc=qsl, cache_indices=cache, initial_state_mode=[rng.choice((0, 1)) for _ in lens],
                  activation_mode=act, pad_slot_id=-1)
        y_ref, cs_ref = oc.causal_conv1d(x, w, None, cs, **kw)
        cs_d = cs.to(dev)
        y = ops.causal_conv1d(x.to(dev), w.to(dev), None, cs_d, **kw)
        keep = torch.ones(qsl[-1], dtype=torch.bool)   # tokens of a padded sequence are not written by the op
        for i in padded:
            keep[qsl[i]:qsl[i + 1]] = False
        if keep.any():
            assert_close(y[keep.to(dev)], y_ref[keep], TOL_BF16, f"y W={W} D={D} lens={lens}")
        assert torch.equal(cs_d.cpu(), cs_ref)
