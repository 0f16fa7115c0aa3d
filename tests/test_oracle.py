"""CPU pins of the oracle (no GPU, no product code): every oracle function is checked against
something that does not share its formula - a different algorithm, a library routine, a closed
form, autograd, or the reference's own deterministic inputs."""
import math

import numpy as np
import pytest
import torch

from oracle import conv1d as oc, decode as od, gdn, gdn_bwd, kda

F = torch.nn.functional


# --------------------------------------------------------------------------- GDN
def test_cfg1_chunked_equals_naive_fp32():
    """Self-check configuration of the benchmark set: fp32, B=1 T=256 H=2 K=V=64, chunk 64, zero initial state, seed 0."""
    d = gdn.make_gdn_inputs(1, 256, 2, 64, 64, seed=0)
    o_n, f_n = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], output_final_state=True, naive=True)
    o_c, f_c = gdn.flash_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], output_final_state=True, naive=False)
    assert o_n.shape == (1, 256, 2, 64) and f_n.shape == (1, 2, 64, 64)
    assert float((o_n - o_c).abs().max()) <= 1e-5
    assert float((f_n - f_c).abs().max()) <= 1e-5


def test_naive_recurrence_against_float64_bruteforce_numpy():
    d = gdn.make_gdn_inputs(1, 20, 1, 8, 5, seed=3, head_first_gates=True)
    o, f = gdn.naive_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], 0.7, output_final_state=True)
    q, k, v = (d[n][0, 0].double().numpy() for n in "qkv")
    g, b = d["g"][0, 0].double().numpy(), d["beta"][0, 0].double().numpy()
    S = np.zeros((8, 5))
    for t in range(20):
        S = math.exp(g[t]) * S
        S = S + np.outer(k[t], b[t] * (v[t] - S.T @ k[t]))     # (I - b k k^T) S + b k v^T
        np.testing.assert_allclose(o[0, 0, t].numpy(), 0.7 * (S.T @ q[t]), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(f[0, 0].numpy(), S, rtol=1e-4, atol=1e-5)


def test_closed_forms():
    d = gdn.make_gdn_inputs(1, 40, 2, 16, 16, seed=1, head_first_gates=True)
    h0 = torch.randn(1, 2, 16, 16, generator=torch.Generator().manual_seed(0))
    # beta = 0: the state only decays
    o, f = gdn.naive_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], torch.zeros_like(d["beta"]), 1.0,
                                                initial_state=h0, output_final_state=True)
    G = torch.cumsum(d["g"], -1)
    assert torch.allclose(o, torch.einsum("bhtk,bhkv->bhtv", d["q"], h0) * torch.exp(G)[..., None], atol=1e-5)
    assert torch.allclose(f, h0 * torch.exp(G[:, :, -1])[..., None, None], atol=1e-5)
    # g = 0, beta = 1, unit keys: the state stores v_t under k_t exactly
    o, _ = gdn.naive_recurrent_gated_delta_rule(d["k"], d["k"], d["v"], torch.zeros_like(d["g"]),
                                                torch.ones_like(d["beta"]), 1.0)
    assert torch.allclose(o, d["v"], atol=1e-4)


@pytest.mark.parametrize("chunk", [16, 32, 64, 128])
def test_chunk_size_invariance_and_varlen(chunk):
    d = gdn.make_gdn_inputs(1, 200, 2, 32, 48, seed=2, head_first_gates=True, Hk=1)
    ref, fref = gdn.naive_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], output_final_state=True)
    o, f = gdn.chunk_gated_delta_rule_fwd(d["q"], d["k"], d["v"], d["g"], d["beta"], output_final_state=True, chunk=chunk)
    assert float((o - ref).abs().max()) < 1e-5 and float((f - fref).abs().max()) < 1e-5
    cu = [0, 7, 7, 90, 200]
    o_v, f_v = gdn.chunk_gated_delta_rule_fwd(d["q"], d["k"], d["v"], d["g"], d["beta"], output_final_state=True,
                                              chunk=chunk, cu_seqlens=cu)
    for n, (s, e) in enumerate(zip(cu, cu[1:])):
        if e == s:
            continue
        o_s, f_s = gdn.naive_recurrent_gated_delta_rule(d["q"][:, :, s:e], d["k"][:, :, s:e], d["v"][:, :, s:e],
                                                        d["g"][:, :, s:e], d["beta"][:, :, s:e], output_final_state=True)
        assert float((o_v[:, :, s:e] - o_s).abs().max()) < 1e-5
        assert float((f_v[n] - f_s[0]).abs().max()) < 1e-5


def test_stage_oracles_against_library_routines():
    gen = torch.Generator().manual_seed(4)
    g = torch.randn(2, 3, 130, generator=gen)
    ref = torch.cat([torch.cumsum(c, -1) for c in g.split(64, dim=-1)], -1)
    assert torch.allclose(gdn.chunk_local_cumsum(g, 64), ref, atol=1e-6)
    rev = torch.cat([torch.flip(torch.cumsum(torch.flip(c, [-1]), -1), [-1]) for c in g.split(64, dim=-1)], -1)
    assert torch.allclose(gdn.chunk_local_cumsum(g, 64, reverse=True, scale=2.0), 2.0 * rev, atol=1e-5)
    # kkt: structural zeros + library matmul
    k = torch.randn(1, 1, 70, 16, generator=gen)
    G = gdn.chunk_local_cumsum(-torch.rand(1, 1, 70, generator=gen), 64)
    beta = torch.rand(1, 1, 70, generator=gen)
    A = gdn.chunk_scaled_dot_kkt(k, G, beta, 64)
    blk = A[0, 0, :64]
    assert float(torch.triu(blk).abs().max()) == 0.0 and float(A[0, 0, 64:, 6:].abs().max()) == 0.0
    i, j = 37, 5
    expect = beta[0, 0, i] * math.exp(float(G[0, 0, i] - G[0, 0, j])) * float(k[0, 0, i] @ k[0, 0, j])
    assert abs(float(blk[i, j]) - expect) < 1e-5
    # solve_tri against numpy.linalg.inv, incl. a tail block
    X = gdn.solve_tri(A)
    inv = np.linalg.inv(np.eye(64) + blk.double().numpy())
    np.testing.assert_allclose(X[0, 0, :64].numpy(), inv, rtol=1e-5, atol=1e-5)
    inv_t = np.linalg.inv(np.eye(6) + A[0, 0, 64:, :6].double().numpy())
    np.testing.assert_allclose(X[0, 0, 64:, :6].numpy(), inv_t, rtol=1e-5, atol=1e-5)


# --------------------------------------------------------------------------- conv1d
def test_conv1d_against_F_conv1d_and_reference_kat_inputs():
    def make_tensor(shape, start):  # test_npu_causal_conv1d.py:154-161
        n = int(np.prod(shape))
        return (torch.arange(start, start + n, dtype=torch.float32).reshape(shape) / 128.0).to(torch.float16)

    x, w, b = make_tensor((2, 4, 16), 1.0), make_tensor((4, 16), 101.0), make_tensor((16,), 201.0)
    cs = make_tensor((2, 3, 16), 301.0)
    for act in (0, 1):
        y, new_cs = oc.causal_conv1d(x, w, b, cs, activation_mode=act)
        ref = F.conv1d(x.float().permute(0, 2, 1), w.float().t().unsqueeze(1), b.float(), padding=3, groups=16)[..., :4]
        ref = F.silu(ref) if act else ref
        assert torch.allclose(y.float(), ref.permute(0, 2, 1).to(torch.float16).float(), atol=2e-3, rtol=2e-3)
        assert torch.equal(new_cs[:, 2], x[:, 3]) and torch.equal(new_cs[:, 0], x[:, 1])
    # with initial state: equals a convolution over [state | x]
    y, new_cs = oc.causal_conv1d(x, w, None, cs, initial_state_mode=[1, 1])
    xc = torch.cat([cs, x], 1).float().permute(0, 2, 1)
    ref = F.conv1d(xc, w.float().t().unsqueeze(1), None, padding=0, groups=16)
    assert torch.allclose(y.float(), ref.permute(0, 2, 1).to(torch.float16).float(), atol=2e-3, rtol=2e-3)


def test_conv1d_short_sequences_shift_the_state():
    x = torch.randn(1, 2, 16).half()
    cs = torch.randn(1, 3, 16).half()
    w = torch.randn(4, 16).half()
    _, new_cs = oc.causal_conv1d(x, w, None, cs, initial_state_mode=[1])
    assert torch.equal(new_cs[0, 0], cs[0, 2]) and torch.equal(new_cs[0, 1:], x[0])
    _, new_cs = oc.causal_conv1d(x, w, None, cs)           # no initial state: zero history
    assert float(new_cs[0, 0].abs().max()) == 0.0


# --------------------------------------------------------------------------- decode
def test_decode_equals_naive_recurrence_with_transposed_state():
    gen = torch.Generator().manual_seed(6)
    T, H, K, V = 6, 2, 8, 12
    q, k = torch.randn(T, H, K, generator=gen), torch.randn(T, H, K, generator=gen)
    v, beta = torch.randn(T, H, V, generator=gen), torch.rand(T, H, generator=gen)
    g = -torch.rand(T, H, generator=gen)
    S0 = torch.randn(2, H, V, K, generator=gen)
    lens = torch.tensor([0, 4, 2], dtype=torch.int32)
    idx = torch.tensor([0, 0, 0, 0, 1, 1], dtype=torch.int32)
    o, S = od.recurrent_gated_delta_rule(q, k, v, S0, beta=beta, scale=0.5, actual_seq_lengths=lens,
                                         ssm_state_indices=idx, g=g)
    for n, (s, e) in enumerate([(0, 4), (4, 6)]):
        tr = lambda x: x[s:e].transpose(0, 1).unsqueeze(0)      # [1,H,L,D]
        o_n, f_n = gdn.naive_recurrent_gated_delta_rule(tr(q), tr(k), tr(v), g[s:e].t().unsqueeze(0),
                                                        beta[s:e].t().unsqueeze(0), 0.5,
                                                        initial_state=S0[n:n + 1].transpose(-1, -2),
                                                        output_final_state=True)
        assert torch.allclose(o[s:e], o_n[0].transpose(0, 1), atol=1e-5)
        assert torch.allclose(S[n], f_n[0].transpose(-1, -2), atol=1e-5)


def test_decode_accepted_tokens_and_no_gate():
    gen = torch.Generator().manual_seed(7)
    T, H, D = 3, 1, 4
    q, k, v = (torch.randn(T, H, D, generator=gen) for _ in range(3))
    beta = torch.rand(T, H, generator=gen)
    S0 = torch.randn(3, H, D, D, generator=gen)
    lens = torch.tensor([0, 3], dtype=torch.int32)
    idx = torch.tensor([0, 1, 2], dtype=torch.int32)
    acc = torch.tensor([2], dtype=torch.int32)
    o, S = od.recurrent_gated_delta_rule(q, k, v, S0, beta=beta, actual_seq_lengths=lens, ssm_state_indices=idx,
                                         num_accepted_tokens=acc, gk=torch.zeros(T, H, D))
    St = S0[1].clone()                                           # slot of token seq0 + accepted - 1
    for t in range(T):
        delta = beta[t, 0] * (v[t, 0] - St[0] @ k[t, 0])
        St[0] = St[0] + torch.outer(delta, k[t, 0])
        assert torch.allclose(o[t, 0], St[0] @ q[t, 0], atol=1e-5)
        assert torch.allclose(S[t], St, atol=1e-5)


# --------------------------------------------------------------------------- KDA
def kda_inputs(B, T, H, K, V, seed=0, gate_scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, H, T, K, generator=gen), dim=-1)
    k = F.normalize(torch.randn(B, H, T, K, generator=gen), dim=-1)
    v = torch.randn(B, H, T, V, generator=gen)
    gate = F.logsigmoid(torch.randn(B, H, T, K, generator=gen)) * gate_scale
    beta = torch.sigmoid(torch.randn(B, H, T, generator=gen))
    return q, k, v, gate, beta


@pytest.mark.parametrize("cu", [None, [0, 5, 70, 150]])
def test_kda_chunked_equals_naive(cu):
    q, k, v, gate, beta = kda_inputs(1, 150, 2, 16, 24, seed=1, gate_scale=0.3)
    h0 = torch.randn(1 if cu is None else 3, 2, 16, 24, generator=torch.Generator().manual_seed(9))
    o_n, f_n = kda.naive_recurrent_kda(q, k, v, gate, beta, 0.3, initial_state=h0, output_final_state=True,
                                       cu_seqlens=cu, compute_dtype=torch.float64)
    gk = kda.kda_gate_cumsum(gate, 64, cu_seqlens=cu)
    out = kda.chunk_kda_fwd(q, k, v, gk, beta, 0.3, 64, initial_state=h0, output_final_state=True, cu_seqlens=cu,
                            compute_dtype=torch.float64)
    assert float((out["o"] - o_n).abs().max()) < 1e-5
    assert float((out["final_state"] - f_n.float()).abs().max()) < 1e-5


@pytest.mark.parametrize("cu", [None, [0, 5, 70, 150]])
def test_fwd_h_with_key_wise_gate_is_the_kda_state_scan(cu):
    """chunk_gated_delta_rule_fwd_h(kg, w, u, gk=gk) walks the same states as the KDA chunk forward (itself pinned
    against the per-token recurrence above): h, v_new and the final state agree."""
    q, k, v, gate, beta = kda_inputs(1, 150, 2, 16, 24, seed=3, gate_scale=0.3)
    h0 = torch.randn(1 if cu is None else 3, 2, 16, 24, generator=torch.Generator().manual_seed(4))
    gk = kda.kda_gate_cumsum(gate, 64, cu_seqlens=cu)
    ref = kda.chunk_kda_fwd(q, k, v, gk, beta, 0.3, 64, initial_state=h0, output_final_state=True, cu_seqlens=cu,
                            compute_dtype=torch.float64)
    h, v_new, final = gdn.chunk_gated_delta_rule_fwd_h(ref["kg"], ref["w"], ref["u"], gk=gk, initial_state=h0,
                                                       output_final_state=True, cu_seqlens=cu, compute_dtype=torch.float64,
                                                       output_dtype=torch.float64)
    assert torch.allclose(h, ref["h"], atol=1e-10) and torch.allclose(v_new, ref["v_new"], atol=1e-10)
    assert torch.allclose(final, ref["final_state"], atol=1e-6)


def test_kda_reduces_to_gdn_for_channel_constant_gate():
    d = gdn.make_gdn_inputs(1, 100, 2, 16, 16, seed=5, head_first_gates=True)
    gate = d["g"][..., None].expand(-1, -1, -1, 16).contiguous()
    o_k, f_k = kda.naive_recurrent_kda(d["q"], d["k"], d["v"], gate, d["beta"], output_final_state=True)
    o_g, f_g = gdn.naive_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], output_final_state=True)
    assert torch.allclose(o_k, o_g, atol=1e-6) and torch.allclose(f_k, f_g, atol=1e-6)


def test_kda_gate_activations():
    gen = torch.Generator().manual_seed(2)
    g = torch.randn(1, 2, 70, 8, generator=gen)
    A_log, dt = torch.randn(2, generator=gen) * 0.3, torch.randn(16, generator=gen) * 0.1
    gk = kda.kda_gate_cumsum(g, 64, A_log=A_log, dt_bias=dt, use_gate_in_kernel=True)
    act = -torch.exp(A_log).view(1, 2, 1, 1) * F.softplus(g + dt.view(1, 2, 1, 8))
    ref = torch.cat([torch.cumsum(c, 2) for c in act.split(64, dim=2)], 2) / math.log(2.0)
    assert torch.allclose(gk, ref, atol=1e-5)
    gk = kda.kda_gate_cumsum(g, 64, A_log=A_log, dt_bias=dt, use_gate_in_kernel=True, safe_gate=True, lower_bound=-3.0)
    act = -3.0 * torch.sigmoid(torch.exp(A_log).view(1, 2, 1, 1) * (g + dt.view(1, 2, 1, 8)))
    ref = torch.cat([torch.cumsum(c, 2) for c in act.split(64, dim=2)], 2) / math.log(2.0)
    assert torch.allclose(gk, ref, atol=1e-5)


@pytest.mark.parametrize("mode", ["g", "gK"])
def test_bwd_dhu_against_autograd(mode):
    """dh0 and dv2 of the reverse scan equal autograd through the forward state recurrence."""
    gen = torch.Generator().manual_seed(8)
    B, H, T, K, V, C = 1, 2, 150, 8, 6, 64
    dd = torch.float64
    q, k, w = (torch.randn(B, H, T, K, generator=gen, dtype=dd) * 0.3 for _ in range(3))
    u = torch.randn(B, H, T, V, generator=gen, dtype=dd).requires_grad_(True)
    do, dv = torch.randn(B, H, T, V, generator=gen, dtype=dd), torch.randn(B, H, T, V, generator=gen, dtype=dd)
    dht = torch.randn(B, H, K, V, generator=gen, dtype=dd)
    h0 = torch.randn(B, H, K, V, generator=gen, dtype=dd).requires_grad_(True)
    if mode == "g":
        g = torch.cat([torch.cumsum(c, -1) for c in (-torch.rand(B, H, T, generator=gen, dtype=dd) * 0.1).split(C, -1)], -1)
    else:
        gK = torch.cat([torch.cumsum(c, 2) for c in (-torch.rand(B, H, T, K, generator=gen, dtype=dd) * 0.1).split(C, 2)], 2)
    S, loss = h0, 0.0
    for s in range(0, T, C):
        e = min(s + C, T)
        vn = u[:, :, s:e] - w[:, :, s:e] @ S
        loss = loss + (vn * dv[:, :, s:e]).sum()
        if mode == "g":
            gc = g[:, :, s:e]
            loss = loss + 0.7 * (((q[:, :, s:e] * torch.exp(gc)[..., None]) @ S) * do[:, :, s:e]).sum()
            S = S * torch.exp(gc[:, :, -1])[..., None, None] + k[:, :, s:e].transpose(-1, -2) @ (vn * torch.exp(gc[:, :, -1:] - gc)[..., None])
        else:
            loss = loss + 0.7 * ((q[:, :, s:e] @ S) * do[:, :, s:e]).sum()
            S = S * torch.exp2(gK[:, :, e - 1])[..., None] + k[:, :, s:e].transpose(-1, -2) @ vn
    loss = loss + (S * dht).sum()
    loss.backward()
    kw = dict(g=g) if mode == "g" else dict(gK=gK)
    dh, dh0, dv2 = kda.chunk_gated_delta_rule_bwd_dhu(q, k, w, do, dv, 0.7, C, dht=dht, compute_dtype=dd, **kw)
    assert torch.allclose(dh0, h0.grad, atol=1e-9)
    assert torch.allclose(dv2, u.grad, atol=1e-9)
    assert torch.allclose(dh[:, :, -1], dht, atol=0)            # state gradient seen by the last chunk


def test_bwd_intra_against_autograd_and_anchored_evaluation():
    """The four accumulations equal autograd through Aqk / Akk as functions of (q, k, gk, beta)."""
    gen = torch.Generator().manual_seed(10)
    B, H, T, K = 1, 2, 70, 8
    dd = torch.float64
    q = torch.randn(B, H, T, K, generator=gen, dtype=dd).requires_grad_(True)
    k = torch.randn(B, H, T, K, generator=gen, dtype=dd).requires_grad_(True)
    beta = torch.rand(B, H, T, generator=gen, dtype=dd).requires_grad_(True)
    inc = -torch.rand(B, H, T, K, generator=gen, dtype=dd) * 0.2
    gk = torch.cat([torch.cumsum(c, 2) for c in inc.split(64, 2)], 2).requires_grad_(True)
    dAqk = torch.randn(B, H, T, 64, generator=gen, dtype=dd)
    dAkk = torch.tril(torch.randn(B, H, T, 64, generator=gen, dtype=dd))
    loss = 0.0
    for s in range(0, T, 64):
        e = min(s + 64, T)
        L = e - s
        dec = torch.exp2(gk[:, :, s:e, None, :] - gk[:, :, None, s:e, :])
        aqk = torch.tril(torch.einsum("bhik,bhijk,bhjk->bhij", q[:, :, s:e], dec, k[:, :, s:e]))
        akk = torch.tril(torch.einsum("bhik,bhijk,bhjk->bhij", k[:, :, s:e], dec, k[:, :, s:e])) * beta[:, :, s:e, None]
        loss = loss + (aqk * dAqk[:, :, s:e, :L]).sum() + (akk * torch.tril(dAkk[:, :, s:e, :L])).sum()
    loss.backward()
    z4, z3 = torch.zeros(B, H, T, K, dtype=dd), torch.zeros(B, H, T, dtype=dd)
    dq, dk, db, dg = kda.chunk_kda_bwd_intra(q.detach(), k.detach(), gk.detach(), beta.detach(), dAqk, dAkk, z4, z4, z3, z4)
    assert torch.allclose(dq, q.grad, atol=1e-9) and torch.allclose(dk, k.grad, atol=1e-9)
    assert torch.allclose(db, beta.grad, atol=1e-9)
    assert torch.allclose(dg, gk.grad / math.log(2.0), atol=1e-9)   # dg is the gradient w.r.t. ln2 * gk


def _cumsum_log2(raw, C, cu=None):
    out = torch.empty_like(raw)
    for b, _, _, s, e in gdn.chunk_spans(raw.shape[0], raw.shape[2], C, cu):
        out[b, :, s:e] = torch.cumsum(raw[b, :, s:e], dim=1) / math.log(2.0)
    return out


@pytest.mark.parametrize("cu", [None, [0, 70, 70, 150]])
def test_kda_bwd_dav_against_autograd(cu):
    """dAqk and dv are the gradients of o_intra = (scale tril(S)) v_new with respect to S and v_new."""
    gen = torch.Generator().manual_seed(21)
    B, H, T, V, C, dd = 1, 2, 150, 6, 64, torch.float64
    S = torch.randn(B, H, T, C, generator=gen, dtype=dd).requires_grad_(True)
    vn = torch.randn(B, H, T, V, generator=gen, dtype=dd).requires_grad_(True)
    do = torch.randn(B, H, T, V, generator=gen, dtype=dd)
    loss, Aqk = 0.0, torch.zeros(B, H, T, C, dtype=dd)
    for b, _, _, s, e in gdn.chunk_spans(B, T, C, cu):
        L = e - s
        A = torch.tril(S[b, :, s:e, :L]) * 0.7
        Aqk[b, :, s:e, :L] = A.detach()
        loss = loss + ((A @ vn[b, :, s:e]) * do[b, :, s:e]).sum()
    loss.backward()
    dA, dv = kda.chunk_kda_bwd_dav(vn.detach(), do, Aqk, 0.7, C, cu_seqlens=cu, compute_dtype=dd)
    assert torch.allclose(dA, S.grad, atol=1e-10) and torch.allclose(dv, vn.grad, atol=1e-10)


@pytest.mark.parametrize("cu,rep", [(None, 1), ([0, 70, 70, 150], 2)])
def test_kda_bwd_dqkwg_against_autograd(cu, rep):
    """dq, dk, dw, dg are the gradients of one chunk step's state-dependent parts with h, dh, dv given."""
    gen = torch.Generator().manual_seed(22)
    B, Hk, T, K, V, C, dd = 1, 2, 150, 8, 6, 64, torch.float64
    Hv = Hk * rep
    NT = gdn.total_chunks(B, T, C, cu)
    q = torch.randn(B, Hk, T, K, generator=gen, dtype=dd).requires_grad_(True)
    k = torch.randn(B, Hk, T, K, generator=gen, dtype=dd).requires_grad_(True)
    w = torch.randn(B, Hv, T, K, generator=gen, dtype=dd).requires_grad_(True)
    gk = _cumsum_log2(-torch.rand(B, Hv, T, K, generator=gen, dtype=dd) * 0.2, C, cu).requires_grad_(True)
    vn, do, dv = (torch.randn(B, Hv, T, V, generator=gen, dtype=dd) for _ in range(3))
    h, dh = (torch.randn(B, Hv, NT, K, V, generator=gen, dtype=dd) for _ in range(2))
    loss = 0.0
    for b, _, ci, s, e in gdn.chunk_spans(B, T, C, cu):
        qc = q[b, :, s:e].repeat_interleave(rep, dim=0)
        kc = k[b, :, s:e].repeat_interleave(rep, dim=0)
        gc = gk[b, :, s:e]
        o = 0.7 * (qc * torch.exp2(gc)) @ h[b, :, ci]
        h_next = torch.exp2(gc[:, -1])[..., None] * h[b, :, ci] + (kc * torch.exp2(gc[:, -1:] - gc)).transpose(1, 2) @ vn[b, :, s:e]
        loss = loss + (o * do[b, :, s:e]).sum() + (h_next * dh[b, :, ci]).sum() - ((w[b, :, s:e] @ h[b, :, ci]) * dv[b, :, s:e]).sum()
    loss.backward()
    dq, dk, dw, dg = kda.chunk_kda_bwd_dqkwg(q.detach(), k.detach(), vn, gk.detach(), h, do, dh, dv, 0.7, C, cu_seqlens=cu,
                                             compute_dtype=dd)
    fold = lambda x: x.view(B, Hk, rep, T, K).sum(2)
    assert torch.allclose(fold(dq), q.grad, atol=1e-9) and torch.allclose(fold(dk), k.grad, atol=1e-9)
    assert torch.allclose(dw, w.grad, atol=1e-9)
    assert torch.allclose(dg, gk.grad / math.log(2.0), atol=1e-9)


@pytest.mark.parametrize("cu,rep", [(None, 1), ([0, 70, 70, 150], 2)])
def test_kda_bwd_wy_against_autograd(cu, rep):
    """dk, dv, dbeta, dg, dM are the gradients of w = (I+M)^-1 (k beta 2^g), u = (I+M)^-1 (v beta), M an independent
    strictly lower matrix."""
    gen = torch.Generator().manual_seed(23)
    B, Hk, T, K, V, C, dd = 1, 2, 150, 8, 6, 64, torch.float64
    Hv = Hk * rep
    k = torch.randn(B, Hk, T, K, generator=gen, dtype=dd).requires_grad_(True)
    v = torch.randn(B, Hv, T, V, generator=gen, dtype=dd).requires_grad_(True)
    beta = torch.rand(B, Hv, T, generator=gen, dtype=dd).requires_grad_(True)
    gk = _cumsum_log2(-torch.rand(B, Hv, T, K, generator=gen, dtype=dd) * 0.2, C, cu).requires_grad_(True)
    M = (torch.randn(B, Hv, T, C, generator=gen, dtype=dd) * 0.2).requires_grad_(True)
    dw = torch.randn(B, Hv, T, K, generator=gen, dtype=dd)
    du = torch.randn(B, Hv, T, V, generator=gen, dtype=dd)
    loss, Akk = 0.0, torch.zeros(B, Hv, T, C, dtype=dd)
    for b, _, _, s, e in gdn.chunk_spans(B, T, C, cu):
        L = e - s
        A = torch.linalg.inv(torch.eye(L, dtype=dd) + torch.tril(M[b, :, s:e, :L], -1))
        Akk[b, :, s:e, :L] = A.detach()
        kc = k[b, :, s:e].repeat_interleave(rep, dim=0)
        bc = beta[b, :, s:e, None]
        loss = loss + ((A @ (kc * bc * torch.exp2(gk[b, :, s:e]))) * dw[b, :, s:e]).sum() + ((A @ (v[b, :, s:e] * bc)) * du[b, :, s:e]).sum()
    loss.backward()
    dk, dv, db, dg, dM = kda.chunk_kda_bwd_wy(k.detach(), v.detach(), beta.detach(), gk.detach(), Akk, dw, du, C,
                                              cu_seqlens=cu, compute_dtype=dd)
    assert torch.allclose(dk.view(B, Hk, rep, T, K).sum(2), k.grad, atol=1e-9)
    assert torch.allclose(dv, v.grad, atol=1e-9) and torch.allclose(db, beta.grad, atol=1e-9)
    assert torch.allclose(dg, gk.grad / math.log(2.0), atol=1e-9)
    assert torch.allclose(dM, M.grad, atol=1e-9)


@pytest.mark.parametrize("cu,rep", [(None, 1), ([0, 70, 70, 150], 2), ([0, 5, 133], 1)])
def test_kda_bwd_composition_against_autograd_through_the_recurrence(cu, rep):
    """The whole chunked backward (every gradient, with an initial state and a final-state gradient) equals fp64
    autograd through the per-token KDA recurrence."""
    gen = torch.Generator().manual_seed(24)
    T = cu[-1] if cu else 150
    B, Hk, K, V, dd = 1, 2, 8, 6, torch.float64
    Hv = Hk * rep
    N = len(cu) - 1 if cu else B
    q = F.normalize(torch.randn(B, Hk, T, K, generator=gen, dtype=dd), dim=-1).requires_grad_(True)
    k = F.normalize(torch.randn(B, Hk, T, K, generator=gen, dtype=dd), dim=-1).requires_grad_(True)
    v = torch.randn(B, Hv, T, V, generator=gen, dtype=dd).requires_grad_(True)
    gate = (F.logsigmoid(torch.randn(B, Hv, T, K, generator=gen, dtype=dd)) * 0.5).requires_grad_(True)
    beta = torch.sigmoid(torch.randn(B, Hv, T, generator=gen, dtype=dd)).requires_grad_(True)
    h0 = (torch.randn(N, Hv, K, V, generator=gen, dtype=dd) * 0.3).requires_grad_(True)
    do = torch.randn(B, Hv, T, V, generator=gen, dtype=dd)
    dht = torch.randn(N, Hv, K, V, generator=gen, dtype=dd)
    o, final = kda.naive_recurrent_kda(q, k, v, gate, beta, 0.7, initial_state=h0, output_final_state=True, cu_seqlens=cu,
                                       compute_dtype=dd)
    ((o * do).sum() + (final * dht).sum()).backward()
    got = kda.chunk_kda_bwd(q.detach(), k.detach(), v.detach(), gate.detach(), beta.detach(), 0.7, do, initial_state=h0.detach(),
                            dht=dht, cu_seqlens=cu, compute_dtype=dd)
    for name, a, e in zip(("dq", "dk", "dv", "dg", "dbeta", "dh0"), got, (q.grad, k.grad, v.grad, gate.grad, beta.grad, h0.grad)):
        assert torch.allclose(a, e, atol=1e-8), f"{name}: {float((a - e).abs().max())}"


# ----------------------------------------------------------------------------
# GDN backward chain: every operator against autograd of the stage it differentiates (fp64)
# ----------------------------------------------------------------------------
def _cumsummed_gate(B, H, T, C, gen, dd, cu=None):
    raw = -torch.rand(B, H, T, generator=gen, dtype=dd) * 0.2
    return raw, gdn.chunk_local_cumsum(raw, C, cu_seqlens=cu, output_dtype=dd)


@pytest.mark.parametrize("cu", [None, [0, 70, 70, 150]])
def test_bwd_dv_local_against_autograd(cu):
    """dv_local is the gradient, with respect to v_new, of the intra-chunk part of the output."""
    gen = torch.Generator().manual_seed(21)
    B, Hk, Hv, T, K, V, C = 1, 1, 2, 150, 8, 6, 64
    dd = torch.float64
    q, k = (torch.randn(B, Hk, T, K, generator=gen, dtype=dd) for _ in range(2))
    v = torch.randn(B, Hv, T, V, generator=gen, dtype=dd).requires_grad_(True)
    do = torch.randn(B, Hv, T, V, generator=gen, dtype=dd)
    _, G = _cumsummed_gate(B, Hv, T, C, gen, dd, cu)
    h = torch.zeros(B, Hv, gdn.total_chunks(B, T, C, cu), K, V, dtype=dd)
    o = gdn.chunk_fwd_o(q, k, v, h, 0.7, g=G, chunk=C, cu_seqlens=cu, compute_dtype=dd, output_dtype=dd)
    (o * do).sum().backward()
    dv = gdn_bwd.chunk_bwd_dv_local(q, k, do, G, 0.7, C, cu_seqlens=cu, compute_dtype=dd, output_dtype=dd)
    assert torch.allclose(dv, v.grad, atol=1e-10)


def test_bwd_dqkwg_against_autograd():
    """One chunk step (v_new = u - w h, output, state update) differentiated by autograd: dq, dk, dw and
    the gradient of the cumsummed gate equal the operator's; several chunks exercise the per-chunk h / dh."""
    gen = torch.Generator().manual_seed(22)
    B, Hk, Hv, T, K, V, C = 1, 1, 2, 150, 8, 6, 64
    dd = torch.float64
    scale = 0.6
    q, k = (torch.randn(B, Hk, T, K, generator=gen, dtype=dd).requires_grad_(True) for _ in range(2))
    w = (torch.randn(B, Hv, T, K, generator=gen, dtype=dd) * 0.3).requires_grad_(True)
    u = torch.randn(B, Hv, T, V, generator=gen, dtype=dd)
    do = torch.randn(B, Hv, T, V, generator=gen, dtype=dd)
    _, G0 = _cumsummed_gate(B, Hv, T, C, gen, dd)
    G = G0.clone().requires_grad_(True)
    NT = gdn.total_chunks(B, T, C)
    # independent per-chunk states and state gradients: the operator treats them as given
    h = torch.randn(B, Hv, NT, K, V, generator=gen, dtype=dd) * 0.5
    dh = torch.randn(B, Hv, NT, K, V, generator=gen, dtype=dd) * 0.5
    qr, kr = q.repeat_interleave(2, 1), k.repeat_interleave(2, 1)
    loss = 0.0
    vns = []
    for ci, s in enumerate(range(0, T, C)):
        e = min(s + C, T)
        gc = G[:, :, s:e]
        S = h[:, :, ci]
        vn = u[:, :, s:e] - w[:, :, s:e] @ S
        vn.retain_grad()
        vns.append(vn)
        dec = torch.tril(torch.exp(torch.clamp(gc[..., :, None] - gc[..., None, :], max=0.0)))
        o = ((qr[:, :, s:e] * torch.exp(gc)[..., None]) @ S + (qr[:, :, s:e] @ kr[:, :, s:e].transpose(-1, -2) * dec) @ vn) * scale
        S_next = S * torch.exp(gc[:, :, -1])[..., None, None] \
            + kr[:, :, s:e].transpose(-1, -2) @ (vn * torch.exp(gc[:, :, -1:] - gc)[..., None])
        loss = loss + (o * do[:, :, s:e]).sum() + (S_next * dh[:, :, ci]).sum()
    loss.backward()
    v_new = torch.cat([t.detach() for t in vns], 2)
    dv = torch.cat([t.grad for t in vns], 2)            # what bwd_dhu hands to dqkwg
    dq, dk, dw, dg = gdn_bwd.chunk_bwd_dqkwg(q.detach(), k.detach(), v_new.detach(), G0, h, do, dh, dv, scale, C,
                                             compute_dtype=dd, output_dtype=dd)
    assert torch.allclose(dq, q.grad, atol=1e-9)
    assert torch.allclose(dk, k.grad, atol=1e-9)
    assert torch.allclose(dw, w.grad, atol=1e-9)
    assert torch.allclose(dg, G.grad, atol=1e-9)


@pytest.mark.parametrize("cu", [None, [0, 64, 81, 150]])
def test_wy_bwd_against_autograd(cu):
    """bwd_da followed by bwd_full is the vector-Jacobian product of (k, v, beta, G) -> (w, u)."""
    gen = torch.Generator().manual_seed(23)
    B, Hk, Hv, T, K, V, C = 1, 1, 2, 150, 8, 6, 64
    dd = torch.float64
    k = F.normalize(torch.randn(B, Hk, T, K, generator=gen, dtype=dd), dim=-1).requires_grad_(True)
    v = torch.randn(B, Hv, T, V, generator=gen, dtype=dd).requires_grad_(True)
    beta = torch.rand(B, Hv, T, generator=gen, dtype=dd).requires_grad_(True)
    _, G0 = _cumsummed_gate(B, Hv, T, C, gen, dd, cu)
    G = G0.clone().requires_grad_(True)
    dw = torch.randn(B, Hv, T, K, generator=gen, dtype=dd)
    du = torch.randn(B, Hv, T, V, generator=gen, dtype=dd)
    # forward stages written with differentiable torch ops only (library inverse, not the oracle's substitution)
    kr = k.repeat_interleave(2, 1)
    ws, us, As = [], [], []
    spans = [(s, min(s + C, T)) for s in range(0, T, C)] if cu is None else \
        [(s, min(s + C, e)) for b0, e in zip(cu, cu[1:]) for s in range(b0, e, C)]
    for s, e in spans:
        gc, bc, kc = G[:, :, s:e], beta[:, :, s:e], kr[:, :, s:e]
        M = torch.tril((kc @ kc.transpose(-1, -2)) * torch.exp(gc[..., :, None] - gc[..., None, :]) * bc[..., None], -1)
        Ainv = torch.linalg.inv(torch.eye(e - s, dtype=dd) + M)
        As.append(torch.nn.functional.pad(Ainv.detach(), (0, C - (e - s))))
        ws.append(Ainv @ (kc * (bc * torch.exp(gc))[..., None]))
        us.append(Ainv @ (v[:, :, s:e] * bc[..., None]))
    ((torch.cat(ws, 2) * dw).sum() + (torch.cat(us, 2) * du).sum()).backward()
    A = torch.cat(As, 2)
    # the oracle's own forward agrees with this construction
    A_or = gdn.solve_tri(gdn.chunk_scaled_dot_kkt(k.detach(), G0, beta.detach(), C, cu_seqlens=cu, compute_dtype=dd),
                         cu_seqlens=cu, compute_dtype=dd, output_dtype=dd)
    assert torch.allclose(A_or, A, atol=1e-10)
    dA = gdn_bwd.prepare_wy_repr_bwd_da(k.detach(), v.detach(), beta.detach(), A, dw, du, G0, C, cu_seqlens=cu,
                                        compute_dtype=dd, output_dtype=dd)
    assert float(torch.tril(dA[:, :, :64, :], -1).abs().max()) == 0.0     # stored transposed: upper triangular
    dk, dv, db, dg = gdn_bwd.prepare_wy_repr_bwd_full(k.detach(), v.detach(), beta.detach(), A, dA, dw, du, G0, C,
                                                      cu_seqlens=cu, compute_dtype=dd, output_dtype=dd)
    assert torch.allclose(dk, k.grad, atol=1e-9)
    assert torch.allclose(dv, v.grad, atol=1e-9)
    assert torch.allclose(db, beta.grad, atol=1e-9)
    assert torch.allclose(dg, G.grad, atol=1e-9)


@pytest.mark.parametrize("cu", [None, [0, 40, 40, 170]])
def test_gdn_backward_composition_against_recurrence_autograd(cu):
    """The composed backward equals autograd through the per-token recurrence for every input, with an
    initial state, a final-state gradient, grouped value heads and a ragged tail."""
    gen = torch.Generator().manual_seed(24)
    B, Hk, Hv, T, K, V, C = (2 if cu is None else 1), 1, 2, 170, 8, 6, 64
    N = B if cu is None else len(cu) - 1
    dd = torch.float64
    q = F.normalize(torch.randn(B, Hk, T, K, generator=gen, dtype=dd), dim=-1).requires_grad_(True)
    k = F.normalize(torch.randn(B, Hk, T, K, generator=gen, dtype=dd), dim=-1).requires_grad_(True)
    v = torch.randn(B, Hv, T, V, generator=gen, dtype=dd).requires_grad_(True)
    g = (-torch.rand(B, Hv, T, generator=gen, dtype=dd) * 0.3).requires_grad_(True)
    beta = torch.rand(B, Hv, T, generator=gen, dtype=dd).requires_grad_(True)
    h0 = (torch.randn(N, Hv, K, V, generator=gen, dtype=dd) * 0.5).requires_grad_(True)
    do = torch.randn(B, Hv, T, V, generator=gen, dtype=dd)
    dht = torch.randn(N, Hv, K, V, generator=gen, dtype=dd)
    o, final = gdn.naive_recurrent_gated_delta_rule(q, k, v, g, beta, 0.5, initial_state=h0, output_final_state=True,
                                                    cu_seqlens=cu, compute_dtype=dd)
    ((o * do).sum() + (final * dht).sum()).backward()
    det = lambda t: t.detach()
    dq, dk, dv, db, dg, dh0 = gdn_bwd.chunk_gated_delta_rule_bwd(
        det(q), det(k), det(v), det(g), det(beta), 0.5, do, initial_state=det(h0), dht=dht, chunk=C, cu_seqlens=cu,
        compute_dtype=dd)
    for name, got, want in (("dq", dq, q.grad), ("dk", dk, k.grad), ("dv", dv, v.grad), ("dbeta", db, beta.grad),
                            ("dg", dg, g.grad), ("dh0", dh0, h0.grad)):
        assert torch.allclose(got, want, atol=1e-8), f"{name}: {(got - want).abs().max().item():.3e}"


# ----------------------------------------------------------------------------
# causal_conv1d: state-update / speculative-decode mode and backward
# ----------------------------------------------------------------------------
def test_conv1d_update_in_pieces_equals_one_prefill():
    """Feeding a sequence piece by piece through the update mode reproduces F.conv1d over the whole sequence,
    for every width, through shuffled cache slots, and leaves the last W-1 inputs in the state."""
    gen = torch.Generator().manual_seed(31)
    for W in (2, 3, 4):
        B, T, D = 3, 11, 16
        x = torch.randn(B, T, D, generator=gen)
        w = torch.randn(W, D, generator=gen)
        b = torch.randn(D, generator=gen)
        full = F.conv1d(x.permute(0, 2, 1), w.t().unsqueeze(1), b, padding=W - 1, groups=D)[..., :T].permute(0, 2, 1)
        cache = [4, 0, 2]
        cs = torch.zeros(6, W - 1, D)
        outs = []
        for s, e in ((0, 1), (1, 4), (4, 5), (5, 11)):
            piece = x[:, s] if e - s == 1 and s == 0 else x[:, s:e]      # also the 2-D one-token form
            y, cs = oc.causal_conv1d_update(piece, w, b, cs, cache_indices=cache)
            outs.append(y.unsqueeze(1) if y.dim() == 2 else y)
        assert torch.allclose(torch.cat(outs, 1), full, atol=1e-5)
        for n, slot in enumerate(cache):
            assert torch.equal(cs[slot], x[n, T - (W - 1):])
        assert float(cs[[1, 3, 5]].abs().max()) == 0.0                  # untouched slots


def test_conv1d_update_padding_and_activation():
    gen = torch.Generator().manual_seed(32)
    x = torch.randn(3, 2, 16, generator=gen)
    w, cs = torch.randn(4, 16, generator=gen), torch.randn(5, 3, 16, generator=gen)
    y, new = oc.causal_conv1d_update(x, w, None, cs, cache_indices=[3, -1, 0], activation_mode=1)
    ref = F.silu(F.conv1d(torch.cat([cs[[3, 0]], x[[0, 2]]], 1).permute(0, 2, 1), w.t().unsqueeze(1), None, groups=16)).permute(0, 2, 1)
    assert torch.allclose(y[[0, 2]], ref, atol=1e-5) and float(y[1].abs().max()) == 0.0
    assert torch.equal(new[[1, 2, 4]], cs[[1, 2, 4]])


def test_conv1d_speculative_decode_tracks_the_accepted_prefix():
    """A speculative-decoding loop: every step proposes S tokens of which only a prefix is accepted; the next step
    passes that count.  The outputs at accepted positions must equal a plain causal convolution of the accepted
    stream (F.conv1d), whatever was drafted beyond it."""
    gen = torch.Generator().manual_seed(33)
    W, D, S = 4, 16, 4
    w, b = torch.randn(W, D, generator=gen), torch.randn(D, generator=gen)
    truth = torch.randn(1, 40, D, generator=gen)
    full = F.conv1d(truth.permute(0, 2, 1), w.t().unsqueeze(1), b, padding=W - 1, groups=D)[..., :40].permute(0, 2, 1)
    cs = torch.zeros(2, (W - 1) + (S - 1), D)
    pos, accepted_prev = 0, None
    for accepted in (2, 4, 1, 3, 4, 2):
        draft = truth[:, pos:pos + S].clone()
        draft[:, accepted:] = torch.randn(1, S - accepted, D, generator=gen)      # rejected tail
        kw = {} if accepted_prev is None else dict(num_accepted_tokens=[accepted_prev])
        if accepted_prev is None:
            # first step: history is the zero state at rows 0..2, i.e. one accepted token of an empty draft
            kw = dict(num_accepted_tokens=[1])
        y, cs = oc.causal_conv1d_update(draft, w, b, cs, cache_indices=[1], **kw)
        assert torch.allclose(y[:, :accepted], full[:, pos:pos + accepted], atol=1e-5)
        pos += accepted
        accepted_prev = accepted


def test_conv1d_bwd_against_autograd():
    """dx, dw, db, dh0 equal autograd through F.conv1d over [state rows 1..W-1 | x], with SiLU, a final-state
    gradient and packed sequences (including one shorter than the kernel)."""
    gen = torch.Generator().manual_seed(34)
    dd = torch.float64
    for W in (2, 3, 4):
        D = 16
        qsl = [0, 2, 9, 10, 21]
        T = qsl[-1]
        N = len(qsl) - 1
        x = torch.randn(T, D, generator=gen, dtype=dd).requires_grad_(True)
        w = torch.randn(W, D, generator=gen, dtype=dd).requires_grad_(True)
        bias = torch.randn(D, generator=gen, dtype=dd).requires_grad_(True)
        h0 = torch.randn(N, W, D, generator=gen, dtype=dd).requires_grad_(True)
        dy = torch.randn(T, D, generator=gen, dtype=dd)
        dht = torch.randn(N, W, D, generator=gen, dtype=dd)
        loss, ys = 0.0, []
        for n, (s, e) in enumerate(zip(qsl, qsl[1:])):
            xp = torch.cat([h0[n, 1:], x[s:e]], 0)
            pre = F.conv1d(xp.t().unsqueeze(0), w.t().unsqueeze(1), bias, groups=D)[0].t()
            ys.append(pre.detach())
            loss = loss + (F.silu(pre) * dy[s:e]).sum()
            if e - s >= W - 1:          # final state = last W-1 inputs (the golden's short-sequence rule differs)
                loss = loss + (x[e - (W - 1):e] * dht[n, 1:]).sum()
        loss.backward()
        long_enough = torch.tensor([e - s >= W - 1 for s, e in zip(qsl, qsl[1:])])
        dht_used = dht * long_enough[:, None, None]
        dx, dw, db, dh0 = oc.causal_conv1d_bwd(x.detach().float(), torch.cat(ys).float(), w.detach().float(), dy.float(),
                                               h0.detach().float(), dht_used.float(), query_start_loc=qsl, activation=1)
        assert torch.allclose(dx.double(), x.grad, atol=1e-4)
        assert torch.allclose(dw.double(), w.grad, atol=1e-4)
        assert torch.allclose(db.double(), bias.grad, atol=1e-4)
        assert torch.allclose(dh0.double(), h0.grad, atol=1e-4)
        assert float(dh0[:, 0].abs().max()) == 0.0
    # dense layout, no activation, no states: the plain transposed convolution
    x = torch.randn(2, 7, 16, generator=gen, dtype=dd).requires_grad_(True)
    w = torch.randn(4, 16, generator=gen, dtype=dd).requires_grad_(True)
    dy = torch.randn(2, 7, 16, generator=gen, dtype=dd)
    (F.conv1d(x.permute(0, 2, 1), w.t().unsqueeze(1), None, padding=3, groups=16)[..., :7].permute(0, 2, 1) * dy).sum().backward()
    dx, dw, db, dh0 = oc.causal_conv1d_bwd(x.detach().float(), None, w.detach().float(), dy.float())
    assert torch.allclose(dx.double(), x.grad, atol=1e-4) and torch.allclose(dw.double(), w.grad, atol=1e-4)
    assert torch.allclose(db.double(), dy.sum((0, 1)), atol=1e-4) and float(dh0.abs().max()) == 0.0


# ----------------------------------------------------------------------------
# recurrent_kda (decode / speculative decode over a state pool)
# ----------------------------------------------------------------------------
def test_recurrent_kda_equals_naive_recurrence_and_gate_operator():
    """Plain case: equals the per-token recurrence already pinned above (head-major, K-first state); the in-kernel
    options equal applying the (separately pinned) gate activation, F.normalize and sigmoid outside."""
    gen = torch.Generator().manual_seed(41)
    B, T, H, HV, K, V = 2, 5, 1, 2, 8, 6
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    v = torch.randn(B, T, HV, V, generator=gen)
    g = -torch.rand(B, T, HV, K, generator=gen) * 0.3
    beta = torch.rand(B, T, HV, generator=gen)
    h0 = torch.randn(B, HV, K, V, generator=gen) * 0.5
    out, pool = kda.recurrent_kda(q, k, v, g, beta, h0, scale=0.7)
    hm = lambda t: t.transpose(1, 2)
    o_ref, f_ref = kda.naive_recurrent_kda(hm(q), hm(k), hm(v), hm(g), hm(beta), 0.7, initial_state=h0, output_final_state=True)
    assert torch.allclose(out, hm(o_ref), atol=1e-5) and torch.allclose(pool, f_ref, atol=1e-5)
    # V-first pool: the transposed state
    out2, pool2 = kda.recurrent_kda(q, k, v, g, beta, h0.transpose(-1, -2).contiguous(), scale=0.7, state_v_first=True)
    assert torch.allclose(out2, out, atol=1e-6) and torch.allclose(pool2.transpose(-1, -2), pool, atol=1e-6)
    # in-kernel options
    raw = torch.randn(B, T, HV, K, generator=gen)
    A_log, dt = torch.randn(HV, generator=gen) * 0.3, torch.randn(HV * K, generator=gen) * 0.1
    braw = torch.randn(B, T, HV, generator=gen)
    for safe in (False, True):
        gate = kda.kda_gate(hm(raw), A_log=A_log, dt_bias=dt.view(HV, K), use_gate_in_kernel=True, safe_gate=safe, lower_bound=-3.0)
        want, wpool = kda.recurrent_kda(F.normalize(q, dim=-1), F.normalize(k, dim=-1), v, hm(gate), 2 * torch.sigmoid(braw), h0, scale=0.7)
        got, gpool = kda.recurrent_kda(q, k, v, raw, braw, h0, scale=0.7, A_log=A_log, dt_bias=dt, use_qk_l2norm_in_kernel=True,
                                       use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True,
                                       safe_gate=safe, lower_bound=-3.0)
        assert torch.allclose(got, want, atol=1e-5) and torch.allclose(gpool, wpool, atol=1e-5)


def test_recurrent_kda_slots_and_speculative_decoding():
    """Packed per-token slots: every token's state lands in its slot and one call equals token-by-token calls.
    Speculative rows [seq, step]: a draft / accept loop reproduces the plain recurrence on the accepted stream."""
    gen = torch.Generator().manual_seed(42)
    H, K, V, cap = 2, 8, 6, 9
    cu = [0, 3, 3, 4, 8]
    T = cu[-1]
    q, k, v = (torch.randn(T, H, d, generator=gen) for d in (K, K, V))
    g = -torch.rand(T, H, K, generator=gen) * 0.3
    beta = torch.rand(T, H, generator=gen)
    pool0 = torch.randn(cap, H, V, K, generator=gen) * 0.5
    slots = torch.tensor([4, 4, 7, 1, 0, 2, 2, 5])
    out, pool = kda.recurrent_kda(q, k, v, g, beta, pool0, cu_seqlens=cu, ssm_state_indices=slots, layout="TND", state_v_first=True)
    # token-by-token: each step is its own one-token sequence that starts from the slot the previous token wrote
    p = pool0.clone()
    for n, (s, e) in enumerate(zip(cu, cu[1:])):
        prev = None
        for t in range(s, e):
            if prev is not None and int(slots[t]) != prev:
                p[int(slots[t])] = p[prev]            # the running state moves on to the next slot
            o1, p = kda.recurrent_kda(q[t:t + 1], k[t:t + 1], v[t:t + 1], g[t:t + 1], beta[t:t + 1], p, cu_seqlens=[0, 1],
                                      ssm_state_indices=slots[t:t + 1], layout="TND", state_v_first=True)
            assert torch.allclose(o1[0], out[t], atol=1e-5)
            prev = int(slots[t])
    assert torch.allclose(p[[4, 7, 1, 0, 2, 5]], pool[[4, 7, 1, 0, 2, 5]], atol=1e-5)
    assert torch.equal(pool[[3, 6, 8]], pool0[[3, 6, 8]])            # untouched slots
    # speculative decoding: two sequences, 3 draft steps each, slot rows fixed across calls
    S = 3
    rows = torch.tensor([[0, 1, 2], [3, 4, 5]])
    truth_len = 12
    tq, tk, tv = (torch.randn(2, truth_len, H, d, generator=gen) for d in (K, K, V))
    tg, tb = -torch.rand(2, truth_len, H, K, generator=gen) * 0.3, torch.rand(2, truth_len, H, generator=gen)
    ref, _ = kda.recurrent_kda(tq, tk, tv, tg, tb, torch.zeros(2, H, V, K), state_v_first=True)
    pool = torch.zeros(6, H, V, K)
    pos = [0, 0]
    accepted = None
    for step_accept in ([2, 3], [1, 1], [3, 2]):
        def draft(src, n):
            d = src[n, pos[n]:pos[n] + S].clone()
            d[step_accept[n]:] = torch.randn_like(d[step_accept[n]:])      # rejected tail: garbage
            return d
        dq, dk, dv, dg, db = (torch.stack([draft(t, 0), draft(t, 1)]) for t in (tq, tk, tv, tg, tb))
        db = db.abs().clamp(max=1.0)
        dg = -dg.abs()
        for n in range(2):      # accepted prefix carries the true values
            a = step_accept[n]
            dg[n, :a], db[n, :a] = tg[n, pos[n]:pos[n] + a], tb[n, pos[n]:pos[n] + a]
        kw = {} if accepted is None else dict(num_accepted_tokens=torch.tensor(accepted))
        if accepted is None:
            kw = dict(num_accepted_tokens=torch.tensor([1, 1]))       # slot of step 0 holds the (zero) start state
        o, pool = kda.recurrent_kda(dq, dk, dv, dg, db, pool, ssm_state_indices=rows, state_v_first=True, **kw)
        for n in range(2):
            a = step_accept[n]
            assert torch.allclose(o[n, :a], ref[n, pos[n]:pos[n] + a], atol=1e-5)
            pos[n] += a
        accepted = step_accept


def test_l2norm_against_F_normalize_and_autograd():
    gen = torch.Generator().manual_seed(51)
    x = torch.randn(3, 5, 16, generator=gen, dtype=torch.float64).requires_grad_(True)
    dy = torch.randn(3, 5, 16, generator=gen, dtype=torch.float64)
    y, rstd = gdn.l2norm_fwd(x.detach(), eps=0.0, compute_dtype=torch.float64)
    assert torch.allclose(y, F.normalize(x.detach(), dim=-1), atol=1e-12)          # eps = 0: the unit vector
    assert torch.allclose(rstd, 1.0 / x.detach().norm(dim=-1), atol=1e-12)
    eps = 1e-2                                                                    # a visible eps: the Triton kernel's formula
    ref = x * torch.rsqrt((x * x).sum(-1, keepdim=True) + eps)
    (ref * dy).sum().backward()
    y, rstd = gdn.l2norm_fwd(x.detach(), eps=eps, compute_dtype=torch.float64)
    assert torch.allclose(y, ref.detach(), atol=1e-12)
    # the backward formula drops the eps term of the exact derivative (as the reference kernel does): exact for eps -> 0
    x2 = torch.randn(4, 8, generator=gen, dtype=torch.float64).requires_grad_(True)
    d2 = torch.randn(4, 8, generator=gen, dtype=torch.float64)
    (F.normalize(x2, dim=-1) * d2).sum().backward()
    y2, r2 = gdn.l2norm_fwd(x2.detach(), eps=0.0, compute_dtype=torch.float64)
    assert torch.allclose(gdn.l2norm_bwd(y2, r2, d2, compute_dtype=torch.float64), x2.grad, atol=1e-10)
