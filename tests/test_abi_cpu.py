"""Boundary tests that need no GPU: the shared library loads and exports every symbol that
include/fla_hip.h declares; the ctypes wrappers build exactly one value per C operand, in the
prototype's order and with the prototype's C types; host-side validation rejects bad calls
before any launch.  Modelled on torch_custom/fla_npu/test/test_aclnn_ctypes_abi.py and
test_ascendc_mutation_contract.py."""
import ctypes
import re
from pathlib import Path
from unittest import mock

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "fla_hip.h"


def declared_symbols():
    text = HEADER.read_text()
    return sorted(set(re.findall(r"\b(fla_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    import fla_hip

    return fla_hip.load_library()


def test_library_exports_every_declared_symbol(lib):
    names = declared_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in fla_hip.h but not exported: {missing}"
    assert lib.fla_abi_version() == 1


def test_every_operator_has_a_query_and_a_launch_symbol():
    names = declared_symbols()
    ops = [n[:-len("_get_workspace_size")] for n in names if n.endswith("_get_workspace_size")]
    assert ops and all(op in names for op in ops)


class FakeTensor:
    def __init__(self, shape, dtype=torch.bfloat16):
        self.shape = tuple(shape)
        self.dtype = dtype

    def dim(self):
        return len(self.shape)

    def contiguous(self):
        return self


class FakeCallContext:
    def __init__(self):
        self.names = []

    def tensor(self, tensor, name="tensor"):
        self.names.append(name)
        from fla_hip.ops._runtime import TENSOR_P
        return TENSOR_P()

    def int_array(self, values):
        self.names.append("int_array")
        from fla_hip.ops._runtime import INT_ARRAY_P
        return INT_ARRAY_P()


def capture_call(fn, *args, **kwargs):
    from fla_hip.ops import _hip_ctypes as H

    captured = {}

    def fake_empty(shape, like, **kw):
        return FakeTensor(shape, kw.get("dtype") or like.dtype)

    def fake_empty_like(t, **kw):
        return FakeTensor(t.shape, kw.get("dtype") or t.dtype)

    def fake_call(name, argtypes, build_args, outputs):
        ctx = FakeCallContext()
        captured.update(name=name, argtypes=list(argtypes), args=build_args(ctx), names=ctx.names)
        return outputs

    def fake_empty_ordered_like(like, *, dtype=None, shape=None, device=None):
        return FakeTensor(like.shape if shape is None else shape, dtype or like.dtype)

    with mock.patch.object(H, "_empty", side_effect=fake_empty), \
            mock.patch.object(H, "_empty_like", side_effect=fake_empty_like), \
            mock.patch.object(H, "_empty_ordered_like", side_effect=fake_empty_ordered_like), \
            mock.patch.object(H, "_call_op", side_effect=fake_call), \
            mock.patch.object(H, "_shape", side_effect=lambda t: tuple(t.shape)):
        out = fn(*args, **kwargs)
    return captured, out


def assert_args_match_argtypes(captured):
    assert len(captured["args"]) == len(captured["argtypes"])
    for value, ctype in zip(captured["args"], captured["argtypes"]):
        assert isinstance(value, ctype), (captured["name"], value, ctype)


def test_fwd_h_wrapper_operand_order_and_outputs():
    from fla_hip.ops import _hip_ctypes as H
    k = FakeTensor((1, 2, 130, 128))
    u = FakeTensor((1, 4, 130, 128))
    g = FakeTensor((1, 4, 130), torch.float32)
    cap, out = capture_call(H.npu_chunk_gated_delta_rule_fwd_h, k, u, u, g, output_final_state=True, chunk_size=None)
    assert cap["name"] == "chunk_gated_delta_rule_fwd_h"
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == ["k", "w", "u", "g", "gk", "initial_state", "h", "v_new", "final_state"]
    assert cap["args"][7].value == 64                           # chunk_size=None -> 64 (_aclnn_ctypes.py:572)
    h, v_new, final = out
    assert h.shape == (1, 4, 3, 128, 128) and final.shape == (1, 4, 128, 128) and final.dtype == torch.float32


def test_fwd_h_varlen_shapes_and_state_layout_check():
    from fla_hip.ops import _hip_ctypes as H
    k = FakeTensor((1, 2, 130, 128))
    u = FakeTensor((1, 2, 130, 64))
    g = FakeTensor((1, 2, 130), torch.float32)
    cap, out = capture_call(H.npu_chunk_gated_delta_rule_fwd_h, k, u, u, g, cu_seqlens=[0, 1, 66, 130], state_v_first=True)
    assert out[0].shape == (1, 2, 4, 64, 128) and out[2] is None
    with pytest.raises(RuntimeError, match="initial_state shape does not match state_v_first"):
        capture_call(H.npu_chunk_gated_delta_rule_fwd_h, k, u, u, g, initial_state=FakeTensor((1, 2, 128, 64), torch.float32),
                     state_v_first=True)
    with pytest.raises(RuntimeError, match=r"^npu_chunk_gated_delta_rule_fwd_h: either g or gk must be provided\.$"):
        H.npu_chunk_gated_delta_rule_fwd_h(k, u, u)


@pytest.mark.parametrize("name,args,kwargs", [
    ("npu_chunk_fwd_o", (FakeTensor((1, 2, 64, 128)),) * 3 + (FakeTensor((1, 2, 1, 128, 128)), 0.1), {"g": FakeTensor((1, 2, 64), torch.float32)}),
    ("npu_recompute_w_u_fwd", (FakeTensor((1, 2, 64, 128)), FakeTensor((1, 2, 64, 128)), FakeTensor((1, 2, 64), torch.float32), FakeTensor((1, 2, 64, 64)), 64), {"g": FakeTensor((1, 2, 64), torch.float32)}),
    ("npu_chunk_scaled_dot_kkt", (FakeTensor((1, 2, 64, 128)), FakeTensor((1, 2, 64), torch.float32), FakeTensor((1, 2, 64), torch.float32)), {}),
    ("npu_solve_tri", (FakeTensor((1, 64, 2, 64)),), {}),
    ("npu_chunk_local_cumsum", (FakeTensor((1, 2, 64), torch.float32), 64), {}),
    ("npu_causal_conv1d", (FakeTensor((2, 8, 32)), FakeTensor((4, 32))), {"head_num": 2}),
])
def test_wrappers_build_one_value_per_c_operand(name, args, kwargs):
    from fla_hip.ops import _hip_ctypes as H
    cap, _ = capture_call(getattr(H, name), *args, **kwargs)
    assert_args_match_argtypes(cap)
    assert cap["argtypes"] == H.OP_ARGTYPES[cap["name"]]


def test_defaults_follow_the_reference():
    import inspect
    from fla_hip.ops import _hip_ctypes as H
    sig = inspect.signature(H.npu_chunk_local_cumsum)
    assert sig.parameters["output_dtype"].default == "float32" and sig.parameters["head_first"].default is True
    assert inspect.signature(H.npu_chunk_scaled_dot_kkt).parameters["chunk_size"].default == 64
    assert inspect.signature(H.npu_solve_tri).parameters["layout"].default == "bsnd"
    assert inspect.signature(H.npu_recurrent_gated_delta_rule).parameters["scale"].default == 1.0
    cap, out = capture_call(H.npu_causal_conv1d, FakeTensor((2, 8, 32)), FakeTensor((4, 32)), head_num=2)
    assert out.shape == (2, 2, 8, 16)                           # [B, head_num, S, D/head_num]


def test_public_namespace_and_mutation_contract():
    from fla_hip import ops
    for name in ("npu_causal_conv1d", "causal_conv1d", "npu_recurrent_gated_delta_rule", "recurrent_gated_delta_rule",
                 "npu_chunk_fwd_o", "chunk_fwd_o", "npu_solve_tri", "chunk_local_cumsum", "chunk_scaled_dot_kkt",
                 "recompute_w_u_fwd", "chunk_gated_delta_rule_fwd_h"):
        assert callable(getattr(ops, name))
    assert ops.MUTATED_ARGUMENTS["recurrent_gated_delta_rule"] == ("state",)
    assert ops.MUTATED_ARGUMENTS["causal_conv1d"] == ("conv_states",)
    with pytest.raises(NotImplementedError):
        ops.npu_fast_gelu_custom(torch.zeros(1))
    state = torch.zeros(1, 1, 4, 4, requires_grad=True)
    with pytest.raises(RuntimeError, match="mutates state in place"):
        ops.recurrent_gated_delta_rule(None, None, None, state, beta=None, actual_seq_lengths=None,
                                       ssm_state_indices=None, g=torch.zeros(1))


def test_recurrent_kda_mutation_follows_the_inplace_flag():
    """`npu_recurrent_kda` overwrites its state pool only with inplace_final_state (MUTATION_PREDICATES,
    ops/ascendc/__init__.py:61-71): then a pool that requires grad is rejected and the version counter of the pool
    is bumped after the call; with the flag off neither happens."""
    from fla_hip import ops
    from fla_hip.ops import _hip_ctypes as H
    assert ops.MUTATED_ARGUMENTS["npu_recurrent_kda"] == ("initial_state",)
    assert ops.MUTATION_PREDICATES["npu_recurrent_kda"]({"inplace_final_state": True}) is True
    assert ops.MUTATION_PREDICATES["npu_recurrent_kda"]({"inplace_final_state": 0}) is False
    calls = []
    guarded = ops._wrap_mutable_op("npu_recurrent_kda", lambda q, k, v, g, beta, initial_state=None, *,
                                   inplace_final_state=True, **kw: calls.append(inplace_final_state) or "out")
    pool = torch.zeros(2, 1, 4, 4, requires_grad=True)
    with pytest.raises(RuntimeError, match="npu_recurrent_kda mutates initial_state in place"):
        guarded(None, None, None, None, None, pool)
    assert not calls                                                    # rejected before the operator ran
    assert guarded(None, None, None, None, None, pool, inplace_final_state=False) == "out"
    plain = torch.zeros(2, 1, 4, 4)
    before = plain._version
    guarded(None, None, None, None, None, plain, inplace_final_state=False)
    assert plain._version == before                                     # not written: no bump
    guarded(None, None, None, None, None, plain)
    assert plain._version == before + 1
    assert calls == [False, False, True]
    # the exported operator is the guarded one
    assert ops.npu_recurrent_kda is ops.recurrent_kda and ops.npu_recurrent_kda is not H.npu_recurrent_kda


def test_recurrent_wrapper_requires_a_gate_before_any_launch():
    from fla_hip.ops import _hip_ctypes as H
    with mock.patch.object(H, "_call_op") as call:
        with pytest.raises(RuntimeError, match=r"^npu_recurrent_gated_delta_rule: either g or gk must be provided\.$"):
            H.npu_recurrent_gated_delta_rule(None, None, None, None, beta=None, actual_seq_lengths=None,
                                             ssm_state_indices=None)
    call.assert_not_called()


def test_library_rejects_null_and_bad_descriptors_without_a_gpu(lib):
    """Status codes and fla_last_error() for calls that fail validation (no launch happens)."""
    from fla_hip.ops._runtime import FlaTensor, TENSOR_P, INT_ARRAY_P
    lib.fla_last_error.restype = ctypes.c_char_p
    ws = ctypes.c_uint64(0)
    fn = lib.fla_chunk_scaled_dot_kkt_get_workspace_size
    fn.restype = ctypes.c_int
    fn.argtypes = [TENSOR_P, TENSOR_P, TENSOR_P, INT_ARRAY_P, INT_ARRAY_P, ctypes.c_int64, TENSOR_P,
                   ctypes.POINTER(ctypes.c_uint64)]
    assert fn(TENSOR_P(), TENSOR_P(), TENSOR_P(), INT_ARRAY_P(), INT_ARRAY_P(), 64, TENSOR_P(), ctypes.byref(ws)) == 1
    assert b"k must not be null" in lib.fla_last_error()
    t = FlaTensor()
    t.data = 16
    t.dtype = 0          # fp32 where bf16 is required
    t.ndim = 4
    for i, d in enumerate((1, 1, 64, 128)):
        t.shape[i] = d
    assert fn(ctypes.pointer(t), TENSOR_P(), TENSOR_P(), INT_ARRAY_P(), INT_ARRAY_P(), 64, TENSOR_P(), ctypes.byref(ws)) == 2
    assert fn(ctypes.pointer(t), TENSOR_P(), TENSOR_P(), INT_ARRAY_P(), INT_ARRAY_P(), 32, TENSOR_P(), ctypes.byref(ws)) == 4
    assert b"chunk_size must be 64" in lib.fla_last_error()


def _descriptor(shape, dtype_code, data=4096, strides=None):
    """A descriptor over a pointer that is never dereferenced (validation and size queries only)."""
    from fla_hip.ops._runtime import FlaTensor
    t = FlaTensor()
    t.data, t.dtype, t.ndim = data, dtype_code, len(shape)
    st = 1
    for i in reversed(range(len(shape))):
        t.shape[i] = shape[i]
        t.stride[i] = st if strides is None else strides[i]
        st *= shape[i]
    return t


def test_value_slab_workspace_and_new_entries_without_a_gpu(lib):
    """Size queries and validation of the entry points that loop value slabs or serve the prefill route; nothing is
    launched.  chunk_bwd_dqkwg with 128-token chunks and V = 256 asks for room for the second pass (dq, dk, dw in the
    element type and dg in fp32, each rounded up to 256 bytes)."""
    from fla_hip.ops._runtime import TENSOR_P, INT_ARRAY_P
    from fla_hip.ops import _hip_ctypes as H
    lib.fla_last_error.restype = ctypes.c_char_p
    BF, F32, I32 = 2, 0, 3
    p = ctypes.pointer
    B, Hh, T, K, V = 1, 2, 256, 128, 256
    qk = _descriptor((B, Hh, T, K), BF)
    vv = _descriptor((B, Hh, T, V), BF)
    g = _descriptor((B, Hh, T), F32)
    h = _descriptor((B, Hh, 2, K, V), BF)
    ws = ctypes.c_uint64(0)
    fn = lib.fla_chunk_bwd_dqkwg_get_workspace_size
    fn.restype = ctypes.c_int
    fn.argtypes = [*H.OP_ARGTYPES["chunk_bwd_dqkwg"], ctypes.POINTER(ctypes.c_uint64)]
    null, nia = TENSOR_P(), INT_ARRAY_P()
    args = [p(qk), p(qk), p(vv), p(g), p(h), p(vv), p(h), p(vv), nia, nia, null, null, 1.0, 128, False, False,
            p(qk), p(qk), p(qk), p(g)]
    assert fn(*args, ctypes.byref(ws)) == 0, lib.fla_last_error()
    assert ws.value == 3 * B * Hh * T * K * 2 + B * Hh * T * 4
    args[13] = 64                                     # 64-token chunks: one pass, the kernel walks both slabs itself
    h64 = _descriptor((B, Hh, 4, K, V), BF)
    args[4] = args[6] = p(h64)
    assert fn(*args, ctypes.byref(ws)) == 0 and ws.value == 0

    fn = lib.fla_gdn_chunk_fwd_state_pool_get_workspace_size
    fn.restype = ctypes.c_int
    fn.argtypes = [*H.OP_ARGTYPES["gdn_chunk_fwd_state_pool"], ctypes.POINTER(ctypes.c_uint64)]
    q4 = _descriptor((1, Hh, T, K), BF)
    gate = _descriptor((1, T, Hh), F32)
    o = _descriptor((1, T, Hh, K), BF)
    pool = _descriptor((5, Hh, K, K), F32, strides=(Hh * K * K, K * K, 1, K))      # V-first rows seen as [rows,H,K,V]
    idx = _descriptor((1,), I32)
    assert fn(p(q4), p(q4), p(q4), p(gate), p(gate), 0.1, p(pool), null, nia, 64, False, p(o), ctypes.byref(ws)) == 1
    assert b"state_indices must not be null" in lib.fla_last_error()
    assert fn(p(q4), p(q4), p(q4), p(gate), p(gate), 0.1, p(pool), p(idx), nia, 64, False, p(o), ctypes.byref(ws)) == 0
    bad_pool = _descriptor((5, Hh, K, K), F32, strides=(Hh * K * K, K * K, 2 * K, 2))
    assert fn(p(q4), p(q4), p(q4), p(gate), p(gate), 0.1, p(bad_pool), p(idx), nia, 64, False, p(o), ctypes.byref(ws)) == 3
    two = _descriptor((2,), I32)                     # one sequence, two indices
    assert fn(p(q4), p(q4), p(q4), p(gate), p(gate), 0.1, p(pool), p(two), nia, 64, False, p(o), ctypes.byref(ws)) == 3

    plan = lib.fla_recurrent_gdn_prefill_plan
    plan.restype = ctypes.c_int
    plan.argtypes = [*H.OP_ARGTYPES["recurrent_gdn_prefill_plan"], ctypes.c_void_p]
    lens = _descriptor((9000,), I32)
    assert plan(p(lens), p(idx), 4, p(_descriptor((8999,), I32)), p(_descriptor((17999,), I32)), None) == 4
    assert b"between 1 and 8192 sequences" in lib.fla_last_error()
    lens = _descriptor((3,), I32)
    assert plan(p(lens), p(idx), 4, p(_descriptor((2,), I32)), p(_descriptor((4,), I32)), None) == 3   # report must be [2B+1]
    assert plan(p(lens), p(idx), 0, p(_descriptor((2,), I32)), p(_descriptor((5,), I32)), None) == 3   # empty pool

    fn = lib.fla_chunk_kda_bwd_dqkwg_wy_intra_get_workspace_size
    fn.restype = ctypes.c_int
    fn.argtypes = [*H.OP_ARGTYPES["chunk_kda_bwd_dqkwg_wy_intra"], ctypes.POINTER(ctypes.c_uint64)]
    T2 = 128
    x = _descriptor((1, Hh, T2, K), BF)
    f = _descriptor((1, Hh, T2, K), F32)
    a = _descriptor((1, Hh, T2, 64), BF)
    hb = _descriptor((1, Hh, 2, K, K), BF)
    beta = _descriptor((1, Hh, T2), F32)
    db = _descriptor((1, Hh, T2), F32)
    base = [p(x), p(x), p(x), p(f), p(hb), p(x), p(hb), p(x), p(x), p(beta), p(a), nia, nia, 0.1, 64]
    assert fn(*base, p(f), p(f), p(f), p(x), p(db), ctypes.byref(ws)) == 0, lib.fla_last_error()
    assert fn(*base, p(x), p(x), p(f), p(x), p(db), ctypes.byref(ws)) == 0          # dq, dk in the element type
    assert fn(*base, p(x), p(f), p(f), p(x), p(db), ctypes.byref(ws)) == 2          # one of each
    assert b"dq and dk must share one dtype" in lib.fla_last_error()


def test_cpu_tensors_are_rejected():
    from fla_hip import ops
    x = torch.zeros(1, 4, 16, dtype=torch.bfloat16)
    with pytest.raises(TypeError, match="ROCm GPU tensor"):
        ops.causal_conv1d(x, torch.zeros(4, 16, dtype=torch.bfloat16))


# ---------------------------------------------------------------------------------------------
# KDA-side wrappers
# ---------------------------------------------------------------------------------------------
class FakeFloatTensor(FakeTensor):
    device = "cuda:0"

    def is_contiguous(self):
        return True


def test_kda_fwd_wrapper_operands_shapes_and_output_policy():
    """Operand order of fla_chunk_kda_fwd (= aclnnChunkKdaFwd, _aclnn_ctypes.py:1230-1262) and the
    12-value visibility mask (_kda_policy.py:16-39)."""
    from fla_hip.ops import _hip_ctypes as H
    B, T, Hk, HV, K, V = 2, 130, 2, 4, 128, 256
    q = FakeTensor((B, T, Hk, K))
    v = FakeTensor((B, T, HV, V))
    g = FakeTensor((B, T, HV, K), torch.float32)
    beta = FakeTensor((B, T, HV), torch.float32)
    cap, out = capture_call(H.npu_chunk_kda_fwd, q, q, v, g, beta, 0.1, 64, output_final_state=True,
                            disable_recompute=True, state_v_first=True)
    assert cap["name"] == "chunk_kda_fwd"
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == [
        "q", "k", "v", "g", "beta", "A_log", "dt_bias", "initial_state", "attn_out", "final_state", "gk", "Aqk", "Akk",
        "w", "u", "qg", "kg", "v_new", "h"]
    assert cap["args"][10].value == b"BSND" and cap["args"][12].value == 64 and cap["args"][16].value is True
    o, final, gk, aqk, akk, w, u, qg, kg, v_new, h, init = out
    assert o.shape == (B, T, HV, V) and final.shape == (B, HV, V, K) and final.dtype == torch.float32
    assert gk.shape == (B, HV, T, K) and gk.dtype == torch.float32
    assert aqk.shape == akk.shape == (B, HV, T, 64)
    assert w.shape == qg.shape == kg.shape == (B, HV, T, K) and u.shape == v_new.shape == (B, HV, T, V)
    assert h.shape == (B, 3, HV, V, K) and init is None
    # rank-3 layouts, varlen chunk count, hidden outputs
    cu = [0, 1, 66, 130]
    q3, v3 = FakeTensor((Hk, T, K)), FakeTensor((HV, T, V))
    g3, b3 = FakeTensor((HV, T, K), torch.float32), FakeTensor((HV, T), torch.float32)
    cap, out = capture_call(H.npu_chunk_kda_fwd, q3, q3, v3, g3, b3, 0.1, layout="NTD", cu_seqlens=cu,
                            return_intermediate_states=True)
    assert out[0].shape == (HV, T, V) and out[10].shape == (4, HV, K, V) and out[1] is None and out[5] is None
    assert H.kda_fwd_optional_output_mask(output_final_state=False, use_gate_in_kernel=True, disable_recompute=False,
                                          return_intermediate_states=False) == (
        True, False, False, True, True, False, False, False, False, False, False, True)


@pytest.mark.parametrize("kwargs,match", [
    (dict(layout="bsnd"), "layout must be uppercase"),
    (dict(chunk_size=32), "chunk_size must be 64 or 128"),
    (dict(layout="TND"), "rank does not match layout"),
    (dict(use_gate_in_kernel=True), "A_log must be float32"),
    (dict(cu_seqlens=[0, 70, 60, 130]), "cu_seqlens must be nondecreasing"),
    (dict(cu_seqlens=[0, 130], chunk_indices=[0, 1, 0, 0, 0, 2]), "canonical sequence-major order"),
    (dict(initial_state=FakeTensor((1, 2, 64, 128), torch.float32)), "initial_state shape/dtype"),
])
def test_kda_fwd_wrapper_rejects_bad_calls_before_launch(kwargs, match):
    from fla_hip.ops import _hip_ctypes as H
    q = FakeTensor((1, 130, 2, 128))
    g = FakeTensor((1, 130, 2, 128), torch.float32)
    beta = FakeTensor((1, 130, 2), torch.float32)
    kw = dict(chunk_size=64)
    kw.update(kwargs)
    with pytest.raises(RuntimeError, match=match):
        capture_call(H.npu_chunk_kda_fwd, q, q, q, g, beta, 0.1, **kw)


def test_kda_gate_and_bwd_wrappers_operands():
    from fla_hip.ops import _hip_ctypes as H
    g = FakeTensor((1, 2, 130, 128), torch.float32)
    cap, out = capture_call(H.npu_kda_gate_cumsum, g, 64, A_log=FakeTensor((2,), torch.float32), use_gate_in_kernel=True,
                            safe_gate=True)
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == ["g", "A_log", "dt_bias", "gk"]
    assert cap["args"][7].value == -5.0 and out.dtype == torch.float32       # lower_bound default (_aclnn_ctypes.py:1292)

    q = FakeTensor((1, 2, 130, 128))
    dv = FakeTensor((1, 4, 130, 64))
    gK = FakeTensor((1, 4, 130, 128), torch.float32)
    cap, (dh, dh0, dv2) = capture_call(H.npu_chunk_gated_delta_rule_bwd_dhu, q, q, FakeTensor((1, 4, 130, 128)), dv, dv,
                                       0.1, 64, gK=gK, h0=FakeTensor((1, 4, 128, 64), torch.float32), use_exp2=None)
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == ["q", "k", "w", "d_o", "dv", "g", "gK", "h0", "dht", "dh", "dh0", "dv2"]
    assert cap["args"][13].value is True                                     # use_exp2=None resolves to "gK given"
    assert dh.shape == dh0.shape == (1, 4, 3, 128, 64) and dv2.shape == dv.shape
    with pytest.raises(ValueError, match="Exactly one of g and gK"):
        capture_call(H.npu_chunk_gated_delta_rule_bwd_dhu, q, q, q, dv, dv, 0.1, 64)
    with pytest.raises(ValueError, match="use_exp2 must be true"):
        capture_call(H.npu_chunk_gated_delta_rule_bwd_dhu, q, q, q, dv, dv, 0.1, 64, gK=gK, use_exp2=False)

    T, Hh, K = 65, 3, 128
    f32 = torch.float32
    mk = lambda shape, dt=f32: FakeFloatTensor(shape, dt)
    qk = mk((1, Hh, T, K), torch.bfloat16)
    args = (qk, qk, mk((1, Hh, T, K)), mk((1, Hh, T), torch.bfloat16), mk((1, Hh, T, 64)), mk((1, Hh, T, 64)),
            mk((1, Hh, T, K)), mk((1, Hh, T, K)), mk((1, Hh, T)), mk((1, Hh, T, K)))
    cap, outs = capture_call(H.npu_chunk_kda_bwd_intra, *args, layout="BNSD")
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == [
        "q", "k", "gk", "beta", "dAqk", "dAkk", "dq", "dk", "db", "dg", "dq_out", "dk_out", "db_out", "dg_out"]
    assert cap["args"][13].value is True and cap["args"][14].value == b"BNSD"
    assert [o.shape for o in outs] == [(1, Hh, T, K), (1, Hh, T, K), (1, Hh, T), (1, Hh, T, K)]
    with pytest.raises(RuntimeError, match="safe_gate=False is reserved"):
        capture_call(H.npu_chunk_kda_bwd_intra, *args, layout="BNSD", safe_gate=False)
    with pytest.raises(RuntimeError, match="TND requires cu_seqlens"):
        capture_call(H.npu_chunk_kda_bwd_intra, *[mk(t.shape[1:], t.dtype) for t in args], layout="TND")
    with pytest.raises(RuntimeError, match="varlen supports TND or BSND"):
        capture_call(H.npu_chunk_kda_bwd_intra, *args, layout="BNSD", cu_seqlens=[0, T])


def test_gdn_backward_wrappers_operands_and_outputs():
    """Operand order equals the aclnn prototypes (_aclnn_ctypes.py:242-279, 397-510); dq / dk take the key-head
    shape, dw the value-head count, and the fp32 side outputs come back in the dtype of beta / g."""
    from fla_hip.ops import _hip_ctypes as H
    B, Hk, Hv, T, K, V = 1, 2, 4, 130, 128, 64
    f32 = torch.float32
    q = FakeFloatTensor((B, Hk, T, K), torch.bfloat16)
    v = FakeFloatTensor((B, Hv, T, V), torch.bfloat16)
    w = FakeFloatTensor((B, Hv, T, K), torch.bfloat16)
    g = FakeFloatTensor((B, Hv, T), f32)
    A = FakeFloatTensor((B, Hv, T, 64), torch.bfloat16)
    h = FakeFloatTensor((B, Hv, 3, K, V), torch.bfloat16)

    cap, out = capture_call(H.npu_chunk_bwd_dv_local, q, q, v, g, 0.1, 64, A=A)
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == ["q", "k", "d_o", "g", "g_gamma", "A", "out"]
    assert out.shape == v.shape and cap["args"][8].value == pytest.approx(0.1) and cap["args"][9].value == 64
    with pytest.raises(NotImplementedError, match="g_gamma"):
        capture_call(H.npu_chunk_bwd_dv_local, q, q, v, g, 0.1, 64, g_gamma=g)

    cap, (dq, dk, dw, dg) = capture_call(H.npu_chunk_bwd_dqkwg, q, q, v, g, h, v, h, v, 64, scale=0.25)
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == [
        "q", "k", "v", "g", "h", "dox", "dh", "dv", "w", "g_gamma", "dq", "dk", "dw", "dg"]
    assert dq.shape == dk.shape == q.shape and dw.shape == (B, Hv, T, K) and dg.shape == g.shape and dg.dtype == f32
    assert cap["args"][12].value == 0.25 and cap["args"][14].value is False and cap["args"][15].value is False
    cap, _ = capture_call(H.npu_chunk_bwd_dqkwg, q, q, v, g, h, v, h, v, 64)
    assert cap["args"][12].value == 1.0                                      # scale=None -> 1.0 (_aclnn_ctypes.py:501)

    cap, dA = capture_call(H.npu_prepare_wy_repr_bwd_da, q, v, g, A, w, v, g, chunk_size=64)
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == ["k", "v", "beta", "A", "dw", "du", "g", "dA"]
    assert dA.shape == A.shape and dA.dtype == A.dtype

    cap, (dk2, dv2, db, dg2) = capture_call(H.npu_prepare_wy_repr_bwd_full, q, v, g, A, A, w, v, g, 64)
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == [
        "k", "v", "beta", "A", "dA", "dw", "du", "g", "dk", "dv", "dbeta", "dg"]
    assert dk2.shape == q.shape and dv2.shape == v.shape and db.shape == g.shape and dg2.shape == g.shape
    assert db.dtype == f32 and dg2.dtype == f32

    cap, (dk2, dv2, db, dg2) = capture_call(H.npu_prepare_wy_repr_bwd, q, v, g, A, w, v, g, 64)    # :284-321
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == [
        "k", "v", "beta", "A", "dw", "du", "g", "dk", "dv", "dbeta", "dg"]
    assert dk2.shape == q.shape and dv2.shape == v.shape and db.shape == g.shape and dg2.dtype == f32


def test_backward_ops_are_exported_under_both_names():
    from fla_hip import ops
    for name in ("chunk_bwd_dv_local", "chunk_bwd_dqkwg", "prepare_wy_repr_bwd_da", "prepare_wy_repr_bwd_full",
                 "prepare_wy_repr_bwd"):
        assert getattr(ops, name) is getattr(ops, "npu_" + name)


def test_conv1d_bwd_and_recurrent_kda_wrappers_operands():
    """Operand order of fla_causal_conv1d_bwd (= aclnnCausalConv1dBwd, _aclnn_ctypes.py:988-1037) and of
    fla_recurrent_kda (= aclnnRecurrentKda, :1468-1493); pre-launch checks of the recurrent wrapper."""
    from fla_hip.ops import _hip_ctypes as H
    x = FakeFloatTensor((2, 9, 32), torch.bfloat16)
    w = FakeFloatTensor((4, 32), torch.bfloat16)
    cap, (dx, dw, db, dh0) = capture_call(H.npu_causal_conv1d_bwd, x, None, w, x, input_layout="BSH")
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"] if n != "int_array"] == ["x", "y", "weight", "dy", "initial_state", "dht", "dx", "dw", "db", "dh0"]
    assert cap["args"][7].value == 0 and cap["args"][8].value == b"BSH"
    assert dx.shape == x.shape and dw.shape == w.shape and db.shape == (32,) and dh0.shape == (2, 4, 32)
    cap, (_, _, _, dh0) = capture_call(H.npu_causal_conv1d_bwd, FakeFloatTensor((18, 32)), None, w, FakeFloatTensor((2, 18, 16)),
                                       query_start_loc=[0, 5, 9, 18], input_layout="NTD")
    assert dh0.shape == (3, 4, 32)
    with pytest.raises(RuntimeError, match="query_start_loc is required for TND"):
        capture_call(H.npu_causal_conv1d_bwd, FakeFloatTensor((18, 32)), None, w, FakeFloatTensor((18, 32)), input_layout="TND")


class FakeDevTensor(FakeFloatTensor):
    def __init__(self, shape, dtype=torch.bfloat16, device="cuda:0"):
        super().__init__(shape, dtype)
        self.device = device

    def numel(self):
        n = 1
        for d in self.shape:
            n *= d
        return n


def test_recurrent_kda_wrapper_checks_and_operands():
    from fla_hip.ops import _hip_ctypes as H
    B, T, Hh, HV, K, V = 2, 2, 2, 4, 128, 128
    q = FakeDevTensor((B, T, Hh, K))
    v = FakeDevTensor((B, T, HV, V))
    g = FakeDevTensor((B, T, HV, K), torch.float32)
    beta = FakeDevTensor((B, T, HV), torch.float32)
    state = FakeDevTensor((B, HV, V, K), torch.float32)
    A_log = FakeDevTensor((HV,), torch.float32)
    cap, (out, final) = capture_call(H.npu_recurrent_kda, q, q, v, g, beta, state, A_log=A_log, use_gate_in_kernel=True,
                                     output_final_state=True, state_v_first=True)
    assert_args_match_argtypes(cap)
    assert [n for n in cap["names"]] == ["q", "k", "v", "g", "beta", "initial_state", "cu_seqlens", "ssm_state_indices", "A_log",
                                         "dt_bias", "num_accepted_tokens", "attn_out", "final_state"]
    assert cap["args"][11].value == b"BSND" and cap["args"][12].value == pytest.approx(K ** -0.5)
    assert cap["args"][13].value is True and cap["args"][14].value is True            # output_final_state, inplace default
    assert cap["args"][20].value == -5.0 and cap["args"][21].value is True            # lower_bound default, state_v_first
    assert out.shape == v.shape and final is state
    _, (_, final) = capture_call(H.npu_recurrent_kda, q, q, v, g, beta, state, state_v_first=True)
    assert final is None                                                               # output_final_state defaults to False
    for kwargs, match in (
        (dict(layout="BNSD"), "layout must be BSND or TND"),
        (dict(layout="TND"), "layout/rank mismatch"),
        (dict(state_v_first=True, safe_gate=True), "require use_gate_in_kernel=True"),
        (dict(state_v_first=True, use_gate_in_kernel=True), r"A_log must be FP32 \[HV\]"),
        (dict(state_v_first=True, use_gate_in_kernel=True, A_log=A_log, safe_gate=True, lower_bound=-6.0), r"lower_bound must be in \[-5,0\)"),
        (dict(state_v_first=True, num_accepted_tokens=FakeDevTensor((B,), torch.int32)), "requires ssm_state_indices"),
    ):
        with pytest.raises(RuntimeError, match=match):
            capture_call(H.npu_recurrent_kda, q, q, v, g, beta, state, **kwargs)
    with pytest.raises(RuntimeError, match="inplace_final_state=True requires initial_state"):
        capture_call(H.npu_recurrent_kda, q, q, v, g, beta, None)
    with pytest.raises(RuntimeError, match="HV must be divisible by H"):
        capture_call(H.npu_recurrent_kda, FakeDevTensor((B, T, 3, K)), FakeDevTensor((B, T, 3, K)), v, g, beta, state, state_v_first=True)


def test_bench_refuses_more_than_one_gpu():
    """This build runs on one GPU: bench.py --gpus N > 1 exits with a message instead of timing anything."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_outputs_follow_the_memory_order_of_their_inputs():
    """dq, dk, dv of the GDN backward operators are allocated in the memory order of q, k, v: contiguous for the
    reference's contiguous [B,H,T,D] operands, a token-major view for ``x.transpose(1, 2)`` of a [B,T,H,D] tensor, so
    that the gradient passes back through the transpose without a copy."""
    from fla_hip.ops import _hip_ctypes as H
    x = torch.empty(2, 3, 5, 8)
    y = H._empty_ordered_like(x)
    assert y.shape == x.shape and y.is_contiguous()
    xt = torch.empty(2, 5, 3, 8).transpose(1, 2)            # [B,H,T,D] view of token-major memory
    yt = H._empty_ordered_like(xt, dtype=torch.float32)
    assert yt.shape == xt.shape and yt.stride() == xt.stride() and yt.dtype == torch.float32
    assert yt.transpose(1, 2).is_contiguous()
    z = H._empty_ordered_like(xt, shape=(2, 3, 5, 16))
    assert z.shape == (2, 3, 5, 16) and z.transpose(1, 2).is_contiguous()
