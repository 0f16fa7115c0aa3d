"""ctypes runtime for ``libfla_hip.so``: tensor / int-array descriptors, device
guard, stream lookup, the two-phase call and status handling.

Counterpart of torch_custom/fla_npu/fla_npu/ops/ascendc/_runtime.py (descriptor
construction :210-273, device guard :153-174, stream pointer :177-188, two-phase
call :388-429, entry ``call_aclnn`` :463-482).
"""
from __future__ import annotations

import ctypes
from typing import Callable, Iterable, Optional, Sequence

FLA_MAX_DIMS = 8
FLA_OK = 0

# fla_dtype values of include/fla_hip.h
_DTYPE_CODES = {"float32": 0, "float16": 1, "bfloat16": 2, "int32": 3, "int64": 4}


class FlaTensor(ctypes.Structure):
    """Mirror of ``struct fla_tensor``."""

    _fields_ = [
        ("data", ctypes.c_void_p),
        ("dtype", ctypes.c_int32),
        ("ndim", ctypes.c_int32),
        ("shape", ctypes.c_int64 * FLA_MAX_DIMS),
        ("stride", ctypes.c_int64 * FLA_MAX_DIMS),
    ]


class FlaIntArray(ctypes.Structure):
    """Mirror of ``struct fla_int_array``."""

    _fields_ = [("data", ctypes.POINTER(ctypes.c_int64)), ("size", ctypes.c_uint64)]


TENSOR_P = ctypes.POINTER(FlaTensor)
INT_ARRAY_P = ctypes.POINTER(FlaIntArray)


def dtype_code(dtype) -> int:
    name = str(dtype).removeprefix("torch.")
    try:
        return _DTYPE_CODES[name]
    except KeyError:
        raise TypeError(f"fla_hip: unsupported tensor dtype {dtype}.") from None


def shape(tensor) -> tuple:
    return tuple(int(d) for d in tensor.shape)


def ensure_gpu_tensor(tensor, name: str):
    import torch

    if not isinstance(tensor, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(tensor)!r}.")
    if tensor.device.type != "cuda":
        raise TypeError(f"{name} must be a ROCm GPU tensor (device 'cuda'), got device {tensor.device}.")
    return tensor


def empty(shape_: Iterable[int], like, *, dtype=None):
    import torch

    return torch.empty(tuple(int(d) for d in shape_), device=like.device, dtype=dtype or like.dtype)


def empty_like(tensor, *, dtype=None):
    import torch

    return torch.empty_like(tensor, dtype=dtype or tensor.dtype, memory_format=torch.contiguous_format)


class CallContext:
    """Builds and keeps alive the descriptors of one library call."""

    def __init__(self, device):
        self.device = device
        self.keepalive = []

    def tensor(self, tensor, name: str = "tensor"):
        if tensor is None:
            return TENSOR_P()
        tensor = ensure_gpu_tensor(tensor, name)
        if tensor.device != self.device:
            raise ValueError(
                f"{name} must be on {self.device}, got {tensor.device}; "
                "one call cannot mix tensors from different devices."
            )
        if tensor.dim() > FLA_MAX_DIMS:
            raise ValueError(f"{name} has rank {tensor.dim()} > {FLA_MAX_DIMS}.")
        desc = FlaTensor()
        desc.data = tensor.data_ptr()
        desc.dtype = dtype_code(tensor.dtype)
        desc.ndim = tensor.dim()
        for i, (d, s) in enumerate(zip(tensor.shape, tensor.stride())):
            desc.shape[i] = int(d)
            desc.stride[i] = int(s)
        self.keepalive.append(desc)
        self.keepalive.append(tensor)
        return ctypes.pointer(desc)

    def int_array(self, values: Optional[Sequence[int]]):
        if values is None:
            return INT_ARRAY_P()
        import torch

        if isinstance(values, torch.Tensor):
            values = values.detach().cpu().flatten().tolist()
        values = tuple(int(v) for v in values)
        if not values:
            return INT_ARRAY_P()
        buf = (ctypes.c_int64 * len(values))(*values)
        desc = FlaIntArray(ctypes.cast(buf, ctypes.POINTER(ctypes.c_int64)), len(values))
        self.keepalive.append(buf)
        self.keepalive.append(desc)
        return ctypes.pointer(desc)


def _first_tensor(outputs):
    import torch

    if isinstance(outputs, torch.Tensor):
        return outputs
    if isinstance(outputs, (tuple, list)):
        for item in outputs:
            found = _first_tensor(item)
            if found is not None:
                return found
    return None


_LIB = None
_BOUND = {}


def _library():
    global _LIB
    if _LIB is None:
        import fla_hip

        _LIB = fla_hip.load_library()
    return _LIB


def _bind(name: str, argtypes: Sequence):
    """Bind ``fla_<name>_get_workspace_size`` and ``fla_<name>`` with explicit argtypes."""
    bound = _BOUND.get(name)
    if bound is None:
        lib = _library()
        query = getattr(lib, f"fla_{name}_get_workspace_size")
        launch = getattr(lib, f"fla_{name}")
        query.argtypes = [*argtypes, ctypes.POINTER(ctypes.c_uint64)]
        query.restype = ctypes.c_int
        launch.argtypes = [*argtypes, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
        launch.restype = ctypes.c_int
        bound = _BOUND[name] = (query, launch)
    return bound


def last_error() -> str:
    msg = _library().fla_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def call_op(name: str, argtypes: Sequence, build_args: Callable[[CallContext], list], outputs):
    """Two-phase call of operator ``name`` on the device of ``outputs``.

    Phase 1 asks for the workspace size, the workspace is a ``uint8`` tensor from
    torch's caching allocator on that device, phase 2 enqueues on the current
    stream of that device.  Nothing synchronises; descriptor memory is released
    when this function returns (the library has consumed it by then).
    """
    import torch

    anchor = _first_tensor(outputs)
    if anchor is None:
        raise RuntimeError(f"fla_{name}: no output tensor to take the device from.")
    ensure_gpu_tensor(anchor, "output")
    device = anchor.device
    query, launch = _bind(name, argtypes)
    with torch.cuda.device(device):
        ctx = CallContext(device)
        args = build_args(ctx)
        ws_size = ctypes.c_uint64(0)
        status = query(*args, ctypes.byref(ws_size))
        if status != FLA_OK:
            raise RuntimeError(f"fla_{name}_get_workspace_size failed with status={status}: {last_error()}")
        workspace = None
        ws_ptr = ctypes.c_void_p()
        if ws_size.value:
            workspace = torch.empty(int(ws_size.value), dtype=torch.uint8, device=device)
            ws_ptr = ctypes.c_void_p(workspace.data_ptr())
        stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
        status = launch(*args, ws_ptr, ws_size, stream)
        if status != FLA_OK:
            raise RuntimeError(f"fla_{name} failed with status={status}: {last_error()}")
        del workspace  # stream-ordered reuse by the caching allocator keeps this safe
    return outputs


def call_op_noalloc(name: str, argtypes: Sequence, build_args: Callable[[CallContext], list], outputs):
    """One-phase call of ``fla_<name>(<operands>, stream)``: an entry point that brings its own scratch memory.
    Nothing is allocated here or inside the library; the caller has allocated ``outputs``."""
    import torch

    anchor = _first_tensor(outputs)
    if anchor is None:
        raise RuntimeError(f"fla_{name}: no output tensor to take the device from.")
    ensure_gpu_tensor(anchor, "output")
    device = anchor.device
    launch = _BOUND.get(name)
    if launch is None:
        launch = getattr(_library(), f"fla_{name}")
        launch.argtypes = [*argtypes, ctypes.c_void_p]
        launch.restype = ctypes.c_int
        _BOUND[name] = launch
    with torch.cuda.device(device):
        ctx = CallContext(device)
        args = build_args(ctx)
        stream = ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
        status = launch(*args, stream)
        if status != FLA_OK:
            raise RuntimeError(f"fla_{name} failed with status={status}: {last_error()}")
    return outputs
