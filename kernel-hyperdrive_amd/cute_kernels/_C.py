"""ctypes binding of ``libcute_hip.so`` (C ABI declared in ``include/cute_hip.h``).

This is the only module that touches the native library.  It plays the part of the reference's
``cpp_jit`` (cute_kernels/jit.py:63-89): kernel launchers elsewhere in the package call
``_C.<function>(tensor, ...)`` and get a kernel launch on torch's current stream.  There is no
fallback: if the library cannot be loaded the first call raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch


# CUTE_HIP_LIBRARY points at another build of the same library (kernel experiments)
_LIB_PATH = os.environ.get("CUTE_HIP_LIBRARY") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "lib", "libcute_hip.so"
)
_ABI_VERSION = 3

_lib = None
_lock = threading.Lock()

CK_F32, CK_F16, CK_BF16 = 0, 1, 2
_DTYPE_CODE = {torch.float32: CK_F32, torch.float16: CK_F16, torch.bfloat16: CK_BF16}

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int
_f32 = ctypes.c_float

# name -> (restype, argtypes); mirrors include/cute_hip.h declaration by declaration
_SIGNATURES = {
    "ck_status_string": (ctypes.c_char_p, [_i32]),
    "ck_abi_version": (_i32, []),
    "ck_add_tensor_forward": (_i32, [_p, _p, _p, _i64, _i32, _i32, _p]),
    "ck_add_scalar_forward": (_i32, [_p, ctypes.c_double, _p, _i64, _i32, _i32, _p]),
    "ck_swiglu_forward": (_i32, [_p, _p, _p, _i64, _i32, _i32, _p]),
    "ck_swiglu_backward": (_i32, [_p, _p, _p, _p, _p, _i64, _i32, _i32, _p]),
    "ck_swiglu_unchunked_forward": (_i32, [_p, _p, _i64, _i64, _i32, _i32, _p]),
    "ck_swiglu_unchunked_backward": (_i32, [_p, _p, _p, _i64, _i64, _i32, _i32, _p]),
    "ck_rmsnorm_forward": (_i32, [_p, _p, _p, _p, _i64, _i64, _f32, _i32, _i32, _p]),
    "ck_residual_rmsnorm_forward": (_i32, [_p, _p, _p, _p, _p, _p, _i64, _i64, _f32, _i32, _i32, _p]),
    "ck_rmsnorm_backward_workspace_size": (_i64, [_i64, _i64]),
    "ck_rmsnorm_backward": (_i32, [_p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _f32, _i32, _i32, _p]),
    "ck_embedding_forward": (_i32, [_p, _i32, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "ck_embedding_backward_workspace_size": (_i64, [_i64, _i64, _i64]),
    "ck_embedding_backward": (_i32, [_p, _i32, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "ck_contiguous_count": (_i32, [_p, _i32, _p, _i64, _i64, _p]),
    "ck_moe_sort_workspace_size": (_i64, [_i64, _i64]),
    "ck_moe_sort": (_i32, [_p, _i32, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "ck_moe_sort_noalloc": (_i32, [_p, _i32, _p, _p, _p, _i64, _i64, _p]),
    "ck_scatter2scatter": (
        _i32,
        [_p, _i64, _p, _i64, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _p, _i32, _p],
    ),
    "ck_scatter2scatter_ws": (
        _i32,
        [_p, _i64, _p, _i64, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _p, _i32, _i32,
         _p, _i64, _p],
    ),
    "ck_scatter2scatter_workspace_size": (_i64, [_i64, _i64, _i64, _i64, _i32]),
    "ck_scatter2scatter_glu": (
        _i32,
        [_p, _i64, _p, _i64, _i64, _i64, _p, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _p],
    ),
    "ck_scatter2scatter_glu_bwd": (
        _i32,
        [_p, _i64, _p, _i64, _i64, _i64, _p, _p, _i64, _p, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _p],
    ),
    "ck_offsets_from_sorted": (_i32, [_p, _p, _i64, _i64, _p]),
    "ck_group_bwd_W": (_i32, [_p, _i64, _p, _i64, _p, _p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _p]),
    "ck_group": (_i32, [_p, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "ck_moe_combine_forward": (_i32, [_p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "ck_moe_combine_backward_gates": (_i32, [_p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "ck_expert_bias_forward": (_i32, [_p, _i64, _p, _i64, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "ck_expert_bias_backward": (_i32, [_p, _i64, _p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "ck_router_topk_softmax_forward": (_i32, [_p, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, _p]),
    "ck_router_topk_softmax_backward": (_i32, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "ck_router_forward": (_i32, [_p, _i64, _p, _i64, _p, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _i32, _p]),
    "ck_router_weight_grad_workspace_size": (_i64, [_i64, _i64, _i64]),
    "ck_router_weight_grad": (_i32, [_p, _p, _i64, _p, _i64, _p, _i64, _i64, _i64, _i64, _i32, _p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def library_path() -> str:
    return _LIB_PATH


def load_library() -> ctypes.CDLL:
    """Load (building first if nothing is built) and type the native library."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            from ._build import build

            build()
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError here = library older than this binding
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.ck_abi_version() != _ABI_VERSION:
            raise RuntimeError(
                f"libcute_hip.so has ABI version {lib.ck_abi_version()}, this package needs {_ABI_VERSION}: rebuild it"
            )
        _lib = lib
    return _lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype ({dtype}); the HIP kernels take float32, float16 and bfloat16") from None


def _ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def _require_gpu(*tensors: torch.Tensor | None) -> torch.device:
    device = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("cute_kernels HIP kernels need GPU tensors; got a tensor on " + str(t.device))
        if device is None:
            device = t.device
        elif t.device != device:
            raise RuntimeError(f"tensors on different devices ({device} and {t.device})")
    if device is None:
        raise RuntimeError("no tensor argument")
    return device


class _Launch:
    """Context for one native call: the tensors' device made current, its stream fetched."""

    __slots__ = ("device", "guard", "stream")

    def __init__(self, *tensors):
        self.device = _require_gpu(*tensors)
        self.guard = None

    def __enter__(self):
        if self.device.index != torch.cuda.current_device():
            self.guard = torch.cuda.device(self.device)
            self.guard.__enter__()
        self.stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


# Optional per-launch timing: while a list is installed here, the grouped-GEMM entry points bracket their
# launch with GPU events recorded on the launch stream and append (name, flop, start, end) to it.
_launch_trace: list | None = None


def set_launch_trace(trace: list | None) -> None:
    global _launch_trace
    _launch_trace = trace


class _Timed:
    __slots__ = ("name", "flop", "start")

    def __init__(self, name: str, flop: float):
        self.name, self.flop = name, flop

    def __enter__(self):
        if _launch_trace is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if _launch_trace is not None:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            _launch_trace.append((self.name, self.flop, self.start, end))
        return False


def _check(status: int, name: str) -> None:
    if status != 0:
        text = load_library().ck_status_string(status).decode()
        raise RuntimeError(f"{name} failed: {text} (status {status})")


def _ids_are_i32(ids: torch.Tensor) -> int:
    if ids.dtype == torch.int32:
        return 1
    if ids.dtype == torch.int64:
        return 0
    raise ValueError(f"index tensor must be int32 or int64, got {ids.dtype}")


def _index_i64(t: torch.Tensor, name: str) -> torch.Tensor:
    """An index tensor as the kernels read it: int64, dense.  The reference's Triton kernels take any integer type
    (they load through typed pointers); the native entry points read int64, so other integer types are converted
    here and anything else is refused - read as int64, an int32 tensor would be twice as long as it is."""
    if t.dtype == torch.int64:
        return t if t.is_contiguous() else t.contiguous()
    if t.dtype in (torch.int32, torch.int16, torch.int8, torch.uint8):
        return t.to(torch.int64).contiguous()
    raise ValueError(f"{name} must be an integer tensor, got {t.dtype}")


def _index_i64_out(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int64 or not t.is_contiguous():
        raise ValueError(f"{name} is written as dense int64; got {t.dtype}, strides {tuple(t.stride())}")


def _same_dtype(ref: torch.Tensor, what: str, **others: torch.Tensor) -> None:
    for name, t in others.items():
        if t is not None and t.dtype != ref.dtype:
            raise ValueError(f"{what}: {name} is {t.dtype}, expected {ref.dtype} like the first operand")


# ---- one Python function per C entry point ----------------------------------------------------------
def _walks_linearly(t: torch.Tensor) -> bool:
    """Dense in memory in some order of its dimensions (a transposed tensor, for instance)."""
    if t.is_contiguous():
        return True
    order = sorted(range(t.dim()), key=lambda d: t.stride(d), reverse=True)
    return t.permute(order).is_contiguous()


def _dense_like(ref: torch.Tensor, what: str, **others: torch.Tensor | None) -> None:
    """The kernels that take no strides read `numel` consecutive elements from every pointer: the operands have to be
    dense, of the first operand's type and number of elements, and laid out like it."""
    for name, t in dict(first=ref, **others).items():
        if t is None:
            continue
        label = name if name != "first" else "the first operand"
        if not _walks_linearly(t) or (t.numel() > 0 and t.stride() != ref.stride() and not
                                      (t.is_contiguous() and ref.is_contiguous())):
            raise ValueError(f"{what}: {label} must be dense in memory and laid out like the first operand")
        if t.dtype != ref.dtype:
            raise ValueError(f"{what}: {name} is {t.dtype}, expected {ref.dtype} like the first operand")
        if t.numel() != ref.numel():
            raise ValueError(f"{what}: {name} has {t.numel()} elements, the first operand {ref.numel()}")


def _dense(what: str, **tensors: torch.Tensor | None) -> None:
    for name, t in tensors.items():
        if t is not None and not t.is_contiguous():
            raise ValueError(f"{what}: {name} must be contiguous")


# All tensors must be contiguous unless a stride is passed explicitly.


def add_tensor_forward(x, y, output, block_size: int) -> None:
    lib = load_library()
    _dense_like(x, "add_tensor_forward", y=y, output=output)
    with _Launch(x, y, output) as L:
        _check(
            lib.ck_add_tensor_forward(_ptr(x), _ptr(y), _ptr(output), x.numel(), dtype_code(x.dtype), block_size,
                                      L.stream),
            "ck_add_tensor_forward",
        )


def add_scalar_forward(x, y: float, output, block_size: int) -> None:
    lib = load_library()
    _dense_like(x, "add_scalar_forward", output=output)
    with _Launch(x, output) as L:
        _check(
            lib.ck_add_scalar_forward(_ptr(x), float(y), _ptr(output), x.numel(), dtype_code(x.dtype), block_size,
                                      L.stream),
            "ck_add_scalar_forward",
        )


def swiglu_forward(gate, up, output, block_size: int) -> None:
    lib = load_library()
    _dense_like(gate, "swiglu_forward", up=up, output=output)
    with _Launch(gate, up, output) as L:
        _check(
            lib.ck_swiglu_forward(_ptr(gate), _ptr(up), _ptr(output), gate.numel(), dtype_code(gate.dtype),
                                  block_size, L.stream),
            "ck_swiglu_forward",
        )


def swiglu_backward(gate, up, output_grad, gate_grad, up_grad, block_size: int) -> None:
    lib = load_library()
    _dense_like(gate, "swiglu_backward", up=up, output_grad=output_grad, gate_grad=gate_grad, up_grad=up_grad)
    with _Launch(gate, up, output_grad, gate_grad, up_grad) as L:
        _check(
            lib.ck_swiglu_backward(_ptr(gate), _ptr(up), _ptr(output_grad), _ptr(gate_grad), _ptr(up_grad),
                                   gate.numel(), dtype_code(gate.dtype), block_size, L.stream),
            "ck_swiglu_backward",
        )


def swiglu_unchunked_forward(x, output, block_size: int) -> None:
    lib = load_library()
    _same_dtype(x, "swiglu_unchunked_forward", output=output)
    _dense("swiglu_unchunked_forward", x=x, output=output)
    if x.size(-1) % 2 != 0 or 2 * output.numel() != x.numel():
        raise ValueError("swiglu_unchunked_forward: the last dimension is (up | gate), the output holds half of it")
    H = x.size(-1)
    B = x.numel() // H if H > 0 else 0
    with _Launch(x, output) as L:
        _check(
            lib.ck_swiglu_unchunked_forward(_ptr(x), _ptr(output), B, H, dtype_code(x.dtype), block_size, L.stream),
            "ck_swiglu_unchunked_forward",
        )


def swiglu_unchunked_backward(x, output_grad, x_grad, block_size: int) -> None:
    lib = load_library()
    _dense_like(x, "swiglu_unchunked_backward", x_grad=x_grad)
    _same_dtype(x, "swiglu_unchunked_backward", output_grad=output_grad)
    _dense("swiglu_unchunked_backward", output_grad=output_grad)
    if x.size(-1) % 2 != 0 or 2 * output_grad.numel() != x.numel():
        raise ValueError("swiglu_unchunked_backward: the last dimension is (up | gate), output_grad holds half of it")
    H = x.size(-1)
    B = x.numel() // H if H > 0 else 0
    with _Launch(x, output_grad, x_grad) as L:
        _check(
            lib.ck_swiglu_unchunked_backward(_ptr(x), _ptr(output_grad), _ptr(x_grad), B, H, dtype_code(x.dtype),
                                             block_size, L.stream),
            "ck_swiglu_unchunked_backward",
        )


def _row_operands(what: str, x, B: int, H: int, weight, rstd, **same_shape) -> None:
    """Dense [B, H] tensors of x's type, a dense weight of H elements, fp32 1/rms of B elements (each may be None).
    Row kernels reduce along the last dimension as it lies in memory, so "dense in some order of the dimensions" is
    not enough here: a transposed tensor would be normalised along the wrong axis."""
    _dense_like(x, what, **same_shape)
    _dense(what, x=x, **same_shape)
    if weight is not None and (weight.numel() != H or not weight.is_contiguous()):
        raise ValueError(f"{what}: the weight must be a dense vector of {H} elements")
    if rstd is not None and (rstd.dtype != torch.float32 or rstd.numel() != B or not rstd.is_contiguous()):
        raise ValueError(f"{what}: the 1 / rms buffer must be dense fp32 with one element per row ({B})")


def rmsnorm_forward(x, weight, output, rstd, eps: float, block_size_b: int = 0) -> None:
    lib = load_library()
    _same_dtype(x, "rmsnorm_forward", weight=weight, output=output)
    H = x.size(-1)
    B = x.numel() // H if H > 0 else 0
    _row_operands("rmsnorm_forward", x, B, H, weight, rstd, output=output)
    with _Launch(x, weight, output, rstd) as L:
        _check(
            lib.ck_rmsnorm_forward(_ptr(x), _ptr(weight), _ptr(output), _ptr(rstd), B, H, eps, dtype_code(x.dtype),
                                   block_size_b, L.stream),
            "ck_rmsnorm_forward",
        )


def residual_rmsnorm_forward(x, residual, weight, output, residual_out, rstd, eps: float, block_size_b: int = 0) -> None:
    """residual_out = x + residual, output = rmsnorm(residual_out); all dense and of one shape and dtype."""
    lib = load_library()
    H = x.size(-1)
    B = x.numel() // H if H > 0 else 0
    for t in (residual, output, residual_out):
        if t.shape != x.shape or t.dtype != x.dtype or not t.is_contiguous():
            raise ValueError("residual_rmsnorm_forward: x, residual, output and residual_out must be dense and alike")
    if not x.is_contiguous():
        raise ValueError("residual_rmsnorm_forward: x must be dense")
    _same_dtype(x, "residual_rmsnorm_forward", weight=weight)
    _row_operands("residual_rmsnorm_forward", x, B, H, weight, rstd)
    with _Launch(x, residual, weight, output, residual_out, rstd) as L:
        _check(
            lib.ck_residual_rmsnorm_forward(_ptr(x), _ptr(residual), _ptr(weight), _ptr(output), _ptr(residual_out),
                                            _ptr(rstd), B, H, eps, dtype_code(x.dtype), block_size_b, L.stream),
            "ck_residual_rmsnorm_forward",
        )


def rmsnorm_backward_workspace_size(B: int, H: int, device: torch.device) -> int:
    lib = load_library()
    with torch.cuda.device(device):
        return lib.ck_rmsnorm_backward_workspace_size(B, H)


def rmsnorm_backward(x, weight, output_grad, rstd, x_grad, weight_grad, workspace, eps: float,
                     block_size_b: int = 0) -> None:
    lib = load_library()
    _same_dtype(x, "rmsnorm_backward", weight=weight, output_grad=output_grad, x_grad=x_grad, weight_grad=weight_grad)
    H = x.size(-1)
    B = x.numel() // H if H > 0 else 0
    _row_operands("rmsnorm_backward", x, B, H, weight, rstd, output_grad=output_grad, x_grad=x_grad)
    if (weight is None) != (weight_grad is None) or (weight_grad is not None and (
            weight_grad.numel() != H or not weight_grad.is_contiguous())):
        raise ValueError("rmsnorm_backward: weight_grad goes with the weight, a dense vector of its size")
    with _Launch(x, weight, output_grad, rstd, x_grad, weight_grad, workspace) as L:
        _check(
            lib.ck_rmsnorm_backward(_ptr(x), _ptr(weight), _ptr(output_grad), _ptr(rstd), _ptr(x_grad),
                                    _ptr(weight_grad), _ptr(workspace),
                                    0 if workspace is None else workspace.numel() * workspace.element_size(), B, H,
                                    eps, dtype_code(x.dtype), block_size_b, L.stream),
            "ck_rmsnorm_backward",
        )


def embedding_forward(input_ids, weight, output) -> None:
    lib = load_library()
    _same_dtype(weight, "embedding_forward", output=output)
    _dense("embedding_forward", input_ids=input_ids, weight=weight, output=output)
    if weight.dim() != 2 or output.numel() != input_ids.numel() * weight.size(1):
        raise ValueError("embedding_forward: weight [V, H], output one row of H per id")
    with _Launch(input_ids, weight, output) as L:
        _check(
            lib.ck_embedding_forward(_ptr(input_ids), _ids_are_i32(input_ids), _ptr(weight), _ptr(output),
                                     input_ids.numel(), weight.size(0), weight.size(1), dtype_code(weight.dtype),
                                     L.stream),
            "ck_embedding_forward",
        )


def embedding_backward_workspace_size(num_ids: int, V: int, H: int) -> int:
    return load_library().ck_embedding_backward_workspace_size(num_ids, V, H)


def embedding_backward(input_ids, output_grad, weight_grad, workspace) -> None:
    lib = load_library()
    _same_dtype(weight_grad, "embedding_backward", output_grad=output_grad)
    _dense("embedding_backward", input_ids=input_ids, output_grad=output_grad, weight_grad=weight_grad,
           workspace=workspace)
    if weight_grad.dim() != 2 or output_grad.numel() != input_ids.numel() * weight_grad.size(1):
        raise ValueError("embedding_backward: weight_grad [V, H], output_grad one row of H per id")
    with _Launch(input_ids, output_grad, weight_grad, workspace) as L:
        _check(
            lib.ck_embedding_backward(_ptr(input_ids), _ids_are_i32(input_ids), _ptr(output_grad), _ptr(weight_grad),
                                      _ptr(workspace), workspace.numel() * workspace.element_size(),
                                      input_ids.numel(), weight_grad.size(0), weight_grad.size(1),
                                      dtype_code(weight_grad.dtype), L.stream),
            "ck_embedding_backward",
        )


def contiguous_count(x, output, size: int) -> None:
    lib = load_library()
    if output.dtype != torch.int32 or not output.is_contiguous() or output.numel() != size:
        raise ValueError("contiguous_count writes a dense int32 tensor of `size` counts")
    if not x.is_contiguous():
        x = x.contiguous()
    with _Launch(x, output) as L:
        _check(
            lib.ck_contiguous_count(_ptr(x), _ids_are_i32(x), _ptr(output), x.numel(), size, L.stream),
            "ck_contiguous_count",
        )


def moe_sort_workspace_size(M: int, E: int) -> int:
    return load_library().ck_moe_sort_workspace_size(M, E)


def moe_sort(expert_ids, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, workspace, E: int) -> None:
    lib = load_library()
    if not expert_ids.is_contiguous():
        expert_ids = expert_ids.contiguous()
    for name, t in (("sorted_expert_idxs", sorted_expert_idxs), ("sorted_scattered_idxs", sorted_scattered_idxs),
                    ("expert_offsets", expert_offsets)):
        _index_i64_out(t, name)
    if sorted_expert_idxs.numel() != expert_ids.numel() or sorted_scattered_idxs.numel() != expert_ids.numel():
        raise ValueError("moe_sort: one sorted id and one position per expert id")
    if expert_offsets.numel() != E:
        raise ValueError("moe_sort: one offset per expert")
    with _Launch(expert_ids, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, workspace) as L:
        _check(
            lib.ck_moe_sort(_ptr(expert_ids), _ids_are_i32(expert_ids), _ptr(sorted_expert_idxs),
                            _ptr(sorted_scattered_idxs), _ptr(expert_offsets), _ptr(workspace),
                            0 if workspace is None else workspace.numel() * workspace.element_size(),
                            expert_ids.numel(), E, L.stream),
            "ck_moe_sort",
        )


MOE_SORT_NOALLOC_SCRATCH_BYTES = 4 * 1024 * 1024


def moe_sort_noalloc(expert_ids, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, E: int) -> None:
    """``moe_sort`` with the workspace inside the library (a fixed device array per GPU): for callers that must
    not allocate.  Calls that overlap on one GPU share that array and race."""
    lib = load_library()
    if not expert_ids.is_contiguous():
        expert_ids = expert_ids.contiguous()
    for name, t in (("sorted_expert_idxs", sorted_expert_idxs), ("sorted_scattered_idxs", sorted_scattered_idxs),
                    ("expert_offsets", expert_offsets)):
        _index_i64_out(t, name)
    if sorted_expert_idxs.numel() != expert_ids.numel() or sorted_scattered_idxs.numel() != expert_ids.numel():
        raise ValueError("moe_sort: one sorted id and one position per expert id")
    if expert_offsets.numel() != E:
        raise ValueError("moe_sort: one offset per expert")
    with _Launch(expert_ids, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets) as L:
        _check(
            lib.ck_moe_sort_noalloc(_ptr(expert_ids), _ids_are_i32(expert_ids), _ptr(sorted_expert_idxs),
                                    _ptr(sorted_scattered_idxs), _ptr(expert_offsets), expert_ids.numel(), E,
                                    L.stream),
            "ck_moe_sort_noalloc",
        )


def offsets_from_sorted(sorted_expert_idxs, expert_offsets) -> None:
    lib = load_library()
    sorted_expert_idxs = _index_i64(sorted_expert_idxs, "sorted_expert_idxs")
    _index_i64_out(expert_offsets, "expert_offsets")
    with _Launch(sorted_expert_idxs, expert_offsets) as L:
        _check(
            lib.ck_offsets_from_sorted(_ptr(sorted_expert_idxs), _ptr(expert_offsets), sorted_expert_idxs.numel(),
                                       expert_offsets.numel(), L.stream),
            "ck_offsets_from_sorted",
        )


def scatter2scatter_workspace_size(num_slots: int, K: int, N: int, E: int, dtype) -> int:
    """Bytes of workspace with which ``scatter2scatter`` splits the tail of its tile grid (0: not for this shape)."""
    return int(load_library().ck_scatter2scatter_workspace_size(num_slots, K, N, E, dtype_code(dtype)))


GEMM_WAVES = (0, 4, 8)  # loops of the matrix-core kernel: the library's choice, four wavefronts per tile, eight


def _waves(waves: int, what: str) -> int:
    if waves not in GEMM_WAVES:
        raise ValueError(f"{what}: waves must be one of {GEMM_WAVES}, got {waves!r}")
    return int(waves)


def scatter2scatter(X, W, sorted_scattered_idxs, expert_offsets, out, fan_out: int, x_grouped: bool,
                    y_grouped: bool, workspace=None, bias=None, waves: int = 0) -> None:
    """X [*, K] (unit column stride), W strided view [E, K, N], out [slots, N] (unit column stride); ``workspace``:
    uint8 tensor of ``scatter2scatter_workspace_size`` bytes or None; ``bias``: [E, N] contiguous or None, added to
    every row of its expert before the row is rounded; ``waves``: the loop of the matrix-core kernel (``GEMM_WAVES``)."""
    waves = _waves(waves, "scatter2scatter")
    lib = load_library()
    if X.stride(1) != 1 or out.stride(1) != 1:
        raise ValueError("scatter2scatter needs unit column stride for X and out")
    _same_dtype(X, "scatter2scatter", W=W, out=out, bias=bias)
    if bias is not None and (tuple(bias.shape) != (W.size(0), out.size(1)) or not bias.is_contiguous()):
        raise ValueError("scatter2scatter: bias must be a contiguous [E, N] tensor")
    if sorted_scattered_idxs is not None:
        sorted_scattered_idxs = _index_i64(sorted_scattered_idxs, "sorted_scattered_idxs")
    expert_offsets = _index_i64(expert_offsets, "expert_offsets")
    if expert_offsets.numel() != W.size(0):
        raise ValueError("scatter2scatter: one expert offset per expert of W")
    flop = 2.0 * out.size(0) * X.size(1) * out.size(1)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with _Launch(X, W, sorted_scattered_idxs, expert_offsets, out, workspace, bias) as L, _Timed("scatter2scatter", flop):
        _check(
            lib.ck_scatter2scatter_ws(_ptr(X), X.stride(0), _ptr(W), W.stride(0), W.stride(1), W.stride(2),
                                      _ptr(sorted_scattered_idxs), _ptr(expert_offsets), _ptr(out), out.stride(0),
                                      out.size(0), X.size(1), out.size(1), W.size(0), fan_out, int(x_grouped),
                                      int(y_grouped), _ptr(bias), dtype_code(X.dtype), waves, _ptr(workspace), ws_bytes,
                                      L.stream),
            "ck_scatter2scatter_ws",
        )


def scatter2scatter_glu(X, W, sorted_scattered_idxs, expert_offsets, h, act, fan_out: int, x_grouped: bool,
                        waves: int = 0) -> None:
    """h [slots, 2I] = gathered X rows times W [E, K, 2I], act [slots, I] = SwiGLU(h); rows grouped by expert."""
    lib = load_library()
    waves = _waves(waves, "scatter2scatter_glu")
    if X.stride(1) != 1 or h.stride(1) != 1 or act.stride(1) != 1:
        raise ValueError("scatter2scatter_glu needs unit column stride for X, h and act")
    if h.size(1) != 2 * act.size(1) or h.size(0) != act.size(0):
        raise ValueError("scatter2scatter_glu: h must be [slots, 2I] and act [slots, I]")
    _same_dtype(X, "scatter2scatter_glu", W=W, h=h, act=act)
    if sorted_scattered_idxs is not None:
        sorted_scattered_idxs = _index_i64(sorted_scattered_idxs, "sorted_scattered_idxs")
    expert_offsets = _index_i64(expert_offsets, "expert_offsets")
    if expert_offsets.numel() != W.size(0):
        raise ValueError("scatter2scatter_glu: one expert offset per expert of W")
    flop = 2.0 * h.size(0) * X.size(1) * h.size(1)
    with _Launch(X, W, sorted_scattered_idxs, expert_offsets, h, act) as L, _Timed("scatter2scatter", flop):
        _check(
            lib.ck_scatter2scatter_glu(_ptr(X), X.stride(0), _ptr(W), W.stride(0), W.stride(1), W.stride(2),
                                       _ptr(sorted_scattered_idxs), _ptr(expert_offsets), _ptr(h), h.stride(0),
                                       _ptr(act), act.stride(0), h.size(0), X.size(1), act.size(1), W.size(0),
                                       fan_out, int(x_grouped), dtype_code(X.dtype), waves, L.stream),
            "ck_scatter2scatter_glu",
        )


def scatter2scatter_glu_bwd(DY, W, expert_offsets, h, d_h, waves: int = 0) -> None:
    """d_h [slots, 2I] = SwiGLU'(h) applied to DY [slots, K] times W [E, K, I]; all rows grouped by expert."""
    lib = load_library()
    waves = _waves(waves, "scatter2scatter_glu_bwd")
    if DY.stride(1) != 1 or h.stride(1) != 1 or d_h.stride(1) != 1:
        raise ValueError("scatter2scatter_glu_bwd needs unit column stride for DY, h and d_h")
    if h.shape != d_h.shape or h.size(1) != 2 * W.size(2) or h.size(0) != DY.size(0):
        raise ValueError("scatter2scatter_glu_bwd: h and d_h must be [slots, 2I] for W [E, K, I]")
    _same_dtype(DY, "scatter2scatter_glu_bwd", W=W, h=h, d_h=d_h)
    expert_offsets = _index_i64(expert_offsets, "expert_offsets")
    if expert_offsets.numel() != W.size(0):
        raise ValueError("scatter2scatter_glu_bwd: one expert offset per expert of W")
    flop = 2.0 * DY.size(0) * DY.size(1) * W.size(2)
    with _Launch(DY, W, expert_offsets, h, d_h) as L, _Timed("scatter2scatter", flop):
        _check(
            lib.ck_scatter2scatter_glu_bwd(_ptr(DY), DY.stride(0), _ptr(W), W.stride(0), W.stride(1), W.stride(2),
                                           _ptr(expert_offsets), _ptr(h), h.stride(0), _ptr(d_h), d_h.stride(0),
                                           DY.size(0), DY.size(1), W.size(2), W.size(0), dtype_code(DY.dtype), waves,
                                           L.stream),
            "ck_scatter2scatter_glu_bwd",
        )


def group_bwd_W(DY, X, expert_offsets, DW, E: int, waves: int = 0) -> None:
    lib = load_library()
    waves = _waves(waves, "group_bwd_W")
    if X.stride(1) != 1 or DY.stride(1) != 1:
        raise ValueError("group_bwd_W needs unit column stride for X and DY")
    _same_dtype(X, "group_bwd_W", DY=DY, DW=DW)
    expert_offsets = _index_i64(expert_offsets, "expert_offsets")
    if expert_offsets.numel() != E or DW.size(0) != E:
        raise ValueError("group_bwd_W: one expert offset and one DW block per expert")
    flop = 2.0 * X.size(0) * X.size(1) * DY.size(1)
    with _Launch(DY, X, expert_offsets, DW) as L, _Timed("group_bwd_W", flop):
        _check(
            lib.ck_group_bwd_W(_ptr(DY), DY.stride(0), _ptr(X), X.stride(0), _ptr(expert_offsets), _ptr(DW),
                               DW.stride(0), DW.stride(1), DW.stride(2), X.size(0), X.size(1), DY.size(1), E,
                               dtype_code(X.dtype), waves, L.stream),
            "ck_group_bwd_W",
        )


def group(A, idx, coeff, out, fan_out: int) -> None:
    lib = load_library()
    if A.stride(1) != 1 or out.stride(1) != 1:
        raise ValueError("group needs unit column stride for A and out")
    _same_dtype(A, "group", coeff=coeff, out=out)
    idx = _index_i64(idx, "the row index")
    if coeff is not None and not coeff.is_contiguous():
        coeff = coeff.contiguous()
    with _Launch(A, idx, coeff, out) as L:
        _check(
            lib.ck_group(_ptr(A), A.stride(0), _ptr(idx), _ptr(coeff), _ptr(out), out.stride(0), idx.numel(),
                         A.size(1), fan_out, dtype_code(A.dtype), L.stream),
            "ck_group",
        )


def moe_combine_forward(expanded, gates, out) -> None:
    """expanded [T, k, H], gates [T, k] (or None: plain sum over the k slots), out [T, H]; all dense."""
    lib = load_library()
    T, k, H = expanded.shape
    _same_dtype(expanded, "moe_combine_forward", gates=gates, out=out)
    _dense("moe_combine_forward", expanded=expanded, gates=gates, out=out)
    if out.numel() != T * H or (gates is not None and gates.numel() != T * k):
        raise ValueError("moe_combine_forward: expanded [T, k, H], gates [T, k], out [T, H]")
    with _Launch(expanded, gates, out) as L:
        _check(
            lib.ck_moe_combine_forward(_ptr(expanded), _ptr(gates), _ptr(out), T, k, H, dtype_code(expanded.dtype),
                                       L.stream),
            "ck_moe_combine_forward",
        )


def moe_combine_backward_gates(expanded, grad_out, d_gates) -> None:
    """expanded [T, k, H], grad_out [T, H], d_gates [T, k]; all dense."""
    lib = load_library()
    T, k, H = expanded.shape
    _same_dtype(expanded, "moe_combine_backward_gates", grad_out=grad_out, d_gates=d_gates)
    _dense("moe_combine_backward_gates", expanded=expanded, grad_out=grad_out, d_gates=d_gates)
    if grad_out.numel() != T * H or d_gates.numel() != T * k:
        raise ValueError("moe_combine_backward_gates: expanded [T, k, H], grad_out [T, H], d_gates [T, k]")
    with _Launch(expanded, grad_out, d_gates) as L:
        _check(
            lib.ck_moe_combine_backward_gates(_ptr(expanded), _ptr(grad_out), _ptr(d_gates), T, k, H,
                                              dtype_code(expanded.dtype), L.stream),
            "ck_moe_combine_backward_gates",
        )


def expert_bias_forward(y, bias, row_index, expert_offsets) -> None:
    """y[r(i)] += bias[expert of sorted position i], in place; row_index None for expert-grouped y, else the
    position -> row map (sorted_scattered_idxs)."""
    lib = load_library()
    if y.stride(1) != 1 or bias.stride(1) != 1:
        raise ValueError("expert_bias_forward needs unit column stride for y and bias")
    if bias.size(1) != y.size(1) or bias.size(0) != expert_offsets.numel():
        raise ValueError("expert_bias_forward: bias must be [num_experts, y.size(1)]")
    if row_index is not None and (row_index.numel() != y.size(0) or row_index.dtype != torch.int64):
        raise ValueError("expert_bias_forward: one int64 row index per row of y")
    if bias.dtype != y.dtype or expert_offsets.dtype != torch.int64:
        raise ValueError("expert_bias_forward: bias in y's dtype, int64 expert offsets")
    if row_index is not None and not row_index.is_contiguous():
        row_index = row_index.contiguous()
    with _Launch(y, bias, row_index, expert_offsets) as L:
        _check(
            lib.ck_expert_bias_forward(_ptr(y), y.stride(0), _ptr(bias), bias.stride(0), _ptr(row_index),
                                       _ptr(expert_offsets), y.size(0), y.size(1), bias.size(0), dtype_code(y.dtype),
                                       L.stream),
            "ck_expert_bias_forward",
        )


def expert_bias_backward(dy, expert_offsets, d_bias) -> None:
    """d_bias[e] = sum of the expert-grouped rows of dy that belong to expert e (every element written)."""
    lib = load_library()
    if dy.stride(1) != 1 or d_bias.stride(1) != 1:
        raise ValueError("expert_bias_backward needs unit column stride for dy and d_bias")
    if d_bias.size(1) != dy.size(1) or d_bias.size(0) != expert_offsets.numel():
        raise ValueError("expert_bias_backward: d_bias must be [num_experts, dy.size(1)]")
    if d_bias.dtype != dy.dtype or expert_offsets.dtype != torch.int64:
        raise ValueError("expert_bias_backward: d_bias in dy's dtype, int64 expert offsets")
    with _Launch(dy, expert_offsets, d_bias) as L:
        _check(
            lib.ck_expert_bias_backward(_ptr(dy), dy.stride(0), _ptr(expert_offsets), _ptr(d_bias), d_bias.stride(0),
                                        dy.size(0), dy.size(1), d_bias.size(0), dtype_code(dy.dtype), L.stream),
            "ck_expert_bias_backward",
        )


ROUTER_MAX_EXPERTS = 1024
ROUTER_MAX_TOP_K = 64
ROUTER_LINEAR_MAX_EXPERTS = 128  # the launch with the router's linear in front


def router_topk_softmax_forward(logits, weights, weights_f32, selected) -> None:
    """logits [T, E] -> selected [T, k] int64 (largest first), weights [T, k] in logits' dtype and in fp32."""
    lib = load_library()
    T, E = logits.shape
    k = selected.size(1)
    if logits.stride(1) != 1:
        raise ValueError("router_topk_softmax_forward needs unit column stride for the logits")
    if weights.dtype != logits.dtype or weights_f32.dtype != torch.float32 or selected.dtype != torch.int64:
        raise ValueError("router_topk_softmax_forward: weights in the logits' dtype, weights_f32 fp32, selected int64")
    for out in (weights, weights_f32, selected):
        if tuple(out.shape) != (T, k) or not out.is_contiguous():
            raise ValueError("router_topk_softmax_forward: outputs must be dense [tokens, k]")
    with _Launch(logits, weights, weights_f32, selected) as L:
        _check(
            lib.ck_router_topk_softmax_forward(_ptr(logits), logits.stride(0), _ptr(weights), _ptr(weights_f32),
                                               _ptr(selected), T, E, k, dtype_code(logits.dtype), L.stream),
            "ck_router_topk_softmax_forward",
        )


def router_forward_supported(x, gate_weight, top_k: int) -> bool:
    """Whether ``router_forward`` takes operands of this type, shape and strides (otherwise: the linear, then
    router_topk_softmax_forward).  Only properties a traced graph knows; the 16-byte alignment of the first elements
    is the caller's to provide."""
    return (
        x.dim() == 2
        and gate_weight.dim() == 2
        and x.dtype in (torch.bfloat16, torch.float16)
        and gate_weight.dtype == x.dtype
        and gate_weight.size(0) <= ROUTER_LINEAR_MAX_EXPERTS
        and top_k <= min(gate_weight.size(0), ROUTER_MAX_TOP_K)
        and x.size(1) % 8 == 0
        and x.stride(1) == 1 and gate_weight.stride(1) == 1
        and x.stride(0) % 8 == 0 and gate_weight.stride(0) % 8 == 0
    )


def router_forward(x, gate_weight, logits, weights, weights_f32, selected) -> None:
    """logits [T, E] = x [T, H] @ gate_weight [E, H]^T (rounded once), and the selection from the stored logits."""
    lib = load_library()
    T, H = x.shape
    E = gate_weight.size(0)
    k = selected.size(1)
    if gate_weight.size(1) != H or gate_weight.dtype != x.dtype:
        raise ValueError("router_forward: gate_weight must be [E, H] in x's dtype")
    if x.stride(1) != 1 or gate_weight.stride(1) != 1:
        raise ValueError("router_forward needs unit column stride for x and gate_weight")
    if tuple(logits.shape) != (T, E) or logits.dtype != x.dtype or logits.stride(1) != 1:
        raise ValueError("router_forward: logits must be [tokens, E] in x's dtype with unit column stride")
    if weights.dtype != x.dtype or weights_f32.dtype != torch.float32 or selected.dtype != torch.int64:
        raise ValueError("router_forward: weights in x's dtype, weights_f32 fp32, selected int64")
    for out in (weights, weights_f32, selected):
        if tuple(out.shape) != (T, k) or not out.is_contiguous():
            raise ValueError("router_forward: weights, weights_f32 and selected must be dense [tokens, k]")
    with _Launch(x, gate_weight, logits, weights, weights_f32, selected) as L:
        _check(
            lib.ck_router_forward(_ptr(x), x.stride(0), _ptr(gate_weight), gate_weight.stride(0), _ptr(logits),
                                  logits.stride(0), _ptr(weights), _ptr(weights_f32), _ptr(selected), T, H, E, k,
                                  dtype_code(x.dtype), L.stream),
            "ck_router_forward",
        )


def router_weight_grad_supported(d_logits, x) -> bool:
    """Whether ``router_weight_grad`` takes operands of this type, shape and strides."""
    return (
        x.dim() == 2
        and d_logits.dim() == 2
        and x.dtype in (torch.bfloat16, torch.float16)
        and d_logits.dtype == x.dtype
        and 0 < d_logits.size(1) <= ROUTER_LINEAR_MAX_EXPERTS
        and x.size(0) > 0 and x.size(0) % 8 == 0
        and x.size(1) % 8 == 0
        and x.stride(1) == 1 and x.stride(0) % 8 == 0
    )


def router_weight_grad_workspace_size(tokens: int, H: int, E: int) -> int:
    return int(load_library().ck_router_weight_grad_workspace_size(tokens, H, E))


def router_weight_grad(d_logits_t, x, d_weight, workspace) -> None:
    """d_weight [E, H] = d_logits_t [E, T] @ x [T, H], fp32 partial sums over pieces of the tokens, one rounding."""
    lib = load_library()
    E, T = d_logits_t.shape
    H = x.size(1)
    if x.size(0) != T or d_logits_t.dtype != x.dtype or d_weight.dtype != x.dtype:
        raise ValueError("router_weight_grad: d_logits_t [E, T], x [T, H] and d_weight [E, H] of one dtype")
    if not d_logits_t.is_contiguous() or x.stride(1) != 1 or d_weight.stride(1) != 1 or tuple(d_weight.shape) != (E, H):
        raise ValueError("router_weight_grad: dense d_logits_t, unit column stride for x and d_weight [E, H]")
    with _Launch(d_logits_t, x, d_weight, workspace) as L:
        _check(
            lib.ck_router_weight_grad(_ptr(d_logits_t), _ptr(x), x.stride(0), _ptr(d_weight), d_weight.stride(0),
                                      _ptr(workspace), workspace.numel() * workspace.element_size(), T, H, E,
                                      dtype_code(x.dtype), L.stream),
            "ck_router_weight_grad",
        )


def router_topk_softmax_backward(d_weights, weights_f32, selected, d_logits) -> None:
    """d_logits [T, E] from d_weights [T, k], the fp32 weights and the selected positions of the forward."""
    lib = load_library()
    T, E = d_logits.shape
    k = selected.size(1)
    if d_logits.stride(1) != 1:
        raise ValueError("router_topk_softmax_backward needs unit column stride for d_logits")
    if d_weights.dtype != d_logits.dtype or weights_f32.dtype != torch.float32 or selected.dtype != torch.int64:
        raise ValueError("router_topk_softmax_backward: d_weights in d_logits' dtype, weights_f32 fp32, selected int64")
    for t in (d_weights, weights_f32, selected):
        if tuple(t.shape) != (T, k) or not t.is_contiguous():
            raise ValueError("router_topk_softmax_backward: d_weights, weights_f32 and selected must be dense [tokens, k]")
    with _Launch(d_weights, weights_f32, selected, d_logits) as L:
        _check(
            lib.ck_router_topk_softmax_backward(_ptr(d_weights), _ptr(weights_f32), _ptr(selected), _ptr(d_logits),
                                                d_logits.stride(0), T, E, k, dtype_code(d_logits.dtype), L.stream),
            "ck_router_topk_softmax_backward",
        )
