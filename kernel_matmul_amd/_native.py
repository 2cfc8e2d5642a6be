"""ctypes binding of libkernel_matmul_amd.so and the tensor marshalling around it.

This is the only module that touches the shared library.  It turns torch tensors into the
(pointer, strides) pairs of the C ABI, passes torch's current HIP stream, allocates outputs
and workspaces with torch, and converts status codes into Python exceptions.  There is no
fallback: if the library is missing, every operator raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Sequence

import torch
from torch import Tensor

from kernel_matmul_amd import _BLOCK_SIZE

KERNEL_TYPES = {"rbf": 0, "spectral": 1, "locally_periodic": 2}
NUM_PARAMS = {"rbf": 2, "spectral": 3, "locally_periodic": 4}
MAX_BATCH_RANK = 6

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
LIB_PATH = os.path.join(_LIB_DIR, "libkernel_matmul_amd.so")

_lib = None

_i64p = ctypes.POINTER(ctypes.c_int64)
_vp = ctypes.c_void_p


class LaunchOptions(ctypes.Structure):
    """Mirror of ``km_launch_options``."""

    _fields_ = [
        ("variant", ctypes.c_int),
        ("rows_per_wave", ctypes.c_int),
        ("col_splits", ctypes.c_int),
        ("reserved", ctypes.c_int),
    ]


def library_available() -> bool:
    return os.path.exists(LIB_PATH)


def load_library():
    """Load the C-ABI library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"kernel_matmul_amd: native library not found at {LIB_PATH}. "
            "Build it with `make -C kernel_matmul_amd/csrc` (needs hipcc, targets gfx950)."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.km_last_error.restype = ctypes.c_char_p
    lib.km_last_error.argtypes = []
    lib.km_version.restype = ctypes.c_int
    lib.km_num_params.restype = ctypes.c_int
    lib.km_num_params.argtypes = [ctypes.c_int]

    f32p, i32p = _vp, _vp
    lib.km_make_ranges.restype = ctypes.c_int
    lib.km_make_ranges.argtypes = [f32p, f32p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                   ctypes.c_float, ctypes.c_int, ctypes.c_int, i32p, i32p]
    lib.km_make_ranges_symmetric.restype = ctypes.c_int
    lib.km_make_ranges_symmetric.argtypes = [f32p, ctypes.c_int64, ctypes.c_int64, ctypes.c_float,
                                             ctypes.c_int, i32p, i32p]
    lib.km_transpose_ranges.restype = ctypes.c_int
    lib.km_transpose_ranges.argtypes = [i32p, i32p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                        ctypes.c_int, ctypes.c_int, i32p, i32p]
    lib.km_make_ranges_device.restype = ctypes.c_int
    lib.km_make_ranges_device.argtypes = lib.km_make_ranges.argtypes + [_vp]
    lib.km_make_ranges_symmetric_device.restype = ctypes.c_int
    lib.km_make_ranges_symmetric_device.argtypes = lib.km_make_ranges_symmetric.argtypes + [_vp]

    tensor = [_vp, _i64p]
    lib.km_matmul.restype = ctypes.c_int
    lib.km_matmul.argtypes = (
        [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]
        + tensor * 6
        + [_vp, ctypes.POINTER(LaunchOptions), _vp]
    )
    lib.km_param_grad_describe.restype = ctypes.c_int
    lib.km_param_grad_describe.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                           ctypes.c_char_p, ctypes.c_size_t]
    lib.km_matmul_describe.restype = ctypes.c_int
    lib.km_matmul_describe.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                       ctypes.c_int64, _vp, ctypes.c_char_p, ctypes.c_size_t]
    lib.km_param_grad_workspace_size.restype = ctypes.c_size_t
    lib.km_param_grad_workspace_size.argtypes = [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64,
                                                 ctypes.c_int64, ctypes.c_int64]
    lib.km_param_grad.restype = ctypes.c_int
    lib.km_param_grad.argtypes = (
        [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]
        + tensor * 7
        + [_vp, _vp, ctypes.c_size_t, _vp]
    )
    lib.km_param_grad_static.restype = ctypes.c_int
    lib.km_param_grad_static.argtypes = (
        [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]
        + tensor * 7
        + [_vp, _vp]
    )
    lib.km_index.restype = ctypes.c_int
    lib.km_index.argtypes = (
        [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64, ctypes.c_int64]
        + tensor * 5
        + [ctypes.c_int, _i64p, ctypes.POINTER(_vp), ctypes.POINTER(_i64p)]
        + tensor * 2
        + [_vp, _vp]
    )
    lib.km_index_bwd_workspace_size.restype = ctypes.c_size_t
    lib.km_index_bwd_workspace_size.argtypes = [ctypes.c_int64]
    lib.km_index_bwd.restype = ctypes.c_int
    lib.km_index_bwd.argtypes = (
        [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64, ctypes.c_int64]
        + tensor * 5
        + [ctypes.c_int, _i64p, ctypes.POINTER(_vp), ctypes.POINTER(_i64p)]
        + tensor * 3
        + [_vp, _vp, ctypes.c_size_t, _vp]
    )
    lib.km_dense.restype = ctypes.c_int
    lib.km_dense.argtypes = (
        [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64, ctypes.c_int64] + tensor * 5 + [_vp, _vp]
    )
    lib.km_dense_bwd.restype = ctypes.c_int
    lib.km_dense_bwd.argtypes = (
        [ctypes.c_int, ctypes.c_int, _i64p, ctypes.c_int64, ctypes.c_int64]
        + tensor * 6
        + [_vp, _vp, ctypes.c_size_t, _vp]
    )
    _lib = lib
    return lib


def _raise(lib, status: int):
    # Every failed check of the reference's entry points is a TORCH_CHECK, i.e. a RuntimeError
    # (native/common/entrypoint.h:3-14).
    raise RuntimeError(lib.km_last_error().decode("utf-8", "replace"))


def _i64(values: Sequence[int]):
    return (ctypes.c_int64 * max(len(values), 1))(*values)


def _ptr(t: Tensor):
    return ctypes.c_void_p(t.data_ptr()) if t.numel() > 0 else ctypes.c_void_p(0)


def _tensor_args(t: Tensor):
    return _ptr(t), _i64(t.stride())


def _stream(device: torch.device):
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(index))


class _on_device:
    """Makes ``device`` current for the launch; costs nothing when it already is."""

    __slots__ = ("_guard",)

    def __init__(self, device: torch.device):
        index = device.index
        self._guard = None
        if index is not None and index != torch.cuda.current_device():
            self._guard = torch.cuda.device(index)

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            return self._guard.__exit__(*exc)
        return False


# Validated calls, keyed by everything the validation looked at (shapes, strides, dtypes,
# devices).  A repeated call with the same signature skips the checks and reuses the ctypes
# stride / size arrays: only the data pointers, the output and the stream are new.
_PREPARED: dict = {}
_PREPARED_LIMIT = 512


def _signature(op: str, kernel_type: str, tensors) -> tuple:
    key = [op, kernel_type]
    for t in tensors:
        key.append(t.shape)
        key.append(t.stride())
        key.append(t.dtype)
        key.append(t.device)
    return tuple(key)


def _remember(key, value):
    if len(_PREPARED) >= _PREPARED_LIMIT:
        _PREPARED.clear()
    _PREPARED[key] = value
    return value


# -- the checks of the reference's entry points (native/common/entrypoint.h:3-14) ----------
def check_cuda(x: Tensor) -> None:
    if not x.is_cuda:
        raise RuntimeError("x must be a CUDA tensor")


def check_int32(x: Tensor) -> None:
    if x.dtype != torch.int32:
        raise RuntimeError("x must be int32")


def check_cuda_int32(x: Tensor) -> None:
    check_cuda(x)
    check_int32(x)


def check_float(x: Tensor) -> None:
    # The reference gets this from mutable_data_ptr<float>() (native/common/accessor.cuh:9).
    if x.dtype != torch.float32:
        names = {torch.float64: "Double", torch.float16: "Half", torch.bfloat16: "BFloat16",
                 torch.int32: "Int", torch.int64: "Long"}
        name = names.get(x.dtype, str(x.dtype).replace("torch.", ""))
        raise RuntimeError(f"expected scalar type Float but found {name}")


def _kernel_id(kernel_type: str) -> int:
    try:
        return KERNEL_TYPES[kernel_type]
    except KeyError:
        raise ValueError(f"Unknown kernel type: {kernel_type}") from None


def _check_batch(name: str, t: Tensor, batch_shape, trailing: int) -> None:
    if t.dim() != len(batch_shape) + trailing or tuple(t.shape[: len(batch_shape)]) != tuple(batch_shape):
        raise RuntimeError(
            f"{name} has shape {tuple(t.shape)}, expected batch shape {tuple(batch_shape)} "
            f"followed by {trailing} dimension(s)"
        )


def _check_matrix_inputs(kernel_type, x1, x2, params, start, end):
    for t in (x1, x2, params):
        check_cuda(t)
        check_float(t)
    check_cuda_int32(start)
    check_cuda_int32(end)
    batch_shape = tuple(x1.shape[:-1])
    if len(batch_shape) > MAX_BATCH_RANK:
        raise RuntimeError(f"at most {MAX_BATCH_RANK} batch dimensions are supported")
    _check_batch("x2", x2, batch_shape, 1)
    _check_batch("params", params, batch_shape, 1)
    _check_batch("start", start, batch_shape, 1)
    _check_batch("end", end, batch_shape, 1)
    if params.shape[-1] != NUM_PARAMS[kernel_type]:
        raise RuntimeError(
            f"{kernel_type} kernel takes {NUM_PARAMS[kernel_type]} parameters, got {params.shape[-1]}"
        )
    rows = -(-x1.shape[-1] // _BLOCK_SIZE)
    if start.shape[-1] != rows or end.shape[-1] != rows:
        raise RuntimeError(f"start/end must have {rows} entries per batch item")
    return batch_shape


def matmul(kernel_type: str, x1: Tensor, x2: Tensor, rhs: Tensor, params: Tensor, start: Tensor,
           end: Tensor, options: LaunchOptions | None = None, out: Tensor | None = None) -> Tensor:
    """out[..., m, k] = K(x1, x2)[mask] @ rhs   (C ABI: km_matmul).

    ``out`` (optional) is a contiguous fp32 tensor of the result's shape to write into."""
    tensors = (x1, x2, rhs, params, start, end)
    key = _signature("matmul", kernel_type, tensors)
    prepared = _PREPARED.get(key)
    if prepared is None:
        kid = _kernel_id(kernel_type)
        check_cuda(rhs)
        check_float(rhs)
        batch_shape = _check_matrix_inputs(kernel_type, x1, x2, params, start, end)
        _check_batch("rhs", rhs, batch_shape, 2)
        m, n, k = x1.shape[-1], x2.shape[-1], rhs.shape[-1]
        if rhs.shape[-2] != n:
            raise RuntimeError(f"rhs has {rhs.shape[-2]} rows, x2 has {n} points")
        prepared = _remember(key, (
            load_library().km_matmul, (kid, len(batch_shape), _i64(batch_shape), m, n, k),
            tuple(_i64(t.stride()) for t in tensors), tuple(t.numel() > 0 for t in tensors),
            (*batch_shape, m, k),
        ))
    fn, head, strides, nonempty, out_shape = prepared
    device = x1.device
    if out is None:
        out = torch.empty(out_shape, dtype=torch.float32, device=device)
    elif (tuple(out.shape) != out_shape or out.dtype != torch.float32 or out.device != device
          or not out.is_contiguous()):
        raise RuntimeError(f"out must be a contiguous float32 tensor of shape {out_shape} on {device}")
    call_args = []
    for t, st, filled in zip(tensors, strides, nonempty):
        call_args.append(t.data_ptr() if filled else None)
        call_args.append(st)
    with _on_device(device):
        status = fn(*head, *call_args, out.data_ptr() if out.numel() > 0 else None,
                    ctypes.byref(options) if options is not None else None, _stream(device))
    if status != 0:
        _raise(load_library(), status)
    return out


def describe_param_grad(kernel_type: str, num_batches: int, m: int, c: int) -> str:
    """Kernels and decomposition of the parameter gradient for this problem (C ABI: km_param_grad_describe)."""
    lib = load_library()
    text = ctypes.create_string_buffer(512)
    status = lib.km_param_grad_describe(_kernel_id(kernel_type), num_batches, m, c, text, len(text))
    if status != 0:
        _raise(lib, status)
    return text.value.decode()


def describe_matmul(kernel_type: str, num_batches: int, m: int, n: int, k: int,
                    options: LaunchOptions | None = None) -> str:
    """Kernel and decomposition the launch table picks for this problem (C ABI: km_matmul_describe)."""
    lib = load_library()
    text = ctypes.create_string_buffer(256)
    status = lib.km_matmul_describe(_kernel_id(kernel_type), num_batches, m, n, k,
                                    ctypes.byref(options) if options is not None else None, text, 256)
    if status != 0:
        _raise(lib, status)
    return text.value.decode()


# device index -> (stream handle, event recorded after the last km_param_grad_static call there)
_STATIC_SCRATCH_USE: dict = {}


def param_grad(kernel_type: str, x1: Tensor, x2: Tensor, left: Tensor, right: Tensor,
               params: Tensor, start: Tensor, end: Tensor, out: Tensor | None = None,
               static_scratch: bool = False) -> Tensor:
    """grad[..., P] of sum((left @ right^T) * K[mask]) w.r.t. params   (C ABI: km_param_grad).

    ``out`` (optional) is a contiguous fp32 tensor [..., P] to write into.  With
    ``static_scratch`` the call goes to km_param_grad_static, which uses the library's per-GPU
    static scratch instead of a workspace allocated here (together with ``out`` the call then
    allocates nothing).  Every GPU has one such array: a call on another stream than the last
    one is ordered behind it with an event; calls issued from several host threads at once, or
    through the C ABI directly, must be kept apart by the caller."""
    tensors = (x1, x2, left, right, params, start, end)
    key = _signature("param_grad", kernel_type, tensors)
    prepared = _PREPARED.get(key)
    if prepared is None:
        kid = _kernel_id(kernel_type)
        for t in (left, right):
            check_cuda(t)
            check_float(t)
        batch_shape = _check_matrix_inputs(kernel_type, x1, x2, params, start, end)
        _check_batch("left", left, batch_shape, 2)
        _check_batch("right", right, batch_shape, 2)
        m, n, c = x1.shape[-1], x2.shape[-1], left.shape[-1]
        if left.shape[-2] != m or right.shape[-2] != n or right.shape[-1] != c:
            raise RuntimeError(
                f"left {tuple(left.shape)} / right {tuple(right.shape)} do not match a {m} x {n} matrix"
            )
        lib = load_library()
        sizes = _i64(batch_shape)
        need = lib.km_param_grad_workspace_size(kid, len(batch_shape), sizes, m, n, c)
        prepared = _remember(key, (
            (kid, len(batch_shape), sizes, m, n, c),
            tuple(_i64(t.stride()) for t in tensors), tuple(t.numel() > 0 for t in tensors),
            (*batch_shape, params.shape[-1]), need,
        ))
    head, strides, nonempty, out_shape, need = prepared
    lib = load_library()
    device = x1.device
    if out is None:
        out = torch.empty(out_shape, dtype=torch.float32, device=device)
    elif (tuple(out.shape) != out_shape or out.dtype != torch.float32 or out.device != device
          or not out.is_contiguous()):
        raise RuntimeError(f"out must be a contiguous float32 tensor of shape {out_shape} on {device}")
    call_args = []
    for t, st, filled in zip(tensors, strides, nonempty):
        call_args.append(t.data_ptr() if filled else None)
        call_args.append(st)
    out_ptr = out.data_ptr() if out.numel() > 0 else None
    if static_scratch:
        with _on_device(device):
            stream = torch.cuda.current_stream(device)
            last = _STATIC_SCRATCH_USE.get(device.index)
            if last is not None and last[0] != stream.cuda_stream:
                # The GPU's one scratch array was last used on another stream: order this call
                # behind that one (calls from several host threads remain the caller's business).
                stream.wait_event(last[1])
            status = lib.km_param_grad_static(*head, *call_args, out_ptr, _stream(device))
            event = last[1] if last is not None else torch.cuda.Event()
            event.record(stream)
            _STATIC_SCRATCH_USE[device.index] = (stream.cuda_stream, event)
    else:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=device)
        with _on_device(device):
            status = lib.km_param_grad(*head, *call_args, out_ptr, workspace.data_ptr(), need,
                                       _stream(device))
    if status != 0:
        _raise(lib, status)
    return out


def index(kernel_type: str, x1: Tensor, x2: Tensor, params: Tensor, start: Tensor, end: Tensor,
          batch_indices: Sequence[Tensor], row_index: Tensor, col_index: Tensor) -> Tensor:
    """out[q] = K[batch_indices[q]..., row_index[q], col_index[q]]   (C ABI: km_index)."""
    kid = _kernel_id(kernel_type)
    batch_shape = _check_matrix_inputs(kernel_type, x1, x2, params, start, end)
    batch_indices = tuple(batch_indices)
    if len(batch_indices) != len(batch_shape):
        raise RuntimeError(
            f"expected {len(batch_shape)} batch index tensors, got {len(batch_indices)}"
        )
    for t in (*batch_indices, row_index, col_index):
        check_cuda_int32(t)
    if row_index.dim() == 0:  # scalar indices: treat as one entry
        result = index(kernel_type, x1, x2, params, start, end,
                       [b.reshape(1) for b in batch_indices], row_index.reshape(1),
                       col_index.reshape(1))
        return result.reshape(())
    shape = tuple(row_index.shape)
    if len(shape) < 1 or len(shape) > MAX_BATCH_RANK + 1:
        raise RuntimeError(f"index tensors must have between 1 and {MAX_BATCH_RANK + 1} dimensions")
    for t in (*batch_indices, col_index):
        if tuple(t.shape) != shape:
            raise RuntimeError("all index tensors must have the same shape")
    lib = load_library()
    out = torch.empty(shape, dtype=torch.float32, device=x1.device)
    rank = len(batch_shape)
    bi_ptrs, bi_strides, _keep = _batch_index_args(batch_indices, rank)
    with _on_device(x1.device):
        status = lib.km_index(
            kid, rank, _i64(batch_shape), x1.shape[-1], x2.shape[-1],
            *_tensor_args(x1), *_tensor_args(x2), *_tensor_args(params),
            *_tensor_args(start), *_tensor_args(end),
            len(shape), _i64(shape), bi_ptrs, bi_strides,
            *_tensor_args(row_index), *_tensor_args(col_index), _ptr(out), _stream(x1.device),
        )
    if status != 0:
        _raise(lib, status)
    return out


def _batch_index_args(batch_indices, rank):
    bi_ptrs = (_vp * max(rank, 1))(*[t.data_ptr() for t in batch_indices])
    stride_arrays = [_i64(t.stride()) for t in batch_indices]
    bi_strides = (_i64p * max(rank, 1))(*[ctypes.cast(a, _i64p) for a in stride_arrays])
    return bi_ptrs, bi_strides, stride_arrays  # the arrays must outlive the call


def index_bwd(kernel_type: str, x1: Tensor, x2: Tensor, params: Tensor, start: Tensor, end: Tensor,
              batch_indices: Sequence[Tensor], row_index: Tensor, col_index: Tensor,
              out_grad: Tensor) -> Tensor:
    """grad[..., P] of sum(out_grad * index(...)) w.r.t. params   (C ABI: km_index_bwd)."""
    kid = _kernel_id(kernel_type)
    batch_shape = _check_matrix_inputs(kernel_type, x1, x2, params, start, end)
    batch_indices = tuple(batch_indices)
    if len(batch_indices) != len(batch_shape):
        raise RuntimeError(
            f"expected {len(batch_shape)} batch index tensors, got {len(batch_indices)}"
        )
    for t in (*batch_indices, row_index, col_index):
        check_cuda_int32(t)
    check_cuda(out_grad)
    check_float(out_grad)
    if row_index.dim() == 0:
        return index_bwd(kernel_type, x1, x2, params, start, end,
                         [b.reshape(1) for b in batch_indices], row_index.reshape(1),
                         col_index.reshape(1), out_grad.reshape(1))
    shape = tuple(row_index.shape)
    for t in (*batch_indices, col_index, out_grad):
        if tuple(t.shape) != shape:
            raise RuntimeError("all index tensors and out_grad must have the same shape")
    lib = load_library()
    rank = len(batch_shape)
    grad = torch.empty((*batch_shape, params.shape[-1]), dtype=torch.float32, device=x1.device)
    need = lib.km_index_bwd_workspace_size(row_index.numel())
    workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=x1.device)
    bi_ptrs, bi_strides, _keep = _batch_index_args(batch_indices, rank)
    with _on_device(x1.device):
        status = lib.km_index_bwd(
            kid, rank, _i64(batch_shape), x1.shape[-1], x2.shape[-1],
            *_tensor_args(x1), *_tensor_args(x2), *_tensor_args(params),
            *_tensor_args(start), *_tensor_args(end),
            len(shape), _i64(shape), bi_ptrs, bi_strides,
            *_tensor_args(row_index), *_tensor_args(col_index), *_tensor_args(out_grad),
            _ptr(grad), ctypes.c_void_p(workspace.data_ptr()), need, _stream(x1.device),
        )
    if status != 0:
        _raise(lib, status)
    return grad


def dense(kernel_type: str, x1: Tensor, x2: Tensor, params: Tensor, start: Tensor,
          end: Tensor) -> Tensor:
    """Masked kernel matrix [..., m, n]   (C ABI: km_dense)."""
    kid = _kernel_id(kernel_type)
    batch_shape = _check_matrix_inputs(kernel_type, x1, x2, params, start, end)
    lib = load_library()
    out = torch.empty((*batch_shape, x1.shape[-1], x2.shape[-1]), dtype=torch.float32, device=x1.device)
    with _on_device(x1.device):
        status = lib.km_dense(
            kid, len(batch_shape), _i64(batch_shape), x1.shape[-1], x2.shape[-1],
            *_tensor_args(x1), *_tensor_args(x2), *_tensor_args(params),
            *_tensor_args(start), *_tensor_args(end), _ptr(out), _stream(x1.device),
        )
    if status != 0:
        _raise(lib, status)
    return out


def dense_bwd(kernel_type: str, x1: Tensor, x2: Tensor, params: Tensor, start: Tensor, end: Tensor,
              out_grad: Tensor) -> Tensor:
    """grad[..., P] of sum(out_grad * dense(...)) w.r.t. params   (C ABI: km_dense_bwd)."""
    kid = _kernel_id(kernel_type)
    check_cuda(out_grad)
    check_float(out_grad)
    batch_shape = _check_matrix_inputs(kernel_type, x1, x2, params, start, end)
    _check_batch("out_grad", out_grad, batch_shape, 2)
    m, n = x1.shape[-1], x2.shape[-1]
    if tuple(out_grad.shape[-2:]) != (m, n):
        raise RuntimeError(f"out_grad has shape {tuple(out_grad.shape)}, expected (..., {m}, {n})")
    lib = load_library()
    sizes = _i64(batch_shape)
    grad = torch.empty((*batch_shape, params.shape[-1]), dtype=torch.float32, device=x1.device)
    need = lib.km_param_grad_workspace_size(kid, len(batch_shape), sizes, m, n, 0)
    workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=x1.device)
    with _on_device(x1.device):
        status = lib.km_dense_bwd(
            kid, len(batch_shape), sizes, m, n,
            *_tensor_args(x1), *_tensor_args(x2), *_tensor_args(params),
            *_tensor_args(start), *_tensor_args(end), *_tensor_args(out_grad),
            _ptr(grad), ctypes.c_void_p(workspace.data_ptr()), need, _stream(x1.device),
        )
    if status != 0:
        _raise(lib, status)
    return grad


# -- ranges ------------------------------------------------------------------------------
def make_ranges_2d(x1: Tensor, x2: Tensor | None, cutoff: float, block_size: int,
                   align: bool) -> tuple[Tensor, Tensor]:
    """Range builders on flattened [batch, n] inputs; result lives on x1's device.

    Host tensors go through the sequential host builders, device tensors through the device
    builders (no host round trip).  The device builders find the scans' results by binary
    search and therefore require what the pattern itself requires: every row of x1 / x2 sorted
    ascending.  On unsorted rows the host and device builders return different (equally
    meaningless) patterns.
    """
    lib = load_library()
    if x1.dtype != torch.float32 or (x2 is not None and x2.dtype != torch.float32):
        raise RuntimeError("expected scalar type Float for range inputs")
    x1c = x1.detach().contiguous()
    x2c = x2.detach().contiguous() if x2 is not None else None
    num_batch, n1 = x1c.shape
    rows = -(-n1 // block_size)
    start = torch.empty((num_batch, rows), dtype=torch.int32, device=x1.device)
    end = torch.empty((num_batch, rows), dtype=torch.int32, device=x1.device)
    if x1.is_cuda:
        if x2c is not None and x2c.device != x1c.device:
            x2c = x2c.to(x1c.device)  # the reference accepts mixed devices (it copies both to the host)
        with _on_device(x1.device):
            if x2c is None:
                status = lib.km_make_ranges_symmetric_device(
                    _ptr(x1c), num_batch, n1, float(cutoff), block_size, _ptr(start), _ptr(end),
                    _stream(x1.device))
            else:
                status = lib.km_make_ranges_device(
                    _ptr(x1c), _ptr(x2c), num_batch, n1, x2c.shape[1], float(cutoff), block_size,
                    int(bool(align)), _ptr(start), _ptr(end), _stream(x1.device))
    else:
        if x2c is None:
            status = lib.km_make_ranges_symmetric(
                _ptr(x1c), num_batch, n1, float(cutoff), block_size, _ptr(start), _ptr(end))
        else:
            x2c = x2c.cpu()
            status = lib.km_make_ranges(
                _ptr(x1c), _ptr(x2c), num_batch, n1, x2c.shape[1], float(cutoff), block_size,
                int(bool(align)), _ptr(start), _ptr(end))
    if status != 0:
        _raise(lib, status)
    return start, end


def transpose_ranges_2d(start: Tensor, end: Tensor, x1_size: int, x2_size: int,
                        block_size: int) -> tuple[Tensor, Tensor]:
    lib = load_library()
    device = start.device
    s = start.detach().to("cpu", torch.int32).contiguous()
    e = end.detach().to("cpu", torch.int32).contiguous()
    num_batch, rows = s.shape
    cols = -(-x2_size // block_size)
    start_t = torch.empty((num_batch, cols), dtype=torch.int32)
    end_t = torch.empty((num_batch, cols), dtype=torch.int32)
    status = lib.km_transpose_ranges(_ptr(s), _ptr(e), num_batch, rows, x1_size, x2_size, block_size,
                                     _ptr(start_t), _ptr(end_t))
    if status != 0:
        _raise(lib, status)
    return start_t.to(device), end_t.to(device)
