"""Drop-in for fairscale's pybind extension ``fairscale.fused_adam_cuda``
(``fairscale/clib/fused_adam_cuda/fused_adam_cuda.cpp:4-8``): copy this file to
``fairscale/fused_adam_cuda.py`` and ``fairscale.optim.Adam`` (``fairscale/optim/adam.py:17,261-276``)
runs its step on ``libfsadam.so``.  Self-contained on purpose: ctypes and torch only.

The library is looked up in ``$FSADAM_LIBRARY``, else as ``libfsadam.so`` on the loader's path.
"""
import ctypes
import os

import torch  # first: the library must bind to the HIP runtime torch has already mapped


class _Tensor(ctypes.Structure):  # FsAdamTensor, include/fsadam.h
    _fields_ = [("p", ctypes.c_void_p), ("m", ctypes.c_void_p), ("v", ctypes.c_void_p),
                ("g", ctypes.c_void_p), ("p_copy", ctypes.c_void_p), ("numel", ctypes.c_int64)]


_lib = ctypes.CDLL(os.environ.get("FSADAM_LIBRARY", "libfsadam.so"))
_f, _i = ctypes.c_float, ctypes.c_int
_lib.fsadam_step.restype = _i
_lib.fsadam_step.argtypes = [ctypes.POINTER(_Tensor), ctypes.c_int64, _i, _f, _f, _f, _f, _f, _f, _f, _i, _i, _i,
                             ctypes.c_void_p, ctypes.c_void_p]
_lib.fsadam_last_error.restype = ctypes.c_char_p

_F32, _F16 = torch.float32, torch.float16


# element types of [p, m, v, g(, p_copy)] per FSADAM_* code: the combinations fused_adam_cuda_kernel.cu:165-263 dispatches on
_DTYPES = {0: (_F32, _F32, _F32, _F32), 1: (_F32, _F32, _F32, _F16, _F16), 2: (_F16, _F32, _F32, _F16), 3: (_F16, _F16, _F16, _F16)}


def _mode(lists):
    """The dtype dispatch of fused_adam_cuda_kernel.cu:165-263 on the first tensor of each list, as FSADAM_* codes."""
    if len(lists) not in (4, 5) or len(lists[0]) == 0:
        raise RuntimeError("tensor_lists must be 4 or 5 non-empty lists")  # multi_tensor_apply.cuh:49-51
    first = tuple(lst[0].dtype for lst in lists)
    for code, dtypes in _DTYPES.items():
        if first == dtypes:
            return code
    raise RuntimeError(f"no kernel for tensor lists of dtypes {first}")  # kernel.cu:167-176,196-199,258,261


def adam(chunk_size, noop_flag, tensor_lists, lr, beta1, beta2, eps, grad_scale, optim_scale, found_inf, step, mode,
         bias_correction, decay):
    """Same 14 positional arguments as the pybind function.  ``chunk_size`` and ``noop_flag`` are ignored
    (the reference kernel never reads ``noop_flag``, fused_adam_cuda_kernel.cu:26).  The kernels index raw memory,
    so what the reference leaves to asserts is checked here for every tensor: dtype per list, one device, equal sizes."""
    code = _mode(tensor_lists)
    dtypes = _DTYPES[code]
    n = len(tensor_lists[0])
    if any(len(lst) != n for lst in tensor_lists):
        raise RuntimeError("Size mismatch among tensor lists")  # multi_tensor_apply.cuh:55
    device = tensor_lists[0][0].device
    rows = (_Tensor * n)()
    for t in range(n):
        cols = [lst[t] for lst in tensor_lists]
        if not all(c.is_contiguous() and c.is_cuda and c.numel() == cols[0].numel() for c in cols):
            raise RuntimeError("tensor lists must hold contiguous device tensors of equal numel")  # multi_tensor_apply.cuh:59-65
        if not all(c.dtype == d and c.device == device for c, d in zip(cols, dtypes)):
            raise RuntimeError(f"tensor {t}: every list must hold one dtype ({dtypes}) on one device")
        rows[t].p, rows[t].m, rows[t].v, rows[t].g = (c.data_ptr() for c in cols[:4])
        rows[t].p_copy = cols[4].data_ptr() if len(cols) == 5 else None
        rows[t].numel = cols[0].numel()
    if found_inf.dtype != _F32 or found_inf.device != device:
        raise RuntimeError("found_inf must be a float32 tensor on the lists' device")
    stream = torch.cuda.current_stream(device).cuda_stream  # the hipStream_t under ROCm
    rc = _lib.fsadam_step(rows, n, code, lr, beta1, beta2, eps, grad_scale, optim_scale, decay, step, mode,
                          bias_correction, found_inf.data_ptr(), stream)
    if rc != 0:
        raise RuntimeError(_lib.fsadam_last_error().decode())
