"""ctypes binding of libtrittention_hip.so (C ABI: include/trittention_hip.h).

PyTorch is used only for device memory and the current HIP stream; tensors
cross the boundary as raw pointers.  There is no fallback: if the library is
missing every call raises.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtrittention_hip.so")
CSRC_DIR = os.path.join(os.path.dirname(_HERE), "csrc")

TRITT_F32, TRITT_BF16, TRITT_F16 = 0, 1, 2
FLAG_AUTO, FLAG_FORCE_GENERIC, FLAG_FORCE_MFMA, FLAG_FLOAT_ATOMICS, FLAG_SPLIT_OPERANDS = 0, 1, 2, 4, 8

_DTYPES = {torch.float32: TRITT_F32, torch.bfloat16: TRITT_BF16, torch.float16: TRITT_F16}

_vp, _i, _f, _sz, _u = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_uint


class Layout(ctypes.Structure):
    """tritt_layout: element strides of a [B,H,T,D] view whose last dimension is dense."""
    _fields_ = [("stride_b", ctypes.c_longlong), ("stride_h", ctypes.c_longlong), ("stride_t", ctypes.c_longlong)]


_lp = ctypes.POINTER(Layout)

_PROTOS = {
    "tritt_version": (_i, []),
    "tritt_status_string": (ctypes.c_char_p, [_i]),
    "tritt_set_tuning": (_i, [_i, _i, ctypes.POINTER(_i)]),
    "tritt_probe_mfma": (_i, [_vp, _i, _i, _vp]),
    "tritt_tdp_fwd_workspace_bytes": (_sz, [_i] * 10 + [_u]),
    "tritt_tdp_fwd": (_i, [_vp] * 7 + [_i] * 5 + [_f] + [_i] * 5 + [_vp, _sz, _u, _vp]),
    "tritt_static_scratch_bytes": (_sz, []),
    "tritt_tdp_fwd_static_scratch": (_i, [_vp] * 7 + [_i] * 5 + [_f] + [_i] * 5 + [_u, _vp]),
    "tritt_tdp_bwd_workspace_bytes": (_sz, [_i] * 10 + [_u]),
    "tritt_tdp_bwd": (_i, [_vp] * 13 + [_i] * 5 + [_f] + [_i] * 5 + [_vp, _sz, _u, _vp]),
    "tritt_dps_fwd_workspace_bytes": (_sz, [_i] * 5 + [_u]),
    "tritt_dps_fwd": (_i, [_vp] * 7 + [_i] * 5 + [_f] + [_i] * 2 + [_vp, _sz, _u, _vp]),
    "tritt_dps_bwd_workspace_bytes": (_sz, [_i] * 5 + [_u]),
    "tritt_dps_bwd": (_i, [_vp] * 13 + [_i] * 5 + [_f] + [_i] * 2 + [_vp, _sz, _u, _vp]),
    "tritt_tdp_fwd_strided_workspace_bytes": (_sz, [_i] * 10 + [_u, _lp]),
    "tritt_tdp_fwd_strided": (_i, [_vp] * 5 + [_lp] + [_vp] * 2 + [_i] * 5 + [_f] + [_i] * 5 + [_vp, _sz, _u, _vp]),
    "tritt_tdp_bwd_strided_workspace_bytes": (_sz, [_i] * 10 + [_u, _lp, _lp]),
    "tritt_tdp_bwd_strided": (_i, [_vp] * 5 + [_lp] + [_vp] * 3 + [_lp] + [_vp] * 5 + [_i] * 5 + [_f] + [_i] * 5
                              + [_vp, _sz, _u, _vp]),
    "tritt_dps_fwd_strided_workspace_bytes": (_sz, [_i] * 5 + [_u, _lp]),
    "tritt_dps_fwd_strided": (_i, [_vp] * 5 + [_lp] + [_vp] * 2 + [_i] * 5 + [_f] + [_i] * 2 + [_vp, _sz, _u, _vp]),
    "tritt_dps_bwd_strided_workspace_bytes": (_sz, [_i] * 5 + [_u, _lp, _lp]),
    "tritt_dps_bwd_strided": (_i, [_vp] * 5 + [_lp] + [_vp] * 3 + [_lp] + [_vp] * 5 + [_i] * 5 + [_f] + [_i] * 2
                              + [_vp, _sz, _u, _vp]),
}

_lib = None


def build(verbose: bool = False) -> str:
    """Compile the HIP sources for gfx950 (always recompiles)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-C", CSRC_DIR, "-B", "-j8"], stdout=out, stderr=out)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
                "(there is no fallback implementation)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _PROTOS.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def exported_symbols():
    return list(_PROTOS)


(TUNE_FWD_SPLITS, TUNE_FWD_BAND, TUNE_BWD_SPLITS, TUNE_BWD128_WAVES, TUNE_F32_VALU, TUNE_DPS_WAVES, TUNE_DPS_PAIR,
 TUNE_DPS_SHARED) = range(8)


def set_tuning(knob: int, value: int) -> int:
    """tritt_set_tuning, returning the previous value; remembered workspace sizes may depend on the knobs."""
    _workspace_sizes.clear()
    previous = _i(0)
    check(lib().tritt_set_tuning(knob, value, ctypes.byref(previous)), "tritt_set_tuning")
    return previous.value


class tuning:
    """``with _lib.tuning(_lib.TUNE_BWD_SPLITS, 4): ...`` (tests and sweeps): sets a knob of the library and
    puts the previous value back on exit."""

    def __init__(self, knob: int, value: int):
        self.knob, self.value = knob, value

    def __enter__(self):
        self.previous = set_tuning(self.knob, self.value)
        return self

    def __exit__(self, *exc):
        set_tuning(self.knob, self.previous)
        return False


_flagged = {}


def flagged_subclass(cls, flags: int):
    """A subclass of an autograd Function whose IMPL_FLAGS is `flags` (one per (class, flags), cached)."""
    flags = int(flags)
    if flags == cls.IMPL_FLAGS:
        return cls
    key = (cls, flags)
    if key not in _flagged:
        _flagged[key] = type(f"{cls.__name__}Flags{flags}", (cls,), {"IMPL_FLAGS": flags})
    return _flagged[key]


def dtype_code(dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16") from None


def check(status: int, what: str):
    if status != 0:
        msg = lib().tritt_status_string(status).decode()
        raise RuntimeError(f"{what} failed: {msg} (status {status})")


def require_gpu(t: torch.Tensor, what: str):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: tensors must live on a GPU (got {t.device}); "
                           "this library has no CPU implementation")


def dense(t):
    """Contiguous and 16-byte aligned (what the library requires of every [B,H,T,D] tensor): a
    contiguous view that starts in the middle of a storage is copied."""
    t = t.contiguous()
    if t.data_ptr() % 16:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def viewable(t) -> bool:
    """Whether the library can read `t` (a [B,H,T,D] view) where it lies: dense last dimension, every other stride
    a non-negative multiple of 16 bytes, 16-byte aligned start (tritt_layout's contract)."""
    unit = 16 // t.element_size()
    B, H, T, D = t.shape
    if (D > 1 and t.stride(3) != 1) or t.data_ptr() % 16:
        return False
    return all(n == 1 or (s >= 0 and s % unit == 0) for n, s in zip((B, H, T), t.stride()[:3]))


def view(t):
    """`t` as the library can take it: the tensor itself when `viewable`, else a dense copy (what the reference
    does with every input: triple_dot_product/flash_trittention.py:64-68)."""
    return t if viewable(t) else dense(t)


def layouts(tensors):
    """A tritt_layout array for `tensors`, or None when every one of them is dense (the plain entry points serve)."""
    if all(t.is_contiguous() for t in tensors):
        return None
    arr = (Layout * len(tensors))()
    for slot, t in zip(arr, tensors):
        # dimensions of extent 1 may carry any stride: the library ignores them, ctypes needs them in range
        slot.stride_b, slot.stride_h, slot.stride_t = (s if n > 1 else 0 for n, s in zip(t.shape[:3], t.stride()[:3]))
    return arr


def layouts_key(arr):
    """Hashable form of a layout array (workspace sizes are remembered per argument tuple)."""
    return None if arr is None else tuple((l.stride_b, l.stride_h, l.stride_t) for l in arr)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def workspace(nbytes: int, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


class on_device:
    """``with on_device(t.device):`` makes the tensor's GPU current around a library call (the backward may run on
    an autograd thread whose current device is another one).  When it already is current, which is the usual case,
    nothing is switched: torch's own guard costs several microseconds per call, as much as a small launch."""

    __slots__ = ("guard",)

    def __init__(self, device):
        self.guard = None if torch.cuda.current_device() == device.index else torch.cuda.device(device)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()
        return self

    def __exit__(self, *exc):
        if self.guard is not None:
            return self.guard.__exit__(*exc)
        return False


_workspace_sizes = {}


def workspace_bytes(query: str, *args) -> int:
    """A `*_workspace_bytes` query of the library, remembered per argument tuple (the answer depends on nothing
    else, except the tuning knobs: `tuning` and the tests' knob changes clear the memory).  Layout arrays in `args`
    enter the key by value."""
    key = (query, tuple(layouts_key(a) if isinstance(a, ctypes.Array) else a for a in args))
    size = _workspace_sizes.get(key)
    if size is None:
        size = _workspace_sizes[key] = getattr(lib(), query)(*args)
    return size
