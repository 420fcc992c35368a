"""ctypes binding of ``libet_hip.so`` — the C ABI declared in ``include/et_abi.h``.

This module is plumbing for the test-suite, ``bench.py`` and the smoke test: it
loads the in-tree shared library, declares argument types, and offers a small
``DeviceBuffer`` on top of ``et_malloc``.  There is no CPU fallback: if the
library is missing, :func:`lib` raises.

The directory name contains a hyphen, so import it with
``__graft_entry__.load_package()`` (module name ``scpaper_2021_amd``).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "lib" / "libet_hip.so"

ET_OK = 0
ET_ERR_INVALID_ARG = -1
ET_ERR_UNSUPPORTED = -2
ET_ERR_ALLOC = -3
ET_ERR_LAUNCH = -4
ET_ERR_IO = -5
ET_ERR_NO_DEVICE = -6

ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
MHA_CAUSAL = 1

_vp = C.c_void_p
_i = C.c_int
_sz = C.c_size_t
_f = C.c_float
_ll = C.c_longlong
_u16 = C.c_uint16

# name -> (argtypes)  ; every function returns int unless listed in _RESTYPES
_SIGNATURES = {
    "et_device_info": (C.c_char_p, _i, C.POINTER(_i), C.POINTER(_i)),
    "et_malloc": (C.POINTER(_vp), _sz),
    "et_free": (_vp,),
    "et_memset": (_vp, _i, _sz, _vp),
    "et_memcpy_h2d": (_vp, _vp, _sz),
    "et_memcpy_d2h": (_vp, _vp, _sz),
    "et_memcpy_d2d": (_vp, _vp, _sz, _vp),
    "et_fill_f16": (_vp, _sz, _u16, _vp),
    "et_fill_i32": (_vp, _sz, C.c_int32, _vp),
    "et_f32_to_f16": (_vp, _vp, _sz, _vp),
    "et_f16_to_f32": (_vp, _vp, _sz, _vp),
    "et_stream_create": (C.POINTER(_vp),),
    "et_stream_destroy": (_vp,),
    "et_stream_sync": (_vp,),
    "et_device_sync": (),
    "et_event_create": (C.POINTER(_vp),),
    "et_event_destroy": (_vp,),
    "et_event_record": (_vp, _vp),
    "et_event_sync": (_vp,),
    "et_event_elapsed_ms": (C.POINTER(_f), _vp, _vp),
    "et_linear_bsr16_f16": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_bsr16_f16_geom": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp),
    "et_linear_dense_f16": (_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_gemm_f16": (_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _ll, _ll, _ll, _vp),
    "et_linear_rowpruned_f16": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_rowpruned_compact_f16": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _vp),
    "et_linear_colpruned_f16": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_mha_fused_f16": (_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _i, _vp),
    "et_skip_layernorm_f16": (_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp),
    "et_layernorm_f16": (_vp, _vp, _vp, _vp, _i, _i, _f, _vp),
    "et_gelu_f16": (_vp, _vp, _sz, _vp),
    "et_relu_f16": (_vp, _vp, _sz, _vp),
    "et_bias_add_f16": (_vp, _vp, _i, _i, _vp),
}
_RESTYPES = {"et_status_string": C.c_char_p, "et_last_error": C.c_char_p}

_lib = None


class EtError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"et status {status}: {message}")
        self.status = status


def lib() -> C.CDLL:
    """The loaded native library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python scpaper-2021_amd/build.py` "
                "(there is no CPU fallback)")
        handle = C.CDLL(str(LIB_PATH))
        for name, args in _SIGNATURES.items():
            fn = getattr(handle, name, None)
            if fn is None:
                continue  # reported by the symbol test, not at import
            fn.argtypes = list(args)
            fn.restype = _i
        handle.et_status_string.argtypes = [_i]
        handle.et_status_string.restype = C.c_char_p
        handle.et_last_error.argtypes = []
        handle.et_last_error.restype = C.c_char_p
        _lib = handle
    return _lib


def check(status: int) -> None:
    if status != ET_OK:
        raise EtError(status, lib().et_last_error().decode(errors="replace"))


def _ptr(x) -> int | None:
    if x is None:
        return None
    if isinstance(x, DeviceBuffer):
        return x.ptr
    return int(x)


class DeviceBuffer:
    """A device allocation owned through et_malloc / et_free."""

    def __init__(self, nbytes: int):
        p = _vp()
        check(lib().et_malloc(C.byref(p), nbytes))
        self.ptr = p.value
        self.nbytes = int(nbytes)
        self.dtype = None
        self.shape = None

    @classmethod
    def from_numpy(cls, arr: np.ndarray) -> "DeviceBuffer":
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.dtype, buf.shape = arr.dtype, arr.shape
        check(lib().et_memcpy_h2d(buf.ptr, arr.ctypes.data, arr.nbytes))
        return buf

    @classmethod
    def empty(cls, shape, dtype) -> "DeviceBuffer":
        dtype = np.dtype(dtype)
        n = int(np.prod(shape)) * dtype.itemsize
        buf = cls(n)
        buf.dtype, buf.shape = dtype, tuple(shape)
        return buf

    def numpy(self, dtype=None, shape=None) -> np.ndarray:
        dtype = np.dtype(dtype or self.dtype)
        shape = tuple(shape if shape is not None else self.shape)
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        check(lib().et_device_sync())
        check(lib().et_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes))
        return out

    def offset(self, nbytes: int) -> int:
        return self.ptr + int(nbytes)

    def free(self) -> None:
        if self.ptr:
            lib().et_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def device_info() -> dict:
    name = C.create_string_buffer(256)
    cu, lds = _i(), _i()
    check(lib().et_device_info(name, 256, C.byref(cu), C.byref(lds)))
    return {"name": name.value.decode(), "num_cu": cu.value, "lds_bytes": lds.value}


def sync() -> None:
    check(lib().et_device_sync())


class Timer:
    """hipEvent pair on a stream (NULL stream by default)."""

    def __init__(self, stream=None):
        self.stream = stream
        self.start, self.stop = _vp(), _vp()
        check(lib().et_event_create(C.byref(self.start)))
        check(lib().et_event_create(C.byref(self.stop)))

    def __enter__(self):
        check(lib().et_event_record(self.start, self.stream))
        return self

    def __exit__(self, *exc):
        check(lib().et_event_record(self.stop, self.stream))
        check(lib().et_event_sync(self.stop))
        ms = _f()
        check(lib().et_event_elapsed_ms(C.byref(ms), self.start, self.stop))
        self.ms = ms.value
        return False

    def __del__(self):
        try:
            lib().et_event_destroy(self.start)
            lib().et_event_destroy(self.stop)
        except Exception:
            pass


# ---------------------------------------------------------------------------
# Thin operator wrappers (device buffers in, status checked).
# ---------------------------------------------------------------------------

def linear_bsr16(row_ptr, col_idx, tiles, bias, X, Y, T, n_in, n_out, act=ACT_NONE, stream=None):
    check(lib().et_linear_bsr16_f16(_ptr(row_ptr), _ptr(col_idx), _ptr(tiles), _ptr(bias), _ptr(X),
                                    _ptr(Y), T, n_in, n_out, act, stream))


def linear_dense(W, bias, X, Y, T, n_in, n_out, act=ACT_NONE, stream=None):
    check(lib().et_linear_dense_f16(_ptr(W), _ptr(bias), _ptr(X), _ptr(Y), T, n_in, n_out, act,
                                    stream))


def gemm(A, B, Cm, M, N, K, lda, ldb, ldc, trans_b=True, batch=1, sa=0, sb=0, sc=0, stream=None):
    check(lib().et_gemm_f16(_ptr(A), _ptr(B), _ptr(Cm), M, N, K, lda, ldb, ldc, int(bool(trans_b)),
                            batch, sa, sb, sc, stream))


def mha_fused(Q, K, V, ldq, ldk, ldv, Z, ldz, mask, lens, B, S, nh, hd, scale, flags=0, stream=None):
    check(lib().et_mha_fused_f16(_ptr(Q), _ptr(K), _ptr(V), ldq, ldk, ldv, _ptr(Z), ldz, _ptr(mask),
                                 _ptr(lens), B, S, nh, hd, scale, flags, stream))


def skip_layernorm(out, src, skip, gamma, beta, rows, H, eps=1e-5, stream=None):
    check(lib().et_skip_layernorm_f16(_ptr(out), _ptr(src), _ptr(skip), _ptr(gamma), _ptr(beta),
                                      rows, H, eps, stream))


def layernorm(out, src, gamma, beta, rows, H, eps=1e-5, stream=None):
    check(lib().et_layernorm_f16(_ptr(out), _ptr(src), _ptr(gamma), _ptr(beta), rows, H, eps, stream))
