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
import os as _os

# ET_LIB_PATH selects another build of the same library (kernel tuning experiments).
LIB_PATH = Path(_os.environ.get("ET_LIB_PATH") or (PKG_DIR / "lib" / "libet_hip.so"))

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
    "et_pool_private_begin": (_sz,),
    "et_pool_private_end": (),
    "et_memset": (_vp, _i, _sz, _vp),
    "et_memcpy_h2d": (_vp, _vp, _sz),
    "et_memcpy_d2h": (_vp, _vp, _sz),
    "et_memcpy_d2d": (_vp, _vp, _sz, _vp),
    "et_memcpy_auto": (_vp, _vp, _sz),
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
    "et_linear_bsr16_f16_f32out": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_skip_layernorm_mixed": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp),
    "et_bsr16_plan_create": (_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, C.POINTER(_vp)),
    "et_bsr16_plan_destroy": (_vp,),
    "et_bsr16_plan_info": (_vp, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)),
    "et_linear_bsr16_planned_f16": (_vp, _vp, _vp, _vp, _vp, _i, _i, _vp),
    "et_bsr16_pack_create": (_vp, _vp, _vp, _i, _i, _i, _i, _i, C.POINTER(_vp)),
    "et_bsr16_pack_create_geom": (_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, C.POINTER(_vp)),
    "et_bsr16_pack_destroy": (_vp,),
    "et_bsr16_pack_info": (_vp, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)),
    "et_linear_bsr16_packed_f16": (_vp, _vp, _vp, _vp, _vp, _i, _i, _vp),
    "et_linear_bsr16_packed_resid_stats_f32": (_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, C.POINTER(_i), _i, _vp),
    "et_norm_linear_bsr16_packed_f32in": (_vp, _vp, _vp, _i, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _vp),
    "et_encoder_chain_supported": (_vp,),
    "et_encoder_chain_f32": (_vp, C.POINTER(_i), _vp),
    "et_encoder_chain_status": (_vp, C.POINTER(_i), C.POINTER(_i)),
    "et_probe_empty": (_i, _i, _vp),
    "et_probe_read": (_vp, _sz, _i, _i, _i, _i, _vp, _vp),
    "et_linear_bsr16_f16_geom": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp),
    "et_skipln_linear_bsr16_f16": (_vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_bsr16_fused_ln_supported": (_i, _i, _i),
    "et_linear_bsr16_resid_stats_f16": (_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, C.POINTER(_i), _i, _i, _i, _vp),
    "et_norm_linear_bsr16_f16": (_vp, _vp, _vp, _i, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_norm_from_stats_f16": (_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _f, _vp),
    "et_linear_dense_f32": (_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_bsr16_f32": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_rowpruned_f32": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_rowpruned_compact_f32": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _vp),
    "et_linear_colpruned_f32": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_vec1x16_f32": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_csr_f32": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_mha_fused_f32": (_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _i, _vp),
    "et_skip_layernorm_f32": (_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp),
    "et_layernorm_f32": (_vp, _vp, _vp, _vp, _i, _i, _f, _vp),
    "et_gelu_f32": (_vp, _vp, _sz, _vp),
    "et_relu_f32": (_vp, _vp, _sz, _vp),
    "et_gather_cols_f16": (_vp, _vp, _vp, _i, _i, _i, _vp),
    "et_linear_colpruned_ws_f16": (_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_colpruned_static_f16": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_dense_f16": (_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_gemm_f16": (_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _ll, _ll, _ll, _vp),
    "et_linear_rowpruned_f16": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_linear_rowpruned_compact_f16": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _vp),
    "et_linear_colpruned_f16": (_vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_mha_fused_f16": (_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _i, _vp),
    "et_mha_fuseo_f16": (_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _i,
                         _vp, _vp, _vp, _vp, _vp, _i, _vp),
    "et_mha_fuseo_f16_geom": (_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _i,
                              _vp, _vp, _vp, _vp, _vp, _i, _i, _vp),
    "et_skip_layernorm_f16": (_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp),
    "et_layernorm_f16": (_vp, _vp, _vp, _vp, _i, _i, _f, _vp),
    "et_gelu_f16": (_vp, _vp, _sz, _vp),
    "et_relu_f16": (_vp, _vp, _sz, _vp),
    "et_bias_add_f16": (_vp, _vp, _i, _i, _vp),
    "et_fill_rows_bias_f16": (_vp, _vp, _i, _i, _vp),
    "et_linear_vec1x16_f16": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_vec1x16_to_dense_f16": (_vp, _vp, _vp, _vp, _i, _i, _vp),
    "et_bsr16_to_dense_f16": (_vp, _vp, _vp, _vp, _i, _i, _vp),
    "et_linear_bsr16_resid_stats_f32_supported": (_i, _i, _i),
    "et_norm_linear_bsr16_f32in_supported": (_i, _i, _i),
    "et_linear_bsr16_resid_stats_f32": (_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp),
    "et_linear_bsr16_resid16_stats_f32": (_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp),
    "et_norm_linear_bsr16_f32in": (_vp, _vp, _i, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_norm_from_stats_f32in": (_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _f, _vp),
    "et_linear_csr_f16": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp),
    "et_mha_compactv_f16": (_vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i,
                            _f, _i, _vp),
    "et_norm_qkv_mha_f32in_supported": (_i, _i, _i, _i, _i),
    "et_qkv_heads_pack_create": (_vp, _vp, _vp, _i, _i, C.POINTER(_vp)),
    "et_norm_qkv_mha_f32in": (_vp, _vp, _vp, _i, _vp, _vp, _f, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _f, _i, _vp),
    "et_qkv_heads_pack_create_folded": (_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, C.POINTER(_vp)),
    "et_mha_probs_f16": (_vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _i, _i, _f, _i, _vp),
    "et_mha_unfused_f16": (_vp, _vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _f, _i, _vp),
    "et_linear_vo_f16": (_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp),
    "et_linear_vo_t_f16": (_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp),
    "et_transpose_heads_f16": (_vp, _vp, _i, _i, _i, _vp),
    "et_mha_vo_f16": (_vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp),
    "et_linear_vo_keys_f16": (_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp),
    "et_mha_vo_otf_f16": (_vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp),
    "et_graph_begin_capture": (_vp,),
    "et_graph_end_capture": (_vp, C.POINTER(_vp)),
    "et_graph_launch": (_vp, _vp),
    "et_graph_destroy": (_vp,),
    "et_model_create": (_vp, C.POINTER(_vp)),
    "et_model_set_bsr16": (_vp, _i, _i, _vp, _vp, _vp, _i, _vp),
    "et_model_set_bsr16_f16": (_vp, _i, _i, _vp, _vp, _vp, _i, _vp),
    "et_model_set_dense": (_vp, _i, _i, _vp, _vp),
    "et_model_set_dense_f16": (_vp, _i, _i, _vp, _vp),
    "et_model_set_norm": (_vp, _i, _i, _vp, _vp),
    "et_model_set_norm_f16": (_vp, _i, _i, _vp, _vp),
    "et_model_set_lens": (_vp, _vp),
    "et_model_set_mask": (_vp, _vp),
    "et_model_finalize": (_vp,),
    "et_model_load": (C.c_char_p, C.c_char_p, _vp, C.POINTER(_vp)),
    "et_model_forward": (_vp, _vp, _vp, _vp),
    "et_model_forward_layer": (_vp, _i, _vp, _vp, _vp),
    "et_model_sync": (_vp,),
    "et_model_launches_per_layer": (_vp, C.POINTER(_i)),
    "et_model_destroy": (_vp,),
    "et_model_f32_create": (_vp, C.POINTER(_vp)),
    "et_model_f32_set_bsr16": (_vp, _i, _i, _vp, _vp, _vp, _i, _vp),
    "et_model_f32_set_dense": (_vp, _i, _i, _vp, _vp),
    "et_model_f32_set_norm": (_vp, _i, _i, _vp, _vp),
    "et_model_f32_set_lens": (_vp, _vp),
    "et_model_f32_finalize": (_vp,),
    "et_model_f32_forward": (_vp, _vp, _vp, _vp),
    "et_model_f32_sync": (_vp,),
    "et_model_f32_destroy": (_vp,),
    "et_fmt_permutation": (C.c_int64, C.c_uint64, _vp),
    "et_fmt_kept_count": (C.c_int64, _f),
    "et_fmt_tile_pattern": (_i, _i, _f, C.c_uint64, _vp, _vp, C.POINTER(_i)),
    "et_fmt_dense_to_bsr16": (_vp, _i, _i, _vp, _vp, _vp, C.POINTER(_i)),
    "et_fmt_row_ids": (_i, _f, C.c_uint64, _vp, C.POINTER(_i)),
    "et_fmt_col_ids": (_i, _f, C.c_uint64, _vp, C.POINTER(_i)),
    "et_fmt_head_ptr": (_vp, _i, _i, _i, _vp),
    "et_fmt_dense_to_1x16": (_vp, _i, _i, _vp, _vp, _vp, C.POINTER(_i)),
    "et_fmt_1x16_pattern": (_i, _i, _f, C.c_uint64, _vp, _vp, C.POINTER(_i)),
    "et_fmt_dense_to_csr": (_vp, _i, _i, _vp, _vp, _vp, C.POINTER(_i)),
    "et_fmt_csr_pattern": (_i, _i, _f, C.c_uint64, _vp, _vp, C.POINTER(_i)),
    "et_fmt_csr_read": (C.c_char_p, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i), _vp, _vp, _vp),
}

W_QKV, W_O, W_FF1, W_FF2 = 0, 1, 2, 3


class ModelDesc(C.Structure):
    _fields_ = [("kdim", _i), ("vdim", _i), ("seq_len", _i), ("nhead", _i), ("dimFF", _i), ("emdim", _i),
                ("nlayer", _i), ("batch", _i), ("act", _i), ("eps", _f), ("causal", _i), ("use_graph", _i), ("mixed", _i)]


class ChainDesc(C.Structure):
    """et_chain_desc of include/et_abi.h"""
    _fields_ = [("o", _vp), ("bias_o", _vp), ("Z", _vp), ("resid", _vp), ("resid16", _vp), ("resid_fin", _vp),
                ("resid_gamma", _vp), ("resid_beta", _vp), ("V1", _vp), ("stats1", _vp),
                ("up", _vp), ("bias_up", _vp), ("gamma1", _vp), ("beta1", _vp), ("eps1", _f), ("fin1", _vp), ("H", _vp),
                ("act", _i),
                ("down", _vp), ("bias_down", _vp), ("V2", _vp), ("stats2", _vp),
                ("qkv", _vp), ("bias_qkv", _vp), ("gamma2", _vp), ("beta2", _vp), ("eps2", _f), ("fin2", _vp), ("QKV", _vp),
                ("T", _i), ("sync", _vp)]


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


def mha_fuseo(Q, K, V, ldq, ldk, ldv, Z, ldz, mask, lens, B, S, nh, hd, scale, flags, o_row_ptr, o_col_idx,
              o_tiles, o_bias, out, emdim, waves=None, stream=None):
    """Fused attention and the tile-sparse output projection in one launch (waves: the tuning form)."""
    head = (_ptr(Q), _ptr(K), _ptr(V), ldq, ldk, ldv, _ptr(Z), ldz, _ptr(mask), _ptr(lens), B, S, nh, hd, scale,
            flags, _ptr(o_row_ptr), _ptr(o_col_idx), _ptr(o_tiles), _ptr(o_bias), _ptr(out), emdim)
    if waves is None:
        check(lib().et_mha_fuseo_f16(*head, stream))
    else:
        check(lib().et_mha_fuseo_f16_geom(*head, waves, stream))


def skip_layernorm(out, src, skip, gamma, beta, rows, H, eps=1e-5, stream=None):
    check(lib().et_skip_layernorm_f16(_ptr(out), _ptr(src), _ptr(skip), _ptr(gamma), _ptr(beta),
                                      rows, H, eps, stream))


def layernorm(out, src, gamma, beta, rows, H, eps=1e-5, stream=None):
    check(lib().et_layernorm_f16(_ptr(out), _ptr(src), _ptr(gamma), _ptr(beta), rows, H, eps, stream))


# ---------------------------------------------------------------------------
# Encoder stack handle (et_model_*)
# ---------------------------------------------------------------------------

def _np_ptr(a):
    return None if a is None else a.ctypes.data


class Model:
    """Encoder stack assembled from host weights; forward replays one HIP graph."""

    def __init__(self, H, nh, dimFF, S, nlayer, batch=1, act=ACT_GELU, eps=1e-5, causal=False, use_graph=True,
                 handle=None, mixed=False):
        self.desc = ModelDesc(H, H, S, nh, dimFF, H, nlayer, batch, act, eps, int(causal), int(use_graph),
                              int(mixed))
        self.rows, self.H = batch * S, H
        if handle is None:
            h = _vp()
            check(lib().et_model_create(C.byref(self.desc), C.byref(h)))
            handle = h.value
        self.handle = handle

    @classmethod
    def load(cls, weights_txt, directory, H, nh, dimFF, S, nlayer, **kw):
        self = cls.__new__(cls)
        Model.__init__(self, H, nh, dimFF, S, nlayer, handle=0, **kw)
        h = _vp()
        check(lib().et_model_load(str(weights_txt).encode(), str(directory).encode(), C.byref(self.desc),
                                  C.byref(h)))
        self.handle = h.value
        return self

    def set_bsr16(self, layer, which, row_ptr, column, data, bias):
        row_ptr = np.ascontiguousarray(row_ptr, np.int32)
        column = np.ascontiguousarray(column, np.int32)
        data = np.ascontiguousarray(data)
        bias = None if bias is None else np.ascontiguousarray(bias, data.dtype)
        fn = lib().et_model_set_bsr16_f16 if data.dtype == np.float16 else lib().et_model_set_bsr16
        assert data.dtype in (np.float16, np.float32)
        # the library reads out/16+1 row pointers, len(column) tiles of 256 values and out biases
        d = self.desc
        n_out = {W_QKV: 2 * d.kdim + d.vdim, W_O: d.emdim, W_FF1: d.dimFF, W_FF2: d.emdim}.get(which)
        if n_out is not None:
            if row_ptr.size != n_out // 16 + 1 or data.size != column.size * 256 or (
                    bias is not None and bias.size != n_out):
                raise ValueError(f"set_bsr16: row_ptr[{row_ptr.size}], column[{column.size}], data[{data.size}] or "
                                 f"bias do not fit a matrix of {n_out} output features")
        check(fn(self.handle, layer, which, _np_ptr(row_ptr), _np_ptr(column), _np_ptr(data), len(column),
                 _np_ptr(bias)))

    def set_dense(self, layer, which, W, bias):
        W = np.ascontiguousarray(W)
        bias = None if bias is None else np.ascontiguousarray(bias, W.dtype)
        fn = lib().et_model_set_dense_f16 if W.dtype == np.float16 else lib().et_model_set_dense
        check(fn(self.handle, layer, which, _np_ptr(W), _np_ptr(bias)))

    def set_norm(self, layer, which, gamma, beta):
        gamma = np.ascontiguousarray(gamma)
        beta = np.ascontiguousarray(beta, gamma.dtype)
        fn = lib().et_model_set_norm_f16 if gamma.dtype == np.float16 else lib().et_model_set_norm
        check(fn(self.handle, layer, which, _np_ptr(gamma), _np_ptr(beta)))

    def launches_per_layer(self) -> int:
        n = _i()
        check(lib().et_model_launches_per_layer(self.handle, C.byref(n)))
        return n.value

    def set_lens(self, lens):
        lens = None if lens is None else np.ascontiguousarray(lens, np.int32)
        check(lib().et_model_set_lens(self.handle, _np_ptr(lens)))

    def set_mask(self, mask):
        mask = None if mask is None else np.ascontiguousarray(mask, np.float16)
        check(lib().et_model_set_mask(self.handle, _np_ptr(mask)))

    def finalize(self):
        check(lib().et_model_finalize(self.handle))

    def forward(self, out, inp, stream=None):
        check(lib().et_model_forward(self.handle, _ptr(out), _ptr(inp), stream))

    def forward_layer(self, layer, out, inp, stream=None):
        check(lib().et_model_forward_layer(self.handle, layer, _ptr(out), _ptr(inp), stream))

    def sync(self):
        check(lib().et_model_sync(self.handle))

    def destroy(self):
        if self.handle:
            lib().et_model_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
