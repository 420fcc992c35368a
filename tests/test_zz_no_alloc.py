"""The allocation-free column-pruned Linear (et_linear_colpruned_static_f16: gathered
activations in a device array built into the library) against the workspace form it is a
variant of (et_linear_colpruned_ws_f16), bit for bit, on two calls in a row — the second on a
smaller problem, so that it runs on a buffer that still holds the first call's data."""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import layers as L
from tests import harness as Hn
from tests.harness import up

pytestmark = pytest.mark.gpu

ACT = {0: "none", 1: "relu", 2: "gelu"}


def run_both(et, T, inp, out, sp, act, seed):
    col_id = F.gen_col_ids(inp, sp, seed=seed)
    nnz = len(col_id)
    cols, b, x = Hn.randn((out, nnz), seed + 1, 0.02), Hn.randn((out,), seed + 2, 0.1), Hn.randn((T, inp), seed + 3)
    d_cols, d_id, d_b, d_x = up(et, cols), up(et, col_id), up(et, b), up(et, x)
    d_ws = et.DeviceBuffer.empty((T, nnz), np.float16)
    d_ref = et.DeviceBuffer.empty((T, out), np.float16)
    d_got = et.DeviceBuffer.empty((T, out), np.float16)
    et.check(et.lib().et_fill_f16(d_got.ptr, T * out, 0x7E00, None))
    et.check(et.lib().et_linear_colpruned_ws_f16(d_cols.ptr, d_id.ptr, nnz, d_b.ptr, d_x.ptr, d_ref.ptr, d_ws.ptr,
                                                 T, inp, out, act, None))
    et.check(et.lib().et_linear_colpruned_static_f16(d_cols.ptr, d_id.ptr, nnz, d_b.ptr, d_x.ptr, d_got.ptr,
                                                     T, inp, out, act, None))
    ref, got = d_ref.numpy(), d_got.numpy()
    want = L.linear_colpruned(Hn.f32(x), Hn.f32(cols), col_id, Hn.f32(b), ACT[act], torch.float16).numpy()
    return ref, got, want


def test_static_scratch_linear_equals_workspace_form_twice(et):
    # first call: 2048 x 1536 kept columns = 6 MiB of the 8 MiB buffer
    ref, got, want = run_both(et, 2048, 3072, 768, 0.5, 2, seed=70)
    assert np.array_equal(ref, got)
    assert Hn.max_abs(got, want) <= 4e-3
    # second call, smaller: runs on a buffer that still holds the first call's gather
    ref, got, want = run_both(et, 64, 768, 3072, 0.75, 0, seed=80)
    assert np.array_equal(ref, got)
    assert Hn.max_abs(got, want) <= 4e-3
    # and a third, larger again, different kept-column count
    ref, got, want = run_both(et, 512, 1024, 256, 0.25, 1, seed=90)
    assert np.array_equal(ref, got)
    assert Hn.max_abs(got, want) <= 4e-3


def test_static_scratch_linear_allocates_nothing(et):
    """Recorded into a HIP graph (stream capture refuses any allocation, and an allocating call would fail the
    capture) and replayed three times with other work between the replays: every replay gives the eager result;
    and the device's free memory is the same before and after eager calls."""
    import ctypes as C
    lib = et.lib()
    T, inp, out, act = 256, 768, 384, 1
    col_id = F.gen_col_ids(inp, 0.5, seed=95)
    nnz = len(col_id)
    d_cols, d_id, d_b = up(et, Hn.randn((out, nnz), 96, 0.02)), up(et, col_id), up(et, Hn.randn((out,), 97, 0.1))
    d_x = up(et, Hn.randn((T, inp), 98))
    d_eager, d_graph = et.DeviceBuffer.empty((T, out), np.float16), et.DeviceBuffer.empty((T, out), np.float16)
    stream = C.c_void_p()
    et.check(lib.et_stream_create(C.byref(stream)))
    args = (d_cols.ptr, d_id.ptr, nnz, d_b.ptr, d_x.ptr)
    hip = C.CDLL("libamdhip64.so")
    free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
    et.check(lib.et_linear_colpruned_static_f16(*args, d_eager.ptr, T, inp, out, act, stream))  # first use: address lookup
    et.check(lib.et_stream_sync(stream))
    assert hip.hipMemGetInfo(C.byref(free0), C.byref(total)) == 0
    for _ in range(3):
        et.check(lib.et_linear_colpruned_static_f16(*args, d_eager.ptr, T, inp, out, act, stream))
    et.check(lib.et_stream_sync(stream))
    assert hip.hipMemGetInfo(C.byref(free1), C.byref(total)) == 0
    assert free1.value == free0.value
    want = d_eager.numpy()
    et.check(lib.et_graph_begin_capture(stream))
    et.check(lib.et_linear_colpruned_static_f16(*args, d_graph.ptr, T, inp, out, act, stream))
    graph = C.c_void_p()
    et.check(lib.et_graph_end_capture(stream, C.byref(graph)))
    for rep in range(3):
        et.check(lib.et_fill_f16(d_graph.ptr, T * out, 0x7E00, stream))  # the program's own work between replays
        et.check(lib.et_graph_launch(graph, stream))
        et.check(lib.et_stream_sync(stream))
        assert np.array_equal(d_graph.numpy(), want), f"replay {rep}"
    et.check(lib.et_graph_destroy(graph))
    et.check(lib.et_stream_destroy(stream))


def test_static_scratch_linear_rejects_what_does_not_fit(et):
    d = et.DeviceBuffer.empty((16,), np.float16)
    # 4096 x 2048 x 2 bytes = 16 MiB > 8 MiB: refused before anything is launched
    st = et.lib().et_linear_colpruned_static_f16(d.ptr, d.ptr, 2048, None, d.ptr, d.ptr, 4096, 4096, 768, 0, None)
    assert st == et.ET_ERR_UNSUPPORTED
    assert b"8388608" in et.lib().et_last_error()
    # empty problems are fine and touch nothing
    et.check(et.lib().et_linear_colpruned_static_f16(d.ptr, d.ptr, 16, None, d.ptr, d.ptr, 0, 32, 16, 0, None))
