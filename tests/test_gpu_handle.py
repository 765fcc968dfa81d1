"""Handle entry points around host memory (enable / disable_access_to_host_mem).

The reference pins memory that already exists (cuda_dataflow_handle.c:604-620); this backend never registers
existing pages: memory from dataflow_amd_alloc_host_mem is accepted as already visible, anything else is refused
with -1, and the refusal leaves no error behind for the next call."""
import ctypes as C

import numpy as np
import pytest

from ml_dataflow_amd import binding as B

pytestmark = pytest.mark.gpu


def test_enable_access_refuses_plain_host_memory_and_accepts_its_own(backend, capfd):
    be = backend
    plain = np.zeros(1 << 16, dtype=np.uint8)
    assert be.h.enable_access_to_host_mem(be.hp, plain.ctypes.data, plain.nbytes, 0) == -1
    assert "dataflow_amd_alloc_host_mem" in capfd.readouterr().err
    assert be.h.disable_access_to_host_mem(be.hp, plain.ctypes.data) == -1
    assert be.h.enable_access_to_host_mem(be.hp, None, 16, 0) == -1
    # no error is left behind: an unrelated device call right after works and round-trips data
    data = np.arange(4096, dtype=np.int32)
    buf = be.upload(data)
    assert (be.read(buf.ptr, data.shape, np.int32) == data).all()
    buf.free()
    own = be.host_alloc(1 << 16)
    assert be.h.enable_access_to_host_mem(be.hp, own, 1 << 16, 0) == 0
    assert be.h.enable_access_to_host_mem(be.hp, own + 4096, 4096, 0) == 0          # an interior range of it
    assert be.h.enable_access_to_host_mem(be.hp, own, 1 << 30, 0) == -1             # a range that runs far past its end
    assert be.h.enable_access_to_host_mem(be.hp, own + 4096, 1 << 16, 0) == -1      # and one that ends just behind it
    capfd.readouterr()
    assert be.h.disable_access_to_host_mem(be.hp, own) == 0
    # still usable by the device afterwards: select_experts writes the per-expert counts through it
    T, E, K = 64, 8, 2
    logits = be.upload(np.zeros((T, E), dtype=np.uint16))
    w, ch = be.alloc(T * K * 4), be.alloc(T * K * 2)
    counts, cum = be.alloc((E + 1) * 4), be.alloc(E * 4)
    be.zero(counts.ptr, (E + 1) * 4, 1)
    be.zero(cum.ptr, E * 4, 1)
    assert be.lib.dataflow_submit_default_select_experts(be.hp, 1, B.DATAFLOW_BF16, T, E, K, logits.ptr, w.ptr, ch.ptr, counts.ptr, cum.ptr, own) == 0
    be.sync()
    host_counts = np.ctypeslib.as_array(C.cast(own, C.POINTER(C.c_int32)), (E,)).copy()
    assert host_counts.tolist() == [T, T] + [0] * (E - 2)         # all-equal logits: every token takes experts 0 and 1
    be.host_free(own)


def test_profiler_hooks_accept_names_and_ranges(backend):
    """name_device / name_handle / name_stream / name_thread forward to the marker library's naming calls where it has them
    (cuda_profiler.c:49-70 forwards to NVTX) and are harmless otherwise; ranges nest; a bad stream id is reported, not used"""
    be = backend
    be.h.profiler_name_device(be.hp, b"gfx950 device 0")
    be.h.profiler_name_handle(be.hp, b"moe backend")
    be.h.profiler_name_stream(be.hp, 1, b"Compute")
    be.h.profiler_name_stream(be.hp, 99, b"no such stream")
    be.h.profiler_name_thread(be.hp, b"test thread")
    be.h.profiler_range_push(b"outer")
    be.h.profiler_range_push(b"inner")
    be.h.profiler_range_pop()
    be.h.profiler_range_pop()
    data = np.arange(1024, dtype=np.int32)                        # the handle works as before afterwards
    buf = be.upload(data)
    assert (be.read(buf.ptr, data.shape, np.int32) == data).all()
    buf.free()
