"""amd_matmul_no_alloc: the matmul with the partial sums of its split along K in the library's own static device
scratch, for callers that cannot allocate.  Called through the C ABI; its output must equal, bit for bit, that of the
existing entry point (the matmul op with a caller's workspace: same kernels, same split) on two calls in a row, the
second with a smaller input; a split that the scratch cannot hold is refused."""
import ctypes as C
import os

import numpy as np
import pytest

from ml_dataflow_amd import binding as B
from util import normal_bf16

pytestmark = pytest.mark.gpu

BF = B.DATAFLOW_BF16
SCRATCH_BYTES = 8 << 20


def entry_point():
    lib = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul.so"))
    fn = lib.amd_matmul_no_alloc
    fn.restype = C.c_int
    fn.argtypes = [C.POINTER(B.DataflowHandle), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float,
                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    return fn


def run_both(be, fn, transa, transb, M, K, N, beta, seed):
    rng = np.random.default_rng(seed)
    A, Bm, Cin = normal_bf16(rng, (M * K,), 0.05), normal_bf16(rng, (N * K,)), normal_bf16(rng, (N * M,))
    d_A, d_B = be.upload(A), be.upload(Bm)
    d_D1, d_D2, d_ws = be.upload(Cin), be.upload(Cin), be.alloc(SCRATCH_BYTES)
    c_dt = BF if beta else B.DATAFLOW_NONE
    assert be.lib.dataflow_submit_matmul(be.hp, 1, BF, BF, c_dt, BF, B.DATAFLOW_FP32, transa, transb, M, K, N, 1.0, beta,
                                         d_A.ptr, d_B.ptr, d_D1.ptr if beta else None, d_D1.ptr, SCRATCH_BYTES, d_ws.ptr) == 0
    assert fn(be.hp, 1, transa, transb, M, K, N, 1.0, beta, d_A.ptr, d_B.ptr, d_D2.ptr if beta else None, d_D2.ptr) == 0
    be.sync(1)
    want, got = be.read(d_D1.ptr, (N, M), np.uint16), be.read(d_D2.ptr, (N, M), np.uint16)
    for buf in (d_A, d_B, d_D1, d_D2, d_ws):
        buf.free()
    return got, want


def test_no_alloc_matmul_equals_the_workspace_matmul(backend, capfd):
    be, fn = backend, entry_point()
    # the router's products (few tiles, long K: split along K through the scratch), large first, then smaller
    for transa, transb, M, K, N, beta in ((1, 0, 64, 4096, 8192, 0.0), (1, 0, 64, 2048, 1000, 0.0),
                                          (0, 1, 4096, 8192, 64, 1.0), (0, 1, 512, 1000, 24, 1.0),
                                          (1, 0, 2048, 512, 2048, 0.0)):          # the last one does not split: no scratch use
        print("case no-alloc matmul ta=%d tb=%d M=%d K=%d N=%d" % (transa, transb, M, K, N), flush=True)
        got, want = run_both(be, fn, transa, transb, M, K, N, beta, seed=M + K + N)
        assert (got == want).all()
    # a split whose partial sums exceed the scratch is refused, with a message, and launches nothing
    M, K, N = 128, 65536, 16384
    d_A, d_B, d_D = be.alloc(M * K * 2), be.alloc(N * K * 2), be.alloc(N * M * 2)
    capfd.readouterr()
    assert fn(be.hp, 1, 1, 0, M, K, N, 1.0, 0.0, d_A.ptr, d_B.ptr, None, d_D.ptr) == -1
    assert "scratch" in capfd.readouterr().err
    for buf in (d_A, d_B, d_D):
        buf.free()
