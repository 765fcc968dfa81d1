"""The four-wave persistent GEMM kernels (one loading and three multiplying waves on the 256 x 288 tile; four waves that
all load and multiply on a 256 x 384 tile) against the eight-wave one: bit for bit, on the shapes they can take.

All kernels keep the LDS tile layouts, the fragment reads and the order of accumulation over k, so every element must
come out identical; the eight-wave kernel itself is held to the oracle in test_gpu_ops.py, and one case here is too.
"""
import ctypes as C
import os

import numpy as np
import pytest

import oracle_lib as O
from ml_dataflow_amd import binding as B
from util import normal_bf16

pytestmark = pytest.mark.gpu

BF = B.DATAFLOW_BF16
CS = 1
AUTO, EIGHT, FOUR, FOUR_384 = 0, 8, 4, 384
OTHERS = [FOUR, FOUR_384, AUTO]          # AUTO: both tilings are launched and the work-groups pick one from the group sizes


@pytest.fixture(scope="module")
def select_kernel(backend):
    lib = C.CDLL(os.path.join(os.path.dirname(B.__file__), "lib", "libamd_matmul.so"))
    lib.amd_matmul_select_kernel.argtypes = [C.c_int]
    yield lib.amd_matmul_select_kernel
    assert lib.amd_matmul_select_kernel(AUTO) == 0


def matmul(be, transa, M, K, N, d_A, d_B, d_D, alpha=1.0):
    assert be.lib.dataflow_submit_matmul(be.hp, CS, BF, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, transa, 0, M, K, N, alpha, 0.0,
                                         d_A.ptr, d_B.ptr, None, d_D.ptr, 0, None) == 0
    be.sync(CS)
    return be.read(d_D.ptr, (N, M), np.uint16)


@pytest.mark.parametrize("other", OTHERS)
@pytest.mark.parametrize("transa", [1, 0])
@pytest.mark.parametrize("M,K,N", [(1024, 128, 8192), (1024, 256, 8192), (512, 1024, 16384), (2048, 4096, 4096), (1000, 384, 8200)])
def test_single_problem_bit_identical(backend, oracle, select_kernel, other, transa, M, K, N):
    print("case w4 single kernel=%d ta=%d M=%d K=%d N=%d" % (other, transa, M, K, N), flush=True)
    be = backend
    rng = np.random.default_rng(M + K + N + transa)
    A = normal_bf16(rng, (M, K) if transa else (K, M), 0.05)
    X = normal_bf16(rng, (N, K))
    d_A, d_B = be.upload(A), be.upload(X)
    d_D8, d_D4 = be.alloc(N * M * 2), be.alloc(N * M * 2)
    be.zero(d_D4.ptr, N * M * 2, CS)
    assert select_kernel(EIGHT) == 0
    alpha = 1.0 if K != 256 else 0.375                      # one shape also with a scale: the epilogues leave the multiply out when alpha is 1
    got8 = matmul(be, transa, M, K, N, d_A, d_B, d_D8, alpha)
    assert select_kernel(other) == 0
    got4 = matmul(be, transa, M, K, N, d_A, d_B, d_D4, alpha)
    assert select_kernel(AUTO) == 0
    bad = got4 != got8
    assert not bad.any(), "%d of %d elements differ, first at %s" % (int(bad.sum()), bad.size, np.argwhere(bad)[:4].tolist())
    if K <= 256:
        want = O.matmul(oracle, transa, 0, M, K, 64, A, np.ascontiguousarray(X[:64]), alpha, 0.0, None)
        g, w = got4[:64].astype(np.uint32) << 16, want.astype(np.uint32) << 16
        diff = np.abs(g.view(np.float32).astype(np.float64) - w.view(np.float32).astype(np.float64))
        assert diff.max() <= 1e-2 * np.abs(w.view(np.float32)).max()
    for d in (d_A, d_B, d_D8, d_D4):
        d.free()


def grouped(be, transa, M, K, total, G, d_cum, d_W, d_X, d_D, gather=None, src_rows=0):
    if gather is None:
        ret = be.lib.dataflow_submit_amd_grouped_matmul(be.hp, CS, BF, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, transa, 0, B.AMD_GROUPED_RAGGED_N,
                                                        M, K, total, G, d_cum.ptr, 1.0, 0.0, d_W.ptr, M * K * 2, d_X.ptr, None, d_D.ptr, 0)
    else:
        ret = be.lib.dataflow_submit_amd_grouped_matmul_gathered(be.hp, CS, BF, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, transa, 0,
                                                                 B.AMD_GROUPED_RAGGED_N, M, K, total, G, d_cum.ptr, 1.0, 0.0, d_W.ptr, M * K * 2,
                                                                 d_X.ptr, None, d_D.ptr, 0, gather.ptr, src_rows)
    assert ret == 0
    be.sync(CS)
    return be.read(d_D.ptr, (total, M), np.uint16)


EDGE_COUNTS = [288, 289, 1, 0, 575, 576, 577, 287, 256, 257, 255, 0, 1152, 1153, 1151, 1024, 1025, 2, 300, 31, 383, 384, 385, 767, 768, 769]


@pytest.mark.parametrize("other", OTHERS)
@pytest.mark.parametrize("transa", [1, 0])
@pytest.mark.parametrize("M,K,counts", [(2048, 128, EDGE_COUNTS), (1024, 512, [1024] * 16), (1024, 1024, [1000, 1100, 1024, 990] * 8),
                                        (1000, 256, [700, 90, 1200, 385] * 12)])      # the last m-tile of every group is partial
def test_ragged_n_bit_identical(backend, select_kernel, other, transa, M, K, counts):
    be = backend
    counts = np.array(counts, dtype=np.int32)
    G, total = len(counts), int(counts.sum())
    print("case w4 grouped-N kernel=%d ta=%d G=%d M=%d K=%d rows=%d" % (other, transa, G, M, K, total), flush=True)
    rng = np.random.default_rng(5 + transa + M + K)
    incl = np.cumsum(counts).astype(np.int32)
    W = normal_bf16(rng, (G, M, K) if transa else (G, K, M), 0.05)
    X = normal_bf16(rng, (total, K))
    d_W, d_X, d_cum = be.upload(W), be.upload(X), be.upload(incl)
    d_D8, d_D4 = be.alloc(total * M * 2), be.alloc(total * M * 2)
    be.zero(d_D4.ptr, total * M * 2, CS)
    assert select_kernel(EIGHT) == 0
    got8 = grouped(be, transa, M, K, total, G, d_cum, d_W, d_X, d_D8)
    assert select_kernel(other) == 0
    got4 = grouped(be, transa, M, K, total, G, d_cum, d_W, d_X, d_D4)
    assert select_kernel(AUTO) == 0
    bad = got4 != got8
    assert not bad.any(), "%d of %d elements differ, first at %s" % (int(bad.sum()), bad.size, np.argwhere(bad)[:4].tolist())
    for d in (d_W, d_X, d_cum, d_D8, d_D4):
        d.free()


@pytest.mark.parametrize("other", OTHERS)
@pytest.mark.parametrize("transa", [1, 0])
@pytest.mark.parametrize("G,M,K,total,src_rows", [(64, 1024, 256, 40000, 5000), (16, 512, 4096, 9000, 2048), (len(EDGE_COUNTS), 2048, 128, sum(EDGE_COUNTS), 700)])
def test_gathered_ragged_n_bit_identical(backend, select_kernel, other, transa, G, M, K, total, src_rows):
    print("case w4 gathered kernel=%d ta=%d G=%d M=%d K=%d rows=%d src=%d" % (other, transa, G, M, K, total, src_rows), flush=True)
    be = backend
    rng = np.random.default_rng(G + M + K + total + transa)
    if G == len(EDGE_COUNTS):
        counts = np.array(EDGE_COUNTS, dtype=np.int32)
    else:
        cuts = np.sort(rng.integers(0, total + 1, size=G - 1))
        counts = np.diff(np.concatenate([[0], cuts, [total]])).astype(np.int32)
    incl = np.cumsum(counts).astype(np.int32)
    W = normal_bf16(rng, (G, M, K) if transa else (G, K, M), 0.05)
    S = normal_bf16(rng, (src_rows, K))
    rowmap = rng.integers(0, src_rows, size=total).astype(np.int32)
    d_W, d_S, d_cum, d_map = be.upload(W), be.upload(S), be.upload(incl), be.upload(rowmap)
    d_D8, d_D4 = be.alloc(total * M * 2), be.alloc(total * M * 2)
    be.zero(d_D4.ptr, total * M * 2, CS)
    assert select_kernel(EIGHT) == 0
    got8 = grouped(be, transa, M, K, total, G, d_cum, d_W, d_S, d_D8, d_map, src_rows)
    assert select_kernel(other) == 0
    got4 = grouped(be, transa, M, K, total, G, d_cum, d_W, d_S, d_D4, d_map, src_rows)
    assert select_kernel(AUTO) == 0
    bad = got4 != got8
    assert not bad.any(), "%d of %d elements differ, first at %s" % (int(bad.sum()), bad.size, np.argwhere(bad)[:4].tolist())
    for d in (d_W, d_S, d_cum, d_map, d_D8, d_D4):
        d.free()
