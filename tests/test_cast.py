"""The two cast ops beside the optimizer step (cast.cu:11-47, 61-113): the oracle pinned against numpy, the HIP
kernels against the oracle through the C ABI.  Every step of both ops is an exactly defined rounding, so the bar is
bit-exact."""
import numpy as np
import pytest

import oracle_lib as O
from util import f32_to_bf16, bf16_to_f32, bf16_to_f64, normal_bf16


def numpy_cast_and_add(alpha, A, beta, Bb):
    """the three roundings with numpy's arithmetic in fp64 (every product and sum below is exact in fp64)"""
    a64 = np.float64(np.float32(alpha)) * A.astype(np.float64)
    t1 = bf16_to_f64(f32_to_bf16(a64.astype(np.float32)))                    # fp32 product first, as the kernel's alpha * A[i]
    beta_b = bf16_to_f64(f32_to_bf16(np.array([beta], np.float32)))[0]
    t2 = bf16_to_f64(f32_to_bf16((beta_b * bf16_to_f64(Bb)).astype(np.float32)))
    return f32_to_bf16((t1 + t2).astype(np.float32))


def make(rng, n):
    A = (rng.standard_normal(n) * 0.01).astype(np.float32)
    Bb = normal_bf16(rng, (n,), 0.5)
    return A, Bb


@pytest.mark.parametrize("n", [1, 7, 1000, 65537])
def test_oracle_cast_is_exact(oracle, n):
    src = normal_bf16(np.random.default_rng(n), (n,), 3.0)
    dst = np.zeros(n, np.float32)
    oracle.oracle_cast_bf16_fp32(n, O.ptr(src), O.ptr(dst))
    assert (dst.view(np.uint32) == (src.astype(np.uint32) << 16)).all()


@pytest.mark.parametrize("n,alpha,beta", [(1, 1.0, 1.0), (1000, 0.25, 1.0), (4099, 1.0 / 3.0, 0.9), (65536, -2.5, 0.3)])
def test_oracle_cast_and_add_is_the_three_roundings(oracle, n, alpha, beta):
    A, Bb = make(np.random.default_rng(n), n)
    got = np.zeros(n, np.uint16)
    oracle.oracle_cast_and_add(n, alpha, O.ptr(A), beta, O.ptr(Bb), O.ptr(got))
    assert (got == numpy_cast_and_add(alpha, A, beta, Bb)).all()


def test_oracle_cast_and_add_special_cases(oracle):
    n = 512
    A, Bb = make(np.random.default_rng(5), n)
    out = np.zeros(n, np.uint16)
    oracle.oracle_cast_and_add(n, 0.0, O.ptr(A), 1.0, O.ptr(Bb), O.ptr(out))          # alpha = 0, beta = 1: B unchanged
    assert (bf16_to_f32(out) == bf16_to_f32(Bb)).all()
    oracle.oracle_cast_and_add(n, 1.0, O.ptr(A), 0.0, O.ptr(Bb), O.ptr(out))          # beta = 0: the rounded cast of A
    assert (bf16_to_f32(out) == bf16_to_f32(f32_to_bf16(A))).all()
    acc = Bb.copy()                                                                   # in place, C aliases B
    oracle.oracle_cast_and_add(n, 1.0, O.ptr(A), 1.0, O.ptr(acc), O.ptr(acc))
    assert (acc == numpy_cast_and_add(1.0, A, 1.0, Bb)).all()


CASES = [(8, 0), (2048, 0), (100003, 0), (1 << 22, 0), (5000, 1), (0, 0)]


@pytest.mark.gpu
@pytest.mark.parametrize("n,offset", CASES)
def test_gpu_cast_matches_oracle(backend, oracle, n, offset):
    """offset 1: arrays that start one element off a 16-byte boundary take the element-wise path"""
    from ml_dataflow_amd import binding as B
    print("case cast n=%d offset=%d" % (n, offset), flush=True)
    be = backend
    BF, F32 = B.DATAFLOW_BF16, B.DATAFLOW_FP32
    src = normal_bf16(np.random.default_rng(n + 1), (n + offset + 1,), 0.5)
    d_src, d_dst = be.upload(src), be.alloc((n + offset + 1) * 4)
    be.zero(d_dst.ptr, (n + offset + 1) * 4)
    assert be.lib.dataflow_submit_cast(be.hp, 1, BF, F32, n, d_src.ptr + 2 * offset, d_dst.ptr + 4 * offset) == 0
    be.sync(1)
    want, part = np.zeros(n, np.float32), src[offset:offset + n].copy()
    oracle.oracle_cast_bf16_fp32(n, O.ptr(part), O.ptr(want))
    assert (be.read(d_dst.ptr + 4 * offset, (n,), np.uint32) == want.view(np.uint32)).all()
    assert be.read(d_dst.ptr + 4 * (offset + n), (1,), np.uint32)[0] == 0             # nothing written past the end
    # only the registered type combination exists
    assert be.lib.dataflow_submit_cast(be.hp, 1, F32, BF, n, d_src.ptr, d_dst.ptr) == -1
    d_src.free(), d_dst.free()


@pytest.mark.gpu
@pytest.mark.parametrize("n,offset", CASES)
def test_gpu_cast_and_add_matches_oracle(backend, oracle, n, offset):
    """an fp32 array folded into a bf16 accumulator, out of place and in place (C aliases B)"""
    from ml_dataflow_amd import binding as B
    print("case cast_and_add n=%d offset=%d" % (n, offset), flush=True)
    be = backend
    BF, F32 = B.DATAFLOW_BF16, B.DATAFLOW_FP32
    A, Bb = make(np.random.default_rng(n + 2), n + offset + 1)
    a, b = A[offset:offset + n].copy(), Bb[offset:offset + n].copy()
    d_A, d_B, d_C = be.upload(A), be.upload(Bb), be.alloc((n + offset + 1) * 2)
    be.zero(d_C.ptr, (n + offset + 1) * 2)
    for alpha, beta in ((1.0, 1.0), (0.37, 0.9)):
        want = np.zeros(n, np.uint16)
        oracle.oracle_cast_and_add(n, alpha, O.ptr(a), beta, O.ptr(b), O.ptr(want))
        assert be.lib.dataflow_submit_cast_and_add(be.hp, 1, F32, BF, BF, n, alpha, d_A.ptr + 4 * offset, beta, d_B.ptr + 2 * offset,
                                                   d_C.ptr + 2 * offset) == 0
        be.sync(1)
        assert (be.read(d_C.ptr + 2 * offset, (n,), np.uint16) == want).all()
    assert be.read(d_C.ptr + 2 * (offset + n), (1,), np.uint16)[0] == 0
    want = np.zeros(n, np.uint16)
    oracle.oracle_cast_and_add(n, 1.0, O.ptr(a), 1.0, O.ptr(b), O.ptr(want))
    assert be.lib.dataflow_submit_cast_and_add(be.hp, 1, F32, BF, BF, n, 1.0, d_A.ptr + 4 * offset, 1.0, d_B.ptr + 2 * offset,
                                               d_B.ptr + 2 * offset) == 0
    be.sync(1)
    assert (be.read(d_B.ptr + 2 * offset, (n,), np.uint16) == want).all()
    assert be.read(d_B.ptr + 2 * (offset + n), (1,), np.uint16)[0] == Bb[offset + n]
    for buf in (d_A, d_B, d_C):
        buf.free()
