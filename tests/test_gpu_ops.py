"""GPU parity of every MoE operator against the CPU oracle, called through the C ABI
(dataflow_submit_* -> handle->submit_op -> gfx950 kernel).

Bar: integer / index / copy results bit-exact; bf16 values within a stated number of bf16 ulps
(2^-7 relative) of the oracle's fp64- or fp32-accumulated result, at most 1e-2 relative overall.
"""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as O
from ml_dataflow_amd import binding as B
from util import f32_to_bf16, bf16_to_f32, bf16_to_f64, normal_bf16, bf16_ulp_diff

pytestmark = pytest.mark.gpu

BF = B.DATAFLOW_BF16
CS = 1          # compute stream


def routed_logits(rng, T, E, coarse):
    v = rng.standard_normal((T, E)).astype(np.float32)
    if coarse:
        v = np.round(v * 4) / 4       # many exact ties
    return f32_to_bf16(v)


def gpu_select(be, logits, K, dt=None):
    dt = BF if dt is None else dt
    T, E = logits.shape
    d_logits = be.upload(logits)
    d_w = be.alloc(T * K * 4)
    d_ch = be.alloc(T * K * 2)
    d_counts = be.alloc((E + 1) * 4)
    d_cum = be.alloc(E * 4)
    host = be.host_alloc(E * 4)
    be.zero(d_counts.ptr, (E + 1) * 4, CS)
    be.zero(d_cum.ptr, E * 4, CS)
    ret = be.lib.dataflow_submit_default_select_experts(be.hp, CS, dt, T, E, K, d_logits.ptr, d_w.ptr, d_ch.ptr, d_counts.ptr, d_cum.ptr, host)
    assert ret == 0
    be.sync(CS)
    out = (be.read(d_w.ptr, (T, K), np.float32), be.read(d_ch.ptr, (T, K), np.uint16), be.read(d_counts.ptr, (E + 1,), np.int32),
           be.read(d_cum.ptr, (E,), np.int32), np.ctypeslib.as_array(C.cast(host, C.POINTER(C.c_int32)), (E,)).copy())
    be.host_free(host)
    return out + (d_ch, d_cum)


@pytest.mark.parametrize("T,E,K,coarse", [
    (256, 8, 2, False), (256, 8, 2, True), (1000, 32, 4, True), (8192, 64, 8, False), (8192, 64, 8, True),
    (777, 7, 3, True), (64, 130, 6, True), (65, 256, 1, False), (33, 16, 5, True), (1, 4, 4, False), (4096, 32, 4, False),
    (200, 64, 12, True), (100, 48, 20, True), (64, 40, 32, True), (300, 2000, 9, False), (31, 32, 32, True), (500, 4096, 2, True)])
def test_select_experts_bit_exact(backend, oracle, T, E, K, coarse):
    print("case select T=%d E=%d K=%d coarse=%s" % (T, E, K, coarse), flush=True)
    rng = np.random.default_rng(T * 31 + E * 7 + K)
    logits = routed_logits(rng, T, E, coarse)
    w_o, ch_o, counts_o, cum_o, host_o = O.select_experts(oracle, logits, K)
    w_g, ch_g, counts_g, cum_g, host_g, _, _ = gpu_select(backend, logits, K)
    assert (ch_g == ch_o).all()
    assert (counts_g[:E] == counts_o[:E]).all()
    assert counts_g[E] == (T + 31) // 32          # the ticket ends equal to the number of work-groups (32 tokens each)
    assert (cum_g == cum_o).all()
    assert (host_g == counts_o[:E]).all()
    np.testing.assert_allclose(w_g, w_o, rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("T,E,K", [(256, 8, 2), (1000, 32, 4), (8192, 64, 8), (777, 7, 3), (5, 4, 4), (1, 3, 1), (65536, 64, 8), (3000, 300, 6),
                                   (8191, 64, 3),        # entry count not a multiple of 8: the last ids are counted one by one
                                   (65537, 64, 1),       # work-groups whose slice lies behind the last entry
                                   (8192, 128, 8), (33000, 1024, 2),     # 16 and 2 private counters per expert and wave
                                   (700, 2000, 3)])      # more experts than the private histograms hold: shared counters
def test_build_expert_mapping_bit_exact(backend, oracle, T, E, K):
    print("case build T=%d E=%d K=%d" % (T, E, K), flush=True)
    be = backend
    rng = np.random.default_rng(T + E + K)
    logits = routed_logits(rng, T, E, True)
    w_o, ch_o, counts_o, cum_o, _ = O.select_experts(oracle, logits, K)
    emap_o, tmap_o, cum_after_o = O.build_expert_mapping(oracle, ch_o, E, cum_o)
    d_ch, d_cum = be.upload(ch_o), be.upload(cum_o)
    d_emap, d_tmap = be.alloc(T * K * 4), be.alloc(T * K * 4)
    be.write(d_emap.ptr, np.full(T * K, -7, dtype=np.int32))
    be.write(d_tmap.ptr, np.full(T * K, -7, dtype=np.int32))
    assert be.lib.dataflow_submit_default_build_expert_mapping(be.hp, CS, T, E, K, d_ch.ptr, d_cum.ptr, d_emap.ptr, d_tmap.ptr) == 0
    be.sync(CS)
    assert (be.read(d_emap.ptr, (T * K,), np.int32) == emap_o).all()
    assert (be.read(d_tmap.ptr, (T, K), np.int32) == tmap_o).all()
    assert (be.read(d_cum.ptr, (E,), np.int32) == cum_after_o).all()       # inclusive post-state


def make_routing(rng, T, E, K):
    chosen = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint16)
    bc = np.bincount(chosen.ravel(), minlength=E).astype(np.int32)
    order = np.argsort(chosen.ravel(), kind="stable")
    tmap = np.empty(T * K, dtype=np.int32)
    tmap[order] = np.arange(T * K, dtype=np.int32)
    return chosen, bc, np.cumsum(bc).astype(np.int32), (order // K).astype(np.int32), tmap.reshape(T, K)


@pytest.mark.parametrize("T,D,E,K", [(256, 512, 8, 2), (100, 2048, 32, 4), (300, 4096, 64, 8), (17, 8, 4, 3), (64, 10000, 8, 2)])
def test_dispatch_bit_exact(backend, oracle, T, D, E, K):
    print("case dispatch T=%d D=%d E=%d K=%d" % (T, D, E, K), flush=True)
    be = backend
    rng = np.random.default_rng(T + D)
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    X = normal_bf16(rng, (T, D))
    d_X, d_tmap, d_z = be.upload(X), be.upload(tmap), be.alloc(T * K * D * 2)
    assert be.lib.dataflow_submit_default_prepare_experts(be.hp, CS, BF, BF, T, D, K, d_X.ptr, d_tmap.ptr, d_z.ptr) == 0
    be.sync(CS)
    zones = be.read(d_z.ptr, (T * K, D), np.uint16)
    want = np.zeros_like(zones)
    oracle.oracle_prepare_experts(T, D, K, O.ptr(X), O.ptr(tmap), O.ptr(want))
    assert (zones == want).all()
    # per-expert variant
    d_counts, d_incl, d_emap = be.upload(counts), be.upload(incl), be.upload(emap)
    for e in (0, E - 1):
        d_ze = be.alloc(max(int(counts[e]), 1) * D * 2)
        assert be.lib.dataflow_submit_default_prepare_expert_zone(be.hp, CS, BF, BF, D, d_X.ptr, e, d_counts.ptr, d_incl.ptr, d_emap.ptr, d_ze.ptr) == 0
        be.sync(CS)
        assert (be.read(d_ze.ptr, (int(counts[e]), D), np.uint16) == want[incl[e] - counts[e]:incl[e]]).all()


@pytest.mark.parametrize("T,D,E,K,with_w", [(256, 512, 8, 2, True), (100, 2048, 32, 4, True), (300, 4096, 64, 8, True),
                                            (300, 4096, 64, 8, False), (17, 8, 4, 3, True), (40, 10000, 8, 5, True)])
def test_combine_bit_exact(backend, oracle, T, D, E, K, with_w):
    print("case combine T=%d D=%d E=%d K=%d w=%s" % (T, D, E, K, with_w), flush=True)
    be = backend
    rng = np.random.default_rng(T * 3 + D + K)
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    zones = normal_bf16(rng, (T * K, D))
    w = rng.random((T, K)).astype(np.float32)
    w[0, 0] = 1.0                                   # the reference special-cases a weight of exactly 1
    resid = normal_bf16(rng, (T, D))
    d_z, d_tmap, d_w, d_out = be.upload(zones), be.upload(tmap), be.upload(w), be.upload(resid)
    assert be.lib.dataflow_submit_default_merge_experts(be.hp, CS, BF, BF, T, D, K, d_z.ptr, d_tmap.ptr, d_w.ptr if with_w else None, d_out.ptr) == 0
    be.sync(CS)
    got = be.read(d_out.ptr, (T, D), np.uint16)
    want = resid.copy()
    oracle.oracle_merge_experts(T, D, K, O.ptr(zones), O.ptr(tmap), O.ptr(w) if with_w else None, O.ptr(want))
    # same fp32 fma chain in the same order: identical bits
    assert (got == want).all()
    # the form that starts from zero instead of reading the row: equal to the oracle's combine into a cleared array,
    # whatever the output buffer held before (here: the result of the call above); rows of -0.0 included
    zones[tmap[1]] = 0x8000
    d_z.free()
    d_z = be.upload(zones)
    assert be.lib.dataflow_submit_amd_merge_experts_fresh(be.hp, CS, BF, BF, T, D, K, d_z.ptr, d_tmap.ptr, d_w.ptr if with_w else None, d_out.ptr) == 0
    be.sync(CS)
    want = np.zeros((T, D), dtype=np.uint16)
    oracle.oracle_merge_experts(T, D, K, O.ptr(zones), O.ptr(tmap), O.ptr(w) if with_w else None, O.ptr(want))
    assert (be.read(d_out.ptr, (T, D), np.uint16) == want).all()


def test_per_expert_combine(backend, oracle):
    be = backend
    rng = np.random.default_rng(5)
    T, D, E, K = 200, 1024, 8, 2
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    zones = normal_bf16(rng, (T * K, D))
    w = (rng.random((T, K)) + 0.1).astype(np.float32)
    d_z, d_incl, d_emap, d_w, d_ch = be.upload(zones), be.upload(incl), be.upload(emap), be.upload(w), be.upload(chosen)
    d_out = be.alloc(T * D * 2)
    be.zero(d_out.ptr, T * D * 2, CS)
    want = np.zeros((T, D), dtype=np.uint16)
    for e in range(E):
        n = int(counts[e])
        base = int(incl[e]) - n
        assert be.lib.dataflow_submit_default_merge_expert_result(be.hp, CS, BF, BF, n, D, K, d_z.ptr + base * D * 2, e, d_incl.ptr, d_emap.ptr,
                                                                  d_w.ptr, d_ch.ptr, d_out.ptr) == 0
        oracle.oracle_merge_expert_result(n, D, K, O.ptr(np.ascontiguousarray(zones[base:base + n])), e, O.ptr(incl), O.ptr(emap),
                                          O.ptr(w), O.ptr(chosen), O.ptr(want))
    be.sync(CS)
    assert (be.read(d_out.ptr, (T, D), np.uint16) == want).all()


@pytest.mark.parametrize("rows,cols", [(512, 1024), (300, 1408), (1, 8), (4097, 1024)])
def test_swiglu_forward_and_backward(backend, oracle, rows, cols):
    print("case swiglu rows=%d cols=%d" % (rows, cols), flush=True)
    be = backend
    rng = np.random.default_rng(rows + cols)
    x1, x3, g = normal_bf16(rng, (rows, cols), 2.0), normal_bf16(rng, (rows, cols), 2.0), normal_bf16(rng, (rows, cols))
    d1, d3, dg = be.upload(x1), be.upload(x3), be.upload(g)
    d_out, d_d1, d_d3 = be.alloc(rows * cols * 2), be.alloc(rows * cols * 2), be.alloc(rows * cols * 2)
    assert be.lib.dataflow_submit_default_swiglu(be.hp, CS, BF, rows, cols, d1.ptr, d3.ptr, d_out.ptr) == 0
    assert be.lib.dataflow_submit_default_swiglu_bwd_x(be.hp, CS, BF, BF, rows, cols, d1.ptr, d3.ptr, dg.ptr, d_d1.ptr, d_d3.ptr) == 0
    be.sync(CS)
    want, w1, w3 = np.zeros_like(x1), np.zeros_like(x1), np.zeros_like(x1)
    oracle.oracle_swiglu(rows, cols, O.ptr(x1), O.ptr(x3), O.ptr(want))
    oracle.oracle_swiglu_bwd_x(rows, cols, O.ptr(x1), O.ptr(x3), O.ptr(g), O.ptr(w1), O.ptr(w3))
    # fast exp / reciprocal on the device: allow 1 bf16 ulp against the oracle's libm result
    assert bf16_ulp_diff(be.read(d_out.ptr, (rows, cols), np.uint16), want).max() <= 1
    assert bf16_ulp_diff(be.read(d_d1.ptr, (rows, cols), np.uint16), w1).max() <= 1
    assert bf16_ulp_diff(be.read(d_d3.ptr, (rows, cols), np.uint16), w3).max() <= 1
    # in place: out aliases x_w1
    assert be.lib.dataflow_submit_default_swiglu(be.hp, CS, BF, rows, cols, d1.ptr, d3.ptr, d1.ptr) == 0
    be.sync(CS)
    assert bf16_ulp_diff(be.read(d1.ptr, (rows, cols), np.uint16), want).max() <= 1


@pytest.mark.parametrize("T,E,K,coarse", [(256, 8, 2, True), (8192, 64, 8, False), (1000, 32, 4, True), (777, 7, 3, True), (64, 130, 6, True),
                                          (65, 256, 1, False), (100, 48, 20, True), (31, 32, 32, True), (300, 2000, 9, False), (1, 4, 4, False)])
def test_select_experts_fp32_bit_exact(backend, oracle, T, E, K, coarse):
    """the op on fp32 logits (select_experts.cu:3-295): integer results bit-exact, weights to fp32 accuracy"""
    print("case select fp32 T=%d E=%d K=%d coarse=%s" % (T, E, K, coarse), flush=True)
    rng = np.random.default_rng(T * 31 + E * 7 + K)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if coarse:
        logits = np.round(logits * 4) / 4
    w_o, ch_o, counts_o, cum_o, host_o = O.select_experts_fp32(oracle, logits, K)
    w_g, ch_g, counts_g, cum_g, host_g, _, _ = gpu_select(backend, logits, K, B.DATAFLOW_FP32)
    assert (ch_g == ch_o).all()
    assert (counts_g[:E] == counts_o[:E]).all() and counts_g[E] == (T + 31) // 32
    assert (cum_g == cum_o).all() and (host_g == counts_o[:E]).all()
    np.testing.assert_allclose(w_g, w_o, rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("dt_name", ["fp32", "fp16"])
@pytest.mark.parametrize("rows,cols", [(64, 1024), (333, 1408), (7, 8), (1, 4096)])
def test_swiglu_fp32_fp16_forward_and_backward(backend, oracle, dt_name, rows, cols):
    """swiglu / swiglu_bwd_x on fp32 and fp16 elements (swiglu.cu:4-64, swiglu_bwd_x.cu:4-109): fp32 within 4e-6 relative of the
    oracle's libm result, fp16 within one step of the element type"""
    print("case swiglu %s rows=%d cols=%d" % (dt_name, rows, cols), flush=True)
    be = backend
    dt, npdt = (B.DATAFLOW_FP32, np.float32) if dt_name == "fp32" else (B.DATAFLOW_FP16, np.float16)
    rng = np.random.default_rng(rows + cols)
    x1, x3, g = [(rng.standard_normal((rows, cols)) * s_).astype(npdt) for s_ in (2.0, 2.0, 1.0)]
    d1, d3, dg = be.upload(x1), be.upload(x3), be.upload(g)
    nbytes = rows * cols * x1.itemsize
    d_out, d_d1, d_d3 = be.alloc(nbytes), be.alloc(nbytes), be.alloc(nbytes)
    assert be.lib.dataflow_submit_default_swiglu(be.hp, CS, dt, rows, cols, d1.ptr, d3.ptr, d_out.ptr) == 0
    assert be.lib.dataflow_submit_default_swiglu_bwd_x(be.hp, CS, dt, dt, rows, cols, d1.ptr, d3.ptr, dg.ptr, d_d1.ptr, d_d3.ptr) == 0
    be.sync(CS)
    want = O.swiglu_typed(oracle, x1, x3)
    w1, w3 = O.swiglu_bwd_x_typed(oracle, x1, x3, g)

    a64, b64, g64 = x1.astype(np.float64), x3.astype(np.float64), g.astype(np.float64)

    def check(got, expect, what, terms=None):
        """one step of the element type on the result, plus fp32 rounding of the terms it is summed from (dX_w1 = g x3 (s + x1 s (1 - s))
        cancels around x1 = -1.28: there the error is that of the terms, not of the small result)"""
        got, expect = got.astype(np.float64), expect.astype(np.float64)
        step = 4e-6 if npdt == np.float32 else 2.0 ** -10                  # fp16: one step of a value's magnitude
        floor = 1e-30 if npdt == np.float32 else 2.0 ** -24                # fp16: the subnormal spacing
        slack = 0.0 if terms is None else 4e-6 * terms
        assert (np.abs(got - expect) <= step * np.abs(expect) + slack + floor).all(), what

    check(be.read(d_out.ptr, (rows, cols), npdt), want, "out")
    check(be.read(d_d1.ptr, (rows, cols), npdt), w1, "dX_w1", terms=np.abs(g64 * b64) * (1.0 + np.abs(a64)))
    check(be.read(d_d3.ptr, (rows, cols), npdt), w3, "dX_w3")
    # in place: out aliases x_w1
    assert be.lib.dataflow_submit_default_swiglu(be.hp, CS, dt, rows, cols, d1.ptr, d3.ptr, d1.ptr) == 0
    be.sync(CS)
    check(be.read(d1.ptr, (rows, cols), npdt), want, "out in place")
    for d in (d1, d3, dg, d_out, d_d1, d_d3):
        d.free()


@pytest.mark.parametrize("T,D,E,K", [(128, 512, 8, 2), (200, 4096, 64, 8), (50, 2048, 32, 4), (9, 16, 4, 3), (30, 10000, 6, 2)])
def test_router_bwd_x_per_expert_and_all(backend, oracle, T, D, E, K):
    print("case router_bwd_x T=%d D=%d E=%d K=%d" % (T, D, E, K), flush=True)
    be = backend
    rng = np.random.default_rng(T + D + E)
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    y = normal_bf16(rng, (T * K, D))
    dY = normal_bf16(rng, (T, D))
    w = (rng.random((T, K)) + 0.05).astype(np.float32)
    # oracle, per expert, in place
    zones_o = y.copy()
    dlog_o = np.zeros((T, E), dtype=np.uint16)
    for e in range(E):
        seg = zones_o[incl[e] - counts[e]:incl[e]]
        oracle.oracle_router_bwd_x(int(counts[e]), D, E, K, e, O.ptr(incl), O.ptr(emap), O.ptr(chosen), O.ptr(w),
                                   seg.ctypes.data, O.ptr(dY), O.ptr(dlog_o), seg.ctypes.data)
    d_incl, d_emap, d_ch, d_w, d_dY, d_tmap = be.upload(incl), be.upload(emap), be.upload(chosen), be.upload(w), be.upload(dY), be.upload(tmap)
    # (a) reference signature, one launch per expert
    d_z = be.upload(y)
    d_dlog = be.alloc(T * E * 2)
    be.zero(d_dlog.ptr, T * E * 2, CS)
    for e in range(E):
        n = int(counts[e])
        zp = d_z.ptr + (int(incl[e]) - n) * D * 2
        assert be.lib.dataflow_submit_router_bwd_x(be.hp, CS, BF, BF, n, D, E, K, e, d_incl.ptr, d_emap.ptr, d_ch.ptr, d_w.ptr,
                                                   zp, d_dY.ptr, d_dlog.ptr, zp) == 0
    be.sync(CS)
    assert (be.read(d_z.ptr, (T * K, D), np.uint16) == zones_o).all()            # exact bf16 product, one rounding
    dlog_g = be.read(d_dlog.ptr, (T, E), np.uint16)
    assert bf16_ulp_diff(dlog_g, dlog_o).max() <= 1                               # fp32 vs fp64 dot, then one rounding
    # (b) grouped addition: all experts in one launch
    d_z2 = be.upload(y)
    be.zero(d_dlog.ptr, T * E * 2, CS)
    assert be.lib.dataflow_submit_amd_router_bwd_x_all(be.hp, CS, BF, BF, T, D, E, K, d_tmap.ptr, d_ch.ptr, d_w.ptr,
                                                       d_z2.ptr, d_dY.ptr, d_dlog.ptr, d_z2.ptr) == 0
    be.sync(CS)
    assert (be.read(d_z2.ptr, (T * K, D), np.uint16) == zones_o).all()
    assert bf16_ulp_diff(be.read(d_dlog.ptr, (T, E), np.uint16), dlog_o).max() <= 1


@pytest.mark.parametrize("T,D,E,K,H", [(128, 512, 8, 2, 256), (200, 1024, 64, 8, 1024), (50, 256, 32, 4, 1408), (9, 16, 4, 3, 8), (1, 64, 4, 2, 520)])
def test_backward_without_recompute_ops(backend, oracle, T, D, E, K, H):
    """the two ops of the backward that does not recompute the expert outputs: the scaled dispatch gives the rows
    router_bwd_x writes (bit-exact); the routed SwiGLU backward gives default_swiglu's h and default_swiglu_bwd_x's
    dx1 / dx3 bit for bit and the router gradient bf16(<h, dh> / w) (fp64 dot product, one rounding: <= 1 step)"""
    print("case no-recompute ops T=%d D=%d E=%d K=%d H=%d" % (T, D, E, K, H), flush=True)
    be = backend
    rng = np.random.default_rng(T + D + E + H)
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    R = T * K
    dY = normal_bf16(rng, (T, D))
    w = (rng.random((T, K)) + 0.05).astype(np.float32)
    # scaled dispatch against the oracle's router_bwd_x rows (its output does not depend on the expert outputs)
    rows_o, dlog_o = normal_bf16(rng, (R, D)), np.zeros((T, E), dtype=np.uint16)
    for e in range(E):
        seg = rows_o[incl[e] - counts[e]:incl[e]]
        oracle.oracle_router_bwd_x(int(counts[e]), D, E, K, e, O.ptr(incl), O.ptr(emap), O.ptr(chosen), O.ptr(w),
                                   seg.ctypes.data, O.ptr(dY), O.ptr(dlog_o), seg.ctypes.data)
    d_dY, d_tmap, d_emap, d_ch, d_w = be.upload(dY), be.upload(tmap), be.upload(emap), be.upload(chosen), be.upload(w)
    d_rows = be.alloc(R * D * 2)
    assert be.lib.dataflow_submit_amd_prepare_experts_scaled(be.hp, CS, BF, BF, T, D, K, d_dY.ptr, d_tmap.ptr, d_w.ptr, d_rows.ptr) == 0
    be.sync(CS)
    assert (be.read(d_rows.ptr, (R, D), np.uint16) == rows_o).all()
    # routed SwiGLU backward
    x1, x3, dh = normal_bf16(rng, (R, H), 2.0), normal_bf16(rng, (R, H), 2.0), normal_bf16(rng, (R, H))
    d_x1, d_x3, d_dh = be.upload(x1), be.upload(x3), be.upload(dh)
    d_h, d_d1, d_d3, d_dlog = be.alloc(R * H * 2), be.alloc(R * H * 2), be.alloc(R * H * 2), be.alloc(T * E * 2)
    d_h2, d_d1b, d_d3b = be.alloc(R * H * 2), be.alloc(R * H * 2), be.alloc(R * H * 2)
    be.zero(d_dlog.ptr, T * E * 2, CS)
    assert be.lib.dataflow_submit_amd_swiglu_bwd_x_routed(be.hp, CS, BF, BF, R, H, E, K, H, H, d_emap.ptr, d_tmap.ptr, d_ch.ptr, d_w.ptr,
                                                          d_x1.ptr, d_x3.ptr, d_dh.ptr, d_dlog.ptr, d_d1.ptr, d_d3.ptr, d_h.ptr) == 0
    assert be.lib.dataflow_submit_default_swiglu(be.hp, CS, BF, R, H, d_x1.ptr, d_x3.ptr, d_h2.ptr) == 0
    assert be.lib.dataflow_submit_default_swiglu_bwd_x(be.hp, CS, BF, BF, R, H, d_x1.ptr, d_x3.ptr, d_dh.ptr, d_d1b.ptr, d_d3b.ptr) == 0
    be.sync(CS)
    h = be.read(d_h.ptr, (R, H), np.uint16)
    assert (h == be.read(d_h2.ptr, (R, H), np.uint16)).all()
    assert (be.read(d_d1.ptr, (R, H), np.uint16) == be.read(d_d1b.ptr, (R, H), np.uint16)).all()
    assert (be.read(d_d3.ptr, (R, H), np.uint16) == be.read(d_d3b.ptr, (R, H), np.uint16)).all()
    want_h = np.zeros_like(x1)
    oracle.oracle_swiglu(R, H, O.ptr(x1), O.ptr(x3), O.ptr(want_h))
    assert bf16_ulp_diff(h, want_h).max() <= 1
    wb = bf16_to_f64(f32_to_bf16(w))
    dots = (bf16_to_f64(h) * bf16_to_f64(dh)).sum(axis=1)                      # per routed row
    want = np.zeros((T, E))
    want[np.repeat(np.arange(T), K), chosen.reshape(-1).astype(np.int64)] = (dots[tmap.reshape(-1)] / wb.reshape(-1))
    got = be.read(d_dlog.ptr, (T, E), np.uint16)
    sel = np.zeros((T, E), dtype=bool)
    sel[np.repeat(np.arange(T), K), chosen.reshape(-1).astype(np.int64)] = True
    assert (got[~sel] == 0).all()                                              # unselected columns stay zero
    scale = np.abs(want).max()
    tiny = np.abs(want) < 2.0 ** -6 * scale
    assert bf16_ulp_diff(got, f32_to_bf16(want.astype(np.float32)))[sel & ~tiny].max(initial=0) <= 1
    assert np.abs(bf16_to_f64(got) - want).max() <= 2.0 ** -8 * scale
    # x1 | x3 side by side per row (row stride 2H), gradients written the same way; the strided forward SwiGLU
    d_x13, d_dx13, d_h3 = be.upload(np.concatenate([x1, x3], axis=1)), be.alloc(2 * R * H * 2), be.alloc(R * H * 2)
    be.zero(d_dlog.ptr, T * E * 2, CS)
    assert be.lib.dataflow_submit_amd_swiglu_bwd_x_routed(be.hp, CS, BF, BF, R, H, E, K, 2 * H, 2 * H, d_emap.ptr, d_tmap.ptr, d_ch.ptr, d_w.ptr,
                                                          d_x13.ptr, d_x13.ptr + 2 * H, d_dh.ptr, d_dlog.ptr, d_dx13.ptr, d_dx13.ptr + 2 * H, d_h.ptr) == 0
    assert be.lib.dataflow_submit_amd_swiglu_strided(be.hp, CS, BF, R, H, 2 * H, d_x13.ptr, d_x13.ptr + 2 * H, d_h3.ptr) == 0
    be.sync(CS)
    dx13 = be.read(d_dx13.ptr, (R, 2 * H), np.uint16)
    assert (dx13[:, :H] == be.read(d_d1b.ptr, (R, H), np.uint16)).all() and (dx13[:, H:] == be.read(d_d3b.ptr, (R, H), np.uint16)).all()
    assert (be.read(d_h.ptr, (R, H), np.uint16) == h).all() and (be.read(d_h3.ptr, (R, H), np.uint16) == h).all()
    assert (be.read(d_dlog.ptr, (T, E), np.uint16) == got).all()
    assert be.lib.dataflow_submit_amd_swiglu_strided(be.hp, CS, BF, R, H, H - 8, d_x13.ptr, d_x13.ptr + 2 * H, d_h3.ptr) == -1   # stride < row length
    # in place: dX_w1 aliases dh
    assert be.lib.dataflow_submit_amd_swiglu_bwd_x_routed(be.hp, CS, BF, BF, R, H, E, K, H, H, d_emap.ptr, d_tmap.ptr, d_ch.ptr, d_w.ptr,
                                                          d_x1.ptr, d_x3.ptr, d_dh.ptr, d_dlog.ptr, d_dh.ptr, d_d3.ptr, d_h.ptr) == 0
    be.sync(CS)
    assert (be.read(d_dh.ptr, (R, H), np.uint16) == be.read(d_d1b.ptr, (R, H), np.uint16)).all()
    assert (be.read(d_dlog.ptr, (T, E), np.uint16) == got).all()


def test_routed_swiglu_backward_with_tiny_and_zero_routing_weights(backend):
    """amd_swiglu_bwd_x_routed divides <h, dh> by bf16(w).  Routing weights from 1 down to 1e-38 and one that is exactly 0:
    every output stays finite; where bf16(w) != 0 the router gradient is bf16(<h, dh> / bf16(w)); where it is 0 the kernel
    writes 0 (the reference's <y, dY> is finite there, but the softmax-gate backward multiplies that entry by w = 0 and
    every other entry of the row by w * d = 0, so nothing downstream differs).  dh is scaled by bf16(w) as in the layer,
    where dh = (bf16(w) dY) W2."""
    be = backend
    rng = np.random.default_rng(5)
    T, E, K, H = 24, 8, 8, 256
    R = T * K
    chosen = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint16)
    # routed row of (t, k): expert-major order, tokens ascending inside an expert (what build_expert_mapping produces)
    order = np.lexsort((np.repeat(np.arange(T), K), chosen.reshape(-1)))
    tmap = np.empty(R, dtype=np.int32)
    tmap[order] = np.arange(R, dtype=np.int32)
    tmap = tmap.reshape(T, K)
    emap = np.repeat(np.arange(T), K)[order].astype(np.int32)
    w = np.tile(np.array([1.0, 0.5, 1e-3, 1e-10, 1e-20, 1e-30, 1e-38, 0.0], dtype=np.float32), (T, 1))
    wb = bf16_to_f64(f32_to_bf16(w))
    assert (wb[:, -1] == 0).all() and (wb[:, :-1] != 0).all()
    x1, x3 = normal_bf16(rng, (R, H), 2.0), normal_bf16(rng, (R, H), 2.0)
    dh = f32_to_bf16((bf16_to_f64(normal_bf16(rng, (R, H))) * wb.reshape(-1)[np.argsort(tmap.reshape(-1))][:, None]).astype(np.float32))
    d_emap, d_tmap, d_ch, d_w = be.upload(emap), be.upload(tmap), be.upload(chosen), be.upload(w)
    d_x1, d_x3, d_dh = be.upload(x1), be.upload(x3), be.upload(dh)
    d_h, d_d1, d_d3, d_dlog = be.alloc(R * H * 2), be.alloc(R * H * 2), be.alloc(R * H * 2), be.alloc(T * E * 2)
    be.zero(d_dlog.ptr, T * E * 2, CS)
    assert be.lib.dataflow_submit_amd_swiglu_bwd_x_routed(be.hp, CS, BF, BF, R, H, E, K, H, H, d_emap.ptr, d_tmap.ptr, d_ch.ptr, d_w.ptr,
                                                          d_x1.ptr, d_x3.ptr, d_dh.ptr, d_dlog.ptr, d_d1.ptr, d_d3.ptr, d_h.ptr) == 0
    be.sync(CS)
    got = be.read(d_dlog.ptr, (T, E), np.uint16)
    for arr in (got, be.read(d_d1.ptr, (R, H), np.uint16), be.read(d_d3.ptr, (R, H), np.uint16), be.read(d_h.ptr, (R, H), np.uint16)):
        assert np.isfinite(bf16_to_f64(arr)).all()
    h = bf16_to_f64(be.read(d_h.ptr, (R, H), np.uint16))
    dots = (h * bf16_to_f64(dh)).sum(axis=1)
    for t in range(T):
        for k in range(K):
            g = got[t, chosen[t, k]]
            if wb[t, k] == 0:
                assert g == 0                                               # the documented value
                continue
            want = dots[tmap[t, k]] / wb[t, k]
            if w[t, k] >= 1e-20:                                            # below, <h, dh> itself is a sum of fp32 denormals
                assert abs(bf16_to_f64(np.array([g], dtype=np.uint16))[0] - want) <= 2.0 ** -7 * max(abs(want), 1e-3)


def test_router_gate_bwd_x(backend, oracle):
    be = backend
    rng = np.random.default_rng(3)
    T, E, K = 1000, 64, 8
    chosen, *_ = make_routing(rng, T, E, K)
    p = rng.random((T, K)).astype(np.float32)
    p /= p.sum(1, keepdims=True)
    d = np.zeros((T, E), dtype=np.float32)
    np.put_along_axis(d, chosen.astype(np.int64), rng.standard_normal((T, K)).astype(np.float32), axis=1)
    d_bits = f32_to_bf16(d)
    d_d, d_ch, d_p = be.upload(d_bits), be.upload(chosen), be.upload(p)
    assert be.lib.dataflow_submit_router_gate_bwd_x(be.hp, CS, BF, BF, T, E, K, d_ch.ptr, d_p.ptr, d_d.ptr) == 0
    be.sync(CS)
    want = d_bits.copy()
    oracle.oracle_router_gate_bwd_x(T, E, K, O.ptr(chosen), O.ptr(p), O.ptr(want))
    assert bf16_ulp_diff(be.read(d_d.ptr, (T, E), np.uint16), want).max() <= 1


def run_gpu_matmul(be, transa, transb, M, K, N, A, Bm, alpha, beta, Cin, workspace_bytes=0):
    d_A, d_B = be.upload(A), be.upload(Bm)
    d_D = be.alloc(max(N * M, 1) * 2)
    c_ptr = None
    c_dt = B.DATAFLOW_NONE
    if Cin is not None:
        be.write(d_D.ptr, Cin)           # C aliases D, as the reference's accumulate calls do
        c_ptr, c_dt = d_D.ptr, BF
    d_ws = be.alloc(workspace_bytes) if workspace_bytes else None
    ret = be.lib.dataflow_submit_matmul(be.hp, CS, BF, BF, c_dt, BF, B.DATAFLOW_FP32, transa, transb, M, K, N, alpha, beta,
                                        d_A.ptr, d_B.ptr, c_ptr, d_D.ptr, workspace_bytes, d_ws.ptr if d_ws else None)
    assert ret == 0
    be.sync(CS)
    return be.read(d_D.ptr, (N, M), np.uint16)


def check_matmul(got, want_o, K):
    """vs the oracle (fp64 accumulate, one rounding): fp32 MFMA accumulation may move a result across a rounding
    boundary, so allow 1 bf16 ulp, and bound the overall relative error by 1e-2 of the output scale"""
    g, w = bf16_to_f64(got), bf16_to_f64(want_o)
    scale = max(np.abs(w).max(), 1e-30)
    assert np.abs(g - w).max() <= 1e-2 * scale
    tiny = np.abs(w) < 2.0 ** -6 * scale                # ulp distance is meaningless next to cancellation
    assert bf16_ulp_diff(got, want_o)[~tiny].max(initial=0) <= 1


MM_SHAPES = [(128, 64, 128), (256, 256, 256), (1024, 512, 300), (96, 72, 40), (8, 8, 1), (1408, 2048, 77), (2048, 1408, 513), (64, 2048, 4096),
             (520, 200, 260)]


@pytest.mark.parametrize("transa,transb", [(1, 0), (0, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("M,K,N", MM_SHAPES)
def test_matmul_layouts(backend, oracle, transa, transb, M, K, N):
    print("case matmul ta=%d tb=%d M=%d K=%d N=%d" % (transa, transb, M, K, N), flush=True)
    rng = np.random.default_rng(M + 3 * K + 7 * N + transa * 2 + transb)
    A = normal_bf16(rng, (M, K) if transa else (K, M))
    Bm = normal_bf16(rng, (K, N) if transb else (N, K), 0.05)
    got = run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 1.0, 0.0, None)
    check_matmul(got, O.matmul(oracle, transa, transb, M, K, N, A, Bm), K)
    Cin = normal_bf16(rng, (N, M))
    got2 = run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 0.5, 1.0, Cin)
    check_matmul(got2, O.matmul(oracle, transa, transb, M, K, N, A, Bm, alpha=0.5, beta=1.0, Cin=Cin), K)


@pytest.mark.parametrize("transa,transb,M,K,N", [
    (1, 0, 64, 4096, 8192),      # router logits of config 4: 64 tiles, K split 4 ways
    (0, 1, 4096, 8192, 64),      # router weight gradient: 32 tiles, K split 8 ways
    (0, 1, 512, 2000, 72),       # K not a multiple of the k-tile or of the split
    (0, 0, 128, 1100, 128),      # one tile; the last split is short
    (1, 1, 264, 1536, 40)])
def test_matmul_split_k_through_the_workspace(backend, oracle, transa, transb, M, K, N):
    """Few tiles and a long K: with a workspace the problem is split along K (fp32 partial sums + one reduction pass);
    the result must meet the same bar as the unsplit run, with and without a C operand, and a workspace that is too
    small must give the unsplit result, not an error."""
    print("case split-k ta=%d tb=%d M=%d K=%d N=%d" % (transa, transb, M, K, N), flush=True)
    rng = np.random.default_rng(M + K + N)
    A = normal_bf16(rng, (M, K) if transa else (K, M))
    Bm = normal_bf16(rng, (K, N) if transb else (N, K), 0.05)
    big = 16 * M * N * 4
    want = O.matmul(oracle, transa, transb, M, K, N, A, Bm)
    check_matmul(run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 1.0, 0.0, None, big), want, K)
    unsplit = run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 1.0, 0.0, None)
    assert (run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 1.0, 0.0, None, M * N * 4) == unsplit).all()
    Cin = normal_bf16(rng, (N, M))
    got = run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 0.5, 1.0, Cin, big)
    check_matmul(got, O.matmul(oracle, transa, transb, M, K, N, A, Bm, alpha=0.5, beta=1.0, Cin=Cin), K)


def test_matmul_random_shapes(backend, oracle):
    """Seeded random problems over every kernel the dispatch can pick (128-tile direct, 256-tile streaming, split-K,
    the general path for sizes that are not multiples of 8), all four layouts, with and without a C operand."""
    rng = np.random.default_rng(20240607)
    cases = []
    for _ in range(10):                                   # small / medium, any size
        cases.append((int(rng.integers(1, 700)), int(rng.integers(1, 900)), int(rng.integers(1, 700))))
    for _ in range(8):                                    # multiples of 8: the direct-to-LDS kernels
        cases.append((8 * int(rng.integers(1, 160)), 8 * int(rng.integers(1, 300)), 8 * int(rng.integers(1, 160))))
    cases += [(2048, 520, 4096), (4096, 264, 2304), (1792, 1032, 4608)]      # enough 256-tiles for the streaming kernel
    cases += [(64, 8 * int(rng.integers(100, 700)), 1024), (1536, 8 * int(rng.integers(100, 700)), 40)]   # split-K candidates
    for n, (M, K, N) in enumerate(cases):
        transa, transb = [(1, 0), (0, 0), (0, 1), (1, 1)][n % 4]
        print("case random matmul %d ta=%d tb=%d M=%d K=%d N=%d" % (n, transa, transb, M, K, N), flush=True)
        A = normal_bf16(rng, (M, K) if transa else (K, M))
        Bm = normal_bf16(rng, (K, N) if transb else (N, K), 0.05)
        ws = 16 * M * N * 4 if n % 2 else 0
        if n % 3 == 0:
            Cin = normal_bf16(rng, (N, M))
            got = run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 0.75, 1.0, Cin, ws)
            check_matmul(got, O.matmul(oracle, transa, transb, M, K, N, A, Bm, alpha=0.75, beta=1.0, Cin=Cin), K)
        else:
            got = run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 1.0, 0.0, None, ws)
            check_matmul(got, O.matmul(oracle, transa, transb, M, K, N, A, Bm), K)


@pytest.mark.parametrize("M,K,N", [(100, 50, 30), (36, 20, 12), (7, 3, 5)])
def test_matmul_unaligned_shapes_take_the_scalar_path(backend, oracle, M, K, N):
    rng = np.random.default_rng(M)
    for transa, transb in [(1, 0), (0, 0), (0, 1)]:
        A = normal_bf16(rng, (M, K) if transa else (K, M))
        Bm = normal_bf16(rng, (K, N) if transb else (N, K))
        got = run_gpu_matmul(backend, transa, transb, M, K, N, A, Bm, 1.0, 0.0, None)
        check_matmul(got, O.matmul(oracle, transa, transb, M, K, N, A, Bm), K)


def test_matmul_special_cases(backend):
    be = backend
    rng = np.random.default_rng(1)
    X = normal_bf16(rng, (300, 256))
    eye = f32_to_bf16(np.eye(256, dtype=np.float32))
    assert (run_gpu_matmul(be, 1, 0, 256, 256, 300, eye, X, 1.0, 0.0, None) == X).all()       # identity weight
    assert (run_gpu_matmul(be, 0, 0, 256, 256, 300, eye, X, 1.0, 0.0, None) == X).all()
    # unsupported dtype is an error, not a silent fallback
    d = be.alloc(1024)
    assert be.lib.dataflow_submit_matmul(be.hp, CS, B.DATAFLOW_FP16, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, 1, 0, 8, 8, 8, 1.0, 0.0,
                                         d.ptr, d.ptr, None, d.ptr, 0, None) == -1


TYPED_KINDS = {O.ELEM_FP32: (B.DATAFLOW_FP32, np.float32), O.ELEM_FP16: (B.DATAFLOW_FP16, np.uint16), O.ELEM_BF16: (BF, np.uint16)}


def typed_operand(rng, shape, kind, scale=1.0):
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    if kind == O.ELEM_FP32:
        return x, x.astype(np.float64)
    if kind == O.ELEM_FP16:
        h = x.astype(np.float16)
        return h.view(np.uint16), h.astype(np.float64)
    b = f32_to_bf16(x)
    return b, bf16_to_f64(b)


def typed_value(bits, kind):
    if kind == O.ELEM_FP32:
        return bits.astype(np.float64)
    if kind == O.ELEM_FP16:
        return bits.view(np.float16).astype(np.float64)
    return bf16_to_f64(bits)


@pytest.mark.parametrize("ab,cd", [(O.ELEM_FP32, O.ELEM_FP32), (O.ELEM_FP16, O.ELEM_FP16), (O.ELEM_FP16, O.ELEM_FP32), (O.ELEM_BF16, O.ELEM_FP32)])
def test_matmul_other_element_types(backend, oracle, ab, cd):
    """The matmul on fp32, fp16 and bf16 -> fp32 (fp32 accumulation) against the oracle's fp64 sum, all four layouts, shapes
    on and off the 128-tile and the k-tile, with and without C.  Bar: the sum of K fp32 terms may differ from the exact
    one by 64 * 2^-24 * sum |a b| (a random walk of K <= 4096 roundings stays far inside); an fp16 result may on top of
    that fall on the other neighbour of the exact value than the oracle's (one unit in the last place: 2^-10 relative, 2^-24
    absolute where it is subnormal)."""
    be = backend
    dt_ab, _ = TYPED_KINDS[ab]
    dt_cd, np_cd = TYPED_KINDS[cd]
    size_cd = 4 if cd == O.ELEM_FP32 else 2
    shapes = [(128, 64, 128), (96, 72, 40), (8, 8, 1), (1, 5, 3), (300, 1031, 260), (520, 200, 77), (256, 2048, 384)]
    for n, (M, K, N) in enumerate(shapes):
        for transa, transb in [(1, 0), (0, 0), (0, 1), (1, 1)]:
            print("case typed matmul ab=%d cd=%d ta=%d tb=%d M=%d K=%d N=%d" % (ab, cd, transa, transb, M, K, N), flush=True)
            rng = np.random.default_rng(ab * 1000 + cd * 100 + n * 10 + transa * 2 + transb)
            A, a64 = typed_operand(rng, (M, K) if transa else (K, M), ab)
            Bm, b64 = typed_operand(rng, (K, N) if transb else (N, K), ab, 0.1)
            Cin, c64 = typed_operand(rng, (N, M), cd)
            opA = a64 if transa else a64.T
            opB = b64 if transb else b64.T
            terms = (np.abs(opA) @ np.abs(opB)).T
            d_A, d_B = be.upload(A), be.upload(Bm)
            for alpha, beta, c in ((1.0, 0.0, None), (0.5, 1.0, Cin)):
                d_D = be.alloc(N * M * size_cd)
                if c is not None:
                    be.write(d_D.ptr, c)
                ret = be.lib.dataflow_submit_matmul(be.hp, CS, dt_ab, dt_ab, dt_cd if c is not None else B.DATAFLOW_NONE, dt_cd, B.DATAFLOW_FP32,
                                                    transa, transb, M, K, N, alpha, beta, d_A.ptr, d_B.ptr,
                                                    d_D.ptr if c is not None else None, d_D.ptr, 0, None)
                assert ret == 0
                be.sync(CS)
                got = be.read(d_D.ptr, (N, M), np_cd)
                want_bits = O.matmul_typed(oracle, ab, cd, transa, transb, M, K, N, A, Bm, alpha=alpha, beta=beta, Cin=c)
                want = typed_value(want_bits, cd)
                tol = 64 * 2.0 ** -24 * (abs(alpha) * terms + (abs(beta) * np.abs(c64) if c is not None else 0.0)) + 1e-30
                if cd == O.ELEM_FP16:
                    tol = tol + 2.0 ** -10 * np.abs(want) + 2.0 ** -24
                err = np.abs(typed_value(got, cd) - want)
                assert (err <= tol).all(), "max excess %g at %s" % ((err - tol).max(), np.argwhere(err > tol)[:3])
    # combinations outside the list stay errors
    d = be.alloc(1024)
    for a_dt, b_dt, c_dt, d_dt, comp in [(B.DATAFLOW_FP32, B.DATAFLOW_FP32, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32),
                                         (B.DATAFLOW_FP16, B.DATAFLOW_FP16, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32),
                                         (B.DATAFLOW_FP16, B.DATAFLOW_FP16, B.DATAFLOW_NONE, B.DATAFLOW_FP16, B.DATAFLOW_FP16),
                                         (B.DATAFLOW_FP32, B.DATAFLOW_FP32, BF, B.DATAFLOW_FP32, B.DATAFLOW_FP32)]:
        beta = 1.0 if c_dt != B.DATAFLOW_NONE else 0.0
        assert be.lib.dataflow_submit_matmul(be.hp, CS, a_dt, b_dt, c_dt, d_dt, comp, 1, 0, 8, 8, 8, 1.0, beta,
                                             d.ptr, d.ptr, d.ptr if beta else None, d.ptr, 0, None) == -1


def ragged_counts(rng, G, total, zero_some):
    cuts = np.sort(rng.integers(0, total + 1, size=G - 1))
    counts = np.diff(np.concatenate([[0], cuts, [total]])).astype(np.int32)
    if zero_some and G > 2:
        counts[1] += counts[2]
        counts[2] = 0
    return counts


@pytest.mark.parametrize("transa", [1, 0])
@pytest.mark.parametrize("G,M,K,total", [(8, 256, 128, 1000), (4, 1408, 512, 700), (64, 1024, 256, 4096), (3, 64, 64, 5)])
def test_grouped_matmul_ragged_n(backend, oracle, transa, G, M, K, total):
    print("case grouped-N ta=%d G=%d M=%d K=%d rows=%d" % (transa, G, M, K, total), flush=True)
    be = backend
    rng = np.random.default_rng(G + M + K + total + transa)
    counts = ragged_counts(rng, G, total, True)
    incl = np.cumsum(counts).astype(np.int32)
    W = normal_bf16(rng, (G, M, K) if transa else (G, K, M), 0.05)
    X = normal_bf16(rng, (total, K))
    Cin = normal_bf16(rng, (total, M))
    d_W, d_X, d_cum = be.upload(W), be.upload(X), be.upload(incl)
    for beta in (0.0, 1.0):
        d_D = be.upload(Cin)
        ret = be.lib.dataflow_submit_amd_grouped_matmul(be.hp, CS, BF, BF, BF if beta else B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32,
                                                        transa, 0, B.AMD_GROUPED_RAGGED_N, M, K, total, G, d_cum.ptr, 1.0, beta,
                                                        d_W.ptr, M * K * 2, d_X.ptr, d_D.ptr if beta else None, d_D.ptr, 0)
        assert ret == 0
        be.sync(CS)
        got = be.read(d_D.ptr, (total, M), np.uint16)
        want = Cin.copy()
        for g in range(G):
            lo, hi = int(incl[g] - counts[g]), int(incl[g])
            if hi > lo:
                want[lo:hi] = O.matmul(oracle, transa, 0, M, K, hi - lo, W[g], np.ascontiguousarray(X[lo:hi]), 1.0, beta,
                                       np.ascontiguousarray(Cin[lo:hi]) if beta else None)
        check_matmul(got, want, K)


@pytest.mark.parametrize("transa", [1, 0])
def test_grouped_matmul_ragged_n_tile_edges(backend, oracle, transa):
    """Large enough for the persistent kernel, whose ragged-N form without C walks the token rows in tiles of 288 (with C:
    256): group sizes on both sides of one, two and four tiles of either height, single rows and empty groups."""
    be = backend
    M, K = 2048, 128
    counts = np.array([288, 289, 1, 0, 575, 576, 577, 287, 256, 257, 255, 0, 1152, 1153, 1151, 1024, 1025, 2, 300, 31], dtype=np.int32)
    G, total = len(counts), int(counts.sum())
    print("case grouped-N tile edges ta=%d G=%d M=%d K=%d rows=%d" % (transa, G, M, K, total), flush=True)
    rng = np.random.default_rng(77 + transa)
    incl = np.cumsum(counts).astype(np.int32)
    W = normal_bf16(rng, (G, M, K) if transa else (G, K, M), 0.05)
    X = normal_bf16(rng, (total, K))
    Cin = normal_bf16(rng, (total, M))
    d_W, d_X, d_cum = be.upload(W), be.upload(X), be.upload(incl)
    for beta in (0.0, 1.0):
        d_D = be.upload(Cin)
        assert be.lib.dataflow_submit_amd_grouped_matmul(be.hp, CS, BF, BF, BF if beta else B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32,
                                                         transa, 0, B.AMD_GROUPED_RAGGED_N, M, K, total, G, d_cum.ptr, 1.0, beta,
                                                         d_W.ptr, M * K * 2, d_X.ptr, d_D.ptr if beta else None, d_D.ptr, 0) == 0
        be.sync(CS)
        got = be.read(d_D.ptr, (total, M), np.uint16)
        want = Cin.copy()
        for g in range(G):
            lo, hi = int(incl[g] - counts[g]), int(incl[g])
            if hi > lo:
                want[lo:hi] = O.matmul(oracle, transa, 0, M, K, hi - lo, W[g], np.ascontiguousarray(X[lo:hi]), 1.0, beta,
                                       np.ascontiguousarray(Cin[lo:hi]) if beta else None)
        check_matmul(got, want, K)
        if beta == 0.0:
            # the same rows through the plain matmul op, group by group (256-row tiles or the small-tile kernels): every
            # element is accumulated over k in the same order whatever the tile, so the results agree bit for bit
            d_P = be.upload(Cin)
            for g in range(G):
                lo, hi = int(incl[g] - counts[g]), int(incl[g])
                if hi > lo:
                    assert be.lib.dataflow_submit_matmul(be.hp, CS, BF, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, transa, 0, M, K, hi - lo, 1.0, 0.0,
                                                         d_W.ptr + g * M * K * 2, d_X.ptr + lo * K * 2, None, d_P.ptr + lo * M * 2, 0, None) == 0
            be.sync(CS)
            per_group = be.read(d_P.ptr, (total, M), np.uint16)
            assert (per_group == got).all(), "%d elements differ from the per-group matmuls" % int((per_group != got).sum())
            d_P.free()
        d_D.free()


@pytest.mark.parametrize("transa", [1, 0])
@pytest.mark.parametrize("G,M,K,total,src_rows", [(8, 256, 128, 1000, 300),        # 128 x 128 tiles, direct-to-LDS loads
                                                   (64, 1024, 256, 40000, 5000),    # 256 x 256 tiles, persistent work-groups
                                                   (16, 512, 4096, 9000, 2048),     # the same with a long K
                                                   (4, 1408, 520, 700, 64),         # K not a multiple of the k-tile
                                                   (3, 64, 36, 5, 2)])              # odd K: the staged kernel
def test_grouped_matmul_gathered_equals_copy_then_matmul(backend, transa, G, M, K, total, src_rows):
    """The gathered form fetches B's rows through a row map; the values that reach the multiplies are those of a packed
    copy, so the result must equal dispatch + grouped matmul bit for bit (checked against this library's own
    ungathered op, which the test above holds to the oracle)."""
    print("case gathered grouped-N ta=%d G=%d M=%d K=%d rows=%d of %d" % (transa, G, M, K, total, src_rows), flush=True)
    be = backend
    rng = np.random.default_rng(G + M + K + total + transa)
    counts = ragged_counts(rng, G, total, True)
    incl = np.cumsum(counts).astype(np.int32)
    W = normal_bf16(rng, (G, M, K) if transa else (G, K, M), 0.05)
    src = normal_bf16(rng, (src_rows, K))
    row_map = rng.integers(0, src_rows, total).astype(np.int32)
    row_map[0], row_map[-1] = src_rows - 1, 0                      # both ends of the source occur
    packed = np.ascontiguousarray(src[row_map])
    Cin = normal_bf16(rng, (total, M))
    d_W, d_src, d_packed, d_cum, d_map = be.upload(W), be.upload(src), be.upload(packed), be.upload(incl), be.upload(row_map)
    for beta in (0.0, 1.0):
        d_want, d_got = be.upload(Cin), be.upload(Cin)
        c_dt = BF if beta else B.DATAFLOW_NONE
        assert be.lib.dataflow_submit_amd_grouped_matmul(be.hp, CS, BF, BF, c_dt, BF, B.DATAFLOW_FP32, transa, 0, B.AMD_GROUPED_RAGGED_N,
                                                         M, K, total, G, d_cum.ptr, 1.0, beta, d_W.ptr, M * K * 2, d_packed.ptr,
                                                         d_want.ptr if beta else None, d_want.ptr, 0) == 0
        assert be.lib.dataflow_submit_amd_grouped_matmul_gathered(be.hp, CS, BF, BF, c_dt, BF, B.DATAFLOW_FP32, transa, 0, B.AMD_GROUPED_RAGGED_N,
                                                                  M, K, total, G, d_cum.ptr, 1.0, beta, d_W.ptr, M * K * 2, d_src.ptr,
                                                                  d_got.ptr if beta else None, d_got.ptr, 0, d_map.ptr, src_rows) == 0
        be.sync(CS)
        got, want = be.read(d_got.ptr, (total, M), np.uint16), be.read(d_want.ptr, (total, M), np.uint16)
        assert (got == want).all(), "beta %g: %d of %d elements differ" % (beta, int((got != want).sum()), got.size)
        d_want.free(), d_got.free()
    # a missing map and a source of 4 GiB or more are refused
    for bad_map, bad_rows in ((None, src_rows), (d_map.ptr, (1 << 32) // (2 * K) + 1)):
        assert be.lib.dataflow_submit_amd_grouped_matmul_gathered(be.hp, CS, BF, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, transa, 0, B.AMD_GROUPED_RAGGED_N,
                                                                  M, K, total, G, d_cum.ptr, 1.0, 0.0, d_W.ptr, M * K * 2, d_src.ptr, None, d_packed.ptr, 0,
                                                                  bad_map, bad_rows) == -1
    be.sync(CS)


@pytest.mark.parametrize("G,M,N,total,src_rows", [(8, 256, 128, 1000, 300),          # 128 x 128 tiles
                                                   (64, 1024, 256, 40000, 5000),      # 256 x 256 tiles, persistent work-groups
                                                   (16, 4096, 512, 9000, 2048),       # the layer's shape: wide rows
                                                   (4, 520, 1408, 700, 64),           # M not a multiple of the tile
                                                   (3, 36, 64, 5, 2)])                # the staged kernel
def test_grouped_matmul_gathered_ragged_k_equals_copy_then_matmul(backend, G, M, N, total, src_rows):
    """Ragged K: the k-rows of A are the gathered ones.  Same bar as above: bit-identical to the packed copy."""
    print("case gathered grouped-K G=%d M=%d N=%d rows=%d of %d" % (G, M, N, total, src_rows), flush=True)
    be = backend
    rng = np.random.default_rng(G + M + N + total)
    counts = ragged_counts(rng, G, total, True)
    incl = np.cumsum(counts).astype(np.int32)
    src = normal_bf16(rng, (src_rows, M))
    row_map = rng.integers(0, src_rows, total).astype(np.int32)
    row_map[0], row_map[-1] = src_rows - 1, 0
    packed = np.ascontiguousarray(src[row_map])
    Bm = normal_bf16(rng, (total, N), 0.05)
    Cin = normal_bf16(rng, (G, N, M))
    d_src, d_packed, d_B, d_cum, d_map = be.upload(src), be.upload(packed), be.upload(Bm), be.upload(incl), be.upload(row_map)
    for beta in (1.0, 0.0):
        d_want, d_got = be.upload(Cin), be.upload(Cin)
        c_dt = BF if beta else B.DATAFLOW_NONE
        assert be.lib.dataflow_submit_amd_grouped_matmul(be.hp, CS, BF, BF, c_dt, BF, B.DATAFLOW_FP32, 0, 1, B.AMD_GROUPED_RAGGED_K,
                                                         M, 0, N, G, d_cum.ptr, 1.0, beta, d_packed.ptr, 0, d_B.ptr,
                                                         d_want.ptr if beta else None, d_want.ptr, N * M * 2) == 0
        assert be.lib.dataflow_submit_amd_grouped_matmul_gathered(be.hp, CS, BF, BF, c_dt, BF, B.DATAFLOW_FP32, 0, 1, B.AMD_GROUPED_RAGGED_K,
                                                                  M, 0, N, G, d_cum.ptr, 1.0, beta, d_src.ptr, 0, d_B.ptr,
                                                                  d_got.ptr if beta else None, d_got.ptr, N * M * 2, d_map.ptr, src_rows) == 0
        be.sync(CS)
        got, want = be.read(d_got.ptr, (G, N, M), np.uint16), be.read(d_want.ptr, (G, N, M), np.uint16)
        assert (got == want).all(), "beta %g: %d of %d elements differ" % (beta, int((got != want).sum()), got.size)
        d_want.free(), d_got.free()


@pytest.mark.parametrize("G,M,N,total", [(8, 256, 128, 1000), (4, 512, 1408, 700), (64, 256, 1024, 4096), (3, 64, 64, 5)])
def test_grouped_matmul_ragged_k(backend, oracle, G, M, N, total):
    print("case grouped-K G=%d M=%d N=%d rows=%d" % (G, M, N, total), flush=True)
    be = backend
    rng = np.random.default_rng(G + M + N + total)
    counts = ragged_counts(rng, G, total, True)
    incl = np.cumsum(counts).astype(np.int32)
    A = normal_bf16(rng, (total, M))             # [K][M] per group, rows packed
    Bm = normal_bf16(rng, (total, N), 0.1)       # [K][N]
    acc0 = normal_bf16(rng, (G, N, M))
    d_A, d_B, d_cum, d_D = be.upload(A), be.upload(Bm), be.upload(incl), be.upload(acc0)
    ret = be.lib.dataflow_submit_amd_grouped_matmul(be.hp, CS, BF, BF, BF, BF, B.DATAFLOW_FP32, 0, 1, B.AMD_GROUPED_RAGGED_K, M, 0, N, G, d_cum.ptr,
                                                    1.0, 1.0, d_A.ptr, 0, d_B.ptr, d_D.ptr, d_D.ptr, N * M * 2)
    assert ret == 0
    be.sync(CS)
    got = be.read(d_D.ptr, (G, N, M), np.uint16)
    for g in range(G):
        lo, hi = int(incl[g] - counts[g]), int(incl[g])
        if hi == lo:
            assert (got[g] == acc0[g]).all()                 # empty group leaves the accumulator untouched
        else:
            want = O.matmul(oracle, 0, 1, M, hi - lo, N, np.ascontiguousarray(A[lo:hi]), np.ascontiguousarray(Bm[lo:hi]), 1.0, 1.0, acc0[g])
            check_matmul(got[g], want, hi - lo)


def test_submit_errors_are_reported(backend):
    be = backend
    d = be.alloc(4096)
    # stream id out of range (cuda_dataflow_handle.c:369-373)
    assert be.lib.dataflow_submit_default_swiglu(be.hp, 99, BF, 1, 8, d.ptr, d.ptr, d.ptr) == -1
    # unregistered dtype combination (cuda_dataflow_handle.c:385-388)
    assert be.lib.dataflow_submit_default_swiglu(be.hp, CS, B.DATAFLOW_FP8E4M3, 1, 8, d.ptr, d.ptr, d.ptr) == -1
    # row length not a multiple of 8
    assert be.lib.dataflow_submit_default_swiglu(be.hp, CS, BF, 1, 12, d.ptr, d.ptr, d.ptr) == -1
    assert be.num_ops == 31                                      # 3 external (matmul, grouped matmul and its gathered form) + 28 native
    be.sync()


def test_diagnostic_probes_run_and_reject_bad_arguments(backend, capfd):
    """The two diagnostic kernels of libamd_matmul_diag.so (MFMA rate, the streaming GEMM's skeleton) launch, finish and leave the
    source untouched; argument combinations they do not implement are refused before any launch."""
    import os
    be = backend
    mm = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul_diag.so"))
    mm.amd_matmul_mfma_probe.restype = C.c_int
    mm.amd_matmul_mfma_probe.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_uint64)]
    mm.amd_matmul_stream_probe.restype = C.c_int
    mm.amd_matmul_stream_probe.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    hp = C.cast(be.hp, C.c_void_p)
    nbytes = 64 << 20
    pattern = np.arange(nbytes // 4, dtype=np.uint32)
    src, word, flops = be.upload(pattern), be.alloc(4096), C.c_uint64()
    be.zero(word.ptr, 4096, CS)
    for mode in range(8):
        print("case mfma probe mode %d" % mode, flush=True)
        assert mm.amd_matmul_mfma_probe(hp, CS, 4, mode, word.ptr, C.byref(flops)) == 0
        assert flops.value > 0
    NO_LOADS, NO_MFMAS, TOUCH, VIA_REGS, PER_GROUP_CLOCKS, ALL_WAVES = 1, 2, 4, 8, 1024, 2048
    for share, slack, flags in ((0, 1, 0), (4, 1, 0), (4, 2, 0), (4, 0, 0), (32, 1, NO_MFMAS), (8, 1, NO_LOADS), (4, 1, TOUCH), (2, 1, TOUCH | NO_MFMAS), (1, 2, 0),
                               (4, 2, VIA_REGS), (8, 2, VIA_REGS | NO_MFMAS),
                               (4, 1, 2 << 4), (8, 0, (63 << 4) | NO_MFMAS), (4, 1, ALL_WAVES), (1, 0, ALL_WAVES | NO_MFMAS)):   # sharers out of step; all waves load
        print("case stream probe share %d slack %d flags %d" % (share, slack, flags), flush=True)
        assert mm.amd_matmul_stream_probe(hp, CS, src.ptr, nbytes, share, slack, flags, 2, word.ptr) == 0
    be.sync(CS)
    assert (be.read(src.ptr, (nbytes // 4,), np.uint32) == pattern).all()
    assert (be.read(word.ptr, (1024,), np.uint32) == 0).all()
    # with per-group clocks every work-group leaves its run time behind the first word
    assert mm.amd_matmul_stream_probe(hp, CS, src.ptr, nbytes, 4, 1, PER_GROUP_CLOCKS | (1 << 4), 2, word.ptr) == 0
    be.sync(CS)
    ticks = be.read(word.ptr, (257,), np.float32)
    assert ticks[0] == 0 and (ticks[1:] > 0).all()
    capfd.readouterr()
    for share, slack, flags, passes, size in ((3, 1, 0, 1, nbytes), (4, 3, 0, 1, nbytes), (4, 1, 4096, 1, nbytes), (4, 2, VIA_REGS | (1 << 4), 1, nbytes), (4, 1, TOUCH | ALL_WAVES, 1, nbytes),
                                              (4, 2, ALL_WAVES, 1, nbytes), (4, 1, VIA_REGS, 1, nbytes), (4, 2, VIA_REGS | TOUCH, 1, nbytes), (4, 1, 0, 0, nbytes), (4, 1, 0, 1, 1 << 20),
                                              (4, 2, TOUCH, 1, nbytes), (4, 1, TOUCH | NO_LOADS, 1, nbytes), (4, 1, NO_LOADS | NO_MFMAS, 1, nbytes)):
        assert mm.amd_matmul_stream_probe(hp, CS, src.ptr, size, share, slack, flags, passes, word.ptr) == -1
    assert "stream probe" in capfd.readouterr().err
    assert mm.amd_matmul_mfma_probe(hp, CS, 0, 0, word.ptr, C.byref(flops)) == -1
    for buf in (src, word):
        buf.free()
