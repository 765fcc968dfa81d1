"""GPU parity of the whole MoE layer (amd_moe_layer_forward / _backward through the C ABI) against the
oracle's restatement of the reference op sequence, for both schedules, plus size-independent properties
at the full benchmark shapes.

Routing is compared bit-exactly by letting the oracle replay the GPU's own bf16 router logits (the two
router products may differ by one rounding, which can legitimately flip a near-tie); the logits themselves
are compared within 1 bf16 ulp.  Values (util.close): every element within 1e-2 of the tensor's scale, within 2 bf16
steps of (its own magnitude + 2 rms), and every element of at least rms magnitude within 2 bf16 steps of the oracle's.
"""
import ctypes as C
import os

import numpy as np
import pytest

import oracle_lib as O
from ml_dataflow_amd import MoeLayer, binding as B
from util import f32_to_bf16, bf16_to_f64, normal_bf16, bf16_ulp_diff, zipf_bias, close, SKEWED_ROUTING_BIAS_SCALE

pytestmark = pytest.mark.gpu

# element-wise bar (bf16 steps) of the fused schedule's router-logit gradient against the oracle's at the benchmark sizes
FUSED_ROUTER_STEPS_AT_SIZE = 24


def make_weights(rng, D, E, H, std=0.02):
    return (normal_bf16(rng, (E, D), std), normal_bf16(rng, (E, H, D), std), normal_bf16(rng, (E, H, D), std),
            normal_bf16(rng, (E, D, H), std))


def run_case(be, oracle, T, D, E, K, H, schedule, seed, bias_scale=None, backward=True, wstd=0.02, fused_router_steps=4):
    rng = np.random.default_rng(seed)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H, wstd)
    X = normal_bf16(rng, (T, D))
    resid = normal_bf16(rng, (T, D))
    dY = normal_bf16(rng, (T, D))
    bias = None
    if bias_scale is not None:
        bias = f32_to_bf16(np.broadcast_to(zipf_bias(rng, E, bias_scale), (T, E)).copy())

    layer = MoeLayer(be, T, D, E, K, H)
    layer.load_weights(Wr, W1, W3, W2)
    d_X, d_out, d_dY, d_dX = be.upload(X), be.upload(resid), be.upload(dY), be.alloc(T * D * 2)
    d_bias = be.upload(bias) if bias is not None else None
    layer.forward(T, d_X.ptr, d_out.ptr, d_bias.ptr if d_bias else None, schedule)
    be.sync()
    L = layer.L
    R = T * K
    g = {
        "logits": be.read(L.x_routed, (T, E), np.uint16), "weights": be.read(L.token_expert_weights, (T, K), np.float32),
        "chosen": be.read(L.chosen_experts, (T, K), np.uint16), "counts": be.read(L.expert_counts, (E + 1,), np.int32),
        "cumsum": be.read(L.expert_counts_cumsum, (E,), np.int32), "emap": be.read(L.expert_mapping, (R,), np.int32),
        "tmap": be.read(L.token_mapping, (T, K), np.int32), "out": be.read(d_out.ptr, (T, D), np.uint16),
        "host_counts": np.ctypeslib.as_array(C.cast(L.host_expert_counts, C.POINTER(C.c_int32)), (E,)).copy(),
    }

    g["x1"], g["x3"] = layer.read_up_projections(T)
    ol = O.Layer(oracle, T, D, E, K, H, Wr, W1, W3, W2)
    own = ol.forward(X, resid, logit_bias=bias)                    # oracle's own logits
    assert bf16_ulp_diff(g["logits"], ol.logits).max() <= 1
    out_o = ol.forward(X, resid, logits=g["logits"])               # replay routing on the GPU's logits
    # integer state: bit-exact
    assert (g["chosen"] == ol.chosen).all()
    assert (g["counts"][:E] == ol.counts[:E]).all() and (g["host_counts"] == ol.counts[:E]).all()
    assert (g["cumsum"] == ol.cumsum).all()
    assert (g["emap"] == ol.expert_mapping).all() and (g["tmap"] == ol.token_mapping).all()
    np.testing.assert_allclose(g["weights"], ol.weights, rtol=2e-6, atol=1e-9)
    close(g["x1"], ol.x1, what="x1")
    close(g["x3"], ol.x3, what="x3")
    close(g["out"], out_o, what="out")

    if backward:
        layer.zero_grads()
        layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
        be.sync()
        dX_o = ol.backward(X, dY)
        dWr, dW1, dW3, dW2 = layer.read_grads()
        # The fused schedule forms the router gradient as <h, dh> / w where the oracle (the reference's order) forms
        # <y, dY>: equal in exact arithmetic, each with its own rounded intermediates (dh and y), so what follows from the
        # router gradient sits further from the oracle than a computation in the oracle's own order: up to 4 steps seen.
        # Neither is the more accurate one: fused_router_gradient_is_as_accurate() compares both with the exact value.
        rs = fused_router_steps if schedule == B.AMD_MOE_FUSED else 2
        close(be.read(d_dX.ptr, (T, D), np.uint16), dX_o, steps=rs, what="dX")
        dx1, dx3 = layer.read_up_projections(T, grads=True)
        close(dx1, ol.dx1, what="dx1")
        close(dx3, ol.dx3, what="dx3")
        close(be.read(L.d_routed, (T, E), np.uint16), ol.dlogits, steps=rs, what="d_routed")
        close(dWr, ol.dWr, steps=rs, what="dWr")
        close(dW1, ol.dW1, what="dW1")
        close(dW3, ol.dW3, what="dW3")
        close(dW2, ol.dW2, what="dW2")
        if schedule == B.AMD_MOE_FUSED:
            fused_router_gradient_is_as_accurate(be.read(L.d_routed, (T, E), np.uint16), ol, W2, dY)
    layer.free()
    return g


def fused_router_gradient_is_as_accurate(d_routed_bits, ol, W2, dY):
    """The router-logit gradient in fp64 from the saved bf16 activations (h = silu(x1) x3, y = h W2^T, d = <y, dY>, then
    the softmax-gate backward d_k <- p_k (d_k - sum_j p_j d_j)), against which the fused schedule's <h, dh> / w must not
    be further off than the oracle's reference-order <bf16(y), dY> is (both carry the rounding of one bf16 intermediate)."""
    f = bf16_to_f64
    T, K, E = ol.T, ol.K, ol.E
    x1, x3 = f(ol.x1), f(ol.x3)
    h = x1 / (1.0 + np.exp(-x1)) * x3
    d = np.zeros((T, K))
    g = f(dY)
    chosen = ol.chosen.astype(np.int64)
    for e in range(E):
        n = int(ol.counts[e])
        rows = np.arange(int(ol.cumsum[e]) - n, int(ol.cumsum[e]))
        if n == 0:
            continue
        tok = ol.expert_mapping[rows]
        val = ((h[rows] @ f(W2[e]).T) * g[tok]).sum(axis=1)
        slot = (chosen[tok] == e).argmax(axis=1)
        d[tok, slot] = val
    p = ol.weights.astype(np.float64)
    exact = p * (d - (p * d).sum(axis=1, keepdims=True))
    cols = (np.repeat(np.arange(T), K), chosen.reshape(-1))
    err_fused = f(d_routed_bits)[cols] - exact.reshape(-1)
    err_oracle = f(ol.dlogits)[cols] - exact.reshape(-1)
    rms = lambda v: float(np.sqrt(np.mean(v * v)))
    assert rms(err_fused) <= 1.25 * rms(err_oracle) + 1e-30, (rms(err_fused), rms(err_oracle))
    assert np.abs(err_fused).max() <= 2.0 * np.abs(err_oracle).max() + 1e-30


# config 1 of the benchmark list (the tiny CPU-runnable case) and smaller ragged ones, both schedules
@pytest.mark.parametrize("schedule", [B.AMD_MOE_GROUPED, B.AMD_MOE_PER_EXPERT, B.AMD_MOE_FUSED])
@pytest.mark.parametrize("T,D,E,K,H", [(256, 512, 8, 2, 1024), (100, 64, 8, 2, 128), (333, 256, 16, 4, 200), (64, 128, 64, 8, 64),
                                       # H * D * 2 bytes not a multiple of 256: w1 and w3 of an expert do not lie back to back, and the
                                       # fused schedule takes its branch with two up-projections and separate x1 / x3
                                       (200, 72, 4, 2, 24)])
def test_layer_forward_backward_parity(backend, oracle, schedule, T, D, E, K, H):
    print("case layer T=%d D=%d E=%d K=%d H=%d schedule=%d" % (T, D, E, K, H, schedule), flush=True)
    run_case(backend, oracle, T, D, E, K, H, schedule, seed=T + D + E + K + H)


def test_layer_with_skewed_routing_and_empty_experts(backend, oracle):
    # strong Zipf bias: most experts get nothing, one gets nearly everything
    g = run_case(backend, oracle, 512, 256, 32, 4, 264, B.AMD_MOE_GROUPED, seed=77, bias_scale=40.0)
    assert (g["counts"][:32] == 0).any() and g["counts"][:32].max() >= 512
    run_case(backend, oracle, 512, 256, 32, 4, 264, B.AMD_MOE_PER_EXPERT, seed=77, bias_scale=40.0)
    # With one routing weight close to 1 the softmax-gate backward p_k (d_k - sum_j p_j d_j) subtracts nearly equal numbers,
    # which amplifies the rounding of the router gradient d in the oracle's order and in the fused schedule's alike: the
    # step bar against the oracle is widened here, the comparison of both with the exact value (run_case) is not.
    run_case(backend, oracle, 512, 256, 32, 4, 264, B.AMD_MOE_FUSED, seed=77, bias_scale=40.0, fused_router_steps=16)


def test_layer_single_token(backend, oracle):
    run_case(backend, oracle, 1, 64, 4, 2, 64, B.AMD_MOE_GROUPED, seed=3)
    run_case(backend, oracle, 1, 64, 4, 2, 64, B.AMD_MOE_PER_EXPERT, seed=3)
    run_case(backend, oracle, 1, 64, 4, 2, 64, B.AMD_MOE_FUSED, seed=3)


@pytest.mark.parametrize("T,D,E,K,H", [(1024, 512, 16, 4, 384),      # every GEMM in the small-tile kernels
                                       (4096, 1024, 8, 4, 512),       # grouped launches in the persistent kernel (256- and 288-row tiles)
                                       (600, 72, 4, 2, 24)])          # w1 / w3 not back to back: the fused schedule's unstacked branch
def test_schedules_agree_bit_for_bit(backend, T, D, E, K, H):
    """every element is accumulated over k in the same order whatever kernel and tile computes it -> identical bits,
    forward and backward, for the per-expert and the grouped schedule; the fused schedule shares the forward and every
    expert-side gradient bit for bit and differs only in what follows from the router gradient (dWr, the router's share
    of dX), which it forms from <h, dh> / w"""
    be = backend
    rng = np.random.default_rng(9)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H)
    X, resid, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    results = []
    for schedule in (B.AMD_MOE_GROUPED, B.AMD_MOE_PER_EXPERT, B.AMD_MOE_FUSED):
        layer = MoeLayer(be, T, D, E, K, H)
        layer.load_weights(Wr, W1, W3, W2)
        d_X, d_out, d_dY, d_dX = be.upload(X), be.upload(resid), be.upload(dY), be.alloc(T * D * 2)
        layer.forward(T, d_X.ptr, d_out.ptr, None, schedule)
        layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
        be.sync()
        L, R = layer.L, T * K
        results.append((be.read(d_out.ptr, (T, D), np.uint16),) + layer.read_up_projections(T) + layer.read_up_projections(T, grads=True)
                       + layer.read_grads()[1:] + (be.read(d_dX.ptr, (T, D), np.uint16), layer.read_grads()[0], be.read(L.d_routed, (T, E), np.uint16)))
        layer.free()
    grouped, per_expert, fused = results
    for a, b in zip(grouped, per_expert):
        assert (a == b).all()
    for a, b in zip(grouped[:8], fused[:8]):                       # out, x1, x3, dx1, dx3, dW1, dW3, dW2
        assert (a == b).all()
    for name, a, b in zip(("dX", "dWr", "d_routed"), grouped[8:], fused[8:]):
        # two roundings of the same exact value (run_case compares each with it); the sums over tokens / experts that
        # give dWr and dX average the difference out again
        # (the larger case sums over more experts per token row and more tokens: a wider bar, as at full size)
        close(b, a, steps=(8 if name == "d_routed" else 4) * (1 if T <= 1024 else 2), what=name)


@pytest.mark.parametrize("T,D,E,K,H", [(1024, 512, 16, 4, 384), (4096, 1024, 8, 4, 512)])
def test_fused_schedule_without_gathered_loads_gives_the_same_bits(backend, T, D, E, K, H):
    """The stacked GEMMs of the fused schedule either fetch the rows of X through expert_mapping in their own loaders or run
    on a dispatched copy (the up-projection for an X of 4 GiB and more, the dW1 | dW3 GEMM by default); AMD_MOE_BWD_GATHER
    makes the backward gather too, AMD_MOE_NO_GATHER forces the copy everywhere.  Same values into the same multiplies:
    every output and gradient agrees bit for bit."""
    be = backend
    rng = np.random.default_rng(31)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H)
    X, resid, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    runs = []
    for packed in (False, True):
        os.environ["AMD_MOE_NO_GATHER" if packed else "AMD_MOE_BWD_GATHER"] = "1"
        try:
            layer = MoeLayer(be, T, D, E, K, H)
            layer.load_weights(Wr, W1, W3, W2)
            d_X, d_out, d_dY, d_dX = be.upload(X), be.upload(resid), be.upload(dY), be.alloc(T * D * 2)
            layer.forward(T, d_X.ptr, d_out.ptr, None, B.AMD_MOE_FUSED)
            layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, B.AMD_MOE_FUSED)
            be.sync()
        finally:
            os.environ.pop("AMD_MOE_NO_GATHER", None)
            os.environ.pop("AMD_MOE_BWD_GATHER", None)
        runs.append((be.read(d_out.ptr, (T, D), np.uint16), be.read(d_dX.ptr, (T, D), np.uint16), be.read(layer.L.d_routed, (T, E), np.uint16))
                    + layer.read_up_projections(T) + layer.read_up_projections(T, grads=True) + tuple(layer.read_grads()))
        layer.free()
        for d in (d_X, d_out, d_dY, d_dX):
            d.free()
    for i, (a, b) in enumerate(zip(*runs)):
        assert (a == b).all(), "output %d differs between the gathered and the packed form" % i


@pytest.mark.parametrize("schedule", [B.AMD_MOE_FUSED, B.AMD_MOE_GROUPED])
def test_two_runs_give_the_same_bits(backend, schedule):
    """nothing in the path depends on the order in which work-groups run: the rows of an expert are in token order
    (stable counting sort, no atomics on positions), every sum has a fixed order, the persistent GEMMs deal their tiles
    statically -> two runs over the same inputs agree bit for bit in every output and every saved mapping"""
    be = backend
    T, D, E, K, H = 4096, 1024, 8, 4, 512
    rng = np.random.default_rng(123)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H)
    X, resid, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    runs = []
    for _ in range(2):
        layer = MoeLayer(be, T, D, E, K, H)
        layer.load_weights(Wr, W1, W3, W2)
        d_X, d_out, d_dY, d_dX = be.upload(X), be.upload(resid), be.upload(dY), be.alloc(T * D * 2)
        layer.forward(T, d_X.ptr, d_out.ptr, None, schedule)
        layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
        be.sync()
        L = layer.L
        runs.append((be.read(d_out.ptr, (T, D), np.uint16), be.read(d_dX.ptr, (T, D), np.uint16), be.read(L.d_routed, (T, E), np.uint16),
                     be.read(L.chosen_experts, (T, K), np.uint16), be.read(L.expert_mapping, (T * K,), np.int32),
                     be.read(L.token_mapping, (T, K), np.int32), be.read(L.expert_counts_cumsum, (E,), np.int32)) + tuple(layer.read_grads()))
        layer.free()
        for d in (d_X, d_out, d_dY, d_dX):
            d.free()
    for i, (a, b) in enumerate(zip(*runs)):
        assert (a == b).all(), "output %d differs between two runs" % i


@pytest.mark.parametrize("schedule", [B.AMD_MOE_GROUPED, B.AMD_MOE_PER_EXPERT, B.AMD_MOE_FUSED])
@pytest.mark.parametrize("T,D,E,K,H,bias_scale", [(512, 256, 32, 4, 264, 40.0),       # most experts without tokens: their gradients must become zero
                                                  (600, 72, 4, 2, 24, None),          # w1 / w3 not back to back
                                                  (4096, 1024, 8, 4, 512, None)])     # the persistent kernels
def test_first_micro_batch_backward_writes_what_clear_and_accumulate_gives(backend, schedule, T, D, E, K, H, bias_scale):
    """AMD_MOE_FIRST_MICRO_BATCH: the weight-gradient GEMMs run with beta = 0 and no C operand over gradient buffers that hold
    NaN patterns; every gradient equals, bit for bit, what zero_grads() followed by the accumulating backward leaves."""
    print("case first micro-batch schedule=%d T=%d D=%d E=%d K=%d H=%d" % (schedule, T, D, E, K, H), flush=True)
    be = backend
    rng = np.random.default_rng(T + E)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H)
    X, resid, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    bias = None if bias_scale is None else f32_to_bf16(np.broadcast_to(zipf_bias(rng, E, bias_scale), (T, E)).copy())
    layer = MoeLayer(be, T, D, E, K, H)
    layer.load_weights(Wr, W1, W3, W2)
    d_X, d_out, d_dY, d_dX = be.upload(X), be.upload(resid), be.upload(dY), be.alloc(T * D * 2)
    d_bias = be.upload(bias) if bias is not None else None
    layer.forward(T, d_X.ptr, d_out.ptr, d_bias.ptr if d_bias else None, schedule)
    be.sync()
    if bias_scale is not None:
        assert (be.read(layer.L.expert_counts, (E,), np.int32) == 0).any()
    layer.zero_grads()
    layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
    be.sync()
    want = tuple(layer.read_grads()) + (be.read(d_dX.ptr, (T, D), np.uint16),)
    dirty = np.full(layer.L.expert_stride_bytes * E // 2, 0x7FC1, np.uint16)
    be.write(layer.L.dw1, dirty)
    be.write(layer.L.dw_router, dirty[:E * D])
    be.sync()
    layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule, first_micro_batch=True)
    be.sync()
    got = tuple(layer.read_grads()) + (be.read(d_dX.ptr, (T, D), np.uint16),)
    for name, a, b in zip(("dWr", "dW1", "dW3", "dW2", "dX"), got, want):
        assert (a == b).all(), "%s: %d of %d elements differ from clear + accumulate" % (name, int((a != b).sum()), a.size)
    # and a second micro-batch accumulates on top of the first: twice the gradient of one, up to the rounding of the sum
    layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
    be.sync()
    for name, a, b in zip(("dWr", "dW1", "dW3", "dW2"), layer.read_grads(), want):
        close(a, f32_to_bf16(2.0 * bf16_to_f64(b).astype(np.float32)), what="2 x " + name)
    layer.free()
    for d in (d_X, d_out, d_dY, d_dX) + ((d_bias,) if d_bias else ()):
        d.free()


def test_backward_schedule_may_differ_from_the_forward_schedule(backend):
    """A grouped forward never waits for the device; a per-expert backward after it reads the per-expert row
    counts on the host and must wait for them itself.  Two batches of the same size with different routing follow
    each other, so stale counts of the first batch would pass a sum check and give wrong row ranges.  Backward over
    another token count than the forward's is refused."""
    be = backend
    T, D, E, K, H = 2048, 256, 16, 4, 128
    rng = np.random.default_rng(11)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H, std=0.05)
    layer = MoeLayer(be, T, D, E, K, H)
    layer.load_weights(Wr, W1, W3, W2)
    d_out, d_dX = be.alloc(T * D * 2), be.alloc(T * D * 2)
    for batch in range(2):
        X, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
        d_X, d_dY = be.upload(X), be.upload(dY)
        results = []
        for fwd, bwd in ((B.AMD_MOE_GROUPED, B.AMD_MOE_GROUPED), (B.AMD_MOE_GROUPED, B.AMD_MOE_PER_EXPERT), (B.AMD_MOE_PER_EXPERT, B.AMD_MOE_GROUPED)):
            be.zero(d_out.ptr, T * D * 2)
            layer.zero_grads()
            layer.forward(T, d_X.ptr, d_out.ptr, None, fwd)
            layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, bwd)          # no sync in between
            be.sync()
            results.append((be.read(d_dX.ptr, (T, D), np.uint16),) + layer.read_grads())
        for other in results[1:]:
            for a, b in zip(results[0], other):
                assert (a == b).all()
        d_X.free(), d_dY.free()
    assert be.lib.amd_moe_layer_backward(be.hp, 1, 2, C.byref(layer.L), T - 1, None, None, None, B.AMD_MOE_GROUPED) == -1
    # the fused schedule saves x1 | x3 side by side per row: no other schedule's backward can read that, nor the reverse
    assert be.lib.amd_moe_layer_backward(be.hp, 1, 2, C.byref(layer.L), T, None, None, None, B.AMD_MOE_FUSED) == -1
    d_X = be.upload(X)
    layer.forward(T, d_X.ptr, d_out.ptr, None, B.AMD_MOE_FUSED)
    be.sync()
    assert be.lib.amd_moe_layer_backward(be.hp, 1, 2, C.byref(layer.L), T, None, None, None, B.AMD_MOE_GROUPED) == -1
    layer.free()


@pytest.mark.parametrize("name,T,D,E,K,H,bias,schedule", [
    ("config2", 8192, 2048, 32, 4, 1408, None, B.AMD_MOE_GROUPED), ("config2", 8192, 2048, 32, 4, 1408, None, B.AMD_MOE_FUSED),
    ("config3", 8192, 2048, 32, 4, 1408, SKEWED_ROUTING_BIAS_SCALE, B.AMD_MOE_GROUPED), ("config3", 8192, 2048, 32, 4, 1408, SKEWED_ROUTING_BIAS_SCALE, B.AMD_MOE_FUSED),
    ("config4", 8192, 4096, 64, 8, 1024, None, B.AMD_MOE_GROUPED), ("config5", 65536, 4096, 64, 8, 1024, None, B.AMD_MOE_GROUPED)])
def test_full_size_properties(backend, oracle, name, T, D, E, K, H, bias, schedule):
    """At the benchmark shapes the oracle's GEMMs are too slow to replay in full; check what does not depend on
    size: routing replayed exactly by the oracle's integer functions, dispatch as a pure copy, combine against
    the oracle given the GPU's expert outputs, and the expert pipeline on sampled rows, on the complete last tile of
    the most loaded expert and (forward-only workloads; the others have it in the backward test) on the complete
    sub-batch of the tokens routed to the least loaded expert."""
    print("case full-size %s schedule %d" % (name, schedule), flush=True)
    be = backend
    rng = np.random.default_rng(42)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H)
    X = normal_bf16(rng, (T, D))
    resid = np.zeros((T, D), dtype=np.uint16)
    bias_m = None
    if bias is not None:
        # scale chosen so the most loaded expert gets nearly 8 times the mean load (8 times = every token)
        bias_m = f32_to_bf16(np.broadcast_to(zipf_bias(rng, E, bias), (T, E)).copy())
    layer = MoeLayer(be, T, D, E, K, H)
    layer.load_weights(Wr, W1, W3, W2)
    d_X, d_out = be.upload(X), be.upload(resid)
    d_bias = be.upload(bias_m) if bias_m is not None else None
    layer.forward(T, d_X.ptr, d_out.ptr, d_bias.ptr if d_bias else None, schedule)
    be.sync()
    L, R = layer.L, T * K
    logits = be.read(L.x_routed, (T, E), np.uint16)
    chosen = be.read(L.chosen_experts, (T, K), np.uint16)
    w = be.read(L.token_expert_weights, (T, K), np.float32)
    counts = be.read(L.expert_counts, (E + 1,), np.int32)
    cumsum = be.read(L.expert_counts_cumsum, (E,), np.int32)
    emap, tmap = be.read(L.expert_mapping, (R,), np.int32), be.read(L.token_mapping, (T, K), np.int32)
    # routing: the oracle's select/build on the GPU's logits
    w_o, ch_o, counts_o, cum_o, _ = O.select_experts(oracle, logits, K)
    emap_o, tmap_o, incl_o = O.build_expert_mapping(oracle, ch_o, E, cum_o)
    assert (chosen == ch_o).all() and (counts[:E] == counts_o[:E]).all() and (cumsum == incl_o).all()
    assert (emap == emap_o).all() and (tmap == tmap_o).all()
    np.testing.assert_allclose(w, w_o, rtol=2e-6, atol=1e-9)
    if bias is not None:
        assert counts[:E].max() >= 7 * (R // E), "workload is not skewed: max %d mean %d" % (counts[:E].max(), R // E)
    # sampled rows of the expert pipeline against the oracle (rows from the first, the largest and the last expert)
    x1 = layer.read_up_projections(T)[0]
    zones = be.read(L.expert_zones, (R, D), np.uint16)              # expert outputs y (w2 result) after forward
    incl = cumsum
    for e in sorted({0, int(np.argmax(counts[:E])), E - 1}):
        n = int(counts[e])
        if n == 0:
            continue
        rows = np.unique(np.clip(np.array([0, n // 2, n - 1]), 0, n - 1)) + int(incl[e]) - n
        xin = np.ascontiguousarray(X[emap[rows]])
        a = O.matmul(oracle, 1, 0, H, D, len(rows), W1[e], xin)
        b = O.matmul(oracle, 1, 0, H, D, len(rows), W3[e], xin)
        hbuf = np.zeros_like(a)
        oracle.oracle_swiglu(len(rows), H, O.ptr(a), O.ptr(b), O.ptr(hbuf))
        y = O.matmul(oracle, 1, 0, D, H, len(rows), W2[e], hbuf)
        close(x1[rows], a, what="x1 rows")
        close(zones[rows], y, steps=4, what="y rows")   # chained roundings (x1, x3, h) ahead of the last product
    # every row of the last (ragged) 256-row tile of the most loaded expert
    e = int(np.argmax(counts[:E]))
    n = int(counts[e])
    rows = np.arange(((n - 1) // 256) * 256, n) + int(incl[e]) - n
    close(x1[rows], O.matmul(oracle, 1, 0, H, D, len(rows), W1[e], np.ascontiguousarray(X[emap[rows]])), what="x1 last tile")
    if name in ("config2", "config3"):
        # the whole sub-batch of the least loaded expert's tokens through the oracle, on the GPU's logits
        e = int(np.argmin(np.where(counts[:E] > 0, counts[:E], R)))
        tokens = np.nonzero((chosen == e).any(axis=1))[0]
        n = len(tokens)
        assert n == counts[e]
        print("  oracle sub-batch: expert %d, %d tokens" % (e, n), flush=True)
        sub = O.Layer(oracle, n, D, E, K, H, Wr, W1, W3, W2)
        out_o = sub.forward(X[tokens], resid[tokens], logits=logits[tokens])
        assert (sub.chosen == chosen[tokens]).all()
        close(be.read(d_out.ptr, (T, D), np.uint16)[tokens], out_o, steps=3, what="out")
        rows_gpu = slice(int(incl[e]) - n, int(incl[e]))
        rows_sub = slice(int(sub.cumsum[e]) - int(sub.counts[e]), int(sub.cumsum[e]))
        x3 = layer.read_up_projections(T)[1]
        close(x1[rows_gpu], sub.x1[rows_sub], steps=3, what="x1")
        close(x3[rows_gpu], sub.x3[rows_sub], steps=3, what="x3")
        del sub, x3
    # combine, given the GPU's own expert outputs: bit-exact
    want = resid.copy()
    oracle.oracle_merge_experts(T, D, K, O.ptr(zones), O.ptr(tmap), O.ptr(w), O.ptr(want))
    assert (be.read(d_out.ptr, (T, D), np.uint16) == want).all()
    # dispatch round trip: zones re-gathered from X are copies of X rows
    assert be.lib.dataflow_submit_default_prepare_experts(be.hp, 1, B.DATAFLOW_BF16, B.DATAFLOW_BF16, T, D, K, d_X.ptr, L.token_mapping, L.expert_zones) == 0
    be.sync()
    z2 = be.read(L.expert_zones, (R, D), np.uint16)
    assert (z2 == X[emap]).all()
    layer.free()


@pytest.mark.parametrize("name,T,schedule", [("config4", 8192, B.AMD_MOE_GROUPED), ("config4", 8192, B.AMD_MOE_FUSED),
                                             ("config5", 65536, B.AMD_MOE_FUSED), ("config5", 65536, B.AMD_MOE_GROUPED)])
def test_full_size_backward(backend, oracle, name, T, schedule):
    """Backward at the benchmark shapes (D 4096, E 64, K 8, H 1024; T 8192 and T 65536).  Everything a token
    contributes is local to the token (routing, its K expert rows, dX, d logits), and an expert's weight gradients
    depend only on its own rows: so the oracle replays the sub-batch made of ALL tokens routed to the least loaded
    expert (about 1000 tokens at T 8192, about 8000 at T 65536: under a minute of CPU) on the GPU's logits, and must
    reproduce the layer output, dX and the router gradient for those tokens and the complete dW1 / dW3 / dW2 of that
    expert.  The other gradients are covered by what does not depend on size: a second backward pass over the same
    inputs adds the same amount again (accumulation with beta = 1), and a third pass in first-micro-batch mode (beta = 0,
    no C operand) writes the first pass's values over them, bit for bit."""
    print("case full-size backward %s schedule %d" % (name, schedule), flush=True)
    be = backend
    D, E, K, H = 4096, 64, 8, 1024
    rng = np.random.default_rng(4242)
    Wr, W1, W3, W2 = make_weights(rng, D, E, H)
    X, resid, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    layer = MoeLayer(be, T, D, E, K, H)
    layer.load_weights(Wr, W1, W3, W2)
    d_X, d_out, d_dY, d_dX = be.upload(X), be.upload(resid), be.upload(dY), be.alloc(T * D * 2)
    layer.forward(T, d_X.ptr, d_out.ptr, None, schedule)
    layer.zero_grads()
    layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
    be.sync()
    L, R = layer.L, T * K
    logits = be.read(L.x_routed, (T, E), np.uint16)
    chosen = be.read(L.chosen_experts, (T, K), np.uint16)
    counts = be.read(L.expert_counts, (E + 1,), np.int32)[:E]
    incl = be.read(L.expert_counts_cumsum, (E,), np.int32)
    dWr1, dW1_1, dW3_1, dW2_1 = layer.read_grads()

    e = int(np.argmin(np.where(counts > 0, counts, R)))
    tokens = np.nonzero((chosen == e).any(axis=1))[0]              # ascending: the order of the expert's rows
    n = len(tokens)
    assert n == counts[e]
    print("  oracle sub-batch: expert %d, %d tokens" % (e, n), flush=True)
    sub = O.Layer(oracle, n, D, E, K, H, Wr, W1, W3, W2)
    out_o = sub.forward(X[tokens], resid[tokens], logits=logits[tokens])
    dX_o = sub.backward(X[tokens], dY[tokens])
    assert (sub.chosen == chosen[tokens]).all()
    # At this size every value has more rounded terms behind it than in the small cases (dot products over 4096
    # elements whose operands were themselves rounded, sums over K = 8 expert rows rounded once or twice on the way): each
    # such rounding may fall differently under fp32 and fp64 accumulation, and the element-wise bar is 3 steps here.
    close(be.read(d_out.ptr, (T, D), np.uint16)[tokens], out_o, steps=3, what="out")
    # The fused schedule has its own form of the router gradient (see run_case).  The reference keeps that gradient in
    # bf16 ahead of the softmax-gate backward p_k (d_k - sum_j p_j d_j), whose subtraction magnifies the last rounding of
    # d: two equally accurate values of d (compared with the exact one below) then give gate outputs several steps
    # apart, and the router's share of dX inherits that.  7 steps seen at this size.
    # (reference-order schedules: 3 steps over the 4 M elements of the 8192-token sub-batch, 4 over the 32 M elements of
    # the 65536-token one, whose worst element is one step further out)
    rs = 10 if schedule == B.AMD_MOE_FUSED else (3 if T <= 8192 else 4)
    close(be.read(d_dX.ptr, (T, D), np.uint16)[tokens], dX_o, steps=rs, what="dX")
    # the gate output itself is held to the tensor-scale bound and, where the exact value is affordable, to the accuracy
    # of the oracle's own value; the more tokens, the larger the worst magnification
    # (fused: element-wise too, on every entry of at least rms magnitude and with the magnification bounded; 13 steps seen)
    close(be.read(L.d_routed, (T, E), np.uint16)[tokens], sub.dlogits, steps=FUSED_ROUTER_STEPS_AT_SIZE if schedule == B.AMD_MOE_FUSED else rs, what="d_routed")
    if schedule == B.AMD_MOE_FUSED:
        fused_router_gradient_is_as_accurate(be.read(L.d_routed, (T, E), np.uint16)[tokens], sub, W2, dY[tokens])
    rows_gpu = slice(int(incl[e]) - n, int(incl[e]))
    rows_sub = slice(int(sub.cumsum[e]) - int(sub.counts[e]), int(sub.cumsum[e]))
    assert sub.counts[e] == n
    x1, x3 = layer.read_up_projections(T)
    dx1, dx3 = layer.read_up_projections(T, grads=True)
    close(x1[rows_gpu], sub.x1[rows_sub], steps=3, what="x1")
    close(x3[rows_gpu], sub.x3[rows_sub], steps=3, what="x3")
    close(dx1[rows_gpu], sub.dx1[rows_sub], steps=3, what="dx1")
    close(dx3[rows_gpu], sub.dx3[rows_sub], steps=3, what="dx3")
    del x1, x3, dx1, dx3
    close(dW1_1[e], sub.dW1[e], steps=3, what="dW1")
    close(dW3_1[e], sub.dW3[e], steps=3, what="dW3")
    close(dW2_1[e], sub.dW2[e], steps=3, what="dW2")
    del sub

    # accumulation: the same backward again adds the same amount (each sum is rounded to bf16 once more)
    print("  second backward pass", flush=True)
    layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
    be.sync()
    for first, second in zip((dWr1, dW1_1, dW3_1, dW2_1), layer.read_grads()):
        scale, worst = 0.0, 0.0
        flat1, flat2 = first.reshape(-1), second.reshape(-1)
        for lo in range(0, flat1.size, 1 << 26):                  # in pieces: the expert gradients are 268 M elements each
            a, b = bf16_to_f64(flat1[lo:lo + (1 << 26)]), bf16_to_f64(flat2[lo:lo + (1 << 26)])
            worst = max(worst, float(np.abs(b - 2.0 * a).max()))
            scale = max(scale, float(np.abs(a).max()))
        assert worst <= 2.0 ** -6 * scale
    if schedule != B.AMD_MOE_PER_EXPERT:
        # first micro-batch mode at size: over the twice-accumulated buffers it writes what clear + accumulate left the first time
        print("  first-micro-batch backward pass", flush=True)
        layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule, first_micro_batch=True)
        be.sync()
        for name_, first, again in zip(("dWr", "dW1", "dW3", "dW2"), (dWr1, dW1_1, dW3_1, dW2_1), layer.read_grads()):
            assert (first == again).all(), "%s: the first-micro-batch backward differs from clear + accumulate" % name_
    layer.free()
