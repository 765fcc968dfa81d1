#!/usr/bin/env python3
"""Benchmark of the MoE-layer hot path on one MI355X.

A "step" is one forward + backward pass of the layer (amd_moe_layer_forward + amd_moe_layer_backward,
fused schedule unless --schedule says otherwise) over one batch of synthetic tokens already resident in HBM.
Prints ONE JSON line.

  value         whole-layer tokens/s (tokens of the batch / mean step time)
  roofline      the dominant kernel (the grouped bf16 MFMA GEMM kernel function with the largest share of step
                time): algorithmic flops per launch / mean launch duration over its launches, timed with HIP
                events recorded on the compute stream around every launch of an op-by-op replay of the same step
  kernels       the same figure for every kernel class of the step (MFMA-bound GEMMs, HBM-bound movers)
  cpu_baseline  the CPU oracle (a port of the reference's kernels; the reference has no CPU MoE path) timed on
                the host cores on a bounded sample of the same workload (fewer tokens, same D/E/K/H)
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from ml_dataflow_amd.synthetic import normal_bf16 as bf16_normal, f32_to_bf16, zipf_bias, SKEWED_ROUTING_BIAS_SCALE  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E

WORKLOADS = {
    # name: (T, D, E, K, H, backward, zipf bias scale)
    "config2_fwd_8192x2048_e32k4_h1408": (8192, 2048, 32, 4, 1408, False, None),
    "config3_fwd_8192x2048_e32k4_h1408_zipf": (8192, 2048, 32, 4, 1408, False, SKEWED_ROUTING_BIAS_SCALE),
    "config4_fwdbwd_8192x4096_e64k8_h1024": (8192, 4096, 64, 8, 1024, True, None),
    "config5_fwdbwd_65536x4096_e64k8_h1024": (65536, 4096, 64, 8, 1024, True, None),
    "config1_fwd_256x512_e8k2_h1024": (256, 512, 8, 2, 1024, False, None),
}
DEFAULT_WORKLOAD = "config4_fwdbwd_8192x4096_e64k8_h1024"
# diagnostics of what the card sustains (M x K x N of one plain GEMM: the up-projection of all tokens as one problem, a
# square one, the down-projection's shape; matrix instructions alone; and a plain copy of rows x width bf16 through the
# dispatch kernel with the identity mapping, at the size of the 8192-token and of the 65536-token workload's routed rows)
SUSTAINED_WORKLOADS = ["gemm_sustained_1024x4096x32768", "gemm_sustained_8192x8192x8192", "gemm_sustained_4096x1024x65536",
                       "mfma_only_random_operands", "mfma_only_small_operands", "mfma_only_varying_operands",
                       "mfma_only_16x16x32_random_operands", "mfma_only_16x16x32_varying_operands",
                       "hbm_copy_65536x4096", "hbm_copy_524288x4096"]
# the streaming GEMM's skeleton (loads, multiplies, barrier and nothing else: amd_matmul_stream_probe) over a table of
# data temperatures, sharing degrees and waits
STREAM_PROBE_WORKLOAD = "gemm_stream_probe"
# ragged-N grouped GEMMs over a table of group sizes and shapes on the eight-wave kernel (256 x 288 tiles), the four-wave
# kernel (256 x 384) and the library's own choice between them: what the device-side rule is calibrated on
TILING_SWEEP_WORKLOAD = "ragged_n_tiling_sweep"
# mode bits of amd_matmul_mfma_probe (include/amd_matmul_diag.h): 1 random operands, 2 the 16x16x32 instruction, 4 operand
# registers that change from instruction to instruction
MFMA_PROBE_MODES = {"mfma_only_small_operands": 0, "mfma_only_random_operands": 1, "mfma_only_varying_operands": 1 | 4,
                    "mfma_only_16x16x32_random_operands": 1 | 2, "mfma_only_16x16x32_varying_operands": 1 | 2 | 4}
# the same three GEMM shapes through the vendor's library (torch.matmul on bf16 tensors): a yardstick for what this
# card gives a bf16 GEMM of such data, not part of the product
VENDOR_WORKLOADS = ["vendor_gemm_1024x4096x32768", "vendor_gemm_8192x8192x8192", "vendor_gemm_4096x1024x65536"]


class HipEvents:
    """hipEvent timing on the stream the kernels are launched on (plain HIP runtime calls through ctypes)."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.pool = []

    def new(self):
        ev = C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(ev)) == 0
        self.pool.append(ev)
        return ev

    def record(self, ev, stream):
        assert self.hip.hipEventRecord(ev, stream) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return float(ms.value)


def replay_step_with_events(be, layer, T, d_X, d_out, d_dY, d_dX, d_bias, backward, ev, stream, fused, first=False):
    """Submits the grouped (or fused) schedule op by op (same ops, same order as amd_moe_layer_forward/_backward, all
    on the compute stream) with an event pair around every launch; returns [(kernel class, ms)].  first: the weight-gradient
    GEMMs as AMD_MOE_FIRST_MICRO_BATCH runs them (beta = 0, no C operand)."""
    from ml_dataflow_amd import binding as B
    lib, hp, L = be.lib, be.hp, layer.L
    D, E, K, H = layer.D, layer.E, layer.K, layer.H
    BF, F32, NONE = B.DATAFLOW_BF16, B.DATAFLOW_FP32, B.DATAFLOW_NONE
    CS = 1
    S = L.expert_stride_bytes
    R = T * K
    cum = L.expert_counts_cumsum
    ws = L.kernel_workspace
    marks = []

    def timed(name, fn, *args):
        a, b = ev.new(), ev.new()
        ev.record(a, stream)
        assert fn(*args) == 0, name
        ev.record(b, stream)
        marks.append((name, a, b))

    def grouped(name, ta, tb, ragged, M, Kd, N, beta, A, sA, Bp, Cp, Dp, sD):
        timed(name, lib.dataflow_submit_amd_grouped_matmul, hp, CS, BF, BF, BF if beta else NONE, BF, F32, ta, tb, ragged, M, Kd, N, E, cum,
              1.0, beta, A, sA, Bp, Cp, Dp, sD)

    wbeta, wdt = (0.0, NONE) if first else (1.0, BF)

    def wc(ptr):
        return None if first else ptr

    bias = d_bias.ptr if d_bias else None
    timed("router_gemm", lib.dataflow_submit_matmul, hp, CS, BF, BF, BF if bias else NONE, BF, F32, 1, 0, E, D, T, 1.0, 1.0 if bias else 0.0,
          L.w_router, d_X.ptr, bias, L.x_routed, L.kernel_workspace_bytes, ws)
    be.zero(L.expert_counts, (E + 1) * 4, CS)
    be.zero(L.expert_counts_cumsum, E * 4, CS)
    timed("select_experts", lib.dataflow_submit_default_select_experts, hp, CS, BF, T, E, K, L.x_routed, L.token_expert_weights, L.chosen_experts,
          L.expert_counts, L.expert_counts_cumsum, L.host_expert_counts)
    timed("build_expert_mapping", lib.dataflow_submit_default_build_expert_mapping, hp, CS, T, E, K, L.chosen_experts, L.expert_counts_cumsum,
          L.expert_mapping, L.token_mapping)
    if fused:
        # no dispatch copy in the fused forward: the up-projection's loaders gather the rows of X through expert_mapping
        timed("gemm_up13", lib.dataflow_submit_amd_grouped_matmul_gathered, hp, CS, BF, BF, NONE, BF, F32, 1, 0, B.AMD_GROUPED_RAGGED_N, 2 * H, D, R, E, cum,
              1.0, 0.0, L.w1, S, d_X.ptr, None, L.x1, 0, L.expert_mapping, T)
        timed("swiglu", lib.dataflow_submit_amd_swiglu_strided, hp, CS, BF, R, H, 2 * H, L.x1, L.x1 + 2 * H, ws)
    else:
        timed("dispatch", lib.dataflow_submit_default_prepare_experts, hp, CS, BF, BF, T, D, K, d_X.ptr, L.token_mapping, L.expert_zones)
        grouped("gemm_tn", 1, 0, B.AMD_GROUPED_RAGGED_N, H, D, R, 0.0, L.w1, S, L.expert_zones, None, L.x1, 0)
        grouped("gemm_tn", 1, 0, B.AMD_GROUPED_RAGGED_N, H, D, R, 0.0, L.w3, S, L.expert_zones, None, L.x3, 0)
        timed("swiglu", lib.dataflow_submit_default_swiglu, hp, CS, BF, R, H, L.x1, L.x3, ws)
    grouped("gemm_tn", 1, 0, B.AMD_GROUPED_RAGGED_N, D, H, R, 0.0, L.w2, S, ws, None, L.expert_zones, 0)
    timed("combine", lib.dataflow_submit_default_merge_experts, hp, CS, BF, BF, T, D, K, L.expert_zones, L.token_mapping, L.token_expert_weights, d_out.ptr)
    if backward:
        be.zero(L.d_routed, T * E * 2, CS)
        if fused:
            timed("dispatch_scaled", lib.dataflow_submit_amd_prepare_experts_scaled, hp, CS, BF, BF, T, D, K, d_dY.ptr, L.token_mapping,
                  L.token_expert_weights, L.expert_zones)
            dh = ws + L.kernel_workspace_bytes // 2
            grouped("gemm_nn", 0, 0, B.AMD_GROUPED_RAGGED_N, H, D, R, 0.0, L.w2, S, L.expert_zones, None, dh, 0)
            timed("swiglu_bwd_x_routed", lib.dataflow_submit_amd_swiglu_bwd_x_routed, hp, CS, BF, BF, R, H, E, K, 2 * H, 2 * H, L.expert_mapping,
                  L.token_mapping, L.chosen_experts, L.token_expert_weights, L.x1, L.x1 + 2 * H, dh, L.d_routed, L.dx1, L.dx1 + 2 * H, ws)
            grouped("gemm_nt_dw", 0, 1, B.AMD_GROUPED_RAGGED_K, H, 0, D, wbeta, ws, 0, L.expert_zones, wc(L.dw2), L.dw2, S)
            grouped("gemm_dx13", 0, 0, B.AMD_GROUPED_RAGGED_N, D, 2 * H, R, 0.0, L.w1, S, L.dx1, None, L.expert_zones, 0)
        else:
            timed("swiglu", lib.dataflow_submit_default_swiglu, hp, CS, BF, R, H, L.x1, L.x3, ws)
            grouped("gemm_tn", 1, 0, B.AMD_GROUPED_RAGGED_N, D, H, R, 0.0, L.w2, S, ws, None, L.expert_zones, 0)
            timed("router_bwd_x", lib.dataflow_submit_amd_router_bwd_x_all, hp, CS, BF, BF, T, D, E, K, L.token_mapping, L.chosen_experts,
                  L.token_expert_weights, L.expert_zones, d_dY.ptr, L.d_routed, L.expert_zones)
            grouped("gemm_nt_dw", 0, 1, B.AMD_GROUPED_RAGGED_K, H, 0, D, wbeta, ws, 0, L.expert_zones, wc(L.dw2), L.dw2, S)
            grouped("gemm_nn", 0, 0, B.AMD_GROUPED_RAGGED_N, H, D, R, 0.0, L.w2, S, L.expert_zones, None, L.dx1, 0)
            timed("swiglu_bwd_x", lib.dataflow_submit_default_swiglu_bwd_x, hp, CS, BF, BF, R, H, L.x1, L.x3, L.dx1, L.dx1, L.dx3)
            grouped("gemm_nn", 0, 0, B.AMD_GROUPED_RAGGED_N, D, H, R, 0.0, L.w1, S, L.dx1, None, L.expert_zones, 0)
            grouped("gemm_nn", 0, 0, B.AMD_GROUPED_RAGGED_N, D, H, R, 1.0, L.w3, S, L.dx3, L.expert_zones, L.expert_zones, 0)
        if fused:
            timed("combine_grad", lib.dataflow_submit_amd_merge_experts_fresh, hp, CS, BF, BF, T, D, K, L.expert_zones, L.token_mapping, None, d_dX.ptr)
        else:
            be.zero(d_dX.ptr, T * D * 2, CS)
            timed("combine_grad", lib.dataflow_submit_default_merge_experts, hp, CS, BF, BF, T, D, K, L.expert_zones, L.token_mapping, None, d_dX.ptr)
        timed("router_gate_bwd_x", lib.dataflow_submit_router_gate_bwd_x, hp, CS, BF, BF, T, E, K, L.chosen_experts, L.token_expert_weights, L.d_routed)
        timed("router_gemm", lib.dataflow_submit_matmul, hp, CS, BF, BF, BF, BF, F32, 0, 0, D, E, T, 1.0, 1.0, L.w_router, L.d_routed, d_dX.ptr, d_dX.ptr,
              L.kernel_workspace_bytes, ws)
        timed("dispatch", lib.dataflow_submit_default_prepare_experts, hp, CS, BF, BF, T, D, K, d_X.ptr, L.token_mapping, L.expert_zones)
        if fused:
            timed("gemm_dw13", lib.dataflow_submit_amd_grouped_matmul, hp, CS, BF, BF, wdt, BF, F32, 0, 1, B.AMD_GROUPED_RAGGED_K, D, 0, 2 * H, E, cum,
                  1.0, wbeta, L.expert_zones, 0, L.dx1, wc(L.dw1), L.dw1, S)
        else:
            grouped("gemm_nt_dw", 0, 1, B.AMD_GROUPED_RAGGED_K, D, 0, H, wbeta, L.expert_zones, 0, L.dx1, wc(L.dw1), L.dw1, S)
            grouped("gemm_nt_dw", 0, 1, B.AMD_GROUPED_RAGGED_K, D, 0, H, wbeta, L.expert_zones, 0, L.dx3, wc(L.dw3), L.dw3, S)
        timed("router_gemm", lib.dataflow_submit_matmul, hp, CS, BF, BF, wdt, BF, F32, 0, 1, D, T, E, 1.0, wbeta, d_X.ptr, L.d_routed, wc(L.dw_router), L.dw_router,
              L.kernel_workspace_bytes, ws)
    be.sync(CS)
    return [(name, ev.elapsed_ms(a, b)) for name, a, b in marks]


# HBM bytes per launch (average over the launches of a class) from two hardware counter runs of this script with
# --calibration-copy (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE), each scaled by what the counter reads for the
# calibration copy of known size (fetch x1.985, write x1.000).  Only valid for the workload and the schedule (fused) they were taken on.
TRAFFIC_SOURCE = ("profiles/moe_layer_%s_hbm_traffic.md: hardware counters of two separate runs of this script, not of this run")
MEASURED_TRAFFIC_BYTES = {
    "config4_fwdbwd_8192x4096_e64k8_h1024": {
        "gemm_up13": 2589760385, "gemm_tn": 1458409166, "gemm_nn": 1540948489, "gemm_nt_dw": 1862856075, "gemm_dx13": 2281766452,
        "gemm_dw13": 3738749644, "dispatch_scaled": 605606034, "swiglu": 400721551, "swiglu_bwd_x_routed": 822827377, "combine": 668834607,
        "combine_grad": 601168066, "dispatch": 604555665,
    },
    "config5_fwdbwd_65536x4096_e64k8_h1024": {
        "gemm_up13": 21330367076, "gemm_tn": 12462374745, "gemm_nn": 9885439367, "gemm_nt_dw": 9458770557, "gemm_dx13": 33712088322,
        "gemm_dw13": 18547757374, "dispatch_scaled": 4844596105, "swiglu": 3205532585, "swiglu_bwd_x_routed": 6617731110, "combine": 5350080114,
        "combine_grad": 4808782033, "dispatch": 4836259094,
    },
}


# kernel function behind each GEMM launch class of the fused schedule, for launches large enough for the persistent kernel
# (libamd_matmul.so's dispatch: ragged-N launches without a C operand walk the token rows in tiles of 288)
_STREAM = "gemm_bf16_stream_kernel<256, %d, 4, 2, %s>"
_W4 = "gemm_bf16_w4_kernel<%s>"
_W4D = "gemm_bf16_w4d_kernel<%s>"
FUSED_GEMM_KERNEL_OF_CLASS = {
    "gemm_up13": _STREAM % (288, "false, false, 1, 1"), "gemm_tn": _STREAM % (288, "false, false, 1, 0"),
    "gemm_nn": _STREAM % (288, "true, false, 1, 0"), "gemm_dx13": _STREAM % (288, "true, false, 1, 0"),
    "gemm_nt_dw": _STREAM % (256, "true, true, 2, 0"), "gemm_dw13": _STREAM % (256, "true, true, 2, 0"),
}


def norm_kernels_with_events(be, T, D, d_X, d_dY, d_dX, ev, stream, backward):
    """The RMS norm that feeds the layer and its backward passes (the calls of dataflow_transformer.c:2567, 3726, 3749),
    each between an event pair; returns [(kernel class, ms)].  rms_norm_bwd_w covers both of its kernels."""
    from ml_dataflow_amd import binding as B
    lib, hp, BF, CS = be.lib, be.hp, B.DATAFLOW_BF16, 1
    w = be.upload(np.full(D, 0x3F80, dtype=np.uint16))
    rms, normed, dw = be.alloc(T * 4), be.alloc(T * D * 2), be.alloc(D * 2)
    ws_bytes = 256 + 512 * D * 4
    ws = be.alloc(ws_bytes)
    be.zero(dw.ptr, D * 2, CS)
    marks = []

    def timed(name, fn, *args):
        a, b = ev.new(), ev.new()
        ev.record(a, stream)
        assert fn(*args) == 0, name
        ev.record(b, stream)
        marks.append((name, a, b))

    timed("rms_norm", lib.dataflow_submit_default_rms_norm, hp, CS, BF, T, D, 1e-5, w.ptr, d_X.ptr, normed.ptr, rms.ptr)
    if backward:
        timed("rms_norm_bwd_x", lib.dataflow_submit_default_rms_norm_bwd_x, hp, CS, BF, BF, T, D, 1e-5, rms.ptr, w.ptr, d_X.ptr, d_dY.ptr,
              d_dX.ptr, normed.ptr)
        timed("rms_norm_bwd_w", lib.dataflow_submit_default_rms_norm_bwd_w, hp, CS, BF, BF, T, D, 1e-5, rms.ptr, d_X.ptr, d_dY.ptr, dw.ptr,
              ws_bytes, ws.ptr)
    be.sync(CS)
    out = [(name, ev.elapsed_ms(a, b)) for name, a, b in marks]
    for buf in (w, rms, normed, dw, ws):
        buf.free()
    return out


def adamw_with_events(be, layer, ev, stream):
    """One AdamW step over all expert weights of the layer (the call of test/dataflow_models/transformer_moe.c:4736 for
    this layer's share of the parameters), moments in freshly zeroed buffers; returns [(kernel class, ms)]."""
    from ml_dataflow_amd import binding as B
    L, BF, CS = layer.L, B.DATAFLOW_BF16, 1
    n = layer.E * (L.expert_stride_bytes // 2)
    mean, var = be.alloc(n * 2), be.alloc(n * 2)
    be.zero(mean.ptr, n * 2, CS)
    be.zero(var.ptr, n * 2, CS)
    a, b = ev.new(), ev.new()
    ev.record(a, stream)
    assert be.lib.dataflow_submit_default_adamw_step(be.hp, CS, BF, BF, BF, BF, n, 1, 0.0, 0.9, 0.999, 0.0, 1e-8, L.w1, L.dw1, mean.ptr, var.ptr) == 0
    ev.record(b, stream)
    be.sync(CS)
    ms = ev.elapsed_ms(a, b)
    mean.free()
    var.free()
    return [("adamw_step", ms)]


def algorithmic_work(T, D, E, K, H, fused):
    """per-launch algorithmic flops (GEMMs) or HBM bytes (movers), the figures the roofline fractions use"""
    R = T * K
    return {
        "gemm_tn": ("mfma", 2.0 * R * D * H), "gemm_nn": ("mfma", 2.0 * R * D * H), "gemm_nt_dw": ("mfma", 2.0 * R * D * H),
        # the fused schedule's launches over the stacked w1 | w3 matrices do the work of two
        "gemm_up13": ("mfma", 4.0 * R * D * H), "gemm_dx13": ("mfma", 4.0 * R * D * H), "gemm_dw13": ("mfma", 4.0 * R * D * H),
        "router_gemm": ("hbm", 2.0 * T * D + 2.0 * E * D + 2.0 * T * E),
        "dispatch": ("hbm", 2.0 * T * D + 4.0 * T * K + 2.0 * R * D), "dispatch_scaled": ("hbm", 2.0 * T * D + 8.0 * T * K + 2.0 * R * D),
        "combine": ("hbm", 2.0 * R * D + 4.0 * T * D + 8.0 * T * K),
        "combine_grad": ("hbm", 2.0 * R * D + (2.0 if fused else 4.0) * T * D + 4.0 * T * K),
        "swiglu": ("hbm", 6.0 * R * H), "swiglu_bwd_x": ("hbm", 10.0 * R * H), "swiglu_bwd_x_routed": ("hbm", 12.0 * R * H + 18.0 * R),
        "router_bwd_x": ("hbm", 2.0 * T * D + 4.0 * R * D + 10.0 * R),
        "select_experts": ("hbm", 2.0 * T * E + 6.0 * T * K + 12.0 * E),
        "build_expert_mapping": ("hbm", 10.0 * T * K),
        "router_gate_bwd_x": ("hbm", 10.0 * T * K),
        # RMS norm around the layer (reported beside the layer's kernels, not part of the timed step)
        "rms_norm": ("hbm", 4.0 * T * D + 4.0 * T), "rms_norm_bwd_x": ("hbm", 10.0 * T * D),
        "rms_norm_bwd_w": ("hbm", 4.0 * T * D + 8.0 * 512 * D),
        # AdamW over all expert weights (3*E*D*H elements): 8 bytes read, 6 written per element
        "adamw_step": ("hbm", 14.0 * 3.0 * E * D * H),
    }


def cpu_baseline(T_sample, D, E, K, H, backward, seed):
    sys.path.insert(0, os.path.join(ROOT, "oracle"))              # the checker's loader; only this leg uses it
    import oracle_lib as O
    oracle = O.load()
    rng = np.random.default_rng(seed)
    Wr = bf16_normal(rng, (E, D), 0.02)
    # the oracle's cost does not depend on the weight values: one expert's matrices are reused for all experts
    W1 = np.broadcast_to(bf16_normal(rng, (1, H, D), 0.02), (E, H, D)).copy()
    W3, W2 = W1.copy(), W1.reshape(E, D, H).copy()
    X, dY = bf16_normal(rng, (T_sample, D), 1.0), bf16_normal(rng, (T_sample, D), 1.0)
    L = O.Layer(oracle, T_sample, D, E, K, H, Wr, W1, W3, W2)
    t0 = time.perf_counter()
    L.forward(X, np.zeros((T_sample, D), dtype=np.uint16))
    if backward:
        L.backward(X, dY)
    dt = time.perf_counter() - t0
    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    return {"value": T_sample / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": "CPU oracle (C restatement of the reference's CUDA kernels, fp64-accumulated GEMMs, OpenMP) on %d of the "
                      "workload's tokens with the same D/E/K/H, %s, %.1f s wall; the reference has no CPU MoE path" %
                      (T_sample, "fwd+bwd" if backward else "fwd", dt)}


def sustained_gemm(args):
    """One GEMM shape launched back to back for a sustained interval (the product's matmul op on one problem), or the
    MFMA-only probe: what the card sustains under its power limit.  Short runs measure the clock governor's
    transients, so the default is 2000 launches; the rate is taken over the second half of them."""
    from ml_dataflow_amd import Backend, binding as B
    be = Backend(0)
    ev, stream = HipEvents(), None
    stream = be.stream(1)
    launches = args.steps if args.steps > 20 else 2000
    BF = B.DATAFLOW_BF16
    moved = None
    if args.workload.startswith("hbm_copy"):
        rows, width = (int(v) for v in args.workload.split("_")[-1].split("x"))
        launches = args.steps if args.steps > 20 else 200
        src, dst = be.alloc(rows * width * 2), be.alloc(rows * width * 2)
        ident = be.upload(np.arange(rows, dtype=np.int32))
        be.zero(src.ptr, rows * width * 2, 1)
        moved = 2 * rows * width * 2 + rows * 4

        def launch():
            assert be.lib.dataflow_submit_default_prepare_experts(be.hp, 1, BF, BF, rows, width, 1, src.ptr, ident.ptr, dst.ptr) == 0
        shape = {"kernel": "default_prepare_experts_bf16_bf16_kernel", "rows": rows, "width": width, "top_k": 1, "mapping": "identity"}
    elif args.workload.startswith("mfma_only"):
        lib = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul_diag.so"))
        lib.amd_matmul_mfma_probe.restype = C.c_int
        lib.amd_matmul_mfma_probe.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_uint64)]
        word, flops = be.alloc(256), C.c_uint64()
        iters = 2048                                   # about 0.5 ms per launch
        mode = MFMA_PROBE_MODES[args.workload]

        def launch():
            assert lib.amd_matmul_mfma_probe(C.cast(be.hp, C.c_void_p), 1, iters, mode, word.ptr, C.byref(flops)) == 0
        shape = {"kernel": "mfma_rate_probe_kernel", "rounds_per_wave": iters, "mode": mode}
    else:
        M, K, N = (int(v) for v in args.workload.split("_")[-1].split("x"))
        rng = np.random.default_rng(42)
        d_A, d_B = be.upload(bf16_normal(rng, (M, K), 0.02)), be.upload(bf16_normal(rng, (N, K), 1.0))
        d_D = be.alloc(N * M * 2)
        flops = C.c_uint64(2 * M * K * N)

        def launch():
            assert be.lib.dataflow_submit_matmul(be.hp, 1, BF, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, 1, 0, M, K, N, 1.0, 0.0,
                                                 d_A.ptr, d_B.ptr, None, d_D.ptr, 0, None) == 0
        shape = {"M": M, "K": K, "N": N, "to_trans_a": 1, "to_trans_b": 0}
    half = launches // 2
    for _ in range(args.warmup):
        launch()
    a, mid, b = ev.new(), ev.new(), ev.new()
    ev.record(a, stream)
    for i in range(launches):
        if i == half:
            ev.record(mid, stream)
        launch()
    ev.record(b, stream)
    be.sync(1)
    first_ms, second_ms = ev.elapsed_ms(a, mid) / half, ev.elapsed_ms(mid, b) / (launches - half)
    if moved is not None:
        gbs = moved / (second_ms * 1e-3) / 1e9
        print(json.dumps({
            "metric": "sustained HBM copy GB/s (%s)" % args.workload, "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
            "steps": launches, "warmup": args.warmup, "ms_per_step": round(second_ms, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic", "config": dict(workload=args.workload, **shape),
            "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None},
            "first_half_ms_per_launch": round(first_ms, 4), "second_half_ms_per_launch": round(second_ms, 4)}))
        be.close()
        return
    tflops = flops.value / (second_ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "sustained bf16 MFMA TFLOP/s (%s)" % args.workload, "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": launches, "warmup": args.warmup, "ms_per_step": round(second_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic", "config": dict(workload=args.workload, **shape),
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": None},
        "first_half_ms_per_launch": round(first_ms, 4), "second_half_ms_per_launch": round(second_ms, 4)}))
    be.close()


def tiling_sweep(args):
    """amd_grouped_matmul (ragged N, no C operand, random bf16 operands) per case on kernel 8, kernel 384 and the default
    choice: three rounds of --steps launches each (8 unless given), alternating, HIP events around each round, the fastest
    round per kernel.  `rule` is what ragged_n_prefers_384 (gemm_kernel.h) picks from the group sizes, restated here."""
    from ml_dataflow_amd import Backend, binding as B
    be = Backend(0)
    ev, stream = HipEvents(), be.stream(1)
    mm = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul.so"))
    mm.amd_matmul_select_kernel.argtypes = [C.c_int]
    BF = B.DATAFLOW_BF16
    rng = np.random.default_rng(0)
    block = bf16_normal(rng, (16 << 20,), 0.5)

    def fill(buf, nbytes):
        for off in range(0, nbytes, block.nbytes):
            be.write(buf.ptr + off, block.view(np.uint8)[:min(block.nbytes, nbytes - off)])

    reps = args.steps if args.steps != 20 else 8
    cases = []
    for (G, M, K) in [(64, 2048, 4096), (64, 4096, 1024), (64, 1024, 4096), (32, 2816, 2048)]:
        for kind, rows in [("even", r) for r in (256, 384, 512, 700, 768, 1024, 1100, 1200, 1536, 2048)] + [("spread", 1024), ("zipf", 1024)]:
            if kind == "even":
                counts = np.full(G, rows, dtype=np.int32)
            elif kind == "spread":
                counts = rng.integers(rows // 2, rows * 3 // 2, size=G).astype(np.int32)
            else:
                w = 1.0 / np.arange(1, G + 1)
                counts = np.maximum(1, w / w.sum() * rows * G).astype(np.int32)
            total = int(counts.sum())
            d_W, d_X, d_D = be.alloc(G * M * K * 2), be.alloc(total * K * 2), be.alloc(total * M * 2)
            d_cum = be.upload(np.cumsum(counts).astype(np.int32))
            fill(d_W, G * M * K * 2)
            fill(d_X, total * K * 2)

            def launch():
                assert be.lib.dataflow_submit_amd_grouped_matmul(be.hp, 1, BF, BF, B.DATAFLOW_NONE, BF, B.DATAFLOW_FP32, 1, 0, B.AMD_GROUPED_RAGGED_N,
                                                                 M, K, total, G, d_cum.ptr, 1.0, 0.0, d_W.ptr, M * K * 2, d_X.ptr, None, d_D.ptr, 0) == 0

            best = {8: 1e9, 384: 1e9, 0: 1e9}
            for _ in range(3):
                for kernel in best:
                    assert mm.amd_matmul_select_kernel(kernel) == 0
                    launch()
                    a, b = ev.new(), ev.new()
                    ev.record(a, stream)
                    for _ in range(reps):
                        launch()
                    ev.record(b, stream)
                    best[kernel] = min(best[kernel], ev.elapsed_ms(a, b) / reps)
            assert mm.amd_matmul_select_kernel(0) == 0
            tiles_m, kt = -(-M // 256), -(-K // 64)
            narrow = -(-tiles_m * int(sum(-(-int(c) // 288) for c in counts)) // 256)
            wide = -(-tiles_m * int(sum(-(-int(c) // 384) for c in counts)) // 256)
            rule = 384 if wide * 640 * (103 * kt + 160) < narrow * 544 * 100 * kt else 8
            cases.append({"groups": G, "M": M, "K": K, "rows": rows if kind == "even" else "%d %s" % (rows, kind), "ms_8": round(best[8], 4),
                          "ms_384": round(best[384], 4), "ms_default": round(best[0], 4), "rule": rule})
            for d in (d_W, d_X, d_D, d_cum):
                d.free()
    right = sum(1 for c in cases if (c["ms_384"] < c["ms_8"]) == (c["rule"] == 384))
    lost = max((c["ms_384"] / c["ms_8"] if c["rule"] == 384 else c["ms_8"] / c["ms_384"]) for c in cases)
    print(json.dumps({"metric": "ragged_n_tiling_sweep", "value": right, "unit": "cases of %d where the rule picks the faster kernel" % len(cases),
                      "n_gpus": 1, "steps": reps, "warmup": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
                      "worst_pick_costs": round(lost, 3), "config": {"workload": args.workload}, "cases": cases}))


def stream_probe(args):
    """amd_matmul_stream_probe (include/amd_matmul_diag.h) over a table of cases: per step and compute unit 64 KiB of operand
    loads into LDS, 64 MFMAs per wave and a barrier.  `cold`: a 1 GiB source of which every 4 MiB region is read once per
    launch by `share` work-groups of a die in step, behind a 1 GiB fill that empties the caches; `cached`: a source as
    large as one pass reads, read again by every pass.  Each case: one untimed launch, then the median of --steps timed
    ones (3 unless given), each between its own pair of events.  Clocks are microseconds x 2400."""
    from ml_dataflow_amd import Backend, binding as B
    be = Backend(0)
    ev, stream = HipEvents(), be.stream(1)
    lib = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul_diag.so"))
    lib.amd_matmul_stream_probe.restype = C.c_int
    lib.amd_matmul_stream_probe.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    GIB, REGION, PASSES, STEPS = 1 << 30, 4 << 20, 4, 64
    src, flush, word = be.alloc(GIB), be.alloc(GIB), be.alloc(256)
    be.zero(src.ptr, GIB, 1)
    NO_LOADS, NO_MFMAS, TOUCH, VIA_REGS = 1, 2, 4, 8
    repeats = args.steps if args.steps != 20 else 3
    cases = [("no loads", False, 4, 1, NO_LOADS)]              # (data, cold, share, slack, flags)
    for data, share in (("cached", 0), ("cached", 32), ("cold", 8), ("cold", 4), ("cold", 2), ("cold", 1)):
        cold = data == "cold"
        cases += [(data, cold, share, slack, flags) for slack, flags in ((1, 0), (2, 0), (0, 0), (1, NO_MFMAS), (0, NO_MFMAS))]
        if cold and share > 1:
            cases.append((data, cold, share, 1, TOUCH))
        cases.append((data, cold, share, 2, VIA_REGS))
    out = []
    for data, cold, share, slack, flags in cases:
        groups = 1 if share == 0 else 256 // share
        src_bytes = GIB if cold else groups * REGION

        def launch():
            assert lib.amd_matmul_stream_probe(C.cast(be.hp, C.c_void_p), 1, src.ptr, src_bytes, share, slack, flags, PASSES, word.ptr) == 0
        launch()
        times = []
        for _ in range(repeats):
            if cold:
                be.zero(flush.ptr, GIB, 1)
            a, b = ev.new(), ev.new()
            ev.record(a, stream)
            launch()
            ev.record(b, stream)
            times.append(ev.elapsed_ms(a, b))
        us = sorted(times)[len(times) // 2] * 1e3 / (PASSES * STEPS)
        out.append({"data": data, "share": share, "wait": {0: "never, no barrier", 1: "end of the step", 2: "end of the next step"}[slack],
                    "loads": not flags & NO_LOADS, "mfmas": not flags & NO_MFMAS, "touch_ahead": bool(flags & TOUCH),
                    "through_registers": bool(flags & VIA_REGS),
                    "us_per_step": round(us, 4), "clocks_at_2400MHz": int(round(us * 2400))})
    # Where the lines come from: regions that are read again by every pass, with working sets from the size of the L2 caches
    # (4 MiB a die) over that of the 256 MiB memory-side cache to beyond it.  (4 passes: the first one is cold.)
    reread = []
    for share in (32, 8, 4):
        groups = 256 // share
        for mult in (1, 2, 4, 8):
            nbytes = min(GIB, groups * REGION * mult)
            if reread and (share, nbytes) == (reread[-1]["share"], reread[-1]["working_set_mib"] << 20):
                continue
            row = {"share": share, "working_set_mib": nbytes >> 20, "per_die_mib": (nbytes >> 20) // 8}
            for key, slack, flags in (("waited_each_step", 1, 0), ("loads_only_never_waited", 0, NO_MFMAS)):
                def launch():
                    assert lib.amd_matmul_stream_probe(C.cast(be.hp, C.c_void_p), 1, src.ptr, nbytes, share, slack, flags, 2 * PASSES, word.ptr) == 0
                launch()
                times = []
                for _ in range(repeats):
                    a, b = ev.new(), ev.new()
                    ev.record(a, stream)
                    launch()
                    ev.record(b, stream)
                    times.append(ev.elapsed_ms(a, b))
                row[key] = int(round(sorted(times)[len(times) // 2] * 1e3 / (2 * PASSES * STEPS) * 2400))
            reread.append(row)
    # Sharers out of step: sharer i of a region starts i * n steps into it, so the lines the others ask for were requested
    # by the first of them n to (share - 1) * n steps earlier; per sharer rank, from each work-group's own clock
    ROTATE_SHIFT, PER_GROUP_CLOCKS = 4, 1024
    clocks = be.alloc(4096)
    rotated = []
    for share in (4, 8):
        for n in (0, 1, 2, 4):
            be.zero(flush.ptr, GIB, 1)
            assert lib.amd_matmul_stream_probe(C.cast(be.hp, C.c_void_p), 1, src.ptr, GIB, share, 1, (n << ROTATE_SHIFT) | PER_GROUP_CLOCKS, PASSES, clocks.ptr) == 0
            be.sync(1)
            ticks = be.read(clocks.ptr, (257,), np.float32)[1:] / 100.0 / (PASSES * STEPS) * 2400
            rank = (np.arange(256) >> 3) % share
            rotated.append({"share": share, "steps_apart": n, "clocks_by_sharer_rank": [int(round(float(ticks[rank == r].mean()))) for r in range(share)]})
    be.sync(1)
    head = next(c for c in out if c["data"] == "cold" and c["share"] == 4 and c["wait"] == "end of the step" and c["loads"] and c["mfmas"]
                and not c["touch_ahead"] and not c["through_registers"])
    print(json.dumps({
        "metric": "clocks per k-tile step of the streaming GEMM's skeleton (64 KiB of loads from HBM shared by 4 work-groups, "
                  "64 MFMAs per wave, one barrier; the multiplies alone are 2048)",
        "value": head["clocks_at_2400MHz"], "unit": "clocks at 2.4 GHz", "n_gpus": 1, "steps": repeats, "warmup": 1,
        "ms_per_step": round(head["us_per_step"] * 1e-3, 7), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {"workload": args.workload, "kernel": "stream_probe_kernel",
                                                          "steps_per_launch": PASSES * STEPS, "bytes_per_step_and_compute_unit": 65536},
        "cases": out, "reread_working_sets": reread, "sharers_out_of_step": rotated}))
    be.close()


def vendor_gemm(args):
    """The M x K x N problem of the gemm_sustained workloads (D[n, m] = sum_k B[n, k] A[m, k]) through torch.matmul, i.e. the
    vendor's GEMM library, with the same operand distributions and launch count; timed with events on torch's stream."""
    import torch
    M, K, N = (int(v) for v in args.workload.split("_")[-1].split("x"))
    launches = args.steps if args.steps > 20 else 2000
    half = launches // 2
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(42)
    A = (torch.randn((M, K), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    Bm = torch.randn((N, K), generator=gen, device=dev).to(torch.bfloat16)
    out = torch.empty((N, M), dtype=torch.bfloat16, device=dev)
    for _ in range(max(args.warmup, 3)):
        torch.matmul(Bm, A.t(), out=out)
    a, mid, b = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    torch.cuda.synchronize()
    a.record()
    for i in range(launches):
        if i == half:
            mid.record()
        torch.matmul(Bm, A.t(), out=out)
    b.record()
    torch.cuda.synchronize()
    first_ms, second_ms = a.elapsed_time(mid) / half, mid.elapsed_time(b) / (launches - half)
    tflops = 2.0 * M * K * N / (second_ms * 1e-3) / 1e12
    print(json.dumps({
        "metric": "sustained bf16 MFMA TFLOP/s (%s)" % args.workload, "value": round(tflops, 1), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": launches, "warmup": args.warmup, "ms_per_step": round(second_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "M": M, "K": K, "N": N, "library": "torch.matmul (torch %s)" % torch.__version__},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": None},
        "first_half_ms_per_launch": round(first_ms, 4), "second_half_ms_per_launch": round(second_ms, 4)}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS) + SUSTAINED_WORKLOADS + VENDOR_WORKLOADS + [STREAM_PROBE_WORKLOAD, TILING_SWEEP_WORKLOAD],
                    help="a layer workload, or one of the sustained-rate diagnostics: one GEMM shape through the matmul op launched "
                         "--steps times back to back (default 2000), or the MFMA-only probe kernel")
    ap.add_argument("--schedule", default="fused", choices=["fused", "grouped", "per_expert"],
                    help="fused: grouped launches, backward without the recompute of the expert outputs (9 expert GEMMs per step); "
                         "grouped: the reference's op sequence with grouped launches (10 expert GEMMs); per_expert: the reference's "
                         "own schedule (host sync after routing, one launch per expert and op)")
    ap.add_argument("--gemm-kernel", type=int, default=0, choices=[0, 8, 4, 384],
                    help="persistent GEMM kernel of the large launches without a C operand (amd_matmul_select_kernel): 0 = the library's "
                         "default (per launch, decided on the device from the group sizes: 8 or 384); 8 = eight waves, loads straight "
                         "into the LDS, 256 x 288 tiles; 384 = four waves that all load and multiply, 256 x 384 tiles; 4 = one loading "
                         "wave and three multiplying waves.  Another one (4 beside 8, else 8) is timed after the step loop and "
                         "reported under gemm_kernel_ab")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="skip the two side measurements (the other GEMM kernel, the first-micro-batch backward): a profiler run then "
                         "sees the accumulating steps' launches only")
    ap.add_argument("--cpu-sample-tokens", type=int, default=8192,
                    help="tokens of the workload the CPU baseline is timed on (the whole of the 8192-token workloads: about 45 s on 16 cores)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="before the steps, launch a plain copy of known size (prepare_experts with top_k 1 and the identity "
                         "mapping, 65536 rows of 8 KiB: 512 MiB read + 512 MiB written) three times, so that a hardware counter "
                         "run can scale FETCH_SIZE / WRITE_SIZE by what they read for it")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the MoE hot path is a single-device kernel path); "
                 "--gpus %d is not supported, run with --gpus 1" % args.gpus)
    if args.workload in SUSTAINED_WORKLOADS:
        return sustained_gemm(args)
    if args.workload in VENDOR_WORKLOADS:
        return vendor_gemm(args)
    if args.workload == STREAM_PROBE_WORKLOAD:
        return stream_probe(args)
    if args.workload == TILING_SWEEP_WORKLOAD:
        return tiling_sweep(args)

    from ml_dataflow_amd import Backend, MoeLayer, binding as B

    T, D, E, K, H, backward, bias_scale = WORKLOADS[args.workload]
    schedule = {"fused": B.AMD_MOE_FUSED, "grouped": B.AMD_MOE_GROUPED, "per_expert": B.AMD_MOE_PER_EXPERT}[args.schedule]
    rng = np.random.default_rng(42)
    be = Backend(0)
    layer = MoeLayer(be, T, D, E, K, H)
    be.write(layer.L.w_router, bf16_normal(rng, (E, D), 0.02))
    for e in range(E):
        be.write(layer.expert_ptr(layer.L.w1, e), bf16_normal(rng, (H, D), 0.02))
        be.write(layer.expert_ptr(layer.L.w3, e), bf16_normal(rng, (H, D), 0.02))
        be.write(layer.expert_ptr(layer.L.w2, e), bf16_normal(rng, (D, H), 0.02))
    d_X = be.upload(bf16_normal(rng, (T, D), 1.0))
    d_dY = be.upload(bf16_normal(rng, (T, D), 1.0))
    d_out, d_dX = be.alloc(T * D * 2), be.alloc(T * D * 2)
    d_bias = None
    if bias_scale is not None:
        d_bias = be.upload(f32_to_bf16(np.broadcast_to(zipf_bias(rng, E, bias_scale), (T, E)).copy()))

    first_micro_batch = [False]          # the timed steps accumulate the weight gradients (beta = 1), as the reference's always do

    def step():
        be.zero(d_out.ptr, T * D * 2, 1)
        layer.forward(T, d_X.ptr, d_out.ptr, d_bias.ptr if d_bias else None, schedule)
        if backward:
            layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule, first_micro_batch=first_micro_batch[0])

    if args.calibration_copy:
        rows, width = 65536, 4096
        src, dst = be.alloc(rows * width * 2), be.alloc(rows * width * 2)
        ident = be.upload(np.arange(rows, dtype=np.int32))
        be.zero(src.ptr, rows * width * 2, 1)
        for _ in range(3):
            assert be.lib.dataflow_submit_default_prepare_experts(be.hp, 1, B.DATAFLOW_BF16, B.DATAFLOW_BF16, rows, width, 1,
                                                                  src.ptr, ident.ptr, dst.ptr) == 0
        be.sync()
        src.free(), dst.free(), ident.free()

    mm = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul.so"))
    mm.amd_matmul_select_kernel.argtypes = [C.c_int]
    assert mm.amd_matmul_select_kernel(args.gemm_kernel) == 0
    for _ in range(args.warmup):
        step()
    be.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    be.sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    counts = be.read(layer.L.expert_counts, (E,), np.int32)

    ev = HipEvents()
    stream = be.stream(1)

    def steps_one_by_one(n):
        """n more steps, each between its own pair of events on the compute stream (every schedule ends a pass there)"""
        marks = []
        for _ in range(n):
            a, b = ev.new(), ev.new()
            ev.record(a, stream)
            step()
            ev.record(b, stream)
            marks.append((a, b))
        be.sync()
        return sorted(ev.elapsed_ms(a, b) for a, b in marks)

    def replay_classes(n, first=False):
        """per-kernel durations: HIP events on the compute stream around every launch of an op-by-op replay"""
        acc = {}
        for i in range(n + 1):
            marks = replay_step_with_events(be, layer, T, d_X, d_out, d_dY, d_dX, d_bias, backward, ev, stream, args.schedule == "fused", first)
            if i == 0:
                continue                               # first replay warms the event pool
            for name, ms in marks:
                acc.setdefault(name, []).append(ms)
        return acc

    per_step = steps_one_by_one(args.steps)
    replays = max(3, min(10, args.steps))
    per_class = replay_classes(replays)
    # the same steps on the other persistent GEMM kernel, in this process on this card (not part of the timed steps above)
    other = 4 if args.gemm_kernel == 8 else 8
    gemm_kernel_ab = None
    if args.schedule == "fused" and not args.headline_only:
        assert mm.amd_matmul_select_kernel(other) == 0
        for _ in range(3):
            step()
        be.sync()
        other_steps = steps_one_by_one(args.steps)
        other_classes = replay_classes(3)
        assert mm.amd_matmul_select_kernel(args.gemm_kernel) == 0
        gemm_kernel_ab = {"kernel": other, "ms_per_step_median": round(other_steps[len(other_steps) // 2], 4), "ms_per_step_min": round(other_steps[0], 4),
                          "gemm_avg_ms": {k: round(float(np.mean(v)), 4) for k, v in other_classes.items() if k.startswith("gemm")},
                          "note": "ragged-N launches without a C operand only (up13, tn, nn, dx13); the weight-gradient launches run the eight-wave kernel either way"}
    # the first micro-batch of an accumulation: weight gradients written with beta = 0 and no C operand.  Reported beside the
    # accumulating steps above, which stay the headline (every later micro-batch, and every step of the reference, is one of those)
    first_mb = None
    if backward and args.schedule != "per_expert" and not args.headline_only:
        first_micro_batch[0] = True
        for _ in range(3):
            step()
        be.sync()
        first_steps = steps_one_by_one(args.steps)
        first_classes = replay_classes(3, first=True)
        first_micro_batch[0] = False
        first_mb = {"ms_per_step_median": round(first_steps[len(first_steps) // 2], 4), "ms_per_step_min": round(first_steps[0], 4),
                    "weight_gradient_gemm_avg_ms": {k: round(float(np.mean(v)), 4) for k, v in first_classes.items() if k in ("gemm_nt_dw", "gemm_dw13")},
                    "weight_gradient_gemm_frac": {k: round(algorithmic_work(T, D, E, K, H, args.schedule == "fused")[k][1] / (float(np.mean(v)) * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)
                                                  for k, v in first_classes.items() if k in ("gemm_nt_dw", "gemm_dw13")},
                    "note": "AMD_MOE_FIRST_MICRO_BATCH: dW written with beta = 0, no C read, no cleared buffers; not the headline"}
    outside_step = set()
    for i in range(replays + 1):
        marks = norm_kernels_with_events(be, T, D, d_X, d_dY, d_dX, ev, stream, backward)
        if backward and i < 3:
            marks += adamw_with_events(be, layer, ev, stream)
        for name, ms in marks:
            outside_step.add(name)
            if i > 0:
                per_class.setdefault(name, []).append(ms)
    work = algorithmic_work(T, D, E, K, H, args.schedule == "fused")
    kernels = {}
    for name, samples in per_class.items():
        bound, amount = work[name]
        avg_ms = float(np.mean(samples))
        launches = len(samples) // replays
        if bound == "mfma":
            achieved, peak, unit = amount / (avg_ms * 1e-3) / 1e12, PEAK_BF16_TFLOPS, "TFLOP/s"
        else:
            achieved, peak, unit = amount / (avg_ms * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
        kernels[name] = {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit, "frac": round(achieved / peak, 4),
                         "avg_ms": round(avg_ms, 4), "launches_per_step": launches, "ms_per_step": round(avg_ms * launches, 4)}
        if name in outside_step:
            kernels[name].update({"launches_per_step": 0, "ms_per_step": 0.0, "in_step": False})
    gemms = {k: v for k, v in kernels.items() if v["bound"] == "mfma"}
    gemm_ms = sum(v["ms_per_step"] for v in gemms.values())
    gemm_flops = sum(work[k][1] * v["launches_per_step"] for k, v in gemms.items())
    measured = MEASURED_TRAFFIC_BYTES.get(args.workload, {}) if args.schedule == "fused" and args.gemm_kernel == 0 else {}
    # The dominant kernel is the kernel function with the most time per step, as in a rocprofv3 --stats table.  The fused
    # schedule launches one of its GEMM kernels twice per step with different shapes (dh, then dx1 W1 + dx3 W3): launch
    # classes that run the same kernel are taken together, flops and durations averaged over its launches.
    big = args.schedule == "fused" and min(D, H) >= 256 and (T * K // 288) * (min(D, H) // 256) >= 128
    kernel_of_class = dict(FUSED_GEMM_KERNEL_OF_CLASS)
    if args.gemm_kernel != 8:
        name = _W4 if args.gemm_kernel == 4 else _W4D
        four = {"gemm_up13": name % "false, 1, 1", "gemm_tn": name % "false, 1, 0", "gemm_nn": name % "true, 1, 0", "gemm_dx13": name % "true, 1, 0"}
        if args.gemm_kernel == 0:
            # the library's rule (ragged_n_prefers_384 in gemm_kernel.h), from the same group sizes: which launches ran on 256 x 384 tiles
            rows_m = {"gemm_up13": 2 * H, "gemm_tn": D, "gemm_nn": H, "gemm_dx13": D}
            k_of = {"gemm_up13": D, "gemm_tn": H, "gemm_nn": D, "gemm_dx13": 2 * H}
            for cls in list(four):
                tiles_m = -(-rows_m[cls] // 256)
                narrow = tiles_m * int(sum(-(-int(c) // 288) for c in counts))
                wide = tiles_m * int(sum(-(-int(c) // 384) for c in counts))
                groups = max(8, min(256, (tiles_m * (T * K // 288 + E) + 7) // 8 * 8))
                even = T * K // E                          # the host's first look: all groups the same size
                even_narrow, even_wide = tiles_m * E * -(-max(even, 1) // 288), tiles_m * E * -(-max(even, 1) // 384)
                kt = -(-k_of[cls] // 64)
                wide_cost, narrow_cost = 640 * (103 * kt + 160), 544 * 100 * kt
                takes_wide = k_of[cls] % 128 == 0 and rows_m[cls] % 8 == 0 and \
                    -(-even_wide // 256) * wide_cost < -(-even_narrow // 256) * narrow_cost and \
                    -(-wide // groups) * wide_cost < -(-narrow // groups) * narrow_cost
                if not takes_wide:
                    del four[cls]
        kernel_of_class.update(four)
    by_kernel = {}
    for k, v in gemms.items():
        by_kernel.setdefault(kernel_of_class[k] if big else k, []).append(k)
    dominant = max(by_kernel, key=lambda name: sum(gemms[k]["ms_per_step"] for k in by_kernel[name]))
    classes = by_kernel[dominant]
    launches = sum(gemms[k]["launches_per_step"] for k in classes)
    dom_ms = sum(gemms[k]["ms_per_step"] for k in classes)
    dom_flops = sum(work[k][1] * gemms[k]["launches_per_step"] for k in classes)
    dom_tflops = dom_flops / (dom_ms * 1e-3) / 1e12
    slowest = min(gemms, key=lambda k: gemms[k]["frac"])
    have_traffic = all(k in measured for k in classes)
    roofline = {"bound": "mfma", "achieved": round(dom_tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(dom_tflops / PEAK_BF16_TFLOPS, 4),
                "traffic": int(sum(measured[k] * gemms[k]["launches_per_step"] for k in classes) / launches) if have_traffic else None,
                "traffic_source": TRAFFIC_SOURCE % args.workload if have_traffic else None,
                "traffic_meaning": "bytes the L2 caches exchanged with the fabric (FETCH_SIZE + WRITE_SIZE); requests that the 256 MiB "
                                   "memory-side cache serves are included, so this is an upper bound on DRAM bytes",
                "kernel": dominant, "launch_classes": classes, "launches_per_step": launches, "avg_launch_ms": round(dom_ms / launches, 4),
                "algorithmic_flops_per_launch": dom_flops / launches,
                "all_grouped_gemms_frac": round(gemm_flops / (gemm_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
                "slowest_gemm_launch_class": {"name": slowest, "frac": gemms[slowest]["frac"], "avg_launch_ms": gemms[slowest]["avg_ms"]}}

    result = {
        "metric": "MoE layer fwd+bwd tokens/sec @8192 tok; grouped-GEMM % bf16 MFMA peak" if args.workload == DEFAULT_WORKLOAD
                  else "MoE layer tokens/sec (%s)" % args.workload,
        "value": round(T / (ms_per_step * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "ms_per_step_median": round(per_step[len(per_step) // 2], 4), "ms_per_step_min": round(per_step[0], 4),
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "gemm_kernel": args.gemm_kernel, "tokens": T, "d_model": D, "experts": E, "top_k": K, "expert_hidden": H,
                   "pass": "fwd+bwd" if backward else "fwd", "schedule": args.schedule,
                   "max_expert_rows": int(counts.max()), "mean_expert_rows": float(T * K / E)},
        "roofline": roofline,
        "kernels": kernels,
    }
    if gemm_kernel_ab:
        result["gemm_kernel_ab"] = gemm_kernel_ab
    if first_mb:
        result["first_micro_batch"] = first_mb
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(min(args.cpu_sample_tokens, T), D, E, K, H, backward, 42)
    layer.free()
    be.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
