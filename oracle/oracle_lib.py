"""ctypes loader for the CPU oracle (oracle/libmoe_oracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.dirname(os.path.abspath(__file__))
_P = C.c_void_p
_I = C.c_int


class OracleMoeLayer(C.Structure):
    _fields_ = [("T", _I), ("D", _I), ("E", _I), ("K", _I), ("H", _I), ("logits_given", _I),
                ("Wr", _P), ("W1", _P), ("W3", _P), ("W2", _P), ("w_stride", C.c_size_t),
                ("logits", _P), ("weights", _P), ("chosen", _P), ("counts", _P), ("cumsum", _P),
                ("expert_mapping", _P), ("token_mapping", _P), ("x1", _P), ("x3", _P),
                ("zones", _P), ("temp", _P),
                ("dx1", _P), ("dx3", _P), ("dlogits", _P), ("dWr", _P), ("dW1", _P), ("dW3", _P), ("dW2", _P)]


SIGS = {
    "oracle_bf16_to_f32": (C.c_float, [C.c_uint16]),
    "oracle_f32_to_bf16": (C.c_uint16, [C.c_float]),
    "oracle_matmul": (None, [_I, _I, _I, _I, _I, C.c_float, C.c_float, _P, _P, _P, _P]),
    "oracle_select_experts": (None, [_I, _I, _I, _P, _P, _P, _P, _P, _P]),
    "oracle_build_expert_mapping": (None, [_I, _I, _I, _P, _P, _P, _P]),
    "oracle_prepare_experts": (None, [_I, _I, _I, _P, _P, _P]),
    "oracle_prepare_expert_zone": (None, [_I, _P, _I, _P, _P, _P, _P]),
    "oracle_swiglu": (None, [_I, _I, _P, _P, _P]),
    "oracle_swiglu_bwd_x": (None, [_I, _I, _P, _P, _P, _P, _P]),
    "oracle_merge_experts": (None, [_I, _I, _I, _P, _P, _P, _P]),
    "oracle_merge_expert_result": (None, [_I, _I, _I, _P, _I, _P, _P, _P, _P, _P]),
    "oracle_router_bwd_x": (None, [_I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P]),
    "oracle_router_gate_bwd_x": (None, [_I, _I, _I, _P, _P, _P]),
    "oracle_rms_norm": (None, [_I, _I, C.c_float, _P, _P, _P, _P]),
    "oracle_rms_norm_recompute": (None, [_I, _I, _P, _P, _P, _P]),
    "oracle_rms_norm_bwd_x": (None, [_I, _I, C.c_float, _P, _P, _P, _P, _P, _P]),
    "oracle_rms_norm_bwd_w": (None, [_I, _I, C.c_float, _P, _P, _P, _P]),
    "oracle_adamw_step": (None, [C.c_uint64, _I, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float, _P, _P, _P, _P]),
    "oracle_cast_bf16_fp32": (None, [C.c_uint64, _P, _P]),
    "oracle_cast_and_add": (None, [C.c_uint64, C.c_float, _P, C.c_float, _P, _P]),
    "oracle_select_experts_fp32": (None, [_I, _I, _I, _P, _P, _P, _P, _P, _P]),
    "oracle_fp16_to_f32": (C.c_float, [C.c_uint16]),
    "oracle_f32_to_fp16": (C.c_uint16, [C.c_float]),
    "oracle_swiglu_typed": (None, [_I, _I, _I, _P, _P, _P]),
    "oracle_swiglu_bwd_x_typed": (None, [_I, _I, _I, _P, _P, _P, _P, _P]),
    "oracle_matmul_typed": (_I, [_I, _I, _I, _I, _I, _I, _I, C.c_float, C.c_float, _P, _P, _P, _P]),
    "oracle_moe_forward": (_I, [C.POINTER(OracleMoeLayer), _P, _P, _P]),
    "oracle_moe_backward": (_I, [C.POINTER(OracleMoeLayer), _P, _P, _P]),
}

_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    path = os.path.join(ORACLE_DIR, "libmoe_oracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "libmoe_oracle.so"])
    lib = C.CDLL(path)
    for name, (res, args) in SIGS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def ptr(a):
    return None if a is None else a.ctypes.data


# ---- numpy-friendly wrappers (all arrays C-contiguous; bf16 as uint16) ----

def matmul(lib, transa, transb, M, K, N, A, B, alpha=1.0, beta=0.0, Cin=None):
    D = np.empty((N, M), dtype=np.uint16)
    if Cin is not None:
        D[...] = Cin
    lib.oracle_matmul(transa, transb, M, K, N, alpha, beta, ptr(A), ptr(B), ptr(D) if Cin is not None else None, ptr(D))
    return D


def select_experts(lib, logits, K):
    T, E = logits.shape
    w = np.zeros((T, K), dtype=np.float32)
    chosen = np.zeros((T, K), dtype=np.uint16)
    counts = np.zeros(E + 1, dtype=np.int32)
    cumsum = np.zeros(E, dtype=np.int32)
    host = np.zeros(E, dtype=np.int32)
    lib.oracle_select_experts(T, E, K, ptr(logits), ptr(w), ptr(chosen), ptr(counts), ptr(cumsum), ptr(host))
    return w, chosen, counts, cumsum, host


def select_experts_fp32(lib, logits, K):
    """logits: float32 [T, E]"""
    T, E = logits.shape
    w = np.zeros((T, K), dtype=np.float32)
    chosen = np.zeros((T, K), dtype=np.uint16)
    counts = np.zeros(E + 1, dtype=np.int32)
    cumsum = np.zeros(E, dtype=np.int32)
    host = np.zeros(E, dtype=np.int32)
    lib.oracle_select_experts_fp32(T, E, K, ptr(logits), ptr(w), ptr(chosen), ptr(counts), ptr(cumsum), ptr(host))
    return w, chosen, counts, cumsum, host


def swiglu_typed(lib, x1, x3):
    """x1, x3: float32 or float16 arrays of one shape [rows, cols]"""
    out = np.empty_like(x1)
    lib.oracle_swiglu_typed(int(x1.dtype == np.float16), x1.shape[0], x1.shape[1], ptr(x1), ptr(x3), ptr(out))
    return out


def swiglu_bwd_x_typed(lib, x1, x3, g):
    d1, d3 = np.empty_like(x1), np.empty_like(x1)
    lib.oracle_swiglu_bwd_x_typed(int(x1.dtype == np.float16), x1.shape[0], x1.shape[1], ptr(x1), ptr(x3), ptr(g), ptr(d1), ptr(d3))
    return d1, d3


ELEM_FP32, ELEM_FP16, ELEM_BF16 = 0, 1, 2


def matmul_typed(lib, ab_kind, cd_kind, transa, transb, M, K, N, A, B, alpha=1.0, beta=0.0, Cin=None):
    """A, B: float32 arrays (fp32) or uint16 bit patterns (fp16, bf16); returns D [N, M] in the same convention"""
    D = np.empty((N, M), dtype=np.float32 if cd_kind == ELEM_FP32 else np.uint16)
    if Cin is not None:
        D[...] = Cin
    assert lib.oracle_matmul_typed(ab_kind, cd_kind, transa, transb, M, K, N, alpha, beta, ptr(A), ptr(B),
                                   ptr(D) if Cin is not None else None, ptr(D)) == 0
    return D


def build_expert_mapping(lib, chosen, E, cumsum_excl):
    T, K = chosen.shape
    cumsum = np.array(cumsum_excl, dtype=np.int32, copy=True)
    emap = np.full(T * K, -1, dtype=np.int32)
    tmap = np.full((T, K), -1, dtype=np.int32)
    lib.oracle_build_expert_mapping(T, E, K, ptr(chosen), ptr(cumsum), ptr(emap), ptr(tmap))
    return emap, tmap, cumsum


class Layer:
    """Owns numpy buffers for an Oracle_Moe_Layer and runs forward / backward."""

    def __init__(self, lib, T, D, E, K, H, Wr, W1, W3, W2):
        self.lib = lib
        self.T, self.D, self.E, self.K, self.H = T, D, E, K, H
        R = T * K
        self.Wr, self.W1, self.W3, self.W2 = [np.ascontiguousarray(w, dtype=np.uint16) for w in (Wr, W1, W3, W2)]
        z = lambda shape, dt=np.uint16: np.zeros(shape, dtype=dt)
        self.logits, self.weights, self.chosen = z((T, E)), z((T, K), np.float32), z((T, K))
        self.counts, self.cumsum = z(E + 1, np.int32), z(E, np.int32)
        self.expert_mapping, self.token_mapping = z(R, np.int32), z((T, K), np.int32)
        self.x1, self.x3, self.zones, self.temp = z((R, H)), z((R, H)), z((R, D)), z((R, H))
        self.dx1, self.dx3, self.dlogits = z((R, H)), z((R, H)), z((T, E))
        self.dWr, self.dW1, self.dW3, self.dW2 = z((E, D)), z((E, H, D)), z((E, H, D)), z((E, D, H))
        s = self.s = OracleMoeLayer()
        s.T, s.D, s.E, s.K, s.H = T, D, E, K, H
        s.w_stride = H * D
        for name in ("Wr", "W1", "W3", "W2", "logits", "weights", "chosen", "counts", "cumsum", "expert_mapping",
                     "token_mapping", "x1", "x3", "zones", "temp", "dx1", "dx3", "dlogits", "dWr", "dW1", "dW3", "dW2"):
            setattr(s, name, getattr(self, name).ctypes.data)

    def forward(self, X, residual, logit_bias=None, logits=None):
        """logits: if given ([T,E] bf16 bits), routing replays these instead of the oracle's own router product"""
        out = np.array(residual, dtype=np.uint16, copy=True)
        self.s.logits_given = 0 if logits is None else 1
        if logits is not None:
            self.logits[...] = logits
        ret = self.lib.oracle_moe_forward(C.byref(self.s), ptr(X), ptr(logit_bias), ptr(out))
        assert ret == 0
        return out

    def backward(self, X, dY):
        dX = np.zeros((self.T, self.D), dtype=np.uint16)
        ret = self.lib.oracle_moe_backward(C.byref(self.s), ptr(X), ptr(dY), ptr(dX))
        assert ret == 0
        return dX
