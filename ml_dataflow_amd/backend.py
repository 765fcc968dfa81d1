"""Thin Python host over the C boundary: handle lifecycle, device buffers and numpy transfers.

Every call goes through the C ABI (the handle's function pointers or the exported submit wrappers);
the classes here own no algorithm.  Device buffers are raw pointers from handle->alloc_mem.
"""
import ctypes as C

import numpy as np

from . import binding as B

STREAM_NAMES = [b"Inbound", b"Compute", b"Secondary Compute", b"Outbound", b"Peer", b"Host Ops", b"Inbound Fwd Context", b"Loss"]
COMPUTE_STREAM = 1      # the stream roles the reference's drivers use (test/dataflow_models/transformer_moe.c:315-327)
SECONDARY_STREAM = 2
INBOUND_STREAM = 0
OUTBOUND_STREAM = 3


class DeviceBuffer:
    """A device allocation made through the handle; freed explicitly or with the backend."""

    def __init__(self, backend, nbytes):
        self.backend = backend
        self.nbytes = int(nbytes)
        self.ptr = backend.h.alloc_mem(backend.hp, max(self.nbytes, 256))
        if not self.ptr:
            raise MemoryError("alloc_mem(%d) failed" % self.nbytes)

    def free(self):
        if self.ptr:
            self.backend.h.free_mem(self.backend.hp, self.ptr)
            self.ptr = None


class Backend:
    """dataflow_init_handle + dataflow_register_default_ops on one GPU."""

    def __init__(self, device_id=0, num_streams=8):
        self.lib = B.load_library()
        self.h = B.DataflowHandle()
        self.hp = C.pointer(self.h)
        names = (C.c_char_p * num_streams)(*[STREAM_NAMES[i] if i < len(STREAM_NAMES) else None for i in range(num_streams)])
        ret = self.lib.dataflow_init_handle(self.hp, B.COMPUTE_HSA, device_id, 0, 0, num_streams, None, names, 1.0)
        if ret != 0:
            raise RuntimeError("dataflow_init_handle failed (is a gfx950 GPU visible?)")
        self.num_ops = self.lib.dataflow_register_default_ops(self.hp)
        if self.num_ops <= 0:
            raise RuntimeError("dataflow_register_default_ops failed: native code objects not loaded")
        self._buffers = []
        self.closed = False

    # ---- device info ----
    @property
    def device_info(self):
        return C.cast(self.h.device_info, C.POINTER(B.HipDeviceInfo)).contents

    def stream(self, stream_id):
        return self.lib.dataflow_amd_get_stream(self.hp, stream_id)

    # ---- memory ----
    def alloc(self, nbytes):
        buf = DeviceBuffer(self, nbytes)
        self._buffers.append(buf)
        return buf

    def upload(self, array, stream_id=INBOUND_STREAM):
        """numpy array -> new device buffer (synchronous)."""
        array = np.ascontiguousarray(array)
        buf = self.alloc(array.nbytes)
        self.write(buf.ptr, array, stream_id)
        return buf

    def write(self, dev_ptr, array, stream_id=INBOUND_STREAM):
        array = np.ascontiguousarray(array)
        if array.nbytes == 0:
            return
        ret = self.h.submit_inbound_transfer(self.hp, stream_id, dev_ptr, array.ctypes.data, array.nbytes)
        if ret != 0 or self.h.sync_stream(self.hp, stream_id) != 0:
            raise RuntimeError("inbound transfer failed")

    def read(self, dev_ptr, shape, dtype, stream_id=OUTBOUND_STREAM):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes == 0:
            return out
        ret = self.h.submit_outbound_transfer(self.hp, stream_id, out.ctypes.data, dev_ptr, out.nbytes)
        if ret != 0 or self.h.sync_stream(self.hp, stream_id) != 0:
            raise RuntimeError("outbound transfer failed")
        return out

    def zero(self, dev_ptr, nbytes, stream_id=-1):
        if self.h.set_mem(self.hp, stream_id, dev_ptr, 0, nbytes) != 0:
            raise RuntimeError("set_mem failed")

    def sync(self, stream_id=None):
        ret = self.h.sync_handle(self.hp) if stream_id is None else self.h.sync_stream(self.hp, stream_id)
        if ret != 0:
            raise RuntimeError("device synchronisation failed (a kernel may have faulted)")

    def host_alloc(self, nbytes):
        ptr = self.lib.dataflow_amd_alloc_host_mem(self.hp, nbytes)
        if not ptr:
            raise MemoryError("dataflow_amd_alloc_host_mem(%d) failed" % nbytes)
        return ptr

    def host_free(self, ptr):
        self.lib.dataflow_amd_free_host_mem(self.hp, ptr)

    def close(self):
        if self.closed:
            return
        for buf in self._buffers:
            buf.free()
        self._buffers = []
        self.lib.dataflow_amd_destroy_handle(self.hp)
        self.closed = True


class MoeLayer:
    """amd_moe_layer_* : one MoE layer's buffers plus forward / backward submission."""

    def __init__(self, backend, max_tokens, model_dim, num_experts, top_k, expert_dim):
        self.be = backend
        self.L = B.AmdMoeLayer()
        self.T, self.D, self.E, self.K, self.H = max_tokens, model_dim, num_experts, top_k, expert_dim
        ret = backend.lib.amd_moe_layer_alloc(backend.hp, C.byref(self.L), max_tokens, model_dim, num_experts, top_k, expert_dim)
        if ret != 0:
            raise RuntimeError("amd_moe_layer_alloc failed")

    def expert_ptr(self, base, e):
        return base + self.L.expert_stride_bytes * e

    def load_weights(self, Wr, W1, W3, W2):
        """Wr [E,D], W1/W3 [E,H,D], W2 [E,D,H] as uint16 (bf16 bits)."""
        self.be.write(self.L.w_router, Wr)
        for e in range(self.E):
            self.be.write(self.expert_ptr(self.L.w1, e), W1[e])
            self.be.write(self.expert_ptr(self.L.w3, e), W3[e])
            self.be.write(self.expert_ptr(self.L.w2, e), W2[e])

    def zero_grads(self):
        self.be.zero(self.L.dw_router, self.E * self.D * 2)
        self.be.zero(self.L.dw1, self.L.expert_stride_bytes * self.E)

    def read_grads(self):
        be, E, D, H = self.be, self.E, self.D, self.H
        dWr = be.read(self.L.dw_router, (E, D), np.uint16)
        dW1 = np.stack([be.read(self.expert_ptr(self.L.dw1, e), (H, D), np.uint16) for e in range(E)])
        dW3 = np.stack([be.read(self.expert_ptr(self.L.dw3, e), (H, D), np.uint16) for e in range(E)])
        dW2 = np.stack([be.read(self.expert_ptr(self.L.dw2, e), (D, H), np.uint16) for e in range(E)])
        return dWr, dW1, dW3, dW2

    def read_up_projections(self, num_tokens, grads=False):
        """(x1, x3) of the last forward, or (dx1, dx3) of the last backward, as [T*K, H] uint16 arrays, whichever way the
        schedule stored them (two arrays, or one [T*K, 2H] array with the pair side by side per row)."""
        R, H = num_tokens * self.K, self.H
        base = self.L.dx1 if grads else self.L.x1
        both = self.be.read(base, (2 * R * H,), np.uint16)
        if self.L.saved_side_by_side:
            both = both.reshape(R, 2 * H)
            return np.ascontiguousarray(both[:, :H]), np.ascontiguousarray(both[:, H:])
        return both[:R * H].reshape(R, H), self.be.read(self.L.dx3 if grads else self.L.x3, (R, H), np.uint16)

    def forward(self, num_tokens, X_ptr, out_ptr, logit_bias_ptr=None, schedule=B.AMD_MOE_GROUPED,
                compute_stream=1, secondary_stream=2):
        ret = self.be.lib.amd_moe_layer_forward(self.be.hp, compute_stream, secondary_stream, C.byref(self.L), num_tokens,
                                                X_ptr, logit_bias_ptr, out_ptr, schedule)
        if ret != 0:
            raise RuntimeError("amd_moe_layer_forward failed")

    def backward(self, num_tokens, X_ptr, dY_ptr, dX_ptr, schedule=B.AMD_MOE_GROUPED, compute_stream=1, secondary_stream=2,
                 first_micro_batch=False):
        """first_micro_batch: the weight gradients are written instead of added to (no cleared buffers needed)."""
        if first_micro_batch:
            schedule |= B.AMD_MOE_FIRST_MICRO_BATCH
        ret = self.be.lib.amd_moe_layer_backward(self.be.hp, compute_stream, secondary_stream, C.byref(self.L), num_tokens,
                                                 X_ptr, dY_ptr, dX_ptr, schedule)
        if ret != 0:
            raise RuntimeError("amd_moe_layer_backward failed")

    def free(self):
        self.be.lib.amd_moe_layer_free(self.be.hp, C.byref(self.L))
