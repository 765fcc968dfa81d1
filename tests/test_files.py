"""The reference's on-disk formats as far as the MoE layer meets them: the per-block weight file
(`combined_layer.weight`, models/init_model.py:205-318 writes it, prep_transformer.c:24-165 + 366-388 lay the block
out and read it) and the naming of saved arrays (dataflow_transformer.c:46-160).

The expected layout is derived here from the writer's side (the arrays init_model.py concatenates, in its order),
not from the C restatement under test; the GPU test loads a file written that way and runs the layer on it.
"""
import ctypes as C
import os

import numpy as np
import pytest

from ml_dataflow_amd import binding as B
from util import normal_bf16


def writer_arrays(rng, D, attn_dim, kv_dim, E, H):
    """The arrays of one block in the order init_model.py appends them to `all_weights` (:205-316)."""
    u = lambda *shape: normal_bf16(rng, shape, 0.02)
    arrays = [("w_attn_norm", u(D)), ("w_q", u(D, attn_dim)), ("w_k", u(D, kv_dim)), ("w_v", u(D, kv_dim)), ("w_o", u(attn_dim, D)),
              ("w_ffn_norm", u(D)), ("w_router", u(E, D))]
    for e in range(E):
        arrays += [("w_1_%d" % e, u(H, D)), ("w_3_%d" % e, u(H, D)), ("w_2_%d" % e, u(D, H))]
    return arrays


@pytest.fixture(scope="module")
def lib():
    return B.load_library()


@pytest.mark.parametrize("D,attn_dim,kv_dim,E,H,align", [(4096, 4096, 1024, 64, 1024, 256), (512, 512, 128, 8, 1024, 256), (128, 128, 64, 4, 64, 256),
                                                        (2048, 2048, 512, 1, 1408, 256), (128, 128, 64, 3, 64, 0)])
def test_offsets_equal_the_writer_side_layout(lib, D, attn_dim, kv_dim, E, H, align):
    """Every size here is a multiple of the alignment, so the file the writer makes by plain concatenation and the
    aligned buffer the reader lays out coincide: offsets must equal the running sum of the array sizes."""
    off = B.AmdMoeBlockOffsets()
    assert lib.amd_moe_block_weight_offsets(D, attn_dim, kv_dim, E, H, B.DATAFLOW_BF16, align, C.byref(off)) == 0
    sizes = [D, D * attn_dim, D * kv_dim, D * kv_dim, attn_dim * D, D, E * D] + [H * D, H * D, D * H] * E
    starts = np.concatenate([[0], np.cumsum(np.array(sizes, dtype=np.int64) * 2)])
    got = [off.w_attn_norm, off.w_q, off.w_k, off.w_v, off.w_o, off.w_ffn_norm, off.w_router, off.w_1, off.w_3, off.w_2]
    assert got == list(starts[:10])
    assert off.expert_stride == 3 * H * D * 2
    assert off.raw_size == off.aligned_size == starts[-1]


def test_offsets_round_up_to_the_alignment(lib):
    """model_dim 24 bf16 = 48 bytes per norm weight: each array starts at the next multiple of 256, as set_offset does
    (prep_transformer.c:3-20); the raw size stays the plain sum."""
    off = B.AmdMoeBlockOffsets()
    D, A, KV, E, H = 24, 24, 8, 2, 40
    assert lib.amd_moe_block_weight_offsets(D, A, KV, E, H, B.DATAFLOW_BF16, 256, C.byref(off)) == 0
    up = lambda v: (v + 255) // 256 * 256
    cur, want = 0, []
    for size in [D, D * A, D * KV, D * KV, A * D, D, E * D] + [H * D, H * D, D * H] * E:
        want.append(cur)
        cur = up(cur + size * 2)
    assert [off.w_attn_norm, off.w_q, off.w_k, off.w_v, off.w_o, off.w_ffn_norm, off.w_router, off.w_1, off.w_3, off.w_2] == want[:10]
    assert off.expert_stride == want[10] - want[7] and off.aligned_size == cur
    assert off.raw_size == 2 * (2 * D + 2 * D * A + 2 * D * KV + E * D + 3 * E * H * D)
    assert lib.amd_moe_block_weight_offsets(D, A, KV, 0, H, B.DATAFLOW_BF16, 256, C.byref(off)) == -1
    assert lib.amd_moe_block_weight_offsets(D, A, KV, E, H, B.DATAFLOW_NONE, 256, C.byref(off)) == -1


def test_saved_array_paths_follow_the_reference_scheme(lib):
    def path(layer, seq, chunk, bwd, name):
        buf = C.create_string_buffer(1024)
        assert lib.amd_moe_saved_array_path(buf, 1024, b"test_transformer_data", layer, seq, chunk, bwd, name) == 0
        return buf.value.decode()
    assert path(3, 0, 2, 0, b"x_routed") == "test_transformer_data/layers_fwd/3/seq_0_chunk_2_x_routed.dat"
    assert path(3, 7, 0, 1, b"x_upstream_grad") == "test_transformer_data/layers_bwd/3/seq_7_chunk_0_x_upstream_grad.dat"
    assert path(5, -1, -1, 1, b"w_2") == "test_transformer_data/model_grads/layers/5/w_2.dat"
    assert path(5, -1, -1, 0, b"w_router") == "test_transformer_data/model/layers/5/w_router.dat"
    assert path(-2, 1, 0, 0, b"x_embedding") == "test_transformer_data/embedding_fwd/seq_1_chunk_0_x_embedding.dat"
    assert path(-1, 1, 0, 1, b"x_logits_loss") == "test_transformer_data/head_bwd/seq_1_chunk_0_x_logits_loss.dat"
    assert path(-1, -1, -1, 1, b"w_head") == "test_transformer_data/model_grads/head/w_head.dat"
    buf = C.create_string_buffer(16)
    assert lib.amd_moe_saved_array_path(buf, 16, b"test_transformer_data", 0, 0, 0, 0, b"x") == -1      # does not fit
    assert lib.amd_moe_saved_array_path(buf, 16, b"d", -3, 0, 0, 0, b"x") == -1


@pytest.mark.gpu
def test_block_file_loads_and_saved_arrays_round_trip(backend, tmp_path):
    """A block file written the way init_model.py writes it, loaded with amd_moe_layer_load_block_file, gives the same
    layer output (bit for bit) as the same weights uploaded array by array; arrays saved with amd_moe_save_array read
    back as the device contents; a truncated file is an error."""
    from ml_dataflow_amd import MoeLayer
    be = backend
    T, D, E, K, H, attn_dim, kv_dim = 200, 256, 8, 2, 384, 256, 64
    rng = np.random.default_rng(11)
    arrays = writer_arrays(rng, D, attn_dim, kv_dim, E, H)
    block = tmp_path / "combined_layer.weight"
    np.concatenate([a.reshape(-1) for _, a in arrays]).tofile(block)
    named = dict(arrays)
    Wr = named["w_router"]
    W1 = np.stack([named["w_1_%d" % e] for e in range(E)])
    W3 = np.stack([named["w_3_%d" % e] for e in range(E)])
    W2 = np.stack([named["w_2_%d" % e] for e in range(E)])
    X, resid = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    d_X = be.upload(X)
    outs = []
    for from_file in (False, True):
        layer = MoeLayer(be, T, D, E, K, H)
        d_norm = be.alloc(D * 2)
        if from_file:
            assert be.lib.amd_moe_layer_load_block_file(be.hp, 0, C.byref(layer.L), str(block).encode(), attn_dim, kv_dim, 256, d_norm.ptr) == 0
            assert (be.read(d_norm.ptr, (D,), np.uint16) == named["w_ffn_norm"]).all()
        else:
            layer.load_weights(Wr, W1, W3, W2)
        d_out = be.upload(resid)
        layer.forward(T, d_X.ptr, d_out.ptr)
        be.sync()
        outs.append(be.read(d_out.ptr, (T, D), np.uint16))
        if from_file:
            save_dir = tmp_path / "saved"
            os.makedirs(save_dir / "layers_fwd" / "0")
            assert be.lib.amd_moe_save_array(be.hp, 1, str(save_dir).encode(), 0, 0, 0, 0, b"x_routed", layer.L.x_routed, T, E, B.DATAFLOW_BF16) == 0
            got = np.fromfile(save_dir / "layers_fwd" / "0" / "seq_0_chunk_0_x_routed.dat", dtype=np.uint16).reshape(T, E)
            assert (got == be.read(layer.L.x_routed, (T, E), np.uint16)).all()
            assert be.lib.amd_moe_save_array(be.hp, 1, str(tmp_path / "missing").encode(), 0, 0, 0, 0, b"x", layer.L.x_routed, T, E, B.DATAFLOW_BF16) == -1
            short = tmp_path / "short.weight"
            np.concatenate([a.reshape(-1) for _, a in arrays])[:-8].tofile(short)
            assert be.lib.amd_moe_layer_load_block_file(be.hp, 0, C.byref(layer.L), str(short).encode(), attn_dim, kv_dim, 256, None) == -1
            assert be.lib.amd_moe_layer_load_block_file(be.hp, 0, C.byref(layer.L), b"/nonexistent/file", attn_dim, kv_dim, 256, None) == -1
        layer.free()
    assert (outs[0] == outs[1]).all()
