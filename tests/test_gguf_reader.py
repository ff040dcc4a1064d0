"""GGUF file -> raw blocks: header parsing, tensor geometry, row / expert ranges, and (on the GPU) the staged upload.

The files are written here, byte by byte, in the layout of the GGUF specification (the reference's own reader test builds
a one-tensor file the same way, tests/test_gguf_iq1m_reader.py:40-57)."""
import struct

import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import block_codec as C
from pocketllm_amd.gguf_reader import GGUFBlockReader

GGML = {"q8_0": 8, "q2_k": 10, "q4_k": 12, "q5_k": 13, "q6_k": 14, "iq2_xxs": 16, "iq4_xs": 23, "iq1_m": 29, "f32": 0}


def _s(text):
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(path, tensors, metadata=(), alignment=32, version=3):
    """tensors: [(name, gguf dims, ggml type id, payload bytes)]; metadata: [(key, value type id, packed value bytes)]."""
    head = bytearray(b"GGUF" + struct.pack("<I", version) + struct.pack("<Q", len(tensors)) + struct.pack("<Q", len(metadata)))
    for key, vtype, packed in metadata:
        head += _s(key) + struct.pack("<I", vtype) + packed
    offsets, pos = [], 0
    for _, _, _, payload in tensors:
        offsets.append(pos)
        pos = (pos + len(payload) + alignment - 1) // alignment * alignment
    for (name, dims, tid, _), off in zip(tensors, offsets):
        head += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<I", tid) + struct.pack("<Q", off)
    while len(head) % alignment:
        head += b"\0"
    data = bytearray()
    for (_, _, _, payload), off in zip(tensors, offsets):
        data += b"\0" * (off - len(data)) + payload
    path.write_bytes(bytes(head + data))


@pytest.fixture()
def sample(tmp_path):
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((24, 512)) * 0.02).astype(np.float32)
    parts = {
        "blk.0.attn_q.weight": ("q4_k", C.quantize_q4_k(w)),
        "blk.0.attn_k.weight": ("q6_k", C.quantize_q6_k(w)),
        "output.weight": ("q8_0", C.pack_q8_0(w[:, :96])),
        "blk.0.ffn_gate_exps.weight": ("iq2_xxs", C.random_iq2_xxs(rng, 3, 16, 2)),
        "blk.0.ffn_down_exps.weight": ("iq1_m", C.random_iq1_m(rng, 3, 32, 1)),
        "blk.0.attn_norm.weight": ("f32", np.ones(512, dtype=np.float32)),
    }
    dims = {"blk.0.attn_q.weight": (512, 24), "blk.0.attn_k.weight": (512, 24), "output.weight": (96, 24),
            "blk.0.ffn_gate_exps.weight": (512, 16, 3), "blk.0.ffn_down_exps.weight": (256, 32, 3), "blk.0.attn_norm.weight": (512,)}
    tensors = [(name, dims[name], GGML[t], np.ascontiguousarray(a).tobytes()) for name, (t, a) in parts.items()]
    metadata = [("general.architecture", 8, _s("test")), ("general.alignment", 4, struct.pack("<I", 64)),
                ("test.layers", 4, struct.pack("<I", 1)), ("test.eps", 6, struct.pack("<f", 1e-5)),
                ("tokenizer.tokens", 9, struct.pack("<I", 8) + struct.pack("<Q", 200) + b"".join(_s(f"t{i}") for i in range(200))),
                ("test.small", 9, struct.pack("<I", 5) + struct.pack("<Q", 3) + struct.pack("<iii", 1, -2, 3))]
    path = tmp_path / "sample.gguf"
    write_gguf(path, tensors, metadata, alignment=64)
    return path, parts


def test_header_metadata_and_geometry(sample):
    path, parts = sample
    with GGUFBlockReader(path) as r:
        assert r.version == 3 and r.alignment == 64 and r.data_offset % 64 == 0
        assert r.metadata["general.architecture"] == "test" and r.metadata["test.layers"] == 1
        assert abs(r.metadata["test.eps"] - 1e-5) < 1e-12 and r.metadata["test.small"] == [1, -2, 3]
        assert r.metadata["tokenizer.tokens"] is None                     # long arrays are skipped, not kept
        assert set(r.tensors) == set(parts)
        info = r.tensors["blk.0.attn_q.weight"]
        assert info.type_name == "q4_k" and info.dimensions == (512, 24) and info.nbytes == 24 * 2 * 144
        assert all(t.absolute_offset % 64 == 0 for t in r.tensors.values())


def test_raw_blocks_are_the_file_bytes(sample):
    path, parts = sample
    with GGUFBlockReader(path) as r:
        for name in ("blk.0.attn_q.weight", "blk.0.attn_k.weight"):
            blocks, type_name, in_dim = r.read_quantized_matrix_blocks(name)
            assert (type_name, in_dim) == (parts[name][0], 512) and blocks.dtype == torch.uint8
            np.testing.assert_array_equal(blocks.numpy(), parts[name][1])
            rows, _, _ = r.read_quantized_matrix_block_rows(name, 5, 7)
            np.testing.assert_array_equal(rows.numpy(), parts[name][1][5:12])
            # the bytes decode to what was quantized
            assert O.rel_l2(O.dequant_rows(blocks.numpy(), type_name, 512), O.dequant_rows(parts[name][1], type_name, 512)) == 0.0
        q8 = r.read_q8_0_blocks("output.weight")
        assert tuple(q8.shape) == (24, 3, 34)
        np.testing.assert_array_equal(q8.numpy(), parts["output.weight"][1])
        np.testing.assert_array_equal(r.read_q8_0_block_rows("output.weight", 20, 4).numpy(), parts["output.weight"][1][20:])
        ex, type_name, in_dim = r.read_routed_layer_blocks("blk.0.ffn_gate_exps.weight")
        assert (type_name, in_dim, tuple(ex.shape)) == ("iq2_xxs", 512, (3, 16, 2, 66))
        np.testing.assert_array_equal(ex.numpy(), parts["blk.0.ffn_gate_exps.weight"][1])
        ex, _, _ = r.read_routed_layer_blocks("blk.0.ffn_down_exps.weight", 1, 2)
        np.testing.assert_array_equal(ex.numpy(), parts["blk.0.ffn_down_exps.weight"][1][1:])
        t = r.quantized_tensor("blk.0.attn_k.weight", row_start=8, row_count=8)
        assert (t.type_name, t.type_id, t.row_elems, t.out_dim, t.row_start) == ("q6_k", 8, 512, 8, 8)


def test_errors_follow_the_reference(sample, tmp_path):
    path, _ = sample
    with GGUFBlockReader(path) as r:
        with pytest.raises(ValueError, match="is not a 2D quantized matrix tensor"):
            r.read_quantized_matrix_blocks("blk.0.ffn_gate_exps.weight")
        with pytest.raises(ValueError, match="is not a routed expert tensor"):
            r.read_routed_layer_blocks("blk.0.attn_q.weight")
        with pytest.raises(ValueError, match="row range"):
            r.read_quantized_matrix_block_rows("blk.0.attn_q.weight", 20, 5)
        with pytest.raises(ValueError, match="expert range"):
            r.read_routed_layer_blocks("blk.0.ffn_gate_exps.weight", 2, 2)
        with pytest.raises(NotImplementedError, match="raw q8_0 blocks"):
            r.read_q8_0_blocks("blk.0.attn_q.weight")
        with pytest.raises(NotImplementedError, match="are not supported"):
            r.read_quantized_matrix_block_rows("output.weight", 0, 1)        # q8_0 has its own readers
        with pytest.raises(KeyError):
            r.read_quantized_matrix_blocks("missing")
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"GGML" + b"\0" * 64)
    with pytest.raises(ValueError, match="not a GGUF file"):
        GGUFBlockReader(bad)
    bad.write_bytes(b"GGUF" + struct.pack("<I", 1) + b"\0" * 64)
    with pytest.raises(ValueError, match="unsupported GGUF version"):
        GGUFBlockReader(bad)
    write_gguf(bad, [("w", (512, 4), GGML["q4_k"], b"\0" * 100)])              # payload shorter than the tensor
    with pytest.raises(ValueError, match="runs past the end"):
        GGUFBlockReader(bad)


@pytest.mark.gpu
def test_upload_feeds_the_kernels(sample):
    from pocketllm_amd.cuda_loader import load_cuda_kernel
    from pocketllm_amd.quantized_ops import QuantizedGGUFLinear
    path, parts = sample
    mod = load_cuda_kernel()
    assert mod is not None
    dev = torch.device("cuda:0")
    with GGUFBlockReader(path) as r:
        t = r.quantized_tensor("blk.0.attn_k.weight", device=dev)
        assert t.blocks.is_cuda
        np.testing.assert_array_equal(t.blocks.cpu().numpy(), parts["blk.0.attn_k.weight"][1])
        x = torch.randn(2, 512, device=dev, dtype=torch.float16)
        y = QuantizedGGUFLinear(t)(x)
        want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(parts["blk.0.attn_k.weight"][1], "q6_k", 512))
        assert np.abs(y.float().cpu().numpy() - want).max() < 2e-2
        ex, _, _ = r.read_routed_layer_blocks("blk.0.ffn_gate_exps.weight", device=dev)
        np.testing.assert_array_equal(ex.cpu().numpy(), parts["blk.0.ffn_gate_exps.weight"][1])


@pytest.mark.gpu
def test_upload_spans_several_staging_chunks(tmp_path):
    rng = np.random.default_rng(9)
    blocks = rng.integers(0, 256, size=(4096, 20, 210), dtype=np.uint8)          # 17 MB: shrink the staging buffers to force chunks
    path = tmp_path / "big.gguf"
    write_gguf(path, [("w", (5120, 4096), GGML["q6_k"], blocks.tobytes())])
    import pocketllm_amd.gguf_reader as G
    old = G._STAGE_BYTES
    G._STAGE_BYTES = 3 << 20
    try:
        with GGUFBlockReader(path) as r:
            got, _, _ = r.read_quantized_matrix_block_rows("w", 100, 3900, device="cuda:0")
            np.testing.assert_array_equal(got.cpu().numpy(), blocks[100:4000])
    finally:
        G._STAGE_BYTES = old
