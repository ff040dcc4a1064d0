"""CPU-only checks: the C-ABI library loads and exports what include/pllm_hip.h declares, the ctypes
table matches the header, and the host-side helpers (encoders, codebooks, loader contract) behave."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import _ffi, block_codec as C, codebooks, cuda_loader, quant_types

ROOT = Path(__file__).resolve().parents[1]
HEADER = (ROOT / "include" / "pllm_hip.h").read_text()


def _declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(pllm_[a-z0-9_]+)\s*\(", text)))


def test_header_and_ctypes_table_agree():
    assert _declared() == sorted(_ffi.SIGNATURES)


def test_every_declaration_cites_the_reference_or_says_it_has_no_counterpart():
    for name in _declared():
        pos = HEADER.index(name + "(")
        comment = HEADER[:pos].rsplit("/*", 1)[-1]
        if name in ("pllm_status_string", "pllm_abi_version") or name.endswith("_workspace_bytes") or name == "pllm_fp8_block_gemm":
            continue        # documented together with their neighbours
        assert ("src/" in comment) or ("cpp_engine/" in comment) or ("no counterpart" in comment), name


@pytest.mark.skipif(not _ffi.LIB_PATH.exists(), reason="libpllm_hip.so not built")
def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(_ffi.LIB_PATH))
    for name in _declared():
        assert hasattr(lib, name), name
    loaded = _ffi.load_library()
    assert loaded.pllm_abi_version() >= 1
    assert [loaded.pllm_gguf_block_bytes(t) for t in range(5)] == [66, 84, 56, 144, 176]
    assert loaded.pllm_gguf_block_bytes(9) == 0
    assert loaded.pllm_status_string(-4) == b"workspace too small"
    # pure host arithmetic of the ABI
    assert loaded.pllm_gguf_quant_gemm_workspace_bytes(3, 1, 5120, 5120, 20) >= 5120 * 2.5
    assert loaded.pllm_gguf_quant_gemm_workspace_bytes(42, 1, 5120, 5120, 20) == 0
    assert loaded.pllm_gguf_moe_workspace_bytes(1, 8, 3072, 1536) > 8 * 3072 * 4


def test_loader_contract_module_or_none(monkeypatch, tmp_path):
    monkeypatch.setattr(cuda_loader, "_NATIVE_MOD", None)
    monkeypatch.setattr(_ffi, "_LIB", None)
    monkeypatch.setattr(_ffi, "LIB_PATH", tmp_path / "missing.so")
    assert cuda_loader.load_cuda_kernel() is None
    from pocketllm_amd.quantized_ops import Q8_0GGUFLinear
    with pytest.raises(RuntimeError, match="native HIP library is required"):
        Q8_0GGUFLinear(torch.zeros(2, 1, 34, dtype=torch.uint8), 32)
    from pocketllm_amd import ops
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.q8_0_weight_gemm(torch.zeros(1, 32), torch.zeros(2, 1, 34, dtype=torch.uint8))


@pytest.mark.skipif(not _ffi.LIB_PATH.exists(), reason="libpllm_hip.so not built")
def test_operator_names_of_the_reference_extension_exist():
    mod = cuda_loader.load_cuda_kernel()
    for name in ("q8_0_gemm_forward", "gguf_quant_gemm_forward", "gguf_quant_gemm_prefill_forward", "gguf_quant_gemm_pair_forward",
                 "gguf_quant_embedding_forward", "gguf_q2k_gemm_dp4a_forward", "gguf_moe_prefill_grouped_forward",
                 "gguf_moe_single_token_iq2_q2k_forward", "gguf_moe_single_token_iq1m_forward", "moe_group_routes",
                 "gguf_single_token_route_slots"):
        assert hasattr(mod, name), name


@pytest.mark.skipif(not _ffi.LIB_PATH.exists(), reason="libpllm_hip.so not built")
def test_argument_checks_run_before_any_gpu_work():
    mod = cuda_loader.load_cuda_kernel()
    x = torch.zeros(1, 512)
    blocks = torch.zeros(4, 2, 144, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="x and blocks must be CUDA tensors"):
        mod.gguf_quant_gemm_forward(x, blocks, 512, 3, torch.empty(0, dtype=torch.int8))
    with pytest.raises(RuntimeError, match="all tensors must be CUDA tensors"):
        mod.q8_0_gemm_forward(x, torch.zeros(4, 16, 34, dtype=torch.uint8), 512)


def test_type_table():
    assert quant_types.GGUF_DENSE_TYPE_IDS["q4_k"] == 3 and quant_types.GGUF_DENSE_TYPE_NAMES[2] == "iq1_m"
    assert quant_types.block_bytes_for_type(4) == 176
    with pytest.raises(RuntimeError, match="unsupported GGUF quant type_id"):
        quant_types.block_bytes_for_type(17)


def test_codebooks_agree_with_oracle_copy():
    np.testing.assert_array_equal(codebooks.iq2xxs_signed_grid(), O.iq2xxs_signed_grid())
    np.testing.assert_array_equal(codebooks.iq1_grid(), O.iq1_grid_i8())
    assert tuple(codebooks.get_iq2xxs_signed_grid_tensor().shape) == (256, 128, 8)
    assert codebooks.get_iq1_grid_tensor().dtype == torch.int8
    np.testing.assert_array_equal(codebooks.iq2xs_grid(), O.iq2xs_grid_u8())
    np.testing.assert_array_equal(codebooks.iq3xxs_grid(), O.iq3xxs_grid_u8())
    # the packed tensor for type ids 5 and 6: entry x sign pattern, IQ3_XXS entries doubled under the two sign halves
    packed = codebooks.get_iq2xs_iq3xxs_signed_grid_tensor()
    assert packed.dtype == torch.int8 and packed.numel() == 512 * 128 * 8 + 256 * 128 * 8
    xs, xxs = codebooks.iq2xs_signed_grid(), codebooks.iq3xxs_signed_grid()
    ks = codebooks.ksigns()
    for g, s_ in ((0, 0), (511, 127), (300, 77)):
        sign = np.where((ks[s_] >> np.arange(8)) & 1, -1, 1)
        np.testing.assert_array_equal(xs[g, s_], O.iq2xs_grid_u8()[g].astype(np.int16) * sign)
        np.testing.assert_array_equal(xxs[g % 256, s_], np.tile(O.iq3xxs_grid_u8()[g % 256].astype(np.int16), 2) * sign)
    assert codebooks.grid_tensor_for_type(3).numel() == 0 and codebooks.grid_tensor_for_type(6).numel() == packed.numel()


@pytest.mark.parametrize("name,enc,bits", [("q4_k", C.quantize_q4_k, 4), ("q5_k", C.quantize_q5_k, 5), ("q2_k", C.quantize_q2_k, 2)])
def test_kquant_encoders_round_trip(name, enc, bits):
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((8, 700)) * 0.02).astype(np.float32)       # ragged K: padded with zeros
    blocks = enc(w)
    assert blocks.shape == (8, 3, O.BLOCK_BYTES[name]) and blocks.dtype == np.uint8
    back = O.dequant_rows(blocks, name, 700)
    err = np.abs(back - w).max()
    assert err < 0.1 * 2.0 ** (4 - bits) * 0.02 * 4 + 1e-3, err


def test_q8_0_packer_matches_reference_recipe():
    rng = np.random.default_rng(4)
    w = rng.standard_normal((5, 70)).astype(np.float32)
    blocks = C.pack_q8_0(w)
    assert blocks.shape == (5, 3, 34)
    # the recipe of tests/test_q8_0_cuda.py:12-24, restated with torch
    padded = torch.zeros(5, 96)
    padded[:, :70] = torch.from_numpy(w)
    view = padded.view(5, 3, 32)
    scales = view.abs().amax(dim=2).clamp_min(1e-6) / 127.0
    q = torch.clamp(torch.round(view / scales.unsqueeze(-1)), -127, 127).to(torch.int8)
    np.testing.assert_array_equal(blocks[..., 2:], q.numpy().view(np.uint8))
    np.testing.assert_array_equal(blocks[..., :2], scales.to(torch.float16).view(torch.uint8).view(5, 3, 2).numpy())


def test_fp8_block_encoder():
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((130, 260)) * 0.02).astype(np.float32)
    codes, scale = C.quantize_fp8_block(w)
    assert codes.shape == (130, 260) and scale.shape == (2, 3)
    back = O.dequant_fp8_block(codes, scale)
    assert np.abs(back - w).max() <= np.abs(w).max() / 448 * 16 + 1e-9      # half an ulp at 3 mantissa bits
    assert ((codes & 0x7f) != 0x7f).all()


def test_random_iq_blocks_have_finite_scales():
    rng = np.random.default_rng(6)
    for name, gen in (("iq2_xxs", C.random_iq2_xxs), ("iq1_m", C.random_iq1_m)):
        blocks = gen(rng, 3, 2)
        vals = O.dequant_rows(blocks, name)
        assert np.isfinite(vals).all() and vals.std() > 0


def test_product_never_touches_the_oracle():
    """The oracle is test infrastructure: nothing under the package imports, reads or links it."""
    import pathlib
    root = pathlib.Path(__file__).resolve().parents[1] / "pocketllm_amd"
    for path in list(root.glob("*.py")) + list((root / "csrc").glob("*")):
        if path.is_file() and path.suffix in (".py", ".hip", ".h", ".inc"):
            assert "oracle" not in path.read_text(errors="replace"), path.name
