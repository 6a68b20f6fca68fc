"""The C-ABI library loads, exports every symbol the header declares, and its host codec matches the oracle."""
import os
import re

import numpy as np
import pytest

from khalamari_amd import _lib
from oracle import gqa_oracle as oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "khm_gqa_sdpa.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(khm_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations parsed"
    lib = _lib.lib()
    missing = sorted(name for name in declared if not hasattr(lib, name))
    assert not missing, f"declared in the header but not exported: {missing}"
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    assert b"gfx950" in lib.khm_version()


def test_reference_side_binding_lists_every_declared_function():
    """The Rust `extern "C"` block a maintainer would add, kept beside the header in the integration notes, names every function of the header."""
    header = open(os.path.join(ROOT, "include", "khm_gqa_sdpa.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(khm_[a-z0-9_]+)\s*\(", header))
    binding = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    bound = set(re.findall(r"pub fn (khm_[a-z0-9_]+)\(", binding))
    assert declared == bound, f"only in the header: {sorted(declared - bound)}; only in the binding: {sorted(bound - declared)}"


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libkhm_gqa_sdpa.so")
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        _lib.lib()


def test_host_fp8_codec_matches_oracle_exhaustively():
    lib = _lib.lib()
    ours = np.array([lib.khm_bf16_to_fp8_e4m3(code) for code in range(65536)], dtype=np.uint8)
    theirs = oracle.bf16_bits_to_fp8(np.arange(65536, dtype=np.uint32).astype(np.uint16))
    assert np.array_equal(ours, theirs)
    decode = np.array([lib.khm_fp8_e4m3_to_bf16(code) for code in range(256)], dtype=np.uint16)
    assert np.array_equal(decode, oracle.fp8_decode_table())


def test_host_bf16_conversion_matches_oracle():
    lib = _lib.lib()
    rng = np.random.default_rng(1)
    values = np.concatenate([rng.standard_normal(2000).astype(np.float32) * 100, np.array([np.inf, -np.inf, 0.0, -0.0, 1.00390625], dtype=np.float32)])
    ours = np.array([lib.khm_f32_to_bf16(float(v)) for v in values], dtype=np.uint16)
    assert np.array_equal(ours, oracle.f32_to_bf16_bits(values))
    assert lib.khm_f32_to_bf16(float("nan")) & 0x7FC0 == 0x7FC0
    assert lib.khm_bf16_to_f32(0x3FC0) == 1.5


def test_fp8_torch_cross_check_in_the_finite_range():
    import torch

    table = oracle.fp8_decode_table()
    finite = np.array([c for c in range(256) if c & 0x7F != 0x7F], dtype=np.uint8)
    as_f32 = torch.from_numpy(finite.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(oracle.bf16_bits_to_f32(table[finite]), as_f32)
    rng = np.random.default_rng(2)
    values = oracle.bf16_round((rng.standard_normal(50000) * 50).astype(np.float32))
    values = values[np.abs(values) <= 448.0]
    ours = oracle.bf16_bits_to_fp8(oracle.f32_to_bf16_bits(values))
    theirs = torch.from_numpy(values).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(ours, theirs)
