"""GPU parity on FP8 E4M3FN K/V pages (the reference's production cache format) against the CPU oracle, through the
C ABI.  K/V are quantised to FP8 before the oracle sees them, as in the reference's tests (sliced_kv_test.rs:171-182,
484-493), so the gate is the bf16 one: |a - e| <= 2e-3 + 1e-2 |e|."""
import numpy as np
import pytest

from khalamari_amd import _lib, sdpa, sliced_q
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, DTYPE_FP8_E4M3FN

from . import gpu_runner, helpers

pytestmark = pytest.mark.gpu


def _decode_case(device, *, hq, hkv, d, tpp, histories, kv_slice, seed, partial_dtype=DTYPE_BF16, **kw):
    q_lens = [1] * len(histories)
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=histories, q_lens=q_lens,
                              seed=seed, fp8_pages=True, **kw)
    _, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 1, kv_slice)
    print(f"fp8 decode case hq={hq} hkv={hkv} d={d} tpp={tpp} histories={histories} slice={kv_slice} seed={seed}", flush=True)
    actual, _ = gpu_runner.run_sliced_kv(w, templates, cu, device, partial_dtype=partial_dtype)
    return helpers.assert_parity(actual, helpers.expected_output(w), f"fp8 decode d={d} tpp={tpp}")


def test_fp8_decode_d128(device):
    """The 35B geometry: Hq64/Hkv8/D128, 16 tokens per 32 KiB page, ragged batch, 512-token partitions."""
    w_page = 2 * 8 * 16 * 128
    assert w_page == 32 * 1024
    print(_decode_case(device, hq=64, hkv=8, d=128, tpp=16, histories=[511, 700, 1500, 33, 0, 15, 16, 2047], kv_slice=512, seed=21))


@pytest.mark.parametrize("partial_dtype", [DTYPE_BF16, DTYPE_F32])
def test_fp8_decode_d256(device, partial_dtype):
    """The 27B geometry: Hq24/Hkv4/D256, 16 tokens per 32 KiB page."""
    print(_decode_case(device, hq=24, hkv=4, d=256, tpp=16, histories=[5000, 2047, 2048, 100], kv_slice=2048, seed=22,
                       partial_dtype=partial_dtype))


@pytest.mark.parametrize("d,tpp", [(128, 8), (256, 8), (256, 32)])
def test_fp8_other_page_sizes(device, d, tpp):
    _decode_case(device, hq=12, hkv=2, d=d, tpp=tpp, histories=[70, 9, 300], kv_slice=64, seed=23 + tpp)


def test_fp8_unaligned_slices_and_nan_garbage(device):
    """Slices that do not align with pages, and the FP8 NaN code in every unused page slot."""
    _decode_case(device, hq=16, hkv=2, d=128, tpp=16, histories=[130, 64, 7], kv_slice=65, seed=29, garbage_bits=0x7F)


def test_fp8_spec_verify_blocks(device):
    """q_len 2..5 causal blocks over FP8 pages: sliced-Q tiles of 17..64 coordinates run on the LDS-tiled kernel that keeps
    the raw FP8 codes in LDS and decodes the fragments it reads."""
    histories, q_lens = [300, 17, 1000, 64], [2, 5, 3, 4]
    w = helpers.make_workload(num_q_heads=32, num_kv_heads=4, head_dim=128, tokens_per_page=16, histories=histories, q_lens=q_lens,
                              seed=33, fp8_pages=True)
    ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 8, 256)
    expected = helpers.expected_output(w)
    for direct in (False,):
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=8, max_q_heads=8,
                                         direct=direct)
        helpers.assert_parity(actual, expected, "fp8 verify")


@pytest.mark.parametrize("tpp", [8, 16, 32])
def test_fp8_spec_verify_blocks_at_head_dim_256(device, tpp):
    """The same blocks at head dim 256 (Hq16/Hkv2, tiles of 8 tokens x 8 heads = 64 coordinates): raw rows of 256 bytes in
    LDS, swizzled by row & 15 on both planes; split into 256- and 100-token slices + Reduce, and unsplit with direct output."""
    histories, q_lens = [300, 17, 1000, 64], [2, 5, 3, 4]
    w = helpers.make_workload(num_q_heads=16, num_kv_heads=2, head_dim=256, tokens_per_page=tpp, histories=histories, q_lens=q_lens,
                              seed=35 + tpp, fp8_pages=True, garbage_bits=0x7F)
    expected = helpers.expected_output(w)
    for kv_slice, direct in [(256, False), (100, False), (1 << 20, True)]:
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 8, kv_slice)
        print(f"fp8 verify d=256 tpp={tpp} kv_slice={kv_slice} direct={direct}", flush=True)
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=8, max_q_heads=8,
                                         direct=direct)
        helpers.assert_parity(actual, expected, f"fp8 verify d=256 tpp={tpp} slice={kv_slice} direct={direct}")


@pytest.mark.parametrize("hq,hkv,d,tile", [(64, 8, 128, 32), (32, 4, 128, 16), (24, 4, 256, 16), (16, 2, 256, 32), (24, 4, 256, 32),
                                           (12, 2, 256, 32)])
def test_fp8_chunked_prefill_onto_a_paged_prefix(device, hq, hkv, d, tile):
    """Causal chunks appended to paged prefixes on FP8 pages: wide Q tiles on the LDS-tiled kernel, whose tiles are
    decoded on their way into LDS; direct output and split-KV + Reduce; the FP8 NaN code in every unused page slot."""
    histories = [0, 333, 1000]
    q_lens = [150, 64, 37]
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=16, histories=histories, q_lens=q_lens,
                              seed=190 + tile, garbage_bits=0x7F, fp8_pages=True)
    expected = helpers.expected_output(w)
    for kv_slice, direct in [(1 << 20, True), (256, False), (100, False)]:
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, tile, kv_slice)
        print(f"fp8 prefill hq={hq} hkv={hkv} d={d} tile={tile} kv_slice={kv_slice} direct={direct}", flush=True)
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=tile,
                                         max_q_heads=hq // hkv, stage=64, direct=direct)
        helpers.assert_parity(actual, expected, f"fp8 prefill tile={tile} slice={kv_slice} direct={direct}")


def test_fp8_long_interior_runs_of_the_twelve_wave_tile_checked_on_every_row(device):
    """Hq12/Hkv2/D256 (six Q heads per KV head, 32-token tiles: 192 columns on twelve waves) over FP8 pages with prefixes of
    a few thousand keys, so that the steady-state loop of the register-staged FP8 tiles carries nearly every tile."""
    histories, q_lens = [3000, 1531], [70, 40]
    w = helpers.make_workload(num_q_heads=12, num_kv_heads=2, head_dim=256, tokens_per_page=16, histories=histories, q_lens=q_lens,
                              seed=611, garbage_bits=0x7F, fp8_pages=True)
    expected = helpers.expected_output(w)
    for kv_slice, direct in [(1 << 20, True), (1024, False)]:
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 32, kv_slice)
        print(f"fp8 twelve-wave tile kv_slice={kv_slice} direct={direct}", flush=True)
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=32, max_q_heads=6,
                                         stage=64, direct=direct)
        helpers.assert_parity(actual, expected, f"fp8 twelve-wave tile slice={kv_slice} direct={direct}")


@pytest.mark.parametrize("tpp", [8, 32])
def test_fp8_prefill_other_page_sizes(device, tpp):
    histories, q_lens = [77, 0], [70, 33]
    w = helpers.make_workload(num_q_heads=16, num_kv_heads=2, head_dim=256, tokens_per_page=tpp, histories=histories, q_lens=q_lens,
                              seed=195 + tpp, fp8_pages=True)
    ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 32, 1 << 20)
    actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=sdpa.MAP_Q_TOKENS_AND_HEADS, max_q_tokens=32, max_q_heads=8,
                                     stage=64, direct=True)
    helpers.assert_parity(actual, helpers.expected_output(w), f"fp8 prefill tpp={tpp}")
