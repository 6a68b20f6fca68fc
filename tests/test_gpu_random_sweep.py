"""Seeded random sweep through the C ABI against the CPU oracle: head geometries, page sizes and formats, page ids per
block, layers, ragged histories and Q lengths, KV slices that are no multiple of anything, partial formats, every kernel
family (split-KV decode, tiled with Reduce, tiled with direct output) over whatever tile variants are legal and built."""
import numpy as np
import pytest

from khalamari_amd import sdpa
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, DTYPE_FP8_E4M3FN, MAP_SLICED_KV

from . import gpu_runner, helpers

HEADS = [(8, 2, 128), (8, 1, 128), (32, 8, 128), (5, 1, 128), (24, 4, 256), (16, 2, 256), (6, 1, 256), (40, 8, 128)]


def _tile_variants(config, kv_dtype, ratio):
    variants = [v for v in sdpa.Registry(config).variants() if v.map_kind != MAP_SLICED_KV and sdpa.has_kernel(config, v, kv_dtype)]
    for kind in (1, 2, 3):
        for max_q_tokens in (1, 2, 4, 8, 16, 32):
            for max_q_heads in sorted({1, 2, 4, min(ratio, 8), ratio}):
                for stage in (16, 32):
                    try:
                        variant = sdpa.ExecutionVariant.sliced_q(config, kind, max_q_tokens, stage, max_q_heads)
                    except Exception:
                        continue
                    if sdpa.supports(variant, config) and sdpa.has_kernel(config, variant, kv_dtype):
                        variants.append(variant)
    return variants


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(7000, 7032))
def test_random_case_matches_oracle(device, seed):
    rng = np.random.default_rng(seed)
    hq, hkv, d = HEADS[rng.integers(len(HEADS))]
    tpp = int(rng.choice([8, 16, 32]))
    fp8 = bool(rng.integers(2))
    page_ids_per_block = int(rng.choice([1, 1, 2]))
    layers = int(rng.choice([1, 2]))
    layer = int(rng.integers(layers))
    requests = int(rng.integers(1, 5))
    mode = str(rng.choice(["decode", "tile", "tile", "direct"]))
    value_scale = float(rng.choice([1.0, 1.0, 0.2]))
    partial_dtype = DTYPE_F32 if rng.integers(4) == 0 else DTYPE_BF16
    config = sdpa.Config(DTYPE_BF16, hq, hkv, d, tpp)
    kv_dtype = DTYPE_FP8_E4M3FN if fp8 else DTYPE_BF16
    histories = [int(rng.integers(0, 2500)) if rng.integers(5) else int(rng.integers(0, 40)) for _ in range(requests)]
    variant = None
    if mode == "decode":
        q_lens = [1] * requests
    else:
        variants = _tile_variants(config, kv_dtype, hq // hkv)
        if not variants:
            pytest.skip(f"no tiled variant is both legal and built for Hq{hq}/Hkv{hkv}/D{d}/page {tpp}")
        variant = variants[rng.integers(len(variants))]
        q_lens = [int(rng.integers(1, 2 * int(variant.map_max_q_tokens) + 2)) for _ in range(requests)]
    kv_slice = int(rng.choice([64, 200, 512, 1000, 4096]))
    what = f"seed {seed}: {mode} Hq{hq}/Hkv{hkv}/D{d} page {tpp} fp8={fp8} ids/block={page_ids_per_block} layer {layer}/{layers} histories={histories} q={q_lens} slice={kv_slice}"
    print(what, flush=True)
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=histories, q_lens=q_lens, seed=seed,
                              num_layers=layers, layer=layer, page_ids_per_block=page_ids_per_block, value_scale=value_scale,
                              garbage_bits=(0x7F if fp8 else 0x7FC0), fp8_pages=fp8)
    expected = helpers.expected_output(w)
    if mode == "decode":
        _, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 1, kv_slice)
        actual, _ = gpu_runner.run_sliced_kv(w, templates, cu, device, partial_dtype=partial_dtype)
    else:
        max_q_tokens = int(variant.map_max_q_tokens)
        ranges, templates, cu = helpers.fixed_slice_plan(histories, q_lens, max_q_tokens, (1 << 30) if mode == "direct" else kv_slice)
        actual = gpu_runner.run_sliced_q(w, ranges, templates, cu, device, kind=int(variant.map_kind), max_q_tokens=max_q_tokens,
                                         max_q_heads=int(variant.map_max_q_heads), stage=int(variant.map_kv_tokens_per_iteration),
                                         direct=(mode == "direct"), partial_dtype=partial_dtype)
    helpers.assert_parity(actual, expected, what)
