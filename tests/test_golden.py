"""Golden fixtures under tests/golden/ (inputs built as the reference's component tests build theirs, expected outputs
frozen from the CPU oracle): the oracle still reproduces them exactly (CPU), and the HIP kernels match them through the
C ABI without the oracle being called (GPU)."""
import glob
import os

import numpy as np
import pytest

from oracle import gqa_oracle as oracle

from . import helpers

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
POISON = 0x4228


def _load(name):
    with np.load(os.path.join(GOLDEN, name)) as data:
        return {key: data[key] for key in data.files}


def _paged_ranges_files():
    return sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLDEN, "paged_ranges_*.npz")))


def _ragged_files():
    return sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLDEN, "ragged_decode_*.npz")))


def test_fixtures_are_present():
    assert len(_paged_ranges_files()) >= 4 and len(_ragged_files()) == 2


@pytest.mark.parametrize("name", _paged_ranges_files())
def test_oracle_reproduces_paged_ranges(name):
    f = _load(name)
    d, tpp = int(f["head_dim"]), int(f["tokens_per_page"])
    geom = oracle.Geometry(6, 2, d, tpp, d ** -0.5, 2, 3, 2, oracle.KV_FP8_E4M3FN if int(f["fp8"]) else oracle.KV_BF16)
    for which in ("plain", "windowed"):
        got = oracle.paged_gqa(geom, f["q_bits"][:18], f["kv_pages"], f["req_slots"][:18], f["page_ids"], f[f"visible_{which}"][:18], layer=1)
        assert np.array_equal(got, f[f"expected_{which}"]), (name, which)
    assert not f["expected_windowed"][17].any()      # an empty visible range gives zeros (sliced_q_test.rs:188-190)


@pytest.mark.parametrize("name", _ragged_files())
def test_oracle_reproduces_ragged_decode(name):
    f = _load(name)
    d = int(f["head_dim"])
    geom = oracle.Geometry(8, 2, d, int(f["tokens_per_page"]), float(f["scale"]), 1, 3, 1)
    got = oracle.paged_gqa(geom, f["q_bits"], f["kv_pages"], f["req_slots"], f["page_ids"], f["visible"])
    assert np.array_equal(got, f["expected"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", _paged_ranges_files())
def test_gpu_matches_paged_ranges_fixture(device, name):
    import torch

    from khalamari_amd import sdpa, sliced_kv, sliced_q
    from khalamari_amd._lib import DTYPE_BF16, DTYPE_FP8_E4M3FN, ReplayU32

    from . import gpu_runner

    f = _load(name)
    d, tpp, fp8 = int(f["head_dim"]), int(f["tokens_per_page"]), bool(int(f["fp8"]))
    page_bytes = 2 * 2 * tpp * d * (1 if fp8 else 2)
    config = sliced_q.Config(6, 2, d, d ** -0.5, page_bytes, sliced_kv.Layout(2, 2, 3, 2), DTYPE_BF16,
                             DTYPE_FP8_E4M3FN if fp8 else DTYPE_BF16)
    shape = sliced_q.Shape(20, 4, 8)
    variant = sdpa.ExecutionVariant.sliced_q_per_head(config.sdpa_config(), 16, 16, 2)
    compute = sliced_q.Compute.new(config, variant, shape)
    dev = lambda a: gpu_runner.to_device(a, device)  # noqa: E731
    q, pages, slots, table, ranges, templates, cu = map(dev, (f["q_bits"], f["kv_pages"], f["req_slots"], f["page_ids"], f["q_token_ranges"],
                                                               f["templates"], f["cu"]))
    partial = torch.zeros(config.partial_output_bytes(variant, shape), dtype=torch.uint8, device=device)
    sums = torch.zeros(config.partial_output_stats_bytes(variant, shape), dtype=torch.uint8, device=device)
    maxs = torch.zeros_like(sums)
    for which in ("plain", "windowed"):
        print(f"golden {name} {which}", flush=True)
        out = torch.full((20, 6, d), POISON, dtype=torch.int16, device=device)
        compute.invoke_map(q=q, kv_pages=pages, req_slots=slots, page_ids=table, visible_kv_token_ranges=dev(f[f"visible_{which}"]),
                           q_token_ranges=ranges, sdpa_map_task_templates=templates, partial_output=partial, partial_exp_sums=sums,
                           partial_max_logits=maxs, page_table_index=ReplayU32.fixed(1), num_active_tokens=ReplayU32.fixed(18),
                           num_active_q_token_tiles=ReplayU32.fixed(3), num_active_kv_splits=ReplayU32.fixed(6))
        compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, q_token_ranges=ranges,
                              cu_sdpa_partial_outputs=cu, output=out, num_active_q_token_tiles=ReplayU32.fixed(3))
        torch.cuda.synchronize()
        actual = gpu_runner.bf16_tensor_to_f32(out)
        helpers.assert_parity(actual[:18], f[f"expected_{which}"], f"{name} {which}")
        assert np.all(out[18:].cpu().numpy() == POISON)


@pytest.mark.gpu
@pytest.mark.parametrize("name", _ragged_files())
def test_gpu_matches_ragged_decode_fixture(device, name):
    import torch

    from khalamari_amd import sdpa, sliced_kv
    from khalamari_amd._lib import ReplayU32

    from . import gpu_runner

    f = _load(name)
    d, tpp = int(f["head_dim"]), int(f["tokens_per_page"])
    config = sliced_kv.Config(8, 2, d, float(f["scale"]), 2 * 2 * tpp * d * 2, sliced_kv.Layout(2, 1, 3, 1))
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), d, 128, 4)
    shape = sliced_kv.Shape(2, 4)
    compute = sliced_kv.Compute(config, variant, shape)
    scratch = sliced_kv.Scratch(device, config, shape)
    dev = lambda a: gpu_runner.to_device(a, device)  # noqa: E731
    out = torch.zeros((2, 8, d), dtype=torch.int16, device=device)
    print(f"golden {name}", flush=True)
    compute.invoke_map(q=dev(f["q_bits"]), kv_pages=dev(f["kv_pages"]), req_slots=dev(f["req_slots"]), page_ids=dev(f["page_ids"]),
                       sdpa_map_task_templates=dev(f["templates"]), partial_exp_sums=scratch.partial_exp_sums,
                       partial_max_logits=scratch.partial_max_logits, partial_output=scratch.partial_output,
                       page_table_index=ReplayU32.fixed(0), num_active_tokens=ReplayU32.fixed(2), num_active_kv_splits=ReplayU32.fixed(4))
    compute.invoke_reduce(partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                          partial_output=scratch.partial_output, cu_sdpa_partial_outputs=dev(f["cu"]), output=out,
                          num_active_tokens=ReplayU32.fixed(2))
    torch.cuda.synchronize()
    helpers.assert_parity(gpu_runner.bf16_tensor_to_f32(out), f["expected"], name)
