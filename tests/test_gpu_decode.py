"""GPU parity of the decode (sliced-KV) path against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32

from . import gpu_runner, helpers

pytestmark = pytest.mark.gpu


def _decode_case(device, *, hq, hkv, d, tpp, histories, kv_slice, seed, partial_dtype=DTYPE_BF16, **kw):
    q_lens = [1] * len(histories)
    w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=tpp, histories=histories,
                              q_lens=q_lens, seed=seed, **kw)
    _, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 1, kv_slice)
    print(f"decode case hq={hq} hkv={hkv} d={d} tpp={tpp} histories={histories} slice={kv_slice} seed={seed}", flush=True)
    actual, _ = gpu_runner.run_sliced_kv(w, templates, cu, device, partial_dtype=partial_dtype)
    expected = helpers.expected_output(w)
    return helpers.assert_parity(actual, expected, f"decode d={d} tpp={tpp}")


def test_config1_single_sequence_identity_pages(device):
    """Benchmark config 1: batch 1, Hq32/Hkv8/D128, context 1024, page 16, identity page table."""
    stats = _decode_case(device, hq=32, hkv=8, d=128, tpp=16, histories=[1023], kv_slice=256, seed=1, permute=False)
    print(stats)


@pytest.mark.parametrize("partial_dtype", [DTYPE_BF16, DTYPE_F32])
def test_ragged_batch_permuted_pages(device, partial_dtype):
    """Config-2 shape at reduced size: ragged contexts, shared permuted pool, 512-token partitions."""
    _decode_case(device, hq=64, hkv=8, d=128, tpp=16, histories=[511, 700, 1500, 33, 0, 15, 16, 2047], kv_slice=512,
                 seed=2, partial_dtype=partial_dtype)


def test_d256_ratio6(device):
    """Config-3 geometry (Hq24/Hkv4/D256) at reduced context with 2048-token partitions."""
    _decode_case(device, hq=24, hkv=4, d=256, tpp=16, histories=[5000, 2047, 2048, 100], kv_slice=2048, seed=3)


@pytest.mark.parametrize("tpp", [8, 32])
@pytest.mark.parametrize("d", [128, 256])
def test_other_page_sizes(device, d, tpp):
    if d == 128 and tpp == 32:
        pytest.skip("(128, 32) is not a reference profile")
    _decode_case(device, hq=12, hkv=2, d=d, tpp=tpp, histories=[70, 9, 300], kv_slice=64, seed=4 + tpp)


def test_unaligned_slices_and_nan_garbage(device):
    """Slices that do not align with pages, and NaN in every unused page slot."""
    _decode_case(device, hq=16, hkv=2, d=128, tpp=16, histories=[130, 64, 7], kv_slice=65, seed=9, garbage_bits=0x7FC0)


@pytest.mark.parametrize("d", [128, 256])
def test_scores_that_keep_outgrowing_the_running_maximum(device, d):
    """Scores rise steadily along the context: the online softmax has to rescale its accumulators again and again."""
    _decode_case(device, hq=24, hkv=4, d=d, tpp=16, histories=[3000, 511, 40], kv_slice=1024, seed=77, key_drift=0.04)


def test_fused_map_reduce_equals_two_launches(device):
    """One-launch Map+Reduce (the last block of a token merges) matches Map followed by Reduce to within one
    rounding of the merge order, and the oracle to the parity gate, also when launched repeatedly on the same
    self-resetting arrival counters, with and without the gate."""
    import torch

    from khalamari_amd import sdpa, sliced_kv
    from khalamari_amd._lib import ReplayU32
    from oracle import gqa_oracle as oracle

    for hq, hkv, d, histories, kv_slice in [(64, 8, 128, [511, 700, 1500, 33, 0, 2047], 512), (24, 4, 256, [5000, 100, 2048], 1024)]:
        q_lens = [1] * len(histories)
        w = helpers.make_workload(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, tokens_per_page=16, histories=histories,
                                  q_lens=q_lens, seed=77)
        _, templates, cu = helpers.fixed_slice_plan(histories, q_lens, 1, kv_slice)
        expected = helpers.expected_output(w)
        gates = oracle.f32_to_bf16_bits(np.random.default_rng(3).standard_normal((len(histories), hq, d), dtype=np.float32))
        for gate in (None, gates):
            two_launch, _ = gpu_runner.run_sliced_kv(w, templates, cu, device, gates=gate)
            config = gpu_runner.component_config(w, sliced_kv.Config)
            variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), d, 128, min(hq // hkv, 8))
            shape = sliced_kv.Shape(w.num_tokens, templates.shape[0])
            compute = sliced_kv.Compute(config, variant, shape)
            scratch = sliced_kv.Scratch(device, config, shape)
            counters = torch.zeros(compute.arrival_counters_bytes(), dtype=torch.uint8, device=device)
            dev = lambda a: gpu_runner.to_device(a, device)
            args = dict(q=dev(w.q_bits), kv_pages=dev(w.kv_pages), req_slots=dev(w.req_slots), page_ids=dev(w.page_ids),
                        sdpa_map_task_templates=dev(templates), partial_exp_sums=scratch.partial_exp_sums,
                        partial_max_logits=scratch.partial_max_logits, partial_output=scratch.partial_output,
                        cu_sdpa_partial_outputs=dev(cu), arrival_counters=counters, page_table_index=ReplayU32.fixed(0),
                        num_active_tokens=ReplayU32.fixed(w.num_tokens), num_active_kv_splits=ReplayU32.fixed(templates.shape[0]),
                        gates=None if gate is None else dev(gate))
            for repeat in range(3):
                out = torch.full((w.num_tokens, hq, d), 0x4228, dtype=torch.int16, device=device)
                print(f"fused map+reduce d={d} gate={gate is not None} repeat={repeat}", flush=True)
                compute.invoke_map_reduce(output=out, **args)
                torch.cuda.synchronize()
                fused = gpu_runner.bf16_tensor_to_f32(out)
                helpers.assert_parity(fused, two_launch, "fused vs two launches", abs_tol=1e-3, rel_tol=8e-3)
                if gate is None:
                    helpers.assert_parity(fused, expected, "fused vs oracle")
                assert int(counters.view(torch.int32).abs().sum().item()) == 0
