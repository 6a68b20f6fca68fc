"""The projection split, Q RMSNorm + RoPE, K RMSNorm + RoPE and the K/V page write as one launch
(khm_gqa_projection_norm_rope_page_write): q_output, gate_output and the pages must hold exactly the bytes that the separate
calls leave there in the order GQA::record enqueues them (crates/inference-executor-metal/src/attn/gqa/backend.rs:358-412):
khm_gqa_qgkv_split (or khm_gqa_qkv_split), khm_rms_norm_rope on the Q rows, khm_k_norm_rope_page_write on the K and V rows."""
import ctypes

import numpy as np
import pytest

from khalamari_amd import _lib
from khalamari_amd import k_norm_rope_page_write as k_writer
from khalamari_amd import kv_page_write as kpw
from khalamari_amd import projection_norm_rope_page_write as prologue
from khalamari_amd import qgkv_split, qkv_split
from khalamari_amd import rms_norm_rope as rnr
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, DTYPE_FP8_E4M3FN, KhmError, ReplayU32
from oracle import gqa_oracle as oracle

YARN = dict(factor=32.0, attention_factor=float(np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0))), beta_fast=32.0,
            beta_slow=1.0, original_max_position_embeddings=8192, truncate=True)
POISON = 0x4228


def _case(hq, hkv, dim, kv_dtype, seed, tokens, gated):
    rng = np.random.default_rng(seed)
    element = 1 if kv_dtype == DTYPE_FP8_E4M3FN else 2
    tokens_per_page, layers, blocks, per_block, slots = 16, 2, 3, 2, 3
    page_bytes = 2 * hkv * tokens_per_page * dim * element
    num_pages = slots * layers * blocks * per_block
    pairs = rng.permutation(slots * blocks * per_block * tokens_per_page)[:tokens]   # distinct (slot, position): no two writes share a row
    width = ((2 if gated else 1) * hq + 2 * hkv) * dim
    return dict(hq=hq, hkv=hkv, dim=dim, kv_dtype=kv_dtype, layers=layers, blocks=blocks, per_block=per_block, slots=slots, tokens=tokens,
                page_bytes=page_bytes, gated=gated, width=width, page_ids=rng.permutation(num_pages).astype(np.uint32),
                req_slots=(pairs % slots).astype(np.uint32), positions=(pairs // slots).astype(np.uint32),
                projection=oracle.f32_to_bf16_bits((rng.standard_normal((tokens, width)) * 3.0).astype(np.float32)),
                q_weight=(0.75 + rng.random(dim) * 0.5).astype(np.float32), k_weight=(0.75 + rng.random(dim) * 0.5).astype(np.float32),
                pages=rng.integers(0, 256, size=num_pages * page_bytes, dtype=np.uint8))


def _configs(case, rope_dim, weight_dtype, yarn):
    def norm(heads, eps):
        config = rnr.Config.bf16(heads, case["dim"], rope_dim, eps, 10_000_000.0).with_norm_weight_dtype(weight_dtype)
        return config.with_rope_scaling(rnr.Yarn(**YARN)) if yarn else config
    page = kpw.Config(case["hkv"], case["dim"], case["page_bytes"], kv_dtype=case["kv_dtype"])
    shape = kpw.Shape(case["tokens"], kpw.PageTableLayout(case["slots"], case["layers"], case["blocks"], case["per_block"]))
    return norm(case["hq"], 1e-6), norm(case["hkv"], 3e-6), page, shape   # the two norms may differ in eps


def _run(device, case, rope_dim, weight_dtype, yarn, active, layer, fused, parameters=False):
    """One pass over a fresh copy of the pool: the fused launch, or the separate calls.  Returns (q_output, gate_output, pages)."""
    import torch

    from . import gpu_runner

    q_norm, k_norm, page, shape = _configs(case, rope_dim, weight_dtype, yarn)
    hq, hkv, dim, tokens, gated = case["hq"], case["hkv"], case["dim"], case["tokens"], case["gated"]
    to = lambda a: gpu_runner.to_device(np.ascontiguousarray(a), device)  # noqa: E731
    weight = lambda w: to(oracle.f32_to_bf16_bits(w) if weight_dtype == DTYPE_BF16 else w)  # noqa: E731
    rows = lambda heads: torch.full((tokens, heads, dim), POISON, dtype=torch.int16, device=device)  # noqa: E731
    projection, pages = to(case["projection"]), to(case["pages"])
    q_weight, k_weight = weight(case["q_weight"]), weight(case["k_weight"])
    req_slots, positions, page_ids = to(case["req_slots"]), to(case["positions"]), to(case["page_ids"])
    q_output, gate_output = rows(hq), rows(hq)
    params = torch.tensor([7, active, layer, 0], dtype=torch.int32, device=device)
    count = ReplayU32.parameter(1) if parameters else ReplayU32.fixed(active)
    table = ReplayU32.parameter(2) if parameters else ReplayU32.fixed(layer)
    if fused:
        prologue.Compute(q_norm, k_norm, page, gated=gated).invoke(
            shape, projection=projection, q_norm_weight=q_weight, k_norm_weight=k_weight, q_output=q_output, gate_output=gate_output if gated else None,
            pages=pages, req_slots=req_slots, flat_token_indices=positions, page_ids=page_ids, num_active_tokens=count, page_table_index=table,
            replay_parameters=params)
    else:
        q, k, v = rows(hq), rows(hkv), rows(hkv)
        if gated:
            qgkv_split.Compute(qgkv_split.Config.bf16(hq, hkv, dim)).invoke(qgkv_split.Shape(tokens), qgkv=projection, q=q, g=gate_output, k=k, v=v,
                                                                             num_active_tokens=count, replay_parameters=params)
        else:
            qkv_split.Compute(qkv_split.Config.bf16(hq, hkv, dim)).invoke(qkv_split.Shape(tokens), qkv=projection, q=q, k=k, v=v,
                                                                           num_active_tokens=count, replay_parameters=params)
        rnr.Compute(q_norm).invoke(rnr.Shape(tokens), input=q, norm_weight=q_weight, flat_token_indices=positions, output=q_output,
                                   num_active_tokens=count, replay_parameters=params)
        k_writer.Compute(k_norm, page).invoke(shape, pages=pages, k=k, v=v, norm_weight=k_weight, req_slots=req_slots, flat_token_indices=positions,
                                              page_ids=page_ids, num_active_tokens=count, page_table_index=table, replay_parameters=params)
    torch.cuda.synchronize()
    assert np.array_equal(projection.cpu().numpy().view(np.uint16), case["projection"]), "the projection was modified"
    return q_output.cpu().numpy().view(np.uint16), gate_output.cpu().numpy().view(np.uint16), pages.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("hq,hkv,dim,rope_dim,kv_dtype,weight_dtype,yarn,gated,tokens,active", [
    (64, 8, 128, 128, DTYPE_FP8_E4M3FN, DTYPE_BF16, False, True, 41, 41),    # benchmark geometry
    (64, 8, 128, 128, DTYPE_BF16, DTYPE_BF16, False, True, 41, 33),
    (24, 4, 256, 256, DTYPE_FP8_E4M3FN, DTYPE_BF16, True, True, 23, 23),     # D 256, Yarn
    (24, 4, 256, 64, DTYPE_BF16, DTYPE_F32, False, True, 23, 7),             # partial rotary, f32 weights
    (16, 2, 128, 128, DTYPE_FP8_E4M3FN, DTYPE_BF16, False, False, 37, 37),   # ungated projection rows
    (5, 1, 64, 32, DTYPE_BF16, DTYPE_BF16, False, True, 19, 18),             # odd head count, 8 lanes per row
    (96, 40, 64, 64, DTYPE_FP8_E4M3FN, DTYPE_F32, True, False, 9, 9),        # 8 lanes per row, many heads
    (24, 12, 512, 256, DTYPE_BF16, DTYPE_BF16, False, True, 6, 5),           # 64 lanes per row, two head groups in both roles
    (64, 8, 128, 128, DTYPE_FP8_E4M3FN, DTYPE_BF16, False, True, 1, 1),      # a single decoded token
])
def test_one_launch_leaves_the_bytes_of_the_separate_calls(device, hq, hkv, dim, rope_dim, kv_dtype, weight_dtype, yarn, gated, tokens, active):
    case = _case(hq, hkv, dim, kv_dtype, seed=hq * 100 + dim + tokens, tokens=tokens, gated=gated)
    for layer, parameters in ((0, False), (1, True)):
        print(f"projection prologue Hq{hq}/Hkv{hkv}/D{dim} rope {rope_dim} kv_dtype={kv_dtype} gated={gated} active={active}/{tokens} "
              f"layer={layer} parameters={parameters}", flush=True)
        fused = _run(device, case, rope_dim, weight_dtype, yarn, active, layer, True, parameters)
        separate = _run(device, case, rope_dim, weight_dtype, yarn, active, layer, False, parameters)
        for name, a, b in zip(("q_output", "gate_output", "pages"), fused, separate):
            assert np.array_equal(a, b), f"{name} differs in {np.count_nonzero(a != b)} places"
        # rows beyond the active count are untouched, and (ungated) so is the whole gate buffer
        assert np.all(fused[0][active:] == POISON) and np.all(fused[1][active if gated else 0:] == POISON)
        assert not np.array_equal(fused[2], case["pages"])


@pytest.mark.gpu
def test_one_launch_against_the_oracle_chain(device):
    """Independent of the separate kernels: the oracle's split, norm + RoPE and page write on the same rows.  Gate rows and V
    bytes are exact; Q rows and K bytes agree up to the producers' one-ulp bound (tests/test_rms_norm_rope.py)."""
    hq, hkv, dim = 16, 2, 128
    case = _case(hq, hkv, dim, DTYPE_FP8_E4M3FN, seed=77, tokens=29, gated=True)
    q_rows, gate_rows, pages = _run(device, case, dim, DTYPE_BF16, False, 29, 1, True)
    zeros = lambda heads: np.zeros(29 * heads * dim, dtype=np.uint16)  # noqa: E731
    q, g, k, v = oracle.qgkv_split(case["projection"], hq, hkv, dim, 29, zeros(hq), zeros(hq), zeros(hkv), zeros(hkv))
    assert np.array_equal(gate_rows.reshape(-1), g)
    weights = [oracle.f32_to_bf16_bits(case[name]) for name in ("q_weight", "k_weight")]
    q_expected = oracle.rms_norm_rope(q.reshape(29, hq, dim), weights[0], case["positions"], hq, dim, dim, 1e-6, 10_000_000.0, io_bf16=True, weight_bf16=True)
    k_expected = oracle.rms_norm_rope(k.reshape(29, hkv, dim), weights[1], case["positions"], hkv, dim, dim, 3e-6, 10_000_000.0, io_bf16=True, weight_bf16=True)
    assert np.mean(q_rows == q_expected) > 0.99
    assert np.max(np.abs(oracle.bf16_bits_to_f32(q_rows) - oracle.bf16_bits_to_f32(q_expected))) < 0.07   # two bf16 ulps at |x| < 8
    def written(k_rows, v_rows):
        return oracle.kv_page_write(case["pages"], k_rows, v_rows, case["req_slots"], case["positions"], case["page_ids"], 29, 1, case["layers"],
                                    case["blocks"], case["per_block"], hkv, dim, 16, case["page_bytes"], True)
    wanted = written(k_expected, v.reshape(29, hkv, dim))
    # which bytes a write of K rows and of V rows touches: 1.0 and -2.0 differ in every FP8 code
    constant = lambda bits: np.full((29, hkv, dim), bits, dtype=np.uint16)  # noqa: E731
    k_bytes = written(constant(0x3F80), constant(0x3F80)) != written(constant(0xC000), constant(0x3F80))
    v_bytes = written(constant(0x3F80), constant(0x3F80)) != written(constant(0x3F80), constant(0xC000))
    assert k_bytes.sum() == v_bytes.sum() == 29 * hkv * dim and not np.any(k_bytes & v_bytes)
    assert np.array_equal(pages[~(k_bytes | v_bytes)], case["pages"][~(k_bytes | v_bytes)])
    assert np.array_equal(pages[v_bytes], wanted[v_bytes])
    assert np.mean(pages[k_bytes] == wanted[k_bytes]) > 0.99


def test_rejections_before_any_device_call():
    buffers = _lib.ProjectionNormRopePageWriteBuffers()
    q_norm, k_norm = rnr.Config.bf16(16, 128, 128, 1e-6, 1e6), rnr.Config.bf16(2, 128, 128, 1e-6, 1e6)
    page = kpw.Config(2, 128, 2 * 2 * 16 * 128)
    shape = kpw.Shape(8, kpw.PageTableLayout(1, 1, 1, 1))

    def call(q=q_norm, k=k_norm, p=page, s=shape, active=ReplayU32.fixed(8)):
        qs, ks, ps, ss = q.as_struct(), k.as_struct(), p.as_struct(), s.as_struct()
        _lib.check(_lib.lib().khm_gqa_projection_norm_rope_page_write(1, ctypes.byref(qs), ctypes.byref(ks), ctypes.byref(ps), ctypes.byref(ss),
                                                                      ctypes.byref(buffers), active, ReplayU32.fixed(0), None, None))
    with pytest.raises(KhmError, match="do not match the page writer's KV heads"):
        call(k=rnr.Config.bf16(4, 128, 128, 1e-6, 1e6))
    with pytest.raises(KhmError, match="takes BF16 projection rows"):
        call(q=rnr.Config.f32(16, 128, 128, 1e-6, 1e6))
    with pytest.raises(KhmError, match="same head_dim, rotation and weight dtype"):
        call(q=rnr.Config.bf16(16, 128, 64, 1e-6, 1e6))
    with pytest.raises(KhmError, match="same head_dim, rotation and weight dtype"):
        call(q=rnr.Config.bf16(16, 128, 128, 1e-6, 2e6))
    with pytest.raises(KhmError, match="GQA projection elements exceeds the shader u32 count domain"):
        call(s=kpw.Shape(1 << 30, kpw.PageTableLayout(1, 1, 1, 1)))
    with pytest.raises(KhmError, match="projection buffer holds 0 bytes, needs 73728"):
        call()
