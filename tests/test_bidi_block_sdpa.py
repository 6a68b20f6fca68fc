"""Dense bidirectional block SDPA (the DFlash2 proposal block): the oracle restatement against an independent float64
reconstruction on the reference's fixtures (CPU), the HIP kernel against the oracle, and the composite of history
partials + block partial through the sliced-Q Reduce (GPU).  Mirrors components/gqa/bidi_block_sdpa_test.rs."""
import numpy as np
import pytest

from khalamari_amd import _lib
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, ReplayU32
from oracle import gqa_oracle as oracle


def _f64_reference(q, k, v, token, head, block_size, hq, hkv, d, scale):
    """Plain softmax attention of one (token, head) over its request block, in float64."""
    q = np.asarray(q, dtype=np.float64).reshape(-1, hq, d)
    k = np.asarray(k, dtype=np.float64).reshape(-1, hkv, d)
    v = np.asarray(v, dtype=np.float64).reshape(-1, hkv, d)
    begin = token // block_size * block_size
    kv_head = head // (hq // hkv)
    scores = k[begin:begin + block_size, kv_head] @ q[token, head] * scale
    weights = np.exp(scores - scores.max())
    return scores.max(), weights.sum(), weights @ v[begin:begin + block_size, kv_head] / weights.sum()


def _request_block_fixture(dtype_bf16):
    """assert_kernel_matches_request_block_bidirectional_reference (bidi_block_sdpa_test.rs:399-470)."""
    hq, hkv, d, block, tokens = 5, 1, 32, 3, 6
    q = (np.arange(tokens * hq * d, dtype=np.float32) * np.float32(0.03125) - np.float32(0.4))
    k = (np.arange(tokens * hkv * d, dtype=np.float32) * np.float32(-0.025) + np.float32(0.3))
    v = (np.arange(tokens * hkv * d, dtype=np.float32) * np.float32(0.05) - np.float32(0.2))
    if dtype_bf16:
        q, k, v = oracle.bf16_round(q), oracle.bf16_round(k), oracle.bf16_round(v)
    ranges = np.array([[0, 3], [3, 6]], dtype=np.uint32)
    cu = np.array([0, 1, 2], dtype=np.uint32)
    return dict(hq=hq, hkv=hkv, d=d, block=block, tokens=tokens, q=q, k=k, v=v, ranges=ranges, cu=cu, max_q=8, slots=8,
                scale=float(np.float32(32.0) ** np.float32(-0.5)))


@pytest.mark.parametrize("dtype_bf16", [False, True])
def test_oracle_matches_float64_reconstruction(dtype_bf16):
    f = _request_block_fixture(dtype_bf16)
    sums, maxs, out = oracle.bidi_block_sdpa(f["q"], f["k"], f["v"], f["ranges"], f["cu"], 2, f["block"], f["max_q"], f["hq"], f["hkv"],
                                             f["d"], f["scale"], f["slots"])
    for token in range(f["tokens"]):
        for head in range(f["hq"]):
            want_max, want_sum, want_out = _f64_reference(f["q"], f["k"], f["v"], token, head, f["block"], f["hq"], f["hkv"], f["d"], f["scale"])
            slot, offset = token // f["block"], token % f["block"]      # the reference's partial_output_index arithmetic
            assert abs(maxs[slot, head, offset] - want_max) < 1e-4
            assert abs(sums[slot, head, offset] - want_sum) < 1e-4
            assert np.abs(out[slot, head, offset] - want_out).max() < 1e-5
    assert np.isnan(sums[2:]).all() and np.isnan(sums[:, :, 3:]).all()          # nothing else is written


def test_validation_messages():
    from khalamari_amd import bidi_block_sdpa as bb

    lib = _lib.lib()
    config = bb.Config(9, 8, 40, 8, 128, 1.0).as_struct()
    shape = bb.Shape(10, 2, 16).as_struct()
    import ctypes
    buffers = _lib.BidiBlockSdpaBuffers()
    status = lib.khm_bidi_block_sdpa(ctypes.byref(config), ctypes.byref(shape), ctypes.byref(buffers), ReplayU32.fixed(2), None, None)
    assert status == _lib.KHM_ERR_INVALID_ARGUMENT and b"complete request blocks" in lib.khm_last_error()   # bidi_block_sdpa_test.rs:21-38


# ---------------------------------------------------------------------------------------------- GPU


def _to(device, array):
    import torch

    array = np.ascontiguousarray(array)
    return torch.from_numpy(array.view(np.uint8).reshape(-1).copy()).to(device)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_bf16", [False, True])
def test_gpu_matches_oracle_on_the_request_block_fixture(device, dtype_bf16):
    import torch

    from khalamari_amd import bidi_block_sdpa as bb

    f = _request_block_fixture(dtype_bf16)
    dtype = DTYPE_BF16 if dtype_bf16 else DTYPE_F32
    config = bb.Config(f["block"], f["max_q"], f["hq"], f["hkv"], f["d"], f["scale"], dtype)
    shape = bb.Shape(f["tokens"], 2, f["slots"])
    pack = (lambda a: oracle.f32_to_bf16_bits(a)) if dtype_bf16 else (lambda a: np.asarray(a, dtype=np.float32))
    stats = config.partial_output_stat_elements(shape)
    sums = torch.full((stats,), float("nan"), dtype=torch.float32, device=device)
    maxs = torch.full((stats,), float("nan"), dtype=torch.float32, device=device)
    partial = torch.zeros(config.partial_output_values(shape) * config.item_size(), dtype=torch.uint8, device=device)
    bb.Compute(config).invoke(shape, ReplayU32.fixed(2), q=_to(device, pack(f["q"])), local_k=_to(device, pack(f["k"])),
                              local_v=_to(device, pack(f["v"])), q_token_ranges=_to(device, f["ranges"]),
                              cu_sdpa_partial_outputs=_to(device, f["cu"]), partial_exp_sums=sums, partial_max_logits=maxs, partial_output=partial)
    torch.cuda.synchronize()
    want_sums, want_maxs, want_out = oracle.bidi_block_sdpa(f["q"], f["k"], f["v"], f["ranges"], f["cu"], 2, f["block"], f["max_q"], f["hq"],
                                                            f["hkv"], f["d"], f["scale"], f["slots"])
    got_sums = sums.cpu().numpy().reshape(want_sums.shape)
    got_maxs = maxs.cpu().numpy().reshape(want_maxs.shape)
    raw = partial.cpu().numpy()
    got_out = (oracle.bf16_bits_to_f32(raw.view(np.uint16)) if dtype_bf16 else raw.view(np.float32)).reshape(want_out.shape)
    written = ~np.isnan(want_sums)
    assert np.array_equal(np.isnan(got_sums), ~written)                          # exactly the same entries are written
    assert np.abs(got_sums[written] - want_sums[written]).max() < 1e-4
    assert np.abs(got_maxs[written] - want_maxs[written]).max() < 1e-4
    assert np.abs(got_out[written] - want_out[written]).max() < (1e-2 if dtype_bf16 else 1e-5)   # bidi_block_sdpa_test.rs:41-48


@pytest.mark.gpu
@pytest.mark.parametrize("hq,hkv,d,block,max_q,dtype_bf16", [
    (16, 2, 128, 8, 8, True),      # the executor's shape: eight tokens x eight heads = four rounds of sixteen tasks
    (24, 4, 256, 16, 16, True),    # head_dim 256: two chunks per lane, 96 tasks per block
    (24, 4, 256, 32, 8, False),    # f32, a 32-token request block of 256 dims: two key tiles (running maximum across tiles)
    (6, 3, 96, 5, 4, True),        # head_dim that is not a multiple of 128, odd block size, ranges shorter than the block
    (4, 1, 32, 40, 64, False),     # ranges that span request blocks (max_q_tokens above the block size)
    (8, 2, 160, 12, 16, True),     # head_dim 160: the second chunk is live in four lanes of a row only
])
def test_gpu_matches_oracle_over_shapes(device, hq, hkv, d, block, max_q, dtype_bf16):
    """Random request blocks through the C ABI against the oracle: several rounds of tasks per thread block, several key
    tiles, partly filled lane rows, and Q ranges cut at max_q_tokens wherever they fall."""
    import torch

    from khalamari_amd import bidi_block_sdpa as bb

    requests = 3
    tokens = requests * block
    rng = np.random.default_rng(hq * 1000 + d + block)
    q = rng.standard_normal(tokens * hq * d).astype(np.float32)
    k = rng.standard_normal(tokens * hkv * d).astype(np.float32)
    v = rng.standard_normal(tokens * hkv * d).astype(np.float32)
    if dtype_bf16:
        q, k, v = oracle.bf16_round(q), oracle.bf16_round(k), oracle.bf16_round(v)
    ranges = np.array([[begin, min(begin + max_q, tokens)] for begin in range(0, tokens, max_q)], dtype=np.uint32)
    num_ranges = ranges.shape[0]
    cu = np.arange(num_ranges + 1, dtype=np.uint32) * 2          # every range owns two slots; the block partial is the second
    slots = 2 * num_ranges
    scale = float(np.float32(d) ** np.float32(-0.5))
    dtype = DTYPE_BF16 if dtype_bf16 else DTYPE_F32
    config = bb.Config(block, max_q, hq, hkv, d, scale, dtype)
    shape = bb.Shape(tokens, num_ranges, slots)
    pack = (lambda a: oracle.f32_to_bf16_bits(a)) if dtype_bf16 else (lambda a: np.asarray(a, dtype=np.float32))
    stats = config.partial_output_stat_elements(shape)
    sums = torch.full((stats,), float("nan"), dtype=torch.float32, device=device)
    maxs = torch.full((stats,), float("nan"), dtype=torch.float32, device=device)
    partial = torch.zeros(config.partial_output_values(shape) * config.item_size(), dtype=torch.uint8, device=device)
    print(f"bidi block shapes: hq={hq} hkv={hkv} d={d} block={block} max_q={max_q} bf16={dtype_bf16} ranges={num_ranges}", flush=True)
    bb.Compute(config).invoke(shape, ReplayU32.fixed(num_ranges), q=_to(device, pack(q)), local_k=_to(device, pack(k)),
                              local_v=_to(device, pack(v)), q_token_ranges=_to(device, ranges), cu_sdpa_partial_outputs=_to(device, cu),
                              partial_exp_sums=sums, partial_max_logits=maxs, partial_output=partial)
    torch.cuda.synchronize()
    want_sums, want_maxs, want_out = oracle.bidi_block_sdpa(q, k, v, ranges, cu, num_ranges, block, max_q, hq, hkv, d, scale, slots)
    got_sums = sums.cpu().numpy().reshape(want_sums.shape)
    got_maxs = maxs.cpu().numpy().reshape(want_maxs.shape)
    raw = partial.cpu().numpy()
    got_out = (oracle.bf16_bits_to_f32(raw.view(np.uint16)) if dtype_bf16 else raw.view(np.float32)).reshape(want_out.shape)
    written = ~np.isnan(want_sums)
    assert written.sum() == tokens * hq
    assert np.array_equal(np.isnan(got_sums), ~written)
    assert np.abs(got_sums[written] - want_sums[written]).max() < 1e-4 * max(1.0, float(want_sums[written].max()))
    assert np.abs(got_maxs[written] - want_maxs[written]).max() < 1e-4
    assert np.abs(got_out[written] - want_out[written]).max() < (1e-2 if dtype_bf16 else 2e-5)


@pytest.mark.gpu
def test_gpu_replay_active_q_token_ranges(device):
    """test_replay_active_q_token_ranges_match_cpu_reference (bidi_block_sdpa_test.rs:50-157)."""
    import torch

    from khalamari_amd import bidi_block_sdpa as bb

    tokens, d = 8, 32
    config = bb.Config(tokens, 1, 1, 1, d, float(np.float32(d) ** np.float32(-0.5)), DTYPE_F32)
    shape = bb.Shape(tokens, tokens, tokens)
    q = np.arange(tokens * d, dtype=np.float32) * np.float32(0.003) - np.float32(0.4)
    k = np.arange(tokens * d, dtype=np.float32) * np.float32(-0.002) + np.float32(0.3)
    v = np.arange(tokens * d, dtype=np.float32) * np.float32(0.004) - np.float32(0.2)
    ranges = np.array([[i, i + 1] for i in range(tokens)], dtype=np.uint32)
    cu = np.arange(tokens + 1, dtype=np.uint32)
    params = torch.zeros(2, dtype=torch.int32, device=device)
    buffers = dict(q=_to(device, q), local_k=_to(device, k), local_v=_to(device, v), q_token_ranges=_to(device, ranges),
                   cu_sdpa_partial_outputs=_to(device, cu))
    compute = bb.Compute(config)
    for active in [1, 8, 3, 7, 2, 6, 4, 5]:
        sums = torch.full((tokens,), -7.0, dtype=torch.float32, device=device)
        maxs = torch.full((tokens,), -7.0, dtype=torch.float32, device=device)
        partial = torch.full((tokens * d,), -7.0, dtype=torch.float32, device=device)
        params[1] = active
        compute.invoke(shape, ReplayU32.parameter(1), partial_exp_sums=sums, partial_max_logits=maxs, partial_output=partial,
                       replay_parameters=params, **buffers)
        torch.cuda.synchronize()
        got = partial.cpu().numpy().reshape(tokens, d)
        for token in range(active):
            want_max, want_sum, want_out = _f64_reference(q, k, v, token, 0, tokens, 1, 1, d, config.scale)
            assert abs(maxs[token].item() - want_max) < 1e-4 and abs(sums[token].item() - want_sum) < 1e-4
            assert np.abs(got[token] - want_out).max() < 1e-4
        assert (got[active:] == -7.0).all() and (sums[active:] == -7.0).all()


@pytest.mark.gpu
@pytest.mark.parametrize("visible_begins", [[0] * 7, [4, 5, 6, 7, 8, 9, 10, 11]])
def test_gpu_history_and_block_composite(device, visible_begins):
    """assert_composite_matches_reference (bidi_block_sdpa_test.rs:170-397): two history partials from the sliced-Q Map on
    FP8 pages plus the block partial, merged by the sliced-Q Reduce, against softmax over history[begin..12] + the block."""
    import torch

    from khalamari_amd import bidi_block_sdpa as bb
    from khalamari_amd import sdpa, sliced_kv, sliced_q
    from khalamari_amd._lib import DTYPE_FP8_E4M3FN

    n, history, hq, hkv, d, tpp = len(visible_begins), 16, 5, 1, 128, 8
    scale = float(np.float32(d) ** np.float32(-0.5))
    q = np.ones((n, hq, d), dtype=np.float32)
    history_k = np.full((history, hkv, d), oracle.fp8_round_trip(np.array([0.17677669], dtype=np.float32))[0], dtype=np.float32)
    history_v = np.full((history, hkv, d), 1.0, dtype=np.float32)
    local_k = oracle.bf16_round(np.full((n, hkv, d), 0.22097087, dtype=np.float32))
    local_v = np.full((n, hkv, d), -1.0, dtype=np.float32)
    geom = oracle.Geometry(hq, hkv, d, tpp, scale, 1, 2, 1, oracle.KV_FP8_E4M3FN)
    pages = oracle.pack_pages(geom, 2, [(history_k, history_v)], [[0, 1]])
    qconfig = sliced_q.Config(hq, hkv, d, scale, geom.page_bytes, sliced_kv.Layout(1, 1, 2, 1), DTYPE_BF16, DTYPE_FP8_E4M3FN)
    qshape = sliced_q.Shape(n, 1, 3)
    variant = sdpa.ExecutionVariant.sliced_q_per_head(qconfig.sdpa_config(), 8, 16, 5)
    map_compute = sliced_q.Compute.new(qconfig, variant, qshape)
    bconfig = bb.Config(n, 8, hq, hkv, d, scale, DTYPE_BF16)
    bshape = bb.Shape(n, 1, 3)
    dev = lambda a: _to(device, a)  # noqa: E731
    q_d = dev(oracle.f32_to_bf16_bits(q))
    ranges = dev(np.array([[0, n]], dtype=np.uint32))
    cu = dev(np.array([0, 3], dtype=np.uint32))
    groups = 3 * 8 * hq
    sums = torch.zeros(groups, dtype=torch.float32, device=device)
    maxs = torch.zeros(groups, dtype=torch.float32, device=device)
    partial = torch.zeros(groups * d * 2, dtype=torch.uint8, device=device)
    out = torch.zeros(n * hq * d, dtype=torch.int16, device=device)
    visible = np.array([[b, 12] for b in visible_begins], dtype=np.uint32)
    templates = np.array([[0, 0, 4], [0, 4, 12], [0xFFFFFFFF] * 3], dtype=np.uint32)
    map_compute.invoke_map(q=q_d, kv_pages=dev(pages), req_slots=dev(np.zeros(n, dtype=np.uint32)), page_ids=dev(np.array([0, 1], dtype=np.uint32)),
                           visible_kv_token_ranges=dev(visible), q_token_ranges=ranges, sdpa_map_task_templates=dev(templates),
                           partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, page_table_index=ReplayU32.fixed(0),
                           num_active_tokens=ReplayU32.fixed(n), num_active_q_token_tiles=ReplayU32.fixed(1), num_active_kv_splits=ReplayU32.fixed(3))
    bb.Compute(bconfig).invoke(bshape, ReplayU32.fixed(1), q=q_d, local_k=dev(oracle.f32_to_bf16_bits(local_k)),
                               local_v=dev(oracle.f32_to_bf16_bits(local_v)), q_token_ranges=ranges, cu_sdpa_partial_outputs=cu,
                               partial_exp_sums=sums, partial_max_logits=maxs, partial_output=partial)
    map_compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, q_token_ranges=ranges,
                              cu_sdpa_partial_outputs=cu, output=out, num_active_q_token_tiles=ReplayU32.fixed(1))
    torch.cuda.synchronize()
    actual = oracle.bf16_bits_to_f32(out.cpu().numpy().view(np.uint16)).reshape(n, hq, d)
    for token, begin in enumerate(visible_begins):
        keys = np.concatenate([history_k[begin:12, 0], local_k[:, 0]]).astype(np.float64)
        values = np.concatenate([history_v[begin:12, 0], local_v[:, 0]]).astype(np.float64)
        scores = keys @ q[token, 0].astype(np.float64) * scale
        weights = np.exp(scores - scores.max())
        expected = weights @ values / weights.sum()
        assert np.abs(actual[token] - expected[None, :]).max() < 1e-2, (token, actual[token, 0, :4], expected[:4])


@pytest.mark.gpu
@pytest.mark.parametrize("fp8_pages,window", [(False, 0xFFFFFFFF), (True, 64)])
def test_gpu_spec_decode_step_from_selected_variant_and_built_metadata(device, fp8_pages, window):
    """A whole proposal step the way the executor drives it (attn/bidi_block_gqa/backend.rs:394-480): variant and capacity
    from the block selector, metadata from the block metadata builder, history partials from the sliced-Q Map over the
    paged cache, the dense block partial, and the Reduce; against a float64 softmax over each row's visible history
    window plus its whole block."""
    import torch

    from khalamari_amd import bidi_block_metadata as bbm
    from khalamari_amd import bidi_block_sdpa as bb
    from khalamari_amd import sdpa, sliced_kv, sliced_q
    from khalamari_amd._lib import DTYPE_FP8_E4M3FN

    rng = np.random.default_rng(11 + int(fp8_pages))
    hq, hkv, d, tpp, block_size = 8, 2, 128, 16, 7
    scale = float(np.float32(d) ** np.float32(-0.5))
    anchors, slots = [37, 150, 600], [2, 0, 1]                 # history lengths; request slots in batch order
    sconfig = sdpa.Config(DTYPE_BF16, hq, hkv, d, tpp)
    variant, capacity = bbm.select(sconfig, len(anchors), block_size)
    assert variant.map_max_q_tokens == 8 and sdpa.has_kernel(sconfig, variant, DTYPE_FP8_E4M3FN if fp8_pages else DTYPE_BF16)
    indices, ranges = [], []
    for anchor in anchors:
        for offset in range(block_size):
            indices.append(anchor + offset)
            ranges.append((max(anchor + offset + 1 - window, 0), anchor))
    meta = bbm.build(slots, indices, ranges, block_size, variant, capacity.max_sdpa_map_task_templates)
    shape = meta.replay_shape
    n = len(indices)

    kv_dtype = oracle.KV_FP8_E4M3FN if fp8_pages else oracle.KV_BF16
    rounding = oracle.fp8_round_trip if fp8_pages else oracle.bf16_round
    num_blocks = -(-max(anchors) // tpp)
    geom = oracle.Geometry(hq, hkv, d, tpp, scale, 1, num_blocks, 1, kv_dtype)
    histories = [(rounding(rng.standard_normal((a, hkv, d)).astype(np.float32)), rounding(rng.standard_normal((a, hkv, d)).astype(np.float32)))
                 for a in anchors]
    pages_per_request = [-(-a // tpp) for a in anchors]
    order = rng.permutation(sum(pages_per_request) + 3)
    page_lists, cursor = [], 0
    for count in pages_per_request:
        page_lists.append([int(x) for x in order[cursor:cursor + count]])
        cursor += count
    pages = oracle.pack_pages(geom, len(order), histories, page_lists, fill_bits=0x7F if fp8_pages else 0x7FC0)   # NaN everywhere else
    table = np.full((3, num_blocks), 0xFFFFFFFF, dtype=np.uint32)       # indexed by request SLOT
    for slot, page_list in zip(slots, page_lists):
        table[slot, :len(page_list)] = page_list
    q = oracle.bf16_round(rng.standard_normal((n, hq, d)).astype(np.float32))
    local_k = oracle.bf16_round(rng.standard_normal((n, hkv, d)).astype(np.float32))
    local_v = oracle.bf16_round(rng.standard_normal((n, hkv, d)).astype(np.float32))

    qconfig = sliced_q.Config(hq, hkv, d, scale, geom.page_bytes, sliced_kv.Layout(3, 1, num_blocks, 1), DTYPE_BF16,
                              DTYPE_FP8_E4M3FN if fp8_pages else DTYPE_BF16)
    qshape = sliced_q.Shape(shape.num_total_tokens, shape.num_total_q_token_tiles, shape.num_total_sdpa_map_task_templates)
    map_compute = sliced_q.Compute.new(qconfig, variant, qshape)
    dev = lambda a: _to(device, a)  # noqa: E731
    q_d, ranges_d, cu_d = dev(oracle.f32_to_bf16_bits(q)), dev(meta.q_token_ranges), dev(meta.cu_sdpa_partial_outputs)
    groups = int(shape.num_total_sdpa_map_task_templates) * int(variant.map_max_q_tokens) * hq
    sums = torch.full((groups,), float("nan"), dtype=torch.float32, device=device)
    maxs = torch.full((groups,), float("nan"), dtype=torch.float32, device=device)
    partial = torch.full((groups * d * 2,), 0xFF, dtype=torch.uint8, device=device)
    out = torch.zeros(n * hq * d, dtype=torch.int16, device=device)
    fixed = ReplayU32.fixed
    map_compute.invoke_map(q=q_d, kv_pages=dev(pages), req_slots=dev(meta.req_slots), page_ids=dev(table),
                           visible_kv_token_ranges=dev(meta.visible_kv_token_ranges), q_token_ranges=ranges_d,
                           sdpa_map_task_templates=dev(meta.sdpa_map_task_templates), partial_output=partial, partial_exp_sums=sums,
                           partial_max_logits=maxs, page_table_index=fixed(0), num_active_tokens=fixed(shape.num_tokens),
                           num_active_q_token_tiles=fixed(shape.num_q_token_tiles), num_active_kv_splits=fixed(shape.num_sdpa_map_task_templates))
    bb.Compute(bb.Config(block_size, int(variant.map_max_q_tokens), hq, hkv, d, scale, DTYPE_BF16)).invoke(
        bb.Shape(shape.num_total_tokens, shape.num_total_q_token_tiles, shape.num_total_sdpa_map_task_templates), fixed(shape.num_q_token_tiles),
        q=q_d, local_k=dev(oracle.f32_to_bf16_bits(local_k)), local_v=dev(oracle.f32_to_bf16_bits(local_v)), q_token_ranges=ranges_d,
        cu_sdpa_partial_outputs=cu_d, partial_exp_sums=sums, partial_max_logits=maxs, partial_output=partial)
    map_compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, q_token_ranges=ranges_d,
                              cu_sdpa_partial_outputs=cu_d, output=out, num_active_q_token_tiles=fixed(shape.num_q_token_tiles))
    torch.cuda.synchronize()
    actual = oracle.bf16_bits_to_f32(out.cpu().numpy().view(np.uint16)).reshape(n, hq, d)
    assert np.isfinite(actual).all()
    for request, anchor in enumerate(anchors):
        rows = slice(request * block_size, (request + 1) * block_size)
        for offset in range(block_size):
            token = request * block_size + offset
            begin = ranges[token][0]
            for head in range(hq):
                kv_head = head // (hq // hkv)
                keys = np.concatenate([histories[request][0][begin:anchor, kv_head], local_k[rows, kv_head]]).astype(np.float64)
                values = np.concatenate([histories[request][1][begin:anchor, kv_head], local_v[rows, kv_head]]).astype(np.float64)
                scores = keys @ q[token, head].astype(np.float64) * scale
                weights = np.exp(scores - scores.max())
                expected = weights @ values / weights.sum()
                error = np.abs(actual[token, head] - expected)
                assert np.all(error <= 2e-3 + 1e-2 * np.abs(expected)), (request, offset, head, error.max())
