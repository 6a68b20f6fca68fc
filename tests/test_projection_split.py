"""Split of the fused input projection into Q, (gate,) K and V rows: the oracle's restatement of the two shaders against
the reference's own expected vectors (CPU), the shape domain the reference rejects (CPU), and the HIP kernels against the
oracle, bit for bit (GPU).  Vectors follow qgkv_split.rs:258-327 and qkv_split.rs:252-306 of the reference."""
import ctypes

import numpy as np
import pytest

from khalamari_amd import _lib, qgkv_split, qkv_split
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, Buffer, KhmError, ReplayU32
from oracle import gqa_oracle as oracle


def _expected_by_slices(projection, gated, hq, hkv, d, active):
    """`expected_*` exactly as the reference tests build them (qgkv_split.rs:297-320, qkv_split.rs:291-300): per token, the
    head pairs' halves (gated) or the leading Q block (ungated), then the K and the V block."""
    q_width, kv_width = hq * d, hkv * d
    width = (2 if gated else 1) * q_width + 2 * kv_width
    q, g, k, v = [], [], [], []
    for token in range(active):
        row = projection[token * width:(token + 1) * width]
        if gated:
            for head in range(hq):
                begin = head * 2 * d
                q.extend(row[begin:begin + d])
                g.extend(row[begin + d:begin + 2 * d])
            kv_begin = 2 * q_width
        else:
            q.extend(row[:q_width])
            kv_begin = q_width
        k.extend(row[kv_begin:kv_begin + kv_width])
        v.extend(row[kv_begin + kv_width:])
    return [np.asarray(a, dtype=projection.dtype) for a in (q, g, k, v)]


@pytest.mark.parametrize("gated,tokens,active_counts", [(True, 4, [1, 4, 3, 2]), (False, 8, [1, 8, 3, 7, 2, 6, 4, 5])])
def test_oracle_matches_the_reference_tests_expected_vectors(gated, tokens, active_counts):
    """test_replay_active_counts (qgkv_split.rs:258-327) and test_replay_matches_reference_across_active_counts
    (qkv_split.rs:252-306): Config::f32(2, 1, 2), the projection holds 0, 1, 2, ..., outputs start zeroed and keep what
    earlier, larger replays wrote beyond the active prefix."""
    hq, hkv, d = 2, 1, 2
    width = (2 if gated else 1) * hq * d + 2 * hkv * d
    projection = np.arange(tokens * width, dtype=np.float32)
    q, g, k, v = (np.zeros(tokens * n, dtype=np.float32) for n in (hq * d, hq * d, hkv * d, hkv * d))
    for active in active_counts:
        if gated:
            q, g, k, v = oracle.qgkv_split(projection, hq, hkv, d, active, q, g, k, v)
        else:
            q, k, v = oracle.qkv_split(projection, hq, hkv, d, active, q, k, v)
        want_q, want_g, want_k, want_v = _expected_by_slices(projection, gated, hq, hkv, d, active)
        assert np.array_equal(q[:want_q.size], want_q) and np.array_equal(k[:want_k.size], want_k)
        assert np.array_equal(v[:want_v.size], want_v)
        if gated:
            assert np.array_equal(g[:want_g.size], want_g)


def test_oracle_leaves_rows_beyond_the_active_prefix_alone():
    hq, hkv, d, tokens = 3, 2, 4, 5
    rng = np.random.default_rng(5)
    projection = rng.integers(0, 1 << 16, size=tokens * (2 * hq + 2 * hkv) * d, dtype=np.uint16)
    before = [np.full(tokens * n, 0xABCD, dtype=np.uint16) for n in (hq * d, hq * d, hkv * d, hkv * d)]
    after = oracle.qgkv_split(projection, hq, hkv, d, 2, *before)
    for got, n in zip(after, (hq * d, hq * d, hkv * d, hkv * d)):
        assert np.all(got[2 * n:] == 0xABCD) and not np.any(got[:2 * n] == 0xABCD)
    # every projection element of the active rows lands in exactly one place
    assert sorted(np.concatenate([a[:2 * n] for a, n in zip(after, (hq * d, hq * d, hkv * d, hkv * d))]).tolist()) == \
        sorted(projection[:2 * (2 * hq + 2 * hkv) * d].tolist())


def test_widths_and_byte_counts():
    """Config::{qgkv_width, qkv_width, *_bytes} (qgkv_split.rs:69-133, qkv_split.rs:69-131)."""
    gated, ungated = qgkv_split.Config.bf16(64, 8, 128), qkv_split.Config.f32(24, 4, 256)
    shape = qgkv_split.Shape(7)
    assert gated.projection_width() == (2 * 64 + 2 * 8) * 128 and ungated.projection_width() == (24 + 2 * 4) * 256
    assert gated.projection_bytes(shape) == 7 * 144 * 128 * 2 and gated.q_bytes(shape) == 7 * 64 * 128 * 2
    assert ungated.kv_bytes(shape) == 7 * 4 * 256 * 4
    with pytest.raises(KhmError, match="GQA fused projection head count must fit u32"):
        qgkv_split.Config.f32(0x7FFFFFFF, 0x7FFFFFFF, 1).projection_width()


def test_shapes_reject_shader_count_overflow():
    """test_shape_rejects_shader_count_overflow of both components (qgkv_split.rs:329-335, qkv_split.rs:308-314)."""
    empty = Buffer(0, 0)
    gated = qgkv_split.Config.f32(1, 1, 1).c()
    with pytest.raises(KhmError, match="^.*\\] GQA projection elements exceeds the shader u32 count domain"):
        _lib.check(_lib.lib().khm_gqa_qgkv_split(ctypes.byref(gated), 1 << 30, empty, empty, empty, empty, empty, ReplayU32.fixed(1), None, None))
    ungated = qkv_split.Config.f32(2, 1, 1).c()
    with pytest.raises(KhmError, match="ungated GQA projection elements exceeds the shader u32 count domain"):
        _lib.check(_lib.lib().khm_gqa_qkv_split(ctypes.byref(ungated), 1 << 30, empty, empty, empty, empty, ReplayU32.fixed(1), None, None))


def test_invocations_reject_bad_arguments_before_any_device_call():
    empty, config = Buffer(0, 0), qgkv_split.Config.bf16(2, 1, 8).c()
    call = lambda tokens, active, c=config: _lib.check(_lib.lib().khm_gqa_qgkv_split(  # noqa: E731
        ctypes.byref(c), tokens, empty, empty, empty, empty, empty, active, None, None))
    with pytest.raises(KhmError, match="requires tokens"):
        call(0, ReplayU32.fixed(1))
    with pytest.raises(KhmError, match="num_active_tokens=5 is outside its replay domain \\[1, 4\\]"):
        call(4, ReplayU32.fixed(5))
    with pytest.raises(KhmError, match="num_active_tokens=0 is outside its replay domain"):
        call(4, ReplayU32.fixed(0))
    with pytest.raises(KhmError, match="replay parameter but no parameter block"):
        call(4, ReplayU32.parameter(0))
    with pytest.raises(KhmError, match="qgkv buffer holds 0 bytes, needs 384"):
        call(4, ReplayU32.fixed(4))
    bad = _lib.ProjectionSplitConfig(2, 1, 8, _lib.DTYPE_FP8_E4M3FN)
    with pytest.raises(KhmError, match="unsupported GQA projection split dtype"):
        call(4, ReplayU32.fixed(4), bad)
    with pytest.raises(KhmError, match="requires Q heads, KV heads and a head dimension"):
        call(4, ReplayU32.fixed(4), _lib.ProjectionSplitConfig(2, 0, 8, DTYPE_BF16))


# ------------------------------------------------------------------------------------------------------------ GPU


def _run(device, gated, dtype, hq, hkv, d, tokens, active, *, parameter=False, byte_offset=0, seed=0):
    """One launch over random bit patterns; returns (device outputs, oracle outputs), each [q, (g,) k, v] as flat arrays."""
    import torch
    np_dtype = np.uint32 if dtype == DTYPE_F32 else np.uint16
    item = np.dtype(np_dtype).itemsize
    width = (2 if gated else 1) * hq * d + 2 * hkv * d
    rng = np.random.default_rng(seed)
    projection = rng.integers(0, 1 << (8 * item), size=tokens * width, dtype=np.uint64).astype(np_dtype)
    sizes = [hq * d] * (2 if gated else 1) + [hkv * d] * 2
    poison = 0xA5A5A5A5 if dtype == DTYPE_F32 else 0xA5A5
    before = [np.full(tokens * n, poison, dtype=np_dtype) for n in sizes]

    def on_device(array):   # a byte offset shifts the buffer off its 256-byte allocation boundary
        raw = torch.zeros(array.nbytes + 256, dtype=torch.uint8, device=device)
        window = raw[byte_offset:byte_offset + array.nbytes]
        window.copy_(torch.from_numpy(array.view(np.uint8)).to(device))
        return window

    source = on_device(projection)
    outputs = [on_device(a) for a in before]
    params = torch.tensor([0, active, 0], dtype=torch.int32, device=device)
    count = ReplayU32.parameter(1) if parameter else ReplayU32.fixed(active)
    cls = qgkv_split if gated else qkv_split
    config = cls.Config(hq, hkv, d, dtype)
    shape = cls.Shape(tokens)
    assert source.numel() == config.projection_bytes(shape) and outputs[0].numel() == config.q_bytes(shape)
    print(f"projection split gated={gated} dtype={dtype} Hq{hq}/Hkv{hkv}/D{d} tokens={tokens} active={active} offset={byte_offset}", flush=True)
    if gated:
        cls.Compute(config).invoke(shape, qgkv=source, q=outputs[0], g=outputs[1], k=outputs[2], v=outputs[3], num_active_tokens=count,
                                   replay_parameters=params)
        want = oracle.qgkv_split(projection, hq, hkv, d, active, *before)
    else:
        cls.Compute(config).invoke(shape, qkv=source, q=outputs[0], k=outputs[1], v=outputs[2], num_active_tokens=count,
                                   replay_parameters=params)
        want = oracle.qkv_split(projection, hq, hkv, d, active, *before)
    torch.cuda.synchronize()
    got = [o.cpu().numpy().view(np_dtype) for o in outputs]
    assert np.array_equal(source.cpu().numpy().view(np_dtype), projection), "the projection was modified"
    return got, list(want)


@pytest.mark.gpu
@pytest.mark.parametrize("gated", [True, False])
def test_device_replays_the_reference_vectors(device, gated):
    """The reference tests' own case (Config::f32(2, 1, 2), projection 0, 1, 2, ...) with the active count read from the
    replay parameter block, every count of the reference's list."""
    import torch

    hq, hkv, d = 2, 1, 2
    tokens, counts = (4, [1, 4, 3, 2]) if gated else (8, [1, 8, 3, 7, 2, 6, 4, 5])
    width = (2 if gated else 1) * hq * d + 2 * hkv * d
    projection = np.arange(tokens * width, dtype=np.float32)
    source = torch.from_numpy(projection).to(device)
    sizes = [hq * d] * (2 if gated else 1) + [hkv * d] * 2
    outputs = [torch.zeros(tokens * n, dtype=torch.float32, device=device) for n in sizes]
    params = torch.zeros(2, dtype=torch.int32, device=device)
    cls = qgkv_split if gated else qkv_split
    compute, shape = cls.Compute(cls.Config.f32(hq, hkv, d)), cls.Shape(tokens)
    for active in counts:
        params.copy_(torch.tensor([active, 0], dtype=torch.int32))
        if gated:
            compute.invoke(shape, qgkv=source, q=outputs[0], g=outputs[1], k=outputs[2], v=outputs[3],
                           num_active_tokens=ReplayU32.parameter(0), replay_parameters=params)
        else:
            compute.invoke(shape, qkv=source, q=outputs[0], k=outputs[1], v=outputs[2], num_active_tokens=ReplayU32.parameter(0),
                           replay_parameters=params)
        torch.cuda.synchronize()
        want = _expected_by_slices(projection, gated, hq, hkv, d, active)
        if not gated:
            want = [want[0], want[2], want[3]]
        for got, expected in zip(outputs, want):
            assert np.array_equal(got.cpu().numpy()[:expected.size], expected)


@pytest.mark.gpu
@pytest.mark.parametrize("gated", [True, False])
@pytest.mark.parametrize("dtype,hq,hkv,d,tokens,active,offset", [
    (DTYPE_BF16, 64, 8, 128, 37, 37, 0),      # benchmark geometry, 16-byte units, a ragged last token group
    (DTYPE_BF16, 24, 4, 256, 9, 6, 0),
    (DTYPE_F32, 16, 2, 128, 11, 10, 0),
    (DTYPE_BF16, 5, 1, 12, 7, 7, 0),          # 24-byte head rows: 8-byte units
    (DTYPE_BF16, 3, 2, 6, 6, 5, 0),           # 12-byte head rows: 4-byte units
    (DTYPE_BF16, 2, 1, 3, 5, 4, 0),           # 6-byte head rows: 2-byte units
    (DTYPE_F32, 2, 1, 1, 9, 9, 0),            # one f32 per head
    (DTYPE_BF16, 8, 2, 64, 10, 3, 8),         # buffers 8 bytes off a 16-byte boundary: 8-byte units
    (DTYPE_BF16, 8, 2, 64, 10, 10, 2),        # 2 bytes off: 2-byte units
    (DTYPE_BF16, 40, 40, 128, 3, 2, 0),       # a row wider than 256 x 16-byte units x several blocks
])
def test_device_matches_the_oracle_bit_for_bit(device, gated, dtype, hq, hkv, d, tokens, active, offset):
    got, want = _run(device, gated, dtype, hq, hkv, d, tokens, active, byte_offset=offset, parameter=(tokens % 2 == 1),
                     seed=hq * 1000 + d)
    for name, a, b in zip(("q", "g", "k", "v") if gated else ("q", "k", "v"), got, want):
        assert np.array_equal(a, b), f"{name} differs in {np.count_nonzero(a != b)} elements"


@pytest.mark.gpu
def test_full_size_prefill_batch_round_trips(device):
    """16384 tokens of the benchmark geometry (604 MB of projection): concatenating the outputs' head rows back in row
    order gives the projection again, which needs no oracle pass over the full size."""
    import torch

    hq, hkv, d, tokens = 64, 8, 128, 16384
    generator = torch.Generator(device=device).manual_seed(3)
    projection = torch.randint(-32768, 32767, (tokens, 2 * hq + 2 * hkv, d), dtype=torch.int16, device=device, generator=generator)
    q, g = (torch.zeros((tokens, hq, d), dtype=torch.int16, device=device) for _ in range(2))
    k, v = (torch.zeros((tokens, hkv, d), dtype=torch.int16, device=device) for _ in range(2))
    config = qgkv_split.Config.bf16(hq, hkv, d)
    print("projection split at full size", flush=True)
    qgkv_split.Compute(config).invoke(qgkv_split.Shape(tokens), qgkv=projection, q=q, g=g, k=k, v=v, num_active_tokens=ReplayU32.fixed(tokens))
    torch.cuda.synchronize()
    rebuilt = torch.cat([torch.stack([q, g], dim=2).reshape(tokens, 2 * hq, d), k, v], dim=1)
    assert torch.equal(rebuilt, projection)
