"""Per-head RMSNorm + rotary embedding: the oracle restatement against the reference's own known answers and against
what the mathematics fixes (CPU), and the HIP kernel against the oracle through the C ABI (GPU).  Vectors follow
components/rms_norm_rope.rs:409-640 of the reference."""
import ctypes

import numpy as np
import pytest

from khalamari_amd import _lib
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, ReplayU32
from oracle import gqa_oracle as oracle

YARN = dict(factor=32.0, attention_factor=float(np.float32(1.0) + np.float32(0.1) * np.log(np.float32(32.0))), beta_fast=32.0,
            beta_slow=1.0, original_max_position_embeddings=8192, truncate=True)


def _yarn_config():
    from khalamari_amd import rms_norm_rope as rnr

    return rnr.Config.f32(1, 128, 128, 1e-6, 10_000_000.0).with_rope_scaling(rnr.Yarn(**YARN))


def _long_context_vectors():
    """test_f32_yarn_matches_cpu_reference_at_long_context (rms_norm_rope.rs:427-492): inputs and the expected row
    built the way that test builds it (f32 arithmetic, libm sine/cosine of the f32 angle)."""
    index = np.arange(128)
    values = ((index * 37 % 29).astype(np.float32) - np.float32(14.0)) / np.float32(8.0)
    weight_bits = oracle.f32_to_bf16_bits((np.float32(0.75) + (index % 11).astype(np.float32) / np.float32(20.0)).astype(np.float32))
    weight = oracle.bf16_bits_to_f32(weight_bits)
    position = 262_143
    acc = np.float32(0.0)
    for value in values:
        acc = np.float32(acc + value * value)
    inv_rms = np.float32(1.0) / np.sqrt(np.float32(acc / np.float32(128.0) + np.float32(1e-6)))
    expected = np.zeros(128, dtype=np.float32)
    for d in range(64):
        ramp = np.clip((np.float32(d) - np.float32(14.0)) / np.float32(29.0 - 14.0), 0.0, 1.0).astype(np.float32)
        yarn_scale = np.float32(1.0) + ramp * np.float32(1.0 / 32.0 - 1.0)
        powf = np.float32(np.power(np.float64(10_000_000.0), -np.float64(np.float32(d / 64.0))))    # libm powf: correctly rounded
        inv_freq = np.float32(powf * yarn_scale)
        theta = np.float32(np.float32(position) * inv_freq)
        sin, cos = np.float32(np.sin(np.float64(theta))), np.float32(np.cos(np.float64(theta)))
        first = weight[d] * values[d] * inv_rms
        second = weight[d + 64] * values[d + 64] * inv_rms
        expected[d] = np.float32(YARN["attention_factor"]) * (first * cos - second * sin)
        expected[d + 64] = np.float32(YARN["attention_factor"]) * (first * sin + second * cos)
    return values, weight_bits, position, expected


ROUNDING_INPUT = np.array([0.73046875, -1.171875, 0.439_453_13, 2.03125], dtype=np.float32)
ROUNDING_WEIGHT = np.array([1.296875, 0.8984375, 1.1015625, 0.703125], dtype=np.float32)


def _rounding_order_expected():
    """test_bf16_preserves_norm_rounding_order (rms_norm_rope.rs:494-539): bf16(weight * bf16(input * inv_rms))."""
    input_bits, weight_bits = oracle.f32_to_bf16_bits(ROUNDING_INPUT), oracle.f32_to_bf16_bits(ROUNDING_WEIGHT)
    x = oracle.bf16_bits_to_f32(input_bits)
    square_sum = np.float32(0.0)
    for value in x:
        square_sum = np.float32(square_sum + value * value)
    inv_rms = np.float32(1.0) / np.sqrt(np.float32(square_sum / np.float32(4.0) + np.float32(1e-6)))
    normalized = oracle.bf16_round((x * inv_rms).astype(np.float32))
    return input_bits, weight_bits, oracle.f32_to_bf16_bits((oracle.bf16_bits_to_f32(weight_bits) * normalized).astype(np.float32))


def _f32_weight_expected():
    """test_bf16_io_with_f32_norm_weight_matches_cpu_reference (rms_norm_rope.rs:541-583): bf16(input * inv_rms * weight)."""
    input_bits = oracle.f32_to_bf16_bits(np.array([0.75, -1.25, 0.5, 2.0], dtype=np.float32))
    weight = np.array([1.3, 0.9, 1.1, 0.7], dtype=np.float32)
    x = oracle.bf16_bits_to_f32(input_bits)
    square_sum = np.float32(0.0)
    for value in x:
        square_sum = np.float32(square_sum + value * value)
    inv_rms = np.float32(1.0) / np.sqrt(np.float32(square_sum / np.float32(4.0) + np.float32(1e-6)))
    return input_bits, weight, oracle.f32_to_bf16_bits((x * inv_rms * weight).astype(np.float32))


# ---------------------------------------------------------------------------------------------- CPU


def test_yarn_correction_range_known_answer():
    """test_yarn_correction_range (rms_norm_rope.rs:409-425): (128, 1e7, beta 32/1, 8192, truncate) -> [14, 29]."""
    assert oracle.yarn_correction_range(128, 10_000_000.0, 32.0, 1.0, 8192, True) == (14.0, 29.0)
    assert _yarn_config().yarn_correction_range() == (14.0, 29.0)


def test_kernel_parameters_host_side_matches_oracle_and_closed_form():
    from khalamari_amd import rms_norm_rope as rnr

    table, factor = rnr.Config.bf16(4, 128, 64, 1e-6, 1_000_000.0).kernel_parameters()
    assert factor == 1.0 and len(table) == 32
    assert table[0] == 1.0 and np.allclose(table[16], 1e-3, rtol=1e-5)          # theta^(-1/2) at the middle pair
    want, _ = oracle.rope_kernel_parameters(64, 1_000_000.0)
    assert np.allclose(table, want, rtol=1e-6)
    table, factor = _yarn_config().kernel_parameters()
    want, want_factor = oracle.rope_kernel_parameters(128, 10_000_000.0, YARN)
    assert np.allclose(table, want, rtol=1e-6) and factor == want_factor
    plain, _ = oracle.rope_kernel_parameters(128, 10_000_000.0)
    # below the range the frequency is untouched, above it is divided by the factor
    assert np.array_equal(want[:15], plain[:15]) and np.allclose(want[29:], plain[29:] / 32.0, rtol=1e-6)


def test_oracle_long_context_yarn_known_answer():
    values, weight_bits, position, expected = _long_context_vectors()
    got = oracle.rms_norm_rope(values, weight_bits, [position], 1, 128, 128, 1e-6, 10_000_000.0, yarn=YARN, weight_bf16=True)
    assert np.abs(got.reshape(-1) - expected).max() < 1e-3      # the reference's tolerance
    assert np.abs(got.reshape(-1) - expected).max() < 1e-6      # same arithmetic, so in fact far closer


def test_oracle_bf16_rounding_order_known_answers():
    input_bits, weight_bits, expected = _rounding_order_expected()
    got = oracle.rms_norm_rope(input_bits, weight_bits, [0], 1, 4, 2, 1e-6, 1_000_000.0, io_bf16=True, weight_bf16=True)
    assert np.array_equal(got.reshape(-1), expected)
    # rounding only once gives other bits for this vector: the test separates the two orders
    x, w = oracle.bf16_bits_to_f32(input_bits), oracle.bf16_bits_to_f32(weight_bits)
    inv_rms = np.float32(1.0) / np.sqrt(np.float32(np.sum(x * x, dtype=np.float32) / 4 + np.float32(1e-6)))
    assert not np.array_equal(oracle.f32_to_bf16_bits((w * x * inv_rms).astype(np.float32)), expected)
    input_bits, weight, expected = _f32_weight_expected()
    got = oracle.rms_norm_rope(input_bits, weight, [0], 1, 4, 2, 1e-6, 1_000_000.0, io_bf16=True)
    assert np.array_equal(got.reshape(-1), expected)


def test_oracle_rotation_invariants():
    """What the mathematics fixes: unit RMS after the norm, a rotation per (d, d + rope_dim/2) pair by position * frequency
    (so pair norms are kept and positions add), and untouched dims past rope_dim."""
    rng = np.random.default_rng(5)
    heads, head_dim, rope_dim, theta = 3, 64, 32, 10_000.0
    x = rng.standard_normal((5, heads, head_dim)).astype(np.float32)
    ones = np.ones(head_dim, dtype=np.float32)
    positions = np.array([0, 1, 7, 100, 4095], dtype=np.uint32)
    out = oracle.rms_norm_rope(x, ones, positions, heads, head_dim, rope_dim, 1e-6, theta)
    assert np.allclose(np.sqrt((out.astype(np.float64) ** 2).mean(axis=-1)), 1.0, atol=1e-4)
    normed = x / np.sqrt((x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True) + 1e-6)
    assert np.allclose(out[0], normed[0], atol=1e-6)                                  # position 0: no rotation
    assert np.allclose(out[..., rope_dim:], normed[..., rope_dim:], atol=1e-6)        # not rotated past rope_dim
    half = rope_dim // 2
    frequency = theta ** (-np.arange(half) / half)
    as_complex = normed[..., :half] + 1j * normed[..., half:rope_dim]
    rotated = as_complex * np.exp(1j * positions[:, None, None] * frequency[None, None, :])
    assert np.allclose(out[..., :half], rotated.real, atol=2e-4) and np.allclose(out[..., half:rope_dim], rotated.imag, atol=2e-4)
    # a weight scales dimension-wise before the rotation
    weight = rng.uniform(0.5, 1.5, head_dim).astype(np.float32)
    weighted = oracle.rms_norm_rope(x, weight, np.zeros(5, dtype=np.uint32), heads, head_dim, rope_dim, 1e-6, theta)
    assert np.allclose(weighted, normed * weight, atol=1e-5)


def test_validation_without_a_gpu():
    from khalamari_amd import rms_norm_rope as rnr

    config = rnr.Config.bf16(2, 4, 4, 1e-6, 1_000_000.0).as_struct()
    buffers = _lib.RmsNormRopeBuffers()
    with pytest.raises(_lib.KhmError, match="RMSNorm/RoPE elements exceeds the shader u32 element-index domain"):
        _lib.check(_lib.lib().khm_rms_norm_rope(ctypes.byref(config), 1 << 30, ctypes.byref(buffers), ReplayU32.fixed(1), None, None))
    with pytest.raises(_lib.KhmError, match="rope_dim must be even"):
        rnr.Config.bf16(2, 4, 3, 1e-6, 1_000_000.0).kernel_parameters()
    with pytest.raises(_lib.KhmError, match="must not exceed head_dim"):
        rnr.Config.bf16(2, 4, 6, 1e-6, 1_000_000.0).kernel_parameters()
    with pytest.raises(_lib.KhmError, match="beta_fast must not be below beta_slow"):
        rnr.Config.bf16(2, 128, 128, 1e-6, 1_000_000.0).with_rope_scaling(rnr.Yarn(4.0, 1.0, 1.0, 32.0, 4096, True)).kernel_parameters()
    with pytest.raises(_lib.KhmError, match="replay domain"):
        small = rnr.Config.bf16(2, 4, 4, 1e-6, 1_000_000.0).as_struct()
        _lib.check(_lib.lib().khm_rms_norm_rope(ctypes.byref(small), 4, ctypes.byref(buffers), ReplayU32.fixed(5), None, None))


# ---------------------------------------------------------------------------------------------- GPU


def _run(config, values, weight, positions, active=None, parameters=None):
    import torch

    from khalamari_amd import rms_norm_rope as rnr

    assert torch.cuda.is_available()
    device = torch.device("cuda:0")
    to = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).to(device)  # noqa: E731
    values = np.ascontiguousarray(values)
    output = torch.full((values.nbytes,), 0x55, dtype=torch.uint8, device=device)
    tokens = len(positions)
    rnr.Compute(config).invoke(rnr.Shape(tokens), input=to(values), norm_weight=to(weight), flat_token_indices=to(np.asarray(positions, dtype=np.uint32)),
                               output=output, num_active_tokens=active if active is not None else ReplayU32.fixed(tokens),
                               replay_parameters=parameters)
    torch.cuda.synchronize()
    return output.cpu().numpy().view(values.dtype).reshape(values.shape)


@pytest.mark.gpu
def test_gpu_reference_known_answers():
    from khalamari_amd import rms_norm_rope as rnr

    values, weight_bits, position, expected = _long_context_vectors()
    got = _run(_yarn_config(), values, weight_bits, [position])
    assert np.abs(got - expected).max() < 1e-3, np.abs(got - expected).max()          # the reference's tolerance
    assert np.abs(got - expected).max() < 1e-5, np.abs(got - expected).max()

    input_bits, weight_bits, expected = _rounding_order_expected()
    got = _run(rnr.Config.bf16(1, 4, 2, 1e-6, 1_000_000.0), input_bits, weight_bits, [0])
    assert np.array_equal(got, expected)
    input_bits, weight, expected = _f32_weight_expected()
    got = _run(rnr.Config.bf16(1, 4, 2, 1e-6, 1_000_000.0).with_norm_weight_dtype(DTYPE_F32), input_bits, weight, [0])
    assert np.array_equal(got, expected)


@pytest.mark.gpu
@pytest.mark.parametrize("heads,head_dim,rope_dim,yarn", [(32, 128, 128, False), (8, 128, 128, True), (16, 256, 64, False), (3, 80, 40, True), (2, 72, 36, False),
                                                         (4, 256, 256, False), (4, 256, 128, True), (5, 64, 64, False), (2, 512, 256, False)])
def test_gpu_f32_rows_match_oracle(heads, head_dim, rope_dim, yarn):
    from khalamari_amd import rms_norm_rope as rnr

    rng = np.random.default_rng(heads * head_dim + rope_dim)
    tokens = 19
    values = rng.standard_normal((tokens, heads, head_dim)).astype(np.float32)
    positions = rng.integers(0, 200_000, tokens).astype(np.uint32)
    scaling = dict(YARN, original_max_position_embeddings=4096) if yarn else None
    for weight_dtype in (DTYPE_BF16, DTYPE_F32):
        weight = rng.uniform(0.5, 1.5, head_dim).astype(np.float32)
        if weight_dtype == DTYPE_BF16:
            weight = oracle.f32_to_bf16_bits(weight)
        config = rnr.Config(heads, head_dim, rope_dim, 1e-6, 1_000_000.0, rnr.Yarn(**scaling) if yarn else None, DTYPE_F32, weight_dtype)
        got = _run(config, values, weight, positions)
        want = oracle.rms_norm_rope(values, weight, positions, heads, head_dim, rope_dim, 1e-6, 1_000_000.0, yarn=scaling,
                                    weight_bf16=weight_dtype == DTYPE_BF16)
        # f32 arithmetic in another summation order and a float sine/cosine: a few ulp of values of magnitude ~4
        assert np.abs(got - want).max() < 2e-5, np.abs(got - want).max()


@pytest.mark.gpu
@pytest.mark.parametrize("heads,head_dim,rope_dim,weight_dtype", [(32, 128, 128, DTYPE_BF16), (8, 128, 128, DTYPE_F32), (16, 256, 64, DTYPE_BF16),
                                                                 (6, 256, 256, DTYPE_BF16), (70, 128, 128, DTYPE_BF16)])
def test_gpu_bf16_rows_match_oracle_and_respect_the_active_count(heads, head_dim, rope_dim, weight_dtype):
    import torch

    from khalamari_amd import rms_norm_rope as rnr

    rng = np.random.default_rng(heads + head_dim + rope_dim)
    tokens, active = 23, 17
    values = oracle.f32_to_bf16_bits(rng.standard_normal((tokens, heads, head_dim)).astype(np.float32))
    positions = rng.integers(0, 131_072, tokens).astype(np.uint32)
    weight = rng.uniform(0.5, 1.5, head_dim).astype(np.float32)
    if weight_dtype == DTYPE_BF16:
        weight = oracle.f32_to_bf16_bits(weight)
    config = rnr.Config(heads, head_dim, rope_dim, 1e-6, 1_000_000.0, None, DTYPE_BF16, weight_dtype)
    block = torch.zeros(4, dtype=torch.int32, device="cuda:0")
    block[1] = active
    got = _run(config, values, weight, positions, active=ReplayU32.parameter(1), parameters=block)
    want = oracle.rms_norm_rope(values, weight, positions, heads, head_dim, rope_dim, 1e-6, 1_000_000.0, io_bf16=True,
                                weight_bf16=weight_dtype == DTYPE_BF16)
    assert np.all(got[active:] == 0x5555)                                    # rows past the active count stay untouched
    got_f, want_f = oracle.bf16_bits_to_f32(got[:active]), oracle.bf16_bits_to_f32(want[:active])
    # the same rounding points; an ulp of inv_rms or of the sine can move a value across one bf16 rounding boundary
    # (a rotated value can sit near zero, so the ulp that bounds the difference is that of its pair's magnitude)
    assert np.mean(got[:active] == want[:active]) > 0.99
    half = rope_dim // 2
    magnitude = np.abs(want_f).copy()
    pair = np.hypot(want_f[..., :half], want_f[..., half:rope_dim])
    magnitude[..., :half], magnitude[..., half:rope_dim] = pair, pair
    ulps = np.abs(got_f - want_f) / (np.maximum(magnitude, 2.0 ** -6) * 2.0 ** -7)
    assert np.mean(ulps <= 1.0) > 0.9999 and ulps.max() <= 2.0, (float(ulps.max()), np.unravel_index(np.argmax(ulps), ulps.shape))
    # every head, also those of a second block of a token, is as exact as the others
    assert np.all((got[:active] == want[:active]).mean(axis=(0, 2)) > 0.98)
