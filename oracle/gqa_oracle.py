"""ctypes front end of the CPU oracle (``oracle/gqa_oracle.c``) plus numpy helpers.

TEST INFRASTRUCTURE ONLY: importable from ``tests/``, the smoke entry and the
``cpu_baseline`` leg of ``bench.py``.  The product package never imports this module.

Reference citations live in ``gqa_oracle.c``; helpers here that restate reference
fixtures cite them inline.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkhm_gqa_oracle.so")

KV_BF16 = 0
KV_FP8_E4M3FN = 1


def build(force: bool = False) -> str:
    """Compile the C oracle with the committed Makefile and return the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True)
    return _LIB_PATH


class _Geom(ctypes.Structure):
    _fields_ = [
        ("num_q_heads", ctypes.c_uint32),
        ("num_kv_heads", ctypes.c_uint32),
        ("head_dim", ctypes.c_uint32),
        ("tokens_per_page", ctypes.c_uint32),
        ("num_gqa_layers", ctypes.c_uint32),
        ("num_blocks", ctypes.c_uint32),
        ("num_page_ids_per_block", ctypes.c_uint32),
        ("kv_dtype", ctypes.c_uint32),
        ("page_bytes", ctypes.c_uint64),
        ("scale", ctypes.c_float),
        ("reserved", ctypes.c_uint32),
    ]


@dataclass(frozen=True)
class Geometry:
    """Static facts of one paged KV cache + head layout (the oracle's view of `Config`)."""

    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    tokens_per_page: int
    scale: float
    num_gqa_layers: int = 1
    num_blocks: int = 1
    num_page_ids_per_block: int = 1
    kv_dtype: int = KV_BF16

    @property
    def kv_element_bytes(self) -> int:
        return 1 if self.kv_dtype == KV_FP8_E4M3FN else 2

    @property
    def page_bytes(self) -> int:
        return 2 * self.num_kv_heads * self.tokens_per_page * self.head_dim * self.kv_element_bytes

    def _c(self) -> _Geom:
        return _Geom(
            self.num_q_heads, self.num_kv_heads, self.head_dim, self.tokens_per_page, self.num_gqa_layers,
            self.num_blocks, self.num_page_ids_per_block, self.kv_dtype, self.page_bytes, self.scale, 0,
        )


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        handle = ctypes.CDLL(_LIB_PATH)
        handle.khm_oracle_bf16_to_f32.restype = ctypes.c_float
        handle.khm_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        handle.khm_oracle_f32_to_bf16.restype = ctypes.c_uint16
        handle.khm_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        handle.khm_oracle_bf16_to_fp8_e4m3.restype = ctypes.c_uint8
        handle.khm_oracle_bf16_to_fp8_e4m3.argtypes = [ctypes.c_uint16]
        handle.khm_oracle_fp8_e4m3_to_bf16.restype = ctypes.c_uint16
        handle.khm_oracle_fp8_e4m3_to_bf16.argtypes = [ctypes.c_uint8]
        handle.khm_oracle_sigmoid.restype = ctypes.c_float
        handle.khm_oracle_sigmoid.argtypes = [ctypes.c_float]
        handle.khm_oracle_softmax.restype = ctypes.c_int
        handle.khm_oracle_projected_gqa.restype = ctypes.c_int
        handle.khm_oracle_paged_gqa.restype = ctypes.c_int
        handle.khm_oracle_map_partials.restype = ctypes.c_int
        handle.khm_oracle_reduce_sliced_kv.restype = None
        handle.khm_oracle_reduce_sliced_q.restype = None
        handle.khm_oracle_gate_f32.restype = None
        handle.khm_oracle_gate_bf16.restype = None
        handle.khm_oracle_max_threads.restype = ctypes.c_int
        _lib = handle
    return _lib


def _ptr(array: np.ndarray, ctype):
    return array.ctypes.data_as(ctypes.POINTER(ctype))


def _c(array, dtype) -> np.ndarray:
    return np.ascontiguousarray(array, dtype=dtype)


# ---------------------------------------------------------------- numpy twins of the scalar codecs


def f32_to_bf16_bits(values) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16 bit patterns (`half` bf16::from_f32; call sites fp8.rs:11-17)."""
    values = np.ascontiguousarray(values, dtype=np.float32)
    bits = values.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, ((bits >> 16) | 0x40).astype(np.uint16), rounded).reshape(values.shape)


def bf16_bits_to_f32(bits) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32).reshape(bits.shape)


def bf16_round(values) -> np.ndarray:
    return bf16_bits_to_f32(f32_to_bf16_bits(values))


def fp8_decode_table() -> np.ndarray:
    """bf16 bit pattern of every E4M3FN code (fp8.rs:47-58), through the C oracle."""
    handle = lib()
    return np.array([handle.khm_oracle_fp8_e4m3_to_bf16(code) for code in range(256)], dtype=np.uint16)


def bf16_bits_to_fp8(bits) -> np.ndarray:
    """Per-element bf16 -> E4M3FN code (fp8.rs:19-45) through a 65536-entry table from the C oracle."""
    global _ENCODE_TABLE
    if _ENCODE_TABLE is None:
        handle = lib()
        _ENCODE_TABLE = np.array([handle.khm_oracle_bf16_to_fp8_e4m3(code) for code in range(65536)], dtype=np.uint8)
    return _ENCODE_TABLE[np.ascontiguousarray(bits, dtype=np.uint16)]


_ENCODE_TABLE = None


def fp8_round_trip(values) -> np.ndarray:
    """f32 -> bf16 -> fp8 -> bf16 -> f32, the K/V quantisation the reference tests apply (sliced_kv_test.rs:484-489)."""
    codes = bf16_bits_to_fp8(f32_to_bf16_bits(values))
    return bf16_bits_to_f32(fp8_decode_table()[codes])


# ---------------------------------------------------------------- reference fixture generators (data, not code)


def lcg_values(count: int, seed: int) -> np.ndarray:
    """`generated_values` of sliced_kv_test.rs:501-509: LCG in [-1, 1)."""
    out = np.empty(count, dtype=np.float32)
    state = seed & 0xFFFFFFFF
    for i in range(count):
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = np.float32(np.float32(state >> 8) / np.float32(16777216.0)) * np.float32(2.0) - np.float32(1.0)
    return out


def lcg_bf16_values(count: int, seed: int) -> np.ndarray:
    """`generated_bf16_values` of sliced_q_test.rs:611-619: LCG in [-0.5, 0.5), rounded to bf16."""
    out = np.empty(count, dtype=np.float32)
    state = seed & 0xFFFFFFFF
    for i in range(count):
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = np.float32(state >> 8) / np.float32(16777216.0) - np.float32(0.5)
    return bf16_round(out)


def pattern_values(count: int, scale: float, offset: int) -> np.ndarray:
    """`fixture_values` of sliced_kv_test.rs:495-499."""
    index = np.arange(count, dtype=np.int64)
    return (((index * 11 + offset) % 23).astype(np.float32) * np.float32(scale) - np.float32(11.0 * scale)).astype(np.float32)


# ---------------------------------------------------------------- wrapped oracle entry points


def softmax(logits) -> np.ndarray:
    logits = _c(logits, np.float32)
    out = np.empty_like(logits)
    status = lib().khm_oracle_softmax(_ptr(logits, ctypes.c_float), ctypes.c_uint64(logits.size), _ptr(out, ctypes.c_float))
    if status != 0:
        raise ValueError("softmax reference requires finite positive total")
    return out


def sigmoid(value: float) -> float:
    return float(lib().khm_oracle_sigmoid(ctypes.c_float(value)))


def projected_gqa(cu_tokens, token_indices, q, k_by_req, v_by_req, num_q_heads, num_kv_heads, head_dim, scale) -> np.ndarray:
    """Dense causal GQA on f32 inputs (reference.rs:15-78)."""
    cu_tokens = _c(cu_tokens, np.uint32)
    token_indices = _c(token_indices, np.uint32)
    q = _c(q, np.float32)
    ks = [_c(k, np.float32) for k in k_by_req]
    vs = [_c(v, np.float32) for v in v_by_req]
    num_reqs = len(token_indices)
    assert len(cu_tokens) == num_reqs + 1 and len(ks) == num_reqs and len(vs) == num_reqs
    total = int(cu_tokens[-1])
    assert q.size == total * num_q_heads * head_dim
    for r in range(num_reqs):
        context = int(token_indices[r]) + int(cu_tokens[r + 1] - cu_tokens[r])
        assert ks[r].size == context * num_kv_heads * head_dim, "K context length mismatch"
        assert vs[r].size == context * num_kv_heads * head_dim, "V context length mismatch"
    pointer_array = ctypes.POINTER(ctypes.c_float) * num_reqs
    out = np.zeros(total * num_q_heads * head_dim, dtype=np.float32)
    status = lib().khm_oracle_projected_gqa(
        ctypes.c_uint32(num_reqs), _ptr(cu_tokens, ctypes.c_uint32), _ptr(token_indices, ctypes.c_uint32),
        _ptr(q, ctypes.c_float), pointer_array(*[_ptr(k, ctypes.c_float) for k in ks]),
        pointer_array(*[_ptr(v, ctypes.c_float) for v in vs]), ctypes.c_uint32(num_q_heads),
        ctypes.c_uint32(num_kv_heads), ctypes.c_uint32(head_dim), ctypes.c_float(scale), _ptr(out, ctypes.c_float),
    )
    if status != 0:
        raise ValueError(f"projected_gqa oracle failed with status {status}")
    return out.reshape(total, num_q_heads, head_dim)


def paged_gqa(geom: Geometry, q_bits, kv_pages, req_slots, page_ids, visible_ranges, layer: int = 0,
              num_threads: int = 1) -> np.ndarray:
    """Paged attention with per-token visible windows; q as bf16 bit patterns [T, Hq, D]."""
    q_bits = _c(q_bits, np.uint16)
    kv_pages = np.ascontiguousarray(kv_pages).view(np.uint8)
    req_slots = _c(req_slots, np.uint32)
    page_ids = _c(page_ids, np.uint32)
    visible_ranges = _c(visible_ranges, np.uint32).reshape(-1)
    num_tokens = req_slots.size
    assert q_bits.size == num_tokens * geom.num_q_heads * geom.head_dim
    assert visible_ranges.size == 2 * num_tokens
    out = np.zeros((num_tokens, geom.num_q_heads, geom.head_dim), dtype=np.float32)
    c_geom = geom._c()
    status = lib().khm_oracle_paged_gqa(
        ctypes.byref(c_geom), ctypes.c_uint32(num_tokens), _ptr(q_bits, ctypes.c_uint16), _ptr(kv_pages, ctypes.c_uint8),
        _ptr(req_slots, ctypes.c_uint32), _ptr(page_ids, ctypes.c_uint32), ctypes.c_uint32(layer),
        _ptr(visible_ranges, ctypes.c_uint32), _ptr(out, ctypes.c_float), ctypes.c_int(num_threads),
    )
    if status != 0:
        raise ValueError(f"paged_gqa oracle failed with status {status}")
    return out


def map_partials(geom: Geometry, templates, q_token_ranges, max_q_tokens, q_bits, kv_pages, req_slots, page_ids,
                 visible_ranges, layer: int = 0, round_partials_bf16: bool = False, fill: float = np.nan):
    """Partial states of every map task template; returns (exp_sums, max_logits, partial)."""
    templates = _c(templates, np.uint32).reshape(-1, 3)
    q_token_ranges = _c(q_token_ranges, np.uint32).reshape(-1, 2)
    q_bits = _c(q_bits, np.uint16)
    kv_pages = np.ascontiguousarray(kv_pages).view(np.uint8)
    req_slots = _c(req_slots, np.uint32)
    page_ids = _c(page_ids, np.uint32)
    visible_ranges = _c(visible_ranges, np.uint32).reshape(-1)
    num_templates = templates.shape[0]
    stats_shape = (num_templates, geom.num_q_heads, max_q_tokens)
    exp_sums = np.full(stats_shape, fill, dtype=np.float32)
    max_logits = np.full(stats_shape, fill, dtype=np.float32)
    partial = np.full(stats_shape + (geom.head_dim,), fill, dtype=np.float32)
    c_geom = geom._c()
    status = lib().khm_oracle_map_partials(
        ctypes.byref(c_geom), ctypes.c_uint32(num_templates), _ptr(templates, ctypes.c_uint32),
        ctypes.c_uint32(q_token_ranges.shape[0]), _ptr(q_token_ranges, ctypes.c_uint32), ctypes.c_uint32(max_q_tokens),
        _ptr(q_bits, ctypes.c_uint16), _ptr(kv_pages, ctypes.c_uint8), _ptr(req_slots, ctypes.c_uint32),
        _ptr(page_ids, ctypes.c_uint32), ctypes.c_uint32(layer), _ptr(visible_ranges, ctypes.c_uint32),
        ctypes.c_int(1 if round_partials_bf16 else 0), _ptr(exp_sums, ctypes.c_float), _ptr(max_logits, ctypes.c_float),
        _ptr(partial, ctypes.c_float),
    )
    if status != 0:
        raise ValueError(f"map_partials oracle failed with status {status}")
    return exp_sums, max_logits, partial


def reduce_sliced_kv(exp_sums, max_logits, partial, cu_partial_outputs, num_tokens, num_q_heads, head_dim) -> np.ndarray:
    exp_sums = _c(exp_sums, np.float32)
    max_logits = _c(max_logits, np.float32)
    partial = _c(partial, np.float32)
    cu = _c(cu_partial_outputs, np.uint32)
    out = np.zeros((num_tokens, num_q_heads, head_dim), dtype=np.float32)
    lib().khm_oracle_reduce_sliced_kv(
        _ptr(exp_sums, ctypes.c_float), _ptr(max_logits, ctypes.c_float), _ptr(partial, ctypes.c_float),
        _ptr(cu, ctypes.c_uint32), ctypes.c_uint32(num_tokens), ctypes.c_uint32(num_q_heads), ctypes.c_uint32(head_dim),
        _ptr(out, ctypes.c_float),
    )
    return out


def reduce_sliced_q(exp_sums, max_logits, partial, q_token_ranges, cu_partial_outputs, max_q_tokens, num_tokens,
                    num_q_heads, head_dim, fill: float = 0.0) -> np.ndarray:
    exp_sums = _c(exp_sums, np.float32)
    max_logits = _c(max_logits, np.float32)
    partial = _c(partial, np.float32)
    q_token_ranges = _c(q_token_ranges, np.uint32).reshape(-1, 2)
    cu = _c(cu_partial_outputs, np.uint32)
    out = np.full((num_tokens, num_q_heads, head_dim), fill, dtype=np.float32)
    lib().khm_oracle_reduce_sliced_q(
        _ptr(exp_sums, ctypes.c_float), _ptr(max_logits, ctypes.c_float), _ptr(partial, ctypes.c_float),
        _ptr(q_token_ranges, ctypes.c_uint32), _ptr(cu, ctypes.c_uint32), ctypes.c_uint32(q_token_ranges.shape[0]),
        ctypes.c_uint32(max_q_tokens), ctypes.c_uint32(num_q_heads), ctypes.c_uint32(head_dim), _ptr(out, ctypes.c_float),
    )
    return out


def gate_f32(attention, gates) -> np.ndarray:
    attention = _c(attention, np.float32)
    gates = _c(gates, np.float32)
    out = np.empty_like(attention)
    lib().khm_oracle_gate_f32(_ptr(attention, ctypes.c_float), _ptr(gates, ctypes.c_float), ctypes.c_uint64(attention.size),
                              _ptr(out, ctypes.c_float))
    return out


def gate_bf16(attention_bits, gate_bits) -> np.ndarray:
    attention_bits = _c(attention_bits, np.uint16)
    gate_bits = _c(gate_bits, np.uint16)
    out = np.empty_like(attention_bits)
    lib().khm_oracle_gate_bf16(_ptr(attention_bits, ctypes.c_uint16), _ptr(gate_bits, ctypes.c_uint16),
                               ctypes.c_uint64(attention_bits.size), _ptr(out, ctypes.c_uint16))
    return out


def max_threads() -> int:
    return int(lib().khm_oracle_max_threads())


# ---------------------------------------------------------------- per-head RMSNorm + rotary embedding


def yarn_correction_range(rope_dim: int, rope_theta: float, beta_fast: float, beta_slow: float, original_max_position_embeddings: int,
                          truncate: bool):
    """`RopeScaling::yarn_kernel_parameters` (components/rms_norm_rope.rs:206-243): the (low, high) rotary-pair range over
    which Yarn ramps from the unscaled to the interpolated frequency.  f64 inside the logarithms, f32 results."""
    def correction(rotations):
        value = rope_dim * np.log(np.float64(original_max_position_embeddings) / (np.float64(np.float32(rotations)) * 2.0 * np.pi))
        return np.float32(value / (2.0 * np.log(np.float64(np.float32(rope_theta)))))

    low = max(correction(beta_fast), np.float32(0.0))
    high = min(correction(beta_slow), np.float32(max(rope_dim - 1, 0)))
    if truncate:
        low, high = np.floor(low), np.ceil(high)
    if not low <= high:
        raise ValueError("Yarn correction range must be ordered")
    if low == high:
        high = np.float32(high + np.float32(0.001))
    return np.float32(low), np.float32(high)


def rope_kernel_parameters(rope_dim: int, rope_theta: float, yarn=None):
    """`RopeScaling::kernel_parameters` (rms_norm_rope.rs:245-270): (inverse_frequencies f32[rope_dim/2], attention_factor).
    `yarn` is None or a dict with factor, attention_factor, beta_fast, beta_slow, original_max_position_embeddings, truncate."""
    rope_half = rope_dim // 2
    dims = np.arange(rope_half, dtype=np.float32)
    # powf(theta, -(d / half)) with f32 operands, correctly rounded (f64 power, then one rounding), as a libm powf returns;
    # numpy's own f32 power is an ulp off for some pairs, and at position 2^18 one ulp of a frequency moves the output by 1e-2
    inverse = np.power(np.float64(np.float32(rope_theta)), -(dims / np.float32(rope_half)).astype(np.float64)).astype(np.float32)
    if yarn is None:
        return inverse, np.float32(1.0)
    low, high = yarn_correction_range(rope_dim, rope_theta, yarn["beta_fast"], yarn["beta_slow"], yarn["original_max_position_embeddings"],
                                      yarn["truncate"])
    ramp = np.clip((dims - low) / (high - low), np.float32(0.0), np.float32(1.0)).astype(np.float32)
    scale = np.float32(1.0) + ramp * (np.float32(1.0) / np.float32(yarn["factor"]) - np.float32(1.0))
    return (inverse * scale).astype(np.float32), np.float32(yarn["attention_factor"])


def rms_norm_rope(input_values, norm_weight, positions, num_heads: int, head_dim: int, rope_dim: int, eps: float, rope_theta: float,
                  yarn=None, io_bf16: bool = False, weight_bf16: bool = False) -> np.ndarray:
    """`rms_norm_rope_impl` (components/metal/rms_norm_rope.metal:22-120) for rows [T][num_heads][head_dim].

    `input_values` / the result are f32 values, or bf16 bit patterns (uint16) when `io_bf16`; `norm_weight` likewise under
    `weight_bf16`.  With bf16 input AND bf16 weight the normalized value and its product with the weight are each
    rounded to bf16 (apply_norm, rms_norm_rope.metal:14-16); every other combination multiplies in f32.  The square sum
    runs over the row in index order in f32."""
    x = bf16_bits_to_f32(input_values) if io_bf16 else np.asarray(input_values, dtype=np.float32)
    w = bf16_bits_to_f32(norm_weight) if weight_bf16 else np.asarray(norm_weight, dtype=np.float32)
    x = x.reshape(-1, num_heads, head_dim)
    positions = np.asarray(positions, dtype=np.uint32)
    inverse, attention_factor = rope_kernel_parameters(rope_dim, rope_theta, yarn)
    rope_half = rope_dim // 2
    out = np.zeros_like(x)
    for token in range(x.shape[0]):
        theta = (np.float32(positions[token]) * inverse).astype(np.float32)
        # the rotation angle is an f32; its sine and cosine are evaluated in f64 and rounded
        cos, sin = np.cos(theta.astype(np.float64)).astype(np.float32), np.sin(theta.astype(np.float64)).astype(np.float32)
        for head in range(num_heads):
            row = x[token, head]
            acc = np.float32(0.0)
            for value in row:
                acc = np.float32(acc + value * value)
            inv_rms = np.float32(1.0) / np.sqrt(np.float32(acc / np.float32(head_dim) + np.float32(eps)), dtype=np.float32)
            if io_bf16 and weight_bf16:
                normed = bf16_round(w * bf16_round(row * inv_rms))
            else:
                normed = (w * row * inv_rms).astype(np.float32)
            first, second = normed[:rope_half], normed[rope_half:rope_dim]
            out[token, head, :rope_half] = attention_factor * (first * cos - second * sin)
            out[token, head, rope_half:rope_dim] = attention_factor * (first * sin + second * cos)
            out[token, head, rope_dim:] = normed[rope_dim:]
    return f32_to_bf16_bits(out) if io_bf16 else out


# ---------------------------------------------------------------- bidirectional block SDPA


def bidi_block_sdpa(q, local_k, local_v, q_token_ranges, cu_partial_outputs, num_active_q_token_ranges: int, block_size: int,
                    max_q_tokens: int, num_q_heads: int, num_kv_heads: int, head_dim: int, scale: float, num_partial_slots: int):
    """Restatement of gqa_bidi_block_sdpa_impl (components/metal/gqa_bidi_block_sdpa.metal:10-93) in f32: every Q token
    of a range attends, unmasked, to the `block_size` local K/V tokens of its request block
    (`local_kv_token_begin = q_token / block_size * block_size`); the partial state goes to slot
    `cu[range + 1] - 1`.  Inputs are f32 arrays (bf16 inputs are widened by the caller).  Returns
    (exp_sums, max_logits, partial_output) in the partial layout `[slots][Hq][max_q_tokens]([D])`; untouched entries
    are NaN so that a test sees what was written.
    """
    q = np.asarray(q, dtype=np.float32).reshape(-1, num_q_heads, head_dim)
    k = np.asarray(local_k, dtype=np.float32).reshape(-1, num_kv_heads, head_dim)
    v = np.asarray(local_v, dtype=np.float32).reshape(-1, num_kv_heads, head_dim)
    ranges = np.asarray(q_token_ranges, dtype=np.uint32).reshape(-1, 2)
    cu = np.asarray(cu_partial_outputs, dtype=np.uint32).reshape(-1)
    sums = np.full((num_partial_slots, num_q_heads, max_q_tokens), np.nan, dtype=np.float32)
    maxs = np.full_like(sums, np.nan)
    out = np.full((num_partial_slots, num_q_heads, max_q_tokens, head_dim), np.nan, dtype=np.float32)
    ratio = num_q_heads // num_kv_heads
    f32 = np.float32
    for r in range(num_active_q_token_ranges):
        begin, end = int(ranges[r, 0]), int(ranges[r, 1])
        slot = int(cu[r + 1]) - 1
        for offset in range(min(end - begin, max_q_tokens)):
            token = begin + offset
            local_begin = token // block_size * block_size
            for head in range(num_q_heads):
                kv_head = head // ratio
                logits = np.empty(block_size, dtype=np.float32)
                for local in range(block_size):
                    score = f32(0.0)
                    for d in range(head_dim):
                        score = f32(score + f32(q[token, head, d] * k[local_begin + local, kv_head, d]))
                    logits[local] = f32(score * f32(scale))
                block_max = logits.max()
                weights = np.exp((logits - block_max).astype(np.float32)).astype(np.float32)
                exp_sum = f32(0.0)
                for w in weights:
                    exp_sum = f32(exp_sum + w)
                sums[slot, head, offset] = exp_sum
                maxs[slot, head, offset] = block_max
                acc = np.zeros(head_dim, dtype=np.float32)
                for local in range(block_size):
                    acc = (acc + weights[local] * v[local_begin + local, kv_head]).astype(np.float32)
                out[slot, head, offset] = acc / exp_sum if exp_sum > 0 else 0.0
    return sums, maxs, out


# ---------------------------------------------------------------- page write


def kv_page_write(pages, flat_k_bits, flat_v_bits, req_slots, flat_token_indices, page_ids, num_active_token_writes: int,
                  layer: int, num_gqa_layers: int, num_blocks: int, num_page_ids_per_block: int, num_kv_heads: int,
                  head_dim: int, tokens_per_page: int, page_bytes: int, fp8_pages: bool) -> np.ndarray:
    """Restatement of gqa_kv_page_write_impl (components/metal/gqa_kv_page_write.metal:33-80): every active write
    scatters its K and V rows through the page table into `[K|V][Hkv][tokens_per_page][D]` pages.

    `pages` is a uint8 array [num_pages * page_bytes] and is returned modified in a copy; `flat_*_bits` are bf16 bit
    patterns [W, Hkv, D].  FP8 pages store `bf16_bits_to_fp8` codes (the reference), bf16 pages the bits themselves.
    """
    out = np.array(pages, dtype=np.uint8, copy=True).reshape(-1)
    element = 1 if fp8_pages else 2
    k = np.asarray(flat_k_bits, dtype=np.uint16).reshape(-1, num_kv_heads, head_dim)
    v = np.asarray(flat_v_bits, dtype=np.uint16).reshape(-1, num_kv_heads, head_dim)
    table = np.asarray(page_ids, dtype=np.uint32).reshape(-1)
    values_per_plane = num_kv_heads * tokens_per_page * head_dim
    for write in range(num_active_token_writes):
        req_slot = int(req_slots[write])
        token = int(flat_token_indices[write])
        block = token // (tokens_per_page * num_page_ids_per_block)
        page_index = (token // tokens_per_page) % num_page_ids_per_block
        page_id = int(table[((req_slot * num_gqa_layers + layer) * num_blocks + block) * num_page_ids_per_block + page_index])
        page_token = token % tokens_per_page
        for head in range(num_kv_heads):
            offset = (head * tokens_per_page + page_token) * head_dim
            for plane, row in ((0, k[write, head]), (1, v[write, head])):
                begin = page_id * page_bytes + (plane * values_per_plane + offset) * element
                if fp8_pages:
                    out[begin:begin + head_dim] = bf16_bits_to_fp8(row)
                else:
                    out[begin:begin + 2 * head_dim] = row.view(np.uint8)
    return out


# ---------------------------------------------------------------- projection split


def qgkv_split(qgkv, num_q_heads: int, num_kv_heads: int, head_dim: int, num_active_tokens: int, q, g, k, v):
    """Restatement of gqa_qgkv_split_impl (components/metal/gqa_qgkv_split.metal:5-44), every thread id at once: element
    `gid` of the first `num_active_tokens` projection rows goes to q, g, k or v by the shader's own index arithmetic.
    `q`, `g`, `k`, `v` are the buffers' contents before the launch (flat, any element type); modified copies come back."""
    source = np.asarray(qgkv).reshape(-1)
    q, g, k, v = (np.array(a, copy=True).reshape(-1) for a in (q, g, k, v))
    q_slots = num_q_heads * head_dim
    kv_slots = num_kv_heads * head_dim
    token_width = 2 * q_slots + 2 * kv_slots
    gid = np.arange(num_active_tokens * token_width, dtype=np.int64)
    token = gid // token_width
    slot_index = gid - token * token_width
    values = source[gid]
    in_qg = slot_index < 2 * q_slots
    qg_pair = slot_index // (2 * head_dim)
    in_pair = slot_index - qg_pair * 2 * head_dim
    target = (token * num_q_heads + qg_pair) * head_dim + (in_pair % head_dim)
    to_q = in_qg & (in_pair < head_dim)
    to_g = in_qg & ~(in_pair < head_dim)
    q[target[to_q]] = values[to_q]
    g[target[to_g]] = values[to_g]
    slot_index = slot_index - 2 * q_slots
    to_k = ~in_qg & (slot_index < kv_slots)
    k[(token * kv_slots + slot_index)[to_k]] = values[to_k]
    slot_index = slot_index - kv_slots
    to_v = ~in_qg & ~to_k
    v[(token * kv_slots + slot_index)[to_v]] = values[to_v]
    return q, g, k, v


def qkv_split(qkv, num_q_heads: int, num_kv_heads: int, head_dim: int, num_active_tokens: int, q, k, v):
    """Restatement of gqa_qkv_split_impl (components/metal/gqa_qkv_split.metal:5-34), every thread id at once."""
    source = np.asarray(qkv).reshape(-1)
    q, k, v = (np.array(a, copy=True).reshape(-1) for a in (q, k, v))
    q_slots = num_q_heads * head_dim
    kv_slots = num_kv_heads * head_dim
    token_width = q_slots + 2 * kv_slots
    gid = np.arange(num_active_tokens * token_width, dtype=np.int64)
    token = gid // token_width
    slot_index = gid - token * token_width
    values = source[gid]
    to_q = slot_index < q_slots
    q[(token * q_slots + slot_index)[to_q]] = values[to_q]
    slot_index = slot_index - q_slots
    to_k = ~to_q & (slot_index < kv_slots)
    k[(token * kv_slots + slot_index)[to_k]] = values[to_k]
    slot_index = slot_index - kv_slots
    to_v = ~to_q & ~to_k
    v[(token * kv_slots + slot_index)[to_v]] = values[to_v]
    return q, k, v


# ---------------------------------------------------------------- page packing (test helper)


def pack_pages(geom: Geometry, num_pages: int, sequences, page_lists, fill_bits: int = 0) -> np.ndarray:
    """Scatter per-sequence K/V (f32 [ctx, Hkv, D], already representable in the KV dtype) into pages.

    Page layout `[K|V][Hkv][tokens_per_page][D]` (docs/executor_gqa.md:257-258;
    kv_page_values of sliced_kv_test.rs:446-472).  ``page_lists[i][p]`` is the physical page of logical
    page ``p`` of sequence ``i``.  Returns a uint8 array [num_pages, page_bytes].
    """
    tpp, hkv, d = geom.tokens_per_page, geom.num_kv_heads, geom.head_dim
    if geom.kv_dtype == KV_FP8_E4M3FN:
        pages = np.full((num_pages, 2, hkv, tpp, d), fill_bits, dtype=np.uint8)
    else:
        pages = np.full((num_pages, 2, hkv, tpp, d), fill_bits, dtype=np.uint16)
    for (k, v), page_list in zip(sequences, page_lists):
        k = np.asarray(k, dtype=np.float32).reshape(-1, hkv, d)
        v = np.asarray(v, dtype=np.float32).reshape(-1, hkv, d)
        ctx = k.shape[0]
        for plane, values in ((0, k), (1, v)):
            bits = f32_to_bf16_bits(values)
            if geom.kv_dtype == KV_FP8_E4M3FN:
                bits = bf16_bits_to_fp8(bits)
            for p in range((ctx + tpp - 1) // tpp):
                chunk = bits[p * tpp:(p + 1) * tpp]  # [n, Hkv, D]
                pages[page_list[p], plane, :, :chunk.shape[0], :] = chunk.transpose(1, 0, 2)
    return pages.reshape(num_pages, -1).view(np.uint8)
