"""ctypes loader for `libkhm_gqa_sdpa.so` and the C structs of `include/khm_gqa_sdpa.h`.

There is no fallback path: when the library is missing or fails to load, importing the
component modules raises.  Build it with `python -m khalamari_amd.build`.
"""
from __future__ import annotations

import ctypes
import os

_PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("KHM_LIB_PATH") or os.path.join(_PACKAGE_DIR, "lib", "libkhm_gqa_sdpa.so")

KHM_OK = 0
KHM_ERR_INVALID_ARGUMENT = -1
KHM_ERR_UNSUPPORTED = -2
KHM_ERR_HIP = -3
KHM_ERR_CAPACITY = -4

DTYPE_F32 = 0
DTYPE_BF16 = 1
DTYPE_FP8_E4M3FN = 2
DTYPE_U32 = 3

MAP_SLICED_KV = 0
MAP_Q_TOKENS_PER_HEAD = 1
MAP_Q_HEADS_PER_TOKEN = 2
MAP_Q_TOKENS_AND_HEADS = 3

u32 = ctypes.c_uint32
u64 = ctypes.c_uint64


class KhmError(RuntimeError):
    """A reference `assert!`/`panic!` condition (or a HIP failure) reported by the C ABI."""

    def __init__(self, status: int, message: str):
        super().__init__(f"[khm status {status}] {message}")
        self.status = status
        self.message = message


class ReplayU32(ctypes.Structure):
    """`ReplayU32::{Fixed, Parameter}`."""

    _fields_ = [("is_parameter", u32), ("value", u32)]

    @staticmethod
    def fixed(value: int) -> "ReplayU32":
        return ReplayU32(0, int(value))

    @staticmethod
    def parameter(index: int) -> "ReplayU32":
        return ReplayU32(1, int(index))


class Buffer(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("len_bytes", u64)]


class PageTableLayout(ctypes.Structure):
    _fields_ = [("num_req_slots", u32), ("num_gqa_layers", u32), ("num_blocks", u32), ("num_page_ids_per_block", u32)]


class SdpaConfig(ctypes.Structure):
    _fields_ = [("io_dtype", u32), ("num_q_heads", u32), ("num_kv_heads", u32), ("head_dim", u32), ("tokens_per_page", u32)]


class SdpaVariant(ctypes.Structure):
    _fields_ = [
        ("map_kind", u32), ("map_max_q_tokens", u32), ("map_max_q_heads", u32), ("map_kv_tokens_per_iteration", u32),
        ("map_required_threads", u32), ("kv_cache_tokens_per_page", u32), ("reduce_max_q_tokens", u32),
        ("reduce_max_q_heads", u32), ("reduce_required_threads", u32),
    ]

    def key(self):
        return tuple(getattr(self, name) for name, _ in self._fields_)

    def __eq__(self, other):
        return isinstance(other, SdpaVariant) and self.key() == other.key()

    def __hash__(self):
        return hash(self.key())

    def __repr__(self):
        return "SdpaVariant(" + ", ".join(f"{name}={getattr(self, name)}" for name, _ in self._fields_) + ")"


class GqaSdpaConfig(ctypes.Structure):
    _fields_ = [
        ("num_q_heads", u32), ("num_kv_heads", u32), ("head_dim", u32), ("scale", ctypes.c_float), ("page_bytes", u32),
        ("page_table_layout", PageTableLayout), ("dtype", u32), ("kv_dtype", u32), ("partial_dtype", u32),
    ]


class GqaSdpaShape(ctypes.Structure):
    _fields_ = [("num_total_tokens", u32), ("num_total_q_token_tiles", u32), ("num_total_sdpa_map_task_templates", u32)]


class SlicedKvMapBuffers(ctypes.Structure):
    _fields_ = [(name, Buffer) for name in (
        "q", "kv_pages", "req_slots", "page_ids", "sdpa_map_task_templates", "partial_exp_sums", "partial_max_logits",
        "partial_output")]


class SlicedKvReduceBuffers(ctypes.Structure):
    _fields_ = [(name, Buffer) for name in (
        "partial_exp_sums", "partial_max_logits", "partial_output", "cu_sdpa_partial_outputs", "output")]


class SlicedKvStaticBuffers(ctypes.Structure):
    _fields_ = [(name, Buffer) for name in (
        "q", "kv_pages", "req_slots", "page_ids", "sdpa_map_task_templates", "cu_sdpa_partial_outputs", "output")]


class SlicedQMapBuffers(ctypes.Structure):
    _fields_ = [(name, Buffer) for name in (
        "q", "kv_pages", "req_slots", "page_ids", "visible_kv_token_ranges", "q_token_ranges", "sdpa_map_task_templates",
        "partial_output", "partial_exp_sums", "partial_max_logits")]


class SlicedQDirectBuffers(ctypes.Structure):
    _fields_ = [(name, Buffer) for name in (
        "q", "kv_pages", "req_slots", "page_ids", "visible_kv_token_ranges", "q_token_ranges", "sdpa_map_task_templates",
        "output")]


class SlicedQReduceBuffers(ctypes.Structure):
    _fields_ = [(name, Buffer) for name in (
        "partial_output", "partial_exp_sums", "partial_max_logits", "q_token_ranges", "cu_sdpa_partial_outputs", "output")]


class RequestShape(ctypes.Structure):
    _fields_ = [("num_history_tokens", u32), ("num_q_tokens", u32)]


class GqaReplayShape(ctypes.Structure):
    _fields_ = [
        ("num_tokens", u32), ("num_total_tokens", u32), ("num_q_token_tiles", u32), ("num_total_q_token_tiles", u32),
        ("num_sdpa_map_task_templates", u32), ("num_total_sdpa_map_task_templates", u32),
        ("reduce_sdpa_partial_outputs", u32),
    ]

    def as_tuple(self):
        return (self.num_tokens, self.num_total_tokens, self.num_q_token_tiles, self.num_total_q_token_tiles,
                self.num_sdpa_map_task_templates, self.num_total_sdpa_map_task_templates,
                bool(self.reduce_sdpa_partial_outputs))


class SelectorLimits(ctypes.Structure):
    _fields_ = [("max_tokens", u32), ("max_map_task_templates", u32), ("partial_state_group_capacity", u64)]


class QTokenRange(ctypes.Structure):
    _fields_ = [("request_index", u32), ("flat_q_token_begin", u32), ("flat_q_token_end", u32), ("num_visible_kv_tokens", u32)]


class MapTaskTemplate(ctypes.Structure):
    _fields_ = [("q_token_range_index", u32), ("kv_token_begin", u32), ("kv_token_end", u32)]


class SelectionMetrics(ctypes.Structure):
    _fields_ = [
        ("num_scheduled_qk_token_pairs", u64), ("num_active_qk_token_pairs", u64), ("num_map_threadblocks_per_kv_head", u64),
        ("num_map_simdgroup_waves_per_kv_head", u64), ("num_active_partial_state_groups", u64),
        ("num_active_partial_states", u64), ("num_reserved_partial_state_groups", u64),
        ("num_replay_reserved_partial_state_groups", u64), ("max_kv_iterations_per_split", u32), ("reserved", u32),
        ("num_logical_qk_token_pairs", u64),
    ]


class PageTableLayoutStruct(ctypes.Structure):
    _fields_ = [("num_req_slots", u32), ("num_gqa_layers", u32), ("num_blocks", u32), ("num_page_ids_per_block", u32)]


class KvPageWriteConfig(ctypes.Structure):
    """`kv_page_write::Config` plus the page element type."""

    _fields_ = [("num_kv_heads", u32), ("head_dim", u32), ("page_bytes", u32), ("dtype", u32), ("kv_dtype", u32)]


class ProjectionSplitConfig(ctypes.Structure):
    """`qgkv_split::Config` / `qkv_split::Config` (qgkv_split.rs:34-40)."""

    _fields_ = [("num_q_heads", u32), ("num_kv_heads", u32), ("head_dim", u32), ("dtype", u32)]


class KvPageWriteShape(ctypes.Structure):
    _fields_ = [("num_total_token_writes", u32), ("page_table_layout", PageTableLayoutStruct)]


class KvPageWriteBuffers(ctypes.Structure):
    _fields_ = [("pages", Buffer), ("flat_k", Buffer), ("flat_v", Buffer), ("req_slots", Buffer), ("flat_token_indices", Buffer),
                ("page_ids", Buffer)]


class BidiBlockSdpaConfig(ctypes.Structure):
    """`bidi_block_sdpa::Config`."""

    _fields_ = [("block_size", u32), ("max_q_tokens", u32), ("num_q_heads", u32), ("num_kv_heads", u32), ("head_dim", u32),
                ("scale", ctypes.c_float), ("dtype", u32)]


class BidiBlockSdpaShape(ctypes.Structure):
    _fields_ = [("num_total_tokens", u32), ("num_total_q_token_ranges", u32), ("num_total_partial_output_slots", u32)]


class BidiBlockSdpaBuffers(ctypes.Structure):
    _fields_ = [("q", Buffer), ("local_k", Buffer), ("local_v", Buffer), ("q_token_ranges", Buffer), ("cu_sdpa_partial_outputs", Buffer),
                ("partial_exp_sums", Buffer), ("partial_max_logits", Buffer), ("partial_output", Buffer)]


class BidiBlockCapacity(ctypes.Structure):
    """`BiDiBlockCapacity` + `BiDiBlockGQACapacity`."""

    _fields_ = [("max_requests", u32), ("block_size", u32), ("max_tokens", u32), ("max_q_tokens", u32), ("max_q_token_ranges", u32),
                ("max_sdpa_map_task_templates", u32), ("max_sdpa_partial_state_groups", u64)]


class RopeScalingStruct(ctypes.Structure):
    """`rms_norm_rope::RopeScaling`; kind 0 = default, 1 = Yarn."""

    _fields_ = [("kind", u32), ("factor", ctypes.c_float), ("attention_factor", ctypes.c_float), ("beta_fast", ctypes.c_float),
                ("beta_slow", ctypes.c_float), ("original_max_position_embeddings", u32), ("truncate", u32)]


class RmsNormRopeConfig(ctypes.Structure):
    """`rms_norm_rope::Config`."""

    _fields_ = [("num_heads", u32), ("head_dim", u32), ("rope_dim", u32), ("eps", ctypes.c_float), ("rope_theta", ctypes.c_float),
                ("rope_scaling", RopeScalingStruct), ("dtype", u32), ("norm_weight_dtype", u32)]


class RmsNormRopeBuffers(ctypes.Structure):
    _fields_ = [("input", Buffer), ("norm_weight", Buffer), ("flat_token_indices", Buffer), ("output", Buffer)]


class KNormRopePageWriteBuffers(ctypes.Structure):
    _fields_ = [("pages", Buffer), ("k", Buffer), ("v", Buffer), ("norm_weight", Buffer), ("req_slots", Buffer),
                ("flat_token_indices", Buffer), ("page_ids", Buffer)]


class ProjectionNormRopePageWriteBuffers(ctypes.Structure):
    _fields_ = [("projection", Buffer), ("q_norm_weight", Buffer), ("k_norm_weight", Buffer), ("q_output", Buffer),
                ("gate_output", Buffer), ("pages", Buffer), ("req_slots", Buffer), ("flat_token_indices", Buffer), ("page_ids", Buffer)]


# Every symbol `include/khm_gqa_sdpa.h` declares; checked by tests/test_abi.py.
EXPORTED_SYMBOLS = (
    "khm_last_error", "khm_version",
    "khm_sdpa_variant_sliced_kv", "khm_sdpa_variant_sliced_q", "khm_sdpa_variant_supports", "khm_sdpa_registry_new",
    "khm_sdpa_variant_has_kernel",
    "khm_gqa_sdpa_num_tokens_per_page", "khm_gqa_sdpa_q_bytes", "khm_gqa_sdpa_page_ids_bytes",
    "khm_sliced_kv_partial_output_stats_bytes", "khm_sliced_kv_partial_output_bytes", "khm_sliced_kv_create",
    "khm_sliced_kv_destroy", "khm_sliced_kv_map_kernel_id", "khm_sliced_kv_reduce_kernel_id", "khm_sliced_kv_map",
    "khm_sliced_kv_reduce", "khm_sliced_kv_reduce_gated", "khm_sliced_kv_arrival_counters_bytes", "khm_sliced_kv_map_reduce",
    "khm_sliced_kv_static_scratch_bytes", "khm_sliced_kv_map_reduce_static",
    "khm_sliced_q_partial_output_bytes", "khm_sliced_q_partial_output_stats_bytes", "khm_sliced_q_create",
    "khm_sliced_q_destroy", "khm_sliced_q_map_kernel_id", "khm_sliced_q_map", "khm_sliced_q_direct", "khm_sliced_q_reduce",
    "khm_sliced_q_direct_gated", "khm_sliced_q_reduce_gated",
    "khm_sliced_q_arrival_counters_bytes", "khm_sliced_q_map_reduce",
    "khm_gqa_activation_gate",
    "khm_gqa_qgkv_width", "khm_gqa_qkv_width", "khm_gqa_qgkv_split", "khm_gqa_qkv_split",
    "khm_bf16_to_fp8_e4m3", "khm_fp8_e4m3_to_bf16", "khm_f32_to_bf16", "khm_bf16_to_f32",
    "khm_fp8_e4m3_to_bf16_device", "khm_bf16_to_fp8_e4m3_device",
    "khm_kv_page_write_num_tokens_per_page", "khm_kv_page_write",
    "khm_bidi_block_sdpa",
    "khm_bidi_block_capacity_new", "khm_bidi_block_select", "khm_bidi_block_metadata_compute",
    "khm_rms_norm_rope_yarn_correction_range", "khm_rms_norm_rope_kernel_parameters", "khm_rms_norm_rope",
    "khm_k_norm_rope_page_write", "khm_gqa_projection_norm_rope_page_write",
    "khm_replay_bucket_policy_create", "khm_replay_bucket_policy_destroy", "khm_replay_bucket_policy_max_capacity",
    "khm_replay_bucket_policy_buckets", "khm_replay_bucket_policy_capacity", "khm_replay_bucket_policy_capacity_allow_zero",
    "khm_request_shapes_from_batch",
    "khm_selector_create", "khm_selector_create_for_partitions", "khm_selector_create_for_lookup", "khm_selector_destroy",
    "khm_selector_limits_get", "khm_selector_variants", "khm_selector_select", "khm_selector_select_partitioned",
    "khm_selection_destroy", "khm_selection_variant", "khm_selection_direct_output", "khm_selection_replay_shape",
    "khm_selection_metrics_get", "khm_selection_num_q_token_ranges", "khm_selection_num_map_task_templates",
    "khm_selection_q_token_ranges", "khm_selection_map_task_templates", "khm_selection_cu_partial_outputs",
    "khm_gqa_metadata_create", "khm_gqa_metadata_destroy", "khm_gqa_metadata_update", "khm_gqa_metadata_buffer",
    "khm_gqa_metadata_host", "khm_gqa_metadata_compute",
)

_lib = None


def lib() -> ctypes.CDLL:
    """Load the shared library once; raises when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the gfx950 library has not been built (python -m khalamari_amd.build). "
            "There is no CPU or PyTorch fallback for this path."
        )
    try:
        # torch bundles the HIP runtime it was built with; load it first so both share one runtime instance.
        import torch  # noqa: F401
    except Exception:  # pragma: no cover - torch is optional for the host-only entry points
        pass
    handle = ctypes.CDLL(LIB_PATH)
    handle.khm_last_error.restype = ctypes.c_char_p
    handle.khm_version.restype = ctypes.c_char_p
    for name in ("khm_gqa_sdpa_q_bytes", "khm_gqa_sdpa_page_ids_bytes", "khm_sliced_kv_partial_output_stats_bytes",
                 "khm_sliced_kv_partial_output_bytes", "khm_sliced_q_partial_output_bytes",
                 "khm_sliced_q_partial_output_stats_bytes", "khm_sliced_kv_arrival_counters_bytes",
                 "khm_sliced_q_arrival_counters_bytes"):
        getattr(handle, name).restype = u64
    handle.khm_gqa_sdpa_num_tokens_per_page.restype = u32
    for name in ("khm_sliced_kv_map_kernel_id", "khm_sliced_kv_reduce_kernel_id", "khm_sliced_q_map_kernel_id"):
        getattr(handle, name).restype = ctypes.c_void_p
        getattr(handle, name).argtypes = [ctypes.c_void_p]
    for name in ("khm_sliced_kv_destroy", "khm_sliced_q_destroy"):
        getattr(handle, name).restype = None
        getattr(handle, name).argtypes = [ctypes.c_void_p]
    handle.khm_bf16_to_fp8_e4m3.restype = ctypes.c_uint8
    handle.khm_bf16_to_fp8_e4m3.argtypes = [ctypes.c_uint16]
    handle.khm_fp8_e4m3_to_bf16.restype = ctypes.c_uint16
    handle.khm_fp8_e4m3_to_bf16.argtypes = [ctypes.c_uint8]
    handle.khm_f32_to_bf16.restype = ctypes.c_uint16
    handle.khm_f32_to_bf16.argtypes = [ctypes.c_float]
    handle.khm_bf16_to_f32.restype = ctypes.c_float
    handle.khm_bf16_to_f32.argtypes = [ctypes.c_uint16]
    handle.khm_sliced_kv_map.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedKvMapBuffers), ReplayU32, ReplayU32, ReplayU32,
                                         ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_kv_reduce.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedKvReduceBuffers), ReplayU32, ctypes.c_void_p,
                                            ctypes.c_void_p]
    handle.khm_sliced_kv_reduce_gated.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedKvReduceBuffers), Buffer, ReplayU32,
                                                  ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_kv_map_reduce.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedKvMapBuffers),
                                                ctypes.POINTER(SlicedKvReduceBuffers), Buffer, Buffer, ReplayU32, ReplayU32, ReplayU32,
                                                ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_kv_static_scratch_bytes.restype = ctypes.c_uint64
    handle.khm_sliced_kv_static_scratch_bytes.argtypes = []
    handle.khm_sliced_kv_map_reduce_static.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedKvStaticBuffers), Buffer, ReplayU32,
                                                       ReplayU32, ReplayU32, ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_q_map_reduce.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedQMapBuffers),
                                               ctypes.POINTER(SlicedQReduceBuffers), Buffer, ReplayU32, ReplayU32, ReplayU32, ReplayU32,
                                               ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_q_map.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedQMapBuffers), ReplayU32, ReplayU32, ReplayU32,
                                        ReplayU32, ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_q_direct.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedQDirectBuffers), ReplayU32, ReplayU32,
                                           ReplayU32, ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_q_reduce.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedQReduceBuffers), ReplayU32, ctypes.c_void_p,
                                           ctypes.c_void_p]
    handle.khm_sliced_q_direct_gated.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedQDirectBuffers), Buffer, ReplayU32, ReplayU32,
                                                 ReplayU32, ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_sliced_q_reduce_gated.argtypes = [ctypes.c_void_p, ctypes.POINTER(SlicedQReduceBuffers), Buffer, ReplayU32, ctypes.c_void_p,
                                                 ctypes.c_void_p]
    handle.khm_gqa_activation_gate.argtypes = [u32, u32, u32, u32, Buffer, Buffer, Buffer, ReplayU32, ctypes.c_void_p,
                                               ctypes.c_void_p]
    handle.khm_gqa_qgkv_width.restype = u64
    handle.khm_gqa_qgkv_width.argtypes = [ctypes.POINTER(ProjectionSplitConfig)]
    handle.khm_gqa_qkv_width.restype = u64
    handle.khm_gqa_qkv_width.argtypes = [ctypes.POINTER(ProjectionSplitConfig)]
    handle.khm_gqa_qgkv_split.argtypes = [ctypes.POINTER(ProjectionSplitConfig), u32, Buffer, Buffer, Buffer, Buffer, Buffer, ReplayU32,
                                          ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_gqa_qkv_split.argtypes = [ctypes.POINTER(ProjectionSplitConfig), u32, Buffer, Buffer, Buffer, Buffer, ReplayU32,
                                         ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_fp8_e4m3_to_bf16_device.argtypes = [Buffer, Buffer, u64, ctypes.c_void_p]
    handle.khm_bf16_to_fp8_e4m3_device.argtypes = [Buffer, Buffer, u64, ctypes.c_void_p]
    handle.khm_kv_page_write_num_tokens_per_page.restype = u32
    handle.khm_kv_page_write_num_tokens_per_page.argtypes = [ctypes.POINTER(KvPageWriteConfig)]
    handle.khm_kv_page_write.argtypes = [ctypes.POINTER(KvPageWriteConfig), ctypes.POINTER(KvPageWriteShape),
                                         ctypes.POINTER(KvPageWriteBuffers), ReplayU32, ReplayU32, ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_bidi_block_sdpa.argtypes = [ctypes.POINTER(BidiBlockSdpaConfig), ctypes.POINTER(BidiBlockSdpaShape),
                                           ctypes.POINTER(BidiBlockSdpaBuffers), ReplayU32, ctypes.c_void_p, ctypes.c_void_p]
    u32_p = ctypes.POINTER(u32)
    handle.khm_bidi_block_capacity_new.argtypes = [u32, u32, u32, ctypes.POINTER(BidiBlockCapacity)]
    handle.khm_bidi_block_select.argtypes = [ctypes.POINTER(SdpaConfig), u32, u32, ctypes.POINTER(SdpaVariant), ctypes.POINTER(BidiBlockCapacity)]
    handle.khm_bidi_block_metadata_compute.argtypes = [u32_p, u32, u32_p, u32_p, u32_p, u32, ctypes.POINTER(SdpaVariant), u32, u32, u32_p, u32_p,
                                                       u32_p, u32_p, u32_p, u32_p, ctypes.POINTER(GqaReplayShape)]
    float_p = ctypes.POINTER(ctypes.c_float)
    handle.khm_rms_norm_rope_yarn_correction_range.argtypes = [ctypes.POINTER(RmsNormRopeConfig), float_p, float_p]
    handle.khm_rms_norm_rope_kernel_parameters.argtypes = [ctypes.POINTER(RmsNormRopeConfig), float_p, u32, float_p]
    handle.khm_rms_norm_rope.argtypes = [ctypes.POINTER(RmsNormRopeConfig), u32, ctypes.POINTER(RmsNormRopeBuffers), ReplayU32,
                                         ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_k_norm_rope_page_write.argtypes = [ctypes.POINTER(RmsNormRopeConfig), ctypes.POINTER(KvPageWriteConfig),
                                                  ctypes.POINTER(KvPageWriteShape), ctypes.POINTER(KNormRopePageWriteBuffers), ReplayU32,
                                                  ReplayU32, ctypes.c_void_p, ctypes.c_void_p]
    handle.khm_gqa_projection_norm_rope_page_write.argtypes = [u32, ctypes.POINTER(RmsNormRopeConfig), ctypes.POINTER(RmsNormRopeConfig),
                                                               ctypes.POINTER(KvPageWriteConfig), ctypes.POINTER(KvPageWriteShape),
                                                               ctypes.POINTER(ProjectionNormRopePageWriteBuffers), ReplayU32, ReplayU32,
                                                               ctypes.c_void_p, ctypes.c_void_p]
    _lib = handle
    return handle


def check(status: int) -> int:
    """Raise `KhmError` for a negative status (the binding-side equivalent of the reference's panic)."""
    if status < 0:
        raise KhmError(status, lib().khm_last_error().decode())
    return status
