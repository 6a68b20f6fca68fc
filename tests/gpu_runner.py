"""Runs a Workload through the C ABI on the GPU (torch provides device memory and the stream only)."""
from __future__ import annotations

import gc

import numpy as np
import torch

from khalamari_amd import sdpa, sliced_kv, sliced_q
from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, DTYPE_FP8_E4M3FN, ReplayU32

from oracle import gqa_oracle as oracle


def to_device(array: np.ndarray, device) -> torch.Tensor:
    array = np.ascontiguousarray(array)
    if array.dtype == np.uint16:
        return torch.from_numpy(array.view(np.int16)).to(device)
    if array.dtype == np.uint32:
        return torch.from_numpy(array.view(np.int32)).to(device)
    return torch.from_numpy(array).to(device)


def capture_graph(record) -> torch.cuda.CUDAGraph:
    """`record()` captured into a HIP graph.  A capture is invalidated by any call that frees or allocates device or pinned
    memory in the process while it is open, and Python runs finalizers of dead reference cycles (a metadata buffer set's
    hipFree, say) whenever its cycle collector fires: collect first, and keep the collector off until the capture ends."""
    gc.collect()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    collector_was_on = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            record()
    finally:
        if collector_was_on:
            gc.enable()
    return graph


def bf16_tensor_to_f32(t: torch.Tensor) -> np.ndarray:
    return oracle.bf16_bits_to_f32(t.cpu().numpy().view(np.uint16))


def component_config(w, cls, partial_dtype=DTYPE_BF16, num_req_slots=None):
    g = w.geom
    layout = sliced_kv.Layout(num_req_slots or w.num_req_slots, g.num_gqa_layers, g.num_blocks, g.num_page_ids_per_block)
    kv_dtype = DTYPE_FP8_E4M3FN if g.kv_dtype == oracle.KV_FP8_E4M3FN else DTYPE_BF16
    return cls(g.num_q_heads, g.num_kv_heads, g.head_dim, g.scale, g.page_bytes, layout, DTYPE_BF16, kv_dtype,
               partial_dtype)


def run_sliced_kv(w, templates, cu, device, *, max_q_heads=None, partial_dtype=DTYPE_BF16, pad_templates=0,
                  gates=None, poison=None):
    """Decode path: Map over (token, kv_begin, kv_end) templates, then the flat Reduce.  Returns f32 [T, Hq, D]."""
    g = w.geom
    config = component_config(w, sliced_kv.Config, partial_dtype)
    ratio = g.num_q_heads // g.num_kv_heads
    variant = sdpa.ExecutionVariant.sliced_kv(config.sdpa_config(), min(max(g.head_dim, 32), 256), 128,
                                              max_q_heads or min(ratio, 8))
    templates = np.asarray(templates, dtype=np.uint32).reshape(-1, 3)
    M = templates.shape[0]
    total = M + pad_templates
    padded = np.full((total, 3), 0xFFFFFFFF, dtype=np.uint32)
    padded[:M] = templates
    shape = sliced_kv.Shape(w.num_tokens, total)
    compute = sliced_kv.Compute(config, variant, shape)
    q = to_device(w.q_bits, device)
    pages = to_device(w.kv_pages, device)
    slots = to_device(w.req_slots, device)
    table = to_device(w.page_ids, device)
    tmpl = to_device(padded, device)
    cu_d = to_device(np.asarray(cu, dtype=np.uint32), device)
    scratch = sliced_kv.Scratch(device, config, shape)
    out = torch.zeros((w.num_tokens, g.num_q_heads, g.head_dim), dtype=torch.int16, device=device)
    if poison is not None:
        out.fill_(poison)
    compute.invoke_map(q=q, kv_pages=pages, req_slots=slots, page_ids=table, sdpa_map_task_templates=tmpl,
                       partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                       partial_output=scratch.partial_output, page_table_index=ReplayU32.fixed(w.layer),
                       num_active_tokens=ReplayU32.fixed(w.num_tokens), num_active_kv_splits=ReplayU32.fixed(M))
    gate_d = to_device(gates, device) if gates is not None else None
    compute.invoke_reduce(partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                          partial_output=scratch.partial_output, cu_sdpa_partial_outputs=cu_d, output=out,
                          num_active_tokens=ReplayU32.fixed(w.num_tokens), gates=gate_d)
    torch.cuda.synchronize()
    return bf16_tensor_to_f32(out), scratch


def run_sliced_q(w, ranges, templates, cu, device, *, kind, max_q_tokens, max_q_heads, stage=16, direct=False,
                 partial_dtype=DTYPE_BF16, poison=0x4228, visible=None, gates=None):
    """Verify / prefill path: Map (or direct) over Q ranges, then the ranged Reduce; `gates` (bf16 bits [T, Hq, D]) fuses
    the sigmoid gate into whichever of the two writes the output.  Returns f32 [T, Hq, D]."""
    g = w.geom
    config = component_config(w, sliced_q.Config, partial_dtype)
    variant = sdpa.ExecutionVariant.sliced_q(config.sdpa_config(), kind, max_q_tokens, stage, max_q_heads)
    ranges = np.asarray(ranges, dtype=np.uint32).reshape(-1, 2)
    templates = np.asarray(templates, dtype=np.uint32).reshape(-1, 3)
    shape = sliced_q.Shape(w.num_tokens, ranges.shape[0], templates.shape[0])
    compute = sliced_q.Compute(config, variant, shape, direct=direct)
    q = to_device(w.q_bits, device)
    pages = to_device(w.kv_pages, device)
    slots = to_device(w.req_slots, device)
    table = to_device(w.page_ids, device)
    vis = to_device(np.asarray(w.visible if visible is None else visible, dtype=np.uint32), device)
    rng_d = to_device(ranges, device)
    tmpl = to_device(templates, device)
    out = torch.full((w.num_tokens, g.num_q_heads, g.head_dim), poison, dtype=torch.int16, device=device)
    common = dict(q=q, kv_pages=pages, req_slots=slots, page_ids=table, visible_kv_token_ranges=vis, q_token_ranges=rng_d,
                  sdpa_map_task_templates=tmpl, page_table_index=ReplayU32.fixed(w.layer),
                  num_active_tokens=ReplayU32.fixed(w.num_tokens),
                  num_active_q_token_tiles=ReplayU32.fixed(ranges.shape[0]))
    gates_d = to_device(gates, device) if gates is not None else None
    if direct:
        compute.invoke_direct(output=out, gates=gates_d, **common)
    else:
        partial = torch.zeros(config.partial_output_bytes(variant, shape), dtype=torch.uint8, device=device)
        sums = torch.zeros(config.partial_output_stats_bytes(variant, shape), dtype=torch.uint8, device=device)
        maxs = torch.zeros(config.partial_output_stats_bytes(variant, shape), dtype=torch.uint8, device=device)
        cu_d = to_device(np.asarray(cu, dtype=np.uint32), device)
        compute.invoke_map(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                           num_active_kv_splits=ReplayU32.fixed(templates.shape[0]), **common)
        compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs, q_token_ranges=rng_d,
                              cu_sdpa_partial_outputs=cu_d, output=out,
                              num_active_q_token_tiles=ReplayU32.fixed(ranges.shape[0]), gates=gates_d)
    torch.cuda.synchronize()
    return bf16_tensor_to_f32(out)
