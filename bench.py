#!/usr/bin/env python3
"""Benchmark of the paged GQA split-KV SDPA path on one MI355X.

`python bench.py [--gpus 1] [--steps K] [--warmup W]` prints ONE JSON line.  A step is one pass of the
hot path (Map + Reduce, or the direct Map) over one batch of synthetic input that already sits in HBM.
The headline workload is config 2 (32 ragged decode requests, 512-token split-KV partitions);
the other synthetic configs are timed briefly and reported under "configs".

Inputs: Q/K/V ~ N(0,1) rounded to bf16 (generated on the device, fixed seeds), context lengths and page
permutations from numpy's PCG64 seeded with the config index.  KV pools rotate between steps (three
distinct pools) so no pool stays resident in the 256 MB Infinity Cache: the HBM figure is a cold one.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
TOKENS_PER_PAGE = 16
NUM_POOLS = 3
# HBM bytes per Map launch from the hardware counters, (FETCH_SIZE * 2.000 + WRITE_SIZE * 1.000) KiB per dispatch:
# two `rocprofv3 --pmc` runs per config, each counter scaled by what it reads for a plain 1 GiB copy kernel
# (`--calibration-copy`).  The summaries with their commands are the text files under profiles/.
MEASURED_MAP_TRAFFIC_BYTES = {2: 565_561_344, 3: 2_153_930_752, 4: 1_446_890_496, 5: 1_202_827_264, 6: 1_068_915_712}
MEASURED_MAP_TRAFFIC_BYTES_FP8_PAGES = {2: 286_631_936, 3: 1_082_411_008, 4: 729_135_104, 5: 869_629_952, 6: 1_614_041_088}

CONFIGS = {
    1: dict(name="config1: B=1 q=1 Hq32/Hkv8/D128 ctx 1024, identity pages", hq=32, hkv=8, d=128, kind="decode", kv_slice=64),
    2: dict(name="config2: B=32 q=1 Hq64/Hkv8/D128 ctx U[512,8192], 20480-page pool, 512-token partitions + LSE reduce",
            hq=64, hkv=8, d=128, kind="decode", kv_slice=512),
    3: dict(name="config3: B=4 q=1 Hq24/Hkv4/D256 ctx 131072, 2048-token partitions, output x sigmoid(gate)",
            hq=24, hkv=4, d=256, kind="decode", kv_slice=2048, gated=True),
    4: dict(name="config4: B=16 spec-verify q=1+k (k in 1..4), ctx U[4096,32768], Hq64/Hkv8/D128", hq=64, hkv=8, d=128,
            kind="verify"),
    5: dict(name="config5: B=8 chunked prefill, 2048-token chunk on prefix U[0,16384], Hq64/Hkv8/D128", hq=64, hkv=8, d=128,
            kind="prefill"),
}
# Not a benchmark config: the lengths of config 5 on the head geometry of config 3, so that the D 256 prefill tiles
# have a measured figure too.  Reported under "configs" as "extra_prefill_d256"; selectable with --config 6.
EXTRA_PREFILL_D256 = 6
CONFIGS[EXTRA_PREFILL_D256] = dict(name="extra: B=8 chunked prefill, 2048-token chunk on prefix U[0,16384], Hq24/Hkv4/D256",
                                   hq=24, hkv=4, d=256, kind="prefill")


SLAB_BYTES = 4096
_slab_reader_lib = None


def slab_read(pool, slab_ids, num_slabs: int, sink, blocks_per_cu: int = 2, run_slabs: int = 1, slab_bytes: int = SLAB_BYTES) -> None:
    """Enqueues, on torch's current stream, a launch that only reads `num_slabs` slabs of `slab_bytes` (4096 or 2048)
    bytes of `pool` from a resident grid, in the Map kernel's lane layout: slab i at byte offset `slab_ids[i] * slab_bytes`,
    or with `run_slabs` > 1 runs of that many consecutive slabs, run j at `slab_ids[j] * run_slabs * slab_bytes`.  The kernel lives in
    `libbench_slab_read.so` beside this file (source `bench_slab_read.hip`): a measurement aid, not part of the library."""
    import ctypes

    import torch

    def nbytes(t):
        return t.numel() * t.element_size()

    status = _bench_aid_lib().bench_slab_read(pool.data_ptr(), nbytes(pool), slab_ids.data_ptr(), nbytes(slab_ids), int(num_slabs),
                                              int(run_slabs), int(slab_bytes), int(blocks_per_cu), sink.data_ptr(), nbytes(sink),
                                              ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    if status != 0:
        raise RuntimeError(f"bench_slab_read failed with status {status}")


def _bench_aid_lib():
    import ctypes

    global _slab_reader_lib
    if _slab_reader_lib is None:
        path = os.path.join(ROOT, "libbench_slab_read.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: run `python -m khalamari_amd.build` (or __graft_entry__.build()) first")
        _slab_reader_lib = ctypes.CDLL(path)
        _slab_reader_lib.bench_slab_read.restype = ctypes.c_int
        _slab_reader_lib.bench_slab_read.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32,
                                                     ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_uint64,
                                                     ctypes.c_void_p]
    return _slab_reader_lib


def config_key(index: int) -> str:
    return "extra_prefill_d256" if index == EXTRA_PREFILL_D256 else f"config{index}"


def sample_lengths(index: int):
    """(histories, q_lens) of a config; numpy PCG64 seeded with the config index."""
    if index == EXTRA_PREFILL_D256:
        return sample_lengths(5)
    rng = np.random.default_rng(index)
    if index == 1:
        return [1023], [1]
    if index == 2:
        contexts = rng.integers(512, 8193, size=32)
        return [int(c) - 1 for c in contexts], [1] * 32
    if index == 3:
        return [131071] * 4, [1] * 4
    if index == 4:
        prior = rng.integers(4096, 32769, size=16)
        drafts = rng.integers(1, 5, size=16)
        return [int(p) for p in prior], [1 + int(k) for k in drafts]
    if index == 5:
        prefix = rng.integers(0, 16385, size=8)
        return [int(p) for p in prefix], [2048] * 8
    raise ValueError(index)


class Workload:
    """One synthetic config resident in HBM plus its recorded launches."""

    def __init__(self, index: int, device, num_pools: int = NUM_POOLS, fp8_pages: bool = False):
        import torch

        from khalamari_amd import batch_metadata, sdpa, sliced_kv, sliced_q
        from khalamari_amd import kv_page_write
        from khalamari_amd._lib import DTYPE_BF16, DTYPE_F32, DTYPE_FP8_E4M3FN, ReplayU32
        from khalamari_amd.selector import GQAReplayBucketPolicy, RequestShape, Selector

        spec = CONFIGS[index]
        self.index, self.spec, self.device = index, spec, device
        hq, hkv, d = spec["hq"], spec["hkv"], spec["d"]
        self.histories, self.q_lens = sample_lengths(index)
        contexts = [h + n for h, n in zip(self.histories, self.q_lens)]
        num_requests = len(contexts)
        pages_per_request = [-(-c // TOKENS_PER_PAGE) for c in contexts]
        pool_pages = max(sum(pages_per_request), 20480 if index == 2 else 0)
        num_blocks = max(pages_per_request)
        rng = np.random.default_rng(1000 + index)
        order = np.arange(pool_pages) if index == 1 else rng.permutation(pool_pages)
        table = np.zeros((num_requests, num_blocks), dtype=np.uint32)
        cursor = 0
        for r, n in enumerate(pages_per_request):
            table[r, :n] = order[cursor:cursor + n]
            cursor += n
        # FP8 E4M3FN pages (the reference's cache format, 32 KiB at these geometries) or bf16 pages (what the five benchmark configs are defined on)
        self.fp8_pages = fp8_pages
        self.kv_element_bytes = 1 if fp8_pages else 2
        kv_dtype = DTYPE_FP8_E4M3FN if fp8_pages else DTYPE_BF16
        self.page_bytes = 2 * hkv * TOKENS_PER_PAGE * d * self.kv_element_bytes
        generator = torch.Generator(device=device)
        generator.manual_seed(index)
        self.kv_pools = []
        for _ in range(num_pools):
            values = torch.randn(pool_pages * self.page_bytes // self.kv_element_bytes, device=device, dtype=torch.float32,
                                 generator=generator).to(torch.bfloat16)
            if fp8_pages:
                codes = torch.empty(values.numel(), dtype=torch.uint8, device=device)
                kv_page_write.fp8_encode_device(values, codes, values.numel())
                values = codes
            self.kv_pools.append(values)
        torch.cuda.synchronize()
        self.num_tokens = sum(self.q_lens)
        self.q = torch.randn((self.num_tokens, hq, d), device=device, dtype=torch.float32, generator=generator).to(torch.bfloat16)
        self.gates = None
        if spec.get("gated"):
            self.gates = torch.randn((self.num_tokens, hq, d), device=device, dtype=torch.float32, generator=generator).to(torch.bfloat16)
        self.page_table = torch.from_numpy(table.reshape(-1).view(np.int32)).to(device)
        self.table_host = table
        self.out = torch.zeros((self.num_tokens, hq, d), dtype=torch.bfloat16, device=device)

        # prepare: selector -> metadata, as GQA::prepare does once per batch
        layout = sliced_kv.Layout(num_requests, 1, num_blocks, 1)
        sconfig = sdpa.Config(DTYPE_BF16, hq, hkv, d, TOKENS_PER_PAGE)
        cu_tokens = [0]
        for n in self.q_lens:
            cu_tokens.append(cu_tokens[-1] + n)
        shapes = RequestShape.from_batch(self.histories, cu_tokens)
        ratio = hq // hkv
        if spec["kind"] == "decode":
            variant = sdpa.ExecutionVariant.sliced_kv(sconfig, d, 128, min(ratio, 8))
            max_splits = max(-(-c // spec["kv_slice"]) for c in contexts)
            selector = Selector.for_partitions(sdpa.Registry.from_variants(sconfig, [variant]), self.num_tokens, num_requests,
                                               lambda v: max_splits)
            limits = selector.limits()
            policy = GQAReplayBucketPolicy(limits.max_tokens, limits.max_map_task_templates)
            selection = selector.select_partitioned(variant, spec["kv_slice"], False, shapes, policy, self.num_tokens)
        else:
            selector = Selector.for_lookup(sconfig, self.num_tokens, layout)
            limits = selector.limits()
            policy = GQAReplayBucketPolicy(limits.max_tokens, limits.max_map_task_templates)
            selection = selector.select(shapes, policy, self.num_tokens)
        self.selection = selection
        self.variant = selection.variant()
        self.direct = selection.direct_output()
        self.metadata = batch_metadata.GQAMetadataBuffers(limits.max_tokens, limits.max_map_task_templates)
        shape = self.metadata.update(list(range(num_requests)), self.histories, cu_tokens, selection)
        self.replay_shape = shape
        self.visible_tokens = sum(contexts)
        partial_dtype = DTYPE_F32 if os.environ.get("KHM_BENCH_PARTIAL", "bf16") == "f32" else DTYPE_BF16
        fixed = ReplayU32.fixed
        md = self.metadata
        # The launch closures hold these tensors, not the workload: a closure over `self` stored on `self` is a reference
        # cycle, and a workload in a cycle keeps its device memory until the cycle collector runs, whenever that is.
        q, page_table, out, gates = self.q, self.page_table, self.out, self.gates
        # Map and Reduce in one launch (the last block of a token merges) pays off when the step is launch-latency
        # bound; large batches keep the two-launch form.  KHM_BENCH_FUSED=0/1 forces either.
        choice = os.environ.get("KHM_BENCH_FUSED", "auto")
        fused = choice == "1" or (choice == "auto" and self.visible_tokens * hkv * d * 4 < (64 << 20))
        fused = fused and not self.direct
        self.fused = fused
        if self.variant.map_kind == sdpa.MAP_SLICED_KV:
            config = sliced_kv.Config(hq, hkv, d, d ** -0.5, self.page_bytes, layout, DTYPE_BF16, kv_dtype, partial_dtype)
            kshape = sliced_kv.Shape(shape.num_total_tokens, shape.num_total_sdpa_map_task_templates)
            compute = sliced_kv.Compute(config, self.variant, kshape)
            scratch = sliced_kv.Scratch(device, config, kshape)
            self._keep = (compute, scratch)

            def launch_map(pool):
                compute.invoke_map(q=q, kv_pages=pool, req_slots=md.req_slots(), page_ids=page_table,
                                   sdpa_map_task_templates=md.sdpa_map_task_templates(), partial_exp_sums=scratch.partial_exp_sums,
                                   partial_max_logits=scratch.partial_max_logits, partial_output=scratch.partial_output,
                                   page_table_index=fixed(0), num_active_tokens=fixed(shape.num_tokens),
                                   num_active_kv_splits=fixed(shape.num_sdpa_map_task_templates))

            def launch_reduce(gates=gates):
                compute.invoke_reduce(partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                                      partial_output=scratch.partial_output, cu_sdpa_partial_outputs=md.cu_sdpa_partial_outputs(),
                                      output=out, num_active_tokens=fixed(shape.num_tokens), gates=gates)

            if fused:
                counters = torch.zeros(compute.arrival_counters_bytes(), dtype=torch.uint8, device=device)
                self._keep += (counters,)

                def launch_map(pool):  # noqa: F811
                    compute.invoke_map_reduce(q=q, kv_pages=pool, req_slots=md.req_slots(), page_ids=page_table,
                                              sdpa_map_task_templates=md.sdpa_map_task_templates(),
                                              partial_exp_sums=scratch.partial_exp_sums, partial_max_logits=scratch.partial_max_logits,
                                              partial_output=scratch.partial_output,
                                              cu_sdpa_partial_outputs=md.cu_sdpa_partial_outputs(), output=out,
                                              arrival_counters=counters, page_table_index=fixed(0),
                                              num_active_tokens=fixed(shape.num_tokens),
                                              num_active_kv_splits=fixed(shape.num_sdpa_map_task_templates), gates=gates)

                launch_reduce = None
        else:
            config = sliced_q.Config(hq, hkv, d, d ** -0.5, self.page_bytes, layout, DTYPE_BF16, kv_dtype, partial_dtype)
            qshape = sliced_q.Shape(shape.num_total_tokens, shape.num_total_q_token_tiles, shape.num_total_sdpa_map_task_templates)
            common = dict(q=q, req_slots=md.req_slots(), page_ids=page_table,
                          visible_kv_token_ranges=md.visible_kv_token_ranges(), q_token_ranges=md.q_token_ranges(),
                          sdpa_map_task_templates=md.sdpa_map_task_templates(), page_table_index=fixed(0),
                          num_active_tokens=fixed(shape.num_tokens), num_active_q_token_tiles=fixed(shape.num_q_token_tiles))
            if self.direct:
                compute = sliced_q.Compute.new_direct(config, self.variant, qshape)
                self._keep = (compute,)

                def launch_map(pool, gates=gates):
                    compute.invoke_direct(kv_pages=pool, output=out, gates=gates, **common)

                launch_reduce = None
            else:
                compute = sliced_q.Compute.new(config, self.variant, qshape)
                partial = torch.zeros(config.partial_output_bytes(self.variant, qshape), dtype=torch.uint8, device=device)
                sums = torch.zeros(config.partial_output_stats_bytes(self.variant, qshape), dtype=torch.uint8, device=device)
                maxs = torch.zeros_like(sums)
                self._keep = (compute, partial, sums, maxs)

                def launch_map(pool):
                    compute.invoke_map(kv_pages=pool, partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                                       num_active_kv_splits=fixed(shape.num_sdpa_map_task_templates), **common)

                def launch_reduce(gates=gates):
                    compute.invoke_reduce(partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                                          q_token_ranges=md.q_token_ranges(), cu_sdpa_partial_outputs=md.cu_sdpa_partial_outputs(),
                                          output=out, num_active_q_token_tiles=fixed(shape.num_q_token_tiles), gates=gates)

                if fused:
                    counters = torch.zeros(compute.arrival_counters_bytes(), dtype=torch.uint8, device=device)
                    self._keep += (counters,)

                    def launch_map(pool):  # noqa: F811
                        compute.invoke_map_reduce(kv_pages=pool, partial_output=partial, partial_exp_sums=sums, partial_max_logits=maxs,
                                                  cu_sdpa_partial_outputs=md.cu_sdpa_partial_outputs(), output=out,
                                                  arrival_counters=counters,
                                                  num_active_kv_splits=fixed(shape.num_sdpa_map_task_templates), **common)

                    launch_reduce = None
        self.launch_map, self.launch_reduce = launch_map, launch_reduce

    # ---- algorithmic work ------------------------------------------------------------------------------
    def algorithmic_bytes(self) -> int:
        """K/V bytes of every visible token once per sequence, plus Q, output and page-table reads."""
        spec = self.spec
        kv = self.visible_tokens * spec["hkv"] * spec["d"] * 2 * self.kv_element_bytes
        qo = 2 * self.num_tokens * spec["hq"] * spec["d"] * 2
        table = sum(-(-(h + n) // TOKENS_PER_PAGE) for h, n in zip(self.histories, self.q_lens)) * 4
        return kv + qo + table

    def algorithmic_flops(self) -> int:
        """4 * Hq * D * sum(C * P + C (C + 1) / 2): two GEMMs, causal-exact."""
        spec = self.spec
        pairs = sum(n * h + n * (n + 1) // 2 for h, n in zip(self.histories, self.q_lens))
        return 4 * spec["hq"] * spec["d"] * pairs

    def map_kernel_name(self) -> str:
        """Name of the HIP kernel the Map launch runs: one 16-column tile (decode) uses the split-KV kernel whose waves
        share nothing, wider Q tiles the LDS-tiled kernel."""
        coordinates = int(self.variant.map_max_q_tokens) * int(self.variant.map_max_q_heads)
        from khalamari_amd import sdpa

        if self.variant.map_kind == sdpa.MAP_SLICED_KV or coordinates <= 16:
            return "split_kv_map_kernel"
        return "tile_map_kernel"

    def step(self, i: int) -> None:
        self.launch_map(self.kv_pools[i % len(self.kv_pools)])
        if self.launch_reduce is not None:
            self.launch_reduce()

    def time_steps(self, steps: int, warmup: int):
        """(ms per step over a clean timed region, mean Map-kernel ms from per-launch HIP events)."""
        import torch

        for i in range(warmup):
            self.step(i)
        torch.cuda.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for i in range(steps):
            self.step(i)
        end.record()
        torch.cuda.synchronize()
        ms_per_step = begin.elapsed_time(end) / steps
        # per-kernel region: events on the launch stream around every Map launch
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for i, (a, b) in enumerate(pairs):
            a.record()
            self.launch_map(self.kv_pools[i % len(self.kv_pools)])
            b.record()
            if self.launch_reduce is not None:
                self.launch_reduce()
        torch.cuda.synchronize()
        map_ms = sorted(a.elapsed_time(b) for a, b in pairs)
        return ms_per_step, float(np.mean(map_ms)), float(map_ms[len(map_ms) // 2])

    def slab_reader(self, steps: int) -> dict:
        """The memory system's own figure for this launch: a kernel that only reads as many bytes as the workload's
        visible K/V, as slabs (4 KB; 2 KB on FP8 pages at head_dim 128: what one page holds contiguously for one plane and
        KV head) at random places of the same pools (rotated like the steps), from a resident grid
        with every wave the same share.  No metadata chain, no softmax, no merge, no ragged tail."""
        import torch

        spec = self.spec
        kv_bytes = self.visible_tokens * spec["hkv"] * spec["d"] * 2 * self.kv_element_bytes
        # what one (page, plane, KV head) holds contiguously, capped at 4 KB: 2 KB on FP8 pages at head_dim 128
        slab_bytes = min(SLAB_BYTES, TOKENS_PER_PAGE * spec["d"] * self.kv_element_bytes)
        pool_slabs = self.kv_pools[0].numel() * self.kv_pools[0].element_size() // slab_bytes
        num_slabs = min(kv_bytes // slab_bytes, pool_slabs)
        order = np.random.Generator(np.random.PCG64(1234)).permutation(pool_slabs)[:num_slabs].astype(np.uint32)
        slab_ids = torch.from_numpy(order.view(np.int32)).to(self.kv_pools[0].device)
        sink = torch.zeros(1, dtype=torch.int32, device=slab_ids.device)
        best = None
        for blocks_per_cu in (2, 4):
            for i in range(3):
                slab_read(self.kv_pools[i % len(self.kv_pools)], slab_ids, num_slabs, sink, blocks_per_cu, 1, slab_bytes)
            pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
            for i, (a, b) in enumerate(pairs):
                a.record()
                slab_read(self.kv_pools[i % len(self.kv_pools)], slab_ids, num_slabs, sink, blocks_per_cu, 1, slab_bytes)
                b.record()
            torch.cuda.synchronize()
            mean_us = float(np.mean([a.elapsed_time(b) for a, b in pairs])) * 1e3
            if best is None or mean_us < best["us"]:
                best = {"us": mean_us, "blocks_per_cu": blocks_per_cu}
        nbytes = num_slabs * slab_bytes
        best.update(bytes=int(nbytes), gbps=nbytes / (best["us"] * 1e-6) / 1e9, slab_bytes=int(slab_bytes),
                    what=f"read-only launch of the workload's K/V bytes as random {slab_bytes // 1024} KB slabs of the same pools, evenly split over a resident grid")
        return best

    def report(self, steps: int, warmup: int) -> dict:
        ms, map_ms, map_ms_median = self.time_steps(steps, warmup)
        spec = self.spec
        result = {
            "workload": spec["name"] + (" [FP8 E4M3FN pages]" if self.fp8_pages else ""),
            "us_per_step": ms * 1e3,
            "map_kernel_us": map_ms * 1e3,
            "map_kernel_us_median": map_ms_median * 1e3,
            "map_kernel": self.map_kernel_name(),
            "map_kind": int(self.variant.map_kind),
            "map_tile": [int(self.variant.map_max_q_tokens), int(self.variant.map_max_q_heads)],
            "direct_output": bool(self.direct),
            "fused_reduce": bool(self.fused),
            "map_task_templates": int(self.replay_shape.num_sdpa_map_task_templates),
            "visible_kv_tokens": int(self.visible_tokens),
        }
        if spec["kind"] == "prefill":
            flops = self.algorithmic_flops()
            result.update(bound="mfma", algorithmic_flops=flops, tflops=flops / (ms * 1e-3) / 1e12,
                          map_tflops=flops / (map_ms * 1e-3) / 1e12)
            result["roofline_frac"] = result["map_tflops"] / MFMA_BF16_PEAK_TFLOPS
        else:
            nbytes = self.algorithmic_bytes()
            result.update(bound="hbm", algorithmic_bytes=nbytes, gbps=nbytes / (ms * 1e-3) / 1e9,
                          map_gbps=nbytes / (map_ms * 1e-3) / 1e9)
            result["roofline_frac"] = result["map_gbps"] / HBM_PEAK_GBPS
            result["slab_reader"] = self.slab_reader(min(steps, 50))
        return result


def cpu_baseline(index: int = 2, seconds_hint: float = 20.0) -> dict:
    """Times the CPU oracle (a port of the reference's scalar f32 attention, gathering through the page table) on a
    bounded sample of the headline workload: the shortest sequences of config 2 until about `seconds_hint` of
    single-thread work is reached, once single-threaded and once on all host cores."""
    from oracle import gqa_oracle as oracle

    spec = CONFIGS[index]
    histories, q_lens = sample_lengths(index)
    order = np.argsort(histories)
    hq, hkv, d = spec["hq"], spec["hkv"], spec["d"]
    # about 0.25 G multiply-adds per second per thread for the strictly ordered scalar loops
    budget_tokens = int(seconds_hint * 0.25e9 / (hq * d * 2))
    chosen, total = [], 0
    for r in order:
        if chosen and total + histories[r] + 1 > budget_tokens:
            break
        chosen.append(int(r))
        total += histories[r] + 1
    rng = np.random.default_rng(7)
    sample_hist = [histories[r] for r in chosen]
    contexts = [h + 1 for h in sample_hist]
    pages = [-(-c // TOKENS_PER_PAGE) for c in contexts]
    geom = oracle.Geometry(hq, hkv, d, TOKENS_PER_PAGE, d ** -0.5, 1, max(pages), 1)
    order_pages = rng.permutation(sum(pages))
    table = np.zeros((len(chosen), max(pages)), dtype=np.uint32)
    cursor = 0
    for i, n in enumerate(pages):
        table[i, :n] = order_pages[cursor:cursor + n]
        cursor += n
    kv = oracle.f32_to_bf16_bits(rng.standard_normal(sum(pages) * geom.page_bytes // 2, dtype=np.float32))
    q = oracle.f32_to_bf16_bits(rng.standard_normal((len(chosen), hq, d), dtype=np.float32))
    slots = np.arange(len(chosen), dtype=np.uint32)
    visible = np.array([[0, c] for c in contexts], dtype=np.uint32)
    nbytes = sum(contexts) * hkv * d * 4
    timings, passes = {}, {}
    threads = oracle.max_threads()
    # the whole config is well under a second of CPU work: repeat it until each leg has run for a few seconds
    for label, n, seconds in (("single_thread", 1, 8.0), ("all_cores", threads, 4.0)):
        count, elapsed = 0, 0.0
        while elapsed < seconds and count < 64:
            start = time.perf_counter()
            oracle.paged_gqa(geom, q, kv.view(np.uint8), slots, table.reshape(-1), visible, num_threads=n)
            elapsed += time.perf_counter() - start
            count += 1
        timings[label] = elapsed / count
        passes[label] = count
    return {
        "value": nbytes / timings["all_cores"] / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{len(chosen)} shortest of the 32 config-2 sequences ({sum(contexts)} KV tokens, {nbytes / 1e6:.1f} MB of K/V), "
                  f"f32 C oracle, OpenMP over (token, KV head); mean of {passes['all_cores']} passes "
                  f"({passes['single_thread']} single-threaded)",
        "seconds": timings["all_cores"],
        "single_thread_value": nbytes / timings["single_thread"] / 1e9,
        "single_thread_seconds": timings["single_thread"],
        "host_cpu": _cpu_model(),
    }


def producer_rows(device, steps: int = 20) -> dict:
    """The kernels that feed the SDPA, at config 5's prefill shape (8 x 2048 new tokens, Hq=64 / Hkv=8, D=128): the split of
    the gated input projection, per-head RMSNorm + RoPE of Q, the K/V page write into FP8 pages, and K RMSNorm + RoPE fused with that write.  All are HBM bound;
    bytes are what the kernel must move."""
    import torch

    from khalamari_amd import kv_page_write, rms_norm_rope
    from khalamari_amd._lib import ReplayU32

    spec = CONFIGS[5]
    hq, hkv, d = spec["hq"], spec["hkv"], spec["d"]
    requests, new_tokens = 8, 2048
    tokens = requests * new_tokens
    generator = torch.Generator(device=device)
    generator.manual_seed(77)

    def timed(launch):
        for _ in range(3):
            launch()
        torch.cuda.synchronize()
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for a, b in pairs:
            a.record()
            launch()
            b.record()
        torch.cuda.synchronize()
        return float(np.mean([a.elapsed_time(b) for a, b in pairs])) * 1e3

    result = {}
    from khalamari_amd import qgkv_split

    split_config = qgkv_split.Config.bf16(hq, hkv, d)
    split_shape = qgkv_split.Shape(tokens)
    projection = torch.randn((tokens, split_config.projection_width()), device=device, dtype=torch.bfloat16, generator=generator)
    split_q, split_g = (torch.empty((tokens, hq, d), device=device, dtype=torch.bfloat16) for _ in range(2))
    split_k, split_v = (torch.empty((tokens, hkv, d), device=device, dtype=torch.bfloat16) for _ in range(2))
    split = qgkv_split.Compute(split_config)
    us = timed(lambda: split.invoke(split_shape, qgkv=projection, q=split_q, g=split_g, k=split_k, v=split_v,
                                    num_active_tokens=ReplayU32.fixed(tokens)))
    nbytes = 2 * split_config.projection_bytes(split_shape)
    result["qgkv_split"] = {"workload": f"projection rows {tokens}x(2x{hq}+2x{hkv})x{d} bf16 -> q, g, k, v", "kernel_us": us,
                            "algorithmic_bytes": nbytes, "gbps": nbytes / us / 1e3, "roofline_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS}

    q = torch.randn((tokens, hq, d), device=device, dtype=torch.float32, generator=generator).to(torch.bfloat16)
    q_out = torch.empty_like(q)
    weight = torch.ones(d, device=device, dtype=torch.bfloat16)
    positions = (torch.arange(tokens, device=device, dtype=torch.int32) % new_tokens).contiguous()
    norm = rms_norm_rope.Compute(rms_norm_rope.Config.bf16(hq, d, d, 1e-6, 1_000_000.0))
    us = timed(lambda: norm.invoke(rms_norm_rope.Shape(tokens), input=q, norm_weight=weight, flat_token_indices=positions, output=q_out,
                                   num_active_tokens=ReplayU32.fixed(tokens)))
    nbytes = 2 * q.numel() * 2
    result["rms_norm_rope"] = {"workload": f"Q rows {tokens}x{hq}x{d} bf16, default RoPE", "kernel_us": us, "algorithmic_bytes": nbytes,
                               "gbps": nbytes / us / 1e3, "roofline_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS}

    pages_per_request = new_tokens // TOKENS_PER_PAGE
    page_bytes = 2 * hkv * TOKENS_PER_PAGE * d
    layout = kv_page_write.PageTableLayout(requests, 1, pages_per_request, 1)
    pages = torch.zeros(requests * pages_per_request * page_bytes, dtype=torch.uint8, device=device)
    page_ids = torch.from_numpy(np.random.default_rng(3).permutation(requests * pages_per_request).astype(np.int32)).to(device)
    flat_k = torch.randn((tokens, hkv, d), device=device, dtype=torch.float32, generator=generator).to(torch.bfloat16)
    flat_v = torch.randn((tokens, hkv, d), device=device, dtype=torch.float32, generator=generator).to(torch.bfloat16)
    req_slots = (torch.arange(tokens, device=device, dtype=torch.int32) // new_tokens).contiguous()
    writer = kv_page_write.Compute(kv_page_write.Config(hkv, d, page_bytes))
    shape = kv_page_write.Shape(tokens, layout)
    us = timed(lambda: writer.invoke(shape, pages=pages, flat_k=flat_k, flat_v=flat_v, req_slots=req_slots, flat_token_indices=positions,
                                     page_ids=page_ids, num_active_token_writes=ReplayU32.fixed(tokens), page_table_index=ReplayU32.fixed(0)))
    nbytes = 2 * flat_k.numel() * 2 + 2 * flat_k.numel()
    result["kv_page_write"] = {"workload": f"K/V rows {tokens}x{hkv}x{d} bf16 -> FP8 E4M3FN pages", "kernel_us": us, "algorithmic_bytes": nbytes,
                               "gbps": nbytes / us / 1e3, "roofline_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS}

    # K RMSNorm + RoPE and the page write in one launch, beside the two launches it replaces (K norm/rope, then the writer)
    from khalamari_amd import k_norm_rope_page_write

    k_norm = rms_norm_rope.Compute(rms_norm_rope.Config.bf16(hkv, d, d, 1e-6, 1_000_000.0))
    k_rows = torch.empty_like(flat_k)

    def two_launches():
        k_norm.invoke(rms_norm_rope.Shape(tokens), input=flat_k, norm_weight=weight, flat_token_indices=positions, output=k_rows,
                      num_active_tokens=ReplayU32.fixed(tokens))
        writer.invoke(shape, pages=pages, flat_k=k_rows, flat_v=flat_v, req_slots=req_slots, flat_token_indices=positions, page_ids=page_ids,
                      num_active_token_writes=ReplayU32.fixed(tokens), page_table_index=ReplayU32.fixed(0))

    fused = k_norm_rope_page_write.Compute(rms_norm_rope.Config.bf16(hkv, d, d, 1e-6, 1_000_000.0), kv_page_write.Config(hkv, d, page_bytes))
    separate_us = timed(two_launches)
    us = timed(lambda: fused.invoke(shape, pages=pages, k=flat_k, v=flat_v, norm_weight=weight, req_slots=req_slots, flat_token_indices=positions,
                                    page_ids=page_ids, num_active_tokens=ReplayU32.fixed(tokens), page_table_index=ReplayU32.fixed(0)))
    result["k_norm_rope_page_write"] = {"workload": f"K RMSNorm + RoPE and K/V rows {tokens}x{hkv}x{d} bf16 -> FP8 E4M3FN pages, one launch",
                                        "kernel_us": us, "algorithmic_bytes": nbytes, "gbps": nbytes / us / 1e3,
                                        "roofline_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS, "two_launches_us": separate_us}

    # everything between the input projection and the SDPA in one launch, beside the three launches it replaces
    # (projection split, Q norm/rope, fused K writer)
    from khalamari_amd import projection_norm_rope_page_write

    q_config, k_config = rms_norm_rope.Config.bf16(hq, d, d, 1e-6, 1_000_000.0), rms_norm_rope.Config.bf16(hkv, d, d, 1e-6, 1_000_000.0)
    prologue = projection_norm_rope_page_write.Compute(q_config, k_config, kv_page_write.Config(hkv, d, page_bytes))
    q_norm = rms_norm_rope.Compute(q_config)

    def three_launches():
        split.invoke(split_shape, qgkv=projection, q=split_q, g=split_g, k=split_k, v=split_v, num_active_tokens=ReplayU32.fixed(tokens))
        q_norm.invoke(rms_norm_rope.Shape(tokens), input=split_q, norm_weight=weight, flat_token_indices=positions, output=q_out,
                      num_active_tokens=ReplayU32.fixed(tokens))
        fused.invoke(shape, pages=pages, k=split_k, v=split_v, norm_weight=weight, req_slots=req_slots, flat_token_indices=positions,
                     page_ids=page_ids, num_active_tokens=ReplayU32.fixed(tokens), page_table_index=ReplayU32.fixed(0))

    separate_us = timed(three_launches)
    us = timed(lambda: prologue.invoke(shape, projection=projection, q_norm_weight=weight, k_norm_weight=weight, q_output=q_out,
                                       gate_output=split_g, pages=pages, req_slots=req_slots, flat_token_indices=positions, page_ids=page_ids,
                                       num_active_tokens=ReplayU32.fixed(tokens), page_table_index=ReplayU32.fixed(0)))
    nbytes = split_config.projection_bytes(split_shape) + 2 * q.numel() * 2 + 2 * flat_k.numel()
    result["projection_norm_rope_page_write"] = {
        "workload": f"projection rows {tokens}x(2x{hq}+2x{hkv})x{d} bf16 -> Q rows (norm + RoPE), gate rows, K (norm + RoPE) / V into FP8 E4M3FN "
                    "pages, one launch", "kernel_us": us, "algorithmic_bytes": nbytes, "gbps": nbytes / us / 1e3,
        "roofline_frac": nbytes / us / 1e3 / HBM_PEAK_GBPS, "three_launches_us": separate_us}
    return result


def layer_rows(device, index: int, fp8_pages: bool = False, replays: int = 30) -> dict:
    """Everything the reference's GQA::record enqueues between the input and the output projection
    (crates/inference-executor-metal/src/attn/gqa/backend.rs:358-421) for one batch of a benchmark config, recorded twice
    into a HIP graph and replayed: as the seven operators of the reference (projection split, Q norm + RoPE, K norm + RoPE,
    K/V page write, Map, Reduce, gate; Map writes the output itself when the selector says so), and as the shortest recording
    of this library (projection kernel, Map, gated Reduce or gated direct output).  Both leave the same bytes."""
    import torch

    from khalamari_amd import activation_gate, kv_page_write, projection_norm_rope_page_write, qgkv_split, rms_norm_rope
    from khalamari_amd._lib import DTYPE_BF16, DTYPE_FP8_E4M3FN, ReplayU32

    workload = Workload(index, device, num_pools=1, fp8_pages=fp8_pages)
    spec = workload.spec
    hq, hkv, d, tokens = spec["hq"], spec["hkv"], spec["d"], workload.num_tokens
    if workload.fused:
        raise RuntimeError("the layer recordings are timed on configs whose Map and Reduce are separate launches")
    pool = workload.kv_pools[0]
    generator = torch.Generator(device=device)
    generator.manual_seed(78)
    split_config = qgkv_split.Config.bf16(hq, hkv, d)
    projection = torch.randn((tokens, split_config.projection_width()), device=device, dtype=torch.bfloat16, generator=generator)
    rows = lambda heads: torch.empty((tokens, heads, d), device=device, dtype=torch.bfloat16)  # noqa: E731
    q_split, g_rows, k_split, v_split, k_normed, gated_out = rows(hq), rows(hq), rows(hkv), rows(hkv), rows(hkv), rows(hq)
    weight = torch.ones(d, device=device, dtype=torch.bfloat16)
    positions = torch.tensor([h + i for h, n in zip(workload.histories, workload.q_lens) for i in range(n)], dtype=torch.int32, device=device)
    req_slots = workload.metadata.req_slots()
    blocks = workload.table_host.shape[1]
    page_config = kv_page_write.Config(hkv, d, workload.page_bytes, kv_dtype=DTYPE_FP8_E4M3FN if fp8_pages else DTYPE_BF16)
    page_shape = kv_page_write.Shape(tokens, kv_page_write.PageTableLayout(len(workload.histories), 1, blocks, 1))
    q_config, k_config = rms_norm_rope.Config.bf16(hq, d, d, 1e-6, 1_000_000.0), rms_norm_rope.Config.bf16(hkv, d, d, 1e-6, 1_000_000.0)
    split, q_norm, k_norm = qgkv_split.Compute(split_config), rms_norm_rope.Compute(q_config), rms_norm_rope.Compute(k_config)
    writer = kv_page_write.Compute(page_config)
    prologue = projection_norm_rope_page_write.Compute(q_config, k_config, page_config)
    active, layer = ReplayU32.fixed(tokens), ReplayU32.fixed(0)

    def seven_operators():
        split.invoke(qgkv_split.Shape(tokens), qgkv=projection, q=q_split, g=g_rows, k=k_split, v=v_split, num_active_tokens=active)
        q_norm.invoke(rms_norm_rope.Shape(tokens), input=q_split, norm_weight=weight, flat_token_indices=positions, output=workload.q,
                      num_active_tokens=active)
        k_norm.invoke(rms_norm_rope.Shape(tokens), input=k_split, norm_weight=weight, flat_token_indices=positions, output=k_normed,
                      num_active_tokens=active)
        writer.invoke(page_shape, pages=pool, flat_k=k_normed, flat_v=v_split, req_slots=req_slots, flat_token_indices=positions,
                      page_ids=workload.page_table, num_active_token_writes=active, page_table_index=layer)
        if workload.launch_reduce is None:
            workload.launch_map(pool, gates=None)
        else:
            workload.launch_map(pool)
            workload.launch_reduce(gates=None)
        activation_gate.invoke(DTYPE_BF16, hq, d, tokens, workload.out, g_rows, gated_out, active)

    def shortest():
        prologue.invoke(page_shape, projection=projection, q_norm_weight=weight, k_norm_weight=weight, q_output=workload.q, gate_output=g_rows,
                        pages=pool, req_slots=req_slots, flat_token_indices=positions, page_ids=workload.page_table, num_active_tokens=active,
                        page_table_index=layer)
        if workload.launch_reduce is None:
            workload.launch_map(pool, gates=g_rows)
        else:
            workload.launch_map(pool)
            workload.launch_reduce(gates=g_rows)

    def replayed(record):
        import gc

        record()
        torch.cuda.synchronize()
        result = workload.out.clone() if record is shortest else gated_out.clone()
        pages_after = pool.clone()
        gc.collect()
        graph = torch.cuda.CUDAGraph()
        gc.disable()   # a collector run inside the capture could free device memory, which invalidates it
        try:
            with torch.cuda.graph(graph):
                record()
        finally:
            gc.enable()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        for _ in range(replays):
            graph.replay()
        end.record()
        torch.cuda.synchronize()
        return begin.elapsed_time(end) * 1e3 / replays, result, pages_after

    seven_us, seven_out, seven_pages = replayed(seven_operators)
    short_us, short_out, short_pages = replayed(shortest)
    return {"workload": spec["name"] + (" [FP8 E4M3FN pages]" if fp8_pages else ""), "tokens": tokens,
            "launches_reference_recording": 7 if workload.launch_reduce is not None else 6,
            "launches_shortest_recording": 3 if workload.launch_reduce is not None else 2,
            "reference_recording_us": seven_us, "shortest_recording_us": short_us,
            "same_output_bytes": bool(torch.equal(seven_out, short_out)), "same_page_bytes": bool(torch.equal(seven_pages, short_pages))}


def slab_run_table(device, index: int = 2, steps: int = 40) -> list:
    """The read-only launch of a config's K/V bytes as contiguous runs of 4 .. 64 KB at random places of its pools: what a
    block that covered several KV heads of a page (longer contiguous reads) could gain over 4 KB slabs."""
    import torch

    workload = Workload(index, device)
    spec = workload.spec
    kv_bytes = workload.visible_tokens * spec["hkv"] * spec["d"] * 2 * workload.kv_element_bytes
    pool_slabs = workload.kv_pools[0].numel() * workload.kv_pools[0].element_size() // SLAB_BYTES
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    rows = []
    for run in (1, 2, 4, 8, 16):
        num_slabs = (kv_bytes // SLAB_BYTES) // run * run
        order = np.random.Generator(np.random.PCG64(1234)).permutation(pool_slabs // run)[:num_slabs // run].astype(np.uint32)
        run_ids = torch.from_numpy(order.view(np.int32)).to(device)
        for blocks_per_cu in (2, 4):
            for i in range(3):
                slab_read(workload.kv_pools[i % NUM_POOLS], run_ids, num_slabs, sink, blocks_per_cu, run)
            pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
            for i, (a, b) in enumerate(pairs):
                a.record()
                slab_read(workload.kv_pools[i % NUM_POOLS], run_ids, num_slabs, sink, blocks_per_cu, run)
                b.record()
            torch.cuda.synchronize()
            us = float(np.mean([a.elapsed_time(b) for a, b in pairs])) * 1e3
            rows.append({"contiguous_kb": run * SLAB_BYTES // 1024, "blocks_per_cu": blocks_per_cu, "us": us,
                         "gbps": num_slabs * SLAB_BYTES / us / 1e3})
    return rows


def _cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as handle:
            for line in handle:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def calibration_copy(device, gib: int = 1) -> None:
    """A plain elementwise copy of `gib` GiB (reads and writes every byte once): what a hardware counter reads for
    this launch, divided by its known size, is the scale factor for the same counter on the Map kernel."""
    import torch

    source = torch.full(((gib << 30) // 4,), 1.0, dtype=torch.float32, device=device)
    target = torch.empty_like(source)
    for _ in range(3):
        torch.mul(source, 1.0, out=target)   # an elementwise kernel, not a DMA blit: it shows up as a dispatch
    torch.cuda.synchronize()
    del source, target
    torch.cuda.empty_cache()


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__)
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--config", type=int, default=2, help="headline config (default 2)")
    parser.add_argument("--only", action="store_true", help="time only the headline config (used for profiling runs)")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    parser.add_argument("--producers", action="store_true",
                        help="time only the kernels that feed the SDPA (RMSNorm + RoPE, K/V page write) and print their JSON (profiling runs)")
    parser.add_argument("--fp8-pages", action="store_true",
                        help="headline config on FP8 E4M3FN pages, the reference's cache format (profiling runs; the default headline keeps bf16 pages)")
    parser.add_argument("--layer", action="store_true",
                        help="time the whole layer between the projections (producers, SDPA, gate) of --config N, as the reference's "
                             "seven operators and as this library's shortest recording, replayed from a HIP graph")
    parser.add_argument("--slab-runs", action="store_true",
                        help="time only the read-only launch of the headline config's K/V bytes as contiguous runs of 4 .. 64 KB and print the table as JSON")
    parser.add_argument("--no-clock-probe", action="store_true", help="accepted and ignored (older command lines)")
    parser.add_argument("--calibration-copy", action="store_true",
                        help="also launch a plain 1 GiB copy kernel, the known-size reference for FETCH_SIZE / WRITE_SIZE counter runs")
    args = parser.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path shards by (sequence, KV head) with no exchange, and this build runs "
              "on a single MI355X; rerun with --gpus 1", file=sys.stderr)
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (no GPU visible)", file=sys.stderr)
        return 2
    device = torch.device("cuda:0")
    if args.calibration_copy:
        calibration_copy(device)
    if args.producers:
        print(json.dumps({"producers": producer_rows(device, steps=max(args.steps, 1))}))
        return 0
    if args.slab_runs:
        print(json.dumps({"slab_runs": slab_run_table(device, args.config)}))
        return 0
    if args.layer:
        print(json.dumps({"layer": layer_rows(device, args.config, fp8_pages=args.fp8_pages)}))
        return 0
    headline = Workload(args.config, device, fp8_pages=args.fp8_pages)
    head = headline.report(args.steps, args.warmup)
    others = {}
    if not args.only:
        del headline
        torch.cuda.empty_cache()
        for index in sorted(CONFIGS):
            if index == args.config:
                continue
            try:
                workload = Workload(index, device)
                others[config_key(index)] = workload.report(max(args.steps // 4, 10), max(args.warmup // 2, 3))
                del workload
                torch.cuda.empty_cache()
            except Exception as error:  # a config whose kernel is not built yet is reported, not hidden
                others[config_key(index)] = {"workload": CONFIGS[index]["name"], "error": str(error)}
        # the reference's production cache format: half the bytes per KV token
        for index in (2, 3, 4, 5):
            try:
                workload = Workload(index, device, fp8_pages=True)
                others[f"config{index}_fp8_pages"] = workload.report(max(args.steps // 4, 10), max(args.warmup // 2, 3))
                del workload
                torch.cuda.empty_cache()
            except Exception as error:
                others[f"config{index}_fp8_pages"] = {"workload": CONFIGS[index]["name"] + " [FP8 E4M3FN pages]", "error": str(error)}
        try:
            others["producers"] = producer_rows(device)
        except Exception as error:
            others["producers"] = {"error": str(error)}
    prefill = head["bound"] == "mfma"
    line = {
        "metric": "paged GQA prefill bf16 MFMA TFLOP/s" if prefill else "paged GQA decode achieved HBM GB/s (split-KV Map + LSE Reduce per step)",
        "value": head["tflops"] if prefill else head["gbps"],
        "unit": "TFLOP/s" if prefill else "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["us_per_step"] / 1e3,
        "us_per_step": head["us_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": head["workload"], "kv_pools_rotated": NUM_POOLS, "map_task_templates": head["map_task_templates"],
                   "visible_kv_tokens": head["visible_kv_tokens"]},
        "roofline": {
            "bound": head["bound"],
            "achieved": head["map_tflops"] if prefill else head["map_gbps"],
            "peak": MFMA_BF16_PEAK_TFLOPS if prefill else HBM_PEAK_GBPS,
            "unit": "TFLOP/s" if prefill else "GB/s",
            "frac": head["roofline_frac"],
            "traffic": (MEASURED_MAP_TRAFFIC_BYTES_FP8_PAGES if args.fp8_pages else MEASURED_MAP_TRAFFIC_BYTES).get(args.config),
            "kernel": head["map_kernel"],
            "kernel_us": head["map_kernel_us"],
            "algorithmic_bytes": head.get("algorithmic_bytes"),
            "algorithmic_flops": head.get("algorithmic_flops"),
            "slab_reader": head.get("slab_reader"),
        },
        "configs": others,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(2)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
