"""bench.py's read-only slab launch (a library of its own beside bench.py): one run on the GPU."""
import numpy as np
import pytest

import bench


@pytest.mark.gpu
def test_gpu_reads_listed_slabs_and_leaves_the_sink_alone(device):
    import torch

    slabs = 1024
    pool = torch.randint(-2**31, 2**31 - 1, (slabs * bench.SLAB_BYTES // 4,), dtype=torch.int32, device=device)
    order = np.random.default_rng(5).permutation(slabs).astype(np.uint32)
    ids = torch.from_numpy(order.view(np.int32)).to(device)
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    for count in (1, 3, slabs):   # fewer slabs than waves, and a full list
        print(f"bench slab read: {count} slabs", flush=True)
        bench.slab_read(pool, ids, count, sink, blocks_per_cu=2)
    torch.cuda.synchronize()
    assert int(sink.item()) == 0
    with pytest.raises(RuntimeError):
        bench.slab_read(pool, ids, 0, sink)          # nothing to read
    with pytest.raises(RuntimeError):
        bench.slab_read(pool, ids, 4, sink, blocks_per_cu=9)


def test_bench_aid_library_exports_its_entry_points():
    import ctypes
    import os

    path = os.path.join(bench.ROOT, "libbench_slab_read.so")
    if not os.path.exists(path):
        pytest.skip("libbench_slab_read.so is not built")
    lib = ctypes.CDLL(path)
    for name in ("bench_slab_read", "bench_mfma_sustained", "bench_mfma_sustained_operand_bytes", "bench_mfma_sustained_sink_bytes",
                 "bench_mfma_sustained_flops", "bench_clock_probe"):
        assert hasattr(lib, name), name


@pytest.mark.gpu
def test_gpu_mfma_loop_reaches_a_plausible_rate_and_clock(device):
    print("bench mfma sustained: 20000 steps per launch", flush=True)
    rows = bench.mfma_sustained_table(device, steps=20000)
    assert len(rows) == 4
    for row in rows:
        print(row, flush=True)
        assert 500.0 < row["tflops"] < 2600.0            # 2.5 PFLOP/s is the published dense bf16 peak
        assert 0.8 < row["shader_clock_ghz"] < 2.6       # 2.4 GHz is the top shader clock
