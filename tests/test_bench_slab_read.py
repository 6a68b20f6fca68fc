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
        bench.slab_read(pool, ids, count, sink, blocks_per_cu=2, slab_bytes=2048)   # the first half of the pool, as 2 KB slabs
    torch.cuda.synchronize()
    assert int(sink.item()) == 0
    with pytest.raises(RuntimeError):
        bench.slab_read(pool, ids, 0, sink)          # nothing to read
    with pytest.raises(RuntimeError):
        bench.slab_read(pool, ids, 4, sink, blocks_per_cu=9)
    with pytest.raises(RuntimeError):
        bench.slab_read(pool, ids, 4, sink, slab_bytes=1024)


def test_bench_aid_library_exports_its_entry_points():
    import ctypes
    import os

    path = os.path.join(bench.ROOT, "libbench_slab_read.so")
    if not os.path.exists(path):
        pytest.skip("libbench_slab_read.so is not built")
    lib = ctypes.CDLL(path)
    assert hasattr(lib, "bench_slab_read")
