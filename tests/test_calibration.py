"""The read-only calibration launch: argument checks on the CPU, one run on the GPU."""
import ctypes

import numpy as np
import pytest

from khalamari_amd import _lib


def _buffer(pointer: int, length: int) -> _lib.Buffer:
    return _lib.Buffer(ctypes.c_void_p(pointer), length)


def test_rejects_bad_arguments_before_touching_a_device():
    lib = _lib.lib()
    ok = _buffer(0x1000, 1 << 20)
    cases = [
        (_buffer(0, 1 << 20), ok, 4, 2, ok),          # null pool
        (ok, _buffer(0x1000, 8), 4, 2, ok),           # fewer ids than slabs
        (ok, ok, 0, 2, ok),                           # nothing to read
        (ok, ok, 4, 0, ok),                           # no blocks
        (ok, ok, 4, 9, ok),                           # more blocks per compute unit than the entry point allows
        (ok, ok, 4, 2, _buffer(0x1000, 2)),           # sink too small
        (_buffer(0x1000, 100), ok, 4, 2, ok),         # pool smaller than one slab
    ]
    for pool, ids, count, blocks, sink in cases:
        assert lib.khm_calibration_slab_read(pool, ids, count, blocks, sink, None) == _lib.KHM_ERR_INVALID_ARGUMENT
        assert lib.khm_last_error()


@pytest.mark.gpu
def test_gpu_reads_listed_slabs_and_leaves_the_sink_alone(device):
    import torch

    from khalamari_amd import calibration

    slabs = 1024
    pool = torch.randint(-2**31, 2**31 - 1, (slabs * calibration.SLAB_BYTES // 4,), dtype=torch.int32, device=device)
    order = np.random.default_rng(5).permutation(slabs).astype(np.uint32)
    ids = torch.from_numpy(order.view(np.int32)).to(device)
    sink = torch.zeros(1, dtype=torch.int32, device=device)
    for count in (1, 3, slabs):   # fewer slabs than waves, and a full list
        print(f"calibration slab read: {count} slabs", flush=True)
        calibration.slab_read(pool, ids, count, sink, blocks_per_cu=2)
    torch.cuda.synchronize()
    assert int(sink.item()) == 0
