"""Measurement aid with no counterpart in the reference: a launch that only reads 4 KB slabs of a K/V pool."""
from __future__ import annotations

from . import _lib
from ._buffers import stream_handle, view

SLAB_BYTES = 4096


def slab_read(pool, slab_ids, num_slabs: int, sink, blocks_per_cu: int = 2, stream=None) -> None:
    """Enqueue a read of `num_slabs` slabs (slab i at byte offset `slab_ids[i] * 4096` of `pool`) from a resident grid,
    with the Map kernel's lane layout and loads in flight; `sink` is a device buffer of at least four bytes."""
    _lib.check(_lib.lib().khm_calibration_slab_read(view(pool), view(slab_ids), int(num_slabs), int(blocks_per_cu), view(sink),
                                                    stream_handle(stream)))
