"""Borrowed device buffers for the C ABI: anything with `data_ptr()` (a torch tensor) or a (ptr, bytes) pair."""
from __future__ import annotations

from ._lib import Buffer


def view(obj) -> Buffer:
    if isinstance(obj, Buffer):
        return obj
    if isinstance(obj, tuple):
        return Buffer(int(obj[0]), int(obj[1]))
    if hasattr(obj, "data_ptr"):
        return Buffer(obj.data_ptr(), obj.numel() * obj.element_size())
    raise TypeError(f"cannot borrow {type(obj).__name__} as a device buffer")


def stream_handle(stream) -> int:
    """hipStream_t of a torch stream (or the current one); 0 is the legacy default stream."""
    if stream is None:
        import torch

        return int(torch.cuda.current_stream().cuda_stream)
    if hasattr(stream, "cuda_stream"):
        return int(stream.cuda_stream)
    return int(stream)


def param_block(block) -> int:
    if block is None:
        return 0
    if hasattr(block, "data_ptr"):
        return int(block.data_ptr())
    return int(block)
