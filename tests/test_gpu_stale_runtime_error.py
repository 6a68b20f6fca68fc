"""A HIP error that the host program left unread in the calling thread (the runtime keeps a thread's last error until it
is read) must not be reported as the failure of this library's next launch."""
import ctypes

import numpy as np
import pytest
import torch

from khalamari_amd import activation_gate
from khalamari_amd._lib import DTYPE_BF16, ReplayU32

pytestmark = pytest.mark.gpu


def _loaded_hip_runtime():
    """The HIP runtime this process already uses, found among its mapped files."""
    for line in open("/proc/self/maps"):
        path = line.split()[-1]
        if "libamdhip64" in path:
            return ctypes.CDLL(path)
    return None


def test_launch_after_an_unread_error_of_the_host_program(device):
    attention = torch.full((4, 2, 8), 0x3F80, dtype=torch.int16, device=device)   # 1.0
    gates = torch.zeros((4, 2, 8), dtype=torch.int16, device=device)              # sigmoid(0) = 0.5
    out = torch.zeros_like(attention)
    torch.cuda.synchronize()
    runtime = _loaded_hip_runtime()
    if runtime is None:
        pytest.skip("the HIP runtime library is not among the mapped files")
    runtime.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    status = runtime.hipMemcpy(None, None, 16, 1)     # a null destination: refused at once, nothing is copied
    assert status != 0
    print(f"host program's failed call returned {status}; launching", flush=True)
    activation_gate.invoke(DTYPE_BF16, 2, 8, 4, attention, gates, out, ReplayU32.fixed(4))   # raises KhmError on a reported failure
    torch.cuda.synchronize()
    assert np.all(out.cpu().numpy() == 0x3F00)   # 0.5
