"""Mirror of `ReplayBucketPolicy` (crates/inference-executor-core/src/replay.rs:1-87)."""
from __future__ import annotations

import ctypes

from . import _lib


class ReplayBucketPolicy:
    def __init__(self, max_capacity: int, topology_boundaries=()):
        handle = ctypes.c_void_p()
        boundaries = (ctypes.c_uint32 * len(topology_boundaries))(*topology_boundaries)
        _lib.check(_lib.lib().khm_replay_bucket_policy_create(ctypes.c_uint32(max_capacity), boundaries,
                                                              len(topology_boundaries), ctypes.byref(handle)))
        self._handle = handle

    @staticmethod
    def with_topology_boundaries(max_capacity: int, topology_boundaries) -> "ReplayBucketPolicy":
        return ReplayBucketPolicy(max_capacity, tuple(topology_boundaries))

    def __del__(self):
        handle = getattr(self, "_handle", None)
        if handle and _lib is not None and getattr(_lib, "_lib", None) is not None:
            _lib._lib.khm_replay_bucket_policy_destroy(handle)
            self._handle = None

    def max_capacity(self) -> int:
        fn = _lib.lib().khm_replay_bucket_policy_max_capacity
        fn.restype = ctypes.c_uint32
        return int(fn(self._handle))

    def buckets(self):
        count = ctypes.c_uint32()
        _lib.check(_lib.lib().khm_replay_bucket_policy_buckets(self._handle, None, 0, ctypes.byref(count)))
        array = (ctypes.c_uint32 * count.value)()
        _lib.check(_lib.lib().khm_replay_bucket_policy_buckets(self._handle, array, count.value, ctypes.byref(count)))
        return list(array)

    def capacity(self, active: int) -> int:
        out = ctypes.c_uint32()
        _lib.check(_lib.lib().khm_replay_bucket_policy_capacity(self._handle, ctypes.c_uint32(active), ctypes.byref(out)))
        return out.value

    def capacity_allow_zero(self, active: int) -> int:
        out = ctypes.c_uint32()
        _lib.check(_lib.lib().khm_replay_bucket_policy_capacity_allow_zero(self._handle, ctypes.c_uint32(active),
                                                                           ctypes.byref(out)))
        return out.value
