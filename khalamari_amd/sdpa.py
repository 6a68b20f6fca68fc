"""Mirror of `components::gqa::sdpa` (crates/inference-backend-metal/src/components/gqa/sdpa.rs):
`Config`, `MapKernelKind`, `ExecutionVariant` constructors and `Registry`."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from . import _lib
from ._lib import (DTYPE_BF16, DTYPE_F32, MAP_Q_HEADS_PER_TOKEN, MAP_Q_TOKENS_AND_HEADS,  # noqa: F401
                   MAP_Q_TOKENS_PER_HEAD, MAP_SLICED_KV, SdpaVariant)


@dataclass(frozen=True)
class Config:
    """`sdpa::Config` (sdpa.rs:219-227)."""

    io_dtype: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    tokens_per_page: int

    def c(self) -> _lib.SdpaConfig:
        return _lib.SdpaConfig(self.io_dtype, self.num_q_heads, self.num_kv_heads, self.head_dim, self.tokens_per_page)

    def q_heads_per_kv_head(self) -> int:
        return self.num_q_heads // self.num_kv_heads


class ExecutionVariant:
    """Constructors of `sdpa::ExecutionVariant` (sdpa.rs:60-160); instances are `SdpaVariant` structs."""

    @staticmethod
    def sliced_kv(config: Config, kv_tokens_per_iteration: int, required_threads: int, max_q_heads: int) -> SdpaVariant:
        out = SdpaVariant()
        c = config.c()
        _lib.check(_lib.lib().khm_sdpa_variant_sliced_kv(ctypes.byref(c), kv_tokens_per_iteration, required_threads,
                                                         max_q_heads, ctypes.byref(out)))
        return out

    @staticmethod
    def sliced_q(config: Config, kind: int, max_q_tokens: int, kv_tokens_per_iteration: int, max_q_heads: int) -> SdpaVariant:
        out = SdpaVariant()
        c = config.c()
        _lib.check(_lib.lib().khm_sdpa_variant_sliced_q(ctypes.byref(c), kind, max_q_tokens, kv_tokens_per_iteration,
                                                        max_q_heads, ctypes.byref(out)))
        return out

    @staticmethod
    def sliced_q_per_head(config: Config, max_q_tokens: int, kv_tokens_per_iteration: int, max_q_heads: int) -> SdpaVariant:
        return ExecutionVariant.sliced_q(config, MAP_Q_TOKENS_PER_HEAD, max_q_tokens, kv_tokens_per_iteration, max_q_heads)


def supports(variant: SdpaVariant, config: Config) -> bool:
    c = config.c()
    return bool(_lib.check(_lib.lib().khm_sdpa_variant_supports(ctypes.byref(variant), ctypes.byref(c))))


def has_kernel(config: Config, variant: SdpaVariant, kv_dtype: int = DTYPE_BF16) -> bool:
    c = config.c()
    return bool(_lib.check(_lib.lib().khm_sdpa_variant_has_kernel(ctypes.byref(c), ctypes.byref(variant), kv_dtype)))


class Registry:
    """`sdpa::Registry` (sdpa.rs:239-302)."""

    def __init__(self, config: Config, variants=None):
        self._config = config
        if variants is None:
            array = (SdpaVariant * 8)()
            count = ctypes.c_uint32()
            c = config.c()
            _lib.check(_lib.lib().khm_sdpa_registry_new(ctypes.byref(c), array, 8, ctypes.byref(count)))
            variants = [SdpaVariant.from_buffer_copy(array[i]) for i in range(count.value)]
        else:
            variants = list(variants)
            if not variants:
                raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT, "GQA SDPA registry requires an execution variant")
            if not all(supports(v, config) for v in variants):
                raise _lib.KhmError(_lib.KHM_ERR_INVALID_ARGUMENT,
                                    "GQA SDPA registry contains an unsupported execution variant")
        self._variants = variants

    @staticmethod
    def from_variants(config: Config, variants) -> "Registry":
        return Registry(config, variants)

    def config(self) -> Config:
        return self._config

    def variants(self):
        return list(self._variants)

    def max_q_tokens_per_map_task(self) -> int:
        return max(v.map_max_q_tokens for v in self._variants)
