"""Plugin hook surface for sparse-attention algorithms under vLLM 0.9.2.

Mirrors the interface of the reference's ``UcmSparseBase``
(ucm/sparse/base.py:56-202): the patched vLLM call sites
(ucm/integration/vllm/patch/0.9.2/vllm-adapt.patch:80-115, :359-364,
:1159-1176) look these methods up by name, so names, argument order and return
conventions are kept; everything else is this package's own.  vLLM is not
imported here, which keeps the surface testable with stand-in objects.
"""
from __future__ import annotations

import enum
import warnings
from abc import ABC, abstractmethod
from typing import Any, List, Optional, Union

INVALID_SLOT = -1  # ucm/sparse/base.py:35: "this request is not sparsified"


class UcmSparseRole(enum.Enum):
    SCHEDULER = 0  # instance living in the scheduler process
    WORKER = 1     # instance living in a worker (model runner) process


class UcmSparseMetadata(ABC):  # noqa: B024
    """Per-step data a plugin builds in build_sparse_meta and reads in its worker hooks."""


class UcmSparseBase(ABC):
    def __init__(self, vllm_config: Any, role: UcmSparseRole):
        self._vllm_config = vllm_config
        self._role = role
        self._sparse_metadata: Optional[UcmSparseMetadata] = None
        self.load_misses = 0            # blocks a device-side load wanted from the KV store and did not find there

    @property
    def role(self) -> UcmSparseRole:
        return self._role

    def _report_missing(self, n: int) -> None:
        """A load that a kernel carries out leaves out a block the store does not hold: the cache block that should
        receive it keeps what it has.  That is counted and said aloud instead of passing unnoticed, and the plugins
        look the block up again at their next load."""
        self.load_misses += n
        warnings.warn(f"{type(self).__name__}: the KV store does not hold {n} of the blocks a load of this step may ask "
                      "for; cache blocks that should receive them keep what they hold", RuntimeWarning, stacklevel=3)

    # ---- worker side -----------------------------------------------------
    def bind_sparse_metadata(self, sparse_metadata: UcmSparseMetadata) -> None:
        self._sparse_metadata = sparse_metadata

    def clear_sparse_metadata(self) -> None:
        self._sparse_metadata = None

    def _get_sparse_metadata(self) -> UcmSparseMetadata:
        assert self._sparse_metadata is not None, "no sparse metadata bound for this step"
        return self._sparse_metadata

    def register_kv_caches(self, kv_caches: dict) -> None:
        """kv_caches: layer name -> that layer's paged KV cache tensor."""

    def execute_begin(self, scheduler_output) -> None:
        """Start of ModelRunner.execute_model, after build_sparse_meta."""

    def execute_finished(self) -> None:
        """End of ModelRunner.execute_model."""

    def attention_begin(self, query, key, value, layer_name: str, forward_context) -> None:
        """Start of unified_attention for one layer; may replace
        forward_context.attn_metadata.block_table / seq_lens."""

    def attention_finished(self, query, key, value, attn_output, layer_name: str, forward_context) -> None:
        """End of unified_attention for one layer."""

    def request_finished_in_worker(self, request_id: Union[int, str]) -> None:
        """Release what the worker holds for a finished request."""

    # ---- scheduler side --------------------------------------------------
    @abstractmethod
    def request_begin(self, request_id: Union[int, str], prompt_token_ids: List[int]) -> None:
        """Scheduler.add_request."""

    def request_finished_in_scheduler(self, request_id: Union[int, str]) -> None:
        """Scheduler.finish_requests."""

    def estimate_num_slots_sparsed(self, request) -> int:
        """Token slots the request needs once sparsified, or INVALID_SLOT."""
        return INVALID_SLOT

    def update_state_after_alloc(self, request, num_blocks: int) -> None:
        """After the KV cache manager allocated blocks for the request."""

    def build_sparse_meta(self, scheduler_output, requests, input_batch, attn_metadata):
        """Once per step, before execute_begin."""

    def allocate_slots(self, request, num_slots_sparsed, coordinator, block_pool, kv_cache_groups):
        """Divert KVCacheManager.allocate_slots for a sparsified request; None = not enough blocks."""
        return None
