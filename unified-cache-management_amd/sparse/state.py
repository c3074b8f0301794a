"""Process-wide plugin instance (ucm/sparse/state.py:21-76): created once by
ensure_ucm_sparse_initialized from the worker / scheduler start-up hooks."""
from __future__ import annotations

from typing import Optional

from .base import UcmSparseBase, UcmSparseRole
from .factory import UcmSparseFactory

_UCM_SPARSE_AGENT: Optional[UcmSparseBase] = None


def ensure_ucm_sparse_initialized(vllm_config, role: UcmSparseRole = UcmSparseRole.WORKER) -> None:
    global _UCM_SPARSE_AGENT
    ktc = getattr(vllm_config, "kv_transfer_config", None)
    if ktc is None or "ucm_sparse_config" not in (ktc.kv_connector_extra_config or {}):
        return
    if _UCM_SPARSE_AGENT is None:
        _UCM_SPARSE_AGENT = UcmSparseFactory.create_sparse_method(vllm_config, role)


def get_ucm_sparse() -> UcmSparseBase:
    if _UCM_SPARSE_AGENT is None:
        raise RuntimeError("UCM sparse agent is not initialized")
    return _UCM_SPARSE_AGENT


def has_ucm_sparse() -> bool:
    return _UCM_SPARSE_AGENT is not None


def reset_ucm_sparse() -> None:
    """Drop the instance (tests)."""
    global _UCM_SPARSE_AGENT
    _UCM_SPARSE_AGENT = None
