"""Name -> plugin registry with lazy imports.  As in the reference
(ucm/sparse/factory.py:12-52) the algorithm is chosen by the FIRST key of
``kv_connector_extra_config["ucm_sparse_config"]``."""
from __future__ import annotations

import importlib
from typing import Callable, Dict

from .base import UcmSparseBase, UcmSparseRole


class UcmSparseFactory:
    _registry: Dict[str, Callable[[], type]] = {}

    @classmethod
    def register_sparse_method(cls, name: str, module_path: str, class_name: str) -> None:
        if name in cls._registry:
            raise ValueError(f"Sparse attention method '{name}' is already registered.")
        cls._registry[name] = lambda: getattr(importlib.import_module(module_path), class_name)

    @classmethod
    def create_sparse_method(cls, config, role: UcmSparseRole) -> UcmSparseBase:
        sparse_cfg = config.kv_transfer_config.kv_connector_extra_config["ucm_sparse_config"]
        name = next(iter(sparse_cfg))
        if name not in cls._registry:
            raise ValueError(f"Unsupported sparse method type: {name}")
        return cls._registry[name]()(config, role)


_PKG = __name__.rsplit(".", 1)[0]
UcmSparseFactory.register_sparse_method("GSA", _PKG + ".gsa.gsa", "GSA")
UcmSparseFactory.register_sparse_method("ESA", _PKG + ".esa.esa", "ESA")
UcmSparseFactory.register_sparse_method("KvComp", _PKG + ".kvcomp.kvcomp", "KvComp")
UcmSparseFactory.register_sparse_method("KVStarMultiStep", _PKG + ".kvstar.multistep", "KVStarMultiStep")
