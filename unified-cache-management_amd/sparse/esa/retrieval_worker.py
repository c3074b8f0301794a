"""ESA retrieval worker on the GPU.

``HipRetrievalBackend`` stands in for the reference's pybind11 class
``RetrievalWorkerBackend`` (ucm/sparse/esa/retrieval/cpy/retrieval_backend.cpp:17-225)
and ``RetrievalWorker`` for its thin Python wrapper
(ucm/sparse/esa/retrieval/retrieval_worker.py:10-34): same four methods
(submit / poll / wait / get_result), same result dictionary, same
``RuntimeError`` messages.  Instead of a pool of host threads scanning a CPU
table, ``submit`` enqueues two kernels on a side HIP stream and records an
event; ``poll`` queries it, ``wait`` blocks on it, ``get_result`` copies the k'
winners back.

The representative table ``data`` ([n_items, dim] fp32) lives in HBM and is
aliased, not copied: rows written later are seen by later submits, as with the
reference's numpy view (retrieval_backend.cpp:19-26).
"""
from __future__ import annotations

import threading
from typing import Dict

import numpy as np
import torch

from ... import ops


class HipRetrievalBackend:
    def __init__(self, data: torch.Tensor):
        if not isinstance(data, torch.Tensor) or not data.is_cuda:
            raise ValueError("data must be a device tensor [n_items, dim] (float32)")
        if data.dim() != 2 or data.dtype != torch.float32 or not data.is_contiguous():
            raise ValueError("data must be a contiguous float32 [n_items, dim] tensor")
        self.data = data
        self.n_items, self.dim = data.shape
        self._stream = torch.cuda.Stream(device=data.device)  # default priority
        self._lock = threading.Lock()
        self._next_req_id = 0
        self._pending: Dict[int, dict] = {}
        self._known = set()

    # -- submit(query f32[B, dim], topk, indexes int32[B, M] padded with -1) -> req_id
    def submit(self, query, topk: int, indexes) -> int:
        dev = self.data.device
        q = query if isinstance(query, torch.Tensor) else torch.as_tensor(np.asarray(query))
        if q.dim() != 2 or q.shape[1] != self.dim:
            raise RuntimeError("Query dim mismatch")
        idx_np = None
        if isinstance(indexes, torch.Tensor):
            idx = indexes
        else:
            idx_np = _pad_rows(indexes)
            idx = torch.from_numpy(idx_np)
        if idx.dim() != 2 or idx.shape[0] != q.shape[0]:
            raise RuntimeError("Query and indexes batch mismatch")
        batch, m = idx.shape
        # the producer of `query` runs on the caller's stream
        ready = torch.cuda.Event()
        ready.record(torch.cuda.current_stream(dev))
        with torch.cuda.stream(self._stream):
            self._stream.wait_event(ready)
            q_dev = q.to(device=dev, dtype=torch.float32, non_blocking=True).contiguous()
            idx_dev = idx.to(device=dev, dtype=torch.int32, non_blocking=True).contiguous()
            stride = max(min(int(topk), m), 1)
            ws = torch.empty((batch, max(m, 1)), dtype=torch.float32, device=dev)
            # indices, score bits and counts share one buffer so that get_result is a single copy to the host
            pack = torch.zeros((3, batch, stride), dtype=torch.int32, device=dev)
            out_idx, out_scores, out_count = pack[0], pack[1].view(torch.float32), pack[2].view(-1)[:batch]
            ops.esa_retrieve(self.data, q_dev, idx_dev, int(topk), ws, out_idx, out_scores, out_count,
                             stream=self._stream.cuda_stream)
            done = torch.cuda.Event()
            done.record(self._stream)
        with self._lock:
            req_id = self._next_req_id
            self._next_req_id += 1
            self._known.add(req_id)
            self._pending[req_id] = dict(done=done, pack=pack, keep=(q_dev, idx_dev, ws), topk=int(topk))
        return req_id

    def poll(self, req_id: int) -> bool:
        with self._lock:
            p = self._pending.get(req_id)
        return p is not None and p["done"].query()

    def wait(self, req_id: int) -> None:
        with self._lock:
            if req_id not in self._known:
                raise RuntimeError("Bad req_id")
            p = self._pending.get(req_id)
        if p is not None:
            p["done"].synchronize()  # releases the GIL while it blocks

    def get_result(self, req_id: int) -> dict:
        with self._lock:
            p = self._pending.get(req_id)
            if p is None or not p["done"].query():
                raise RuntimeError("Result not ready")
            del self._pending[req_id]  # a result can be fetched once, like the reference's erase
        host = p["pack"].cpu().numpy()                 # [3, batch, stride]: one copy, one wait
        batch = host.shape[1]
        counts = host[2].reshape(-1)[:batch]
        k = int(counts[0]) if batch else 0  # the reference sizes the arrays by request 0's result
        return {"indices": np.ascontiguousarray(host[0][:, :k]), "scores": np.ascontiguousarray(host[1][:, :k]).view(np.float32)}

    def discard(self, req_id: int) -> None:
        """Forgets a submitted request whose result will not be fetched (its owner finished) and releases its
        device buffers; the reference keeps such results until the process ends."""
        with self._lock:
            self._pending.pop(req_id, None)


def _pad_rows(indexes) -> np.ndarray:
    """list of per-request slot lists (or a 2-D array) -> int32 [B, M] padded with -1."""
    if isinstance(indexes, np.ndarray) and indexes.ndim == 2:
        return np.ascontiguousarray(indexes, dtype=np.int32)
    rows = [np.asarray(r, dtype=np.int32).reshape(-1) for r in indexes]
    m = max((len(r) for r in rows), default=0)
    out = np.full((len(rows), m), -1, np.int32)
    for i, r in enumerate(rows):
        out[i, : len(r)] = r
    return out


class RetrievalWorker:
    """Dtype/device front of the backend (retrieval_worker.py:10-34): queries in
    the model dtype are widened to float32; they stay on the device."""

    def __init__(self, cpp_worker: HipRetrievalBackend):
        self.cpp_worker = cpp_worker

    @classmethod
    def handle_input(cls, input):  # noqa: A002  (reference's parameter name)
        if input.dtype != torch.float32:
            input = input.to(torch.float32)
        return input

    def submit(self, query, topk, indexes):
        return self.cpp_worker.submit(self.handle_input(query), topk, indexes)

    def poll(self, req_id):
        return self.cpp_worker.poll(req_id)

    def get_result(self, req_id):
        return self.cpp_worker.get_result(req_id)

    def wait(self, req_id):
        return self.cpp_worker.wait(req_id)
