"""KVStar retrieval on the GPU behind the reference's ``kvstar_retrieve`` module
surface (ucm/sparse/kvstar/retrieve/py_intf/py_intf.cpp:14-133):

    task_id = AsyncRetrieveByCPU(query_group, blk_repre, d_pruned_index, topk, req_id, device_type)
    Wait(task_id)
    GetTaskResult(task_id) -> {"status": "SUCCESS", "data": [block indices]}

``query_group`` is fp16 ``[x, q_heads, d]`` and ``blk_repre`` fp16 ``[n, M, kv_heads,
d_pruned]`` as in ``ReqPerLayerState.retrieval_async`` (ucm/sparse/kvstar/multistep.py:240-265),
but both live on the device: the reference's thread pool (retrieve_task_manager.cpp,
retrieve_task_runner.cpp) becomes a side stream, a task's completion an event.
``extract_block_repre`` is the device twin of multistep.py:279-316; it returns a ``BlockRepre``,
which reports the reference's shape ``(n, M, kv_heads, d_pruned)`` and supports the block slices
the plugin takes (``[init:-local]``, multistep.py:495-497) but keeps the values in the order the
score kernel streams (``[kv_heads, n, d_pad/8, M, 8]``); ``dense()`` gives the reference's tensor.
A plain ``[n, M, kv_heads, d_pruned]`` tensor is accepted too and repacked once per call.

Block order in ``data``: descending by (vote, index), the order in which the reference's heap is
emptied (simd_compute_kernel.cpp:969-977).  It is restored on the device (``ops.kvstar_order``) and
read back once per launch, for all its tasks, when the first of them is asked for its list; the
device copy (``DeviceResult``) lets a caller load the chosen blocks without reading the list at all.
"""
from __future__ import annotations

import enum
import itertools
import threading
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ... import ops


class DeviceType(enum.Enum):
    CPU = 0
    GPU = 1


CPU, GPU = DeviceType.CPU, DeviceType.GPU


@dataclass
class SetupParam:
    """Accepted for interface compatibility; NUMA placement has no meaning here."""
    cpuNumaIds: List[int]
    physicalCorePerNuma: int
    allocRatio: float
    blkRepreSize: int
    deviceType: DeviceType
    totalTpSize: int
    localRankId: int


class _Results:
    """What one launch leaves behind for its tasks: the chosen blocks in the reference's order on the device
    (``idx`` int32 [n_tasks, stride], ``cnt`` int32 [n_tasks]).  The host's copy is made when the first task of the
    launch is asked for its list, for all of them at once."""

    def __init__(self, event, votes, idx, cnt, keep=()):
        self.event, self.votes, self.idx, self.cnt, self.keep = event, votes, idx, cnt, keep
        self._host = None

    def host(self):
        if self._host is None:
            self.event.synchronize()
            self._host = (self.idx.cpu(), self.cnt.cpu())
        return self._host

    def chosen(self, row: int) -> List[int]:
        idx, cnt = self.host()
        return idx[row, : int(cnt[row])].tolist()


@dataclass
class _Task:
    results: Optional[_Results]
    row: int = 0                        # this task's row of the launch's results
    error: Optional[str] = None

    @property
    def event(self):
        return None if self.results is None else self.results.event


_tasks: Dict[int, _Task] = {}
_ids = itertools.count(1)
_lock = threading.Lock()
_stream: Optional[torch.cuda.Stream] = None
_layer_pointers: Dict[int, "ops.LayerPointers"] = {}     # one pointer table per key cache seen by extract_block_repre


def Setup(param: SetupParam) -> None:  # noqa: N802 (reference name)
    global _stream
    if _stream is None:
        _stream = torch.cuda.Stream()  # default priority


class BlockRepre:
    """Sub-block representatives of n blocks in the score kernel's order; ``table`` is fp16
    [kv_heads, n, d_pad/8, M, 8] (possibly a block slice of a bigger table)."""

    def __init__(self, table: torch.Tensor, d_pruned: int):
        self.table = table
        self.d_pruned = int(d_pruned)

    @property
    def shape(self) -> torch.Size:
        h, n, _, m, _ = self.table.shape
        return torch.Size((n, m, h, self.d_pruned))

    dtype = property(lambda self: self.table.dtype)
    device = property(lambda self: self.table.device)

    def dim(self) -> int:
        return 4

    def __len__(self) -> int:
        return self.table.shape[1]

    def __getitem__(self, blocks) -> "BlockRepre":
        if not isinstance(blocks, slice) or blocks.step not in (None, 1):
            raise TypeError("BlockRepre supports contiguous block slices only; use dense() for anything else")
        return BlockRepre(self.table[:, blocks], self.d_pruned)

    def dense(self) -> torch.Tensor:
        """The reference's [n, M, kv_heads, d_pruned] tensor (a copy)."""
        return ops.kvstar_table_to_reference(self.table)[..., : self.d_pruned].contiguous()


def AsyncRetrieveByCPU(query_group: torch.Tensor, blk_repre: torch.Tensor, d_pruned_index, topk: int, req_id: int,
                       device_type: DeviceType = CPU) -> int:  # noqa: N802
    """Queues one retrieval; returns its task id.  Shape errors are reported through the task
    result ("FAILURE" + the reference's message), as the reference's worker thread does."""
    global _stream
    if _stream is None:
        _stream = torch.cuda.Stream()
    task_id = next(_ids)
    try:
        if query_group.dim() != 3:
            raise RuntimeError("Query shape must be 3D (x, H, d).")
        if blk_repre.dim() != 4:
            raise RuntimeError("BlockRep shape must be 4D (n, M, h, d).")
        packed = isinstance(blk_repre, BlockRepre)
        x, hq, d_orig = query_group.shape
        n, m, h, dp = blk_repre.shape
        if hq % h != 0:
            raise RuntimeError("Num_q_heads must be a divisible by num_kv_heads.")
        pruned = sel = None
        if d_pruned_index is not None:
            if tuple(d_pruned_index.shape) != (h, dp):
                raise RuntimeError("dPrunedIndex shape is inconsistent with K's shape.")
            pruned = d_pruned_index.to(device=blk_repre.device, dtype=torch.int32).reshape(1, h, dp).contiguous()
            sel = torch.zeros(1, dtype=torch.int32, device=blk_repre.device)
        elif d_orig != dp:
            raise RuntimeError("Dimension mismatch: No dPrunedIndex, but Q and K head dims differ.")
        if query_group.dtype != torch.float16 or blk_repre.dtype != torch.float16:
            raise RuntimeError("query group and block representatives must be float16 device tensors")
        dev = blk_repre.device
        ready = torch.cuda.Event()
        ready.record()
        with torch.cuda.stream(_stream):
            _stream.wait_event(ready)
            table = blk_repre.table if packed else ops.kvstar_table_from_reference(blk_repre)
            q = query_group.contiguous()
            votes = torch.zeros(max(n, 1), dtype=torch.float32, device=dev)
            k = min(int(topk), n)
            idx = torch.zeros((1, max(n, 1)), dtype=torch.int32, device=dev)
            cnt = torch.zeros(1, dtype=torch.int32, device=dev)
            keep = (table, q, pruned, sel)
            if n > 0 and k > 0:
                seg_off = torch.zeros(1, dtype=torch.int32, device=dev)
                seg_len = torch.full((1,), n, dtype=torch.int32, device=dev)
                ws = ops.kvstar_workspace(1, h, x * (hq // h), n, m, table.shape[2] * 8, dev)
                ops.kvstar_votes(q, torch.zeros(1, dtype=torch.int64, device=dev), x, hq, table, seg_off, seg_len, n, votes,
                                 ws, d_pruned=dp, pruned=pruned, pruned_sel=sel)
                ops.kvstar_topk(votes, seg_off, seg_len, torch.full((1,), k, dtype=torch.int32, device=dev), n, idx, cnt)
                ops.kvstar_order(votes, seg_off, seg_len, k, idx, cnt)
                keep += (seg_off, seg_len, ws)
            results = _Results(torch.cuda.Event(), votes, idx, cnt, keep)
            results.event.record(_stream)
        task = _Task(results, 0)
    except RuntimeError as e:
        task = _Task(None, error=str(e))
    with _lock:
        _tasks[task_id] = task
    return task_id


def AsyncRetrieveBatch(query_groups, blk_repres, d_pruned_indexes, topks, req_ids=None, device_type: DeviceType = CPU) -> List[int]:  # noqa: N802
    """Several retrievals (the requests of one layer) in one launch; returns one task id per entry, to be used
    with Wait / GetTaskResult like those of AsyncRetrieveByCPU.  Every entry must have the same number of query
    tokens, heads and kept channels, and a BlockRepre (extract_block_repre's result) as representatives;
    ``query_groups`` is a list of fp16 [x, q_heads, d] tensors or one fp16 tensor [n_tasks, x, q_heads, d]."""
    global _stream
    if _stream is None:
        _stream = torch.cuda.Stream()
    n_tasks = len(query_groups)
    if n_tasks == 0:
        return []
    ids = [next(_ids) for _ in range(n_tasks)]
    try:
        q0, r0 = query_groups[0], blk_repres[0]
        if any(not isinstance(r, BlockRepre) for r in blk_repres):
            raise RuntimeError("AsyncRetrieveBatch takes BlockRepre representatives")
        x, hq, d_orig = q0.shape
        _, m, h, dp = r0.shape
        stacked = isinstance(query_groups, torch.Tensor)      # [n_tasks, x, q_heads, d] in one tensor
        if stacked and query_groups.dtype != torch.float16:
            raise RuntimeError("query groups must be float16")
        for qg, r in zip(query_groups, blk_repres):
            if tuple(r.shape[1:]) != (m, h, dp) or (not stacked and (tuple(qg.shape) != (x, hq, d_orig) or qg.dtype != torch.float16)):
                raise RuntimeError("the entries of a batch must agree in query tokens, heads, sub-blocks and kept channels")
        if hq % h != 0:
            raise RuntimeError("Num_q_heads must be a divisible by num_kv_heads.")
        with_lists = d_pruned_indexes is not None and any(i is not None for i in d_pruned_indexes)
        if with_lists:
            if any(i is None or tuple(i.shape) != (h, dp) for i in d_pruned_indexes):
                raise RuntimeError("dPrunedIndex shape is inconsistent with K's shape.")
        elif d_orig != dp:
            raise RuntimeError("Dimension mismatch: No dPrunedIndex, but Q and K head dims differ.")
        dev = r0.device
        lens = [int(r.shape[0]) for r in blk_repres]
        offs = [0]
        for n in lens[:-1]:
            offs.append(offs[-1] + n)
        total, longest = sum(lens), max(lens)
        ready = torch.cuda.Event()
        ready.record()
        with torch.cuda.stream(_stream):
            _stream.wait_event(ready)
            q = query_groups.contiguous() if stacked else torch.stack([qg.contiguous() for qg in query_groups])
            pruned = sel = None
            if with_lists:
                pruned = torch.stack([i.to(device=dev, dtype=torch.int32) for i in d_pruned_indexes]).contiguous()
                sel = torch.arange(n_tasks, dtype=torch.int32, device=dev)
            meta_d = ops.upload(torch.tensor([offs, lens, [min(int(k), n) for k, n in zip(topks, lens)]], dtype=torch.int32), dev)
            q_off = torch.arange(n_tasks, dtype=torch.int64, device=dev) * (x * hq * d_orig)
            votes = torch.zeros(max(total, 1), dtype=torch.float32, device=dev)
            idx = torch.zeros((n_tasks, max(longest, 1)), dtype=torch.int32, device=dev)
            cnt = torch.zeros(n_tasks, dtype=torch.int32, device=dev)
            keep = (q, pruned, sel, meta_d, q_off, tuple(r.table for r in blk_repres))
            if longest > 0:
                ws = ops.kvstar_workspace(n_tasks, h, x * (hq // h), longest, m, r0.table.shape[2] * 8, dev)
                ptrs = ops.kvstar_votes_tables(q, q_off, x, hq, [r.table for r in blk_repres], meta_d[0], meta_d[1], longest, votes, ws,
                                               d_pruned=dp, pruned=pruned, pruned_sel=sel)
                ops.kvstar_topk(votes, meta_d[0], meta_d[1], meta_d[2], longest, idx, cnt)
                ops.kvstar_order(votes, meta_d[0], meta_d[1], longest, idx, cnt)
                keep += (ws, ptrs)
            results = _Results(torch.cuda.Event(), votes, idx, cnt, keep)
            results.event.record(_stream)
        tasks = [_Task(results, i) for i in range(n_tasks)]
    except RuntimeError as e:
        tasks = [_Task(None, error=str(e)) for _ in range(n_tasks)]
    with _lock:
        for i, t in zip(ids, tasks):
            _tasks[i] = t
    return ids


def RegisterBatch(results: _Results, n_tasks: int) -> List[int]:  # noqa: N802
    """Task ids for the rows of a launch somebody else queued (``results.event`` recorded after it): row i becomes
    a task that Wait / GetTaskResult / DeviceResult / Forget treat like one of AsyncRetrieveBatch's."""
    ids = [next(_ids) for _ in range(n_tasks)]
    with _lock:
        for row, task_id in enumerate(ids):
            _tasks[task_id] = _Task(results, row)
    return ids


def Wait(task_id: int) -> None:  # noqa: N802
    with _lock:
        task = _tasks.get(task_id)
    if task is not None and task.event is not None:
        task.event.synchronize()


def GetTaskResult(task_id: int):  # noqa: N802
    """Status dictionary of a task (py_intf.cpp:55-95); None for an id that is not (or no longer) known.  A finished
    task is handed out once: delivering "SUCCESS" or "FAILURE" forgets the task and releases its device buffers
    (the reference keeps every result for the life of the process)."""
    with _lock:
        task = _tasks.get(task_id)
    if task is None:
        return None
    if task.error is not None:
        with _lock:
            _tasks.pop(task_id, None)
        return {"status": "FAILURE", "error": task.error}
    if not task.event.query():
        return {"status": "RUNNING"}
    data = task.results.chosen(task.row)
    with _lock:
        _tasks.pop(task_id, None)
    return {"status": "SUCCESS", "data": data}


def DeviceResult(task_id: int):  # noqa: N802
    """(results, row) of a queued task, for callers that use the chosen blocks on the device: ``results.idx[row,
    :results.cnt[row]]`` are valid on any stream that has waited for ``results.event``.  Raises the task's error if
    it failed at submission; the task stays known until GetTaskResult or Forget."""
    with _lock:
        task = _tasks.get(task_id)
    if task is None:
        return None
    if task.error is not None:
        raise RuntimeError(task.error)
    return task.results, task.row


def Forget(task_id: int) -> None:  # noqa: N802
    with _lock:
        _tasks.pop(task_id, None)


def ForgetBatch(task_ids) -> None:  # noqa: N802
    with _lock:
        for task_id in task_ids:
            _tasks.pop(task_id, None)


def extract_block_repre(k_cache: torch.Tensor, vllm_block_ids: List[int], merge: int, prune_ratio: float = 1.0,
                        d_pruned_index: Optional[torch.Tensor] = None, prune_dim_enable: bool = False):
    """Sub-block representatives of cache blocks ``vllm_block_ids`` (multistep.py:279-316).
    Returns (BlockRepre of shape (n, M, kv_heads, d_pruned), d_pruned_index int64 [kv_heads, d_pruned] or None).  With ``prune_dim_enable`` and a ratio below 0.98 the channels with the largest mean |k|
    over these blocks are kept per head (the reference's choice, :284-292); otherwise a given index is reused."""
    n_total, block_size, kv_heads, head_dim = k_cache.shape
    dev = k_cache.device
    n = len(vllm_block_ids)
    ids = ops.upload(torch.tensor(vllm_block_ids, dtype=torch.int32), dev)
    rows = torch.arange(n, dtype=torch.int32, device=dev)
    known = _layer_pointers.get(k_cache.data_ptr())
    if known is None or known.tensors[0].shape != k_cache.shape:
        if len(_layer_pointers) > 256:                   # caches come and go with engines; the table stays small
            _layer_pointers.clear()
        known = _layer_pointers[k_cache.data_ptr()] = ops.LayerPointers([k_cache])
    if prune_dim_enable and prune_ratio < 0.98:
        # mean |k| per (head, channel) over all tokens of these blocks: the blocks' own means of |k|, read from the
        # paged cache in one pass, averaged (the reference gathers the blocks and takes one mean, :284-290)
        per_block = torch.empty((1, n, kv_heads * head_dim), dtype=torch.float32, device=dev)
        ops.block_mean(known, ids, rows, per_block, block_size, kv_heads, head_dim, n_total, mode=ops.MEAN_F32 | ops.MEAN_ABS)
        absmean = per_block[0].mean(dim=0).view(kv_heads, head_dim)
        _, d_pruned_index = torch.topk(absmean, k=round(head_dim * prune_ratio), dim=-1)
        d_pruned_index = d_pruned_index.contiguous()
    d_pruned = head_dim if d_pruned_index is None else d_pruned_index.shape[1]
    d_pad = (d_pruned + 15) // 16 * 16
    table = ops.kvstar_table(1, kv_heads, n, block_size // merge, d_pad, dev)
    pruned32 = None if d_pruned_index is None else d_pruned_index.to(torch.int32).contiguous()
    ops.kvstar_block_repre(known, ids, rows, table, block_size, kv_heads, head_dim, n_total, merge, pruned=pruned32)
    return BlockRepre(table[0], d_pruned), d_pruned_index
