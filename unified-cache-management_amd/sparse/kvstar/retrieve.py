"""KVStar retrieval on the GPU behind the reference's ``kvstar_retrieve`` module
surface (ucm/sparse/kvstar/retrieve/py_intf/py_intf.cpp:14-133):

    task_id = AsyncRetrieveByCPU(query_group, blk_repre, d_pruned_index, topk, req_id, device_type)
    Wait(task_id)
    GetTaskResult(task_id) -> {"status": "SUCCESS", "data": [block indices]}

``query_group`` is fp16 ``[x, q_heads, d]`` and ``blk_repre`` fp16 ``[n, M, kv_heads,
d_pruned]`` as in ``ReqPerLayerState.retrieval_async`` (ucm/sparse/kvstar/multistep.py:240-265),
but both live on the device: the reference's thread pool (retrieve_task_manager.cpp,
retrieve_task_runner.cpp) becomes a side stream, a task's completion an event.
``extract_block_repre`` is the device twin of multistep.py:279-316; what it returns has the
reference's shape but is a view of head-major storage (``[kv_heads, n, M, d_pad]``, the
order the score kernel streams), and stays one under row slices such as ``[init:-local]``.
A tensor in any other memory order is accepted too and repacked once per call.

Block order in ``data``: descending vote, lower index first among equals (what the
reference's portable kernel returns; its AVX2 build returns the same set unordered).
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


@dataclass
class _Task:
    event: Optional[torch.cuda.Event]
    votes: Optional[torch.Tensor]
    idx: Optional[torch.Tensor]
    cnt: Optional[torch.Tensor]
    keep: tuple = ()
    error: Optional[str] = None


_tasks: Dict[int, _Task] = {}
_ids = itertools.count(1)
_lock = threading.Lock()
_stream: Optional[torch.cuda.Stream] = None


def Setup(param: SetupParam) -> None:  # noqa: N802 (reference name)
    global _stream
    if _stream is None:
        _stream = torch.cuda.Stream()  # default priority


def _head_major(blk_repre: torch.Tensor) -> torch.Tensor:
    """[n, M, h, dp] (reference order of the dims) -> fp16 [h, n, M, d_pad] whose (n, M, d_pad) part is dense."""
    n, m, h, dp = blk_repre.shape
    hm = blk_repre.permute(2, 0, 1, 3)
    d_phys = hm.stride(2) if m > 1 or n > 1 else dp
    if hm.stride(3) == 1 and d_phys % 16 == 0 and 0 <= d_phys - dp < 16 and hm.stride(2) == d_phys \
            and hm.stride(1) == m * d_phys and hm.data_ptr() % 16 == 0 \
            and (h == 1 or (hm.stride(0) % 8 == 0 and hm.stride(0) >= n * m * d_phys)):
        # already head-major (what extract_block_repre hands out); widen the view to the padded columns (zeros)
        return torch.as_strided(hm, (h, n, m, d_phys), (hm.stride(0), m * d_phys, d_phys, 1))
    out = torch.zeros((h, n, m, (dp + 15) // 16 * 16), dtype=blk_repre.dtype, device=blk_repre.device)
    out[..., :dp] = hm
    return out


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
            table = _head_major(blk_repre)
            q = query_group.contiguous()
            votes = torch.zeros(max(n, 1), dtype=torch.float32, device=dev)
            k = min(int(topk), n)
            idx = torch.zeros((1, 1, max(n, 1)), dtype=torch.int32, device=dev)
            cnt = torch.zeros((1, 1), dtype=torch.int32, device=dev)
            keep = (table, q, pruned, sel)
            if n > 0 and k > 0:
                seg_off = torch.zeros(1, dtype=torch.int32, device=dev)
                seg_len = torch.full((1,), n, dtype=torch.int32, device=dev)
                ws = ops.kvstar_workspace(1, h, x * (hq // h), n, m, dev)
                ops.kvstar_votes(q, torch.zeros(1, dtype=torch.int64, device=dev), x, hq, table, seg_off, seg_len, n, votes,
                                 ws, d_pruned=dp, pruned=pruned, pruned_sel=sel)
                ops.topk_windows(votes.view(1, -1), seg_off, seg_len, torch.full((1,), k, dtype=torch.int32, device=dev), n,
                                 idx, cnt, start_w=0, end_w=0)
                keep += (seg_off, seg_len, ws)
            event = torch.cuda.Event()
            event.record(_stream)
        task = _Task(event, votes, idx, cnt, keep)
    except RuntimeError as e:
        task = _Task(None, None, None, None, error=str(e))
    with _lock:
        _tasks[task_id] = task
    return task_id


def Wait(task_id: int) -> None:  # noqa: N802
    with _lock:
        task = _tasks.get(task_id)
    if task is not None and task.event is not None:
        task.event.synchronize()


def GetTaskResult(task_id: int):  # noqa: N802
    with _lock:
        task = _tasks.get(task_id)
    if task is None:
        return None
    if task.error is not None:
        return {"status": "FAILURE", "error": task.error}
    if not task.event.query():
        return {"status": "RUNNING"}
    n = int(task.cnt[0, 0])
    chosen = task.idx[0, 0, :n].long()
    order = torch.argsort(task.votes[chosen], descending=True, stable=True)   # chosen is ascending: ties keep the lower index first
    task.keep = ()
    return {"status": "SUCCESS", "data": chosen[order].tolist()}


def extract_block_repre(k_cache: torch.Tensor, vllm_block_ids: List[int], merge: int, prune_ratio: float = 1.0,
                        d_pruned_index: Optional[torch.Tensor] = None, prune_dim_enable: bool = False):
    """Sub-block representatives of cache blocks ``vllm_block_ids`` (multistep.py:279-316).
    Returns (fp16 of shape [n, M, kv_heads, d_pad] - a view of head-major storage - with zero columns past
    d_pruned, d_pruned_index int64 [kv_heads, d_pruned] or None).  With ``prune_dim_enable`` and a ratio below 0.98 the channels with the largest mean |k|
    over these blocks are kept per head (the reference's choice, :284-292); otherwise a given index is reused."""
    n_total, block_size, kv_heads, head_dim = k_cache.shape
    dev = k_cache.device
    ids = torch.tensor(vllm_block_ids, dtype=torch.int32, device=dev)
    if prune_dim_enable and prune_ratio < 0.98:
        absmean = k_cache[ids.long()].reshape(-1, kv_heads, head_dim).to(torch.float32).abs().mean(dim=0)
        _, d_pruned_index = torch.topk(absmean, k=round(head_dim * prune_ratio), dim=-1)
        d_pruned_index = d_pruned_index.contiguous()
    d_pruned = head_dim if d_pruned_index is None else d_pruned_index.shape[1]
    d_pad = (d_pruned + 15) // 16 * 16
    repre = torch.empty((1, kv_heads, len(vllm_block_ids), block_size // merge, d_pad), dtype=torch.float16, device=dev)
    pruned32 = None if d_pruned_index is None else d_pruned_index.to(torch.int32).contiguous()
    ops.kvstar_block_repre(ops.LayerPointers([k_cache]), ids, torch.arange(len(vllm_block_ids), dtype=torch.int32, device=dev),
                           repre, block_size, kv_heads, head_dim, n_total, merge, pruned=pruned32)
    return repre[0].permute(1, 2, 0, 3), d_pruned_index
