"""A KV block store with the surface of the reference's ``UcmKVStoreBase``
(ucm/store/ucmstore.py:39-204), kept in one staging buffer and moved by the
batched copy kernel.

The reference's stores receive, per call, one tensor view per block
(``k_cache[id]``, ucm/sparse/esa/esa.py:254-258) plus a byte offset inside the
stored block (``get_offset``, esa.py:124-135: [layer][K|V][rank]); the DRAM
store then issues one ``copy_`` per block (ucm/store/dramstore/dramstore_connector.py:112-166)
and the NFS store one memcpy per 256 KiB shard.  Here a stored block is a slot
of ``kv_block_size`` bytes in a single buffer (HBM by default - 288 GB makes an
on-device block store practical - or pinned host memory), and a whole
load/dump call becomes ONE launch of ``ucm_copy_batch`` over two pointer arrays,
the twin of the reference device layer's H2DBatch/D2HBatch
(ucm/store/device/cuda/cuda_device.cu:47-81).

Config keys (same names as the DRAM store): ``max_cache_size`` bytes,
``kv_block_size`` bytes of one stored block (all layers, K and V), plus
``device`` ("cuda" | "pinned") and ``role``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

import torch

from .. import ops

SUCCESS = 0
FAILURE = -1


class Task:
    """Handle of one transfer (ucm/store/ucmstore.py:31-36)."""


@dataclass
class HipTask(Task):
    task_id: str = "1"
    event: Optional[Any] = None
    keep: Optional[tuple] = None  # pointer arrays stay alive until the copy ran


class UcmHipBlockStore:
    def __init__(self, config: Dict):
        self.config = config
        self.kv_block_size = int(config.get("kv_block_size", 262144))
        self.max_cache_byte = int(config.get("max_cache_size", 5368709120))
        self.max_block_num = self.max_cache_byte // self.kv_block_size
        self.role = config.get("role", "worker")
        self.slot_of: Dict[str, int] = {}
        self.committed = set()
        self.free_slots = list(range(self.max_block_num - 1, -1, -1))
        self._buffer: Optional[torch.Tensor] = None
        self._stream: Optional[torch.cuda.Stream] = None
        self._where = config.get("device", "cuda")

    # ---- storage -----------------------------------------------------------
    def _ensure_buffer(self) -> torch.Tensor:
        if self._buffer is None:
            nbytes = self.max_block_num * self.kv_block_size
            if self._where == "pinned":
                self._buffer = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
            else:
                self._buffer = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            self._stream = torch.cuda.Stream()  # default priority
        return self._buffer

    def cc_store(self) -> int:
        return 0

    def device_pool(self) -> Tuple[torch.Tensor, int]:
        """The buffer holding every stored block (slot i at byte i*kv_block_size) and the size of a stored block:
        what a kernel needs to read blocks in place (``slot_of`` maps a block hash to its slot).  Plugins that find
        this method plan and run their loads on the device instead of calling ``load`` block by block."""
        return self._ensure_buffer(), self.kv_block_size

    def create(self, block_ids: List[str]) -> List[int]:
        """Reserves a slot per block hash; FAILURE for those that do not fit."""
        out = []
        for b in block_ids:
            if b in self.slot_of:
                out.append(SUCCESS)
            elif self.free_slots:
                self.slot_of[b] = self.free_slots.pop()
                out.append(SUCCESS)
            else:
                out.append(FAILURE)
        return out

    def lookup(self, block_ids: List[str]) -> List[bool]:
        return [b in self.committed for b in block_ids]

    def prefetch(self, block_ids: List[str]) -> None:
        pass

    def commit(self, block_ids: List[str], is_success: bool = True) -> None:
        for b in block_ids:
            if is_success:
                if b in self.slot_of:
                    self.committed.add(b)
            elif b in self.slot_of and b not in self.committed:
                self.free_slots.append(self.slot_of.pop(b))

    # ---- transfers -----------------------------------------------------------
    def _move(self, block_ids: List[str], offset: List[int], addrs: List[int], sizes: List[int], to_store: bool) -> HipTask:
        task = HipTask()
        if not block_ids:
            task.event = None
            return task
        if len(set(sizes)) != 1 or sizes[0] % 16:
            raise ValueError("all pieces of one call must have the same size, a multiple of 16 bytes")
        buf = self._ensure_buffer()
        base = buf.data_ptr()
        store_ptrs = []
        for b, off in zip(block_ids, offset):
            if b not in self.slot_of:
                if not to_store or self.create([b])[0] != SUCCESS:
                    task.task_id = "-1"      # unknown block on load, or store full on dump
                    return task
            if off < 0 or off + sizes[0] > self.kv_block_size:
                raise ValueError("offset outside the stored block")
            store_ptrs.append(base + self.slot_of[b] * self.kv_block_size + off)
        dev = torch.device("cuda", torch.cuda.current_device())
        host = torch.tensor([store_ptrs, addrs], dtype=torch.int64)
        ready = torch.cuda.Event()
        ready.record()                       # the caller's stream produced / will consume the tensors
        with torch.cuda.stream(self._stream):
            self._stream.wait_event(ready)
            ptrs = ops.upload(host, dev)     # staged through reused pinned memory, copied on this stream
            dst, src = (ptrs[0], ptrs[1]) if to_store else (ptrs[1], ptrs[0])
            ops.copy_batch(dst, src, sizes[0])
            task.event = torch.cuda.Event()
            task.event.record(self._stream)
        task.keep = (ptrs,)
        return task

    @staticmethod
    def _views(tensors: List[torch.Tensor]) -> Tuple[List[int], List[int]]:
        for t in tensors:
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError("block tensors must be contiguous device tensors")
        return [t.data_ptr() for t in tensors], [t.numel() * t.element_size() for t in tensors]

    def load(self, block_ids: List[str], offset: List[int], dst_tensor: List[torch.Tensor]) -> Task:
        addrs, sizes = self._views(dst_tensor)
        return self._move(block_ids, offset, addrs, sizes, to_store=False)

    def dump(self, block_ids: List[str], offset: List[int], src_tensor: List[torch.Tensor]) -> Task:
        addrs, sizes = self._views(src_tensor)
        return self._move(block_ids, offset, addrs, sizes, to_store=True)

    @staticmethod
    def _checked(addrs: List[int], sizes: List[int]) -> List[int]:
        """Raw addresses go straight to a copy kernel: each must be memory a kernel can touch (device memory or
        pinned host memory); pageable host memory is refused here, on the host."""
        from .. import _lib

        can = _lib.lib().ucm_kernel_can_access
        for a, n in zip(addrs, sizes):
            if not can(int(a), int(n)):
                raise ValueError(f"address {int(a):#x} is not device or pinned host memory")
        return [int(a) for a in addrs]

    def fetch_data(self, block_ids: List[str], offset: List[int], dst_addr: List[int], size: List[int]) -> Task:
        return self._move(block_ids, offset, self._checked(dst_addr, size), list(size), to_store=False)

    def dump_data(self, block_ids: List[str], offset: List[int], src_addr: List[int], size: List[int]) -> Task:
        return self._move(block_ids, offset, self._checked(src_addr, size), list(size), to_store=True)

    def wait(self, task: HipTask) -> int:
        if task.task_id == "-1":
            return FAILURE
        if task.event is not None:
            task.event.synchronize()
        task.keep = None
        return SUCCESS

    def check(self, task: HipTask) -> Tuple[int, bool]:
        if task.task_id == "-1":
            return FAILURE, True
        return SUCCESS, task.event is None or task.event.query()
