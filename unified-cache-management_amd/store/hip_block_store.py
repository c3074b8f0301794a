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
``device`` ("cuda" | "pinned"), ``role`` and ``host_spill_blocks``.

``host_spill_blocks`` > 0 puts a tier of pinned host memory behind a pool in
HBM, moved through the library's device object the way the reference's stores
move shards through theirs (``IBufferedDevice``: GetBuffer + D2HAsync /
H2DAsync + AppendCallback, ucm/store/device/ibuffered_device.h:32-66,
ucm/store/device/cuda/cuda_device.cu:115-178): when ``create`` finds the pool
full, the committed block that was used longest ago is copied to a pinned
buffer on the store's stream and its slot handed on; a ``load`` (or ``hold``)
of a spilled block copies it back first.  Both copies are asynchronous; their
completion callbacks do the bookkeeping (``spills_done`` / buffers back to the
ring).  Blocks that kernels read in place (``device_pool`` + ``slot_of``) are
``hold``-ed by the plugins for as long as a request may load them and are never
spilled; ``generation`` counts the spills for callers that cache slot numbers
without holding.
"""
from __future__ import annotations

from collections import OrderedDict
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
        # the pinned-host tier behind a pool in HBM
        self.host_blocks = int(config.get("host_spill_blocks", 0)) if self._where == "cuda" else 0
        self._device = None                              # the library's device object: pinned buffers, stream, callbacks
        self.host_of: Dict[str, Any] = {}                # spilled block -> its pinned buffer
        self._lru: "OrderedDict[str, None]" = OrderedDict()   # committed blocks in the pool, coldest first
        self._held: Dict[str, int] = {}                  # blocks kernels may read in place: never spilled
        self.generation = 0                              # bumped whenever a block leaves the pool
        self.spills = self.spills_done = self.reloads = 0
        self._last_write = None                          # event after the last copy into the pool on the store's stream

    # ---- storage -----------------------------------------------------------
    def _ensure_buffer(self) -> torch.Tensor:
        if self._buffer is None:
            nbytes = self.max_block_num * self.kv_block_size
            if self._where == "pinned":
                self._buffer = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
            else:
                self._buffer = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            if self.host_blocks:
                from .hip_device import HipDevice

                self._device = HipDevice(torch.cuda.current_device(), self.kv_block_size, self.host_blocks)
                self._device.Setup()
                self._stream = torch.cuda.ExternalStream(self._device.stream)   # spills, reloads and moves in one order
            else:
                self._stream = torch.cuda.Stream()  # default priority
        return self._buffer

    # ---- the host tier -------------------------------------------------------
    def _slot(self) -> Optional[int]:
        """A free slot of the pool, making one by spilling the coldest block nobody holds if need be."""
        if self.free_slots:
            return self.free_slots.pop()
        if not self.host_blocks or len(self.host_of) >= self.host_blocks:
            return None
        self._ensure_buffer()
        victim = next((b for b in self._lru if not self._held.get(b)), None)
        if victim is None:
            return None
        buf = self._device.GetBuffer(self.kv_block_size)
        if buf is None:
            return None
        slot = self.slot_of.pop(victim)
        del self._lru[victim]
        ready = torch.cuda.Event()                       # the block may have been written on the caller's stream
        ready.record()
        self._stream.wait_event(ready)
        self._device.D2HAsync(buf.ptr, self._ensure_buffer().data_ptr() + slot * self.kv_block_size, self.kv_block_size)
        self._device.AppendCallback(self._spill_done)
        self.host_of[victim] = buf
        self.spills += 1
        self.generation += 1
        # whoever writes the slot next, on whatever stream, comes after the copy that empties it
        done = torch.cuda.Event()
        done.record(self._stream)
        torch.cuda.current_stream().wait_event(done)
        return slot

    def _spill_done(self, ok: bool) -> None:             # (on the runtime's callback thread)
        self.spills_done += 1 if ok else 0

    def _reload(self, block: str) -> bool:
        """A spilled block back into the pool (asynchronous, on the store's stream)."""
        slot = self._slot()
        if slot is None:
            return False
        buf = self.host_of.pop(block)
        self._device.H2DAsync(self._ensure_buffer().data_ptr() + slot * self.kv_block_size, buf.ptr, self.kv_block_size)
        self._device.AppendCallback(lambda ok, b=buf: b.release())     # the buffer goes back to the ring when the copy is through
        self.slot_of[block] = slot
        self._lru[block] = None
        self.reloads += 1
        self._wrote()
        return True

    def _wrote(self) -> None:
        if self._last_write is None:
            self._last_write = torch.cuda.Event()
        self._last_write.record(self._stream)

    def wait_for_writes(self) -> None:
        """Makes the current stream wait (on the device, not the host) for everything the store's stream has copied
        into the pool so far: kernels that read stored blocks in place call it before they do."""
        if self._last_write is not None:
            torch.cuda.current_stream().wait_event(self._last_write)

    def hold(self, block_ids: List[str]) -> List[int]:
        """Slots of blocks that kernels are going to read in place (-1: the store does not have it): spilled ones come
        back into the pool first, and none of them leaves it before ``release``."""
        self._ensure_buffer()
        out = []
        for b in block_ids:
            if b in self.host_of and not self._reload(b):
                out.append(-1)
                continue
            slot = self.slot_of.get(b, -1)
            if slot >= 0:
                self._held[b] = self._held.get(b, 0) + 1
            out.append(slot)
        self.wait_for_writes()
        return out

    def release(self, block_ids: List[str]) -> None:
        for b in block_ids:
            n = self._held.get(b, 0) - 1
            if n > 0:
                self._held[b] = n
            else:
                self._held.pop(b, None)

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
            if b in self.slot_of or b in self.host_of:
                out.append(SUCCESS)
                continue
            slot = self._slot()
            if slot is None:
                out.append(FAILURE)
            else:
                self.slot_of[b] = slot
                out.append(SUCCESS)
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
                    self._lru[b] = None
                    self._lru.move_to_end(b)
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
            if b in self.host_of and not self._reload(b):
                task.task_id = "-1"          # spilled, and no slot to bring it back into
                return task
            if b not in self.slot_of:
                if not to_store or self.create([b])[0] != SUCCESS:
                    task.task_id = "-1"      # unknown block on load, or store full on dump
                    return task
            if b in self._lru:
                self._lru.move_to_end(b)
            if off < 0 or off + sizes[0] > self.kv_block_size:
                raise ValueError("offset outside the stored block")
            store_ptrs.append(base + self.slot_of[b] * self.kv_block_size + off)
        dev = torch.device("cuda", torch.cuda.current_device())
        host = torch.tensor([store_ptrs, addrs], dtype=torch.int64)
        # the pointer arrays are allocated and filled on the caller's stream (nothing is ever allocated on the store's
        # stream: a tensor freed after that stream is gone could not be handed back to the allocator)
        ptrs = ops.upload(host, dev)
        ready = torch.cuda.Event()
        ready.record()                       # the caller's stream produced / will consume the tensors
        with torch.cuda.stream(self._stream):
            self._stream.wait_event(ready)
            dst, src = (ptrs[0], ptrs[1]) if to_store else (ptrs[1], ptrs[0])
            ops.copy_batch(dst, src, sizes[0])
            task.event = torch.cuda.Event()
            task.event.record(self._stream)
            if to_store:
                self._wrote()
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
