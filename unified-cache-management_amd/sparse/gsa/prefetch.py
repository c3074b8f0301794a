"""The GSA prefetch engine's native object on the GPU.

``GSAPrefetchEngineC`` keeps the method names and call protocol of the
reference's pybind11 class (ucm/sparse/gsa/prefetch/src/pybinds.cpp:13-24,
include/kvcache_pre.h:68-152): the Python side hands it four tensors it shares
with the engine (free blocks, success block tables and their lengths),
registers each request's resident blocks (``set_blocks_map`` /
``add_blocks_map``), and after every top-k calls ``set_blocks_table_info`` +
``run_async_prefetch_bs``; ``get_prefetch_status`` then tells when
``obtain_load_blocks`` / ``obtain_miss_idxs`` can be read.

What differs is where it runs.  The reference walks std::map containers on a
worker thread (16 OpenMP threads over the layers, requests one after the
other, src/kvcache_pre.cpp:274-311); here the shared tensors live in device
memory, a request's maps are a row of device arrays, and one
``ucm_prefetch_plan`` launch does every request and layer of the call.  The
results stay on the device: ``load_missing`` moves the missed blocks from a
device-addressable pool into the cache blocks chosen for them without the host
seeing either list.  The ``obtain_*`` accessors copy them back for callers
written against the reference's surface.

Limits (the reference's containers have none): 256 resident blocks and 256
selected blocks per request; ``set_blocks_map`` / ``add_blocks_map`` and
``run_async_prefetch_bs`` raise ``ValueError`` beyond them.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ... import ops


class GSAPrefetchEngineC:
    def __init__(self, free_block: torch.Tensor, load_success_blocks: torch.Tensor, free_block_len: torch.Tensor,
                 success_table_len: torch.Tensor, is_log: bool = False, max_requests: Optional[int] = None):
        for t in (free_block, load_success_blocks, free_block_len, success_table_len):
            if not t.is_cuda or t.dtype != torch.int32 or not t.is_contiguous():
                raise ValueError("the engine's tensors must be contiguous int32 device tensors")
        self.free_block, self.free_block_len = free_block, free_block_len
        self.success_blocks, self.success_len = load_success_blocks, success_table_len
        self.n_layers, self.max_bs, self.max_len = load_success_blocks.shape
        self.device = free_block.device
        self.cap = 256                                   # resident blocks per request the kernel handles
        self.topk_stride = min(self.max_len, 256)
        rows = self.max_bs if max_requests is None else max_requests
        i32 = dict(dtype=torch.int32, device=self.device)
        self.map_block = torch.full((rows, self.cap), -1, **i32)
        self.map_len = torch.zeros(rows, **i32)
        self.map_idx = torch.full((self.n_layers, rows, self.cap), -1, **i32)
        self.load_blocks = torch.full((self.n_layers, rows, self.cap), -1, **i32)
        self.load_count = torch.zeros((self.n_layers, rows), **i32)
        self.miss_idxs = torch.full((self.n_layers, rows, self.topk_stride), -1, **i32)
        self.miss_count = torch.zeros((self.n_layers, rows), **i32)
        self._free_rows = list(range(rows - 1, -1, -1))
        self._row_of: Dict[int, int] = {}
        self._blocks: Dict[int, List[int]] = {}          # host mirror of map_block rows (block ids never change on the device)
        self._topk: Optional[torch.Tensor] = None
        self._topk_width = 0
        self._step = 0
        self._done: Optional[torch.cuda.Event] = None
        self._status = True
        self._run_rows: List[int] = []
        self._run_dev = None

    # ---- block maps ---------------------------------------------------------------------------------
    def set_blocks_map(self, req_id: int, block_table_list: List[int], select_index: List[int]) -> None:
        """Resident blocks of a request: cache block block_table_list[idx] holds logical block idx, for every idx of
        select_index, in every layer (kvcache_pre.cpp:136-153)."""
        if len(select_index) > self.cap:
            raise ValueError(f"more than {self.cap} resident blocks per request")
        row = self._row_of.get(req_id)
        if row is None:
            if not self._free_rows:
                raise RuntimeError("GSAPrefetchEngineC: no free request row")
            row = self._free_rows.pop()
            self._row_of[req_id] = row
        # the reference's maps keep the LAST idx written for a block id and every idx's block: a block named twice
        # would leave them inconsistent, so it is refused here
        blocks = [int(block_table_list[i]) for i in select_index]
        if len(set(blocks)) != len(blocks):
            raise ValueError("a cache block may hold one logical block")
        self._blocks[req_id] = blocks
        n = len(blocks)
        host = torch.tensor([blocks, [int(i) for i in select_index]], dtype=torch.int32).to(self.device)
        self.map_block[row].fill_(-1)
        self.map_idx[:, row].fill_(-1)
        if n:
            self.map_block[row, :n] = host[0]
            self.map_idx[:, row, :n] = host[1]
        self.map_len[row] = n

    def add_blocks_map(self, req_id: int, idx: int, block_id: int) -> None:
        """One more resident block (a block the request grew by), in every layer (kvcache_pre.cpp:155-173)."""
        if req_id not in self._row_of:
            self.set_blocks_map(req_id, {idx: block_id}, [idx])
            return
        row, blocks = self._row_of[req_id], self._blocks[req_id]
        if block_id in blocks:
            pos = blocks.index(block_id)
        else:
            if len(blocks) >= self.cap:
                raise ValueError(f"more than {self.cap} resident blocks per request")
            pos = len(blocks)
            blocks.append(int(block_id))
            self.map_block[row, pos] = int(block_id)
            self.map_len[row] = len(blocks)
        self.map_idx[:, row, pos] = int(idx)

    def del_blocks_map(self, req_id: int) -> None:
        row = self._row_of.pop(req_id, None)
        if row is not None:
            self._blocks.pop(req_id, None)
            self.map_len[row] = 0
            self._free_rows.append(row)

    # ---- one prefetch round ---------------------------------------------------------------------------
    def set_blocks_table_info(self, block_tables: torch.Tensor, block_lengths: torch.Tensor, input_topk_buf: torch.Tensor,
                              step: int) -> None:
        """The tables this round writes and the selections it reads ([layers, batch, >= topk] logical block
        indices, int32 or int64; copied, as the reference clones them, kvcache_pre.cpp:358-366)."""
        self.success_blocks, self.success_len = block_tables, block_lengths
        width = min(input_topk_buf.shape[2], self.topk_stride)
        topk = torch.zeros((self.n_layers, input_topk_buf.shape[1], self.topk_stride), dtype=torch.int32, device=self.device)
        topk[:, :, :width] = input_topk_buf[:, :, :width].to(device=self.device, dtype=torch.int32)
        self._topk = topk
        self._topk_width = width
        self._step = step

    def run_async_prefetch_bs(self, req_ids: List[int], topk_lens: List[int], bs_indexes: List[int], rank: int = 0) -> None:
        """Hit / miss / free-list round for the listed requests (request i reads selection row i of the buffer and
        owns batch slot bs_indexes[i]); asynchronous on the current stream."""
        if self._topk is None:
            raise RuntimeError("set_blocks_table_info must be called before run_async_prefetch_bs")
        if len(req_ids) > self.max_bs:
            raise RuntimeError(f"batch of {len(req_ids)} requests exceeds max_bs {self.max_bs}")
        rows = [self._row_of.get(int(r), -1) for r in req_ids]       # unknown requests are skipped by the kernel
        if self._topk.shape[1] < len(req_ids):
            raise ValueError("selection buffer has fewer rows than requests")
        if max((int(k) for k in topk_lens), default=0) > min(self.topk_stride, self._topk_width):
            raise ValueError(f"a selection of more than {min(self.topk_stride, self._topk_width)} blocks: the engine holds "
                             f"{self.topk_stride} per request and the buffer of this round {self._topk_width}")
        meta = torch.tensor([rows, [int(k) for k in topk_lens], [int(b) for b in bs_indexes]], dtype=torch.int32).pin_memory()
        meta_d = meta.to(self.device, non_blocking=True)
        topk = self._topk[:, : len(req_ids)].contiguous()
        self._status = False
        ops.prefetch_plan(self.map_block, self.map_len, self.map_idx, topk, meta_d[1], meta_d[0], meta_d[2],
                          self.free_block, self.free_block_len, self.success_blocks, self.success_len, self.load_blocks,
                          self.load_count, self.miss_idxs, self.miss_count)
        self._done = torch.cuda.Event()
        self._done.record()
        self._run_rows, self._run_dev = rows, (meta, meta_d, topk)

    def get_prefetch_status(self) -> bool:
        if not self._status and self._done is not None and self._done.query():
            self._status = True
        return self._status

    def set_prefetch_status(self, flag: bool) -> None:
        self._status = bool(flag)

    # ---- results -----------------------------------------------------------------------------------------
    def _per_request(self, table: torch.Tensor, count: torch.Tensor) -> List[List[List[int]]]:
        if self._done is not None:
            self._done.synchronize()
        t, c = table.cpu(), count.cpu()
        out = []
        for row in self._run_rows:
            out.append([[] if row < 0 else t[l, row, : int(c[l, row])].tolist() for l in range(self.n_layers)])
        return out

    def obtain_load_blocks(self) -> List[List[List[int]]]:
        """[request of the last round][layer] -> cache blocks that receive a load, in order."""
        return self._per_request(self.load_blocks, self.load_count)

    def obtain_miss_idxs(self) -> List[List[List[int]]]:
        """[request of the last round][layer] -> every missed logical block, in selection order; the first
        len(load blocks) of them are the ones that are loaded."""
        return self._per_request(self.miss_idxs, self.miss_count)

    def obtain_blocks_map(self) -> Dict[int, List[Dict[int, int]]]:
        """request id -> per layer {cache block: logical block it holds}."""
        if self._done is not None:
            self._done.synchronize()
        idx = self.map_idx.cpu()
        return {req: [dict(zip(self._blocks[req], idx[l, row, : len(self._blocks[req])].tolist()))
                      for l in range(self.n_layers)] for req, row in self._row_of.items()}

    # ---- device-side consumers ----------------------------------------------------------------------------
    def row_of(self, req_id: int) -> int:
        """Row of the engine's tables (and of load_missing's src_table) that holds the request, -1 if unknown."""
        return self._row_of.get(int(req_id), -1)

    def run_rows_device(self) -> torch.Tensor:
        """Table rows of the last round's requests (int32 device tensor; -1 for requests the engine does not know)."""
        return self._run_dev[1][0]

    def load_missing(self, layers: ops.LayerPointers, kv_stride: int, block_bytes: int, num_blocks: int,
                     pool: torch.Tensor, pool_block_bytes: int, src_table: torch.Tensor) -> None:
        """Loads the last round's served misses of every layer: stored block src_table[row][logical block] of the pool
        ([block][layer][K|V], device or pinned host memory) goes into the cache block the round chose for it - the
        reference's connector.load of block hashes into all_need_load_block (ucm/sparse/gsa/gsa.py:835-866), as one
        launch on the current stream.  src_table int32 [rows, M] is the caller's hash -> pool lookup, done once per
        request."""
        ops.kv_load_planned(layers, 0, 0, self.n_layers, kv_stride, block_bytes, num_blocks, pool, pool_block_bytes,
                            self.miss_idxs, src_table, self.load_blocks, self.run_rows_device(), load_count=self.load_count)
