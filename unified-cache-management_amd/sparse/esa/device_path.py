"""Batched, device-resident decode path of the ESA plugin.

The reference drives retrieval and loads one request and one layer at a time
(ucm/sparse/esa/esa.py:286-339): a ``submit`` with the request's slot list, a
``wait`` + ``get_result`` on the host, Python set arithmetic for the delta
against ``pre_topk_block_hashes``, and one ``store.load`` per K and V with a
tensor view per block.  When the store's blocks are device-addressable
(``UcmHipBlockStore``) none of that needs the host:

* every live request owns a ROW of a few persistent device tables - its slot
  list per layer (``ReqStatePerLayer.slots``), its k, the pool block of each of
  its stored blocks (the hash -> store lookup, done once), the cache blocks of
  its first ``top_k`` vLLM blocks, and per layer what those blocks hold
  (``pre_topk_block_hashes``);
* a layer's hook issues ONE ``ucm_esa_retrieve_rows`` for all requests that
  retrieve in this step, ONE ``ucm_delta_plan_rows`` for all that load, and the
  last layer's hook ONE ``ucm_kv_load_planned`` that moves the missing blocks of
  all layers from the pool into the cache;
* per step the host uploads one small descriptor (which rows retrieve, which
  load, where their query token sits) from pinned memory.

The state machine over ``step % retrieval_stride`` is the reference's.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from ... import _lib, ops
from ..utils import HeldBlocks


@dataclass
class DeviceRequest:
    """Host-side record of one request in the device tables."""
    row: int
    block_hashes: List[str]
    sparse_range: int
    top_k: int
    slots: List[List[int]] = field(default_factory=list)      # per layer, for the pools
    n_repre: int = 0                                          # representatives written (blocks)
    pending: bool = False                                     # a retrieval waits to be turned into loads
    dst_ids: tuple = ()                                       # cache blocks of the first top_k vLLM blocks, as uploaded
    src_ready: bool = False                                   # every block of the sparse range was found in the store
    src_missing: int = 0                                      # how many were not, at the last look
    skipped: bool = False                                     # a load ran while some were missing
    held: Optional[HeldBlocks] = None                         # its stored blocks stay in the store's pool while it lives


class StepPlan:
    """What one engine step does, as device index arrays (one upload)."""

    def __init__(self):
        self.first_rows = self.first_qpos = None      # step == 1: retrieve + plan + load before the layer's attention
        self.retrieve_rows = self.retrieve_qpos = None
        self.load_rows = None
        self.n_first = self.n_retrieve = self.n_load = 0
        self.m_first = self.m_retrieve = 0            # longest slot list among the rows
        self.prefill = None                           # (ids_dev [n], slots_dev [L, n]) of requests ending prefill


class EsaDeviceTables:
    def __init__(self, n_layers: int, max_rows: int, max_blocks: int, max_slots: int, device):
        i32 = dict(dtype=torch.int32, device=device)
        self.n_layers, self.max_rows, self.max_blocks, self.max_slots = n_layers, max_rows, max_blocks, max_slots
        self.slot_table = torch.full((n_layers, max_rows, max_blocks), -1, **i32)
        self.topk_rows = torch.zeros(max_rows, **i32)
        self.out_idx = torch.full((n_layers, max_rows, max_slots), -1, **i32)
        self.out_pos = torch.full((n_layers, max_rows, max_slots), -1, **i32)
        self.out_scores = torch.zeros((n_layers, max_rows, max_slots), dtype=torch.float32, device=device)
        self.out_count = torch.zeros((n_layers, max_rows), **i32)
        self.resident = torch.full((n_layers, max_rows, max_slots), -1, **i32)
        self.load_sel = torch.full((n_layers, max_rows, max_slots), -1, **i32)
        self.slot_of_sel = torch.full((n_layers, max_rows, max_slots), -1, **i32)
        self.miss_count = torch.zeros((n_layers, max_rows), **i32)
        self.src_table = torch.full((max_rows, max_blocks), -1, **i32)
        self.dst_table = torch.full((max_rows, max_slots), -1, **i32)
        self.scores_ws = torch.empty(max_rows * max_blocks, dtype=torch.float32, device=device)
        self.free_rows = list(range(max_rows - 1, -1, -1))
        self.device = device

    def allocate_row(self) -> int:
        if not self.free_rows:
            raise RuntimeError("ESA device tables: more live requests than max_num_seqs rows")
        row = self.free_rows.pop()
        self.slot_table[:, row].fill_(-1)
        self.resident[:, row].fill_(-1)
        self.out_count[:, row].zero_()
        self.src_table[row].fill_(-1)
        self.dst_table[row].fill_(-1)
        return row

    def release_row(self, row: int) -> None:
        self.free_rows.append(row)

    def upload(self, parts: List[List[int]]) -> List[Optional[torch.Tensor]]:
        """The integer lists side by side in one device tensor, sent in one copy (pinned staging whose reuse waits
        for the copy that last read it); returns a view per list, None for an empty one."""
        flat = [x for p in parts for x in p]
        if not flat:
            return [None] * len(parts)
        dev = ops.upload(torch.tensor(flat, dtype=torch.int32), self.device)
        views, pos = [], 0
        for p in parts:
            views.append(dev[pos : pos + len(p)] if p else None)
            pos += len(p)
        return views


class EsaDevicePath:
    """Owns the tables and runs the batched hooks for an ``ESA`` plugin instance."""

    def __init__(self, esa, pool: torch.Tensor, pool_block_bytes: int, device):
        self.esa = esa
        self.pool, self.pool_block_bytes = pool, pool_block_bytes
        max_blocks = max(esa.max_model_len // esa.block_size, 1)
        max_slots = max(int(max_blocks * esa.esa_cfg["sparse_ratio"]), 1)
        if max_slots > 1024:
            raise ValueError("ESA device path: more than 1024 sparse slots per request")
        self.tables = EsaDeviceTables(esa.total_num_hidden_layers, esa.max_num_seqs, max_blocks, max_slots, device)
        self.reqs: Dict[object, DeviceRequest] = {}
        self.plan = StepPlan()
        self.kv_caches: List[Optional[torch.Tensor]] = [None] * esa.total_num_hidden_layers
        self._kv_one: List[Optional[ops.LayerPointers]] = [None] * esa.total_num_hidden_layers
        self._kv_all: Optional[ops.LayerPointers] = None
        self.device = device
        # a layer's retrieval and plan go to the library with addresses taken once: the tables are this object's own,
        # and slicing and re-validating a dozen tensors per layer and step took twice the time of the calls themselves
        self._retr_const: List[Optional[tuple]] = [None] * esa.total_num_hidden_layers
        self._plan_const: List[Optional[tuple]] = [None] * esa.total_num_hidden_layers

    # ---- caches ----------------------------------------------------------------------------
    def register_kv_cache(self, layer_id: int, kv_cache: torch.Tensor) -> None:
        cur = self.kv_caches[layer_id]
        if cur is not None and cur.data_ptr() == kv_cache.data_ptr():
            return
        self.kv_caches[layer_id] = kv_cache
        self._kv_one[layer_id] = ops.LayerPointers([kv_cache])
        self._kv_all = None
        if all(c is not None for c in self.kv_caches):
            self._kv_all = ops.LayerPointers(self.kv_caches)

    def _geometry(self, layer_id: int):
        kv = self.kv_caches[layer_id]
        return kv.stride(0) * kv.element_size(), kv.stride(1) * kv.element_size(), kv.shape[1]

    # ---- per step ----------------------------------------------------------------------------
    def build_step(self, metas) -> None:
        """metas: the step's ReqMeta list (sparsified requests only).  Decides what every request does in this
        step (esa.py:366-399) and uploads the index arrays."""
        esa, t = self.esa, self.tables
        stride = esa.esa_cfg["retrieval_stride"]
        wait = getattr(esa.connector, "wait_for_writes", None)
        if wait is not None:
            wait()                       # blocks dumped through the store's stream are read in place by this step's loads
        first, first_q, retr, retr_q, load = [], [], [], [], []
        m_first = m_retr = 0
        prefill = []
        for meta in metas:
            st = self.reqs.get(meta.request_id)
            if st is None:
                st = self._new_request(meta)
            if meta.is_prefill:
                if meta.is_last_chunk and st.n_repre == 0 and st.sparse_range > 0:
                    prefill.append((st, meta))
                continue
            step = meta.step
            if step == 0 or st.n_repre == 0 or st.top_k <= 0:
                continue
            if not st.src_ready:
                self._upload_sources(st)
            ids = tuple(meta.vllm_block_ids[: st.top_k])
            if ids != st.dst_ids:
                t.dst_table[st.row, : len(ids)] = torch.tensor(ids, dtype=torch.int32, device=self.device)
                st.dst_ids = ids
            if st.src_missing and (step == 1 or (step % stride == 0 and st.pending)):
                esa._report_missing(st.src_missing)
                st.skipped = True
            if step == 1:
                first.append(st.row)
                first_q.append(meta.query_start_loc)
                m_first = max(m_first, st.n_repre)
                st.pending = False
                continue
            if step % stride == 2 % stride:
                retr.append(st.row)
                retr_q.append(meta.query_start_loc)
                m_retr = max(m_retr, st.n_repre)
                st.pending = True
            if step % stride == 0 and st.pending:
                load.append(st.row)
                st.pending = False
        p = StepPlan()
        p.n_first, p.n_retrieve, p.n_load = len(first), len(retr), len(load)
        p.m_first, p.m_retrieve = m_first, m_retr
        if first or retr or load:
            p.first_rows, p.first_qpos, p.retrieve_rows, p.retrieve_qpos, p.load_rows = t.upload(
                [first, first_q, retr, retr_q, load])
        if prefill:
            p.prefill = self._allocate_repre(prefill)
        self.plan = p

    def _new_request(self, meta) -> DeviceRequest:
        esa = self.esa
        n, local = meta.num_prompt_tokens, esa.esa_cfg["local_window_sz"]
        sparse_range = n // esa.block_size - (local if n % esa.block_size == 0 else local - 1)
        sparse_range = max(sparse_range, 0)
        top_k = int(sparse_range * esa.esa_cfg["sparse_ratio"])
        row = self.tables.allocate_row()
        self.tables.topk_rows[row] = top_k
        st = DeviceRequest(row=row, block_hashes=esa.prompt_block_hashes(meta.prompt_token_ids), sparse_range=sparse_range,
                           top_k=top_k)
        self.reqs[meta.request_id] = st
        return st

    def _upload_sources(self, st: DeviceRequest) -> None:
        """hash -> pool block of the request's sparse range (esa.py:306-310 looks hashes up per retrieval): once, when
        the store holds them all; otherwise again at every step until it does.  A load that ran in between left the
        missing blocks out while the plan counted them as present, so once more of them are found the request's
        resident lists are forgotten and its next load brings in everything it selects."""
        if st.held is None:
            st.held = HeldBlocks(self.esa.connector)
        src = st.held.slots(st.block_hashes[: st.sparse_range])
        missing = src.count(-1)
        if src:
            self.tables.src_table[st.row, : len(src)] = ops.upload(torch.tensor(src, dtype=torch.int32), self.device)
        if st.skipped and missing < st.src_missing:
            self.tables.resident[:, st.row].fill_(-1)
            st.skipped = False
        st.src_missing, st.src_ready = missing, missing == 0

    def _allocate_repre(self, prefill):
        """Rows of every layer's table for the requests that finish their prefill in this step
        (block_repre_data, esa.py:353-364); the means themselves are taken layer by layer in attention_finished."""
        esa, t = self.esa, self.tables
        ids, per_layer = [], [[] for _ in range(t.n_layers)]
        for st, meta in prefill:
            blk = meta.vllm_block_ids[: st.sparse_range]
            n = len(blk)
            ids.extend(blk)
            st.slots = []
            for l in range(t.n_layers):
                got = esa.layer_pools[l].allocate(n)
                st.slots.append(got)
                per_layer[l].extend(got)
            st.n_repre = n
        ids_dev = torch.tensor(ids, dtype=torch.int32, device=self.device)
        slots_dev = torch.tensor(per_layer, dtype=torch.int32, device=self.device)
        pos = 0
        for st, _ in prefill:
            t.slot_table[:, st.row, : st.n_repre] = slots_dev[:, pos : pos + st.n_repre]
            pos += st.n_repre
        return ids_dev, slots_dev

    # ---- hooks ----------------------------------------------------------------------------------
    def _queries(self, query: torch.Tensor, qpos: torch.Tensor) -> torch.Tensor:
        """The group-mean query of every request of the call, flattened, fp32 (esa.py:286-296: the mean is taken in
        the model dtype, the worker widens it)."""
        esa = self.esa
        q = query.index_select(0, qpos)
        b, hq, _ = q.shape
        if hq > esa.num_key_heads:
            q = q.view(b, esa.num_key_heads, -1, esa.head_size).mean(2)
        elif hq < esa.num_key_heads:
            q = torch.repeat_interleave(q, esa.num_key_heads // hq, 1)
        return q.reshape(b, -1).to(torch.float32)

    def _retrieve(self, layer_id: int, query: torch.Tensor, rows: torch.Tensor, qpos: torch.Tensor, m: int) -> None:
        t = self.tables
        q = self._queries(query, qpos)
        table = self.esa.data                                # [layers, slots, dim]
        c = self._retr_const[layer_id]
        if c is None or c[0] is not table:                   # first call of a layer: through the checked wrapper
            data = table[layer_id]
            ops.esa_retrieve_rows(data, q, t.slot_table[layer_id], m, rows, t.topk_rows, t.max_slots, t.scores_ws,
                                  t.out_idx[layer_id], t.out_pos[layer_id], t.out_scores[layer_id], t.out_count[layer_id])
            self._retr_const[layer_id] = (table, data.data_ptr(), data.shape[0], data.shape[1], t.slot_table[layer_id].data_ptr(),
                                          t.max_rows, t.max_blocks, t.topk_rows.data_ptr(), t.max_slots, t.scores_ws.data_ptr(),
                                          t.out_idx[layer_id].data_ptr(), t.out_pos[layer_id].data_ptr(),
                                          t.out_scores[layer_id].data_ptr(), t.out_count[layer_id].data_ptr())
            return
        batch = rows.numel()
        if m > c[6] or batch > c[5] or q.shape != (batch, c[3]) or q.dtype is not torch.float32 or not q.is_contiguous() \
                or rows.dtype is not torch.int32 or not rows.is_cuda:
            raise ValueError("ESA device path: queries or rows do not fit the tables")
        rc = _lib.lib().ucm_esa_retrieve_rows(c[1], c[2], c[3], q.data_ptr(), c[4], c[5], c[6], m, rows.data_ptr(), batch, c[7],
                                             c[8], c[9], c[10], c[11], c[12], c[13], c[8], ops.current_stream())
        if rc != 0:
            raise _lib.UcmHipError("ucm_esa_retrieve_rows", rc, _lib.lib().ucm_last_error().decode())

    def _plan(self, layer_id: int, rows: torch.Tensor) -> None:
        t, l = self.tables, slice(layer_id, layer_id + 1)
        c = self._plan_const[layer_id]
        if c is None:
            ops.delta_plan_rows(t.out_pos[l], t.out_pos[l], t.out_count[l], rows, t.resident[l], t.load_sel[l],
                                t.slot_of_sel[l], t.miss_count[l])
            self._plan_const[layer_id] = (t.out_pos[l].data_ptr(), t.out_count[l].data_ptr(), t.resident[l].data_ptr(),
                                          t.load_sel[l].data_ptr(), t.slot_of_sel[l].data_ptr(), t.miss_count[l].data_ptr())
            return
        if rows.numel() > t.max_rows or rows.dtype is not torch.int32 or not rows.is_cuda:
            raise ValueError("ESA device path: rows do not fit the tables")
        rc = _lib.lib().ucm_delta_plan_rows(c[0], c[0], c[1], rows.data_ptr(), rows.numel(), t.max_rows, 1, t.max_slots, c[2],
                                           t.max_slots, c[3], c[4], c[5], ops.current_stream())
        if rc != 0:
            raise _lib.UcmHipError("ucm_delta_plan_rows", rc, _lib.lib().ucm_last_error().decode())

    def _load(self, first_layer: int, n_layers: int, rows: torch.Tensor) -> None:
        t = self.tables
        kv_stride, block_bytes, num_blocks = self._geometry(first_layer)
        ptrs, base = (self._kv_all, first_layer) if self._kv_all is not None else (self._kv_one[first_layer], 0)
        if self._kv_all is None and n_layers != 1:
            raise RuntimeError("ESA device path: not every layer's cache is registered")
        ops.kv_load_planned(ptrs, base, first_layer, n_layers, kv_stride, block_bytes, num_blocks, self.pool,
                            self.pool_block_bytes, t.load_sel[first_layer : first_layer + n_layers], t.src_table,
                            t.dst_table, rows)

    def attention_begin(self, layer_id: int, query: torch.Tensor) -> None:
        p = self.plan
        if p.n_first:   # step 1: retrieval and loads happen before this layer's attention (esa.py:372-377)
            self._retrieve(layer_id, query, p.first_rows, p.first_qpos, p.m_first)
            self._plan(layer_id, p.first_rows)
            self._load(layer_id, 1, p.first_rows)

    def attention_finished(self, layer_id: int, query: torch.Tensor) -> None:
        p, esa = self.plan, self.esa
        if p.prefill is not None:
            ids_dev, slots_dev = p.prefill
            ops.block_mean(esa._layer_ptrs[layer_id], ids_dev, slots_dev[layer_id], esa.data[layer_id : layer_id + 1],
                           esa.block_size, esa.num_key_heads, esa.head_size, esa._num_blocks[layer_id],
                           mode=ops.MEAN_BF16_ROUND)
        if p.n_retrieve:
            self._retrieve(layer_id, query, p.retrieve_rows, p.retrieve_qpos, p.m_retrieve)
        if p.n_load:
            self._plan(layer_id, p.load_rows)
            if self._kv_all is None:
                self._load(layer_id, 1, p.load_rows)
            elif layer_id == self.tables.n_layers - 1:
                self._load(0, self.tables.n_layers, p.load_rows)   # the missing blocks of all layers in one launch

    def request_finished(self, request_id) -> None:
        st = self.reqs.pop(request_id, None)
        if st is None:
            return
        for l, slots in enumerate(st.slots):
            self.esa.layer_pools[l].free(slots)
        if st.held is not None:
            st.held.release()
        self.tables.release_row(st.row)
