"""KVStar's decode steps for all requests of a layer at once.

The reference walks its requests one by one in every layer hook (ucm/sparse/kvstar/multistep.py:693-760): a clone
of the step's query token per request and layer, a retrieval task per request and layer every ``retrieval_stride``
steps, a ``store.load`` pair per request and layer one stride later.  On the device none of that needs a request
at a time, and most steps need nothing but the clone.  Here a layer hook of a decode step issues

* ONE launch that copies the step's query tokens of all requests aside, as fp16, into the layer's ring of query
  groups (``ucm_kvstar_park_queries``; the index arrays are the same for every layer and go down once per step),
* on the steps in which requests complete a group: ONE votes / selection / order launch triple on the side stream
  for all of them (``ucm_kvstar_votes_tables`` reads the groups straight from the ring),
* on the steps in which a stride's winners are due: ONE ``ucm_kv_load_planned`` that follows the lists on the
  device, after the side stream's event.

Everything that does not change between two retrievals of the same requests - the pointer arrays of their
representative tables, their channel lists, the segment descriptors, the tables that turn a list entry into a stored
block and a list position into a cache block - is built once per set of requests and kept.  The per-request,
per-layer state objects of the reference stay what they are for everybody who looks at them (``block_hashes``,
``blk_repre``, ``task_waiter``, ``step_group_retrieve_result`` ...), but no decode step calls into them.

The schedule over ``step % retrieval_stride`` is the reference's (multistep.py:365-387, 503-521).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ... import _lib, ops
from ...sparse.utils import HeldBlocks
from . import retrieve as kvstar_retrieve

_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_Q_CODES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16}


class _Batch:
    """What the requests of one retrieval (or one load) share in every layer; built once per set of requests."""

    def __init__(self, members, topks, device):
        self.states = [states for _, states, _ in members]          # per request: its per-layer state objects
        states0 = [states[0] for states in self.states]
        lens = [int(st.blk_repre.shape[0]) for st in states0]
        offs = [0]
        for n in lens[:-1]:
            offs.append(offs[-1] + n)
        self.n = len(lens)
        self.lens, self.total, self.longest = lens, sum(lens), max(lens)
        self.topks = [min(int(k), n) for k, n in zip(topks, lens)]
        self.meta = ops.upload(torch.tensor([offs, lens, self.topks], dtype=torch.int32), device)   # seg_off, seg_len, topk
        self.per_layer: Dict[int, tuple] = {}
        self.src_table: Optional[torch.Tensor] = None
        self.src_complete = False
        self.dst_table: Optional[torch.Tensor] = None
        self.dst_host = torch.full((self.n, max(self.longest, 1)), -1, dtype=torch.int32)
        self.dst_rows: List[Optional[tuple]] = [None] * self.n
        self.launched: Dict[tuple, tuple] = {}             # (record, layer) -> (results, task ids) of a launch not yet loaded
        self.loaded: Dict[int, list] = {}                  # layer -> task ids of the launch whose lists were loaded last


class KVStarLayerPath:
    def __init__(self, plugin, device):
        self.plugin = plugin
        self.device = device
        cfg = plugin.kvstar_multistep_cfg
        self.stride = int(cfg["retrieval_stride"])
        self.rows: Dict[object, int] = {}
        self.free_rows: List[int] = []
        self.n_rows = 0
        self.rings: Dict[int, torch.Tensor] = {}          # layer -> fp16 [rows, 2 groups, stride, q_heads * head_dim]
        self.row_elems = 0
        self.batches: Dict[tuple, _Batch] = {}
        self.held: Dict[object, HeldBlocks] = {}           # per request: its stored blocks stay in the store's pool
        self.step: dict = {}
        self.side = None
        self.reading: Dict[int, object] = {}               # layer -> event of the side stream's last launch that reads its ring
        self._dev_index = 0

    # ---- rows of the rings ------------------------------------------------------------------------------------
    def _row_of(self, request_id) -> int:
        row = self.rows.get(request_id)
        if row is None:
            row = self.free_rows.pop() if self.free_rows else self._grow()
            self.rows[request_id] = row
        return row

    def _grow(self) -> int:
        old = self.n_rows
        self.n_rows = max(16, 2 * old)
        self.free_rows.extend(range(self.n_rows - 1, old, -1))
        for l, ring in list(self.rings.items()):           # (rare: more live requests than ever before)
            bigger = torch.zeros((self.n_rows,) + tuple(ring.shape[1:]), dtype=ring.dtype, device=ring.device)
            bigger[:old] = ring
            self.rings[l] = bigger
        return old

    def request_finished(self, request_id) -> None:
        row = self.rows.pop(request_id, None)
        if row is not None:
            self.free_rows.append(row)
        held = self.held.pop(request_id, None)
        if held is not None:
            held.release()
        for key in [k for k in self.batches if request_id in k[0]]:
            del self.batches[key]

    def _ring(self, layer_id: int, query: torch.Tensor) -> torch.Tensor:
        ring = self.rings.get(layer_id)
        if ring is None:
            self.row_elems = query.shape[-2] * query.shape[-1]
            ring = self.rings[layer_id] = torch.zeros((self.n_rows, 2, self.stride, self.row_elems), dtype=torch.float16,
                                                      device=query.device)
        return ring

    # ---- per step ---------------------------------------------------------------------------------------------
    def build_step(self, metadata, ReqStage) -> None:
        """Decides what this step does for every request (the same in every layer) and uploads the index arrays."""
        stride, plugin = self.stride, self.plugin
        park_src: List[int] = []
        park_at: List[tuple] = []                          # (row, group plane, place)
        queue, first, load, ending = [], [], [], []
        for meta in metadata.requests:
            row = self._row_of(meta.request_id)
            if meta.stage == ReqStage.PREFILL:
                places = meta.query_offload_info
                if places:
                    start = meta.query_start_loc + meta.query_len - len(places)
                    for rel, place in enumerate(places):
                        park_src.append(start + rel)
                        park_at.append((row, 0, place))
                if meta.is_last_chunk:
                    ending.append(meta)
                continue
            states = plugin.req_states.get(meta.request_id)
            if not states or states[0] is None or states[0].blk_repre is None:
                continue
            step = meta.step
            plane = (1 + (step - 1) // stride) % 2          # the prefill group lives in plane 0, decode groups alternate
            park_src.append(meta.query_start_loc)
            park_at.append((row, plane, (step - 1) % stride))
            member = (meta, states, row)
            if step % stride == 0:
                queue.append((member, "decode" + str(step + 1 - stride), plane, stride))
            if step == 1:
                first.append((member, "prefill", 0, min(stride, meta.num_prompt_tokens)))
            if step >= 2 * stride and step % stride == 0:
                load.append((member, "decode" + str((int(math.ceil((step + 1) / stride)) - 3) * stride + 1)))
        self.step = {"n_park": len(park_src), "park_src": park_src, "park_at": park_at, "queue": queue, "first": first,
                     "load": load, "ending": ending, "cache": {}, "owner": metadata}

    def _park_arrays(self):
        st = self.step
        found = st["cache"].get("park")
        if found is None:
            per_group = self.stride * self.row_elems
            dst = [((row * 2 + plane) * self.stride + place) * self.row_elems for row, plane, place in st["park_at"]]
            both = ops.upload(torch.tensor([st["park_src"], dst], dtype=torch.int64), self.device)
            found = st["cache"]["park"] = (both[0].to(torch.int32), both[1], per_group)
        return found

    # ---- hooks ------------------------------------------------------------------------------------------------
    def attention_begin(self, layer_id: int, layer_name: str, query: torch.Tensor, forward_context) -> None:
        st = self.step
        if self.device is None:
            self.device = query.device
            self._dev_index = query.device.index if query.device.index is not None else torch.cuda.current_device()
        busy = self.reading.pop(layer_id, None)
        if busy is not None:
            # the side stream's last votes launch of this layer reads the ring; it was queued at least a step ago
            torch.cuda.current_stream().wait_event(busy)
        if st["n_park"]:
            ring = self._ring(layer_id, query)
            src, dst, _ = self._park_arrays()
            code = _Q_CODES.get(query.dtype)
            if code is None or not query.is_contiguous():
                raise ValueError("query must be a contiguous bfloat16, float16 or float32 tensor")
            _lib.call("ucm_kvstar_park_queries", query.data_ptr(), code, query.shape[0], self.row_elems, src.data_ptr(),
                      dst.data_ptr(), st["n_park"], ring.data_ptr(), ring.numel(), self._stream())
        if st["first"]:
            # first decode step: windows back in place, the prefill group's votes, and their winners loaded right away
            sink = []
            for (meta, states, _), _, _, _ in st["first"]:
                states[layer_id].req_meta = meta
                sink.append((states[layer_id], "restore"))
            self.plugin._flush_windows(sink, layer_name, forward_context)
        if st["queue"]:
            self._retrieve("queue", st["queue"], layer_id, query)
        if st["first"]:
            self._retrieve("first", st["first"], layer_id, query)
            self._load("first", [(member, record) for member, record, _, _ in st["first"]], layer_id, layer_name, forward_context)

    def attention_finished(self, layer_id: int, layer_name: str, forward_context) -> None:
        if self.step["load"]:
            self._load("due", self.step["load"], layer_id, layer_name, forward_context)

    def _stream(self) -> int:
        return _raw_stream(self._dev_index) if _raw_stream is not None else ops.current_stream()

    # ---- retrieval --------------------------------------------------------------------------------------------
    def _candidates(self, meta, state) -> List[int]:
        n_keep = math.ceil(state.blk_repre.shape[0] * state.sparse_cfg["sparse_ratio"])
        return meta.vllm_block_ids[state.init_window_sz : n_keep + state.init_window_sz]

    def _batch(self, members, x: int) -> _Batch:
        key = (tuple(meta.request_id for meta, _, _ in members), x)
        batch = self.batches.get(key)
        if batch is None:
            topks = [len(self._candidates(meta, states[0])) for meta, states, _ in members]
            batch = self.batches[key] = _Batch(members, topks, self.device)
        return batch

    def _retrieve(self, which: str, entries, layer_id: int, query: torch.Tensor) -> None:
        """One votes / selection / order launch triple on the side stream for the requests that complete a query
        group in this step (retrieval_async per request in the reference, multistep.py:240-268)."""
        cache = self.step["cache"]
        groups = cache.get(which)
        if groups is None:                                  # the same for every layer
            groups = cache[which] = []
            by_x: Dict[tuple, list] = {}
            for member, record, plane, x in entries:
                meta, states, row = member
                if len(self._candidates(meta, states[0])) == 0:
                    for st in states:                       # nothing to choose from: the record is an empty list
                        dict.__setitem__(st.step_group_retrieve_result, record, [])
                        dict.__setitem__(st.step_group_retrieve_indices, record, [])
                    continue
                by_x.setdefault((x, record), []).append((member, record, plane))      # one launch per group record
            for (x, _), part in by_x.items():
                batch = self._batch([m for m, _, _ in part], x)
                per_group = self.stride * self.row_elems
                q_off = [(row * 2 + plane) * per_group + (self.stride - x) * self.row_elems for (_, _, row), _, plane in part]
                groups.append((batch, part, x, ops.upload(torch.tensor(q_off, dtype=torch.int64), self.device)))
        if self.side is None:
            self.side = torch.cuda.Stream()                 # default priority
        for batch, part, x, q_off in groups:
            self._launch(batch, part, x, q_off, layer_id, query)

    def _layer_tables(self, batch: _Batch, part, layer_id: int):
        found = batch.per_layer.get(layer_id)
        if found is None:
            states = [member[1][layer_id] for member, _, _ in part]
            tables = [st.blk_repre.table for st in states]
            kv_heads, _, pieces, m, _ = tables[0].shape
            strides = [ops._kvstar_cell_strides(t, "table") for t in tables]
            row_strides = {rs for t, (_, rs) in zip(tables, strides) if t.shape[1] > 1}
            if len(row_strides) > 1:
                raise ValueError("the representative tables of one layer must share a row stride")
            row_stride = row_strides.pop() if row_strides else pieces * m * 8
            ptrs = ops.upload(torch.tensor([[t.data_ptr() for t in tables], [hs for hs, _ in strides]], dtype=torch.int64), self.device)
            pruned = sel = None
            if states[0].d_pruned_index is not None:
                pruned = torch.stack([st.d_pruned_index32 for st in states]).contiguous()
                sel = torch.arange(batch.n, dtype=torch.int32, device=self.device)
            d_pruned = states[0].blk_repre.d_pruned
            found = batch.per_layer[layer_id] = dict(
                ptrs=ptrs, row_stride=row_stride, pruned=pruned, sel=sel, m=m, kv_heads=kv_heads, d_pad=pieces * 8,
                d_pruned=d_pruned, votes=torch.zeros(max(batch.total, 1), dtype=torch.float32, device=self.device), ws={},
                keep=tables)
        return found

    def _launch(self, batch: _Batch, part, x: int, q_off: torch.Tensor, layer_id: int, query: torch.Tensor) -> None:
        lt = self._layer_tables(batch, part, layer_id)
        ring = self.rings[layer_id]
        hq, d_orig = query.shape[-2], query.shape[-1]
        ws = lt["ws"].get(x)
        if ws is None:
            ws = lt["ws"][x] = ops.kvstar_workspace(batch.n, lt["kv_heads"], x * (hq // lt["kv_heads"]), batch.longest, lt["m"],
                                                   lt["d_pad"], self.device)
        idx = torch.empty((batch.n, max(batch.longest, 1)), dtype=torch.int32, device=self.device)
        cnt = torch.empty(batch.n, dtype=torch.int32, device=self.device)
        side = self.side
        idx.record_stream(side)
        cnt.record_stream(side)
        ready = torch.cuda.Event()
        ready.record()
        side.wait_event(ready)
        s = side.cuda_stream
        meta, votes = batch.meta, lt["votes"]
        pruned, sel = lt["pruned"], lt["sel"]
        _lib.call("ucm_kvstar_votes_tables", ring.data_ptr(), ring.numel(), q_off.data_ptr(), x, hq, d_orig,
                  None if pruned is None else pruned.data_ptr(), 0 if pruned is None else pruned.shape[0],
                  None if sel is None else sel.data_ptr(), lt["ptrs"][0].data_ptr(), lt["ptrs"][1].data_ptr(), lt["row_stride"],
                  meta[0].data_ptr(), meta[1].data_ptr(), batch.n, batch.longest, lt["m"], lt["kv_heads"], lt["d_pruned"],
                  lt["d_pad"], ws[0].data_ptr(), ws[0].numel(), ws[1].data_ptr(), ws[1].numel(), votes.data_ptr(), votes.numel(),
                  0, s)
        _lib.call("ucm_kvstar_topk", votes.data_ptr(), votes.numel(), meta[0].data_ptr(), meta[1].data_ptr(), meta[2].data_ptr(),
                  batch.n, batch.longest, idx.data_ptr(), idx.shape[1], cnt.data_ptr(), s)
        _lib.call("ucm_kvstar_order", votes.data_ptr(), votes.numel(), meta[0].data_ptr(), meta[1].data_ptr(), batch.n,
                  batch.longest, idx.data_ptr(), idx.shape[1], cnt.data_ptr(), s)
        done = torch.cuda.Event()
        done.record(side)
        self.reading[layer_id] = done
        results = kvstar_retrieve._Results(done, votes, idx, cnt, (batch, q_off))
        results.batch = batch
        ids = kvstar_retrieve.RegisterBatch(results, batch.n)
        for (member, record, _), task_id in zip(part, ids):
            member[1][layer_id].task_waiter[record] = task_id
        batch.launched[(part[0][1], layer_id)] = (results, ids)

    # ---- loads ------------------------------------------------------------------------------------------------
    def _load(self, which: str, entries, layer_id: int, layer_name: str, forward_context) -> None:
        """The winners of a group into the requests' candidate cache blocks (load_retrieve_result_async per request
        in the reference, multistep.py:410-450): per launch that produced the lists, one kernel follows them.  Which
        launches those are is found through the requests' tasks at the step's first layer; every layer of a step was
        launched for the same requests in the same rows."""
        cache = self.step["cache"]
        plan = cache.get(("load", which))
        if plan is None:
            plan = cache[("load", which)] = []
            groups: Dict[tuple, list] = {}
            for member, record in entries:
                task_id = member[1][layer_id].task_waiter.get(record)
                if task_id is None:                          # (nothing was queued: no candidates)
                    continue
                found = kvstar_retrieve.DeviceResult(task_id)
                if found is None:
                    raise RuntimeError(f"retrieval task {task_id} of layer {layer_id} is not known")
                groups.setdefault((id(found[0].batch), record), []).append((member, found[0].batch, found[1]))
            for (_, record), members in groups.items():
                batch = members[0][1]
                rows = [row for _, _, row in members]
                rows_dev = None if rows == list(range(batch.n)) else ops.upload(torch.tensor(rows, dtype=torch.int32), self.device)
                plan.append((batch, record, members, rows_dev))
        if not plan:
            return
        kv = forward_context.no_compile_layers[layer_name].kv_cache[forward_context.virtual_engine]
        known = self.plugin._layer_ptrs.get(layer_name)
        if known is None or known[0] != kv.data_ptr():
            known = self.plugin._layer_ptrs[layer_name] = (kv.data_ptr(), ops.LayerPointers([kv]))
        es = kv.element_size()
        pool, pool_block_bytes = self.plugin.connector.device_pool()
        stream = torch.cuda.current_stream()
        for batch, record, members, rows_dev in plan:
            launched = batch.launched.pop((record, layer_id), None)
            if launched is None:                             # loaded already
                continue
            results, ids = launched
            src, dst = self._load_tables(batch, members)
            stream.wait_event(results.event)
            ops.kv_load_planned(known[1], 0, layer_id, 1, kv.stride(0) * es, kv.stride(1) * es, kv.shape[1], pool, pool_block_bytes,
                                results.idx.unsqueeze(0), src, dst, rows_dev, load_count=results.cnt.unsqueeze(0))
            # the lists stay readable (step_group_retrieve_result) until the next group's load of this layer
            before = batch.loaded.get(layer_id)
            if before is not None:
                kvstar_retrieve.ForgetBatch(before)
            batch.loaded[layer_id] = ids

    def _load_tables(self, batch: _Batch, members):
        """src: the store's block of every prompt block a request's list can name; dst: the cache block of every list
        position.  Both are the same in every layer.  The sources are resolved again at every load as long as the store
        lacked one of them (a block that arrives later is then found, and every look that still misses is counted and
        warned about); a request's destinations when its candidate blocks have changed."""
        if not batch.src_complete and ("src", id(batch)) not in self.step["cache"]:
            self.step["cache"][("src", id(batch))] = True           # once per step, not once per layer
            src = torch.full((batch.n, max(batch.longest, 1)), -1, dtype=torch.int32)
            missing = 0
            for row, states in enumerate(batch.states):
                st = states[0]
                rid = st.req_meta.request_id
                held = self.held.get(rid)
                if held is None:
                    held = self.held[rid] = HeldBlocks(self.plugin.connector)
                stored = held.slots(st.block_hashes[st.init_window_sz : st.init_window_sz + batch.lens[row]])
                missing += stored.count(-1)
                src[row, : len(stored)] = torch.tensor(stored, dtype=torch.int32)
            if missing:
                self.plugin._report_missing(missing)
            batch.src_table = ops.upload(src, self.device)
            batch.src_complete = missing == 0
        width = batch.dst_host.shape[1]
        changed = batch.dst_table is None
        for member, _, row in members:
            cands = tuple(self._candidates(member[0], member[1][0])[:width])
            if batch.dst_rows[row] != cands:
                batch.dst_rows[row] = cands
                batch.dst_host[row] = -1
                batch.dst_host[row, : len(cands)] = torch.tensor(cands, dtype=torch.int32)
                changed = True
        if changed:
            batch.dst_table = ops.upload(batch.dst_host, self.device)
        return batch.src_table, batch.dst_table
