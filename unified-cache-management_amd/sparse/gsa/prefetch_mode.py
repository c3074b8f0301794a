"""GSA with ``ptopk_prefetch_enable``: the hooks' side of the prefetch engine.

In this mode (the reference's ``PTOPK_PREFETCH_ENABLE``, ucm/sparse/utils.py:11) a long request gives most of its
cache blocks back at its first decode step and keeps ``max_topk + 1`` of them as its resident set.  Attention no
longer reads a table chosen from all the request's blocks but the engine's: every few steps the latest selection is
compared with what is resident, missed blocks are loaded from the KV store into resident blocks the selection does
not use, and the table the round wrote becomes the one attention reads at the round after.  The Python side of that
protocol is ``GSAPrefetchBase`` (ucm/sparse/gsa/prefetch/prefetch_engine.py:125-553) and the parts of ``GSA`` that
dump blocks to the store and load the round's misses (ucm/sparse/gsa/gsa.py:690-745, 821-866); this module is their
counterpart on top of ``GSAPrefetchEngineC`` (prefetch.py), with every table on the device:

* ``use_table`` / ``use_len``: the block table attention reads, per layer and request row (``use_block_table``);
  ``succ_table`` / ``succ_len``: the one the next round writes (``m_load_success_list``); swapped at every round
  (deal_async_prefetch :193-238);
* first decode step of a request (``_first_topk_deal`` :327-379): both tables list the cache blocks at the
  request's ``remain_idx``, the free list those at ``prefetch_idx``, and the engine learns which logical block every
  resident cache block holds;
* every step (``_gsa_block_len_pre`` :381-425): sequence lengths from the table lengths, and a block the request has
  just grown by joins the table (and, at the next round, the other table and the engine's map);
* a round (every ``prefetch_stride`` = 6 steps with a sparsified request in the batch): swap, one
  ``ucm_prefetch_plan`` launch, one ``ucm_kv_load_planned`` for the misses it could serve - all on the step's stream,
  no host synchronisation;
* every block whose representative is taken goes to the store under the reference's name ``req_<id>_blk_<n>``
  (gsa.py:715-745), this layer's K and V slice in one pointer-array copy.

Which logical blocks the windows stand for follows the reference with one exception: the saved local window is
written into the last ``local`` resident blocks, so those blocks hold the last ``local`` blocks the request had when
it was sparsified; the reference names them after the request's length one step later (``real_length``, :366-368),
which is off by one block when the first decoded token opens a new block.

Scheduler side: the reference has no ``allocate_slots`` for GSA; ``GSA.allocate_slots`` here keeps a request's first
``sparse_len`` blocks (which still hold logical blocks 0 .. max_topk) and whatever it holds beyond its prompt.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ... import ops
from ..utils import HeldBlocks
from .prefetch import GSAPrefetchEngineC


class GsaPrefetchMode:
    def __init__(self, gsa, store, device):
        if store is None or not hasattr(store, "device_pool"):
            raise RuntimeError("GSA prefetch mode needs a KV store whose blocks a kernel can read (device_pool())")
        self.gsa, self.store, self.device = gsa, store, device
        L, MB, W = gsa.layer_num, gsa.max_bs, gsa.max_block_len
        i32 = dict(dtype=torch.int32, device=device)
        self.use_table = torch.zeros((L, MB, W), **i32)
        self.succ_table = torch.zeros((L, MB, W), **i32)
        self.use_len = torch.zeros((L, MB), **i32)
        self.succ_len = torch.zeros((L, MB), **i32)
        self.free_block = torch.zeros((L, MB, W), **i32)
        self.free_len = torch.zeros((L, MB), **i32)
        self.seq_len = torch.zeros((L, MB), **i32)
        self.engine = GSAPrefetchEngineC(self.free_block, self.succ_table, self.free_len, self.succ_len, max_requests=MB)
        self.src_table = torch.full((MB, W), -1, **i32)           # engine row x logical block -> block of the store's pool
        self.pool, self.pool_block_bytes = store.device_pool()
        self.stride = int(gsa.prefetch_stride)
        self.space = 0                                            # steps since the last round (prefetch_space)
        self.rounds = 0
        self.engine_id: Dict[object, int] = {}                    # request id -> the integer the engine knows it by
        self._next_id = 0
        self.to_map: Dict[object, List[tuple]] = {}               # blocks to tell the engine about at the next round
        self.to_table: Dict[object, List[int]] = {}               # ... and to append to the table that round activates
        self.batch: List = []
        self.held: Dict[object, HeldBlocks] = {}                  # per request: its stored blocks stay in the store's pool
        self.ready = set()                                        # requests whose table rows have been set up
        self.bt_step = self.seq_step = None
        self._save_key = None
        self._save = None

    # ---- names ------------------------------------------------------------------------------------------------
    @staticmethod
    def block_hash(request_id, logical: int) -> str:
        return f"req_{request_id}_blk_{logical}"                  # gsa.py:471-473

    def _engine_id(self, request_id) -> int:
        known = self.engine_id.get(request_id)
        if known is None:
            known = self.engine_id[request_id] = self._next_id
            self._next_id += 1
        return known

    def round_due(self) -> bool:
        """The step that is about to run ends with a round of the engine."""
        return self.space >= self.stride - 1

    # ---- execute_begin ------------------------------------------------------------------------------------------
    def begin_step(self, by_index: List) -> None:
        """Tables and sequence lengths of this step's batch (model_input_del, prefetch_engine.py:125-171)."""
        gsa = self.gsa
        cache_map, bs = gsa.topk_kpre_manger.cache_map, gsa.block_size
        self.batch = [st for st in by_index if st is not None]
        rows = [cache_map[st.req_id] for st in self.batch]
        dev = self.device
        plain_rows, plain_lens, plain_seq, plain_blocks = [], [], [], []
        dec_rows, dec_slot, grow_rows, grow_blocks = [], [], [], []
        for st, row in zip(self.batch, rows):
            if not st.is_decode():
                # prefill: the request's own blocks and length (:416-425)
                plain_rows.append(row)
                plain_lens.append(len(st.blocks))
                plain_seq.append(st.get_seq_len())
                plain_blocks.append(st.blocks)
                self.to_map[st.req_id], self.to_table[st.req_id] = [], []
                self.ready.discard(st.req_id)
                continue
            if st.remain_idx is not None:
                self._first_deal(st, row)
            elif st.req_id not in self.ready:
                # a request whose first decode step ran while the mode was idle (no sparsified request in the batch):
                # it holds all its blocks
                plain = ops.upload(torch.tensor(st.phys, dtype=torch.int32), dev)
                for table, lens in ((self.use_table, self.use_len), (self.succ_table, self.succ_len)):
                    table[:, row, : len(st.phys)] = plain
                    lens[:, row] = len(st.phys) - (1 if st.get_seq_len() % bs == 1 else 0)
                self.ready.add(st.req_id)
            slot = st.get_seq_len() % bs
            dec_rows.append(row)
            dec_slot.append(slot)
            if slot == 1:
                # the token of this step opens a block: it joins the table now, the other table and the engine's map
                # at the next round (:395-410)
                last = st.phys[-1]
                grow_rows.append(row)
                grow_blocks.append(last)
                self.to_table.setdefault(st.req_id, []).append(last)
                self.to_map.setdefault(st.req_id, []).append((len(st.blocks) - 1, last))
        if plain_rows:
            width = max(plain_lens)
            host = torch.zeros((len(plain_rows), width), dtype=torch.int32)
            for i, blocks in enumerate(plain_blocks):
                host[i, : len(blocks)] = torch.tensor(blocks, dtype=torch.int32)
            at = ops.upload(torch.tensor([plain_rows, plain_lens, plain_seq], dtype=torch.int32), dev).long()
            self.use_table[:, at[0], :width] = ops.upload(host, dev)
            self.use_len[:, at[0]] = at[1].to(torch.int32)
            self.seq_len[:, at[0]] = at[2].to(torch.int32)
        if dec_rows:
            d = ops.upload(torch.tensor([dec_rows, dec_slot], dtype=torch.int32), dev)
            at, slot = d[0].long(), d[1]
            n = self.use_len[:, at]                                # [L, decode requests], before this step's growth
            self.seq_len[:, at] = torch.where(slot == 0, n * bs, torch.where(slot == 1, n * bs + 1, (n - 1) * bs + slot))
        if grow_rows:
            g = ops.upload(torch.tensor([grow_rows, grow_blocks], dtype=torch.int32), dev)
            self._append(self.use_table, self.use_len, g[0].long(), g[1])
        rows_dev = ops.upload(torch.tensor(rows, dtype=torch.int64), dev)
        self.bt_step = self.use_table.index_select(1, rows_dev)   # [L, batch, W], the step's requests in batch order
        self.seq_step = self.seq_len.index_select(1, rows_dev)

    @staticmethod
    def _append(table: torch.Tensor, lens: torch.Tensor, at: torch.Tensor, blocks: torch.Tensor) -> None:
        """table[l, at[i], lens[l, at[i]]] = blocks[i] and lens[l, at[i]] += 1, every layer."""
        pos = lens[:, at].long().unsqueeze(2)                      # [L, n, 1]
        rows = table[:, at]                                        # a copy [L, n, W]
        rows.scatter_(2, pos, blocks.view(1, -1, 1).expand(table.shape[0], -1, 1))
        table[:, at] = rows
        lens[:, at] += 1

    def _first_deal(self, st, row: int) -> None:
        """First decode step of a request (_first_topk_deal, prefetch_engine.py:327-379)."""
        gsa, dev = self.gsa, self.device
        phys, remain, free = st.phys, list(st.remain_idx), list(st.prefetch_idx)
        in_use = [phys[x] for x in remain]
        spare = [phys[x] for x in free]
        both = ops.upload(torch.tensor(in_use + spare, dtype=torch.int32), dev)
        n_use, n_free = len(in_use), len(spare)
        self.use_table[:, row, :n_use] = both[:n_use]
        self.succ_table[:, row, :n_use] = both[:n_use]
        self.use_len[:, row] = n_use
        self.succ_len[:, row] = n_use
        self.free_len[:, row] = n_free
        if n_free:
            self.free_block[:, row, :n_free] = both[n_use:]
        self.to_map[st.req_id], self.to_table[st.req_id] = [], []
        self.ready.add(st.req_id)
        if not st.is_gsa():
            return
        # which logical block every resident cache block holds: the blocks at remain_idx and prefetch_idx their own
        # number, the last `local` of remain_idx the local window that was written into them
        local = gsa.min_topk - 1
        logical = remain[:-local] + list(range(st.prompt_blocks - local, st.prompt_blocks))
        table = {idx: phys[pos] for idx, pos in zip(free + logical, free + remain)}
        eid = self._engine_id(st.req_id)
        self.engine.set_blocks_map(eid, table, free + logical)
        self._sources(st, self.engine.row_of(eid), range(st.prompt_blocks))

    def _sources(self, st, engine_row: int, logical) -> None:
        """Where the store keeps the request's logical blocks (the hash -> pool block lookup, once per block)."""
        logical = list(logical)
        if not logical:
            return
        held = self.held.get(st.req_id)
        if held is None:
            held = self.held[st.req_id] = HeldBlocks(self.store)
        slots = held.slots([self.block_hash(st.req_id, i) for i in logical])
        # (the request's last block is still being written and comes to the store when it is full; it is inside the
        # selection's window until then and never asked for)
        missing = sum(1 for i, s in zip(logical, slots) if s < 0 and i < st._repre_done)
        if missing:
            self.gsa._report_missing(missing)
        at = ops.upload(torch.tensor(logical, dtype=torch.int64), self.device)
        self.src_table[engine_row].index_copy_(0, at, ops.upload(torch.tensor(slots, dtype=torch.int32), self.device))

    # ---- attention_finished -------------------------------------------------------------------------------------
    def save_blocks(self, layer_id: int, kv_cache: torch.Tensor) -> None:
        """The blocks whose representatives this step takes go to the store, this layer's K and V slices in one
        pointer-array copy (launch_transfer_task("dump", ...) per layer, gsa.py:715-745)."""
        gsa = self.gsa
        key = gsa.model_input
        if self._save_key is not key:                             # the same lists in every layer's hook
            self._save_key, self._save = key, None
            hashes, blocks, owners = [], [], []
            for st in key.get("batch", []):
                if st is None:
                    continue
                for logical, block in zip(st.calc_logical, st.calc_block_table):
                    hashes.append(self.block_hash(st.req_id, logical))
                    blocks.append(block)
                    owners.append((st, logical))
            if not hashes:
                return
            if any(rc != 0 for rc in self.store.create(hashes)):
                raise RuntimeError("GSA prefetch mode: the KV store has no room for this step's blocks")
            slots = [self.store.slot_of[h] for h in hashes]
            es = kv_cache.element_size()
            block_bytes, kv_stride = kv_cache.stride(1) * es, kv_cache.stride(0) * es
            i64 = dict(dtype=torch.int64)
            src = ops.upload(torch.tensor(blocks, **i64) * block_bytes, self.device)
            dst = ops.upload(torch.tensor(slots, **i64) * self.pool_block_bytes + self.pool.data_ptr(), self.device)
            self._save = (torch.cat([src, src + kv_stride]), torch.cat([dst, dst + block_bytes]), block_bytes, hashes)
            for (st, logical), slot in zip(owners, slots):       # a sparsified request can be asked for them from now on
                eid = self.engine_id.get(st.req_id)
                if eid is not None and self.engine.row_of(eid) >= 0:
                    self._sources(st, self.engine.row_of(eid), [logical])
        if self._save is None:
            return
        src, dst, block_bytes, hashes = self._save
        ops.copy_batch(dst + layer_id * 2 * block_bytes, src + kv_cache.data_ptr(), block_bytes)
        if layer_id == gsa.layer_num - 1:
            self.store.commit(hashes)

    # ---- execute_finished ---------------------------------------------------------------------------------------
    def end_step(self) -> None:
        """A round of the engine every ``prefetch_stride`` steps that have a sparsified request
        (deal_async_prefetch, prefetch_engine.py:193-238, and the loads of gsa.py:821-866)."""
        gsa = self.gsa
        if not gsa.model_input.get("any_gsa"):
            return
        if self.space < self.stride - 1:
            self.space += 1
            return
        self.space = 0
        self.rounds += 1
        self.use_table, self.succ_table = self.succ_table, self.use_table
        self.use_len, self.succ_len = self.succ_len, self.use_len
        cache_map = gsa.topk_kpre_manger.cache_map
        req_ids, topk_lens, rows = [], [], []
        grow_rows, grow_blocks = [], []
        for st in self.batch:
            row = cache_map[st.req_id]
            for logical, block in self.to_map.get(st.req_id, []):
                if st.req_id in self.engine_id:
                    self.engine.add_blocks_map(self.engine_id[st.req_id], logical, block)
            for block in self.to_table.get(st.req_id, []):
                grow_rows.append(row)
                grow_blocks.append(block)
            self.to_map[st.req_id], self.to_table[st.req_id] = [], []
            req_ids.append(self.engine_id.get(st.req_id, -1))
            rows.append(row)
            n = len(st.blocks)
            k = gsa._topk_len(n) if st.is_gsa() else 0
            topk_lens.append(min(k, n))
        for r, b in zip(grow_rows, grow_blocks):                   # (one at a time: a request may have grown twice)
            one = torch.tensor([r], dtype=torch.int64, device=self.device)
            self._append(self.use_table, self.use_len, one, torch.tensor([b], dtype=torch.int32, device=self.device))
        order = [st.index_in_batch for st in self.batch]
        topk = gsa.topk_caches[:, : len(order)] if order == list(range(len(order))) else gsa.topk_caches[:, order]
        self.engine.set_blocks_table_info(self.succ_table, self.succ_len, topk, gsa.step_count)
        self.engine.run_async_prefetch_bs(req_ids, topk_lens, rows)
        layers, kv_stride, block_bytes, num_blocks = gsa._all_layers()
        self.engine.load_missing(layers, kv_stride, block_bytes, num_blocks, self.pool, self.pool_block_bytes, self.src_table)

    def request_finished(self, request_id) -> None:
        eid = self.engine_id.pop(request_id, None)
        if eid is not None:
            self.engine.del_blocks_map(eid)
        self.to_map.pop(request_id, None)
        self.to_table.pop(request_id, None)
        self.ready.discard(request_id)
        held = self.held.pop(request_id, None)
        if held is not None:
            held.release()
