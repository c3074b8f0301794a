"""Batched, device-resident retrieval step of the KvComp plugin.

The reference scores and loads one request and one layer at a time
(ucm/sparse/kvcomp/kvcomp.py:361-389): the query slice of the request, its
group mean, the hash codes, the Hamming scores against the request's blocks, a
``topk`` whose result comes back to the host as a list, the list turned into
block hashes and two ``store.load`` calls with a tensor view per block, and a
wait for them.  When the store's blocks are device-addressable
(``UcmHipBlockStore.device_pool``) a layer's hook needs none of the host round
trips and covers all requests of the step at once:

* every request owns a row (its segment of the summary tables, which the plugin
  already keeps); per step the host uploads one descriptor from pinned memory -
  for each request that retrieves, the first candidate block, how many
  candidates, how many to pick, which token of the step's batch is its query;
* the hook takes the group means of all those queries with the reference's own
  torch expression, then ONE ``ucm_hash_encode_queries``, ONE
  ``ucm_hash_score_blocks``, ONE ``ucm_topk_windows`` (ascending picks, as the
  reference sorts them) and ONE ``ucm_kv_load_planned`` that copies pick j of
  every request from the store's pool into that request's j-th middle cache
  block, K and V - what ``launch_transfer_task("load", hashes, mid)`` does
  (:283-323), without the wait.

With ``"delta_loads": true`` the load is a delta: the plugin remembers which candidate each middle cache block
holds (per layer and request), ``ucm_delta_plan`` keeps the picks that are already there where they are and pairs the
missing ones with the blocks whose candidate was not picked again, and ``ucm_kv_load_planned`` moves only those - the
same set of blocks in the request's middle cache blocks as the reference leaves there, in another order (the reference
reloads every pick at every retrieval, :283-323, pick j into the j-th block).

Which steps retrieve, which blocks are candidates and how many are picked are
the reference's rules (``ReqStatePerLayer.retrieval`` :202-258).  Blocks that
became full (``save_blocks`` :325-347) are dumped into the pool and hashed for
all requests of a layer with one pointer-array copy and one launch; the windows
kept aside at the end of a prefill and written back at the first decode step
(:260-274, :392-404) take one pointer-array copy per layer each way.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ... import ops
from ..utils import HeldBlocks


class KvCompDevicePath:
    def __init__(self, plugin, pool: torch.Tensor, pool_block_bytes: int, device):
        self.plugin, self.pool, self.pool_block_bytes, self.device = plugin, pool, pool_block_bytes, device
        L, rows, mb, h = plugin.total_num_hidden_layers, plugin.max_num_seqs, plugin.max_blocks, plugin.num_key_heads
        i32 = dict(dtype=torch.int32, device=device)
        self.rows, self.max_blocks = rows, mb
        self.idx = torch.full((L, rows, mb), -1, **i32)           # picks, as offsets from the row's first candidate
        self.cnt = torch.zeros((L, rows), **i32)
        self.src_table = torch.full((rows, mb), -1, **i32)        # candidate i of a row -> block of the store's pool
        self.dst_table = torch.full((rows, mb), -1, **i32)        # pick j of a row -> cache block
        self.q_codes = torch.empty((1, rows, h, 16), dtype=torch.uint8, device=device)
        self.q_sum = torch.empty((1, rows, 128), dtype=torch.int16, device=device)
        self.qbar = torch.empty((1, rows, h, 16), dtype=torch.uint8, device=device)
        # per-step descriptor, one entry per retrieving request: seg_off, seg_len, topk_len, its token in the step's
        # query tensor, its table row; filled on the host and sent in one copy
        self._desc = torch.empty((5, rows), dtype=torch.int32)
        # delta loads: the candidate (offset from the row's first) each middle cache block holds, -1 = none of them
        self.delta = bool(plugin.cfg.get("delta_loads", False))
        self.resident = torch.full((L, rows, mb), -1, **i32) if self.delta else None
        self.res_step = self.load_step = self.slot_step = self.miss_step = self._res_rows = None
        self._forget: List[int] = []                              # rows whose load left blocks out: planned afresh next time
        self.n_layers = L
        self.n_src: Dict[object, int] = {}                        # candidates of a request whose pool block is uploaded
        self.src_absent: Dict[object, List[int]] = {}             # ... and those the store did not hold at the last look
        self.held: Dict[object, HeldBlocks] = {}                  # per request: its stored blocks stay in the store's pool
        self.dst_ids: Dict[object, tuple] = {}
        self.active: List[object] = []                            # requests that retrieve in this step
        self.first_of: Dict[object, int] = {}
        self.seg_off = self.seg_len = self.topk_len = self.tokens = self.src_step = self.dst_step = None
        self.slot_of_step: Dict[object, int] = {}
        self.max_len = self.total = 0
        self._save_key = None
        self.windows: Dict[object, torch.Tensor] = {}              # per request: [layer][K|V][window block] bytes
        self.win_shape: Dict[object, tuple] = {}
        self._win_key: Dict[str, object] = {}
        self._win_lists: Dict[str, tuple] = {}
        self._save_src = self._save_dst = self._save_ids = self._save_rows = None
        self._kv: Dict[int, ops.LayerPointers] = {}
        self._geom: Dict[int, tuple] = {}

    def register_kv_cache(self, layer_id: int, kv_cache: torch.Tensor) -> None:
        if layer_id not in self._kv or self._geom[layer_id][3] != kv_cache.data_ptr():
            self._kv[layer_id] = ops.LayerPointers([kv_cache])
            self._geom[layer_id] = (kv_cache.stride(0) * kv_cache.element_size(), kv_cache.stride(1) * kv_cache.element_size(),
                                    kv_cache.shape[1], kv_cache.data_ptr())

    # ---- per step ---------------------------------------------------------------------------
    def build_step(self, metas, query_start: List[int]) -> None:
        """metas: the step's requests; query_start[i]: first token of request i in the step's query tensor.  Fills
        the descriptor for the requests that retrieve in this step (kvcomp.py:361-371, :202-215)."""
        p = self.plugin
        stride, init, local = p.cfg["retrieval_stride"], p.cfg["init_window_sz"], p.cfg["local_window_sz"]
        self._commit_resident()
        self.active, self.max_len, self.total = [], 0, 0
        rows = self.rows
        host = None
        for meta, a in zip(metas, query_start):
            states = p.req_states.get(meta.request_id)
            st = states[0] if states else None
            if st is None or not st.block_size or meta.step % stride != 1 or meta.num_scheduled_tokens != 1:
                continue
            n_blocks = st.num_blocks_hashed
            mid = meta.vllm_block_ids[init:-local]
            top_k, first, end = len(mid), init, n_blocks - local + 1
            if end <= first or top_k <= 0:
                continue
            count = end - first
            k = count if top_k >= n_blocks else min(top_k, count)     # every candidate, or the best top_k of them
            row = p.segment_base(meta.request_id) // p.max_blocks
            if host is None:
                host = self._desc.numpy()
            n = len(self.active)
            host[0, n], host[1, n], host[2, n], host[3, n], host[4, n] = row * p.max_blocks + first, count, k, a, row
            self.active.append(meta.request_id)
            self.first_of[meta.request_id] = first
            self.max_len = max(self.max_len, count)
            self.total += count
            self._sources(meta.request_id, row, first, count)
            ids = tuple(mid[:k])
            if self.dst_ids.get(meta.request_id) != ids:
                self.dst_table[row, : len(ids)] = torch.tensor(ids, dtype=torch.int32, device=self.device)
                self.dst_ids[meta.request_id] = ids
                if self.delta:
                    self.resident[:, row] = -1               # other cache blocks: what they hold is not known
            if self.delta and self.src_absent.get(meta.request_id):
                self._forget.append(row)                     # the plan will count blocks as loaded that the load leaves out
        if host is not None:
            n = len(self.active)
            d = ops.upload(self._desc[:, :n], self.device)      # (pinned staging whose reuse waits for its last copy)
            self.seg_off, self.seg_len, self.topk_len, self.tokens = d[0, :n], d[1, :n], d[2, :n], d[3, :n]
            table_rows = d[4, :n].long()
            self.src_step = self.src_table.index_select(0, table_rows)      # the step's requests side by side
            self.dst_step = self.dst_table.index_select(0, table_rows)
            self.slot_of_step = {r: i for i, r in enumerate(self.active)}
            if self.delta:
                w = max(len(self.dst_ids[r]) for r in self.active)           # middle cache blocks of the widest request
                if w > 1024:
                    raise ValueError(f"delta_loads plans at most 1024 middle blocks per request ({w} here)")
                # [layers, the step's requests, middle blocks]
                self.res_step = self.resident.index_select(1, table_rows)[:, :, :w].contiguous()
                self.load_step, self.slot_step = torch.empty_like(self.res_step), torch.empty_like(self.idx[:, :n])
                self.miss_step = torch.zeros((self.n_layers, n), dtype=torch.int32, device=self.device)
                self._res_rows = table_rows

    def _commit_resident(self) -> None:
        """What the step's plans left in the middle blocks goes back into the requests' rows (after the last layer's
        hook, or before the next step is built)."""
        if self._res_rows is not None:
            self.resident[:, :, : self.res_step.shape[2]].index_copy_(1, self._res_rows, self.res_step)
            self._res_rows = None
        if self._forget:
            self.resident[:, torch.tensor(self._forget, dtype=torch.int64, device=self.device)] = -1
            self._forget = []

    def _sources(self, request_id, row: int, first: int, count: int) -> None:
        """Pool blocks of candidates first .. first+count-1: the hash -> store lookup, once per block the store holds;
        one it does not hold (its dump found no room, or has not happened) is looked up again at every retrieval, and
        reported while it stays away - the retrieval's load leaves it out."""
        done = self.n_src.get(request_id, 0)
        absent = self.src_absent.get(request_id)
        if done >= count and not absent:
            return
        from .kvcomp import ReqStatePerLayer                 # (the plugin module imports this one)

        held = self.held.get(request_id)
        if held is None:
            held = self.held[request_id] = HeldBlocks(self.plugin.connector)
        name = ReqStatePerLayer.block_hash
        if absent:
            looked = held.slots([name(request_id, first + i) for i in absent])
            found = [(i, slot) for i, slot in zip(absent, looked) if slot >= 0]
            if found:
                at = torch.tensor([i for i, _ in found], dtype=torch.int64, device=self.device)
                self.src_table[row].index_copy_(0, at, ops.upload(torch.tensor([s for _, s in found], dtype=torch.int32), self.device))
                gone = {i for i, _ in found}
                absent = [i for i in absent if i not in gone]
        if done < count:
            src = held.slots([name(request_id, first + i) for i in range(done, count)])
            self.src_table[row, done:count] = ops.upload(torch.tensor(src, dtype=torch.int32), self.device)
            absent = (absent or []) + [done + i for i, s in enumerate(src) if s < 0]
            self.n_src[request_id] = count
        self.src_absent[request_id] = absent or []
        if absent:
            self.plugin._report_missing(len(absent))

    # ---- hook -------------------------------------------------------------------------------
    def attention_begin(self, layer_id: int, query: torch.Tensor) -> None:
        if not self.active:
            return
        p = self.plugin
        h, d, b = p.num_key_heads, p.head_size, len(self.active)
        q = query.index_select(0, self.tokens.long())                 # [b, q heads, d], the model's dtype
        hq = q.shape[1]
        if hq > h:                                                    # kvcomp.py:228-233
            q = q.view(b, h, -1, d).mean(2)
        elif hq < h:
            q = torch.repeat_interleave(q, h // hq, 1)
        q = q.to(p.hash_encoder.dtype).reshape(1, b, h, d).contiguous()
        q_codes, q_sum, qbar = self.q_codes[:, :b], self.q_sum[:, :b], self.qbar[:, :b]
        ops.hash_encode_queries(q, p.hash_encoder.hash_weights, h, q_codes, q_sum, qbar, b)
        l = slice(layer_id, layer_id + 1)
        ops.hash_score_blocks(0, q_sum, qbar, p.colsum[l], p.block_codes[l], self.seg_off, self.seg_len, self.total,
                              p.scores[l], round_fp16=bool(p.cfg["fp16_scores"]))
        idx, cnt = self.idx[l, :b], self.cnt[l, :b]
        ops.topk_windows(p.scores[l], self.seg_off, self.seg_len, self.topk_len, self.max_len, idx, cnt, start_w=0, end_w=0)
        kv_stride, block_bytes, num_blocks, _ = self._geom[layer_id]
        if self.delta:
            ops.delta_plan(idx, idx, cnt, self.res_step[l], self.load_step[l], self.slot_step[l], self.miss_step[l])
            ops.kv_load_planned(self._kv[layer_id], 0, layer_id, 1, kv_stride, block_bytes, num_blocks, self.pool,
                                self.pool_block_bytes, self.load_step[l], self.src_step, self.dst_step, None)
            if layer_id == self.n_layers - 1:
                self._commit_resident()
            return
        ops.kv_load_planned(self._kv[layer_id], 0, layer_id, 1, kv_stride, block_bytes, num_blocks, self.pool,
                            self.pool_block_bytes, idx, self.src_step, self.dst_step, None, load_count=cnt)

    # ---- blocks that became full --------------------------------------------------------------
    def save_blocks(self, layer_id: int, step_key, batch) -> bool:
        """batch: (request, cache blocks, logical numbers) of every request with full blocks to save in this step
        (the same lists in every layer's hook).  One pointer-array copy moves this layer's K and V slices of all of
        them into the store's pool - what ``launch_transfer_task("dump", ...)`` does per request (kvcomp.py:325-347)
        - and one launch writes their codes and column sums.  False (nothing done) when the store has no room."""
        from .kvcomp import ReqStatePerLayer

        p = self.plugin
        kv_stride, block_bytes, num_blocks, base = self._geom[layer_id]
        if step_key is not self._save_key:
            store = p.connector
            hashes = [ReqStatePerLayer.block_hash(r, b) for r, _, logical in batch for b in logical]
            made = [h for h in hashes if h not in store.slot_of]
            if any(rc != 0 for rc in store.create(hashes)):
                store.commit(made, False)        # the slots this call reserved go back: nothing was written into them
                return False
            physical = [b for _, blocks, _ in batch for b in blocks]
            rows = [p.segment_base(r) + b for r, _, logical in batch for b in logical]
            i64 = dict(dtype=torch.int64, device=self.device)
            src = torch.tensor(physical, **i64) * block_bytes
            dst = torch.tensor([store.slot_of[h] for h in hashes], **i64) * self.pool_block_bytes + self.pool.data_ptr()
            self._save_src = torch.cat([src, src + kv_stride])                  # K slices, then V slices
            self._save_dst = torch.cat([dst, dst + block_bytes])
            self._save_ids = torch.tensor(physical, dtype=torch.int32, device=self.device)
            self._save_rows = torch.tensor(rows, dtype=torch.int32, device=self.device)
            self._save_key = step_key
        ops.copy_batch(self._save_dst + layer_id * 2 * block_bytes, self._save_src + base, block_bytes)
        l = slice(layer_id, layer_id + 1)
        p.hash_encoder.encode_cache_blocks(p._layer_ptrs[layer_id], self._save_ids, self._save_rows, p.block_size,
                                           p.num_key_heads, p._num_blocks[layer_id], p.colsum[l], p.block_codes[l],
                                           None if p.token_codes is None else p.token_codes[l])
        return True

    # ---- the windows kept aside at the end of the prefill ---------------------------------------
    def _window_blocks(self, ids: List[int], n_head: Optional[int] = None, n_tail: Optional[int] = None) -> List[int]:
        init, local = self.plugin.cfg["init_window_sz"], self.plugin.cfg["local_window_sz"]
        if n_head is None:                                   # kvcomp.py:260-274
            n_head = len(ids[:init])
            n_tail = min(local, len(ids[init:]))
        return ids[:n_head] + (ids[-n_tail:] if n_tail > 0 else [])

    def _window_copy(self, layer_id: int, step_key, which: str, metas, to_windows: bool) -> None:
        """One pointer-array copy between the window blocks of all ``metas`` in this layer's cache and the requests'
        window buffers ([layer][K|V][window block]); the address lists are built at the step's first hook."""
        kv_stride, block_bytes, _, base = self._geom[layer_id]
        if self._win_key.get(which) is not step_key:
            cache_off, win_addr, win_lstride = [], [], []
            L = self.plugin.total_num_hidden_layers
            for meta in metas:
                rid = meta.request_id
                if to_windows:
                    blocks = self._window_blocks(meta.vllm_block_ids)
                    n_head = len(meta.vllm_block_ids[: self.plugin.cfg["init_window_sz"]])
                    self.win_shape[rid] = (n_head, len(blocks) - n_head)
                    self.windows[rid] = torch.empty(L * 2 * len(blocks) * block_bytes, dtype=torch.uint8, device=self.device)
                else:
                    n_head, n_tail = self.win_shape[rid]
                    if len(meta.vllm_block_ids) < max(n_head, n_tail):
                        # (upstream's indexed assignment fails on the same lists: kvcomp.py:392-404)
                        raise ValueError(f"KvComp: request {rid} holds {len(meta.vllm_block_ids)} cache blocks, fewer than "
                                         f"one of its saved windows ({n_head} and {n_tail} blocks)")
                    blocks = self._window_blocks(meta.vllm_block_ids, n_head, n_tail)
                n, ptr = len(blocks), self.windows[rid].data_ptr()
                # a request whose new block list is shorter than its two windows together gets a cache block named
                # twice on the way back: the reference writes the first window, then the last one over it
                # (kvcomp.py:392-404), so of the copies into one block only the last is made
                last = {b: j for j, b in enumerate(blocks)}
                for kv in range(2):
                    for j, b in enumerate(blocks):
                        if not to_windows and last[b] != j:
                            continue
                        cache_off.append(kv * kv_stride + b * block_bytes)
                        win_addr.append(ptr + (kv * n + j) * block_bytes)
                        win_lstride.append(2 * n * block_bytes)
            i64 = dict(dtype=torch.int64, device=self.device)
            self._win_lists[which] = tuple(torch.tensor(x, **i64) for x in (cache_off, win_addr, win_lstride))
            self._win_key[which] = step_key
        cache_off, win_addr, win_lstride = self._win_lists[which]
        if cache_off.numel() == 0:
            return
        in_cache, in_windows = cache_off + base, win_addr + win_lstride * layer_id
        if to_windows:
            ops.copy_batch(in_windows, in_cache, block_bytes)
        else:
            ops.copy_batch(in_cache, in_windows, block_bytes)

    def save_windows(self, layer_id: int, step_key, metas) -> None:
        """The first ``init_window_sz`` and last ``local_window_sz`` blocks of every request that finishes its
        prefill in this step, copied aside (``construct_init_and_local_window``, kvcomp.py:260-274)."""
        self._window_copy(layer_id, step_key, "save", metas, True)

    def restore_windows(self, layer_id: int, step_key, metas) -> None:
        """... and written back into the request's new first and last blocks at its first decode step
        (``prepare_init_and_local_window``, kvcomp.py:392-404)."""
        self._window_copy(layer_id, step_key, "restore", metas, False)

    def selection(self, layer_id: int, request_id) -> Optional[List[int]]:
        """Logical blocks picked for the request in this layer, ascending (reads back).  Valid until the next step in
        which any request retrieves: the tables hold the latest retrieval only."""
        i = self.slot_of_step.get(request_id)
        if i is None:
            return None
        n = int(self.cnt[layer_id, i])
        return [self.first_of[request_id] + int(x) for x in self.idx[layer_id, i, :n].tolist()]

    def resident_blocks(self, layer_id: int, request_id) -> Optional[List[int]]:
        """Delta loads: the logical block each middle cache block of the request holds after its latest retrieval (-1:
        none), in the order of the request's middle cache blocks (reads back)."""
        if not self.delta or request_id not in self.dst_ids:
            return None
        self._commit_resident()
        p = self.plugin
        row = p.segment_base(request_id) // p.max_blocks
        first = self.first_of[request_id]
        return [first + int(x) if x >= 0 else -1 for x in self.resident[layer_id, row, : len(self.dst_ids[request_id])].tolist()]

    def request_finished(self, request_id) -> None:
        if self.delta and request_id in self.dst_ids:
            self._commit_resident()
            p = self.plugin
            self.resident[:, p.segment_base(request_id) // p.max_blocks] = -1
        held = self.held.pop(request_id, None)
        if held is not None:
            held.release()
        for table in (self.n_src, self.src_absent, self.dst_ids, self.first_of, self.windows, self.win_shape):
            table.pop(request_id, None)
