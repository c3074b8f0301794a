"""GSA-shaped sparse-attention plugin whose retrieval runs on the GPU.

Same hook surface and per-step flow as the reference's ``GSA``
(ucm/sparse/gsa/gsa.py:415-1031): block representatives are refreshed after
each layer's attention (``copy_k``, :634-654), each request's last query token
drives a top-k over its block representatives (``copy_q`` :616-632 +
``CalKpreAndTopk``), and ``attention_begin`` swaps the layer's block table and
sequence lengths for sparse ones (:656-686, built by
``GSAPrefetchBase._no_gsa_input_deal``,
ucm/sparse/gsa/prefetch/prefetch_engine.py:507-553).

What differs is where it runs.  The reference moves queries and block means to
the host, scores them with OpenMP loops and uses the result a few steps later.
Here the representative table, the scores and the per-layer sparse block
tables never leave HBM: ``attention_begin`` enqueues the scoring and selection
kernels of that layer on the model's own stream, and the attention kernel of
the same layer already reads the fresh table.  No host synchronisation happens
in any hook; per-step metadata goes down in one pinned-memory copy.

vLLM is not imported: the hooks only touch attributes of the objects they are
handed (``scheduler_output.num_scheduled_tokens``, ``requests[id].block_ids``,
``forward_context.no_compile_layers[name].kv_cache``, ``attn_metadata.block_table``
...), so stand-in objects drive the class in the tests.
"""
from __future__ import annotations

import ctypes
import math
from itertools import accumulate, count
from typing import Dict, List, Optional, Union

import numpy as np
import torch

from ... import _lib, ops
from ..base import INVALID_SLOT, UcmSparseBase, UcmSparseMetadata, UcmSparseRole
from ..utils import (
    INIT_WINDOW_BLOCKS,
    LOCAL_WINDOW_BLOCKS,
    MAX_BS,
    MAX_TOPK_LEN,
    MIN_TOPK_LEN,
    SEG_PREFILL_THRESHOLD,
    compute_topk_len,
)

ReqType = Union[str, int]
_serials = count()
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_Q_CODES = {torch.bfloat16: _lib.DTYPE_BF16, torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16}


class GSAReqStat:
    """Per-request bookkeeping (role of the reference's GSAReqStat, gsa.py:66-239):
    the request's cache blocks, the representative rows they map to, and which
    blocks need their representative (re)computed after this step."""

    def __init__(self, req_id: ReqType, slot_offset: int, block_size: int, threshold: int):
        self.req_id = req_id
        self.slot_offset = slot_offset
        self.block_size = block_size
        self.threshold = threshold
        self.blocks: List[int] = []
        self.blocks_version = 0           # counts the changes of `blocks`
        self.serial = next(_serials)      # a request id may come back with another request behind it
        self.calc_block_table: List[int] = []
        self.calc_repre_slot_mapping: List[int] = []
        self.num_computed_tokens = 0
        self.num_scheduled_tokens = 0
        self.num_prompt_tokens = 0
        self.num_output_tokens = 0
        self.index_in_batch = 0
        self._repre_done = 0  # blocks [0, _repre_done) have a representative
        # prefetch mode (the reference's PTOPK_PREFETCH_ENABLE): which logical blocks stay resident once the
        # request is sparsified, which resident blocks start out free, and the saved local window
        self.remain_idx: Optional[List[int]] = None
        self.prefetch_idx: Optional[List[int]] = None
        self.sparse_len = 0
        self.local_window_kv: Optional[torch.Tensor] = None   # [blocks, layers, K|V, block bytes]
        self.phys: List[int] = []         # prefetch mode, decode: the cache blocks the request holds (the scheduler's list)
        self.prompt_blocks = 0            # ... and how many logical blocks it had when it was sparsified
        self.calc_logical: List[int] = [] # logical numbers of the blocks in calc_block_table

    # -- state queries (same meaning as the reference's) ---------------------
    def is_decode(self) -> bool:
        return self.num_prompt_tokens <= self.num_computed_tokens

    def is_gsa(self) -> bool:
        return self.num_prompt_tokens > self.threshold and self.is_decode()

    def is_last_chunk(self) -> bool:
        return self.num_computed_tokens + self.num_scheduled_tokens >= self.num_prompt_tokens

    def get_seq_len(self) -> int:
        return self.num_computed_tokens + self.num_scheduled_tokens

    def get_sparse_and_free_block(self, prefetch: bool, min_topk: int, max_topk: int, ratio: float) -> None:
        """The resident set at the first decode step (GSAReqStat._get_sparse_and_free_block, gsa.py:156-186): with
        n blocks and k = compute_topk_len(n), logical blocks 0 .. max_topk stand for the request's sparse cache
        blocks; the first k - local and the last local of them are in use (remain_idx), the ones in between start
        out free (prefetch_idx); local = min_topk - 1."""
        if self.num_prompt_tokens != self.num_computed_tokens:
            self.remain_idx = self.prefetch_idx = None
            return
        n = len(self.blocks)
        if self.num_prompt_tokens > self.threshold and prefetch:
            local = min_topk - 1
            remain_len = compute_topk_len(n, min_topk, max_topk, ratio)
            if remain_len > max_topk:
                prefetch_len, idx = 0, list(range(remain_len))
            else:
                prefetch_len, idx = max_topk - remain_len + 1, list(range(max_topk + 1))
            assert local < remain_len
            self.remain_idx = idx[: remain_len - local] + idx[-local:]
            self.prefetch_idx = idx[remain_len - local : -local]
            self.sparse_len = remain_len + prefetch_len
        else:
            self.remain_idx, self.prefetch_idx, self.sparse_len = list(range(n)), [], n

    @property
    def repre_slot_mapping(self) -> List[int]:
        return [self.slot_offset + i for i in range(len(self.blocks))]

    def update(self, num_scheduled_tokens: int, req_state, index_in_batch: int, prefetch=None) -> None:
        self.num_computed_tokens = req_state.num_computed_tokens
        self.num_scheduled_tokens = num_scheduled_tokens
        self.num_prompt_tokens = len(req_state.prompt_token_ids)
        self.num_output_tokens = len(req_state.output_token_ids)
        self.index_in_batch = index_in_batch
        src = req_state.block_ids[0]
        if prefetch is not None and self.blocks and self.is_decode():
            self._update_sparsified(src, prefetch)
            return
        # (a decoding request's list only grows at its end: the copy is made when the list changed)
        mid = len(src) // 2
        if len(src) != len(self.blocks) or (src and (src[-1] != self.blocks[-1] or src[0] != self.blocks[0]
                                                     or src[mid] != self.blocks[mid])):
            self.blocks = list(src)
            self.blocks_version += 1
        # A block gets its representative once every one of its tokens is in
        # the cache, i.e. after the step that fills it.
        full_after_step = self.get_seq_len() // self.block_size
        full_after_step = min(full_after_step, len(self.blocks))
        todo = range(self._repre_done, full_after_step)
        self.calc_block_table = [self.blocks[i] for i in todo]
        self.calc_repre_slot_mapping = [self.slot_offset + i for i in todo]
        self.calc_logical = list(todo)
        self._repre_done = max(self._repre_done, full_after_step)

    def _update_sparsified(self, src: List[int], prefetch) -> None:
        """A decoding request in prefetch mode (GSAReqStat.updata_req_state, gsa.py:133-154): ``blocks`` stays the
        list of LOGICAL blocks - one entry per block of the sequence, a block the request grows by is appended -
        while the cache blocks it really holds are the scheduler's list ``phys``: the resident blocks first, then
        the blocks decoded into.  The block being written is always the last of ``phys``; it gets its
        representative (and goes to the store) after the step that fills it."""
        # decided from the blocks the request held BEFORE the scheduler swapped in its sparse block list
        self.get_sparse_and_free_block(True, *prefetch)
        if self.remain_idx is not None:
            self.prompt_blocks = len(self.blocks)
        self.phys = list(src)
        if len(src) != self.sparse_len:
            self.blocks = self.blocks + [src[-1]]
            self.blocks_version += 1
            self.sparse_len = len(src)
        full_after_step = min(self.get_seq_len() // self.block_size, len(self.blocks))
        self.calc_block_table, self.calc_repre_slot_mapping, self.calc_logical = [], [], []
        if full_after_step > self._repre_done:
            last = len(self.blocks) - 1
            self.calc_block_table = [src[-1]]
            self.calc_repre_slot_mapping = [self.slot_offset + last]
            self.calc_logical = [last]
            self._repre_done = full_after_step


class GSAMetaData(UcmSparseMetadata):
    def __init__(self, block_size: int, device):
        self.gsa_stats: Dict[ReqType, GSAReqStat] = {}
        self.block_size = block_size
        self.device = device


class TopKAndKpreManger:
    """Hands each live request one of max_num row ranges of the representative
    table (gsa.py:323-351; spelling of the class name kept)."""

    def __init__(self, max_num: int):
        self.cache_map: Dict[ReqType, int] = {}
        self.max_num = max_num
        self.free_cache = list(range(max_num))

    def free(self, req_id: ReqType) -> bool:
        if req_id not in self.cache_map:
            return False
        self.free_cache.append(self.cache_map.pop(req_id))
        return True

    def alloc(self, req_id: ReqType) -> Optional[int]:
        if not self.free_cache:
            return None
        self.cache_map[req_id] = self.free_cache.pop(0)
        return self.cache_map[req_id]

    def is_exist(self, req_id: ReqType) -> bool:
        return req_id in self.cache_map


class GSA(UcmSparseBase):
    def __init__(self, vllm_config, role: UcmSparseRole, store=None):
        super().__init__(vllm_config, role)
        self.connector = store            # prefetch mode: the KV store the request's blocks go to and come back from
        mc, pc = vllm_config.model_config, vllm_config.parallel_config
        self.block_size = vllm_config.cache_config.block_size
        self.num_key_heads = mc.get_num_kv_heads(pc)
        self.num_q_heads = mc.get_num_attention_heads(pc)
        self.head_size = mc.get_head_size()
        self.layer_num = mc.get_num_layers(pc)
        self.max_block_len = math.ceil(mc.max_model_len / self.block_size)
        sched = getattr(vllm_config, "scheduler_config", None)
        self.max_bs = min(MAX_BS, getattr(sched, "max_num_seqs", MAX_BS))
        extra = vllm_config.kv_transfer_config.kv_connector_extra_config
        cfg = dict((extra.get("ucm_sparse_config") or {}).get("GSA") or {})
        self.threshold = int(cfg.get("seg_prefill_threshold", SEG_PREFILL_THRESHOLD))
        self.retrieval_stride = max(1, int(cfg.get("retrieval_stride", 1)))
        self.min_topk = int(cfg.get("min_topk_len", MIN_TOPK_LEN))
        self.max_topk = int(cfg.get("max_topk_len", MAX_TOPK_LEN))
        self.topk_ratio = float(cfg.get("sparse_ratio", 0.3))
        self.init_window = int(cfg.get("init_window_sz", INIT_WINDOW_BLOCKS))
        self.local_window = int(cfg.get("local_window_sz", LOCAL_WINDOW_BLOCKS))
        # "bfloat16": the table keeps the rounded means the live reference path stores (gsa.py:640-652) in
        # that type, half the bytes to score; "float32": fp32 means, the KRepreComputer contract
        # the reference's PTOPK_PREFETCH_ENABLE (ucm/sparse/utils.py:11, off as shipped): sparsified requests give
        # most of their cache blocks back, so the local window is kept aside at the end of the prefill and
        # written into the blocks that stand for it afterwards
        self.ptopk_prefetch = bool(cfg.get("ptopk_prefetch_enable", False))
        self.prefetch_stride = max(1, int(cfg.get("prefetch_stride", 6)))   # steps between two rounds of the prefetch engine
        self._pf = None                   # prefetch mode's tables and engine (prefetch_mode.py), built with the device state
        # 0: a layer's blocks are scored with the layer's own queries just before its attention (one launch per layer).
        # 1: the reference's timing - a layer's hook only keeps the step's last query tokens (copy_q, gsa.py:616-632) and
        # the step after scores every layer with them in ONE launch before the model runs, as the reference's block
        # tables of a step come from queries of an earlier one (gsa.py:672-679); a request's first sparsified step
        # still scores layer by layer.  Prefetch mode keeps its own timing (its rounds read the step's selection).
        self.retrieval_lag = int(cfg.get("retrieval_lag", 0))
        if self.retrieval_lag not in (0, 1):
            raise ValueError("retrieval_lag must be 0 (same step) or 1 (the step after)")
        self.repre_dtype = torch.bfloat16 if cfg.get("repre_dtype", "float32") == "bfloat16" else torch.float32
        self.repre_mode = ops.MEAN_BF16_STORE if self.repre_dtype == torch.bfloat16 else ops.MEAN_F32

        self.topk_kpre_manger = TopKAndKpreManger(self.max_bs)
        self.gsa_stats: Dict[ReqType, GSAReqStat] = {}
        self.gsa_metadata: Optional[GSAMetaData] = None
        self.model_input: dict = {}
        self.step_count = 0
        self.k_cache: Dict[int, torch.Tensor] = {}
        self.v_cache: Dict[int, torch.Tensor] = {}
        self._dev_ready = False
        self._layer_ptrs: Dict[int, ops.LayerPointers] = {}
        self._kv_all: Optional[ops.LayerPointers] = None   # every layer's (2, blocks, ...) cache, for whole-block moves
        self._kv_full: Dict[int, torch.Tensor] = {}
        self._scored: set = set()  # sparsified requests whose blocks have been scored at least once
        self._layer_of: Dict[str, int] = {}
        self._fast: Optional[list] = None   # set by execute_begin for a step that takes the one-launch path in every layer
        self._seen_layers = None          # the engine's table of layers once every layer's cache has been registered from it
        self._tables_signature = None     # (request, blocks, last block) per batch slot of the block tables on the device
        self._tables_dev: Optional[torch.Tensor] = None
        self.q_stage: Optional[torch.Tensor] = None   # retrieval_lag 1: [layers, table partitions, q_heads, head_size], the kept queries
        self._parked: set = set()         # requests whose queries of the step before are in q_stage, every layer
        self._parking: Optional[tuple] = None   # this step keeps its queries: (requests, source rows, partitions, n)
        self._lagged: Optional[list] = None     # this step's selection was made in execute_begin: per-layer views

    # ------------------------------------------------------------------ device state
    def _ensure_device_state(self, device) -> None:
        if self._dev_ready:
            return
        rows = self.max_bs * self.max_block_len
        row = self.num_key_heads * self.head_size
        L = self.layer_num
        self.device = device
        self._dev_index = device.index if device.index is not None else torch.cuda.current_device()
        self.kpre_caches = torch.zeros((L, rows, row), dtype=self.repre_dtype, device=device)
        self.scores = torch.zeros((L, rows), dtype=torch.float32, device=device)
        self.topk_caches = torch.zeros((L, self.max_bs, self.max_block_len), dtype=torch.int32, device=device)
        self.block_tables_mp = torch.zeros_like(self.topk_caches)
        self.topk_counts = torch.zeros((L, self.max_bs), dtype=torch.int32, device=device)
        self.gsa_seq_len = torch.zeros((L, self.max_bs), dtype=torch.int32, device=device)
        # two pinned staging buffers for the per-step descriptors, used alternately
        cap = (6 + 3 * self.max_block_len) * self.max_bs
        self._host_desc = [torch.zeros(cap, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._host_free = [None, None]  # event recorded after each buffer's last upload
        # attention_begin runs once per layer and decode step: it goes to the library with addresses computed
        # here and in execute_begin instead of slicing six tensors and re-validating them every time (the
        # shapes are this plugin's own and do not change)
        self._layer_addr = [
            (self.kpre_caches[l].data_ptr(), self.scores[l].data_ptr(), self.topk_caches[l].data_ptr(),
             self.topk_counts[l].data_ptr(), self.block_tables_mp[l].data_ptr(), self.gsa_seq_len[l].data_ptr())
            for l in range(L)
        ]
        self._repre_code = _lib.DTYPE_BF16 if self.repre_dtype == torch.bfloat16 else _lib.DTYPE_F32
        self._views: Dict[int, list] = {}  # batch size -> per-layer (block table, sequence lengths) views
        # scoring and selection of a layer are ONE library call with ONE argument block: everything that does not
        # change between layers is filled in here and in execute_begin, attention_begin sets the layer and its
        # queries.  The ticket counters of the fused launch are zero between calls.
        self.tickets = torch.zeros((L, self.max_bs), dtype=torch.int32, device=device)
        self._sel = _lib.ScoreSelectArgs(
            q_heads=self.num_q_heads, repre=self.kpre_caches.data_ptr(), repre_dtype=self._repre_code,
            repre_layer_stride=self.kpre_caches.stride(0), repre_rows=rows, kv_heads=self.num_key_heads,
            head_dim=self.head_size, scores=self.scores.data_ptr(), scores_layer_stride=self.scores.stride(0),
            start_w=self.init_window, end_w=self.local_window, idx_out=self.topk_caches.data_ptr(),
            count_out=self.topk_counts.data_ptr(), out_stride=self.max_block_len, bt_stride=self.max_block_len,
            phys_out=self.block_tables_mp.data_ptr(), sparse_seq_lens=self.gsa_seq_len.data_ptr(),
            block_size=self.block_size, tickets=self.tickets.data_ptr(),
            idx_layer_stride=self.topk_caches.stride(0), count_layer_stride=self.topk_counts.stride(0))
        self._sel_addr = ctypes.addressof(self._sel)
        # retrieval_lag 1: the same call over every layer at once, its queries the kept ones
        self._sel_all = _lib.ScoreSelectArgs()
        ctypes.memmove(ctypes.addressof(self._sel_all), self._sel_addr, ctypes.sizeof(self._sel))
        self._sel_all.first_layer, self._sel_all.n_layers = 0, L
        self._park_rows = _lib.lib().ucm_park_rows
        self._score_select = _lib.lib().ucm_score_select
        self._fused_ok = self.max_block_len <= 1024     # longer requests take the two launches
        self._dev_ready = True

    def _topk_len(self, n_blocks: int) -> int:
        return compute_topk_len(n_blocks, self.min_topk, self.max_topk, self.topk_ratio)

    def _prefetch_mode(self):
        if self._pf is None:
            from .prefetch_mode import GsaPrefetchMode

            self._pf = GsaPrefetchMode(self, self.connector, self.device)
        return self._pf

    def register_kv_caches(self, kv_caches: dict) -> None:
        for name, cache in kv_caches.items():
            self._register_layer(int(name.split(".")[2]), cache)

    def _register_layer(self, layer_id: int, kv_cache) -> None:
        known = self._kv_full.get(layer_id)
        if known is kv_cache or (known is not None and isinstance(kv_cache, torch.Tensor) and isinstance(known, torch.Tensor)
                                 and known.data_ptr() == kv_cache.data_ptr()):
            return
        if kv_cache[0].dtype == torch.float16 and self.repre_dtype == torch.bfloat16:
            raise ValueError("a float16 KV cache needs repre_dtype float32: the bfloat16 table holds the means of a bfloat16 model")
        self.k_cache[layer_id], self.v_cache[layer_id] = kv_cache[0], kv_cache[1]
        self._layer_ptrs[layer_id] = ops.LayerPointers([kv_cache[0]])
        self._kv_full[layer_id] = kv_cache
        self._kv_all = None
        self._ensure_device_state(kv_cache[0].device)

    def _all_layers(self):
        """(pointer table over every layer's cache, bytes between the K and V planes, bytes of a block, blocks)."""
        if self._kv_all is None:
            if len(self._kv_full) != self.layer_num or not all(isinstance(c, torch.Tensor) for c in self._kv_full.values()):
                raise RuntimeError("whole-block moves need every layer's cache registered as one (2, blocks, ...) tensor")
            self._kv_all = ops.LayerPointers([self._kv_full[l] for l in range(self.layer_num)])
        kv = self._kv_full[0]
        return self._kv_all, kv.stride(0) * kv.element_size(), kv.stride(1) * kv.element_size(), kv.shape[1]

    # ------------------------------------------------------------------ local window (prefetch mode)
    def _gsa_sparse_local_kv(self) -> None:
        """End of the step that finishes a long request's prefill: the K and V of its last ``local`` blocks, every
        layer, are kept aside (gsa.py:995-1031) - one gather launch instead of a clone per block, layer and plane."""
        local = self.min_topk - 1
        for st in self.model_input.get("batch", []):
            if st is None or st.is_decode() or not st.is_last_chunk() or st.num_prompt_tokens <= self.threshold:
                continue
            layers, kv_stride, block_bytes, num_blocks = self._all_layers()
            ids = torch.tensor(st.blocks[-local:], dtype=torch.int32, device=self.device)
            st.local_window_kv = torch.empty((ids.numel(), self.layer_num, 2, block_bytes), dtype=torch.uint8, device=self.device)
            ops.kv_gather_blocks(layers, kv_stride, block_bytes, num_blocks, ids, st.local_window_kv)

    def _init_sparse_local_kv(self, scheduler_output, requests) -> None:
        """First decode step of such a request: the saved window goes into the cache blocks that now stand for it,
        the last ``local`` entries of remain_idx (gsa.py:956-993), as one scatter launch."""
        local = self.min_topk - 1
        for req_id in scheduler_output.num_scheduled_tokens:
            st = self.gsa_stats.get(req_id)
            if st is None or st.num_prompt_tokens <= self.threshold or st.local_window_kv is None:
                continue
            if st.num_computed_tokens != st.num_prompt_tokens:
                continue
            assert st.remain_idx is not None
            blocks = requests[req_id].block_ids[0]
            ids = torch.tensor([blocks[x] for x in st.remain_idx[-local:]], dtype=torch.int32, device=self.device)
            layers, kv_stride, block_bytes, num_blocks = self._all_layers()
            ops.kv_scatter_blocks(layers, kv_stride, block_bytes, num_blocks, ids, st.local_window_kv)

    def maybe_register_kv_cache(self, forward_context, layer_name: str) -> None:
        attn = forward_context.no_compile_layers[layer_name]
        self._register_layer(self._layer_id(layer_name), attn.kv_cache[forward_context.virtual_engine])

    # ------------------------------------------------------------------ per-step metadata
    def build_sparse_meta(self, scheduler_output, requests, input_batch, attn_metadata) -> None:
        meta = GSAMetaData(self.block_size, getattr(self, "device", None))
        meta.gsa_stats = self.gsa_stats
        new_ids = {r.req_id for r in getattr(scheduler_output, "scheduled_new_reqs", [])}
        for req_id, n_tok in scheduler_output.num_scheduled_tokens.items():
            if req_id in new_ids and req_id in self.gsa_stats:
                self.request_finished_in_worker(req_id)  # id reused by a new request
            if not self.topk_kpre_manger.is_exist(req_id):
                if self.topk_kpre_manger.alloc(req_id) is None:
                    raise RuntimeError("more live requests than representative-table partitions")
            if req_id not in self.gsa_stats:
                self.gsa_stats[req_id] = GSAReqStat(
                    req_id, self.max_block_len * self.topk_kpre_manger.cache_map[req_id], self.block_size,
                    self.threshold)
            self.gsa_stats[req_id].update(n_tok, requests[req_id], input_batch.req_id_to_index[req_id],
                                          (self.min_topk, self.max_topk, self.topk_ratio) if self.ptopk_prefetch else None)
        self.gsa_metadata = meta
        self._sparse_metadata = meta
        self._fast = None
        if self.ptopk_prefetch:
            self._init_sparse_local_kv(scheduler_output, requests)

        batch = len(scheduler_output.num_scheduled_tokens)
        by_index: List[Optional[GSAReqStat]] = [None] * batch
        query_locals = [0] * (batch + 1)
        calc_blocks: List[int] = []
        calc_slots: List[int] = []
        for req_id, n_tok in scheduler_output.num_scheduled_tokens.items():
            st = self.gsa_stats[req_id]
            by_index[st.index_in_batch] = st
            query_locals[st.index_in_batch + 1] = n_tok
            calc_blocks += st.calc_block_table
            calc_slots += st.calc_repre_slot_mapping
        query_locals = list(accumulate(query_locals))
        self.model_input = {
            "calc_block_table": calc_blocks,
            "calc_repre_slot_mapping": calc_slots,
            "query_locals": query_locals,
            "batch": by_index,
        }

    def execute_begin(self, scheduler_output) -> None:
        """Packs this step's descriptors and sends them down in one copy."""
        by_index: List[Optional[GSAReqStat]] = self.model_input.get("batch", [])
        batch = len(by_index)
        gsa_ids = {st.req_id for st in by_index if st is not None and st.is_gsa()}
        any_gsa = bool(gsa_ids)
        self.model_input["any_gsa"] = any_gsa
        # score on every retrieval_stride-th step, and whenever a request is sparsified for the first time
        is_topk = any_gsa and (self.step_count % self.retrieval_stride == 0 or not gsa_ids <= self._scored)
        if any_gsa and self.ptopk_prefetch and self._dev_ready and self._prefetch_mode().round_due():
            is_topk = True                # the round at the end of this step reads this step's selection
        self.model_input["is_topk"] = is_topk
        self._fast = self._lagged = self._parking = None
        if is_topk:
            self._scored |= gsa_ids
        if not any_gsa or not self._dev_ready:
            return
        width = self.max_block_len
        n_calc = len(self.model_input["calc_block_table"])
        # The block tables go down only when a request's list changed or the batch was reordered (a decoding
        # request's list grows by one entry every block_size steps); the six descriptor rows and the block-mean
        # lists go down every step.  One int32 host buffer, one copy.
        signature = tuple((st.serial, st.blocks_version) if st is not None else None for st in by_index)
        tables_known = signature == self._tables_signature
        slot = self.step_count & 1
        if self._host_free[slot] is not None:
            self._host_free[slot].synchronize()  # upload of two steps ago; long finished
        n_tables = 0 if tables_known else batch * width
        host = self._host_desc[slot][: 6 * batch + n_tables + 2 * n_calc]
        hn = host.numpy()                    # the same pinned memory; numpy fills it several times faster than torch indexing
        desc = hn[: 6 * batch].reshape(6, batch)
        if not tables_known:
            tables = hn[6 * batch : 6 * batch + n_tables].reshape(batch, width)
            tables[:] = 0
        max_len = total = 0
        query_locals = self.model_input["query_locals"]
        rows = []                            # per request: first table row, blocks, k, its last query token, tokens so far, table partition
        min_topk, max_topk, ratio = self.min_topk, self.max_topk, self.topk_ratio
        for i, st in enumerate(by_index):
            if st is None:
                rows.append((0, 0, 0, 0, 0, -1))
                continue
            n = len(st.blocks)
            # k >= n keeps every block (short or prefilling requests)
            k = compute_topk_len(n, min_topk, max_topk, ratio) if st.is_gsa() else n
            rows.append((st.slot_offset, n, k if k > 1 else 1, query_locals[i + 1] - 1,
                         st.num_computed_tokens + st.num_scheduled_tokens, st.slot_offset // width))
            if not tables_known:
                tables[i, :n] = st.blocks
            if n > max_len:
                max_len = n
            total += n
        desc[:] = np.array(rows, dtype=np.int32).T
        tail = hn[6 * batch + n_tables :]
        tail[:n_calc] = self.model_input["calc_block_table"]
        tail[n_calc:] = self.model_input["calc_repre_slot_mapping"]
        dev = host.to(self.device, non_blocking=True)
        if self._host_free[slot] is None:
            self._host_free[slot] = torch.cuda.Event()
        self._host_free[slot].record()
        d = dev[: 6 * batch].view(6, batch)
        if not tables_known:
            self._tables_dev = dev[6 * batch : 6 * batch + n_tables].view(batch, width)
            self._tables_signature = signature
        self.model_input.update(
            seg_off=d[0], seg_len=d[1], topk_len=d[2], q_rows=d[3], seq_lens=d[4],
            block_tables=self._tables_dev,
            calc_blocks_dev=dev[6 * batch + n_tables : 6 * batch + n_tables + n_calc],
            calc_slots_dev=dev[6 * batch + n_tables + n_calc :],
            max_len=max_len, total=total, n_batch=batch,
        )
        base = d.data_ptr()
        self.model_input["addr"] = (base, base + 4 * batch, base + 8 * batch, base + 12 * batch, base + 16 * batch,
                                    self._tables_dev.data_ptr())
        a = self._sel
        a.seg_off, a.seg_len, a.topk_len, a.q_rows, a.seq_lens, a.block_tables = self.model_input["addr"]
        a.n_req, a.max_seg_len, a.total_blocks = batch, max_len, total
        lag = self.retrieval_lag and not self.ptopk_prefetch and self._fused_ok and _raw_stream is not None
        if lag and (self.retrieval_stride == 1 or (self.step_count + 1) % self.retrieval_stride == 0):
            # the step after may select with this step's queries: every layer keeps them
            self._parking = ({st.req_id for st in by_index if st is not None}, base + 12 * batch, base + 20 * batch, batch)
        if self.ptopk_prefetch:
            # attention reads the engine's tables; the selection is kept as logical block numbers for the next round
            a.block_tables = a.phys_out = a.sparse_seq_lens = None
            self._prefetch_mode().begin_step(by_index)
        elif lag and is_topk and self.q_stage is not None and gsa_ids <= self._parked:
            # every sparsified request's queries of the step before are at hand: one launch for all layers, now
            b = self._sel_all
            b.seg_off, b.seg_len, b.topk_len, b.seq_lens, b.block_tables = a.seg_off, a.seg_len, a.topk_len, a.seq_lens, a.block_tables
            b.q_rows = base + 20 * batch
            b.n_req, b.max_seg_len, b.total_blocks = batch, max_len, total
            rc = self._score_select(ctypes.addressof(b), _raw_stream(self._dev_index))
            if rc != 0:
                raise _lib.UcmHipError("ucm_score_select", rc, _lib.lib().ucm_last_error().decode())
            self._lagged = self._batch_views(batch)
        elif is_topk and self._fused_ok and _raw_stream is not None:
            self._fast = self._batch_views(batch)

    def _batch_views(self, n: int) -> list:
        """Per layer: (sparse block table, sparse sequence lengths) of a batch of n requests."""
        views = self._views.get(n)
        if views is None:
            views = self._views[n] = [(self.block_tables_mp[k, :n], self.gsa_seq_len[k, :n]) for k in range(self.layer_num)]
        return views

    def execute_finished(self) -> None:
        if self.ptopk_prefetch:
            self._gsa_sparse_local_kv()
            if self._pf is not None:
                self._pf.end_step()
        self._parked = self._parking[0] if self._parking is not None else set()
        self._parking = None
        self.step_count += 1

    # ------------------------------------------------------------------ per-layer hooks
    def _layer_id(self, layer_name: str) -> int:
        l = self._layer_of.get(layer_name)
        if l is None:
            l = self._layer_of[layer_name] = int(layer_name.split(".")[2])
        return l

    def attention_begin(self, query, key, value, layer_name: str, forward_context) -> None:
        # the layer's cache is looked at when the engine's table of layers is not the one seen before (the caches are
        # allocated once; the reference re-reads them in every hook, gsa.py:866-877)
        layers = forward_context.no_compile_layers
        if layers is not self._seen_layers or layer_name not in self._layer_of:
            self.maybe_register_kv_cache(forward_context, layer_name)
            if len(self._kv_full) == self.layer_num:
                self._seen_layers = layers
        parking = self._parking
        if parking is not None:
            # the last query token of every request goes to the request's row of the kept queries of this layer
            # (copy_q, gsa.py:616-632), for the selection the next step makes before its model runs
            l = self._layer_of[layer_name]
            if self.q_stage is None:
                self._make_stage(query)
            if query.dtype is not self._stage_dtype or query.shape[1:] != self._stage_row or not query.is_contiguous():
                raise ValueError("query must be a contiguous device tensor [tokens, q_heads, head_size] of the type the first step had")
            rc = self._park_rows(query.data_ptr(), query.shape[0], parking[1], self._stage_addr[l], self.max_bs, parking[2],
                                 parking[3], self._stage_row_bytes, _raw_stream(self._dev_index))
            if rc != 0:
                raise _lib.UcmHipError("ucm_park_rows", rc, _lib.lib().ucm_last_error().decode())
        if self._lagged is not None:
            md = forward_context.attn_metadata
            if isinstance(md, dict):
                md = md[layer_name]
            md.block_table, md.seq_lens = self._lagged[self._layer_of[layer_name]]
            return
        fast = self._fast
        if fast is not None:
            # the step scores and selects with the one-launch call: everything but the layer and its queries was
            # filled in by execute_begin
            l = self._layer_of[layer_name]
            q_code = _Q_CODES.get(query.dtype)
            if q_code is None or not query.is_contiguous() or query.shape[-1] != self.head_size:
                raise ValueError("query must be a contiguous bfloat16, float16 or float32 device tensor [tokens, q_heads, head_size]")
            a = self._sel
            a.q, a.q_dtype, a.q_layer_stride, a.first_layer = query.data_ptr(), q_code, query.numel(), l
            rc = self._score_select(self._sel_addr, _raw_stream(self._dev_index))
            if rc != 0:
                raise _lib.UcmHipError("ucm_score_select", rc, _lib.lib().ucm_last_error().decode())
            md = forward_context.attn_metadata
            if isinstance(md, dict):
                md = md[layer_name]
            md.block_table, md.seq_lens = fast[l]
            return
        mi = self.model_input
        if not mi.get("any_gsa") or "seg_off" not in mi:
            return
        l = self._layer_of[layer_name]
        n = mi["n_batch"]
        stream = _raw_stream(self._dev_index) if _raw_stream is not None else ops.current_stream()
        if mi["is_topk"]:
            q_code = _Q_CODES.get(query.dtype)
            if q_code is None:
                raise ValueError("query must be bfloat16, float16 or float32")
            if not (query.is_cuda and query.is_contiguous()) or query.shape[-1] != self.head_size:
                raise ValueError("query must be a contiguous device tensor [tokens, q_heads, head_size]")
        if mi["is_topk"] and self._fused_ok:
            # scores of every block and the selection from them: one launch (the last scoring workgroup of a
            # request runs its selection), block-table lookup and sparse lengths on the way out
            a = self._sel
            a.q, a.q_dtype, a.q_layer_stride, a.first_layer = query.data_ptr(), q_code, query.numel(), l
            rc = self._score_select(self._sel_addr, stream)
            if rc != 0:
                raise _lib.UcmHipError("ucm_score_select", rc, _lib.lib().ucm_last_error().decode())
        elif mi["is_topk"] or not self.ptopk_prefetch:
            seg_off, seg_len, topk_len, q_rows, seq_lens, tables = mi["addr"]
            repre, scores, idx, counts, phys, sparse_len = self._layer_addr[l]
            if self.ptopk_prefetch:
                tables = phys = sparse_len = None
            rows = self.kpre_caches.shape[1]
            if mi["is_topk"]:
                _lib.call("ucm_score_blocks", query.data_ptr(), q_code, query.numel(), q_rows, self.num_q_heads, repre,
                          self._repre_code, self.kpre_caches.stride(0), rows, 1, seg_off, seg_len, n, mi["max_len"],
                          mi["total"], 1, self.num_key_heads, self.head_size, scores, self.scores.stride(0), 1.0, 0, stream)
            # selection from the last scores with this step's lengths, block-table lookup, sparse lengths
            _lib.call("ucm_topk_windows", scores, self.scores.stride(0), rows, seg_off, seg_len, topk_len, n, mi["max_len"],
                      1, self.init_window, self.local_window, idx, self.max_block_len, counts, tables, self.max_block_len,
                      phys, seq_lens, self.block_size, sparse_len, stream)
        md = forward_context.attn_metadata
        md = md[layer_name] if isinstance(md, dict) else md
        if self.ptopk_prefetch:
            md.block_table, md.seq_lens = self._pf.bt_step[l], self._pf.seq_step[l]
        else:
            md.block_table, md.seq_lens = self._batch_views(n)[l]

    def _make_stage(self, query) -> None:
        """The kept queries [layers, table partitions, q_heads, head_size], in the type of the model's queries."""
        if _Q_CODES.get(query.dtype) is None:
            raise ValueError("query must be bfloat16, float16 or float32")
        stage = self.q_stage = torch.zeros((self.layer_num, self.max_bs, self.num_q_heads, self.head_size),
                                           dtype=query.dtype, device=self.device)
        b = self._sel_all
        b.q, b.q_dtype, b.q_layer_stride = stage.data_ptr(), _Q_CODES[query.dtype], stage.stride(0)
        self._stage_dtype, self._stage_row = query.dtype, stage.shape[2:]
        self._stage_row_bytes = stage.stride(1) * stage.element_size()
        self._stage_addr = [stage[l].data_ptr() for l in range(self.layer_num)]

    def attention_finished(self, query, key, value, attn_output, layer_name: str, forward_context) -> None:
        # (the layer's cache was looked at in attention_begin of the same step)
        if self.model_input.get("calc_block_table"):
            self.copy_k(layer_name, forward_context)
            if self.ptopk_prefetch:
                l = self._layer_id(layer_name)
                self._prefetch_mode().save_blocks(l, self._kv_full[l])

    def copy_k(self, layer_name: str, forward_context) -> None:
        """Representatives of the blocks this step filled (gsa.py:634-654), reduced in place on the device."""
        blocks = self.model_input.get("calc_block_table") or []
        if not blocks:
            return
        l = self._layer_id(layer_name)
        if "calc_blocks_dev" in self.model_input:
            ids, slots = self.model_input["calc_blocks_dev"], self.model_input["calc_slots_dev"]
        else:  # a step without any sparsified request still has to keep the table current
            ids = torch.tensor(blocks, dtype=torch.int32, device=self.device)
            slots = torch.tensor(self.model_input["calc_repre_slot_mapping"], dtype=torch.int32, device=self.device)
            self.model_input["calc_blocks_dev"], self.model_input["calc_slots_dev"] = ids, slots
        k_cache = self.k_cache[l]
        ops.block_mean(self._layer_ptrs[l], ids, slots, self.kpre_caches[l : l + 1], self.block_size,
                       self.num_key_heads, self.head_size, k_cache.shape[0], mode=self.repre_mode)

    def request_finished_in_worker(self, request_id: ReqType) -> None:
        self.topk_kpre_manger.free(request_id)
        self.gsa_stats.pop(request_id, None)
        self._scored.discard(request_id)
        self._parked.discard(request_id)
        if self._pf is not None:
            self._pf.request_finished(request_id)

    # ------------------------------------------------------------------ scheduler side
    def request_begin(self, request_id: ReqType, prompt_token_ids: List[int]) -> None:
        pass

    def estimate_num_slots_sparsed(self, request) -> int:
        """Token slots of a sparsified request (gsa.py:891-912): the blocks decoded so far plus max_topk + 1 sparse
        blocks, minus the unused tail of the last block.  INVALID_SLOT unless prefetch mode is on (the reference's
        PTOPK_PREFETCH_ENABLE is off as shipped), during prefill and for prompts below the threshold."""
        if not self.ptopk_prefetch or request.num_output_tokens == 0 or request.num_prompt_tokens <= self.threshold:
            return INVALID_SLOT
        bs = self.block_size
        num_prompt_blocks = math.ceil(request.num_prompt_tokens / bs)
        num_all_blocks = math.ceil(request.num_tokens / bs)
        topk_len = compute_topk_len(num_prompt_blocks, self.min_topk, self.max_topk, self.topk_ratio)
        prefetch_len = 0 if topk_len > self.max_topk else self.max_topk - topk_len + 1
        num_sparse_blocks = num_all_blocks - num_prompt_blocks + topk_len + prefetch_len
        flaw = request.num_tokens % bs
        return num_sparse_blocks * bs - (bs - flaw if flaw else 0)

    def allocate_slots(self, request, num_slots_sparsed, coordinator, block_pool, kv_cache_groups):
        """Prefetch mode, scheduler side.  The reference leaves this to the base class, which does nothing; what its
        worker side assumes (_first_topk_deal reads the resident blocks at positions 0 .. max_topk of the request's
        block list, prefetch_engine.py:327-379) is written out here: at its first decode step a long request keeps
        its first ``max_topk + 1`` blocks - they still hold logical blocks 0 .. max_topk - and whatever it holds
        beyond its prompt's blocks, returns the rest to the pool, and is then allocated for the sparsified length."""
        blocks = coordinator.get_blocks(request.request_id)[0]
        kept = list(blocks)
        if request.num_computed_tokens == request.num_prompt_tokens:
            n_prompt = math.ceil(request.num_prompt_tokens / self.block_size)
            k = self._topk_len(n_prompt)
            keep = k + (0 if k > self.max_topk else self.max_topk - k + 1)
            kept, returned = list(blocks[:keep]) + list(blocks[n_prompt:]), list(blocks[keep:n_prompt])
            for block in blocks:
                block_pool._maybe_evict_cached_block(block)
            block_pool.free_blocks(returned)
            coordinator.single_type_managers[0].req_to_blocks[request.request_id] = kept
        empty = tuple([] for _ in range(len(kv_cache_groups)))
        n_new = coordinator.get_num_blocks_to_allocate(request_id=request.request_id, num_tokens=num_slots_sparsed,
                                                       new_computed_blocks=empty)
        if n_new > block_pool.get_num_free_blocks():
            return None
        coordinator.allocate_new_blocks(request.request_id, num_slots_sparsed)
        from ..esa.esa import _kv_cache_blocks

        return _kv_cache_blocks(kept)
