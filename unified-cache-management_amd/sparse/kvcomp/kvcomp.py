"""KvComp-shaped sparse-attention plugin: hash-code retrieval per request and
layer, selected blocks loaded from a KV store into the request's cache blocks.

Follows the reference's ``KvComp`` (ucm/sparse/kvcomp/kvcomp.py:432-587) and its
``ReqStatePerLayer`` (:157-429) hook for hook:

* ``attention_finished`` - every block that became full is dumped to the store
  under ``req_<id>_blk_<n>`` and hashed (``save_blocks`` :325-347); at the last
  prefill chunk the first ``init_window_sz`` and last ``local_window_sz`` blocks
  are kept aside (``construct_init_and_local_window`` :260-274);
* ``attention_begin`` on decode steps with ``step % retrieval_stride == 1``
  (:361-389) - the windows are written back once (``prepare_init_and_local_window``
  :392-404), the blocks between them are scored against the step's query and
  the best ``len(vllm_block_ids[init:-local])`` are loaded into those cache
  blocks, ascending.

What changes underneath: a block's representation is not its 16 KiB of token
codes but the 2 KiB of per-(head, bit) column sums S[h][c] = #ones - #zeros over
the block's tokens, because the reference's score
    sum over (query head i, kv head j, token s) of <+-1(q_i), +-1(k_js)>   (:237-247)
equals <sum_i u(q_i), sum_j S[j]> exactly in integers; codes, sums, scores and
the selection are one kernel each.  The reference evaluates that sum in fp16;
``fp16_scores`` (default on) rounds the exact integer to fp16 once, which is what
an exact fp16 evaluation would return; ties are broken towards the lower block.
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Union

import torch

from ... import ops
from ..base import INVALID_SLOT, UcmSparseBase, UcmSparseMetadata, UcmSparseRole
from ..esa.esa import get_offset
from .device_path import KvCompDevicePath
from .hash_encoder import HashEncoder

ReqType = Union[str, int]

INIT_WINDOW_SZ = 1
LOCAL_WINDOW_SZ = 2
SPARSE_RATIO = 0.3
RETRIEVAL_STRIDE = 4


@dataclass
class ReqMeta:
    request_id: ReqType
    index_in_batch: int
    num_prompt_tokens: int
    num_output_tokens: int
    num_scheduled_tokens: int
    num_computed_tokens: int
    num_sparsed_tokens: int
    vllm_block_ids: List[int]

    @property
    def step(self) -> int:
        return self.num_output_tokens

    @property
    def is_prefill(self) -> bool:
        return self.num_output_tokens == 0

    @property
    def is_last_chunk(self) -> bool:
        return self.num_computed_tokens + self.num_scheduled_tokens >= self.num_prompt_tokens


@dataclass
class KvCompSparseMetaData(UcmSparseMetadata):
    requests: List[ReqMeta] = field(default_factory=list)
    finished_req_ids: List[ReqType] = field(default_factory=list)

    def add_request(self, *args, **kwargs) -> None:
        self.requests.append(ReqMeta(*args, **kwargs))


class ReqStatePerLayer:
    """One request in one layer (kvcomp.py:157-429)."""

    def __init__(self, req_meta: ReqMeta, layer_name: str, rank: int, tp_size: int, store_instance, plugin: "KvComp"):
        self.layer_name = layer_name
        self.layer_id = int(layer_name.split(".")[2])
        self.req_meta = req_meta
        self.rank, self.tp_size = rank, tp_size
        self.store_instance = store_instance
        self.plugin = plugin
        self.init_window_sz, self.local_window_sz = plugin.cfg["init_window_sz"], plugin.cfg["local_window_sz"]
        self.num_blocks_hashed = 0                       # rows of this request's segment that hold a block
        self.init_window = self.local_window = None
        self.block_size = None
        self.k_cache = self.v_cache = None
        self.tasks: Dict[int, object] = {}
        self._last_selection: Optional[List[int]] = None

    @property
    def last_selection(self) -> Optional[List[int]]:
        """Logical block ids of the last retrieval, ascending (read back from the device tables when the batched
        path made it)."""
        dev = self.plugin._dev
        got = dev.selection(self.layer_id, self.req_meta.request_id) if dev is not None else None
        return self._last_selection if got is None else got

    @classmethod
    def block_hash(cls, request_id, block_id) -> str:
        return f"req_{request_id}_blk_{block_id}"

    def update_meta(self, req_meta: ReqMeta) -> None:
        self.req_meta = req_meta

    def maybe_register_kv_cache(self, forward_context) -> None:
        if self.block_size:
            return
        attn = forward_context.no_compile_layers[self.layer_name]
        kv_cache = attn.kv_cache[forward_context.virtual_engine]
        self.k_cache, self.v_cache = kv_cache[0], kv_cache[1]
        self.block_size = self.k_cache.shape[1]
        self.num_key_heads, self.head_size = self.k_cache.shape[2], self.k_cache.shape[3]
        self.plugin.register_layer_cache(self.layer_id, self.k_cache, kv_cache)

    # ---- retrieval -----------------------------------------------------------------------
    def retrieval(self, query: torch.Tensor, top_k: int) -> List[str]:
        n_blocks = self.num_blocks_hashed
        first, end = self.init_window_sz, n_blocks - self.local_window_sz + 1
        if top_k >= n_blocks:
            chosen = list(range(first, end))
        elif end <= first or top_k <= 0:
            chosen = []
        else:
            ntokens, num_q_heads, _ = query.shape
            if num_q_heads > self.num_key_heads:
                query = query.view(ntokens, self.num_key_heads, -1, self.head_size).mean(2)
            elif num_q_heads < self.num_key_heads:
                query = torch.repeat_interleave(query, self.num_key_heads // num_q_heads, 1)
            picked = self.plugin.score_and_select(self.layer_id, self.req_meta.request_id, query, first, end - first,
                                                  min(top_k, end - first))
            chosen = [first + int(i) for i in picked]
        self._last_selection = chosen
        return [self.block_hash(self.req_meta.request_id, b) for b in chosen]

    # ---- windows -------------------------------------------------------------------------
    def construct_init_and_local_window(self) -> None:
        ids = self.req_meta.vllm_block_ids
        head = ids[: self.init_window_sz]
        self.init_window = (self.k_cache[head].clone(), self.v_cache[head].clone())
        n_local = min(self.local_window_sz, len(ids[self.init_window_sz:]))
        if n_local > 0:
            tail = ids[-n_local:]
            self.local_window = (self.k_cache[tail].clone(), self.v_cache[tail].clone())

    def prepare_init_and_local_window(self) -> None:
        if self.req_meta.step != 1 or self.init_window is None:
            return
        ids = self.req_meta.vllm_block_ids
        self.k_cache[ids[: self.init_window_sz]] = self.init_window[0]
        self.v_cache[ids[: self.init_window_sz]] = self.init_window[1]
        if self.local_window is None:
            return
        n_local = self.local_window[0].shape[0]
        self.k_cache[ids[-n_local:]] = self.local_window[0]
        self.v_cache[ids[-n_local:]] = self.local_window[1]

    # ---- transfers -----------------------------------------------------------------------
    def launch_transfer_task(self, transfer_type: str, block_hashes: List[str], vllm_block_ids: List[int]) -> None:
        n = min(len(block_hashes), len(vllm_block_ids))
        if n == 0:
            return
        block_hashes, vllm_block_ids = block_hashes[:n], vllm_block_ids[:n]
        fn = getattr(self.store_instance, transfer_type)
        shape = (self.block_size, self.num_key_heads, self.head_size)
        precision = self.k_cache.element_size()
        off_k = [get_offset(shape, self.rank, self.tp_size, precision, self.layer_id, False)] * n
        off_v = [get_offset(shape, self.rank, self.tp_size, precision, self.layer_id, True)] * n
        self.tasks[hash((tuple(block_hashes), transfer_type, "key"))] = fn(
            block_hashes, off_k, [self.k_cache[i] for i in vllm_block_ids])
        self.tasks[hash((tuple(block_hashes), transfer_type, "value"))] = fn(
            block_hashes, off_v, [self.v_cache[i] for i in vllm_block_ids])

    def wait_for_task_done(self) -> None:
        for task in self.tasks.values():
            self.store_instance.wait(task)
        self.tasks.clear()

    def blocks_to_save(self, num_blocks_need_dump: int):
        """(cache blocks, their logical numbers) that became full (kvcomp.py:325-335), counted as saved."""
        if num_blocks_need_dump <= 0:
            return [], []
        ids = self.req_meta.vllm_block_ids
        done = self.num_blocks_hashed
        logical = list(range(done, done + num_blocks_need_dump))
        if self.req_meta.is_prefill:
            physical = ids[done : done + num_blocks_need_dump]
        else:
            physical = ids[-1:]
            logical = logical[:1]
        self.num_blocks_hashed += len(logical)
        return physical, logical

    def save_blocks(self, num_blocks_need_dump: int) -> None:
        physical, logical = self.blocks_to_save(num_blocks_need_dump)
        if not logical:
            return
        hashes = [self.block_hash(self.req_meta.request_id, b) for b in logical]
        self.launch_transfer_task("dump", hashes, physical)
        self.plugin.hash_blocks(self.layer_id, self.req_meta.request_id, physical, logical)

    # ---- hooks ---------------------------------------------------------------------------
    def attention_begin(self, query, key, value, forward_context) -> None:
        if self.req_meta.step % self.plugin.cfg["retrieval_stride"] != 1 or not self.block_size:
            return
        attn_md = forward_context.attn_metadata
        if isinstance(attn_md, dict):
            attn_md = attn_md[self.layer_name]
        a = int(attn_md.query_start_loc[self.req_meta.index_in_batch])
        current_query = query[a : a + self.req_meta.num_scheduled_tokens]
        mid = self.req_meta.vllm_block_ids[self.init_window_sz : -self.local_window_sz]
        self.wait_for_task_done()
        self.prepare_init_and_local_window()
        hashes = self.retrieval(current_query, len(mid))
        self.launch_transfer_task("load", hashes, mid)
        self.wait_for_task_done()

    def attention_finished(self, query, key, value, attn_output, forward_context, batch=None) -> None:
        """batch: a list the blocks to save are appended to instead of being dumped and hashed here (the plugin
        then saves the blocks of all requests of the layer at once)."""
        self.maybe_register_kv_cache(forward_context)
        updated = self.req_meta.num_computed_tokens + self.req_meta.num_scheduled_tokens
        n = updated // self.block_size - self.num_blocks_hashed
        if batch is None:
            self.save_blocks(n)
        else:
            physical, logical = self.blocks_to_save(n)
            if logical:
                batch.append((self.req_meta.request_id, physical, logical))
        if self.req_meta.is_prefill and self.req_meta.is_last_chunk:
            if batch is None:
                self.construct_init_and_local_window()
            self.wait_for_task_done()


class KvComp(UcmSparseBase):
    def __init__(self, vllm_config, role: UcmSparseRole, store=None):
        super().__init__(vllm_config, role)
        mc, pc = vllm_config.model_config, vllm_config.parallel_config
        self.rank = getattr(pc, "rank", 0)
        self.tp_size = getattr(pc, "tensor_parallel_size", 1)
        self.block_size = vllm_config.cache_config.block_size
        extra = vllm_config.kv_transfer_config.kv_connector_extra_config
        self.cfg = dict(extra.get("ucm_sparse_config", {}).get("KvComp", {}))
        path = extra.get("kvcomp_config_path")
        if path:                                           # the reference's JSON (kvcomp_config.py): head_dim, hash_bits
            with open(path) as f:
                js = json.load(f)
            self.cfg.setdefault("head_dim", js.get("head_dim", 128))
            self.cfg.setdefault("hash_bits", js.get("hash_bits", 128))
            # the reference refuses a file written for another model (kvcomp.py:458-464)
            n_model = getattr(getattr(mc, "hf_text_config", None), "num_hidden_layers", None)
            n_file = js.get("num_hidden_layers")
            assert n_model is None or n_file is None or n_file == n_model, (
                f"kvcomp_config.num_hidden_layers {n_file} != "
                f"vllm_config.model_config.hf_text_config.num_hidden_layers {n_model}")
        for key, default in (("init_window_sz", INIT_WINDOW_SZ), ("local_window_sz", LOCAL_WINDOW_SZ),
                             ("sparse_ratio", SPARSE_RATIO), ("retrieval_stride", RETRIEVAL_STRIDE),
                             ("hash_bits", 128), ("fp16_scores", True), ("keep_token_codes", False)):
            self.cfg.setdefault(key, default)
        self.num_key_heads = mc.get_num_kv_heads(pc)
        self.head_size = mc.get_head_size()
        self.cfg.setdefault("head_dim", self.head_size)
        self.total_num_hidden_layers = mc.get_num_layers(pc)
        self.max_blocks = -(-mc.max_model_len // self.block_size)
        self.max_num_seqs = vllm_config.scheduler_config.max_num_seqs
        self.connector = store                            # anything with the UcmKVStoreBase load / dump / wait methods
        self.req_states: Dict[ReqType, List[Optional[ReqStatePerLayer]]] = {}
        self.segment_of: Dict[ReqType, int] = {}
        self.free_segments = list(range(self.max_num_seqs - 1, -1, -1))
        self.hash_encoder: Optional[HashEncoder] = None
        self.colsum = self.block_codes = self.token_codes = None
        self._layer_ptrs: Dict[int, ops.LayerPointers] = {}
        self._num_blocks: Dict[int, int] = {}
        # "device_loads": the batched retrieval step that scores, selects and loads on the device for all requests
        # of a layer at once (needs a store whose blocks a kernel can read, i.e. one with device_pool()); False
        # keeps the per-request path, which works with any store
        # (the stored-block layout the kernels address is the one of a single rank, get_offset with tp_size 1)
        self._device_loads = bool(self.cfg.get("device_loads", True)) and self.tp_size == 1
        self._dev: Optional[KvCompDevicePath] = None
        self._dev_step_built = True
        self._quiet = False
        self._kv_caches: Dict[int, torch.Tensor] = {}

    # ---- device tables -------------------------------------------------------------------
    def register_layer_cache(self, layer_id: int, k_cache: torch.Tensor, kv_cache: Optional[torch.Tensor] = None) -> None:
        dev = k_cache.device
        if kv_cache is not None:
            self._kv_caches[layer_id] = kv_cache
            if self._dev is not None:
                self._dev.register_kv_cache(layer_id, kv_cache)
        if self.hash_encoder is None:
            self.hash_encoder = HashEncoder(self.cfg["head_dim"], self.cfg["hash_bits"], k_cache.dtype, dev)
            L, rows, h = self.total_num_hidden_layers, self.max_num_seqs * self.max_blocks, self.num_key_heads
            self.colsum = torch.zeros((L, rows, h, 128), dtype=torch.int16, device=dev)
            self.block_codes = torch.zeros((L, rows, h, 16), dtype=torch.uint8, device=dev)
            if self.cfg["keep_token_codes"]:
                self.token_codes = torch.zeros((L, rows, self.block_size, h, 16), dtype=torch.uint8, device=dev)
            self.scores = torch.zeros((L, rows), dtype=torch.float32, device=dev)
        if layer_id not in self._layer_ptrs or self._layer_ptrs[layer_id].tensors[0].data_ptr() != k_cache.data_ptr():
            self._layer_ptrs[layer_id] = ops.LayerPointers([k_cache])
            self._num_blocks[layer_id] = k_cache.shape[0]

    def segment_base(self, request_id: ReqType) -> int:
        if request_id not in self.segment_of:
            assert self.free_segments, "more sparsified requests than max_num_seqs"
            self.segment_of[request_id] = self.free_segments.pop()
        return self.segment_of[request_id] * self.max_blocks

    def hash_blocks(self, layer_id: int, request_id: ReqType, physical: List[int], logical: List[int]) -> None:
        """Codes and column sums of cache blocks ``physical`` into rows base + ``logical`` of the layer's tables."""
        dev = self.colsum.device
        base = self.segment_base(request_id)
        ids = torch.tensor(physical, dtype=torch.int32, device=dev)
        slots = torch.tensor([base + b for b in logical], dtype=torch.int32, device=dev)
        l = slice(layer_id, layer_id + 1)
        self.hash_encoder.encode_cache_blocks(self._layer_ptrs[layer_id], ids, slots, self.block_size, self.num_key_heads,
                                              self._num_blocks[layer_id], self.colsum[l], self.block_codes[l],
                                              None if self.token_codes is None else self.token_codes[l])

    def score_and_select(self, layer_id: int, request_id: ReqType, query: torch.Tensor, first: int, count: int,
                         top_k: int) -> List[int]:
        """query [tokens, kv_heads, head_size] (group means); scores blocks first .. first+count-1 of the
        request and returns the top_k of them, as offsets from ``first``, ascending."""
        dev = self.colsum.device
        t, h, d = query.shape
        q = query.to(self.hash_encoder.dtype).reshape(1, 1, t * h, d).contiguous()
        q_codes = torch.empty((1, 1, t * h, 16), dtype=torch.uint8, device=dev)
        q_sum = torch.empty((1, 1, 128), dtype=torch.int16, device=dev)
        qbar = torch.empty((1, 1, h, 16), dtype=torch.uint8, device=dev)
        ops.hash_encode_queries(q, self.hash_encoder.hash_weights, h, q_codes, q_sum, qbar, 1)
        base = self.segment_base(request_id)
        seg_off = torch.tensor([base + first], dtype=torch.int32, device=dev)
        seg_len = torch.tensor([count], dtype=torch.int32, device=dev)
        l = slice(layer_id, layer_id + 1)
        ops.hash_score_blocks(0, q_sum, qbar, self.colsum[l], self.block_codes[l], seg_off, seg_len, count, self.scores[l],
                              round_fp16=bool(self.cfg["fp16_scores"]))
        idx = torch.empty((1, 1, count), dtype=torch.int32, device=dev)
        cnt = torch.empty((1, 1), dtype=torch.int32, device=dev)
        ops.topk_windows(self.scores[l], seg_off, seg_len, torch.tensor([top_k], dtype=torch.int32, device=dev), count,
                         idx, cnt, start_w=0, end_w=0)
        n = int(cnt[0, 0])
        return idx[0, 0, :n].tolist()

    # ---- worker hooks ----------------------------------------------------------------------
    def _state(self, req_meta: ReqMeta, layer_name: str) -> ReqStatePerLayer:
        layer_id = int(layer_name.split(".")[2])
        states = self.req_states.setdefault(req_meta.request_id, [None] * self.total_num_hidden_layers)
        if states[layer_id] is None:
            states[layer_id] = ReqStatePerLayer(req_meta, layer_name, self.rank, self.tp_size, self.connector, self)
        return states[layer_id]

    def _batched(self, layer_name: str, forward_context) -> Optional[KvCompDevicePath]:
        """The batched path (created at the first hook that sees a device-addressable store), with this layer's
        cache registered; None when the store's blocks cannot be read by a kernel."""
        if not self._device_loads or not hasattr(self.connector, "device_pool"):
            return None
        layer_id = int(layer_name.split(".")[2])
        if layer_id not in self._kv_caches:
            kv_cache = forward_context.no_compile_layers[layer_name].kv_cache[forward_context.virtual_engine]
            self.register_layer_cache(layer_id, kv_cache[0], kv_cache)
        if self._dev is None:
            pool, pool_block_bytes = self.connector.device_pool()
            self._dev = KvCompDevicePath(self, pool, pool_block_bytes, self.colsum.device)
            for l, kv in self._kv_caches.items():
                self._dev.register_kv_cache(l, kv)
        return self._dev

    def _device_step(self, layer_name: str, forward_context) -> Optional[KvCompDevicePath]:
        """The batched path, with this step's descriptor built (at the step's first hook: the token positions come
        with the forward context), or None when the store's blocks cannot be read by a kernel."""
        if self._batched(layer_name, forward_context) is None:
            return None
        if not self._dev_step_built:
            attn_md = forward_context.attn_metadata
            if isinstance(attn_md, dict):
                attn_md = attn_md[layer_name]
            starts = attn_md.query_start_loc.tolist()
            metas = self._sparse_metadata.requests
            self._dev.build_step(metas, [int(starts[m.index_in_batch]) for m in metas])
            self._dev_step_built = True
        return self._dev

    def attention_begin(self, query, key, value, layer_name: str, forward_context) -> None:
        if self._quiet:
            return
        dev = self._device_step(layer_name, forward_context)
        batched = set(dev.active) if dev is not None else ()
        for req_meta in self._sparse_metadata.requests:
            st = self._state(req_meta, layer_name)
            st.update_meta(req_meta)
            if req_meta.request_id in batched:          # dumps done and windows back in place, then one call for all
                st.wait_for_task_done()
                st.prepare_init_and_local_window()
            else:
                st.attention_begin(query, key, value, forward_context)
        if dev is not None:
            layer_id = int(layer_name.split(".")[2])
            first = [m for m in self._sparse_metadata.requests if m.step == 1 and m.request_id in dev.windows]
            if first:
                dev.restore_windows(layer_id, self._sparse_metadata, first)
            if batched:
                dev.attention_begin(layer_id, query)

    def attention_finished(self, query, key, value, attn_output, layer_name: str, forward_context) -> None:
        # with a device-addressable store the full blocks of all requests are dumped and hashed in one go, and the
        # windows of those that finish their prefill copied aside in one go
        if self._quiet:
            return
        dev = self._batched(layer_name, forward_context)
        batch = [] if dev is not None else None
        for req_meta in self._sparse_metadata.requests:
            st = self._state(req_meta, layer_name)
            st.update_meta(req_meta)
            st.attention_finished(query, key, value, attn_output, forward_context, batch)
        layer_id = int(layer_name.split(".")[2])
        if dev is not None:
            ending = [m for m in self._sparse_metadata.requests if m.is_prefill and m.is_last_chunk]
            if ending:
                dev.save_windows(layer_id, self._sparse_metadata, ending)
        if batch:
            if not dev.save_blocks(layer_id, self._sparse_metadata, batch):      # the store is full: block by block
                for request_id, physical, logical in batch:
                    st = self.req_states[request_id][layer_id]
                    st.launch_transfer_task("dump", [st.block_hash(request_id, b) for b in logical], physical)
                    self.hash_blocks(layer_id, request_id, physical, logical)

    def build_sparse_meta(self, scheduler_output, requests, input_batch, attn_metadata=None) -> None:
        meta = KvCompSparseMetaData()
        sparsed = getattr(scheduler_output, "req_sparsed_slots", {}) or {}
        for req_id, n_tok in scheduler_output.num_scheduled_tokens.items():
            req = requests[req_id]
            if len(req.prompt_token_ids) > self.block_size:
                meta.add_request(req_id, input_batch.req_id_to_index[req_id], len(req.prompt_token_ids),
                                 len(req.output_token_ids), n_tok, req.num_computed_tokens,
                                 sparsed.get(req_id, INVALID_SLOT), req.block_ids[0])
        self._sparse_metadata = meta
        self._dev_step_built = False
        self._quiet = self._quiet_step(meta.requests)

    def _quiet_step(self, metas) -> bool:
        """True when no hook of this step has anything to do on the batched path: every request decodes, none is at
        a retrieval step or at its first decode step (windows), none fills a block, and every layer has seen every
        request before.  The hooks then return at once instead of walking the requests in every layer (three decode
        steps of four with the default stride)."""
        if self._dev is None:
            return False
        stride, bs = self.cfg["retrieval_stride"], self.block_size
        for m in metas:
            states = self.req_states.get(m.request_id)
            if m.is_prefill or m.step % stride == 1 or states is None or any(st is None or not st.block_size for st in states):
                return False
            if (m.num_computed_tokens + m.num_scheduled_tokens) // bs > states[0].num_blocks_hashed or states[0].tasks:
                return False
        return True

    def request_finished_in_worker(self, request_id: ReqType) -> None:
        self.req_states.pop(request_id, None)
        if self._dev is not None:
            self._dev.request_finished(request_id)
        if request_id in self.segment_of:
            self.free_segments.append(self.segment_of.pop(request_id))

    # ---- scheduler side ----------------------------------------------------------------------
    def request_begin(self, request_id: ReqType, prompt_token_ids: List[int]) -> None:
        pass

    def estimate_num_slots_sparsed(self, request) -> int:
        """kvcomp.py:571-587."""
        if request.num_output_tokens == 0 or request.num_prompt_tokens < self.block_size:
            return INVALID_SLOT
        num_blocks = math.ceil(request.num_tokens / self.block_size)
        init, local = self.cfg["init_window_sz"], self.cfg["local_window_sz"]
        mid = int((num_blocks - init - local) * self.cfg["sparse_ratio"])
        flaw = request.num_tokens % self.block_size
        if flaw:
            flaw = self.block_size - flaw
        return (init + mid + local) * self.block_size - flaw
