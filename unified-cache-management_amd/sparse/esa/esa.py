"""ESA-shaped sparse-attention plugin: per-request, per-layer retrieval through
the GPU retrieval worker and delta loads of the chosen blocks from a KV store.

Follows the reference's ``ESA`` (ucm/sparse/esa/esa.py:402-587) and its
``ReqStatePerLayer`` state machine (:157-399) hook for hook:

* last prefill chunk  - ``block_repre_data`` (:353-364): the representatives of
  the request's first ``sparse_range`` blocks go into rows of the layer's
  table handed out by a ``ReprePool``;
* decode, ``step % retrieval_stride == 2`` - ``start_retrieval`` (:286-301):
  group-mean query, ``submit`` to the layer's retrieval worker;
* ``== 0`` - ``wait_retrieval_and_start_load`` (:303-339): slots -> block hashes,
  delta against what the request's first ``top_k`` cache blocks already hold,
  ``store.load`` of the missing ones;
* ``== 1`` - ``wait_transfer_task_done`` (:279-284).

What changes is the machinery underneath: the table is a device tensor and the
mean is taken by ``ucm_block_mean`` straight from the paged cache (bf16-rounded,
as the reference's ``k_cache[ids].mean(1)`` stores it); the worker is
``HipRetrievalBackend``; a store only needs the ``UcmKVStoreBase`` methods
``load`` / ``dump`` / ``wait`` (``UcmHipBlockStore`` does each as one batched
launch).  Scheduler-side slot accounting (``estimate_num_slots_sparsed``,
``allocate_slots``, :537-587) is host arithmetic and kept as is.
"""
from __future__ import annotations

import hashlib
import math
import pickle
from dataclasses import dataclass, field
from functools import lru_cache
from typing import Dict, List, Optional, Union

import torch

from ... import ops
from ..base import INVALID_SLOT, UcmSparseBase, UcmSparseMetadata, UcmSparseRole
from .device_path import EsaDevicePath
from .retrieval_worker import HipRetrievalBackend, RetrievalWorker

ReqType = Union[str, int]


class ReprePool:
    """Free-list of representative rows (esa.py:34-48)."""

    def __init__(self, num_slots: int):
        self.free_slots = list(range(num_slots - 1, -1, -1))
        self.allocated = set()

    def allocate(self, num_new_slots: int) -> List[int]:
        assert len(self.free_slots) >= num_new_slots, "Not enough free slots"
        if num_new_slots <= 0:
            return []
        got = self.free_slots[-num_new_slots:][::-1]           # the order repeated pop() hands them out in
        del self.free_slots[-num_new_slots:]
        self.allocated.update(got)
        return got

    def free(self, slots) -> None:
        for s in slots:
            if s in self.allocated:
                self.allocated.discard(s)
                self.free_slots.append(s)


@dataclass
class ReqMeta:
    request_id: ReqType
    index_in_batch: int
    num_scheduled_tokens: int
    num_computed_tokens: int
    vllm_block_ids: List[int]
    query_start_loc: int
    prompt_token_ids: List[int]
    output_token_ids: List[int]

    @property
    def step(self) -> int:
        return self.num_output_tokens

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_output_tokens(self) -> int:
        return len(self.output_token_ids)

    @property
    def is_prefill(self) -> bool:
        return self.num_output_tokens == 0

    @property
    def is_last_chunk(self) -> bool:
        return self.num_computed_tokens + self.num_scheduled_tokens >= self.num_prompt_tokens


@dataclass
class ESASparseMetaData(UcmSparseMetadata):
    requests: List[ReqMeta] = field(default_factory=list)
    finished_req_ids: List[ReqType] = field(default_factory=list)

    def add_request(self, *args, **kwargs) -> None:
        self.requests.append(ReqMeta(*args, **kwargs))


def get_offset(block_shape, rank, tp_size, precision, layer_id, is_v, is_mla=False) -> int:
    """Byte offset of one layer's K or V slice of one TP rank inside a stored
    block laid out [layer][K|V][rank] (esa.py:124-135)."""
    block_size, heads_per_tp, head_size = block_shape
    k_sz = block_size * heads_per_tp * head_size * precision
    v_sz = 0 if is_mla else k_sz
    layer_size = (k_sz + v_sz) * tp_size
    k_off = layer_size * layer_id if is_mla else layer_size * layer_id + layer_size // tp_size * rank
    return k_off + k_sz if is_v else k_off


@lru_cache(maxsize=None)
def _md5_int(obj) -> int:
    return int.from_bytes(hashlib.md5(pickle.dumps(obj, protocol=pickle.HIGHEST_PROTOCOL)).digest(), byteorder="big")


def block_hash_func(parent_block_hash, curr_block_token_ids) -> int:
    """Chained block hash, the same value the reference computes (esa.py:138-150),
    so blocks dumped by either side are found by the other."""
    if not parent_block_hash:
        parent_block_hash = _md5_int("UCMHASHSEED")
    return _md5_int((parent_block_hash, tuple(curr_block_token_ids)))


class ReqStatePerLayer:
    """One request in one layer (esa.py:157-399)."""

    def __init__(self, req_meta: ReqMeta, layer_name: str, rank: int, tp_size: int, store_instance, esa: "ESA"):
        self.layer_name = layer_name
        self.layer_id = int(layer_name.split(".")[2])
        self.req_meta = req_meta
        self.rank, self.tp_size = rank, tp_size
        self.store_instance = store_instance
        self.esa = esa
        self.esa_cfg = esa.esa_cfg
        self.block_size = esa.block_size
        self.num_key_heads, self.head_size = esa.num_key_heads, esa.head_size
        self.retrieval_worker: RetrievalWorker = esa.retrieval_workers[self.layer_id]
        self.repre_pool: ReprePool = esa.layer_pools[self.layer_id]
        self.slots: List[int] = []
        self.slots_to_relative_indexes: Dict[int, int] = {}
        self.retrieval_task = None
        self.k_cache = self.v_cache = None
        self.tasks: Dict[int, object] = {}
        self.block_hashes: Optional[List[str]] = None
        self.pre_topk_block_hashes: Dict[int, str] = {}
        self.init_static_flag = False
        self.sparse_range = self.get_sparse_prefill_range()

    # ---- static data -----------------------------------------------------------
    def set_block_hashes(self, token_ids) -> None:
        if self.block_hashes is None:
            self.block_hashes = self.esa.prompt_block_hashes(token_ids)

    def update_meta(self, req_meta: ReqMeta) -> None:
        self.req_meta = req_meta

    def maybe_register_static_data(self, forward_context) -> None:
        if self.init_static_flag:
            return
        attn = forward_context.no_compile_layers[self.layer_name]
        kv_cache = attn.kv_cache[forward_context.virtual_engine]
        self.k_cache, self.v_cache = kv_cache[0], kv_cache[1]
        self.esa.register_layer_cache(self.layer_id, self.k_cache)
        self.set_block_hashes(self.req_meta.prompt_token_ids)
        self.init_static_flag = True

    def get_sparse_prefill_range(self) -> int:
        n, local = self.req_meta.num_prompt_tokens, self.esa_cfg["local_window_sz"]
        if n % self.block_size == 0:
            return n // self.block_size - local
        return n // self.block_size - (local - 1)

    # ---- transfers ---------------------------------------------------------------
    def launch_transfer_task(self, transfer_type: str, block_hashes: List[str], vllm_block_ids: List[int]) -> None:
        if not block_hashes:
            return
        fn = getattr(self.store_instance, transfer_type)
        shape = (self.block_size, self.num_key_heads, self.head_size)
        precision = self.k_cache.element_size()
        n = len(block_hashes)
        off_k = [get_offset(shape, self.rank, self.tp_size, precision, self.layer_id, False)] * n
        off_v = [get_offset(shape, self.rank, self.tp_size, precision, self.layer_id, True)] * n
        self.tasks[hash((tuple(block_hashes), transfer_type, "key"))] = fn(
            block_hashes, off_k, [self.k_cache[i] for i in vllm_block_ids])
        self.tasks[hash((tuple(block_hashes), transfer_type, "value"))] = fn(
            block_hashes, off_v, [self.v_cache[i] for i in vllm_block_ids])

    def wait_transfer_task_done(self) -> None:
        for task in self.tasks.values():
            self.store_instance.wait(task)
        self.tasks.clear()

    # ---- representatives -------------------------------------------------------
    def block_repre_data(self) -> None:
        ids = self.req_meta.vllm_block_ids[: self.sparse_range]
        if not ids:
            return
        new_slots = self.repre_pool.allocate(len(ids))
        base = len(self.slots)
        for i, slot in enumerate(new_slots):
            self.slots_to_relative_indexes[slot] = base + i
        self.slots.extend(new_slots)
        self.slots_dev = torch.tensor([self.slots], dtype=torch.int32, device=self.k_cache.device)   # one index row
        self.esa.write_block_repre(self.layer_id, ids, new_slots)

    # ---- retrieval -----------------------------------------------------------------
    def top_k(self) -> int:
        return int(self.sparse_range * self.esa_cfg["sparse_ratio"])

    def start_retrieval(self, batch_query: torch.Tensor, forward_context) -> None:
        a = self.req_meta.query_start_loc
        query = batch_query[a : a + self.req_meta.num_scheduled_tokens]
        ntokens, num_q_heads, _ = query.shape
        if num_q_heads > self.num_key_heads:
            query = query.view(ntokens, self.num_key_heads, -1, self.head_size).mean(2)
        elif num_q_heads < self.num_key_heads:
            query = torch.repeat_interleave(query, self.num_key_heads // num_q_heads, 1)
        # the reference submits every scheduled token's query with ONE index row (esa.py:297-301) and reads row 0
        # of the result (:305); in decode there is one token
        self.retrieval_task = self.retrieval_worker.submit(query.reshape(ntokens, -1)[:1], topk=self.top_k(),
                                                           indexes=self.slots_dev)

    def wait_retrieval_and_start_load(self) -> None:
        self.retrieval_worker.wait(self.retrieval_task)
        result = self.retrieval_worker.get_result(self.retrieval_task)
        rel = [self.slots_to_relative_indexes[int(s)] for s in result["indices"][0]]
        block_hashes = [self.block_hashes[i] for i in rel]
        resident_ids = self.req_meta.vllm_block_ids[: self.top_k()]
        # delta: cache blocks that already hold a wanted block keep it, the others receive the missing ones
        wanted = set(block_hashes)
        matched = {b: h for b, h in self.pre_topk_block_hashes.items() if b in resident_ids and h in wanted}
        have = set(matched.values())
        free_ids = [b for b in resident_ids if b not in matched]
        missing = [h for h in block_hashes if h not in have]
        pairs = list(zip(free_ids, missing))
        self.pre_topk_block_hashes = dict(matched)
        self.pre_topk_block_hashes.update(pairs)
        self.last_loaded = pairs
        self.launch_transfer_task("load", [h for _, h in pairs], [b for b, _ in pairs])
        self.retrieval_task = None

    # ---- hooks -----------------------------------------------------------------------
    def attention_begin(self, query, key, value, forward_context) -> None:
        self.maybe_register_static_data(forward_context)
        stride = self.esa_cfg["retrieval_stride"]
        if self.req_meta.step % stride == 1:
            if self.req_meta.step == 1:
                self.start_retrieval(query, forward_context)
                self.wait_retrieval_and_start_load()
            self.wait_transfer_task_done()

    def attention_finished(self, query, key, value, attn_output, forward_context) -> None:
        self.maybe_register_static_data(forward_context)
        if self.req_meta.is_prefill and self.req_meta.is_last_chunk:
            self.block_repre_data()
            return
        if self.req_meta.step == 0:
            return
        stride = self.esa_cfg["retrieval_stride"]
        if self.req_meta.step % stride == 2 % stride and self.slots:
            self.start_retrieval(query, forward_context)
        if self.req_meta.step % stride == 0 and self.retrieval_task is not None:
            self.wait_retrieval_and_start_load()


class ESA(UcmSparseBase):
    def __init__(self, vllm_config, role: UcmSparseRole, store=None):
        super().__init__(vllm_config, role)
        mc, pc = vllm_config.model_config, vllm_config.parallel_config
        self.rank = getattr(pc, "rank", 0)
        self.tp_size = getattr(pc, "tensor_parallel_size", 1)
        extra = vllm_config.kv_transfer_config.kv_connector_extra_config
        self.esa_cfg = dict(extra["ucm_sparse_config"]["ESA"])
        for key, default in (("init_window_sz", 1), ("local_window_sz", 2), ("min_blocks", 4),
                             ("sparse_ratio", 0.3), ("retrieval_stride", 5)):
            self.esa_cfg.setdefault(key, default)
        self.block_size = vllm_config.cache_config.block_size
        self.num_key_heads = mc.get_num_kv_heads(pc)
        self.head_size = mc.get_head_size()
        self.total_num_hidden_layers = mc.get_num_layers(pc)
        self.max_model_len = mc.max_model_len
        self.max_num_seqs = vllm_config.scheduler_config.max_num_seqs
        self.num_slots = self.max_model_len * self.max_num_seqs // self.block_size
        self.dim = self.num_key_heads * self.head_size
        self.connector = store  # anything with the UcmKVStoreBase load / dump / wait methods
        self.req_states: Dict[ReqType, List[Optional[ReqStatePerLayer]]] = {}
        self.layer_pools = [ReprePool(self.num_slots) for _ in range(self.total_num_hidden_layers)]
        self.data: Optional[torch.Tensor] = None            # [layers, num_slots, dim] fp32, allocated with the first cache
        self.retrieval_workers: List[Optional[RetrievalWorker]] = [None] * self.total_num_hidden_layers
        self._layer_ptrs: Dict[int, ops.LayerPointers] = {}
        self._num_blocks: Dict[int, int] = {}
        # "device_loads": the batched path that plans and loads on the device (needs a store whose blocks a
        # kernel can read, i.e. one with device_pool()); False keeps the per-request host path for any store
        # (the stored-block layout the load kernel addresses is a single rank's, get_offset with tp_size 1)
        self._device_loads = (bool(self.esa_cfg.get("device_loads", True)) and hasattr(store, "device_pool")
                              and self.tp_size == 1)
        self._dev: Optional[EsaDevicePath] = None

    def prompt_block_hashes(self, token_ids) -> List[str]:
        """Chained hashes of the prompt's full blocks (esa.py:205-219)."""
        out, parent = [], None
        for start in range(0, len(token_ids), self.block_size):
            chunk = token_ids[start : start + self.block_size]
            if len(chunk) < self.block_size:
                break
            parent = block_hash_func(parent, tuple(chunk))
            out.append(str(parent))
        return out

    # ---- device tables -----------------------------------------------------------------
    def _allocate_tables(self, device) -> None:
        if self.data is None:
            self.data = torch.zeros((self.total_num_hidden_layers, self.num_slots, self.dim), dtype=torch.float32,
                                    device=device)
            for l in range(self.total_num_hidden_layers):
                self.retrieval_workers[l] = RetrievalWorker(HipRetrievalBackend(self.data[l]))

    def register_layer_cache(self, layer_id: int, k_cache: torch.Tensor) -> None:
        self._allocate_tables(k_cache.device)
        if layer_id not in self._layer_ptrs or self._layer_ptrs[layer_id].tensors[0].data_ptr() != k_cache.data_ptr():
            self._layer_ptrs[layer_id] = ops.LayerPointers([k_cache])
            self._num_blocks[layer_id] = k_cache.shape[0]

    def write_block_repre(self, layer_id: int, vllm_block_ids: List[int], slots: List[int]) -> None:
        dev = self.data.device
        ids = torch.tensor(vllm_block_ids, dtype=torch.int32, device=dev)
        sl = torch.tensor(slots, dtype=torch.int32, device=dev)
        ops.block_mean(self._layer_ptrs[layer_id], ids, sl, self.data[layer_id : layer_id + 1], self.block_size,
                       self.num_key_heads, self.head_size, self._num_blocks[layer_id], mode=ops.MEAN_BF16_ROUND)

    # ---- worker hooks ---------------------------------------------------------------------
    def create_layerwise_req_state(self, req_meta: ReqMeta, layer_name: str, forward_context) -> ReqStatePerLayer:
        layer_id = int(layer_name.split(".")[2])
        states = self.req_states.setdefault(req_meta.request_id, [None] * self.total_num_hidden_layers)
        if states[layer_id] is None:
            if self.data is None:   # the workers exist once the first cache has been seen
                attn = forward_context.no_compile_layers[layer_name]
                self.register_layer_cache(layer_id, attn.kv_cache[forward_context.virtual_engine][0])
            states[layer_id] = ReqStatePerLayer(req_meta, layer_name, self.rank, self.tp_size, self.connector, self)
        return states[layer_id]

    def _device_layer(self, layer_name: str, forward_context) -> int:
        layer_id = int(layer_name.split(".")[2])
        if self._dev.kv_caches[layer_id] is None:
            kv_cache = forward_context.no_compile_layers[layer_name].kv_cache[forward_context.virtual_engine]
            self.register_layer_cache(layer_id, kv_cache[0])
            self._dev.register_kv_cache(layer_id, kv_cache)
        return layer_id

    def attention_begin(self, query, key, value, layer_name: str, forward_context) -> None:
        if self._dev is not None:
            if self._sparse_metadata.requests:
                self._dev.attention_begin(self._device_layer(layer_name, forward_context), query)
            return
        for req_meta in self._sparse_metadata.requests:
            st = self.create_layerwise_req_state(req_meta, layer_name, forward_context)
            st.update_meta(req_meta)
            st.attention_begin(query, key, value, forward_context)

    def attention_finished(self, query, key, value, attn_output, layer_name: str, forward_context) -> None:
        if self._dev is not None:
            if self._sparse_metadata.requests:
                self._dev.attention_finished(self._device_layer(layer_name, forward_context), query)
            return
        for req_meta in self._sparse_metadata.requests:
            st = self.create_layerwise_req_state(req_meta, layer_name, forward_context)
            st.update_meta(req_meta)
            st.attention_finished(query, key, value, attn_output, forward_context)

    def is_sparsed_request(self, req) -> bool:
        return len(req.prompt_token_ids) >= self.block_size * self.esa_cfg["min_blocks"]

    def build_sparse_meta(self, scheduler_output, requests, input_batch, attn_metadata) -> None:
        meta = ESASparseMetaData()
        if isinstance(attn_metadata, dict):
            attn_metadata = next(iter(attn_metadata.values()))
        for req_id, n_tok in scheduler_output.num_scheduled_tokens.items():
            req = requests[req_id]
            if not self.is_sparsed_request(req):
                continue
            idx = input_batch.req_id_to_index[req_id]
            meta.add_request(req_id, idx, n_tok, req.num_computed_tokens, req.block_ids[0],
                             int(attn_metadata.query_start_loc[idx]), req.prompt_token_ids, req.output_token_ids)
        self._sparse_metadata = meta
        if self._device_loads and meta.requests:
            if self._dev is None:
                dev = torch.device("cuda", torch.cuda.current_device())
                pool, pool_block_bytes = self.connector.device_pool()
                self._dev = EsaDevicePath(self, pool, pool_block_bytes, dev)
                self._allocate_tables(dev)
            self._dev.build_step(meta.requests)

    def request_finished_in_worker(self, request_id: ReqType) -> None:
        if self._dev is not None:
            self._dev.request_finished(request_id)
        for st in self.req_states.pop(request_id, []):
            if st is not None:
                st.repre_pool.free(st.slots)
                if st.retrieval_task is not None:     # a retrieval nobody will fetch: drop its device buffers
                    st.retrieval_worker.cpp_worker.discard(st.retrieval_task)

    # ---- scheduler side -------------------------------------------------------------------------
    def request_begin(self, request_id: ReqType, prompt_token_ids: List[int]) -> None:
        pass

    def estimate_num_slots_sparsed(self, request) -> int:
        if request.num_output_tokens == 0 or not self.is_sparsed_request(request):
            return INVALID_SLOT
        n, out_len, bs = request.num_prompt_tokens, request.num_output_tokens, self.block_size
        local = self.esa_cfg["local_window_sz"]
        flaw = n % bs
        if flaw == 0:
            sparse_range, local_window = n // bs - local, bs * local + out_len
        else:
            sparse_range, local_window = n // bs - (local - 1), flaw + bs * (local - 1) + out_len
        return int(sparse_range * self.esa_cfg["sparse_ratio"]) * bs + local_window

    def allocate_slots(self, request, num_slots_sparsed, coordinator, block_pool, kv_cache_groups):
        """Keeps the last ceil(slots/block_size) blocks of the request, returns the others to the pool
        and allocates for the sparsified length (esa.py:557-587)."""
        need = math.ceil(num_slots_sparsed / self.block_size)
        blocks = coordinator.get_blocks(request.request_id)[0]
        first_kept = len(blocks) - need
        kept, returned = [], []
        for i, block in enumerate(blocks):
            (kept if i >= first_kept else returned).append(block)
            block_pool._maybe_evict_cached_block(block)
        block_pool.free_blocks(returned)
        coordinator.single_type_managers[0].req_to_blocks[request.request_id] = kept
        empty = tuple([] for _ in range(len(kv_cache_groups)))
        n_new = coordinator.get_num_blocks_to_allocate(request_id=request.request_id, num_tokens=num_slots_sparsed,
                                                       new_computed_blocks=empty)
        if n_new > block_pool.get_num_free_blocks():
            return None
        coordinator.allocate_new_blocks(request.request_id, num_slots_sparsed)
        return _kv_cache_blocks(kept)


def _kv_cache_blocks(kept):
    """vLLM's KVCacheBlocks when vLLM is importable, else a plain stand-in with the same field."""
    try:
        from vllm.v1.core.kv_cache_manager import KVCacheBlocks  # type: ignore

        return KVCacheBlocks(tuple([kept]))
    except Exception:  # vLLM absent (tests)
        from types import SimpleNamespace

        return SimpleNamespace(blocks=tuple([kept]))
