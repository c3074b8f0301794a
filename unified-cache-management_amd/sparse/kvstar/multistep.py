"""KVStar multi-step sparse-attention plugin: every ``retrieval_stride`` decode
steps the queries of the last stride vote for the prompt blocks to keep; the
winners are loaded from the KV store into the request's candidate cache blocks
two strides later, so a retrieval never stalls a decode step.

Follows the reference's ``KVStarMultiStep`` (ucm/sparse/kvstar/multistep.py:607-846)
and ``ReqPerLayerState`` (:175-604) hook for hook and keeps its bookkeeping names
(``standby_query_group``, ``step_group_retrieve_result``, ``task_waiter``, the
``"prefill"`` / ``"decode<N>"`` group records):

* prefill: the queries of the last ``retrieval_stride`` prompt tokens are parked
  (``offload_prefill_query`` :388-408); at the last chunk the sub-block
  representatives of all full prompt blocks are taken (``compute_block_repre``
  :483-501, with channel pruning when ``blk_repre_dim_prune_ratio < 0.98``) and
  the init / local window blocks are copied aside;
* decode step 1: windows written back, the prefill group's retrieval runs and
  its result is loaded into the candidate blocks (:377-387);
* decode step s: the query joins group ``decode<1 + stride*((s-1)//stride)>``
  (:461-481); at ``s % stride == 0`` that group's retrieval is queued (:370-374),
  and from ``s >= 2*stride`` the result of the group before it is loaded in
  ``attention_finished`` (:513-521), waited for at ``s % stride == 1`` (:387).

What changes underneath: queries, representatives and votes stay on the device
(``retrieve.py``: the reference's CPU thread pool is a side stream), the
representatives come from one kernel over the paged cache, and there is no NUMA
binding to do.  Block hashes are the chained md5 of the prompt's token blocks
(``utils.py:22-36``), the ones the connector dumped the blocks under.
"""
from __future__ import annotations

import enum
import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Union

import torch

from ..base import INVALID_SLOT, UcmSparseBase, UcmSparseMetadata, UcmSparseRole
from ..esa.esa import _kv_cache_blocks, block_hash_func, get_offset
from ..utils import HeldBlocks
from ... import ops
from . import retrieve as kvstar_retrieve
from .layer_path import KVStarLayerPath

ReqType = Union[str, int]

DEFAULTS = {
    "init_window_sz": 1,
    "local_window_sz": 2,
    "sparse_ratio": 0.25,
    "retrieval_stride": 8,
    "blk_repre_dim_prune_ratio": 0.25,
    "blk_repre_inner_token_merge": 2,
    "batch_retrieval": True,      # not in the reference: one launch per layer for all requests that retrieve in a step
    "device_loads": True,         # not in the reference: with a store whose blocks a kernel can read (device_pool()),
                                  # the blocks every request of a layer loads move in one pointer-array copy, and so
                                  # do the window blocks the requests of a layer save or write back
    "device_plans": True,         # not in the reference: with device_loads, the chosen blocks are loaded by a kernel
                                  # that follows the retrieval's own list on the device; the host reads the list only
                                  # when step_group_retrieve_result / _indices are looked at
}


class _RetrievalBatch:
    """The retrievals the requests of one layer queue during one attention_begin, launched together."""

    def __init__(self):
        self.entries = []     # (state, record, the group's query tokens [H, d] each, topk)
        self.after = []       # what the states still have to do once their tasks exist

    def flush(self) -> None:
        groups: Dict[tuple, list] = {}
        for e in self.entries:
            state, _, tokens, _ = e
            groups.setdefault((len(tokens), tuple(tokens[0].shape), state.d_pruned_index is None,
                               tuple(state.blk_repre.shape[1:])), []).append(e)
        for members in groups.values():
            # one stack and one conversion for the query groups of all members (torch.stack(...).to(float16) per
            # request in the reference, multistep.py:252-254)
            x = len(members[0][2])
            q = torch.stack([t for _, _, tokens, _ in members for t in tokens]).to(torch.float16)
            q = q.view(len(members), x, *q.shape[1:])
            for i, (st, record, _, _) in enumerate(members):
                st.do_retrieve_query_group[record] = q[i]
            ids = kvstar_retrieve.AsyncRetrieveBatch(
                q, [st.blk_repre for st, _, _, _ in members],
                [st.d_pruned_index32 for st, _, _, _ in members], [k for _, _, _, k in members])
            for (st, record, _, _), task_id in zip(members, ids):
                st.task_waiter[record] = task_id
        for fn in self.after:
            fn()
        self.entries, self.after = [], []


class _Collected(dict):
    """``step_group_retrieve_result`` / ``step_group_retrieve_indices`` of a request: a record whose blocks were
    loaded straight from the device list is read back the first time somebody asks for it."""

    def __init__(self, collect):
        super().__init__()
        self._collect = collect

    def __missing__(self, record):
        self._collect(record)
        return dict.__getitem__(self, record)


class ReqStage(enum.Enum):
    PREFILL = enum.auto()
    DECODE = enum.auto()


@dataclass
class ReqMeta:
    """multistep.py:43-130."""
    request_id: ReqType
    index_in_batch: int
    num_prompt_tokens: int
    num_output_tokens: int
    num_scheduled_tokens: int
    num_computed_tokens: int
    num_sparsed_tokens: int
    vllm_block_ids: List[int]
    token_blk_size: int
    prompt_token_ids: List[int]
    query_start_loc: int = -1
    query_len: int = -1
    retrieval_stride: int = 8
    block_hashes: List[str] = field(default_factory=list)

    def set_block_hashes(self, token_ids) -> List[str]:
        hashes, parent = [], None
        for start in range(0, len(token_ids), self.token_blk_size):
            chunk = token_ids[start : start + self.token_blk_size]
            if len(chunk) < self.token_blk_size:
                break
            parent = block_hash_func(parent, tuple(chunk))
            hashes.append(str(parent))
        return hashes

    @property
    def req_block_hashes(self) -> List[str]:
        if not self.block_hashes:
            self.block_hashes = self.set_block_hashes(self.prompt_token_ids)
        return self.block_hashes

    @property
    def step(self) -> int:
        return self.num_output_tokens

    @property
    def stage(self) -> ReqStage:
        return ReqStage.DECODE if self.num_output_tokens > 0 else ReqStage.PREFILL

    @property
    def is_last_chunk(self) -> bool:
        return self.num_computed_tokens + self.num_scheduled_tokens >= self.num_prompt_tokens

    @property
    def prefill_fully_blk_num(self) -> int:
        return self.num_prompt_tokens // self.token_blk_size

    @property
    def query_offload_info(self) -> Optional[List[int]]:
        """Places in the retrieval group of the tokens this step contributes: in prefill the chunk's share of
        the prompt's last ``retrieval_stride`` tokens (None if it has none), in decode the step's own place."""
        if self.stage == ReqStage.PREFILL:
            end_pos = self.num_computed_tokens + self.num_scheduled_tokens
            if end_pos < self.num_prompt_tokens - self.retrieval_stride:
                return None
            end_in_group = self.retrieval_stride - (self.num_prompt_tokens - end_pos)
            count = min(end_in_group, self.num_scheduled_tokens)
            return list(range(end_in_group - count, end_in_group))
        return [self.num_output_tokens % self.retrieval_stride]


@dataclass
class KVStarMultiStepSparseMetaData(UcmSparseMetadata):
    requests: List[ReqMeta] = field(default_factory=list)
    finished_req_ids: List[ReqType] = field(default_factory=list)

    def add_request(self, *args, **kwargs) -> None:
        self.requests.append(ReqMeta(*args, **kwargs))


class ReqPerLayerState:
    """One request in one layer (multistep.py:175-604)."""

    def __init__(self, req_meta: ReqMeta, layer_name: str, rank: int, tp_size: int, store_instance, store_name, sparse_cfg):
        self.sparse_cfg = sparse_cfg
        self.layer_name = layer_name
        self.layer_id = int(layer_name.split(".")[2])
        self.blk_repre = None                           # kvstar_retrieve.BlockRepre of the blocks between the windows
        self.block_hashes: List[str] = []
        self.num_tokens = 0
        self.store_instance, self.store_name = store_instance, store_name
        self.req_meta = req_meta
        self._init_window = self._local_window = None
        self._kept = None                                # (buffer [K|V][window block], first, init blocks, local blocks)
        self.init_window_sz, self.local_window_sz = sparse_cfg["init_window_sz"], sparse_cfg["local_window_sz"]
        self.block_size = None
        self._kv = None                                  # the layer's cache [K|V][block][token][head][channel]
        self.d_pruned_index = None
        self.local_tp_rank, self.total_tp_size = rank, tp_size
        self.blk_trans_tasks: Dict[int, object] = {}
        self.load_sink: Optional[list] = None            # set by the plugin: loads are collected, not issued here
        self.plan_sink: Optional[list] = None            # set by the plugin: loads that follow the device's own list
        self.standby_row: Optional[torch.Tensor] = None  # set by the plugin: this step's query token, already copied aside
        self.window_sink: Optional[list] = None          # set by the plugin: window copies are collected, not issued here
        self.repre_sink: Optional[list] = None           # set by the plugin: representatives of a layer's requests in one go
        self._d_pruned_index32 = None
        self.standby_query_group: Dict[str, list] = {}
        self.do_retrieve_query_group: Dict[str, torch.Tensor] = {}
        self.step_group_retrieve_result: Dict[str, List[str]] = _Collected(self._collect_planned)
        self.step_group_retrieve_indices: Dict[str, List[int]] = _Collected(self._collect_planned)   # as indices into blk_repre
        self._planned: Dict[str, tuple] = {}             # record -> (task id, results, row) of a load planned on the device
        self.task_waiter: Dict[str, int] = {}
        self.num_blocks_dumped = 0

    # the layer's K and V planes and the window copies, as the reference's attributes of these names; the views are made
    # when somebody asks for them (the paths that handle a layer's requests together work on addresses)
    k_cache = property(lambda self: None if self._kv is None else self._kv[0])
    v_cache = property(lambda self: None if self._kv is None else self._kv[1])

    def _window(self, which: int):
        if self._kept is None:
            return self._local_window if which else self._init_window
        kept, at, n_init, n_local = self._kept
        if which == 0:
            return kept[0, at : at + n_init], kept[1, at : at + n_init]
        return (kept[0, at + n_init : at + n_init + n_local], kept[1, at + n_init : at + n_init + n_local]) if n_local else None

    def _set_window(self, which: int, value) -> None:
        if self._kept is not None:                       # leaving the shared buffer: both windows become plain tensors
            self._init_window, self._local_window, self._kept = self._window(0), self._window(1), None
        if which:
            self._local_window = value
        else:
            self._init_window = value

    init_window = property(lambda self: self._window(0), lambda self, v: self._set_window(0, v))
    local_window = property(lambda self: self._window(1), lambda self, v: self._set_window(1, v))

    @classmethod
    def block_hash(cls, request_id, block_id) -> str:
        return f"req_{request_id}_blk_{block_id}"

    # ---- retrieval -----------------------------------------------------------------------
    def get_retrieve_record(self, cur_step: int) -> str:
        return "prefill" if cur_step == 1 else "decode" + str(cur_step - self.sparse_cfg["retrieval_stride"])

    def retrieval_async(self, cur_step: int, topk: int, retrieve_device: str = "cpu", batch: Optional[_RetrievalBatch] = None) -> None:
        """Queues the vote of one query group over the request's representatives (multistep.py:240-268); with
        ``batch`` the task is only listed, and launched with the layer's other requests."""
        record = self.get_retrieve_record(cur_step)
        if topk == 0:
            self.step_group_retrieve_result[record] = []
            self.step_group_retrieve_indices[record] = []
            return
        group = [x for x in self.standby_query_group[record] if x is not None]
        if batch is not None:
            batch.entries.append((self, record, group, topk))
            return
        self.do_retrieve_query_group[record] = torch.stack(group).to(torch.float16).contiguous()
        self.task_waiter[record] = kvstar_retrieve.AsyncRetrieveByCPU(
            self.do_retrieve_query_group[record], self.blk_repre, self.d_pruned_index, topk,
            hash(self.req_meta.request_id) & 0x7FFFFFFF, kvstar_retrieve.CPU)

    def extract_block_repre(self, vllm_block_ids: List[int], prune_dim_enable: bool = False):
        """Sub-block representatives of the listed cache blocks (multistep.py:279-316)."""
        if not vllm_block_ids or vllm_block_ids[-1] < 2:          # the reference's own guard, kept as it is (:280-281)
            return None
        repre, index = kvstar_retrieve.extract_block_repre(
            self.k_cache, vllm_block_ids, self.sparse_cfg["blk_repre_inner_token_merge"],
            prune_ratio=self.sparse_cfg["blk_repre_dim_prune_ratio"], d_pruned_index=self.d_pruned_index,
            prune_dim_enable=prune_dim_enable)
        self.d_pruned_index = index
        self._d_pruned_index32 = None
        return repre

    @property
    def d_pruned_index32(self):
        """The kept channels as the kernels take them (int32), converted once."""
        if self.d_pruned_index is not None and self._d_pruned_index32 is None:
            self._d_pruned_index32 = self.d_pruned_index.to(torch.int32).contiguous()
        return self._d_pruned_index32

    def get_retrieve_candidate_block_ids(self) -> List[int]:
        n_keep = math.ceil(self.blk_repre.shape[0] * self.sparse_cfg["sparse_ratio"])
        return self.req_meta.vllm_block_ids[self.init_window_sz : n_keep + self.init_window_sz]

    def get_decode_step_record(self):
        stride = self.sparse_cfg["retrieval_stride"]
        step = self.req_meta.step
        return "decode" + str(((step - 1) // stride) * stride + 1), (step - 1) % stride

    def save_to_standby(self, group_record: str, in_query_group_idx: int, query_relative_idx: int, tokens_to_offload) -> None:
        if group_record not in self.standby_query_group:
            self.standby_query_group[group_record] = [None] * self.sparse_cfg["retrieval_stride"]
        self.standby_query_group[group_record][in_query_group_idx] = tokens_to_offload[query_relative_idx].clone()

    def offload_prefill_query(self, query, query_len: int, query_start_loc: int) -> None:
        places = self.req_meta.query_offload_info
        if not places:
            return
        assert query_len >= len(places)
        # one copy of the chunk's share of the group; every place keeps a view of it
        tail = query[query_start_loc + query_len - len(places) : query_start_loc + query_len].clone()
        group = self.standby_query_group.setdefault("prefill", [None] * self.sparse_cfg["retrieval_stride"])
        for rel, place in enumerate(places):
            group[place] = tail[rel]

    def load_retrieve_result_async(self, load_step: int, candidate_swap_vllm_block_ids: List[int]) -> None:
        """Collects the result of the group two strides back (the prefill group early on) and starts loading
        the chosen blocks into the candidate cache blocks (multistep.py:410-450)."""
        stride = self.sparse_cfg["retrieval_stride"]
        if load_step <= stride * 2:
            record = "prefill"
        else:
            record = "decode" + str((int(math.ceil(load_step / stride)) - 3) * stride + 1)
        if (self.plan_sink is not None and record in self.task_waiter and record not in self._planned
                and dict.get(self.step_group_retrieve_result, record) is None):
            # the chosen blocks never come to the host: the load follows the device's list, after the side stream's
            # event, and the bookkeeping lists are read back only if somebody looks at them
            task_id = self.task_waiter[record]
            found = kvstar_retrieve.DeviceResult(task_id)
            if found is None:
                raise RuntimeError(f"retrieval task {task_id} of layer {self.layer_id} is not known")
            for old_task, _, _ in self._planned.values():
                kvstar_retrieve.Forget(old_task)
            self._planned = {record: (task_id,) + found}
            del self.standby_query_group[record]
            del self.do_retrieve_query_group[record]
            if record != "prefill" or load_step == 1:
                self.plan_sink.append((self, found[0], found[1], list(candidate_swap_vllm_block_ids)))
            return
        if dict.get(self.step_group_retrieve_result, record) is None and record in self._planned:
            self._collect_planned(record)
        if self.step_group_retrieve_result.get(record) is None:
            task_id = self.task_waiter[record]
            kvstar_retrieve.Wait(task_id)
            result = kvstar_retrieve.GetTaskResult(task_id)
            del self.standby_query_group[record]
            del self.do_retrieve_query_group[record]
            if result["status"] != "SUCCESS":
                raise RuntimeError(f"retrieval task {task_id} of layer {self.layer_id} failed: {result}")
            chosen = [int(i) for i in result["data"]]
            self.step_group_retrieve_indices[record] = chosen
            self.step_group_retrieve_result[record] = [self.block_hashes[i + self.init_window_sz] for i in chosen]
        hashes = self.step_group_retrieve_result[record]
        if (record != "prefill" or load_step == 1) and len(hashes) > 0:
            self.launch_transfer_task("load", hashes, candidate_swap_vllm_block_ids)

    def _collect_planned(self, record: str) -> None:
        """The host's copy of a list whose blocks were loaded on the device (KeyError if there is none)."""
        found = self._planned.get(record)
        if found is None:
            # (a load issued for the layer's requests together leaves no entry per request: the task itself is asked)
            found = kvstar_retrieve.DeviceResult(self.task_waiter[record])
            if found is None:
                raise KeyError(record)
            found = (None,) + found
        _, results, row = found
        chosen = results.chosen(row)
        dict.__setitem__(self.step_group_retrieve_indices, record, chosen)
        dict.__setitem__(self.step_group_retrieve_result, record, [self.block_hashes[i + self.init_window_sz] for i in chosen])

    def release(self) -> None:
        """The request is over: retrievals nobody will collect are dropped, and with them the buffers of their launch
        once its last task is gone (the reference keeps every result for the life of the process)."""
        for task_id, _, _ in self._planned.values():
            kvstar_retrieve.Forget(task_id)
        for task_id in self.task_waiter.values():
            kvstar_retrieve.Forget(task_id)
        self._planned = {}
        self.task_waiter = {}

    # ---- windows -------------------------------------------------------------------------
    def window_blocks(self):
        """(cache blocks of the init window, cache blocks of the local window) as the request stands now."""
        ids = self.req_meta.vllm_block_ids
        n_local = min(self.local_window_sz, len(ids[self.init_window_sz :]))
        return ids[: self.init_window_sz], (ids[-n_local:] if n_local > 0 else [])

    def prepare_init_and_local_window(self) -> None:
        if self.window_sink is not None:
            self.window_sink.append((self, "restore"))
            return
        ids = self.req_meta.vllm_block_ids
        self.k_cache[ids[: self.init_window_sz]] = self.init_window[0]
        self.v_cache[ids[: self.init_window_sz]] = self.init_window[1]
        if self.local_window is None:
            return
        n_local = self.local_window[0].shape[0]
        self.k_cache[ids[-n_local:]] = self.local_window[0]
        self.v_cache[ids[-n_local:]] = self.local_window[1]

    def construct_init_and_local_window(self) -> None:
        if self.window_sink is not None:
            self.window_sink.append((self, "save"))
            return
        ids = self.req_meta.vllm_block_ids
        head = ids[: self.init_window_sz]
        self.init_window = (self.k_cache[head].clone(), self.v_cache[head].clone())
        n_local = min(self.local_window_sz, len(ids[self.init_window_sz :]))
        if n_local > 0:
            tail = ids[-n_local:]
            self.local_window = (self.k_cache[tail].clone(), self.v_cache[tail].clone())

    def compute_block_repre(self, num_blocks_need_dump: int) -> None:
        if self.req_meta.stage != ReqStage.PREFILL or not self.req_meta.is_last_chunk:
            return
        ids = self.req_meta.vllm_block_ids[: self.num_blocks_dumped + num_blocks_need_dump]
        if self.repre_sink is not None and ids and ids[-1] >= 2:
            self.repre_sink.append((self, list(ids)))   # taken with the layer's other requests (set_block_repre follows)
            return
        self.set_block_repre(self.extract_block_repre(ids, prune_dim_enable=True))

    def set_block_repre(self, repre) -> None:
        """The representatives of all full prompt blocks are in: the ones between the windows are kept, the window
        blocks copied aside (multistep.py:483-501)."""
        if repre is not None:
            repre = None if repre.shape[0] <= 2 else repre[self.init_window_sz : -self.local_window_sz]
        self.blk_repre = repre
        self.construct_init_and_local_window()

    # ---- hooks ---------------------------------------------------------------------------
    def attention_begin(self, query, key, value, forward_context, batch: Optional[_RetrievalBatch] = None) -> None:
        meta = self.req_meta
        if meta.stage == ReqStage.PREFILL:
            self.offload_prefill_query(query, meta.query_len, meta.query_start_loc)
            return
        if self.blk_repre is None:
            return
        assert meta.query_len == 1, "KVStar series sparse attention doesn't support spec_decode now"
        stride = self.sparse_cfg["retrieval_stride"]
        group_record, place = self.get_decode_step_record()
        if self.standby_row is not None:
            self.standby_query_group.setdefault(group_record, [None] * stride)[place] = self.standby_row
        else:
            self.save_to_standby(group_record, place, meta.query_start_loc, query)
        later = (lambda fn: fn()) if batch is None else batch.after.append   # with a batch: once the tasks exist
        if meta.step % stride == 0:
            self.retrieval_async(meta.step + 1, len(self.get_retrieve_candidate_block_ids()), batch=batch)
        if meta.step == 1:
            self.prepare_init_and_local_window()
            candidates = self.get_retrieve_candidate_block_ids()
            self.wait_for_blk_transfer_task_done()
            self.retrieval_async(meta.step, len(candidates), batch=batch)
            step = meta.step
            later(lambda: self.load_retrieve_result_async(step, candidates))
        if meta.step % stride == 1:
            later(self.wait_for_blk_transfer_task_done)

    def attention_finished(self, query, key, value, attn_output, forward_context) -> None:
        meta = self.req_meta
        if meta.stage != ReqStage.PREFILL:
            stride = self.sparse_cfg["retrieval_stride"]
            if self.blk_repre is not None and meta.step >= stride * 2 and meta.step % stride == 0:
                self.load_retrieve_result_async(meta.step + 1, self.get_retrieve_candidate_block_ids())
            return
        self.maybe_register_kv_cache(forward_context)
        updated = meta.num_computed_tokens + meta.num_scheduled_tokens
        need_dump = updated // self.block_size - self.num_blocks_dumped
        self.num_tokens = updated
        self.compute_block_repre(need_dump)

    def maybe_register_kv_cache(self, forward_context) -> None:
        if self.block_size:
            return
        attn = forward_context.no_compile_layers[self.layer_name]
        self._kv = attn.kv_cache[forward_context.virtual_engine]
        _, _, self.block_size, self.num_key_heads, self.head_size = self._kv.shape
        self.block_hashes = self.req_meta.req_block_hashes

    def update_meta(self, req_meta: ReqMeta, forward_context=None) -> None:
        self.req_meta = req_meta

    # ---- transfers -----------------------------------------------------------------------
    def launch_transfer_task(self, transfer_type: str, block_hashes: List[str], vllm_block_ids: List[int]) -> None:
        n = min(len(block_hashes), len(vllm_block_ids))
        if n == 0:
            return
        block_hashes, vllm_block_ids = list(block_hashes[:n]), list(vllm_block_ids[:n])
        if transfer_type == "load" and self.load_sink is not None:
            self.load_sink.append((block_hashes, vllm_block_ids))
            return
        fn = getattr(self.store_instance, transfer_type)
        shape = (self.block_size, self.num_key_heads, self.head_size)
        precision = self.k_cache.element_size()
        off_k = [get_offset(shape, self.local_tp_rank, self.total_tp_size, precision, self.layer_id, False)] * n
        off_v = [get_offset(shape, self.local_tp_rank, self.total_tp_size, precision, self.layer_id, True)] * n
        self.blk_trans_tasks[hash((tuple(block_hashes), transfer_type, "key"))] = fn(
            block_hashes, off_k, [self.k_cache[i] for i in vllm_block_ids])
        self.blk_trans_tasks[hash((tuple(block_hashes), transfer_type, "value"))] = fn(
            block_hashes, off_v, [self.v_cache[i] for i in vllm_block_ids])

    def wait_for_blk_transfer_task_done(self) -> None:
        for task in self.blk_trans_tasks.values():
            self.store_instance.wait(task)
        self.blk_trans_tasks.clear()


class KVStarMultiStep(UcmSparseBase):
    """Plugin object (multistep.py:607-846).  ``store``: anything with the ``UcmKVStoreBase`` load / wait
    methods; under vLLM it is the connector of the KV transfer group."""

    def __init__(self, vllm_config, role: UcmSparseRole, store=None):
        super().__init__(vllm_config=vllm_config, role=role)
        self.req_states: Dict[ReqType, List[Optional[ReqPerLayerState]]] = {}
        self.local_tp_rank = vllm_config.parallel_config.rank
        self.total_tp_size = vllm_config.parallel_config.tensor_parallel_size
        hf_config = getattr(vllm_config.model_config, "hf_config", None)
        self.total_num_hidden_layers = (hf_config.num_hidden_layers if hf_config is not None
                                        else vllm_config.model_config.get_num_layers(vllm_config.parallel_config))
        extra = vllm_config.kv_transfer_config.kv_connector_extra_config
        self.kvstar_multistep_cfg = dict(DEFAULTS)
        self.kvstar_multistep_cfg.update(extra["ucm_sparse_config"].get("KVStarMultiStep") or {})
        self.connector_name = extra.get("ucm_connector_name")
        self.connector = store
        self.token_blk_size = vllm_config.cache_config.block_size
        self._step_cache: Dict[object, tuple] = {}       # what every layer's hooks of one step share (tables, indices)
        self._layer_ptrs: Dict[str, tuple] = {}
        self._layer_ids: Dict[str, int] = {}
        self._layer_slots: Dict[str, int] = {}             # layers in the order their hooks first ran
        self._n_slots = 0                                  # how many there were in a complete step (0: none seen yet)
        self._path: Optional[KVStarLayerPath] = None       # the decode steps of a layer's requests at once (see _hook)
        if role == UcmSparseRole.WORKER:
            kvstar_retrieve.Setup(kvstar_retrieve.SetupParam(
                cpuNumaIds=[], physicalCorePerNuma=0, allocRatio=0.75, blkRepreSize=4096, deviceType=kvstar_retrieve.CPU,
                totalTpSize=self.total_tp_size, localRankId=self.local_tp_rank))
            if self.connector is None:
                try:  # under vLLM: the connector of the KV transfer group, as the reference takes it (:637-642)
                    from vllm.distributed.kv_transfer import get_kv_transfer_group  # type: ignore

                    self.connector = get_kv_transfer_group().connector
                except Exception:
                    self.connector = None

    def create_layerwise_req_state(self, req_meta: ReqMeta, layer_name: str) -> ReqPerLayerState:
        layer_id = int(layer_name.split(".")[2])
        states = self.req_states.setdefault(req_meta.request_id, [None] * self.total_num_hidden_layers)
        if states[layer_id] is None:
            states[layer_id] = ReqPerLayerState(req_meta, layer_name, self.local_tp_rank, self.total_tp_size, self.connector,
                                                self.connector_name, self.kvstar_multistep_cfg)
        return states[layer_id]

    def request_begin(self, request_id: ReqType, prompt_token_ids: List[int]) -> None:
        pass

    # ---- worker side ---------------------------------------------------------------------
    def request_finished_in_worker(self, request_id: ReqType) -> None:
        for state in self.req_states.pop(request_id, None) or []:
            if state is not None:
                state.release()
        if self._path is not None:
            self._path.request_finished(request_id)

    def _layer_path(self) -> Optional[KVStarLayerPath]:
        """The path that handles a layer's requests together (layer_path.py); it needs what the three switches stand
        for: batched retrieval, a store whose blocks a kernel can read, loads that follow the device's lists."""
        cfg = self.kvstar_multistep_cfg
        if self._path is None and cfg["batch_retrieval"] and cfg["device_plans"] and self._load_sink() is not None:
            self._path = KVStarLayerPath(self, None)
        return self._path

    def _load_sink(self) -> Optional[list]:
        """A list that collects the loads of a hook's requests, when they can be carried out as one copy: the store's
        blocks must be readable by a kernel, in the stored layout of a single rank (get_offset with tp_size 1)."""
        if (self.kvstar_multistep_cfg["device_loads"] and hasattr(self.connector, "device_pool")
                and self.total_tp_size == 1):
            return []
        return None

    def _flush_loads(self, sink: list, layer_name: str, forward_context) -> None:
        """One pointer-array copy for every (stored block -> cache block) pair the hook's requests asked for, K and V
        (launch_transfer_task("load", ...) per request, multistep.py:452-480).  A block the store does not hold is
        left out and reported (the per-request path gives up the whole request's load in that case)."""
        if not sink:
            return
        layer_id = int(layer_name.split(".")[2])
        kv = forward_context.no_compile_layers[layer_name].kv_cache[forward_context.virtual_engine]
        pool, pool_block_bytes = self.connector.device_pool()
        es = kv.element_size()
        kv_stride, block_bytes = kv.stride(0) * es, kv.stride(1) * es
        cache, stored = kv.data_ptr(), pool.data_ptr() + layer_id * 2 * block_bytes
        dst, src = [], []
        missing = 0
        # (held while the copy is queued: a store with a tier behind its pool brings spilled blocks back first, and
        # orders whatever it does to these slots later after this stream's work)
        held = HeldBlocks(self.connector)
        for hashes, ids in sink:
            for slot, b in zip(held.slots(hashes), ids):
                if slot < 0:
                    missing += 1
                    continue
                for plane in (0, 1):
                    src.append(stored + slot * pool_block_bytes + plane * block_bytes)
                    dst.append(cache + plane * kv_stride + b * block_bytes)
        if missing:
            self._report_missing(missing)
        if src:
            # a block list shorter than the request's two windows together (this plugin's own slot estimate never
            # leaves one; another scheduler might) names a cache block twice on the way back: the reference writes
            # the init window, then the local one over it (multistep.py:348-362), so of the copies into one block
            # only the last is made (the copies of one launch are not ordered)
            last = {d: i for i, d in enumerate(dst)}
            if len(last) != len(dst):
                keep = [i for i, d in enumerate(dst) if last[d] == i]
                dst, src = [dst[i] for i in keep], [src[i] for i in keep]
            ptrs = ops.upload(torch.tensor([dst, src], dtype=torch.int64), kv.device)
            ops.copy_batch(ptrs[0], ptrs[1], block_bytes)
        held.release()

    def _flush_planned(self, plan: list, layer_name: str, forward_context) -> None:
        """The loads whose lists stay on the device: per launch that produced them, one ucm_kv_load_planned follows
        the ordered lists (j-th chosen block -> j-th candidate cache block, multistep.py:410-450) once the side
        stream's event has passed.  The tables that turn a list entry into a stored block and a list position into a
        cache block are the same for every layer of a step and are built at the first."""
        if not plan:
            return
        layer_id = int(layer_name.split(".")[2])
        kv = forward_context.no_compile_layers[layer_name].kv_cache[forward_context.virtual_engine]
        known = self._layer_ptrs.get(layer_name)
        if known is None or known[0] != kv.data_ptr():
            known = self._layer_ptrs[layer_name] = (kv.data_ptr(), ops.LayerPointers([kv]))
        es = kv.element_size()
        pool, pool_block_bytes = self.connector.device_pool()
        groups: Dict[int, list] = {}
        for entry in plan:
            groups.setdefault(id(entry[1]), []).append(entry)
        stream = torch.cuda.current_stream()
        for members in groups.values():
            results = members[0][1]
            n_rows, width = results.idx.shape
            key = (n_rows, width, tuple((st.req_meta.request_id, row) for st, _, row, _ in members))
            tables = self._step_cache.get(key)
            if tables is None:
                held = self._step_cache.setdefault("held", HeldBlocks(self.connector))   # until the step's last layer
                longest = max(len(st.block_hashes) for st, _, _, _ in members)
                src = torch.full((n_rows, max(longest, 1)), -1, dtype=torch.int32)
                dst = torch.full((n_rows, width), -1, dtype=torch.int32)
                missing = 0
                for st, _, row, candidates in members:
                    first = st.init_window_sz
                    stored = held.slots(st.block_hashes[first : first + st.blk_repre.shape[0]])
                    missing += stored.count(-1)
                    src[row, : len(stored)] = torch.tensor(stored, dtype=torch.int32)
                    dst[row, : min(len(candidates), width)] = torch.tensor(candidates[:width], dtype=torch.int32)
                if missing:
                    self._report_missing(missing)
                rows = [row for _, _, row, _ in members]
                both = ops.upload(torch.cat([src.view(-1), dst.view(-1), torch.tensor(rows, dtype=torch.int32)]), kv.device)
                tables = self._step_cache[key] = (both[: src.numel()].view(src.shape),
                                                   both[src.numel() : src.numel() + dst.numel()].view(dst.shape),
                                                   None if rows == list(range(n_rows)) else both[src.numel() + dst.numel() :])
            stream.wait_event(results.event)
            results.idx.record_stream(stream)
            results.cnt.record_stream(stream)
            ops.kv_load_planned(known[1], 0, layer_id, 1, kv.stride(0) * es, kv.stride(1) * es, kv.shape[1], pool, pool_block_bytes,
                                results.idx.unsqueeze(0), tables[0], tables[1], tables[2], load_count=results.cnt.unsqueeze(0))

    def _of_all_layers(self, what, layer_name: str, make):
        """Layer ``layer_name``'s part of a buffer that every layer of this step needs in the same shape: once the
        number of layers is known (a step has gone by), ``make(n)`` allocates for all of them at the first, instead
        of one device allocation per layer."""
        slot = self._layer_slots.setdefault(layer_name, len(self._layer_slots))
        if slot >= self._n_slots:
            return make(1)[0]
        whole = self._step_cache.get(what)
        if whole is None:
            whole = self._step_cache[what] = make(self._n_slots)
        return whole[slot]

    def _flush_windows(self, sink: list, layer_name: str, forward_context) -> None:
        """The window copies of a hook's requests as one pointer-array copy: "save" keeps the init and local window
        blocks of a request that ends its prefill (multistep.py:326-346: four indexed clones per request), "restore"
        writes them back into the blocks the request holds at its first decode step (:348-362)."""
        if not sink:
            return
        kv = forward_context.no_compile_layers[layer_name].kv_cache[forward_context.virtual_engine]
        es = kv.element_size()
        kv_stride, block_bytes = kv.stride(0) * es, kv.stride(1) * es
        if not kv[0, 0].is_contiguous():
            raise ValueError("cache blocks must be contiguous")
        cache = kv.data_ptr()
        dst, src = [], []
        saves = [(st, st.window_blocks()) for st, what in sink if what == "save"]
        if saves:
            total = sum(len(head) + len(tail) for _, (head, tail) in saves)
            kept = self._of_all_layers(("kept", total), layer_name, lambda n: torch.empty(
                (n, 2, total) + tuple(kv.shape[2:]), dtype=kv.dtype, device=kv.device))                # [K|V][window block]
            base, at = kept.data_ptr(), 0
            for st, (head, tail) in saves:
                st._init_window = st._local_window = None
                st._kept = (kept, at, len(head), len(tail))
                for j, b in enumerate(list(head) + list(tail)):
                    for plane in (0, 1):
                        src.append(cache + plane * kv_stride + b * block_bytes)
                        dst.append(base + (plane * total + at + j) * block_bytes)
                at += len(head) + len(tail)
        for st, what in sink:
            if what != "restore":
                continue
            ids = st.req_meta.vllm_block_ids
            if st._kept is not None:
                kept, at, n_init, n_local = st._kept
                base, total = kept.data_ptr(), kept.shape[1]
                blocks = list(ids[: st.init_window_sz][:n_init]) + (list(ids[-n_local:]) if n_local else [])
                for plane in (0, 1):
                    for j, b in enumerate(blocks):
                        src.append(base + (plane * total + at + j) * block_bytes)
                        dst.append(cache + plane * kv_stride + b * block_bytes)
                continue
            init, local = st.init_window, st.local_window
            for plane in (0, 1):
                for j, b in enumerate(ids[: st.init_window_sz]):
                    src.append(init[plane][j].data_ptr())
                    dst.append(cache + plane * kv_stride + b * block_bytes)
                if local is not None:
                    n_local = local[plane].shape[0]
                    for j, b in enumerate(ids[-n_local:]):
                        src.append(local[plane][j].data_ptr())
                        dst.append(cache + plane * kv_stride + b * block_bytes)
        if src:
            ptrs = ops.upload(torch.tensor([dst, src], dtype=torch.int64), kv.device)
            ops.copy_batch(ptrs[0], ptrs[1], block_bytes)

    def _flush_repre(self, sink: list, layer_name: str, forward_context) -> None:
        """Sub-block representatives and channel choice of every request that ends its prefill in this step, for one
        layer: one pass over the paged cache for the blocks' mean |k| (of all requests), one mean per request over
        its blocks, one top-k for the kept channels, one launch that writes every request's representatives with its
        own channels (``extract_block_repre`` per request in the reference, multistep.py:279-316).  The requests'
        tables are row ranges of one tensor."""
        if not sink:
            return
        cfg = self.kvstar_multistep_cfg
        kv = forward_context.no_compile_layers[layer_name].kv_cache[forward_context.virtual_engine]
        k_cache = kv[0]
        n_total, block_size, kv_heads, head_dim = k_cache.shape
        dev = k_cache.device
        known = self._layer_ptrs.get(("k", layer_name))
        if known is None or known[0] != k_cache.data_ptr():
            known = self._layer_ptrs[("k", layer_name)] = (k_cache.data_ptr(), ops.LayerPointers([k_cache]))
        key = ("repre", tuple(st.req_meta.request_id for st, _ in sink))
        shared = self._step_cache.get(key)
        if shared is None:        # the same for every layer of the step
            counts = [len(ids) for _, ids in sink]
            flat = [b for _, ids in sink for b in ids]
            which = [r for r, n in enumerate(counts) for _ in range(n)]
            both = ops.upload(torch.tensor([flat, which], dtype=torch.int32), dev)
            shared = self._step_cache[key] = (both[0], both[1], torch.arange(len(flat), dtype=torch.int32, device=dev),
                                               torch.tensor(counts, dtype=torch.int64, device=dev), counts)
        ids_dev, which_dev, rows, counts_dev, counts = shared
        n = ids_dev.numel()
        merge, ratio = cfg["blk_repre_inner_token_merge"], cfg["blk_repre_dim_prune_ratio"]
        index = lists32 = None
        if ratio < 0.98:
            # mean |k| per (head, channel) over all tokens of a request's blocks: the blocks' own means of |k|, read
            # from the paged cache in one pass, averaged per request
            per_block = torch.empty((1, n, kv_heads * head_dim), dtype=torch.float32, device=dev)
            ops.block_mean(known[1], ids_dev, rows, per_block, block_size, kv_heads, head_dim, n_total,
                           mode=ops.MEAN_F32 | ops.MEAN_ABS)
            absmean = torch.segment_reduce(per_block[0], "mean", lengths=counts_dev, axis=0, unsafe=True)
            _, index = torch.topk(absmean.view(len(counts), kv_heads, head_dim), k=round(head_dim * ratio), dim=-1)
            lists32 = index.to(torch.int32)
        d_pruned = head_dim if index is None else index.shape[-1]
        d_pad = (d_pruned + 15) // 16 * 16
        table = self._of_all_layers(("table", n, d_pad), layer_name, lambda layers: ops.kvstar_table(
            layers, kv_heads, n, block_size // merge, d_pad, dev)).unsqueeze(0)
        ops.kvstar_block_repre(known[1], ids_dev, rows, table, block_size, kv_heads, head_dim, n_total, merge, pruned=lists32,
                               pruned_sel=None if lists32 is None else which_dev)
        at = 0
        for r, (st, _) in enumerate(sink):
            if index is not None:
                st.d_pruned_index, st._d_pruned_index32 = index[r], lists32[r]
            st.set_block_repre(kvstar_retrieve.BlockRepre(table[0][:, at : at + counts[r]], d_pruned))
            at += counts[r]

    def _standby_rows(self, query):
        """The decoding requests' query tokens of this layer copied aside in one go (``query[start].clone()`` per
        request in the reference, multistep.py:318-324); every request then keeps a view of its row."""
        found = self._step_cache.get("standby")
        if found is None:
            place, starts = {}, []
            for m in self._sparse_metadata.requests:
                if m.stage == ReqStage.DECODE:
                    place[m.request_id] = len(starts)
                    starts.append(m.query_start_loc)
            index = ops.upload(torch.tensor(starts, dtype=torch.int64), query.device) if len(starts) > 1 else None
            found = self._step_cache["standby"] = (index, place)
        if found[0] is None:
            return None, None
        return query.index_select(0, found[0]), found[1]

    def _hook(self, which: str, layer_name: str, forward_context, *args) -> None:
        requests = self._sparse_metadata.requests
        path = self._path
        if path is not None:
            if path.step.get("owner") is not self._sparse_metadata:      # metadata bound by somebody else
                path.build_step(self._sparse_metadata, ReqStage)
            # decode steps: nothing per request; what is left for the per-request objects are the requests that end
            # their prefill in this step (representatives, channel choice, windows aside)
            layer_id = self._layer_ids.get(layer_name)
            if layer_id is None:
                layer_id = self._layer_ids[layer_name] = int(layer_name.split(".")[2])
            if which == "attention_begin":
                path.attention_begin(layer_id, layer_name, args[0], forward_context)
                return
            path.attention_finished(layer_id, layer_name, forward_context)
            requests = path.step["ending"]
            if not requests:
                return
        batch = _RetrievalBatch() if which == "attention_begin" and self.kvstar_multistep_cfg["batch_retrieval"] else None
        sink = self._load_sink()
        plan = [] if sink is not None and self.kvstar_multistep_cfg["device_plans"] else None
        windows = [] if self.kvstar_multistep_cfg["device_loads"] else None
        repres = [] if which == "attention_finished" else None
        rows = place = None
        if which == "attention_begin":
            rows, place = self._standby_rows(args[0])
        for req_meta in requests:
            state = self.create_layerwise_req_state(req_meta, layer_name)
            state.update_meta(req_meta, forward_context)
            state.load_sink, state.plan_sink, state.window_sink, state.repre_sink = sink, plan, windows, repres
            state.standby_row = None if rows is None or req_meta.request_id not in place else rows[place[req_meta.request_id]]
            if which == "attention_begin":
                state.attention_begin(*args, forward_context, batch=batch)
            else:
                state.attention_finished(*args, forward_context)
        if batch is not None:
            batch.flush()
        self._flush_repre(repres, layer_name, forward_context)      # (before the windows: it queues the ending requests' saves)
        self._flush_windows(windows, layer_name, forward_context)
        self._flush_loads(sink, layer_name, forward_context)
        self._flush_planned(plan, layer_name, forward_context)

    def attention_begin(self, query, key, value, layer_name: str, forward_context) -> None:
        self._hook("attention_begin", layer_name, forward_context, query, key, value)

    def attention_finished(self, query, key, value, attn_output, layer_name: str, forward_context) -> None:
        self._hook("attention_finished", layer_name, forward_context, query, key, value, attn_output)

    def build_sparse_meta(self, scheduler_output, requests, input_batch, attn_metadata=None) -> None:
        meta = KVStarMultiStepSparseMetaData()
        if isinstance(attn_metadata, dict):
            attn_metadata = next(iter(attn_metadata.values()))
        starts = attn_metadata.query_start_loc
        for req_id, n_sched in scheduler_output.num_scheduled_tokens.items():
            req = requests[req_id]
            if len(req.prompt_token_ids) <= self.token_blk_size:
                continue
            row = input_batch.req_id_to_index[req_id]
            q_start = int(starts[row])
            meta.add_request(req_id, row, len(req.prompt_token_ids), len(req.output_token_ids), n_sched,
                             req.num_computed_tokens, scheduler_output.req_sparsed_slots[req_id], req.block_ids[0],
                             self.token_blk_size, req.prompt_token_ids, q_start, int(starts[row + 1]) - q_start,
                             self.kvstar_multistep_cfg["retrieval_stride"])
        self._sparse_metadata = meta
        held = self._step_cache.get("held")
        if held is not None:
            held.release()
        self._step_cache = {}
        self._n_slots = len(self._layer_slots)
        path = self._layer_path() if self.role == UcmSparseRole.WORKER else None
        if path is not None:
            path.build_step(meta, ReqStage)

    # ---- scheduler side ------------------------------------------------------------------
    def estimate_num_slots_sparsed(self, request) -> int:
        """Token slots of a decoding request: the windows, sparse_ratio of the prompt blocks between them,
        and everything generated since (multistep.py:775-814)."""
        if request.num_output_tokens == 0:
            return INVALID_SLOT
        bs = self.token_blk_size
        cfg = self.kvstar_multistep_cfg
        n_prefill = request.num_prompt_tokens // bs
        n_fixed = min(cfg["init_window_sz"] + cfg["local_window_sz"], n_prefill)
        n_saved = math.ceil((n_prefill - n_fixed) * cfg["sparse_ratio"])
        n_dense = math.ceil(request.num_tokens / bs)
        budget = n_dense - (n_prefill - n_saved - n_fixed)
        tail = request.num_tokens % bs
        return (budget - 1) * bs + tail if tail else budget * bs

    def allocate_slots(self, request, num_slots_sparsed, coordinator, block_pool, kv_cache_groups):
        """Keeps the last ceil(slots/block_size) blocks of the request, returns the others to the pool and
        allocates for the sparsified length (multistep.py:816-846)."""
        need = math.ceil(num_slots_sparsed / self.token_blk_size)
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
