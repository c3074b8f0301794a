"""``CalKpreAndTopk`` with the method surface of the reference's pybind11 module
``gsa_offload_ops`` (ucm/sparse/gsa/offload_ops/src/pybinds.cpp:9-25,
include/cal_kpre_and_topk.h:47-59), running on the GPU.

The reference object owns a copy thread and a calculate thread: queries are
pulled to the host one request at a time and the block scores and the top-k
are computed by OpenMP loops, layer after layer, while the model runs.  Here
every ``add_copy_req`` simply enqueues, on the caller's stream, the copy of the
queries into ``q_cache`` and then (when a top-k was requested for the step) the
scoring and selection kernels of that layer; results land in the caller-owned
``topk_cache`` tensors, which must be device tensors.  ``is_calculate_finish``
is an event query.

All tensors handed in (kpre caches, top-k caches) must live on the device; the
representatives are fp32 ``[rows, numKpre, kv_heads, head_dim]`` per layer, the
shape of the reference's ``kpre_caches``
(ucm/sparse/gsa/prefetch/prefetch_engine.py:64-77); with numKpre > 1 a row is
read as the reference's kernel reads it, kv head outermost.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ... import ops
from ..utils import INIT_WINDOW_BLOCKS, LOCAL_WINDOW_BLOCKS


def _common_layer_stride(tensors: Sequence[torch.Tensor]) -> Optional[int]:
    """Element stride between consecutive per-layer tensors if they are equally
    spaced views of one allocation, else None."""
    if len(tensors) < 2:
        return 0
    es = tensors[0].element_size()
    step = tensors[1].data_ptr() - tensors[0].data_ptr()
    if step <= 0 or step % es:
        return None
    for a, b in zip(tensors[:-1], tensors[1:]):
        if b.data_ptr() - a.data_ptr() != step or a.shape != b.shape:
            return None
    return step // es


class CalKpreAndTopk:
    def __init__(self, layer_num: int, block_size: int, max_bs: int, num_heads: int, head_size: int,
                 device: Optional[torch.device] = None):
        self.layer_num, self.block_size, self.max_bs = layer_num, block_size, max_bs
        self.q_heads, self.head_size = num_heads, head_size
        self.kv_heads, self.num_kpre = num_heads, 1
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
        self._q_all = torch.zeros((layer_num, max_bs, num_heads, head_size), dtype=torch.float32, device=self.device)
        self.q_cache: List[torch.Tensor] = list(self._q_all.unbind(0))
        self.k_cache: List[torch.Tensor] = []   # unused: block means are taken from the paged cache directly
        self._kpre: List[torch.Tensor] = []
        self._kpre_stride: Optional[int] = None
        self._topk_cache: List[torch.Tensor] = []
        self._topk_lens: List[int] = []
        self._cal_topk_idx: List[int] = []
        self._is_decode: List[bool] = []
        self._need_topk = False
        self._calc_block_table: Optional[torch.Tensor] = None
        self._calc_slots: List[int] = []
        self._desc = None
        self._slot_mapping: List[List[int]] = []
        self._done: Optional[torch.cuda.Event] = None
        self.init_window, self.local_window = INIT_WINDOW_BLOCKS, LOCAL_WINDOW_BLOCKS

    # ---- configuration ---------------------------------------------------
    def set_kpre_method_param(self, num_heads: int, num_kpre: int) -> None:
        """num_kpre representatives per (block, kv head): a block's score then takes, per head, the largest of the
        dots with them.  A row of the kpre caches is read the way the reference's kernel reads it, [kv head]
        [representative][channel] (select_topk_block.cpp: headBase = h * numKrepre * headSize)."""
        if num_kpre < 1 or num_heads * num_kpre > 16 or 16 % (num_heads * num_kpre):
            raise ValueError("kv heads x numKpre must be 1, 2, 4, 8 or 16")
        self.kv_heads, self.num_kpre = num_heads, num_kpre

    def set_kpre_cache(self, kpre_cache: Sequence[torch.Tensor]) -> None:
        row = self.kv_heads * self.num_kpre * self.head_size
        for t in kpre_cache:
            if not t.is_cuda or t.dtype != torch.float32 or not t.is_contiguous() or t[0].numel() != row:
                raise ValueError("kpre caches must be contiguous float32 device tensors [rows, numKpre, kv_heads, head_dim]")
        self._kpre = list(kpre_cache)
        self._kpre_stride = _common_layer_stride(self._kpre)

    def set_topk_cache(self, topk_cache: Sequence[torch.Tensor], topk_lens: Sequence[int]) -> None:
        for t in topk_cache:
            if not t.is_cuda or t.dtype != torch.int32 or t.dim() != 2 or not t.is_contiguous():
                raise ValueError("top-k caches must be contiguous int32 device tensors [batch, width]")
        self._topk_cache, self._topk_lens = list(topk_cache), [int(x) for x in topk_lens]

    def set_common_param(self, cal_topk_idx: Sequence[int], is_decode: Sequence[bool]) -> None:
        self._cal_topk_idx, self._is_decode = [int(x) for x in cal_topk_idx], [bool(x) for x in is_decode]

    def set_topk_param(self, repre_slot_mapping: Sequence[Sequence[int]]) -> None:
        """Arms the top-k of this step.  Entry i of the batch owns the contiguous
        representative rows repre_slot_mapping[i][0] .. +len-1
        (cal_kpre_and_topk.cpp:229-235); only decode entries are scored."""
        if len(repre_slot_mapping) != len(self._is_decode):
            raise ValueError("repre_slot_mapping must have one entry per batch entry")
        self._slot_mapping = [list(r) for r in repre_slot_mapping]
        self._desc = None  # packed when the first layer fires: the top-k lengths arrive after this call
        self._need_topk = True

    def _pack_descriptors(self) -> None:
        repre_slot_mapping = self._slot_mapping
        n = len(self._is_decode)
        seg_off, seg_len, topk, q_rows = [0] * n, [0] * n, [0] * n, [0] * n
        j = 0
        for i in range(n):
            if not self._is_decode[i]:
                continue
            seg_off[i], seg_len[i] = int(repre_slot_mapping[i][0]), len(repre_slot_mapping[i])
            topk[i], q_rows[i] = self._topk_lens[j], self._cal_topk_idx[j]
            j += 1
        host = torch.tensor([seg_off, seg_len, topk, q_rows], dtype=torch.int32).pin_memory()
        self._desc = dict(dev=host.to(self.device, non_blocking=True), host=host, n=n,
                          max_len=max(seg_len, default=0), total=sum(seg_len))

    def set_kpre_param(self, calc_block_table: torch.Tensor, calc_repre_slot_mapping: Sequence[int]) -> None:
        self._calc_block_table = calc_block_table
        self._calc_slots = [int(x) for x in calc_repre_slot_mapping]

    # ---- per-layer triggers ------------------------------------------------
    def add_copy_req(self, need_cal_kpre: bool, layer_idx: int, locations: Sequence[int], tensor: torch.Tensor) -> None:
        """locations non-empty: `tensor` holds one query row per batch entry
        ([batch, q_heads, head_dim]); rows whose location is -1 are skipped
        (cal_kpre_and_topk.cpp:134-150).  The layer's top-k follows at once.
        locations empty: the key side of the layer is ready; nothing to do here,
        the block means are produced by ucm_block_mean from the paged cache."""
        if len(locations) == 0:
            return
        keep = [i for i, loc in enumerate(locations) if loc != -1]
        if keep:
            sel = torch.tensor(keep, dtype=torch.long, device=self.device)
            self.q_cache[layer_idx].index_copy_(0, sel, tensor[sel].to(torch.float32))
        self.set_topk_data_ready(layer_idx)

    def set_kpre_data_ready(self, layer_idx: int) -> bool:
        return True

    def set_topk_data_ready(self, layer_idx: int) -> None:
        if not self._need_topk:
            return
        if self._desc is None:
            self._pack_descriptors()
        d = self._desc
        seg_off, seg_len, topk, q_rows = d["dev"][0], d["dev"][1], d["dev"][2], d["dev"][3]
        if d["max_len"] > 0:
            out = self._topk_cache[layer_idx]
            if out.shape[0] < d["n"] or out.shape[1] < d["max_len"]:
                raise ValueError("top-k cache too small for this batch")
            rows = self._kpre[layer_idx].shape[0]
            repre = self._kpre[layer_idx].view(1, rows, -1)
            scores = self._scores_buffer(rows)
            counts = self._counts_buffer(d["n"])
            ops.score_blocks(self.q_cache[layer_idx].unsqueeze(0), repre, seg_off, seg_len, d["max_len"],
                             self.kv_heads, scores, q_rows=q_rows, total_blocks=d["total"], num_repre=self.num_kpre)
            ops.topk_windows(scores, seg_off, seg_len, topk, d["max_len"], out[: d["n"]].unsqueeze(0), counts,
                             start_w=self.init_window, end_w=self.local_window)
        if layer_idx == self.layer_num - 1:
            self._done = torch.cuda.Event()
            self._done.record()
            self._need_topk = False

    def is_calculate_finish(self) -> bool:
        return self._done is None or self._done.query()

    # ---- scratch owned by the object (allocated once, grown on demand) ------
    def _scores_buffer(self, rows: int) -> torch.Tensor:
        buf = getattr(self, "_scores", None)
        if buf is None or buf.shape[1] < rows:
            self._scores = buf = torch.empty((1, rows), dtype=torch.float32, device=self.device)
        return buf

    def _counts_buffer(self, n: int) -> torch.Tensor:
        buf = getattr(self, "_counts", None)
        if buf is None or buf.shape[1] < n:
            self._counts = buf = torch.empty((1, max(n, 1)), dtype=torch.int32, device=self.device)
        return buf[:, :n]
