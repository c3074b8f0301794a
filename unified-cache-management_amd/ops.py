"""Torch-tensor front end of libucm_hip.so.

Every function takes CUDA(HIP) tensors, checks shapes/dtypes/contiguity on the
host, and enqueues the kernel on torch's current stream through the C ABI
(raw pointers only).  Nothing here computes on the CPU.
"""
from __future__ import annotations

import threading
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import MEAN_ABS, MEAN_BF16_ROUND, MEAN_BF16_STORE, MEAN_F32, MEAN_KEYS_F16, UcmHipError  # noqa: F401


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """torch's current stream on the current device as a raw handle.  The plugins call this twice per layer
    and decode step; building a torch.cuda.Stream object each time costs ~8 us, the raw query ~0.3 us."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def current_stream() -> int:
    """Raw handle of torch's current stream, for callers that go to the library themselves."""
    return _stream()


def _dev(t: torch.Tensor, dtype, name: str) -> int:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t.data_ptr()


def _opt(t: Optional[torch.Tensor], dtype, name: str):
    return None if t is None else _dev(t, dtype, name)


class _UploadRing:
    """Pinned staging for the small descriptor tables the wrappers and plugins send to the device many times per
    step: a slot is reused once the copy queued from it has completed (an event per slot), so no call allocates
    pinned memory.  Anything larger than a slot takes the allocator's route."""

    def __init__(self, slots: int = 64, slot_bytes: int = 1 << 16):
        self.slots, self.slot_bytes = slots, slot_bytes
        self.buf = None
        self.events = [None] * slots
        self.next = 0
        self.lock = threading.Lock()

    def put(self, host: torch.Tensor, device) -> torch.Tensor:
        nbytes = host.numel() * host.element_size()
        if nbytes > self.slot_bytes or nbytes == 0:
            return host.pin_memory().to(device, non_blocking=True)
        with self.lock:
            if self.buf is None:
                self.buf = torch.empty((self.slots, self.slot_bytes), dtype=torch.uint8, pin_memory=True)
            i = self.next
            self.next = (i + 1) % self.slots
            if self.events[i] is None:
                self.events[i] = torch.cuda.Event()
            else:
                self.events[i].synchronize()
            stage = self.buf[i, :nbytes].view(host.dtype).view(host.shape)
            stage.copy_(host)
            out = stage.to(device, non_blocking=True)
            self.events[i].record(torch.cuda.current_stream(device))   # the stream the copy was queued on
        return out


_rings: dict = {}        # one per device: a slot's event belongs to the device it was first recorded on


def upload(host: torch.Tensor, device) -> torch.Tensor:
    """A host tensor's values in a new device tensor, copied on the current stream without blocking the host."""
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    ring = _rings.get(index)
    if ring is None:
        ring = _rings.setdefault(index, _UploadRing())
    return ring.put(host.contiguous(), device)


class LayerPointers:
    """Device array of per-layer base pointers (one int64 tensor, built once).

    ``tensors`` are the per-layer cache tensors; they are kept alive here.
    ``sub(l)`` is the address of entry l, i.e. a one-layer pointer array.
    """

    def __init__(self, tensors: Sequence[torch.Tensor]):
        self.tensors = list(tensors)
        for t in self.tensors:
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError("layer tensors must be contiguous device tensors")
            if t.data_ptr() % 16:
                raise ValueError("layer tensors must be 16-byte aligned")
        self.table = torch.tensor([t.data_ptr() for t in self.tensors], dtype=torch.int64,
                                  device=self.tensors[0].device)

    def __len__(self) -> int:
        return len(self.tensors)

    def ptr(self, first_layer: int = 0) -> int:
        return self.table.data_ptr() + 8 * first_layer


def block_mean(k_layers: LayerPointers, block_ids: torch.Tensor, slots: torch.Tensor, repre: torch.Tensor,
               block_size: int, kv_heads: int, head_dim: int, num_blocks: int, mode: int = MEAN_F32,
               first_layer: int = 0, n_layers: Optional[int] = None) -> None:
    """repre: [L, rows, kv_heads*head_dim], fp32 (mode MEAN_F32 / MEAN_BF16_ROUND) or
    bf16 (the mode is then MEAN_BF16_STORE whatever was passed); rows ``slots`` of layers
    first_layer.. are overwritten with the means of cache blocks ``block_ids`` (``mode | MEAN_ABS``: of their
    absolute values).  The caches behind ``k_layers`` are bfloat16 or float16; with float16 ones MEAN_BF16_ROUND rounds
    to float16 (the cache's type) and a bfloat16 table is refused."""
    if repre.dim() != 3 or repre.shape[2] != kv_heads * head_dim:
        raise ValueError("repre must be [layers, rows, kv_heads*head_dim]")
    n_layers = len(k_layers) - first_layer if n_layers is None else n_layers
    if first_layer < 0 or first_layer + n_layers > min(len(k_layers), repre.shape[0]):
        raise ValueError("layer range outside the tables")
    if block_ids.numel() != slots.numel():
        raise ValueError("block_ids and slots differ in length")
    if repre.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("repre must be float32 or bfloat16")
    of_abs = mode & MEAN_ABS
    mode &= ~(MEAN_ABS | MEAN_KEYS_F16)
    if k_layers.tensors[first_layer].dtype == torch.float16:
        of_abs |= MEAN_KEYS_F16
    if repre.dtype == torch.bfloat16:
        mode = MEAN_BF16_STORE
    elif mode == MEAN_BF16_STORE:
        raise ValueError("MEAN_BF16_STORE needs a bfloat16 table")
    mode |= of_abs
    rp = _dev(repre, repre.dtype, "repre") + first_layer * repre.stride(0) * repre.element_size()
    _lib.call("ucm_block_mean", k_layers.ptr(first_layer), n_layers, num_blocks,
              _dev(block_ids, torch.int32, "block_ids"), _dev(slots, torch.int32, "slots"), block_ids.numel(),
              block_size, kv_heads, head_dim, rp, repre.shape[1], repre.stride(0), mode, _stream())


def score_blocks(q: torch.Tensor, repre: torch.Tensor, seg_off: torch.Tensor, seg_len: torch.Tensor,
                 max_seg_len: int, kv_heads: int, scores: torch.Tensor,
                 q_rows: Optional[torch.Tensor] = None, first_layer: int = 0,
                 n_layers: Optional[int] = None, total_blocks: int = 0, scale: float = 1.0, num_repre: int = 1,
                 tile_blocks: int = 0) -> None:
    """q: [L, rows, q_heads, head_dim] fp32, bf16 or fp16; repre: fp32 or bf16 [L, rows, kv_heads*num_repre*head_dim];
    scores: fp32 [L, rows].  Layers first_layer .. first_layer+n_layers-1 are scored.
    total_blocks: sum of seg_len when the host knows it (tighter grid), else 0.  scale multiplies every score
    (1/kv_heads: the mean over all q heads the reference's torch variant ranks by).  tile_blocks: blocks per
    workgroup, 0 = the library's choice (benchmarks and tests)."""
    if q.dim() != 4 or repre.dim() != 3 or scores.dim() != 2:
        raise ValueError("q [L,rows,Hq,D], repre [L,rows,Hkv*D], scores [L,rows] expected")
    head_dim, q_heads = q.shape[3], q.shape[2]
    if repre.shape[2] != kv_heads * num_repre * head_dim:
        raise ValueError("repre row does not match kv_heads*num_repre*head_dim")
    if repre.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("repre must be float32 or bfloat16")
    qd = _q_code(q)
    n_layers = repre.shape[0] - first_layer if n_layers is None else n_layers
    if first_layer < 0 or first_layer + n_layers > min(q.shape[0], repre.shape[0], scores.shape[0]):
        raise ValueError("layer range outside the tables")
    n_req = seg_off.numel()
    if seg_len.numel() != n_req or (q_rows is not None and q_rows.numel() != n_req):
        raise ValueError("seg_off / seg_len / q_rows differ in length")
    if q_rows is None and q.shape[1] < n_req:
        raise ValueError("q has fewer rows than requests")
    if scores.shape[1] < repre.shape[1]:
        raise ValueError("scores row shorter than the representative table")
    es = q.element_size()
    _lib.call("ucm_score_blocks", _dev(q, q.dtype, "q") + first_layer * q.stride(0) * es, qd, q.stride(0),
              _opt(q_rows, torch.int32, "q_rows"), q_heads,
              _dev(repre, repre.dtype, "repre") + first_layer * repre.stride(0) * repre.element_size(),
              _lib.DTYPE_BF16 if repre.dtype == torch.bfloat16 else _lib.DTYPE_F32, repre.stride(0), repre.shape[1],
              num_repre, _dev(seg_off, torch.int32, "seg_off"), _dev(seg_len, torch.int32, "seg_len"), n_req, max_seg_len,
              total_blocks, n_layers, kv_heads, head_dim,
              _dev(scores, torch.float32, "scores") + first_layer * scores.stride(0) * 4, scores.stride(0),
              float(scale), int(tile_blocks), _stream())


def _q_code(q: torch.Tensor) -> int:
    code = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16}.get(q.dtype)
    if code is None:
        raise ValueError("q must be float32, bfloat16 or float16")
    return code


def score_select(q: torch.Tensor, repre: torch.Tensor, seg_off: torch.Tensor, seg_len: torch.Tensor,
                 topk_len: torch.Tensor, max_seg_len: int, kv_heads: int, scores: torch.Tensor, idx_out: torch.Tensor,
                 count_out: torch.Tensor, tickets: torch.Tensor, start_w: int = 1, end_w: int = 2,
                 q_rows: Optional[torch.Tensor] = None, block_tables: Optional[torch.Tensor] = None,
                 phys_out: Optional[torch.Tensor] = None, seq_lens: Optional[torch.Tensor] = None, block_size: int = 0,
                 sparse_seq_lens: Optional[torch.Tensor] = None, first_layer: int = 0, n_layers: Optional[int] = None,
                 scale: float = 1.0, num_repre: int = 1, tile_blocks: int = 0, total_blocks: int = 0) -> None:
    """score_blocks and topk_windows as one launch (ucm_score_select): q [L, rows, q_heads, head_dim] whose layer 0
    belongs to ``first_layer``... of the tables; tickets int32 [L, n_req], zero before the first call and left zero."""
    if q.dim() != 4 or repre.dim() != 3 or scores.dim() != 2:
        raise ValueError("q [L,rows,Hq,D], repre [L,rows,Hkv*D], scores [L,rows] expected")
    head_dim, q_heads = q.shape[3], q.shape[2]
    if repre.shape[2] != kv_heads * num_repre * head_dim:
        raise ValueError("repre row does not match kv_heads*num_repre*head_dim")
    n_req = seg_off.numel()
    n_layers = q.shape[0] if n_layers is None else n_layers
    if first_layer < 0 or first_layer + n_layers > min(repre.shape[0], scores.shape[0], idx_out.shape[0]) or n_layers > q.shape[0]:
        raise ValueError("layer range outside the tables")
    if idx_out.dim() != 3 or idx_out.shape[1] != n_req or count_out.shape != idx_out.shape[:2] or tickets.shape != count_out.shape:
        raise ValueError("idx_out [L,n_req,stride], count_out and tickets [L,n_req] expected")
    if scores.shape[1] < repre.shape[1]:
        raise ValueError("scores row shorter than the representative table")
    if phys_out is not None and phys_out.shape != idx_out.shape:
        raise ValueError("phys_out must have idx_out's shape")
    if sparse_seq_lens is not None and sparse_seq_lens.shape != count_out.shape:
        raise ValueError("sparse_seq_lens must have count_out's shape")
    args = _lib.ScoreSelectArgs(
        q=_dev(q, q.dtype, "q"), q_dtype=_q_code(q), q_heads=q_heads, q_layer_stride=q.stride(0),
        q_rows=_opt(q_rows, torch.int32, "q_rows"), repre=_dev(repre, repre.dtype, "repre"),
        repre_dtype=_lib.DTYPE_BF16 if repre.dtype == torch.bfloat16 else _lib.DTYPE_F32,
        repre_layer_stride=repre.stride(0), repre_rows=repre.shape[1], seg_off=_dev(seg_off, torch.int32, "seg_off"),
        seg_len=_dev(seg_len, torch.int32, "seg_len"), topk_len=_dev(topk_len, torch.int32, "topk_len"), n_req=n_req,
        max_seg_len=max_seg_len, first_layer=first_layer, kv_heads=kv_heads, head_dim=head_dim,
        scores=_dev(scores, torch.float32, "scores"), scores_layer_stride=scores.stride(0), tile_blocks=int(tile_blocks),
        start_w=start_w, end_w=end_w, idx_out=_dev(idx_out, torch.int32, "idx_out"),
        count_out=_dev(count_out, torch.int32, "count_out"), out_stride=idx_out.shape[2],
        bt_stride=0 if block_tables is None else block_tables.shape[1],
        block_tables=_opt(block_tables, torch.int32, "block_tables"), phys_out=_opt(phys_out, torch.int32, "phys_out"),
        seq_lens=_opt(seq_lens, torch.int32, "seq_lens"), sparse_seq_lens=_opt(sparse_seq_lens, torch.int32, "sparse_seq_lens"),
        block_size=block_size, tickets=_dev(tickets, torch.int32, "tickets"))
    args.n_layers, args.num_repre, args.scale, args.total_blocks = n_layers, num_repre, float(scale), int(total_blocks)
    import ctypes as C

    _lib.call("ucm_score_select", C.addressof(args), _stream())


def topk_windows(scores: torch.Tensor, seg_off: torch.Tensor, seg_len: torch.Tensor, topk_len: torch.Tensor,
                 max_seg_len: int, idx_out: torch.Tensor, count_out: torch.Tensor, start_w: int = 1,
                 end_w: int = 2, block_tables: Optional[torch.Tensor] = None,
                 phys_out: Optional[torch.Tensor] = None, seq_lens: Optional[torch.Tensor] = None,
                 block_size: int = 0, sparse_seq_lens: Optional[torch.Tensor] = None, first_layer: int = 0,
                 n_layers: Optional[int] = None) -> None:
    """scores fp32 [L, rows]; idx_out/phys_out int32 [L, n_req, stride]; count_out int32 [L, n_req]."""
    n_req = seg_off.numel()
    if idx_out.dim() != 3 or idx_out.shape[1] != n_req or count_out.shape != idx_out.shape[:2]:
        raise ValueError("idx_out [L,n_req,stride] and count_out [L,n_req] expected")
    n_layers = scores.shape[0] - first_layer if n_layers is None else n_layers
    if first_layer < 0 or first_layer + n_layers > min(scores.shape[0], idx_out.shape[0]):
        raise ValueError("layer range outside the tables")
    if phys_out is not None and phys_out.shape != idx_out.shape:
        raise ValueError("phys_out must have idx_out's shape")
    if block_tables is not None and (block_tables.dim() != 2 or block_tables.shape[0] != n_req):
        raise ValueError("block_tables must be [n_req, stride]")
    if sparse_seq_lens is not None and sparse_seq_lens.shape != count_out.shape:
        raise ValueError("sparse_seq_lens must have count_out's shape")
    o = first_layer * idx_out.stride(0) * 4
    c = first_layer * count_out.stride(0) * 4
    _lib.call("ucm_topk_windows", _dev(scores, torch.float32, "scores") + first_layer * scores.stride(0) * 4,
              scores.stride(0), scores.shape[1], _dev(seg_off, torch.int32, "seg_off"), _dev(seg_len, torch.int32, "seg_len"),
              _dev(topk_len, torch.int32, "topk_len"), n_req, max_seg_len, n_layers, start_w, end_w,
              _dev(idx_out, torch.int32, "idx_out") + o, idx_out.shape[2],
              _dev(count_out, torch.int32, "count_out") + c,
              _opt(block_tables, torch.int32, "block_tables"),
              0 if block_tables is None else block_tables.shape[1],
              None if phys_out is None else _dev(phys_out, torch.int32, "phys_out") + o,
              _opt(seq_lens, torch.int32, "seq_lens"), block_size,
              None if sparse_seq_lens is None else _dev(sparse_seq_lens, torch.int32, "sparse_seq_lens") + c,
              _stream())


def kvstar_topk(votes: torch.Tensor, seg_off: torch.Tensor, seg_len: torch.Tensor, topk_len: torch.Tensor,
                max_seg_len: int, idx_out: torch.Tensor, count_out: torch.Tensor) -> None:
    """votes fp32 [rows]; idx_out int32 [n_tasks, stride] (ascending block indices); count_out int32 [n_tasks]."""
    n_tasks = seg_off.numel()
    if idx_out.dim() != 2 or idx_out.shape[0] != n_tasks or count_out.numel() != n_tasks:
        raise ValueError("idx_out [n_tasks,stride] and count_out [n_tasks] expected")
    _lib.call("ucm_kvstar_topk", _dev(votes, torch.float32, "votes"), votes.numel(), _dev(seg_off, torch.int32, "seg_off"),
              _dev(seg_len, torch.int32, "seg_len"), _dev(topk_len, torch.int32, "topk_len"), n_tasks, max_seg_len,
              _dev(idx_out, torch.int32, "idx_out"), idx_out.shape[1], _dev(count_out, torch.int32, "count_out"),
              _stream())


def kvstar_order(votes: torch.Tensor, seg_off: torch.Tensor, seg_len: torch.Tensor, max_count: int, idx: torch.Tensor,
                 count: torch.Tensor) -> None:
    """Puts every task's chosen blocks (kvstar_topk's idx [n_tasks, stride] and count [n_tasks]) into the order the
    reference returns them in: descending by (vote, index)."""
    n_tasks = count.numel()
    if idx.dim() != 2 or idx.shape[0] != n_tasks or seg_off.numel() != n_tasks or seg_len.numel() != n_tasks:
        raise ValueError("idx [n_tasks, stride] and seg_off, seg_len, count [n_tasks] expected")
    _lib.call("ucm_kvstar_order", _dev(votes, torch.float32, "votes"), votes.numel(), _dev(seg_off, torch.int32, "seg_off"),
              _dev(seg_len, torch.int32, "seg_len"), n_tasks, max_count, _dev(idx, torch.int32, "idx"), idx.shape[1],
              _dev(count, torch.int32, "count"), _stream())


def esa_retrieve(data: torch.Tensor, q: torch.Tensor, indexes: torch.Tensor, topk: int, scores_ws: torch.Tensor,
                 out_idx: torch.Tensor, out_scores: torch.Tensor, out_count: torch.Tensor,
                 stream: Optional[int] = None) -> None:
    """data fp32 [N, dim]; q fp32 [B, dim]; indexes int32 [B, M] (-1 padded); outputs [B, stride]."""
    if data.dim() != 2 or q.dim() != 2 or indexes.dim() != 2:
        raise ValueError("data [N,dim], q [B,dim], indexes [B,M] expected")
    batch, m = indexes.shape
    if q.shape != (batch, data.shape[1]):
        raise ValueError("q must be [B, dim]")
    if scores_ws.numel() < batch * m or out_idx.shape != out_scores.shape or out_idx.shape[0] != batch:
        raise ValueError("workspace / outputs too small")
    _lib.call("ucm_esa_retrieve", _dev(data, torch.float32, "data"), data.shape[0], data.shape[1],
              _dev(q, torch.float32, "q"), _dev(indexes, torch.int32, "indexes"), batch, m, int(topk),
              _dev(scores_ws, torch.float32, "scores_ws"), _dev(out_idx, torch.int32, "out_idx"),
              _dev(out_scores, torch.float32, "out_scores"), _dev(out_count, torch.int32, "out_count"),
              out_idx.shape[1], _stream() if stream is None else stream)


def delta_plan(sel: torch.Tensor, sel_phys: torch.Tensor, count: torch.Tensor, resident: torch.Tensor,
               load_phys: torch.Tensor, slot_of_sel: torch.Tensor, miss_count: torch.Tensor) -> None:
    """sel / sel_phys / slot_of_sel int32 [L, n_req, stride]; count / miss_count int32 [L, n_req];
    resident / load_phys int32 [L, n_req, n_slots] (resident is updated in place)."""
    n_layers, n_req, stride = sel.shape
    if sel_phys.shape != sel.shape or slot_of_sel.shape != sel.shape or count.shape != (n_layers, n_req) \
            or miss_count.shape != count.shape or resident.shape[:2] != (n_layers, n_req) \
            or load_phys.shape != resident.shape:
        raise ValueError("delta_plan: inconsistent shapes")
    _lib.call("ucm_delta_plan", _dev(sel, torch.int32, "sel"), _dev(sel_phys, torch.int32, "sel_phys"),
              _dev(count, torch.int32, "count"), n_req, n_layers, stride, _dev(resident, torch.int32, "resident"),
              resident.shape[2], _dev(load_phys, torch.int32, "load_phys"),
              _dev(slot_of_sel, torch.int32, "slot_of_sel"), _dev(miss_count, torch.int32, "miss_count"), _stream())


def esa_retrieve_rows(data: torch.Tensor, q: torch.Tensor, slot_table: torch.Tensor, m: int, rows: torch.Tensor,
                      topk_rows: torch.Tensor, max_topk: int, scores_ws: torch.Tensor, out_idx: torch.Tensor,
                      out_pos: Optional[torch.Tensor], out_scores: torch.Tensor, out_count: torch.Tensor) -> None:
    """data fp32 [N, dim]; q fp32 [B, dim]; slot_table int32 [table_rows, stride] (-1 padded), of which the first
    ``m`` entries of a row are looked at; rows int32 [B]; topk_rows int32 [table_rows]; out_idx / out_pos /
    out_scores [table_rows, out_stride]; out_count int32 [table_rows]."""
    if data.dim() != 2 or q.dim() != 2 or slot_table.dim() != 2 or q.shape[1] != data.shape[1]:
        raise ValueError("data [N,dim], q [B,dim], slot_table [rows,stride] expected")
    batch, (table_rows, stride) = rows.numel(), slot_table.shape
    if m > stride:
        raise ValueError("m exceeds the table's row length")
    if q.shape[0] != batch or scores_ws.numel() < batch * m:
        raise ValueError("q / scores_ws do not cover the batch")
    if out_idx.shape[0] != table_rows or out_scores.shape != out_idx.shape or out_count.numel() != table_rows \
            or topk_rows.numel() != table_rows or (out_pos is not None and out_pos.shape != out_idx.shape):
        raise ValueError("per-row outputs must have one row per table row")
    _lib.call("ucm_esa_retrieve_rows", _dev(data, torch.float32, "data"), data.shape[0], data.shape[1],
              _dev(q, torch.float32, "q"), _dev(slot_table, torch.int32, "slot_table"), table_rows, stride, int(m),
              _dev(rows, torch.int32, "rows"), batch, _dev(topk_rows, torch.int32, "topk_rows"), int(max_topk),
              _dev(scores_ws, torch.float32, "scores_ws"), _dev(out_idx, torch.int32, "out_idx"),
              _opt(out_pos, torch.int32, "out_pos"), _dev(out_scores, torch.float32, "out_scores"),
              _dev(out_count, torch.int32, "out_count"), out_idx.shape[1], _stream())


def delta_plan_rows(sel: torch.Tensor, sel_phys: torch.Tensor, count: torch.Tensor, rows: torch.Tensor,
                    resident: torch.Tensor, load_phys: torch.Tensor, slot_of_sel: torch.Tensor,
                    miss_count: torch.Tensor) -> None:
    """As delta_plan, every array [L, table_rows, ...]; only the rows listed in ``rows`` (int32 [B]) are planned."""
    n_layers, table_rows, stride = sel.shape
    if sel_phys.shape != sel.shape or slot_of_sel.shape != sel.shape or count.shape != (n_layers, table_rows) \
            or miss_count.shape != count.shape or resident.shape[:2] != (n_layers, table_rows) \
            or load_phys.shape != resident.shape:
        raise ValueError("delta_plan_rows: inconsistent shapes")
    _lib.call("ucm_delta_plan_rows", _dev(sel, torch.int32, "sel"), _dev(sel_phys, torch.int32, "sel_phys"),
              _dev(count, torch.int32, "count"), _dev(rows, torch.int32, "rows"), rows.numel(), table_rows, n_layers,
              stride, _dev(resident, torch.int32, "resident"), resident.shape[2],
              _dev(load_phys, torch.int32, "load_phys"), _dev(slot_of_sel, torch.int32, "slot_of_sel"),
              _dev(miss_count, torch.int32, "miss_count"), _stream())


def kv_load_planned(layers: LayerPointers, ptr_first: int, store_first_layer: int, n_layers: int, kv_stride: int,
                    block_bytes: int, num_blocks: int, pool: torch.Tensor, pool_block_bytes: int,
                    load_sel: torch.Tensor, src_table: torch.Tensor, dst_table: torch.Tensor,
                    rows: Optional[torch.Tensor], load_count: Optional[torch.Tensor] = None, rank: int = 0,
                    tp_size: int = 1) -> None:
    """pool: uint8 buffer of stored blocks ([block][layer][K|V], device or pinned host memory); load_sel int32
    [n_layers, table_rows, n_slots]: the plan of model layers store_first_layer.., whose cache pointers are entries
    ptr_first.. of ``layers``; src_table int32 [table_rows, M]; dst_table int32 [table_rows, >= n_slots], or
    [n_layers, table_rows, >= n_slots] when every layer has destinations of its own; load_count int32
    [n_layers, table_rows] or None; rows int32 [B] or None (all table rows).  tp_size > 1: the stored blocks are the ones
    tp_size ranks share ([layer][rank][K|V] slices of block_bytes each) and ``rank``'s slices are read."""
    if load_sel.dim() != 3 or load_sel.shape[0] != n_layers:
        raise ValueError("load_sel must be [n_layers, table_rows, n_slots]")
    table_rows, n_slots = load_sel.shape[1], load_sel.shape[2]
    per_layer = dst_table.dim() == 3
    if src_table.shape[0] != table_rows or dst_table.shape[-2] != table_rows or dst_table.shape[-1] < n_slots \
            or (per_layer and dst_table.shape[0] != n_layers):
        raise ValueError("src_table / dst_table must have one row per table row")
    if load_count is not None and load_count.shape != (n_layers, table_rows):
        raise ValueError("load_count must be [n_layers, table_rows]")
    if ptr_first < 0 or ptr_first + n_layers > len(layers):
        raise ValueError("layer range outside the pointer table")
    nbytes = pool.numel() * pool.element_size()
    _lib.call("ucm_kv_load_planned_tp", layers.ptr(ptr_first), n_layers, kv_stride, block_bytes, num_blocks,
              _staging_ptr(pool, 0), nbytes // pool_block_bytes, pool_block_bytes, store_first_layer,
              _dev(load_sel, torch.int32, "load_sel"), n_slots, _dev(src_table, torch.int32, "src_table"),
              src_table.shape[1], _dev(dst_table, torch.int32, "dst_table"), dst_table.shape[-1],
              dst_table.stride(0) if per_layer else 0, _opt(load_count, torch.int32, "load_count"),
              _opt(rows, torch.int32, "rows"), table_rows if rows is None else rows.numel(), table_rows, int(rank),
              int(tp_size), _stream())


def prefetch_plan(map_block: torch.Tensor, map_len: torch.Tensor, map_idx: torch.Tensor, topk_idx: torch.Tensor,
                  topk_len: torch.Tensor, rows: torch.Tensor, bs_index: torch.Tensor, free_block: torch.Tensor,
                  free_len: torch.Tensor, success_blocks: torch.Tensor, success_len: torch.Tensor,
                  load_blocks: torch.Tensor, load_count: torch.Tensor, miss_idxs: torch.Tensor,
                  miss_count: torch.Tensor) -> None:
    """map_block int32 [table_rows, cap]; map_idx int32 [L, table_rows, cap]; topk_idx int32 [L, B, stride];
    free_block / success_blocks int32 [L, max_bs, row_len]; free_len / success_len int32 [L, max_bs];
    load_blocks int32 [L, table_rows, cap]; miss_idxs int32 [L, table_rows, stride]; counts int32 [L, table_rows]."""
    n_layers, table_rows, cap = map_idx.shape
    batch = rows.numel()
    if map_block.shape != (table_rows, cap) or map_len.numel() != table_rows:
        raise ValueError("map_block [table_rows, cap] / map_len [table_rows] expected")
    if topk_idx.dim() != 3 or topk_idx.shape[:2] != (n_layers, batch) or topk_len.numel() != batch or bs_index.numel() != batch:
        raise ValueError("topk_idx [L, B, stride], topk_len / rows / bs_index [B] expected")
    max_bs, row_len = free_block.shape[1], free_block.shape[2]
    if free_block.shape[0] != n_layers or success_blocks.shape != free_block.shape or free_len.shape != (n_layers, max_bs) \
            or success_len.shape != free_len.shape:
        raise ValueError("free / success tables must be [L, max_bs, row_len] and [L, max_bs]")
    if load_blocks.shape != (n_layers, table_rows, cap) or miss_idxs.shape != (n_layers, table_rows, topk_idx.shape[2]) \
            or load_count.shape != (n_layers, table_rows) or miss_count.shape != load_count.shape:
        raise ValueError("load / miss outputs have the wrong shape")
    _lib.call("ucm_prefetch_plan", _dev(map_block, torch.int32, "map_block"), _dev(map_len, torch.int32, "map_len"),
              _dev(map_idx, torch.int32, "map_idx"), table_rows, cap, _dev(topk_idx, torch.int32, "topk_idx"),
              topk_idx.shape[2], _dev(topk_len, torch.int32, "topk_len"), _dev(rows, torch.int32, "rows"),
              _dev(bs_index, torch.int32, "bs_index"), batch, n_layers, max_bs, row_len,
              _dev(free_block, torch.int32, "free_block"), _dev(free_len, torch.int32, "free_len"),
              _dev(success_blocks, torch.int32, "success_blocks"), _dev(success_len, torch.int32, "success_len"),
              _dev(load_blocks, torch.int32, "load_blocks"), _dev(load_count, torch.int32, "load_count"),
              _dev(miss_idxs, torch.int32, "miss_idxs"), _dev(miss_count, torch.int32, "miss_count"), _stream())


HASH_SCORE_SUM, HASH_SCORE_BLOCK_CODE = 0, 1


def hash_encode_blocks(k_layers: LayerPointers, block_ids: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                       n: int, w: torch.Tensor, block_size: int, kv_heads: int, num_blocks: int,
                       colsum: torch.Tensor, block_codes: torch.Tensor,
                       token_codes: Optional[torch.Tensor] = None, workgroups: int = 0) -> None:
    """w [128, 128] in the caches' type (bfloat16 or float16); colsum int16 [L, rows, kv_heads, 128]; block_codes uint8
    [L, rows, kv_heads, 16]; token_codes uint8 [L, rows, block_size, kv_heads, 16] or None; workgroups: persistent
    workgroups over all layers, 0 = the library's choice (benchmarks and tests)."""
    key_dtype = k_layers.tensors[0].dtype if k_layers.tensors else w.dtype
    if key_dtype not in (torch.bfloat16, torch.float16) or w.dtype != key_dtype:
        raise ValueError("hash_encode_blocks takes bfloat16 or float16 key caches and weights of the same type")
    if w.shape != (128, 128):
        raise ValueError("w must be [128, 128]")
    n_layers, rows = colsum.shape[0], colsum.shape[1]
    if colsum.shape != (n_layers, rows, kv_heads, 128) or block_codes.shape != (n_layers, rows, kv_heads, 16):
        raise ValueError("colsum [L,rows,Hkv,128] / block_codes [L,rows,Hkv,16] expected")
    if n_layers != len(k_layers):
        raise ValueError("one output layer per cache layer")
    if token_codes is not None and token_codes.shape != (n_layers, rows, block_size, kv_heads, 16):
        raise ValueError("token_codes must be [L, rows, block_size, kv_heads, 16]")
    _lib.call("ucm_hash_encode_blocks_f16" if key_dtype == torch.float16 else "ucm_hash_encode_blocks", k_layers.ptr(), n_layers,
              num_blocks, _opt(block_ids, torch.int32, "block_ids"),
              _opt(slots, torch.int32, "slots"), n, block_size, kv_heads, 128, _dev(w, key_dtype, "w"), 128, rows,
              _opt(token_codes, torch.uint8, "token_codes"), 0 if token_codes is None else token_codes.stride(0),
              _dev(colsum, torch.int16, "colsum"), colsum.stride(0), _dev(block_codes, torch.uint8, "block_codes"),
              block_codes.stride(0), int(workgroups), _stream())


def hash_encode_queries(q: torch.Tensor, w: torch.Tensor, kv_heads: int, q_codes: torch.Tensor, q_sum: torch.Tensor,
                        qbar_codes: torch.Tensor, n_req: int, q_rows: Optional[torch.Tensor] = None) -> None:
    """q bf16 [L, rows, q_heads, 128] (or float16 with float16 weights); q_codes u8
    [L, n_req, q_heads, 16]; q_sum int16 [L, n_req, 128]; qbar_codes u8 [L, n_req, kv_heads, 16]."""
    n_layers, _, q_heads, d = q.shape
    if q.dtype not in (torch.bfloat16, torch.float16) or w.dtype != q.dtype:
        raise ValueError("hash_encode_queries takes bfloat16 or float16 queries and weights of the same type")
    if q_codes.shape != (n_layers, n_req, q_heads, 16) or q_sum.shape != (n_layers, n_req, 128) \
            or qbar_codes.shape != (n_layers, n_req, kv_heads, 16):
        raise ValueError("query code outputs have the wrong shape")
    if q_rows is None and q.shape[1] < n_req:
        raise ValueError("q has fewer rows than requests")
    _lib.call("ucm_hash_encode_queries_f16" if q.dtype == torch.float16 else "ucm_hash_encode_queries", _dev(q, q.dtype, "q"),
              q.stride(0), _opt(q_rows, torch.int32, "q_rows"), n_req, n_layers, q_heads, kv_heads, d, _dev(w, q.dtype, "w"), 128,
              _dev(q_codes, torch.uint8, "q_codes"), _dev(q_sum, torch.int16, "q_sum"),
              _dev(qbar_codes, torch.uint8, "qbar_codes"), _stream())


def hash_score_blocks(mode: int, q_sum: torch.Tensor, qbar_codes: torch.Tensor, colsum: torch.Tensor,
                      block_codes: torch.Tensor, seg_off: torch.Tensor, seg_len: torch.Tensor, total_blocks: int,
                      scores: torch.Tensor, round_fp16: bool = False) -> None:
    n_layers, rows, kv_heads, _ = colsum.shape
    n_req = seg_off.numel()
    if scores.dim() != 2 or scores.shape[0] != n_layers or scores.shape[1] < rows:
        raise ValueError("scores must be [L, >= rows]")
    _lib.call("ucm_hash_score_blocks", mode, _dev(q_sum, torch.int16, "q_sum"), _dev(qbar_codes, torch.uint8, "qbar_codes"),
              _dev(colsum, torch.int16, "colsum"), colsum.stride(0), _dev(block_codes, torch.uint8, "block_codes"),
              block_codes.stride(0), rows, _dev(seg_off, torch.int32, "seg_off"), _dev(seg_len, torch.int32, "seg_len"),
              n_req, total_blocks, n_layers, kv_heads, 128, _dev(scores, torch.float32, "scores"), scores.stride(0),
              int(round_fp16), _stream())


def copy_batch(dst_ptrs: torch.Tensor, src_ptrs: torch.Tensor, size: int) -> None:
    """dst_ptrs/src_ptrs: int64 device tensors of raw addresses; copies size bytes each."""
    if dst_ptrs.numel() != src_ptrs.numel():
        raise ValueError("pointer arrays differ in length")
    _lib.call("ucm_copy_batch", _dev(dst_ptrs, torch.int64, "dst_ptrs"), _dev(src_ptrs, torch.int64, "src_ptrs"),
              dst_ptrs.numel(), size, _stream())


def park_rows(src: torch.Tensor, src_idx: torch.Tensor, dst: torch.Tensor, dst_idx: Optional[torch.Tensor] = None) -> None:
    """dst[dst_idx[i]] = src[src_idx[i]] for 2-D (or flattened to rows) contiguous device tensors of one dtype and row
    size; dst_idx None: row i.  Pairs with an index outside its tensor are skipped."""
    if src.dtype != dst.dtype or not (src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("src and dst must be contiguous device tensors of one dtype")
    if src.dim() < 2 or dst.dim() < 2 or src.shape[1:] != dst.shape[1:]:
        raise ValueError("src and dst must be arrays of rows of one shape")
    n = src_idx.numel()
    if dst_idx is not None and dst_idx.numel() != n:
        raise ValueError("index arrays differ in length")
    row_bytes = src[0].numel() * src.element_size()
    _lib.call("ucm_park_rows", src.data_ptr(), src.shape[0], _dev(src_idx, torch.int32, "src_idx"), dst.data_ptr(),
              dst.shape[0], _opt(dst_idx, torch.int32, "dst_idx"), n, row_bytes, _stream())


def _staging_ptr(staging: torch.Tensor, need: int) -> int:
    if not (staging.is_cuda or staging.is_pinned()):
        raise ValueError("staging must be device or pinned host memory")
    if not staging.is_contiguous() or staging.numel() * staging.element_size() < need:
        raise ValueError(f"staging must be contiguous and hold {need} bytes")
    return staging.data_ptr()


def kv_gather_blocks(layers: LayerPointers, kv_stride: int, block_bytes: int, num_blocks: int,
                     block_ids: torch.Tensor, staging: torch.Tensor, rank: int = 0, tp_size: int = 1) -> None:
    """Cache blocks ``block_ids`` of every layer into ``staging`` in the stored-block layout; with tp_size > 1 the
    staging blocks are the wider ones tp_size ranks share ([layer][rank][K|V]) and only ``rank``'s slices are written."""
    n = block_ids.numel()
    _lib.call("ucm_kv_gather_blocks_tp", layers.ptr(), len(layers), kv_stride, block_bytes, num_blocks,
              _dev(block_ids, torch.int32, "block_ids"), n,
              _staging_ptr(staging, n * len(layers) * 2 * block_bytes * tp_size), int(rank), int(tp_size), _stream())


def kv_scatter_blocks(layers: LayerPointers, kv_stride: int, block_bytes: int, num_blocks: int,
                      block_ids: torch.Tensor, staging: torch.Tensor, rank: int = 0, tp_size: int = 1) -> None:
    n = block_ids.numel()
    _lib.call("ucm_kv_scatter_blocks_tp", layers.ptr(), len(layers), kv_stride, block_bytes, num_blocks,
              _dev(block_ids, torch.int32, "block_ids"), n,
              _staging_ptr(staging, n * len(layers) * 2 * block_bytes * tp_size), int(rank), int(tp_size), _stream())


def kv_gather_selected(layers: LayerPointers, kv_stride: int, block_bytes: int, num_blocks: int,
                       phys: torch.Tensor, count: torch.Tensor, dst_off: torch.Tensor, region_k: torch.Tensor,
                       max_count: int, staging: torch.Tensor, staging_blocks: int) -> None:
    """phys int32 [L, n_req, stride], count int32 [L, n_req]; staging holds staging_blocks blocks."""
    if phys.dim() != 3 or phys.shape[0] != len(layers) or count.shape != phys.shape[:2]:
        raise ValueError("phys [L,n_req,stride] / count [L,n_req] expected")
    n_req = phys.shape[1]
    if dst_off.numel() != n_req or region_k.numel() != n_req:
        raise ValueError("dst_off / region_k must have one entry per request")
    _lib.call("ucm_kv_gather_selected", layers.ptr(), len(layers), kv_stride, block_bytes, num_blocks,
              _dev(phys, torch.int32, "phys"), _dev(count, torch.int32, "count"), n_req, phys.shape[2],
              _dev(dst_off, torch.int64, "dst_off"), _dev(region_k, torch.int32, "region_k"), max_count,
              _staging_ptr(staging, staging_blocks * block_bytes), staging_blocks, _stream())


def kvstar_table(n_layers: int, kv_heads: int, rows: int, sub_blocks: int, d_pad: int, device,
                 layout: str = "head") -> torch.Tensor:
    """Empty KVStar representative table, fp16, indexed [L, kv_heads, rows, d_pad/8, M, 8]: per kv head and block
    a cell with the 16-byte pieces (8 channels) of the M sub-blocks side by side, the order the score kernel
    streams.  layout "head" keeps a plane per kv head, "row" the kv heads of a row next to each other in memory
    (the returned tensor is then a permuted view); the kernels take either and run equally fast on both."""
    if d_pad % 16 != 0:
        raise ValueError("d_pad must be a multiple of 16")
    if layout == "head":
        return torch.empty((n_layers, kv_heads, rows, d_pad // 8, sub_blocks, 8), dtype=torch.float16, device=device)
    if layout != "row":
        raise ValueError("layout must be 'row' or 'head'")
    return torch.empty((n_layers, rows, kv_heads, d_pad // 8, sub_blocks, 8), dtype=torch.float16,
                       device=device).permute(0, 2, 1, 3, 4, 5)


def _kvstar_cell_strides(t: torch.Tensor, what: str):
    """(head stride, row stride) in elements of a [kv_heads, rows, d_pad/8, M, 8] view whose cells are dense."""
    kv_heads, rows, pieces, m, _ = t.shape
    cell = pieces * m * 8
    if rows and kv_heads and not t[0, 0].is_contiguous():
        raise ValueError(f"{what}: a (kv head, row) cell [d_pad/8, M, 8] must be contiguous")
    row_stride = t.stride(1) if rows > 1 else cell
    head_stride = t.stride(0) if kv_heads > 1 else max(rows, 1) * row_stride
    return head_stride, row_stride


def kvstar_table_to_reference(table: torch.Tensor) -> torch.Tensor:
    """[..., kv_heads, rows, d_pad/8, M, 8] -> the reference's [..., rows, M, kv_heads, d_pad] (a copy)."""
    h, rows, pieces, m, _ = table.shape[-5:]
    lead = tuple(range(table.dim() - 5))
    k = len(lead)
    return table.permute(*lead, k + 1, k + 3, k, k + 2, k + 4).reshape(*table.shape[:-5], rows, m, h, pieces * 8)


def kvstar_table_from_reference(repre: torch.Tensor, layout: str = "head") -> torch.Tensor:
    """The reference's [rows, M, kv_heads, d] -> fp16 indexed [kv_heads, rows, d_pad/8, M, 8], columns zero padded to
    16; in memory the heads of a row next to each other (layout "row") or a plane per head ("head")."""
    rows, m, h, d = repre.shape
    d_pad = (d + 15) // 16 * 16
    padded = torch.zeros((rows, m, h, d_pad), dtype=torch.float16, device=repre.device)
    padded[..., :d] = repre
    cells = padded.view(rows, m, h, d_pad // 8, 8)
    if layout == "head":
        return cells.permute(2, 0, 3, 1, 4).contiguous()
    if layout != "row":
        raise ValueError("layout must be 'row' or 'head'")
    return cells.permute(0, 2, 3, 1, 4).contiguous().permute(1, 0, 2, 3, 4)


def kvstar_block_repre(k_layers: LayerPointers, block_ids: torch.Tensor, slots: torch.Tensor, repre: torch.Tensor,
                       block_size: int, kv_heads: int, head_dim: int, num_blocks: int, merge: int,
                       pruned: Optional[torch.Tensor] = None, pruned_sel: Optional[torch.Tensor] = None) -> None:
    """repre: a kvstar_table ([L, kv_heads, rows, d_pad/8, M, 8] fp16); the caches bfloat16 or float16; pruned int32 [kv_heads, d_pruned] (one set of
    channel lists for every layer), [L, kv_heads, d_pruned] (lists per layer) or None.  With pruned_sel (int32 [n]:
    the list each listed block is pruned by) pruned is [n_lists, kv_heads, d_pruned] or [L, n_lists, kv_heads, d_pruned]."""
    key_dtype = _lib.DTYPE_F16 if k_layers.tensors and k_layers.tensors[0].dtype == torch.float16 else _lib.DTYPE_BF16
    if repre.dim() != 6 or repre.dtype != torch.float16 or repre.shape[4] * merge != block_size or \
            repre.shape[1] != kv_heads or repre.shape[5] != 8:
        raise ValueError("repre must be float16 [L, kv_heads, rows, d_pad/8, block_size/merge, 8]")
    head_stride, row_stride = _kvstar_cell_strides(repre[0], "repre")
    if len(k_layers) != repre.shape[0]:
        raise ValueError("one table layer per cache layer")
    if block_ids.numel() != slots.numel():
        raise ValueError("block_ids and slots differ in length")
    d_pruned = head_dim if pruned is None else pruned.shape[-1]
    n_lists = 0
    if pruned_sel is not None:
        if pruned is None or pruned.dim() not in (3, 4) or pruned_sel.numel() != block_ids.numel():
            raise ValueError("pruned_sel needs pruned [n_lists, kv_heads, d_pruned] (or one such set per layer) and one entry per block")
        per_layer = pruned.dim() == 4
        n_lists = pruned.shape[-3]
    else:
        per_layer = pruned is not None and pruned.dim() == 3
    if pruned is not None and (pruned.shape[-2] != kv_heads or (per_layer and pruned.shape[0] != repre.shape[0])):
        raise ValueError("pruned must be [kv_heads, d_pruned] or [layers, kv_heads, d_pruned]")
    _lib.call("ucm_kvstar_block_repre_keys", k_layers.ptr(), key_dtype, repre.shape[0], num_blocks, _dev(block_ids, torch.int32, "block_ids"),
              _dev(slots, torch.int32, "slots"), block_ids.numel(), block_size, kv_heads, head_dim, merge,
              _opt(pruned, torch.int32, "pruned"), pruned.stride(0) if per_layer else 0,
              _opt(pruned_sel, torch.int32, "pruned_sel"), n_lists, d_pruned, repre.shape[3] * 8,
              repre.data_ptr(),
              repre.shape[2], repre.stride(0), head_stride, row_stride, _stream())


def kvstar_workspace(n_tasks: int, kv_heads: int, rows_per_head: int, max_blocks: int, sub_blocks: int, d_pad: int,
                     device, tiles_per_wave: int = 0) -> tuple:
    """Scratch of ucm_kvstar_votes for a call of this shape; rows_per_head = query tokens * (q_heads / kv_heads),
    d_pad = padded channels per representative (the table's d_pad); tiles_per_wave as passed to the votes call."""
    import ctypes as C

    a, b = C.c_int64(0), C.c_int64(0)
    _lib.call("ucm_kvstar_workspace_floats", n_tasks, kv_heads, rows_per_head, max_blocks, sub_blocks, d_pad,
              int(tiles_per_wave), C.addressof(a), C.addressof(b))
    return (torch.empty(max(a.value, 1), dtype=torch.float32, device=device),
            torch.empty(max(b.value, 1), dtype=torch.float32, device=device))


def kvstar_votes(q: torch.Tensor, q_off: torch.Tensor, n_tokens: int, q_heads: int, repre: torch.Tensor,
                 seg_off: torch.Tensor, seg_len: torch.Tensor, max_blocks: int, votes: torch.Tensor, workspace: tuple,
                 d_pruned: Optional[int] = None, pruned: Optional[torch.Tensor] = None,
                 pruned_sel: Optional[torch.Tensor] = None, tiles_per_wave: int = 0) -> None:
    """q fp16 (any shape; task t reads [n_tokens, q_heads, d_orig] from element q_off[t]); repre: one layer of a
    kvstar_table, fp16 [kv_heads, rows, d_pad/8, M, 8] (head planes may be strided: a row slice of a bigger
    table is fine); votes fp32 [>= rows]; pruned int32 [n_lists, kv_heads, d_pruned]."""
    if repre.dim() != 5 or repre.dtype != torch.float16 or not repre.is_cuda or repre.shape[4] != 8:
        raise ValueError("repre must be a float16 device tensor [kv_heads, rows, d_pad/8, M, 8]")
    kv_heads, rows, pieces, m, _ = repre.shape
    d_pad = pieces * 8
    head_stride, row_stride = _kvstar_cell_strides(repre, "repre")
    d_orig = q.shape[-1]
    n_tasks = seg_off.numel()
    if seg_len.numel() != n_tasks or q_off.numel() != n_tasks:
        raise ValueError("q_off / seg_off / seg_len differ in length")
    if pruned is not None:
        if pruned.dim() != 3 or pruned.shape[1] != kv_heads or pruned_sel is None or pruned_sel.numel() != n_tasks:
            raise ValueError("pruned must be [n_lists, kv_heads, d_pruned] with one pruned_sel entry per task")
        d_pruned = pruned.shape[2]
    elif d_pruned is None:
        d_pruned = d_orig
    if votes.numel() < rows:
        raise ValueError("votes shorter than the representative table")
    ws_max, ws_part = workspace
    _lib.call("ucm_kvstar_votes", _dev(q, torch.float16, "q"), q.numel(), _dev(q_off, torch.int64, "q_off"), n_tokens, q_heads,
              d_orig, _opt(pruned, torch.int32, "pruned"), 0 if pruned is None else pruned.shape[0],
              _opt(pruned_sel, torch.int32, "pruned_sel"), repre.data_ptr(), rows, head_stride, row_stride, _dev(seg_off, torch.int32, "seg_off"), _dev(seg_len, torch.int32, "seg_len"), n_tasks, max_blocks, m,
              kv_heads, d_pruned, d_pad, _dev(ws_max, torch.float32, "ws_max"), ws_max.numel(), _dev(ws_part, torch.float32, "ws_part"), ws_part.numel(),
              _dev(votes, torch.float32, "votes"), int(tiles_per_wave), _stream())


def kvstar_votes_tables(q: torch.Tensor, q_off: torch.Tensor, n_tokens: int, q_heads: int, tables, seg_off: torch.Tensor,
                        seg_len: torch.Tensor, max_blocks: int, votes: torch.Tensor, workspace: tuple,
                        d_pruned: Optional[int] = None, pruned: Optional[torch.Tensor] = None,
                        pruned_sel: Optional[torch.Tensor] = None, tiles_per_wave: int = 0):
    """kvstar_votes for tasks that each bring a table of their own: tables[t] fp16 [kv_heads, rows_t, d_pad/8, M, 8]
    (block 0 of task t = its row 0); seg_off only places the votes.  Returns the device pointer arrays, which the
    caller keeps alive until the stream has run the call."""
    n_tasks = len(tables)
    if n_tasks == 0:
        return None
    kv_heads, _, pieces, m, _ = tables[0].shape
    cell = pieces * m * 8
    strides = []
    for t in tables:
        if t.dim() != 5 or t.dtype != torch.float16 or not t.is_cuda or t.shape[0] != kv_heads or t.shape[2:] != tables[0].shape[2:]:
            raise ValueError("every table must be a float16 device tensor [kv_heads, rows, d_pad/8, M, 8] of the same M and d_pad")
        strides.append(_kvstar_cell_strides(t, "table"))
    # one row stride for the call: tables of a single row fit any
    row_strides = {rs for t, (_, rs) in zip(tables, strides) if t.shape[1] > 1}
    if len(row_strides) > 1:
        raise ValueError("the tables of one call must share a row stride (all head planes, or all rows of kv_heads cells)")
    row_stride = row_strides.pop() if row_strides else cell
    d_orig = q.shape[-1]
    if seg_off.numel() != n_tasks or seg_len.numel() != n_tasks or q_off.numel() != n_tasks:
        raise ValueError("q_off / seg_off / seg_len / tables differ in length")
    if pruned is not None:
        if pruned.dim() != 3 or pruned.shape[1] != kv_heads or pruned_sel is None or pruned_sel.numel() != n_tasks:
            raise ValueError("pruned must be [n_lists, kv_heads, d_pruned] with one pruned_sel entry per task")
        d_pruned = pruned.shape[2]
    elif d_pruned is None:
        d_pruned = d_orig
    dev = upload(torch.tensor([[t.data_ptr() for t in tables], [hs for hs, _ in strides]], dtype=torch.int64), tables[0].device)
    ws_max, ws_part = workspace
    _lib.call("ucm_kvstar_votes_tables", _dev(q, torch.float16, "q"), q.numel(), _dev(q_off, torch.int64, "q_off"), n_tokens, q_heads,
              d_orig, _opt(pruned, torch.int32, "pruned"), 0 if pruned is None else pruned.shape[0],
              _opt(pruned_sel, torch.int32, "pruned_sel"), dev[0].data_ptr(), dev[1].data_ptr(),
              row_stride, _dev(seg_off, torch.int32, "seg_off"), _dev(seg_len, torch.int32, "seg_len"), n_tasks, max_blocks, m,
              kv_heads, d_pruned, pieces * 8, _dev(ws_max, torch.float32, "ws_max"), ws_max.numel(), _dev(ws_part, torch.float32, "ws_part"), ws_part.numel(),
              _dev(votes, torch.float32, "votes"), votes.numel(), int(tiles_per_wave), _stream())
    return dev
