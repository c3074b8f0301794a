"""ctypes access to the CPU oracle (``liborc.so``) and, where it was built, to
the reference's own translation units (``_ref/libucm_ref.so``).

TEST INFRASTRUCTURE ONLY.  Importers: the test-suite, ``__graft_entry__.smoke``
and the ``cpu_baseline`` leg of ``bench.py``.  The shipped package never
imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORC_PATH = os.path.join(_HERE, "liborc.so")
_REF_DIR = os.path.join(_HERE, "_ref")
_REF_PATH = os.path.join(_REF_DIR, "libucm_ref.so")

_u32, _i32, _i64, _f32 = C.c_uint32, C.c_int32, C.c_int64, C.c_float
_p = C.c_void_p


def build(with_ref: bool | None = None) -> None:
    """Run the Makefile (liborc.so; the reference TUs when the tree is there)."""
    target = ["all"] if with_ref is None else (["all", "ref"] if with_ref else ["liborc.so"])
    subprocess.check_call(["make", "-C", _HERE, "-s"] + target)


def _load_orc() -> C.CDLL:
    if not os.path.exists(_ORC_PATH):
        build(with_ref=False)
    return C.CDLL(_ORC_PATH)


_orc = _load_orc()


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _sig(lib, name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_orc_vector_mean = _sig(_orc, "orc_vector_mean", None, _p, _p, _u32, _u32)
_orc_k_repre_block = _sig(_orc, "orc_k_repre_block", None, _p, _u32, _u32, _u32, _p)
_orc_block_mean_paged = _sig(_orc, "orc_block_mean_paged", None, _p, _p, _p, _u32, _u32, _u32, _u32, _p, C.c_int)
_orc_block_mean_paged_f16 = _sig(_orc, "orc_block_mean_paged_f16", None, _p, _p, _p, _u32, _u32, _u32, _u32, _p, C.c_int)
_orc_q_head_mean = _sig(_orc, "orc_q_head_mean", None, _p, _u32, _u32, _u32)
_orc_dot16 = _sig(_orc, "orc_dot16", _f32, _p, _p, _u32)
_orc_kq_scores = _sig(_orc, "orc_kq_scores", None, _p, _p, _u32, _u32, _u32, _u32, _p)
_orc_topk_windows = _sig(_orc, "orc_topk_windows", _i32, _p, _u32, _u32, _u32, _u32, _p)
_orc_topk_windows_i32 = _sig(_orc, "orc_topk_windows_i32", _i32, _p, _u32, _u32, _u32, _u32, _p)
_orc_select_topk = _sig(_orc, "orc_select_topk", _i32, _p, _p, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _p, _p)
_orc_select_topk_bs = _sig(_orc, "orc_select_topk_bs", None, _p, _p, _p, _p, _p, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _p, _u32, _p, _p)
_orc_compute_topk_len = _sig(_orc, "orc_compute_topk_len", _i32, _i32)
_orc_esa_retrieve = _sig(_orc, "orc_esa_retrieve", _i32, _p, _u32, _p, _p, _u32, _i32, _p, _p)
_orc_block_table_gather = _sig(_orc, "orc_block_table_gather", _i32, _p, _p, _i32, _i32, _i32, _p)
_orc_get_offset = _sig(_orc, "orc_get_offset", _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, C.c_int, C.c_int)
_orc_kv_move_blocks = _sig(_orc, "orc_kv_move_blocks", None, _p, _u32, C.c_size_t, C.c_size_t, _p, _u32, _p, C.c_int)
_orc_kv_gather_selected = _sig(_orc, "orc_kv_gather_selected", None, _p, _u32, C.c_size_t, C.c_size_t, _p, _p, _u32, _u32, _p, _p, _p)
_orc_delta_plan = _sig(_orc, "orc_delta_plan", _i32, _p, _p, _i32, _p, _i32, _p, _p)
_orc_hash_encode = _sig(_orc, "orc_hash_encode", None, _p, _p, _u32, _u32, _u32, _p)
_orc_hash_encode_f32 = _sig(_orc, "orc_hash_encode_f32", None, _p, _p, _u32, _u32, _u32, _p)
_orc_hash_colsum = _sig(_orc, "orc_hash_colsum", None, _p, _u32, _u32, _u32, _u32, _p)
_orc_hash_scores_sum = _sig(_orc, "orc_hash_scores_sum", None, _p, _u32, _p, _u32, _u32, _u32, _u32, _p)
_orc_hash_majority = _sig(_orc, "orc_hash_majority", None, _p, _u32, _u32, _u32, _u32, _p)
_orc_hash_scores_block = _sig(_orc, "orc_hash_scores_block", None, _p, _p, _u32, _u32, _u32, _p)
_orc_f16_to_f32 = _sig(_orc, "orc_f16_to_f32", _f32, C.c_uint16)
_orc_f32_to_f16 = _sig(_orc, "orc_f32_to_f16", C.c_uint16, _f32)
_orc_kvstar_block_repre = _sig(_orc, "orc_kvstar_block_repre", None, _p, _p, _p, _u32, _u32, _u32, _u32, _u32, _p, _u32,
                               _u32, _p)
_orc_kvstar_block_repre_f16 = _sig(_orc, "orc_kvstar_block_repre_f16", None, _p, _p, _p, _u32, _u32, _u32, _u32, _u32, _p, _u32,
                                   _u32, _p)
_orc_kvstar_retrieve = _sig(_orc, "orc_kvstar_retrieve", _i32, _p, _u32, _u32, _u32, _p, _u32, _u32, _u32, _u32, _u32, _p,
                            _u32, _p, _p)
_orc_f32_to_bf16 = _sig(_orc, "orc_f32_to_bf16", C.c_uint16, _f32)
_orc_prefetch_run = _sig(_orc, "orc_prefetch_run", _i32, _p, _p, _i32, _p, _i32, _p, _p, _p, _i32, _p, _p, _p, _p)
_orc_kvstar_topk = _sig(_orc, "orc_kvstar_topk", _i32, _p, _u32, _u32, _p)


# ---------------------------------------------------------------- bf16 helpers

def bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns (uint16), round-to-nearest-even."""
    u = _c(x, np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (_c(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


# ------------------------------------------------------------------ the oracle

def vector_mean(vectors: np.ndarray) -> np.ndarray:
    v = _c(vectors, np.float32)
    num_k, dim = v.shape
    out = np.empty(dim, np.float32)
    _orc_vector_mean(_ptr(v), _ptr(out), dim, num_k)
    return out


def k_repre_block(k_array: np.ndarray) -> np.ndarray:
    """k_array [kHead, blockSize, headSize] fp32 -> [kHead, headSize]."""
    k = _c(k_array, np.float32)
    h, t, d = k.shape
    out = np.empty((h, d), np.float32)
    _orc_k_repre_block(_ptr(k), h, t, d, _ptr(out))
    return out


def block_mean_paged(k_cache_bits, block_ids, slots, repre, round_bf16=False, keys_f16=False) -> None:
    """k_cache_bits uint16 [num_blocks, T, H, D] (bf16 bit patterns, or fp16 ones with keys_f16: round_bf16 then
    rounds to fp16, the cache's own type); writes repre[slots[i]] in place."""
    kc = _c(k_cache_bits, np.uint16)
    _, t, h, d = kc.shape
    ids, sl = _c(block_ids, np.int32), _c(slots, np.int32)
    assert repre.dtype == np.float32 and repre.flags.c_contiguous
    fn = _orc_block_mean_paged_f16 if keys_f16 else _orc_block_mean_paged
    fn(_ptr(kc), _ptr(ids), _ptr(sl), len(ids), t, h, d, _ptr(repre), int(round_bf16))


def q_head_mean(q: np.ndarray, k_head: int) -> np.ndarray:
    """q [qHead, D] fp32 -> [kHead, D] (computed in place on a copy, like the reference)."""
    w = _c(q, np.float32).copy()
    q_head, d = w.shape
    _orc_q_head_mean(_ptr(w), k_head, q_head, d)
    return w[:k_head].copy()


def dot16(q: np.ndarray, k: np.ndarray) -> np.float32:
    a, b = _c(q, np.float32), _c(k, np.float32)
    return np.float32(_orc_dot16(_ptr(a), _ptr(b), a.size))


def kq_scores(q_mean: np.ndarray, k_repre: np.ndarray) -> np.ndarray:
    """q_mean [kHead, D]; k_repre [n, kHead, numKrepre, D] -> scores [n]."""
    qm, kr = _c(q_mean, np.float32), _c(k_repre, np.float32)
    n, h, r, d = kr.shape
    out = np.empty(n, np.float32)
    _orc_kq_scores(_ptr(qm), _ptr(kr), n, h, r, d, _ptr(out))
    return out


def topk_windows(scores: np.ndarray, k: int, start_w: int = 1, end_w: int = 2) -> np.ndarray:
    if np.issubdtype(np.asarray(scores).dtype, np.integer):
        s = _c(scores, np.int32)
        fn = _orc_topk_windows_i32
    else:
        s = _c(scores, np.float32)
        fn = _orc_topk_windows
    out = np.empty(max(len(s), k) + start_w + end_w, np.int32)
    cnt = fn(_ptr(s), len(s), k, start_w, end_w, _ptr(out))
    return out[:cnt].copy()


def select_topk(q, k_repre, k, start_w=1, end_w=2):
    """q [qHead, D]; k_repre [n, kHead, numKrepre, D] -> (indices, scores)."""
    w = _c(q, np.float32).copy()
    kr = _c(k_repre, np.float32)
    n, h, r, d = kr.shape
    out = np.empty(max(n, k) + start_w + end_w, np.int32)
    scores = np.empty(n, np.float32)
    cnt = _orc_select_topk(_ptr(w), _ptr(kr), n, h, w.shape[0], r, d, k, start_w, end_w, _ptr(out), _ptr(scores))
    return out[:cnt].copy(), scores


def select_topk_bs(q, repre, seg_off, seg_len, topk_len, k_head, num_krepre=1, start_w=1, end_w=2, out_stride=None):
    """q [B, qHead, D]; repre [rows, kHead*numKrepre*D].  Returns (idx [B, stride], count [B], scores [rows])."""
    w = _c(q, np.float32).copy()
    rp = _c(repre, np.float32)
    so, sl, tk = _c(seg_off, np.int32), _c(seg_len, np.int32), _c(topk_len, np.int32)
    b, q_head, d = w.shape
    if out_stride is None:
        out_stride = int(max(sl.max(initial=0), tk.max(initial=0))) + start_w + end_w
    out = np.full((b, out_stride), -1, np.int32)
    cnt = np.zeros(b, np.int32)
    scores = np.zeros(rp.shape[0], np.float32)
    _orc_select_topk_bs(_ptr(w), _ptr(rp), _ptr(so), _ptr(sl), _ptr(tk), b, k_head, q_head, num_krepre, d,
                        start_w, end_w, _ptr(out), out_stride, _ptr(cnt), _ptr(scores))
    return out, cnt, scores


def compute_topk_len(raw_seq_len: int) -> int:
    return int(_orc_compute_topk_len(int(raw_seq_len)))


def esa_retrieve(data: np.ndarray, q: np.ndarray, indexes: np.ndarray, topk: int):
    """One request of the ESA backend: (indices int32[k'], scores f32[k'])."""
    dt, qq, ix = _c(data, np.float32), _c(q, np.float32), _c(indexes, np.int32)
    out_i = np.empty(len(ix) + 1, np.int32)
    out_s = np.empty(len(ix) + 1, np.float32)
    cnt = _orc_esa_retrieve(_ptr(dt), dt.shape[1], _ptr(qq), _ptr(ix), len(ix), topk, _ptr(out_i), _ptr(out_s))
    return out_i[:cnt].copy(), out_s[:cnt].copy()


def block_table_gather(block_table, topk_idx, seq_len: int, block_size: int):
    bt, ti = _c(block_table, np.int32), _c(topk_idx, np.int32)
    out = np.empty(len(ti), np.int32)
    sl = _orc_block_table_gather(_ptr(bt), _ptr(ti), len(ti), seq_len, block_size, _ptr(out))
    return out, int(sl)


def get_offset(block_shape, rank, tp_size, precision, layer_id, is_v, is_mla=False) -> int:
    bs, h, d = block_shape
    return int(_orc_get_offset(bs, h, d, rank, tp_size, precision, layer_id, int(is_v), int(is_mla)))


def _layer_ptrs(layers):
    arr = (C.c_void_p * len(layers))(*[a.ctypes.data for a in layers])
    return arr


def kv_move_blocks(layers, kv_stride, block_bytes, block_ids, staging, to_staging: bool) -> None:
    """layers: list of uint8 arrays (one per layer, K plane at 0, V plane at kv_stride)."""
    ids = _c(block_ids, np.int32)
    _orc_kv_move_blocks(_layer_ptrs(layers), len(layers), kv_stride, block_bytes, _ptr(ids), len(ids),
                        _ptr(staging), int(to_staging))


def kv_gather_selected(layers, kv_stride, block_bytes, phys, count, dst_off, region_k, staging) -> None:
    ph, ct = _c(phys, np.int32), _c(count, np.int32)
    n_layers, n_req, stride = ph.shape
    do, rk = _c(dst_off, np.int64), _c(region_k, np.int32)
    _orc_kv_gather_selected(_layer_ptrs(layers), n_layers, kv_stride, block_bytes, _ptr(ph), _ptr(ct), n_req,
                            stride, _ptr(do), _ptr(rk), _ptr(staging))


def delta_plan(sel, sel_phys, resident):
    """One (layer, request): returns (load_phys [n_slots], slot_of_sel [len(sel)], moved); resident is updated in place."""
    s, sp = _c(sel, np.int32), _c(sel_phys, np.int32)
    assert resident.dtype == np.int32 and resident.flags.c_contiguous
    load = np.empty(len(resident), np.int32)
    slot_of = np.full(max(len(s), 1), -1, np.int32)
    moved = _orc_delta_plan(_ptr(s), _ptr(sp), len(s), _ptr(resident), len(resident), _ptr(load), _ptr(slot_of))
    return load, slot_of[: len(s)], int(moved)


def hash_encode(x_bits: np.ndarray, w: np.ndarray) -> np.ndarray:
    """x_bits uint16 [..., dim] (bf16), w fp32 [dim, bits] -> uint8 [..., bits/8]."""
    xb, ww = _c(x_bits, np.uint16), _c(w, np.float32)
    dim, bits = ww.shape
    n = xb.size // dim
    out = np.empty((n, bits // 8), np.uint8)
    _orc_hash_encode(_ptr(xb), _ptr(ww), n, dim, bits, _ptr(out))
    return out.reshape(xb.shape[:-1] + (bits // 8,))


def hash_encode_f32(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """x fp32 [..., dim], w fp32 [dim, bits] -> uint8 [..., bits/8]."""
    xx, ww = _c(x, np.float32), _c(w, np.float32)
    dim, bits = ww.shape
    n = xx.size // dim
    out = np.empty((n, bits // 8), np.uint8)
    _orc_hash_encode_f32(_ptr(xx), _ptr(ww), n, dim, bits, _ptr(out))
    return out.reshape(xx.shape[:-1] + (bits // 8,))


def hash_colsum(token_codes: np.ndarray) -> np.ndarray:
    """token_codes [n, block_size, kv_heads, nbytes] -> int16 [n, kv_heads, nbytes*8] (#ones - #zeros)."""
    tc = _c(token_codes, np.uint8)
    n, t, h, nb = tc.shape
    out = np.empty((n, h, nb * 8), np.int16)
    _orc_hash_colsum(_ptr(tc), n, t, h, nb, _ptr(out))
    return out


def hash_scores_sum(q_codes: np.ndarray, key_codes: np.ndarray) -> np.ndarray:
    """q_codes [q_heads, nbytes]; key_codes [n, kv_heads, block_size, nbytes] -> int32 [n]."""
    qc, kc = _c(q_codes, np.uint8), _c(key_codes, np.uint8)
    n, h, t, nb = kc.shape
    out = np.empty(n, np.int32)
    _orc_hash_scores_sum(_ptr(qc), qc.shape[0], _ptr(kc), n, h, t, nb, _ptr(out))
    return out


def hash_majority(token_codes: np.ndarray) -> np.ndarray:
    """token_codes [n, block_size, kv_heads, nbytes] -> [n, kv_heads, nbytes]."""
    tc = _c(token_codes, np.uint8)
    n, t, h, nb = tc.shape
    out = np.empty((n, h, nb), np.uint8)
    _orc_hash_majority(_ptr(tc), n, t, h, nb, _ptr(out))
    return out


def hash_scores_block(q_codes: np.ndarray, block_codes: np.ndarray) -> np.ndarray:
    qc, bc = _c(q_codes, np.uint8), _c(block_codes, np.uint8)
    n, h, nb = bc.shape
    out = np.empty(n, np.int32)
    _orc_hash_scores_block(_ptr(qc), _ptr(bc), n, h, nb, _ptr(out))
    return out


# ------------------------------------------- the reference's own compiled TUs

def f16_to_f32(h: int) -> float:
    return float(_orc_f16_to_f32(int(h)))


def f32_to_f16(f: float) -> int:
    return int(_orc_f32_to_f16(float(f)))


def kvstar_block_repre(cache_bits: np.ndarray, block_ids, slots, merge: int, repre: np.ndarray, pruned=None,
                       keys_f16: bool = False) -> None:
    """cache_bits uint16 [num_blocks, block_size, kv_heads, head_dim] (bf16, or fp16 with keys_f16); repre uint16 (fp16)
    [rows, M, kv_heads, d_pad], rows ``slots`` are overwritten; pruned int32 [kv_heads, d_pruned] or None."""
    cb = _c(cache_bits, np.uint16)
    _, bs, h, d = cb.shape
    ids, sl = _c(block_ids, np.int32), _c(slots, np.int32)
    assert repre.dtype == np.uint16 and repre.flags.c_contiguous and repre.shape[1] == bs // merge and repre.shape[2] == h
    pr = None if pruned is None else _c(pruned, np.int32)
    dp = d if pr is None else pr.shape[1]
    fn = _orc_kvstar_block_repre_f16 if keys_f16 else _orc_kvstar_block_repre
    fn(_ptr(cb), _ptr(ids), _ptr(sl), len(ids), bs, h, d, merge, None if pr is None else _ptr(pr), dp, repre.shape[3], _ptr(repre))


def kvstar_retrieve(q_bits: np.ndarray, repre: np.ndarray, topk: int, pruned=None, d_pruned: int | None = None):
    """q_bits uint16 (fp16) [tokens, q_heads, d_orig]; repre uint16 (fp16) [n_blocks, M, kv_heads, d_pad]
    -> (top-k block indices by descending score, final scores fp32 [n_blocks])."""
    qb, rp = _c(q_bits, np.uint16), _c(repre, np.uint16)
    x, hq, d = qb.shape
    n, m, h, d_pad = rp.shape
    pr = None if pruned is None else _c(pruned, np.int32)
    dp = (d_pad if d_pruned is None else d_pruned) if pr is None else pr.shape[1]
    final = np.zeros(n, np.float32)
    idx = np.zeros(max(min(topk, n), 1), np.int32)
    k = _orc_kvstar_retrieve(_ptr(qb), x, hq, d, _ptr(rp), n, m, h, dp, d_pad, None if pr is None else _ptr(pr), topk,
                             _ptr(final), _ptr(idx))
    return idx[:k].copy(), final


def kvstar_topk(final_scores: np.ndarray, topk: int) -> np.ndarray:
    """The heap top-k of KVStar::Execute on given per-block scores: indices, descending by (score, index)."""
    f = _c(final_scores, np.float32)
    out = np.zeros(max(min(int(topk), len(f)), 1), np.int32)
    k = _orc_kvstar_topk(_ptr(f), len(f), int(topk), _ptr(out))
    return out[:k].copy()


def prefetch_run(map_block, map_idx, topk, free_block, free_len: int, success_cap: int):
    """One (request, layer) of the GSA prefetch engine.  map_idx (int32 array) is updated in place.  Returns
    (success_blocks [success_cap], success_len, load_blocks, miss_idxs, new_free_list)."""
    mb = _c(map_block, np.int32)
    assert map_idx.dtype == np.int32 and map_idx.flags.c_contiguous and len(map_idx) == len(mb)
    tk = _c(topk, np.int32)
    fb = np.zeros(max(len(mb), len(free_block), 1), np.int32)
    fb[: len(free_block)] = free_block
    fl, sl, nm = C.c_int32(int(free_len)), C.c_int32(0), C.c_int32(0)
    succ = np.zeros(max(success_cap, 1), np.int32)
    loads = np.zeros(max(len(tk), 1), np.int32)
    miss = np.zeros(max(len(tk), 1), np.int32)
    n_load = _orc_prefetch_run(_ptr(mb), _ptr(map_idx), len(mb), _ptr(tk), len(tk), _ptr(fb), C.byref(fl), _ptr(succ),
                               success_cap, C.byref(sl), _ptr(loads), _ptr(miss), C.byref(nm))
    if n_load < 0:
        raise ValueError("free list names a block that is not in the map")
    return succ[:success_cap], int(sl.value), loads[:n_load].copy(), miss[: nm.value].copy(), fb[: fl.value].copy()


def f32_to_bf16(x: float) -> int:
    return int(_orc_f32_to_bf16(float(x)))


class _Ref:
    """Lazy handle on oracle/_ref (present only where the reference tree was)."""

    def __init__(self):
        self._lib = None

    @property
    def available(self) -> bool:
        return os.path.exists(_REF_PATH)

    @property
    def lib(self) -> C.CDLL:
        if self._lib is None:
            lib = C.CDLL(_REF_PATH)
            _sig(lib, "ref_simd_name", C.c_char_p)
            _sig(lib, "ref_vector_dot", _f32, _p, _p, _u32)
            _sig(lib, "ref_vector_mean", None, _p, _p, _u32, _u32)
            _sig(lib, "ref_k_repre_block", None, _p, _u32, _u32, _u32, _p)
            _sig(lib, "ref_q_head_mean", None, _p, _u32, _u32, _u32)
            _sig(lib, "ref_kq_scores", None, _p, _p, _u32, _u32, _u32, _u32, _p)
            _sig(lib, "ref_select_topk", None, _p, _p, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _p)
            _sig(lib, "ref_select_topk_bs", None, _p, _p, _p, _p, _p, _u32, _u32, _u32, _u32, _u32, _p, _u32)
            self._lib = lib
        return self._lib

    def simd_name(self) -> str:
        return self.lib.ref_simd_name().decode()

    def vector_dot(self, q, k) -> np.float32:
        a, b = _c(q, np.float32), _c(k, np.float32)
        return np.float32(self.lib.ref_vector_dot(_ptr(a), _ptr(b), a.size))

    def vector_mean(self, vectors) -> np.ndarray:
        v = _c(vectors, np.float32)
        out = np.empty(v.shape[1], np.float32)
        self.lib.ref_vector_mean(_ptr(v), _ptr(out), v.shape[1], v.shape[0])
        return out

    def k_repre_block(self, k_array) -> np.ndarray:
        k = _c(k_array, np.float32)
        h, t, d = k.shape
        out = np.empty((h, d), np.float32)
        self.lib.ref_k_repre_block(_ptr(k), h, t, d, _ptr(out))
        return out

    def q_head_mean(self, q, k_head) -> np.ndarray:
        w = _c(q, np.float32).copy()
        self.lib.ref_q_head_mean(_ptr(w), k_head, w.shape[0], w.shape[1])
        return w[:k_head].copy()

    def kq_scores(self, q_mean, k_repre) -> np.ndarray:
        qm, kr = _c(q_mean, np.float32), _c(k_repre, np.float32)
        n, h, r, d = kr.shape
        out = np.empty(n, np.float32)
        self.lib.ref_kq_scores(_ptr(qm), _ptr(kr), n, h, r, d, _ptr(out))
        return out

    def select_topk(self, q, k_repre, k, start_w=1, end_w=2) -> np.ndarray:
        w = _c(q, np.float32).copy()
        kr = _c(k_repre, np.float32)
        n, h, r, d = kr.shape
        sentinel = -7
        out = np.full(max(n, k) + start_w + end_w + 1, sentinel, np.int32)
        self.lib.ref_select_topk(_ptr(w), _ptr(kr), n, h, w.shape[0], r, d, k, start_w, end_w, _ptr(out))
        identity = (start_w + end_w >= n) or (k >= n) or (k == 0)
        return out[: (n if identity else k)].copy()

    def select_topk_bs(self, q, repre, seg_off, seg_len, topk_len, k_head, num_krepre=1, out_stride=None):
        w = _c(q, np.float32).copy()
        rp = _c(repre, np.float32)
        so, sl, tk = _c(seg_off, np.int32), _c(seg_len, np.int32), _c(topk_len, np.int32)
        b, q_head, d = w.shape
        if out_stride is None:
            out_stride = int(max(sl.max(initial=0), tk.max(initial=0))) + 4
        out = np.full((b, out_stride), -1, np.int32)
        self.lib.ref_select_topk_bs(_ptr(w), _ptr(rp), _ptr(so), _ptr(sl), _ptr(tk), b, k_head, q_head,
                                    num_krepre, d, _ptr(out), out_stride)
        return out

    def gsa_prefetch_module(self):
        """The reference's GSA prefetch engine built as a python extension (or None)."""
        if not os.path.isdir(_REF_DIR) or not any(f.startswith("gsa_prefetch") for f in os.listdir(_REF_DIR)):
            return None
        import torch  # noqa: F401  (the extension links against libtorch)

        if _REF_DIR not in sys.path:
            sys.path.insert(0, _REF_DIR)
        import gsa_prefetch  # noqa: E402  (compiled from the reference's C++)

        return gsa_prefetch

    def retrieval_backend_module(self):
        """The reference's ESA backend built as a python extension (or None)."""
        if not os.path.isdir(_REF_DIR) or not any(f.startswith("retrieval_backend") for f in os.listdir(_REF_DIR)):
            return None
        if _REF_DIR not in sys.path:
            sys.path.insert(0, _REF_DIR)
        import retrieval_backend  # noqa: E402  (compiled from the reference's C++)

        return retrieval_backend


ref = _Ref()
