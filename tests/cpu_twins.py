"""One scripted pass over the dense retrieval path - representatives, scores, selection with block-table lookup,
delta plan, gathers and the block moves - written once against the C ABI's prototypes and run either through
libucm_hip.so on device buffers or through the oracle's `_cpu` twins (oracle/ucm_cpu_abi.c) on host buffers.
The argument lists of the two runs are identical except for where the pointers point."""
import contextlib
import ctypes as C
import os

import numpy as np

import oracle
import synth

TWINS = ["ucm_block_mean", "ucm_score_blocks", "ucm_topk_windows", "ucm_score_select", "ucm_kv_gather_blocks", "ucm_kv_scatter_blocks",
         "ucm_kv_gather_blocks_tp", "ucm_kv_scatter_blocks_tp", "ucm_kv_load_planned_tp",
         "ucm_kv_gather_selected", "ucm_delta_plan", "ucm_hash_encode_blocks", "ucm_hash_encode_queries",
         "ucm_hash_score_blocks", "ucm_esa_retrieve", "ucm_esa_retrieve_rows", "ucm_delta_plan_rows", "ucm_copy_batch",
         "ucm_kv_load_planned", "ucm_kvstar_topk", "ucm_kvstar_order", "ucm_prefetch_plan", "ucm_kvstar_block_repre",
         "ucm_kvstar_votes", "ucm_kvstar_votes_tables", "ucm_kvstar_park_queries", "ucm_park_rows", "ucm_kvstar_block_repre_keys",
         "ucm_hash_encode_blocks_f16", "ucm_hash_encode_queries_f16"]


@contextlib.contextmanager
def reseeded(offset: int):
    """Every input of the scripted passes drawn from other seeds (the shapes, the ids that are out of range on purpose
    and the order of the calls stay as they are): synth's generators take seed + offset while the block runs."""
    names = ("normal_f32", "normal_bf16_bits", "normal_bf16_as_f32", "ints", "permutation")
    kept = {n: getattr(synth, n) for n in names}
    try:
        for n, f in kept.items():
            setattr(synth, n, (lambda f: lambda seed, *a, **k: f(seed + offset, *a, **k))(f))
        yield
    finally:
        for n, f in kept.items():
            setattr(synth, n, f)


def twin_caller(signatures):
    """call(name, *args) for the host twins, bound with the argument types the device library's binding uses."""
    lib = C.CDLL(os.path.join(os.path.dirname(oracle.__file__), "liborc.so"))
    for name in TWINS:
        fn = getattr(lib, name + "_cpu")
        fn.argtypes, fn.restype = signatures[name], C.c_int

    def call(name, *args):
        rc = getattr(lib, name + "_cpu")(*args)
        if rc != 0:
            raise RuntimeError(f"{name}_cpu returned {rc}")
    return call


class HostSide:
    def up(self, a):
        return np.ascontiguousarray(a).copy()

    def ptr(self, a):
        return a.ctypes.data

    def pointers(self, arrays):
        self._keep = getattr(self, "_keep", []) + [np.array([a.ctypes.data for a in arrays], np.uint64)]
        return self._keep[-1].ctypes.data

    def down(self, a):
        return a

    def sync(self):
        pass


class DeviceSide:
    def __init__(self, ops, dev):
        import torch

        self.torch, self.ops, self.dev = torch, ops, dev

    def up(self, a):
        a = np.ascontiguousarray(a)
        view = a.view(np.int16) if a.dtype == np.uint16 else a      # torch has no uint16 arithmetic type to hold bf16 bits
        t = self.torch.from_numpy(view.copy()).to(self.dev)
        if a.dtype == np.uint16:
            # (the tensor itself is kept, not its address: a freed tensor's address comes back with another type behind it)
            self._u16 = getattr(self, "_u16", {})
            self._u16[id(t)] = t
        return t

    def ptr(self, t):
        return t.data_ptr()

    def pointers(self, tensors):
        self._keep = getattr(self, "_keep", []) + [self.ops.LayerPointers(tensors)]
        return self._keep[-1].ptr()

    def down(self, t):
        a = t.cpu().numpy()
        return a.view(np.uint16) if getattr(self, "_u16", {}).get(id(t)) is t else a

    def sync(self):
        self.torch.cuda.synchronize()


L, NB, BS, HKV, D, G = 2, 12, 16, 2, 64, 4
HQ, ROW = HKV * G, HKV * D
BLOCK_BYTES = BS * HKV * D * 2
KV_STRIDE = NB * BLOCK_BYTES
LENS = np.array([4, 0, 6], np.int32)
OFF = np.array([0, 4, 4], np.int32)
ROWS = 10


def inputs():
    caches = [synth.normal_bf16_bits(7000 + l, (2, NB, BS, HKV, D)) for l in range(L)]
    ids = synth.permutation(7010, NB)[:ROWS].astype(np.int32)
    ids_bad = np.concatenate([ids, [-1, NB]]).astype(np.int32)        # two ids the call must skip
    slots = np.concatenate([np.arange(ROWS), [3, 4]]).astype(np.int32)
    q32 = synth.normal_f32(7020, (L, 5, HQ, D))
    q16 = oracle.bf16_bits(synth.normal_f32(7021, (L, 5, HQ, D)))
    q_rows = np.array([4, 1, 2], np.int32)
    topk = np.array([3, 1, 4], np.int32)
    tables = np.stack([synth.permutation(7030 + r, NB)[:8] for r in range(3)]).astype(np.int32)
    seq_lens = np.array([4 * BS - 5, 0, 6 * BS], np.int32)
    return dict(caches=caches, ids=ids_bad, slots=slots, q32=q32, q16=q16, q_rows=q_rows, topk=topk, tables=tables,
                seq_lens=seq_lens)


def run(call, side):
    """Every output of the pass, as numpy arrays."""
    x = inputs()
    out = {}
    caches = [side.up(c) for c in x["caches"]]
    k_planes = side.pointers(caches)                                 # a layer's K plane comes first
    ids, slots = side.up(x["ids"]), side.up(x["slots"])
    n = len(x["ids"])
    # 1. representatives in the three modes
    tabs = {}
    for mode, dtype in ((0, np.float32), (1, np.float32), (2, np.uint16), (4, np.float32)):      # 4: of the absolute values
        t = side.up(np.full((L, ROWS, ROW), 7, dtype))
        call("ucm_block_mean", k_planes, L, NB, side.ptr(ids), side.ptr(slots), n, BS, HKV, D, side.ptr(t), ROWS, ROWS * ROW,
             mode, None)
        tabs[mode] = t
        out[f"repre{mode}"] = t
    # 2. scores: fp32 queries on the fp32 table; bf16 queries picked by q_rows on the bf16 table, scaled
    seg_off, seg_len = side.up(OFF), side.up(LENS)
    s32 = side.up(np.full((L, ROWS), -3, np.float32))
    q32 = side.up(x["q32"])
    call("ucm_score_blocks", side.ptr(q32), 0, 5 * HQ * D, None, HQ, side.ptr(tabs[0]), 0, ROWS * ROW, ROWS, 1, side.ptr(seg_off),
         side.ptr(seg_len), 3, 6, 10, L, HKV, D, side.ptr(s32), ROWS, 1.0, 0, None)
    s16 = side.up(np.full((L, ROWS), -3, np.float32))
    q16, q_rows = side.up(x["q16"]), side.up(x["q_rows"])
    call("ucm_score_blocks", side.ptr(q16), 1, 5 * HQ * D, side.ptr(q_rows), HQ, side.ptr(tabs[2]), 1, ROWS * ROW, ROWS, 1,
         side.ptr(seg_off), side.ptr(seg_len), 3, 6, 0, L, HKV, D, side.ptr(s16), ROWS, 0.5, 0, None)
    out["scores32"], out["scores16"] = s32, s16
    # 3. selection with the block-table lookup and the sparse lengths
    topk, tables, seq_lens = side.up(x["topk"]), side.up(x["tables"]), side.up(x["seq_lens"])
    idx, phys = side.up(np.full((L, 3, 6), -1, np.int32)), side.up(np.full((L, 3, 6), -1, np.int32))
    cnt, sparse = side.up(np.full((L, 3), -1, np.int32)), side.up(np.full((L, 3), -1, np.int32))
    call("ucm_topk_windows", side.ptr(s16), ROWS, ROWS, side.ptr(seg_off), side.ptr(seg_len), side.ptr(topk), 3, 6, L, 1, 1,
         side.ptr(idx), 6, side.ptr(cnt), side.ptr(tables), 8, side.ptr(phys), side.ptr(seq_lens), BS, side.ptr(sparse), None)
    out.update(idx=idx, phys=phys, cnt=cnt, sparse=sparse)
    # 3b. the same scores and selection as one launch: every output must equal the two calls'
    import ctypes as C

    from ucm_amd import _lib

    # (its output tables are kept for four requests, of which this batch uses three: layer strides of their own)
    f_scores = side.up(np.full((L, ROWS), -3, np.float32))
    f_idx, f_phys = side.up(np.full((L, 4, 6), -1, np.int32)), side.up(np.full((L, 4, 6), -1, np.int32))
    f_cnt, f_sparse = side.up(np.full((L, 4), -1, np.int32)), side.up(np.full((L, 4), -1, np.int32))
    tickets = side.up(np.zeros((L, 4), np.int32))
    args = _lib.ScoreSelectArgs(
        q=side.ptr(q16), q_dtype=1, q_heads=HQ, q_layer_stride=5 * HQ * D, q_rows=side.ptr(q_rows), repre=side.ptr(tabs[2]),
        repre_dtype=1, repre_layer_stride=ROWS * ROW, repre_rows=ROWS, seg_off=side.ptr(seg_off), seg_len=side.ptr(seg_len),
        topk_len=side.ptr(topk), n_req=3, max_seg_len=6, first_layer=0, kv_heads=HKV, head_dim=D, scores=side.ptr(f_scores),
        scores_layer_stride=ROWS, start_w=1, end_w=1, idx_out=side.ptr(f_idx), count_out=side.ptr(f_cnt), out_stride=6,
        bt_stride=8, block_tables=side.ptr(tables), phys_out=side.ptr(f_phys), seq_lens=side.ptr(seq_lens),
        sparse_seq_lens=side.ptr(f_sparse), block_size=BS, tickets=side.ptr(tickets), idx_layer_stride=4 * 6,
        count_layer_stride=4)
    args.n_layers, args.scale = L, 0.5
    call("ucm_score_select", C.addressof(args), None)
    out.update(f_scores=f_scores, f_idx=f_idx, f_phys=f_phys, f_cnt=f_cnt, f_sparse=f_sparse, tickets=tickets)
    # 4. delta plan, twice: empty slots first, then the other scores' selection against what the first left
    resident = side.up(np.full((L, 3, 4), -1, np.int32))
    load, slot_of, miss = (side.up(np.full(s, -9, np.int32)) for s in ((L, 3, 4), (L, 3, 6), (L, 3)))
    call("ucm_delta_plan", side.ptr(idx), side.ptr(phys), side.ptr(cnt), 3, L, 6, side.ptr(resident), 4, side.ptr(load),
         side.ptr(slot_of), side.ptr(miss), None)
    side.sync()
    out.update(resident1=side.up(side.down(resident)), load1=side.up(side.down(load)), miss1=side.up(side.down(miss)))
    idx2, phys2, cnt2 = (side.up(np.full(s, -1, np.int32)) for s in ((L, 3, 6), (L, 3, 6), (L, 3)))
    call("ucm_topk_windows", side.ptr(s32), ROWS, ROWS, side.ptr(seg_off), side.ptr(seg_len), side.ptr(topk), 3, 6, L, 1, 1,
         side.ptr(idx2), 6, side.ptr(cnt2), side.ptr(tables), 8, side.ptr(phys2), None, BS, None, None)
    call("ucm_delta_plan", side.ptr(idx2), side.ptr(phys2), side.ptr(cnt2), 3, L, 6, side.ptr(resident), 4, side.ptr(load),
         side.ptr(slot_of), side.ptr(miss), None)
    out.update(idx2=idx2, resident2=resident, load2=load, slot_of2=slot_of, miss2=miss)
    # 5. gather of the first selection, and of the second plan's loads (its -1 entries are skipped)
    layers = side.pointers(caches)
    dst_off, region_k = side.up(np.array([0, 16, 16], np.int64)), side.up(np.array([4, 0, 4], np.int32))
    for name, p, c in (("gathered", phys, cnt), ("loaded", load, side.up(np.full((L, 3), 4, np.int32)))):
        staging = side.up(np.zeros((2 * 2 * L * 4, BLOCK_BYTES), np.uint8))
        stride = 6 if name == "gathered" else 4
        call("ucm_kv_gather_selected", layers, L, KV_STRIDE, BLOCK_BYTES, NB, side.ptr(p), side.ptr(c), 3, stride,
             side.ptr(dst_off), side.ptr(region_k), 4, side.ptr(staging), 2 * 2 * L * 4, None)
        out[name] = staging
    # 6. block moves: out of the cache, and back into an empty one
    move = side.up(np.array([5, -2, 0, 11], np.int32))
    staging = side.up(np.zeros((4, L, 2, BLOCK_BYTES), np.uint8))
    call("ucm_kv_gather_blocks", layers, L, KV_STRIDE, BLOCK_BYTES, NB, side.ptr(move), 4, side.ptr(staging), None)
    empty = [side.up(np.zeros((2, NB, BS, HKV, D), np.uint16)) for _ in range(L)]
    call("ucm_kv_scatter_blocks", side.pointers(empty), L, KV_STRIDE, BLOCK_BYTES, NB, side.ptr(move), 4, side.ptr(staging), None)
    out["moved"] = staging
    for l in range(L):
        out[f"restored{l}"] = empty[l]
    # 7. the same moves for rank 1 of 3 ranks that share the stored block: only that rank's slices are touched
    wide = side.up(np.full((4, L, 3, 2, BLOCK_BYTES), 0xEE, np.uint8))
    call("ucm_kv_gather_blocks_tp", layers, L, KV_STRIDE, BLOCK_BYTES, NB, side.ptr(move), 4, side.ptr(wide), 1, 3, None)
    empty_tp = [side.up(np.zeros((2, NB, BS, HKV, D), np.uint16)) for _ in range(L)]
    call("ucm_kv_scatter_blocks_tp", side.pointers(empty_tp), L, KV_STRIDE, BLOCK_BYTES, NB, side.ptr(move), 4, side.ptr(wide), 1, 3,
         None)
    out["moved_tp"] = wide
    for l in range(L):
        out[f"restored_tp{l}"] = empty_tp[l]
    side.sync()
    return {k: np.array(side.down(v)) for k, v in out.items()}, x


def run_bounds(call, side):
    """Segment descriptors that point outside the tables: the call declares fewer rows than the buffers hold (the
    table starts PAD rows into its buffer), so a descriptor that were followed would land in memory the test owns and
    show up in the padding.  Request 0 is in range, request 1 starts below row 0, request 2 ends past the last row."""
    import ctypes as C

    from ucm_amd import _lib

    PAD = 4
    x = inputs()
    repre_h = synth.normal_f32(7050, (L, ROWS + 2 * PAD, ROW))
    repre = side.up(repre_h)
    scores = side.up(np.full((L, ROWS + 2 * PAD), -3, np.float32))
    q32 = side.up(x["q32"])
    seg_off, seg_len = side.up(np.array([1, -2, 7], np.int32)), side.up(np.array([4, 3, 5], np.int32))
    topk = side.up(np.array([2, 2, 2], np.int32))
    stride_t, stride_s = (ROWS + 2 * PAD) * ROW, ROWS + 2 * PAD
    call("ucm_score_blocks", side.ptr(q32), 0, 5 * HQ * D, None, HQ, side.ptr(repre) + PAD * ROW * 4, 0, stride_t, ROWS, 1,
         side.ptr(seg_off), side.ptr(seg_len), 3, 6, 0, L, HKV, D, side.ptr(scores) + PAD * 4, stride_s, 1.0, 0, None)
    idx, cnt = side.up(np.full((L, 3, 6), -1, np.int32)), side.up(np.full((L, 3), -1, np.int32))
    call("ucm_topk_windows", side.ptr(scores) + PAD * 4, stride_s, ROWS, side.ptr(seg_off), side.ptr(seg_len), side.ptr(topk),
         3, 6, L, 0, 0, side.ptr(idx), 6, side.ptr(cnt), None, 0, None, None, BS, None, None)
    f_scores = side.up(np.full((L, ROWS + 2 * PAD), -3, np.float32))
    f_idx, f_cnt = side.up(np.full((L, 3, 6), -1, np.int32)), side.up(np.full((L, 3), -1, np.int32))
    tickets = side.up(np.zeros((L, 3), np.int32))
    args = _lib.ScoreSelectArgs(
        q=side.ptr(q32), q_dtype=0, q_heads=HQ, q_layer_stride=5 * HQ * D, repre=side.ptr(repre) + PAD * ROW * 4, repre_dtype=0,
        repre_layer_stride=stride_t, repre_rows=ROWS, seg_off=side.ptr(seg_off), seg_len=side.ptr(seg_len),
        topk_len=side.ptr(topk), n_req=3, max_seg_len=6, first_layer=0, kv_heads=HKV, head_dim=D,
        scores=side.ptr(f_scores) + PAD * 4, scores_layer_stride=stride_s, start_w=0, end_w=0, idx_out=side.ptr(f_idx),
        count_out=side.ptr(f_cnt), out_stride=6, tickets=side.ptr(tickets))
    args.n_layers = L
    call("ucm_score_select", C.addressof(args), None)
    side.sync()
    out = dict(scores=scores, idx=idx, cnt=cnt, f_scores=f_scores, f_idx=f_idx, f_cnt=f_cnt, tickets=tickets)
    return {k: np.array(side.down(v)) for k, v in out.items()}, dict(repre=repre_h, q32=x["q32"], pad=PAD)


HL, HNB, HBS, HHKV, HHQ, HD = 2, 7, 16, 2, 8, 128
H_LENS = np.array([3, 0, 2], np.int32)
H_OFF = np.array([0, 3, 3], np.int32)
H_ROWS = 6


def hash_inputs():
    keys = [synth.normal_bf16_bits(7100 + l, (HNB, HBS, HHKV, HD)) for l in range(HL)]
    w = oracle.bf16_bits(synth.normal_f32(7110, (HD, 128)) * np.float32(2.0))
    q = synth.normal_bf16_bits(7111, (HL, 4, HHQ, HD))
    ids = np.array([4, 0, 6, -3, 2, 1, 5, HNB], np.int32)              # two ids the call must skip
    slots = np.array([0, 1, 2, 3, 3, 4, 5, 5], np.int32)
    # a float16 model: keys, queries (one head per kv head) and weights in float16, subnormal components among them
    rng = np.random.default_rng(7120)
    keys16 = [(rng.standard_normal((HNB, HBS, HHKV, HD)) * rng.choice([3e-6, 0.02, 1.0, 200.0], size=(HNB, HBS, HHKV, 1)))
              .astype(np.float16) for _ in range(HL)]
    w16 = (rng.standard_normal((HD, 128)) * 2.0).astype(np.float16)
    q16 = (rng.standard_normal((HL, 4, HHKV, HD)) * rng.choice([1e-5, 1.0], size=(HL, 4, HHKV, 1))).astype(np.float16)
    return dict(keys=keys, w=w, q=q, ids=ids, slots=slots, q_rows=np.array([3, 0, 1], np.int32), keys16=keys16, w16=w16, q16=q16)


def run_hash(call, side):
    """The hash-code path: block codes and summaries, query codes, both scores."""
    x = hash_inputs()
    keys = [side.up(k) for k in x["keys"]]
    w, q = side.up(x["w"]), side.up(x["q"])
    ids, slots, q_rows = side.up(x["ids"]), side.up(x["slots"]), side.up(x["q_rows"])
    tcodes = side.up(np.full((HL, H_ROWS, HBS, HHKV, 16), 0xEE, np.uint8))
    colsum = side.up(np.full((HL, H_ROWS, HHKV, 128), 77, np.int16))
    bcodes = side.up(np.full((HL, H_ROWS, HHKV, 16), 0xEE, np.uint8))
    call("ucm_hash_encode_blocks", side.pointers(keys), HL, HNB, side.ptr(ids), side.ptr(slots), len(x["ids"]), HBS, HHKV, HD,
         side.ptr(w), 128, H_ROWS, side.ptr(tcodes), H_ROWS * HBS * HHKV * 16, side.ptr(colsum), H_ROWS * HHKV * 128,
         side.ptr(bcodes), H_ROWS * HHKV * 16, 0, None)
    q_codes = side.up(np.full((HL, 3, HHQ, 16), 0xEE, np.uint8))
    q_sum = side.up(np.full((HL, 3, 128), 77, np.int16))
    qbar = side.up(np.full((HL, 3, HHKV, 16), 0xEE, np.uint8))
    call("ucm_hash_encode_queries", side.ptr(q), 4 * HHQ * HD, side.ptr(q_rows), 3, HL, HHQ, HHKV, HD, side.ptr(w), 128,
         side.ptr(q_codes), side.ptr(q_sum), side.ptr(qbar), None)
    seg_off, seg_len = side.up(H_OFF), side.up(H_LENS)
    out = dict(token_codes=tcodes, colsum=colsum, block_codes=bcodes, q_codes=q_codes, q_sum=q_sum, qbar=qbar)
    for name, mode, fp16 in (("score_sum", 0, 0), ("score_sum_fp16", 0, 1), ("score_code", 1, 0)):
        sc = side.up(np.full((HL, H_ROWS), -3, np.float32))
        call("ucm_hash_score_blocks", mode, side.ptr(q_sum), side.ptr(qbar), side.ptr(colsum), H_ROWS * HHKV * 128,
             side.ptr(bcodes), H_ROWS * HHKV * 16, H_ROWS, side.ptr(seg_off), side.ptr(seg_len), 3, 5, HL, HHKV, 128, side.ptr(sc),
             H_ROWS, fp16, None)
        out[name] = sc
    # descriptors outside the summary tables: the first request starts below row 0, the third ends past the last row the
    # call names (one row fewer than the tables hold, so a request that were followed would stay inside owned memory)
    bad_off, bad_len = side.up(np.array([-1, 3, 3], np.int32)), side.up(np.array([2, 0, 3], np.int32))
    for name, mode in (("score_sum_bad", 0), ("score_code_bad", 1)):
        sc = side.up(np.full((HL, H_ROWS), -3, np.float32))
        call("ucm_hash_score_blocks", mode, side.ptr(q_sum) , side.ptr(qbar), side.ptr(colsum), H_ROWS * HHKV * 128,
             side.ptr(bcodes), H_ROWS * HHKV * 16, H_ROWS - 1, side.ptr(bad_off), side.ptr(bad_len), 3, 5, HL, HHKV, 128,
             side.ptr(sc), H_ROWS, 0, None)
        out[name] = sc
    # the float16 entry points on the same lists
    keys16 = [side.up(k.view(np.uint16)) for k in x["keys16"]]
    w16, q16 = side.up(x["w16"].view(np.uint16)), side.up(x["q16"].view(np.uint16))
    t16 = side.up(np.full((HL, H_ROWS, HBS, HHKV, 16), 0xEE, np.uint8))
    c16 = side.up(np.full((HL, H_ROWS, HHKV, 128), 77, np.int16))
    b16 = side.up(np.full((HL, H_ROWS, HHKV, 16), 0xEE, np.uint8))
    call("ucm_hash_encode_blocks_f16", side.pointers(keys16), HL, HNB, side.ptr(ids), side.ptr(slots), len(x["ids"]), HBS, HHKV, HD,
         side.ptr(w16), 128, H_ROWS, side.ptr(t16), H_ROWS * HBS * HHKV * 16, side.ptr(c16), H_ROWS * HHKV * 128,
         side.ptr(b16), H_ROWS * HHKV * 16, 0, None)
    qc16 = side.up(np.full((HL, 3, HHKV, 16), 0xEE, np.uint8))
    qs16 = side.up(np.full((HL, 3, 128), 77, np.int16))
    qb16 = side.up(np.full((HL, 3, HHKV, 16), 0xEE, np.uint8))
    call("ucm_hash_encode_queries_f16", side.ptr(q16), 4 * HHKV * HD, side.ptr(q_rows), 3, HL, HHKV, HHKV, HD, side.ptr(w16), 128,
         side.ptr(qc16), side.ptr(qs16), side.ptr(qb16), None)
    # the same queries as HHKV heads around one kv head: the mean codes of a grouped float16 model
    qcg = side.up(np.full((HL, 3, HHKV, 16), 0xEE, np.uint8))
    qsg = side.up(np.full((HL, 3, 128), 77, np.int16))
    qbg = side.up(np.full((HL, 3, 1, 16), 0xEE, np.uint8))
    call("ucm_hash_encode_queries_f16", side.ptr(q16), 4 * HHKV * HD, side.ptr(q_rows), 3, HL, HHKV, 1, HD, side.ptr(w16), 128,
         side.ptr(qcg), side.ptr(qsg), side.ptr(qbg), None)
    out.update(token_codes_f16=t16, colsum_f16=c16, block_codes_f16=b16, q_codes_f16=qc16, q_sum_f16=qs16, qbar_f16=qb16,
               q_codes_f16_grouped=qcg, q_sum_f16_grouped=qsg, qbar_f16_grouped=qbg)
    side.sync()
    return {k: np.array(side.down(v)) for k, v in out.items()}, x


E_ITEMS, E_DIM, E_M, E_ROWS, E_L, E_SLOTS = 40, 64, 12, 5, 2, 6


def esa_inputs():
    data = synth.normal_f32(7200, (E_ITEMS, E_DIM))
    data[7] = data[3]                                                  # equal scores: the earlier list entry wins
    data[11] = 0.0
    data[12] = -0.0 * np.ones(E_DIM, np.float32)                       # +0 and -0 rank as equal
    q = synth.normal_f32(7201, (3, E_DIM))
    lists = np.full((3, E_M), -1, np.int32)
    lists[0, :9] = [5, 3, -1, 7, E_ITEMS, 11, 12, 30, 2]               # a hole, an id outside the table
    lists[1, :2] = [9, 9]                                              # the same row twice
    lists[2] = synth.permutation(7202, E_ITEMS)[:E_M]
    table = np.full((E_ROWS, E_M + 3), -1, np.int32)                   # persistent rows, wider than m
    table[4, :E_M], table[0, :E_M], table[2, :E_M] = lists[0], lists[1], lists[2]
    rows = np.array([4, 0, 2, E_ROWS, -1], np.int32)                   # two requests outside the table: no-ops
    topk_rows = np.array([1, 9, 4, 9, 3], np.int32)
    return dict(data=data, q=q, lists=lists, table=table, rows=rows, topk_rows=topk_rows)


def run_esa(call, side):
    """The ESA worker's retrieval, batched and over a persistent table, and the resident-set plan of its winners."""
    x = esa_inputs()
    data, q = side.up(x["data"]), side.up(x["q"])
    lists, table, rows, topk_rows = side.up(x["lists"]), side.up(x["table"]), side.up(x["rows"]), side.up(x["topk_rows"])
    ws = side.up(np.zeros((5, E_M), np.float32))
    out = {}
    for topk in (4, 0, 20):
        oi, os_, oc = (side.up(np.full((3, E_M), -7, np.int32)), side.up(np.full((3, E_M), -7, np.float32)),
                       side.up(np.full(3, -7, np.int32)))
        call("ucm_esa_retrieve", side.ptr(data), E_ITEMS, E_DIM, side.ptr(q), side.ptr(lists), 3, E_M, topk, side.ptr(ws),
             side.ptr(oi), side.ptr(os_), side.ptr(oc), E_M, None)
        out.update({f"idx{topk}": oi, f"scores{topk}": os_, f"count{topk}": oc})
    q5 = side.up(np.concatenate([x["q"], x["q"][:2]]))                 # five requests, two of them without a row
    ri, rp, rs, rc = (side.up(np.full((E_ROWS, 5), -7, np.int32)), side.up(np.full((E_ROWS, 5), -7, np.int32)),
                      side.up(np.full((E_ROWS, 5), -7, np.float32)), side.up(np.full(E_ROWS, -7, np.int32)))
    call("ucm_esa_retrieve_rows", side.ptr(data), E_ITEMS, E_DIM, side.ptr(q5), side.ptr(table), E_ROWS, E_M + 3, E_M,
         side.ptr(rows), 5, side.ptr(topk_rows), 5, side.ptr(ws), side.ptr(ri), side.ptr(rp), side.ptr(rs), side.ptr(rc), 5, None)
    out.update(rows_idx=ri, rows_pos=rp, rows_scores=rs, rows_count=rc)
    # the winners' list positions are the request's logical blocks: two plans in a row over [layers][rows][slots]
    resident = side.up(np.full((E_L, E_ROWS, E_SLOTS), -1, np.int32))
    load, slot_of, miss = (side.up(np.full((E_L, E_ROWS, E_SLOTS), -7, np.int32)), side.up(np.full((E_L, E_ROWS, 5), -7, np.int32)),
                           side.up(np.full((E_L, E_ROWS), -7, np.int32)))
    side.sync()
    pos_h, cnt_h = np.array(side.down(rp)), np.array(side.down(rc))
    sel_h = np.stack([pos_h, pos_h[:, ::-1].copy()])                   # layer 1 sees the winners in another order
    cnt_l = np.stack([cnt_h, cnt_h])
    for r in range(E_ROWS):
        if cnt_h[r] >= 0:
            sel_h[1, r, : cnt_h[r]] = pos_h[r, : cnt_h[r]][::-1]
    sel, cnt = side.up(sel_h.astype(np.int32)), side.up(cnt_l.astype(np.int32))
    for step in (1, 2):
        if step == 2:                                                  # second step: one winner replaced per request
            sel_h = sel_h.copy()
            for r in range(E_ROWS):
                if cnt_h[r] > 0:                                       # by the lowest position that did not win
                    sel_h[:, r, 0] = min(set(range(E_M)) - set(pos_h[r, : cnt_h[r]].tolist()))
            sel = side.up(sel_h.astype(np.int32))
        call("ucm_delta_plan_rows", side.ptr(sel), side.ptr(sel), side.ptr(cnt), side.ptr(rows), 5, E_ROWS, E_L, 5,
             side.ptr(resident), E_SLOTS, side.ptr(load), side.ptr(slot_of), side.ptr(miss), None)
        side.sync()
        out.update({f"resident{step}": np.array(side.down(resident)).copy(), f"load{step}": np.array(side.down(load)).copy(),
                    f"slot_of{step}": np.array(side.down(slot_of)).copy(), f"miss{step}": np.array(side.down(miss)).copy()})
    side.sync()
    return {k: (v if isinstance(v, np.ndarray) else np.array(side.down(v))) for k, v in out.items()}, x


# ---- KVStar's selection, the prefetch bookkeeping and the loads that follow it --------------------------------------
P_L, P_ROWS, P_CAP, P_TOPK, P_MAX_BS, P_ROW_LEN, P_NB, P_POOL = 2, 3, 8, 6, 4, 8, 40, 24
P_BLOCK_BYTES = 256


def more_inputs():
    rng = np.random.default_rng(7300)
    lens = np.array([7, 1, 40, 100, 0], np.int32)
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    ks = np.array([3, 1, 40, 17, 2], np.int32)                         # the third task keeps everything
    votes = (rng.integers(0, 4, int(lens.sum())) * 0.25).astype(np.float32)
    votes[off[3] : off[3] + 10] *= -1                                  # negative votes and both zeros
    # prefetch: per request the resident cache blocks (the same in every layer) and, per layer, what they hold
    map_block = np.full((P_ROWS, P_CAP), -1, np.int32)
    map_len = np.array([6, 8, 5], np.int32)
    map_idx = np.full((P_L, P_ROWS, P_CAP), -1, np.int32)
    for r in range(P_ROWS):
        map_block[r, : map_len[r]] = 2 + r * P_CAP + rng.permutation(P_CAP)[: map_len[r]]
        for l in range(P_L):
            map_idx[l, r, : map_len[r]] = rng.permutation(12)[: map_len[r]]
    rows = np.array([2, 0, P_ROWS, 1], np.int32)                       # the third request names no row of the table
    bs_index = np.array([0, 3, 1, 2], np.int32)
    topk_len = np.array([5, 6, 4, 0], np.int32)                        # the fourth selects nothing: skipped
    topk_idx = np.stack([np.stack([rng.permutation(12)[:P_TOPK] for _ in range(4)]) for _ in range(P_L)]).astype(np.int32)
    free_block = np.zeros((P_L, P_MAX_BS, P_ROW_LEN), np.int32)
    free_len = np.zeros((P_L, P_MAX_BS), np.int32)
    for l in range(P_L):
        for i in (0, 1):                                               # a free list = some of the request's blocks
            r, b = rows[i], bs_index[i]
            pick = rng.permutation(map_len[r])[:4]
            free_block[l, b, :4] = map_block[r, pick]
            free_len[l, b] = 4
    src_table = np.stack([rng.permutation(P_POOL)[:12] for _ in range(P_ROWS)]).astype(np.int32)
    src_table[0, 3] = -1                                               # a logical block the store does not hold
    pool = rng.integers(0, 256, (P_POOL, P_L, 2, P_BLOCK_BYTES)).astype(np.uint8)
    return dict(lens=lens, off=off, ks=ks, votes=votes, map_block=map_block, map_len=map_len, map_idx=map_idx, rows=rows,
                bs_index=bs_index, topk_len=topk_len, topk_idx=topk_idx, free_block=free_block, free_len=free_len,
                src_table=src_table, pool=pool)


def run_more(call, side):
    """KVStar's selection and its return order; a pointer-array copy; a round of the prefetch bookkeeping and the
    loads it plans, from a pool in the stored layout into two layers' caches."""
    x = more_inputs()
    out = {}
    n_tasks, longest = len(x["lens"]), int(x["lens"].max())
    votes, off, lens, ks = side.up(x["votes"]), side.up(x["off"]), side.up(x["lens"]), side.up(x["ks"])
    idx, cnt = side.up(np.full((n_tasks, longest), -1, np.int32)), side.up(np.full(n_tasks, -1, np.int32))
    n_votes = len(x["votes"])
    call("ucm_kvstar_topk", side.ptr(votes), n_votes, side.ptr(off), side.ptr(lens), side.ptr(ks), n_tasks, longest, side.ptr(idx),
         longest, side.ptr(cnt), None)
    side.sync()
    out["chosen"] = np.array(side.down(idx)).copy()
    call("ucm_kvstar_order", side.ptr(votes), n_votes, side.ptr(off), side.ptr(lens), n_tasks, longest, side.ptr(idx), longest,
         side.ptr(cnt), None)
    out.update(ordered=idx, chosen_count=cnt)
    # the same with a votes array declared 50 entries shorter: the task that reaches past it (the fourth) selects
    # nothing and its row is left alone by both calls; a task that starts below 0 likewise
    off_bad = x["off"].copy()
    off_bad[0] = -3
    off_b = side.up(off_bad)
    idx_b, cnt_b = side.up(np.full((n_tasks, longest), -1, np.int32)), side.up(np.full(n_tasks, -1, np.int32))
    call("ucm_kvstar_topk", side.ptr(votes), n_votes - 50, side.ptr(off_b), side.ptr(lens), side.ptr(ks), n_tasks, longest,
         side.ptr(idx_b), longest, side.ptr(cnt_b), None)
    call("ucm_kvstar_order", side.ptr(votes), n_votes - 50, side.ptr(off_b), side.ptr(lens), n_tasks, longest, side.ptr(idx_b),
         longest, side.ptr(cnt_b), None)
    out.update(ordered_bad=idx_b, chosen_count_bad=cnt_b)
    # pointer-array copy: three pieces of 64 bytes, the last two swapped
    a, b = side.up(np.arange(192, dtype=np.uint8)), side.up(np.zeros(192, np.uint8))
    src = side.up(np.array([side.ptr(a), side.ptr(a) + 128, side.ptr(a) + 64], np.int64))
    dst = side.up(np.array([side.ptr(b), side.ptr(b) + 64, side.ptr(b) + 128], np.int64))
    call("ucm_copy_batch", side.ptr(dst), side.ptr(src), 3, 64, None)
    out["copied"] = b
    # one round of the prefetch bookkeeping
    map_block, map_len, map_idx = side.up(x["map_block"]), side.up(x["map_len"]), side.up(x["map_idx"])
    rows, bs_index, topk_len, topk_idx = side.up(x["rows"]), side.up(x["bs_index"]), side.up(x["topk_len"]), side.up(x["topk_idx"])
    free_block, free_len = side.up(x["free_block"]), side.up(x["free_len"])
    succ, succ_len = side.up(np.full((P_L, P_MAX_BS, P_ROW_LEN), -5, np.int32)), side.up(np.full((P_L, P_MAX_BS), -5, np.int32))
    load_blocks, load_count = side.up(np.full((P_L, P_ROWS, P_CAP), -1, np.int32)), side.up(np.full((P_L, P_ROWS), -5, np.int32))
    miss_idxs, miss_count = side.up(np.full((P_L, P_ROWS, P_TOPK), -1, np.int32)), side.up(np.full((P_L, P_ROWS), -5, np.int32))
    call("ucm_prefetch_plan", side.ptr(map_block), side.ptr(map_len), side.ptr(map_idx), P_ROWS, P_CAP, side.ptr(topk_idx), P_TOPK,
         side.ptr(topk_len), side.ptr(rows), side.ptr(bs_index), 4, P_L, P_MAX_BS, P_ROW_LEN, side.ptr(free_block),
         side.ptr(free_len), side.ptr(succ), side.ptr(succ_len), side.ptr(load_blocks), side.ptr(load_count),
         side.ptr(miss_idxs), side.ptr(miss_count), None)
    out.update(map_idx=map_idx, free_block=free_block, free_len=free_len, success=succ, success_len=succ_len,
               load_blocks=load_blocks, load_count=load_count, miss_idxs=miss_idxs, miss_count=miss_count)
    # the loads it planned: miss j of a row goes into load block j, K and V of both layers
    caches = [side.up(np.zeros((2, P_NB, P_BLOCK_BYTES), np.uint8)) for _ in range(P_L)]
    layers = side.pointers(caches)
    pool, src_table = side.up(x["pool"]), side.up(x["src_table"])
    call("ucm_kv_load_planned", layers, P_L, P_NB * P_BLOCK_BYTES, P_BLOCK_BYTES, P_NB, side.ptr(pool), P_POOL,
         P_L * 2 * P_BLOCK_BYTES, 0, side.ptr(miss_idxs), P_TOPK, side.ptr(src_table), 12, side.ptr(load_blocks), P_CAP,
         P_ROWS * P_CAP, side.ptr(load_count), side.ptr(rows), 4, P_ROWS, None)
    for l in range(P_L):
        out[f"cache{l}"] = caches[l]
    # the same loads out of stored blocks that two ranks share, for rank 1: [block][layer][rank][K|V]
    caches_tp = [side.up(np.zeros((2, P_NB, P_BLOCK_BYTES), np.uint8)) for _ in range(P_L)]
    pool_tp = np.full((P_POOL, P_L, 2, 2, P_BLOCK_BYTES), 0xEE, np.uint8)
    pool_tp[:, :, 1] = np.asarray(x["pool"]).reshape(P_POOL, P_L, 2, P_BLOCK_BYTES)
    pool_tp = side.up(pool_tp)
    call("ucm_kv_load_planned_tp", side.pointers(caches_tp), P_L, P_NB * P_BLOCK_BYTES, P_BLOCK_BYTES, P_NB, side.ptr(pool_tp),
         P_POOL, P_L * 4 * P_BLOCK_BYTES, 0, side.ptr(miss_idxs), P_TOPK, side.ptr(src_table), 12, side.ptr(load_blocks), P_CAP,
         P_ROWS * P_CAP, side.ptr(load_count), side.ptr(rows), 4, P_ROWS, 1, 2, None)
    for l in range(P_L):
        out[f"cache_tp{l}"] = caches_tp[l]
    side.sync()
    return {k: (v if isinstance(v, np.ndarray) else np.array(side.down(v))) for k, v in out.items()}, x


# ---- KVStar's representatives and votes ------------------------------------------------------------------------
K_L, K_NB, K_BS, K_HKV, K_D, K_MERGE, K_ROWS, K_G, K_X = 2, 10, 16, 2, 64, 4, 8, 2, 2
K_M, K_DP, K_DPAD = K_BS // K_MERGE, 20, 32
K_OFF, K_LEN = np.array([0, 3, 3], np.int32), np.array([3, 0, 5], np.int32)


def kvstar_inputs():
    rng = np.random.default_rng(7400)
    caches = [synth.normal_bf16_bits(7400 + l, (K_NB, K_BS, K_HKV, K_D)) for l in range(K_L)]
    ids = np.array([7, 2, 9, -1, 0, 4, 5, K_NB, 1, 3], np.int32)      # two ids the call must skip
    slots = np.array([0, 1, 2, 3, 3, 4, 5, 6, 6, 7], np.int32)
    lists = np.stack([np.stack([np.sort(rng.permutation(K_D)[:K_DP]) for _ in range(K_HKV)]) for _ in range(K_L)]).astype(np.int32)
    q = (rng.standard_normal((3, K_X, K_HKV * K_G, K_D)) * 0.5).astype(np.float16).view(np.uint16)
    return dict(caches=caches, ids=ids, slots=slots, lists=lists, q=q)


def run_kvstar(call, side):
    """Sub-block representatives with and without channel pruning into tables of head planes, then the votes of
    three tasks (one empty) over layer 0's pruned table, once as rows of the shared table and once as tables of
    their own."""
    import ctypes as C

    from ucm_amd import _lib

    x = kvstar_inputs()
    out = {}
    caches = [side.up(c) for c in x["caches"]]
    k_layers = side.pointers(caches)
    ids, slots, lists = side.up(x["ids"]), side.up(x["slots"]), side.up(x["lists"])
    tables = {}
    for name, pr, dp, d_pad in (("full", None, K_D, K_D), ("pruned", lists, K_DP, K_DPAD)):
        cell = d_pad * K_M
        t = side.up(np.full((K_L, K_HKV, K_ROWS, cell), 0x3c00, np.uint16))            # fp16 ones where nothing is written
        call("ucm_kvstar_block_repre", k_layers, K_L, K_NB, side.ptr(ids), side.ptr(slots), len(x["ids"]), K_BS, K_HKV, K_D,
             K_MERGE, None if pr is None else side.ptr(pr), 0 if pr is None else K_HKV * K_DP, None, 0, dp, d_pad, side.ptr(t),
             K_ROWS, K_HKV * K_ROWS * cell, K_ROWS * cell, cell, None)
        tables[name] = t
        out["table_" + name] = t
    # every listed block pruned by a list of its own choice: the two layers' lists as the two lists of EVERY layer,
    # blocks alternating between them, one naming a list that does not exist (skipped)
    cell = K_DPAD * K_M
    sel_h = (np.arange(len(x["ids"])) % 2).astype(np.int32)
    sel_h[5] = 2
    t, sel_in = side.up(np.full((K_L, K_HKV, K_ROWS, cell), 0x3c00, np.uint16)), side.up(sel_h)
    call("ucm_kvstar_block_repre", k_layers, K_L, K_NB, side.ptr(ids), side.ptr(slots), len(x["ids"]), K_BS, K_HKV, K_D, K_MERGE,
         side.ptr(lists), 0, side.ptr(sel_in), K_L, K_DP, K_DPAD, side.ptr(t), K_ROWS, K_HKV * K_ROWS * cell, K_ROWS * cell,
         cell, None)
    out["table_by_block"] = t
    x["list_sel"] = sel_h
    side.sync()
    # votes over layer 0 of the pruned table
    cell = K_DPAD * K_M
    q, seg_off, seg_len = side.up(x["q"]), side.up(K_OFF), side.up(K_LEN)
    q_off = side.up((np.arange(3) * K_X * K_HKV * K_G * K_D).astype(np.int64))
    sel = side.up(np.zeros(3, np.int32))
    mf, pf = C.c_int64(), C.c_int64()
    _lib.call("ucm_kvstar_workspace_floats", 3, K_HKV, K_X * K_G, 5, K_M, K_DPAD, 0, C.byref(mf), C.byref(pf))
    ws_max, ws_part = side.up(np.zeros(max(mf.value, 1), np.float32)), side.up(np.zeros(max(pf.value, 1), np.float32))
    votes = side.up(np.full(K_ROWS, -3, np.float32))
    q_elems = int(np.prod(x["q"].shape))
    call("ucm_kvstar_votes", side.ptr(q), q_elems, side.ptr(q_off), K_X, K_HKV * K_G, K_D, side.ptr(lists), K_L, side.ptr(sel),
         side.ptr(tables["pruned"]), K_ROWS, K_ROWS * cell, cell, side.ptr(seg_off), side.ptr(seg_len), 3, 5, K_M, K_HKV, K_DP,
         K_DPAD, side.ptr(ws_max), mf.value, side.ptr(ws_part), pf.value, side.ptr(votes), 0, None)
    out["votes"] = votes
    # descriptors the call must not follow: a query block that ends past the buffer (declared one task shorter), a
    # channel list that does not exist, rows past the table (declared two rows shorter).  Each of the three tasks
    # breaks one rule in turn, the other two vote as before.
    q_need = K_X * K_HKV * K_G * K_D
    for case in range(3):
        bad_sel = np.zeros(3, np.int32)
        bad_sel[0] = K_L if case == 1 else 0
        sel_b = side.up(bad_sel)
        votes_b = side.up(np.full(K_ROWS, -3, np.float32))
        call("ucm_kvstar_votes", side.ptr(q), q_elems - (q_need if case == 0 else 0), side.ptr(q_off), K_X, K_HKV * K_G, K_D,
             side.ptr(lists), K_L, side.ptr(sel_b), side.ptr(tables["pruned"]), K_ROWS - (2 if case == 2 else 0), K_ROWS * cell,
             cell, side.ptr(seg_off), side.ptr(seg_len), 3, 5, K_M, K_HKV, K_DP, K_DPAD, side.ptr(ws_max), mf.value,
             side.ptr(ws_part), pf.value, side.ptr(votes_b), 0, None)
        out[f"votes_bad{case}"] = votes_b
    base = side.ptr(tables["pruned"])
    task_tables = side.up(np.array([base + int(a) * cell * 2 for a in K_OFF], np.int64))
    head_strides = side.up(np.full(3, K_ROWS * cell, np.int64))
    votes_t = side.up(np.full(K_ROWS, -3, np.float32))
    call("ucm_kvstar_votes_tables", side.ptr(q), q_elems, side.ptr(q_off), K_X, K_HKV * K_G, K_D, side.ptr(lists), K_L,
         side.ptr(sel), side.ptr(task_tables), side.ptr(head_strides), cell, side.ptr(seg_off), side.ptr(seg_len), 3, 5, K_M,
         K_HKV, K_DP, K_DPAD, side.ptr(ws_max), mf.value, side.ptr(ws_part), pf.value, side.ptr(votes_t), K_ROWS, 0, None)
    out["votes_tables"] = votes_t
    # query tokens parked as fp16 from bf16, fp16 and fp32 queries: rows out of order, one row and one place out of range
    row_elems = K_HKV * K_G * K_D
    rng = np.random.default_rng(7410)
    qf = (rng.standard_normal((6, row_elems)) * np.array([1e-6, 1.0, 300.0, 7e4, 1.0, 1.0], np.float32)[:, None]).astype(np.float32)
    qf[4, :4] = [np.inf, -np.inf, 0.0, -0.0]
    src = side.up(np.array([5, 0, 6, 3, 2, 1], np.int32))                  # 6 is past the queries
    dst = side.up((np.array([0, 2, 3, 1, 9, 4], np.int64)) * row_elems)     # 9 is past the ring of 6 rows
    with np.errstate(over="ignore"):
        q_half = qf.astype(np.float16).view(np.uint16)
    for name, code, arr in (("park_f32", 0, qf), ("park_bf16", 1, oracle.bf16_bits(qf)), ("park_f16", 2, q_half)):
        ring, q_in = side.up(np.full((6, row_elems), 0x3c00, np.uint16)), side.up(arr)
        call("ucm_kvstar_park_queries", side.ptr(q_in), code, 6, row_elems, side.ptr(src), side.ptr(dst), 6, side.ptr(ring),
             6 * row_elems, None)
        side.sync()
        out[name] = ring
    x["park_q"] = qf
    # rows of one array into rows of another (a step's query rows kept for the next step's selection): out of order,
    # a source row past the array, a negative one, a destination past the array; with and without destination indices
    rows_src = side.up(np.arange(7 * 48, dtype=np.int32).reshape(7, 48))
    pick = side.up(np.array([6, 0, 7, 3, -1, 2], np.int32))
    put = side.up(np.array([1, 4, 0, 5, 2, 9], np.int32))
    for name, where in (("rows_indexed", put), ("rows_in_order", None)):
        rows_dst = side.up(np.full((6, 48), -5, np.int32))
        call("ucm_park_rows", side.ptr(rows_src), 7, side.ptr(pick), side.ptr(rows_dst), 6, None if where is None else side.ptr(where),
             6, 48 * 4, None)
        side.sync()
        out[name] = rows_dst
    side.sync()
    return {k: (v if isinstance(v, np.ndarray) else np.array(side.down(v))) for k, v in out.items()}, x

