"""The GSA prefetch-engine protocol replayed on the CPU oracle (oracle.prefetch_run per request and layer): the
checker for the reference's compiled engine (tests/test_oracle_pins.py), for the golden vectors, and for the device
engine (tests/test_gpu_prefetch.py).  Test infrastructure only."""
import numpy as np

import oracle as O


class OracleEngine:
    def __init__(self, n_layers, max_bs=8, max_len=64):
        self.n_layers, self.max_len = n_layers, max_len
        self.free = np.zeros((n_layers, max_bs, max_len), np.int32)
        self.free_len = np.zeros((n_layers, max_bs), np.int32)
        self.success = np.zeros((n_layers, max_bs, max_len), np.int32)
        self.success_len = np.zeros((n_layers, max_bs), np.int32)
        self.blocks = {}      # req -> block ids (slot order)
        self.idx = {}         # req -> [layer] int32 array, logical block held by each slot

    def set_blocks_map(self, req, table, select):
        self.blocks[req] = [table[i] for i in select]
        self.idx[req] = [np.array(select, np.int32) for _ in range(self.n_layers)]

    def add_blocks_map(self, req, idx, block):
        self.blocks[req].append(block)
        self.idx[req] = [np.append(a, np.int32(idx)).astype(np.int32) for a in self.idx[req]]

    def run(self, req_ids, topk, bs_indexes):
        """topk[r][l] = selection of request r in layer l.  Returns (loads, misses) as [request][layer] lists."""
        loads, misses = [], []
        for r, req in enumerate(req_ids):
            b = bs_indexes[r]
            lr, mr = [], []
            for l in range(self.n_layers):
                succ, sl, ld, ms, fr = O.prefetch_run(self.blocks[req], self.idx[req][l], topk[r][l],
                                                      self.free[l, b, : self.free_len[l, b]], self.free_len[l, b], self.max_len)
                self.success[l, b] = succ
                self.success_len[l, b] = sl
                self.free[l, b, : len(fr)] = fr
                self.free_len[l, b] = len(fr)
                lr.append(ld.tolist())
                mr.append(ms.tolist() if len(ld) or len(ms) else [])
            loads.append(lr)
            misses.append(mr)
        return loads, misses

    def maps(self, req):
        return [dict(zip(self.blocks[req], a.tolist())) for a in self.idx[req]]


def replay(n_layers, reqs, runs, max_bs=8, max_len=64):
    """The scenario of tests/golden/make_golden.py through the oracle; same result records as run_reference_prefetch."""
    eng = OracleEngine(n_layers, max_bs, max_len)
    for rq in reqs:
        eng.set_blocks_map(rq["req_id"], rq["table"], rq["select"])
        eng.free[:, rq["bs_index"], : len(rq["free"])] = rq["free"]
        eng.free_len[:, rq["bs_index"]] = len(rq["free"])
    out = []
    for run in runs:
        for r, idx, blk in run["adds"]:
            eng.add_blocks_map(reqs[r]["req_id"], idx, blk)
        loads, misses = eng.run([rq["req_id"] for rq in reqs], run["topk"], [rq["bs_index"] for rq in reqs])
        out.append(dict(success=eng.success.copy(), success_len=eng.success_len.copy(), free=eng.free.copy(),
                        free_len=eng.free_len.copy(), loads=loads, misses=misses,
                        maps={rq["req_id"]: eng.maps(rq["req_id"]) for rq in reqs}))
    return out


def same_result(a, b, free_valid_only=True):
    """Compares two result records; entries of a free list beyond its length are leftovers and not compared."""
    assert np.array_equal(a["success"], b["success"]) and np.array_equal(a["success_len"], b["success_len"])
    assert np.array_equal(a["free_len"], b["free_len"])
    L, B, _ = a["free"].shape
    for l in range(L):
        for s in range(B):
            n = a["free_len"][l, s]
            assert np.array_equal(a["free"][l, s, :n], b["free"][l, s, :n]), (l, s)
    assert a["loads"] == b["loads"], (a["loads"], b["loads"])
    assert a["misses"] == b["misses"], (a["misses"], b["misses"])
    assert a["maps"] == b["maps"]
