"""Writes tests/golden/*.npz from the reference's own C++ compiled in
oracle/_ref (see oracle/Makefile).  Needs the reference tree at build time, so
it runs only in the build container; the fixtures it writes are data (seeds,
shapes, expected outputs) and travel everywhere.

    python tests/golden/make_golden.py

Inputs come from tests/synth.py (integer-only generator), so a fixture holds
just the seed and shape of each case plus what the reference returned.
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle  # noqa: E402
import synth  # noqa: E402


def cases_select():
    """(name, seed, n_blocks, q_heads, kv_heads, head_dim, k, start_w, end_w, bf16_repre)"""
    return [
        ("llama_cfg1_small", 11, 96, 32, 8, 128, 19, 1, 2, 0),
        ("llama_bf16_repre", 12, 80, 32, 8, 128, 19, 1, 2, 1),
        ("qwen72_g8", 13, 70, 64, 8, 128, 17, 1, 2, 0),
        ("mha_no_group", 14, 40, 4, 4, 64, 9, 1, 2, 0),
        ("tiny_heads", 15, 33, 8, 2, 32, 8, 1, 2, 0),
        ("identity_k_ge_n", 16, 12, 32, 8, 128, 12, 1, 2, 0),
        ("identity_n_le_3", 17, 3, 32, 8, 128, 2, 1, 2, 0),
        ("wide_windows", 18, 50, 16, 4, 128, 14, 3, 5, 0),
        ("k_equals_windows", 19, 30, 16, 4, 128, 3, 1, 2, 0),
    ]


def select_inputs(seed, n, hq, hkv, d, bf16_repre):
    q = synth.normal_bf16_as_f32(seed, (hq, d))
    repre = synth.normal_f32(seed + 1000, (n, hkv, 1, d)) * np.float32(0.25)
    if bf16_repre:
        repre = synth.bf16_widen(synth.bf16_round_bits(repre))
    return q, repre


def prefetch_scenarios():
    """(seed, layers, requests, runs) of the GSA prefetch-engine cases."""
    return [(2100, 2, 3, 4), (2200, 3, 5, 6), (2300, 1, 1, 5), (2400, 4, 6, 3)]


def prefetch_scenario(seed, n_layers, n_req, n_runs):
    """A deterministic call sequence for GSAPrefetchEngineC: per request a block table, the resident logical blocks
    (set_blocks_map's selectIndex), an initial free list (a subset of the resident blocks, the reference's
    prefetch_blocks), and per run either a (layer-wise different) selection or, now and then, a block appended by
    add_blocks_map first.  Requests sit in shuffled batch slots.  Some selections exceed what the free list can
    serve, and free-listed blocks become hits."""
    pool = synth.permutation(seed, 600)
    reqs, used = [], 0
    slots = synth.permutation(seed + 1, 8)
    for r in range(n_req):
        n = int(synth.ints(seed + 10 + r, 1, 8, 40)[0])
        table = [int(x) for x in pool[used : used + n]]
        used += n + 6                                   # room for appended blocks
        m = int(synth.ints(seed + 30 + r, 1, 4, n)[0])
        select = sorted(int(x) for x in synth.permutation(seed + 50 + r, n)[:m])
        n_free = int(synth.ints(seed + 70 + r, 1, 0, m)[0])
        free = [table[select[int(i)]] for i in synth.permutation(seed + 90 + r, m)[:n_free]]
        reqs.append(dict(req_id=100 + 7 * r, bs_index=int(slots[r]), table=table, select=select, free=free,
                         spare=[int(x) for x in pool[used - 6 : used]]))
    runs = []
    for t in range(n_runs):
        run = dict(adds=[], topk=[])
        for r, rq in enumerate(reqs):
            n = len(rq["table"]) + sum(1 for run_ in runs for a in run_["adds"] if a[0] == r)
            if t > 0 and int(synth.ints(seed + 200 + 13 * t + r, 1, 0, 2)[0]) == 0 and n - len(rq["table"]) < 6:
                run["adds"].append((r, n, rq["spare"][n - len(rq["table"])]))     # (request, logical idx, cache block)
                n += 1
            k = int(synth.ints(seed + 300 + 17 * t + r, 1, 1, min(len(rq["select"]) + 3, n))[0])
            run["topk"].append([[int(x) for x in synth.permutation(seed + 400 + 100 * t + 10 * r + l, n)[:k]]
                                for l in range(n_layers)])
        runs.append(run)
    return reqs, runs


def run_reference_prefetch(gp, n_layers, reqs, runs, max_bs=8, max_len=64):
    """Drives the reference's engine (compiled in oracle/_ref) through a scenario; returns per run what it left in
    its tensors and accessors."""
    import time

    import torch

    i32 = dict(dtype=torch.int32)
    free = torch.zeros((n_layers, max_bs, max_len), **i32)
    free_len = torch.zeros((n_layers, max_bs), **i32)
    success = torch.zeros((n_layers, max_bs, max_len), **i32)
    success_len = torch.zeros((n_layers, max_bs), **i32)
    eng = gp.GSAPrefetchEngineC(free, success, free_len, success_len, False)
    for rq in reqs:
        eng.set_blocks_map(rq["req_id"], list(rq["table"]), list(rq["select"]))
        free[:, rq["bs_index"], : len(rq["free"])] = torch.tensor(rq["free"], **i32)
        free_len[:, rq["bs_index"]] = len(rq["free"])
    results = []
    for t, run in enumerate(runs):
        for r, idx, blk in run["adds"]:
            eng.add_blocks_map(reqs[r]["req_id"], idx, blk)
        buf = torch.zeros((n_layers, len(reqs), max_len), dtype=torch.int64)
        for r in range(len(reqs)):
            for l in range(n_layers):
                tk = run["topk"][r][l]
                buf[l, r, : len(tk)] = torch.tensor(tk, dtype=torch.int64)
        eng.set_blocks_table_info(success, success_len, buf, t)
        eng.run_async_prefetch_bs([rq["req_id"] for rq in reqs], [len(run["topk"][r][0]) for r in range(len(reqs))],
                                  [rq["bs_index"] for rq in reqs], 0)
        while not eng.get_prefetch_status():
            time.sleep(0.001)
        maps = eng.obtain_blocks_map()
        results.append(dict(success=success.clone().numpy(), success_len=success_len.clone().numpy(),
                            free=free.clone().numpy(), free_len=free_len.clone().numpy(),
                            loads=eng.obtain_load_blocks(), misses=eng.obtain_miss_idxs(),
                            maps={rq["req_id"]: [dict(m) for m in maps[rq["req_id"]]] for rq in reqs}))
    for rq in reqs:
        eng.del_blocks_map(rq["req_id"])
    return results


def main():
    assert oracle.ref.available, "build oracle/_ref first (make -C oracle)"
    ref = oracle.ref
    out = {}
    meta = {"simd": ref.simd_name(), "select": [], "dot": [], "mean": [], "ties": [], "esa": []}

    for name, seed, n, hq, hkv, d, k, sw, ew, b16 in cases_select():
        q, repre = select_inputs(seed, n, hq, hkv, d, b16)
        qm = ref.q_head_mean(q, hkv)
        out[f"select/{name}/qmean"] = qm
        out[f"select/{name}/scores"] = ref.kq_scores(qm, repre)
        out[f"select/{name}/idx"] = ref.select_topk(q, repre, k, sw, ew)
        meta["select"].append([name, seed, n, hq, hkv, d, k, sw, ew, b16])

    for i, dim in enumerate([1, 7, 16, 31, 128, 144, 1024]):
        q = synth.normal_f32(200 + i, (dim,))
        kk = synth.normal_f32(300 + i, (dim,))
        out[f"dot/{dim}"] = np.array([ref.vector_dot(q, kk)], np.float32)
        meta["dot"].append([dim, 200 + i, 300 + i])

    for i, (num_k, dim) in enumerate([(1, 16), (4, 128), (8, 128), (128, 128), (5, 19)]):
        v = synth.normal_bf16_as_f32(400 + i, (num_k, dim))
        out[f"mean/{num_k}x{dim}"] = ref.vector_mean(v)
        meta["mean"].append([num_k, dim, 400 + i])

    # one block through ComputeKRepreBlock ([kHead, blockSize, headSize])
    kb = synth.normal_bf16_as_f32(450, (8, 128, 128))
    out["krepre/8x128x128"] = ref.k_repre_block(kb)

    # selection with many equal scores; scores are fed through a 1-dim
    # "representative" so the public SelectTopK sees them unchanged
    q1 = np.ones((1, 1), np.float32)
    for i in range(24):
        n = int(synth.ints(500 + i, 1, 4, 40)[0])
        k = int(synth.ints(600 + i, 1, 1, n + 2)[0])
        sw = int(synth.ints(700 + i, 1, 0, 2)[0])
        ew = int(synth.ints(800 + i, 1, 0, 3)[0])
        sc = synth.ints(900 + i, n, 0, 3).astype(np.float32)
        out[f"ties/{i}"] = ref.select_topk(q1, sc.reshape(n, 1, 1, 1), k, sw, ew)
        meta["ties"].append([i, n, k, sw, ew, 900 + i])

    # ESA backend (retrieval_backend.cpp): scores of the best k in descending order
    rb = ref.retrieval_backend_module()
    if rb is not None:
        for i, (rows, dim, b, m, topk) in enumerate([(300, 1024, 2, 120, 20), (64, 256, 3, 64, 100), (50, 1024, 1, 30, 7)]):
            data = synth.normal_bf16_as_f32(1000 + i, (rows, dim))
            q = synth.normal_bf16_as_f32(1100 + i, (b, dim))
            idx = np.stack([synth.permutation(1200 + i * 8 + r, rows)[:m] for r in range(b)]).astype(np.int32)
            idx[:, m - 3:] = -1  # padding entries
            be = rb.RetrievalWorkerBackend(data)
            rid = be.submit(q, topk, idx)
            be.wait(rid)
            res = be.get_result(rid)
            out[f"esa/{i}/indices"] = np.asarray(res["indices"], np.int32)
            out[f"esa/{i}/scores"] = np.asarray(res["scores"], np.float32)
            meta["esa"].append([i, rows, dim, b, m, topk, 1000 + i, 1100 + i, 1200 + i * 8])
            del be

    # GSA prefetch engine (kvcache_pre.cpp): success tables, free lists, loads and misses of every run
    gp = ref.gsa_prefetch_module()
    meta["prefetch"] = []
    if gp is not None:
        for seed, n_layers, n_req, n_runs in prefetch_scenarios():
            reqs, runs = prefetch_scenario(seed, n_layers, n_req, n_runs)
            res = run_reference_prefetch(gp, n_layers, reqs, runs)
            for t, r in enumerate(res):
                key = f"prefetch/{seed}/{t}"
                out[key + "/success"], out[key + "/success_len"] = r["success"], r["success_len"]
                out[key + "/free"], out[key + "/free_len"] = r["free"], r["free_len"]
                flat = lambda x: np.array([v for per_req in x for per_layer in per_req for v in [len(per_layer)] + list(per_layer)], np.int32)
                out[key + "/loads"], out[key + "/misses"] = flat(r["loads"]), flat(r["misses"])
                out[key + "/maps"] = np.array([v for rq in reqs for m in r["maps"][rq["req_id"]]
                                               for kv in [(len(m), -1)] + sorted(m.items()) for v in kv], np.int32)
            meta["prefetch"].append([seed, n_layers, n_req, n_runs])

    out["meta"] = np.frombuffer(json.dumps(meta).encode(), np.uint8)
    path = os.path.join(HERE, "gsa_esa_reference.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
