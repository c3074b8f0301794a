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

    out["meta"] = np.frombuffer(json.dumps(meta).encode(), np.uint8)
    path = os.path.join(HERE, "gsa_esa_reference.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
