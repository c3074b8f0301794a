"""Pins the CPU oracle (oracle/ucm_oracle.c) before anything is compared with
it: (1) against the golden vectors written from the reference's own C++
(tests/golden/make_golden.py), (2) against that compiled C++ directly where
oracle/_ref exists, (3) against closed forms / brute force chosen so that a
dropped term, a wrong index or a flipped comparison fails."""
import itertools

import numpy as np
import pytest

import oracle as O
import synth
from golden.make_golden import cases_select, select_inputs

bits = lambda a: np.ascontiguousarray(a, np.float32).view(np.uint32)


# ------------------------------------------------------------------ golden

def test_golden_select_cases(golden):
    z, meta = golden
    assert meta["simd"] == "x86_64 AVX512F"
    assert [c[0] for c in meta["select"]] == [c[0] for c in cases_select()]
    for name, seed, n, hq, hkv, d, k, sw, ew, b16 in meta["select"]:
        q, repre = select_inputs(seed, n, hq, hkv, d, b16)
        qm = O.q_head_mean(q, hkv)
        assert np.array_equal(bits(qm), bits(z[f"select/{name}/qmean"])), name
        assert np.array_equal(bits(O.kq_scores(qm, repre)), bits(z[f"select/{name}/scores"])), name
        idx, scores = O.select_topk(q, repre, k, sw, ew)
        assert np.array_equal(idx, z[f"select/{name}/idx"]), name
        assert np.array_equal(bits(scores), bits(z[f"select/{name}/scores"])), name


def test_golden_dot_mean_krepre(golden):
    z, meta = golden
    for dim, s1, s2 in meta["dot"]:
        got = O.dot16(synth.normal_f32(s1, (dim,)), synth.normal_f32(s2, (dim,)))
        assert bits(got)[()] == bits(z[f"dot/{dim}"])[0], dim
    for num_k, dim, seed in meta["mean"]:
        v = synth.normal_bf16_as_f32(seed, (num_k, dim))
        assert np.array_equal(bits(O.vector_mean(v)), bits(z[f"mean/{num_k}x{dim}"]))
    kb = synth.normal_bf16_as_f32(450, (8, 128, 128))
    want = z["krepre/8x128x128"]
    assert np.array_equal(bits(O.k_repre_block(kb)), bits(want))
    # the paged-cache entry point reads [T][H][D] bf16 instead of [H][T][D] fp32
    cache = synth.bf16_round_bits(kb.transpose(1, 0, 2))[None]
    repre = np.zeros((3, 8 * 128), np.float32)
    O.block_mean_paged(cache, [0], [2], repre)
    assert np.array_equal(bits(repre[2]), bits(want.reshape(-1)))
    assert not repre[:2].any()


def test_golden_ties(golden):
    z, meta = golden
    for i, n, k, sw, ew, seed in meta["ties"]:
        sc = synth.ints(seed, n, 0, 3).astype(np.float32)
        assert np.array_equal(O.topk_windows(sc, k, sw, ew), z[f"ties/{i}"]), (i, n, k, sw, ew)


def test_golden_esa_backend(golden):
    z, meta = golden
    assert meta["esa"], "fixture was written without the ESA backend"
    for i, rows, dim, b, m, topk, s_data, s_q, s_idx in meta["esa"]:
        data = synth.normal_bf16_as_f32(s_data, (rows, dim))
        q = synth.normal_bf16_as_f32(s_q, (b, dim))
        idx = np.stack([synth.permutation(s_idx + r, rows)[:m] for r in range(b)]).astype(np.int32)
        idx[:, m - 3:] = -1
        for r in range(b):
            gi, gs = O.esa_retrieve(data, q[r], idx[r], topk)
            want_s = z[f"esa/{i}/scores"][r]
            want_i = z[f"esa/{i}/indices"][r]
            assert np.array_equal(bits(gs), bits(want_s))
            assert len(np.unique(want_s)) == len(want_s)  # no ties in the fixture, so order is pinned
            assert np.array_equal(gi, want_i)


# ------------------------------------------- the compiled reference, live

needs_ref = pytest.mark.skipif(not O.ref.available, reason="oracle/_ref not built (reference tree absent)")


@needs_ref
def test_ref_dot_and_mean_random():
    rng = np.random.default_rng(5)
    for dim in [1, 3, 16, 17, 48, 128, 130, 1024, 1037]:
        for _ in range(60):
            q = rng.standard_normal(dim).astype(np.float32) * np.float32(rng.uniform(1e-3, 1e3))
            k = rng.standard_normal(dim).astype(np.float32)
            assert bits(O.dot16(q, k))[()] == bits(O.ref.vector_dot(q, k))[()]
    for num_k, dim in itertools.product([1, 2, 4, 8, 127, 128], [1, 16, 40, 128]):
        v = rng.standard_normal((num_k, dim)).astype(np.float32)
        assert np.array_equal(bits(O.vector_mean(v)), bits(O.ref.vector_mean(v)))


@needs_ref
def test_ref_select_random_shapes():
    rng = np.random.default_rng(6)
    for trial in range(40):
        hkv = int(rng.choice([1, 2, 4, 8]))
        g = int(rng.choice([1, 2, 4, 8]))
        d = int(rng.choice([32, 64, 128]))
        n = int(rng.integers(1, 200))
        k = int(rng.integers(1, 60))
        q = synth.normal_bf16_as_f32(2000 + trial, (hkv * g, d))
        repre = synth.normal_f32(3000 + trial, (n, hkv, 1, d))
        assert np.array_equal(bits(O.q_head_mean(q, hkv)), bits(O.ref.q_head_mean(q, hkv)))
        idx, scores = O.select_topk(q, repre, k)
        assert np.array_equal(bits(scores), bits(O.ref.kq_scores(O.ref.q_head_mean(q, hkv), repre)))
        assert np.array_equal(idx, O.ref.select_topk(q, repre, k)), (trial, n, k)


@needs_ref
def test_ref_num_krepre_max():
    """numKrepre > 1 takes the best representative per head (fmax)."""
    for trial in range(10):
        q = synth.normal_f32(4000 + trial, (8, 128))
        repre = synth.normal_f32(4100 + trial, (37, 8, 3, 128))
        assert np.array_equal(bits(O.kq_scores(q, repre)), bits(O.ref.kq_scores(q, repre)))


@needs_ref
def test_ref_ties_exhaustive_small():
    q1 = np.ones((1, 1), np.float32)
    rng = np.random.default_rng(7)
    for _ in range(3000):
        n = int(rng.integers(1, 15))
        k = int(rng.integers(1, 17))
        sw, ew = int(rng.integers(0, 3)), int(rng.integers(0, 4))
        sc = rng.integers(0, 3, n).astype(np.float32)
        want = O.ref.select_topk(q1, sc.reshape(n, 1, 1, 1), k, sw, ew)
        assert np.array_equal(O.topk_windows(sc, k, sw, ew), want), (n, k, sw, ew, sc)


@needs_ref
def test_ref_batch_entry_point():
    lens = np.array([5, 40, 3, 130, 64], np.int32)
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    tk = np.array([O.compute_topk_len(int(n)) for n in lens], np.int32)
    q = synth.normal_bf16_as_f32(5000, (len(lens), 32, 128))
    repre = synth.normal_f32(5001, (int(lens.sum()), 8 * 128))
    idx, cnt, _ = O.select_topk_bs(q, repre, off, lens, tk, 8, out_stride=140)
    want = O.ref.select_topk_bs(q, repre, off, lens, tk, 8, out_stride=140)
    for r in range(len(lens)):
        assert np.array_equal(idx[r, : cnt[r]], want[r, : cnt[r]])


@needs_ref
def test_ref_esa_backend_live():
    rb = O.ref.retrieval_backend_module()
    if rb is None:
        pytest.skip("retrieval_backend extension not built")
    data = synth.normal_bf16_as_f32(6000, (200, 1024))
    be = rb.RetrievalWorkerBackend(data)
    q = synth.normal_bf16_as_f32(6001, (2, 1024))
    idx = np.stack([synth.permutation(6002 + r, 200)[:150] for r in range(2)]).astype(np.int32)
    rid = be.submit(q, 33, idx)
    be.wait(rid)
    res = be.get_result(rid)
    for r in range(2):
        gi, gs = O.esa_retrieve(data, q[r], idx[r], 33)
        assert np.array_equal(bits(gs), bits(res["scores"][r]))
        assert np.array_equal(gi, res["indices"][r])


# ------------------------------------------------ closed forms, brute force

def test_dot16_lane_structure():
    """Each of the 16 lanes is its own fma chain; a one-hot probe at every
    position must come back exactly, and the butterfly must be
    ((l0+l8)+(l4+l12)) + ((l2+l10)+(l6+l14)) + ... : checked with values whose
    sum depends on the association."""
    for pos in range(128):
        q = np.zeros(128, np.float32)
        k = np.zeros(128, np.float32)
        q[pos], k[pos] = 3.0, 0.5
        assert O.dot16(q, k) == np.float32(1.5)
    lane = np.array([1e8, 1, -1e8, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1], np.float32)
    f = np.float32
    a = [f(lane[j + 8] + lane[j]) for j in range(8)]
    b = [f(a[j + 4] + a[j]) for j in range(4)]
    want = f(f(b[0] + b[2]) + f(b[1] + b[3]))
    assert O.dot16(lane, np.ones(16, np.float32)) == want
    assert want != np.float32(np.sum(lane.astype(np.float64)))  # the probe does depend on the order
    # fma, not mul-then-add: (1+2^-12)^2 - 1 keeps the 2^-24 term only when fused
    x = np.float32(1 + 2.0 ** -12)
    q = np.zeros(32, np.float32)
    k = np.zeros(32, np.float32)
    q[0], k[0] = 1.0, -1.0
    q[16], k[16] = x, x
    assert O.dot16(q, k) == np.float32(2.0 ** -11 + 2.0 ** -24)


def test_mean_is_sequential_fp32():
    v = np.array([[1e8], [1.0], [-1e8], [1.0]], np.float32)
    f = np.float32
    want = f(f(f(f(v[0, 0] + v[1, 0]) + v[2, 0]) + v[3, 0]) * f(0.25))
    assert O.vector_mean(v)[0] == want == f(0.25)
    q = np.arange(4 * 8, dtype=np.float32).reshape(4, 8)
    assert np.array_equal(O.q_head_mean(q, 2), np.stack([q[:2].mean(0), q[2:].mean(0)]))
    assert np.array_equal(O.q_head_mean(q, 4), q)


def test_topk_windows_brute_force():
    rng = np.random.default_rng(8)
    for _ in range(2000):
        n = int(rng.integers(1, 12))
        k = int(rng.integers(0, 14))
        sw, ew = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        sc = rng.integers(0, 4, n).astype(np.float32)
        got = O.topk_windows(sc, k, sw, ew)
        if sw + ew >= n or k >= n or k == 0:
            assert np.array_equal(got, np.arange(n))
            continue
        mid = sorted(range(sw, n - ew), key=lambda i: (-sc[i], i))[: max(k - sw - ew, 0)]
        full = list(range(sw)) + mid + list(range(n - ew, n))
        want = sorted(full[:k]) if k >= sw + ew else full[:k]
        assert list(got) == want, (n, k, sw, ew, sc)
        assert len(got) == k and all(np.diff(got) > 0)


def test_compute_topk_len_closed_form():
    for n in range(0, 400):
        t = int(n * 0.3)
        want = min(32, n) if t < 32 else (48 if t > 48 else t)
        assert O.compute_topk_len(n) == want
    assert O.compute_topk_len(256) == 48 and O.compute_topk_len(20) == 20 and O.compute_topk_len(120) == 36


def test_get_offset_and_block_table():
    shape = (128, 8, 128)
    k_sz = 128 * 8 * 128 * 2
    assert O.get_offset(shape, 0, 1, 2, 0, False) == 0
    assert O.get_offset(shape, 0, 1, 2, 0, True) == k_sz
    assert O.get_offset(shape, 0, 1, 2, 5, False) == 5 * 2 * k_sz
    assert O.get_offset(shape, 1, 2, 2, 3, True) == 3 * 4 * k_sz + 2 * k_sz + k_sz
    assert O.get_offset(shape, 1, 2, 2, 3, False, is_mla=True) == 3 * 2 * k_sz
    table = np.array([9, 4, 7, 1, 3], np.int32)
    phys, sl = O.block_table_gather(table, [0, 2, 4], 5 * 128, 128)
    assert list(phys) == [9, 7, 3] and sl == 3 * 128
    _, sl = O.block_table_gather(table, [0, 2, 4], 4 * 128 + 17, 128)
    assert sl == 2 * 128 + 17


def test_kv_moves_round_trip():
    n_layers, nb, bb = 3, 11, 64
    rng = np.random.default_rng(9)
    layers = [rng.integers(0, 256, 2 * nb * bb, dtype=np.uint8) for _ in range(n_layers)]
    ids = np.array([7, 0, 10, 3], np.int32)
    staging = np.zeros(len(ids) * n_layers * 2 * bb, np.uint8)
    O.kv_move_blocks(layers, nb * bb, bb, ids, staging, True)
    st = staging.reshape(len(ids), n_layers, 2, bb)
    for i, b in enumerate(ids):
        for l in range(n_layers):
            for kv in range(2):
                assert np.array_equal(st[i, l, kv], layers[l].reshape(2, nb, bb)[kv, b])
                off = O.get_offset((bb, 1, 1), 0, 1, 1, l, bool(kv))
                assert np.array_equal(staging[i * n_layers * 2 * bb + off:][:bb], st[i, l, kv])
    fresh = [np.zeros_like(a) for a in layers]
    O.kv_move_blocks(fresh, nb * bb, bb, ids, staging, False)
    for l in range(n_layers):
        f, o = fresh[l].reshape(2, nb, bb), layers[l].reshape(2, nb, bb)
        assert np.array_equal(f[:, ids], o[:, ids])
        rest = np.setdiff1d(np.arange(nb), ids)
        assert not f[:, rest].any()


def test_hash_closed_forms():
    rng = np.random.default_rng(10)
    dim, nbits = 16, 24
    w = rng.standard_normal((dim, nbits)).astype(np.float32) * 2
    xb = synth.normal_bf16_bits(7000, (5, 3, dim))
    x = synth.bf16_widen(xb).astype(np.float64)
    proj = x @ w.astype(np.float64)
    want_bits = (proj > 0).astype(np.uint8).reshape(5, 3, nbits // 8, 8)
    want = (want_bits * (1 << np.arange(8, dtype=np.uint8))).sum(-1).astype(np.uint8)
    got = O.hash_encode(xb, w)
    assert got.shape == (5, 3, 3) and np.array_equal(got, want)
    # sum score == explicit +-1 inner products
    qc = rng.integers(0, 256, (4, 3), dtype=np.uint8)
    kc = rng.integers(0, 256, (6, 2, 5, 3), dtype=np.uint8)
    un = lambda c: np.unpackbits(c, axis=-1, bitorder="little").astype(np.int64) * 2 - 1
    want = np.einsum("id,njsd->n", un(qc), un(kc))
    assert np.array_equal(O.hash_scores_sum(qc, kc), want)
    # majority vote and popcount similarity
    tc = rng.integers(0, 256, (3, 8, 2, 3), dtype=np.uint8)
    ones = np.unpackbits(tc, axis=-1, bitorder="little").sum(1)
    want_codes = np.packbits((2 * ones > 8).astype(np.uint8), axis=-1, bitorder="little")
    assert np.array_equal(O.hash_majority(tc), want_codes)
    q2 = rng.integers(0, 256, (2, 3), dtype=np.uint8)
    sim = (nbits - np.unpackbits(q2[None] ^ want_codes, axis=-1).sum(-1)).sum(-1)
    assert np.array_equal(O.hash_scores_block(q2, want_codes), sim)


def test_delta_plan_against_set_arithmetic():
    """The reference's delta load in terms of sets (esa.py:312-338): what stays is resident AND selected, what is
    loaded is selected minus resident, and it goes into slots whose block is no longer selected."""
    rng = np.random.default_rng(11)
    for _ in range(500):
        n_slots = int(rng.integers(1, 20))
        k = int(rng.integers(0, n_slots + 3))
        universe = int(rng.integers(max(k, 1), 60))
        resident = rng.permutation(universe)[:n_slots].astype(np.int32)
        resident = np.concatenate([resident, np.full(n_slots - len(resident), -1, np.int32)])
        resident[rng.random(n_slots) < 0.2] = -1
        before = resident.copy()
        sel = np.sort(rng.permutation(universe)[:k]).astype(np.int32)
        phys = (sel * 7 + 3).astype(np.int32)
        load, slot_of, moved = O.delta_plan(sel, phys, resident)
        kk = min(k, n_slots)
        old, new = set(before[before >= 0].tolist()), set(sel[:kk].tolist())
        assert moved == len(new - old)
        assert set(load[load >= 0].tolist()) == {b * 7 + 3 for b in new - old}
        for j in range(n_slots):
            if before[j] in new:
                assert load[j] == -1 and resident[j] == before[j]       # hit: untouched
            elif load[j] >= 0:
                assert resident[j] in (new - old) and load[j] == resident[j] * 7 + 3
            else:
                assert resident[j] == -1                                 # dropped and not refilled
        assert set(resident[resident >= 0].tolist()) == new
        for i in range(kk):
            assert resident[slot_of[i]] == sel[i]
        # misses fill freed slots in ascending order
        filled = [j for j in range(n_slots) if load[j] >= 0]
        assert [resident[j] for j in filled] == sorted(new - old)


def test_half_conversions_against_numpy():
    """orc_f16_to_f32 over every bit pattern, orc_f32_to_f16 on values around every rounding boundary."""
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    for h in range(65536):
        got = O.f16_to_f32(h)
        assert (np.isnan(got) and np.isnan(want[h])) or got == want[h], h
    rng = np.random.default_rng(5)
    vals = [0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 6.1e-5, 6.0e-5, 2.0 ** -14]
    vals += list(rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32))
    # exact midpoints between neighbouring halves (ties to even) and their float neighbours
    for h in rng.integers(0, 0x7bff, 2000):
        a, b = np.uint16(h).view(np.float16).astype(np.float32), np.uint16(h + 1).view(np.float16).astype(np.float32)
        mid = np.float32((np.float64(a) + np.float64(b)) / 2)
        vals += [mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)), -mid]
    with np.errstate(over="ignore"):
        for v in vals:
            v = np.float32(v)
            assert O.f32_to_f16(float(v)) == int(v.astype(np.float16).view(np.uint16)), v


def _votes_fp64(q, rep):
    """Softmax-vote in float64 straight from its definition."""
    x, hq, d = q.shape
    n, m, hkv, _ = rep.shape
    g = hq // hkv
    keys = rep.astype(np.float64).reshape(n * m, hkv, -1)
    votes = np.zeros(n)
    for t in range(x):
        for head in range(hq):
            s = keys[:, head // g, :] @ q[t, head].astype(np.float64)
            p = np.exp(s - s.max())
            votes += (p / p.sum()).reshape(n, m).sum(1)
    return votes


def test_kvstar_retrieve_closed_forms():
    """No build of the reference pins the KVStar restatement (it needs spdlog); what does: the definition
    evaluated in float64, sum(votes) = rows, invariance under a per-row shift of the scores, the channel
    gather, sub-block means by hand.  The selection step has a test of its own (test_kvstar_heap_tie_rule)."""
    for seed, (x, hq, hkv, d, m, n) in enumerate([(5, 8, 2, 64, 4, 23), (1, 4, 4, 16, 1, 7), (8, 32, 8, 128, 8, 40), (3, 6, 3, 48, 2, 1)]):
        rep = (synth.normal_f32(40 + seed, (n, m, hkv, d)) * np.float32(0.3)).astype(np.float16)
        q = (synth.normal_f32(50 + seed, (x, hq, d)) * np.float32(0.3)).astype(np.float16)
        k = max(n // 3, 1)
        idx, final = O.kvstar_retrieve(q.view(np.uint16), rep.view(np.uint16), k)
        want = _votes_fp64(q, rep)
        assert np.allclose(final, want, rtol=1e-5, atol=1e-6)
        assert abs(final.sum() - x * hq) < 1e-4 * x * hq
        assert sorted(idx) == sorted(np.argsort(-want, kind="stable")[:k]) or np.min(np.diff(np.sort(want))) < 1e-6
        assert list(idx) == sorted(idx, key=lambda i: (final[i], i), reverse=True)
        # a dropped or transposed head mapping would show here: zeroing the keys of one kv head flattens its rows' softmax
        rep0 = rep.copy()
        rep0[:, :, 0, :] = 0
        _, f0 = O.kvstar_retrieve(q.view(np.uint16), rep0.view(np.uint16), k)
        assert np.allclose(f0, _votes_fp64(q, rep0), rtol=1e-5, atol=1e-6)
        # channel gather: scoring pruned keys against the full query equals scoring them against the gathered query
        dp = max(d // 2, 1)
        pr = np.stack([synth.permutation(60 + seed * 8 + h, d)[:dp] for h in range(hkv)]).astype(np.int32)
        rep_p = np.ascontiguousarray(rep[..., :dp])
        _, fp = O.kvstar_retrieve(q.view(np.uint16), rep_p.view(np.uint16), k, pruned=pr)
        g = hq // hkv
        q_g = np.stack([q[:, h, :][:, pr[h // g]] for h in range(hq)], axis=1)
        assert np.allclose(fp, _votes_fp64(q_g, rep_p), rtol=1e-5, atol=1e-6)
        # padded table columns are ignored
        pad = np.zeros((n, m, hkv, dp + 5), np.float16)
        pad[..., :dp] = rep_p
        pad[..., dp:] = 9.0
        _, fpad = O.kvstar_retrieve(q.view(np.uint16), pad.view(np.uint16), k, pruned=pr)
        assert np.array_equal(fpad, fp)


def test_kvstar_block_repre_by_hand():
    bs, hkv, d, merge = 8, 2, 4, 4
    cache = synth.normal_bf16_bits(70, (3, bs, hkv, d))
    out = np.zeros((5, bs // merge, hkv, 16), np.uint16)
    pr = np.array([[2, 0, 3], [1, 3, 0]], np.int32)
    O.kvstar_block_repre(cache, [2, 0], [4, 1], merge, out, pruned=pr)
    wide = synth.bf16_widen(cache)
    for blk, slot in ((2, 4), (0, 1)):
        for m in range(bs // merge):
            for h in range(hkv):
                for p in range(3):
                    acc = np.float32(0)
                    vals = wide[blk, m * merge : (m + 1) * merge, h, pr[h, p]]
                    acc = vals[0]
                    for v in vals[1:]:
                        acc = np.float32(acc + v)
                    acc = np.float32(acc * np.float32(1.0 / merge))
                    b16 = synth.bf16_widen(synth.bf16_round_bits(np.array([acc], np.float32)))[0]
                    assert out[slot, m, h, p] == np.float32(b16).astype(np.float16).view(np.uint16)
                assert not out[slot, m, h, 3:].any()
    assert not out[[0, 2, 3]].any()


def test_kvstar_block_repre_of_fp16_keys_by_hand():
    """A float16 cache: sequential fp32 sums of the widened keys, times 1/merge, rounded once to float16 - numpy's own
    float16 conversions on both ends; merges 4 (the product is exact) and 3 (it is rounded to fp32 first)."""
    for merge, bs in ((4, 8), (3, 12)):
        hkv, d = 2, 4
        rng = np.random.default_rng(71 + merge)
        keys = (rng.standard_normal((3, bs, hkv, d)) * np.array([1.0, 300.0, 1e-4, 30.0])).astype(np.float16)
        out = np.zeros((5, bs // merge, hkv, 16), np.uint16)
        pr = np.array([[2, 0, 3], [1, 3, 0]], np.int32)
        O.kvstar_block_repre(keys.view(np.uint16), [2, 0], [4, 1], merge, out, pruned=pr, keys_f16=True)
        wide = keys.astype(np.float32)
        for blk, slot in ((2, 4), (0, 1)):
            for m in range(bs // merge):
                for h in range(hkv):
                    for p in range(3):
                        vals = wide[blk, m * merge : (m + 1) * merge, h, pr[h, p]]
                        acc = vals[0]
                        for v in vals[1:]:
                            acc = np.float32(acc + v)
                        acc = np.float32(acc * np.float32(1.0 / merge))
                        assert out[slot, m, h, p] == acc.astype(np.float16).view(np.uint16), (merge, blk, m, h, p)
                    assert not out[slot, m, h, 3:].any()
        assert not out[[0, 2, 3]].any()


# ------------------------------------------ helpers the GPU tests use as ground truth

def test_bf16_rounding_against_torch():
    """orc_f32_to_bf16 (and the numpy twin the tests use) against torch's float32 -> bfloat16 conversion, a
    library routine: random values over the whole exponent range, every exact midpoint between neighbouring
    bf16 values with its two float neighbours (ties go to even), zeros, subnormals, overflow to inf, inf, NaN."""
    import torch

    rng = np.random.default_rng(21)
    u = rng.integers(0, 2**32, 200000, dtype=np.uint64).astype(np.uint32)
    hi = rng.integers(0, 2**16, 40000, dtype=np.uint64).astype(np.uint32) << 16
    mids = hi | np.uint32(0x8000)                          # exactly half way between bf16 `hi` and the next one
    special = np.array([0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x007FFFFF, 0x00800000, 0x7F7FFFFF, 0xFF7FFFFF,
                        0x7F7F8000, 0x7F7F7FFF, 0x7F800000, 0xFF800000, 0x7FC00000, 0x7F800001, 0xFFFFFFFF, 0x7FBFFFFF,
                        0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001], np.uint32)
    allu = np.concatenate([u, mids, mids - np.uint32(1), mids + np.uint32(1), special])
    x = allu.view(np.float32)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got_np = O.bf16_bits(x)
    nan = np.isnan(x)
    assert np.array_equal(got_np[~nan], want[~nan])
    assert np.all((want[nan] & 0x7F80) == 0x7F80) and np.all((got_np[nan] & 0x7F80) == 0x7F80) and np.all(got_np[nan] & 0x7F)
    pick = np.concatenate([rng.integers(0, len(u), 3000), np.arange(len(u), len(allu))])
    for i in pick:
        g = O.f32_to_bf16(x[i])
        if nan[i]:
            assert (g & 0x7F80) == 0x7F80 and (g & 0x7F)
        else:
            assert g == want[i], hex(int(allu[i]))
    assert np.array_equal(synth.bf16_round_bits(x[~nan]), want[~nan])     # the generator's own rounding, same rule


def test_block_mean_bf16_rounding_mode():
    """round_bf16=True stores the sequential fp32 mean rounded once to bf16 (what the live torch path keeps,
    gsa.py:640-652): equal, bit for bit, to torch's rounding of the unrounded oracle mean; within one bf16 step of
    the exactly (float64) computed mean rounded once, and equal to it except where the fp32 sum sits at a tie."""
    import torch

    cache = synth.normal_bf16_bits(800, (6, 128, 8, 128))
    ids, slots = [4, 1, 5], [0, 2, 1]
    plain = np.zeros((3, 1024), np.float32)
    rounded = np.zeros((3, 1024), np.float32)
    O.block_mean_paged(cache, ids, slots, plain)
    O.block_mean_paged(cache, ids, slots, rounded, round_bf16=True)
    want = torch.from_numpy(plain).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(bits(rounded), bits(want))
    exact = synth.bf16_widen(cache).astype(np.float64)[ids].mean(axis=1).reshape(3, 1024)[np.argsort(slots)]
    once = torch.from_numpy(exact).to(torch.float32).to(torch.bfloat16).to(torch.float32).numpy()
    step = np.abs(once) * 2.0 ** -7 + 1e-30
    assert np.all(np.abs(rounded - once) <= step)
    assert np.mean(rounded == once) > 0.99


def test_block_mean_of_fp16_keys():
    """The fp16-cache variant: numpy's own float16 -> float32 widening, fp32 adds in token order written out as a loop,
    * (1/T); rounded once to float16 by numpy in the rounding mode.  Also through the C-ABI twin with its key-type flag."""
    import ctypes as C

    rng = np.random.default_rng(801)
    keys = (rng.standard_normal((5, 16, 2, 8)) * 3).astype(np.float16)
    keys[0, 3, 1, 2], keys[1, 0, 0, 0] = np.float16(6.1e-5), np.float16(-65504.0)     # a subnormal-range and the largest value
    cache = keys.view(np.uint16)
    ids, slots = [3, 0, 1], [1, 2, 0]
    plain, rounded = np.zeros((3, 16), np.float32), np.zeros((3, 16), np.float32)
    O.block_mean_paged(cache, ids, slots, plain, keys_f16=True)
    O.block_mean_paged(cache, ids, slots, rounded, round_bf16=True, keys_f16=True)
    for b, s in zip(ids, slots):
        acc = keys[b, 0].astype(np.float32).reshape(-1)
        for t in range(1, 16):
            acc = acc + keys[b, t].astype(np.float32).reshape(-1)
        want = acc * np.float32(1.0 / 16)
        assert np.array_equal(bits(plain[s]), bits(want))
        assert np.array_equal(bits(rounded[s]), bits(want.astype(np.float16).astype(np.float32)))
    # the twin: flag 8 selects the fp16 reading, mode 1 the rounding, mode 2 (a bf16 table) is not offered
    lib = C.CDLL(O._ORC_PATH)
    layers = (C.c_void_p * 1)(cache.ctypes.data)
    ids_a, slots_a = np.array(ids, np.int32), np.array(slots, np.int32)
    for mode, want in ((8, plain), (9, rounded)):
        out = np.zeros((3, 16), np.float32)
        rc = lib.ucm_block_mean_cpu(layers, 1, 5, ids_a.ctypes.data_as(C.c_void_p), slots_a.ctypes.data_as(C.c_void_p), 3, 16, 2, 8,
                                    out.ctypes.data_as(C.c_void_p), 3, C.c_int64(48), mode, None)
        assert rc == 0 and np.array_equal(bits(out), bits(want))
    assert lib.ucm_block_mean_cpu(layers, 1, 5, ids_a.ctypes.data_as(C.c_void_p), slots_a.ctypes.data_as(C.c_void_p), 3, 16, 2, 8,
                                  out.ctypes.data_as(C.c_void_p), 3, C.c_int64(48), 10, None) == -95


def test_hash_colsum_closed_form():
    rng = np.random.default_rng(22)
    for n, t, h, nb in [(3, 128, 8, 16), (2, 7, 1, 3), (1, 1, 2, 1), (4, 64, 4, 16)]:
        tc = rng.integers(0, 256, (n, t, h, nb), dtype=np.uint8)
        ones = np.unpackbits(tc, axis=-1, bitorder="little").astype(np.int64).sum(axis=1)   # [n, h, nb*8]
        assert np.array_equal(O.hash_colsum(tc), (2 * ones - t).astype(np.int16))
    tc = np.zeros((1, 128, 1, 16), np.uint8)
    tc[0, :, 0, 5] = 0x81                                   # bits 40 and 47 set in every token
    cs = O.hash_colsum(tc)[0, 0]
    assert cs[40] == 128 and cs[47] == 128 and cs[41] == -128 and cs.sum() == 2 * 128 - 126 * 128


def _exact_sign_codes(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """Bits of sign(x . W[:, c]) > 0 with the products summed exactly (python integers over a common power of two)."""
    from fractions import Fraction

    n, dim = x.shape
    nbits = w.shape[1]
    wf = [[Fraction(float(w[d, c])) for c in range(nbits)] for d in range(dim)]
    out = np.zeros((n, nbits), np.uint8)
    for i in range(n):
        xf = [Fraction(float(v)) for v in x[i]]
        for c in range(nbits):
            out[i, c] = sum((xf[d] * wf[d][c] for d in range(dim) if xf[d] != 0), Fraction(0)) > 0
    return np.packbits(out, axis=-1, bitorder="little")


def test_hash_encode_128x128_against_exact_sign():
    """Both encoders at the shape every kernel runs (head_dim 128, 128 bits): against the float64 matrix product of
    numpy where the projection is clear of zero, against exactly summed products on rows built to cancel (a
    projection of exactly 0 is NOT positive: the bit is 0), and the LSB-first packing by construction."""
    rng = np.random.default_rng(23)
    dim = nbits = 128
    w = synth.bf16_widen(synth.bf16_round_bits(rng.standard_normal((dim, nbits)).astype(np.float32) * 2))
    xb = synth.normal_bf16_bits(8100, (300, dim))
    x = synth.bf16_widen(xb)
    proj = x.astype(np.float64) @ w.astype(np.float64)
    clear = np.abs(proj) > 1e-9 * (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64))
    assert clear.mean() > 0.999
    want = np.packbits((proj > 0).astype(np.uint8), axis=-1, bitorder="little")
    got_b, got_f = O.hash_encode(xb, w), O.hash_encode_f32(x, w)
    unp = lambda c: np.unpackbits(c, axis=-1, bitorder="little")
    assert np.array_equal(unp(got_b)[clear], unp(want)[clear]) and np.array_equal(unp(got_f)[clear], unp(want)[clear])
    exact = _exact_sign_codes(x[:4], w)
    assert np.array_equal(got_b[:4], exact) and np.array_equal(got_f[:4], exact)
    # cancelling rows: x has two equal entries, column c of W has opposite entries there -> projection exactly 0
    xc = np.zeros((3, dim), np.float32)
    wc = w.copy()
    xc[0, [3, 77]] = 1.5
    wc[3, 10], wc[77, 10] = 0.625, -0.625                   # column 10: exactly zero -> bit 0
    wc[3, 11], wc[77, 11] = 0.625, -0.5                     # column 11: +0.1875 -> bit 1
    wc[3, 12], wc[77, 12] = 0.5, -0.625                     # column 12: negative -> bit 0
    xc[1] = 0                                               # all-zero vector: every bit 0
    xc[2, 127] = -2.0 ** -120                               # tiny negative times column sign
    for enc, arg in ((O.hash_encode, synth.bf16_round_bits(xc)), (O.hash_encode_f32, xc)):
        codes = enc(arg, wc)
        b = unp(codes)
        assert (b[0, 10], b[0, 11], b[0, 12]) == (0, 1, 0)
        assert not codes[1].any()
        assert np.array_equal(b[2], (wc[127] < 0).astype(np.uint8))
        assert np.array_equal(codes, _exact_sign_codes(xc, wc))
    # packing: bit j of byte b is column 8b+j
    one = np.zeros((1, dim), np.float32)
    one[0, 0] = 1.0
    wp = -np.ones((dim, nbits), np.float32)
    wp[0, 8 * 5 + 3] = 1.0
    codes = O.hash_encode_f32(one, wp)[0]
    assert codes[5] == 1 << 3 and codes.sum() == 1 << 3
    # an fp32 input that is not a bf16 value must not be rounded on the way in
    xf = np.zeros((1, dim), np.float32)
    xf[0, 0], xf[0, 1] = np.float32(1 + 2.0 ** -20), -1.0
    w2 = np.zeros((dim, nbits), np.float32)
    w2[0, 0] = w2[1, 0] = 1.0
    assert O.hash_encode_f32(xf, w2)[0, 0] & 1 == 1


def test_kv_gather_selected_placement():
    """orc_kv_gather_selected against the placement rule spelled out with numpy indexing, on a poisoned staging
    buffer: request r's region starts dst_off[r] blocks in and is [layer][K|V][region_k[r]] blocks; only the first
    count[l][r] entries of phys are followed; nothing else is touched."""
    rng = np.random.default_rng(24)
    n_layers, nb, bb, n_req, stride = 3, 13, 32, 4, 6
    layers = [rng.integers(0, 256, 2 * nb * bb, dtype=np.uint8) for _ in range(n_layers)]
    count = rng.integers(0, stride + 1, (n_layers, n_req)).astype(np.int32)
    count[0, 1] = 0
    phys = rng.integers(0, nb, (n_layers, n_req, stride)).astype(np.int32)
    region_k = count.max(axis=0).astype(np.int32) + np.array([0, 2, 0, 1], np.int32)
    order = [2, 0, 3, 1]                                     # regions need not be in request order
    dst_off = np.zeros(n_req, np.int64)
    pos = 1
    for r in order:
        dst_off[r] = pos
        pos += n_layers * 2 * int(region_k[r]) + 1           # a one-block gap after every region
    staging = np.full(pos * bb, 0xA5, np.uint8)
    O.kv_gather_selected(layers, nb * bb, bb, phys, count, dst_off, region_k, staging)
    want = np.full((pos, bb), 0xA5, np.uint8)
    for l in range(n_layers):
        planes = layers[l].reshape(2, nb, bb)
        for r in range(n_req):
            for kv in range(2):
                for j in range(count[l, r]):
                    want[dst_off[r] + (l * 2 + kv) * region_k[r] + j] = planes[kv, phys[l, r, j]]
    assert np.array_equal(staging.reshape(pos, bb), want)
    assert (want == 0xA5).all(axis=1).sum() >= n_req + 1      # the gaps and unused tails stayed poisoned


def test_topk_windows_i32_brute_force():
    rng = np.random.default_rng(25)
    for _ in range(2000):
        n = int(rng.integers(1, 14))
        k = int(rng.integers(0, 16))
        sw, ew = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        sc = rng.integers(-3, 3, n).astype(np.int32) * (1 if rng.random() < 0.5 else 1 << 20)
        got = O.topk_windows(sc, k, sw, ew)
        assert got.dtype == np.int32
        if sw + ew >= n or k >= n or k == 0:
            assert np.array_equal(got, np.arange(n))
            continue
        mid = sorted(range(sw, n - ew), key=lambda i: (-int(sc[i]), i))[: max(k - sw - ew, 0)]
        full = list(range(sw)) + mid + list(range(n - ew, n))
        want = sorted(full[:k]) if k >= sw + ew else full[:k]
        assert list(got) == want, (n, k, sw, ew, sc)
    # scores beyond float32's 24 bits would tie after a conversion; the supported range (|s| < 2^24) does not
    sc = np.array([0, (1 << 24) - 1, (1 << 24) - 2, 5, -(1 << 24) + 1, 0], np.int32)
    assert list(O.topk_windows(sc, 4, 1, 2)) == [0, 1, 4, 5]
    assert list(O.topk_windows(sc, 5, 1, 2)) == [0, 1, 2, 4, 5]


def _heap_topk(scores, k):
    """KVStar's selection (simd_compute_kernel.cpp:955-977) with python's heapq, whose smallest-first order over
    (score, index) tuples is std::priority_queue<pair, vector, greater>'s."""
    import heapq

    heap = []
    for n, s in enumerate(scores):
        if len(heap) < k:
            heapq.heappush(heap, (float(s), n))
        elif heap and s > heap[0][0]:
            heapq.heapreplace(heap, (float(s), n))
    out = [0] * len(heap)
    pos = len(heap) - 1
    while heap:
        out[pos] = heapq.heappop(heap)[1]
        pos -= 1
    return out


def kvstar_heap_closed_form(scores, k):
    """The same selection without a heap (what the device code evaluates): with T the k-th largest score, every
    block above T is kept; ties at T enter while fewer than k blocks >= T have been seen and leave, lowest index
    first, once per block above T that arrives later.  So with P the shortest prefix holding k blocks >= T and
    g_P / g the blocks above T in P / in all, the ties kept are those of P from rank g - g_P on."""
    n = len(scores)
    if k >= n:
        keep = list(range(n))
    else:
        T = sorted(scores, reverse=True)[k - 1]
        seen = g_p = 0
        ties_in_p = []
        for i, s in enumerate(scores):
            if s >= T:
                seen += 1
                if s > T:
                    g_p += 1
                else:
                    ties_in_p.append(i)
                if seen == k:
                    break
        g = sum(1 for s in scores if s > T)
        keep = [i for i, s in enumerate(scores) if s > T] + ties_in_p[g - g_p:]
    return sorted(keep, key=lambda i: (scores[i], i), reverse=True)


def test_kvstar_heap_tie_rule():
    """The worked example: votes [a, b, a, b] with b > a and k = 3.  Blocks 0, 1, 2 fill the heap; block 3 (b) is
    greater than the smallest pair (a, 0) and replaces it; popping smallest-first from the back gives (b,3), (b,1),
    (a,2) -> [3, 1, 2].  (A lowest-index-first sort would give [1, 3, 0]: a different block at the k boundary.)"""
    assert list(O.kvstar_topk(np.array([1, 2, 1, 2], np.float32), 3)) == [3, 1, 2]
    assert list(O.kvstar_topk(np.array([2, 1, 1, 1], np.float32), 2)) == [0, 1]      # equal to the minimum: not replaced
    assert list(O.kvstar_topk(np.array([1, 1, 2, 2], np.float32), 3)) == [3, 2, 1]
    assert list(O.kvstar_topk(np.array([5, 4], np.float32), 7)) == [0, 1]
    rng = np.random.default_rng(26)
    for _ in range(3000):
        n = int(rng.integers(1, 24))
        k = int(rng.integers(1, 26))
        sc = rng.integers(0, 4, n).astype(np.float32)
        want = _heap_topk(sc, k)
        assert list(O.kvstar_topk(sc, k)) == want, (sc, k)
        assert kvstar_heap_closed_form(list(sc), k) == want, (sc, k)
    # through the retrieval entry point: identical blocks get identical votes
    rep = np.zeros((4, 2, 1, 16), np.float16)
    rep[1] = rep[3] = 0.5
    q = np.ones((1, 1, 16), np.float16)
    idx, final = O.kvstar_retrieve(q.view(np.uint16), rep.view(np.uint16), 3)
    assert final[1] == final[3] and final[0] == final[2] and list(idx) == [3, 1, 2]


# ------------------------------------------------ GSA prefetch engine bookkeeping

@needs_ref
def test_ref_prefetch_engine_live():
    """orc_prefetch_run, replayed over whole call sequences, against the reference's own GSAPrefetchEngineC compiled
    from kvcache_pre.cpp: success tables, success lengths, rebuilt free lists, loads, misses and block maps of
    every run, every layer, every request."""
    from golden.make_golden import prefetch_scenario, prefetch_scenarios, run_reference_prefetch
    from prefetch_model import replay, same_result

    gp = O.ref.gsa_prefetch_module()
    if gp is None:
        pytest.skip("gsa_prefetch extension not built")
    cases = prefetch_scenarios() + [(3000 + 31 * i, 1 + i % 3, 1 + i % 4, 4) for i in range(12)]
    served_short = hit_in_free = 0
    for seed, n_layers, n_req, n_runs in cases:
        reqs, runs = prefetch_scenario(seed, n_layers, n_req, n_runs)
        want = run_reference_prefetch(gp, n_layers, reqs, runs)
        got = replay(n_layers, reqs, runs)
        for w, g in zip(want, got):
            same_result(w, g)
            served_short += sum(len(ld) < len(ms) for lr, mr in zip(w["loads"], w["misses"]) for ld, ms in zip(lr, mr))
    assert served_short > 0          # the cases do include selections the free list could not serve


def test_golden_prefetch_engine(golden):
    from golden.make_golden import prefetch_scenario
    from prefetch_model import replay

    z, meta = golden
    assert meta.get("prefetch"), "fixture was written without the prefetch engine"
    flat = lambda x: np.array([v for per_req in x for per_layer in per_req for v in [len(per_layer)] + list(per_layer)], np.int32)
    for seed, n_layers, n_req, n_runs in meta["prefetch"]:
        reqs, runs = prefetch_scenario(seed, n_layers, n_req, n_runs)
        for t, g in enumerate(replay(n_layers, reqs, runs)):
            key = f"prefetch/{seed}/{t}"
            assert np.array_equal(g["success"], z[key + "/success"]) and np.array_equal(g["success_len"], z[key + "/success_len"])
            assert np.array_equal(g["free_len"], z[key + "/free_len"])
            for l in range(n_layers):
                for s in range(g["free"].shape[1]):
                    n = g["free_len"][l, s]
                    assert np.array_equal(g["free"][l, s, :n], z[key + "/free"][l, s, :n])
            assert np.array_equal(flat(g["loads"]), z[key + "/loads"]) and np.array_equal(flat(g["misses"]), z[key + "/misses"])
            maps = np.array([v for rq in reqs for m in g["maps"][rq["req_id"]]
                             for kv in [(len(m), -1)] + sorted(m.items()) for v in kv], np.int32)
            assert np.array_equal(maps, z[key + "/maps"])


def test_prefetch_run_by_hand():
    """A case small enough to follow: cache blocks 50, 60, 70, 80 hold logical blocks 0, 1, 2, 3; the free list names 70
    then 60.  Selecting [3, 9, 1, 8]: 3 and 1 are hits (blocks 80, 60); 9 and 8 miss.  The free list offers 70 (taken
    by 9), then 60 - a hit, passed over - and is then exhausted, so 8 stays unserved.  Success table by logical
    index: 1 -> 60, 3 -> 80, 9 -> 70.  New free list: blocks outside the hit set by id: [50]."""
    idx = np.array([0, 1, 2, 3], np.int32)
    succ, sl, loads, miss, free = O.prefetch_run([50, 60, 70, 80], idx, [3, 9, 1, 8], [70, 60], 2, 6)
    assert loads.tolist() == [70] and miss.tolist() == [9, 8]
    assert succ.tolist() == [60, 80, 70, 0, 0, 0] and sl == 3
    assert free.tolist() == [50] and idx.tolist() == [0, 1, 9, 3]
    with pytest.raises(ValueError):
        O.prefetch_run([50, 60], np.array([0, 1], np.int32), [5], [99], 1, 4)
