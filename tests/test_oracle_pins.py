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
    gather, sub-block means by hand, brute force on a tiny case with a tie."""
    for seed, (x, hq, hkv, d, m, n) in enumerate([(5, 8, 2, 64, 4, 23), (1, 4, 4, 16, 1, 7), (8, 32, 8, 128, 8, 40), (3, 6, 3, 48, 2, 1)]):
        rep = (synth.normal_f32(40 + seed, (n, m, hkv, d)) * np.float32(0.3)).astype(np.float16)
        q = (synth.normal_f32(50 + seed, (x, hq, d)) * np.float32(0.3)).astype(np.float16)
        k = max(n // 3, 1)
        idx, final = O.kvstar_retrieve(q.view(np.uint16), rep.view(np.uint16), k)
        want = _votes_fp64(q, rep)
        assert np.allclose(final, want, rtol=1e-5, atol=1e-6)
        assert abs(final.sum() - x * hq) < 1e-4 * x * hq
        assert list(idx) == list(np.argsort(-want, kind="stable")[:k]) or np.min(np.diff(np.sort(want))) < 1e-6
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
    # ties: identical blocks get identical votes and the lower index comes first
    rep = np.zeros((4, 2, 1, 16), np.float16)
    rep[1] = rep[3] = 0.5
    q = np.ones((1, 1, 16), np.float16)
    idx, final = O.kvstar_retrieve(q.view(np.uint16), rep.view(np.uint16), 3)
    assert final[1] == final[3] and final[0] == final[2] and list(idx) == [1, 3, 0]


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
