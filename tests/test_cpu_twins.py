"""The oracle's `_cpu` twins of the C ABI (oracle/ucm_cpu_abi.c): same prototypes as the device entry points, host
pointers.  Here, without a GPU: they load with the device binding's argument types and reproduce the oracle's own
functions on a scripted pass; with a GPU (tests/test_gpu_kernels.py) the same pass through libucm_hip.so gives the
same bytes."""
import numpy as np

import cpu_twins
import oracle as O


def test_twins_reproduce_the_oracle(ucm):
    from ucm_amd import _lib

    got, x = cpu_twins.run(cpu_twins.twin_caller(_lib.SIGNATURES), cpu_twins.HostSide())
    L, ROWS, ROW, HKV = cpu_twins.L, cpu_twins.ROWS, cpu_twins.ROW, cpu_twins.HKV
    ids, slots = x["ids"][:ROWS], x["slots"][:ROWS]            # the two out-of-range ids behind them are skipped
    for l in range(L):
        for mode, rounded in ((0, False), (1, True)):
            want = np.full((ROWS, ROW), 7, np.float32)
            O.block_mean_paged(x["caches"][l][0], ids, slots, want, round_bf16=rounded)
            assert np.array_equal(got[f"repre{mode}"][l].view(np.uint32), want.view(np.uint32))
        assert np.array_equal(got["repre2"][l], O.bf16_bits(got["repre1"][l]))
        want = np.full((ROWS, ROW), 7, np.float32)
        O.block_mean_paged(x["caches"][l][0] & np.uint16(0x7fff), ids, slots, want)
        assert np.array_equal(got["repre4"][l].view(np.uint32), want.view(np.uint32))
    # scores and selection, per request, against the oracle's batch call
    table16 = O.bf16_to_f32(got["repre2"])
    for l in range(L):
        q = O.bf16_to_f32(x["q16"][l][x["q_rows"]])
        idx, cnt, scores = O.select_topk_bs(q, table16[l], cpu_twins.OFF, cpu_twins.LENS, x["topk"], HKV, start_w=1, end_w=1,
                                            out_stride=6)
        for r, (a, n) in enumerate(zip(cpu_twins.OFF, cpu_twins.LENS)):
            assert np.array_equal(got["scores16"][l, a : a + n], scores[a : a + n] * np.float32(0.5))
            assert got["cnt"][l, r] == cnt[r] and np.array_equal(got["idx"][l, r, : cnt[r]], idx[r, : cnt[r]])
            assert np.array_equal(got["phys"][l, r, : cnt[r]], x["tables"][r][idx[r, : cnt[r]]])
            if n:
                assert got["sparse"][l, r] == (x["seq_lens"][r] if cnt[r] >= n else
                                                O.block_table_gather(x["tables"][r], idx[r, : cnt[r]], int(x["seq_lens"][r]),
                                                                     cpu_twins.BS)[1])
    # the one-launch entry point gives what the two calls gave, and leaves its tickets at zero
    assert np.array_equal(got["f_scores"].view(np.uint32), got["scores16"].view(np.uint32))
    for a, b in (("f_idx", "idx"), ("f_phys", "phys"), ("f_cnt", "cnt"), ("f_sparse", "sparse")):
        assert np.array_equal(got[a][:, :3], got[b]) and (got[a][:, 3] == -1).all(), a      # the fourth request's row is not this batch's
    assert not got["tickets"].any()
    # the first plan fills empty slots in order; the moves restore exactly the listed blocks
    assert np.array_equal(got["resident1"][:, 0, :3], got["idx"][:, 0, :3]) and (got["resident1"][:, 1] == -1).all()
    assert np.array_equal(got["miss1"], got["cnt"])
    for l in range(L):
        want = np.zeros_like(x["caches"][l])
        for b in (5, 0, 11):
            want[:, b] = x["caches"][l][:, b]
        assert np.array_equal(got[f"restored{l}"], want)
        assert np.array_equal(got[f"restored_tp{l}"], want)
    # one rank of three that share the stored block: its slices sit where get_offset says, the others' bytes stay
    wide = got["moved_tp"]                               # [4 blocks][layer][rank][K|V][bytes]
    flat = wide.reshape(4, -1)
    assert (wide[:, :, [0, 2]] == 0xEE).all() and (wide[1] == 0xEE).all()
    for i, b in ((0, 5), (2, 0), (3, 11)):
        for l in range(L):
            for kv in (0, 1):
                at = O.get_offset((1, 1, cpu_twins.BLOCK_BYTES), 1, 3, 1, l, bool(kv))
                want = x["caches"][l][kv, b].reshape(-1).view(np.uint8)
                assert np.array_equal(flat[i, at : at + cpu_twins.BLOCK_BYTES], want), (i, l, kv)


def test_descriptors_outside_the_tables_are_not_followed(ucm):
    """seg_off / seg_len live in device memory: a request whose rows do not lie inside the table the call names is
    skipped by the scores (its scores, and the padding around the table, keep what they held) and selects nothing."""
    from ucm_amd import _lib

    got, x = cpu_twins.run_bounds(cpu_twins.twin_caller(_lib.SIGNATURES), cpu_twins.HostSide())
    pad, rows = x["pad"], cpu_twins.ROWS
    for key in ("scores", "f_scores"):
        sc = got[key]
        assert (sc[:, :pad + 1] == -3).all() and (sc[:, pad + 5:] == -3).all(), key        # only rows 1..4 were written
        for l in range(cpu_twins.L):
            _, _, want = O.select_topk_bs(x["q32"][l][:1], x["repre"][l][pad + 1 : pad + 5], np.array([0], np.int32),
                                          np.array([4], np.int32), np.array([2], np.int32), cpu_twins.HKV, start_w=0, end_w=0)
            assert np.array_equal(sc[l, pad + 1 : pad + 5].view(np.uint32), want[:4].view(np.uint32)), (key, l)
    for ck, ik in (("cnt", "idx"), ("f_cnt", "f_idx")):
        assert (got[ck][:, 0] == 2).all() and (got[ck][:, 1:] == 0).all(), ck
        assert (got[ik][:, 1:] == -1).all(), ik
    assert np.array_equal(got["idx"], got["f_idx"]) and not got["tickets"].any()


def test_hash_twins_reproduce_the_oracle(ucm):
    from ucm_amd import _lib

    got, x = cpu_twins.run_hash(cpu_twins.twin_caller(_lib.SIGNATURES), cpu_twins.HostSide())
    w = O.bf16_to_f32(x["w"])
    live = [i for i, b in enumerate(x["ids"]) if 0 <= b < cpu_twins.HNB]
    # a slot named twice keeps the later block (the calls are serial on the host)
    final = {int(x["slots"][i]): int(x["ids"][i]) for i in live}
    for l in range(cpu_twins.HL):
        for slot, blk in final.items():
            codes = O.hash_encode(x["keys"][l][blk], w)                      # [tokens, kv heads, 16]
            assert np.array_equal(got["token_codes"][l, slot], codes)
            assert np.array_equal(got["colsum"][l, slot], O.hash_colsum(codes[None])[0])
            assert np.array_equal(got["block_codes"][l, slot], O.hash_majority(codes[None])[0])
        for r, row in enumerate(x["q_rows"]):
            qc = O.hash_encode(x["q"][l, row], w)
            assert np.array_equal(got["q_codes"][l, r], qc)
            for a, n in ((cpu_twins.H_OFF[r], cpu_twins.H_LENS[r]),):
                if n:
                    keys = np.ascontiguousarray(got["token_codes"][l, a : a + n].transpose(0, 2, 1, 3))   # [block, head, token, 16]
                    assert np.array_equal(got["score_sum"][l, a : a + n], O.hash_scores_sum(qc, keys).astype(np.float32))
                    assert np.array_equal(got["score_code"][l, a : a + n],
                                          O.hash_scores_block(got["qbar"][l, r], got["block_codes"][l, a : a + n]).astype(np.float32))
    assert np.array_equal(got["score_sum_fp16"], got["score_sum"].astype(np.float16).astype(np.float32))
    # requests outside the declared rows were not scored; the empty one in between has nothing to score either way
    assert (got["score_sum_bad"] == -3).all() and (got["score_code_bad"] == -3).all()
    # the float16 entry points: the signs of numpy's own float64 products of the widened values, summed in order
    w16 = x["w16"].astype(np.float64)
    for l in range(cpu_twins.HL):
        for slot, blk in final.items():
            k = x["keys16"][l][blk].astype(np.float64)                          # [tokens, kv heads, 128]
            acc = np.zeros(k.shape[:2] + (128,))
            for d_ in range(cpu_twins.HD):
                acc += k[..., d_, None] * w16[d_]
            codes = np.packbits(acc > 0, axis=-1, bitorder="little")
            assert np.array_equal(got["token_codes_f16"][l, slot], codes)
            assert np.array_equal(got["colsum_f16"][l, slot], O.hash_colsum(codes[None])[0])
            assert np.array_equal(got["block_codes_f16"][l, slot], O.hash_majority(codes[None])[0])
        for r, row in enumerate(x["q_rows"]):
            qv = x["q16"][l, row].astype(np.float64)
            acc = np.zeros((qv.shape[0], 128))
            for d_ in range(cpu_twins.HD):
                acc += qv[:, d_, None] * w16[d_]
            qc = np.packbits(acc > 0, axis=-1, bitorder="little")
            assert np.array_equal(got["q_codes_f16"][l, r], qc)
            assert np.array_equal(got["qbar_f16"][l, r], qc)                    # one head per kv head: the mean is the row
            assert np.array_equal(got["q_sum_f16"][l, r], (np.unpackbits(qc, axis=-1, bitorder="little").astype(np.int32) * 2 - 1).sum(0))
            # all heads around one kv head: the fp32 mean in head order, then its exact signs
            q32 = x["q16"][l, row].astype(np.float32)
            mean = q32[0]
            for h in range(1, q32.shape[0]):
                mean = mean + q32[h]
            mean = mean * (np.float32(1.0) / np.float32(q32.shape[0]))
            accm = np.zeros(128)
            for d_ in range(cpu_twins.HD):
                accm += np.float64(mean[d_]) * w16[d_]
            assert np.array_equal(got["qbar_f16_grouped"][l, r, 0], np.packbits(accm > 0, bitorder="little"))
            assert np.array_equal(got["q_codes_f16_grouped"][l, r], qc)
            assert np.array_equal(got["q_sum_f16_grouped"][l, r], got["q_sum_f16"][l, r])


def test_esa_twins_reproduce_the_oracle(ucm):
    from ucm_amd import _lib

    got, x = cpu_twins.run_esa(cpu_twins.twin_caller(_lib.SIGNATURES), cpu_twins.HostSide())
    n_items = cpu_twins.E_ITEMS
    for topk in (4, 0, 20):
        for b in range(3):
            live = x["lists"][b][(x["lists"][b] >= 0) & (x["lists"][b] < n_items)]      # holes and foreign ids are skipped
            idx, sc = O.esa_retrieve(x["data"], x["q"][b], live, topk)
            n = got[f"count{topk}"][b]
            assert n == len(idx) == min(len(live), topk)
            assert np.array_equal(got[f"idx{topk}"][b, :n], idx)
            assert np.array_equal(got[f"scores{topk}"][b, :n].view(np.uint32), sc.view(np.uint32))
            assert (got[f"idx{topk}"][b, n:] == -7).all()
    # worked by hand: rows 11 (+0) and 12 (-0) tie at 0 and come in list order; the duplicate of row 3 follows row 3
    order = got["idx20"][0, :7].tolist()
    assert order.index(11) + 1 == order.index(12) and order.index(3) + 1 == order.index(7)
    # the table variant: request b -> row rows[b], its own k, positions within the slot list
    for b, row in enumerate(x["rows"][:3]):
        k = min(5, int(x["topk_rows"][row]))
        lst = x["table"][row, : cpu_twins.E_M]
        live = lst[(lst >= 0) & (lst < n_items)]
        idx, sc = O.esa_retrieve(x["data"], x["q"][b], live, k)
        n = got["rows_count"][row]
        assert n == len(idx) and np.array_equal(got["rows_idx"][row, :n], idx)
        assert np.array_equal(lst[got["rows_pos"][row, :n]], idx)
    assert (got["rows_count"][[1, 3]] == -7).all()                     # rows no request of the call owns
    # plans: first step loads every winner; second step loads exactly the one replaced, into the slot it freed
    for l in range(cpu_twins.E_L):
        for row in (4, 0, 2):
            n = got["rows_count"][row]
            assert got["miss1"][l, row] == n and sorted(got["resident1"][l, row, :n]) == sorted(got["rows_pos"][row, :n])
            assert got["miss2"][l, row] == 1 and (got["load2"][l, row] >= 0).sum() == 1
            slot = int(np.argmax(got["load2"][l, row] >= 0))
            assert got["resident2"][l, row, slot] == got["load2"][l, row, slot]
            assert got["resident1"][l, row, slot] not in got["resident2"][l, row]


def test_selection_prefetch_and_load_twins_reproduce_the_oracle(ucm):
    from ucm_amd import _lib

    got, x = cpu_twins.run_more(cpu_twins.twin_caller(_lib.SIGNATURES), cpu_twins.HostSide())
    # KVStar's selection: the oracle's literal heap gives the order, its sorted copy the ascending list
    for t, (a, n, k) in enumerate(zip(x["off"], x["lens"], x["ks"])):
        if n == 0:
            assert got["chosen_count"][t] == 0
            continue
        want = O.kvstar_topk(x["votes"][a : a + n], int(k))
        assert got["chosen_count"][t] == len(want)
        assert got["chosen"][t, : len(want)].tolist() == sorted(want.tolist())
        assert got["ordered"][t, : len(want)].tolist() == want.tolist()
        assert (got["ordered"][t, len(want):] == -1).all()
    # with the votes declared shorter and a task starting below them: those two select nothing, the others as before
    assert got["chosen_count_bad"][0] == 0 and got["chosen_count_bad"][3] == 0
    assert (got["ordered_bad"][[0, 3]] == -1).all()
    for t in (1, 2, 4):
        assert got["chosen_count_bad"][t] == got["chosen_count"][t] and np.array_equal(got["ordered_bad"][t], got["ordered"][t])
    assert np.array_equal(got["copied"], np.concatenate([np.arange(64), np.arange(128, 192), np.arange(64, 128)]).astype(np.uint8))
    # the prefetch round, request by request and layer by layer, against the oracle's single run
    P = cpu_twins
    want_cache = [np.zeros((2, P.P_NB, P.P_BLOCK_BYTES), np.uint8) for _ in range(P.P_L)]
    for l in range(P.P_L):
        for i in (0, 1):
            r, b = int(x["rows"][i]), int(x["bs_index"][i])
            n = int(x["map_len"][r])
            m_idx = x["map_idx"][l, r, :n].copy()
            succ, succ_len, loads, miss, free = O.prefetch_run(x["map_block"][r, :n], m_idx, x["topk_idx"][l, i, : x["topk_len"][i]],
                                                              x["free_block"][l, b, : x["free_len"][l, b]], int(x["free_len"][l, b]),
                                                              P.P_ROW_LEN)
            assert np.array_equal(got["map_idx"][l, r, :n], m_idx)
            assert np.array_equal(got["success"][l, b], succ) and got["success_len"][l, b] == succ_len
            assert got["load_count"][l, r] == len(loads) and np.array_equal(got["load_blocks"][l, r, : len(loads)], loads)
            assert got["miss_count"][l, r] == len(miss) and np.array_equal(got["miss_idxs"][l, r, : len(miss)], miss)
            assert got["free_len"][l, b] == len(free) and np.array_equal(got["free_block"][l, b, : len(free)], free)
            for j, blk in enumerate(loads):                        # the planned loads, placed by hand
                stored = x["src_table"][r, miss[j]]
                if stored >= 0:
                    want_cache[l][:, blk] = x["pool"][stored, l]
        # rows no request of the call reached keep what they held; a request that selects nothing reports zero loads
        assert got["load_count"][l, 1] == 0 and got["miss_count"][l, 1] == 0
        assert np.array_equal(got["map_idx"][l, 1], x["map_idx"][l, 1])
        assert (got["success"][l, [1, 2]] == -5).all()
        assert np.array_equal(got[f"cache{l}"], want_cache[l])
        assert np.array_equal(got[f"cache_tp{l}"], want_cache[l])      # the same blocks out of rank 1's slices of wider stored blocks
    assert any(c.any() for c in want_cache)


def test_kvstar_twins_reproduce_the_oracle(ucm):
    from ucm_amd import _lib

    got, x = cpu_twins.run_kvstar(cpu_twins.twin_caller(_lib.SIGNATURES), cpu_twins.HostSide())
    K = cpu_twins
    live = [(int(b), int(s)) for b, s in zip(x["ids"], x["slots"]) if 0 <= b < K.K_NB]
    final = dict((s, b) for b, s in live)                              # a slot named twice keeps the later block
    for name, d_pad in (("full", K.K_D), ("pruned", K.K_DPAD)):
        # cells [d_pad/8][M][8] of (layer, head, row) back into the reference's [row][M][head][d]
        cells = got["table_" + name].reshape(K.K_L, K.K_HKV, K.K_ROWS, d_pad // 8, K.K_M, 8)
        ref = cells.transpose(0, 2, 4, 1, 3, 5).reshape(K.K_L, K.K_ROWS, K.K_M, K.K_HKV, d_pad)
        for l in range(K.K_L):
            want = np.full((K.K_ROWS, K.K_M, K.K_HKV, d_pad), 0x3c00, np.uint16)
            O.kvstar_block_repre(x["caches"][l], np.array(list(final.values()), np.int32), np.array(list(final.keys()), np.int32),
                                 K.K_MERGE, want, pruned=None if name == "full" else x["lists"][l])
            assert np.array_equal(ref[l], want), (name, l)
            if name == "pruned":
                assert (ref[l][..., K.K_DP:] == 0).all() and (ref[l][..., : K.K_DP] != 0).any()
    assert set(final) == set(range(K.K_ROWS))
    # a list per listed block: every block against the oracle run with the list it names; the one that names no list is skipped
    cells = got["table_by_block"].reshape(K.K_L, K.K_HKV, K.K_ROWS, K.K_DPAD // 8, K.K_M, 8)
    by_block = cells.transpose(0, 2, 4, 1, 3, 5).reshape(K.K_L, K.K_ROWS, K.K_M, K.K_HKV, K.K_DPAD)
    last = {}
    for i, (b, s_) in enumerate(zip(x["ids"], x["slots"])):
        if 0 <= b < K.K_NB and x["list_sel"][i] < K.K_L:
            last[int(s_)] = (int(b), int(x["list_sel"][i]))
    for l in range(K.K_L):
        want = np.full((K.K_ROWS, K.K_M, K.K_HKV, K.K_DPAD), 0x3c00, np.uint16)
        for slot, (b, which) in last.items():
            O.kvstar_block_repre(x["caches"][l], np.array([b], np.int32), np.array([slot], np.int32), K.K_MERGE, want,
                                 pruned=x["lists"][which])
        assert np.array_equal(by_block[l], want), l
    for key in ("votes", "votes_tables"):
        for t, (a, n) in enumerate(zip(K.K_OFF, K.K_LEN)):
            if n:
                _, want = O.kvstar_retrieve(x["q"][t], np.ascontiguousarray(ref[0][a : a + n]), 1, pruned=x["lists"][0])
                assert np.array_equal(got[key][a : a + n].view(np.uint32), want.view(np.uint32)), (key, t)
                assert abs(float(want.sum()) - K.K_X * K.K_HKV * K.K_G) < 1e-3          # every query row votes with weight one
    assert np.array_equal(got["votes"], got["votes_tables"])
    # parked query tokens: numpy's own float32 -> float16 conversion (round to nearest even, overflow to inf); the row
    # past the queries and the place past the ring change nothing
    qf = x["park_q"]
    want = np.full((6, qf.shape[1]), 0x3c00, np.uint16)
    with np.errstate(over="ignore"):
        for s_, d_ in ((5, 0), (0, 2), (3, 1), (1, 4)):
            want[d_] = qf[s_].astype(np.float16).view(np.uint16)
        assert np.array_equal(got["park_f32"], want), np.argwhere(got["park_f32"] != want)[:4]
        want16 = want.copy()
        for s_, d_ in ((5, 0), (0, 2), (3, 1), (1, 4)):
            want16[d_] = O.bf16_to_f32(O.bf16_bits(qf[s_])).astype(np.float16).view(np.uint16)
        assert np.array_equal(got["park_bf16"], want16)
        assert np.array_equal(got["park_f16"][[0, 2, 1, 4]], qf[[5, 0, 3, 1]].astype(np.float16).view(np.uint16))
    # rows moved by index: pairs (6 -> 1), (0 -> 4), (3 -> 5) land, the rest name a row outside an array
    src_rows = np.arange(7 * 48, dtype=np.int32).reshape(7, 48)
    want_rows = np.full((6, 48), -5, np.int32)
    want_rows[[1, 4, 5]] = src_rows[[6, 0, 3]]
    assert np.array_equal(got["rows_indexed"], want_rows)
    want_rows = np.full((6, 48), -5, np.int32)
    want_rows[[0, 1, 3, 5]] = src_rows[[6, 0, 3, 2]]
    assert np.array_equal(got["rows_in_order"], want_rows)
    # a task whose query block, channel list or rows lie outside what the call declares is skipped: its votes keep
    # the fill value, the other tasks' are unchanged
    a0, n0, a2, n2 = K.K_OFF[0], K.K_LEN[0], K.K_OFF[2], K.K_LEN[2]
    assert (got["votes_bad0"][a2 : a2 + n2] == -3).all() and np.array_equal(got["votes_bad0"][a0 : a0 + n0], got["votes"][a0 : a0 + n0])
    assert (got["votes_bad1"][a0 : a0 + n0] == -3).all() and np.array_equal(got["votes_bad1"][a2 : a2 + n2], got["votes"][a2 : a2 + n2])
    assert (got["votes_bad2"][a2 : a2 + n2] == -3).all() and np.array_equal(got["votes_bad2"][a0 : a0 + n0], got["votes"][a0 : a0 + n0])

