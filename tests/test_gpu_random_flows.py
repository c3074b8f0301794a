"""The whole dense path on randomly drawn shapes (seeded, so every run sees the same cases): block means ->
scores -> selection with block tables and sparse lengths -> two resident-set plans -> gather, each stage against
the CPU oracle.  The fixed-shape tests pick their edge cases by hand; this one draws head counts, group sizes, head
dims, block sizes, window sizes, empty and one-block requests, k = 0 and k beyond the request together."""
import math
import types

import numpy as np
import pytest
import torch

import oracle as O
import synth
from test_gpu_kernels import bf16_dev, bits, check_against_oracle, i32, run_select

pytestmark = pytest.mark.gpu


def draw(seed):
    rng = np.random.default_rng(9000 + seed)
    c = dict(hkv=int(rng.choice([1, 2, 4, 8])), g=int(rng.choice([1, 2, 4, 8])), d=int(rng.choice([64, 128])),
             bs=int(rng.choice([4, 16, 32, 128])), n_layers=int(rng.integers(1, 4)), n_req=int(rng.integers(1, 9)),
             sw=int(rng.integers(0, 4)), ew=int(rng.integers(0, 4)), bf16_table=bool(rng.integers(0, 2)),
             bf16_q=bool(rng.integers(0, 2)))
    lens = rng.integers(0, 41, c["n_req"]).astype(np.int32)
    lens[rng.integers(0, c["n_req"])] = rng.choice([0, 1, 2])        # always one degenerate request
    if lens.sum() == 0:
        lens[0] = 7
    topk = np.array([rng.integers(0, n + 4) for n in lens], np.int32)
    topk[rng.integers(0, c["n_req"])] = 0
    c.update(lens=lens, topk=topk, rng=rng)
    return c


@pytest.mark.parametrize("seed", range(32))
def test_random_flow(ucm, dev, seed):
    from ucm_amd import ops

    c = draw(seed)
    rng, lens, topk = c["rng"], c["lens"], c["topk"]
    hkv, d, bs, n_layers, n_req = c["hkv"], c["d"], c["bs"], c["n_layers"], c["n_req"]
    hq, row, rows = hkv * c["g"], hkv * d, int(lens.sum())
    nb = rows + int(rng.integers(1, 9))
    bb = bs * row * 2
    caches_h = [synth.normal_bf16_bits(9100 + 7 * seed + l, (2, nb, bs, hkv, d)) for l in range(n_layers)]
    caches = [bf16_dev(x, dev) for x in caches_h]
    lp = ops.LayerPointers(caches)
    table = rng.permutation(nb)[:rows].astype(np.int32)              # row of the ragged batch -> cache block
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)

    # ---- representatives, in the table's own element type
    dtype = torch.bfloat16 if c["bf16_table"] else torch.float32
    repre = torch.full((n_layers, rows, row), 3.0, dtype=dtype, device=dev)
    ops.block_mean(lp, i32(table, dev), i32(np.arange(rows), dev), repre, bs, hkv, d, nb)
    repre_h = repre.float().cpu().numpy()
    for l in range(n_layers):
        want = np.zeros((rows, row), np.float32)
        O.block_mean_paged(caches_h[l][0], table, np.arange(rows), want, round_bf16=c["bf16_table"])
        assert np.array_equal(bits(repre_h[l]), bits(want)), ("mean", l)

    # ---- scores and selection, with the block-table lookup and the sparse lengths
    q = synth.normal_bf16_as_f32(9200 + seed, (n_layers, n_req, hq, d))
    bt = np.full((n_req, max(int(lens.max()), 1)), -5, np.int32)
    for r, n in enumerate(lens):
        bt[r, :n] = table[off[r] : off[r] + n]
    seq_lens = np.array([max(0, n * bs - int(rng.integers(0, bs))) for n in lens], np.int32)
    out = run_select(ops, dev, q, repre_h, lens, topk, hkv, c["sw"], c["ew"],
                     q_dtype=torch.bfloat16 if c["bf16_q"] else torch.float32, block_tables=bt, seq_lens=seq_lens,
                     block_size=bs, repre_dtype=dtype)
    check_against_oracle(out, q, repre_h, lens, topk, hkv, c["sw"], c["ew"])
    for l in range(n_layers):
        for r, n in enumerate(lens):
            k = out["cnt"][l, r]
            if topk[r] == 0 or n == 0:
                continue
            picked = out["idx"][l, r, :k]
            assert np.array_equal(out["phys"][l, r, :k], bt[r, picked]), ("phys", l, r)
            want_len = seq_lens[r] if k >= n else O.block_table_gather(bt[r], picked, int(seq_lens[r]), bs)[1]
            assert out["sparse_seq_lens"][l, r] == want_len, ("sparse length", l, r)

    # ---- two plans (the second with every request's selection shifted by one block) and the gathers they drive
    stride = out["idx"].shape[2]
    n_slots = max(int(out["cnt"].max()), 1)
    cnt = out["cnt"].copy()
    cnt[:, topk == 0] = 0                                             # no selection was written for k = 0
    resident = torch.full((n_layers, n_req, n_slots), -1, dtype=torch.int32, device=dev)
    res_h = np.full((n_layers, n_req, n_slots), -1, np.int32)
    region = np.full(n_req, n_slots, np.int32)
    dst_off = np.arange(n_req, dtype=np.int64) * n_slots * n_layers * 2
    total = n_req * n_slots * n_layers * 2
    staging = torch.zeros(total * bb, dtype=torch.uint8, device=dev)
    stage_h = np.zeros(total * bb, np.uint8)
    flat = [x.view(np.uint8).reshape(-1) for x in caches_h]
    sel = out["idx"].copy()
    for step in range(2):
        if step == 1:
            for l in range(n_layers):
                for r, n in enumerate(lens):
                    k = cnt[l, r]
                    if k and n > k:                                   # swap the last pick for a block that was not picked
                        sel[l, r, k - 1] = np.setdiff1d(np.arange(n), sel[l, r, :k])[0]
        phys = np.full_like(sel, -1)
        for l in range(n_layers):
            for r in range(n_req):
                phys[l, r, : cnt[l, r]] = bt[r, sel[l, r, : cnt[l, r]]]
        load = torch.full((n_layers, n_req, n_slots), -7, dtype=torch.int32, device=dev)
        slot_of = torch.full((n_layers, n_req, stride), -7, dtype=torch.int32, device=dev)
        miss = torch.full((n_layers, n_req), -7, dtype=torch.int32, device=dev)
        ops.delta_plan(i32(sel, dev), i32(phys, dev), i32(cnt, dev), resident, load, slot_of, miss)
        ops.kv_gather_selected(lp, nb * bb, bb, nb, load, i32(np.full((n_layers, n_req), n_slots), dev),
                               torch.from_numpy(dst_off).to(dev), i32(region, dev), n_slots, staging, total)
        torch.cuda.synchronize()
        load_h = np.empty((n_layers, n_req, n_slots), np.int32)
        for l in range(n_layers):
            for r in range(n_req):
                k = cnt[l, r]
                w_load, w_slot, w_moved = O.delta_plan(sel[l, r, :k], phys[l, r, :k], res_h[l, r])
                load_h[l, r] = w_load
                assert np.array_equal(load[l, r].cpu().numpy(), w_load), ("load", step, l, r)
                assert np.array_equal(slot_of[l, r, :k].cpu().numpy(), w_slot), ("slot", step, l, r)
                assert int(miss[l, r]) == w_moved, ("miss", step, l, r)
        assert np.array_equal(resident.cpu().numpy(), res_h), ("resident", step)
        for l in range(n_layers):                                     # slots whose entry is -1 keep what they hold
            for r in range(n_req):
                for slot in np.nonzero(load_h[l, r] >= 0)[0]:
                    for kv in range(2):
                        src = kv * nb * bb + int(load_h[l, r, slot]) * bb
                        dst = (int(dst_off[r]) + (l * 2 + kv) * n_slots + int(slot)) * bb
                        stage_h[dst : dst + bb] = flat[l][src : src + bb]
        assert np.array_equal(staging.cpu().numpy(), stage_h), ("staging", step)


@pytest.mark.parametrize("seed", range(10))
def test_random_hash_flow(ucm, dev, seed):
    """The hash-code path on drawn shapes: token codes, column sums and majority codes of listed blocks (ids and
    slots that must be skipped among them), query codes through q_rows, both scores (plain and fp16-rounded),
    selection - every stage against the oracle."""
    from ucm_amd import ops
    from test_gpu_hash import make_weights

    rng = np.random.default_rng(9500 + seed)
    hkv = int(rng.choice([1, 2, 4, 8]))
    g = int(rng.choice([1, 2, 4, 8]))
    bs = int(rng.choice([32 // hkv, 64 // hkv * 3, 128, 16 * int(rng.integers(1, 9))]))
    if (bs * hkv) % 32:
        bs = 32
    n_layers, n_req = int(rng.integers(1, 4)), int(rng.integers(1, 7))
    hq = hkv * g
    lens = rng.integers(0, 25, n_req).astype(np.int32)
    lens[rng.integers(0, n_req)] = rng.choice([0, 1])
    if lens.sum() == 0:
        lens[0] = 5
    rows = int(lens.sum())
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    nb = rows + 3
    w_bits, w_f32 = make_weights(9600 + seed)
    keys_h = [synth.normal_bf16_bits(9700 + 5 * seed + l, (nb, bs, hkv, 128)) for l in range(n_layers)]
    for k in keys_h:
        k[0, 0, 0, :] = 0                                              # a vector whose projections are all exactly 0
        k[1, 0, 0, :] = k[1, min(1, bs - 1), 0, :] ^ np.uint16(0x8000)
    lp = ops.LayerPointers([bf16_dev(k, dev) for k in keys_h])
    ids = np.concatenate([rng.permutation(nb)[:rows], [-1, nb]]).astype(np.int32)     # two entries to skip
    slots = np.concatenate([rng.permutation(rows), [0, 1]]).astype(np.int32)
    colsum = torch.full((n_layers, rows, hkv, 128), 77, dtype=torch.int16, device=dev)
    bcodes = torch.full((n_layers, rows, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    tcodes = torch.full((n_layers, rows, bs, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    wd = bf16_dev(w_bits, dev)
    ops.hash_encode_blocks(lp, i32(ids, dev), i32(slots, dev), len(ids), wd, bs, hkv, nb, colsum, bcodes, token_codes=tcodes)
    colsum2, bcodes2 = torch.zeros_like(colsum), torch.zeros_like(bcodes)
    ops.hash_encode_blocks(lp, i32(ids, dev), i32(slots, dev), len(ids), wd, bs, hkv, nb, colsum2, bcodes2)
    torch.cuda.synchronize()
    tc = tcodes.cpu().numpy()
    for l in range(n_layers):
        want = O.hash_encode(keys_h[l][ids[:rows]], w_f32)
        assert np.array_equal(tc[l][slots[:rows]], want), ("token codes", l)
        assert np.array_equal(colsum[l].cpu().numpy()[slots[:rows]], O.hash_colsum(want)), ("column sums", l)
        assert np.array_equal(bcodes[l].cpu().numpy()[slots[:rows]], O.hash_majority(want)), ("block codes", l)
    assert torch.equal(colsum2, colsum) and torch.equal(bcodes2, bcodes)               # the summaries-only variant

    n_tok = n_req + 2
    q_h = synth.normal_bf16_bits(9800 + seed, (n_layers, n_tok, hq, 128))
    q_rows = rng.permutation(n_tok)[:n_req].astype(np.int32)
    q_codes = torch.zeros((n_layers, n_req, hq, 16), dtype=torch.uint8, device=dev)
    q_sum = torch.zeros((n_layers, n_req, 128), dtype=torch.int16, device=dev)
    qbar = torch.zeros((n_layers, n_req, hkv, 16), dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(bf16_dev(q_h, dev), wd, hkv, q_codes, q_sum, qbar, n_req, q_rows=i32(q_rows, dev))
    torch.cuda.synchronize()
    for l in range(n_layers):
        want_q = O.hash_encode(q_h[l][q_rows], w_f32)
        assert np.array_equal(q_codes[l].cpu().numpy(), want_q), ("query codes", l)
        pm = np.unpackbits(want_q, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
        assert np.array_equal(q_sum[l].cpu().numpy(), pm.sum(1)), ("query sums", l)
        qm = np.stack([O.q_head_mean(synth.bf16_widen(q_h[l][r]), hkv) for r in q_rows])
        assert np.array_equal(qbar[l].cpu().numpy(), O.hash_encode_f32(qm, w_f32)), ("mean codes", l)

    sw, ew = int(rng.integers(0, 3)), int(rng.integers(0, 3))
    topk = np.array([rng.integers(0, n + 3) for n in lens], np.int32)
    for mode, rnd in ((ops.HASH_SCORE_SUM, False), (ops.HASH_SCORE_SUM, True), (ops.HASH_SCORE_BLOCK_CODE, False)):
        scores = torch.full((n_layers, rows), -1.0, device=dev)
        ops.hash_score_blocks(mode, q_sum, qbar, colsum, bcodes, i32(off, dev), i32(lens, dev), rows, scores, round_fp16=rnd)
        mx = max(int(lens.max()), 1)
        idx = torch.full((n_layers, n_req, mx), -1, dtype=torch.int32, device=dev)
        cnt = torch.zeros((n_layers, n_req), dtype=torch.int32, device=dev)
        ops.topk_windows(scores, i32(off, dev), i32(lens, dev), i32(topk, dev), mx, idx, cnt, start_w=sw, end_w=ew)
        torch.cuda.synchronize()
        sc = scores.cpu().numpy()
        for l in range(n_layers):
            for r, n in enumerate(lens):
                a = off[r]
                if mode == ops.HASH_SCORE_SUM:
                    key_codes = tc[l][a : a + n].transpose(0, 2, 1, 3)
                    want = O.hash_scores_sum(q_codes[l, r].cpu().numpy(), key_codes).astype(np.float32)
                    if rnd:
                        want = want.astype(np.float16).astype(np.float32)
                else:
                    want = O.hash_scores_block(qbar[l, r].cpu().numpy(), bcodes[l, a : a + n].cpu().numpy()).astype(np.float32)
                assert np.array_equal(sc[l, a : a + n], want), ("scores", mode, rnd, l, r)
                if topk[r] > 0 and n > 0:
                    sel = O.topk_windows(want, int(topk[r]), sw, ew)
                    assert cnt[l, r] == len(sel) and np.array_equal(idx[l, r, : len(sel)].cpu().numpy(), sel), ("selection", mode, l, r)


@pytest.mark.parametrize("seed", range(12))
def test_random_esa_retrieval(ucm, dev, seed):
    """The ESA worker's retrieval on drawn shapes: table dims from 4 to 1024, candidate lists with holes, foreign ids
    and repeated rows, lists shorter and longer than a rank group, k from 0 to beyond the list; the batched call and
    the persistent-table call against the oracle (scores bit for bit, equal scores in list order)."""
    from ucm_amd import ops

    rng = np.random.default_rng(9900 + seed)
    dim = int(rng.choice([4, 64, 128, 1024, 4 * int(rng.integers(1, 90))]))
    n_items = int(rng.integers(1, 400))
    batch = int(rng.integers(1, 7))
    m = int(rng.choice([1, 5, 64, 300, 1025, int(rng.integers(1, 1500))]))
    data = synth.normal_f32(9910 + seed, (n_items, dim))
    if n_items > 3:
        data[1] = data[3]                                              # equal scores
    q = synth.normal_f32(9920 + seed, (batch, dim))
    lists = rng.integers(0, n_items, (batch, m)).astype(np.int32)       # repeats are likely
    lists[rng.random((batch, m)) < 0.2] = -1
    lists[rng.random((batch, m)) < 0.05] = n_items + 3                  # outside the table: skipped
    lists[0, m // 2 :] = -1                                             # a short list in a wide batch
    for topk in (0, int(rng.integers(1, m + 5)), m + 7):
        stride = max(min(topk, m), 1)
        oi = torch.full((batch, stride), -7, dtype=torch.int32, device=dev)
        os_ = torch.full((batch, stride), -7.0, device=dev)
        oc = torch.full((batch,), -7, dtype=torch.int32, device=dev)
        ws = torch.zeros(batch * m, device=dev)
        ops.esa_retrieve(torch.from_numpy(data).to(dev), torch.from_numpy(q).to(dev), i32(lists, dev), topk, ws, oi, os_, oc)
        torch.cuda.synchronize()
        for b in range(batch):
            live = lists[b][(lists[b] >= 0) & (lists[b] < n_items)]
            idx, sc = O.esa_retrieve(data, q[b], live, topk)
            n = int(oc[b])
            assert n == len(idx), (topk, b)
            assert np.array_equal(oi[b, :n].cpu().numpy(), idx), (topk, b)
            assert np.array_equal(bits(os_[b, :n].cpu().numpy()), bits(sc)), (topk, b)
            assert (oi[b, n:] == -7).all(), (topk, b)
    # persistent rows: request b of the call owns row rows[b]; each row has its own k
    table_rows = batch + 2
    table = np.full((table_rows, m + 2), -1, np.int32)
    rows = rng.permutation(table_rows)[:batch].astype(np.int32)
    table[rows, :m] = lists
    topk_rows = rng.integers(0, m + 3, table_rows).astype(np.int32)
    max_topk = int(topk_rows.max())
    stride = max(min(max_topk, m), 1)
    ri = torch.full((table_rows, stride), -7, dtype=torch.int32, device=dev)
    rp, rs = torch.full_like(ri, -7), torch.full((table_rows, stride), -7.0, device=dev)
    rc = torch.full((table_rows,), -7, dtype=torch.int32, device=dev)
    ops.esa_retrieve_rows(torch.from_numpy(data).to(dev), torch.from_numpy(q).to(dev), i32(table, dev), m, i32(rows, dev),
                          i32(topk_rows, dev), max_topk, torch.zeros(batch * m, device=dev), ri, rp, rs, rc)
    torch.cuda.synchronize()
    for b, row in enumerate(rows):
        live = lists[b][(lists[b] >= 0) & (lists[b] < n_items)]
        idx, sc = O.esa_retrieve(data, q[b], live, int(topk_rows[row]))
        n = int(rc[row])
        assert n == len(idx) and np.array_equal(ri[row, :n].cpu().numpy(), idx), ("rows", b)
        assert np.array_equal(bits(rs[row, :n].cpu().numpy()), bits(sc)), ("rows", b)
        pos = rp[row, :n].cpu().numpy()
        assert np.array_equal(lists[b][pos], idx) and len(set(pos.tolist())) == n, ("positions", b)
    others = np.setdiff1d(np.arange(table_rows), rows)
    assert (rc[torch.from_numpy(others).to(dev)] == -7).all()


def kvstar_random_scenario(dev, seed, overrides):
    """Five requests with drawn prompt lengths, arrival steps, prefill chunkings and lifetimes go through the KVStar
    plugin's hooks on stand-in vLLM objects (head counts, stride, merge, sparse ratio and channel pruning drawn too);
    the connector's part (the prompt's blocks stored under their hashes) and the scheduler's (the request shrunk to
    its sparse budget, stale blocks zeroed) happen before a request's first decode step.  Returns, per engine step,
    the requests scheduled and a position-weighted checksum of every layer's cache."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.esa.esa import get_offset
    from ucm_amd.sparse.factory import UcmSparseFactory
    from ucm_amd.store.hip_block_store import UcmHipBlockStore
    from test_gpu_host_layer import make_config

    ns = types.SimpleNamespace
    rng = np.random.default_rng(seed)
    L, d, bs = 3, 128, 16
    hkv = int(rng.choice([2, 4])); hq = hkv * int(rng.choice([2, 4]))
    stride = int(rng.choice([2, 4])); merge = int(rng.choice([2, 4]))
    ratio = float(rng.choice([0.25, 0.5])); prune = float(rng.choice([1.0, 0.5]))
    R = 5
    blocks = rng.integers(6, 41, R); arrive = rng.integers(0, 6, R); chunks = rng.integers(1, 4, R)
    n_decode = rng.integers(stride * 2 + 2, stride * 4 + 4, R)
    nb = int(blocks.sum()) + R + 4
    cfg = make_config(hq, hkv, d, L, bs, 16 * 64, {})
    settings = {"retrieval_stride": stride, "sparse_ratio": ratio, "blk_repre_dim_prune_ratio": prune, "blk_repre_inner_token_merge": merge}
    settings.update(overrides)
    cfg.kv_transfer_config.kv_connector_extra_config = {"ucm_sparse_config": {"KVStarMultiStep": settings}}
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": nb * L * 2 * slice_bytes})
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    plugin.connector = store
    g = torch.Generator(device=dev); g.manual_seed(seed)
    caches = [(torch.randn(2, nb, bs, hkv, d, device=dev, generator=g) * 0.3).to(torch.bfloat16) for _ in range(L)]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    reqs, first = {}, 2
    for r in range(R):
        n_prompt = int(blocks[r]) * bs + int(rng.integers(1, bs))
        ids = list(range(first, first + int(blocks[r]) + 1)); first += int(blocks[r]) + 1
        cuts = sorted(rng.choice(np.arange(1, n_prompt), int(chunks[r]) - 1, replace=False).tolist()) if chunks[r] > 1 else []
        sizes = [b - a for a, b in zip([0] + cuts, cuts + [n_prompt])]
        reqs[str(r)] = ns(block_ids=[ids], num_computed_tokens=0, prompt_token_ids=[int(t) for t in synth.permutation(seed * 10 + r, 100000)[:n_prompt]],
                          output_token_ids=[], num_prompt_tokens=n_prompt, num_output_tokens=0, num_tokens=n_prompt, request_id=str(r),
                          full_ids=ids, sizes=sizes, left=int(n_decode[r]), done=False, stored=False)
    ib = ns(req_id_to_index={str(r): r for r in range(R)})
    digests = []
    weights = None
    t = 0
    while not all(q.done for q in reqs.values()):
        sched = {}
        for r in range(R):
            q = reqs[str(r)]
            if q.done or arrive[r] > t:
                continue
            if q.sizes:
                sched[r] = q.sizes.pop(0)
            else:
                if not q.stored:                       # first decode step: the connector stored the prompt, the scheduler shrank it
                    hashes = plugin.req_states[str(r)][0].block_hashes
                    assert store.create(hashes) == [0] * len(hashes)
                    for l in range(L):
                        for kv in range(2):
                            off = get_offset((bs, hkv, d), 0, 1, 2, l, bool(kv))
                            store.wait(store.dump(hashes, [off] * len(hashes), [caches[l][kv][i] for i in q.full_ids[: len(hashes)]]))
                    store.commit(hashes)
                    q.output_token_ids.append(1); q.num_output_tokens, q.num_tokens = 1, q.num_prompt_tokens + 1
                    q.block_ids = [q.full_ids[-math.ceil(plugin.estimate_num_slots_sparsed(q) / bs):]]
                    for l in range(L):
                        caches[l][:, q.block_ids[0][:-1]] = 0
                    q.stored = True
                else:
                    q.output_token_ids.append(1); q.num_output_tokens += 1; q.num_tokens += 1
                sched[r] = 1
        if sched:
            so = ns(num_scheduled_tokens={str(r): n for r, n in sched.items()}, req_sparsed_slots={str(r): 0 for r in sched})
            starts = [0] * (R + 1)
            for r in range(R):
                starts[r + 1] = starts[r] + sched.get(r, 0)
            md = ns(query_start_loc=torch.tensor(starts))
            fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=md)
            qt = (torch.randn(starts[-1], hq, d, device=dev, generator=g) * 0.3).to(torch.bfloat16)
            plugin.build_sparse_meta(so, reqs, ib, md)
            for l in range(L):
                plugin.attention_begin(qt, None, None, names[l], fc)
                plugin.attention_finished(qt, None, None, None, names[l], fc)
            for r, n in sched.items():
                q = reqs[str(r)]
                q.num_computed_tokens += n
                if q.stored:
                    q.left -= 1
                    if q.left == 0:
                        for st in plugin.req_states[str(r)]:
                            if st is not None: st.wait_for_blk_transfer_task_done()
                        plugin.request_finished_in_worker(str(r)); q.done = True
            for rr, states in plugin.req_states.items():
                for st in states:
                    if st is not None: st.wait_for_blk_transfer_task_done()
            torch.cuda.synchronize()
            row = []
            for c in caches:
                flat = c.view(torch.int16).reshape(-1).to(torch.int64)
                if weights is None or weights.numel() != flat.numel():
                    weights = torch.arange(flat.numel(), device=dev) % 65521 + 1
                row.append(int((flat * weights).sum()))
            digests.append((t, tuple(sorted(sched)), tuple(row)))
        t += 1
    return digests, (hkv, hq, stride, merge, ratio, prune, blocks.tolist(), arrive.tolist(), chunks.tolist(), n_decode.tolist())


@pytest.mark.parametrize("seed", range(8))
def test_random_kvstar_plugin_flow(ucm, dev, seed):
    """The three ways the KVStar plugin loads what a retrieval chose - a kernel following the list on the device, one
    pointer-array copy per layer from the lists read back, one store.load per request and K|V - behind the same
    batched retrievals: the same bytes in every cache after every engine step, and no retrieval task left behind."""
    from ucm_amd.sparse.kvstar import retrieve as kvstar_retrieve

    before = len(kvstar_retrieve._tasks)
    planned, drawn = kvstar_random_scenario(dev, seed, {})
    by_request, _ = kvstar_random_scenario(dev, seed, {"device_loads": False, "device_plans": False})
    from_lists, _ = kvstar_random_scenario(dev, seed, {"device_plans": False})
    assert len(planned) == len(by_request) == len(from_lists) > 0
    for a, b, c in zip(planned, by_request, from_lists):
        assert a == b == c, (drawn, a[:2])
    assert len(kvstar_retrieve._tasks) == before
