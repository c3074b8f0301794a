"""The benchmark definition's configurations 2 (the one the metric is quoted on) and 5 at their full sizes, every
result compared with the CPU oracle: scores bit for bit, selected indices, block-table lookup, every gathered byte,
two delta steps against orc_delta_plan; hash codes of a sampled block per (layer, request), all column sums, block
codes, both integer scores and the selection in whole layers."""
import numpy as np
import pytest
import torch

import oracle as O
import synth

pytestmark = pytest.mark.gpu

bits = lambda a: np.ascontiguousarray(a, np.float32).view(np.uint32)


def i32(x, dev):
    return torch.tensor(np.asarray(x), dtype=torch.int32, device=dev)


def test_config2_full_size_retrieval_gather_and_delta(ucm, dev):
    """16 requests of 32..512 blocks (4096..65536 tokens), Llama-3-8B shape, 32 layers, a bf16 paged cache of about
    70 GB addressed through a random block table, k = max(16, 3 %) + 1 first + 2 last blocks."""
    from ucm_amd import ops

    n_req, n_layers, hq, hkv, d, bs = 16, 32, 32, 8, 128, 128
    row, block_bytes = hkv * d, bs * hkv * d * 2
    lens = synth.ragged_lengths(2020, n_req, 4096, 65536)
    topk = np.array([max(16, int(0.03 * n)) + 3 for n in lens], np.int32)
    rows = nb = int(lens.sum())
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    table_h = synth.permutation(2021, nb)
    max_len, max_k = int(lens.max()), int(topk.max())
    gen = torch.Generator(device=dev)
    gen.manual_seed(2022)
    caches = [torch.empty((2, nb, bs, hkv, d), dtype=torch.bfloat16, device=dev).normal_(generator=gen) for _ in range(n_layers)]
    layers = ops.LayerPointers(caches)
    bt_h = np.zeros((n_req, max_len), np.int32)
    for r in range(n_req):
        bt_h[r, : lens[r]] = table_h[off[r] : off[r] + lens[r]]
    seg_off, seg_len, topk_d, bt = i32(off, dev), i32(lens, dev), i32(topk, dev), i32(bt_h, dev)
    repre = torch.zeros(n_layers, rows, row, dtype=torch.bfloat16, device=dev)
    ops.block_mean(layers, i32(table_h, dev), torch.arange(rows, dtype=torch.int32, device=dev), repre, bs, hkv, d, nb)
    scores = torch.zeros(n_layers, rows, device=dev)
    idx = torch.full((n_layers, n_req, max_len), -1, dtype=torch.int32, device=dev)
    phys = torch.full_like(idx, -1)
    cnt = torch.zeros(n_layers, n_req, dtype=torch.int32, device=dev)
    region_h = topk.copy()
    dst_off_h = np.concatenate([[0], np.cumsum(region_h.astype(np.int64) * n_layers * 2)[:-1]]).astype(np.int64)
    total_blocks = int((region_h.astype(np.int64) * n_layers * 2).sum())
    staging = torch.zeros(total_blocks * block_bytes, dtype=torch.uint8, device=dev)
    kv_stride = nb * block_bytes
    st = staging.view(torch.bfloat16).view(-1, bs, hkv, d)

    def retrieve(q):
        ops.score_blocks(q, repre, seg_off, seg_len, max_len, hkv, scores, total_blocks=rows)
        ops.topk_windows(scores, seg_off, seg_len, topk_d, max_len, idx, cnt, block_tables=bt, phys_out=phys)

    # ---- one full step: score, select, gather
    q = torch.empty((n_layers, n_req, hq, d), dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    retrieve(q)
    ops.kv_gather_selected(layers, kv_stride, block_bytes, nb, phys, cnt, torch.from_numpy(dst_off_h).to(dev), i32(region_h, dev),
                           max_k, staging, total_blocks)
    torch.cuda.synchronize()
    q_h = q.float().cpu().numpy()
    sc_h, idx_h, cnt_h, phys_h = scores.cpu().numpy(), idx.cpu().numpy(), cnt.cpu().numpy(), phys.cpu().numpy()
    # a sampled block mean against the oracle, rounded to the table's dtype (all of them are covered at smaller sizes)
    kc0 = caches[0][0][int(table_h[7])].view(torch.int16).cpu().numpy().view(np.uint16)[None]
    want_rep = np.zeros((1, row), np.float32)
    O.block_mean_paged(kc0, [0], [0], want_rep, round_bf16=True)
    assert np.array_equal(bits(repre[0, 7].float().cpu().numpy()), bits(want_rep[0]))
    for l in range(n_layers):
        rep = repre[l].float().cpu().numpy()
        widx, wcnt, wsc = O.select_topk_bs(q_h[l], rep, off, lens, topk, hkv, out_stride=max_len + 4)
        assert np.array_equal(bits(wsc), bits(sc_h[l])), f"scores differ in layer {l}"
        assert np.array_equal(wcnt, cnt_h[l]) and np.array_equal(wcnt, topk)
        for r in range(n_req):
            assert np.array_equal(widx[r, : wcnt[r]], idx_h[l, r, : wcnt[r]]), (l, r)
            assert np.array_equal(phys_h[l, r, : wcnt[r]], bt_h[r][widx[r, : wcnt[r]]]), (l, r)
    for l in range(n_layers):
        for r in range(n_req):
            k = int(topk[r])
            sel = phys[l, r, :k].long()
            for kv in range(2):
                o = int(dst_off_h[r]) + (l * 2 + kv) * k
                assert torch.equal(st[o : o + k], caches[l][kv][sel]), (l, r, kv)

    # ---- two delta steps: staging slots keep their blocks, only the missing ones move
    n_slots = max_k
    resident = torch.full((n_layers, n_req, n_slots), -1, dtype=torch.int32, device=dev)
    load_phys = torch.empty_like(resident)
    slot_of = torch.full_like(idx, -1)
    miss = torch.zeros_like(cnt)
    slots_count = torch.full_like(cnt, n_slots)
    d_total = int(n_req * n_slots * n_layers * 2)
    d_off = torch.arange(n_req, dtype=torch.int64, device=dev) * (n_slots * n_layers * 2)
    d_region = torch.full((n_req,), n_slots, dtype=torch.int32, device=dev)
    d_staging = torch.zeros(d_total * block_bytes, dtype=torch.uint8, device=dev)
    d_st = d_staging.view(torch.bfloat16).view(-1, bs, hkv, d)
    res_h = np.full((n_layers, n_req, n_slots), -1, np.int32)
    q_t = q.float()
    moved_total = 0
    for step in range(2):
        if step:
            q_t = 0.95 * q_t + (1 - 0.95 ** 2) ** 0.5 * torch.randn(q_t.shape, device=dev, generator=gen)
        qb = q_t.to(torch.bfloat16)
        retrieve(qb)
        ops.delta_plan(idx, phys, cnt, resident, load_phys, slot_of, miss)
        ops.kv_gather_selected(layers, kv_stride, block_bytes, nb, load_phys, slots_count, d_off, d_region, n_slots, d_staging, d_total)
        torch.cuda.synchronize()
        idx_h, cnt_h, phys_h = idx.cpu().numpy(), cnt.cpu().numpy(), phys.cpu().numpy()
        load_h, slot_h, miss_h, got_res = load_phys.cpu().numpy(), slot_of.cpu().numpy(), miss.cpu().numpy(), resident.cpu().numpy()
        for l in range(n_layers):
            for r in range(n_req):
                k = int(cnt_h[l, r])
                wl, ws, moved = O.delta_plan(idx_h[l, r, :k], phys_h[l, r, :k], res_h[l, r])
                assert moved == miss_h[l, r] and np.array_equal(wl, load_h[l, r]), (step, l, r)
                assert np.array_equal(ws, slot_h[l, r, :k]) and np.array_equal(res_h[l, r], got_res[l, r]), (step, l, r)
                moved_total += moved if step else 0
        for l in (0, 13, n_layers - 1):
            for r in range(n_req):
                k = int(cnt_h[l, r])
                slots_lr = slot_of[l, r, :k].long()
                for kv in range(2):
                    o = r * (n_slots * n_layers * 2) + (l * 2 + kv) * n_slots
                    assert torch.equal(d_st[o + slots_lr], caches[l][kv][phys[l, r, :k].long()]), (step, l, r, kv)
    assert 0 < moved_total < int(topk.sum()) * n_layers          # the second step moved some blocks, not all


def test_config5_full_size_hash_retrieval(ucm, dev):
    """32 requests of 64..256 blocks (8192..32768 tokens), 8 kv heads, 32 layers, 128-bit codes from a seeded Gaussian
    128 x 128 matrix: token codes of one sampled block per (layer, request) against the oracle's exact projection,
    and - in two whole layers - every column sum, majority code, query code, both integer block scores and the
    selection, computed by the oracle from the token codes."""
    from ucm_amd import ops

    n_req, n_layers, hq, hkv, bs = 32, 32, 32, 8, 128
    lens = synth.ragged_lengths(2050, n_req, 8192, 32768)
    rows = int(lens.sum())
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    topk = np.array([max(16, int(0.03 * n)) + 3 for n in lens], np.int32)
    w_bits = synth.bf16_round_bits(synth.normal_f32(2051, (128, 128)))
    w_f32 = synth.bf16_widen(w_bits)
    wd = torch.from_numpy(w_bits.view(np.int16)).to(dev).view(torch.bfloat16)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2052)
    ids_h = synth.permutation(2053, rows)
    caches = [torch.empty((rows, bs, hkv, 128), dtype=torch.bfloat16, device=dev).normal_(generator=gen) for _ in range(n_layers)]
    colsum = torch.zeros((n_layers, rows, hkv, 128), dtype=torch.int16, device=dev)
    bcodes = torch.zeros((n_layers, rows, hkv, 16), dtype=torch.uint8, device=dev)
    tcodes = torch.zeros((n_layers, rows, bs, hkv, 16), dtype=torch.uint8, device=dev)
    ops.hash_encode_blocks(ops.LayerPointers(caches), i32(ids_h, dev), None, rows, wd, bs, hkv, rows, colsum, bcodes, token_codes=tcodes)
    q = torch.empty((n_layers, n_req, hq, 128), dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    q_codes = torch.zeros((n_layers, n_req, hq, 16), dtype=torch.uint8, device=dev)
    q_sum = torch.zeros((n_layers, n_req, 128), dtype=torch.int16, device=dev)
    qbar = torch.zeros((n_layers, n_req, hkv, 16), dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(q, wd, hkv, q_codes, q_sum, qbar, n_req)
    torch.cuda.synchronize()
    # one sampled block per (layer, request)
    pick = np.array([[off[r] + int(synth.ints(2060 + 40 * l + r, 1, 0, int(lens[r]) - 1)[0]) for r in range(n_req)]
                     for l in range(n_layers)])
    for l in range(n_layers):
        sel = torch.from_numpy(pick[l]).to(dev)
        keys = caches[l][torch.from_numpy(ids_h[pick[l]].astype(np.int64)).to(dev)].view(torch.int16).cpu().numpy().view(np.uint16)
        want = O.hash_encode(keys, w_f32)                              # [n_req, bs, hkv, 16]
        assert np.array_equal(tcodes[l][sel].cpu().numpy(), want), l
    seg_off, seg_len, topk_d = i32(off, dev), i32(lens, dev), i32(topk, dev)
    max_len = int(lens.max())
    q_bits = q.view(torch.int16).cpu().numpy().view(np.uint16)
    for l in (3, n_layers - 1):
        tc = tcodes[l].cpu().numpy()
        want_sum, want_maj = O.hash_colsum(tc), O.hash_majority(tc)
        assert np.array_equal(colsum[l].cpu().numpy(), want_sum) and np.array_equal(bcodes[l].cpu().numpy(), want_maj)
        want_q = O.hash_encode(q_bits[l], w_f32)
        assert np.array_equal(q_codes[l].cpu().numpy(), want_q)
        pm = np.unpackbits(want_q, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
        assert np.array_equal(q_sum[l].cpu().numpy(), pm.sum(1))
        qm = np.stack([O.q_head_mean(synth.bf16_widen(q_bits[l][r]), hkv) for r in range(n_req)])
        want_qbar = O.hash_encode_f32(qm, w_f32)
        assert np.array_equal(qbar[l].cpu().numpy(), want_qbar)
        for mode in (ops.HASH_SCORE_BLOCK_CODE, ops.HASH_SCORE_SUM):
            scores = torch.full((n_layers, rows), -1.0, device=dev)
            ops.hash_score_blocks(mode, q_sum, qbar, colsum, bcodes, seg_off, seg_len, rows, scores)
            idx = torch.full((n_layers, n_req, max_len), -1, dtype=torch.int32, device=dev)
            cnt = torch.zeros((n_layers, n_req), dtype=torch.int32, device=dev)
            ops.topk_windows(scores, seg_off, seg_len, topk_d, max_len, idx, cnt)
            torch.cuda.synchronize()
            sc, idx_h, cnt_h = scores[l].cpu().numpy(), idx[l].cpu().numpy(), cnt[l].cpu().numpy()
            for r in range(n_req):
                a, n = int(off[r]), int(lens[r])
                if mode == ops.HASH_SCORE_BLOCK_CODE:
                    want = O.hash_scores_block(want_qbar[r], want_maj[a : a + n])
                else:
                    want = O.hash_scores_sum(want_q[r], tc[a : a + n].transpose(0, 2, 1, 3))
                assert np.array_equal(sc[a : a + n], want.astype(np.float32)), (l, mode, r)
                sel = O.topk_windows(want.astype(np.int32), int(topk[r]))
                assert cnt_h[r] == len(sel) and np.array_equal(idx_h[r, : len(sel)], sel), (l, mode, r)


def test_config4_full_size_long_context_scores_selection_and_incremental_update(ucm, dev):
    """8 requests of 512..1024 blocks (65536..131072 tokens), Qwen2-72B attention shape (64 query heads, 8 kv heads,
    head_dim 128), all 80 layers, k = max(16, 2 %) + 1 first + 2 last blocks.  The representative table is the input
    at this size (the keys of 80 layers would not fit the device: 8 x 1024 x 80 x 512 KiB); the incremental update
    of a decode step - only the block a request just filled is reduced, every other row stays - is done on one
    cache block per request and layer."""
    from ucm_amd import ops

    n_req, n_layers, hq, hkv, d, bs = 8, 80, 64, 8, 128, 128
    row = hkv * d
    lens = synth.ragged_lengths(2040, n_req, 65536, 131072)
    assert lens.min() >= 512 and lens.max() <= 1024
    topk = np.array([max(16, int(0.02 * n)) + 3 for n in lens], np.int32)
    rows = int(lens.sum())
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    max_len = int(lens.max())
    gen = torch.Generator(device=dev)
    gen.manual_seed(2041)
    # bf16 values both sides hold exactly: block means of N(0,1) keys have a standard deviation of 1/sqrt(128)
    repre = (torch.empty((n_layers, rows, row), dtype=torch.float32, device=dev).normal_(generator=gen) * 0.0884).to(torch.bfloat16)
    q = torch.empty((n_layers, n_req, hq, d), dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    seg_off, seg_len, topk_d = i32(off, dev), i32(lens, dev), i32(topk, dev)
    scores = torch.zeros(n_layers, rows, device=dev)
    idx = torch.full((n_layers, n_req, max_len), -1, dtype=torch.int32, device=dev)
    cnt = torch.zeros(n_layers, n_req, dtype=torch.int32, device=dev)

    def check(layers_to_check):
        torch.cuda.synchronize()
        q_h, sc_h, idx_h, cnt_h = q.float().cpu().numpy(), scores.cpu().numpy(), idx.cpu().numpy(), cnt.cpu().numpy()
        for l in layers_to_check:
            widx, wcnt, wsc = O.select_topk_bs(q_h[l], repre[l].float().cpu().numpy(), off, lens, topk, hkv, out_stride=max_len + 4)
            assert np.array_equal(bits(wsc), bits(sc_h[l])), f"scores differ in layer {l}"
            assert np.array_equal(wcnt, cnt_h[l]) and np.array_equal(wcnt, topk)
            for r in range(n_req):
                assert np.array_equal(widx[r, : wcnt[r]], idx_h[l, r, : wcnt[r]]), (l, r)
                # what the rule fixes whatever the scores: first block, last two, ascending, no repeats
                got = idx_h[l, r, : wcnt[r]]
                assert got[0] == 0 and got[-1] == lens[r] - 1 and got[-2] == lens[r] - 2 and (np.diff(got) > 0).all()

    ops.score_blocks(q, repre, seg_off, seg_len, max_len, hkv, scores, total_blocks=rows)
    ops.topk_windows(scores, seg_off, seg_len, topk_d, max_len, idx, cnt)
    check(range(n_layers))

    # ---- decode step: each request's last block has just been filled; only its row of the table changes
    nb = 2 * n_req
    caches = [torch.empty((nb, bs, hkv, d), dtype=torch.bfloat16, device=dev).normal_(generator=gen) for _ in range(n_layers)]
    new_ids = synth.permutation(2042, nb)[:n_req].astype(np.int32)
    new_rows = (off + lens - 1).astype(np.int32)
    before = repre.clone()
    ops.block_mean(ops.LayerPointers(caches), i32(new_ids, dev), i32(new_rows, dev), repre, bs, hkv, d, nb)
    torch.cuda.synchronize()
    untouched = np.ones(rows, bool)
    untouched[new_rows] = False
    keep = torch.from_numpy(untouched).to(dev)
    assert torch.equal(repre[:, keep], before[:, keep])
    for l in (0, 41, n_layers - 1):
        want = np.zeros((n_req, row), np.float32)
        O.block_mean_paged(caches[l].view(torch.int16).cpu().numpy().view(np.uint16), new_ids, np.arange(n_req), want, round_bf16=True)
        assert np.array_equal(bits(repre[l, torch.from_numpy(new_rows.astype(np.int64)).to(dev)].float().cpu().numpy()), bits(want))
    q = torch.empty((n_layers, n_req, hq, d), dtype=torch.bfloat16, device=dev).normal_(generator=gen)
    ops.score_blocks(q, repre, seg_off, seg_len, max_len, hkv, scores, total_blocks=rows)
    ops.topk_windows(scores, seg_off, seg_len, topk_d, max_len, idx, cnt)
    check((0, 17, 41, n_layers - 1))
