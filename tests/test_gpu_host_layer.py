"""The host-side mirror of the reference's plugin / worker interfaces, driven the
way patched vLLM drives it (stand-in objects instead of vLLM's), with every
result checked against the CPU oracle."""
import types

import numpy as np
import pytest
import torch

import oracle as O
import synth

pytestmark = pytest.mark.gpu

bits = lambda a: np.ascontiguousarray(a, np.float32).view(np.uint32)


# ------------------------------------------------------- retrieval worker

def test_retrieval_worker_golden_vectors(ucm, dev, golden):
    """submit / wait / get_result against what the reference's own backend returned."""
    from ucm_amd.sparse.esa.retrieval_worker import HipRetrievalBackend, RetrievalWorker

    z, meta = golden
    for i, rows, dim, b, m, topk, s_data, s_q, s_idx in meta["esa"]:
        data = torch.from_numpy(synth.normal_bf16_as_f32(s_data, (rows, dim))).to(dev)
        q = torch.from_numpy(synth.normal_bf16_as_f32(s_q, (b, dim))).to(dev).to(torch.bfloat16)
        idx = np.stack([synth.permutation(s_idx + r, rows)[:m] for r in range(b)]).astype(np.int32)
        idx[:, m - 3:] = -1
        worker = RetrievalWorker(HipRetrievalBackend(data))
        rid = worker.submit(q, topk=topk, indexes=idx)
        worker.wait(rid)
        assert worker.poll(rid)
        res = worker.get_result(rid)
        assert res["indices"].dtype == np.int32 and res["scores"].dtype == np.float32
        assert np.array_equal(res["indices"], z[f"esa/{i}/indices"])
        assert np.array_equal(bits(res["scores"]), bits(z[f"esa/{i}/scores"]))
        with pytest.raises(RuntimeError, match="Result not ready"):
            worker.get_result(rid)  # a result is handed out once


def test_retrieval_worker_protocol_and_errors(ucm, dev):
    from ucm_amd.sparse.esa.retrieval_worker import HipRetrievalBackend, RetrievalWorker

    rows, dim = 500, 1024
    data = torch.from_numpy(synth.normal_bf16_as_f32(700, (rows, dim))).to(dev)
    backend = HipRetrievalBackend(data)
    worker = RetrievalWorker(backend)
    with pytest.raises(RuntimeError, match="Query dim mismatch"):
        backend.submit(torch.zeros(1, dim - 1, device=dev), 3, [[1, 2]])
    with pytest.raises(RuntimeError, match="Query and indexes batch mismatch"):
        backend.submit(torch.zeros(2, dim, device=dev), 3, [[1, 2]])
    with pytest.raises(RuntimeError, match="Bad req_id"):
        backend.wait(12345)
    # the way ESA calls it: one request, a python list of slot lists (esa.py:297-301)
    slots = [int(s) for s in synth.permutation(701, rows)[:333]]
    q = torch.from_numpy(synth.normal_bf16_as_f32(702, (1, dim))).to(dev)
    ids = [worker.submit(q, topk=40, indexes=[slots]) for _ in range(3)]
    assert ids == sorted(set(ids))  # fresh increasing ids
    for rid in ids:
        worker.wait(rid)
        res = worker.get_result(rid)
        wi, ws = O.esa_retrieve(data.cpu().numpy(), q.cpu().numpy()[0], np.array(slots, np.int32), 40)
        assert np.array_equal(res["indices"][0], wi) and np.array_equal(bits(res["scores"][0]), bits(ws))
    # topk larger than the candidate list returns every candidate, best first
    rid = worker.submit(q, topk=5000, indexes=[slots[:17]])
    worker.wait(rid)
    res = worker.get_result(rid)
    assert res["indices"].shape == (1, 17) and np.all(np.diff(res["scores"][0]) <= 0)
    # rows written after construction are visible: the table is aliased, not copied
    data[slots[5]] = 100.0 * q[0]
    rid = worker.submit(q, topk=1, indexes=[slots])
    worker.wait(rid)
    assert worker.get_result(rid)["indices"][0, 0] == slots[5]
    # ties: equal rows come out in index-row order
    data[7] = data[3]
    rid = worker.submit(q, topk=2, indexes=[[7, 3]])
    worker.wait(rid)
    assert list(worker.get_result(rid)["indices"][0]) == [7, 3]


def test_esa_retrieve_wide_and_ragged_rows(ucm, dev):
    """Batch of requests, -1 padding in the middle, out-of-range slots, dims that are not a multiple of the tile."""
    from ucm_amd import ops

    # the last case: the widest row the entry point takes (8192 candidates: the rank kernel's 64 KiB of dynamic LDS)
    for rows, dim, b, m, topk in [(900, 1024, 4, 700, 210), (64, 36, 3, 9, 4), (3000, 256, 2, 2500, 900), (9000, 64, 2, 8192, 3000)]:
        data_h = synth.normal_bf16_as_f32(710 + dim, (rows, dim))
        q_h = synth.normal_bf16_as_f32(711 + dim, (b, dim))
        idx = np.stack([synth.permutation(712 + r, rows)[:m] for r in range(b)]).astype(np.int32)
        idx[:, ::5] = -1
        idx[0, 1] = rows + 7  # outside the table: skipped like a padding entry
        out_idx = torch.full((b, min(topk, m)), -1, dtype=torch.int32, device=dev)
        out_scores = torch.zeros((b, min(topk, m)), device=dev)
        out_cnt = torch.zeros(b, dtype=torch.int32, device=dev)
        ws = torch.empty(b, m, device=dev)
        ops.esa_retrieve(torch.from_numpy(data_h).to(dev), torch.from_numpy(q_h).to(dev),
                         torch.from_numpy(idx).to(dev), topk, ws, out_idx, out_scores, out_cnt)
        for r in range(b):
            row = idx[r].copy()
            row[row >= rows] = -1
            wi, wsc = O.esa_retrieve(data_h, q_h[r], row, topk)
            c = int(out_cnt[r])
            assert c == len(wi)
            assert np.array_equal(out_idx[r, :c].cpu().numpy(), wi)
            assert np.array_equal(bits(out_scores[r, :c].cpu().numpy()), bits(wsc))


# ------------------------------------------------ CalKpreAndTopk surface

def test_cal_kpre_and_topk_surface(ucm, dev):
    """The reference's call sequence (gsa.py:484-512, :914-954, :616-632) against the GPU object."""
    from ucm_amd.sparse.gsa.offload_ops import CalKpreAndTopk

    L, bs, max_bs, hq, hkv, d, max_blocks = 3, 128, 8, 32, 8, 128, 64
    obj = CalKpreAndTopk(L, bs, max_bs, hq, d, device=dev)
    obj.set_kpre_method_param(hkv, 1)
    kpre_all = torch.from_numpy(synth.normal_f32(720, (L, max_bs * max_blocks, 1, hkv, d))).to(dev)
    obj.set_kpre_cache(list(kpre_all.unbind(0)))
    # batch of 4: entries 0 and 2 decode with 50 and 37 blocks, 1 and 3 do not
    is_decode = [True, False, True, False]
    lens = [50, 0, 37, 0]
    slot_map = [[max_blocks * (i + 1) + j for j in range(max(n, 1))] for i, n in enumerate(lens)]
    topk_lens = [O.compute_topk_len(50), O.compute_topk_len(37)]
    topk_cache = [torch.full((4, max_blocks), -1, dtype=torch.int32, device=dev) for _ in range(L)]
    obj.set_common_param([0, 2], is_decode)
    obj.set_topk_param(slot_map)
    obj.set_topk_cache(topk_cache, topk_lens)
    q = synth.normal_bf16_as_f32(721, (L, 4, hq, d))
    for l in range(L):
        qd = torch.from_numpy(q[l]).to(dev).to(torch.bfloat16)
        obj.add_copy_req(False, l, [5, -1, 9, -1], qd)   # locations: -1 = not a decode entry
    torch.cuda.synchronize()
    assert obj.is_calculate_finish()
    kp = kpre_all.cpu().numpy().reshape(L, max_bs * max_blocks, hkv * d)
    for l in range(L):
        got = topk_cache[l].cpu().numpy()
        for i, j in ((0, 0), (2, 1)):
            want, _ = O.select_topk(q[l, i], kp[l, slot_map[i][0] : slot_map[i][0] + lens[i]].reshape(lens[i], hkv, 1, d),
                                    topk_lens[j])
            assert np.array_equal(got[i, : len(want)], want), (l, i)
        assert np.all(got[1] == -1) and np.all(got[3] == -1)
        assert np.array_equal(obj.q_cache[l][0].cpu().numpy(), q[l, 0])
    with pytest.raises(ValueError):
        obj.set_kpre_method_param(hkv, 3)
    # two representatives per (block, kv head): a row of the cache is read [kv head][representative][channel], as
    # the reference's kernel reads it
    obj = CalKpreAndTopk(L, bs, max_bs, hq, d, device=dev)
    obj.set_kpre_method_param(hkv, 2)
    kpre_all = torch.from_numpy(synth.normal_f32(722, (L, max_bs * max_blocks, 2, hkv, d))).to(dev)
    obj.set_kpre_cache(list(kpre_all.unbind(0)))
    topk_cache = [torch.full((4, max_blocks), -1, dtype=torch.int32, device=dev) for _ in range(L)]
    obj.set_common_param([0, 2], is_decode)
    obj.set_topk_param(slot_map)
    obj.set_topk_cache(topk_cache, topk_lens)
    for l in range(L):
        obj.add_copy_req(False, l, [5, -1, 9, -1], torch.from_numpy(q[l]).to(dev).to(torch.bfloat16))
    torch.cuda.synchronize()
    kp = kpre_all.cpu().numpy().reshape(L, max_bs * max_blocks, hkv * 2 * d)
    for l in range(L):
        got = topk_cache[l].cpu().numpy()
        for i, j in ((0, 0), (2, 1)):
            want, _ = O.select_topk(q[l, i], kp[l, slot_map[i][0] : slot_map[i][0] + lens[i]].reshape(lens[i], hkv, 2, d),
                                    topk_lens[j])
            assert np.array_equal(got[i, : len(want)], want), (l, i)


# ------------------------------------------------------------ GSA plugin

class _ModelConfig:
    def __init__(self, hq, hkv, d, layers, max_model_len):
        self.hq, self.hkv, self.d, self.layers, self.max_model_len = hq, hkv, d, layers, max_model_len

    def get_num_kv_heads(self, pc):
        return self.hkv

    def get_num_attention_heads(self, pc):
        return self.hq

    def get_head_size(self):
        return self.d

    def get_num_layers(self, pc):
        return self.layers


def make_config(hq, hkv, d, layers, block_size, max_model_len, gsa_cfg):
    ns = types.SimpleNamespace
    return ns(model_config=_ModelConfig(hq, hkv, d, layers, max_model_len), parallel_config=ns(rank=0, tensor_parallel_size=1),
              cache_config=ns(block_size=block_size), scheduler_config=ns(max_num_seqs=4),
              kv_transfer_config=ns(kv_connector_extra_config={"ucm_sparse_config": {"GSA": gsa_cfg}}))


def topk_len(n, lo, hi):
    t = int(n * 0.3)
    return min(lo, n) if t < lo else min(t, hi)


@pytest.mark.parametrize("repre_dtype,model,lag", [("float32", "bfloat16", 0), ("bfloat16", "bfloat16", 0), ("float32", "float16", 0),
                                                   ("bfloat16", "bfloat16", 1), ("float32", "float16", 1)])
def test_gsa_plugin_decode_flow(ucm, dev, repre_dtype, model, lag):
    """Two requests through prefill and 40 decode steps, two layers: after every attention_begin the
    layer's block table and sequence lengths must be what the oracle selects from the same cache.
    With a bfloat16 table the representatives are the rounded means of the live reference path; a model that runs
    in float16 (cache, keys and queries) goes through the same hooks with an fp32 table.  With retrieval_lag 1 a
    step's selection comes from the queries of the step before (the request's first sparsified step apart), scored
    over the table and the block lists of the step that uses it, in one launch before the first layer runs."""
    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseRole
    from ucm_amd.sparse.factory import UcmSparseFactory
    from ucm_amd.sparse.gsa.gsa import GSA

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 64, 2, 16, 120
    lo, hi = 6, 10
    cfg = make_config(hq, hkv, d, L, bs, 16 * 60, {"seg_prefill_threshold": 100, "min_topk_len": lo, "max_topk_len": hi,
                                                   "repre_dtype": repre_dtype, "retrieval_lag": lag})
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    assert isinstance(plugin, GSA)
    assert plugin.repre_dtype == getattr(torch, repre_dtype)   # the table itself is allocated at the first step
    assert plugin.estimate_num_slots_sparsed(ns()) == INVALID_SLOT
    plugin.request_begin("A", [])

    g = torch.Generator(device=dev)
    g.manual_seed(5)
    model = getattr(torch, model)
    caches = [torch.zeros(2, nb, bs, hkv, d, dtype=model, device=dev) for _ in range(L)]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=None)
    free_blocks = [int(x) for x in synth.permutation(730, nb)]
    prompts = {"A": 300, "B": 50}
    reqs = {r: ns(block_ids=[[]], num_computed_tokens=0, prompt_token_ids=[1] * n, output_token_ids=[]) for r, n in prompts.items()}
    repre_h = {r: [np.zeros((60, hkv * d), np.float32) for _ in range(L)] for r in prompts}
    done_blocks = {r: 0 for r in prompts}
    saw_sparse = 0
    q_before = [None] * L                    # request A's query of the step before, per layer
    lagged_steps = 0

    for step in range(41):
        sched = {}
        for r, st in reqs.items():
            n_new = prompts[r] if step == 0 else 1
            need = -(-(st.num_computed_tokens + n_new) // bs)
            while len(st.block_ids[0]) < need:
                st.block_ids[0].append(free_blocks.pop())
            sched[r] = n_new
        so = ns(num_scheduled_tokens=sched, scheduled_new_reqs=[ns(req_id=r) for r in reqs] if step == 0 else [],
                scheduled_cached_reqs=ns(req_ids=[] if step == 0 else list(reqs)))
        ib = ns(req_id_to_index={"A": 0, "B": 1})
        n_tok = sum(sched.values())
        seq_lens = [reqs[r].num_computed_tokens + sched[r] for r in ("A", "B")]
        width = 60
        bt = torch.zeros(2, width, dtype=torch.int32, device=dev)
        for i, r in enumerate(("A", "B")):
            bt[i, : len(reqs[r].block_ids[0])] = torch.tensor(reqs[r].block_ids[0], dtype=torch.int32)
        plugin.build_sparse_meta(so, reqs, ib, None)
        plugin.execute_begin(so)
        # with the lag, every step after the first sparsified one has its selection before the model runs
        assert (plugin._lagged is not None) == (lag == 1 and step >= 2)
        lagged_steps += int(plugin._lagged is not None)
        for l in range(L):
            md = ns(block_table=bt.clone(), seq_lens=torch.tensor(seq_lens, dtype=torch.int32, device=dev))
            fc.attn_metadata = {names[l]: md}
            query = torch.randn(n_tok, hq, d, device=dev, generator=g).to(model)
            key = torch.randn(n_tok, hkv, d, device=dev, generator=g).to(model)
            # the model writes this step's keys into the paged cache before attention runs
            t0 = 0
            for r in ("A", "B"):
                for t in range(sched[r]):
                    pos = reqs[r].num_computed_tokens + t
                    caches[l][0, reqs[r].block_ids[0][pos // bs], pos % bs] = key[t0 + t]
                t0 += sched[r]
            plugin.attention_begin(query, key, key, names[l], fc)
            torch.cuda.synchronize()
            if step > 0:
                # request A is sparsified, B keeps everything
                nA = len(reqs["A"].block_ids[0])
                k = topk_len(nA, lo, hi)
                qA = query[0].float().cpu().numpy()  # A's only (= last) token is row 0 of the batch
                if lag and step >= 2:
                    qA, q_before[l] = q_before[l], qA
                else:
                    q_before[l] = qA
                want_idx, _ = O.select_topk(qA, repre_h["A"][l][:nA].reshape(nA, hkv, 1, d), k)
                phys, want_len = O.block_table_gather(reqs["A"].block_ids[0], want_idx, seq_lens[0], bs)
                got_bt, got_len = md.block_table.cpu().numpy(), md.seq_lens.cpu().numpy()
                assert got_len[0] == want_len, (step, l)
                assert np.array_equal(got_bt[0, : len(phys)], phys), (step, l)
                nB = len(reqs["B"].block_ids[0])
                assert got_len[1] == seq_lens[1] and np.array_equal(got_bt[1, :nB], reqs["B"].block_ids[0])
                saw_sparse += int(len(phys) < nA)
            else:
                assert md.block_table.data_ptr() != plugin.block_tables_mp.data_ptr()  # prefill: untouched
            plugin.attention_finished(query, key, key, None, names[l], fc)
            # oracle-side table: a block is reduced after the step that fills it
            for r in ("A", "B"):
                full = min(seq_lens[("A", "B").index(r)] // bs, len(reqs[r].block_ids[0]))
                todo = list(range(done_blocks[r], full))
                if todo:
                    kc = caches[l][0].view(torch.int16).cpu().numpy().view(np.uint16)
                    O.block_mean_paged(kc, [reqs[r].block_ids[0][i] for i in todo], todo, repre_h[r][l],
                                       round_bf16=(repre_dtype == "bfloat16"), keys_f16=(model == torch.float16))
        for r in ("A", "B"):
            done_blocks[r] = max(done_blocks[r], min(seq_lens[("A", "B").index(r)] // bs, len(reqs[r].block_ids[0])))
        plugin.execute_finished()
        torch.cuda.synchronize()
        # the device table equals the oracle's
        offA = plugin.gsa_stats["A"].slot_offset
        for l in range(L):
            assert plugin.kpre_caches.dtype == getattr(torch, repre_dtype)
            got = plugin.kpre_caches[l, offA : offA + done_blocks["A"]].float().cpu().numpy()
            assert np.array_equal(bits(got), bits(repre_h["A"][l][: done_blocks["A"]])), (step, l)
        for r, st in reqs.items():
            st.num_computed_tokens += sched[r]
            st.output_token_ids.append(7)
    assert saw_sparse >= 2 * 39  # every decode step of every layer really dropped blocks
    assert lagged_steps == (39 if lag else 0)
    plugin.request_finished_in_worker("A")
    assert "A" not in plugin.gsa_stats and not plugin.topk_kpre_manger.is_exist("A")


def test_gsa_retrieval_lag_with_a_request_that_arrives_later(ucm, dev):
    """retrieval_lag 1 while the batch changes: request A decodes from step 1 and leaves after step 7, request C's prompt
    arrives at step 4 (A decoding beside it) and C decodes from step 5, request D arrives at step 8.  Every selection a layer's attention sees must be the oracle's for
    the query the request had in the step before - for C's first decode step that is the last token of its prompt, kept
    during the step that prefilled it - over the representatives and block lists of the step that uses it."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 64, 2, 16, 160
    lo, hi = 6, 10
    cfg = make_config(hq, hkv, d, L, bs, 16 * 60, {"seg_prefill_threshold": 100, "min_topk_len": lo, "max_topk_len": hi,
                                                   "repre_dtype": "bfloat16", "retrieval_lag": 1})
    plugin = GSA(cfg, UcmSparseRole.WORKER)
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    caches = [torch.zeros(2, nb, bs, hkv, d, dtype=torch.bfloat16, device=dev) for _ in range(L)]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=None)
    free_blocks = [int(x) for x in synth.permutation(731, nb)]
    prompts, arrives, leaves = {"A": 290, "C": 410, "D": 330}, {"A": 0, "C": 4, "D": 8}, {"A": 7}
    reqs = {r: ns(block_ids=[[]], num_computed_tokens=0, prompt_token_ids=[1] * n, output_token_ids=[]) for r, n in prompts.items()}
    repre_h = {r: [np.zeros((60, hkv * d), np.float32) for _ in range(L)] for r in prompts}
    done_blocks = {r: 0 for r in prompts}
    q_before = {r: [None] * L for r in prompts}
    lagged, checked = [], 0
    for step in range(12):
        for r, last in leaves.items():
            if step == last + 1:
                plugin.request_finished_in_worker(r)             # A is done
        live = [r for r in prompts if arrives[r] <= step <= leaves.get(r, 99)]
        sched = {r: (prompts[r] if step == arrives[r] else 1) for r in live}
        for r in live:
            need = -(-(reqs[r].num_computed_tokens + sched[r]) // bs)
            while len(reqs[r].block_ids[0]) < need:
                reqs[r].block_ids[0].append(free_blocks.pop())
        so = ns(num_scheduled_tokens=sched, scheduled_new_reqs=[ns(req_id=r) for r in live if step == arrives[r]])
        ib = ns(req_id_to_index={r: i for i, r in enumerate(live)})
        seq_lens = {r: reqs[r].num_computed_tokens + sched[r] for r in live}
        plugin.build_sparse_meta(so, {r: reqs[r] for r in live}, ib, None)
        plugin.execute_begin(so)
        lagged.append(plugin._lagged is not None)
        for l in range(L):
            md = ns(block_table=None, seq_lens=None)
            fc.attn_metadata = {names[l]: md}
            n_tok = sum(sched.values())
            query = torch.randn(n_tok, hq, d, device=dev, generator=g).to(torch.bfloat16)
            key = torch.randn(n_tok, hkv, d, device=dev, generator=g).to(torch.bfloat16)
            t0, last_row = 0, {}
            for r in live:
                for t in range(sched[r]):
                    pos = reqs[r].num_computed_tokens + t
                    caches[l][0, reqs[r].block_ids[0][pos // bs], pos % bs] = key[t0 + t]
                t0 += sched[r]
                last_row[r] = t0 - 1
            plugin.attention_begin(query, key, key, names[l], fc)
            torch.cuda.synchronize()
            for i, r in enumerate(live):
                q_now = query[last_row[r]].float().cpu().numpy()
                if step > arrives[r]:                                     # a decode step of a sparsified request
                    n = len(reqs[r].block_ids[0])
                    q_use = q_before[r][l] if lagged[-1] else q_now
                    want_idx, _ = O.select_topk(q_use, repre_h[r][l][:n].reshape(n, hkv, 1, d), topk_len(n, lo, hi))
                    phys, want_len = O.block_table_gather(reqs[r].block_ids[0], want_idx, seq_lens[r], bs)
                    assert int(md.seq_lens[i]) == want_len, (step, l, r)
                    assert np.array_equal(md.block_table[i, : len(phys)].cpu().numpy(), phys), (step, l, r)
                    checked += 1
                q_before[r][l] = q_now
            plugin.attention_finished(query, key, key, None, names[l], fc)
            for r in live:
                full = min(seq_lens[r] // bs, len(reqs[r].block_ids[0]))
                todo = list(range(done_blocks[r], full))
                if todo:
                    kc = caches[l][0].view(torch.int16).cpu().numpy().view(np.uint16)
                    O.block_mean_paged(kc, [reqs[r].block_ids[0][i] for i in todo], todo, repre_h[r][l], round_bf16=True)
        for r in live:
            done_blocks[r] = max(done_blocks[r], min(seq_lens[r] // bs, len(reqs[r].block_ids[0])))
            reqs[r].num_computed_tokens += sched[r]
            reqs[r].output_token_ids.append(7)
        plugin.execute_finished()
    # step 1 scores layer by layer (nothing was kept during the prefill-only step 0); from step 2 on one launch per step,
    # the step C's prompt runs beside A's decode, C's first decode step, the step after A has left and D's arrival included
    assert lagged == [False, False] + [True] * 10
    assert "A" not in plugin.gsa_stats and "A" not in plugin._parked and set(plugin.gsa_stats) == {"C", "D"}
    assert checked == L * (7 + 7 + 3)


@pytest.mark.parametrize("lag", [0, 1])
@pytest.mark.parametrize("seed", [11, 12, 13])
def test_gsa_drawn_scenarios(ucm, dev, seed, lag):
    """Thirty steps of a drawn batch: up to four requests at a time, prompts of 40 to 520 tokens (those of at most
    100 are never sparsified; those above 256 are prefilled in two chunks), arrivals and departures at random steps,
    a request id coming back with another request behind it, batch indices that shift when a request leaves.  After
    every layer's attention_begin a sparsified request's row of the block table and its length are the oracle's
    selection - from the query of the step before wherever the step was scored ahead of the model - and a request that
    is not sparsified keeps its own blocks; after every step the table of representatives holds the oracle's rows."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 64, 2, 16, 200
    lo, hi, threshold, chunk = 6, 10, 100, 256
    cfg = make_config(hq, hkv, d, L, bs, 16 * 60, {"seg_prefill_threshold": threshold, "min_topk_len": lo, "max_topk_len": hi,
                                                   "repre_dtype": "bfloat16", "retrieval_lag": lag})
    plugin = GSA(cfg, UcmSparseRole.WORKER)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    rng = np.random.RandomState(seed)
    caches = [torch.zeros(2, nb, bs, hkv, d, dtype=torch.bfloat16, device=dev) for _ in range(L)]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=None)
    free_blocks = [int(x) for x in synth.permutation(740 + seed, nb)]
    ids = ["A", "B", "C", "D", "E"]
    reqs, prompts, repre_h, done_blocks, q_before = {}, {}, {}, {}, {}
    live, leaving = [], []
    checked = kept_whole = lagged_steps = came_back = 0
    seen = set()
    for step in range(30):
        for r in leaving:
            plugin.request_finished_in_worker(r)
            free_blocks.extend(reqs[r].block_ids[0])
            live.remove(r)
        leaving = []
        new = []
        idle = [r for r in ids if r not in live]
        if idle and len(live) < 4 and (step == 0 or rng.rand() < 0.4):
            r = idle[rng.randint(len(idle))]
            came_back += int(r in seen)
            seen.add(r)
            prompts[r] = int(rng.choice([rng.randint(40, 101), rng.randint(101, 257), rng.randint(257, 521)], p=[0.2, 0.4, 0.4]))
            reqs[r] = ns(block_ids=[[]], num_computed_tokens=0, prompt_token_ids=[1] * prompts[r], output_token_ids=[])
            repre_h[r] = [np.zeros((60, hkv * d), np.float32) for _ in range(L)]
            done_blocks[r], q_before[r] = 0, [None] * L
            live.append(r)
            new.append(r)
        if not live:
            continue
        sched = {r: (min(chunk, prompts[r] - reqs[r].num_computed_tokens) if reqs[r].num_computed_tokens < prompts[r] else 1)
                 for r in live}
        for r in live:
            need = -(-(reqs[r].num_computed_tokens + sched[r]) // bs)
            while len(reqs[r].block_ids[0]) < need:
                reqs[r].block_ids[0].append(free_blocks.pop())
        so = ns(num_scheduled_tokens=sched, scheduled_new_reqs=[ns(req_id=r) for r in new])
        ib = ns(req_id_to_index={r: i for i, r in enumerate(live)})
        seq_lens = {r: reqs[r].num_computed_tokens + sched[r] for r in live}
        sparsified = {r: prompts[r] > threshold and reqs[r].num_computed_tokens >= prompts[r] for r in live}
        plugin.build_sparse_meta(so, {r: reqs[r] for r in live}, ib, None)
        plugin.execute_begin(so)
        lagged = plugin._lagged is not None
        assert not lagged or lag == 1
        lagged_steps += int(lagged)
        for l in range(L):
            md = ns(block_table=None, seq_lens=None)
            fc.attn_metadata = {names[l]: md}
            n_tok = sum(sched.values())
            query = torch.randn(n_tok, hq, d, device=dev, generator=g).to(torch.bfloat16)
            key = torch.randn(n_tok, hkv, d, device=dev, generator=g).to(torch.bfloat16)
            t0, last_row = 0, {}
            for r in live:
                for t in range(sched[r]):
                    pos = reqs[r].num_computed_tokens + t
                    caches[l][0, reqs[r].block_ids[0][pos // bs], pos % bs] = key[t0 + t]
                t0 += sched[r]
                last_row[r] = t0 - 1
            plugin.attention_begin(query, key, key, names[l], fc)
            torch.cuda.synchronize()
            assert (md.block_table is not None) == any(sparsified.values()), (step, l)
            for i, r in enumerate(live):
                q_now = query[last_row[r]].float().cpu().numpy()
                n = len(reqs[r].block_ids[0])
                if sparsified[r]:
                    q_use = q_before[r][l] if lagged else q_now
                    want_idx, _ = O.select_topk(q_use, repre_h[r][l][:n].reshape(n, hkv, 1, d), topk_len(n, lo, hi))
                    phys, want_len = O.block_table_gather(reqs[r].block_ids[0], want_idx, seq_lens[r], bs)
                    assert int(md.seq_lens[i]) == want_len, (step, l, r)
                    assert np.array_equal(md.block_table[i, : len(phys)].cpu().numpy(), phys), (step, l, r)
                    checked += 1
                elif md.block_table is not None:
                    assert int(md.seq_lens[i]) == seq_lens[r], (step, l, r)
                    assert np.array_equal(md.block_table[i, :n].cpu().numpy(), reqs[r].block_ids[0]), (step, l, r)
                    kept_whole += 1
                q_before[r][l] = q_now
            plugin.attention_finished(query, key, key, None, names[l], fc)
            for r in live:
                full = min(seq_lens[r] // bs, len(reqs[r].block_ids[0]))
                todo = list(range(done_blocks[r], full))
                if todo:
                    kc = caches[l][0].view(torch.int16).cpu().numpy().view(np.uint16)
                    O.block_mean_paged(kc, [reqs[r].block_ids[0][i] for i in todo], todo, repre_h[r][l], round_bf16=True)
        plugin.execute_finished()
        torch.cuda.synchronize()
        for r in live:
            done_blocks[r] = max(done_blocks[r], min(seq_lens[r] // bs, len(reqs[r].block_ids[0])))
            off = plugin.gsa_stats[r].slot_offset
            for l in range(L):
                got = plugin.kpre_caches[l, off : off + done_blocks[r]].float().cpu().numpy()
                assert np.array_equal(bits(got), bits(repre_h[r][l][: done_blocks[r]])), (step, l, r)
            reqs[r].num_computed_tokens += sched[r]
            if reqs[r].num_computed_tokens > prompts[r] - 1:
                reqs[r].output_token_ids.append(7)
            if reqs[r].num_computed_tokens >= prompts[r] + 2 and rng.rand() < 0.12:
                leaving.append(r)
    assert checked >= 15 * L and kept_whole >= L, (checked, kept_whole, came_back)
    assert set(plugin.gsa_stats) == set(live)
    if lag:
        assert lagged_steps >= 8


@pytest.mark.parametrize("lag", [0, 1])
def test_gsa_plugin_at_serving_size(ucm, dev, lag):
    """Sixteen requests of 280 to 400 blocks of 128 tokens, 32 layers, Llama-3-8B head shape, through the plugin's
    hooks as the benchmark's plugin leg drives them (two cache tensors stand behind the 32 layers): after each of four
    decode steps every layer's row of the block table and its length are the oracle's selection for every request,
    from the representatives the plugin's own table holds and the queries the layer was handed - this step's, or
    with retrieval_lag 1 and from the second decode step on the step before's."""
    import plugin_bench as PB
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA

    L, n_req, bs = 32, 16, PB.BS
    rng = np.random.default_rng(41)
    lens = rng.integers(280, 401, n_req)
    nb = int(lens.sum()) + 8
    g = torch.Generator(device=dev)
    g.manual_seed(42)
    two = [torch.empty((2, nb, bs, PB.HKV, PB.D), dtype=torch.bfloat16, device=dev).normal_(0.0, 1.0, generator=g) for _ in range(2)]
    caches = [two[l % 2] for l in range(L)]
    perm = rng.permutation(nb)
    starts = np.concatenate([[0], np.cumsum(lens)])
    block_lists = [[int(x) for x in perm[starts[r] : starts[r + 1]]] for r in range(n_req)]
    cfg = PB.make_config(L, 65536, n_req, "GSA", {"seg_prefill_threshold": 0, "repre_dtype": "bfloat16", "retrieval_lag": lag})
    plugin = GSA(cfg, UcmSparseRole.WORKER)
    h = PB.Harness(torch, dev, plugin, caches, PB._prompt_shape(lens), block_lists, 43, with_execute_hooks=True)
    h.step("prefill", {rid: r.num_prompt_tokens for rid, r in h.reqs.items()}, query_rows=16)
    torch.cuda.synchronize()
    q_before, dropped = None, 0
    for step in range(1, 5):
        h.decode_token()
        h.step("decode", {rid: 1 for rid in h.reqs})
        torch.cuda.synchronize()
        qs = [q.float().cpu().numpy() for q in h.last_queries]
        lagged = lag == 1 and step >= 2
        tables = plugin.block_tables_mp.cpu().numpy()
        seq_out = plugin.gsa_seq_len.cpu().numpy()
        for l in range(L):
            table = plugin.kpre_caches[l].float().cpu().numpy()
            for i, rid in enumerate(h.order):
                st = plugin.gsa_stats[rid]
                n = len(block_lists[i])
                q = (q_before if lagged else qs)[l][i]
                k = plugin._topk_len(n)
                want_idx, _ = O.select_topk(q, table[st.slot_offset : st.slot_offset + n].reshape(n, PB.HKV, 1, PB.D), k)
                seq_len = h.reqs[rid].num_computed_tokens          # (the harness has already counted this step's token)
                phys, want_len = O.block_table_gather(block_lists[i], want_idx, seq_len, bs)
                assert seq_out[l, i] == want_len, (step, l, rid)
                assert np.array_equal(tables[l, i, : len(phys)], phys), (step, l, rid)
                dropped += int(len(phys) < n)
        q_before = qs
    assert dropped == 4 * L * n_req
    for rid in list(h.reqs):
        plugin.request_finished_in_worker(rid)


@pytest.mark.parametrize("lag", [0, 1])
def test_gsa_retrieval_stride_reuses_scores(ucm, dev, lag):
    """With retrieval_stride 3 the scores of the last retrieval are re-selected with the current lengths
    on the steps in between (the last two blocks are always kept, so the newest block is never missing);
    a request is scored on its first sparsified step whatever the stride.  With retrieval_lag 1 the queries are kept
    only on the step before a retrieval, and that retrieval (step 3) is the one launch before the model runs."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 64, 1, 16, 64
    cfg = make_config(hq, hkv, d, L, bs, 16 * 40, {"seg_prefill_threshold": 10, "min_topk_len": 5, "max_topk_len": 5,
                                                   "retrieval_stride": 3, "retrieval_lag": lag})
    plugin = GSA(cfg, UcmSparseRole.WORKER)
    cache = torch.randn(2, nb, bs, hkv, d, device=dev).to(torch.bfloat16)
    name = "model.layers.0.self_attn.attn"
    fc = ns(no_compile_layers={name: ns(kv_cache=[cache])}, virtual_engine=0, attn_metadata=None)
    st = ns(block_ids=[list(range(20))], num_computed_tokens=0, prompt_token_ids=[1] * 318, output_token_ids=[])
    ib = ns(req_id_to_index={"A": 0})
    tables, scored = [], []
    for step in range(5):
        n_new = 318 if step == 0 else 1
        if step == 3:
            st.block_ids[0].append(33)  # token 320 opens block 21
        so = ns(num_scheduled_tokens={"A": n_new}, scheduled_new_reqs=[ns(req_id="A")] if step == 0 else [])
        plugin.build_sparse_meta(so, {"A": st}, ib, None)
        plugin.execute_begin(so)
        scored.append(plugin.model_input["is_topk"])
        assert (plugin._lagged is not None) == (lag == 1 and step == 3)
        assert (plugin._parking is not None) == (lag == 1 and step == 2)
        md = ns(block_table=None, seq_lens=None)
        fc.attn_metadata = md
        q = torch.randn(n_new, hq, d, device=dev).to(torch.bfloat16)
        plugin.attention_begin(q, None, None, name, fc)
        plugin.attention_finished(q, None, None, None, name, fc)
        plugin.execute_finished()
        torch.cuda.synchronize()
        st.num_computed_tokens += n_new
        st.output_token_ids.append(1)
        if step > 0:
            cnt = int(plugin.topk_counts[0, 0])
            tables.append((md.block_table[0, :cnt].cpu().tolist(), int(md.seq_lens[0])))
        else:
            assert md.block_table is None  # prefill: the layer's metadata is left alone
    assert scored == [False, True, False, True, False]
    assert tables[0][0] == tables[1][0] and tables[0][0][-2:] == [18, 19]     # step 2 re-selects step 1's scores
    assert tables[2][0][-2:] == [19, 33] and tables[3][0] == tables[2][0]      # the new block is in the local window
    assert all(len(t[0]) == 5 and t[0][0] == 0 for t in tables)
    assert [t[1] for t in tables] == [4 * 16 + 15, 5 * 16, 4 * 16 + 1, 4 * 16 + 2]


def test_gsa_local_window_save_and_restore(ucm, dev):
    """Prefetch mode: at the end of a long request's prefill the last `local` blocks are kept aside, K and V, every
    layer; at its first decode step they are written into the cache blocks that now stand for the window (the last
    `local` entries of remain_idx), whatever those blocks held (gsa.py:956-1031)."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 64, 3, 16, 200
    lo, hi = 6, 10                                              # local window = lo - 1 = 5 blocks
    cfg = make_config(hq, hkv, d, L, bs, 16 * 120, {"seg_prefill_threshold": 100, "min_topk_len": lo, "max_topk_len": hi,
                                                    "ptopk_prefetch_enable": True})
    plugin = GSA(cfg, UcmSparseRole.WORKER)
    caches = [torch.randn(2, nb, bs, hkv, d, device=dev).to(torch.bfloat16) for _ in range(L)]
    plugin.register_kv_caches({f"model.layers.{l}.self_attn.attn": caches[l] for l in range(L)})
    n_blocks = 40
    prompt_len = n_blocks * bs
    prompt_blocks = [int(x) for x in synth.permutation(950, nb)[:n_blocks]]
    short_blocks = [int(x) for x in synth.permutation(951, nb)[100:104]]
    reqs = {"long": ns(block_ids=[prompt_blocks], num_computed_tokens=0, prompt_token_ids=[1] * prompt_len, output_token_ids=[]),
            "short": ns(block_ids=[short_blocks], num_computed_tokens=0, prompt_token_ids=[1] * 60, output_token_ids=[])}
    ib = ns(req_id_to_index={"long": 0, "short": 1})
    so = ns(num_scheduled_tokens={"long": prompt_len, "short": 60}, scheduled_new_reqs=[ns(req_id="long"), ns(req_id="short")])
    plugin.build_sparse_meta(so, reqs, ib, None)
    plugin.execute_begin(so)
    plugin.execute_finished()                                   # the prefill step ends: the window is saved
    st = plugin.gsa_stats["long"]
    assert plugin.gsa_stats["short"].local_window_kv is None and st.local_window_kv.shape[:3] == (lo - 1, L, 2)
    window = [c[:, prompt_blocks[-(lo - 1):]].clone() for c in caches]
    # the scheduler now gives the request its sparse block list: k = compute_topk_len(40) = 10 (the cap) -> 10 + 1
    # sparse blocks, and one more for the token being decoded; everything in the cache is overwritten in between
    sparse_blocks = [int(x) for x in synth.permutation(952, nb)[150:162]]
    for c in caches:
        c.normal_()
    before = [c.clone() for c in caches]
    reqs["long"].block_ids = [sparse_blocks]
    reqs["long"].num_computed_tokens = prompt_len
    reqs["long"].output_token_ids = [1]
    so = ns(num_scheduled_tokens={"long": 1}, scheduled_new_reqs=[])
    plugin.build_sparse_meta(so, reqs, ns(req_id_to_index={"long": 0}), None)
    torch.cuda.synchronize()
    assert st.remain_idx == list(range(5)) + list(range(6, 11)) and st.prefetch_idx == [5]
    target = [sparse_blocks[x] for x in st.remain_idx[-(lo - 1):]]
    for l in range(L):
        assert torch.equal(caches[l][:, target], window[l])
        rest = [b for b in range(nb) if b not in target]
        assert torch.equal(caches[l][:, rest], before[l][:, rest])


# ------------------------------------------------- block store + ESA plugin

def test_hip_block_store_round_trip(ucm, dev):
    """dump / load through the store surface of the reference (one tensor view per block, byte offsets
    inside the stored block) move exactly the bytes, as one batched launch per call."""
    from ucm_amd.sparse.esa.esa import get_offset
    from ucm_amd.store.hip_block_store import FAILURE, SUCCESS, UcmHipBlockStore

    L, nb, bs, hkv, d = 3, 20, 16, 2, 64
    shape = (bs, hkv, d)
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 6 * L * 2 * slice_bytes, "role": "worker"})
    caches = [torch.randn(2, nb, bs, hkv, d, device=dev).to(torch.bfloat16) for _ in range(L)]
    hashes = [f"h{i}" for i in range(6)]
    ids = [3, 17, 0, 9, 11, 5]
    assert store.create(hashes) == [SUCCESS] * 6 and store.create(["overflow"]) == [FAILURE]
    assert store.lookup(hashes) == [False] * 6
    tasks = []
    for l in range(L):
        for kv in range(2):
            off = [get_offset(shape, 0, 1, 2, l, bool(kv))] * 6
            tasks.append(store.dump(hashes, off, [caches[l][kv][i] for i in ids]))
    assert all(store.wait(t) == SUCCESS for t in tasks)
    store.commit(hashes, True)
    assert store.lookup(hashes + ["nope"]) == [True] * 6 + [False]
    # stored-block layout is [layer][K|V] at get_offset, one slot per hash
    buf = store._buffer.view(store.max_block_num, L, 2, slice_bytes)
    for j, i in enumerate(ids):
        for l in range(L):
            for kv in range(2):
                assert torch.equal(buf[store.slot_of[hashes[j]], l, kv], caches[l][kv][i].reshape(-1).view(torch.uint8))
    # load a permuted subset into other cache blocks
    fresh = [torch.zeros_like(c) for c in caches]
    pick, dst = [4, 1, 2], [7, 8, 19]
    tasks = []
    for l in range(L):
        for kv in range(2):
            off = [get_offset(shape, 0, 1, 2, l, bool(kv))] * 3
            tasks.append(store.load([hashes[p] for p in pick], off, [fresh[l][kv][b] for b in dst]))
    assert all(store.check(t)[0] == SUCCESS for t in tasks)
    assert all(store.wait(t) == SUCCESS for t in tasks)
    for l in range(L):
        for kv in range(2):
            for p, b in zip(pick, dst):
                assert torch.equal(fresh[l][kv][b], caches[l][kv][ids[p]])
            rest = [b for b in range(nb) if b not in dst]
            assert not fresh[l][kv][rest].any()
    assert store.wait(store.load(["unknown"], [0], [fresh[0][0][0]])) == FAILURE
    # raw addresses (fetch_data / dump_data): device memory passes, pageable host memory is refused before any launch
    raw = torch.zeros(slice_bytes, dtype=torch.uint8, device=dev)
    assert store.wait(store.fetch_data([hashes[0]], [0], [raw.data_ptr()], [slice_bytes])) == SUCCESS
    assert torch.equal(raw, caches[0][0][ids[0]].reshape(-1).view(torch.uint8))
    pageable = np.zeros(slice_bytes + 64, np.uint8)
    with pytest.raises(ValueError, match="not device or pinned"):
        store.fetch_data([hashes[0]], [0], [pageable.ctypes.data + (-pageable.ctypes.data) % 16], [slice_bytes])
    # a store in pinned host memory behaves the same
    host = UcmHipBlockStore({"kv_block_size": slice_bytes, "max_cache_size": 4 * slice_bytes, "device": "pinned"})
    t = host.dump(["a"], [0], [caches[0][0][2]])
    assert host.wait(t) == SUCCESS
    out = torch.zeros_like(caches[0][0][2])
    assert host.wait(host.load(["a"], [0], [out])) == SUCCESS and torch.equal(out, caches[0][0][2])


def test_esa_plugin_flow(ucm, dev):
    """Prefill + decode of one request through the ESA-shaped plugin: representatives at the last prefill chunk,
    retrieval through the worker, delta loads from the store into the request's first top_k cache blocks."""
    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseRole
    from ucm_amd.sparse.esa.esa import ESA, block_hash_func, get_offset
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 64, 2, 16, 64
    cfg = make_config(hq, hkv, d, L, bs, 16 * 64, {})
    cfg.kv_transfer_config.kv_connector_extra_config = {"ucm_sparse_config": {"ESA": {
        "init_window_sz": 1, "local_window_sz": 2, "min_blocks": 4, "sparse_ratio": 0.3, "retrieval_stride": 5,
        "device_loads": False}}}                             # the per-request path through store.load (any store)
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 40 * L * 2 * slice_bytes})
    plugin = ESA(cfg, UcmSparseRole.WORKER, store=store)
    n_prompt = 20 * bs + 5                                   # 20 full blocks + 5 tokens
    prompt = [int(x) for x in synth.ints(900, n_prompt, 0, 30000)]
    block_ids = [int(x) for x in synth.permutation(901, nb)[:22]]
    req = ns(block_ids=[block_ids], num_computed_tokens=0, prompt_token_ids=prompt, output_token_ids=[],
             num_prompt_tokens=n_prompt, num_output_tokens=0, request_id="A")
    assert plugin.estimate_num_slots_sparsed(req) == INVALID_SLOT          # nothing to sparsify during prefill
    caches = [torch.randn(2, nb, bs, hkv, d, device=dev).to(torch.bfloat16) for _ in range(L)]
    original = [c.clone() for c in caches]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=None)
    ib = ns(req_id_to_index={"A": 0})
    md = ns(query_start_loc=torch.tensor([0, 1]))
    sparse_range, top_k = 19, 5                              # 20 - (local_window_sz - 1); int(19 * 0.3)

    def run_step(n_tok):
        so = ns(num_scheduled_tokens={"A": n_tok})
        plugin.build_sparse_meta(so, {"A": req}, ib, md)
        qs = []
        for l in range(L):
            q = torch.randn(n_tok, hq, d, device=dev).to(torch.bfloat16)
            qs.append(q)
            plugin.attention_begin(q, None, None, names[l], fc)
            plugin.attention_finished(q, None, None, None, names[l], fc)
        req.num_computed_tokens += n_tok
        return qs

    run_step(n_prompt)                                       # prefill: representatives of the first 19 blocks
    torch.cuda.synchronize()
    states = plugin.req_states["A"]
    hashes, parent = [], None
    for b in range(20):
        parent = block_hash_func(parent, tuple(prompt[b * bs : (b + 1) * bs]))
        hashes.append(str(parent))
    assert states[0].block_hashes == hashes and states[0].sparse_range == sparse_range
    rep_h = []
    for l in range(L):
        assert len(states[l].slots) == sparse_range
        kc = original[l][0].view(torch.int16).cpu().numpy().view(np.uint16)
        want = np.zeros((plugin.num_slots, hkv * d), np.float32)
        O.block_mean_paged(kc, block_ids[:sparse_range], states[l].slots, want, round_bf16=True)
        assert np.array_equal(bits(plugin.data[l].cpu().numpy()), bits(want))
        rep_h.append(want)
    # what the prefix-cache connector does after prefill: every full prompt block goes to the store
    for l in range(L):
        for kv in range(2):
            off = [get_offset((bs, hkv, d), 0, 1, 2, l, bool(kv))] * 20
            assert store.wait(store.dump(hashes, off, [caches[l][kv][b] for b in block_ids[:20]])) == 0
    store.commit(hashes)

    def expected_selection(l, q):
        qm = q[0].view(hkv, hq // hkv, d).mean(1).float().reshape(-1).cpu().numpy()   # the plugin's mean is taken in bf16
        idx, _ = O.esa_retrieve(rep_h[l], qm, np.array(states[l].slots, np.int32), top_k)
        return [states[l].slots_to_relative_indexes[int(s)] for s in idx]

    resident = block_ids[:top_k]
    held = [dict() for _ in range(L)]                        # cache block -> logical block it holds after the loads
    for step in range(1, 8):
        req.output_token_ids.append(1)
        req.num_output_tokens = step
        # the retrieval of steps 2 (submitted in attention_finished) is consumed at step 5
        qs = run_step(1)
        torch.cuda.synchronize()
        for l in range(L):
            st = states[l]
            if step == 1:
                want = expected_selection(l, qs[l])
                assert sorted(st.pre_topk_block_hashes.values()) == sorted(hashes[i] for i in want)
                held[l] = {b: hashes.index(h) for b, h in st.pre_topk_block_hashes.items()}
                assert set(held[l]) <= set(resident) and len(st.last_loaded) == top_k
            if step == 2:
                pending_q = qs
                assert st.retrieval_task is not None
            if step == 5:
                want = set(expected_selection(l, pending_q[l]))
                new_held = {b: hashes.index(h) for b, h in st.pre_topk_block_hashes.items()}
                assert set(new_held.values()) == want
                kept = {b for b in new_held if held[l].get(b) == new_held[b]}
                assert {b for b, _ in st.last_loaded} == set(new_held) - kept       # only missing blocks were loaded
                held[l] = new_held
            if step >= 6:
                assert not st.tasks                           # transfers were waited for at step % stride == 1
            if step in (1, 6, 7):
                # the request's first top_k cache blocks hold exactly the selected blocks, K and V
                for b, logical in held[l].items():
                    for kv in range(2):
                        assert torch.equal(caches[l][kv][b], original[l][kv][block_ids[logical]]), (step, l, b)
    assert plugin.estimate_num_slots_sparsed(req) == top_k * bs + (5 + bs * 1 + 7)
    plugin.request_finished_in_worker("A")
    assert "A" not in plugin.req_states and len(plugin.layer_pools[0].allocated) == 0


def test_hip_block_store_spills_to_pinned_host_and_reloads(ucm, dev):
    """A pool of 4 slots in HBM with a tier of 6 pinned buffers behind it: the fifth block pushes the one used longest
    ago out (an asynchronous copy on the store's stream, finished by a callback), loading a spilled block brings it
    back, held blocks stay, and every block reads back the bytes that were dumped."""
    from ucm_amd.store.hip_block_store import FAILURE, SUCCESS, UcmHipBlockStore

    kvb = 2 * 4096
    store = UcmHipBlockStore({"kv_block_size": kvb, "max_cache_size": 4 * kvb, "host_spill_blocks": 6})
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    data = [torch.randint(0, 255, (kvb,), dtype=torch.uint8, device=dev, generator=g) for _ in range(10)]
    names = [f"b{i}" for i in range(10)]

    def put(i):
        assert store.create([names[i]]) == [SUCCESS]
        assert store.wait(store.dump([names[i]], [0], [data[i]])) == SUCCESS
        store.commit([names[i]])

    def get(i):
        out = torch.zeros(kvb, dtype=torch.uint8, device=dev)
        assert store.wait(store.load([names[i]], [0], [out])) == SUCCESS
        return out

    for i in range(4):
        put(i)
    assert store.spills == 0 and store.generation == 0
    assert torch.equal(get(0), data[0])                      # touching b0 makes b1 the coldest
    put(4)
    assert store.spills == 1 and "b1" in store.host_of and "b1" not in store.slot_of and store.generation == 1
    assert store.lookup(names[:5]) == [True] * 5
    held = store.hold(["b2", "b3"])                          # kernels will read these in place: they may not leave
    assert held == [store.slot_of["b2"], store.slot_of["b3"]]
    put(5)
    put(6)
    assert set(store.host_of) == {"b1", "b0", "b4"} and store.spills == 3
    assert store.create(["b7"]) == [FAILURE] or "b7" in store.slot_of   # only b5 / b6 can leave now
    store.release(["b2", "b3"])
    # a spilled block comes back through load (and pushes another one out), bytes intact; so does one through hold
    assert torch.equal(get(1), data[1]) and "b1" in store.slot_of and store.reloads == 1
    slot = store.hold(["b0"])[0]
    assert slot == store.slot_of["b0"] and store.reloads == 2
    pool, _ = store.device_pool()
    torch.cuda.synchronize()
    assert torch.equal(pool[slot * kvb : (slot + 1) * kvb], data[0])
    store.release(["b0"])
    for i in range(7):
        if names[i] in store.slot_of or names[i] in store.host_of:
            assert torch.equal(get(i), data[i]), i
    store._device.Synchronized()
    assert store.spills_done == store.spills                 # every spill's callback has run
    # the tier is bounded too: 4 slots + 6 buffers hold 10 blocks, the eleventh is refused
    for i in range(7, 10):
        put(i)
    assert store.create(["b10"]) == [FAILURE]
