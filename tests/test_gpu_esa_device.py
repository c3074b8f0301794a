"""The ESA plugin's batched device path (retrieve -> delta plan -> planned loads, no host round trip) driven the way
patched vLLM drives the hooks: 16 requests at different stages of their decode in every engine step, 32 layers.
After every step the request's first top_k cache blocks must hold, K and V, exactly the blocks the oracle selects
(orc_esa_retrieve) and places (orc_delta_plan) from the same queries.  Host time of the hooks is printed per kind
of step."""
import time
import types

import numpy as np
import pytest
import torch

import oracle as O
import synth

pytestmark = pytest.mark.gpu

bits = lambda a: np.ascontiguousarray(a, np.float32).view(np.uint32)
ns = types.SimpleNamespace


class _ModelConfig:
    def __init__(self, hq, hkv, d, layers, max_model_len):
        self.hq, self.hkv, self.d, self.layers, self.max_model_len = hq, hkv, d, layers, max_model_len

    def get_num_kv_heads(self, pc):
        return self.hkv

    def get_head_size(self):
        return self.d

    def get_num_layers(self, pc):
        return self.layers


def _config(hq, hkv, d, layers, bs, max_model_len, max_num_seqs, esa_cfg):
    return ns(model_config=_ModelConfig(hq, hkv, d, layers, max_model_len), parallel_config=ns(rank=0, tensor_parallel_size=1),
              cache_config=ns(block_size=bs), scheduler_config=ns(max_num_seqs=max_num_seqs),
              kv_transfer_config=ns(kv_connector_extra_config={"ucm_sparse_config": {"ESA": esa_cfg}}))


@pytest.mark.parametrize("pool_where,model_dtype,churn,serving", [
    ("cuda", "bfloat16", False, False), ("pinned", "bfloat16", False, False), ("cuda", "float16", False, False),
    ("cuda", "bfloat16", True, False), ("cuda", "bfloat16", True, True)])
def test_esa_device_path_flow(ucm, dev, pool_where, model_dtype, churn, serving):
    """churn: three requests finish before step 7 and three others start at step 8, in the table rows, representative
    slots and batch positions the first three gave back.  serving: Llama-3-8B's head shape and blocks of 128 tokens
    (eight layers), instead of the small shape the other cases run in 32 layers."""
    from ucm_amd import ops
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.esa.esa import ESA
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    hq, hkv, d, L, bs = (32, 8, 128, 8, 128) if serving else (8, 2, 64, 32, 16)
    n_req = 16 if pool_where == "cuda" else 5
    nb = 2048
    stride_cfg = 5
    max_blocks = 128 if pool_where == "cuda" else 400        # 38 sparse slots at most (one wave plans them) / 120 (a workgroup)
    cfg = _config(hq, hkv, d, L, bs, max_blocks * bs, 24, {"init_window_sz": 1, "local_window_sz": 2, "min_blocks": 4,
                                                     "sparse_ratio": 0.3, "retrieval_stride": stride_cfg})
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 1800 * L * 2 * slice_bytes,
                              "device": pool_where})
    plugin = ESA(cfg, UcmSparseRole.WORKER, store=store)
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    model_dtype = getattr(torch, model_dtype)       # the cache's and the queries' type: the means are rounded to it
    caches = [torch.randn(2, nb, bs, hkv, d, device=dev, generator=g).to(model_dtype) for _ in range(L)]
    original = [c.clone() for c in caches]
    all_layers = ops.LayerPointers(caches)
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=None)

    # requests: different prompt lengths, each starting its prefill at a different engine step
    perm = synth.permutation(77, nb)
    reqs, used = {}, 0
    late = 3 if churn else 0
    for i in range(n_req + late):
        n_blocks = int(synth.ints(300 + i, 1, 12, 100)[0])
        if churn and i in (3, n_req + 1):                    # two short ones: 3 and 5 blocks (min_blocks is 4)
            n_blocks = 3 if i == 3 else 5
        n_prompt = n_blocks * bs + (0 if i % 3 == 0 else int(synth.ints(400 + i, 1, 1, bs - 1)[0]))
        total = n_blocks + 3
        ids = [int(x) for x in perm[used : used + total]]
        used += total
        prompt = [int(x) for x in synth.ints(500 + i, n_prompt, 0, 30000)]
        reqs[f"r{i}"] = ns(request_id=f"r{i}", block_ids=[ids], num_computed_tokens=0, prompt_token_ids=prompt,
                           output_token_ids=[], num_prompt_tokens=n_prompt, start=i % 4 if i < n_req else 8, index=i,
                           done=False)
    assert used <= nb

    # host model of every (request, layer)
    model, keys_h = {}, {}
    host_ms = {"prefill": [], "first": [], "retrieve": [], "load": [], "idle": []}

    def engine_step(t):
        active = [r for r in reqs.values() if r.start <= t and not r.done]
        sched, qsl, pos = {}, [], 0
        for r in active:
            n_tok = r.num_prompt_tokens if r.num_computed_tokens == 0 else 1
            sched[r.request_id] = n_tok
            qsl.append(pos)
            pos += n_tok
        ib = ns(req_id_to_index={r.request_id: j for j, r in enumerate(active)})
        md = ns(query_start_loc=torch.tensor(qsl + [pos]))
        so = ns(num_scheduled_tokens=sched)
        qs = [torch.randn(pos, hq, d, device=dev, generator=g).to(model_dtype) for _ in range(L)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        plugin.build_sparse_meta(so, {r.request_id: r for r in active}, ib, md)
        for l in range(L):
            plugin.attention_begin(qs[l], None, None, names[l], fc)
            plugin.attention_finished(qs[l], None, None, None, names[l], fc)
        host = (time.perf_counter() - t0) * 1e3
        torch.cuda.synchronize()
        p = plugin._dev.plan
        kind = ("prefill" if p.prefill is not None else "first" if p.n_first else "load" if p.n_load else
                "retrieve" if p.n_retrieve else "idle")
        host_ms[kind].append(host)
        return active, qsl, qs

    def expected_selection(m, l, q_tok):
        qm = q_tok.view(hkv, hq // hkv, d).mean(1).float().reshape(-1).cpu().numpy()      # the plugin's mean is taken in bf16
        idx, _ = O.esa_retrieve(m["rep"][l], qm, np.array(m["slots"][l], np.int32), m["top_k"])
        pos_of = {s: i for i, s in enumerate(m["slots"][l])}
        return np.array([pos_of[int(s)] for s in idx], np.int32)

    def check_caches(r, m):
        ids = r.block_ids[0]
        dst = torch.tensor(ids[: m["top_k"]], device=dev)
        for l in range(L):
            res = m["resident"][l]
            held = res >= 0
            if not held.any():
                continue
            src = torch.tensor([ids[b] for b in res[held]], device=dev)
            got = caches[l].index_select(1, dst[torch.from_numpy(held).to(dev)])
            assert torch.equal(got, original[l].index_select(1, src)), (r.request_id, l)

    n_steps = 14
    for t in range(n_steps):
        if churn and t == 7:
            for rid in ("r0", "r5", "r10"):
                plugin.request_finished_in_worker(rid)
                reqs[rid].done = True
            assert len(plugin._dev.tables.free_rows) == 24 - sum(1 for r in reqs.values() if r.start < 7 and not r.done and r.num_prompt_tokens >= 4 * bs)
        active, qsl, qs = engine_step(t)
        for j, r in enumerate(active):
            rid = r.request_id
            if r.num_computed_tokens == 0:
                # ---- the prefill step just ran: the plugin wrote the representatives
                if r.num_prompt_tokens < 4 * bs:             # below min_blocks: the plugin leaves the request alone
                    assert rid not in plugin._dev.reqs
                    model[rid] = dict(top_k=0)
                    r.num_computed_tokens = r.num_prompt_tokens
                    r.output_token_ids.append(1)
                    continue
                st = plugin._dev.reqs[rid]
                n_full = r.num_prompt_tokens // bs
                sparse_range = n_full - (2 if r.num_prompt_tokens % bs == 0 else 1)
                top_k = int(sparse_range * 0.3)
                assert (st.sparse_range, st.top_k, st.n_repre) == (sparse_range, top_k, sparse_range)
                m = dict(top_k=top_k, slots=[list(s) for s in st.slots], rep=[], sel=[None] * L,
                         resident=[np.full(top_k, -1, np.int32) for _ in range(L)])
                ids = r.block_ids[0]
                for l in range(L):
                    if l not in keys_h:                    # (a layer's keys as the oracle reads them, fetched once)
                        keys_h[l] = original[l][0].view(torch.int16).cpu().numpy().view(np.uint16)
                    kc = keys_h[l]
                    want = np.zeros((plugin.num_slots, hkv * d), np.float32)
                    O.block_mean_paged(kc, ids[:sparse_range], m["slots"][l], want, round_bf16=True,
                                       keys_f16=(model_dtype == torch.float16))
                    got = plugin.data[l][m["slots"][l]].cpu().numpy()
                    assert np.array_equal(bits(got), bits(want[m["slots"][l]])), (rid, l)
                    m["rep"].append(want)
                model[rid] = m
                # what the prefix-cache connector does after prefill: every full prompt block goes to the store
                hashes = st.block_hashes
                assert len(hashes) == n_full
                assert store.create(hashes) == [0] * n_full
                slots = [store.slot_of[h] for h in hashes]
                assert slots == list(range(slots[0], slots[0] + n_full))
                pool, kvb = store.device_pool()
                ops.kv_gather_blocks(all_layers, caches[0].stride(0) * 2, slice_bytes, nb,
                                     torch.tensor(ids[:n_full], dtype=torch.int32, device=dev), pool[slots[0] * kvb :])
                store.commit(hashes)
                torch.cuda.synchronize()
                r.num_computed_tokens = r.num_prompt_tokens
                r.output_token_ids.append(1)
                continue
            m, step = model[rid], len(r.output_token_ids)
            if m["top_k"] > 0:
                retrieve_now = step == 1 or step % stride_cfg == 2 % stride_cfg
                load_now = step == 1 or (step % stride_cfg == 0 and m["sel"][0] is not None)
                for l in range(L):
                    if retrieve_now:
                        m["sel"][l] = expected_selection(m, l, qs[l][qsl[j]])
                    if load_now:
                        O.delta_plan(m["sel"][l], m["sel"][l], m["resident"][l])
                if load_now:
                    for l in range(L):
                        assert sorted(m["resident"][l].tolist()) == sorted(m["sel"][l].tolist())
                    m["sel"] = [None] * L
                check_caches(r, m)
            r.num_computed_tokens += 1
            r.output_token_ids.append(1)
    # every kind of step was seen; everything outside the requests' sparse slots is untouched
    # (a step is named for the first kind of work it holds; with late arrivals some kinds are never alone in a step)
    assert all(host_ms[k] for k in (("prefill", "first") if churn else ("prefill", "first", "retrieve", "load")))
    touched = torch.zeros(nb, dtype=torch.bool, device=dev)
    for rid, m in model.items():
        touched[torch.tensor(reqs[rid].block_ids[0][: m["top_k"]], dtype=torch.long, device=dev)] = True
    for l in range(L):
        assert torch.equal(caches[l][:, ~touched], original[l][:, ~touched])
    print("\nESA device path, %d requests x %d layers, host ms per engine step (hooks only): " % (n_req, L) +
          ", ".join(f"{k} {np.median(v):.2f} (n={len(v)})" for k, v in host_ms.items() if v))
    assert len(plugin._dev.reqs) == sum(1 for r in reqs.values() if not r.done and r.num_prompt_tokens >= 4 * bs)
    for rid, r in reqs.items():
        if not r.done:
            plugin.request_finished_in_worker(rid)
    assert not plugin._dev.reqs and len(plugin.layer_pools[0].allocated) == 0
    assert len(plugin._dev.tables.free_rows) == 24


def test_esa_device_path_store_hole(ucm, dev):
    """The store lacks every other prompt block when the first load is due: the load leaves them out and says so (a
    warning, a counter); once they are there, the plugin finds them, forgets what it believed resident and the next
    load brings every selected block in - after which the cache holds what the resident lists say."""
    from ucm_amd import ops
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.esa.esa import ESA
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    hq, hkv, d, L, bs, nb, stride = 8, 2, 64, 2, 16, 128, 5
    cfg = _config(hq, hkv, d, L, bs, 64 * bs, 4, {"init_window_sz": 1, "local_window_sz": 2, "min_blocks": 4,
                                                 "sparse_ratio": 0.3, "retrieval_stride": stride})
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 64 * L * 2 * slice_bytes})
    plugin = ESA(cfg, UcmSparseRole.WORKER, store=store)
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    caches = [torch.randn(2, nb, bs, hkv, d, device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    original = [c.clone() for c in caches]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=None)
    n_full = 40
    ids = [int(x) for x in synth.permutation(78, nb)[: n_full + 3]]
    req = ns(request_id="h", block_ids=[ids], num_computed_tokens=0, output_token_ids=[], num_prompt_tokens=n_full * bs + 3,
             prompt_token_ids=[int(x) for x in synth.ints(501, n_full * bs + 3, 0, 30000)])

    def engine_step():
        n_tok = req.num_prompt_tokens if req.num_computed_tokens == 0 else 1
        md = ns(query_start_loc=torch.tensor([0, n_tok]))
        plugin.build_sparse_meta(ns(num_scheduled_tokens={"h": n_tok}), {"h": req}, ns(req_id_to_index={"h": 0}), md)
        for l in range(L):
            q = torch.randn(n_tok, hq, d, device=dev, generator=g).to(torch.bfloat16)
            plugin.attention_begin(q, None, None, names[l], fc)
            plugin.attention_finished(q, None, None, None, names[l], fc)
        torch.cuda.synchronize()
        req.num_computed_tokens += n_tok
        req.output_token_ids.append(1)

    def to_store(which):
        hashes = plugin._dev.reqs["h"].block_hashes
        some = [hashes[i] for i in which]
        assert store.create(some) == [0] * len(some)
        pool, kvb = store.device_pool()
        for i, h in zip(which, some):
            ops.kv_gather_blocks(ops.LayerPointers(original), original[0].stride(0) * 2, slice_bytes, nb,
                                 torch.tensor([ids[i]], dtype=torch.int32, device=dev), pool[store.slot_of[h] * kvb :])
        store.commit(some)
        torch.cuda.synchronize()

    def held_blocks_match():
        st, t = plugin._dev.reqs["h"], plugin._dev.tables
        for l in range(L):
            res = t.resident[l, st.row, : st.top_k].cpu().numpy()
            assert (res >= 0).all()
            for j, b in enumerate(res):
                if not torch.equal(caches[l][:, ids[j]], original[l][:, ids[int(b)]]):
                    return False
        return True

    engine_step()                                            # prefill: representatives
    late = list(range(0, n_full, 2))
    to_store([i for i in range(n_full) if i not in late])
    st = plugin._dev.reqs["h"]
    n_late = len([i for i in late if i < st.sparse_range])
    with pytest.warns(RuntimeWarning, match="does not hold"):
        engine_step()                                        # decode step 1: retrieve, plan, load - with holes
    assert plugin.load_misses == n_late and not st.src_ready and st.skipped
    assert not held_blocks_match()                           # (blocks were left out; the lists say they are there)
    to_store(late)
    for step in range(2, 2 * stride + 1):                    # retrieval at step 2 and 7, loads at 5 and 10
        engine_step()
        if step == 2:
            assert st.src_ready and not st.skipped and plugin.load_misses == n_late
            assert int((plugin._dev.tables.resident[:, st.row] >= 0).sum()) == 0
        if step in (stride, 2 * stride):
            assert held_blocks_match()
    plugin.request_finished_in_worker("h")
