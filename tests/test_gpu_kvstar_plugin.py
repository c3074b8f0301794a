"""KVStarMultiStep host layer: the reference's hook sequence on stand-in vLLM objects, selections against the CPU oracle."""
import math
import types

import numpy as np
import pytest
import torch

import oracle as O
import synth
from test_gpu_host_layer import make_config
from test_gpu_kvstar import VOTE_ATOL, VOTE_RTOL, check_selection

pytestmark = pytest.mark.gpu


def bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("prune_ratio,chunks,batched,device_loads,device_plans,hole,model", [
    (1.0, 1, True, True, True, False, "bfloat16"), (0.5, 3, True, False, True, False, "bfloat16"),
    (0.25, 1, False, True, True, False, "bfloat16"), (0.25, 1, True, False, False, False, "bfloat16"),
    (0.25, 1, True, True, False, False, "bfloat16"), (0.5, 3, True, True, True, False, "bfloat16"),
    (0.25, 1, True, True, True, True, "bfloat16"), (0.25, 1, False, True, True, True, "bfloat16"),
    (0.25, 1, True, True, False, True, "bfloat16"), (0.25, 1, True, True, True, "spill", "bfloat16"),
    (0.25, 1, False, True, True, "spill", "bfloat16"), (0.25, 1, True, True, False, "spill", "bfloat16"),
    (0.25, 1, True, True, True, False, "float16"), (1.0, 3, False, True, True, False, "float16")])
def test_kvstar_plugin_flow(ucm, dev, prune_ratio, chunks, batched, device_loads, device_plans, hole, model):
    """Prefill (one chunk, or three) of 24 full blocks + 5 tokens, then 13 decode steps with stride 4: step 1 restores
    the windows and loads what the prefill group's vote picks; the vote of decode steps 1-4 is queued at step 4 and
    its winners are loaded at step 8; steps 5-8 at step 8 / 12.  Selections are checked against the CPU oracle on the
    same keys and queries.  ``hole``: at the first load the store lacks some of the prompt's blocks - the load leaves them
    out, says so (a warning, a counter) and looks again at the next load, by which time they have arrived.  ``hole ==
    "spill"``: the store's pool is smaller than the prompt and has pinned host memory behind it - the blocks a load may
    ask for come back into the pool when the request first loads, and stay.  ``model``: the type of the cache and of the
    queries (a float16 model's representatives are rounded once, to float16)."""
    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseRole
    from ucm_amd.sparse.factory import UcmSparseFactory
    from ucm_amd.sparse.kvstar.multistep import KVStarMultiStep
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 128, 2, 16, 80
    stride, merge, ratio = 4, 4, 0.25
    cfg = make_config(hq, hkv, d, L, bs, 16 * 64, {})
    cfg.kv_transfer_config.kv_connector_extra_config = {"ucm_sparse_config": {"KVStarMultiStep": {
        "retrieval_stride": stride, "sparse_ratio": ratio, "blk_repre_dim_prune_ratio": prune_ratio,
        "blk_repre_inner_token_merge": merge, "batch_retrieval": batched, "device_loads": device_loads,
        "device_plans": device_plans}}}
    slice_bytes = bs * hkv * d * 2
    spill, hole = hole == "spill", hole is True
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": (22 if spill else 40) * L * 2 * slice_bytes,
                              "host_spill_blocks": 8 if spill else 0})
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    assert isinstance(plugin, KVStarMultiStep)
    plugin.connector = store

    n_full, n_prompt = 24, 24 * bs + 5
    tokens = [int(t) for t in synth.permutation(1400, 1000)[:n_prompt]]
    full_ids = [int(x) + 2 for x in synth.permutation(1401, nb - 2)[:25]]   # vLLM block ids (0 and 1 stay unused)
    req = ns(block_ids=[list(full_ids)], num_computed_tokens=0, prompt_token_ids=tokens, output_token_ids=[],
             num_prompt_tokens=n_prompt, num_output_tokens=0, num_tokens=n_prompt, request_id="7")
    g = torch.Generator(device=dev)
    g.manual_seed(21)
    model = getattr(torch, model)
    caches = [(torch.randn(2, nb, bs, hkv, d, device=dev, generator=g) * 0.3).to(model) for _ in range(L)]
    original = [c.clone() for c in caches]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    ib = ns(req_id_to_index={"7": 0})

    def run_step(n_tok):
        so = ns(num_scheduled_tokens={"7": n_tok}, req_sparsed_slots={"7": 0})
        md = ns(query_start_loc=torch.tensor([0, n_tok]))
        fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=md)
        plugin.build_sparse_meta(so, {"7": req}, ib, md)
        qs = []
        for l in range(L):
            q = (torch.randn(n_tok, hq, d, device=dev, generator=g) * 0.3).to(model)
            qs.append(q)
            plugin.attention_begin(q, None, None, names[l], fc)
            plugin.attention_finished(q, None, None, None, names[l], fc)
        req.num_computed_tokens += n_tok
        return qs

    # ---- prefill; the last `stride` prompt tokens' queries form the "prefill" group
    sizes = [n_prompt] if chunks == 1 else [200, n_prompt - 200 - 3, 3]
    prompt_q = [[] for _ in range(L)]
    for n_tok in sizes:
        for l, q in enumerate(run_step(n_tok)):
            prompt_q[l].append(q)
    groups = {"prefill": [torch.cat(prompt_q[l])[-stride:] for l in range(L)]}
    states = plugin.req_states["7"]
    hashes = states[0].block_hashes
    assert len(hashes) == n_full and hashes == states[1].block_hashes

    # what the connector does in a deployment: the prompt's full blocks are in the store under their chained hashes
    from ucm_amd.sparse.esa.esa import get_offset

    def to_store(which):
        some = [hashes[i] for i in which]
        assert store.create(some) == [0] * len(some)
        for l in range(L):
            for kv in range(2):
                off = get_offset((bs, hkv, d), 0, 1, 2, l, bool(kv))
                store.wait(store.dump(some, [off] * len(some), [original[l][kv][full_ids[i]] for i in which]))
        store.commit(some)

    late = list(range(1, n_full - 2, 2)) if hole else []     # every other block between the windows arrives late
    if spill:                                                # 24 blocks into 22 slots: the two stored first leave the pool
        to_store(list(range(12)))
        to_store(list(range(12, n_full)))
        assert store.spills == 2 and set(store.host_of) == {hashes[0], hashes[1]}
    else:
        to_store([i for i in range(n_full) if i not in late])

    # representatives: blocks 1 .. 21 (init window 1, local window 2), against the oracle on the same keys
    want_repre, pruned = [], []
    for l in range(L):
        st = states[l]
        dp = round(d * prune_ratio)
        assert st.blk_repre.shape == (n_full - 3, bs // merge, hkv, dp)
        pr = None if prune_ratio >= 0.98 else st.d_pruned_index.cpu().numpy().astype(np.int32)
        w = np.zeros((n_full, bs // merge, hkv, (dp + 15) // 16 * 16), np.uint16)
        O.kvstar_block_repre(bits(original[l][0]), np.array(full_ids[:n_full], np.int32), np.arange(n_full, dtype=np.int32), merge, w,
                             pruned=pr, keys_f16=(model == torch.float16))
        assert np.array_equal(bits(st.blk_repre.dense()), w[1:-2][..., :dp])
        want_repre.append(w[1:-2])
        pruned.append(pr)
        assert torch.equal(st.init_window[0], original[l][0][full_ids[:1]])
        assert torch.equal(st.local_window[1], original[l][1][full_ids[-2:]])

    # ---- the scheduler shrinks the request: init + ceil(21 * 0.25) = 6 candidates + local 2 + the tail block
    req.output_token_ids.append(1)
    req.num_output_tokens, req.num_tokens = 1, n_prompt + 1
    slots = plugin.estimate_num_slots_sparsed(req)
    n_keep = math.ceil((n_full - 3) * ratio)
    assert slots == (1 + n_keep + 2) * bs + 6
    kept = full_ids[-math.ceil(slots / bs):]
    assert len(kept) == 1 + n_keep + 2 + 1
    req.block_ids = [list(kept)]
    for l in range(L):                                       # what was in the kept blocks is stale now
        caches[l][:, kept[:-1]] = 0

    def expect(record, l):
        qg = groups[record][l].to(torch.float16)
        dp = round(d * prune_ratio)
        _, votes = O.kvstar_retrieve(bits(qg), want_repre[l], n_keep, pruned=pruned[l], d_pruned=dp)
        return votes

    def check_loaded(record, l, absent=(), before=None):
        st = states[l]
        # with the loads planned on the device nobody has read the list yet; looking at it fetches the host copy
        assert (record in st.step_group_retrieve_indices) == (not (device_loads and device_plans))
        chosen = st.step_group_retrieve_indices[record]
        votes = expect(record, l)
        check_selection(chosen, votes, n_keep)
        assert all(votes[a] >= votes[b] - (VOTE_ATOL + VOTE_RTOL * abs(votes[b]) * 4) for a, b in zip(chosen, chosen[1:]))
        assert st.step_group_retrieve_result[record] == [hashes[i + 1] for i in chosen]
        for kv in range(2):                                  # candidate block j holds the j-th winner, K and V
            got = caches[l][kv][kept[1 : 1 + n_keep]]
            want = original[l][kv][[full_ids[i + 1] for i in chosen]]
            if absent:                                       # a block the store lacked: the cache block keeps what it held
                for j, i in enumerate(chosen):
                    if i + 1 in absent:
                        want[j] = before[l][kv][kept[1 + j]]
            assert torch.equal(got, want), (record, l, kv)

    decode_q = {l: [] for l in range(L)}
    for step in range(1, 14):
        if step > 1:
            req.output_token_ids.append(1)
            req.num_output_tokens, req.num_tokens = step, n_prompt + step
        before = [c.clone() for c in caches]
        if hole and step == 1:
            with pytest.warns(RuntimeWarning, match="does not hold"):
                qs = run_step(1)
            assert plugin.load_misses >= 1
        else:
            qs = run_step(1)
        if hole and step == 1:
            to_store(late)
            seen = plugin.load_misses
        for l, q in enumerate(qs):
            decode_q[l].append(q[0])
        if step % stride == 0:
            groups["decode" + str(step - stride + 1)] = [torch.stack(decode_q[l][-stride:]) for l in range(L)]
        torch.cuda.synchronize()
        for l in range(L):
            st = states[l]
            if step == 1:
                st.wait_for_blk_transfer_task_done()
                check_loaded("prefill", l, late, before)
                for kv in range(2):                          # windows written back around the candidates
                    assert torch.equal(caches[l][kv][kept[0]], original[l][kv][full_ids[0]])
                    assert torch.equal(caches[l][kv][kept[-2:]], original[l][kv][full_ids[-2:]])
            if step == 4:
                assert "decode1" in st.task_waiter and "decode1" not in st.step_group_retrieve_result
            if step == 8:                                    # attention_finished of step 8 collects decode1 and loads it
                st.wait_for_blk_transfer_task_done()
                check_loaded("decode1", l)
                assert "decode5" in st.task_waiter
            if step == 12:
                st.wait_for_blk_transfer_task_done()
                check_loaded("decode5", l)
            if step in (9, 13):
                assert not st.blk_trans_tasks                # waited for at the first step of a stride
    if hole:
        assert plugin.load_misses == seen                    # nothing was missing any more at the later loads
    if spill:
        assert plugin.load_misses == 0
        if device_plans:                                     # (the lists stay on the device: every block a list may name was held)
            assert store.reloads >= 1 and hashes[1] in store.slot_of
    plugin.request_finished_in_worker("7")
    assert "7" not in plugin.req_states


def kvstar_serving_scenario(dev, overrides, n_steps, timing):
    """16 requests of 32-200 prompt blocks, 32 layers: one prefill step for all, then n_steps decode steps with the
    reference's stride of 8 (votes queued at steps 8 and 16, the first decode group's winners loaded at 16).
    Returns a position-weighted checksum of every layer's cache after steps 1, 8, 16 and the last one, and every
    request's chosen lists of layer 0 and the last layer.  Request 5 finishes after step 12, between the queueing of its
    votes and their load, so the load of step 16 follows 15 of the 16 rows of the launch that produced the lists."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.esa.esa import get_offset
    from ucm_amd.sparse.factory import UcmSparseFactory
    from ucm_amd.store.hip_block_store import UcmHipBlockStore
    import time

    from ucm_amd.sparse.kvstar import retrieve as kvstar_retrieve

    tasks_before = len(kvstar_retrieve._tasks)
    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, R = 32, 8, 128, 32, 16, 16
    lens = [32 + (37 * r * 13) % 169 for r in range(R)]
    nb = sum(lens) + R + 8
    cfg = make_config(hq, hkv, d, L, bs, 16 * 256, {})
    settings = {"retrieval_stride": 8, "sparse_ratio": 0.25, "blk_repre_dim_prune_ratio": 0.25, "blk_repre_inner_token_merge": 2}
    settings.update(overrides)
    cfg.kv_transfer_config.kv_connector_extra_config = {"ucm_sparse_config": {"KVStarMultiStep": settings}}
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": nb * L * 2 * slice_bytes})
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    plugin.connector = store
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    caches = [(torch.randn(2, nb, bs, hkv, d, device=dev, generator=g) * 0.3).to(torch.bfloat16) for _ in range(L)]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    reqs, first = {}, 2
    for r in range(R):
        n_prompt = lens[r] * bs + 5
        ids = list(range(first, first + lens[r] + 1))
        first += lens[r] + 1
        reqs[str(r)] = ns(block_ids=[ids], num_computed_tokens=0, prompt_token_ids=[int(t) for t in synth.permutation(1400 + r, 100000)[:n_prompt]],
                          output_token_ids=[], num_prompt_tokens=n_prompt, num_output_tokens=0, num_tokens=n_prompt, request_id=str(r),
                          full_ids=ids)
    ib = ns(req_id_to_index={str(r): r for r in range(R)})

    active = list(range(R))

    def run_step(n_toks, label):
        so = ns(num_scheduled_tokens={str(r): n_toks[r] for r in active}, req_sparsed_slots={str(r): 0 for r in active})
        starts = [0] * (R + 1)
        for r in range(R):
            starts[r + 1] = starts[r] + (n_toks[r] if r in active else 0)
        md = ns(query_start_loc=torch.tensor(starts))
        fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=md)
        q = (torch.randn(starts[-1], hq, d, device=dev, generator=g) * 0.3).to(torch.bfloat16)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        plugin.build_sparse_meta(so, reqs, ib, md)
        for l in range(L):
            plugin.attention_begin(q, None, None, names[l], fc)
            plugin.attention_finished(q, None, None, None, names[l], fc)
        timing.setdefault(label, []).append(1e3 * (time.perf_counter() - t0))
        torch.cuda.synchronize()
        for r in active:
            reqs[str(r)].num_computed_tokens += n_toks[r]

    def digest():
        weights = None
        out = []
        for c in caches:
            flat = c.view(torch.int16).reshape(-1).to(torch.int64)
            if weights is None:
                weights = torch.arange(flat.numel(), device=dev) % 65521 + 1
            out.append(int((flat * weights).sum()))
        return out

    run_step([reqs[str(r)].num_prompt_tokens for r in range(R)], "prefill")
    for r in range(R):                                   # the connector's part: the prompt's blocks under their hashes
        hashes = plugin.req_states[str(r)][0].block_hashes
        assert store.create(hashes) == [0] * len(hashes)
        for l in range(L):
            for kv in range(2):
                off = get_offset((bs, hkv, d), 0, 1, 2, l, bool(kv))
                store.wait(store.dump(hashes, [off] * len(hashes), [caches[l][kv][i] for i in reqs[str(r)].full_ids[: len(hashes)]]))
        store.commit(hashes)
    for r in range(R):                                   # the scheduler shrinks every request
        req = reqs[str(r)]
        req.output_token_ids.append(1)
        req.num_output_tokens, req.num_tokens = 1, req.num_prompt_tokens + 1
        req.block_ids = [req.full_ids[-math.ceil(plugin.estimate_num_slots_sparsed(req) / bs):]]
        for l in range(L):
            caches[l][:, req.block_ids[0][:-1]] = 0
    digests, chosen = {}, {}
    for step in range(1, n_steps + 1):
        if step == 13:
            plugin.request_finished_in_worker("5")
            active.remove(5)
        if step > 1:
            for r in active:
                req = reqs[str(r)]
                req.output_token_ids.append(1)
                req.num_output_tokens, req.num_tokens = step, req.num_prompt_tokens + step
        kind = "first decode" if step == 1 else "queue + load" if step % 8 == 0 and step >= 16 else "queue" if step % 8 == 0 else "plain"
        run_step([1] * R, kind)
        if step in (1, 8, 16, n_steps):
            for r in active:
                for st in (plugin.req_states[str(r)][0], plugin.req_states[str(r)][L - 1]):
                    st.wait_for_blk_transfer_task_done()
            torch.cuda.synchronize()
            digests[step] = digest()
        if step in (1, 16):
            record = "prefill" if step == 1 else "decode1"
            chosen[step] = [[list(plugin.req_states[str(r)][l].step_group_retrieve_indices[record]) for l in (0, L - 1)] for r in active]
    for r in active:                                     # every request ends: no retrieval task is left behind
        plugin.request_finished_in_worker(str(r))
    assert len(kvstar_retrieve._tasks) == tasks_before and not plugin.req_states
    return digests, chosen


def test_kvstar_plugin_at_serving_size(ucm, dev):
    """The device path (loads planned from the device's own lists, window and standby copies once per layer) against
    the host path behind the same batched retrievals (every list read back, two store.load calls per request and
    layer): the same lists and the same bytes in every cache of every layer.  The reference's flow (one retrieval per
    request and layer as well) runs a launch of its own per request, whose votes may differ from the batched launch's
    in the last bits and swap two near-equal blocks of a list, so it is only timed here; the host time of the hooks
    is printed for all three."""
    t_dev, t_host, t_ref = {}, {}, {}
    got = kvstar_serving_scenario(dev, {}, 17, t_dev)
    torch.cuda.empty_cache()
    want = kvstar_serving_scenario(dev, {"device_loads": False, "device_plans": False}, 17, t_host)
    assert got[1] == want[1]
    assert got[0] == want[0]
    torch.cuda.empty_cache()
    kvstar_serving_scenario(dev, {"batch_retrieval": False, "device_loads": False, "device_plans": False}, 17, t_ref)
    for kind in t_dev:
        print(f"KVStar hooks, 16 requests x 32 layers, {kind}: {np.median(t_dev[kind]):.1f} ms of host time per step "
              f"(lists on the host {np.median(t_host[kind]):.1f} ms, the reference's flow {np.median(t_ref[kind]):.1f} ms)")


@pytest.mark.parametrize("n_full", [2, 3, 4])
def test_kvstar_windows_of_a_short_request(ucm, dev, n_full):
    """A prompt of two to four full blocks and a few tokens - no more blocks than the init and local windows cover, so
    nothing lies between them to choose from: prefill, the scheduler's shrink and the first decode step through the
    batched path (one launch for all window copies) and through the per-request path (torch's indexed assignments, one
    after the other) leave the same bytes in every cache, and the request's last two blocks hold its local window."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.factory import UcmSparseFactory
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 128, 2, 16, 24
    n_prompt = n_full * bs + 5
    full_ids = [int(x) + 2 for x in synth.permutation(1410 + n_full, nb - 2)[: n_full + 1]]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    results = []
    for device_loads in (True, False):
        cfg = make_config(hq, hkv, d, L, bs, 16 * 64, {})
        cfg.kv_transfer_config.kv_connector_extra_config = {"ucm_sparse_config": {"KVStarMultiStep": {
            "retrieval_stride": 4, "sparse_ratio": 0.25, "blk_repre_dim_prune_ratio": 1.0, "blk_repre_inner_token_merge": 4,
            "device_loads": device_loads, "device_plans": device_loads}}}
        slice_bytes = bs * hkv * d * 2
        plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
        plugin.connector = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 16 * L * 2 * slice_bytes})
        g = torch.Generator(device=dev)
        g.manual_seed(33)
        caches = [(torch.randn(2, nb, bs, hkv, d, device=dev, generator=g) * 0.3).to(torch.bfloat16) for _ in range(L)]
        original = [c.clone() for c in caches]
        req = ns(block_ids=[list(full_ids)], num_computed_tokens=0, prompt_token_ids=list(range(7, 7 + n_prompt)), output_token_ids=[],
                 num_prompt_tokens=n_prompt, num_output_tokens=0, num_tokens=n_prompt, request_id="9")
        ib = ns(req_id_to_index={"9": 0})

        def run_step(n_tok):
            so = ns(num_scheduled_tokens={"9": n_tok}, req_sparsed_slots={"9": 0})
            md = ns(query_start_loc=torch.tensor([0, n_tok]))
            fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=md)
            plugin.build_sparse_meta(so, {"9": req}, ib, md)
            for l in range(L):
                q = (torch.randn(n_tok, hq, d, device=dev, generator=g) * 0.3).to(torch.bfloat16)
                plugin.attention_begin(q, None, None, names[l], fc)
                plugin.attention_finished(q, None, None, None, names[l], fc)
            req.num_computed_tokens += n_tok

        run_step(n_prompt)
        hashes = plugin.req_states["9"][0].block_hashes
        store = plugin.connector
        assert store.create(hashes) == [0] * len(hashes)
        from ucm_amd.sparse.esa.esa import get_offset
        for l in range(L):
            for kv in range(2):
                off = get_offset((bs, hkv, d), 0, 1, 2, l, bool(kv))
                store.wait(store.dump(hashes, [off] * len(hashes), [original[l][kv][full_ids[i]] for i in range(len(hashes))]))
        store.commit(hashes)
        req.output_token_ids.append(1)
        req.num_output_tokens, req.num_tokens = 1, n_prompt + 1
        slots = plugin.estimate_num_slots_sparsed(req)
        kept = full_ids[-math.ceil(slots / bs):] if slots > 0 else list(full_ids)
        req.block_ids = [list(kept)]
        run_step(1)
        torch.cuda.synchronize()
        for l in range(L):
            plugin.req_states["9"][l].wait_for_blk_transfer_task_done()
        torch.cuda.synchronize()
        results.append((kept, [c.clone() for c in caches], original))
    (kept_a, caches_a, original), (kept_b, caches_b, _) = results
    assert kept_a == kept_b
    for l in range(L):
        assert torch.equal(caches_a[l], caches_b[l]), l
        # the request's last two blocks hold the local window, whatever else the list is short for
        n_local = min(2, len(kept_a))
        want = original[l][:, full_ids[: n_full + 1][-2:][-n_local:]]
        assert torch.equal(caches_a[l][:, kept_a[-n_local:]], want), l
