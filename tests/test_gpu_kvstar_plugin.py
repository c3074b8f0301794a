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


@pytest.mark.parametrize("prune_ratio,chunks,batched,device_loads", [(1.0, 1, True, True), (0.5, 3, True, False), (0.25, 1, False, True),
                                                                     (0.25, 1, True, False)])
def test_kvstar_plugin_flow(ucm, dev, prune_ratio, chunks, batched, device_loads):
    """Prefill (one chunk, or three) of 24 full blocks + 5 tokens, then 13 decode steps with stride 4: step 1 restores
    the windows and loads what the prefill group's vote picks; the vote of decode steps 1-4 is queued at step 4 and
    its winners are loaded at step 8; steps 5-8 at step 8 / 12.  Selections are checked against the CPU oracle on the
    same keys and queries."""
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
        "blk_repre_inner_token_merge": merge, "batch_retrieval": batched, "device_loads": device_loads}}}
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 40 * L * 2 * slice_bytes})
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
    caches = [(torch.randn(2, nb, bs, hkv, d, device=dev, generator=g) * 0.3).to(torch.bfloat16) for _ in range(L)]
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
            q = (torch.randn(n_tok, hq, d, device=dev, generator=g) * 0.3).to(torch.bfloat16)
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
    assert store.create(hashes) == [0] * n_full
    from ucm_amd.sparse.esa.esa import get_offset
    for l in range(L):
        for kv in range(2):
            off = get_offset((bs, hkv, d), 0, 1, 2, l, bool(kv))
            store.wait(store.dump(hashes, [off] * n_full, [original[l][kv][i] for i in full_ids[:n_full]]))
    store.commit(hashes)

    # representatives: blocks 1 .. 21 (init window 1, local window 2), against the oracle on the same keys
    want_repre, pruned = [], []
    for l in range(L):
        st = states[l]
        dp = round(d * prune_ratio)
        assert st.blk_repre.shape == (n_full - 3, bs // merge, hkv, dp)
        pr = None if prune_ratio >= 0.98 else st.d_pruned_index.cpu().numpy().astype(np.int32)
        w = np.zeros((n_full, bs // merge, hkv, (dp + 15) // 16 * 16), np.uint16)
        O.kvstar_block_repre(bits(original[l][0]), np.array(full_ids[:n_full], np.int32), np.arange(n_full, dtype=np.int32), merge, w,
                             pruned=pr)
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

    def check_loaded(record, l):
        st = states[l]
        chosen = st.step_group_retrieve_indices[record]
        votes = expect(record, l)
        check_selection(chosen, votes, n_keep)
        assert all(votes[a] >= votes[b] - (VOTE_ATOL + VOTE_RTOL * abs(votes[b]) * 4) for a, b in zip(chosen, chosen[1:]))
        assert st.step_group_retrieve_result[record] == [hashes[i + 1] for i in chosen]
        for kv in range(2):                                  # candidate block j holds the j-th winner, K and V
            got = caches[l][kv][kept[1 : 1 + n_keep]]
            assert torch.equal(got, original[l][kv][[full_ids[i + 1] for i in chosen]]), (record, l, kv)

    decode_q = {l: [] for l in range(L)}
    for step in range(1, 14):
        if step > 1:
            req.output_token_ids.append(1)
            req.num_output_tokens, req.num_tokens = step, n_prompt + step
        for l, q in enumerate(run_step(1)):
            decode_q[l].append(q[0])
        if step % stride == 0:
            groups["decode" + str(step - stride + 1)] = [torch.stack(decode_q[l][-stride:]) for l in range(L)]
        torch.cuda.synchronize()
        for l in range(L):
            st = states[l]
            if step == 1:
                st.wait_for_blk_transfer_task_done()
                check_loaded("prefill", l)
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
    plugin.request_finished_in_worker("7")
    assert "7" not in plugin.req_states
