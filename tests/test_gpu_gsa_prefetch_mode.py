"""GSA with ptopk_prefetch_enable, hooks to engine to store: a host replay of the reference's protocol
(prefetch_engine.py:125-468, gsa.py:690-745, 821-866) with the CPU oracle's engine round (orc_prefetch_run) against the
plugin's device tables, step by step, and the cache blocks attention is pointed at against the keys and values they
should hold."""
import types

import numpy as np
import pytest
import torch

import oracle as O
import synth
from test_gpu_host_layer import make_config, topk_len

pytestmark = pytest.mark.gpu
ns = types.SimpleNamespace


class Model:
    """One request, as the reference's Python side sees it."""

    def __init__(self, rid, prompt_blocks, n_prompt_tokens, L):
        self.rid, self.prompt_ids, self.n_prompt, self.L = rid, list(prompt_blocks), n_prompt_tokens, L
        self.logical_phys = list(prompt_blocks)      # "blocks" of GSAReqStat: one entry per logical block
        self.phys = list(prompt_blocks)              # the scheduler's list
        self.use = self.succ = self.free = None      # per layer lists
        self.map = None                              # per layer {cache block: logical block}
        self.to_map, self.to_table = [], []
        self.sparse = False


@pytest.mark.parametrize("stride", [3, 1])
def test_gsa_prefetch_mode_flow(ucm, dev, stride):
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    hq, hkv, d, L, bs, nb = 8, 2, 64, 3, 16, 400
    lo, hi, ratio = 6, 10, 0.3
    local = lo - 1
    cfg = make_config(hq, hkv, d, L, bs, 16 * 120, {"seg_prefill_threshold": 100, "min_topk_len": lo, "max_topk_len": hi,
                                                    "ptopk_prefetch_enable": True, "prefetch_stride": stride})
    slice_bytes = bs * hkv * d * 2
    store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 200 * L * 2 * slice_bytes})
    plugin = GSA(cfg, UcmSparseRole.WORKER, store=store)
    g = torch.Generator(device=dev)
    g.manual_seed(77)
    caches = [torch.randn(2, nb, bs, hkv, d, device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    plugin.register_kv_caches({names[l]: caches[l] for l in range(L)})
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0, attn_metadata=None)

    perm = [int(x) for x in synth.permutation(960, nb)]
    pool_free = perm[200:]                              # blocks the scheduler hands out during decode
    # A: 40 full blocks + 5 tokens; B: exactly 35 blocks (its first decoded token opens a block) - it ends after engine
    # step 25; C: short, never sparse; D: 38 blocks + 9 tokens, arrives at engine step 10, while the others decode
    shapes = {"A": (41, 40 * bs + 5), "B": (35, 35 * bs), "C": (4, 60), "D": (39, 38 * bs + 9)}
    arrive, leave = {"A": 0, "B": 0, "C": 0, "D": 10}, {"B": 25}
    reqs, models, at = {}, {}, 0
    for rid, (n_blocks, n_tok) in shapes.items():
        ids = perm[at : at + n_blocks]
        at += n_blocks
        reqs[rid] = ns(block_ids=[list(ids)], num_computed_tokens=0, prompt_token_ids=[1] * n_tok, output_token_ids=[])
        models[rid] = Model(rid, ids, n_tok, L)
    truth = {rid: [dict() for _ in range(L)] for rid in shapes}    # per layer {logical block: its K and V}
    tokens = {r: 0 for r in shapes}                                 # tokens in the sequence so far
    k_of = lambda n: topk_len(n, lo, hi)

    def run_step(order, n_tokens, new=()):
        so = ns(num_scheduled_tokens={r: n_tokens[r] for r in order}, scheduled_new_reqs=[ns(req_id=r) for r in new])
        ib = ns(req_id_to_index={r: i for i, r in enumerate(order)})
        starts = np.concatenate([[0], np.cumsum([n_tokens[r] for r in order])])
        md = ns(query_start_loc=torch.tensor(starts), block_table=None, seq_lens=None)
        fc.attn_metadata = md
        plugin.build_sparse_meta(so, reqs, ib, md)
        plugin.execute_begin(so)
        seen = []
        for l in range(L):
            q = (torch.randn(int(starts[-1]), hq, d, device=dev, generator=g) * 0.3).to(torch.bfloat16)
            plugin.attention_begin(q, None, None, names[l], fc)
            seen.append((None if md.block_table is None else md.block_table.clone(),
                         None if md.seq_lens is None else md.seq_lens.clone()))
            plugin.attention_finished(q, None, None, None, names[l], fc)
        plugin.execute_finished()
        torch.cuda.synchronize()
        for r in order:
            reqs[r].num_computed_tokens += n_tokens[r]
        return seen

    def after_prefill(rid):
        """Every full block is in the store; then the scheduler's part (GSA.allocate_slots): a long request keeps its
        first sparse_len blocks, the rest is somebody else's."""
        m = models[rid]
        n_full = shapes[rid][1] // bs
        for j in range(len(m.prompt_ids)):
            for l in range(L):
                truth[rid][l][j] = caches[l][:, m.prompt_ids[j]].clone()
        assert all(store.lookup([f"req_{rid}_blk_{j}"]) == [True] for j in range(n_full))
        assert f"req_{rid}_blk_{n_full}" not in store.slot_of
        tokens[rid] = shapes[rid][1]
        if shapes[rid][1] <= 100:
            return
        n_p = len(m.prompt_ids)
        k = k_of(n_p)
        sparse_len = k + (0 if k > hi else hi - k + 1)
        released = m.prompt_ids[sparse_len:]
        m.phys = m.prompt_ids[:sparse_len]
        m.sparse, m.n_p = True, n_p
        for l in range(L):
            caches[l][:, released] = 7.0

    def grow(rid):
        """The scheduler's part of a decode step: a block for the token if it opens one."""
        m = models[rid]
        if tokens[rid] % bs == 0:
            blk = pool_free.pop()
            m.phys.append(blk)
            m.logical_phys.append(blk)
            for l in range(L):
                truth[rid][l][len(m.logical_phys) - 1] = caches[l][:, blk].clone()
            return blk
        return None

    row_of = lambda rid: plugin.topk_kpre_manger.cache_map[rid]

    def holds_what_the_maps_say(step, l, m):
        """Every block of the table attention reads holds the logical block the engine's map names (a round's loads
        go to blocks outside that table)."""
        pending = dict((b, j) for j, b in m.to_map)
        for b in m.use[l]:
            j = m.map[l].get(b, pending.get(b))
            assert j is not None, (step, l, m.rid, b)
            assert torch.equal(caches[l][:, b], truth[m.rid][l][j]), (step, l, m.rid, b, j)

    pf = None
    space = rounds = n_loaded = 0
    decoded = {r: 0 for r in shapes}                                # decode steps a request has taken
    live = []
    for step in range(0, 40):
        for rid in [r for r in live if leave.get(r, 99) < step]:
            plugin.request_finished_in_worker(rid)
            live.remove(rid)
            assert rid not in pf.engine_id and rid not in pf.ready
        new = [r for r in shapes if arrive[r] == step]
        live += new
        order = list(live)
        n_tokens, grown = {}, {}
        for rid in order:
            if rid in new:
                n_tokens[rid] = shapes[rid][1]
                continue
            grown[rid] = grow(rid)
            tokens[rid] += 1
            decoded[rid] += 1
            reqs[rid].output_token_ids.append(1)
            reqs[rid].block_ids = [list(models[rid].phys)]
            n_tokens[rid] = 1
        seen = run_step(order, n_tokens, new)
        for rid in new:
            after_prefill(rid)
        if step == 0:
            assert all(t is None for t, _ in seen)                   # nobody decodes: the layer's metadata is left alone
            continue
        pf = plugin._pf
        round_now = space >= stride - 1
        space = 0 if round_now else space + 1
        # ---- replay: first deal, lengths, growth
        for rid in order:
            m = models[rid]
            if rid in new:                                          # a prefill step: its own blocks, its real length
                m.use = [list(m.prompt_ids) for _ in range(L)]
                m.succ = None
                m.seq_want = [shapes[rid][1]] * L
                m.to_map, m.to_table = [], []
                continue
            slot = tokens[rid] % bs
            if decoded[rid] == 1:
                if m.sparse:
                    n_p, k = m.n_p, k_of(m.n_p)
                    idx = list(range(hi + 1)) if k <= hi else list(range(k))
                    remain = idx[: k - local] + idx[-local:]
                    free = idx[k - local : -local]
                    in_use = [m.phys[x] for x in remain]
                    m.use = [list(in_use) for _ in range(L)]
                    m.succ = [list(in_use) for _ in range(L)]
                    m.free = [[m.phys[x] for x in free] for _ in range(L)]
                    logical = remain[:-local] + list(range(n_p - local, n_p))
                    m.map = [dict(zip([m.phys[x] for x in free + remain], free + logical)) for _ in range(L)]
                    for l in range(L):                  # the saved window was written into the last `local` of them
                        for x, j in zip(remain[-local:], range(n_p - local, n_p)):
                            assert torch.equal(caches[l][:, m.phys[x]], truth[rid][l][j]), (rid, l, j)
                else:
                    m.use = [list(m.prompt_ids) for _ in range(L)]
                    m.succ = [list(m.prompt_ids) for _ in range(L)]
            m.seq_want = []
            for l in range(L):
                n = len(m.use[l])
                m.seq_want.append(n * bs if slot == 0 else n * bs + 1 if slot == 1 else (n - 1) * bs + slot)
            if slot == 1:
                blk = grown[rid]
                assert blk is not None
                for l in range(L):
                    m.use[l].append(blk)
                m.to_table.append(blk)
                m.to_map.append((len(m.logical_phys) - 1, blk))
        # ---- what attention was handed in this step
        for l in range(L):
            table, lens = seen[l]
            for i, rid in enumerate(order):
                m = models[rid]
                assert int(lens[i]) == m.seq_want[l], (step, l, rid)
                n = len(m.use[l])
                assert table[i, :n].tolist() == m.use[l], (step, l, rid)
                if m.sparse and rid not in new and not round_now:
                    holds_what_the_maps_say(step, l, m)
        # ---- the round at the end of the step
        if round_now:
            rounds += 1
            for i, rid in enumerate(order):
                m = models[rid]
                if rid in new:
                    continue                                        # (its rows are set up again at its first decode step)
                m.use, m.succ = m.succ, m.use
                for j, b in m.to_map:
                    if m.sparse:
                        for l in range(L):
                            m.map[l][b] = j
                for b in m.to_table:
                    for l in range(L):
                        m.use[l].append(b)
                m.to_map, m.to_table = [], []
                if not m.sparse:
                    continue
                n = len(m.logical_phys)
                k = min(k_of(n), n)
                for l in range(L):
                    topk = plugin.topk_caches[l, i, :k].cpu().numpy()
                    assert int(plugin.topk_counts[l, i]) == k
                    blocks = np.array(sorted(m.map[l]), np.int32)
                    idxs = np.array([m.map[l][b] for b in blocks], np.int32)
                    succ, n_succ, loads, miss, free = O.prefetch_run(blocks, idxs, topk, np.array(m.free[l], np.int32),
                                                                     len(m.free[l]), plugin.max_block_len)
                    m.map[l] = dict(zip(blocks.tolist(), idxs.tolist()))
                    m.succ[l] = succ[:n_succ].tolist()
                    m.free[l] = free.tolist()
                    row = row_of(rid)
                    assert pf.succ_table[l, row, :n_succ].tolist() == m.succ[l], (step, l, rid)
                    assert int(pf.succ_len[l, row]) == n_succ
                    assert pf.free_block[l, row, : len(free)].tolist() == m.free[l] and int(pf.free_len[l, row]) == len(free)
                    # the blocks the round loaded hold what they were loaded for, and none of them is in the table
                    # attention reads until the next round
                    for b, j in zip(loads.tolist(), miss.tolist()):
                        assert torch.equal(caches[l][:, b], truth[rid][l][j]), (step, l, rid, b, j)
                        assert b not in m.use[l]
                    n_loaded += len(loads)
                    assert pf.use_table[l, row, : len(m.use[l])].tolist() == m.use[l] and int(pf.use_len[l, row]) == len(m.use[l])
                    holds_what_the_maps_say(step, l, m)
            got = pf.engine.obtain_blocks_map()
            for rid in order:
                if models[rid].sparse and rid not in new:
                    for l in range(L):
                        assert got[pf.engine_id[rid]][l] == models[rid].map[l], (step, l, rid)
    assert rounds == pf.rounds and rounds >= 39 // stride - 1
    assert plugin.load_misses == 0 and n_loaded > 0
    assert sorted(live) == ["A", "C", "D"] and decoded["D"] == 29
    for rid in live:
        plugin.request_finished_in_worker(rid)
    assert not pf.engine_id and not pf.ready
