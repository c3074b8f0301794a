"""The GSA prefetch engine on the device (ucm_prefetch_plan behind the reference's GSAPrefetchEngineC surface) against
the CPU oracle's replay of the same call sequences - itself pinned by the reference's compiled engine and the golden
vectors (tests/test_oracle_pins.py) - and the loads it plans against the bytes of the pool."""
import numpy as np
import pytest
import torch

import synth
from golden.make_golden import prefetch_scenario, prefetch_scenarios
from prefetch_model import replay, same_result

pytestmark = pytest.mark.gpu


def run_device(dev, n_layers, reqs, runs, max_bs=8, max_len=64):
    from ucm_amd.sparse.gsa.prefetch import GSAPrefetchEngineC

    i32 = dict(dtype=torch.int32, device=dev)
    free = torch.zeros((n_layers, max_bs, max_len), **i32)
    free_len = torch.zeros((n_layers, max_bs), **i32)
    success = torch.full((n_layers, max_bs, max_len), 7, **i32)      # the round zero-fills the rows it writes
    success_len = torch.zeros((n_layers, max_bs), **i32)
    eng = GSAPrefetchEngineC(free, success, free_len, success_len, False)
    for rq in reqs:
        eng.set_blocks_map(rq["req_id"], list(rq["table"]), list(rq["select"]))
        free[:, rq["bs_index"], : len(rq["free"])] = torch.tensor(rq["free"], **i32)
        free_len[:, rq["bs_index"]] = len(rq["free"])
        success[:, rq["bs_index"]] = 0
    results = []
    for t, run in enumerate(runs):
        for r, idx, blk in run["adds"]:
            eng.add_blocks_map(reqs[r]["req_id"], idx, blk)
        buf = torch.zeros((n_layers, len(reqs), max_len), dtype=torch.int64)
        for r in range(len(reqs)):
            for l in range(n_layers):
                tk = run["topk"][r][l]
                buf[l, r, : len(tk)] = torch.tensor(tk, dtype=torch.int64)
        eng.set_blocks_table_info(success, success_len, buf, t)
        eng.run_async_prefetch_bs([rq["req_id"] for rq in reqs], [len(run["topk"][r][0]) for r in range(len(reqs))],
                                  [rq["bs_index"] for rq in reqs], 0)
        loads, misses = eng.obtain_load_blocks(), eng.obtain_miss_idxs()
        assert eng.get_prefetch_status()
        maps = eng.obtain_blocks_map()
        live = torch.zeros(max_bs, dtype=torch.bool)
        live[[rq["bs_index"] for rq in reqs]] = True
        s = success.cpu().numpy().copy()
        s[:, ~live.numpy()] = 0                                        # slots no request owns keep their fill
        results.append(dict(success=s, success_len=success_len.cpu().numpy(), free=free.cpu().numpy(),
                            free_len=free_len.cpu().numpy(), loads=loads, misses=misses,
                            maps={rq["req_id"]: maps[rq["req_id"]] for rq in reqs}))
    return eng, results


@pytest.mark.parametrize("case", prefetch_scenarios() + [(3000 + 31 * i, 1 + i % 3, 1 + i % 4, 4) for i in range(12)])
def test_prefetch_engine_matches_oracle(ucm, dev, case):
    seed, n_layers, n_req, n_runs = case
    reqs, runs = prefetch_scenario(seed, n_layers, n_req, n_runs)
    _, got = run_device(dev, n_layers, reqs, runs)
    want = replay(n_layers, reqs, runs)
    for w, g in zip(want, got):
        same_result(w, g)


def test_prefetch_engine_golden(ucm, dev, golden):
    z, meta = golden
    flat = lambda x: np.array([v for per_req in x for per_layer in per_req for v in [len(per_layer)] + list(per_layer)], np.int32)
    for seed, n_layers, n_req, n_runs in meta["prefetch"]:
        reqs, runs = prefetch_scenario(seed, n_layers, n_req, n_runs)
        _, got = run_device(dev, n_layers, reqs, runs)
        for t, g in enumerate(got):
            key = f"prefetch/{seed}/{t}"
            assert np.array_equal(g["success"], z[key + "/success"]) and np.array_equal(g["success_len"], z[key + "/success_len"])
            assert np.array_equal(flat(g["loads"]), z[key + "/loads"]) and np.array_equal(flat(g["misses"]), z[key + "/misses"])
            assert np.array_equal(g["free_len"], z[key + "/free_len"])


def test_prefetch_engine_skips_and_errors(ucm, dev):
    from ucm_amd.sparse.gsa.prefetch import GSAPrefetchEngineC

    i32 = dict(dtype=torch.int32, device=dev)
    L, B, M = 2, 4, 32
    free, success = torch.zeros((L, B, M), **i32), torch.full((L, B, M), 5, **i32)
    free_len, success_len = torch.zeros((L, B), **i32), torch.full((L, B), 9, **i32)
    eng = GSAPrefetchEngineC(free, success, free_len, success_len)
    with pytest.raises(RuntimeError):
        eng.run_async_prefetch_bs([1], [3], [0])                      # no selection buffer yet
    with pytest.raises(ValueError):
        eng.set_blocks_map(1, [10, 10, 12], [0, 1])                   # one cache block for two logical blocks
    eng.set_blocks_map(1, [10, 11, 12, 13], [0, 2])
    eng.set_blocks_table_info(success, success_len, torch.tensor([[[0, 2, 0], [0, 0, 0]]] * L, dtype=torch.int32), 0)
    # request 77 is unknown and request 1's second entry has no selection: both are skipped, their slots untouched
    eng.run_async_prefetch_bs([1, 77], [2, 2], [3, 1])
    assert eng.obtain_load_blocks() == [[[], []], [[], []]]
    assert success[:, 3, :3].tolist() == [[10, 12, 0]] * L and success_len[:, 3].tolist() == [2, 2]
    assert success[:, 1].eq(5).all() and success_len[:, 1].tolist() == [9, 9]
    eng.run_async_prefetch_bs([1], [0], [2])                          # topk_len 0: skipped
    assert success[:, 2].eq(5).all()
    with pytest.raises(ValueError, match="selection of more than 3"):
        eng.run_async_prefetch_bs([1], [4], [2])                      # longer than the round's buffer: refused, not cut
    eng.del_blocks_map(1)
    eng.del_blocks_map(1)
    assert eng.obtain_blocks_map() == {}


def test_prefetch_load_missing_moves_the_planned_blocks(ucm, dev):
    """A round's served misses are loaded from a pool of stored blocks ([block][layer][K|V]) into the cache blocks the
    round picked, K and V, all layers in one launch; unserved misses and hits move nothing."""
    from ucm_amd import ops

    L, nb, bs, hkv, d = 3, 80, 16, 2, 64
    slice_bytes = bs * hkv * d * 2
    seed, n_req, n_runs = 2200, 5, 6
    reqs, runs = prefetch_scenario(seed, L, n_req, n_runs)
    top_block = max(max(rq["table"] + rq["spare"]) for rq in reqs) + 1
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    caches = [torch.randn(2, top_block, bs, hkv, d, device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    layers = ops.LayerPointers(caches)
    # the pool holds logical block i of request r at pool slot 50*r + i, filled with a pattern of its own
    pool = torch.randint(0, 255, (50 * n_req, L, 2, slice_bytes), dtype=torch.uint8, device=dev, generator=g)
    eng, _ = run_device(dev, L, reqs, runs[:1])
    src = torch.full((eng.map_block.shape[0], 50), -1, dtype=torch.int32, device=dev)
    for r, rq in enumerate(reqs):
        src[eng._row_of[rq["req_id"]]] = torch.arange(50 * r, 50 * r + 50, dtype=torch.int32, device=dev)
    before = [c.clone() for c in caches]
    loads, misses = eng.obtain_load_blocks(), eng.obtain_miss_idxs()
    eng.load_missing(layers, caches[0].stride(0) * 2, slice_bytes, top_block, pool.view(-1), L * 2 * slice_bytes, src)
    torch.cuda.synchronize()
    moved = 0
    for l in range(L):
        touched = set()
        for r in range(n_req):
            for blk, logical in zip(loads[r][l], misses[r][l]):
                for kv in range(2):
                    assert torch.equal(caches[l][kv][blk].reshape(-1).view(torch.uint8), pool[50 * r + logical, l, kv])
                touched.add(blk)
                moved += 1
        rest = torch.tensor([b for b in range(top_block) if b not in touched], device=dev)
        assert torch.equal(caches[l][:, rest], before[l][:, rest])
    assert moved > 0
