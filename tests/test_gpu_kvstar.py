"""KVStar softmax-vote retrieval: HIP kernels against the CPU oracle (fp32, tolerance stated per check)."""
import numpy as np
import pytest
import torch

import oracle as O
import synth

pytestmark = pytest.mark.gpu

# votes are sums of softmax probabilities; kernel and oracle differ in fp32 summation order and in exp()
VOTE_RTOL, VOTE_ATOL = 2e-4, 2e-6


def f16_bits(a):
    return np.ascontiguousarray(a, np.float32).astype(np.float16).view(np.uint16)


def dev_f16(bits, dev):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(dev).view(torch.float16)


def check_selection(got_idx, want_final, k):
    """The selected set may differ from the oracle's only by blocks whose votes tie within tolerance."""
    n = len(want_final)
    k = min(k, n)
    assert len(got_idx) == k and len(set(got_idx)) == k
    if k == 0:
        return
    order = np.argsort(-want_final, kind="stable")
    kth = want_final[order[k - 1]]
    tol = VOTE_ATOL + VOTE_RTOL * abs(kth) * 4
    for i in got_idx:
        assert want_final[i] >= kth - tol, (i, want_final[i], kth)
    for i in order[:k]:
        if want_final[i] > kth + tol:
            assert i in got_idx, (i, want_final[i], kth)


@pytest.mark.parametrize("merge,hkv,d,bs", [(16, 8, 128, 128), (32, 2, 64, 128), (4, 4, 128, 16), (128, 1, 128, 128), (16, 2, 128, 32),
                                            (2, 8, 128, 128), (1, 2, 64, 128)])   # the last two: 64 and 128 sub-blocks per block
def test_kvstar_block_repre(ucm, dev, merge, hkv, d, bs):
    from ucm_amd import ops

    n_layers, nb, rows = 2, 11, 14
    caches_h = [synth.normal_bf16_bits(1000 + l, (nb, bs, hkv, d)) for l in range(n_layers)]
    caches = [torch.from_numpy(c.view(np.int16)).to(dev).view(torch.bfloat16) for c in caches_h]
    lp = ops.LayerPointers(caches)
    ids = synth.permutation(1010, nb)[:9].astype(np.int32)
    slots = synth.permutation(1011, rows)[:9].astype(np.int32)
    M = bs // merge
    for d_pruned, layout in ((d, "row"), (d - 13, "row"), (16, "row"), (d, "head"), (16, "head")):
        pruned = None if d_pruned == d else np.stack([synth.permutation(1020 + h, d)[:d_pruned] for h in range(hkv)]).astype(np.int32)
        d_pad = (d_pruned + 15) // 16 * 16
        repre = ops.kvstar_table(n_layers, hkv, rows, M, d_pad, dev, layout).fill_(3.0)      # indexed [L, h, rows, d_pad/8, M, 8]
        ops.kvstar_block_repre(lp, torch.from_numpy(ids).to(dev), torch.from_numpy(slots).to(dev), repre, bs, hkv, d, nb, merge,
                               pruned=None if pruned is None else torch.from_numpy(pruned).to(dev))
        got = ops.kvstar_table_to_reference(repre).contiguous().view(torch.int16).cpu().numpy().view(np.uint16)   # oracle's order
        for l in range(n_layers):
            want = np.full((rows, M, hkv, d_pad), np.float16(3.0).view(np.uint16), np.uint16)
            O.kvstar_block_repre(caches_h[l], ids, slots, merge, want, pruned=pruned)
            assert np.array_equal(got[l], want), (d_pruned, l)
    # against torch's own mean in the model dtype (what the reference calls): equal up to one bf16 step of the summation order
    t = caches[0][torch.from_numpy(ids.astype(np.int64)).to(dev)].reshape(9, M, merge, hkv, d).mean(dim=2).to(torch.float16)
    repre = ops.kvstar_table(n_layers, hkv, rows, M, d, dev).zero_()
    ops.kvstar_block_repre(lp, torch.from_numpy(ids).to(dev), torch.from_numpy(slots).to(dev), repre, bs, hkv, d, nb, merge)
    mine = ops.kvstar_table_to_reference(repre[0])[torch.from_numpy(slots.astype(np.int64)).to(dev)]
    assert torch.allclose(mine.float(), t.float(), rtol=2 ** -7, atol=1e-6)


@pytest.mark.parametrize("merge,hkv,d,bs", [(2, 8, 128, 128), (4, 2, 64, 32), (16, 4, 128, 128), (3, 2, 64, 48)])
def test_kvstar_block_repre_of_fp16_keys(ucm, dev, merge, hkv, d, bs):
    """A float16 model: the cache is float16, the means are rounded once to float16 (merge 3 goes through the kernel
    for arbitrary sub-block sizes); the result is what torch's mean() gives in float16 up to the order of the sums."""
    from ucm_amd import ops

    n_layers, nb, rows = 2, 9, 12
    rng = np.random.default_rng(1090 + merge)
    caches_h = [(rng.standard_normal((nb, bs, hkv, d)) * rng.choice([1e-3, 1.0, 40.0], size=(nb, 1, 1, d))).astype(np.float16)
                for _ in range(n_layers)]
    caches = [torch.from_numpy(c).to(dev) for c in caches_h]
    lp = ops.LayerPointers(caches)
    ids = synth.permutation(1091, nb)[:7].astype(np.int32)
    slots = synth.permutation(1092, rows)[:7].astype(np.int32)
    M = bs // merge
    for d_pruned, layout in ((d, "head"), (16, "head"), (d - 8, "row")):
        pruned = None if d_pruned == d else np.stack([synth.permutation(1093 + h, d)[:d_pruned] for h in range(hkv)]).astype(np.int32)
        d_pad = (d_pruned + 15) // 16 * 16
        repre = ops.kvstar_table(n_layers, hkv, rows, M, d_pad, dev, layout).fill_(3.0)
        ops.kvstar_block_repre(lp, torch.from_numpy(ids).to(dev), torch.from_numpy(slots).to(dev), repre, bs, hkv, d, nb, merge,
                               pruned=None if pruned is None else torch.from_numpy(pruned).to(dev))
        got = ops.kvstar_table_to_reference(repre).contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
        for l in range(n_layers):
            want = np.full((rows, M, hkv, d_pad), np.float16(3.0).view(np.uint16), np.uint16)
            O.kvstar_block_repre(caches_h[l].view(np.uint16), ids, slots, merge, want, pruned=pruned, keys_f16=True)
            assert np.array_equal(got[l], want), (d_pruned, l)
    t = caches[0][torch.from_numpy(ids.astype(np.int64)).to(dev)].reshape(7, M, merge, hkv, d).mean(dim=2)
    repre = ops.kvstar_table(n_layers, hkv, rows, M, d, dev).zero_()
    ops.kvstar_block_repre(lp, torch.from_numpy(ids).to(dev), torch.from_numpy(slots).to(dev), repre, bs, hkv, d, nb, merge)
    mine = ops.kvstar_table_to_reference(repre[0])[torch.from_numpy(slots.astype(np.int64)).to(dev)]
    assert torch.allclose(mine.float(), t.float(), rtol=2 ** -10, atol=1e-6)


@pytest.mark.parametrize("merge", [2, 16, 3])      # the persistent kernel, and the one for other sub-block sizes (16 and 3)
def test_kvstar_block_repre_channel_lists_per_layer(ucm, dev, merge):
    """One launch over all layers with a different set of kept channels in each (the reference picks them per layer
    state, multistep.py:284-304): every layer against the oracle run with that layer's lists."""
    from ucm_amd import ops

    n_layers, nb, rows, hkv, d, bs = 5, 13, 16, 4, 128, 48
    dp, M = 37, bs // merge
    d_pad = (dp + 15) // 16 * 16
    caches_h = [synth.normal_bf16_bits(1500 + l, (nb, bs, hkv, d)) for l in range(n_layers)]
    caches = [torch.from_numpy(c.view(np.int16)).to(dev).view(torch.bfloat16) for c in caches_h]
    ids = synth.permutation(1510, nb)[:10].astype(np.int32)
    slots = synth.permutation(1511, rows)[:10].astype(np.int32)
    pruned = np.stack([[synth.permutation(1520 + 10 * l + h, d)[:dp] for h in range(hkv)] for l in range(n_layers)]).astype(np.int32)
    repre = ops.kvstar_table(n_layers, hkv, rows, M, d_pad, dev).fill_(3.0)
    ops.kvstar_block_repre(ops.LayerPointers(caches), torch.from_numpy(ids).to(dev), torch.from_numpy(slots).to(dev), repre, bs,
                           hkv, d, nb, merge, pruned=torch.from_numpy(pruned).to(dev))
    got = ops.kvstar_table_to_reference(repre).contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    for l in range(n_layers):
        want = np.full((rows, M, hkv, d_pad), np.float16(3.0).view(np.uint16), np.uint16)
        O.kvstar_block_repre(caches_h[l], ids, slots, merge, want, pruned=pruned[l])
        assert np.array_equal(got[l], want), l
    with pytest.raises(ValueError):
        ops.kvstar_block_repre(ops.LayerPointers(caches), torch.from_numpy(ids).to(dev), torch.from_numpy(slots).to(dev), repre,
                               bs, hkv, d, nb, merge, pruned=torch.from_numpy(pruned[:2]).to(dev))


def run_votes(ops, dev, q_bits_list, repre_bits, lens, n_tokens, hq, pruned=None, pruned_sel=None, d_pruned=None, layout="head",
              tiles_per_wave=0):
    """q_bits_list: per task uint16 [x, hq, d]; repre_bits uint16 [rows, M, hkv, d_pad]; tasks own consecutive row ranges."""
    lens = np.asarray(lens, np.int32)
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    q = dev_f16(np.stack(q_bits_list), dev)
    q_off = torch.arange(len(lens), dtype=torch.int64, device=dev) * q[0].numel()
    rows, M, hkv, _ = repre_bits.shape
    table = ops.kvstar_table_from_reference(dev_f16(repre_bits, dev), layout)         # indexed [h, rows, d_pad/8, M, 8]
    assert torch.equal(ops.kvstar_table_to_reference(table), dev_f16(repre_bits, dev))
    votes = torch.full((rows,), -7.0, device=dev)
    ws = ops.kvstar_workspace(len(lens), hkv, n_tokens * (hq // hkv), int(lens.max(initial=0)), M, table.shape[2] * 8, dev,
                              tiles_per_wave=tiles_per_wave)
    ops.kvstar_votes(q, q_off, n_tokens, hq, table, torch.from_numpy(off).to(dev), torch.from_numpy(lens).to(dev),
                     int(lens.max(initial=0)), votes, ws, d_pruned=d_pruned,
                     pruned=None if pruned is None else torch.from_numpy(pruned).to(dev),
                     pruned_sel=None if pruned_sel is None else torch.tensor(pruned_sel, dtype=torch.int32, device=dev),
                     tiles_per_wave=tiles_per_wave)
    torch.cuda.synchronize()
    return votes.cpu().numpy(), off


@pytest.mark.parametrize("x,hq,hkv,d,M", [(8, 32, 8, 128, 8), (8, 16, 2, 64, 4), (3, 8, 8, 128, 1), (1, 4, 1, 128, 32),
                                          (5, 24, 4, 96, 2), (8, 64, 8, 128, 16), (8, 32, 8, 128, 64), (4, 8, 2, 64, 128),
                                          (8, 32, 8, 32, 64), (4, 16, 4, 32, 2), (4, 64, 4, 32, 8), (2, 8, 8, 48, 16)])
def test_kvstar_votes_match_oracle(ucm, dev, x, hq, hkv, d, M):
    from ucm_amd import ops

    lens = [37, 1, 0, 130, 64, 257] if M <= 8 else [37, 1, 0, 70]
    rows = int(np.sum(lens))
    scale = np.float32(0.25)                                  # keeps the softmax from collapsing onto one sub-block
    repre = f16_bits(synth.normal_f32(1100, (rows, M, hkv, d)) * scale)
    qs = [f16_bits(synth.normal_f32(1101 + t, (x, hq, d)) * scale) for t in range(len(lens))]
    wants = {t: O.kvstar_retrieve(qs[t], repre[sum(lens[:t]) : sum(lens[:t]) + n], topk=max(n // 3, 1))[1]
             for t, n in enumerate(lens) if n}
    # 0: automatic, -1: per-task plane in LDS, n: chunks of 4n tiles; table rows of kv_heads cells, or head planes
    for tiles_per_wave, layout in ((0, "row"), (-1, "row"), (1, "row"), (3, "row"), (0, "head"), (-1, "head"), (3, "head")):
        got, off = run_votes(ops, dev, qs, repre, lens, x, hq, layout=layout, tiles_per_wave=tiles_per_wave)
        for t, n in enumerate(lens):
            if n == 0:
                continue
            assert np.allclose(got[off[t] : off[t] + n], wants[t], rtol=VOTE_RTOL, atol=VOTE_ATOL), (tiles_per_wave, t, n)
            # what the mathematics fixes whatever the order: every row's probabilities add up to one
            assert abs(got[off[t] : off[t] + n].sum() - x * hq) < 1e-3 * x * hq


def test_kvstar_many_short_tasks_take_the_in_lds_path(ucm, dev):
    """Enough (task, kv head) pairs that the automatic choice is one workgroup per pair with the task's
    per-block sums in LDS; ragged lengths including empty tasks."""
    from ucm_amd import ops

    x, hq, hkv, d, M = 8, 32, 8, 128, 8
    lens = [int(v) for v in synth.permutation(1150, 150) % 41]     # 0..40 blocks, 150 tasks -> 1200 (task, kv head) pairs
    rows = int(np.sum(lens))
    repre = f16_bits(synth.normal_f32(1151, (rows, M, hkv, d)) * np.float32(0.25))
    qs = [f16_bits(synth.normal_f32(1152 + t, (x, hq, d)) * np.float32(0.25)) for t in range(len(lens))]
    got, off = run_votes(ops, dev, qs, repre, lens, x, hq)
    for t, n in enumerate(lens):
        if n == 0:
            continue
        want = O.kvstar_retrieve(qs[t], repre[off[t] : off[t] + n], topk=1)[1]
        assert np.allclose(got[off[t] : off[t] + n], want, rtol=VOTE_RTOL, atol=VOTE_ATOL), (t, n)


@pytest.mark.parametrize("d,M", [(128, 8), (32, 64)])
@pytest.mark.parametrize("slope", [2.0, -2.0, 7.0])
def test_kvstar_scores_drifting_far_from_the_first_span(ucm, dev, d, M, slope):
    """The kernel takes a wave's exponentials relative to the largest score of the wave's first span.  Scores that
    climb by hundreds along the task make it raise that reference and redo spans (a slope of 7 per block passes
    the limit from one span to the next); scores that fall by hundreds underflow to zero votes, as the exact
    softmax does in fp32.  Both paths, same tolerance as everywhere."""
    from ucm_amd import ops

    x, hq, hkv, n = 4, 8, 2, 200
    lens = [n, 3]
    rows = int(np.sum(lens))
    base = (np.arange(rows, dtype=np.float32) * np.float32(slope))[:, None, None, None]     # the block's score level
    noise = synth.normal_f32(1170, (rows, M, hkv, d)) * np.float32(0.125)
    repre = f16_bits(base * np.float32(2.0 / d) + noise)                                    # times q = 0.5: score = level + noise
    qs = [f16_bits(np.full((x, hq, d), 0.5, dtype=np.float32) + synth.normal_f32(1171 + t, (x, hq, d)) * np.float32(0.03125))
          for t in range(2)]
    for tiles_per_wave in (-1, 3):
        got, off = run_votes(ops, dev, qs, repre, lens, x, hq, tiles_per_wave=tiles_per_wave)
        for t, m in enumerate(lens):
            want = O.kvstar_retrieve(qs[t], repre[off[t] : off[t] + m], topk=1)[1]
            assert np.isfinite(got[off[t] : off[t] + m]).all()
            assert np.allclose(got[off[t] : off[t] + m], want, rtol=VOTE_RTOL, atol=VOTE_ATOL), (tiles_per_wave, t)
            assert abs(got[off[t] : off[t] + m].sum() - x * hq) < 1e-3 * x * hq


@pytest.mark.parametrize("M,d", [(64, 32), (8, 128)])
def test_kvstar_full_size_vote_sums_and_block_order(ucm, dev, M, d):
    """The multi-query retrieval at the size of the ragged batch of configs[1] (16 requests of 32..512 blocks x 32
    layers = 512 tasks, 8 query tokens x 32 heads each), through what holds at any size: a task's votes are
    probabilities summed over its 256 (token, head) rows, so they are non-negative and add up to 256; and a vote
    belongs to its block, so a table with every task's blocks in reverse order gives the same votes reversed
    (other summation order: equal to rounding).  Three tasks are also compared with the CPU oracle."""
    from ucm_amd import ops

    x, hq, hkv, n_layers, n_req = 8, 32, 8, 32, 16
    lens_req = 32 + synth.permutation(1180, 4096)[:n_req] % 481            # 32..512 blocks
    lens = np.tile(lens_req, n_layers).astype(np.int32)
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    rows, n_tasks, longest = int(lens.sum()), len(lens), int(lens.max())
    gen = torch.Generator(device=dev)
    gen.manual_seed(1181)
    table = (torch.empty((hkv, rows, d // 8, M, 8), device=dev).normal_(generator=gen) * 0.25).to(torch.float16)
    q = (torch.empty((n_tasks, x, hq, d), device=dev).normal_(generator=gen) * 0.25).to(torch.float16)
    q_off = torch.arange(n_tasks, dtype=torch.int64, device=dev) * (x * hq * d)
    seg_off, seg_len = torch.from_numpy(off).to(dev), torch.from_numpy(lens).to(dev)
    ws = ops.kvstar_workspace(n_tasks, hkv, x * hq // hkv, longest, M, d, dev)
    votes = torch.full((rows,), -7.0, device=dev)
    ops.kvstar_votes(q, q_off, x, hq, table, seg_off, seg_len, longest, votes, ws)
    # the same tasks with their blocks in reverse order
    src = torch.cat([torch.arange(int(o) + int(n) - 1, int(o) - 1, -1) for o, n in zip(off, lens)]).to(dev)
    votes_rev = torch.full((rows,), -7.0, device=dev)
    ops.kvstar_votes(q, q_off, x, hq, table[:, src].contiguous(), seg_off, seg_len, longest, votes_rev, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(votes).all() and (votes >= 0).all()
    sums = torch.zeros(n_tasks, device=dev, dtype=torch.float64).index_add_(
        0, torch.repeat_interleave(torch.arange(n_tasks, device=dev), seg_len.long()), votes.double())
    assert torch.allclose(sums, torch.full_like(sums, x * hq), rtol=1e-4), (sums.min().item(), sums.max().item())
    assert torch.allclose(votes_rev[src], votes, rtol=VOTE_RTOL, atol=VOTE_ATOL)
    ref_order = ops.kvstar_table_to_reference(table)                       # [rows, M, hkv, d]
    for t in (0, n_tasks // 2 + 3, n_tasks - 1):
        o, n = int(off[t]), int(lens[t])
        want = O.kvstar_retrieve(q[t].view(torch.int16).cpu().numpy().view(np.uint16),
                                 ref_order[o : o + n].contiguous().view(torch.int16).cpu().numpy().view(np.uint16), topk=1)[1]
        assert np.allclose(votes[o : o + n].cpu().numpy(), want, rtol=VOTE_RTOL, atol=VOTE_ATOL), t


def test_kvstar_workspace_sized_for_another_path_is_refused(ucm, dev):
    """The path depends on a process-wide knob; a workspace sized before the knob changed is rejected on the host."""
    from ucm_amd import _lib, ops

    x, hq, hkv, d, M, n_tasks, blocks = 8, 32, 8, 128, 8, 32, 40
    table = torch.zeros(hkv, n_tasks * blocks, d // 8, M, 8, dtype=torch.float16, device=dev)
    q = torch.zeros(n_tasks, x, hq, d, dtype=torch.float16, device=dev)
    q_off = torch.arange(n_tasks, dtype=torch.int64, device=dev) * (x * hq * d)
    seg_off = torch.arange(n_tasks, dtype=torch.int32, device=dev) * blocks
    seg_len = torch.full((n_tasks,), blocks, dtype=torch.int32, device=dev)
    votes = torch.zeros(n_tasks * blocks, device=dev)
    ws = ops.kvstar_workspace(n_tasks, hkv, x * hq // hkv, blocks, M, d, dev)      # 256 (task, kv head) pairs: the in-LDS path
    with pytest.raises(_lib.UcmHipError) as e:
        ops.kvstar_votes(q, q_off, x, hq, table, seg_off, seg_len, blocks, votes, ws, tiles_per_wave=3)
    assert e.value.code == _lib.EINVAL and "workspace" in str(e.value)
    ops.kvstar_votes(q, q_off, x, hq, table, seg_off, seg_len, blocks, votes, ws)  # the path it was sized for
    torch.cuda.synchronize()
    assert np.allclose(votes.cpu().numpy(), x * hq / blocks, rtol=1e-5)            # all-zero scores: uniform votes


@pytest.mark.parametrize("longest", [1200, 1400])
def test_kvstar_long_task_plane_in_lds_or_not(ucm, dev, longest):
    """1200 blocks x 32 rows is a 150 KiB plane: the in-LDS path at its largest; 1400 blocks do not fit, and the
    request for the in-LDS path falls back to the workspace path."""
    from ucm_amd import ops

    x, hq, hkv, d, M = 8, 8, 2, 128, 8
    lens = [longest, 5]
    rows = int(np.sum(lens))
    repre = f16_bits(synth.normal_f32(1160, (rows, M, hkv, d)) * np.float32(0.25))
    qs = [f16_bits(synth.normal_f32(1161 + t, (x, hq, d)) * np.float32(0.25)) for t in range(2)]
    got, off = run_votes(ops, dev, qs, repre, lens, x, hq, tiles_per_wave=-1)
    for t, n in enumerate(lens):
        want = O.kvstar_retrieve(qs[t], repre[off[t] : off[t] + n], topk=1)[1]
        assert np.allclose(got[off[t] : off[t] + n], want, rtol=VOTE_RTOL, atol=VOTE_ATOL), (t, n)


@pytest.mark.parametrize("M,dp", [(8, 77), (64, 32)])          # 77 kept channels: table rows padded to 80; 64 / 32: the reference's defaults
@pytest.mark.parametrize("tiles_per_wave", [0, -1])
def test_kvstar_pruned_channels_and_selection(ucm, dev, tiles_per_wave, M, dp):
    from ucm_amd import ops

    _pruned_channels_and_selection(ops, dev, M, dp, tiles_per_wave)


def _pruned_channels_and_selection(ops, dev, M, dp, tiles_per_wave):

    x, hq, hkv, d = 8, 32, 8, 128
    lens = [90, 33]
    rows = int(np.sum(lens))
    pruned = np.stack([[synth.permutation(1200 + 10 * t + h, d)[:dp] for h in range(hkv)] for t in range(2)]).astype(np.int32)
    d_pad = (dp + 15) // 16 * 16
    repre = np.zeros((rows, M, hkv, d_pad), np.uint16)
    repre[..., :dp] = f16_bits(synth.normal_f32(1201, (rows, M, hkv, dp)) * np.float32(0.3))
    qs = [f16_bits(synth.normal_f32(1202 + t, (x, hq, d)) * np.float32(0.3)) for t in range(2)]
    got, off = run_votes(ops, dev, qs, repre, lens, x, hq, pruned=pruned, pruned_sel=[1, 0], tiles_per_wave=tiles_per_wave)
    for t, n in enumerate(lens):
        sel = [1, 0][t]
        idx, want = O.kvstar_retrieve(qs[t], repre[off[t] : off[t] + n], topk=n // 4, pruned=pruned[sel])
        assert np.allclose(got[off[t] : off[t] + n], want, rtol=VOTE_RTOL, atol=VOTE_ATOL), t
        k = n // 4
        seg_off, seg_len = torch.tensor([off[t]], dtype=torch.int32, device=dev), torch.tensor([n], dtype=torch.int32, device=dev)
        out = torch.zeros((1, 1, n), dtype=torch.int32, device=dev)
        cnt = torch.zeros((1, 1), dtype=torch.int32, device=dev)
        ops.kvstar_topk(torch.from_numpy(got).to(dev), seg_off, seg_len, torch.tensor([k], dtype=torch.int32, device=dev), n, out[0], cnt[0])
        check_selection(out[0, 0, : int(cnt[0, 0])].tolist(), want, k)


def test_kvstar_retrieve_module_surface(ucm, dev):
    """The reference's kvstar_retrieve calls, on device tensors: keys -> sub-block means (with channel pruning)
    -> AsyncRetrieveByCPU / Wait / GetTaskResult."""
    from ucm_amd.sparse.kvstar import retrieve as kvstar_retrieve

    hq, hkv, d, bs, nb, merge = 16, 4, 128, 32, 40, 8
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    k_cache = (torch.randn(nb, bs, hkv, d, device=dev, generator=g) * 0.3).to(torch.bfloat16)
    ids = [int(i) for i in synth.permutation(1300, nb)[:30]]
    kvstar_retrieve.Setup(kvstar_retrieve.SetupParam([0], 8, 0.5, 0, kvstar_retrieve.CPU, 1, 0))
    for ratio in (1.0, 0.6):
        repre, index = kvstar_retrieve.extract_block_repre(k_cache, ids, merge, prune_ratio=ratio, prune_dim_enable=True)
        dp = round(d * ratio)
        assert repre.shape == (30, bs // merge, hkv, dp) and repre.dtype == torch.float16 and repre.dim() == 4
        assert repre.table.shape == (hkv, 30, (dp + 15) // 16 * 2, bs // merge, 8)   # the score kernel's order
        assert (index is None) == (ratio == 1.0)
        cache_bits = k_cache.view(torch.int16).cpu().numpy().view(np.uint16)
        want = np.zeros((30, bs // merge, hkv, (dp + 15) // 16 * 16), np.uint16)
        pr = None if index is None else index.cpu().numpy().astype(np.int32)
        O.kvstar_block_repre(cache_bits, ids, np.arange(30), merge, want, pruned=pr)
        assert np.array_equal(repre.dense().view(torch.int16).cpu().numpy().view(np.uint16), want[..., :dp])
        if index is not None:                                  # the kept channels are those with the largest mean |k|
            # (as torch computes that statistic - one mean over all tokens - up to the summation order: a channel
            # whose mean is within rounding of the last kept one's may be exchanged for it)
            am = k_cache[torch.tensor(ids, device=dev)].reshape(-1, hkv, d).float().abs().mean(0)
            kept = torch.gather(am, 1, index)
            assert index.shape == (hkv, dp) and all(len(set(row.tolist())) == dp for row in index)
            assert (kept >= torch.topk(am, dp, dim=-1).values[:, -1:] * (1 - 1e-5)).all()
            assert (kept[:, :-1] >= kept[:, 1:] * (1 - 1e-5)).all()       # and they come largest first
        blk = repre[1:-2]                                      # the reference keeps [init:-local] (multistep.py:495-497): still a view
        assert blk.shape == (27, bs // merge, hkv, dp) and blk.table.data_ptr() != repre.table.data_ptr()
        if ratio == 1.0:
            blk = blk.dense()                                  # and a plain [n, M, h, d] tensor is accepted as well
        q = (torch.randn(8, hq, d, device=dev, generator=g) * 0.3).to(torch.float16)
        tid = kvstar_retrieve.AsyncRetrieveByCPU(q, blk, index, 9, 7, kvstar_retrieve.CPU)
        kvstar_retrieve.Wait(tid)
        res = kvstar_retrieve.GetTaskResult(tid)
        assert res["status"] == "SUCCESS" and len(res["data"]) == 9
        padded = want[1:-2]
        idx, final = O.kvstar_retrieve(q.view(torch.int16).cpu().numpy().view(np.uint16), padded, 9, pruned=pr, d_pruned=dp)
        check_selection(res["data"], final, 9)
        assert all(final[a] >= final[b] - 1e-5 for a, b in zip(res["data"], res["data"][1:]))   # descending votes
    # errors arrive through the task result, with the reference's messages
    bad = kvstar_retrieve.AsyncRetrieveByCPU(q[0], blk, index, 3, 7, kvstar_retrieve.CPU)
    assert kvstar_retrieve.GetTaskResult(bad) == {"status": "FAILURE", "error": "Query shape must be 3D (x, H, d)."}
    bad = kvstar_retrieve.AsyncRetrieveByCPU(q[:, :6], blk, index, 3, 7, kvstar_retrieve.CPU)
    assert kvstar_retrieve.GetTaskResult(bad)["error"] == "Num_q_heads must be a divisible by num_kv_heads."
    assert kvstar_retrieve.GetTaskResult(123456) is None


@pytest.mark.parametrize("ratio", [1.0, 0.25])
def test_kvstar_retrieve_batch(ucm, dev, ratio):
    """AsyncRetrieveBatch: the requests of a layer in one launch, each with a table (and channel list) of its own;
    every task must return what AsyncRetrieveByCPU returns for it alone."""
    from ucm_amd.sparse.kvstar import retrieve as kvstar_retrieve

    hq, hkv, d, bs, nb, merge = 16, 4, 128, 32, 90, 2
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    k_cache = (torch.randn(nb, bs, hkv, d, device=dev, generator=g) * 0.3).to(torch.bfloat16)
    order = [int(i) + 2 for i in synth.permutation(1500, nb - 2)]
    lens, topks = [30, 1, 41, 7], [9, 1, 12, 7]
    repres, indexes, qs, at = [], [], [], 0
    for n in lens:
        r, i = kvstar_retrieve.extract_block_repre(k_cache, order[at : at + n], merge, prune_ratio=ratio, prune_dim_enable=True)
        at += n
        repres.append(r)
        indexes.append(i)
        qs.append((torch.randn(8, hq, d, device=dev, generator=g) * 0.3).to(torch.float16))
    tids = kvstar_retrieve.AsyncRetrieveBatch(qs, repres, indexes, topks)
    assert len(tids) == len(lens)
    for t, tid in enumerate(tids):
        kvstar_retrieve.Wait(tid)
        got = kvstar_retrieve.GetTaskResult(tid)
        alone = kvstar_retrieve.AsyncRetrieveByCPU(qs[t], repres[t], indexes[t], topks[t], t, kvstar_retrieve.CPU)
        kvstar_retrieve.Wait(alone)
        want = kvstar_retrieve.GetTaskResult(alone)
        assert got["status"] == "SUCCESS" and len(got["data"]) == min(topks[t], lens[t])
        dp = repres[t].shape[3]
        pr = None if indexes[t] is None else indexes[t].cpu().numpy().astype(np.int32)
        padded = np.zeros((lens[t], bs // merge, hkv, (dp + 15) // 16 * 16), np.uint16)
        padded[..., :dp] = repres[t].dense().view(torch.int16).cpu().numpy().view(np.uint16)
        _, votes = O.kvstar_retrieve(qs[t].view(torch.int16).cpu().numpy().view(np.uint16), padded, topks[t], pruned=pr, d_pruned=dp)
        check_selection(got["data"], votes, topks[t])
        check_selection(want["data"], votes, topks[t])
    bad = kvstar_retrieve.AsyncRetrieveBatch(qs[:2], [repres[0], repres[1].dense()], indexes[:2], topks[:2])
    assert kvstar_retrieve.GetTaskResult(bad[1])["status"] == "FAILURE"
    assert kvstar_retrieve.AsyncRetrieveBatch([], [], [], []) == []


@pytest.mark.parametrize("max_len", [64, 100, 256, 700, 3000])
def test_kvstar_topk_heap_ties(ucm, dev, max_len):
    """ucm_kvstar_topk against the oracle's literal heap on votes full of ties (few distinct values), one launch for
    many tasks of ragged length: the chosen SET must be the heap's, and sorting it by (vote, index) descending must
    give the heap's order."""
    from ucm_amd import ops

    rng = np.random.default_rng(max_len)
    n_tasks = 150
    lens = rng.integers(1, max_len + 1, n_tasks).astype(np.int32)
    lens[0], lens[1] = max_len, 1
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    ks = np.array([max(1, int(rng.integers(1, n + 3))) for n in lens], np.int32)
    ks[2] = lens[2]                                             # k == n: everything
    votes = rng.integers(0, 4, int(lens.sum())).astype(np.float32) * np.float32(0.25)
    votes[off[3] : off[3] + lens[3]] = 1.0                      # one task with all votes equal
    idx = torch.full((n_tasks, max_len), -1, dtype=torch.int32, device=dev)
    cnt = torch.zeros(n_tasks, dtype=torch.int32, device=dev)
    t = lambda a: torch.from_numpy(a).to(dev)
    votes[off[4] : off[4] + lens[4]] *= -1.0                    # negative votes and both zeros
    ops.kvstar_topk(t(votes), t(off), t(lens), t(ks), max_len, idx, cnt)
    ordered = idx.clone()
    ops.kvstar_order(t(votes), t(off), t(lens), max_len, ordered, cnt)   # the reference's return order, on the device
    torch.cuda.synchronize()
    idx, cnt, ordered = idx.cpu().numpy(), cnt.cpu().numpy(), ordered.cpu().numpy()
    for i in range(n_tasks):
        v = votes[off[i] : off[i] + lens[i]]
        want = O.kvstar_topk(v, int(ks[i]))
        got = idx[i, : cnt[i]]
        assert cnt[i] == len(want) == min(ks[i], lens[i])
        assert np.all(np.diff(got) > 0)
        assert sorted(want.tolist()) == got.tolist(), (i, lens[i], ks[i])
        assert sorted(got.tolist(), key=lambda b: (v[b], b), reverse=True) == want.tolist()
        assert ordered[i, : cnt[i]].tolist() == want.tolist(), (i, lens[i], ks[i])
    for a in (idx, ordered):
        assert np.all(a[np.arange(max_len)[None, :] >= cnt[:, None]] == -1)


def test_kvstar_get_task_result_tie_order(ucm, dev):
    """Through the module surface: blocks 1 and 3 identical, 0 and 2 identical and lower; k = 3.  The reference's heap
    returns [3, 1, 2] (simd_compute_kernel.cpp:955-977)."""
    from ucm_amd.sparse.kvstar import retrieve as kvstar_retrieve

    rep = torch.zeros(4, 2, 1, 16, dtype=torch.float16, device=dev)
    rep[1] = rep[3] = 0.5
    q = torch.ones(1, 1, 16, dtype=torch.float16, device=dev)
    kvstar_retrieve.Setup(kvstar_retrieve.SetupParam([0], 8, 0.5, 0, kvstar_retrieve.CPU, 1, 0))
    tid = kvstar_retrieve.AsyncRetrieveByCPU(q, rep, None, 3, 0, kvstar_retrieve.CPU)
    kvstar_retrieve.Wait(tid)
    res = kvstar_retrieve.GetTaskResult(tid)
    assert res["status"] == "SUCCESS" and res["data"] == [3, 1, 2]
