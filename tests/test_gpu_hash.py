"""Hash-code retrieval (KvComp style) against the oracle: token codes, block
summaries, query codes, both integer block scores and the selection.  All
results are integers / bit strings, so every comparison is exact."""
import numpy as np
import pytest
import torch

import oracle as O
import synth

pytestmark = pytest.mark.gpu


def i32(x, dev):
    return torch.tensor(np.asarray(x), dtype=torch.int32, device=dev)


def bf16_dev(bits_u16, dev):
    return torch.from_numpy(np.ascontiguousarray(bits_u16).view(np.int16)).to(dev).view(torch.bfloat16)


def make_weights(seed):
    """N(0, 2^2) weights in bf16, as HashEncoder draws them (hash_encoder.py:65-71)."""
    bits = synth.bf16_round_bits(synth.normal_f32(seed, (128, 128)) * np.float32(2.0))
    return bits, synth.bf16_widen(bits)


# the last four: more than 63 tiles in a block, so the column counters are flushed inside the tile loop too
@pytest.mark.parametrize("hkv,bs", [(8, 128), (2, 16), (4, 64), (1, 32), (8, 272), (4, 520), (2, 1040), (1, 2080)])
def test_hash_encode_blocks(ucm, dev, hkv, bs):
    from ucm_amd import ops

    n_layers, nb, rows = 2, 9, 12
    w_bits, w_f32 = make_weights(800)
    caches_h = [synth.normal_bf16_bits(801 + l, (nb, bs, hkv, 128)) for l in range(n_layers)]
    # adversarial rows: exact cancellation (projection exactly 0 -> bit 0), near cancellation, huge dynamic range
    w2 = w_f32.copy()
    for l in range(n_layers):
        c = caches_h[l]
        c[0, 0, 0, :] = 0
        c[0, 1, 0, :] = 0
        c[0, 1, 0, 5] = synth.bf16_round_bits(np.array([3.0], np.float32))[0]
        big = synth.bf16_round_bits(np.array([1.0e4, -1.0e4, 1.0e-4], np.float32))
        c[1, 2, 0, :3] = big
        c[2, 3, 0, :] = c[2, 4, 0, :] ^ np.uint16(0x8000)  # exact negation of another row
    caches = [bf16_dev(c, dev) for c in caches_h]
    lp = ops.LayerPointers(caches)
    ids = synth.permutation(810, nb)[:7]
    slots = synth.permutation(811, rows)[:7]
    colsum = torch.full((n_layers, rows, hkv, 128), 77, dtype=torch.int16, device=dev)
    bcodes = torch.full((n_layers, rows, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    tcodes = torch.full((n_layers, rows, bs, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_blocks(lp, i32(ids, dev), i32(slots, dev), len(ids), bf16_dev(w_bits, dev), bs, hkv, nb,
                           colsum, bcodes, token_codes=tcodes)
    torch.cuda.synchronize()
    got_t, got_s, got_b = tcodes.cpu().numpy(), colsum.cpu().numpy(), bcodes.cpu().numpy()
    for l in range(n_layers):
        want_t = O.hash_encode(caches_h[l][ids], w2)                # [7, bs, hkv, 16]
        assert np.array_equal(got_t[l][slots], want_t), l
        assert np.array_equal(got_s[l][slots], O.hash_colsum(want_t)), l
        assert np.array_equal(got_b[l][slots], O.hash_majority(want_t)), l
        rest = np.setdiff1d(np.arange(rows), slots)
        assert np.all(got_t[l][rest] == 0xEE) and np.all(got_s[l][rest] == 77) and np.all(got_b[l][rest] == 0xEE)
    # the all-zero vector projects to exactly 0 everywhere: every bit is 0
    s0 = slots[list(ids).index(0)] if 0 in ids else None
    if s0 is not None:
        assert not got_t[0][s0, 0, 0].any()
    # without the token codes the summaries are the same
    colsum2, bcodes2 = torch.zeros_like(colsum), torch.zeros_like(bcodes)
    ops.hash_encode_blocks(lp, i32(ids, dev), i32(slots, dev), len(ids), bf16_dev(w_bits, dev), bs, hkv, nb,
                           colsum2, bcodes2)
    assert torch.equal(colsum2[:, torch.from_numpy(slots.astype(np.int64)).to(dev)],
                       colsum[:, torch.from_numpy(slots.astype(np.int64)).to(dev)])


@pytest.mark.parametrize("hkv,bs", [(8, 128), (2, 48), (1, 160), (4, 8)])
def test_hash_encode_persistent_waves_and_queue_overflow(ucm, dev, hkv, bs):
    """One workgroup per layer walks the whole list (every wave takes several blocks, the
    next block's first keys are fetched while the current one is finished), with odd and
    single tile counts, bad ids in the list, and blocks whose every projection needs the
    exact redo: x = (+B at dim 0, s at dim 8, -B at dim 16) against weights with row 16
    equal to row 0 cancels to s*w[8][c] exactly, while fp32 accumulation loses s next to B,
    so the matrix-core sign is wrong for about half of the columns and thousands of queue
    entries per tile have to be redone and patched."""
    from ucm_amd import ops

    n_layers, nb, rows = 2, 23, 30
    w = synth.normal_f32(830, (128, 128)) * np.float32(2.0)
    w[16] = w[0]
    w_bits = synth.bf16_round_bits(w)
    w_f32 = synth.bf16_widen(w_bits)
    one = lambda v: synth.bf16_round_bits(np.array([v], np.float32))[0]
    caches_h = [synth.normal_bf16_bits(831 + l, (nb, bs, hkv, 128)) for l in range(n_layers)]
    for l in range(n_layers):
        c = caches_h[l]
        for blk in (2, 3, 11, 20):                      # whole blocks of cancelling keys
            c[blk] = 0
            c[blk, :, :, 0] = one(4096.0)
            c[blk, :, :, 16] = one(-4096.0)
            small = np.array([one(((-1.0) ** (t + h)) * 2.0 ** -20 * (1 + ((t * 7 + h) % 8) / 8.0))
                              for t in range(bs) for h in range(hkv)], np.uint16).reshape(bs, hkv)
            c[blk, :, :, 8] = small
        c[5, bs // 2:] = 0                              # half a block of all-zero keys
    caches = [bf16_dev(c, dev) for c in caches_h]
    lp = ops.LayerPointers(caches)
    ids = np.concatenate([synth.permutation(832, nb), [2, 3]]).astype(np.int32)
    slots = synth.permutation(833, rows)[: len(ids)].astype(np.int32)
    ids_bad, slots_bad = ids.copy(), slots.copy()
    ids_bad[[1, 6, 7, 13]] = [-1, nb, 1 << 30, nb + 5]      # skipped, never dereferenced
    slots_bad[[9, 20]] = [rows, -3]
    live = np.array([i for i in range(len(ids)) if 0 <= ids_bad[i] < nb and 0 <= slots_bad[i] < rows])
    for groups in (n_layers, 2 * n_layers, 0):
        colsum = torch.full((n_layers, rows, hkv, 128), 77, dtype=torch.int16, device=dev)
        bcodes = torch.full((n_layers, rows, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
        tcodes = torch.full((n_layers, rows, bs, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
        ops.hash_encode_blocks(lp, i32(ids_bad, dev), i32(slots_bad, dev), len(ids), bf16_dev(w_bits, dev), bs, hkv,
                               nb, colsum, bcodes, token_codes=tcodes, workgroups=groups)
        colsum2, bcodes2 = torch.full_like(colsum, 77), torch.full_like(bcodes, 0xEE)
        ops.hash_encode_blocks(lp, i32(ids_bad, dev), i32(slots_bad, dev), len(ids), bf16_dev(w_bits, dev), bs, hkv,
                               nb, colsum2, bcodes2, workgroups=groups)
        torch.cuda.synchronize()
        got_t, got_s, got_b = tcodes.cpu().numpy(), colsum.cpu().numpy(), bcodes.cpu().numpy()
        assert torch.equal(colsum, colsum2) and torch.equal(bcodes, bcodes2), groups
        for l in range(n_layers):
            want_t = O.hash_encode(caches_h[l][ids_bad[live]], w_f32)
            assert np.array_equal(got_t[l][slots_bad[live]], want_t), (groups, l)
            assert np.array_equal(got_s[l][slots_bad[live]], O.hash_colsum(want_t)), (groups, l)
            assert np.array_equal(got_b[l][slots_bad[live]], O.hash_majority(want_t)), (groups, l)
            rest = np.setdiff1d(np.arange(rows), slots_bad[live])
            assert np.all(got_t[l][rest] == 0xEE) and np.all(got_s[l][rest] == 77) and np.all(got_b[l][rest] == 0xEE)
            # the construction did what it is for: the cancelling keys' codes follow sign(s * w[8][c])
            k = list(live).index(len(ids) - 2)      # block 2, appended at the end of the list
            sgn = synth.bf16_widen(caches_h[l][2, :, :, 8])[..., None] * w_f32[8][None, None, :] > 0
            assert np.array_equal(np.unpackbits(want_t[k], axis=-1, bitorder="little").astype(bool), sgn)


def test_config5_full_size_negated_keys_give_complement_codes(ucm, dev):
    """The hash configuration at its full size (32 requests of 64..256 blocks, 8 kv heads, 32 layers, 128-bit
    codes), checked through what the arithmetic fixes at any size: negating a key negates its exact projection,
    so a bit of -K's token code is the complement of K's unless the projection is exactly 0 (bit 0 both times:
    `> 0` is strict; a few per ten million sums of bf16 products do cancel exactly), a column sum is
    #ones - #zeros of its column over the block's tokens, and the majority code is `column sum > 0`.
    Eight layers at a time, fresh keys each time, so that the keys and their negation stay around 22 GB."""
    from ucm_amd import ops

    hkv, bs, n_req, group = 8, 128, 32, 8
    lens = 64 + synth.permutation(880, 4096)[:n_req] % 193          # 64..256 blocks per request
    rows = int(lens.sum())
    w_bits, w_f32 = make_weights(881)
    w = bf16_dev(w_bits, dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(882)
    ids = torch.randperm(rows, device=dev, generator=gen).to(torch.int32)
    shifts = torch.arange(8, device=dev, dtype=torch.uint8)

    def recount(tcodes_layer):                                      # [rows, bs, hkv, 16] -> #ones per (row, head, column)
        bits = (tcodes_layer.view(rows, bs, hkv, 16, 1) >> shifts) & 1
        return bits.view(rows, bs, hkv, 128).sum(dim=1, dtype=torch.int32)

    def majority(colsum):
        return ((colsum > 0).view(group, rows, hkv, 16, 8).to(torch.uint8) << shifts).sum(dim=-1, dtype=torch.uint8)

    exact_zeros = 0
    for part in range(32 // group):
        caches = [torch.empty((rows, bs, hkv, 128), dtype=torch.bfloat16, device=dev).normal_(generator=gen)
                  for _ in range(group)]
        negated = [-c for c in caches]
        out = []
        for layers in (caches, negated):
            colsum = torch.zeros((group, rows, hkv, 128), dtype=torch.int16, device=dev)
            bcodes = torch.zeros((group, rows, hkv, 16), dtype=torch.uint8, device=dev)
            tcodes = torch.zeros((group, rows, bs, hkv, 16), dtype=torch.uint8, device=dev)
            ops.hash_encode_blocks(ops.LayerPointers(layers), ids, None, rows, w, bs, hkv, rows, colsum, bcodes,
                                   token_codes=tcodes)
            out.append((colsum, bcodes, tcodes))
        torch.cuda.synchronize()
        (s_pos, b_pos, t_pos), (s_neg, b_neg, t_neg) = out
        assert not (t_pos & t_neg).any(), part                      # never positive both ways
        both_zero = ~(t_pos | t_neg)                                # bits that are 0 both ways: exact zeros only
        where = both_zero.nonzero()
        assert where.shape[0] < 1e-6 * both_zero.numel() * 8, (part, where.shape[0])
        for l, r, t, h, byte in where[:4].cpu().numpy():            # ... which a few of them are shown to be
            x = caches[l][int(ids[r])][t, h].double().cpu().numpy()
            cols = [8 * byte + j for j in range(8) if (int(both_zero[l, r, t, h, byte]) >> j) & 1]
            assert cols and all(float(x @ w_f32[:, c].astype(np.float64)) == 0.0 for c in cols), (part, l, r, t, h, byte)
        exact_zeros += where.shape[0]
        for l in (0, group - 1):
            ones_pos, ones_neg = recount(t_pos[l]), recount(t_neg[l])
            assert torch.equal(s_pos[l].to(torch.int32), 2 * ones_pos - bs), (part, l)
            assert torch.equal(s_neg[l].to(torch.int32), 2 * ones_neg - bs), (part, l)
        assert torch.equal(b_pos, majority(s_pos)) and torch.equal(b_neg, majority(s_neg)), part
        del caches, negated, out
    print("exact zero projections met:", exact_zeros)


@pytest.mark.parametrize("hq,hkv", [(64, 8), (128, 8), (8, 8), (28, 4), (6, 2), (40, 1)])
def test_hash_query_codes_for_other_head_counts(ucm, dev, hq, hkv):
    """Query codes, their +-1 sums and the group-mean codes for head counts that take one chunk of staged
    vectors, several, and a last chunk that is not full (the kernel stages forty vectors at a time)."""
    from ucm_amd import ops

    n_layers, n_req = 2, 3
    w_bits, w_f32 = make_weights(840)
    q_h = synth.normal_bf16_bits(841 + hq, (n_layers, n_req, hq, 128))
    q_h[0, 1, 0, :] = 0                                        # an all-zero query: every projection is 0, every bit 0
    q_codes = torch.full((n_layers, n_req, hq, 16), 0xEE, dtype=torch.uint8, device=dev)
    q_sum = torch.full((n_layers, n_req, 128), 77, dtype=torch.int16, device=dev)
    qbar = torch.full((n_layers, n_req, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(bf16_dev(q_h, dev), bf16_dev(w_bits, dev), hkv, q_codes, q_sum, qbar, n_req)
    torch.cuda.synchronize()
    for l in range(n_layers):
        want_q = O.hash_encode(q_h[l], w_f32)
        assert np.array_equal(q_codes[l].cpu().numpy(), want_q), l
        pm = np.unpackbits(want_q, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
        assert np.array_equal(q_sum[l].cpu().numpy(), pm.sum(1)), l
        qm = np.stack([O.q_head_mean(synth.bf16_widen(q_h[l][r]), hkv) for r in range(n_req)])
        assert np.array_equal(qbar[l].cpu().numpy(), O.hash_encode_f32(qm, w_f32)), l
    assert not q_codes[0, 1, 0].any()


def test_hash_query_codes_near_zero_projections_and_scales(ucm, dev):
    """Query rows and group means whose projections cancel exactly, or down to one small term, and vectors
    scaled from 2^-100 to 2^100: the kernel projects on the matrix cores in fp32 and redoes results within
    its error bound exactly, so every sign must still be the oracle's (strict > 0: a projection of exactly
    zero is bit 0)."""
    from ucm_amd import ops

    hq, hkv, n_layers, n_req = 32, 8, 2, 6
    g = hq // hkv
    w_bits, _ = make_weights(860)
    w_bits[1] = w_bits[0]                      # two equal weight rows: (t, -t, 0, ...) projects to exactly 0
    w_bits[5] = w_bits[4] ^ 0x8000             # and a negated pair: (t, t, ...) on dims 4, 5 cancels too
    w_f32 = synth.bf16_widen(w_bits)
    f = synth.normal_f32(861, (n_layers, n_req, hq, 128))
    one, tiny = np.float32(1.0), np.float32(2.0 ** -40)
    # request 0: rows that cancel exactly; every second one keeps a term 2^-40 of the others' size on dim 2
    f[:, 0] = 0
    f[:, 0, :, 0], f[:, 0, :, 1] = 3.0, -3.0
    f[:, 0, :, 4], f[:, 0, :, 5] = 0.75, 0.75
    f[:, 0, 1::2, 2] = tiny * np.where(np.arange(hq // 2) % 2 == 0, one, -one)
    # request 1: heads of a group are negations of each other, so the group means are exactly zero ...
    f[:, 1, 1::2] = -f[:, 1, 0::2]
    # request 2: ... or cancel down to one small term
    f[:, 2, 1::2] = -f[:, 2, 0::2]
    # requests 3 and 4: tiny and huge vectors; request 5 mixes the scales of its rows
    f[:, 3] *= np.float32(2.0 ** -100)
    f[:, 4] *= np.float32(2.0 ** 100)
    f[:, 5] *= (np.float32(2.0) ** np.linspace(-90, 90, hq)).astype(np.float32)[None, :, None]
    q_h = synth.bf16_round_bits(f)
    q_h[:, 1, 1::2] = q_h[:, 1, 0::2] ^ 0x8000          # exact negations after rounding as well
    q_h[:, 2, 1::2] = q_h[:, 2, 0::2] ^ 0x8000
    q_h[:, 2, :, 7] = 0                                 # (added to a term of size 1 it would be rounded away)
    q_h[:, 2, 0::g, 7] = synth.bf16_round_bits(np.float32(2.0 ** -30))
    q_codes = torch.full((n_layers, n_req, hq, 16), 0xEE, dtype=torch.uint8, device=dev)
    q_sum = torch.full((n_layers, n_req, 128), 77, dtype=torch.int16, device=dev)
    qbar = torch.full((n_layers, n_req, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(bf16_dev(q_h, dev), bf16_dev(w_bits, dev), hkv, q_codes, q_sum, qbar, n_req)
    torch.cuda.synchronize()
    for l in range(n_layers):
        want_q = O.hash_encode(q_h[l], w_f32)
        assert np.array_equal(q_codes[l].cpu().numpy(), want_q), l
        pm = np.unpackbits(want_q, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
        assert np.array_equal(q_sum[l].cpu().numpy(), pm.sum(1)), l
        qm = np.stack([O.q_head_mean(synth.bf16_widen(q_h[l][r]), hkv) for r in range(n_req)])
        want_bar = O.hash_encode_f32(qm, w_f32)
        assert np.array_equal(qbar[l].cpu().numpy(), want_bar), l
        # the cases are what they claim to be
        assert not want_q[0, 0::2].any() and want_q[0, 1::2].any()
        assert not want_bar[1].any() and want_bar[2].any()
        assert want_q[3].any() and want_q[4].any()


def test_hash_query_rows_outside_the_layer_are_skipped(ucm, dev):
    """A request whose q_rows entry is negative or past the layer's queries leaves its outputs untouched."""
    from ucm_amd import ops

    hq, hkv, n_tok = 32, 8, 5
    w_bits, w_f32 = make_weights(870)
    q_h = synth.normal_bf16_bits(871, (2, n_tok, hq, 128))
    q_rows = np.array([4, -3, 5, 0], np.int32)
    q_codes = torch.full((2, 4, hq, 16), 0xEE, dtype=torch.uint8, device=dev)
    q_sum = torch.full((2, 4, 128), 77, dtype=torch.int16, device=dev)
    qbar = torch.full((2, 4, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(bf16_dev(q_h, dev), bf16_dev(w_bits, dev), hkv, q_codes, q_sum, qbar, 4, q_rows=i32(q_rows, dev))
    torch.cuda.synchronize()
    for l in range(2):
        for r, row in enumerate(q_rows):
            if 0 <= row < n_tok:
                assert np.array_equal(q_codes[l, r].cpu().numpy(), O.hash_encode(q_h[l, row], w_f32)), (l, r)
            else:
                assert (q_codes[l, r] == 0xEE).all() and (q_sum[l, r] == 77).all() and (qbar[l, r] == 0xEE).all(), (l, r)


def test_hash_queries_scores_and_selection(ucm, dev):
    """Config-5 shape in small: ragged batch, 8 kv heads, 32 query heads, 2 layers."""
    from ucm_amd import ops

    n_layers, hq, hkv, bs = 2, 32, 8, 128
    lens = np.array([5, 33, 1, 64, 17, 3], np.int32)
    rows = int(lens.sum())
    off = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    w_bits, w_f32 = make_weights(820)
    g = torch.Generator(device=dev)
    g.manual_seed(821)
    caches = [torch.randn(rows, bs, hkv, 128, device=dev, generator=g).to(torch.bfloat16) for _ in range(n_layers)]
    lp = ops.LayerPointers(caches)
    colsum = torch.zeros((n_layers, rows, hkv, 128), dtype=torch.int16, device=dev)
    bcodes = torch.zeros((n_layers, rows, hkv, 16), dtype=torch.uint8, device=dev)
    tcodes = torch.zeros((n_layers, rows, bs, hkv, 16), dtype=torch.uint8, device=dev)
    wd = bf16_dev(w_bits, dev)
    ops.hash_encode_blocks(lp, None, None, rows, wd, bs, hkv, rows, colsum, bcodes, token_codes=tcodes)
    q_h = synth.normal_bf16_bits(822, (n_layers, len(lens) + 2, hq, 128))
    q_rows = np.array([3, 0, 7, 1, 2, 5], np.int32)
    q_codes = torch.zeros((n_layers, len(lens), hq, 16), dtype=torch.uint8, device=dev)
    q_sum = torch.zeros((n_layers, len(lens), 128), dtype=torch.int16, device=dev)
    qbar = torch.zeros((n_layers, len(lens), hkv, 16), dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(bf16_dev(q_h, dev), wd, hkv, q_codes, q_sum, qbar, len(lens), q_rows=i32(q_rows, dev))
    torch.cuda.synchronize()
    tc = tcodes.cpu().numpy()
    for l in range(n_layers):
        kc = caches[l].view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(tc[l], O.hash_encode(kc, w_f32)), l
        want_q = O.hash_encode(q_h[l][q_rows], w_f32)
        assert np.array_equal(q_codes[l].cpu().numpy(), want_q)
        pm = np.unpackbits(want_q, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
        assert np.array_equal(q_sum[l].cpu().numpy(), pm.sum(1))
        qm = np.stack([O.q_head_mean(synth.bf16_widen(q_h[l][r]), hkv) for r in q_rows])
        assert np.array_equal(qbar[l].cpu().numpy(), O.hash_encode_f32(qm, w_f32))

    for mode, rnd in ((ops.HASH_SCORE_SUM, False), (ops.HASH_SCORE_SUM, True), (ops.HASH_SCORE_BLOCK_CODE, False)):
        scores = torch.full((n_layers, rows), -1.0, device=dev)
        ops.hash_score_blocks(mode, q_sum, qbar, colsum, bcodes, i32(off, dev), i32(lens, dev), rows, scores,
                              round_fp16=rnd)
        topk = np.array([max(2, n // 3) + 2 for n in lens], np.int32)
        idx = torch.full((n_layers, len(lens), int(lens.max())), -1, dtype=torch.int32, device=dev)
        cnt = torch.zeros((n_layers, len(lens)), dtype=torch.int32, device=dev)
        # KvComp keeps the first block and the last one out of the candidates (kvcomp.py:219-221)
        ops.topk_windows(scores, i32(off, dev), i32(lens, dev), i32(topk, dev), int(lens.max()), idx, cnt,
                         start_w=1, end_w=1)
        torch.cuda.synchronize()
        sc = scores.cpu().numpy()
        for l in range(n_layers):
            for r, n in enumerate(lens):
                a = off[r]
                if mode == ops.HASH_SCORE_SUM:
                    key_codes = tc[l][a : a + n].transpose(0, 2, 1, 3)      # [n, hkv, bs, 16] as the reference stores them
                    want = O.hash_scores_sum(q_codes[l, r].cpu().numpy(), key_codes).astype(np.float32)
                    if rnd:
                        want = want.astype(np.float16).astype(np.float32)
                else:
                    want = O.hash_scores_block(qbar[l, r].cpu().numpy(), bcodes[l, a : a + n].cpu().numpy()).astype(np.float32)
                assert np.array_equal(sc[l, a : a + n], want), (mode, rnd, l, r)
                sel = O.topk_windows(want, int(topk[r]), 1, 1)
                assert cnt[l, r] == len(sel) and np.array_equal(idx[l, r, : len(sel)].cpu().numpy(), sel), (mode, l, r)


def cancelling_keys(seed, w_f32, n_vec, perm):
    """Vectors whose projection on one chosen weight column is built to cancel: the 128 dims are taken in pairs (in
    the order `perm`), the second element of a pair being the bf16 neighbour that brings the running sum closest to
    zero, with magnitudes that fall off at a rate drawn per vector.  The projection ends between 2^-45 and 2^-18 of
    ||x|| ||w|| while the partial sums along the way are as large as any - the worst case for a sum accumulated in
    fp32 in whatever order.  Returns bf16 bits [n_vec, 128] and the column each vector was built against."""
    rng = np.random.default_rng(seed)
    cols = rng.integers(0, 128, n_vec)
    wc = w_f32.T[cols].astype(np.float64)                                # [n_vec, 128]
    rate = rng.random((n_vec, 1)) * 0.35
    a = synth.bf16_widen(synth.bf16_round_bits((rng.standard_normal((n_vec, 64)) * 2.0 ** (-rate * np.arange(64))).astype(np.float32)))
    x = np.zeros((n_vec, 128), np.float32)
    r = np.zeros(n_vec)
    for i in range(64):
        p0, p1 = perm[2 * i], perm[2 * i + 1]
        w1 = np.where(wc[:, p1] == 0, 1.0, wc[:, p1])
        t0 = a[:, i].astype(np.float64) * wc[:, p0]
        ideal = (-(r + t0) / w1).astype(np.float32)
        ideal = np.clip(ideal, -1e30, 1e30)
        lo = (ideal.view(np.uint32) & np.uint32(0xffff0000)).view(np.float32)            # towards zero
        hi = ((ideal.view(np.uint32) & np.uint32(0xffff0000)) + np.uint32(0x10000)).view(np.float32)
        y = np.where(np.abs(r + t0 + lo.astype(np.float64) * w1) <= np.abs(r + t0 + hi.astype(np.float64) * w1), lo, hi)
        y = np.where(np.isfinite(y) & (np.abs(y) < 1e20), y, np.float32(0))
        x[:, p0], x[:, p1] = a[:, i], y
        r = r + t0 + y.astype(np.float64) * wc[:, p1]
    bits_ = synth.bf16_round_bits(x)
    assert np.array_equal(synth.bf16_widen(bits_), x)                                    # every value is a bf16 value
    return bits_, cols


@pytest.mark.parametrize("paired", ["neighbours", "scattered"])
def test_hash_encode_projections_built_to_cancel(ucm, dev, paired):
    """Seven thousand key vectors, each built so that its projection on one weight column cancels down to between
    2^-45 and 2^-18 of ||x|| ||w|| (neighbouring dims paired, or dims paired at random so that the cancellation spans
    the matrix instructions): the signs - those the matrix cores keep and those that are redone - must be the
    oracle's, and so must the column sums."""
    from ucm_amd import ops

    hkv, bs, nb = 8, 128, 7
    w_bits, w_f32 = make_weights(880)
    perm = np.arange(128) if paired == "neighbours" else np.random.default_rng(881).permutation(128)
    x_bits, cols = cancelling_keys(882, w_f32, nb * bs * hkv, perm)
    x64 = synth.bf16_widen(x_bits).astype(np.float64)
    ratio = np.abs((x64 * w_f32.T[cols]).sum(1)) / (np.linalg.norm(x64, axis=1) * np.linalg.norm(w_f32.T[cols].astype(np.float64), axis=1))
    assert np.median(ratio) < 2.0 ** -24 and (ratio > 2.0 ** -24).sum() > 500 and (ratio < 2.0 ** -30).sum() > 500
    keys_h = x_bits.reshape(nb, bs, hkv, 128)
    lp = ops.LayerPointers([bf16_dev(keys_h, dev)])
    colsum = torch.zeros((1, nb, hkv, 128), dtype=torch.int16, device=dev)
    bcodes = torch.zeros((1, nb, hkv, 16), dtype=torch.uint8, device=dev)
    tcodes = torch.zeros((1, nb, bs, hkv, 16), dtype=torch.uint8, device=dev)
    ops.hash_encode_blocks(lp, None, None, nb, bf16_dev(w_bits, dev), bs, hkv, nb, colsum, bcodes, token_codes=tcodes)
    torch.cuda.synchronize()
    want = O.hash_encode(keys_h, w_f32)
    assert np.array_equal(tcodes[0].cpu().numpy(), want)
    assert np.array_equal(colsum[0].cpu().numpy(), O.hash_colsum(want))
    assert np.array_equal(bcodes[0].cpu().numpy(), O.hash_majority(want))


def test_hash_encode_keys_beyond_the_fp32_range(ucm, dev):
    """Keys whose fp32 sums overflow on the way (components up to 3e38: the exact sum may be finite and of either
    sign where the matrix cores hold an infinity or a NaN), keys with infinite components and keys with NaN: the
    codes are still the signs of the sums accumulated exactly, d ascending (NaN is not > 0: bit 0), because a key
    without a finite error bound has all its results redone."""
    from ucm_amd import ops

    hkv, bs, nb = 8, 128, 6
    w_bits, w_f32 = make_weights(890)
    rng = np.random.default_rng(891)
    keys_h = synth.normal_bf16_bits(892, (nb, bs, hkv, 128))
    raw = rng.integers(0, 1 << 16, size=(bs, hkv, 128), dtype=np.uint16)
    keys_h[0] = raw                                                    # any bit pattern: NaN, infinities, 1e38 next to 1e-38
    finite = raw.copy()
    finite[(finite & 0x7F80) == 0x7F80] &= 0xFF7F                      # exponent 255 -> 254: the same without NaN and infinity
    keys_h[1] = finite
    huge = synth.bf16_round_bits((rng.standard_normal((bs, hkv, 128)) * 1e38).clip(-3e38, 3e38).astype(np.float32))
    keys_h[2] = huge                                                   # every partial sum is out of range
    keys_h[3, ::3, :, 17] = 0x7F80                                     # one +inf in otherwise ordinary keys
    keys_h[3, 1::3, :, 40] = 0xFF80                                    # ... or +inf and -inf
    keys_h[3, 1::3, :, 90] = 0x7F80
    keys_h[4, ::2, :, 5] = 0x7FC0                                      # one NaN
    keys_h[5, :, ::2, 0] = synth.bf16_round_bits(np.array([2.5e38], np.float32))[0]    # one component that alone overflows
    lp = ops.LayerPointers([bf16_dev(keys_h, dev)])
    colsum = torch.zeros((1, nb, hkv, 128), dtype=torch.int16, device=dev)
    bcodes = torch.zeros((1, nb, hkv, 16), dtype=torch.uint8, device=dev)
    tcodes = torch.zeros((1, nb, bs, hkv, 16), dtype=torch.uint8, device=dev)
    ops.hash_encode_blocks(lp, None, None, nb, bf16_dev(w_bits, dev), bs, hkv, nb, colsum, bcodes, token_codes=tcodes)
    torch.cuda.synchronize()
    with np.errstate(all="ignore"):
        want = O.hash_encode(keys_h, w_f32)
    # the cases are what they claim to be: fp32 sums of block 2 are not finite, its exact sums have both signs
    x2 = synth.bf16_widen(huge).reshape(-1, 128)
    with np.errstate(all="ignore"):
        assert not np.isfinite(x2 @ w_f32).any()
    assert 0.3 < np.unpackbits(want[2]).mean() < 0.7
    assert not want[4, ::2].any() and want[4, 1::2].any()
    got = tcodes[0].cpu().numpy()
    for b in range(nb):
        assert np.array_equal(got[b], want[b]), b
    assert np.array_equal(colsum[0].cpu().numpy(), O.hash_colsum(want))
    assert np.array_equal(bcodes[0].cpu().numpy(), O.hash_majority(want))
    # the summaries alone (no token codes) take the same path
    colsum2, bcodes2 = torch.zeros_like(colsum), torch.zeros_like(bcodes)
    ops.hash_encode_blocks(lp, None, None, nb, bf16_dev(w_bits, dev), bs, hkv, nb, colsum2, bcodes2)
    assert torch.equal(colsum2, colsum) and torch.equal(bcodes2, bcodes)


def test_hash_query_codes_beyond_the_fp32_range(ucm, dev):
    """Query rows with components up to 3e38 (one head per kv head, so that the group mean is the row itself): a
    tile whose largest norm is not finite is redone whole, the signs are those of the exact sums."""
    from ucm_amd import ops

    hq = hkv = 8
    n_layers, n_req = 1, 4
    w_bits, w_f32 = make_weights(895)
    rng = np.random.default_rng(896)
    q_h = synth.normal_bf16_bits(897, (n_layers, n_req, hq, 128))
    q_h[0, 1] = synth.bf16_round_bits((rng.standard_normal((hq, 128)) * 1e38).clip(-3e38, 3e38).astype(np.float32))
    q_h[0, 2, ::2] = q_h[0, 1, ::2]                                    # huge rows next to ordinary ones
    q_h[0, 3, :, 9] = synth.bf16_round_bits(np.array([2.5e38], np.float32))[0]
    q_codes = torch.full((n_layers, n_req, hq, 16), 0xEE, dtype=torch.uint8, device=dev)
    q_sum = torch.full((n_layers, n_req, 128), 77, dtype=torch.int16, device=dev)
    qbar = torch.full((n_layers, n_req, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(bf16_dev(q_h, dev), bf16_dev(w_bits, dev), hkv, q_codes, q_sum, qbar, n_req)
    torch.cuda.synchronize()
    want_q = O.hash_encode(q_h[0], w_f32)
    assert 0.3 < np.unpackbits(want_q[1]).mean() < 0.7
    assert np.array_equal(q_codes[0].cpu().numpy(), want_q)
    pm = np.unpackbits(want_q, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
    assert np.array_equal(q_sum[0].cpu().numpy(), pm.sum(1))
    assert np.array_equal(qbar[0].cpu().numpy(), want_q)               # a group of one head: the mean is the row


# ------------------------------------------------------------ a float16 model

def exact_codes(x64, w64):
    """Signs of the products summed in float64, d ascending: [..., 128] x [128, 128] -> uint8 [..., 16]."""
    acc = np.zeros(x64.shape[:-1] + (128,))
    with np.errstate(all="ignore"):
        for d_ in range(128):
            acc = acc + x64[..., d_, None] * w64[d_]
    return np.packbits(acc > 0, axis=-1, bitorder="little")


def f16_dev(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.parametrize("hkv,bs", [(8, 128), (2, 16), (1, 32), (4, 520), (8, 272)])
def test_hash_encode_blocks_of_a_float16_model(ucm, dev, hkv, bs):
    """Float16 keys and weights (ucm_hash_encode_blocks_f16): the codes are the signs of the exactly accumulated
    float16 products - the oracle's float64 sums of the widened values and numpy's own agree on that - with rows
    that cancel exactly, rows of subnormal components (the matrix instruction takes them as they are), rows at the
    top of float16's range, infinities and NaN."""
    from ucm_amd import ops

    n_layers, nb, rows = 2, 9, 12
    rng = np.random.default_rng(1500 + hkv + bs)
    w16 = (rng.standard_normal((128, 128)) * 2.0).astype(np.float16)
    caches_h = [(rng.standard_normal((nb, bs, hkv, 128)) * rng.choice([1e-3, 1.0, 30.0], size=(nb, bs, hkv, 1))).astype(np.float16)
                for _ in range(n_layers)]
    for c in caches_h:
        c[0, 0, 0, :] = 0
        c[0, 1, 0, :] = 0
        c[0, 1, 0, 5] = 3.0
        c[1, 2, 0, :3] = [1.0e4, -1.0e4, 1.0e-4]
        c[2, 3, 0, :] = -c[2, 4, 0, :]
        c[3, 0, 0, :] = (rng.standard_normal(128) * 2e-6).astype(np.float16)          # all components subnormal
        c[3, 1, 0, :] = (rng.standard_normal(128) * 2e-6).astype(np.float16)
        c[3, 1, 0, 7] = 0.5                                                            # ... but one
        c[4, 0, 0, :] = (rng.standard_normal(128) * 3e4).clip(-65504, 65504).astype(np.float16)
        c[4, 1, 0, 9] = np.inf
        c[4, 2, 0, 9], c[4, 2, 0, 77] = np.inf, -np.inf
        c[4, 3, 0, 100] = np.nan
    caches = [f16_dev(c, dev) for c in caches_h]
    lp = ops.LayerPointers(caches)
    ids = synth.permutation(1510, nb)[:7]
    slots = synth.permutation(1511, rows)[:7]
    colsum = torch.full((n_layers, rows, hkv, 128), 77, dtype=torch.int16, device=dev)
    bcodes = torch.full((n_layers, rows, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    tcodes = torch.full((n_layers, rows, bs, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_blocks(lp, i32(ids, dev), i32(slots, dev), len(ids), f16_dev(w16, dev), bs, hkv, nb, colsum, bcodes,
                           token_codes=tcodes)
    torch.cuda.synchronize()
    got_t, got_s, got_b = tcodes.cpu().numpy(), colsum.cpu().numpy(), bcodes.cpu().numpy()
    w_f32 = w16.astype(np.float32)
    for l in range(n_layers):
        with np.errstate(all="ignore"):
            want_t = O.hash_encode_f32(caches_h[l][ids].astype(np.float32), w_f32)
        if l == 0:
            assert np.array_equal(want_t, exact_codes(caches_h[l][ids].astype(np.float64), w16.astype(np.float64)))
        assert np.array_equal(got_t[l][slots], want_t), l
        assert np.array_equal(got_s[l][slots], O.hash_colsum(want_t)), l
        assert np.array_equal(got_b[l][slots], O.hash_majority(want_t)), l
        rest = np.setdiff1d(np.arange(rows), slots)
        assert np.all(got_t[l][rest] == 0xEE) and np.all(got_s[l][rest] == 77) and np.all(got_b[l][rest] == 0xEE)
    colsum2, bcodes2 = torch.zeros_like(colsum), torch.zeros_like(bcodes)
    ops.hash_encode_blocks(lp, i32(ids, dev), i32(slots, dev), len(ids), f16_dev(w16, dev), bs, hkv, nb, colsum2, bcodes2)
    at = torch.from_numpy(slots.astype(np.int64)).to(dev)
    assert torch.equal(colsum2[:, at], colsum[:, at]) and torch.equal(bcodes2[:, at], bcodes[:, at])
    # keys of one type with weights of the other are refused
    with pytest.raises(ValueError):
        ops.hash_encode_blocks(lp, None, None, nb, f16_dev(w16, dev).to(torch.bfloat16), bs, hkv, nb, colsum, bcodes)


@pytest.mark.parametrize("paired", ["neighbours", "scattered"])
def test_hash_encode_float16_projections_built_to_cancel(ucm, dev, paired):
    """Float16 key vectors built so that their projection on one weight column cancels down to a sliver of
    ||x|| ||w|| while the partial sums stay large: every sign, the matrix cores' and the redone ones', is the exact one."""
    from ucm_amd import ops

    hkv, bs, nb = 8, 128, 6
    n_vec = nb * bs * hkv
    rng = np.random.default_rng(1520)
    w16 = (rng.standard_normal((128, 128)) * 2.0).astype(np.float16)
    w64 = w16.astype(np.float64)
    perm = np.arange(128) if paired == "neighbours" else rng.permutation(128)
    cols = rng.integers(0, 128, n_vec)
    wc = w64.T[cols]
    rate = rng.random((n_vec, 1)) * 0.12                       # (float16 has 40 binades: the magnitudes fall off slowly)
    a = (rng.standard_normal((n_vec, 64)) * 2.0 ** (-rate * np.arange(64))).astype(np.float16)
    x = np.zeros((n_vec, 128), np.float16)
    r = np.zeros(n_vec)
    for i in range(64):
        p0, p1 = perm[2 * i], perm[2 * i + 1]
        w1 = np.where(wc[:, p1] == 0, 1.0, wc[:, p1])
        t0 = a[:, i].astype(np.float64) * wc[:, p0]
        ideal = np.clip(-(r + t0) / w1, -6e4, 6e4)
        near = ideal.astype(np.float16)
        cands = np.stack([near, np.nextafter(near, np.float16(np.inf)), np.nextafter(near, np.float16(-np.inf))])
        cands = np.where(np.isfinite(cands), cands, near[None])
        err = np.abs(r + t0 + cands.astype(np.float64) * w1)
        y = np.take_along_axis(cands, err.argmin(0)[None], 0)[0]
        x[:, p0], x[:, p1] = a[:, i], y
        r = r + t0 + y.astype(np.float64) * wc[:, p1]
    x64 = x.astype(np.float64)
    ratio = np.abs((x64 * wc).sum(1)) / (np.linalg.norm(x64, axis=1) * np.linalg.norm(wc, axis=1))
    assert np.median(ratio) < 2.0 ** -14 and (ratio < 2.0 ** -17).sum() > 300      # (eleven bits: the slivers are wider than bfloat16's)
    keys_h = x.reshape(nb, bs, hkv, 128)
    lp = ops.LayerPointers([f16_dev(keys_h, dev)])
    colsum = torch.zeros((1, nb, hkv, 128), dtype=torch.int16, device=dev)
    bcodes = torch.zeros((1, nb, hkv, 16), dtype=torch.uint8, device=dev)
    tcodes = torch.zeros((1, nb, bs, hkv, 16), dtype=torch.uint8, device=dev)
    ops.hash_encode_blocks(lp, None, None, nb, f16_dev(w16, dev), bs, hkv, nb, colsum, bcodes, token_codes=tcodes)
    torch.cuda.synchronize()
    want = O.hash_encode_f32(keys_h.astype(np.float32), w16.astype(np.float32))
    assert np.array_equal(tcodes[0].cpu().numpy(), want)
    assert np.array_equal(colsum[0].cpu().numpy(), O.hash_colsum(want))
    assert np.array_equal(bcodes[0].cpu().numpy(), O.hash_majority(want))


@pytest.mark.parametrize("g", [2, 3, 4, 8])
def test_hash_query_mean_codes_of_a_float16_model_with_grouped_heads(ucm, dev, g):
    """Several float16 query heads per kv head: the mean codes are the exact signs of (fp32 sequential sum * 1/g) . w,
    also where the heads of a group cancel down to a few low bits, for subnormal rows and for large ones; the
    per-head codes and their sums are unchanged by the grouping."""
    from ucm_amd import ops

    hkv, n_layers, n_req = 8, 2, 5
    hq = hkv * g
    rng = np.random.default_rng(1531 + g)
    w16 = (rng.standard_normal((128, 128)) * 2.0).astype(np.float16)
    q = rng.standard_normal((n_layers, n_req, hq, 128)).astype(np.float32)
    q[:, 1] *= 3e-6                                            # subnormal components
    q[:, 2] *= 1500.0
    q16 = q.astype(np.float16)
    # request 3: the heads of a group cancel but for the last bit of one component of one of them
    q16[:, 3, 1::g] = -q16[:, 3, 0::g]
    if g > 2:
        q16[:, 3].reshape(n_layers, hkv, g, 128)[:, :, 2:] = 0
    q16[:, 3, 0::g, 7] = np.nextafter(q16[:, 3, 0::g, 7], np.float16(np.inf))
    q_codes = torch.full((n_layers, n_req, hq, 16), 0xEE, dtype=torch.uint8, device=dev)
    q_sum = torch.full((n_layers, n_req, 128), 77, dtype=torch.int16, device=dev)
    qbar = torch.full((n_layers, n_req, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(f16_dev(q16, dev), f16_dev(w16, dev), hkv, q_codes, q_sum, qbar, n_req)
    torch.cuda.synchronize()
    inv = np.float32(1.0) / np.float32(g)
    for l in range(n_layers):
        want = exact_codes(q16[l].astype(np.float64), w16.astype(np.float64))
        assert np.array_equal(q_codes[l].cpu().numpy(), want), l
        pm = np.unpackbits(want, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
        assert np.array_equal(q_sum[l].cpu().numpy(), pm.sum(1)), l
        grouped = q16[l].astype(np.float32).reshape(n_req, hkv, g, 128)
        mean = grouped[:, :, 0]
        for j in range(1, g):
            mean = mean + grouped[:, :, j]                     # fp32, head order
        mean = mean * inv
        want_bar = exact_codes(mean.astype(np.float64), w16.astype(np.float64))
        for r in range(n_req):
            assert np.array_equal(O.q_head_mean(q16[l, r].astype(np.float32), hkv), mean[r])
        assert np.array_equal(qbar[l].cpu().numpy(), want_bar), l
        assert want_bar[3].any() and not np.array_equal(want_bar[3], want_bar[0])


def test_hash_query_codes_of_a_float16_model(ucm, dev):
    """Float16 queries and weights, one query head per kv head (what the plugin passes after its own group mean):
    codes, their +-1 sums and the mean codes (the rows' own codes); rows that cancel exactly or down to one small
    term, rows of subnormal components and rows of large ones."""
    from ucm_amd import ops

    hkv, n_layers, n_req = 8, 2, 6
    rng = np.random.default_rng(1530)
    w16 = (rng.standard_normal((128, 128)) * 2.0).astype(np.float16)
    w16[1] = w16[0]
    w16[5] = -w16[4]
    q = rng.standard_normal((n_layers, n_req, hkv, 128)).astype(np.float32)
    q[:, 0] = 0
    q[:, 0, :, 0], q[:, 0, :, 1] = 3.0, -3.0                   # cancels exactly against the equal weight rows
    q[:, 0, :, 4], q[:, 0, :, 5] = 0.75, 0.75
    q[:, 0, 1::2, 2] = 2.0 ** -14                              # every second row keeps one small term
    q[:, 1] *= 2e-6                                            # subnormal components
    q[:, 2] *= 2000.0
    q[:, 3] *= (2.0 ** np.linspace(-20, 12, hkv))[None, :, None]
    q16 = q.astype(np.float16)
    q_codes = torch.full((n_layers, n_req, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    q_sum = torch.full((n_layers, n_req, 128), 77, dtype=torch.int16, device=dev)
    qbar = torch.full((n_layers, n_req, hkv, 16), 0xEE, dtype=torch.uint8, device=dev)
    ops.hash_encode_queries(f16_dev(q16, dev), f16_dev(w16, dev), hkv, q_codes, q_sum, qbar, n_req)
    torch.cuda.synchronize()
    for l in range(n_layers):
        want = exact_codes(q16[l].astype(np.float64), w16.astype(np.float64))
        assert np.array_equal(want, O.hash_encode_f32(q16[l].astype(np.float32), w16.astype(np.float32)))
        assert np.array_equal(q_codes[l].cpu().numpy(), want), l
        assert np.array_equal(qbar[l].cpu().numpy(), want), l
        pm = np.unpackbits(want, axis=-1, bitorder="little").astype(np.int32) * 2 - 1
        assert np.array_equal(q_sum[l].cpu().numpy(), pm.sum(1)), l
        assert not want[0, 0::2].any() and want[0, 1::2].any() and want[1].any()
