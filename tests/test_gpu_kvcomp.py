"""KvComp-shaped host layer (HashEncoder + plugin) against the CPU oracle."""
import types

import numpy as np
import pytest
import torch

import oracle as O
import synth
from test_gpu_host_layer import make_config

pytestmark = pytest.mark.gpu


def bf16_bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def test_hash_encoder_surface(ucm, dev):
    from ucm_amd.sparse.kvcomp.hash_encoder import HashEncoder

    enc = HashEncoder(128, 128, torch.bfloat16, dev)
    assert enc.hash_weights.shape == (128, 128) and enc.hash_numbers == 16
    assert 1.5 < float(enc.hash_weights.float().std()) < 2.5          # N(0, std 2), hash_encoder.py:65-71
    w_bits = synth.bf16_round_bits(synth.normal_f32(950, (128, 128)) * np.float32(2.0))
    w = torch.from_numpy(w_bits.view(np.int16)).to(dev).view(torch.bfloat16)
    enc.set_hash_weight(w)
    with pytest.raises(ValueError):
        enc.set_hash_weight(w[:, :64])
    with pytest.raises(ValueError):
        enc.set_hash_weight(w.float())
    with pytest.raises(ValueError):
        enc.compute_hash(torch.zeros(4, 64, dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError):
        HashEncoder(128, 100, torch.bfloat16, dev)
    with pytest.raises(ValueError):
        HashEncoder(64, 128, torch.bfloat16, dev)                       # not built: refused, no other path
    for shape in [(3, 5, 128), (1, 128), (64, 128), (7, 2, 3, 128), (0, 128)]:
        x_bits = synth.normal_bf16_bits(951 + len(shape), shape)
        x = torch.from_numpy(x_bits.view(np.int16)).to(dev).view(torch.bfloat16)
        got = enc.compute_hash(x)
        assert got.shape == shape[:-1] + (16,) and got.dtype == torch.uint8
        if x.numel():
            assert np.array_equal(got.cpu().numpy(), O.hash_encode(x_bits, synth.bf16_widen(w_bits))), shape
    # fp32 input is converted to the encoder's dtype first (hash_encoder.py:121-122)
    xf = torch.from_numpy(synth.normal_f32(960, (9, 128))).to(dev)
    assert torch.equal(enc.compute_hash(xf), enc.compute_hash(xf.to(torch.bfloat16)))
    # unpack: +-1 in fp16, bit j of byte b is column 8b+j
    codes = enc.compute_hash(xf)
    pm = enc._unpack_hash(codes)
    assert pm.dtype == torch.float16 and pm.shape == (9, 128)
    want = np.unpackbits(codes.cpu().numpy(), axis=-1, bitorder="little").astype(np.float32) * 2 - 1
    assert np.array_equal(pm.float().cpu().numpy(), want)


def test_kvcomp_plugin_flow(ucm, dev):
    """Prefill of 20 full blocks + 5 tokens, then decode on the sparsified block list: windows restored at step 1,
    retrieval at steps 1 and 5 picks what the oracle picks from the same keys, the chosen blocks land in the
    request's middle cache blocks in ascending order, a block filled during decode is dumped and hashed."""
    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseRole
    from ucm_amd.sparse.factory import UcmSparseFactory
    from ucm_amd.sparse.kvcomp.kvcomp import KvComp
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    ns = types.SimpleNamespace
    hq, hkv, d, L, bs, nb = 8, 2, 128, 2, 16, 64
    cfg = make_config(hq, hkv, d, L, bs, 16 * 64, {})
    cfg.kv_transfer_config.kv_connector_extra_config = {"ucm_sparse_config": {"KvComp": {"keep_token_codes": True}}}
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    assert isinstance(plugin, KvComp)
    slice_bytes = bs * hkv * d * 2
    plugin.connector = store = UcmHipBlockStore({"kv_block_size": L * 2 * slice_bytes, "max_cache_size": 40 * L * 2 * slice_bytes})

    n_prompt = 20 * bs + 5
    full_ids = [int(x) for x in synth.permutation(970, nb)[:21]]
    req = ns(block_ids=[list(full_ids)], num_computed_tokens=0, prompt_token_ids=[1] * n_prompt, output_token_ids=[],
             num_prompt_tokens=n_prompt, num_output_tokens=0, num_tokens=n_prompt, request_id="A")
    assert plugin.estimate_num_slots_sparsed(req) == INVALID_SLOT
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    caches = [torch.randn(2, nb, bs, hkv, d, device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    original = [c.clone() for c in caches]
    names = [f"model.layers.{l}.self_attn.attn" for l in range(L)]
    fc = ns(no_compile_layers={names[l]: ns(kv_cache=[caches[l]]) for l in range(L)}, virtual_engine=0,
            attn_metadata=ns(query_start_loc=torch.tensor([0, 1])))
    ib = ns(req_id_to_index={"A": 0})

    def run_step(n_tok):
        so = ns(num_scheduled_tokens={"A": n_tok}, req_sparsed_slots={"A": 0})
        plugin.build_sparse_meta(so, {"A": req}, ib)
        qs = []
        for l in range(L):
            q = torch.randn(n_tok, hq, d, device=dev, generator=g).to(torch.bfloat16)
            qs.append(q)
            plugin.attention_begin(q, None, None, names[l], fc)
            plugin.attention_finished(q, None, None, None, names[l], fc)
        req.num_computed_tokens += n_tok
        return qs

    run_step(n_prompt)
    torch.cuda.synchronize()
    w_f32 = plugin.hash_encoder.hash_weights.float().cpu().numpy()
    states = plugin.req_states["A"]
    base = plugin.segment_base("A")
    key_codes = []                                           # per layer: [20, bs, hkv, 16] of the original blocks
    for l in range(L):
        assert states[l].num_blocks_hashed == 20
        want = O.hash_encode(bf16_bits(original[l][0][full_ids[:20]]), w_f32)
        assert np.array_equal(plugin.token_codes[l, base : base + 20].cpu().numpy(), want)
        assert np.array_equal(plugin.colsum[l, base : base + 20].cpu().numpy(), O.hash_colsum(want))
        key_codes.append(want)
        assert all(store.lookup([f"req_A_blk_{b}"]) == [False] for b in range(20))   # dumped, not committed by the plugin
        assert all(f"req_A_blk_{b}" in store.slot_of for b in range(20))

    # the scheduler now shrinks the request to init + 30 % of the middle + local blocks (kvcomp.py:571-587)
    req.output_token_ids.append(7)
    req.num_output_tokens, req.num_tokens = 1, n_prompt + 1
    slots = plugin.estimate_num_slots_sparsed(req)
    n_total = -(-(n_prompt + 1) // bs)                      # 21 blocks
    mid = int((n_total - 1 - 2) * 0.3)                      # 5
    assert slots == (1 + mid + 2) * bs - (bs - (n_prompt + 1) % bs)
    kept = full_ids[-(-(-slots // bs)):]                    # the last ceil(slots / bs) = 8 cache blocks
    assert len(kept) == 1 + mid + 2
    req.block_ids = [list(kept)]

    def expected(l, q, n_hashed):
        qm = q[0].view(hkv, hq // hkv, d).mean(1)                                        # bf16 group mean, as the plugin takes it
        q_codes = O.hash_encode(bf16_bits(qm), w_f32)                                    # [hkv, 16]
        first, end = 1, n_hashed - 2 + 1
        kc = key_codes[l][first:end].transpose(0, 2, 1, 3)                               # [n, hkv, bs, 16]
        sc = O.hash_scores_sum(q_codes, kc).astype(np.float16)                           # the reference's fp16 scores
        order = np.argsort(-sc.astype(np.float32), kind="stable")[:mid]
        return sorted(first + int(i) for i in order)

    for step in range(1, 7):
        if step > 1:
            req.output_token_ids.append(7)
            req.num_output_tokens = step
            req.num_tokens = n_prompt + step
        qs = run_step(1)
        torch.cuda.synchronize()
        for l in range(L):
            st = states[l]
            if step in (1, 5):
                want = expected(l, qs[l], 20)
                assert st.last_selection == want, (step, l)
                for kv in range(2):
                    got = caches[l][kv][kept[1 : 1 + mid]]
                    assert torch.equal(got, original[l][kv][[full_ids[b] for b in want]]), (step, l, kv)
                    # windows: logical block 0 in the first kept block, the last two logical blocks in the last two
                    assert torch.equal(caches[l][kv][kept[0]], original[l][kv][full_ids[0]])
            else:
                assert st.last_selection == expected(l, qs_at[l], 20) if step < 5 else True
        if step in (1, 5):
            qs_at = qs
    # step 1 restored the local window as it was at the end of prefill (blocks 19 and 20 of the prompt)
    # and decode kept writing into the last block; the block that filled up is dumped and hashed
    req.output_token_ids.extend([7] * 12)
    req.num_output_tokens = 18
    req.num_tokens = n_prompt + 18
    req.num_computed_tokens = n_prompt + 10                  # 335 tokens computed: this step completes block 20
    for l in range(L):
        caches[l][0][kept[-1]] = torch.randn(bs, hkv, d, device=dev, generator=g).to(torch.bfloat16)
    run_step(1)
    torch.cuda.synchronize()
    for l in range(L):
        assert states[l].num_blocks_hashed == 21
        want = O.hash_encode(bf16_bits(caches[l][0][kept[-1]])[None], w_f32)
        assert np.array_equal(plugin.token_codes[l, base + 20].cpu().numpy(), want[0])
        assert "req_A_blk_20" in store.slot_of
    plugin.request_finished_in_worker("A")
    assert "A" not in plugin.req_states and "A" not in plugin.segment_of
