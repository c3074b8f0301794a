"""Host-side logic that needs no GPU: the hook surface, the registry, request
bookkeeping and the top-k length rule."""
import math
import inspect
import types

import pytest

import oracle as O

ns = types.SimpleNamespace


class _ModelConfig:
    max_model_len = 4096

    def get_num_kv_heads(self, pc):
        return 8

    def get_num_attention_heads(self, pc):
        return 32

    def get_head_size(self):
        return 128

    def get_num_layers(self, pc):
        return 4


def make_config(name="GSA", cfg=None):
    return ns(model_config=_ModelConfig(), parallel_config=ns(), cache_config=ns(block_size=128),
              scheduler_config=ns(max_num_seqs=8),
              kv_transfer_config=ns(kv_connector_extra_config={"ucm_sparse_config": {name: cfg or {}}}))


def test_hook_surface_matches_the_patched_call_sites(ucm):
    """Names and positional parameters vLLM's patched call sites use
    (vllm-adapt.patch:80-115, :359-364, :573-574, :1159-1176)."""
    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseBase

    want = {
        "bind_sparse_metadata": ["sparse_metadata"],
        "clear_sparse_metadata": [],
        "register_kv_caches": ["kv_caches"],
        "execute_begin": ["scheduler_output"],
        "execute_finished": [],
        "attention_begin": ["query", "key", "value", "layer_name", "forward_context"],
        "attention_finished": ["query", "key", "value", "attn_output", "layer_name", "forward_context"],
        "request_finished_in_worker": ["request_id"],
        "request_begin": ["request_id", "prompt_token_ids"],
        "request_finished_in_scheduler": ["request_id"],
        "estimate_num_slots_sparsed": ["request"],
        "update_state_after_alloc": ["request", "num_blocks"],
        "build_sparse_meta": ["scheduler_output", "requests", "input_batch", "attn_metadata"],
        "allocate_slots": ["request", "num_slots_sparsed", "coordinator", "block_pool", "kv_cache_groups"],
    }
    for name, params in want.items():
        sig = inspect.signature(getattr(UcmSparseBase, name))
        assert list(sig.parameters)[1:] == params, name
    assert INVALID_SLOT == -1
    with pytest.raises(TypeError):
        UcmSparseBase(None, None)  # request_begin is abstract, as in the reference

    class Minimal(UcmSparseBase):
        def request_begin(self, request_id, prompt_token_ids):
            pass

    m = Minimal(None, None)
    assert m.estimate_num_slots_sparsed(None) == INVALID_SLOT and m.allocate_slots(1, 2, 3, 4, 5) is None
    with pytest.raises(AssertionError):
        m._get_sparse_metadata()
    m.bind_sparse_metadata("x")
    assert m._get_sparse_metadata() == "x"
    m.clear_sparse_metadata()


def test_factory_and_process_state(ucm):
    from ucm_amd.sparse import state
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.factory import UcmSparseFactory
    from ucm_amd.sparse.gsa.gsa import GSA

    state.reset_ucm_sparse()
    assert not state.has_ucm_sparse()
    with pytest.raises(RuntimeError, match="not initialized"):
        state.get_ucm_sparse()
    state.ensure_ucm_sparse_initialized(ns(kv_transfer_config=None))
    state.ensure_ucm_sparse_initialized(ns(kv_transfer_config=ns(kv_connector_extra_config={})))
    assert not state.has_ucm_sparse()
    state.ensure_ucm_sparse_initialized(make_config(), UcmSparseRole.SCHEDULER)
    agent = state.get_ucm_sparse()
    assert isinstance(agent, GSA) and agent.role == UcmSparseRole.SCHEDULER
    state.ensure_ucm_sparse_initialized(make_config())
    assert state.get_ucm_sparse() is agent  # created once per process
    state.reset_ucm_sparse()
    with pytest.raises(ValueError, match="Unsupported sparse method"):
        UcmSparseFactory.create_sparse_method(make_config("NoSuchMethod"), UcmSparseRole.WORKER)
    with pytest.raises(ValueError, match="already registered"):
        UcmSparseFactory.register_sparse_method("GSA", "x", "y")


def test_compute_topk_len_matches_the_oracle(ucm):
    from ucm_amd.sparse.utils import compute_topk_len

    for n in range(0, 600):
        assert compute_topk_len(n) == O.compute_topk_len(n)
    assert compute_topk_len(30, 6, 10) == 9 and compute_topk_len(10, 6, 10) == 6 and compute_topk_len(4, 6, 10) == 4


def test_request_bookkeeping(ucm):
    from ucm_amd.sparse.gsa.gsa import GSAReqStat, TopKAndKpreManger

    mgr = TopKAndKpreManger(2)
    assert mgr.alloc("a") == 0 and mgr.alloc("b") == 1 and mgr.alloc("c") is None
    assert mgr.free("a") and not mgr.free("a") and mgr.alloc("c") == 0 and mgr.is_exist("c")

    st = GSAReqStat("r", slot_offset=1000, block_size=16, threshold=40)
    req = ns(block_ids=[[5, 9, 2]], num_computed_tokens=0, prompt_token_ids=[0] * 60, output_token_ids=[])
    st.update(40, req, 0)                       # first prefill chunk: 40 of 60 tokens -> blocks 0 and 1 are full
    assert st.calc_block_table == [5, 9] and st.calc_repre_slot_mapping == [1000, 1001]
    assert not st.is_decode() and not st.is_gsa() and not st.is_last_chunk()
    req.num_computed_tokens, req.block_ids = 40, [[5, 9, 2, 7]]
    st.update(20, req, 0)                       # last chunk: 60 tokens -> block 2 full, block 3 partial
    assert st.is_last_chunk() and st.calc_block_table == [2] and st.calc_repre_slot_mapping == [1002]
    req.num_computed_tokens, req.output_token_ids = 60, [1]
    st.update(1, req, 3)                        # decode, 61 tokens
    assert st.is_decode() and st.is_gsa() and st.calc_block_table == [] and st.index_in_batch == 3
    assert st.repre_slot_mapping == [1000, 1001, 1002, 1003]
    req.num_computed_tokens = 63
    st.update(1, req, 0)                        # token 64 fills block 3
    assert st.calc_block_table == [7] and st.calc_repre_slot_mapping == [1003] and st.get_seq_len() == 64
    req.num_computed_tokens, req.block_ids = 64, [[5, 9, 2, 7, 11]]
    st.update(1, req, 0)
    assert st.calc_block_table == []            # the new block has one token; nothing to reduce yet
    short = GSAReqStat("s", 0, 16, threshold=40)
    short.update(30, ns(block_ids=[[1, 2]], num_computed_tokens=0, prompt_token_ids=[0] * 30, output_token_ids=[]), 0)
    assert not short.is_gsa()


def test_gsa_plugin_metadata_without_a_gpu(ucm):
    """build_sparse_meta is pure host work: slots, block-mean lists and query offsets for a mixed batch."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA

    plugin = GSA(make_config(cfg={"seg_prefill_threshold": 200}), UcmSparseRole.WORKER)
    assert plugin.max_block_len == 32 and plugin.max_bs == 8 and plugin.layer_num == 4
    reqs = {
        "x": ns(block_ids=[[3, 4, 5]], num_computed_tokens=0, prompt_token_ids=[0] * 300, output_token_ids=[]),
        "y": ns(block_ids=[[8]], num_computed_tokens=0, prompt_token_ids=[0] * 100, output_token_ids=[]),
    }
    so = ns(num_scheduled_tokens={"x": 300, "y": 100}, scheduled_new_reqs=[ns(req_id="x"), ns(req_id="y")])
    plugin.build_sparse_meta(so, reqs, ns(req_id_to_index={"x": 1, "y": 0}), None)
    mi = plugin.model_input
    assert mi["query_locals"] == [0, 100, 400]
    assert mi["calc_block_table"] == [3, 4] and mi["calc_repre_slot_mapping"] == [0, 1]  # x owns partition 0
    assert plugin.gsa_stats["y"].slot_offset == 32 and mi["batch"][0].req_id == "y"
    plugin.execute_begin(so)
    assert mi["any_gsa"] is False and mi["is_topk"] is False
    plugin.execute_finished()
    plugin.request_finished_in_worker("x")
    assert "x" not in plugin.gsa_stats and plugin.topk_kpre_manger.free_cache[-1] == 0
    # the options that choose when a selection is made and applied
    assert plugin.retrieval_lag == 0 and GSA(make_config(cfg={"retrieval_lag": 1}), UcmSparseRole.WORKER).retrieval_lag == 1
    with pytest.raises(ValueError, match="retrieval_lag"):
        GSA(make_config(cfg={"retrieval_lag": 2}), UcmSparseRole.WORKER)


def test_esa_scheduler_side_and_helpers(ucm):
    """ESA's slot estimate, block keeping and hash chain are host arithmetic (esa.py:124-150, :537-587)."""
    import hashlib
    import pickle

    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseRole
    from ucm_amd.sparse.esa.esa import ESA, ReprePool, block_hash_func, get_offset
    from ucm_amd.sparse.factory import UcmSparseFactory

    cfg = make_config("ESA", {"init_window_sz": 1, "local_window_sz": 2, "min_blocks": 4, "sparse_ratio": 0.3,
                              "retrieval_stride": 5})
    esa = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.SCHEDULER)
    assert isinstance(esa, ESA) and esa.num_slots == 4096 * 8 // 128

    def request(n_prompt, n_out):
        return ns(request_id="r", prompt_token_ids=[0] * n_prompt, num_prompt_tokens=n_prompt, num_output_tokens=n_out)

    assert esa.estimate_num_slots_sparsed(request(2000, 0)) == INVALID_SLOT      # still prefilling
    assert esa.estimate_num_slots_sparsed(request(300, 3)) == INVALID_SLOT       # shorter than min_blocks blocks
    # 2048 tokens = 16 full blocks: sparse_range 14, keep int(14*0.3)=4 blocks + 2 local blocks + outputs
    assert esa.estimate_num_slots_sparsed(request(2048, 3)) == 4 * 128 + 2 * 128 + 3
    # 2000 tokens: 15 full blocks + 80: sparse_range 14, local = 80 + 128 + outputs
    assert esa.estimate_num_slots_sparsed(request(2000, 7)) == 4 * 128 + 80 + 128 + 7

    freed, evicted = [], []
    blocks = list(range(100, 116))
    mgr = ns(req_to_blocks={"r": blocks})
    coordinator = ns(get_blocks=lambda rid: [blocks], single_type_managers=[mgr],
                     get_num_blocks_to_allocate=lambda request_id, num_tokens, new_computed_blocks: 1,
                     allocate_new_blocks=lambda rid, n: None)
    pool = ns(_maybe_evict_cached_block=evicted.append, free_blocks=freed.extend, get_num_free_blocks=lambda: 5)
    out = esa.allocate_slots(request(2048, 3), 4 * 128 + 2 * 128 + 3, coordinator, pool, [None])
    assert mgr.req_to_blocks["r"] == blocks[-7:] and freed == blocks[:-7] and evicted == blocks
    assert out.blocks == (blocks[-7:],)
    pool.get_num_free_blocks = lambda: 0
    assert esa.allocate_slots(request(2048, 3), 771, coordinator, pool, [None]) is None

    seed = int.from_bytes(hashlib.md5(pickle.dumps("UCMHASHSEED", protocol=pickle.HIGHEST_PROTOCOL)).digest(), "big")
    h1 = block_hash_func(None, (1, 2, 3))
    assert h1 == int.from_bytes(hashlib.md5(pickle.dumps((seed, (1, 2, 3)), protocol=pickle.HIGHEST_PROTOCOL)).digest(), "big")
    assert block_hash_func(h1, [4, 5]) == block_hash_func(h1, (4, 5)) != h1
    for args in [((128, 8, 128), 0, 1, 2, 0, False), ((128, 8, 128), 1, 2, 2, 3, True), ((128, 8, 128), 0, 1, 2, 5, True)]:
        assert get_offset(*args) == O.get_offset(*args)

    pool2 = ReprePool(5)
    a = pool2.allocate(3)
    assert a == [0, 1, 2] and pool2.allocated == {0, 1, 2}
    pool2.free([1])
    assert pool2.allocate(3) == [1, 3, 4]
    with pytest.raises(AssertionError):
        pool2.allocate(1)


def test_kvstar_req_meta_query_offload_info(ucm):
    """Which places of the retrieval group a prefill chunk fills (multistep.py:103-130): only the prompt's last
    `retrieval_stride` tokens are kept, whatever the chunking."""
    from ucm_amd.sparse.kvstar.multistep import ReqMeta, ReqStage

    def meta(computed, scheduled, prompt=100, out=0, stride=8):
        return ReqMeta("r", 0, prompt, out, scheduled, computed, 0, [], 16, [0] * prompt, 0, scheduled, stride)

    assert meta(0, 50).query_offload_info is None                     # ends before token 92
    assert meta(0, 100).query_offload_info == list(range(8))          # one chunk: all eight places
    assert meta(50, 45).query_offload_info == [0, 1, 2]               # tokens 92..94
    assert meta(95, 5).query_offload_info == [3, 4, 5, 6, 7]
    assert meta(0, 93).query_offload_info == [0]
    assert meta(97, 3, prompt=100).query_offload_info == [5, 6, 7]
    m = meta(100, 1, out=13)
    assert m.stage == ReqStage.DECODE and m.query_offload_info == [13 % 8] and m.step == 13
    assert meta(0, 99).is_last_chunk is False and meta(60, 40).is_last_chunk is True
    hashes = ReqMeta("r", 0, 40, 0, 40, 0, 0, [], 16, list(range(40))).req_block_hashes
    assert len(hashes) == 2 and len(set(hashes)) == 2                 # full blocks only, chained


def test_kvstar_scheduler_side(ucm):
    """estimate_num_slots_sparsed / allocate_slots are host arithmetic (multistep.py:775-846)."""
    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseRole
    from ucm_amd.sparse.kvstar.multistep import KVStarMultiStep

    ns = types.SimpleNamespace
    cfg = make_config("KVStarMultiStep", {"sparse_ratio": 0.25})
    cfg.cache_config.block_size = 16
    cfg.parallel_config = ns(rank=0, tensor_parallel_size=1)
    cfg.model_config.hf_config = ns(num_hidden_layers=2)
    plugin = KVStarMultiStep(cfg, UcmSparseRole.SCHEDULER)
    assert plugin.estimate_num_slots_sparsed(ns(num_output_tokens=0)) == INVALID_SLOT
    for n_prompt, n_out in [(16 * 40 + 3, 1), (16 * 40, 7), (16 * 2 + 1, 5), (16 * 41, 16)]:
        req = ns(num_output_tokens=n_out, num_prompt_tokens=n_prompt, num_tokens=n_prompt + n_out)
        full = n_prompt // 16
        fixed = min(3, full)
        saved = math.ceil((full - fixed) * 0.25)
        blocks = math.ceil((n_prompt + n_out) / 16) - (full - saved - fixed)
        tail = (n_prompt + n_out) % 16
        assert plugin.estimate_num_slots_sparsed(req) == ((blocks - 1) * 16 + tail if tail else blocks * 16)

    class Pool:
        def __init__(self):
            self.freed, self.evicted = [], []

        def _maybe_evict_cached_block(self, b):
            self.evicted.append(b)

        def free_blocks(self, bl):
            self.freed.extend(bl)

        def get_num_free_blocks(self):
            return 1

    held = list(range(100, 110))
    mgr = ns(req_to_blocks={})
    calls = []
    coord = ns(get_blocks=lambda rid: [held], single_type_managers=[mgr],
               get_num_blocks_to_allocate=lambda request_id, num_tokens, new_computed_blocks: calls.append(num_tokens) or 1,
               allocate_new_blocks=lambda rid, n: calls.append(("alloc", n)))
    pool = Pool()
    got = plugin.allocate_slots(ns(request_id="A"), 16 * 3 + 2, coord, pool, [None])
    assert mgr.req_to_blocks["A"] == held[-4:] and pool.freed == held[:-4] and pool.evicted == held
    assert got.blocks == (held[-4:],) and calls == [50, ("alloc", 50)]
    coord.get_num_blocks_to_allocate = lambda request_id, num_tokens, new_computed_blocks: 2
    assert plugin.allocate_slots(ns(request_id="A"), 50, coord, Pool(), [None]) is None


def test_gsa_prefetch_mode_resident_set_and_slots(ucm):
    """The resident set of a sparsified request (gsa.py:156-186) and the slots it is given (gsa.py:891-912), checked
    against values worked out by hand from the reference's constants (min 32, max 48, ratio 0.3, local = 31)."""
    from ucm_amd.sparse.base import INVALID_SLOT, UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA, GSAReqStat

    st = GSAReqStat("a", 0, 128, 8400)
    st.blocks = list(range(100))                      # 100 blocks -> k = int(30.0) = 30 < 32 -> min(32, 100) = 32
    st.num_prompt_tokens = st.num_computed_tokens = 100 * 128
    st.get_sparse_and_free_block(True, 32, 48, 0.3)
    # blocks 0..48 stand for the sparse cache; in use: the first 32 - 31 = 1 and the last 31; free in between
    assert st.remain_idx == [0] + list(range(18, 49)) and st.prefetch_idx == list(range(1, 18))
    assert st.sparse_len == 32 + 17 and len(st.remain_idx) == 32
    st.blocks = list(range(200))                      # k = int(60.0) -> capped at 48
    st.num_prompt_tokens = st.num_computed_tokens = 200 * 128
    st.get_sparse_and_free_block(True, 32, 48, 0.3)
    assert st.remain_idx == list(range(17)) + list(range(18, 49)) and st.prefetch_idx == [17] and st.sparse_len == 49
    st.get_sparse_and_free_block(False, 32, 48, 0.3)  # prefetch mode off: everything stays
    assert st.remain_idx == list(range(200)) and st.prefetch_idx == [] and st.sparse_len == 200
    st.num_computed_tokens += 1                       # past the first decode step: no longer decided here
    st.get_sparse_and_free_block(True, 32, 48, 0.3)
    assert st.remain_idx is None and st.prefetch_idx is None

    plugin = GSA(make_config(cfg={"ptopk_prefetch_enable": True}), UcmSparseRole.SCHEDULER)
    req = ns(num_prompt_tokens=100 * 128, num_output_tokens=5, num_tokens=100 * 128 + 5)
    # 101 blocks in all, 100 of the prompt: 1 + 32 + 17 = 50 blocks, the last one holding 5 tokens
    assert plugin.estimate_num_slots_sparsed(req) == 50 * 128 - (128 - 5)
    req = ns(num_prompt_tokens=200 * 128 + 7, num_output_tokens=121, num_tokens=201 * 128)
    assert plugin.estimate_num_slots_sparsed(req) == (201 - 201 + 48 + 1) * 128
    assert plugin.estimate_num_slots_sparsed(ns(num_prompt_tokens=8400, num_output_tokens=5, num_tokens=8405)) == INVALID_SLOT
    assert plugin.estimate_num_slots_sparsed(ns(num_prompt_tokens=9000, num_output_tokens=0, num_tokens=9000)) == INVALID_SLOT
    off = GSA(make_config(), UcmSparseRole.SCHEDULER)
    assert off.estimate_num_slots_sparsed(ns(num_prompt_tokens=100 * 128, num_output_tokens=5, num_tokens=100 * 128 + 5)) == INVALID_SLOT

    # the scheduler's half (not in the reference): at the first decode step the request keeps its first max_topk + 1
    # blocks and what it holds beyond its prompt, later steps only allocate
    class Pool:
        def __init__(self):
            self.freed, self.evicted = [], []

        def _maybe_evict_cached_block(self, b):
            self.evicted.append(b)

        def free_blocks(self, bl):
            self.freed.extend(bl)

        def get_num_free_blocks(self):
            return 1

    held = list(range(500, 602))                      # 101 blocks of the prompt (100 full + 5 tokens... ) and one more
    mgr = ns(req_to_blocks={})
    calls = []
    coord = ns(get_blocks=lambda rid: [held], single_type_managers=[mgr],
               get_num_blocks_to_allocate=lambda request_id, num_tokens, new_computed_blocks: calls.append(num_tokens) or 1,
               allocate_new_blocks=lambda rid, n: calls.append(("alloc", n)))
    pool = Pool()
    req = ns(request_id="A", num_prompt_tokens=100 * 128 + 5, num_computed_tokens=100 * 128 + 5, num_output_tokens=1,
             num_tokens=100 * 128 + 6)
    got = plugin.allocate_slots(req, 4000, coord, pool, [None])
    assert mgr.req_to_blocks["A"] == held[:49] + held[101:] and pool.freed == held[49:101] and pool.evicted == held
    assert got.blocks == (held[:49] + held[101:],) and calls == [4000, ("alloc", 4000)]
    req.num_computed_tokens += 1                      # a later step: nothing is returned any more
    pool2, mgr.req_to_blocks = Pool(), {}
    got = plugin.allocate_slots(req, 4001, coord, pool2, [None])
    assert pool2.freed == [] and mgr.req_to_blocks == {} and got.blocks == (held,)
    coord.get_num_blocks_to_allocate = lambda request_id, num_tokens, new_computed_blocks: 2
    assert plugin.allocate_slots(req, 4001, coord, Pool(), [None]) is None


def test_kvcomp_reads_the_reference_config_file(ucm, tmp_path):
    """KvComp takes head_dim and hash_bits from the reference's JSON (kvcomp_config.py:36-80; the files under
    kvcomp/configs have these keys) and refuses one written for a model with another number of layers
    (kvcomp.py:452-464)."""
    import json

    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.kvcomp.kvcomp import KvComp

    js = {"model_name": "Qwen/Qwen3-4B", "is_mla": False, "hash_weight_type": "random", "num_hidden_layers": 36,
          "seq_len_threshhold": 2048, "chunk_size": 128, "chunk_repre_method": "max", "head_dim": 128,
          "hash_bits": 128, "top_k_ratio_per_layer": [1, 1] + [0.3] * 34, "top_k_index_reuse": [-1] * 36,
          "must_select_blocks": [0, -2, -1], "hash_weight": None}
    path = tmp_path / "kvcomp.json"
    path.write_text(json.dumps(js))
    cfg = make_config("KvComp", {})
    cfg.parallel_config = ns(rank=0, tensor_parallel_size=1)
    cfg.kv_transfer_config.kv_connector_extra_config["kvcomp_config_path"] = str(path)
    cfg.model_config.hf_text_config = ns(num_hidden_layers=36)
    plugin = KvComp(cfg, UcmSparseRole.SCHEDULER)
    assert plugin.cfg["head_dim"] == 128 and plugin.cfg["hash_bits"] == 128
    cfg.model_config.hf_text_config = ns(num_hidden_layers=32)
    with pytest.raises(AssertionError, match="num_hidden_layers 36"):
        KvComp(cfg, UcmSparseRole.SCHEDULER)
