"""Host-inclusive timing of the four sparse-attention plugins, driven the way patched vLLM drives their hooks.

bench.py's `value` is what a C caller of libucm_hip.so sees.  A vLLM user sees the plugin: per engine step
`build_sparse_meta` (+ `execute_begin`), then per layer `attention_begin` and `attention_finished`, all on the
model-runner thread.  Each leg here runs those hooks with stand-in objects for the scheduler output, the request
states, the input batch and the forward context (vLLM itself is not imported) on the ragged batch of the benchmark's
second configuration - 16 requests of 32..512 blocks of 128 tokens, 32 layers, Llama-3-8B head shape - and reports
per kind of step

* host_us: time the hooks take on the host, launches included, nothing waited for (the model-runner thread's cost),
* wall_us: from the first hook to the device having finished what the hooks queued (there is no model in between,
  so this is the hooks' host time plus whatever device work outlasts it).

The cache blocks the ESA, KvComp and KVStar legs load into are overwritten: the legs run after bench.py's checks.
"""
from __future__ import annotations

import math
import time
import types

import numpy as np

ns = types.SimpleNamespace
HQ, HKV, D, BS = 32, 8, 128, 128


class ModelConfig:
    def __init__(self, layers: int, max_model_len: int):
        self.layers, self.max_model_len = layers, max_model_len

    def get_num_kv_heads(self, pc):
        return HKV

    def get_num_attention_heads(self, pc):
        return HQ

    def get_head_size(self):
        return D

    def get_num_layers(self, pc):
        return self.layers


def make_config(layers: int, max_model_len: int, max_num_seqs: int, name: str, plugin_cfg: dict):
    return ns(model_config=ModelConfig(layers, max_model_len), parallel_config=ns(rank=0, tensor_parallel_size=1),
              cache_config=ns(block_size=BS), scheduler_config=ns(max_num_seqs=max_num_seqs),
              kv_transfer_config=ns(kv_connector_extra_config={"ucm_sparse_config": {name: plugin_cfg}}))


def layer_names(n_layers: int):
    return [f"model.layers.{l}.self_attn.attn" for l in range(n_layers)]


class Harness:
    """The engine side of a leg: requests with their block lists and token counts, and `step`, which runs one
    engine step's hooks and times them."""

    def __init__(self, torch, dev, plugin, caches, prompt_tokens, block_ids, seed: int, with_execute_hooks: bool = False):
        self.torch, self.dev, self.plugin, self.caches = torch, dev, plugin, caches
        self.n_layers = len(caches)
        self.names = layer_names(self.n_layers)
        self.fc = ns(no_compile_layers={n: ns(kv_cache=[c]) for n, c in zip(self.names, caches)}, virtual_engine=0,
                     attn_metadata=None)
        self.with_execute_hooks = with_execute_hooks
        rng = np.random.default_rng(seed)
        self.reqs = {}
        for r, (n_tok, ids) in enumerate(zip(prompt_tokens, block_ids)):
            rid = f"r{r}"
            self.reqs[rid] = ns(request_id=rid, req_id=rid, block_ids=[list(ids)], full_ids=list(ids), num_computed_tokens=0,
                                prompt_token_ids=[int(t) for t in rng.integers(0, 32000, n_tok)], output_token_ids=[],
                                num_prompt_tokens=n_tok, num_output_tokens=0, num_tokens=n_tok)
        self.order = list(self.reqs)
        self.g = torch.Generator(device=dev)
        self.g.manual_seed(seed)
        self.times = {}
        self.rho = 0.0                 # correlation of a layer's decode queries from one step to the next (0: independent draws)
        self._last_q = None

    def decode_token(self) -> None:
        """Every request has produced one more token (what the engine does between two decode steps)."""
        for r in self.reqs.values():
            r.output_token_ids.append(7)
            r.num_output_tokens += 1
            r.num_tokens += 1

    def step(self, kind: str, n_tokens: dict, query_rows=None, one_query: bool = False) -> None:
        """One engine step: n_tokens[request id] tokens scheduled; the query tensor holds one row per scheduled
        token (or query_rows rows when the hooks of this step never look at the prompt's queries); one_query: every
        layer is handed the same tensor (a prompt's queries are gigabytes per layer)."""
        torch, plugin = self.torch, self.plugin
        live = [rid for rid in self.order if rid in n_tokens]
        starts = [0]
        for rid in live:
            starts.append(starts[-1] + n_tokens[rid])
        rows = starts[-1] if query_rows is None else query_rows
        draw = lambda: torch.empty((rows, HQ, D), dtype=torch.bfloat16, device=self.dev).normal_(0.0, 0.3, generator=self.g)
        qs = [draw()] * self.n_layers if one_query else [draw() for _ in range(self.n_layers)]
        if self.rho > 0.0 and not one_query:
            # decode queries that drift: q_t = rho q_(t-1) + sqrt(1 - rho^2) noise, layer by layer (the same batch as before)
            if self._last_q is not None and self._last_q[0].shape == qs[0].shape:
                qs = [(self.rho * a.float() + math.sqrt(1.0 - self.rho ** 2) * b.float()).to(torch.bfloat16)
                      for a, b in zip(self._last_q, qs)]
            self._last_q = qs
        self.last_queries = qs         # what this step's hooks are handed, layer by layer (tests look at them)
        so = ns(num_scheduled_tokens=dict((rid, n_tokens[rid]) for rid in live), req_sparsed_slots={rid: 0 for rid in live},
                scheduled_new_reqs=[ns(req_id=rid) for rid in live if self.reqs[rid].num_computed_tokens == 0],
                scheduled_cached_reqs=ns(req_ids=[rid for rid in live if self.reqs[rid].num_computed_tokens > 0]))
        ib = ns(req_id_to_index={rid: i for i, rid in enumerate(live)})
        md = ns(query_start_loc=torch.tensor(starts), block_table=None, seq_lens=None)
        self.fc.attn_metadata = md
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        plugin.build_sparse_meta(so, self.reqs, ib, md)
        if self.with_execute_hooks:
            plugin.execute_begin(so)
        for l, name in enumerate(self.names):
            plugin.attention_begin(qs[l], None, None, name, self.fc)
            plugin.attention_finished(qs[l], None, None, None, name, self.fc)
        if self.with_execute_hooks:
            plugin.execute_finished()
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        self.times.setdefault(kind, []).append(((t1 - t0) * 1e6, (t2 - t0) * 1e6))
        for rid in live:
            self.reqs[rid].num_computed_tokens += n_tokens[rid]

    def report(self) -> dict:
        out = {}
        for kind, rows in self.times.items():
            host, wall = np.array(rows).T
            out[kind] = {"steps": len(rows), "host_us": round(float(np.median(host)), 1), "wall_us": round(float(np.median(wall)), 1)}
        return out


def _prompt_shape(lens):
    """Prompt lengths that leave room in every request's last block for the decode steps of a leg: all but the last
    block full, 40 tokens in the last."""
    return [int(n - 1) * BS + 40 for n in lens]


def gsa_leg(torch, dev, caches, lens, block_tables, steps: int, seed: int, lag: int = 0) -> dict:
    """GSA: every decode step scores all blocks of every request and swaps each layer's block table and sequence
    lengths for the sparse ones - one library call per layer with the layer's own queries (lag 0), or the layer's
    hook only keeps the queries and the next step scores every layer in one launch before its model runs (lag 1)."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.gsa.gsa import GSA

    n_layers = len(caches)
    cfg = make_config(n_layers, 65536, len(lens), "GSA", {"seg_prefill_threshold": 0, "repre_dtype": "bfloat16", "retrieval_lag": lag})
    plugin = GSA(cfg, UcmSparseRole.WORKER)

    def wave(w: int) -> dict:
        h = Harness(torch, dev, plugin, caches, _prompt_shape(lens), block_tables, seed, with_execute_hooks=True)
        h.step("prefill (representatives of every full block, 32 layers)", {rid: r.num_prompt_tokens for rid, r in h.reqs.items()},
               query_rows=16)
        for i in range(3 + steps):
            h.decode_token()
            h.step("warm" if i < 3 else "decode", {rid: 1 for rid in h.reqs})
        h.times.pop("warm")
        out = h.report()
        out["selected_blocks_layer0"] = [int(x) for x in plugin.topk_counts[0, : len(lens)].tolist()]
        for rid in list(h.reqs):
            plugin.request_finished_in_worker(rid)
        return out

    return _second_wave(wave)


def _second_wave(wave) -> dict:
    """A leg serves two waves of requests with one plugin object and reports the second: what a plugin costs in a
    server that has served before (the first wave pays for the first use of every torch operator and kernel, for
    the store's pool and for the plugin's own tables; its figures say nothing about the steps that follow)."""
    import gc

    wave(0)
    gc.collect()
    return wave(1)


def _store(torch, n_layers: int, blocks: int):
    """A device-resident block store with room for the prompts' blocks (both waves bring the same prompts, so the second
    finds its hashes there and writes the same slots again), its pool allocated up front."""
    from ucm_amd.store.hip_block_store import UcmHipBlockStore

    slice_bytes = BS * HKV * D * 2
    store = UcmHipBlockStore({"kv_block_size": n_layers * 2 * slice_bytes, "max_cache_size": blocks * n_layers * 2 * slice_bytes})
    store.device_pool()
    return store


def _dump_prompt_blocks(torch, dev, ops, store, caches, hashes, ids) -> None:
    """What the prefix-cache connector does after a prefill: the prompt's full blocks go to the store under their
    hashes, every layer, K and V (one gather launch into the store's pool)."""
    n = len(hashes)
    assert store.create(hashes) == [0] * n
    slots = [store.slot_of[h] for h in hashes]
    assert slots == list(range(slots[0], slots[0] + n))
    pool, block_bytes = store.device_pool()
    layers = ops.LayerPointers(caches)
    kv = caches[0]
    ops.kv_gather_blocks(layers, kv.stride(0) * kv.element_size(), kv.stride(1) * kv.element_size(), kv.shape[1],
                         torch.tensor(ids[:n], dtype=torch.int32, device=dev), pool[slots[0] * block_bytes :])
    store.commit(hashes)


def esa_leg(torch, dev, caches, lens, block_tables, seed: int) -> dict:
    """ESA, device path: retrieval at step % 5 == 2, delta loads at step % 5 == 0, both before the first decode
    step's attention."""
    from ucm_amd import ops
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.esa.esa import ESA

    n_layers = len(caches)
    store = _store(torch, n_layers, int(sum(lens)))
    cfg = make_config(n_layers, 65536, len(lens), "ESA", {"init_window_sz": 1, "local_window_sz": 2, "min_blocks": 4,
                                                        "sparse_ratio": 0.3, "retrieval_stride": 5})
    plugin = ESA(cfg, UcmSparseRole.WORKER, store=store)
    kinds = {1: "first decode step (retrieve + plan + load per layer)", 2: "retrieve", 0: "plan + load"}   # by step % 5

    def wave(w: int) -> dict:
        h = Harness(torch, dev, plugin, caches, _prompt_shape(lens), block_tables, seed)
        h.step("prefill (representatives)", {rid: r.num_prompt_tokens for rid, r in h.reqs.items()}, query_rows=16)
        for rid, r in h.reqs.items():
            _dump_prompt_blocks(torch, dev, ops, store, caches, plugin._dev.reqs[rid].block_hashes, r.full_ids)
        for step in range(1, 13):
            h.decode_token()
            h.step(kinds[1] if step == 1 else {2: kinds[2], 0: kinds[0]}.get(step % 5, "idle"), {rid: 1 for rid in h.reqs})
        out = h.report()
        for rid in list(h.reqs):
            plugin.request_finished_in_worker(rid)
        return out

    return _second_wave(wave)


def kvcomp_leg(torch, dev, caches, lens, block_tables, seed: int, delta: bool = False, rho: float = 0.0) -> dict:
    """KvComp, device path: hash codes of every prompt block at the end of the prefill (and the blocks into the
    store), the scheduler shrinks the block lists, then a retrieval every fourth decode step.  ``delta``: the
    retrieval's load moves only the picks the middle cache blocks do not hold yet (how many depends on how far the
    queries drift between retrievals: ``rho`` per step)."""
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.factory import UcmSparseFactory

    n_layers = len(caches)
    torch.manual_seed(seed)                                            # the plugin draws its hash weights from the global generator
    cfg = make_config(n_layers, 65536, len(lens) + 1, "KvComp", {"device_loads": True, "delta_loads": delta})
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    plugin.connector = _store(torch, n_layers, int(sum(lens)))

    def wave(w: int) -> dict:
        h = Harness(torch, dev, plugin, caches, _prompt_shape(lens), block_tables, seed)
        h.rho = rho
        h.step("prefill end (hash codes + blocks to the store, 32 layers)", {rid: r.num_prompt_tokens for rid, r in h.reqs.items()},
               query_rows=16)
        for step in range(1, 10):
            h.decode_token()
            if step == 1:
                for r in h.reqs.values():                              # the scheduler shrinks the block list (kvcomp.py:571-587)
                    slots = plugin.estimate_num_slots_sparsed(r)
                    r.block_ids = [r.full_ids[: -(-r.num_tokens // BS)][-(-(-slots // BS)):]]
            h.step("first decode step (windows back, retrieval, loads)" if step == 1 else "decode", {rid: 1 for rid in h.reqs})
        out = h.report()
        # the decode steps are of two kinds: those in which requests retrieve (every retrieval_stride-th) and the rest
        dec = np.array(h.times["decode"])
        cut = float(np.median(dec[:, 0])) * 2
        busy, plain = dec[dec[:, 0] > cut], dec[dec[:, 0] <= cut]
        out.pop("decode")
        if len(busy):
            out["retrieve step"] = {"steps": len(busy), "host_us": round(float(np.median(busy[:, 0])), 1),
                                    "wall_us": round(float(np.median(busy[:, 1])), 1)}
        out["plain step"] = {"steps": len(plain), "host_us": round(float(np.median(plain[:, 0])), 1),
                             "wall_us": round(float(np.median(plain[:, 1])), 1)}
        if delta and plugin._dev is not None and plugin._dev.miss_step is not None:
            picks = int(plugin._dev.cnt[:, : len(lens)].sum())
            out["blocks_moved_by_the_last_retrieval"] = {"moved": int(plugin._dev.miss_step.sum()), "picked": picks}
        for rid in list(h.reqs):
            plugin.request_finished_in_worker(rid)
        return out

    return _second_wave(wave)


def kvstar_leg(torch, dev, caches, lens, block_tables, seed: int) -> dict:
    """KVStar: sub-block representatives and channel choice at the end of the prefill, then strides of eight decode
    steps - seven that only park the step's query token, one that queues the stride's votes (and, from the second
    stride on, loads the winners of the stride before)."""
    from ucm_amd import ops
    from ucm_amd.sparse.base import UcmSparseRole
    from ucm_amd.sparse.factory import UcmSparseFactory

    n_layers = len(caches)
    stride = 8
    cfg = make_config(n_layers, 65536, len(lens), "KVStarMultiStep",
                      {"retrieval_stride": stride, "sparse_ratio": 0.25, "blk_repre_dim_prune_ratio": 0.25,
                       "blk_repre_inner_token_merge": 2})
    store = _store(torch, n_layers, int(sum(lens)))
    plugin = UcmSparseFactory.create_sparse_method(cfg, UcmSparseRole.WORKER)
    plugin.connector = store

    def wave(w: int) -> dict:
        h = Harness(torch, dev, plugin, caches, _prompt_shape(lens), block_tables, seed)
        h.step("prefill end (representatives + channel choice, 32 layers)", {rid: r.num_prompt_tokens for rid, r in h.reqs.items()},
               one_query=True)
        for rid, r in h.reqs.items():
            _dump_prompt_blocks(torch, dev, ops, store, caches, plugin.req_states[rid][0].block_hashes, r.full_ids)
        n_steps = 3 * stride + 1
        for step in range(1, n_steps + 1):
            h.decode_token()
            if step == 1:
                for r in h.reqs.values():                                  # the scheduler shrinks every request (multistep.py:816-846)
                    r.block_ids = [r.full_ids[-math.ceil(plugin.estimate_num_slots_sparsed(r) / BS):]]
            kind = ("first decode step (windows back, prefill group's votes and their load)" if step == 1 else
                    "queue + load" if step % stride == 0 and step >= 2 * stride else "queue" if step % stride == 0 else "plain")
            h.step(kind, {rid: 1 for rid in h.reqs})
        out = h.report()
        # one stride in steady state: seven plain steps and one that queues and loads
        if "queue + load" in out and "plain" in out:
            out["average_over_a_stride"] = {
                "host_us": round(((stride - 1) * out["plain"]["host_us"] + out["queue + load"]["host_us"]) / stride, 1),
                "wall_us": round(((stride - 1) * out["plain"]["wall_us"] + out["queue + load"]["wall_us"]) / stride, 1)}
        for rid in list(h.reqs):
            plugin.request_finished_in_worker(rid)
        return out

    return _second_wave(wave)
