"""Decode-step benchmark of the sparse-retrieval hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (configs[1] of the benchmark definition): a ragged continuous batch of 16 requests,
context lengths uniform in [4096, 65536] tokens rounded to the 128-token block,
Llama-3-8B attention shape (32 query heads / 8 kv heads / head_dim 128, bf16),
all 32 layers.  One step = for every layer and request: score all block
representatives against the request's query, select top-k = max(16, 3 % of the
blocks) plus the first block and the last two, and gather the selected K and V
blocks from the bf16 paged cache into a contiguous per-request buffer.
Two launches per step (scores with each request's selection run by its last scoring
workgroup, then the gather), no host round trip between; --two-launch scores and
selects in launches of their own.

Prints ONE JSON line.  `value` is microseconds per decode step with all inputs
resident in HBM; `roofline` describes the dominant kernel (the gather),
`roofline_score` the scoring kernel, `cpu_baseline` the same step on the host
(the reference's CPU retrieval algorithm + a memcpy gather).
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time
import zlib

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def measured_traffic(role: str, kernel: str, workload: dict):
    """HBM bytes per launch that rocprofv3 --pmc measured for `kernel` (profiles/traffic.json), or None when the
    file has no entry for this role whose workload (layers, seed, blocks ...) is exactly this run's.  The file
    names the kernel each figure belongs to: a figure is never quoted for a kernel other than the one this run
    launched."""
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        entry = json.load(f)["entries"].get(role)
    if entry is None or entry.get("workload") != workload:
        return None
    if entry["kernel"] != kernel:
        raise SystemExit(f"profiles/traffic.json holds the traffic of {entry['kernel']} for '{role}', but this run launched "
                         f"{kernel}: re-measure before quoting it")
    return int(entry["hbm_bytes_per_launch"])

N_REQ, N_LAYERS, HQ, HKV, D, BS = 16, 32, 32, 8, 128, 128
ROW = HKV * D
BLOCK_BYTES = BS * ROW * 2


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--seed", type=int, default=2024)
    ap.add_argument("--layers", type=int, default=N_LAYERS, help="fewer layers only for quick experiments")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-check", action="store_true", help="skip the oracle check of the last step")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--delta-rho", type=float, nargs="+", default=[0.95, 0.0, 0.9, 0.99],
                    help="correlation(s) of consecutive decode queries in the delta-gather leg (0 = independent); the "
                         "first one is the `delta_gather` object of the line, all of them its `by_correlation` list")
    ap.add_argument("--no-delta", action="store_true", help="skip the delta-gather leg")
    ap.add_argument("--two-launch", action="store_true",
                    help="score and select as two launches (ucm_score_blocks, ucm_topk_windows) instead of the one-launch "
                         "ucm_score_select")
    ap.add_argument("--repre-dtype", choices=["bf16", "f32"], default="bf16",
                    help="element type of the representative table: bf16 = the rounded means the live reference "
                         "path stores, kept as they are; f32 = the same values widened (the CPU path's table)")
    ap.add_argument("--hash-leg", action="store_true",
                    help="also time the hash-code retrieval variant (the configs[4] shape of the benchmark definition) on the same caches")
    ap.add_argument("--hash-distinct", type=int, default=0,
                    help="hash leg: name only this many distinct cache blocks in the encode's block list, over and over "
                         "(8: the key loads are served from cache, which times the compute side of the kernel on its own); "
                         "0 = every block once")
    ap.add_argument("--no-legs", action="store_true",
                    help="only the decode step (and its delta-gather leg): none of the --*-leg measurements.  Without this "
                         "flag and without any --*-leg flag, every leg runs; naming legs runs exactly those.")
    ap.add_argument("--hash-heads-sweep", action="store_true",
                    help="hash leg: also time the summaries-only encode with the same cache bytes read as blocks of 4, 2 "
                         "and 1 kv heads (what a tensor-parallel rank holds)")
    ap.add_argument("--prefetch-leg", action="store_true",
                    help="also time the GSA prefetch engine's round at this batch: hits / misses / free list of every "
                         "(request, layer) on the device plus the loads of the served misses from a device-resident "
                         "pool of stored blocks (needs about as much memory again as the KV cache)")
    ap.add_argument("--moves-leg", action="store_true",
                    help="also time the block-id driven load/dump (the configs[2] shape of the benchmark definition: 64 requests "
                         "x 16 blocks, all layers, K and V, random block table) on the same caches")
    ap.add_argument("--esa-leg", action="store_true",
                    help="also time the ESA retrieval backend (slot-list scoring + top-k) at three shapes")
    ap.add_argument("--config1-leg", action="store_true",
                    help="also time configs[0] of the benchmark definition: one request of 32768 tokens (256 blocks), one layer")
    ap.add_argument("--config4-leg", action="store_true",
                    help="also time configs[3]: 8 requests of 512-1024 blocks, 64 query heads (groups of 8), 80 layers, bf16 "
                         "and fp32 representative tables, with the block mean of the one block per request that fills up")
    ap.add_argument("--plugin-leg", action="store_true",
                    help="also run the four plugins' hooks (GSA, ESA, KvComp, KVStar) on this batch with stand-in objects for "
                         "vLLM's and report the host time and the host-inclusive time of their steps (plugin_bench.py; "
                         "needs about as much memory again as the KV cache for the store the loads come from)")
    ap.add_argument("--kvstar-leg", action="store_true",
                    help="also time the multi-query softmax-vote retrieval (KVStar: 8 query tokens per request) on the same "
                         "ragged batch")
    ap.add_argument("--kvstar-layout", choices=["row", "head"], default="head",
                    help="memory order of the KVStar representative table: the kv heads of a block next to each other "
                         "(row) or a plane per kv head (head)")
    ap.add_argument("--kvstar-merge", type=int, default=2,
                    help="tokens averaged into one sub-block representative (reference default 2: 64 per 128-token block)")
    ap.add_argument("--kvstar-prune", type=float, default=0.25,
                    help="share of the head's channels kept in the representatives (reference default 0.25; 1 = all)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 1 GiB copy (copy_batch_kernel) so that rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE readings can be scaled against a kernel of known traffic")
    args = ap.parse_args()
    leg_flags = ("hash_leg", "prefetch_leg", "moves_leg", "esa_leg", "kvstar_leg", "config1_leg", "config4_leg", "plugin_leg")
    run_all = not args.no_legs and not any(getattr(args, f) for f in leg_flags)
    for f in leg_flags:
        setattr(args, f, run_all or (getattr(args, f) and not args.no_legs))
    return args


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: the retrieval path is per-GPU and this build has no multi-GPU leg "
              f"(--gpus {args.gpus} refused)", file=sys.stderr)
        sys.exit(2)

    import torch

    import __graft_entry__ as ge

    ge.load_package()
    from ucm_amd import ops

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    n_layers = args.layers
    rng = np.random.default_rng(args.seed)
    lens = rng.integers(4096 // BS, 65536 // BS + 1, N_REQ).astype(np.int32)       # blocks per request
    topk = np.array([max(16, int(0.03 * n)) + 3 for n in lens], np.int32)          # total incl. windows
    rows = int(lens.sum())
    nb = rows                                                                        # pool = exactly the live blocks
    seg_off_h = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
    table_h = rng.permutation(nb).astype(np.int32)                                  # random block table over the pool
    max_len, max_k = int(lens.max()), int(topk.max())

    # ---- device state: paged KV cache, block tables, representatives
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)

    def score_name(f32_table: bool) -> str:
        return "score_kernel" if f32_table else "score_kernel_bf16"

    def leg_rng(name: str):
        """Every leg draws from generators of its own (seeded by the run's seed and the leg's name), so that its
        workload does not depend on which other legs ran before it."""
        return np.random.default_rng([args.seed, zlib.crc32(name.encode())])

    def leg_gen(name: str):
        gen = torch.Generator(device=dev)
        gen.manual_seed((args.seed << 32) + zlib.crc32(name.encode()))
        return gen

    caches = []
    for _ in range(n_layers):
        c = torch.empty((2, nb, BS, HKV, D), dtype=torch.bfloat16, device=dev)
        c.normal_(generator=g)
        caches.append(c)
    layers = ops.LayerPointers(caches)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=dev)
    seg_off, seg_len, topk_d, table = i32(seg_off_h), i32(lens), i32(topk), i32(table_h)
    bt_h = np.zeros((N_REQ, max_len), np.int32)
    for r in range(N_REQ):
        bt_h[r, : lens[r]] = table_h[seg_off_h[r] : seg_off_h[r] + lens[r]]
    bt = i32(bt_h)
    repre = torch.zeros(n_layers, rows, ROW, device=dev,
                        dtype=torch.bfloat16 if args.repre_dtype == "bf16" else torch.float32)
    rep_es = repre.element_size()
    slots = torch.arange(rows, dtype=torch.int32, device=dev)

    def prefill():
        ops.block_mean(layers, table, slots, repre, BS, HKV, D, nb, mode=ops.MEAN_BF16_ROUND)

    prefill()
    torch.cuda.synchronize()
    ev = lambda: torch.cuda.Event(enable_timing=True)
    a, b = ev(), ev()
    a.record()
    prefill()
    b.record()
    torch.cuda.synchronize()
    mean_ms = a.elapsed_time(b)
    mean_bytes = n_layers * rows * (BLOCK_BYTES + ROW * rep_es)

    n_q = args.steps + args.warmup
    qs = torch.empty((n_q, n_layers, N_REQ, HQ, D), dtype=torch.bfloat16, device=dev)
    qs.normal_(generator=g)
    scores = torch.zeros(n_layers, rows, device=dev)
    idx = torch.full((n_layers, N_REQ, max_len), -1, dtype=torch.int32, device=dev)
    phys = torch.full_like(idx, -1)
    cnt = torch.zeros(n_layers, N_REQ, dtype=torch.int32, device=dev)
    region_h = topk.copy()
    dst_off_h = np.concatenate([[0], np.cumsum(region_h.astype(np.int64) * n_layers * 2)[:-1]]).astype(np.int64)
    total_blocks = int((region_h.astype(np.int64) * n_layers * 2).sum())
    region, dst_off = i32(region_h), torch.from_numpy(dst_off_h).to(dev)
    staging = torch.empty(total_blocks * BLOCK_BYTES, dtype=torch.uint8, device=dev)
    kv_stride = nb * BLOCK_BYTES

    tickets = torch.zeros_like(cnt)

    def step(q, events=None):
        if events:
            events[0].record()
        if args.two_launch:
            ops.score_blocks(q, repre, seg_off, seg_len, max_len, HKV, scores, total_blocks=rows)
            if events:
                events[1].record()
            ops.topk_windows(scores, seg_off, seg_len, topk_d, max_len, idx, cnt, block_tables=bt, phys_out=phys)
        else:
            # one launch: the last scoring workgroup of a (layer, request) runs its selection
            ops.score_select(q, repre, seg_off, seg_len, topk_d, max_len, HKV, scores, idx, cnt, tickets, block_tables=bt,
                             phys_out=phys, total_blocks=rows)
        if events:
            events[2].record()
        ops.kv_gather_selected(layers, kv_stride, BLOCK_BYTES, nb, phys, cnt, dst_off, region, max_k, staging,
                               total_blocks)
        if events:
            events[3].record()

    if args.calibrate_copy:
        gib = 1 << 30
        src = torch.empty(gib, dtype=torch.uint8, device=dev).random_(generator=leg_gen("calibrate"))
        dst = torch.empty_like(src)
        ops.copy_batch(torch.tensor([dst.data_ptr()], dtype=torch.int64, device=dev),
                       torch.tensor([src.data_ptr()], dtype=torch.int64, device=dev), gib)
        torch.cuda.synchronize()
        assert torch.equal(src, dst)
        del src, dst

    for w in range(args.warmup):
        step(qs[w])
    torch.cuda.synchronize()
    all_events = [[ev() for _ in range(4)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for s in range(args.steps):
        step(qs[args.warmup + s], all_events[s])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    if args.two_launch:
        k_ms = np.array([[e[i].elapsed_time(e[i + 1]) for i in range(3)] for e in all_events]).mean(0)
        score_ms, topk_ms, gather_ms = (float(x) for x in k_ms)
    else:       # one launch scores and selects: two spans per step
        k_ms = np.array([[e[0].elapsed_time(e[2]), e[2].elapsed_time(e[3])] for e in all_events]).mean(0)
        score_ms, topk_ms, gather_ms = float(k_ms[0]), 0.0, float(k_ms[1])

    n_sel = int(topk.astype(np.int64).sum()) * n_layers
    gather_bytes = 2 * n_sel * 2 * BLOCK_BYTES                                     # K and V, read + write
    score_bytes = n_layers * (rows * ROW * rep_es + N_REQ * HQ * D * 2 + rows * 4)  # representatives + bf16 q + scores
    gbs = lambda nbytes, ms: nbytes / (ms * 1e-3) / 1e9

    # ---- delta-gather leg: staging slots keep their blocks between steps, only missing blocks move
    delta = None
    if not args.no_delta:
        n_slots = max_k
        load_phys = torch.empty((n_layers, N_REQ, n_slots), dtype=torch.int32, device=dev)
        slot_of = torch.empty_like(idx)
        miss = torch.zeros_like(cnt)
        slots_count = torch.full_like(cnt, n_slots)
        noise = torch.empty(qs[0].shape, dtype=torch.float32, device=dev)
        st = staging.view(torch.bfloat16).view(-1, BS, HKV, D)

        def delta_run(rho: float) -> dict:
            gen = leg_gen(f"delta {rho}")
            resident = torch.full((n_layers, N_REQ, n_slots), -1, dtype=torch.int32, device=dev)
            q_t = qs[0].float()

            def delta_step(record=None):
                nonlocal q_t
                noise.normal_(generator=gen)
                q_t = rho * q_t + (1.0 - rho * rho) ** 0.5 * noise       # stationary N(0,1) sequence
                qb = q_t.to(torch.bfloat16)
                if record:
                    record[0].record()
                ops.score_select(qb, repre, seg_off, seg_len, topk_d, max_len, HKV, scores, idx, cnt, tickets, block_tables=bt,
                                 phys_out=phys, total_blocks=rows)
                ops.delta_plan(idx, phys, cnt, resident, load_phys, slot_of, miss)
                ops.kv_gather_selected(layers, kv_stride, BLOCK_BYTES, nb, load_phys, slots_count, dst_off, region, n_slots,
                                       staging, total_blocks)
                if record:
                    record[1].record()

            for _ in range(max(args.warmup, 2)):
                delta_step()                                              # the first step fills every slot
            torch.cuda.synchronize()
            d_events = [(ev(), ev()) for _ in range(args.steps)]
            moved = torch.zeros((), dtype=torch.int64, device=dev)
            for s_ in range(args.steps):
                delta_step(d_events[s_])
                moved += miss.sum()
            torch.cuda.synchronize()
            d_ms = float(np.mean([a_.elapsed_time(b_) for a_, b_ in d_events]))
            moved_per_step = float(moved.item()) / args.steps
            # the staging slots must hold exactly the selected blocks (checked on a sample of layers)
            for l in (0, n_layers // 2, n_layers - 1):
                for r in range(N_REQ):
                    k = int(cnt[l, r])
                    slots_lr = slot_of[l, r, :k].long()
                    for kv in range(2):
                        o = int(dst_off_h[r]) + (l * 2 + kv) * n_slots
                        assert torch.equal(st[o + slots_lr], caches[l][kv][phys[l, r, :k].long()]), "delta staging differs"
            return {"query_correlation": rho, "us_per_step": round(d_ms * 1e3, 1), "blocks_moved_per_step": round(moved_per_step, 1),
                    "hit_rate": round(1.0 - moved_per_step / n_sel, 4)}

        runs = [delta_run(float(rho)) for rho in args.delta_rho]
        delta = dict(runs[0])
        delta.update({
            "blocks_selected_per_step": n_sel,
            "by_correlation": runs,
            "note": "score + select (one launch) + resident-set plan + gather of missing blocks only; consecutive queries follow "
                    "q' = rho*q + sqrt(1-rho^2)*noise (synthetic); staging verified against the source blocks",
        })

    # ---- hash-code retrieval leg (configs[4]): 32 requests of 64-256 blocks, 32 layers, 128-bit codes.
    # The key blocks are the K and V planes of the caches above read as one pool of 2*nb blocks.
    # ---- load/dump leg: 1024 random blocks of every layer between the paged cache and a staging buffer in the
    # stored-block order [block][layer][K|V]; the scatter writes what the gather read, so the cache is unchanged
    moves_leg = None
    if args.moves_leg:
        m_blocks = 64 * 16
        m_ids = i32(leg_rng("moves").permutation(nb)[:m_blocks])
        m_stage = torch.empty(m_blocks * n_layers * 2 * BLOCK_BYTES, dtype=torch.uint8, device=dev)

        def timed_move(fn, reps=10):
            fn()
            torch.cuda.synchronize()
            e0, e1 = ev(), ev()
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / reps

        mv_gather_ms = timed_move(lambda: ops.kv_gather_blocks(layers, kv_stride, BLOCK_BYTES, nb, m_ids, m_stage))
        scatter_ms = timed_move(lambda: ops.kv_scatter_blocks(layers, kv_stride, BLOCK_BYTES, nb, m_ids, m_stage))
        move_bytes = 2 * m_blocks * n_layers * 2 * BLOCK_BYTES
        moves_leg = {
            "workload": f"configs[2]: {m_blocks} blocks x {n_layers} layers x (K, V) x {BLOCK_BYTES} B, random block table over "
                        f"{nb} blocks per layer",
            "algorithmic_bytes": move_bytes,
            "gather_ms": round(mv_gather_ms, 3), "scatter_ms": round(scatter_ms, 3),
            "gather_GBps": round(gbs(move_bytes, mv_gather_ms), 1), "scatter_GBps": round(gbs(move_bytes, scatter_ms), 1),
            "frac": [round(gbs(move_bytes, mv_gather_ms) / HBM_PEAK_GBS, 4), round(gbs(move_bytes, scatter_ms) / HBM_PEAK_GBS, 4)],
        }
        del m_stage

    hash_leg = None
    if args.hash_leg:
        h_req = 32
        h_rng, h_gen = leg_rng("hash"), leg_gen("hash")
        h_lens = h_rng.integers(64, 257, h_req).astype(np.int32)
        h_rows = int(h_lens.sum())
        h_off = np.concatenate([[0], np.cumsum(h_lens)[:-1]]).astype(np.int32)
        pool = 2 * nb
        h_ids_h = (h_rng.permutation(pool)[:h_rows] if h_rows <= pool else h_rng.integers(0, pool, h_rows)).astype(np.int32)
        if args.hash_distinct > 0:
            h_ids_h = h_ids_h[np.arange(h_rows) % args.hash_distinct]
        h_ids, h_slots = i32(h_ids_h), torch.arange(h_rows, dtype=torch.int32, device=dev)
        w_hash = (torch.randn(128, 128, device=dev, generator=h_gen) * 2.0).to(torch.bfloat16)
        colsum = torch.zeros((n_layers, h_rows, HKV, 128), dtype=torch.int16, device=dev)
        bcodes = torch.zeros((n_layers, h_rows, HKV, 16), dtype=torch.uint8, device=dev)
        tcodes = torch.zeros((n_layers, h_rows, BS, HKV, 16), dtype=torch.uint8, device=dev)
        hq = torch.empty((n_layers, h_req, HQ, D), dtype=torch.bfloat16, device=dev).normal_(generator=h_gen)
        q_codes = torch.zeros((n_layers, h_req, HQ, 16), dtype=torch.uint8, device=dev)
        q_sum = torch.zeros((n_layers, h_req, 128), dtype=torch.int16, device=dev)
        qbar = torch.zeros((n_layers, h_req, HKV, 16), dtype=torch.uint8, device=dev)
        h_scores = torch.zeros(n_layers, h_rows, device=dev)
        h_topk = np.maximum(16, (0.03 * h_lens).astype(np.int32)) + 3
        h_idx = torch.zeros((n_layers, h_req, int(h_lens.max())), dtype=torch.int32, device=dev)
        h_cnt = torch.zeros((n_layers, h_req), dtype=torch.int32, device=dev)
        h_so, h_sl, h_tk = i32(h_off), i32(h_lens), i32(h_topk)

        def timed(fn, reps):
            fn()
            torch.cuda.synchronize()
            e0, e1 = ev(), ev()
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / reps

        enc = lambda tc: ops.hash_encode_blocks(layers, h_ids, h_slots, h_rows, w_hash, BS, HKV, pool, colsum, bcodes,
                                                token_codes=tc)
        enc_ms = timed(lambda: enc(tcodes), 3)
        enc_sum_ms = timed(lambda: enc(None), 3)
        enc(tcodes)
        q_ms = timed(lambda: ops.hash_encode_queries(hq, w_hash, HKV, q_codes, q_sum, qbar, h_req), 10)
        sc_ms = timed(lambda: ops.hash_score_blocks(0, q_sum, qbar, colsum, bcodes, h_so, h_sl, h_rows, h_scores), 10)
        sc1_ms = timed(lambda: ops.hash_score_blocks(1, q_sum, qbar, colsum, bcodes, h_so, h_sl, h_rows, h_scores), 10)
        ops.hash_score_blocks(0, q_sum, qbar, colsum, bcodes, h_so, h_sl, h_rows, h_scores)
        tk_ms = timed(lambda: ops.topk_windows(h_scores, h_so, h_sl, h_tk, int(h_lens.max()), h_idx, h_cnt), 10)
        heads_sweep = None
        if args.hash_heads_sweep:
            # the same bytes as blocks of fewer heads: a [128][8][128] block is 8/h blocks of [128][h][128], and the
            # block list names all of them; the summary tables keep their size
            heads_sweep = {}
            for h in (8, 4, 2, 1):
                f = HKV // h
                ids_h = (h_ids.view(-1, 1) * f + torch.arange(f, dtype=torch.int32, device=dev)).reshape(-1).contiguous()
                slots_h = torch.arange(h_rows * f, dtype=torch.int32, device=dev)
                cs_h, bc_h = colsum.view(n_layers, h_rows * f, h, 128), bcodes.view(n_layers, h_rows * f, h, 16)
                ms = timed(lambda: ops.hash_encode_blocks(layers, ids_h, slots_h, h_rows * f, w_hash, BS, h, pool * f, cs_h, bc_h), 3)
                heads_sweep[str(h)] = {"blocks": h_rows * f, "ms": round(ms, 3)}
            enc(tcodes)                                  # the tables hold the 8-head results again
        key_bytes = n_layers * h_rows * BLOCK_BYTES
        enc_bytes = key_bytes + n_layers * h_rows * (BS * HKV * 16 + HKV * 128 * 2 + HKV * 16)
        hash_checked = None
        # HBM bytes per launch measured with rocprofv3 --pmc on exactly this workload, as for the gather below
        hash_workload = {"seed": args.seed, "layers": n_layers, "blocks": h_rows, "distinct": args.hash_distinct}
        if not args.no_check:
            import oracle  # checker only

            w_f32 = w_hash.float().cpu().numpy()
            for l in (0, n_layers - 1):
                pool_l = caches[l].view(2 * nb, BS, HKV, D)
                for row in (0, h_rows // 2, h_rows - 1):
                    keys = pool_l[int(h_ids_h[row])].view(torch.int16).cpu().numpy().view(np.uint16)
                    want = oracle.hash_encode(keys[None], w_f32)
                    assert np.array_equal(tcodes[l, row].cpu().numpy(), want[0]), "token codes differ"
                    assert np.array_equal(colsum[l, row].cpu().numpy(), oracle.hash_colsum(want)[0]), "column sums differ"
                    assert np.array_equal(bcodes[l, row].cpu().numpy(), oracle.hash_majority(want)[0]), "block codes differ"
            hash_checked = "token codes, column sums and majority codes of 6 sampled blocks equal the CPU oracle"
        hash_leg = {
            "workload": f"configs[4]: {h_req} requests, {h_rows} blocks of 128 tokens, {n_layers} layers, 8 kv heads, 128-bit codes"
                        + (f" (block list names {args.hash_distinct} distinct blocks: key loads served from cache)" if args.hash_distinct else ""),
            "encode_ms": round(enc_ms, 3),
            "encode_read_GBps": round(gbs(key_bytes, enc_ms), 1),
            "roofline": {"kernel": "hash_encode_blocks_kernel", "bound": "hbm", "achieved": round(gbs(enc_bytes, enc_ms), 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs(enc_bytes, enc_ms) / HBM_PEAK_GBS, 4),
                         "traffic": measured_traffic("hash_encode", "hash_encode_blocks_kernel", hash_workload),
                         "algorithmic_bytes": enc_bytes,
                         "mfma_TFLOPs": round(2.0 * n_layers * h_rows * BS * HKV * 128 * 128 / (enc_ms * 1e-3) / 1e12, 1)},
            "encode_summaries_only_ms": round(enc_sum_ms, 3),
            "encode_summaries_only_ms_by_kv_heads": heads_sweep,
            "decode_step_us": {"query_codes": round(q_ms * 1e3, 1), "score": round(sc_ms * 1e3, 1),
                               "score_block_code": round(sc1_ms * 1e3, 1), "select": round(tk_ms * 1e3, 1)},
            "checked": hash_checked,
        }
        del colsum, bcodes, tcodes

    # ---- KVStar leg: every (layer, request) is one task; 8 query tokens x 32 heads vote over the request's
    # blocks through block_size/merge sub-block representatives each (means of `merge` tokens of the same key
    # cache, fp16, kv head outermost), a share of the channels kept per (layer, kv head)
    kvstar_leg = None
    if args.kvstar_leg:
        kx, merge = 8, args.kvstar_merge
        k_gen = leg_gen("kvstar")
        km = BS // merge
        kdp = D if args.kvstar_prune >= 0.98 else round(D * args.kvstar_prune)
        kd_pad = (kdp + 15) // 16 * 16
        # kept channels: a seeded choice per (layer, kv head) (the reference keeps those with the largest mean |k|)
        kpr = None
        if kdp < D:
            kpr = torch.stack([torch.stack([torch.randperm(D, device=dev, generator=k_gen)[:kdp] for _ in range(HKV)])
                               for _ in range(n_layers)]).to(torch.int32)
        # one table over all layers, indexed [kv head][row][cell]: row of (layer l, block b) = l * rows + b
        if args.kvstar_layout == "row":      # the kv heads of a row next to each other in memory
            kmem = torch.empty((n_layers * rows, HKV, kd_pad // 8, km, 8), dtype=torch.float16, device=dev)
            flat = kmem.permute(1, 0, 2, 3, 4)
            ktab = kmem.view(n_layers, rows, HKV, kd_pad // 8, km, 8).permute(0, 2, 1, 3, 4, 5)
        else:                                # a plane per kv head
            flat = torch.empty((HKV, n_layers * rows, kd_pad // 8, km, 8), dtype=torch.float16, device=dev)
            ktab = flat.view(HKV, n_layers, rows, kd_pad // 8, km, 8).permute(1, 0, 2, 3, 4, 5)
        ev0, ev1 = ev(), ev()
        ops.kvstar_block_repre(layers, table, slots, ktab, BS, HKV, D, nb, merge, pruned=kpr)   # channel lists per layer
        torch.cuda.synchronize()
        krep_all = []
        for _ in range(5):
            ev0.record()
            ops.kvstar_block_repre(layers, table, slots, ktab, BS, HKV, D, nb, merge, pruned=kpr)   # one launch for all layers
            ev1.record()
            torch.cuda.synchronize()
            krep_all.append(ev0.elapsed_time(ev1))
        krep_ms = sorted(krep_all)[len(krep_all) // 2]
        krep_bytes = n_layers * rows * (BLOCK_BYTES + HKV * km * kd_pad * 2)
        n_tasks = n_layers * N_REQ
        k_off = (seg_off_h[None, :].astype(np.int64) + (np.arange(n_layers, dtype=np.int64) * rows)[:, None]).reshape(-1)
        k_len = np.tile(lens, n_layers)
        kq = (torch.randn(n_tasks, kx, HQ, D, device=dev, generator=k_gen) * 0.25).to(torch.float16)
        kq_off = torch.arange(n_tasks, dtype=torch.int64, device=dev) * (kx * HQ * D)
        ksel = None if kpr is None else torch.arange(n_layers, dtype=torch.int32, device=dev).repeat_interleave(N_REQ)
        kvotes = torch.zeros(n_layers * rows, device=dev)
        kws = ops.kvstar_workspace(n_tasks, HKV, kx * HQ // HKV, max_len, km, kd_pad, dev)
        kso, ksl = i32(k_off), i32(k_len)
        ktk = i32(np.tile(topk, n_layers))
        kidx = torch.zeros((1, n_tasks, max_len), dtype=torch.int32, device=dev)
        kcnt = torch.zeros((1, n_tasks), dtype=torch.int32, device=dev)

        def kvstar_step():
            ops.kvstar_votes(kq, kq_off, kx, HQ, flat, kso, ksl, max_len, kvotes, kws, d_pruned=kdp, pruned=kpr, pruned_sel=ksel)
            ops.kvstar_topk(kvotes, kso, ksl, ktk, max_len, kidx[0], kcnt[0])
            ops.kvstar_order(kvotes, kso, ksl, max_len, kidx[0], kcnt[0])     # the order the reference returns them in

        for _ in range(2):
            kvstar_step()
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(args.steps):
            kvstar_step()
        ev1.record()
        torch.cuda.synchronize()
        kv_ms = ev0.elapsed_time(ev1) / args.steps
        kv_bytes = flat.numel() * 2 + kq.numel() * 2 + kvotes.numel() * 4
        kv_checked = None
        if not args.no_check:
            import oracle  # checker only

            kv_cpu_s, kv_cpu_blocks = 0.0, 0
            for t_ in (0, n_tasks // 2 + 3, n_tasks - 1):
                a_, n_ = int(k_off[t_]), int(k_len[t_])
                rep_ref = ops.kvstar_table_to_reference(flat[:, a_ : a_ + n_]).contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
                pr_ = None if kpr is None else kpr[t_ // N_REQ].cpu().numpy().astype(np.int32)
                q_ref = kq[t_].view(torch.int16).cpu().numpy().view(np.uint16)
                t0_ = time.perf_counter()
                _, want = oracle.kvstar_retrieve(q_ref, rep_ref, int(topk[t_ % N_REQ]), pruned=pr_, d_pruned=kdp)
                kv_cpu_s += time.perf_counter() - t0_
                kv_cpu_blocks += n_
                got = kvotes[a_ : a_ + n_].cpu().numpy()
                assert np.allclose(got, want, rtol=2e-4, atol=2e-6), "KVStar votes differ from the CPU oracle"
                # the selection and its order are exact functions of the votes: the oracle's heap on the device's own votes
                heap = oracle.kvstar_topk(got, int(topk[t_ % N_REQ]))
                assert kidx[0, t_, : int(kcnt[0, t_])].cpu().numpy().tolist() == heap.tolist(), "KVStar selection differs from the heap"
            kv_checked = ("votes of 3 sampled tasks within rtol 2e-4 / atol 2e-6 of the CPU oracle (fp32, other summation order); "
                          "their chosen blocks, in order, equal the oracle's heap on the same votes")
        kv_workload = {"seed": args.seed, "layers": n_layers, "blocks": rows, "merge": merge, "channels": kdp}
        kvstar_leg = {
            "workload": f"{n_tasks} tasks (layer x request), {kx} query tokens x {HQ} heads, {rows} blocks x {km} sub-block "
                        f"representatives per layer, {kdp} of {D} channels, fp16",
            "table_layout": args.kvstar_layout,
            "block_repre_ms": round(krep_ms, 3),
            "block_repre_ms_all": [round(x, 3) for x in krep_all],
            "block_repre_GBps": round(gbs(krep_bytes, krep_ms), 1),
            "block_repre_frac": round(gbs(krep_bytes, krep_ms) / HBM_PEAK_GBS, 4),
            "block_repre_traffic": measured_traffic("kvstar_repre", "kvstar_repre_kernel", kv_workload),
            "block_repre_algorithmic_bytes": krep_bytes,
            "us_per_step": round(kv_ms * 1e3, 1),
            "roofline": {"kernel": "kvstar_score_kernel (+ head sum, select, order)", "bound": "hbm",
                         "achieved": round(gbs(kv_bytes, kv_ms), 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(gbs(kv_bytes, kv_ms) / HBM_PEAK_GBS, 4),
                         "traffic": measured_traffic("kvstar_votes", "kvstar_score_kernel", kv_workload),
                         "algorithmic_bytes": kv_bytes,
                         "mfma_TFLOPs": round(2.0 * n_layers * rows * km * HQ * kx * kd_pad / (kv_ms * 1e-3) / 1e12, 1)},
            "checked": kv_checked,
            "cpu_port": None if kv_checked is None else {
                "value": round(kv_cpu_s / kv_cpu_blocks * int(k_len.sum()) * 1e6, 1), "unit": "us/step", "cores": 1, "kind": "port",
                "sample": f"the scalar C restatement on the 3 checked tasks ({kv_cpu_blocks} of {int(k_len.sum())} (block, layer) "
                          f"pairs), scaled by blocks"},
        }
        del ktab, flat, kws, kpr

    # ---- ESA leg: the retrieval worker's backend call (scores of a slot list against a flat query in the
    # reference's sequential order, best k in descending order) on a 16384-row table of 1024-wide representatives
    esa_leg = None
    if args.esa_leg:
        e_rng, e_gen = leg_rng("esa"), leg_gen("esa")
        e_data = torch.randn(16384, HKV * D, device=dev, generator=e_gen)
        esa_leg = []
        for e_b, e_m, e_k in ((1, 512, 150), (64, 512, 150), (1, 8000, 3000)):
            e_q = torch.randn(e_b, HKV * D, device=dev, generator=e_gen)
            e_idx = i32(np.stack([e_rng.permutation(16384)[:e_m] for _ in range(e_b)]))
            e_ws = torch.zeros(e_b * e_m, device=dev)
            e_oi = torch.zeros(e_b, e_k, dtype=torch.int32, device=dev)
            e_os = torch.zeros(e_b, e_k, device=dev)
            e_oc = torch.zeros(e_b, dtype=torch.int32, device=dev)
            for _ in range(3):
                ops.esa_retrieve(e_data, e_q, e_idx, e_k, e_ws, e_oi, e_os, e_oc)
            torch.cuda.synchronize()
            e0, e1 = ev(), ev()
            e0.record()
            for _ in range(50):
                ops.esa_retrieve(e_data, e_q, e_idx, e_k, e_ws, e_oi, e_os, e_oc)
            e1.record()
            torch.cuda.synchronize()
            esa_leg.append({"requests": e_b, "candidates": e_m, "topk": e_k,
                            "us_per_call": round(e0.elapsed_time(e1) / 50 * 1000, 1)})
        del e_data

    # ---- configs[0]: one request of 32768 tokens (256 blocks), one layer: block means from the paged cache, then
    # scores + selection (k = 16 + first 1 + last 2) in one launch.  Latency-bound at this size: the figures are
    # times, the bandwidths only say how far from streaming a single small launch is.
    config1_leg = None
    if args.config1_leg:
        c_rng, c_gen = leg_rng("config1"), leg_gen("config1")
        c_n, c_k = 256, 19
        c_ids = i32(c_rng.permutation(nb)[:c_n])
        c_slots = torch.arange(c_n, dtype=torch.int32, device=dev)
        c_rep = torch.zeros((1, c_n, ROW), dtype=repre.dtype, device=dev)
        c_layer = ops.LayerPointers([caches[0][0]])
        c_q = torch.empty((1, 1, HQ, D), dtype=torch.bfloat16, device=dev).normal_(generator=c_gen)
        c_off, c_len, c_topk = i32([0]), i32([c_n]), i32([c_k])
        c_scores = torch.zeros(1, c_n, device=dev)
        c_idx = torch.full((1, 1, c_n), -1, dtype=torch.int32, device=dev)
        c_cnt, c_tickets = torch.zeros((1, 1), dtype=torch.int32, device=dev), torch.zeros((1, 1), dtype=torch.int32, device=dev)

        def timed_us(fn, reps=50):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            e0, e1 = ev(), ev()
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / reps * 1e3

        c_mean_us = timed_us(lambda: ops.block_mean(c_layer, c_ids, c_slots, c_rep, BS, HKV, D, nb, mode=ops.MEAN_BF16_ROUND))
        c_retr_us = timed_us(lambda: ops.score_select(c_q, c_rep, c_off, c_len, c_topk, c_n, HKV, c_scores, c_idx, c_cnt, c_tickets,
                                                      total_blocks=c_n))
        c_two_us = timed_us(lambda: (ops.score_blocks(c_q, c_rep, c_off, c_len, c_n, HKV, c_scores, total_blocks=c_n),
                                     ops.topk_windows(c_scores, c_off, c_len, c_topk, c_n, c_idx, c_cnt)))
        c_cpu_us = c_checked = None
        if not args.no_check or not args.no_cpu:
            import oracle  # checker / baseline only

            c_rep_h = c_rep[0].float().cpu().numpy()
            c_q_h = c_q[0].float().cpu().numpy()
            lens1, off1, k1 = np.array([c_n], np.int32), np.array([0], np.int32), np.array([c_k], np.int32)
            if not args.no_check:
                kc = caches[0][0].view(torch.int16)[c_ids.long()].cpu().numpy().view(np.uint16)
                want_rep = np.zeros((c_n, ROW), np.float32)
                oracle.block_mean_paged(kc, np.arange(c_n, dtype=np.int32), np.arange(c_n, dtype=np.int32), want_rep, round_bf16=True)
                assert np.array_equal(want_rep.view(np.uint32), c_rep_h.view(np.uint32)), "configs[0]: block means differ"
                widx, wcnt, wsc = oracle.select_topk_bs(c_q_h, c_rep_h, off1, lens1, k1, HKV, out_stride=c_n + 4)
                assert np.array_equal(wsc.view(np.uint32), c_scores[0].cpu().numpy().view(np.uint32)), "configs[0]: scores differ"
                assert int(c_cnt[0, 0]) == int(wcnt[0]) and np.array_equal(c_idx[0, 0, : wcnt[0]].cpu().numpy(), widx[0, : wcnt[0]])
                c_checked = "block means, fp32 scores and the selection equal the CPU oracle"
            if not args.no_cpu:
                ref_ok = oracle.ref.available and _cpu_has_avx512()
                fn = oracle.ref.select_topk_bs if ref_ok else oracle.select_topk_bs
                fn(c_q_h, c_rep_h, off1, lens1, k1, HKV, out_stride=c_n + 4)
                s0 = time.perf_counter()
                for _ in range(200):
                    fn(c_q_h, c_rep_h, off1, lens1, k1, HKV, out_stride=c_n + 4)
                c_cpu_us = (time.perf_counter() - s0) / 200 * 1e6
        c_mean_bytes = c_n * (BLOCK_BYTES + ROW * rep_es)
        c_score_bytes = c_n * ROW * rep_es + HQ * D * 2 + c_n * 4
        config1_leg = {
            "workload": f"configs[0]: 1 request x {c_n} blocks (32768 tokens), 1 layer, k = 16 + 1 first + 2 last, "
                        f"{args.repre_dtype} representatives",
            "block_mean_us": round(c_mean_us, 1), "retrieval_us": round(c_retr_us, 1), "retrieval_two_launches_us": round(c_two_us, 1),
            "roofline_block_mean": {"kernel": "block_mean_kernel", "bound": "hbm", "achieved": round(c_mean_bytes / c_mean_us / 1e3, 1),
                                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(c_mean_bytes / c_mean_us / 1e3 / HBM_PEAK_GBS, 4),
                                    "traffic": None, "algorithmic_bytes": c_mean_bytes},
            "roofline": {"kernel": score_name(args.repre_dtype == "f32"), "bound": "hbm", "achieved": round(c_score_bytes / c_retr_us / 1e3, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(c_score_bytes / c_retr_us / 1e3 / HBM_PEAK_GBS, 4),
                         "traffic": None, "algorithmic_bytes": c_score_bytes,
                         "note": "one workgroup chain of a few microseconds: launch latency, not bandwidth, is what this size measures"},
            "cpu_reference_retrieval_us": None if c_cpu_us is None else round(c_cpu_us, 1),
            "checked": c_checked,
        }

    # ---- configs[3]: 8 requests of 512-1024 blocks, 64 query heads in groups of 8, 80 layers; one decode step =
    # scores + selection of all layers (one launch), and - on the steps in which a request's last block fills up -
    # the block mean of one block per request, every layer.  The tables hold random bf16 values: the step does not
    # read the KV cache, and 80 layers of it would not fit beside the 32-layer one.
    config4_leg = None
    if args.config4_leg:
        f_rng, f_gen = leg_rng("config4"), leg_gen("config4")
        f_req, f_layers, f_hq = 8, 80, 64
        f_lens = f_rng.integers(512, 1025, f_req).astype(np.int32)
        f_rows, f_max = int(f_lens.sum()), int(f_lens.max())
        f_off_h = np.concatenate([[0], np.cumsum(f_lens)[:-1]]).astype(np.int32)
        f_topk_h = np.array([max(16, int(0.02 * n)) + 3 for n in f_lens], np.int32)
        f_off, f_len, f_topk = i32(f_off_h), i32(f_lens), i32(f_topk_h)
        f_q = torch.empty((f_layers, f_req, f_hq, D), dtype=torch.bfloat16, device=dev).normal_(generator=f_gen)
        f_scores = torch.zeros(f_layers, f_rows, device=dev)
        f_idx = torch.full((f_layers, f_req, f_max), -1, dtype=torch.int32, device=dev)
        f_cnt, f_tickets = torch.zeros((f_layers, f_req), dtype=torch.int32, device=dev), torch.zeros((f_layers, f_req), dtype=torch.int32, device=dev)
        f_tab16 = torch.empty((f_layers, f_rows, ROW), dtype=torch.bfloat16, device=dev).normal_(generator=f_gen)
        f_out = {}
        f_e0, f_e1 = ev(), ev()
        for name, tab in (("bf16", f_tab16), ("f32", None)):
            if tab is None:
                tab = f_tab16.float()                                   # the same values widened: the CPU path's table
            run = lambda: ops.score_select(f_q, tab, f_off, f_len, f_topk, f_max, HKV, f_scores, f_idx, f_cnt, f_tickets,
                                           total_blocks=f_rows)
            for _ in range(3):
                run()
            torch.cuda.synchronize()
            f_e0.record()
            for _ in range(args.steps):
                run()
            f_e1.record()
            torch.cuda.synchronize()
            us = f_e0.elapsed_time(f_e1) / args.steps * 1e3
            nbytes = f_layers * (f_rows * ROW * tab.element_size() + f_req * f_hq * D * 2 + f_rows * 4)
            f_kernel = "score_kernel_bf16" if name == "bf16" else "score_kernel"
            f_out[name] = {"retrieval_us": round(us, 1),
                           "roofline": {"kernel": f_kernel, "bound": "hbm",
                                        "achieved": round(nbytes / us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                        "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                                        "traffic": measured_traffic(f"config4_score_{name}_select", f_kernel,
                                                                    {"seed": args.seed, "layers": f_layers, "blocks": f_rows}),
                                        "algorithmic_bytes": nbytes}}
            if name == "f32":
                f_tab32 = tab
        # the incremental representative: the block that filled up, one per request, all 80 layers in one launch
        # (the 80 key planes are the 32 layers' K planes named again and again)
        f_planes = ops.LayerPointers([caches[l % n_layers][0] for l in range(f_layers)])
        f_new_ids = [i32(f_rng.permutation(nb)[:f_req]) for _ in range(args.steps + 3)]   # other blocks every time: nothing cached
        f_new_slots = i32(f_off_h + f_lens - 1)
        inc = lambda i: ops.block_mean(f_planes, f_new_ids[i], f_new_slots, f_tab16, BS, HKV, D, nb, mode=ops.MEAN_BF16_ROUND)
        for i in range(3):
            inc(i)
        torch.cuda.synchronize()
        f_e0.record()
        for i in range(args.steps):
            inc(3 + i)
        f_e1.record()
        torch.cuda.synchronize()
        f_inc_us = f_e0.elapsed_time(f_e1) / args.steps * 1e3
        f_inc_bytes = f_layers * f_req * (BLOCK_BYTES + ROW * 2)
        f_cpu_us = f_checked = None
        if not args.no_check or not args.no_cpu:
            import oracle  # checker / baseline only

            ops.score_select(f_q, f_tab32, f_off, f_len, f_topk, f_max, HKV, f_scores, f_idx, f_cnt, f_tickets, total_blocks=f_rows)
            torch.cuda.synchronize()
            f_q_h = f_q.float().cpu().numpy()
            if not args.no_check:
                for l in (0, f_layers // 2, f_layers - 1):
                    widx, wcnt, wsc = oracle.select_topk_bs(f_q_h[l], f_tab32[l].cpu().numpy(), f_off_h, f_lens, f_topk_h, HKV,
                                                            out_stride=f_max + 4)
                    assert np.array_equal(wsc.view(np.uint32), f_scores[l].cpu().numpy().view(np.uint32)), f"configs[3]: scores differ ({l})"
                    got_i, got_c = f_idx[l].cpu().numpy(), f_cnt[l].cpu().numpy()
                    for r in range(f_req):
                        assert got_c[r] == wcnt[r] and np.array_equal(got_i[r, : wcnt[r]], widx[r, : wcnt[r]]), f"configs[3]: selection differs ({l},{r})"
                f_checked = "fp32 scores and selections of 3 of the 80 layers equal the CPU oracle"
            if not args.no_cpu:
                ref_ok = oracle.ref.available and _cpu_has_avx512()
                fn = oracle.ref.select_topk_bs if ref_ok else oracle.select_topk_bs
                f_rep_h = f_tab32.cpu().numpy()

                def f_cpu_step():
                    for l in range(f_layers):
                        fn(f_q_h[l], f_rep_h[l], f_off_h, f_lens, f_topk_h, HKV, out_stride=f_max + 4)

                f_cpu_step()
                f_reps, f_acc = 0, 0.0
                while f_acc < 4.0 and f_reps < 50:
                    s0 = time.perf_counter()
                    f_cpu_step()
                    f_acc += time.perf_counter() - s0
                    f_reps += 1
                f_cpu_us = f_acc / f_reps * 1e6
                del f_rep_h
        config4_leg = {
            "workload": f"configs[3]: {f_req} requests, {f_rows} blocks ({int(f_lens.min())}-{f_max} each), {f_hq} query heads in groups of "
                        f"{f_hq // HKV}, {f_layers} layers, k = max(16, 2%) + 1 first + 2 last",
            "bf16_table": f_out["bf16"], "f32_table": f_out["f32"],
            "incremental_block_mean": {"blocks_per_launch": f_req * f_layers, "us": round(f_inc_us, 1),
                                       "GBps": round(f_inc_bytes / f_inc_us / 1e3, 1),
                                       "note": "one block per request and layer, 80 layers in one launch; runs on the steps in "
                                               "which a request's last block fills up (every 128th per request)"},
            "cpu_reference_retrieval_us": None if f_cpu_us is None else round(f_cpu_us, 1),
            "cpu_reference": None if f_cpu_us is None else
                f"the reference's own translation units where AVX-512 is present (else the port), {min(16, os.cpu_count() or 1)} OpenMP "
                "threads over blocks, requests and layers serial, fp32 table in host memory",
            "checked": f_checked,
        }
        del f_tab16, f_tab32, f_scores, f_idx

    # ---- check the last step against the CPU oracle (selection, scores, gathered bytes)
    if not args.no_check:
        step(qs[n_q - 1])                                             # re-run the last full step: the delta leg reused the buffers
        torch.cuda.synchronize()
    checked = None
    if not args.no_check:
        import oracle  # checker only

        q_last = qs[n_q - 1].float().cpu().numpy()
        idx_h, cnt_h, phys_h = idx.cpu().numpy(), cnt.cpu().numpy(), phys.cpu().numpy()
        scores_h = scores.cpu().numpy()
        for l in range(n_layers):
            rep = repre[l].float().cpu().numpy()
            widx, wcnt, wsc = oracle.select_topk_bs(q_last[l], rep, seg_off_h, lens, topk, HKV, out_stride=max_len + 4)
            assert np.array_equal(wsc.view(np.uint32), scores_h[l].view(np.uint32)), f"scores differ in layer {l}"
            assert np.array_equal(wcnt, cnt_h[l]), f"counts differ in layer {l}"
            for r in range(N_REQ):
                assert np.array_equal(widx[r, : wcnt[r]], idx_h[l, r, : wcnt[r]]), f"selection differs ({l},{r})"
                assert np.array_equal(phys_h[l, r, : wcnt[r]], bt_h[r][widx[r, : wcnt[r]]])
        # gathered bytes: every staged block equals its source block (device-side compare, all of them)
        st = staging.view(torch.bfloat16).view(-1, BS, HKV, D)
        for l in range(n_layers):
            for r in range(N_REQ):
                k = int(topk[r])
                sel = phys[l, r, :k].long()
                for kv in range(2):
                    o = int(dst_off_h[r]) + (l * 2 + kv) * k
                    assert torch.equal(st[o : o + k], caches[l][kv][sel]), f"gathered bytes differ ({l},{r},{kv})"
        checked = "last step: fp32 scores, selected indices, block-table lookup and all gathered bytes equal the CPU oracle / source blocks"

    # ---- CPU baseline: the reference's CPU retrieval (same arithmetic, its threading) + memcpy gather
    cpu = None
    if not args.no_cpu:
        import oracle

        threads = min(16, os.cpu_count() or 1)
        os.environ.setdefault("OMP_NUM_THREADS", str(threads))
        rep_h = repre.float().cpu().numpy()
        q_h = qs[0].float().cpu().numpy()
        use_ref = oracle.ref.available and _cpu_has_avx512()
        out_stride = max_len + 4

        def cpu_retrieval():
            for l in range(n_layers):
                if use_ref:
                    oracle.ref.select_topk_bs(q_h[l], rep_h[l], seg_off_h, lens, topk, HKV, out_stride=out_stride)
                else:
                    oracle.select_topk_bs(q_h[l], rep_h[l], seg_off_h, lens, topk, HKV, out_stride=out_stride)

        cpu_retrieval()
        reps, t_acc = 0, 0.0
        while t_acc < args.cpu_seconds * 0.6 and reps < 200:
            s0 = time.perf_counter()
            cpu_retrieval()
            t_acc += time.perf_counter() - s0
            reps += 1
        cpu_retr_us = t_acc / reps * 1e6
        # gather sample: a few layers of the cache on the host, the selected blocks copied by the same host threads as
        # the retrieval part, extrapolated to all layers
        g_layers = min(2, n_layers)
        host_layers = [caches[l].view(torch.uint8).reshape(-1).cpu().numpy() for l in range(g_layers)]
        g_total = int((region_h.astype(np.int64) * g_layers * 2).sum())
        g_off = np.concatenate([[0], np.cumsum(region_h.astype(np.int64) * g_layers * 2)[:-1]]).astype(np.int64)
        g_stage = np.empty(g_total * BLOCK_BYTES, np.uint8)
        ph, ch = phys.cpu().numpy()[:g_layers].copy(), cnt.cpu().numpy()[:g_layers].copy()
        oracle.kv_gather_selected(host_layers, kv_stride, BLOCK_BYTES, ph, ch, g_off, region_h, g_stage)
        greps, g_acc = 0, 0.0
        while g_acc < args.cpu_seconds * 0.4 and greps < 50:
            s0 = time.perf_counter()
            oracle.kv_gather_selected(host_layers, kv_stride, BLOCK_BYTES, ph, ch, g_off, region_h, g_stage)
            g_acc += time.perf_counter() - s0
            greps += 1
        cpu_gather_us = g_acc / greps * 1e6 * (n_layers / g_layers)
        cpu = {
            "value": round(cpu_retr_us + cpu_gather_us, 1),
            "unit": "us/step",
            "cores": threads,
            "kind": "reference" if use_ref else "port",
            "retrieval_us": round(cpu_retr_us, 1),
            "gather_us": round(cpu_gather_us, 1),
            "sample": (f"retrieval: {reps} full steps (all {n_layers} layers x {N_REQ} requests, fp32 representatives "
                       f"resident in host DRAM, {threads} OpenMP threads over blocks, requests and layers serial); "
                       f"gather: EXTRAPOLATED from {g_layers} of {n_layers} layers ({greps} passes, memcpy of the selected "
                       f"blocks on {threads} OpenMP threads, time x{n_layers // g_layers})"),
            "host_cpus": os.cpu_count(),
        }

    # ---- prefetch leg: one round of the GSA prefetch engine per decode step - which selected blocks are resident,
    # which free cache block takes each missing one, the new block tables - and the loads it plans, from a pool of
    # stored blocks in device memory.  Runs last: it overwrites cache blocks.
    prefetch_leg = None
    if args.prefetch_leg:
        from ucm_amd.sparse.gsa.gsa import GSAReqStat
        from ucm_amd.sparse.gsa.prefetch import GSAPrefetchEngineC
        from ucm_amd.sparse.utils import LOCAL_WINDOW_SZ, MAX_TOPK_LEN, MIN_TOPK_LEN, compute_topk_len

        p_gen = leg_gen("prefetch")
        width = 64                                          # table row: MAX_TOPK_LEN + 1 resident blocks fit
        i32z = lambda *shape: torch.zeros(shape, dtype=torch.int32, device=dev)
        p_free, p_free_len = i32z(n_layers, N_REQ, width), i32z(n_layers, N_REQ)
        p_succ, p_succ_len = i32z(n_layers, N_REQ, width), i32z(n_layers, N_REQ)
        eng = GSAPrefetchEngineC(p_free, p_succ, p_free_len, p_succ_len, False)
        p_topk_h = np.array([compute_topk_len(int(n)) for n in lens], np.int32)      # 30 % of the blocks, 32..48
        resident_h = []
        for r in range(N_REQ):
            n = int(lens[r])
            st_ = GSAReqStat(r, 0, BS, 0)
            st_.blocks = [int(x) for x in bt_h[r, :n]]
            st_.num_prompt_tokens = st_.num_computed_tokens = n * BS
            st_.get_sparse_and_free_block(True, MIN_TOPK_LEN, MAX_TOPK_LEN, 0.3)
            # positions 0..MAX_TOPK_LEN of the request's block list are the cache blocks it keeps; the last
            # LOCAL_WINDOW_SZ of the used ones hold the request's last logical blocks (prefetch_engine.py:327-379)
            used, spare = st_.remain_idx, st_.prefetch_idx
            logical = spare + used[:-LOCAL_WINDOW_SZ] + list(range(n - LOCAL_WINDOW_SZ, n))
            holder = {i: st_.blocks[i] for i in spare + used[:-LOCAL_WINDOW_SZ]}
            holder.update({n - LOCAL_WINDOW_SZ + j: st_.blocks[p_] for j, p_ in enumerate(used[-LOCAL_WINDOW_SZ:])})
            eng.set_blocks_map(r, holder, logical)
            p_free[:, r, : len(spare)] = i32([st_.blocks[x] for x in spare])
            p_free_len[:, r] = len(spare)
            resident_h.append((holder, logical, [st_.blocks[x] for x in spare]))
        pool = torch.empty((rows, n_layers, 2, BLOCK_BYTES), dtype=torch.uint8, device=dev)
        for l0 in range(0, rows, 256):                      # stored blocks are K and V values like the caches' (the loads
            pool[l0 : l0 + 256].view(torch.bfloat16).normal_(generator=p_gen)       # write them into the caches later legs read)
        src_table = torch.full((N_REQ, max_len), -1, dtype=torch.int32, device=dev)
        for r in range(N_REQ):
            src_table[eng.row_of(r), : lens[r]] = torch.arange(int(seg_off_h[r]), int(seg_off_h[r] + lens[r]), dtype=torch.int32, device=dev)
        p_topk = i32(p_topk_h)
        p_idx = torch.full((n_layers, N_REQ, max_len), -1, dtype=torch.int32, device=dev)
        p_cnt = torch.zeros(n_layers, N_REQ, dtype=torch.int32, device=dev)
        req_ids, bs_idx, tk_list = list(range(N_REQ)), list(range(N_REQ)), [int(k) for k in p_topk_h]
        rho = float(args.delta_rho[0])
        q_cur = qs[0].float()
        n_rounds = 4 + min(args.steps, 16)
        ev_p = [[ev() for _ in range(4)] for _ in range(n_rounds)]
        loads_per_round, topk_rounds = [], []
        for t in range(n_rounds):
            if t:
                q_cur = rho * q_cur + (1.0 - rho * rho) ** 0.5 * torch.randn(q_cur.shape, device=dev, generator=p_gen)
            ops.score_blocks(q_cur.to(torch.bfloat16), repre, seg_off, seg_len, max_len, HKV, scores, total_blocks=rows)
            ops.topk_windows(scores, seg_off, seg_len, p_topk, max_len, p_idx, p_cnt)
            sel = p_idx[:, :, :MAX_TOPK_LEN].contiguous()
            ev_p[t][0].record()
            eng.set_blocks_table_info(p_succ, p_succ_len, sel, t)
            ev_p[t][1].record()
            eng.run_async_prefetch_bs(req_ids, tk_list, bs_idx, 0)
            ev_p[t][2].record()
            eng.load_missing(layers, kv_stride, BLOCK_BYTES, nb, pool.view(-1), n_layers * 2 * BLOCK_BYTES, src_table)
            ev_p[t][3].record()
            loads_per_round.append(eng.load_count.sum())
            topk_rounds.append(sel)
        torch.cuda.synchronize()
        p_ms = np.array([[e[i].elapsed_time(e[i + 1]) for i in range(3)] for e in ev_p[4:]]).mean(0)   # rounds 0-3 warm the set up
        loads_h = [int(x) for x in loads_per_round]
        steady = float(np.mean(loads_h[4:]))
        sel_per_round = int(p_topk_h.sum()) * n_layers
        load_bytes = 2 * steady * 2 * BLOCK_BYTES
        p_checked = None
        if not args.no_check:
            # the blocks the last round loaded hold the bytes of the stored blocks it named
            lb, mi = eng.obtain_load_blocks(), eng.obtain_miss_idxs()
            n_cmp = 0
            for r in range(N_REQ):
                for l in (0, n_layers // 2, n_layers - 1):
                    for blk, idx_ in zip(lb[r][l], mi[r][l]):
                        for kv in range(2):
                            got = caches[l][kv][blk].view(torch.uint8).reshape(-1)
                            assert torch.equal(got, pool[int(seg_off_h[r]) + idx_, l, kv]), f"prefetch load differs ({r},{l},{blk})"
                        n_cmp += 1
            p_checked = f"{n_cmp} blocks loaded by the last round (3 layers x all requests) hold the stored blocks' bytes, K and V"
        # the reference's own engine (kvcache_pre.cpp compiled against torch into oracle/_ref) on the same rounds
        cpu_round_us = None
        if not args.no_cpu:
            import oracle

            gp = oracle.ref.gsa_prefetch_module()
            if gp is not None:
                c32 = dict(dtype=torch.int32)
                c_free, c_free_len = torch.zeros((n_layers, N_REQ, width), **c32), torch.zeros((n_layers, N_REQ), **c32)
                c_succ, c_succ_len = torch.zeros((n_layers, N_REQ, width), **c32), torch.zeros((n_layers, N_REQ), **c32)
                ceng = gp.GSAPrefetchEngineC(c_free, c_succ, c_free_len, c_succ_len, False)
                for r, (holder, logical, spare_blocks) in enumerate(resident_h):
                    table_list = [0] * int(lens[r])
                    for i_, b_ in holder.items():
                        table_list[i_] = b_
                    ceng.set_blocks_map(r, table_list, logical)
                    c_free[:, r, : len(spare_blocks)] = torch.tensor(spare_blocks, **c32)
                    c_free_len[:, r] = len(spare_blocks)
                t_cpu = []
                for t, sel in enumerate(topk_rounds):
                    buf = sel.cpu().to(torch.int64)
                    s0 = time.perf_counter()
                    ceng.set_blocks_table_info(c_succ, c_succ_len, buf, t)
                    ceng.run_async_prefetch_bs(req_ids, tk_list, bs_idx, 0)
                    while not ceng.get_prefetch_status():
                        time.sleep(0.00005)
                    t_cpu.append(time.perf_counter() - s0)
                cpu_round_us = float(np.mean(t_cpu[4:]) * 1e6)
                assert torch.equal(c_succ_len, p_succ_len.cpu()) and torch.equal(c_succ, p_succ.cpu()), \
                    "device and reference engines left different block tables"
        prefetch_leg = {
            "workload": f"{N_REQ} requests x {n_layers} layers, {MAX_TOPK_LEN + 1} cache blocks kept per request, "
                        f"{int(p_topk_h.min())}-{int(p_topk_h.max())} blocks selected per (request, layer), consecutive queries "
                        f"correlated with rho = {rho} (synthetic), stored blocks [block][layer][K|V] in device memory",
            "us_per_round": round(float(p_ms.sum()) * 1e3, 1),
            "table_info_us": round(float(p_ms[0]) * 1e3, 1),
            "plan_us": round(float(p_ms[1]) * 1e3, 1),
            "loads_us": round(float(p_ms[2]) * 1e3, 1),
            "blocks_selected_per_round": sel_per_round,
            "blocks_loaded_per_round": round(steady, 1),
            "hit_rate": round(1.0 - steady / sel_per_round, 4),
            "loads_GBps": round(gbs(load_bytes, float(p_ms[2])), 1) if steady else None,
            "cpu_reference_plan_us": None if cpu_round_us is None else round(cpu_round_us, 1),
            "cpu_reference": None if cpu_round_us is None else
                "GSAPrefetchEngineC of the reference (kvcache_pre.cpp, its worker thread + 16 OpenMP threads over layers) on the "
                "same selections: set_blocks_table_info + run_async_prefetch_bs until get_prefetch_status(); bookkeeping "
                "only, the reference loads through its store connector afterwards; tables equal the device's",
            "checked": p_checked,
        }
        del pool

    # ---- plugin leg: the four plugins' hooks on this batch, host time included (runs last: loads overwrite cache blocks)
    plugin_leg = None
    if args.plugin_leg:
        import plugin_bench

        block_lists = [[int(x) for x in bt_h[r, : lens[r]]] for r in range(N_REQ)]
        del staging
        gc.collect()
        torch.cuda.empty_cache()
        plugin_leg = {"device_memory_free_GB": round(torch.cuda.mem_get_info(dev)[0] / 1e9, 1),
                      "note": "hooks driven by stand-in objects for vLLM's (plugin_bench.py), 16 requests x "
                              f"{n_layers} layers; host_us = the hooks' time on the model-runner thread, wall_us = until the "
                              "device has finished what they queued (no model runs in between); medians per kind of step"}
        for name, leg in (("GSA", lambda: plugin_bench.gsa_leg(torch, dev, caches, lens, block_lists, args.steps, args.seed)),
                          ("GSA, retrieval_lag 1", lambda: plugin_bench.gsa_leg(torch, dev, caches, lens, block_lists, args.steps, args.seed, 1)),
                          ("ESA", lambda: plugin_bench.esa_leg(torch, dev, caches, lens, block_lists, args.seed)),
                          ("KvComp", lambda: plugin_bench.kvcomp_leg(torch, dev, caches, lens, block_lists, args.seed)),
                          ("KvComp, delta_loads (decode queries drift with correlation 0.95 per step)",
                           lambda: plugin_bench.kvcomp_leg(torch, dev, caches, lens, block_lists, args.seed, True, 0.95)),
                          ("KVStar", lambda: plugin_bench.kvstar_leg(torch, dev, caches, lens, block_lists, args.seed))):
            plugin_leg[name] = leg()
            gc.collect()                                     # the leg's plugin and its store (a KV cache's worth of memory)
            torch.cuda.empty_cache()

    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on exactly this workload
    # (profiles/bench_config2_kernels.md); other workloads have no measurement
    main_workload = {"seed": args.seed, "layers": n_layers, "blocks": rows}
    score_kernel_name = "score_kernel_bf16" if args.repre_dtype == "bf16" else "score_kernel"   # what the scoring calls launch
    traffic_gather = measured_traffic("gather", "kv_gather_selected_kernel", main_workload)
    traffic_score = measured_traffic("score_" + args.repre_dtype + ("" if args.two_launch else "_select"), score_kernel_name,
                                     main_workload)

    out = {
        "metric": "us per decode step (32-layer retrieval+gather)",
        "value": round(ms_per_step * 1e3, 1),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "dtype_detail": "bf16 keys and queries, scores accumulated and compared in fp32, KV blocks moved as bytes",
        "data": "synthetic (seeded N(0,1) bf16 keys, values and queries; random block table)",
        "config": {
            "workload": "configs[1]: ragged batch of 16 requests, 4096-65536 tokens, Llama-3-8B attention shape, "
                        f"{n_layers} layers, k = max(16, 3%) + 1 first + 2 last, full gather of selected K and V blocks",
            "representatives": ("bf16 table (block means rounded to the model dtype, as the live reference path stores them)"
                                if args.repre_dtype == "bf16" else "fp32 table holding the bf16-rounded block means"),
            "blocks_per_request": [int(x) for x in lens],
            "total_blocks": rows,
            "selected_blocks_per_step": n_sel,
            "kv_cache_GB": round(n_layers * 2 * nb * BLOCK_BYTES / 1e9, 1),
        },
        "kernels_us": ({"score": round(score_ms * 1e3, 1), "select": round(topk_ms * 1e3, 1), "gather": round(gather_ms * 1e3, 1)}
                       if args.two_launch else {"score_select": round(score_ms * 1e3, 1), "gather": round(gather_ms * 1e3, 1)}),
        "launches_per_step": 3 if args.two_launch else 2,
        "retrieval_us": round((score_ms + topk_ms) * 1e3, 1),
        "roofline": {
            "kernel": "kv_gather_selected_kernel",
            "bound": "hbm",
            "achieved": round(gbs(gather_bytes, gather_ms), 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs(gather_bytes, gather_ms) / HBM_PEAK_GBS, 4),
            "traffic": traffic_gather,
            "algorithmic_bytes": gather_bytes,
        },
        "roofline_score": {
            "kernel": score_kernel_name + ("" if args.two_launch else " (scores, and each request's selection by its last workgroup)"),
            "bound": "hbm",
            "achieved": round(gbs(score_bytes, score_ms), 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs(score_bytes, score_ms) / HBM_PEAK_GBS, 4),
            "traffic": traffic_score,
            "algorithmic_bytes": score_bytes,
        },
        "block_mean_prefill": {"ms": round(mean_ms, 3), "GBps": round(gbs(mean_bytes, mean_ms), 1),
                               "frac": round(gbs(mean_bytes, mean_ms) / HBM_PEAK_GBS, 4)},
        "delta_gather": delta,
        "config1": config1_leg,
        "config4": config4_leg,
        "plugin_steps": plugin_leg,
        "kv_moves": moves_leg,
        "prefetch_round": prefetch_leg,
        "hash_retrieval": hash_leg,
        "esa_retrieval": esa_leg,
        "kvstar_retrieval": kvstar_leg,
        "cpu_baseline": cpu,
        "checked": checked,
    }
    print(json.dumps(out))


def _cpu_has_avx512() -> bool:
    try:
        with open("/proc/cpuinfo") as f:
            return "avx512f" in f.read()
    except OSError:
        return False


if __name__ == "__main__":
    main()
