#!/usr/bin/env python3
"""Benchmark of the speculative-decoding verify step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2_verify_4k]

One "step" = one pass of the verify hot path over one batch of synthetic MiniCPM4-8B-shaped input,
with every input already resident in HBM: for each of the 32 layers append the 60 tree rows' K/V and
run tree-masked attention (one fused kernel + the split merge) over the paged cache (4096-token prefix + 60 tree rows), then the target
lm_head (73448 x 4096) with fused arg-max, greedy tree acceptance and accepted-path KV compaction in
all layers.  The step is captured into a HIP graph (the reference replays a CUDA graph for
decode as well) and replayed; exactly K replays are timed between synchronisations.  At 4K context
the K/V of all layers would fit the 256 MB last-level cache, so the timed steps rotate over four
distinct copies of the K/V pools (one graph each): every pass over K/V comes from HBM.  The time of
replays on a single copy is reported beside it (`us_per_step_one_kv_set`).

Prints ONE JSON line.  `value` is microseconds per step (lower is better).  `roofline` is for the
kernel that takes the largest share of the step; `kernels` lists all of them; `contexts` gives the
step time at 4K / 32K / 128K context; `cpu_baseline` is the CPU oracle timed on this host on a
bounded sample of the same workload (a reported baseline only).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0

# HBM bytes per launch on c2_verify_4k with the automatic split count, from rocprofv3's FETCH_SIZE and
# WRITE_SIZE counters (KiB per dispatch, one counter per run, eager launches), each scaled by what the
# same counter read for a plain 256 MiB copy (x2.000 and x1.000): the table and the two commands are in
# profiles/verify_step_hbm_traffic.md.  Counters cannot be read from inside this process, so the figures
# are carried here as constants and are reported only for the workload they were measured on.
MEASURED_TRAFFIC_KIB = {
    "tree_attn_split_kernel+tree_attn_combine_kernel": 6367 + 8494 + 8710 + 480,
    "head_gemm_chunked_kernel<4,4,256,2>+head_argmax_finalize_kernel": 592012 + 128 + 1052 + 2,
    "tree_accept_kernel+kv_compact_kernel+accepted_ids_kernel": 6 + 1137 + 335 + 4,
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2_verify_4k")
    ap.add_argument("--splits", type=int, default=0, help="force the KV split count of tree attention (0 = auto)")
    ap.add_argument("--no-contexts", action="store_true", help="skip the 32K / 128K context step timings")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-probes", action="store_true", help="skip the MFMA-rate probe of the machine")
    ap.add_argument("--accept-depth", type=int, default=3, help="draft tokens the rigged tree gets accepted")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run a plain 256 MiB device copy three times: the known-size kernel that scales "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    return ap.parse_args()


class Workload:
    """Synthetic tensors of one configuration, resident on the GPU."""

    def __init__(self, torch, name, accept_depth, seed=0):
        import numpy as np
        from cpm.cu_amd import synth
        from cpm.cu_amd.kvcache import PagedKVCache
        cfg = dict(synth.CONFIGS[name])
        shp = synth.MINICPM4_8B
        self.name, self.cfg, self.shape = name, cfg, shp
        L, P, T = cfg["layers"], cfg["prefix"], cfg["T"]
        Hq, Hkv, D, H, V = shp["q_heads"], shp["kv_heads"], shp["head_dim"], shp["hidden"], shp["vocab"]
        self.L, self.P, self.T = L, P, T
        dev = torch.device("cuda:0")
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        S = P + T
        npages = (S + 255) // 256 + 1
        table = synth.rng(seed, 4).permutation(npages).astype(np.int32)  # seeded page-table permutation
        self.cache = PagedKVCache(L, Hkv, npages, device=dev, block_table=table)
        for l in range(L):  # ~N(0,1) prefix K/V, written page by page in the kernels' layout
            self.cache.k[l].normal_(generator=g)
            self.cache.v[l].normal_(generator=g)
        rn = lambda *s, std=1.0: (torch.randn(*s, device=dev, dtype=torch.float32, generator=g) * std).to(torch.float16)
        self.q = [rn(T, Hq, D) for _ in range(L)]
        self.k_new = [rn(T, Hkv, D) for _ in range(L)]
        self.v_new = [rn(T, Hkv, D) for _ in range(L)]
        self.hidden = rn(T, H)
        self.w = rn(V, H, std=0.02)
        self.tree = synth.eagle_tree(cfg["num_iter"], cfg["topk"], T, seed)
        tm = torch.from_numpy(self.tree.mask.view(np.int64)).to(dev)
        self.mask = tm
        self.parent = torch.from_numpy(self.tree.parent).to(dev)
        self.pos = torch.from_numpy(self.tree.positions(P)).to(dev)
        self.accept_depth = min(accept_depth, int(self.tree.depth.max()))
        self.draft_ids = None  # rigged from the target arg-max once it is known
        self.attn_out = [torch.empty(T, Hq, D, dtype=torch.float16, device=dev) for _ in range(L)]

    def rig_draft(self, torch, gt_np):
        from cpm.cu_amd import synth
        pred, self.leaf = synth.draft_ids_for_accept(self.tree, gt_np, self.accept_depth, self.shape["vocab"], 1)
        self.draft_np = pred
        self.draft_ids = torch.from_numpy(pred).cuda()

    def flops_attention_layer(self):
        s = self.shape
        return 4.0 * s["q_heads"] * self.T * s["head_dim"] * (self.P + self.T)

    def bytes_attention_layer(self):
        s = self.shape
        return 2.0 * (self.P + self.T) * s["kv_heads"] * s["head_dim"] * 2 + 2.0 * self.T * s["q_heads"] * s["head_dim"] * 2

    def bytes_target_head(self):
        s = self.shape
        return s["vocab"] * s["hidden"] * 2.0 + self.T * s["hidden"] * 2.0 + self.T * 4.0


def timed_replays(torch, fn, steps, warmup, use_graph):
    """Capture fn() once (unless disabled), run `warmup` untimed and exactly `steps` timed calls.
    `fn` may be a list of callables: each is captured on its own and the calls cycle through them."""
    fns = list(fn) if isinstance(fn, (list, tuple)) else [fn]
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        runs = []
        for f in fns:
            f()  # eager once: allocates workspaces outside capture
            stream.synchronize()
            if use_graph:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    f()
                runs.append(graph.replay)
            else:
                runs.append(f)
        for i in range(warmup):
            runs[i % len(runs)]()
        stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(stream)
        for i in range(steps):
            runs[i % len(runs)]()
        e1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        ev_ms = e0.elapsed_time(e1)
    return ev_ms / steps, wall_ms / steps


def machine_probes(torch):
    """What this GPU gives a kernel that does nothing but MFMAs from registers: with all-zero operands and
    with random ones -- the sustained rate depends on the bits (clocks follow the power drawn).
    Event-timed, eager."""
    import bench_probes
    out = {}
    n = bench_probes.load().bench_mfma_rate_probe_operand_bytes() // 2
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    for name, data in (("zero_operands", torch.zeros(n, dtype=torch.float16, device="cuda")),
                       ("random_operands", torch.randn(n, device="cuda", generator=g).to(torch.float16))):
        bench_probes.mfma_rate_probe(data, 200)
        torch.cuda.synchronize()
        best = 0.0
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            flops, _ = bench_probes.mfma_rate_probe(data, 40000)
            e1.record()
            torch.cuda.synchronize()
            best = max(best, flops / (e0.elapsed_time(e1) * 1e-3) / 1e12)
        out["mfma_tflops_" + name] = round(best, 1)
    out["note"] = "v_mfma_f32_32x32x16_f16 from registers, 256 workgroups x 8 waves, nothing else in the loop"
    return out


def cpu_baseline(torch, wl, layers_sampled=2):
    """CPU oracle on a bounded sample: `layers_sampled` attention layers + the full target head +
    acceptance + compaction of those layers; the per-step figure scales the attention part to 32 layers."""
    import numpy as np
    import oracle
    P, T = wl.P, wl.T
    S = P + T
    ks, vs, qs = [], [], []
    for l in range(layers_sampled):
        k, v = wl.cache.read_logical(l, 0, S)
        ks.append(k.cpu().numpy())
        vs.append(v.cpu().numpy())
        qs.append(wl.q[l].cpu().numpy())
    hid = wl.hidden.cpu().numpy()
    w = wl.w.cpu().numpy()
    t0 = time.perf_counter()
    for l in range(layers_sampled):
        oracle.tree_attention(qs[l], ks[l], vs[l], wl.tree.mask, P)
    t_attn = (time.perf_counter() - t0) / layers_sampled
    t0 = time.perf_counter()
    gt = oracle.argmax(oracle.lm_head(hid, w))
    t_head = time.perf_counter() - t0
    t0 = time.perf_counter()
    a, node, path = oracle.tree_accept(wl.draft_np, gt, wl.tree.positions(P), P, wl.tree.mask, wl.tree.parent)
    flat = [x.reshape(S, -1).copy() for l in range(layers_sampled) for x in (ks[l], vs[l])]
    ids = oracle.kv_compact(flat, P, path, gt)
    t_tail = time.perf_counter() - t0
    step_us = (t_attn * wl.L + t_head + t_tail) * 1e6
    return dict(value=round(step_us, 1), unit="us/step", cores=oracle.num_threads(), kind="port",
                head_and_tail_us=round((t_head + t_tail) * 1e6, 1),
                sample="%d of %d attention layers timed (x%d extrapolated) + full target head/arg-max + acceptance + compaction; "
                       "attention %.1f ms/layer, head %.1f ms" % (layers_sampled, wl.L, wl.L, t_attn * 1e3, t_head * 1e3)), (a, ids, gt)


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on one GPU; --gpus %d is not supported (nothing in it is sharded)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    from cpm.cu_amd import lib, ops
    from cpm.cu_amd.driver import VerifyStep
    lib.get()  # fails loudly without the HIP library
    torch.cuda.set_device(0)
    use_graph = not args.no_graph

    if args.traffic_probe:
        src = torch.full((256 << 20,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    wl = Workload(torch, args.workload, args.accept_depth)
    ctx_name = "%dK" % (wl.P // 1024) if wl.P % 1024 == 0 else str(wl.P)
    metric_name = "verify us/step @8B shape, %d-node tree, %s ctx" % (wl.T, ctx_name)
    wl_desc = ("%s: %d layers x (KV append + tree attention, %dq/%dkv heads, d%d, %d-token paged prefix + %d-node tree) + "
               "target head %dx%d with arg-max + tree acceptance + KV compaction"
               % (args.workload, wl.L, wl.shape["q_heads"], wl.shape["kv_heads"], wl.shape["head_dim"], wl.P, wl.T,
                  wl.shape["vocab"], wl.shape["hidden"]))
    # the head weights are kept in the library's tiled layout, as its model-level loader keeps them
    w_t = ops.tile_head_weight(wl.w)
    vs = VerifyStep(wl.cache, w_t, wl.mask, wl.parent, wl.pos, wl.P)
    # target arg-max once, to rig the draft ids for the chosen accept length
    gt = ops.lm_head_argmax(wl.hidden, w_t)
    torch.cuda.synchronize()
    wl.rig_draft(torch, gt.cpu().numpy())

    def full_step():
        vs.enqueue(wl.q, wl.k_new, wl.v_new, wl.hidden, wl.draft_ids, attn_out=wl.attn_out, splits=args.splits)

    # The 32 layers' K/V at 4K context (~150 MB) fit the 256 MB last-level cache, so replays of the step on
    # one set of pools are partly served from it.  The headline therefore rotates the timed steps over
    # KV_SETS distinct copies of the pools (step i works on copy i % KV_SETS): every pass over K/V comes
    # from HBM, as it does in a decode loop that streams the dense layers' weights in between.  Longer
    # contexts exceed the cache by themselves and use one set.
    KV_SETS = 4 if wl.P <= 8192 else 1
    caches = [wl.cache]
    if KV_SETS > 1:
        from cpm.cu_amd.kvcache import PagedKVCache
        for _ in range(KV_SETS - 1):
            c2 = PagedKVCache(wl.L, wl.cache.Hkv, wl.cache.num_pages, device="cuda", block_table=wl.cache.block_table)
            for l in range(wl.L):
                c2.k[l].copy_(wl.cache.k[l])
                c2.v[l].copy_(wl.cache.v[l])
            caches.append(c2)
    rot_steps = [vs] + [VerifyStep(c, w_t, wl.mask, wl.parent, wl.pos, wl.P) for c in caches[1:]]

    def step_on(st):
        return lambda: st.enqueue(wl.q, wl.k_new, wl.v_new, wl.hidden, wl.draft_ids, attn_out=wl.attn_out, splits=args.splits)

    ms_step, wall_ms = timed_replays(torch, [step_on(st) for st in rot_steps], args.steps, args.warmup, use_graph)
    results = [st.result() for st in rot_steps]
    a_gpu, ids_gpu = results[0]
    sets_agree = all(r[0] == a_gpu and np.array_equal(r[1], ids_gpu) for r in results)
    ms_step_warm = timed_replays(torch, full_step, max(5, args.steps // 2), 2, use_graph)[0] if KV_SETS > 1 else ms_step
    del rot_steps

    # ---- per-operator timings (same inputs, each operator alone, graph-replayed) ----
    reps = max(5, args.steps // 5)

    def attn_all_layers():  # with the KV append of the tree rows fused in, as in the step
        for l in range(wl.L):
            ops.tree_attention(wl.q[l], wl.cache, l, vs.kv_len, vs.max_kv_len, wl.mask, num_splits=args.splits, out=wl.attn_out[l],
                               k_new=wl.k_new[l], v_new=wl.v_new[l])

    HEAD_REP = 4  # several repetitions per graph, so that the graph launch itself does not dominate

    def head_only():
        for _ in range(HEAD_REP):
            ops.lm_head_argmax(wl.hidden, w_t, gt=vs.gt)

    TAIL_REP = 8  # several repetitions per graph, so that the graph launch itself does not dominate

    def accept_compact():
        for _ in range(TAIL_REP):
            vs.pred.copy_(wl.draft_ids)
            ops.tree_accept(vs.pred, vs.gt, wl.pos, vs.cache_length, wl.mask, wl.parent, best=vs.best)
            ops.kv_compact(wl.cache, vs.pred, vs.gt, vs.cache_length, vs.best, wl.T)

    # the one-call tail of verify(): the same two launches also gather the accepted hidden rows, write
    # next position ids and the packed (a, ids) result (length advance off here: the call is repeated)
    prev_hidden = torch.zeros_like(wl.hidden)
    next_pos = torch.zeros(wl.T, dtype=torch.int32, device="cuda")
    packed = torch.zeros(1 + wl.T, dtype=torch.int32, device="cuda")

    def accept_commit():
        for _ in range(TAIL_REP):
            vs.pred.copy_(wl.draft_ids)
            ops.tree_accept(vs.pred, vs.gt, wl.pos, vs.cache_length, wl.mask, wl.parent, best=vs.best)
            ops.accept_commit(wl.cache, vs.pred, vs.gt, vs.cache_length, vs.best, wl.T, hidden=wl.hidden, prev_hidden=prev_hidden,
                              next_position_ids=next_pos, result=packed)

    # rotary embedding of the tree rows: fused into the attention kernel (one table per step) against the
    # reference's order (one in-place launch per layer in front of the attention)
    inv_freq = torch.tensor((10000.0 ** (-np.arange(64, dtype=np.float64) / 64)).astype(np.float32), device="cuda")
    q_scratch = [t.clone() for t in wl.q]
    k_scratch = [t.clone() for t in wl.k_new]

    def attn_rope_fused():
        table = ops.rope_table(wl.pos, inv_freq)
        for l in range(wl.L):
            ops.tree_attention(wl.q[l], wl.cache, l, vs.kv_len, vs.max_kv_len, wl.mask, num_splits=args.splits, out=wl.attn_out[l],
                               k_new=wl.k_new[l], v_new=wl.v_new[l], rope=table)

    def attn_rope_separate():
        table = ops.rope_table(wl.pos, inv_freq)
        for l in range(wl.L):
            ops.rope_apply_(table, q_scratch[l], k_scratch[l])
            ops.tree_attention(q_scratch[l], wl.cache, l, vs.kv_len, vs.max_kv_len, wl.mask, num_splits=args.splits, out=wl.attn_out[l],
                               k_new=k_scratch[l], v_new=wl.v_new[l])

    ms_attn_warm = timed_replays(torch, attn_all_layers, reps, 2, use_graph)[0] / wl.L
    ms_attn = ms_attn_warm
    if KV_SETS > 1:  # as the headline: every pass over K/V from HBM
        def attn_cold():
            for c in caches:
                for l in range(wl.L):
                    ops.tree_attention(wl.q[l], c, l, vs.kv_len, vs.max_kv_len, wl.mask, num_splits=args.splits, out=wl.attn_out[l],
                                       k_new=wl.k_new[l], v_new=wl.v_new[l])
        ms_attn = timed_replays(torch, attn_cold, reps, 2, use_graph)[0] / (wl.L * KV_SETS)
    ms_rope_fused = timed_replays(torch, attn_rope_fused, reps, 2, use_graph)[0] / wl.L
    ms_rope_sep = timed_replays(torch, attn_rope_separate, reps, 2, use_graph)[0] / wl.L
    del q_scratch, k_scratch
    ms_commit = timed_replays(torch, accept_commit, reps, 2, use_graph)[0] / TAIL_REP
    ms_head = timed_replays(torch, head_only, reps, 2, use_graph)[0] / HEAD_REP
    ms_tail = timed_replays(torch, accept_compact, reps, 2, use_graph)[0] / TAIL_REP

    attn_tflops = wl.flops_attention_layer() / (ms_attn * 1e-3) / 1e12
    attn_gbs = wl.bytes_attention_layer() / (ms_attn * 1e-3) / 1e9
    head_gbs = wl.bytes_target_head() / (ms_head * 1e-3) / 1e9
    tail_bytes = 2 * a_gpu * 2 * wl.L * wl.shape["kv_heads"] * wl.shape["head_dim"] * 2  # compaction: a rows, read + written
    tail_gbs = tail_bytes / (ms_tail * 1e-3) / 1e9
    kernels = [
        dict(kernel="tree_attn_split_kernel+tree_attn_combine_kernel", launches_per_step=wl.L, us_per_launch=round(ms_attn * 1e3, 2),
             bound="mfma", achieved=round(attn_tflops, 2), peak=MFMA_F16_PEAK_TFLOPS, unit="TFLOP/s",
             frac=round(attn_tflops / MFMA_F16_PEAK_TFLOPS, 4), hbm_gbs=round(attn_gbs, 1), traffic=None,
             us_per_launch_one_kv_set=round(ms_attn_warm * 1e3, 2)),
        dict(kernel="head_gemm_chunked_kernel<4,4,256,2>+head_argmax_finalize_kernel", launches_per_step=1, us_per_launch=round(ms_head * 1e3, 2),
             bound="hbm", achieved=round(head_gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(head_gbs / HBM_PEAK_GBS, 4),
             traffic=None),
        dict(kernel="tree_accept_kernel+kv_compact_kernel+accepted_ids_kernel", launches_per_step=1,
             us_per_launch=round(ms_tail * 1e3, 2), bound="hbm", achieved=round(tail_gbs, 2), peak=HBM_PEAK_GBS, unit="GB/s",
             frac=round(tail_gbs / HBM_PEAK_GBS, 5), traffic=None,
             note="accepted rows read and written once in every layer's K and V: %d bytes at accept length %d; three launches of latency, "
                  "not bandwidth" % (tail_bytes, a_gpu)),
    ]
    if args.workload == "c2_verify_4k" and args.splits == 0:
        for k in kernels:
            k["traffic"] = MEASURED_TRAFFIC_KIB[k["kernel"]] * 1024
            k["traffic_unit"] = "bytes/launch"
    dominant = max(kernels, key=lambda k: k["us_per_launch"] * k["launches_per_step"])
    roofline = {k: dominant[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")}
    roofline["kernel"] = dominant["kernel"]
    roofline["us_per_launch"] = dominant["us_per_launch"]

    # ---- FR-Spec draft head (config 3 shape), reported beside the verify step ----
    from cpm.cu_amd import synth
    remap = torch.from_numpy(synth.frspec_remap(wl.shape["vocab"], wl.shape["frspec_vocab"], 0)).cuda()
    w_sub = ops.tile_head_weight(wl.w, remap)  # remap_copy fused with the re-tiling
    hid10 = wl.hidden[:10].contiguous()
    def fr_head():
        for _ in range(HEAD_REP):
            ops.frspec_head_topk(hid10, w_sub, remap, 10)
    ms_fr = timed_replays(torch, fr_head, reps, 2, use_graph)[0] / HEAD_REP
    fr_bytes = wl.shape["frspec_vocab"] * wl.shape["hidden"] * 2.0 + 10 * wl.shape["hidden"] * 2.0 + 10 * 10 * 6.0
    fr_gbs = fr_bytes / (ms_fr * 1e-3) / 1e9
    frspec = dict(kernel="head_gemm_chunked_kernel<1,2,512,2>+topk_row_kernel", us_per_call=round(ms_fr * 1e3, 2), bound="hbm",
                  achieved=round(fr_gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(fr_gbs / HBM_PEAK_GBS, 4))

    # ---- the FR-Spec head from a cold cache ----
    # Its matrix (268 MB) nearly fits the last-level cache as well, so replays on one copy are partly served
    # from it.  Here every replay walks several distinct copies, so each pass misses.
    cold = None
    draft = None
    if KV_SETS > 1:
        FR_SETS = 3
        w_subs = [w_sub] + [ops.tile_head_weight(wl.w, remap) for _ in range(FR_SETS - 1)]

        def fr_cold():
            for w in w_subs:
                ops.frspec_head_topk(hid10, w, remap, 10)
        ms_fr_cold = timed_replays(torch, fr_cold, reps, 2, use_graph)[0] / FR_SETS

        # ---- the draft side of the path: one whole draft of the FR-Spec drafter (6 rounds of 10) ----
        # Per round: the drafter layer's own attention (10 queries, mask over 10*d columns, block sliding
        # window of 1024 tokens, its own one-layer cache), the FR-Spec head with log-softmax + top-10 + id
        # map-back, and the tree bookkeeping kernel; the final top-59 + tree build at the end.  The dense
        # parts of the drafter layer (fc, projections, FFN) are not on the path and are not run; the head
        # reads a different copy of its matrix every round, as it would after their weights.
        from cpm.cu_amd.kvcache import PagedKVCache
        k_it, n_it = 10, 6
        dtree = ops.DraftTree(k_it, n_it, remap)
        dcache = PagedKVCache(1, wl.cache.Hkv, wl.cache.num_pages, device="cuda", block_table=wl.cache.block_table)
        dcache.k[0].copy_(wl.cache.k[0])
        dcache.v[0].copy_(wl.cache.v[0])
        hid1 = wl.hidden[:1].contiguous()
        qd = wl.q[0][:k_it].contiguous()
        kd = wl.k_new[0][:k_it].contiguous()
        vd = wl.v_new[0][:k_it].contiguous()
        d_len = [torch.tensor([wl.P + k_it * d], dtype=torch.int32, device="cuda") for d in range(n_it)]
        d_out = torch.empty_like(qd)
        tree_ids = torch.full((wl.T,), -1, dtype=torch.int32, device="cuda")

        def draft_path():
            r = ops.frspec_head_topk(hid1, w_subs[0], remap, k_it)
            dtree.begin(r["val"][0], r["pos"][0])
            for d in range(1, n_it):
                ops.tree_attention(qd, dcache, 0, d_len[d], vs.max_kv_len, dtree.draft_mask, out=d_out, k_new=kd, v_new=vd,
                                   mask_k_range=k_it * d, block_window_size=1024)
                r = ops.frspec_head_topk(hid10, w_subs[d % FR_SETS], remap, k_it)
                dtree.extend(d, r["val"], r["pos"])
            dtree.finish(wl.T, vs.cache_length, tree_draft_ids=tree_ids)
        ms_draft = timed_replays(torch, draft_path, reps, 2, use_graph)[0]
        draft = {"us_per_draft": round(ms_draft * 1e3, 1), "rounds": n_it, "topk_per_round": k_it, "tree_size": wl.T,
                 "operators": "6 x (FR-Spec head + log-softmax + top-10 + id map-back) + 5 x drafter-layer attention "
                              "(window 1024) + tree bookkeeping (begin, 5 x extend, finish)"}
        del w_subs, dcache, dtree
        cold = {"frspec_head_us_per_call": round(ms_fr_cold * 1e3, 2), "frspec_weight_copies_rotated": FR_SETS,
                "frspec_frac_hbm": round(fr_bytes / (ms_fr_cold * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "note": "the FR-Spec head with every replay walking distinct copies of its matrix, so that no pass is served "
                        "from the 256 MB last-level cache; frspec_head above replays one copy"}
    del w_sub, caches
    torch.cuda.empty_cache()

    # ---- CPU oracle on the host cores + parity of the step's integer results ----
    cpu = None
    parity = None
    if not args.no_cpu_baseline:
        import oracle
        cpu, (a_cpu, ids_cpu, gt_cpu) = cpu_baseline(torch, wl)
        gt_gpu = vs.gt.cpu().numpy()
        a_st, _, path_st = oracle.tree_accept(wl.draft_np, gt_gpu, wl.tree.positions(wl.P), wl.P, wl.tree.mask, wl.tree.parent)
        parity = dict(accept_length_gpu=a_gpu, accept_length_oracle=int(a_cpu),
                      ids_equal_oracle=bool(a_gpu == a_cpu and np.array_equal(ids_gpu, ids_cpu)),
                      staged_equal=bool(a_gpu == a_st and np.array_equal(ids_gpu, gt_gpu[path_st])),
                      kv_sets_agree=bool(sets_agree),
                      argmax_rows_equal=int((gt_gpu == gt_cpu).sum()), rows=int(wl.T))

    # ---- the same step at longer contexts ----
    contexts = {str(wl.P): round(ms_step * 1e3, 1)}
    ctx_attn = {str(wl.P): round(ms_attn * 1e3, 2)}
    if not args.no_contexts and args.workload == "c2_verify_4k":
        w_keep, hid_keep = wl.w, wl.hidden
        del vs, wl
        torch.cuda.empty_cache()
        for name in ("c4_verify_32k", "c4_verify_128k"):
            w2 = Workload.__new__(Workload)
            Workload.__init__(w2, torch, name, args.accept_depth)
            w2.w, w2.hidden = w_keep, hid_keep  # same head
            v2 = VerifyStep(w2.cache, w_t, w2.mask, w2.parent, w2.pos, w2.P)
            w2.rig_draft(torch, gt.cpu().numpy())
            n = max(3, args.steps // 5)
            ms2 = timed_replays(torch, lambda: v2.enqueue(w2.q, w2.k_new, w2.v_new, w2.hidden, w2.draft_ids, attn_out=w2.attn_out,
                                                          splits=args.splits), n, 2, use_graph)[0]

            def attn2():
                for l in range(w2.L):
                    ops.tree_attention(w2.q[l], w2.cache, l, v2.kv_len, v2.max_kv_len, w2.mask, num_splits=args.splits, out=w2.attn_out[l],
                                       k_new=w2.k_new[l], v_new=w2.v_new[l])
            ms_a2 = timed_replays(torch, attn2, n, 2, use_graph)[0] / w2.L
            contexts[str(w2.P)] = round(ms2 * 1e3, 1)
            tf2 = w2.flops_attention_layer() / (ms_a2 * 1e-3) / 1e12
            ctx_attn[str(w2.P)] = dict(us_per_layer=round(ms_a2 * 1e3, 2), tflops=round(tf2, 1),
                                       frac_mfma=round(tf2 / MFMA_F16_PEAK_TFLOPS, 4))
            if cpu is not None:
                # the CPU oracle on ONE layer of this context (bounded sample), extrapolated to the step with the
                # head and tail times of the 4K sample
                import oracle
                S2 = w2.P + w2.T
                k2, v2k = w2.cache.read_logical(0, 0, S2)
                k2, v2k, q2 = k2.cpu().numpy(), v2k.cpu().numpy(), w2.q[0].cpu().numpy()
                t0 = time.perf_counter()
                oracle.tree_attention(q2, k2, v2k, w2.tree.mask, w2.P)
                t_layer = time.perf_counter() - t0
                cpu.setdefault("contexts", {})[str(w2.P)] = dict(
                    attention_ms_per_layer=round(t_layer * 1e3, 1),
                    us_per_step_extrapolated=round(t_layer * 1e6 * w2.L + cpu["head_and_tail_us"], 1),
                    sample="1 of %d attention layers timed once" % w2.L)
                del k2, v2k, q2
            del v2, w2
            torch.cuda.empty_cache()

    # ---- what the matrix pipes sustain on this GPU (last, so that its heat does not touch the figures above) ----
    probes = None if args.no_probes else machine_probes(torch)
    if probes is not None:
        ceiling = probes["mfma_tflops_random_operands"]
        if roofline["bound"] == "mfma":  # the same achieved figure against MFMAs alone on random operands
            roofline["measured_ceiling"] = ceiling
            roofline["frac_of_measured_ceiling"] = round(roofline["achieved"] / ceiling, 4)
        for v in ctx_attn.values():
            if isinstance(v, dict):
                v["frac_of_measured_ceiling"] = round(v["tflops"] / ceiling, 4)

    out = {
        "metric": metric_name,
        "value": round(ms_step * 1e3, 1),
        "unit": "us/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": wl_desc, "batch": 1, "graph_replay": use_graph, "kv_splits": args.splits or "auto", "kv_sets_rotated": KV_SETS},
        "wall_ms_per_step": round(wall_ms, 5),
        "us_per_step_one_kv_set": round(ms_step_warm * 1e3, 1),
        "roofline": roofline,
        "machine_probes": probes,
        "kernels": kernels,
        "frspec_head": frspec,
        "cold_cache": cold,
        "draft_path": draft,
        "attention_with_rope": {"fused_us_per_layer": round(ms_rope_fused * 1e3, 2), "separate_launch_us_per_layer": round(ms_rope_sep * 1e3, 2),
                                "note": "rotary embedding of q and the appended K rows; table computed once per step"},
        "commit_tail": {"kernel": "tree_accept_kernel+kv_compact_kernel(with hidden-row gather)+accepted_ids_kernel(ids, positions, packed result)",
                        "us_per_call": round(ms_commit * 1e3, 2)},
        "contexts_us_per_step": contexts,
        "attention_by_context": ctx_attn,
        "cpu_baseline": cpu,
        "parity": parity,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
