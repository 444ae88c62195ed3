#!/usr/bin/env python3
"""Benchmark of the speculative-decoding verify step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2_verify_4k]

One "step" = one pass of the verify hot path over one batch of synthetic MiniCPM4-8B-shaped input, with every
input already resident in HBM: for each of the 32 layers append the 60 tree rows' K/V and run tree-masked attention
over the paged cache (4096-token prefix + 60 tree rows), then the target lm_head (73448 x 4096) with its arg-max,
greedy tree acceptance and accepted-path KV compaction in all layers.

The step runs where a user of the library runs it: on the library's own storage (`cpmcu_init_storage` pools, the
loaded lm_head) through `cpmcu_verify_step` with the library's own HIP graph (captured once per padded length, as
the reference captures decode, src/entry.cu:475-492) on the library's stream.  Exactly K graph launches are timed
with events on that stream.  At 4K context the K/V of all layers would fit the 256 MB last-level cache, so the timed
steps rotate over four distinct sets of K/V pages of the same pools (four page tables, one graph each): every pass
over K/V comes from HBM.  The time of replays on a single set is reported beside it (`us_per_step_one_kv_set`).

Prints ONE JSON line.  `value` is microseconds per step (lower is better).  `roofline` is for the kernel that takes
the largest share of the step; `kernels` lists all of them (names as reported by the library for the dispatch
actually taken); `contexts_us_per_step` gives the step at 4K / 32K / 128K context; `cpu_baseline` is the CPU oracle
timed on this host on a bounded sample of the same workload (a reported baseline only).
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0

# HBM bytes per launch on c2_verify_4k with the automatic split count, from rocprofv3's FETCH_SIZE and WRITE_SIZE
# counters (KiB per dispatch, one counter per run, eager launches), each scaled by what the same counter read for a
# plain 256 MiB copy (x2.000 and x1.000): the table and the two commands are in profiles/verify_step_hbm_traffic.md.
# Counters cannot be read from inside this process, so the figures are carried here as constants, keyed by the kernel
# names the library reports for the dispatch taken: a different instantiation finds no entry and reports null.
MEASURED_TRAFFIC = {
    "source": "profiles/verify_step_hbm_traffic.md, profiles/tree_attention_long_context_traffic.md",
    # the library the counters were read on (git rev-parse --short HEAD of that run, all figures)
    "measured_at_commit": "5ad0aba",
    "kib_per_launch": {
        "tree_attn_split_kernel<2,false>": 15185 + 9463,  # the merge of the split partials runs inside the launch
        "head_gemm_stream_kernel<4,2,256>": 591978 + 128,
    },
    # the attention launch at the longer contexts (32 splits of 256-row workgroups), by prefix length
    "attention_kib_per_launch_by_context": {"32768": 52487 + 17894, "131072": 150806 + 17894},
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2_verify_4k")
    ap.add_argument("--no-contexts", action="store_true", help="skip the 32K / 128K context step timings")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="enqueue the step's launches eagerly instead of replaying the library's HIP graph")
    ap.add_argument("--no-probes", action="store_true", help="skip the MFMA-rate probe of the machine and the power probe of the attention launch")
    ap.add_argument("--no-operators", action="store_true", help="skip the per-operator timings (heads, tail, draft path)")
    ap.add_argument("--accept-depth", type=int, default=3, help="draft tokens the rigged tree gets accepted")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run a plain 256 MiB device copy three times: the known-size kernel that scales "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    return ap.parse_args()


WARM_MS = 40.0  # operator timings first replay for this long: clocks settle over tens of milliseconds after a change of kernel mix


def timed_torch(torch, fn, steps, warmup, use_graph=True, warm_ms=0.0):
    """Operator timings on a torch side stream: fn() captured once into a graph (unless disabled), `warmup` untimed calls
    (and further ones until warm_ms have passed) and exactly `steps` timed calls between two events on that stream.
    fn may be a list: the calls cycle through it."""
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
        t_w = time.perf_counter()
        while (time.perf_counter() - t_w) * 1e3 < warm_ms:
            for i in range(len(runs)):
                runs[i]()
            stream.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        for i in range(steps):
            runs[i % len(runs)]()
        e1.record(stream)
        stream.synchronize()
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


class StepBuffers:
    """The static input / output buffers of the verify step, as cpmcu/llm.py keeps them for the reference."""

    def __init__(self, torch, L, T, Hq, Hkv, D, H, gen):
        dev = "cuda"
        rn = lambda *s: torch.randn(*s, device=dev, dtype=torch.float32, generator=gen).to(torch.float16)
        self.q = [rn(T, Hq, D) for _ in range(L)]
        self.k_new = [rn(T, Hkv, D) for _ in range(L)]
        self.v_new = [rn(T, Hkv, D) for _ in range(L)]
        self.attn_out = [torch.empty(T, Hq, D, dtype=torch.float16, device=dev) for _ in range(L)]
        self.hidden = rn(T, H)
        self.draft_ids = torch.zeros(T, dtype=torch.int32, device=dev)
        self.accepted = torch.zeros(T, dtype=torch.int32, device=dev)
        self.gt = torch.zeros(T, dtype=torch.int32, device=dev)
        self.result = torch.zeros(1 + T, dtype=torch.int32).pin_memory()  # (a, ids): written by the GPU


def run_context(torch, np, model, synth, oracle_mod, args, name, bufs, tree, use_graph, kv_sets, gen, want_cpu):
    """The verify step of one configuration on the library's storage: fills the pools, captures / replays the
    library's graph(s), times K launches on the library's stream, checks the integer results against the oracle."""
    from cpm.cu_amd import ops
    cfg = dict(synth.CONFIGS[name])
    shp = synth.MINICPM4_8B
    L, P, T = cfg["layers"], cfg["prefix"], cfg["T"]
    Hq, Hkv = shp["q_heads"], shp["kv_heads"]
    S = P + T
    npages = (S + 255) // 256 + 1
    assert kv_sets * npages <= model.num_pages, "the library's pools are too small for %s" % name
    # page tables: set i lives in physical pages [i * npages, (i + 1) * npages), permuted by a seeded permutation
    tables = []
    for i in range(kv_sets):
        perm = synth.rng(cfg["seed"], 4 + i).permutation(npages).astype(np.int32) + i * npages
        tables.append(torch.from_numpy(perm).cuda())
    for l in range(L):  # ~N(0,1) K/V, written in the pools' own layout
        model._k[l][: kv_sets * npages].normal_(generator=gen)
        model._v[l][: kv_sets * npages].normal_(generator=gen)
    mask = torch.from_numpy(tree.mask.view(np.int64)).cuda()
    parent = torch.from_numpy(tree.parent).cuda()
    pos = torch.from_numpy(tree.positions(P)).cuda()
    clen = torch.tensor([P], dtype=torch.int32, device="cuda")
    kvlen = torch.tensor([S], dtype=torch.int32, device="cuda")
    padded = (S + 127) // 128 * 128  # padded_length, cpmcu/llm.py:273
    torch.cuda.synchronize()

    def step(i):
        model.verify_step(T, padded, bufs.q, bufs.k_new, bufs.v_new, bufs.attn_out, bufs.hidden, bufs.draft_ids, pos, clen, kvlen,
                          mask, parent, bufs.accepted, gt_out=bufs.gt, result=bufs.result, block_table=tables[i % kv_sets],
                          cuda_graph=use_graph)

    # target arg-max once (through the step itself), to rig the draft ids for the chosen accept length
    step(0)
    model.synchronize()
    gt_np = bufs.gt.cpu().numpy()
    depth = min(args.accept_depth, int(tree.depth.max()))
    draft_np, leaf = synth.draft_ids_for_accept(tree, gt_np, depth, shp["vocab"], 1)
    bufs.draft_ids.copy_(torch.from_numpy(draft_np).cuda())
    torch.cuda.synchronize()

    stream = model.stream()

    def timed(steps, warmup, sets):
        for i in range(max(warmup, sets)):  # every graph is captured (and launched once) before the timed region
            step(i % sets)
        model.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for i in range(steps):
            step(i % sets)
        e1.record(stream)
        model.synchronize()
        wall = (time.perf_counter() - t0) * 1e3
        return e0.elapsed_time(e1) / steps, wall / steps

    results = []
    for i in range(kv_sets):
        step(i)
        model.synchronize()
        a = int(bufs.result[0])
        results.append((a, bufs.result[1:1 + a].numpy().copy()))
    steps = args.steps if name == args.workload else max(10, args.steps // 5)
    ms_step, wall_ms = timed(steps, args.warmup, kv_sets)
    ms_one = timed(max(5, steps // 2), 2, 1)[0] if kv_sets > 1 else ms_step

    out = dict(name=name, P=P, T=T, L=L, ms_step=ms_step, wall_ms=wall_ms, ms_one_set=ms_one, steps=steps, results=results,
               draft_np=draft_np, gt_np=gt_np, tables=tables, padded=padded, mask=mask, parent=parent, pos=pos, clen=clen,
               kvlen=kvlen, npages=npages)
    caches = [model.cache(block_table=t) for t in tables]
    # what the last step left at rows [P, P + a) of layer 0 and of the last layer (the attention-alone timing below
    # appends the tree rows again)
    a0 = results[0][0]
    out["compacted"] = {l: tuple(t.cpu().numpy().reshape(a0, -1) for t in caches[0].read_logical(l, P, a0)) for l in (0, L - 1)}

    # attention alone: 32 layers on the same pools (operator level, torch side stream), every K/V pass from HBM

    def attn_all():
        for c in caches:
            for l in range(L):
                ops.tree_attention(bufs.q[l], c, l, kvlen, padded, mask, out=bufs.attn_out[l], k_new=bufs.k_new[l], v_new=bufs.v_new[l])
    reps = max(10, steps // 5)  # >= 320 timed launches per figure
    out["ms_attn"] = timed_torch(torch, attn_all, reps, 2) / (L * kv_sets)
    if kv_sets > 1:
        def attn_one():
            for l in range(L):
                ops.tree_attention(bufs.q[l], caches[0], l, kvlen, padded, mask, out=bufs.attn_out[l], k_new=bufs.k_new[l], v_new=bufs.v_new[l])
        out["ms_attn_one_set"] = timed_torch(torch, attn_one, reps, 2) / L
    else:
        out["ms_attn_one_set"] = out["ms_attn"]
    out["attn_plan"] = ops.attention_plan(T, Hq, Hkv, padded)
    out["caches"] = caches

    # the CPU oracle on a bounded sample of this context: one attention layer, 1 warm-up + median of 3
    if want_cpu:
        k_all, v_all = caches[0].read_logical(0, 0, S)
        k_np, v_np, q_np = k_all.cpu().numpy(), v_all.cpu().numpy(), bufs.q[0].cpu().numpy()
        del k_all, v_all
        times = []
        for rep in range(4):
            t0 = time.perf_counter()
            oracle_mod.tree_attention(q_np, k_np, v_np, tree.mask, P)
            times.append(time.perf_counter() - t0)
        out["cpu_attn_s"] = statistics.median(times[1:])
    return out


def context_parity(np, oracle_mod, run, bufs, tree):
    """The integer results of one context's step against the oracle: acceptance on the device's own arg-max
    (accept length, ids), and the compacted rows of the first and the last layer against the oracle's path."""
    P, T = run["P"], run["T"]
    a_gpu, ids_gpu = run["results"][0]
    gt_gpu = run["gt_np"]
    a_st, _, path_st = oracle_mod.tree_accept(run["draft_np"], gt_gpu, tree.positions(P), P, tree.mask, tree.parent)
    rows_ok = a_gpu == len(path_st)
    for l, (kd_, vd_) in run["compacted"].items():
        kn, vn = bufs.k_new[l].cpu().numpy().reshape(T, -1), bufs.v_new[l].cpu().numpy().reshape(T, -1)
        rows_ok = bool(rows_ok and np.array_equal(kd_, kn[path_st]) and np.array_equal(vd_, vn[path_st]))
    return dict(accept_length_gpu=int(a_gpu), accept_length_oracle=int(a_st),
                ids_equal_oracle=bool(a_gpu == a_st and np.array_equal(ids_gpu, gt_gpu[path_st])),
                compacted_rows_equal=rows_ok,
                kv_sets_agree=bool(all(r[0] == a_gpu and np.array_equal(r[1], ids_gpu) for r in run["results"])))


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


def power_probe(torch, np, synth, seconds=0.6):
    """The tree-attention launch at 32K and 128K context on all-zero and on random Q/K/V, with the board power read
    from the driver's hwmon file (every 20 ms) while the launches run: the time of the same launch depends on the
    data, and the board's power limit is why.  Four layers' pools per context, replayed as one graph."""
    import glob
    import threading
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    files = []
    for h in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
        for f in ("power1_average", "power1_input"):
            if os.path.exists(os.path.join(h, f)):
                files.append(os.path.join(h, f))
    cap = None
    for h in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
        if os.path.exists(os.path.join(h, "power1_cap")):
            try:
                cap = int(open(os.path.join(h, "power1_cap")).read()) / 1e6
            except (OSError, ValueError):
                pass
            break
    shp = synth.MINICPM4_8B
    T, Hq, Hkv, D, L = 60, shp["q_heads"], shp["kv_heads"], shp["head_dim"], 4
    tree = synth.eagle_tree(6, 10, T, 0)
    mask = torch.from_numpy(tree.mask.view(np.int64)).cuda()
    out = {"power_file": files[0] if files else None, "power_cap_w": cap, "layers_per_graph": L, "contexts": {}}
    for P in (32768, 131072):
        S = P + T
        cache = PagedKVCache(L, Hkv, (S + 255) // 256 + 1)
        kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
        padded = (S + 127) // 128 * 128
        row = {}
        for mode in ("zeros", "random"):
            for l in range(L):
                if mode == "zeros":
                    cache.k[l].zero_()
                    cache.v[l].zero_()
                else:
                    cache.k[l].normal_()
                    cache.v[l].normal_()
            q = torch.zeros(T, Hq, D, device="cuda").half() if mode == "zeros" else torch.randn(T, Hq, D, device="cuda").half()
            o = torch.empty_like(q)
            call = lambda l: ops.tree_attention(q, cache, l, kv_len, padded, mask, out=o)
            call(0)
            torch.cuda.synchronize()
            st = torch.cuda.Stream()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(st):
                with torch.cuda.graph(g, stream=st):
                    for l in range(L):
                        call(l)
            samples, stop = [], [False]

            def sampler():
                while not stop[0]:
                    if files:
                        try:
                            samples.append(int(open(files[0]).read()) / 1e6)
                        except (OSError, ValueError):
                            pass
                    time.sleep(0.02)
            th = threading.Thread(target=sampler)
            th.start()
            n = max(20, int(seconds * 1e6 / (150.0 * L * P / 131072 + 15 * L)))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            with torch.cuda.stream(st):
                for _ in range(n // 4):
                    g.replay()
                e0.record(st)
                for _ in range(n):
                    g.replay()
                e1.record(st)
            torch.cuda.synchronize()
            stop[0] = True
            th.join()
            us = e0.elapsed_time(e1) * 1e3 / (n * L)
            tail = sorted(samples[len(samples) // 2:]) if samples else []
            row[mode] = {"us_per_layer": round(us, 2), "tflops": round(4.0 * Hq * T * D * S / us / 1e6, 1),
                         "board_power_w_median": round(tail[len(tail) // 2], 0) if tail else None,
                         "board_power_w_max": round(max(samples), 0) if samples else None, "power_samples": len(samples)}
            del g
        out["contexts"][str(P)] = row
        del cache
        torch.cuda.empty_cache()
    out["note"] = ("the same attention launch on all-zero and on random fp16 data; power is the driver's reading over the second half of "
                   "the run; a zero in every operand draws less, so the clock stays higher")
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this path is measured on one GPU; --gpus %d is not supported (nothing in it is sharded)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    from cpm.cu_amd import synth
    if args.workload not in synth.CONFIGS:
        sys.exit("bench.py: unknown workload %s (one of %s)" % (args.workload, ", ".join(synth.CONFIGS)))
    import numpy as np
    import torch
    from cpm.cu_amd import lib, ops, synth
    from cpm.cu_amd.model import PathModel
    lib.get()  # fails loudly without the HIP library
    torch.cuda.set_device(0)
    use_graph = not args.no_graph
    want_cpu = not args.no_cpu_baseline
    oracle_mod = None
    if want_cpu:
        import oracle as oracle_mod

    if args.traffic_probe:
        src = torch.full((256 << 20,), 7, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    shp = synth.MINICPM4_8B
    cfg = dict(synth.CONFIGS[args.workload])
    L, T = cfg["layers"], cfg["T"]
    Hq, Hkv, D, H, V = shp["q_heads"], shp["kv_heads"], shp["head_dim"], shp["hidden"], shp["vocab"]
    names = [args.workload]
    if not args.no_contexts and args.workload == "c2_verify_4k":
        names += ["c4_verify_32k", "c4_verify_128k"]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(cfg["seed"])

    # ---- the library's model: heads + paged pools sized for the longest context of this run ----
    kv_sets_of = lambda n: 4 if synth.CONFIGS[n]["prefix"] <= 8192 else 1
    pages_needed = max(kv_sets_of(n) * ((synth.CONFIGS[n]["prefix"] + synth.CONFIGS[n]["T"] + 255) // 256 + 1) for n in names)
    page_bytes_all_layers = (L + 1) * 2 * Hkv * 256 * D * 2  # target layers + the drafter's one layer, K and V
    total_mem = torch.cuda.mem_get_info()[1]
    want_bytes = pages_needed * page_bytes_all_layers * 1.15 + 3 * V * H * 2 + (1 << 30)
    memory_limit = min(0.9, want_bytes / total_mem)
    w_dev = (torch.randn(V, H, device="cuda", dtype=torch.float32, generator=gen) * 0.02).to(torch.float16)
    w_host = w_dev.cpu().numpy()
    remap_np = synth.frspec_remap(V, shp["frspec_vocab"], 0)
    # the drafter's masks have 64 bits, as the reference's: top-k x rounds <= 64 columns, trees of up to 64 nodes.  A wider tree
    # (config 5) is synthetic on the verify side, and the draft side is timed with as many rounds of its top-k as fit.
    draft_rounds = min(cfg["num_iter"], 64 // cfg["topk"])
    model = PathModel(V, L, H, Hq, Hkv, memory_limit=memory_limit, scale_lmhead=1.0, frspec_vocab=shp["frspec_vocab"], tree_size=T,
                      num_iter=draft_rounds, topk=cfg["topk"], draft_layers=1, eagle_window=1024)
    assert model.num_pages >= pages_needed, (model.num_pages, pages_needed)
    model.load_head(w_host, remap_np)
    bufs = StepBuffers(torch, L, T, Hq, Hkv, D, H, gen)
    tree = synth.eagle_tree(cfg["num_iter"], cfg["topk"], T, cfg["seed"])

    main_run = run_context(torch, np, model, synth, oracle_mod, args, args.workload, bufs, tree, use_graph,
                           kv_sets_of(args.workload), gen, want_cpu)
    P = main_run["P"]
    ms_step, ms_attn = main_run["ms_step"], main_run["ms_attn"]
    a_gpu, ids_gpu = main_run["results"][0]
    sets_agree = all(r[0] == a_gpu and np.array_equal(r[1], ids_gpu) for r in main_run["results"])
    ctx_name = "%dK" % (P // 1024) if P % 1024 == 0 else str(P)
    metric_name = "verify us/step @8B shape, %d-node tree, %s ctx" % (T, ctx_name)
    wl_desc = ("%s: %d layers x (KV append + tree attention, %dq/%dkv heads, d%d, %d-token paged prefix + %d-node tree) + "
               "target head %dx%d with arg-max + tree acceptance + KV compaction, on the library's storage through "
               "cpmcu_verify_step" % (args.workload, L, Hq, Hkv, D, P, T, V, H))

    flops_attn = lambda Pc: 4.0 * Hq * T * D * (Pc + T)
    bytes_attn = lambda Pc: 2.0 * (Pc + T) * Hkv * D * 2 + 2.0 * T * Hq * D * 2
    bytes_head = V * H * 2.0 + T * H * 2.0 + T * 4.0

    # ---- per-operator timings on the main workload (operator level, same pools and buffers, graph-replayed) ----
    kernels, frspec, cold, draft, rope_cmp, bf16 = [], None, None, None, None, None
    attn_tflops = flops_attn(P) / (ms_attn * 1e-3) / 1e12
    attn_name = main_run["attn_plan"][0]
    kernels.append(dict(kernel=attn_name, launches_per_step=L, us_per_launch=round(ms_attn * 1e3, 2), bound="mfma",
                        achieved=round(attn_tflops, 2), peak=MFMA_F16_PEAK_TFLOPS, unit="TFLOP/s",
                        frac=round(attn_tflops / MFMA_F16_PEAK_TFLOPS, 4),
                        hbm_gbs=round(bytes_attn(P) / (ms_attn * 1e-3) / 1e9, 1), traffic=None,
                        kv_splits=main_run["attn_plan"][1], workgroups=main_run["attn_plan"][3],
                        us_per_launch_one_kv_set=round(main_run["ms_attn_one_set"] * 1e3, 2)))
    if not args.no_operators:
        reps = max(5, args.steps // 5)
        w_t = ops.tile_head_weight(w_dev)  # the layout the library's loader keeps
        cache0 = main_run["caches"][0]
        mask, parent, pos, clen, kvlen, padded = (main_run[k] for k in ("mask", "parent", "pos", "clen", "kvlen", "padded"))
        HEAD_REP, TAIL_REP = 4, 8  # several repetitions per graph, so that the graph launch itself does not dominate
        head_name = ops.head_plan(T, w_t)[0]

        def timed_model(fn, n_rep):
            """fn(): model-level calls, recorded into a library graph and replayed on the library's stream."""
            gid = model.capture(fn)
            st_ = model.stream()
            t_w = time.perf_counter()
            while (time.perf_counter() - t_w) * 1e3 < WARM_MS:  # (the first replays run at ramping clocks)
                model.replay(gid)
                model.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(st_)
            for _ in range(n_rep):
                model.replay(gid)
            e1.record(st_)
            model.synchronize()
            return e0.elapsed_time(e1) / n_rep

        # the target head on the library's own copy of the weights (cpmcu_decode_lm_head: GEMM + arg-max finish)
        def head_model():
            for _ in range(HEAD_REP):
                model.L.decode_lm_head(T, bufs.hidden.data_ptr(), 0, bufs.gt.data_ptr())
        ms_head_model = timed_model(head_model, reps) / HEAD_REP

        def head_only():  # the GEMM alone, on a separately allocated copy of the tiled weights
            for _ in range(HEAD_REP):
                ops.lm_head_partials(bufs.hidden, w_t)
        ms_head = timed_torch(torch, head_only, reps, 2, warm_ms=WARM_MS) / HEAD_REP
        # the same GEMM where the step has it, behind the 32 attention launches (every K/V set in turn): replays of the head
        # alone keep HBM at its limit without a pause, and the head then runs slower than it does inside a step
        all_caches = main_run["caches"]

        def attn_layers(c):
            for l in range(L):
                ops.tree_attention(bufs.q[l], c, l, kvlen, padded, mask, out=bufs.attn_out[l], k_new=bufs.k_new[l], v_new=bufs.v_new[l])

        def attn_then_head():
            for c in all_caches:
                attn_layers(c)
                ops.lm_head_partials(bufs.hidden, w_t)

        def attn_without_head():
            for c in all_caches:
                attn_layers(c)
        ms_head_in_step = (timed_torch(torch, attn_then_head, reps, 2, warm_ms=WARM_MS) -
                           timed_torch(torch, attn_without_head, reps, 2, warm_ms=WARM_MS)) / len(all_caches)
        parts = ops.lm_head_partials(bufs.hidden, w_t)
        best = torch.zeros(2, dtype=torch.int32, device="cuda")
        path = torch.zeros(T, dtype=torch.int32, device="cuda")

        def tail_only():  # arg-max finish + acceptance + compaction + ids in one launch
            for _ in range(TAIL_REP):
                ops.verify_tail(cache0, bufs.draft_ids, parts, pos, clen, mask, parent, gt_out=bufs.gt, best=best, path=path,
                                accepted_ids=bufs.accepted)
        ms_tail = timed_torch(torch, tail_only, reps, 2, warm_ms=WARM_MS) / TAIL_REP
        head_gbs = bytes_head / (ms_head * 1e-3) / 1e9
        head_tail_gbs = bytes_head / ((ms_head + ms_tail) * 1e-3) / 1e9
        tail_bytes = 2 * a_gpu * 2 * L * Hkv * D * 2  # compaction: a rows, read + written, in every K and V cache
        head_model_gbs = bytes_head / (ms_head_model * 1e-3) / 1e9
        kernels.append(dict(kernel=head_name, launches_per_step=1, us_per_launch=round(ms_head * 1e3, 2), bound="hbm",
                            achieved=round(head_gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(head_gbs / HBM_PEAK_GBS, 4), traffic=None,
                            frac_with_tail_launch=round(head_tail_gbs / HBM_PEAK_GBS, 4),
                            us_behind_attention=round(ms_head_in_step * 1e3, 2),
                            frac_behind_attention=round(bytes_head / (ms_head_in_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                            note="the target head's GEMM on a separately allocated copy of the weights, replayed back to back "
                                 "(us_per_launch, frac) and where the step has it (us_behind_attention: a graph of the %d attention "
                                 "launches + the GEMM minus the same graph without it, over every K/V set); in the step its arg-max is "
                                 "finished inside the tail launch (frac_with_tail_launch charges that whole launch -- acceptance and "
                                 "compaction included -- to the back-to-back figure)" % L))
        kernels.append(dict(kernel=head_name + "+head_argmax_finalize_kernel", launches_per_step=0, us_per_launch=round(ms_head_model * 1e3, 2),
                            bound="hbm", achieved=round(head_model_gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                            frac=round(head_model_gbs / HBM_PEAK_GBS, 4), traffic=None,
                            note="the target head with its arg-max as an operator of its own (cpmcu_decode_lm_head on the library's "
                                 "weights, two launches); not part of the step, which finishes the arg-max in its tail"))
        kernels.append(dict(kernel="verify_tail_kernel", launches_per_step=1, us_per_launch=round(ms_tail * 1e3, 2), bound="hbm",
                            achieved=round(tail_bytes / (ms_tail * 1e-3) / 1e9, 2), peak=HBM_PEAK_GBS, unit="GB/s",
                            frac=round(tail_bytes / (ms_tail * 1e-3) / 1e9 / HBM_PEAK_GBS, 5), traffic=None,
                            note="arg-max finish + acceptance + compaction of %d bytes at accept length %d + ids: one launch of latency, "
                                 "not bandwidth" % (tail_bytes, a_gpu)))

        # rotary embedding of the tree rows: fused into the attention kernel (one table per step) against the reference's
        # order (one in-place launch per layer in front of the attention)
        inv_freq = torch.tensor((10000.0 ** (-np.arange(64, dtype=np.float64) / 64)).astype(np.float32), device="cuda")
        q_scratch = [t.clone() for t in bufs.q]
        k_scratch = [t.clone() for t in bufs.k_new]

        def attn_rope_fused():
            table = ops.rope_table(pos, inv_freq)
            for l in range(L):
                ops.tree_attention(bufs.q[l], cache0, l, kvlen, padded, mask, out=bufs.attn_out[l], k_new=bufs.k_new[l],
                                   v_new=bufs.v_new[l], rope=table)

        def attn_rope_separate():
            table = ops.rope_table(pos, inv_freq)
            for l in range(L):
                ops.rope_apply_(table, q_scratch[l], k_scratch[l])
                ops.tree_attention(q_scratch[l], cache0, l, kvlen, padded, mask, out=bufs.attn_out[l], k_new=k_scratch[l],
                                   v_new=bufs.v_new[l])
        rope_cmp = {"fused_us_per_layer": round(timed_torch(torch, attn_rope_fused, reps, 2) / L * 1e3, 2),
                    "separate_launch_us_per_layer": round(timed_torch(torch, attn_rope_separate, reps, 2) / L * 1e3, 2),
                    "note": "rotary embedding of q and the appended K rows; table computed once per step; one K/V set"}
        del q_scratch, k_scratch

        # ---- FR-Spec draft head (config 3 shape) ----
        remap = torch.from_numpy(remap_np).cuda()
        FR_SETS = 3
        w_subs = [ops.tile_head_weight(w_dev, remap) for _ in range(FR_SETS)]  # remap_copy fused with the re-tiling
        hid10 = bufs.hidden[:10].contiguous()
        fr_name = ops.frspec_head_plan(10, w_subs[0], 10)

        def fr_head():
            for _ in range(HEAD_REP):
                ops.frspec_head_topk(hid10, w_subs[0], remap, 10)
        ms_fr = timed_torch(torch, fr_head, reps, 2, warm_ms=WARM_MS) / HEAD_REP
        fr_bytes = shp["frspec_vocab"] * H * 2.0 + 10 * H * 2.0 + 10 * 10 * 6.0
        fr_gbs = fr_bytes / (ms_fr * 1e-3) / 1e9
        frspec = dict(kernel=fr_name, us_per_call=round(ms_fr * 1e3, 2), bound="hbm", achieved=round(fr_gbs, 1), peak=HBM_PEAK_GBS,
                      unit="GB/s", frac=round(fr_gbs / HBM_PEAK_GBS, 4))

        # the same call as ONE launch (option frspec_fused: every GEMM workgroup publishes its best keys per row as tagged
        # words, the first workgroups to finish rank a row each), which is no faster and therefore not the default
        lib.get().set_option(b"frspec_fused", 1)
        frspec["one_launch_kernel"] = ops.frspec_head_plan(10, w_subs[0], 10)
        frspec["one_launch_us_per_call"] = round(timed_torch(torch, fr_head, reps, 2, warm_ms=WARM_MS) / HEAD_REP * 1e3, 2)
        lib.get().set_option(b"frspec_fused", 0)

        # through the library's own sub-matrix and buffers (cpmcu_draft_head)
        fr_val = torch.zeros((10, 10), dtype=torch.float16, device="cuda")
        fr_pos = torch.zeros((10, 10), dtype=torch.int32, device="cuda")
        fr_ids = torch.zeros((10, 10), dtype=torch.int32, device="cuda")

        def fr_model():
            for _ in range(HEAD_REP):
                model.L.draft_head(10, hid10.data_ptr(), fr_val.data_ptr(), fr_pos.data_ptr(), fr_ids.data_ptr())
        ms_fr_model = timed_model(fr_model, reps) / HEAD_REP
        frspec["model_level_us_per_call"] = round(ms_fr_model * 1e3, 2)
        frspec["model_level_frac"] = round(fr_bytes / (ms_fr_model * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)

        # the same head from a cold cache: its matrix (268 MB) nearly fits the last-level cache, so replays on one copy are
        # partly served from it; here every replay walks several distinct copies, so each pass misses
        def fr_cold():
            for w in w_subs:
                ops.frspec_head_topk(hid10, w, remap, 10)
        ms_fr_cold = timed_torch(torch, fr_cold, reps, 2, warm_ms=WARM_MS) / FR_SETS
        cold = {"frspec_head_us_per_call": round(ms_fr_cold * 1e3, 2), "frspec_weight_copies_rotated": FR_SETS,
                "frspec_frac_hbm": round(fr_bytes / (ms_fr_cold * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "note": "the FR-Spec head with every replay walking distinct copies of its matrix, so that no pass is served "
                        "from the 256 MB last-level cache; frspec_head above replays one copy"}

        lib.get().set_option(b"frspec_fused", 1)
        cold["frspec_one_launch_us_per_call"] = round(timed_torch(torch, fr_cold, reps, 2, warm_ms=WARM_MS) / FR_SETS * 1e3, 2)
        lib.get().set_option(b"frspec_fused", 0)

        # ---- the draft side of the path: one whole draft of the FR-Spec drafter (6 rounds of 10) ----
        # Per round: the drafter layer's own attention (10 queries, mask over 10*d columns, block sliding window of 1024
        # tokens, its own one-layer cache), the FR-Spec head with log-softmax + top-10 + id map-back, and the tree
        # bookkeeping kernel; the final top-59 + tree build at the end.  The dense parts of the drafter layer (fc,
        # projections, FFN) are not on the path and are not run; the head reads a different copy of its matrix every
        # round, as it would after their weights.
        k_it, n_it = cfg["topk"], draft_rounds
        Td = min(T, 64)  # src/model/minicpm4/minicpm4_eagle.cuh:69
        dtree = ops.DraftTree(k_it, n_it, remap)
        dcache = model.cache(block_table=main_run["tables"][0], num_layers=L + 1)  # layer L: the drafter's own cache
        dcache.k[L][: main_run["npages"]].copy_(dcache.k[0][: main_run["npages"]])
        dcache.v[L][: main_run["npages"]].copy_(dcache.v[0][: main_run["npages"]])
        hid1, hid_k = bufs.hidden[:1].contiguous(), bufs.hidden[:k_it].contiguous()  # k hidden rows per round after the first
        qd, kd, vd = bufs.q[0][:k_it].contiguous(), bufs.k_new[0][:k_it].contiguous(), bufs.v_new[0][:k_it].contiguous()
        d_len = [torch.tensor([P + k_it * d], dtype=torch.int32, device="cuda") for d in range(n_it)]
        d_out = torch.empty_like(qd)
        tree_ids = torch.full((Td,), -1, dtype=torch.int32, device="cuda")

        def draft_path():
            r = ops.frspec_head_topk(hid1, w_subs[0], remap, k_it)
            dtree.begin(r["val"][0], r["pos"][0])
            for d in range(1, n_it):
                ops.tree_attention(qd, dcache, L, d_len[d], padded, dtree.draft_mask, out=d_out, k_new=kd, v_new=vd,
                                   mask_k_range=k_it * d, block_window_size=1024)
                r = ops.frspec_head_topk(hid_k, w_subs[d % FR_SETS], remap, k_it)
                dtree.extend(d, r["val"], r["pos"])
            dtree.finish(Td, clen, tree_draft_ids=tree_ids)
        ms_draft_cold = timed_torch(torch, draft_path, reps, 2)

        # the same draft through the library's own model-level calls (drafter state, FR-Spec sub-matrix and the drafter
        # layer's cache owned by the library), recorded once into a library graph and replayed on the library's stream.
        # One copy of the matrix here: part of it stays in the last-level cache from round to round.
        next_ids = torch.zeros(k_it, dtype=torch.int32, device="cuda")
        prows = torch.zeros(k_it, dtype=torch.int32, device="cuda")
        dmask = torch.zeros(k_it, dtype=torch.int64, device="cuda")
        t_pos = torch.zeros(T, dtype=torch.int32, device="cuda")
        t_mask = torch.zeros(T, dtype=torch.int64, device="cuda")
        t_par = torch.zeros(T, dtype=torch.int32, device="cuda")
        model.set_block_table(main_run["tables"][0])
        torch.cuda.synchronize()

        def draft_model_level():
            model.draft_round(0, hid1, next_ids, None, dmask)
            for d in range(1, n_it):
                model.draft_attention(0, k_it, padded, qd, kd, vd, d_len[d], dmask, k_it * d, d_out)
                model.draft_round(d, hid_k, next_ids, prows, dmask)
            model.draft_finish(tree_ids, t_pos, clen, t_mask, t_par)
        gid = model.capture(draft_model_level)
        lib_stream = model.stream()
        for _ in range(3):
            model.replay(gid)
        model.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(lib_stream)
        for _ in range(reps):
            model.replay(gid)
        e1.record(lib_stream)
        model.synchronize()
        ms_draft = e0.elapsed_time(e1) / reps
        draft = {"us_per_draft": round(ms_draft * 1e3, 1), "us_per_draft_cold_matrix": round(ms_draft_cold * 1e3, 1),
                 "rounds": n_it, "topk_per_round": k_it, "tree_size": Td,
                 "operators": "%d x (FR-Spec head + log-softmax + top-%d + id map-back) + %d x drafter-layer attention "
                              "(window 1024) + tree bookkeeping (begin, %d x extend, finish)" % (n_it, k_it, n_it - 1, n_it - 1),
                 "note": "us_per_draft: cpmcu_draft_round / cpmcu_draft_attention / cpmcu_draft_finish on the library's model, "
                         "replayed as a library graph; us_per_draft_cold_matrix: the same operators with every round reading a "
                         "different copy of the FR-Spec matrix (as after the drafter layer's dense weights)"}
        # ---- the same kernels in bfloat16 (torch_dtype = 1): timing only, on the same buffers read as bfloat16 patterns ----
        lib.get().set_option(b"dtype", 1)
        try:
            def attn_bf16():
                for l in range(L):
                    ops.tree_attention(bufs.q[l], cache0, l, kvlen, padded, mask, out=bufs.attn_out[l], k_new=bufs.k_new[l], v_new=bufs.v_new[l])

            def head_bf16():
                for _ in range(HEAD_REP):
                    ops.lm_head_partials(bufs.hidden, w_t)

            as_bf16 = lambda t: t.to(torch.bfloat16).view(torch.float16)  # the same values, rounded to bfloat16, as 16-bit patterns
            w_subs_bf16 = [ops.tile_head_weight(as_bf16(w_dev), remap) for _ in range(FR_SETS)]
            hid10_bf16 = as_bf16(hid10)

            def fr_bf16():
                for w in w_subs_bf16:
                    ops.frspec_head_topk(hid10_bf16, w, remap, 10)
            bf16 = {"attention_us_per_layer_one_kv_set": round(timed_torch(torch, attn_bf16, reps, 2) / L * 1e3, 2),
                    "target_head_us": round(timed_torch(torch, head_bf16, reps, 2, warm_ms=WARM_MS) / HEAD_REP * 1e3, 2),
                    "frspec_head_us_per_call_cold": round(timed_torch(torch, fr_bf16, reps, 2, warm_ms=WARM_MS) / FR_SETS * 1e3, 2),
                    "note": "the bfloat16 instantiations of the same kernels (v_mfma_*_bf16), same shapes; the headline runs in fp16"}
        finally:
            lib.get().set_option(b"dtype", 0)
        del w_subs_bf16
        del w_subs, dtree, dcache, w_t
        torch.cuda.empty_cache()

    if args.workload == "c2_verify_4k":
        for k in kernels:
            kib = MEASURED_TRAFFIC["kib_per_launch"].get(k["kernel"])
            if kib is not None:
                k["traffic"] = kib * 1024
                k["traffic_unit"] = "bytes/launch"
    dominant = max(kernels, key=lambda k: k["us_per_launch"] * k["launches_per_step"])  # (operators outside the step count 0)
    roofline = {k: dominant[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")}
    roofline["kernel"] = dominant["kernel"]
    roofline["us_per_launch"] = dominant["us_per_launch"]

    # ---- CPU oracle on the host cores + parity of the step's integer results ----
    cpu = None
    parity = None
    if want_cpu:
        hid = bufs.hidden.cpu().numpy()
        head_times, gt_cpu = [], None
        for rep in range(4):  # 1 warm-up + 3 timed
            t0 = time.perf_counter()
            gt_cpu = oracle_mod.argmax(oracle_mod.lm_head(hid, w_host))
            head_times.append(time.perf_counter() - t0)
        t_head = statistics.median(head_times[1:])
        tail_times = []
        S = P + T
        # one layer's two caches as they were before the compaction: the prefix from the pool, the tree rows from the inputs
        kp_, vp_ = main_run["caches"][0].read_logical(0, 0, P)
        k_new0, v_new0 = bufs.k_new[0].cpu().numpy().reshape(T, -1), bufs.v_new[0].cpu().numpy().reshape(T, -1)
        flat0 = [np.concatenate([kp_.cpu().numpy().reshape(P, -1), k_new0]), np.concatenate([vp_.cpu().numpy().reshape(P, -1), v_new0])]
        for rep in range(4):
            flat = [x.copy() for x in flat0]
            t0 = time.perf_counter()
            a_cpu, node_cpu, path_cpu = oracle_mod.tree_accept(main_run["draft_np"], gt_cpu, tree.positions(P), P, tree.mask, tree.parent)
            ids_cpu = oracle_mod.kv_compact(flat, P, path_cpu, gt_cpu)
            tail_times.append(time.perf_counter() - t0)
        t_tail = statistics.median(tail_times[1:]) * L  # one layer's two caches timed, all layers' extrapolated
        t_attn = main_run["cpu_attn_s"]
        step_us = (t_attn * L + t_head + t_tail) * 1e6
        cpu = dict(value=round(step_us, 1), unit="us/step", cores=oracle_mod.num_threads(), kind="port",
                   head_and_tail_us=round((t_head + t_tail) * 1e6, 1),
                   sample="1 of %d attention layers (x%d extrapolated) + the full target head/arg-max + acceptance + compaction of one "
                          "layer's caches (x%d); each timed 4 times, first discarded, median of 3; attention %.1f ms/layer, head %.1f ms"
                          % (L, L, L, t_attn * 1e3, t_head * 1e3))
        gt_gpu = main_run["gt_np"]
        a_st, _, path_st = oracle_mod.tree_accept(main_run["draft_np"], gt_gpu, tree.positions(P), P, tree.mask, tree.parent)
        # the compacted rows of the first and the last layer (first K/V set) against the oracle's compaction of the same rows
        rows_ok = a_gpu == len(path_st) and np.array_equal(flat[0][P:P + a_gpu], k_new0[path_cpu])
        for l, (kd_, vd_) in main_run["compacted"].items():
            kn, vn = bufs.k_new[l].cpu().numpy().reshape(T, -1), bufs.v_new[l].cpu().numpy().reshape(T, -1)
            rows_ok = bool(rows_ok and np.array_equal(kd_, kn[path_st]) and np.array_equal(vd_, vn[path_st]))
        parity = dict(accept_length_gpu=a_gpu, accept_length_oracle=int(a_cpu),
                      ids_equal_oracle=bool(a_gpu == a_cpu and np.array_equal(ids_gpu, ids_cpu)),
                      staged_equal=bool(a_gpu == a_st and np.array_equal(ids_gpu, gt_gpu[path_st])),
                      compacted_rows_equal=rows_ok, kv_sets_agree=bool(sets_agree),
                      argmax_rows_equal=int((gt_gpu == gt_cpu).sum()), rows=int(T))

    # ---- the same step at longer contexts (same model, pools refilled) ----
    contexts = {str(P): round(ms_step * 1e3, 1)}
    ctx_attn = {str(P): dict(us_per_layer=round(ms_attn * 1e3, 2), tflops=round(attn_tflops, 1),
                             frac_mfma=round(attn_tflops / MFMA_F16_PEAK_TFLOPS, 4), kernel=attn_name,
                             step_minus_attention_us=round((ms_step - L * ms_attn) * 1e3, 1))}
    main_run.pop("caches", None)
    for name in names[1:]:
        r = run_context(torch, np, model, synth, oracle_mod, args, name, bufs, tree, use_graph, kv_sets_of(name), gen, want_cpu)
        Pc = r["P"]
        contexts[str(Pc)] = round(r["ms_step"] * 1e3, 1)
        tf = flops_attn(Pc) / (r["ms_attn"] * 1e-3) / 1e12
        ctx_attn[str(Pc)] = dict(us_per_layer=round(r["ms_attn"] * 1e3, 2), tflops=round(tf, 1), frac_mfma=round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                                 kernel=r["attn_plan"][0], step_minus_attention_us=round((r["ms_step"] - L * r["ms_attn"]) * 1e3, 1))
        kib = MEASURED_TRAFFIC["attention_kib_per_launch_by_context"].get(str(Pc))
        if kib is not None and r["attn_plan"][0] == "tree_attn_split_kernel<1,false>":
            ctx_attn[str(Pc)]["traffic"] = kib * 1024
            ctx_attn[str(Pc)]["algorithmic_bytes"] = int(bytes_attn(Pc))
        if parity is not None:  # acceptance on the device's arg-max + compacted rows, as for the headline context
            parity.setdefault("contexts", {})[str(Pc)] = context_parity(np, oracle_mod, r, bufs, tree)
        if cpu is not None:
            cpu.setdefault("contexts", {})[str(Pc)] = dict(
                attention_ms_per_layer=round(r["cpu_attn_s"] * 1e3, 1),
                us_per_step_extrapolated=round(r["cpu_attn_s"] * 1e6 * L + cpu["head_and_tail_us"], 1),
                sample="1 of %d attention layers timed 4 times, first discarded, median of 3" % L)
        r.pop("caches", None)
        del r
        torch.cuda.empty_cache()

    model.close()

    # ---- what the matrix pipes sustain on this GPU (last, so that its heat does not touch the figures above) ----
    probes = None if args.no_probes else machine_probes(torch)
    power = None if args.no_probes else power_probe(torch, np, synth)
    if probes is not None:
        ceiling = probes["mfma_tflops_random_operands"]
        if roofline["bound"] == "mfma":  # the same achieved figure against MFMAs alone on random operands
            roofline["measured_ceiling"] = ceiling
            roofline["frac_of_measured_ceiling"] = round(roofline["achieved"] / ceiling, 4)
        for v in ctx_attn.values():
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
        "config": {"workload": wl_desc, "batch": 1, "library_graph": use_graph, "kv_splits": main_run["attn_plan"][1],
                   "kv_sets_rotated": kv_sets_of(args.workload),
                   "launches_per_step": L * (main_run["attn_plan"][0].count("+") + 1) + 2},
        "wall_ms_per_step": round(main_run["wall_ms"], 5),
        "us_per_step_one_kv_set": round(main_run["ms_one_set"] * 1e3, 1),
        "roofline": roofline,
        "machine_probes": probes,
        "power_probe": power,
        "kernels": kernels,
        "traffic_source": MEASURED_TRAFFIC["source"],
        "traffic_measured_at_commit": MEASURED_TRAFFIC["measured_at_commit"],
        "frspec_head": frspec,
        "cold_cache": cold,
        "draft_path": draft,
        "attention_with_rope": rope_cmp,
        "bf16": bf16,
        "contexts_us_per_step": contexts,
        "attention_by_context": ctx_attn,
        "cpu_baseline": cpu,
        "parity": parity,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
