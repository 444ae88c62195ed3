"""Timings of the operators over ranges of shapes, with the kernels the library picks for each: looks for cliffs in the launch plans.

    python -m cpm.cu_amd.sweep attention [--groups] [--heads Hq,Hkv] [--graph]
                                                      tree attention, prefix 256..131072 x tree rows 1..128 (us per layer);
                                                      --groups: the automatic choice beside both kernel shapes forced;
                                                      --heads: query / KV head counts other than 32,2;
                                                      --graph: timed inside replayed graphs (short contexts are
                                                      launch-bound when enqueued from Python)
    python -m cpm.cu_amd.sweep head                   target head (arg-max), rows 1..128 x vocabulary 8K..256K x hidden 2048/4096/8192
    python -m cpm.cu_amd.sweep frspec                 FR-Spec head + log-softmax + top-k + id map-back, vocabulary 8K..73448 x rows x k
    python -m cpm.cu_amd.sweep topk                   top-k of fp16 rows, row length 64..152K x rows 1..60 x k 1..128
    python -m cpm.cu_amd.sweep window                 the drafter layer's attention (k queries, block window of 1024 tokens): the
                                                      library's plan beside both kernel shapes and forced split counts

Eager launches on cuda:0, random fp16 data, event-timed; attention rotates over several layers' K/V pools and the heads over
copies of the weight matrix, so that no pass is served from the last-level cache.  Fractions are of 8 TB/s (heads) and TFLOP/s
are 4 * Hq * T * D * S per layer (attention).
"""
import sys

import numpy as np


def _time(torch, fn, reps):
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3


def _time_graph(torch, fn, reps, inner):
    """us per call of fn inside a replayed graph of `inner` calls: launch gaps as a decode loop has them, no Python in between."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    g, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            for _ in range(inner):
                fn()
    for _ in range(3):
        g.replay()
    torch.cuda.synchronize()
    return _time(torch, g.replay, reps) / inner


def attention(torch, with_groups, Hq=32, Hkv=2, graph=False):
    from . import lib, ops, synth
    from .kvcache import PagedKVCache
    D = 128
    L = lib.get()
    prefixes = [256, 1024, 2048, 4096, 8192, 16384, 32768, 65536, 131072]
    rows = [1, 8, 16, 24, 32, 40, 48, 60, 64, 96, 128]
    print("tree attention, %d query / %d KV heads: us per layer (kernel shape <G>, KV splits, +c: merge launch)" % (Hq, Hkv))
    print("%8s" % "P \\ T" + "".join("%22d" % t for t in rows))
    for P in prefixes:
        line = "%8d" % P
        for T in rows:
            mask = None
            if 1 < T <= 64:
                mask = torch.from_numpy(synth.eagle_tree(6, 10, T, 0).mask.view(np.int64)).cuda()
            S = P + T
            nl = 6 if P <= 32768 else 3
            cache = PagedKVCache(nl, Hkv, (S + 255) // 256 + 1)
            for l in range(nl):
                cache.k[l].normal_()
                cache.v[l].normal_()
            q = torch.randn(T, Hq, D, device="cuda").half()
            kn = torch.randn(T, Hkv, D, device="cuda").half()
            vn = torch.randn(T, Hkv, D, device="cuda").half()
            kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
            out = torch.empty_like(q)
            pad = (S + 127) // 128 * 128

            def run():
                for l in range(nl):
                    ops.tree_attention(q, cache, l, kv_len, pad, mask, out=out, k_new=kn, v_new=vn)
            cell = []
            for G in ((0, 1, 2) if with_groups else (0,)):
                L.set_option(b"attn_kv_groups", G)
                for _ in range(3):
                    run()
                torch.cuda.synchronize()
                us = (_time_graph(torch, run, 12, 1) if graph else _time(torch, run, 12 if P <= 32768 else 6)) / nl
                kernels, splits, groups, _ = ops.attention_plan(T, Hq, Hkv, pad)
                cell.append("%.1f <%d> s%d%s" % (us, groups, splits, "+c" if "combine" in kernels else ""))
            L.set_option(b"attn_kv_groups", 0)
            line += "%22s" % cell[0] if not with_groups else "  [" + " | ".join(cell) + "]"
            del cache
        print(line, flush=True)


def head(torch):
    from . import ops
    rows = [1, 16, 17, 32, 33, 60, 64, 100, 128]
    for H in (2048, 4096, 8192):
        print("target head, hidden size %d: fraction of 8 TB/s (kernel)" % H)
        print("%8s" % "V \\ n" + "".join("%20d" % n for n in rows))
        for V in (8192, 16384, 32768, 50000, 73448, 100000, 131072, 151936, 200000, 262144):
            w = (torch.randn(V, H, device="cuda") * 0.02).half()
            copies = [ops.tile_head_weight(w) for _ in range(2 if V * H * 2 < 1.5e9 else 1)]
            del w
            line = "%8d" % V
            for n in rows:
                hid = torch.randn(n, H, device="cuda").half()
                name = ops.head_plan(n, copies[0])[0].replace("head_gemm_", "").replace("stream_kernel", "S").replace("chunked_kernel", "C")

                def run():
                    for c in copies:
                        ops.lm_head_argmax(hid, c)
                for _ in range(3):
                    run()
                torch.cuda.synchronize()
                us = _time(torch, run, 10) / len(copies)
                line += "%20s" % ("%.2f %s" % (V * H * 2 / us * 1e-3 / 8000, name))
            print(line, flush=True)
            del copies


def frspec(torch):
    from . import ops
    H = 4096
    print("FR-Spec head + log-softmax + top-k + id map-back, hidden size %d: us per call, fraction of 8 TB/s" % H)
    for Vs in (8192, 16384, 32768, 40960, 49152, 65536, 73448):
        w = (torch.randn(Vs, H, device="cuda") * 0.02).half()
        copies = [ops.tile_head_weight(w) for _ in range(3)]
        remap = torch.arange(Vs, dtype=torch.int32, device="cuda")
        del w
        for n, k in ((1, 10), (10, 1), (10, 10), (16, 16)):
            hid = torch.randn(n, H, device="cuda").half()

            def run():
                for c in copies:
                    ops.frspec_head_topk(hid, c, remap, k)
            for _ in range(3):
                run()
            torch.cuda.synchronize()
            us = _time(torch, run, 10) / 3
            print("  V' = %6d  rows %2d  k %2d   %6.1f us  %.2f   %s" % (Vs, n, k, us, Vs * H * 2 / us * 1e-3 / 8000, ops.frspec_head_plan(n, copies[0], k)), flush=True)
        del copies


def topk(torch):
    from . import ops
    tops = [1, 10, 16, 32, 64, 128]
    for n in (1, 10, 60):
        print("top-k of %d fp16 rows: us per call (k across, row length down)" % n)
        print("%8s" % "dim \\ k" + "".join("%9d" % k for k in tops))
        for dim in (64, 510, 640, 1000, 4096, 8192, 16384, 32001, 32768, 32776, 65536, 73448, 151643, 151936):
            xs = [torch.randn(n, dim, device="cuda").half() for _ in range(4)]
            line = "%8d" % dim
            for k in tops:
                if k > dim:
                    line += "%9s" % "-"
                    continue

                def run():
                    for x in xs:
                        ops.topk(x, k)
                try:
                    for _ in range(3):
                        run()
                except ValueError:  # a shape the operator refuses
                    line += "%9s" % "refused"
                    continue
                torch.cuda.synchronize()
                line += "%9.1f" % (_time(torch, run, 10) / len(xs))
            print(line, flush=True)


def window(torch):
    from . import lib, ops
    from .kvcache import PagedKVCache
    Hq, Hkv, D = 32, 2, 128
    L = lib.get()
    splits = (0, 2, 4, 8, 12, 16)
    print("drafter-layer attention, %d query / %d KV heads, block window 1024: us per call in a replayed graph (0 = the library's choice)" % (Hq, Hkv))
    print("%28s" % "shape <G> \\ splits" + "".join("%8d" % ns for ns in splits))
    for P in (4096, 32768):
        for k, d in ((10, 1), (10, 5), (16, 3)):
            S = P + k * d
            cache = PagedKVCache(4, Hkv, (S + 255) // 256 + 2)
            for l in range(4):
                cache.k[l].normal_()
                cache.v[l].normal_()
            q = torch.randn(k, Hq, D, device="cuda").half()
            kn = torch.randn(k, Hkv, D, device="cuda").half()
            vn = torch.randn_like(kn)
            kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
            mask = torch.from_numpy(np.random.default_rng(0).integers(1, 2 ** min(k * d, 62), size=k, dtype=np.int64)).cuda()
            out = torch.empty_like(q)
            pad = (S + 127) // 128 * 128
            for G in (0, 1, 2):
                L.set_option(b"attn_kv_groups", G)
                line = "%28s" % ("P %d, %d queries, round %d, <%d>" % (P, k, d, G))
                for ns in splits:
                    def run():
                        for l in range(4):
                            ops.tree_attention(q, cache, l, kv_len, pad, mask, out=out, k_new=kn, v_new=vn, mask_k_range=k * d,
                                               block_window_size=1024, num_splits=ns)
                    line += "%8.1f" % (_time_graph(torch, run, 20, 2) / 4)
                print(line, flush=True)
            L.set_option(b"attn_kv_groups", 0)
            del cache


def main(argv):
    if not argv or argv[0] not in ("attention", "head", "frspec", "topk", "window"):
        print(__doc__)
        return 2
    import torch
    from . import lib
    lib.get()  # raises if libcpmcu_amd.so is missing
    torch.cuda.set_device(0)
    if argv[0] == "attention":
        heads = argv[argv.index("--heads") + 1].split(",") if "--heads" in argv else (32, 2)
        attention(torch, "--groups" in argv[1:], int(heads[0]), int(heads[1]), "--graph" in argv[1:])
    elif argv[0] == "head":
        head(torch)
    elif argv[0] == "topk":
        topk(torch)
    elif argv[0] == "window":
        window(torch)
    else:
        frspec(torch)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
