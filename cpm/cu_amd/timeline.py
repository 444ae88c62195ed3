"""Where the time of a launch goes, from wall-clock stamps taken inside the kernels.

    python -m cpm.cu_amd.timeline attention [P ...] [--rows T]   tree attention, T-node tree (default 60), prefix lengths P (default 4096)
    python -m cpm.cu_amd.timeline head [n ...]          target head 73448 x 4096, n hidden rows (default 60 16)
    python -m cpm.cu_amd.timeline frspec                FR-Spec head 32768 x 4096, 10 rows: two launches and one launch

Runs on libcpmcu_amd_timeline.so, the build of the same sources with the stamps of csrc/timeline.h compiled in (the
product library has none of them).  Every figure is microseconds from the start of the earliest workgroup of the launch;
a stamp is thread 0's read of the 100 MHz wall clock, so it is good to 10 ns and says when *that* thread got there.
Operands are random fp16 data; the weight matrix is rotated over three copies so that no pass is served from the
last-level cache.
"""
import ctypes
import os
import sys

import numpy as np


def _load():
    from . import build, lib as libmod
    if not os.path.exists(build.TIMELINE_LIB_PATH):
        raise ImportError("%s is missing: run `python -m cpm.cu_amd.build`" % build.TIMELINE_LIB_PATH)
    libmod.LIB_PATH = build.TIMELINE_LIB_PATH  # before the first lib.get()
    L = libmod.get()
    for name in ("cpmcu_timeline_read_head", "cpmcu_timeline_read_attention", "cpmcu_timeline_read_topk"):
        getattr(L.raw, name).argtypes = [ctypes.c_void_p]
        getattr(L.raw, name).restype = ctypes.c_int
    return L


def _read(L, which, nwg):
    buf = np.zeros(1024 * 16, np.uint64)
    rc = getattr(L.raw, "cpmcu_timeline_read_" + which)(buf.ctypes.data)
    if rc != 0:
        raise RuntimeError("reading the timeline records failed")
    return buf.reshape(1024, 16).astype(np.int64)[:nwg]


def _spread(name, x):
    return "  %-34s min %6.2f  median %6.2f  p90 %6.2f  max %6.2f" % (name, x.min(), np.median(x), np.percentile(x, 90), x.max())


def attention(L, torch, prefixes, T=60):
    from . import ops, synth
    from .kvcache import PagedKVCache
    Hq, Hkv, D, NL = 32, 2, 128, 8
    mask = None  # one row, or a chain beyond 64 rows
    if 1 < T <= 64:
        mask = torch.from_numpy(synth.eagle_tree(6, 10, T, 0).mask.view(np.int64)).cuda()
    for P in prefixes:
        S = P + T
        cache = PagedKVCache(NL, Hkv, (S + 255) // 256 + 1)
        for l in range(NL):
            cache.k[l].normal_()
            cache.v[l].normal_()
        q = torch.randn(T, Hq, D, device="cuda").half()
        kn = torch.randn(T, Hkv, D, device="cuda").half()
        vn = torch.randn(T, Hkv, D, device="cuda").half()
        kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
        out = torch.empty_like(q)
        pad = (S + 127) // 128 * 128
        for _ in range(6):
            for l in range(NL):
                ops.tree_attention(q, cache, l, kv_len, pad, mask, out=out, k_new=kn, v_new=vn)
        torch.cuda.synchronize()
        _read(L, "attention", 1024)  # clears
        ops.tree_attention(q, cache, 0, kv_len, pad, mask, out=out, k_new=kn, v_new=vn)
        d = _read(L, "attention", 1024)
        buf_mask = d[:, 0] > 0
        d = d[buf_mask]
        t0 = d[:, 0].min()
        rel = (d[:, :8] - t0) / 100.0
        kernels, splits, groups, wgs = ops.attention_plan(T, Hq, Hkv, pad)
        print("tree attention, %d-token prefix + %d-node tree: %s, %d splits, %d workgroups recorded" % (P, T, kernels, splits, len(d)))
        for i, name in enumerate(["start", "K loop entered", "K loop left", "KV groups merged", "partials issued", "partials acknowledged",
                                  "all splits of the unit arrived", "end (own share merged, output stored)"]):
            if i >= 5 and not d[:, i].any():
                continue  # the merge is a launch of its own: the split launch ends with its partials
            print(_spread(name, rel[:, i]))
        tiles = d[:, 9]
        merged = d[:, 7].any()
        for nt in np.unique(tiles):
            r = rel[tiles == nt]
            if merged:
                print("  workgroups with %d tiles (%d): loop left %.2f, arrived %.2f, end %.2f (medians)" % (nt, len(r), np.median(r[:, 2]), np.median(r[:, 6]), np.median(r[:, 7])))
            else:
                print("  workgroups with %d tiles (%d): loop left %.2f, partials issued %.2f (medians)" % (nt, len(r), np.median(r[:, 2]), np.median(r[:, 4])))
        wg = np.nonzero(buf_mask)[0]
        print("  K loop left by XCD (workgroup number mod 8), medians: " + " ".join("%.1f" % np.median(rel[wg % 8 == x, 2]) for x in range(8)))
        last = d[d[:, 10] == d[:, 10].max()]  # the last split: the appended rows and the end of the stream
        rl = (last - t0) / 100.0
        second = "%.2f" % np.median(rl[:, 12]) if (last[:, 12] != 0).all() else "none"  # a split of one or two tiles has no second iteration: no stamp
        print("  last split (%d workgroups, %s tiles): loop entered %.2f, second iteration %s, patch begun %.2f, V patch begun %.2f, patch done %.2f, loop left %.2f (medians; patch of the M-tile-0 workgroups done %.2f)" %
              (len(last), "/".join(str(x) for x in np.unique(last[:, 9])), np.median(rl[:, 1]), second, np.median(rl[:, 14]), np.median(rl[:, 13]), np.median(rl[:, 15]), np.median(rl[:, 2]),
               np.median(rl[last[:, 11] == 0][:, 15])))
        del cache


def _head_records(L, nwg):
    d = _read(L, "head", nwg)
    t0 = d[:, 0].min()
    return d, t0


def head(L, torch, rows):
    from . import ops
    V, H, copies = 73448, 4096, 3
    ws = [ops.tile_head_weight((torch.randn(V, H, device="cuda") * 0.02).half()) for _ in range(copies)]
    for n in rows:
        hid = torch.randn(n, H, device="cuda").half()
        name, wgs = ops.head_plan(n, ws[0])
        for _ in range(4):
            for w in ws:
                ops.lm_head_argmax(hid, w, head_scale=0.5)
        torch.cuda.synchronize()
        _read(L, "head", 1024)
        ops.lm_head_argmax(hid, ws[0], head_scale=0.5)
        d, t0 = _head_records(L, wgs)
        rel = (d[:, :5] - t0) / 100.0
        waves = (d[:, 8:16] - t0) / 100.0
        print("target head %d x %d, %d hidden rows: %s, %d workgroups" % (V, H, n, name, wgs))
        for i, nm in enumerate(["start", "wave 0 out of the K loop", "full passes folded", "shared last pass folded", "partials written"]):
            print(_spread(nm, rel[:, i]))
        print(_spread("every wave out of the K loop", waves))
        last = waves.max(axis=1)
        print("  last wave out of the loop to the end of the workgroup: median %.2f, for the last workgroup %.2f" %
              (np.median(rel[:, 4] - last), rel[:, 4].max() - last.max()))
        print("  loop end by XCD (workgroup number mod 8), medians: " + " ".join("%.1f" % np.median(last[np.arange(wgs) % 8 == x]) for x in range(8)))


def frspec(L, torch):
    from . import lib as libmod, ops
    V, H, n, k, copies = 32768, 4096, 10, 10, 3
    ws = [ops.tile_head_weight((torch.randn(V, H, device="cuda") * 0.02).half()) for _ in range(copies)]
    hid = torch.randn(n, H, device="cuda").half()
    remap = torch.arange(V, dtype=torch.int32, device="cuda")
    for fused in (0, 1):
        libmod.get().set_option(b"frspec_fused", fused)
        for _ in range(6):
            for w in ws:
                ops.frspec_head_topk(hid, w, remap, k)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            for w in ws:
                ops.frspec_head_topk(hid, w, remap, k)
        e1.record()
        torch.cuda.synchronize()
        print("FR-Spec head %d x %d, %d rows, top-%d: %s, %.2f us per call (eager, rotated copies, stamps compiled in)" %
              (V, H, n, k, ops.frspec_head_plan(n, ws[0], k), e0.elapsed_time(e1) / (20 * copies) * 1e3))
        _read(L, "head", 1024)
        _read(L, "topk", 16)
        ops.frspec_head_topk(hid, ws[0], remap, k)
        d, t0 = _head_records(L, 256)
        rel = (d - t0) / 100.0
        waves = rel[:, 8:16] if not fused else None
        print(_spread("start", rel[:, 0]))
        print(_spread("wave 0 out of the K loop", rel[:, 1]))
        print(_spread("statistics / partials out", rel[:, 4]))
        if fused:
            print(_spread("keys published", rel[:, 5]))
            print(_spread("stores acknowledged", rel[:, 6]))
            fin = d[(d[:, 12] > 0) & (d[:, 12] <= n)]
            for r in fin[np.argsort(fin[:, 12])]:
                f = (r - t0) / 100.0
                print("    finisher of row %d: own loop left %.2f, place known %.2f, all words seen %.2f, bound %.2f, candidates listed %.2f (%d), row written %.2f" %
                      (r[12] - 1, f[1], f[7], f[9], f[10], f[11], r[14], f[13]))
            print("  last keys published %.2f, last row written %.2f" % (rel[:, 5].max(), ((fin[:, 13] - t0) / 100.0).max()))
        else:
            print(_spread("every wave out of the K loop", waves))
            # the row kernel that follows (records of its own clock origin: its first workgroup's start)
            tk = _read(L, "topk", n)
            gemm_end = rel[:, 4].max()
            tr = (tk[:, :7] - tk[:, 0].min()) / 100.0
            print("  topk_row_kernel<true> (%d workgroups of 1024 threads), from the start of its first workgroup, which comes %.2f us after the GEMM's last partials:" %
                  (n, (tk[:, 0].min() - t0) / 100.0 - gemm_end))
            for i, nm in enumerate(["start", "row in registers", "bound and statistics known", "candidate lanes in LDS", "candidates extracted", "ranked", "outputs written"]):
                print(_spread(nm, tr[:, i]))
    libmod.get().set_option(b"frspec_fused", 0)


def main(argv):
    import torch
    if not argv or argv[0] not in ("attention", "head", "frspec"):
        print(__doc__)
        return 2
    L = _load()
    torch.cuda.set_device(0)
    if argv[0] == "attention":
        rest, T = argv[1:], 60
        if "--rows" in rest:
            i = rest.index("--rows")
            T = int(rest[i + 1])
            rest = rest[:i] + rest[i + 2:]
        attention(L, torch, [int(x) for x in rest] or [4096], T)
    elif argv[0] == "head":
        head(L, torch, [int(x) for x in argv[1:]] or [60, 16])
    else:
        frspec(L, torch)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
