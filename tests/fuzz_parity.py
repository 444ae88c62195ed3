"""Time-boxed random parity runs of every operator of the path against the CPU oracle, on cuda:0.

    python tests/fuzz_parity.py [seconds (default 480)] [first seed (default 1000)] [stages, comma-separated (default all)]

Not collected by pytest (the suites in test_gpu_*.py are the fixed, seeded cases); this draws fresh shapes and data for as
long as it is given and applies the same checks through the tests' own helpers: tree attention in its three input modes
(values to fp16 tolerance, appended cache rows bit for bit), the target head's arg-max, the FR-Spec head with log-softmax,
top-k and id map-back, the stand-alone top-k (ties, -inf, wide ranges), acceptance / compaction / the one-launch tail,
the draft-tree construction (all bit-exact), sequences of model-level verify steps enqueued eagerly and replayed as the
library's graphs, a speculative loop on a toy target against plain greedy decoding, and the bfloat16 instantiations of the
attention and the two heads; the FR-Spec head's one-launch form is held to the two-launch one.  Shapes the C-ABI refuses by contract (a documented limit) are counted, not
failures.  Exit status 1 and one line per mismatch (operator, seed, message) if anything differs.
"""
import os
import sys
import time
import warnings

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np  # noqa: E402


def main(argv):
    import torch
    import oracle as orc
    from cpm.cu_amd import lib, ops, synth
    import test_gpu_accept as t_accept
    import test_gpu_attention as t_attention
    import test_gpu_bf16 as t_bf16
    import test_gpu_draft_tree as t_draft
    import test_gpu_frspec_fused as t_fused
    import test_gpu_heads as t_heads
    import test_gpu_spec_loop as t_loop
    import test_gpu_verify_step as t_step
    import pytest
    from util import to_dev, to_np

    budget = float(argv[0]) if len(argv) > 0 else 480.0
    first_seed = int(argv[1]) if len(argv) > 1 else 1000
    lib.get()  # raises if libcpmcu_amd.so is missing: nothing here runs without the HIP library
    torch.cuda.set_device(0)
    warnings.simplefilter("ignore")
    fails = []

    def run(name, fn, secs):
        t0 = last = time.time()
        n = refused = 0
        while time.time() - t0 < secs:
            if time.time() - last > 30:  # a sign of life for whoever watches the output
                last = time.time()
                print("  %s: %d cases so far" % (name, n), flush=True)
            seed = first_seed + n
            try:
                fn(seed)
            except ValueError as e:  # CPMCU_ERR_INVALID_ARGUMENT: a shape outside a documented limit
                if "limit" not in str(e) and "outside" not in str(e):
                    raise
                refused += 1
            except pytest.skip.Exception:  # an arg-max near-tie the test itself declares undecidable
                refused += 1
            except AssertionError as e:
                fails.append((name, seed, str(e)[:300]))
                print("MISMATCH", name, seed, str(e)[:300], flush=True)
            n += 1
        print("%s: %d cases (%d refused by the API or undecidable) in %.0f s, %d mismatches so far" % (name, n, refused, time.time() - t0, len(fails)), flush=True)

    def attention(seed):
        g = synth.rng(seed, 91)
        edges_p = [0, 1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049]
        edges_t = [1, 2, 3, 8, 15, 16, 17, 31, 32, 33, 60, 63, 64, 65, 100, 127, 128]
        P = int(edges_p[g.integers(len(edges_p))]) if g.random() < 0.5 else int(g.integers(0, 5000))
        T = int(edges_t[g.integers(len(edges_t))]) if g.random() < 0.6 else int(g.integers(1, 129))
        mode = ["in_cache", "append", "append_rope"][int(g.integers(3))]
        splits = [0, 0, 0, 1, 2, 3, 5, 7, 16, 17, 24, 32, 33, 64, 100, 128][int(g.integers(16))]
        slack = [0, 0, 1, 63, 64, 200, 1000][int(g.integers(7))]
        lib.get().set_option(b"attn_kv_groups", int(g.integers(3)))  # 0 = the library's choice
        try:
            t_attention.test_randomised_shape_sweep(torch, orc, P, T, mode, splits, slack, seed)
        finally:
            lib.get().set_option(b"attn_kv_groups", 0)

    def head_counts(seed):
        g = synth.rng(seed, 102)
        HKV = int([1, 1, 2, 3, 4, 8, 16, 32][g.integers(8)])
        HQ = HKV * int([1, 1, 2, 3, 4, 5, 8, 16][g.integers(8)])
        t_attention._heads_case(torch, orc, HQ, HKV, int(g.integers(0, 4000)), int(g.integers(1, 129)), ["in_cache", "append", "append_rope"][int(g.integers(3))], seed)

    def target_head(seed):
        g = synth.rng(seed, 92)
        n = int(g.integers(1, 129))
        V = int(g.integers(16, 40000))
        H = int([512, 1024, 2048, 4096][g.integers(4)])
        if H >= 2048:
            V = min(V, 12000)
        elif g.random() < 0.2:  # one to twelve passes over the CUs' wave slots: the streaming kernel's shapes and grids
            V, H = int(g.integers(33000, 420000)), 512
        t_heads._argmax_check(torch, orc, n, V=V, H=H, seed=seed, scale=[None, 0.5, 1.7][int(g.integers(3))], tiled=bool(g.integers(2)))

    def frspec_head(seed):
        g = synth.rng(seed, 93)
        n = int(g.integers(1, 17))
        H = int([512, 1024][g.integers(2)])
        Vs = int(g.integers(2, 4200)) * 8 - (int(g.integers(8)) if g.random() < 0.3 else 0)
        V = Vs + int(g.integers(0, 5000))
        t_heads._frspec_check(torch, orc, n, V, Vs, H, int(g.integers(1, 33)), seed, tiled=bool(g.integers(2)))

    def topk(seed):
        g = synth.rng(seed, 94)
        n = int(g.integers(1, 6))
        dim = int(g.integers(1, 40000)) if g.random() < 0.7 else int(g.integers(4096, 17000)) * 8  # the latter: slices of the row kernel
        top = int(g.integers(1, min(dim, 128) + 1))
        kind = int(g.integers(4))
        if kind == 0:
            x = g.standard_normal((n, dim)).astype(np.float16)
        elif kind == 1:
            x = g.integers(-3, 3, size=(n, dim)).astype(np.float16)  # ties everywhere
        elif kind == 2:
            x = np.full((n, dim), -np.inf, np.float16)  # mostly -inf
            idx = g.integers(0, dim, size=max(1, dim // 50))
            x[:, idx] = g.standard_normal(len(idx)).astype(np.float16)
        else:
            x = (g.standard_normal((n, dim)) * np.exp(g.standard_normal((n, dim)) * 2)).astype(np.float16)
        chunk_form = g.random() < 0.1 and -(-dim // 2048) * top <= 2048  # one case in ten: the chunk + merge form
        if chunk_form:
            lib.get().set_option(b"topk_row_kernel", 0)
        try:
            val, pos = ops.topk(to_dev(torch, x), top)
            torch.cuda.synchronize()
        finally:
            if chunk_form:
                lib.get().set_option(b"topk_row_kernel", 1)
        v_ref, p_ref = orc.topk(x, top)
        what = "n=%d dim=%d top=%d kind=%d chunk_form=%d" % (n, dim, top, kind, chunk_form)
        assert np.array_equal(to_np(pos), p_ref), "top-k positions, " + what
        assert np.array_equal(to_np(val).view(np.uint16), v_ref.view(np.uint16)), "top-k values, " + what

    def tail(seed):
        g = synth.rng(seed, 95)
        T = int(g.integers(1, 129))
        tree = synth.random_tree(T, seed, max_children=int(g.integers(1, 8)), max_depth=int(g.integers(1, 14)))
        P = int(g.integers(0, 1200))
        depth = int(g.integers(0, int(tree.depth.max()) + 1))
        kind = int(g.integers(3))
        if kind == 0:
            t_accept._compact_case(torch, orc, tree, P, depth, layers=2, seed=seed, page_perm=bool(g.integers(2)))
        elif kind == 1:
            t_accept._tail_case(torch, orc, tree, P, depth, layers=2, seed=seed, H=512, V=int(g.integers(200, 5000)), from_partials=bool(g.integers(2)))
        else:
            t_accept._commit_case(torch, orc, tree, P, depth, layers=2, seed=seed)

    def draft_tree(seed):
        g = synth.rng(seed, 96)
        k = int(g.integers(1, 17))
        num_iter = min(int(g.integers(2, 9)), max(2, 64 // k))  # k * num_iter fits the 64-bit draft mask
        T = int(g.integers(2, min(128, 1 + k * num_iter) + 1))
        t_draft.test_draft_tree_equals_oracle(torch, orc, k, num_iter, T, seed, bool(g.integers(2)), bool(g.integers(2)))

    def verify_steps(seed):
        g = synth.rng(seed, 97)
        T = int(g.integers(2, 129))  # beyond 64 nodes: two mask words per row
        t_step._graph_replays_equal_eager_steps(torch, orc, seed, T=T, P0=int(g.integers(0, 3000)), STEPS=int(g.integers(3, 13)), LAYERS=int(g.integers(1, 4)),
                                                V=int(g.integers(500, 6000)), num_iter=8, topk=min(8, T - 1), min_paddings=1)

    def speculative_loop(seed):
        t_loop._speculative_loop(torch, orc, seed)

    def bf16_operators(seed):
        g = synth.rng(seed, 98)
        L = lib.get()

        def set_option(name, value):
            L.set_option(name.encode(), int(value))
        set_option("dtype", 1)
        orc.set_dtype("bf16")
        try:
            kind = int(g.integers(3))
            if kind == 0:
                t_bf16.test_bf16_tree_attention_with_fused_append(torch, orc, None, set_option, int(g.integers(1, 3)), int(g.integers(0, 5000)),
                                                                  int(g.integers(2, 61)), bool(g.integers(2)))
            elif kind == 1:
                H = int([512, 1024, 2048][g.integers(3)])
                t_bf16.test_bf16_target_head_and_argmax(torch, orc, None, int(g.integers(1, 129)), int(g.integers(16, 12000)), H, bool(g.integers(2)),
                                                        [None, 0.3125][int(g.integers(2))])
            else:
                Vs = int(g.integers(2, 2100)) * 8
                t_bf16.test_bf16_frspec_head_topk(torch, orc, None, int(g.integers(1, 17)), Vs + int(g.integers(0, 3000)), Vs, int([512, 1024][g.integers(2)]),
                                                  int(g.integers(1, 33)), bool(g.integers(2)))
        finally:
            orc.set_dtype("f16")
            set_option("dtype", 0)
            set_option("attn_kv_groups", 0)

    def windows(seed):
        # the drafter's own layers: a mask over k*d columns, the block sliding window; and the window under a verify-sized tree
        g = synth.rng(seed, 100)
        kind = int(g.integers(3))
        window = int([128, 256, 512, 1024, 2048, 4096][g.integers(6)])
        if kind == 2:
            t_attention.test_tree_block_window_with_rope(torch, orc, int(g.integers(0, 6000)), int(g.integers(1, 65)), window, bool(g.integers(2)))
            return
        k = int(g.integers(1, 17))
        d = int(g.integers(1, min(8, 64 // k) + 1))
        P0 = int(g.integers(0, 5000))
        if kind == 0:
            t_attention.test_draft_layer_mask_range(torch, orc, k, d, P0, seed)
        else:
            t_attention.test_draft_layer_block_window(torch, orc, k, d, P0, window, int([0, 0, 1, 2, 3, 5][g.integers(6)]), seed)

    def merge_forms(seed):
        # the merge inside the split launch against the separate combine launch: bit-identical outputs when the split count
        # is the same (left to the library, the two forms may partition the keys differently: other roundings)
        g = synth.rng(seed, 101)
        L = lib.get()
        try:
            t_attention.test_merge_in_launch_equals_separate_merge(torch, lambda name, v: L.set_option(name.encode(), int(v)), int(g.integers(0, 9000)),
                                                                   int(g.integers(1, 129)), int([1, 2, 3, 4, 5, 7, 8, 11, 16, 24, 32][g.integers(11)]),
                                                                   bool(g.integers(2)), bool(g.integers(2)))
        finally:
            L.set_option(b"attn_merge_in_launch", 1)

    fused_weights = {}

    def frspec_one_launch(seed):
        # the one-launch form (option frspec_fused) against the two-launch form, which the "frspec" stage holds to the oracle
        g = synth.rng(seed, 99)
        H = 512
        V = int([2048, 4096, 8192, 16384, 32768, 32768, 37568, 50000, 65536][g.integers(9)])
        std = float([0.02, 0.02, 0.002, 0.0003, 0.0][g.integers(5)])
        n, k = int(g.integers(1, 17)), int(g.integers(1, 17))
        if (V, std) not in fused_weights:
            if len(fused_weights) > 5:
                fused_weights.clear()
            w = synth.normal_f16((V, H), seed, 2, std=std) if std > 0 else np.zeros((V, H), np.float16)
            if g.random() < 0.3:
                w[g.integers(1, V, size=V // 3)] = w[0]
            fused_weights[(V, std)] = ops.tile_head_weight(to_dev(torch, w))
        hid = (synth.normal_f16((n, H), seed, 1).astype(np.float32) * float([1.0, 0.1, 4.0][g.integers(3)])).astype(np.float16)
        remap = g.permutation(V + 1000)[:V].astype(np.int32)
        one, two = t_fused._both_forms(torch, lambda name, v: lib.get().set_option(name.encode(), int(v)), hid, fused_weights[(V, std)],
                                       to_dev(torch, remap), k)
        t_fused._assert_same(one, two, "V=%d n=%d k=%d std=%g" % (V, n, k, std))
        lib.get().synchronize()  # a wait that ran out would be an error here

    stages = [("attention", "tree attention", attention), ("heads", "tree attention with other query / KV head counts", head_counts), ("head", "target head", target_head), ("frspec", "FR-Spec head", frspec_head),
              ("topk", "top-k", topk), ("tail", "accept / compaction / tail", tail), ("draft", "draft tree", draft_tree),
              ("steps", "verify steps, eager and as graph replays", verify_steps), ("loop", "speculative loop against greedy decoding", speculative_loop),
              ("window", "drafter-layer attention: mask range, block window; window under a tree with rotary embedding", windows),
              ("merge", "attention merged inside the launch against the combine launch", merge_forms),
              ("fused", "FR-Spec head in one launch against the two-launch form", frspec_one_launch),
              ("bf16", "bfloat16: attention with fused append, target head, FR-Spec head", bf16_operators)]
    if len(argv) > 2:
        wanted = argv[2].split(",")
        unknown = [w for w in wanted if w not in [k for k, _, _ in stages]]
        if unknown:
            print("unknown stage(s) %s; stages: %s" % (unknown, ", ".join(k for k, _, _ in stages)))
            return 2
        stages = [st for st in stages if st[0] in wanted]
    for _, name, fn in stages:
        run(name, fn, budget / len(stages))
    rows = t_fused._rows_seen(lib)
    if any(rows):
        print("one-launch FR-Spec rows: %d finished from the published keys, %d redone from the logits, %d waits ran out" % rows)
    print("mismatches: %d" % len(fails))
    for f in fails:
        print(f)
    return 1 if fails else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
