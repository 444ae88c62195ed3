"""Consecutive verify steps with everything length-related on the device: the one-call tail of
verify() advances the prefix length, and one captured HIP graph per padded length is replayed
(the reference keys its decode graph on (padded_length, T), src/entry.cu:475-492, and sets the length
from the host every iteration, cpmcu/speculative/tree_drafter.py:222).

The same sequence of steps is run twice on identical inputs: eagerly, with the host writing the
prefix length before every step as the reference's loop does, and as graph replays in which the host
writes nothing but the step's inputs.  Accept lengths, accepted ids and the whole cache must agree
bit for bit; attention outputs agree to fp16 rounding (the two runs bound the KV length differently,
which moves the split boundaries).
"""
import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 2, 128
LAYERS, H, VOCAB, T = 3, 512, 2048, 24
P0, STEPS = 1000, 14


def _prefill(torch, cache, seed):
    for layer in range(LAYERS):
        k = synth.normal_f16((P0, HKV, D), seed, 10 + layer)
        v = synth.normal_f16((P0, HKV, D), seed, 50 + layer)
        cache.write_logical(layer, 0, to_dev(torch, k), to_dev(torch, v))


def test_graph_replayed_steps_equal_host_driven_steps(gpu, orc):
    from cpm.cu_amd import ops
    from cpm.cu_amd.driver import GraphedSteps, VerifyStep
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    seed = 3
    tree = synth.random_tree(T, seed, max_children=3, max_depth=6)
    depth = torch.from_numpy(tree.depth.astype(np.int32)).cuda()
    mask = torch.from_numpy(tree.mask.view(np.int64)).cuda()
    parent = to_dev(torch, tree.parent)
    head = to_dev(torch, synth.normal_f16((VOCAB, H), seed, 2, std=0.02))
    npages = (P0 + STEPS * 7 + T + 255) // 256 + 2
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32)

    # per-step inputs; the draft ids are rigged on the device's own arg-max so that the accept length is known
    inputs = []
    rg = synth.rng(seed, 8)
    for s in range(STEPS):
        q = [to_dev(torch, synth.normal_f16((T, HQ, D), seed, 1000 + 10 * s + l)) for l in range(LAYERS)]
        k = [to_dev(torch, synth.normal_f16((T, HKV, D), seed, 2000 + 10 * s + l)) for l in range(LAYERS)]
        v = [to_dev(torch, synth.normal_f16((T, HKV, D), seed, 3000 + 10 * s + l)) for l in range(LAYERS)]
        hidden = to_dev(torch, synth.normal_f16((T, H), seed, 4000 + s))
        gt = to_np(ops.lm_head_argmax(hidden, head))
        want_depth = int(rg.integers(0, int(tree.depth.max()) + 1))
        pred, leaf = synth.draft_ids_for_accept(tree, gt, want_depth, VOCAB, seed * 100 + s)
        inputs.append(dict(q=q, k=k, v=v, hidden=hidden, pred=to_dev(torch, pred), gt=gt, depth=want_depth, path=tree.path_to(leaf)))

    # run 1: eager, the host sets the lengths before every step
    cache_a = PagedKVCache(LAYERS, HKV, npages, block_table=table)
    _prefill(torch, cache_a, seed)
    P = P0
    hist_a, outs_a = [], []
    for s, x in enumerate(inputs):
        pos = torch.from_numpy(tree.positions(P)).cuda()
        st = VerifyStep(cache_a, head, mask, parent, pos, P)
        st.enqueue(x["q"], x["k"], x["v"], x["hidden"], x["pred"])
        a, ids = st.result()
        assert a == x["depth"] + 1 and np.array_equal(ids, x["gt"][x["path"]])
        hist_a.append((a, ids.tolist()))
        outs_a.append(to_np(st.attn_out).copy())
        P += a

    # run 2: graph replays, lengths advance on the device
    cache_b = PagedKVCache(LAYERS, HKV, npages, block_table=table)
    _prefill(torch, cache_b, seed)
    step = VerifyStep(cache_b, head, mask, parent, torch.from_numpy(tree.positions(P0)).cuda(), P0, commit=True)
    gs = GraphedSteps(step, LAYERS, HQ, HKV, H, pad_to=32)
    bq, bk, bv, bh, bd = gs.buffers()
    Pb = P0
    for s, x in enumerate(inputs):
        for l in range(LAYERS):
            bq[l].copy_(x["q"][l])
            bk[l].copy_(x["k"][l])
            bv[l].copy_(x["v"][l])
        bh.copy_(x["hidden"])
        bd.copy_(x["pred"])
        # (the tree positions follow the device-side prefix length by themselves: the step's tail advances them)
        assert np.array_equal(to_np(step.pos), tree.positions(Pb))
        a, ids = gs.run()
        assert (a, ids.tolist()) == hist_a[s], "step %d: graph replay (%d, %s) vs host-driven %s" % (s, a, ids.tolist(), hist_a[s])
        assert np.array_equal(to_np(step.prev_hidden)[:a].view(np.uint16), to_np(x["hidden"])[x["path"]].view(np.uint16))
        assert np.array_equal(to_np(step.next_positions)[:a], Pb + np.arange(a))
        assert_close_f16(to_np(gs.attn_out[LAYERS - 1]), outs_a[s], "attention output of step %d" % s)
        Pb += a
        assert int(to_np(step.cache_length)[0]) == Pb and int(to_np(step.kv_len)[0]) == Pb + T
    assert Pb == P and len(gs.graphs) >= 2, "the run should have crossed a padded length (%d graphs)" % len(gs.graphs)

    for layer in range(LAYERS):
        ka, va = cache_a.read_logical(layer, 0, P)
        kb, vb = cache_b.read_logical(layer, 0, P)
        assert np.array_equal(to_np(ka).view(np.uint16), to_np(kb).view(np.uint16))
        assert np.array_equal(to_np(va).view(np.uint16), to_np(vb).view(np.uint16))
