"""The HIP path (through the C-ABI) against the committed fixtures: the hand-worked cases of
tests/golden/handworked.json and the frozen vectors of tests/golden/vectors.npz.  Integer results
must be equal; fp16 results within max-abs 2e-2 / max-rel 1e-2 (tests/util.py)."""
import json
import os
import sys

import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLD)
import cases  # noqa: E402
from test_golden_cpu import uniform_attention_inputs  # noqa: E402


@pytest.fixture(scope="module")
def hand():
    with open(os.path.join(GOLD, "handworked.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(GOLD, "vectors.npz"), allow_pickle=False)


def _attend(torch, P, tree, q, k, v, fused):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    S = P + tree.T
    npages = (S + 255) // 256 + 1
    cache = PagedKVCache(1, cases.HKV, npages, block_table=np.arange(npages)[::-1].copy(), fill=float("nan"))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    if fused:
        if P:
            cache.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
        out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, tree.mask),
                                 k_new=to_dev(torch, k[P:]), v_new=to_dev(torch, v[P:]))
    else:
        cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
        out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, tree.mask))
    torch.cuda.synchronize()
    return to_np(out)


@pytest.mark.parametrize("fused", [False, True])
def test_hand_attention_uniform(gpu, hand, fused):
    c = hand["attention_uniform"]
    tree, P, q, k, v = uniform_attention_inputs(c)
    out = _attend(gpu, P, tree, q, k, v, fused).astype(np.float32)
    for i, e in enumerate(c["expected"]):
        assert np.allclose(out[i], e, atol=4e-3), (i, out[i].min(), out[i].max(), e)


@pytest.mark.parametrize("fused", [False, True])
def test_frozen_attention(gpu, vec, fused):
    for name in cases.ATTENTION_CASES:
        P, tree, q, k, v = cases.attention_inputs(name)
        assert cases.sha(q, k, v, tree.mask) == bytes(vec[name + "/inputs_sha"]).decode()
        assert_close_f16(_attend(gpu, P, tree, q, k, v, fused), vec[name + "/out"], name)


def test_hand_accept_and_compact(gpu, hand):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    for c in hand["accept"]:
        tree = synth.tree_from_parents(c["parent"])
        T, P = tree.T, 9
        pred = to_dev(torch, np.array(c["pred"], np.int32))
        gt = to_dev(torch, np.array(c["gt"], np.int32))
        cl = torch.tensor([P], dtype=torch.int32, device="cuda")
        best = ops.tree_accept(pred, gt, to_dev(torch, tree.positions(P)), cl, to_dev(torch, tree.mask), to_dev(torch, tree.parent))
        torch.cuda.synchronize()
        a, node = (int(x) for x in best.cpu())
        assert a == c["a"] and node == c["path"][-1] and to_np(pred)[:a].tolist() == c["path"], c["_comment"]
    # compaction with the overlapping path of the fixture, rows labelled by constants
    c = hand["compact"]
    P, path = c["P"], c["path"]
    rows = np.array(c["rows"], np.float16)
    T = len(rows) - P
    cache = PagedKVCache(2, cases.HKV, 1)
    full = np.broadcast_to(rows[:, None, None], (len(rows), cases.HKV, cases.D)).astype(np.float16).copy()
    for l in range(2):
        cache.write_logical(l, 0, to_dev(torch, full), to_dev(torch, full + 0.5))
    pred = torch.zeros(T, dtype=torch.int32, device="cuda")
    pred[:len(path)] = to_dev(torch, np.array(path, np.int32))
    gt = to_dev(torch, (np.arange(T) + 70).astype(np.int32))
    best = to_dev(torch, np.array([len(path), path[-1]], np.int32))
    ops.kv_compact(cache, pred, gt, torch.tensor([P], dtype=torch.int32, device="cuda"), best, T)
    torch.cuda.synchronize()
    n = len(c["expected_prefix"])
    for l in range(2):
        kk, vv = cache.read_logical(l, 0, n)
        assert to_np(kk)[:, 0, 0].tolist() == c["expected_prefix"] and bool((kk == kk[:, :1, :1]).all())
        assert (to_np(vv)[:, 0, 0] - 0.5).tolist() == c["expected_prefix"] and bool((vv == vv[:, :1, :1]).all())
    assert to_np(pred)[:len(path)].tolist() == [70 + p for p in path]  # pred[:a] <- accepted ids


def test_hand_topk_argmax(gpu, hand):
    from cpm.cu_amd import ops
    torch = gpu
    for c in hand["topk"]:
        val, pos = ops.topk(to_dev(torch, np.array([c["x"]], np.float16)), c["k"])
        torch.cuda.synchronize()
        assert to_np(val)[0].astype(np.float32).tolist() == c["val"] and to_np(pos)[0].tolist() == c["pos"], c["_comment"]
    # arg-max through the head: an identity-like weight matrix reproduces x as the logits
    for c in hand["argmax"]:
        x = np.array(c["x"], np.float16)
        w = np.zeros((len(x), cases.H), np.float16)
        w[:, 0] = x
        hid = np.zeros((1, cases.H), np.float16)
        hid[0, 0] = 1.0
        gt = ops.lm_head_argmax(to_dev(torch, hid), to_dev(torch, w))
        torch.cuda.synchronize()
        assert int(gt[0]) == c["expected"]


def test_frozen_head_topk(gpu, vec):
    from cpm.cu_amd import ops
    torch = gpu
    hid, w, remap = cases.head_inputs()
    k = cases.HEAD_CASE["k"]
    gt, logits = ops.lm_head_argmax(to_dev(torch, hid), to_dev(torch, w), want_logits=True)
    torch.cuda.synchronize()
    assert_close_f16(to_np(logits), vec["head/logits"], "target head logits")
    ref = vec["head/logits"].astype(np.float32)
    for i in range(hid.shape[0]):  # equal unless the deciding margin is inside the logit tolerance
        if int(gt[i]) != int(vec["head/argmax"][i]):
            assert abs(ref[i, int(gt[i])] - ref[i].max()) <= 2e-2
    w_sub = ops.gather_rows(to_dev(torch, w), to_dev(torch, remap))
    r = ops.frspec_head_topk(to_dev(torch, hid), w_sub, to_dev(torch, remap), k)
    torch.cuda.synchronize()
    assert_close_f16(to_np(r["logits"]), vec["head/sub_logits"], "FR-Spec logits")
    assert_close_f16(to_np(r["val"]), vec["head/topk_val"], "top-k log-probs")
    pos, ids = to_np(r["pos"]), to_np(r["ids"])
    assert np.array_equal(ids, remap[pos])
    sub = vec["head/sub_logits"].astype(np.float32)
    for i in range(hid.shape[0]):  # same candidates unless separated by less than the tolerance
        kth = np.sort(sub[i])[-k]
        assert np.all(sub[i, pos[i]] >= kth - 2e-2)
        if np.all(np.abs(np.diff(np.sort(sub[i])[-k - 1:])) > 4e-2):
            assert pos[i].tolist() == vec["head/topk_pos"][i].tolist() and ids[i].tolist() == vec["head/topk_ids"][i].tolist()


def test_frozen_accept_compact(gpu, vec):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    for name in cases.ACCEPT_CASES:
        tree, pred_np, gt_np, P, _ = cases.accept_inputs(name)
        T = tree.T
        S = P + T
        npages = (S + 255) // 256
        cache = PagedKVCache(2, cases.HKV, npages)
        kv = [(synth.normal_f16((S, cases.HKV, cases.D), 900 + l, 1), synth.normal_f16((S, cases.HKV, cases.D), 900 + l, 2)) for l in range(2)]
        for l in range(2):
            cache.write_logical(l, 0, to_dev(torch, kv[l][0]), to_dev(torch, kv[l][1]))
        pred, gt = to_dev(torch, pred_np), to_dev(torch, gt_np)
        cl = torch.tensor([P], dtype=torch.int32, device="cuda")
        best = ops.tree_accept(pred, gt, to_dev(torch, tree.positions(P)), cl, to_dev(torch, tree.mask), to_dev(torch, tree.parent))
        ops.kv_compact(cache, pred, gt, cl, best, T)
        torch.cuda.synchronize()
        a, node = vec[name + "/a_node"].tolist()
        path = vec[name + "/path"]
        assert [int(x) for x in best.cpu()] == [a, node], name
        assert np.array_equal(to_np(pred)[:a], vec[name + "/ids"]), name
        for l in range(2):
            kk, vv = cache.read_logical(l, 0, P + a)
            want_k = np.concatenate([kv[l][0][:P], kv[l][0][P + path]])
            want_v = np.concatenate([kv[l][1][:P], kv[l][1][P + path]])
            assert np.array_equal(to_np(kk).view(np.uint16), want_k.view(np.uint16)), name
            assert np.array_equal(to_np(vv).view(np.uint16), want_v.view(np.uint16)), name
