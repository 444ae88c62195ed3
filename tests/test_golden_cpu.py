"""The CPU oracle against the committed fixtures: the hand-worked cases (answers derived from the
definitions, independent of any code here) and the frozen vectors of tests/golden/vectors.npz."""
import json
import os
import sys

import numpy as np
import pytest

from cpm.cu_amd import synth

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLD)
import cases  # noqa: E402


@pytest.fixture(scope="module")
def hand():
    with open(os.path.join(GOLD, "handworked.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(GOLD, "vectors.npz"), allow_pickle=False)


def uniform_attention_inputs(c):
    """K = 0 everywhere, V rows constant: the output of row i is the mean of the V constants it sees."""
    tree = synth.tree_from_parents(c["tree_parent"])
    P, T = len(c["prefix_v"]), tree.T
    vals = np.array(c["prefix_v"] + c["tree_v"], np.float16)
    q = synth.normal_f16((T, cases.HQ, cases.D), 7, 1)
    k = np.zeros((P + T, cases.HKV, cases.D), np.float16)
    v = np.broadcast_to(vals[:, None, None], (P + T, cases.HKV, cases.D)).astype(np.float16).copy()
    return tree, P, q, k, v


def test_hand_attention_uniform(orc, hand):
    c = hand["attention_uniform"]
    tree, P, q, k, v = uniform_attention_inputs(c)
    out = orc.tree_attention(q, k, v, tree.mask, P).astype(np.float32)
    for i, e in enumerate(c["expected"]):
        assert np.allclose(out[i], e, atol=2e-3), (i, out[i].min(), out[i].max(), e)


def test_hand_accept(orc, hand):
    for c in hand["accept"]:
        tree = synth.tree_from_parents(c["parent"])
        P = 9
        a, node, path = orc.tree_accept(c["pred"], c["gt"], tree.positions(P), P, tree.mask, tree.parent)
        assert a == c["a"] and path.tolist() == c["path"] and node == c["path"][-1], c["_comment"]
        assert np.asarray(c["gt"])[path].tolist() == c["ids"]


def test_hand_compact(orc, hand):
    c = hand["compact"]
    cache = np.repeat(np.array(c["rows"], np.float16)[:, None], 8, axis=1).copy()
    gt = np.arange(4, dtype=np.int32)
    orc.kv_compact([cache], c["P"], c["path"], gt)
    n = len(c["expected_prefix"])
    assert cache[:n, 0].tolist() == c["expected_prefix"] and np.all(cache[:n] == cache[:n, :1])


def test_hand_topk_argmax(orc, hand):
    for c in hand["topk"]:
        val, pos = orc.topk(np.array([c["x"]], np.float16), c["k"])
        assert val[0].astype(np.float32).tolist() == c["val"] and pos[0].tolist() == c["pos"], c["_comment"]
    for c in hand["argmax"]:
        assert int(orc.argmax(np.array([c["x"]], np.float16))[0]) == c["expected"]


def _sha(a):
    return bytes(a).decode()


def test_frozen_attention(orc, vec):
    for name in cases.ATTENTION_CASES:
        P, tree, q, k, v = cases.attention_inputs(name)
        assert cases.sha(q, k, v, tree.mask) == _sha(vec[name + "/inputs_sha"]), "input generator changed: regenerate the fixtures"
        out = orc.tree_attention(q, k, v, tree.mask, P)
        assert np.array_equal(out.view(np.uint16), vec[name + "/out"].view(np.uint16)), name


def test_frozen_head_topk(orc, vec):
    hid, w, remap = cases.head_inputs()
    assert cases.sha(hid, w, remap) == _sha(vec["head/inputs_sha"])
    logits = orc.lm_head(hid, w)
    assert np.array_equal(logits.view(np.uint16), vec["head/logits"].view(np.uint16))
    assert np.array_equal(orc.argmax(logits), vec["head/argmax"])
    sub = orc.lm_head(hid, orc.gather_rows(w, remap))
    assert np.array_equal(sub.view(np.uint16), vec["head/sub_logits"].view(np.uint16))
    logp, _, _ = orc.log_softmax(sub)
    val, pos = orc.topk(logp, cases.HEAD_CASE["k"])
    assert np.array_equal(val.view(np.uint16), vec["head/topk_val"].view(np.uint16))
    assert np.array_equal(pos, vec["head/topk_pos"]) and np.array_equal(orc.remap(pos, remap), vec["head/topk_ids"])


def test_frozen_accept_compact(orc, vec):
    for name in cases.ACCEPT_CASES:
        tree, pred, gt, P, caches = cases.accept_inputs(name)
        assert cases.sha(pred, gt, tree.parent, tree.mask) == _sha(vec[name + "/inputs_sha"])
        a, node, path = orc.tree_accept(pred, gt, tree.positions(P), P, tree.mask, tree.parent)
        assert [a, node] == vec[name + "/a_node"].tolist() and np.array_equal(path, vec[name + "/path"])
        ids = orc.kv_compact(caches, P, path, gt)
        assert np.array_equal(ids, vec[name + "/ids"])
        assert cases.sha(*[c[:P + a] for c in caches]) == _sha(vec[name + "/cache_sha"])
