#!/usr/bin/env python3
"""Writes tests/golden/vectors.npz: expected outputs of the CPU oracle for the cases in cases.py.

    python tests/golden/make_vectors.py

The reference's own tests hold no vectors and the reference cannot be imported or built in this
environment, so these fixtures do not come from the reference: they freeze the oracle's results (the
oracle itself is pinned by closed forms, library routines and brute force in test_oracle_pins.py and
by the hand-worked cases in handworked.json).  The GPU tests compare the HIP path with these
committed files; a CPU test checks that today's oracle still reproduces them.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)

import cases  # noqa: E402
import oracle  # noqa: E402


def main():
    out = {}
    for name in cases.ATTENTION_CASES:
        P, tree, q, k, v = cases.attention_inputs(name)
        out[name + "/inputs_sha"] = np.frombuffer(cases.sha(q, k, v, tree.mask).encode(), np.uint8)
        out[name + "/out"] = oracle.tree_attention(q, k, v, tree.mask, P)
    hid, w, remap = cases.head_inputs()
    c = cases.HEAD_CASE
    out["head/inputs_sha"] = np.frombuffer(cases.sha(hid, w, remap).encode(), np.uint8)
    logits = oracle.lm_head(hid, w)
    out["head/logits"] = logits
    out["head/argmax"] = oracle.argmax(logits)
    sub = oracle.lm_head(hid, oracle.gather_rows(w, remap))
    logp, m, lse = oracle.log_softmax(sub)
    val, pos = oracle.topk(logp, c["k"])
    out["head/sub_logits"] = sub
    out["head/topk_val"] = val
    out["head/topk_pos"] = pos
    out["head/topk_ids"] = oracle.remap(pos, remap)
    for name in cases.ACCEPT_CASES:
        tree, pred, gt, P, caches = cases.accept_inputs(name)
        a, node, path = oracle.tree_accept(pred, gt, tree.positions(P), P, tree.mask, tree.parent)
        ids = oracle.kv_compact(caches, P, path, gt)
        out[name + "/inputs_sha"] = np.frombuffer(cases.sha(pred, gt, tree.parent, tree.mask).encode(), np.uint8)
        out[name + "/a_node"] = np.array([a, node], np.int32)
        out[name + "/path"] = path
        out[name + "/ids"] = ids
        out[name + "/cache_sha"] = np.frombuffer(cases.sha(*[c_[:P + a] for c_ in caches]).encode(), np.uint8)
    path_out = os.path.join(HERE, "vectors.npz")
    np.savez_compressed(path_out, **out)
    print("wrote %s: %d arrays, %d bytes" % (path_out, len(out), os.path.getsize(path_out)))


if __name__ == "__main__":
    main()
