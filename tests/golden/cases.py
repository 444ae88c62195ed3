"""Definitions of the committed fixture cases: seeded inputs, rebuilt the same way by the generator
(make_vectors.py), by the CPU tests and by the GPU tests.  Inputs are not stored in the fixture file,
only their SHA-256 and the expected outputs; a changed input generator shows up as a hash mismatch.
"""
import hashlib

import numpy as np

from cpm.cu_amd import synth

HQ, HKV, D, H = 32, 2, 128, 4096

ATTENTION_CASES = {
    # name: (P, T, seed, tree kind)
    "attn_tree_p70_t6": (70, 6, 101, "random"),
    "attn_chain_p0_t5": (0, 5, 102, "chain"),
    "attn_tree_p300_t9": (300, 9, 103, "random"),
}

HEAD_CASE = dict(n=4, V=1536, Vsub=512, k=10, seed=201)

ACCEPT_CASES = {
    # name: (T, seed, accept depth)
    "accept_t16_d0": (16, 301, 0),
    "accept_t16_d3": (16, 302, 3),
    "accept_t60_d5": (60, 303, 5),
    "accept_t128_d6": (128, 304, 6),
}


def sha(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        a = np.ascontiguousarray(a)
        h.update(str(a.dtype).encode() + str(a.shape).encode() + a.tobytes())
    return h.hexdigest()


def attention_inputs(name):
    P, T, seed, kind = ATTENTION_CASES[name]
    tree = synth.chain_tree(T) if kind == "chain" else synth.random_tree(T, seed, max_children=3, max_depth=4)
    q = synth.normal_f16((T, HQ, D), seed, 1)
    k = synth.normal_f16((P + T, HKV, D), seed, 2)
    v = synth.normal_f16((P + T, HKV, D), seed, 3)
    return P, tree, q, k, v


def head_inputs():
    c = HEAD_CASE
    hid = synth.normal_f16((c["n"], H), c["seed"], 1)
    w = synth.normal_f16((c["V"], H), c["seed"], 2, 0.02)
    remap = synth.frspec_remap(c["V"], c["Vsub"], c["seed"])
    return hid, w, remap


def accept_inputs(name):
    T, seed, depth = ACCEPT_CASES[name]
    tree = synth.random_tree(T, seed, max_children=4, max_depth=8)
    depth = min(depth, int(tree.depth.max()))
    gt = synth.rng(seed, 5).integers(0, 1000, size=T).astype(np.int32)
    pred, leaf = synth.draft_ids_for_accept(tree, gt, depth, 1000, seed)
    P = 37 + T
    # two small flat caches (rows x 64 halves) that the accepted path compacts
    caches = [synth.normal_f16((P + T, 64), seed, 10 + i) for i in range(2)]
    return tree, pred, gt, P, caches
