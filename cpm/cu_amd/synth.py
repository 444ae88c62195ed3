"""Seeded synthetic inputs of the verify/draft path (numpy only, deterministic across machines).

Trees follow the invariants of the reference's dynamic EAGLE tree
(src/model/eagle.cuh:188-218, src/model/minicpm4/minicpm4_eagle.cuh:319-393): node 0 is the root,
``parent[i] < i``, ``pos[i] = pos[parent[i]] + 1``, ``mask[i] = mask[parent[i]] | 1 << i``, at most
``topk`` children per node, depth <= ``num_iter``, and nodes are ordered by descending cumulative
score -- so depth is NOT monotone in the node index.
"""
from dataclasses import dataclass

import numpy as np


def rng(seed, stream=0):
    return np.random.Generator(np.random.Philox(key=[int(seed), int(stream)]))


def mask_words(T):
    return (T + 63) // 64


@dataclass
class Tree:
    parent: np.ndarray  # int32 [T], parent[0] = 0 (never read for the root)
    depth: np.ndarray   # int32 [T], root = 0
    mask: np.ndarray    # uint64 [T, W]

    @property
    def T(self):
        return int(self.parent.size)

    def positions(self, P):
        return (P + self.depth).astype(np.int32)

    def path_to(self, node):
        out = []
        while True:
            out.append(int(node))
            if node == 0:
                break
            node = int(self.parent[node])
        return out[::-1]


def masks_from_parents(parent):
    T = len(parent)
    W = mask_words(T)
    bits = [0] * T
    bits[0] = 1
    for i in range(1, T):
        bits[i] = bits[int(parent[i])] | (1 << i)
    mask = np.zeros((T, W), np.uint64)
    for i in range(T):
        for w in range(W):
            mask[i, w] = (bits[i] >> (64 * w)) & 0xFFFFFFFFFFFFFFFF
    return mask


def tree_from_parents(parent):
    parent = np.asarray(parent, np.int32).copy()
    parent[0] = 0
    depth = np.zeros(len(parent), np.int32)
    for i in range(1, len(parent)):
        assert 0 <= parent[i] < i
        depth[i] = depth[parent[i]] + 1
    return Tree(parent, depth, masks_from_parents(parent))


def chain_tree(T):
    return tree_from_parents([0] + list(range(T - 1)))


def eagle_tree(num_iter, topk, T, seed):
    """Simulates the draft loop's bookkeeping with random log-probs and keeps the T-1 best nodes."""
    g = rng(seed, 101)
    # history entries: (score, parent_history_index or -1, depth)
    hist = []
    lp = -np.sort(g.exponential(1.0, topk))  # descending log-probs
    cur = []
    for j in range(topk):
        hist.append((lp[j] - 1e-3 * j, -1, 1))
        cur.append(len(hist) - 1)
    for d in range(1, num_iter):
        cand = []
        for r, hidx in enumerate(cur):
            base = hist[hidx][0]
            lp = -np.sort(g.exponential(1.0, topk)) - 0.05
            for j in range(topk):
                hist.append((base + lp[j] - 1e-3 * j, hidx, d + 1))
                cand.append(len(hist) - 1)
        cand.sort(key=lambda h: (-hist[h][0], h))
        cur = cand[:topk]
    order = sorted(range(len(hist)), key=lambda h: (-hist[h][0], h))[: T - 1]
    node_of = {h: i + 1 for i, h in enumerate(order)}
    parent = [0] * T
    for h, i in node_of.items():
        ph = hist[h][1]
        parent[i] = 0 if ph < 0 else node_of[ph]  # scores decrease along a path, so the parent is selected
    return tree_from_parents(parent)


def random_tree(T, seed, max_children=4, max_depth=8):
    """Unstructured valid tree for property tests (parents drawn uniformly among eligible nodes)."""
    g = rng(seed, 102)
    parent = [0] * T
    depth = [0] * T
    nchild = [0] * T
    for i in range(1, T):
        elig = [j for j in range(i) if nchild[j] < max_children and depth[j] < max_depth]
        p = elig[int(g.integers(len(elig)))] if elig else 0
        parent[i] = p
        depth[i] = depth[p] + 1
        nchild[p] += 1
    return tree_from_parents(parent)


def draft_ids_for_accept(tree, gt, accept_depth, vocab, seed, leaf=None):
    """Draft ids (pred) such that greedy acceptance takes exactly ``accept_depth`` draft tokens.

    The deepest accepted node is ``leaf`` (default: a seeded choice among nodes of that depth).
    pred[i] == gt[parent[i]] along the root->leaf path; everywhere else the draft differs from the
    target's choice, and sibling tokens are distinct.  pred[0] is the root token (never compared).
    """
    g = rng(seed, 103)
    T = tree.T
    if leaf is None:
        cands = [i for i in range(T) if tree.depth[i] == accept_depth]
        assert cands, "no node at depth %d" % accept_depth
        leaf = cands[int(g.integers(len(cands)))]
    assert tree.depth[leaf] == accept_depth
    on_path = set(tree.path_to(leaf))
    pred = np.zeros(T, np.int32)
    pred[0] = int(g.integers(vocab))
    used = {}
    for i in range(1, T):
        p = int(tree.parent[i])
        taken = used.setdefault(p, set())
        if i in on_path:
            tok = int(gt[p])
        else:
            assert len(taken) + 1 < vocab, "node %d has more children than the vocabulary has distinct tokens" % p
            while True:
                tok = int(g.integers(vocab))
                if tok != int(gt[p]) and tok not in taken:
                    break
        assert tok not in taken
        taken.add(tok)
        pred[i] = tok
    return pred, leaf


def normal_f16(shape, seed, stream, std=1.0):
    return (rng(seed, stream).standard_normal(shape, dtype=np.float32) * std).astype(np.float16)


def frspec_remap(vocab, frspec_vocab, seed):
    """token_id_remap: the first ``frspec_vocab`` entries of a seeded permutation of the vocabulary."""
    return rng(seed, 104).permutation(vocab)[:frspec_vocab].astype(np.int32)


# the benchmark configurations (shapes only)
MINICPM4_8B = dict(layers=32, hidden=4096, q_heads=32, kv_heads=2, head_dim=128, vocab=73448, frspec_vocab=32768)
CONFIGS = {
    "c1_plumbing": dict(layers=1, prefix=1024, T=16, num_iter=4, topk=4, seed=0),
    "c2_verify_4k": dict(layers=32, prefix=4096, T=60, num_iter=6, topk=10, seed=0),
    "c4_verify_32k": dict(layers=32, prefix=32768, T=60, num_iter=6, topk=10, seed=0),
    "c4_verify_128k": dict(layers=32, prefix=131072, T=60, num_iter=6, topk=10, seed=0),
    "c5_wide_32k": dict(layers=32, prefix=32768, T=128, num_iter=8, topk=16, seed=0),
}


def draft_topk_rows(n, k, vocab, seed, stream=0, dyadic=False):
    """Synthetic top-k output of the draft head for n rows: log-probs <= 0 in descending order
    (fp16) and distinct positions per row.  dyadic=True draws multiples of 1/64 in (-4, 0], whose
    sums along a draft path stay exact in fp16."""
    g = rng(seed, 200 + stream)
    if dyadic:
        val = -(g.integers(0, 256, size=(n, k)).astype(np.float32) / 64.0)
    else:
        val = -np.abs(g.standard_normal((n, k)).astype(np.float32)) * 2.0
    val = -np.sort(-val, axis=1)
    pos = np.stack([g.choice(vocab, size=k, replace=False) for _ in range(n)]).astype(np.int32)
    return val.astype(np.float16), pos
