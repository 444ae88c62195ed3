"""Oracle pins for the draft-tree construction (src/model/minicpm4/minicpm4_eagle.cuh:319-393):
an independent reconstruction with explicit node records, and a hand-worked case."""
import numpy as np
import pytest

from cpm.cu_amd import synth


class Node:
    def __init__(self, idx, parent, token, logp, depth):
        self.idx, self.parent, self.token, self.logp, self.depth = idx, parent, token, logp, depth


def reconstruct(k, num_iter, T, P, rows_val, rows_pos, remap):
    """Independent statement of what the drafter builds: every candidate the draft visits is a node
    with a parent and a cumulative log-prob (exact arithmetic on dyadic inputs); each iteration
    keeps the k best new candidates alive; the tree is the T-1 best candidates overall, ordered by
    (log-prob descending, visiting order), and each one's mask is itself plus its ancestors."""
    nodes = []  # visiting order == index in the reference's history arrays
    live = []
    v, p = rows_val[0][0], rows_pos[0][0]
    for j in range(k):
        nodes.append(Node(len(nodes), None, int(p[j]), float(v[j]), 1))
        live.append(nodes[-1])
    for d in range(1, num_iter):
        new = []
        for i, par in enumerate(live):
            for j in range(k):
                nd = Node(len(nodes), par, int(rows_pos[d][i][j]), par.logp + float(rows_val[d][i][j]), d + 1)
                nodes.append(nd)
                new.append(nd)
        live = sorted(new, key=lambda n: (-n.logp, n.idx))[:k]
    chosen = sorted(nodes, key=lambda n: (-n.logp, n.idx))[:T - 1]
    index_of = {n.idx: i + 1 for i, n in enumerate(chosen)}
    ids, pos, parent, mask = [-1], [P], [0], [1]
    for i, n in enumerate(chosen, start=1):
        ids.append(int(remap[n.token]) if remap is not None else n.token)
        pos.append(P + n.depth)
        par = 0 if n.parent is None else index_of[n.parent.idx]
        parent.append(par)
        m, a = 1 << i, n.parent
        while a is not None:
            m |= 1 << index_of[a.idx]
            a = a.parent
        mask.append(m | 1)
    return ids, pos, parent, mask


def run_oracle(orc, k, num_iter, T, P, rows_val, rows_pos, remap):
    t = orc.DraftTree(k, num_iter, remap)
    trace = [t.begin(rows_val[0][0], rows_pos[0][0]).copy()]
    for d in range(1, num_iter):
        ids, rows, _ = t.extend(d, rows_val[d], rows_pos[d])
        trace.append((ids.copy(), rows.copy(), t.mask.copy()))
    return t.finish(T, P), trace


def make_rows(k, num_iter, vocab, seed, dyadic=True):
    vals, poss = [], []
    for d in range(num_iter):
        n = 1 if d == 0 else k
        v, p = synth.draft_topk_rows(n, k, vocab, seed, stream=d, dyadic=dyadic)
        vals.append(v)
        poss.append(p)
    return vals, poss


@pytest.mark.parametrize("k,num_iter,T,seed,with_remap", [(2, 2, 4, 1, False), (3, 3, 10, 2, True), (4, 4, 16, 3, True),
                                                           (10, 6, 60, 4, True), (10, 6, 64, 5, False), (8, 8, 32, 6, True),
                                                           (10, 3, 128, 7, True)])
def test_oracle_matches_reconstruction(orc, k, num_iter, T, seed, with_remap):
    vocab, full = 500, 2000
    remap = synth.frspec_remap(full, vocab, seed) if with_remap else None
    vals, poss = make_rows(k, num_iter, vocab, seed)
    P = 100 + seed
    (ids, pos, mask, parent), _ = run_oracle(orc, k, num_iter, T, P, vals, poss, remap)
    r_ids, r_pos, r_parent, r_mask = reconstruct(k, num_iter, T, P, vals, poss, remap)
    assert ids.tolist() == r_ids and pos.tolist() == r_pos and parent.tolist() == r_parent
    got = [sum(int(mask[i, w]) << (64 * w) for w in range(mask.shape[1])) for i in range(T)]
    assert got == r_mask
    # structural invariants of the tree the verify path consumes
    for i in range(1, T):
        assert parent[i] < i and pos[i] == pos[parent[i]] + 1
        assert got[i] == got[parent[i]] | (1 << i)


def test_hand_worked_two_iterations(orc):
    """k = 2, two iterations, worked out by hand: first row -0.5 (token 7), -1.0 (token 3); the
    children of the first are -0.25 (1), -2 (2), of the second -0.125 (5), -0.5 (6).  Cumulative:
    -0.75, -2.5, -1.125, -1.5.  The three best of all six are -0.5, -0.75, -1.0: the first
    candidate, its first child, the second candidate."""
    t = orc.DraftTree(2, 2)
    assert t.begin(np.array([-0.5, -1.0], np.float16), [7, 3]).tolist() == [7, 3]
    ids, rows, cum = t.extend(1, np.array([[-0.25, -2], [-0.125, -0.5]], np.float16), [[1, 2], [5, 6]])
    assert cum.astype(np.float32).tolist() == [[-0.75, -2.5], [-1.125, -1.5]]
    assert ids.tolist() == [1, 5] and rows.tolist() == [0, 1] and t.mask.tolist() == [0b0101, 0b1010]
    ids, pos, mask, parent = t.finish(4, 10)
    assert ids.tolist() == [-1, 7, 1, 3] and pos.tolist() == [10, 11, 12, 11]
    assert parent.tolist() == [0, 0, 1, 0] and mask[:, 0].tolist() == [0b0001, 0b0011, 0b0111, 0b1001]


def test_fp16_cumsum_rounding(orc):
    """cumsum adds in half precision (src/model/eagle.cuh:103-106): 1024 + 0.5 rounds to 1024."""
    t = orc.DraftTree(1, 2)
    t.begin(np.array([-1024.0], np.float16), [0])
    _, _, cum = t.extend(1, np.array([[-0.5]], np.float16), [[0]])
    assert float(cum[0, 0]) == -1024.0
