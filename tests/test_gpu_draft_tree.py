"""GPU parity of the draft-tree construction kernels (through the C-ABI) against the CPU oracle:
every output is integer or a bit pattern, so the bar is equality."""
import numpy as np
import pytest

from cpm.cu_amd import synth
from test_draft_tree_cpu import make_rows, run_oracle
from util import to_dev, to_np

pytestmark = pytest.mark.gpu


def run_gpu(torch, k, num_iter, T, P, vals, poss, remap):
    from cpm.cu_amd import ops
    t = ops.DraftTree(k, num_iter, None if remap is None else to_dev(torch, remap))
    trace = [to_np(t.begin(to_dev(torch, vals[0][0]), to_dev(torch, poss[0][0]))).copy()]
    cums = []
    for d in range(1, num_iter):
        v = to_dev(torch, vals[d])
        ids, rows, mask = t.extend(d, v, to_dev(torch, poss[d]))
        torch.cuda.synchronize()
        trace.append((to_np(ids).copy(), to_np(rows).copy(), to_np(mask).view(np.uint64).copy()))
        cums.append(to_np(v))
    cl = torch.tensor([P], dtype=torch.int32, device="cuda")
    ids, pos, mask, parent = t.finish(T, cl)
    torch.cuda.synchronize()
    return (to_np(ids), to_np(pos), to_np(mask).view(np.uint64), to_np(parent)), trace, cums


@pytest.mark.parametrize("k,num_iter,T,seed,with_remap,dyadic", [(2, 2, 4, 1, False, True), (3, 3, 10, 2, True, False),
                                                                  (10, 6, 60, 4, True, False), (10, 6, 64, 5, False, True),
                                                                  (8, 8, 32, 6, True, False), (10, 3, 128, 7, True, False),
                                                                  (32, 2, 100, 8, True, False), (1, 5, 5, 9, False, False)])
def test_draft_tree_equals_oracle(gpu, orc, k, num_iter, T, seed, with_remap, dyadic):
    torch = gpu
    vocab, full = 500, 2000
    remap = synth.frspec_remap(full, vocab, seed) if with_remap else None
    vals, poss = make_rows(k, num_iter, vocab, seed, dyadic=dyadic)
    P = 4096 + seed
    (o_ids, o_pos, o_mask, o_parent), o_trace = run_oracle(orc, k, num_iter, T, P, vals, poss, remap)
    (g_ids, g_pos, g_mask, g_parent), g_trace, _ = run_gpu(torch, k, num_iter, T, P, vals, poss, remap)
    assert np.array_equal(g_trace[0], o_trace[0])
    for d in range(1, num_iter):
        for a, b in zip(g_trace[d], o_trace[d]):
            assert np.array_equal(a, b), "iteration %d" % d
    assert np.array_equal(g_ids[1:], o_ids[1:]) and g_ids[0] == -1
    assert np.array_equal(g_pos, o_pos) and np.array_equal(g_parent, o_parent)
    assert np.array_equal(g_mask, o_mask)


def test_heavy_ties(gpu, orc):
    """All log-probs equal: every choice is made by the index rule alone."""
    torch = gpu
    k, num_iter, T = 4, 4, 20
    vals = [np.full((1 if d == 0 else k, k), -0.5, np.float16) for d in range(num_iter)]
    poss = [np.arange((1 if d == 0 else k) * k, dtype=np.int32).reshape(-1, k) + 10 * d for d in range(num_iter)]
    (o_ids, o_pos, o_mask, o_parent), _ = run_oracle(orc, k, num_iter, T, 7, vals, poss, None)
    (g_ids, g_pos, g_mask, g_parent), _, _ = run_gpu(torch, k, num_iter, T, 7, vals, poss, None)
    assert np.array_equal(g_ids[1:], o_ids[1:]) and np.array_equal(g_pos, o_pos)
    assert np.array_equal(g_parent, o_parent) and np.array_equal(g_mask, o_mask)


def test_tree_feeds_the_verify_path(gpu, orc):
    """The tree the draft kernels build is consumed as is by acceptance: plant the target's choices
    along one root path of the built tree and check the accept length."""
    from cpm.cu_amd import ops
    torch = gpu
    k, num_iter, T, P = 10, 6, 60, 4096
    vocab, full = 500, 2000
    remap = synth.frspec_remap(full, vocab, 11)
    vals, poss = make_rows(k, num_iter, vocab, 11, dyadic=False)
    t = ops.DraftTree(k, num_iter, to_dev(torch, remap))
    t.begin(to_dev(torch, vals[0][0]), to_dev(torch, poss[0][0]))
    for d in range(1, num_iter):
        t.extend(d, to_dev(torch, vals[d]), to_dev(torch, poss[d]))
    cl = torch.tensor([P], dtype=torch.int32, device="cuda")
    ids = torch.full((T,), -1, dtype=torch.int32, device="cuda")
    ids[0] = 1234  # the root token is the caller's
    ids, pos, mask, parent = t.finish(T, cl, tree_draft_ids=ids)
    torch.cuda.synchronize()
    ids_np, par_np = to_np(ids), to_np(parent)
    depth = to_np(pos) - P
    leaf = int(np.argmax(depth))  # a deepest node
    path = [leaf]
    while path[-1] != 0:
        path.append(int(par_np[path[-1]]))
    path = path[::-1]
    gt = np.full(T, full + 5, np.int32)  # matches nothing ...
    for a, b in zip(path[:-1], path[1:]):
        gt[a] = ids_np[b]                # ... except along the chosen path
    pred = ids.clone()
    best = ops.tree_accept(pred, to_dev(torch, gt), pos, cl, mask, parent)
    torch.cuda.synchronize()
    assert int(best[0]) == len(path) and int(best[1]) == leaf
    assert to_np(pred)[:len(path)].tolist() == path


def test_argument_errors(gpu):
    from cpm.cu_amd import ops
    with pytest.raises(ValueError):
        ops.DraftTree(10, 7).begin(gpu.zeros(10, dtype=gpu.float16, device="cuda"), gpu.zeros(10, dtype=gpu.int32, device="cuda"))
