"""GPU parity of greedy tree acceptance and accepted-path KV compaction (bit-exact) and of the
model-level entry points that mirror the reference's pybind module, all through the C-ABI."""
import ctypes

import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 2, 128
VOCAB = 73448


def _accept_case(torch, orc, tree, P, pred, gt):
    from cpm.cu_amd import ops
    pos = tree.positions(P)
    d_pred = to_dev(torch, pred)
    best = ops.tree_accept(d_pred, to_dev(torch, gt), to_dev(torch, pos), torch.tensor([P], dtype=torch.int32, device="cuda"),
                           to_dev(torch, tree.mask), to_dev(torch, tree.parent))
    torch.cuda.synchronize()
    a_ref, node_ref, path_ref = orc.tree_accept(pred, gt, pos, P, tree.mask, tree.parent)
    best = to_np(best)
    assert best[0] == a_ref and best[1] == node_ref
    assert np.array_equal(to_np(d_pred)[:a_ref], path_ref)
    return a_ref, path_ref


@pytest.mark.parametrize("T,num_iter,topk", [(16, 4, 4), (60, 6, 10), (64, 6, 10), (128, 8, 16), (100, 8, 16)])
def test_accept_rigged_depths(gpu, orc, T, num_iter, topk):
    """Every reachable accept length, on EAGLE-shaped trees whose depth is not monotone in the index."""
    for seed in range(4):
        tree = synth.eagle_tree(num_iter, topk, T, seed)
        gt = synth.rng(seed, 9).integers(0, VOCAB, T).astype(np.int32)
        for depth in range(int(tree.depth.max()) + 1):
            pred, leaf = synth.draft_ids_for_accept(tree, gt, depth, VOCAB, seed * 100 + depth)
            a, path = _accept_case(gpu, orc, tree, 4096 + seed, pred, gt)
            assert a == depth + 1 and list(path) == tree.path_to(leaf)


def test_accept_random_and_duplicate_siblings(gpu, orc):
    """Tiny vocabulary: many accidental matches and duplicate sibling tokens -> the tournament's tie rule matters."""
    for seed in range(40):
        T = int(synth.rng(seed, 1).integers(1, 129))
        tree = synth.random_tree(T, seed, max_children=6, max_depth=12)
        g = synth.rng(seed, 2)
        pred = g.integers(0, 3, T).astype(np.int32)
        gt = g.integers(0, 3, T).astype(np.int32)
        _accept_case(gpu, orc, tree, int(g.integers(0, 100000)), pred, gt)


def _compact_case(torch, orc, tree, P, leaf_depth, layers, seed, page_perm=True):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    T = tree.T
    S = P + T
    npages = (S + 255) // 256 + 1
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32) if page_perm else None
    cache = PagedKVCache(layers, HKV, npages, block_table=table)
    flat = []
    for layer in range(layers):
        k = synth.normal_f16((S, HKV, D), seed, 10 + layer)
        v = synth.normal_f16((S, HKV, D), seed, 50 + layer)
        cache.write_logical(layer, 0, to_dev(torch, k), to_dev(torch, v))
        flat += [k.reshape(S, HKV * D).copy(), v.reshape(S, HKV * D).copy()]
    gt = synth.rng(seed, 9).integers(0, VOCAB, T).astype(np.int32)
    pred, leaf = synth.draft_ids_for_accept(tree, gt, leaf_depth, VOCAB, seed)
    pos = tree.positions(P)
    d_pred, d_gt = to_dev(torch, pred), to_dev(torch, gt)
    d_P = torch.tensor([P], dtype=torch.int32, device="cuda")
    best = ops.tree_accept(d_pred, d_gt, to_dev(torch, pos), d_P, to_dev(torch, tree.mask), to_dev(torch, tree.parent))
    ops.kv_compact(cache, d_pred, d_gt, d_P, best, T)
    torch.cuda.synchronize()
    a, _, path = orc.tree_accept(pred, gt, pos, P, tree.mask, tree.parent)
    ids = orc.kv_compact(flat, P, path, gt)
    assert to_np(best)[0] == a
    assert np.array_equal(to_np(d_pred)[:a], ids)  # accepted token ids
    assert np.array_equal(ids, gt[path])
    for layer in range(layers):
        k_dev, v_dev = cache.read_logical(layer, 0, P + a)
        assert np.array_equal(to_np(k_dev).reshape(P + a, -1).view(np.uint16), flat[2 * layer][: P + a].view(np.uint16))
        assert np.array_equal(to_np(v_dev).reshape(P + a, -1).view(np.uint16), flat[2 * layer + 1][: P + a].view(np.uint16))
    return a, path


def test_compaction_config_shapes(gpu, orc):
    tree = synth.eagle_tree(6, 10, 60, seed=0)
    for depth in range(int(tree.depth.max()) + 1):
        _compact_case(gpu, orc, tree, 4096 - 7, depth, layers=4, seed=depth)
    wide = synth.eagle_tree(8, 16, 128, seed=1)
    for depth in (0, 3, int(wide.depth.max())):
        _compact_case(gpu, orc, wide, 1000, depth, layers=3, seed=20 + depth)


def test_compaction_overlap_and_long_paths(gpu, orc):
    """path = [0, 2, 3]: row P+2 is a source for d=1 and a destination for d=2; plus a 128-long chain
    path (several read/write batches) and the identity path."""
    t = synth.tree_from_parents([0, 0, 0, 2])  # nodes 2 and 3 form the path 0 -> 2 -> 3
    a, path = _compact_case(gpu, orc, t, 300, 2, layers=2, seed=1)
    assert list(path) == [0, 2, 3]
    chain = synth.chain_tree(128)
    a, path = _compact_case(gpu, orc, chain, 250, 127, layers=2, seed=2)
    assert a == 128 and list(path) == list(range(128))
    # a deep path with gaps: every second node of a chain-with-twigs
    parents = [0]
    for i in range(1, 100):
        parents.append(i - 1 if i % 2 == 0 else max(i - 2, 0))
    _compact_case(gpu, orc, synth.tree_from_parents(parents), 511, 49, layers=2, seed=3)


def _commit_case(torch, orc, tree, P, leaf_depth, layers, seed, H=512, pinned_result=False):
    """cpmcu_accept_commit against the oracle's restatement of verify()'s tail and against the separate operators."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    T = tree.T
    S = P + T
    npages = (S + 255) // 256 + 1
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32)
    caches = [PagedKVCache(layers, HKV, npages, block_table=table) for _ in range(2)]
    flat = []
    for layer in range(layers):
        k = synth.normal_f16((S, HKV, D), seed, 10 + layer)
        v = synth.normal_f16((S, HKV, D), seed, 50 + layer)
        for c in caches:
            c.write_logical(layer, 0, to_dev(torch, k), to_dev(torch, v))
        flat += [k.reshape(S, HKV * D).copy(), v.reshape(S, HKV * D).copy()]
    gt = synth.rng(seed, 9).integers(0, VOCAB, T).astype(np.int32)
    pred, leaf = synth.draft_ids_for_accept(tree, gt, leaf_depth, VOCAB, seed)
    hidden = synth.normal_f16((T, H), seed, 90)
    pos = tree.positions(P)
    a, _, path = orc.tree_accept(pred, gt, pos, P, tree.mask, tree.parent)
    want = orc.accept_commit(flat, P, path, gt, hidden)
    assert np.array_equal(want["prev_hidden"].view(np.uint16), hidden[path].view(np.uint16))

    d_gt, d_pos, d_mask, d_par = to_dev(torch, gt), to_dev(torch, pos), to_dev(torch, tree.mask), to_dev(torch, tree.parent)
    # separate operators on the first copy
    p1 = to_dev(torch, pred)
    len1 = torch.tensor([P], dtype=torch.int32, device="cuda")
    best1 = ops.tree_accept(p1, d_gt, d_pos, len1, d_mask, d_par)
    ops.kv_compact(caches[0], p1, d_gt, len1, best1, T)
    # the one-call form on the second
    p2 = to_dev(torch, pred)
    len2 = torch.tensor([P], dtype=torch.int32, device="cuda")
    best2 = ops.tree_accept(p2, d_gt, d_pos, len2, d_mask, d_par)
    d_hidden = to_dev(torch, hidden)
    prev = torch.full((T, H), 7.0, dtype=torch.float16, device="cuda")
    npos = torch.full((T,), -1, dtype=torch.int32, device="cuda")
    if pinned_result:
        result = torch.full((1 + T,), -1, dtype=torch.int32).pin_memory()
    else:
        result = torch.full((1 + T,), -1, dtype=torch.int32, device="cuda")
    ops.accept_commit(caches[1], p2, d_gt, len2, best2, T, hidden=d_hidden, prev_hidden=prev, next_position_ids=npos,
                      result=result, advance_length=True, next_root=True)
    torch.cuda.synchronize()
    res = result.numpy() if pinned_result else to_np(result)
    assert int(to_np(best2)[0]) == a and res[0] == a
    assert np.array_equal(res[: 1 + a], want["result"])
    assert np.all(res[1 + a:] == -1)
    assert int(to_np(len2)[0]) == want["new_length"] == P + a and int(to_np(len1)[0]) == P
    assert np.array_equal(to_np(npos)[:a], want["next_pos"]) and np.all(to_np(npos)[a:] == -1)
    assert np.array_equal(to_np(prev)[:a].view(np.uint16), want["prev_hidden"].view(np.uint16))
    assert np.all(to_np(prev)[a:] == 7.0)  # rows beyond the accept length are not touched
    ids1 = to_np(p1)[:a]
    ids2 = to_np(p2)[:a].copy()
    assert int(ids2[0]) == want["next_root"]  # the next tree's root
    ids2[0] = res[1]
    assert np.array_equal(ids1, ids2) and np.array_equal(ids1, want["result"][1:])
    for layer in range(layers):
        for c in caches:
            k_dev, v_dev = c.read_logical(layer, 0, P + a)
            assert np.array_equal(to_np(k_dev).reshape(P + a, -1).view(np.uint16), flat[2 * layer][: P + a].view(np.uint16))
            assert np.array_equal(to_np(v_dev).reshape(P + a, -1).view(np.uint16), flat[2 * layer + 1][: P + a].view(np.uint16))
    return a


def test_accept_commit_every_depth(gpu, orc):
    tree = synth.eagle_tree(6, 10, 60, seed=0)
    for depth in range(int(tree.depth.max()) + 1):
        assert _commit_case(gpu, orc, tree, 4096 - 7, depth, layers=3, seed=depth) == depth + 1
    wide = synth.eagle_tree(8, 16, 128, seed=1)
    _commit_case(gpu, orc, wide, 1000, int(wide.depth.max()), layers=2, seed=31, H=4096)
    _commit_case(gpu, orc, synth.chain_tree(128), 250, 127, layers=2, seed=32, H=64)


def test_accept_commit_result_in_pinned_host_memory(gpu, orc):
    """The packed (a, ids) result written straight into pinned host memory: one synchronisation, no copy call."""
    tree = synth.eagle_tree(6, 10, 60, seed=2)
    _commit_case(gpu, orc, tree, 777, 3, layers=2, seed=40, pinned_result=True)


def test_accept_commit_argument_checks(gpu):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    cache = PagedKVCache(1, HKV, 2)
    i32 = lambda n: torch.zeros(n, dtype=torch.int32, device="cuda")
    hidden = torch.zeros((4, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        ops.accept_commit(cache, i32(4), i32(4), i32(1), i32(2), 4, hidden=hidden)  # hidden without prev_hidden
    with pytest.raises(ValueError):
        ops.accept_commit(cache, i32(4), i32(4), i32(1), i32(2), 129)  # max_accept beyond the tree limit
    odd = torch.zeros((4, 60), dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        ops.accept_commit(cache, i32(4), i32(4), i32(1), i32(2), 4, hidden=odd, prev_hidden=odd.clone())  # 60 % 8


def _tail_case(torch, orc, tree, P, leaf_depth, layers, seed, H=512, V=3000, from_partials=False):
    """cpmcu_verify_tail (+ cpmcu_verify_tail_inplace) against the oracle's acceptance, compaction and tail bookkeeping,
    with gt given or left as the head's per-workgroup partials."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    T = tree.T
    S = P + T
    npages = (S + 255) // 256 + 1
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32)
    cache = PagedKVCache(layers, HKV, npages, block_table=table)
    flat = []
    for layer in range(layers):
        k = synth.normal_f16((S, HKV, D), seed, 10 + layer)
        v = synth.normal_f16((S, HKV, D), seed, 50 + layer)
        cache.write_logical(layer, 0, to_dev(torch, k), to_dev(torch, v))
        flat += [k.reshape(S, HKV * D).copy(), v.reshape(S, HKV * D).copy()]
    hidden = synth.normal_f16((T, H), seed, 90)
    d_hidden = to_dev(torch, hidden)
    if from_partials:
        w = to_dev(torch, synth.normal_f16((V, H), seed, 91, std=0.02))
        wt = ops.tile_head_weight(w)
        gt = to_np(ops.lm_head_argmax(d_hidden, wt))  # the two-launch head: what the partials must finish to
    else:
        gt = synth.rng(seed, 9).integers(0, VOCAB, T).astype(np.int32)
    pred, leaf = synth.draft_ids_for_accept(tree, gt, leaf_depth, V if from_partials else VOCAB, seed)
    pos = tree.positions(P)
    a, node, path = orc.tree_accept(pred, gt, pos, P, tree.mask, tree.parent)
    want = orc.accept_commit(flat, P, path, gt, hidden)
    d_pred, d_pos, d_mask, d_par = to_dev(torch, pred), to_dev(torch, pos), to_dev(torch, tree.mask), to_dev(torch, tree.parent)
    d_len = torch.tensor([P], dtype=torch.int32, device="cuda")
    d_kvlen = torch.tensor([P + T], dtype=torch.int32, device="cuda")
    i32 = lambda n, fill=-1: torch.full((n,), fill, dtype=torch.int32, device="cuda")
    gt_out, best, pth, ids, npos, result = i32(T), i32(2), i32(T), i32(T), i32(T), i32(1 + T)
    prev = torch.full((T, H), 7.0, dtype=torch.float16, device="cuda")
    src = ops.lm_head_partials(d_hidden, wt) if from_partials else to_dev(torch, gt)
    ops.verify_tail(cache, d_pred, src, d_pos, d_len, d_mask, d_par, hidden=d_hidden, prev_hidden=prev, gt_out=gt_out, best=best,
                    path=pth, accepted_ids=ids, next_position_ids=npos, result=result)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(d_pred), pred), "the draft ids are read only"
    assert np.array_equal(to_np(gt_out), gt)
    assert to_np(best).tolist() == [a, node]
    assert np.array_equal(to_np(pth)[:a], path) and np.all(to_np(pth)[a:] == -1)
    assert np.array_equal(to_np(ids)[:a], want["result"][1:]) and np.all(to_np(ids)[a:] == -1)
    assert np.array_equal(to_np(result)[: 1 + a], want["result"]) and np.all(to_np(result)[1 + a:] == -1)
    assert np.array_equal(to_np(npos)[:a], want["next_pos"]) and np.all(to_np(npos)[a:] == -1)
    assert np.array_equal(to_np(prev)[:a].view(np.uint16), want["prev_hidden"].view(np.uint16)) and np.all(to_np(prev)[a:] == 7.0)
    assert int(to_np(d_len)[0]) == P
    for layer in range(layers):
        k_dev, v_dev = cache.read_logical(layer, 0, P + a)
        assert np.array_equal(to_np(k_dev).reshape(P + a, -1).view(np.uint16), flat[2 * layer][: P + a].view(np.uint16))
        assert np.array_equal(to_np(v_dev).reshape(P + a, -1).view(np.uint16), flat[2 * layer + 1][: P + a].view(np.uint16))
    # the in-place part: ids into pred, lengths and positions advanced; then the next-root form
    p2 = to_dev(torch, pred)
    ops.verify_tail_inplace(best, ids, pred=p2, cache_length=d_len, kv_len=d_kvlen, position_ids=d_pos, advance_length=True)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(p2)[:a], want["result"][1:]) and np.array_equal(to_np(p2)[a:], pred[a:])
    assert int(to_np(d_len)[0]) == want["new_length"] and int(to_np(d_kvlen)[0]) == P + T + a
    assert np.array_equal(to_np(d_pos), tree.positions(P + a))
    p3 = to_dev(torch, pred)
    ops.verify_tail_inplace(best, ids, pred=p3, next_root=True)
    torch.cuda.synchronize()
    assert int(to_np(p3)[0]) == want["next_root"] and np.array_equal(to_np(p3)[1:], pred[1:])
    return a


def test_verify_tail_every_depth(gpu, orc):
    tree = synth.eagle_tree(6, 10, 60, seed=0)
    for depth in range(int(tree.depth.max()) + 1):
        assert _tail_case(gpu, orc, tree, 4096 - 7, depth, layers=3, seed=depth) == depth + 1
    wide = synth.eagle_tree(8, 16, 128, seed=3)
    for depth in (0, 5, 8):
        _tail_case(gpu, orc, wide, 1000, depth, layers=2, seed=31 + depth, H=1024)
    _tail_case(gpu, orc, synth.chain_tree(128), 250, 127, layers=2, seed=32, H=64)   # several read/write batches
    _tail_case(gpu, orc, synth.tree_from_parents([0, 0, 0, 2]), 300, 2, layers=2, seed=33)  # path [0, 2, 3]: overlap
    _tail_case(gpu, orc, synth.chain_tree(1), 77, 0, layers=1, seed=34)


@pytest.mark.parametrize("T,num_iter,topk", [(16, 4, 4), (17, 4, 4), (60, 6, 10), (64, 6, 10), (100, 8, 16), (128, 8, 16)])
def test_verify_tail_finishes_the_head_partials(gpu, orc, T, num_iter, topk):
    """gt left as the head GEMM's per-workgroup partials (one row-block count per kernel shape): the tail's own
    finish must give the arg-max of the two-launch head, and everything behind it follows."""
    tree = synth.eagle_tree(num_iter, topk, T, seed=T)
    _tail_case(gpu, orc, tree, 513, min(2, int(tree.depth.max())), layers=2, seed=T, H=512, V=40000, from_partials=True)


@pytest.mark.parametrize("hkv", [1, 8, 32])
def test_compaction_and_tail_with_other_kv_head_counts(gpu, orc, monkeypatch, hkv):
    """Compaction, the one-launch tail and the commit on caches of 1, 8 and 32 KV heads (the configurations have 2)."""
    import sys
    monkeypatch.setattr(sys.modules[__name__], "HKV", hkv)
    for seed in range(3):
        g = synth.rng(seed, 5)
        tree = synth.random_tree(int(g.integers(2, 65)), seed, max_children=4, max_depth=8)
        depth = int(g.integers(0, int(tree.depth.max()) + 1))
        _compact_case(gpu, orc, tree, int(g.integers(0, 900)), depth, layers=2, seed=seed)
        _tail_case(gpu, orc, tree, int(g.integers(0, 900)), depth, layers=2, seed=seed, H=512, V=3000, from_partials=bool(seed & 1))
        _commit_case(gpu, orc, tree, int(g.integers(0, 900)), depth, layers=2, seed=seed)


def test_verify_tail_random_trees_duplicate_siblings(gpu, orc):
    """Tiny vocabulary: accidental matches and duplicate sibling tokens, so the tournament's tie rule decides."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    cache = PagedKVCache(1, HKV, 3)
    for seed in range(30):
        T = int(synth.rng(seed, 1).integers(1, 129))
        tree = synth.random_tree(T, seed, max_children=6, max_depth=12)
        g = synth.rng(seed, 2)
        pred = g.integers(0, 3, T).astype(np.int32)
        gt = g.integers(0, 3, T).astype(np.int32)
        P = int(g.integers(0, 300))
        pos = tree.positions(P)
        a, node, path = orc.tree_accept(pred, gt, pos, P, tree.mask, tree.parent)
        best = torch.zeros(2, dtype=torch.int32, device="cuda")
        pth = torch.zeros(T, dtype=torch.int32, device="cuda")
        ids = torch.zeros(T, dtype=torch.int32, device="cuda")
        ops.verify_tail(cache, to_dev(torch, pred), to_dev(torch, gt), to_dev(torch, pos), torch.tensor([P], dtype=torch.int32, device="cuda"),
                        to_dev(torch, tree.mask), to_dev(torch, tree.parent), best=best, path=pth, accepted_ids=ids)
        torch.cuda.synchronize()
        assert to_np(best).tolist() == [a, node], seed
        assert np.array_equal(to_np(pth)[:a], path) and np.array_equal(to_np(ids)[:a], gt[path])


def test_model_level_entry_points(gpu, orc):
    """init_* -> init_storage -> load_model -> decode_attention / decode_lm_head / draft_head /
    verify_and_fix on the library-owned paged cache, against the oracle; and the error contract."""
    from cpm.cu_amd import lib as libmod
    torch = gpu
    L = libmod.get()
    V, Vs, H, layers, T, P = 6000, 4096, 512, 3, 60, 700
    keep = []  # device tensors must outlive the asynchronous calls that use their addresses

    def dev(a):
        t = to_dev(torch, a)
        keep.append(t)
        return t.data_ptr()
    with pytest.raises(RuntimeError):
        L.init_base_model(0.02, V, layers, H, 1024, HQ, HKV, D, 1e-5, 2, 2048, 1.0, 1.0, 1.0)  # neither fp16 (0) nor bf16 (1)
    with pytest.raises(ValueError):
        L.init_base_model(0.02, V, layers, H, 1024, HQ, HKV, 64, 1e-5, 0, 2048, 1.0, 1.0, 1.0)  # head_dim
    L.init_base_model(0.02, V, layers, H, 1024, HQ, HKV, D, 1e-5, 0, 2048, 1.0, 0.5, 1.0)
    with pytest.raises(RuntimeError):
        L.verify_and_fix(1, 1, 1, 1, 1, 1, 1, None)  # storage not initialised
    with pytest.raises(ValueError):
        L.init_minicpm4_eagle_model(1, 6, 10, 65, 0, False, 128, 1024, Vs, 1.0, True, True)  # tree_size > 64
    L.init_minicpm4_eagle_model(1, 6, 10, T, 0, False, 128, 1024, Vs, 1.0, True, True)
    ctx = ctypes.c_int(0)
    L.init_storage(ctypes.byref(ctx))
    assert ctx.value >= 4096 and ctx.value % 256 == 0
    w = synth.normal_f16((V, H), 1, 2, std=0.02)
    remap = synth.frspec_remap(V, Vs, 1)
    with pytest.raises(ValueError):
        L.load_model(b"model.layers.0.mlp.up_proj.weight", w.ctypes.data)
    with pytest.raises(RuntimeError):
        L.load_model(b"lm_head.weight", w.ctypes.data)  # token_id_remap must come first
    L.load_model(b"eagle.token_id_remap", remap.ctypes.data)
    L.load_model(b"lm_head.weight", w.ctypes.data)
    for fn, args in (("prefill", (1, 0, 0, 0, 0)), ("decode", (1, 128, 0, 0, 0, 0, 0, 0)), ("draft", (0, 0, 0, 0, 0))):
        with pytest.raises(RuntimeError):
            getattr(L, fn)(*args)

    # a permuted page table, then one verify step over 3 layers
    npages = 8
    table = synth.rng(3, 4).permutation(npages).astype(np.int32)
    L.set_block_table(table.ctypes.data_as(ctypes.c_void_p), npages)
    tree = synth.eagle_tree(6, 10, T, seed=2)
    S = P + T
    cl = torch.tensor([0], dtype=torch.int32, device="cuda")
    flat, outs = [], []
    for layer in range(layers):
        k = synth.normal_f16((S, HKV, D), 7, 10 + layer)
        v = synth.normal_f16((S, HKV, D), 7, 50 + layer)
        q = synth.normal_f16((T, HQ, D), 7, 90 + layer)
        # prefix goes in through the same entry point in chunks of <= 64 rows (a causal-chain "prefill")
        done = 0
        dummy = torch.empty((64, HQ, D), dtype=torch.float16, device="cuda")
        while done < P:
            n = min(64, P - done)
            cl.fill_(done + n)
            L.decode_attention(layer, n, done + n, dev(q[:1].repeat(n, 0)),
                               dev(k[done:done + n]), dev(v[done:done + n]),
                               cl.data_ptr(), 0, dummy.data_ptr())
            L.synchronize()
            done += n
        cl.fill_(S)  # cache_length pre-incremented by T, as cpmcu/llm.py:272 does
        out = torch.empty((T, HQ, D), dtype=torch.float16, device="cuda")
        L.decode_attention(layer, T, (S + 127) // 128 * 128, dev(q), dev(k[P:]),
                           dev(v[P:]), cl.data_ptr(), dev(tree.mask), out.data_ptr())
        L.synchronize()
        assert_close_f16(to_np(out), orc.tree_attention(q, k, v, tree.mask, P), "decode_attention layer %d" % layer)
        flat += [k.reshape(S, -1).copy(), v.reshape(S, -1).copy()]

    # the drafter's own layer: separate cache, block sliding window of 1024 tokens (eagle_window_size above);
    # prefix through causal chunks, then one draft round with Mask(eagle_mask_2d, k, k * d)
    with pytest.raises(ValueError):
        L.draft_attention(1, 1, 128, 1, 1, 1, 1, 0, 0, 1)  # only one drafter layer
    kd, dd, Pd = 10, 3, 1500
    Sd = Pd + kd * dd
    kq = synth.normal_f16((kd, HQ, D), 9, 1)
    kk = synth.normal_f16((Sd, HKV, D), 9, 2)
    vv = synth.normal_f16((Sd, HKV, D), 9, 3)
    g9 = synth.rng(9, 4)
    bits = g9.integers(0, 2, size=(kd, kd * dd)).astype(np.uint64)
    for i in range(kd):
        bits[i, kd * dd - kd + i] = 1
    dmask = np.array([sum(int(bits[i, j]) << j for j in range(kd * dd)) for i in range(kd)], np.uint64)
    done = 0
    while done < Sd - kd:
        n = min(64, Sd - kd - done)
        cl.fill_(done + n)
        L.draft_attention(0, n, done + n, dev(kq[:1].repeat(n, 0)), dev(kk[done:done + n]), dev(vv[done:done + n]),
                          cl.data_ptr(), 0, 0, dummy.data_ptr())
        L.synchronize()
        done += n
    cl.fill_(Sd)
    dout = torch.empty((kd, HQ, D), dtype=torch.float16, device="cuda")
    L.draft_attention(0, kd, (Sd + 127) // 128 * 128, dev(kq), dev(kk[Sd - kd:]), dev(vv[Sd - kd:]), cl.data_ptr(), dev(dmask),
                      kd * dd, dout.data_ptr())
    L.synchronize()
    ref_w = orc.tree_attention(kq, kk, vv, dmask.reshape(kd, 1), Sd - kd, mask_k_range=kd * dd, block_window_size=1024)
    assert_close_f16(to_np(dout), ref_w, "draft_attention with the block window")
    ref_full = orc.tree_attention(kq, kk, vv, dmask.reshape(kd, 1), Sd - kd, mask_k_range=kd * dd)
    assert np.abs(ref_w.astype(np.float32) - ref_full.astype(np.float32)).max() > 1e-3  # the window cut keys off

    hid = synth.normal_f16((T, H), 7, 200)
    logits = torch.empty((64, V), dtype=torch.float16, device="cuda")
    gt = torch.empty(T, dtype=torch.int32, device="cuda")
    L.decode_lm_head(T, dev(hid), logits.data_ptr(), gt.data_ptr())
    L.synchronize()
    z_ref = orc.lm_head(hid, w, head_scale=0.5)
    assert_close_f16(to_np(logits[:T]), z_ref, "decode_lm_head")
    gt_np = to_np(gt)
    assert np.array_equal(gt_np, orc.argmax(to_np(logits[:T])))

    k_top = 10
    val = torch.empty((k_top, k_top), dtype=torch.float16, device="cuda")
    pos = torch.empty((k_top, k_top), dtype=torch.int32, device="cuda")
    ids = torch.empty((k_top, k_top), dtype=torch.int32, device="cuda")
    L.draft_head(k_top, dev(hid[:k_top]), val.data_ptr(), pos.data_ptr(), ids.data_ptr())
    L.synchronize()
    assert np.array_equal(to_np(ids), remap[to_np(pos)])
    lp_ref, _, _ = orc.log_softmax(orc.lm_head(hid[:k_top], w[remap]))
    assert_close_f16(to_np(val), np.take_along_axis(lp_ref, to_np(pos).astype(np.int64), 1), "draft_head log-probs")

    # verify_and_fix: accept 3 draft tokens, compact all layers, pred <- accepted ids
    pred, leaf = synth.draft_ids_for_accept(tree, gt_np, 3, V, 5)
    d_pred = to_dev(torch, pred)
    cl.fill_(P)
    acc = ctypes.c_int(0)
    L.verify_and_fix(T, d_pred.data_ptr(), gt.data_ptr(), dev(tree.positions(P)), cl.data_ptr(),
                     dev(tree.mask), dev(tree.parent), ctypes.byref(acc))
    a, _, path = orc.tree_accept(pred, gt_np, tree.positions(P), P, tree.mask, tree.parent)
    ids_ref = orc.kv_compact(flat, P, path, gt_np)
    assert acc.value == a == 4
    assert np.array_equal(to_np(d_pred)[:a], ids_ref)
    # the compacted cache, seen through the API: one more decode step (a single new token) must
    # attend over prefix + accepted rows exactly as the oracle does on the compacted flat caches
    kp, npg = ctypes.c_uint64(), ctypes.c_int()
    L.model_pointers(0, ctypes.byref(kp), None, None, ctypes.byref(npg))
    assert kp.value != 0 and npg.value >= npages
    S2 = P + a + 1
    one = synth.chain_tree(1)
    for layer in range(layers):
        kn = synth.normal_f16((1, HKV, D), 8, 10 + layer)
        vn = synth.normal_f16((1, HKV, D), 8, 50 + layer)
        qn = synth.normal_f16((1, HQ, D), 8, 90 + layer)
        cl.fill_(S2)
        out = torch.empty((1, HQ, D), dtype=torch.float16, device="cuda")
        L.decode_attention(layer, 1, (S2 + 127) // 128 * 128, dev(qn), dev(kn),
                           dev(vn), cl.data_ptr(), 0, out.data_ptr())
        L.synchronize()
        k_flat = np.concatenate([flat[2 * layer][: P + a].reshape(-1, HKV, D), kn])
        v_flat = np.concatenate([flat[2 * layer + 1][: P + a].reshape(-1, HKV, D), vn])
        assert_close_f16(to_np(out), orc.tree_attention(qn, k_flat, v_flat, one.mask, P + a), "post-compaction decode layer %d" % layer)
    L.print_perf_summary()
    L.shutdown()
