"""Pins of the CPU oracle (CPU only).

The reference ships no golden vectors, fixtures or assertions for this path (its tests/ holds two
manual generation scripts) and its CUDA sources cannot be built here, so each oracle function is
pinned by what the mathematics fixes: closed forms in fp64, library routines on special cases
(numpy, scipy, torch CPU scaled_dot_product_attention), invariants, and brute force on small inputs.
Each check is chosen so that a plausible slip (wrong head-group mapping, transposed operand, wrong
tie direction, dropped causal bound, off-by-one in the tournament) fails it.
"""
import itertools

import numpy as np
import pytest
import scipy.special

from cpm.cu_amd import synth


# ----------------------------------------------------------------------------- fp16 helpers
def test_f16_to_f32_all_patterns(orc):
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    for sw in (False, True):
        got = orc.f16_to_f32(bits, software=sw)
        nan = np.isnan(ref)  # the hardware conversion quiets signalling NaNs; payloads are not compared
        assert np.array_equal(got.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])
        assert np.all(np.isnan(got[nan]))


def test_f32_to_f16_rounding(orc):
    g = synth.rng(1, 1)
    x = np.concatenate([
        g.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** g.integers(-9, 6, 200000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25,
                  np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -14, 6.1e-5, 5.96e-8, 1e-10], np.float32),
        # exact ties between adjacent halves (round to even), normal and subnormal
        (np.arange(1024, 1100, dtype=np.float32) + 0.5) * np.float32(2.0 ** -10),
        (np.arange(0, 64, dtype=np.float32) + 0.5) * np.float32(2.0 ** -24),
    ])
    ref = x.astype(np.float16).view(np.uint16)
    for sw in (False, True):
        assert np.array_equal(orc.f32_to_f16(x, software=sw), ref)


# ----------------------------------------------------------------------------- A1 attention
def _attention_fp64(q, k, v, mask, P):
    """Closed form, written independently of the oracle: explicit boolean visibility + fp64 softmax."""
    T, Hq, D = q.shape
    S, Hkv, _ = k.shape
    group = Hq // Hkv
    vis = np.zeros((T, S), bool)
    vis[:, :P] = True
    for i in range(T):
        for j in range(T):
            if (int(mask[i, j // 64]) >> (j % 64)) & 1 and j <= i:
                vis[i, P + j] = True
    kk = np.repeat(k.astype(np.float64), group, axis=1)  # kv head of q head h is h // group
    vv = np.repeat(v.astype(np.float64), group, axis=1)
    s = np.einsum("ihd,chd->hic", q.astype(np.float64), kk) / np.sqrt(D)
    s = np.where(vis[None], s, -np.inf)
    p = scipy.special.softmax(s, axis=-1)
    lse = scipy.special.logsumexp(s, axis=-1)
    return np.einsum("hic,chd->ihd", p, vv), lse.T


@pytest.mark.parametrize("T,P,Hq,Hkv,seed", [(16, 200, 8, 2, 0), (60, 333, 32, 2, 1), (128, 70, 4, 4, 2), (5, 0, 6, 3, 3)])
def test_attention_closed_form(orc, T, P, Hq, Hkv, seed):
    tree = synth.random_tree(T, seed, max_children=4, max_depth=9)
    q = synth.normal_f16((T, Hq, 128), seed, 1)
    k = synth.normal_f16((P + T, Hkv, 128), seed, 2)
    v = synth.normal_f16((P + T, Hkv, 128), seed, 3)
    out, lse = orc.tree_attention(q, k, v, tree.mask, P, return_lse=True)
    ref, lse_ref = _attention_fp64(q, k, v, tree.mask, P)
    # fp16 output + fp16 P: a few fp16 ulps of values that are O(1)
    assert np.abs(out.astype(np.float64) - ref).max() < 4e-3
    assert np.abs(lse - lse_ref).max() < 1e-3


def test_attention_matches_torch_sdpa(orc):
    """Chain tree == causal decode over prefix + new tokens; arbitrary tree == boolean attn_mask SDPA."""
    import torch
    T, P, Hq, Hkv = 12, 50, 8, 2
    q = synth.normal_f16((T, Hq, 128), 4, 1)
    k = synth.normal_f16((P + T, Hkv, 128), 4, 2)
    v = synth.normal_f16((P + T, Hkv, 128), 4, 3)
    tq = torch.from_numpy(q.astype(np.float32)).permute(1, 0, 2)[None]
    tk = torch.from_numpy(k.astype(np.float32)).permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)[None]
    tv = torch.from_numpy(v.astype(np.float32)).permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)[None]
    for tree in (synth.chain_tree(T), synth.random_tree(T, 9, 3, 5)):
        vis = torch.zeros(T, P + T, dtype=torch.bool)
        vis[:, :P] = True
        for i in range(T):
            for j in range(T):
                vis[i, P + j] = bool((int(tree.mask[i, 0]) >> j) & 1)
        ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=vis)[0].permute(1, 0, 2).numpy()
        out = orc.tree_attention(q, k, v, tree.mask, P).astype(np.float32)
        assert np.abs(out - ref).max() < 4e-3
    # the chain is also torch's own causal path (bottom-right aligned): check through an explicit tril
    tril = torch.ones(T, P + T, dtype=torch.bool).tril(diagonal=P)
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=tril)[0].permute(1, 0, 2).numpy()
    assert np.abs(orc.tree_attention(q, k, v, synth.chain_tree(T).mask, P).astype(np.float32) - ref).max() < 4e-3


def test_attention_invariants(orc):
    T, P, Hq, Hkv = 20, 90, 8, 2
    tree = synth.random_tree(T, 5, 3, 6)
    q = synth.normal_f16((T, Hq, 128), 5, 1)
    k = synth.normal_f16((P + T, Hkv, 128), 5, 2)
    v = synth.normal_f16((P + T, Hkv, 128), 5, 3)
    base = orc.tree_attention(q, k, v, tree.mask, P)
    # (a) perturbing a non-ancestor's K/V leaves a row bit-identical
    victim = 11
    k2, v2 = k.copy(), v.copy()
    k2[P + victim] += np.float16(2.0)
    v2[P + victim] -= np.float16(3.0)
    pert = orc.tree_attention(q, k2, v2, tree.mask, P)
    sees = np.array([(int(tree.mask[i, 0]) >> victim) & 1 for i in range(T)], bool)
    assert np.array_equal(base[~sees], pert[~sees]) and not np.array_equal(base[sees], pert[sees])
    # (b) GQA: heads [0, group) read kv head 0, [group, 2*group) kv head 1 -> swapping kv heads and
    #     the two q-head groups swaps the output groups
    g = Hq // Hkv
    q_sw = np.concatenate([q[:, g:], q[:, :g]], axis=1)
    out_sw = orc.tree_attention(q_sw, k[:, ::-1].copy(), v[:, ::-1].copy(), tree.mask, P)
    assert np.array_equal(out_sw, np.concatenate([base[:, g:], base[:, :g]], axis=1))
    # (c) root-only tree == single-token decode over the prefix plus itself
    one = orc.tree_attention(q[:1], k[: P + 1], v[: P + 1], synth.chain_tree(1).mask, P)
    ref, _ = _attention_fp64(q[:1], k[: P + 1], v[: P + 1], synth.chain_tree(1).mask, P)
    assert np.abs(one.astype(np.float64) - ref).max() < 4e-3
    # (d) the causal bound j <= i holds even if a (malformed) mask sets a forward bit
    bad = tree.mask.copy()
    bad[3, 0] |= np.uint64(1 << 15)
    assert np.array_equal(orc.tree_attention(q, k, v, bad, P)[3], base[3])
    # (e) scale is applied to the scores: doubling q at half the scale is the same problem
    out_h = orc.tree_attention((q.astype(np.float32) * 2).astype(np.float16), k, v, tree.mask, P, scale=0.5 / np.sqrt(128))
    assert np.abs(out_h.astype(np.float32) - base.astype(np.float32)).max() < 2e-3


# ----------------------------------------------------------------------------- heads
def test_lm_head_fp64_and_gather_identity(orc):
    n, V, H = 7, 900, 256
    hid = synth.normal_f16((n, H), 6, 1)
    w = synth.normal_f16((V, H), 6, 2, std=0.05)
    z = orc.lm_head(hid, w)
    ref = hid.astype(np.float64) @ w.astype(np.float64).T
    assert z.shape == (n, V)  # a transposed result would not even have this shape's values
    assert np.abs(z.astype(np.float64) - ref).max() <= np.abs(ref).max() * 2.0 ** -10
    remap = synth.frspec_remap(V, 300, 6)
    sub = orc.gather_rows(w, remap)
    assert np.array_equal(sub.view(np.uint16), w[remap].view(np.uint16))
    # logits'[:, r] == logits_full[:, token_id_remap[r]] bit for bit (same row, same order)
    assert np.array_equal(orc.lm_head(hid, sub).view(np.uint16), z[:, remap].view(np.uint16))
    # head_scale: hidden is pre-scaled and ROUNDED to fp16 before the product
    sc = 0.3
    pre = (hid.astype(np.float32) * np.float32(np.float16(sc))).astype(np.float16)
    assert np.array_equal(orc.lm_head(hid, w, head_scale=sc).view(np.uint16), orc.lm_head(pre, w).view(np.uint16))


def test_log_softmax(orc):
    x = (synth.rng(7, 1).standard_normal((4, 5000)) * 2).astype(np.float16)
    lp, m, lse = orc.log_softmax(x)
    ref = scipy.special.log_softmax(x.astype(np.float64), axis=1)
    ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(lp.astype(np.float64) - ref) <= ulp)  # within one fp16 ulp of the fp64 value
    assert np.array_equal(m, x.astype(np.float32).max(1))
    assert np.allclose(lse, scipy.special.logsumexp(x.astype(np.float64), axis=1) - m, atol=1e-5)
    # exact case: one finite entry per row (sum = 1, log = 0): lp = x - max exactly
    y = np.full((2, 64), -np.inf, np.float16)
    y[0, 5] = 3.5
    y[1, 60] = -2.25
    lp2, _, lse2 = orc.log_softmax(y)
    assert lp2[0, 5] == 0 and lp2[1, 60] == 0 and np.all(lse2 == 0)
    assert np.all(np.isneginf(np.delete(lp2[0], 5)))
    # staged variant applies exactly (x - m) - lse in fp32, rounded once
    st = orc.log_softmax_apply(x, m, lse)
    assert np.array_equal(st.view(np.uint16), lp.view(np.uint16))


def _topk_numpy(x, top):
    xf = x.astype(np.float32)
    pos = np.stack([np.lexsort((np.arange(x.shape[1]), -r))[:top] for r in xf]).astype(np.int32)
    return np.take_along_axis(x, pos.astype(np.int64), 1), pos


@pytest.mark.parametrize("n,dim,top", [(3, 1000, 10), (1, 510, 59), (2, 100, 100), (4, 4096, 32), (1, 1, 1)])
def test_topk_vs_lexsort(orc, n, dim, top):
    g = synth.rng(dim, top)
    for x in (g.standard_normal((n, dim)).astype(np.float16),            # tie-free-ish
              g.integers(-2, 3, (n, dim)).astype(np.float16),            # heavy ties
              np.where(g.random((n, dim)) < 0.7, -np.inf, g.standard_normal((n, dim))).astype(np.float16)):
        val, pos = orc.topk(x, top)
        v_ref, p_ref = _topk_numpy(x, top)
        assert np.array_equal(pos, p_ref)
        assert np.array_equal(val.view(np.uint16), v_ref.view(np.uint16))


def test_topk_tie_direction_and_signed_zero(orc):
    x = np.array([[1, 3, 3, -0.0, 0.0, 3, 2]], np.float16)
    val, pos = orc.topk(x, 7)
    assert pos.tolist() == [[1, 2, 5, 6, 0, 3, 4]]  # equal values: LOWER index first; -0 == +0


def test_argmax_lowest_index(orc):
    x = synth.rng(8, 1).integers(-5, 6, (6, 999)).astype(np.float16)
    assert np.array_equal(orc.argmax(x), np.argmax(x.astype(np.float32), axis=1))
    x[0, :] = -np.inf
    x[1, 998] = 100
    assert orc.argmax(x)[0] == 0 and orc.argmax(x)[1] == 998


def test_remap(orc):
    table = synth.frspec_remap(5000, 1000, 3)
    pos = synth.rng(3, 2).integers(0, 1000, 59).astype(np.int32)
    assert np.array_equal(orc.remap(pos, table), table[pos])


# ----------------------------------------------------------------------------- A4 acceptance
def _bitrev(i, bits):
    return int(format(i, "0%db" % bits)[::-1], 2)


def _accept_bruteforce(tree, pred, gt, P):
    """Walk parent pointers (not masks): node i is accepted iff every non-root node on its root path
    matches its parent's target token.  Deepest wins; among equals the reference's strictly-greater
    tournament keeps the node whose bit-reversed slot index is smallest."""
    T = tree.T
    ok = [True] * T
    for i in range(1, T):
        ok[i] = ok[int(tree.parent[i])] and pred[i] == gt[int(tree.parent[i])]
    best_depth = max(int(tree.depth[i]) for i in range(T) if ok[i])
    bits = 6 if T <= 64 else 7
    cands = [i for i in range(T) if ok[i] and tree.depth[i] == best_depth]
    if best_depth == 0:
        node = 0  # score 1 is also what rejected nodes and empty slots carry, all reporting index 0
    else:
        node = min(cands, key=lambda i: _bitrev(i, bits))
    return best_depth + 1, node, tree.path_to(node)


def test_accept_bruteforce_small_trees_exhaustive(orc):
    """All parent arrays of 5-node trees x all pred/gt over a 2-token vocabulary."""
    P = 17
    for parents in itertools.product(*[range(i) for i in range(1, 5)]):
        tree = synth.tree_from_parents((0,) + parents)
        for bits in range(1 << 9):
            pred = np.array([0] + [(bits >> b) & 1 for b in range(4)], np.int32)
            gt = np.array([(bits >> (4 + b)) & 1 for b in range(5)], np.int32)
            a, node, path = orc.tree_accept(pred, gt, tree.positions(P), P, tree.mask, tree.parent)
            a_ref, node_ref, path_ref = _accept_bruteforce(tree, pred, gt, P)
            assert (a, node, list(path)) == (a_ref, node_ref, path_ref)


@pytest.mark.parametrize("T", [2, 33, 60, 64, 65, 100, 128])
def test_accept_bruteforce_random(orc, T):
    for seed in range(60):
        tree = synth.random_tree(T, seed, max_children=5, max_depth=12) if seed % 2 else synth.eagle_tree(8, 16, T, seed) if T > 20 else synth.random_tree(T, seed)
        g = synth.rng(seed, T)
        vocab = int(g.choice([2, 3, 50]))
        pred = g.integers(0, vocab, T).astype(np.int32)
        gt = g.integers(0, vocab, T).astype(np.int32)
        P = int(g.integers(0, 200000))
        a, node, path = orc.tree_accept(pred, gt, tree.positions(P), P, tree.mask, tree.parent)
        a_ref, node_ref, path_ref = _accept_bruteforce(tree, pred, gt, P)
        assert (a, node, list(path)) == (a_ref, node_ref, path_ref)
        assert path[0] == 0 and all(path[i] < path[i + 1] for i in range(a - 1))  # strictly increasing
        assert all(tree.depth[path[d]] == d for d in range(a))


def test_accept_chain_is_longest_prefix_match(orc):
    """Chain tree == sequential verification (cf. seq_verify_kernel, src/model/drafter.cuh:6-40)."""
    T = 40
    tree = synth.chain_tree(T)
    g = synth.rng(2, 2)
    for _ in range(50):
        gt = g.integers(0, 4, T).astype(np.int32)
        pred = np.concatenate([[7], gt[:-1]]).astype(np.int32)  # perfect draft
        cut = int(g.integers(1, T + 1))
        if cut < T:
            pred[cut] = gt[cut - 1] + 1  # first mismatch at position `cut`
        a, node, path = orc.tree_accept(pred, gt, tree.positions(5), 5, tree.mask, tree.parent)
        assert a == cut and node == cut - 1 and list(path) == list(range(cut))


def test_accept_rigged_depths(orc):
    for T, it, k in ((16, 4, 4), (60, 6, 10), (128, 8, 16)):
        tree = synth.eagle_tree(it, k, T, seed=0)
        assert not np.all(np.diff(tree.depth) >= 0), "generator must produce non-monotone depth order"
        gt = synth.rng(0, 9).integers(0, 73448, T).astype(np.int32)
        for depth in range(int(tree.depth.max()) + 1):
            pred, leaf = synth.draft_ids_for_accept(tree, gt, depth, 73448, depth)
            a, node, path = orc.tree_accept(pred, gt, tree.positions(4096), 4096, tree.mask, tree.parent)
            assert a == depth + 1 and node == (leaf if depth else 0) and list(path) == tree.path_to(leaf)


# ----------------------------------------------------------------------------- A5 compaction
def test_compaction_is_a_row_permutation(orc):
    g = synth.rng(4, 4)
    P, T, rows = 37, 20, 64
    for path in ([0], [0, 1, 2, 3], [0, 2, 3], [0, 5, 9, 19], [0, 19]):
        caches = [g.standard_normal((P + T, rows)).astype(np.float16) for _ in range(6)]
        before = [c.copy() for c in caches]
        gt = g.integers(0, 1000, T).astype(np.int32)
        ids = orc.kv_compact(caches, P, np.array(path, np.int32), gt)
        assert np.array_equal(ids, gt[path])
        for c, b in zip(caches, before):
            assert np.array_equal(c[:P], b[:P])                                  # prefix untouched
            assert np.array_equal(c[P:P + len(path)], b[P + np.array(path)])     # dst[P+d] = src[P+path[d]]
            assert np.array_equal(c[P + len(path):], b[P + len(path):])          # the rest is not written


def test_attention_mask_range_wider_than_queries(orc):
    """mask_k_range > T (the drafter's own attention, src/model/minicpm4/minicpm4_eagle.cuh:359) against torch's
    CPU scaled_dot_product_attention with an explicit boolean mask built from the definition: key
    column c is visible to query i iff c <= P + i and (c < S - R or bit c - (S - R) of mask[i])."""
    import torch
    g = synth.rng(5, 55)
    T, R, P, Hq, Hkv, D = 5, 20, 37, 4, 2, 32
    S = P + T
    q = g.standard_normal((T, Hq, D)).astype(np.float16)
    k = g.standard_normal((S, Hkv, D)).astype(np.float16)
    v = g.standard_normal((S, Hkv, D)).astype(np.float16)
    bits = g.integers(0, 2, size=(T, R)).astype(np.uint64)
    for i in range(T):
        bits[i, R - T + i] = 1  # a query always sees its own key
    mask = np.array([[sum(int(bits[i, j]) << j for j in range(R))] for i in range(T)], np.uint64)
    out = orc.tree_attention(q, k, v, mask, P, mask_k_range=R).astype(np.float32)
    vis = np.zeros((T, S), bool)
    for i in range(T):
        for c in range(S):
            vis[i, c] = c <= P + i and (c < S - R or bool(bits[i, c - (S - R)]))
    qt = torch.from_numpy(q.astype(np.float32)).permute(1, 0, 2)                          # [Hq, T, D]
    kt = torch.from_numpy(k.astype(np.float32)).permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)
    vt = torch.from_numpy(v.astype(np.float32)).permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=torch.from_numpy(vis)).permute(1, 0, 2).numpy()
    assert np.abs(out - ref).max() < 5e-3


def _window_first_key(P, window):
    """First visible key of the block sliding window, written out from the reference's arithmetic
    (src/flash_attn/src/flash_blockmask.h:16,32 with kBlockN = 128, loop_step_idx = 0): an independent
    restatement in Python integers, used only to build the expected visible sets below."""
    q_block_idx = P
    k_window_left = (q_block_idx + 127) // 128 - window // 128
    return max(k_window_left, 0) * 128


@pytest.mark.parametrize("P,window", [(100, 128), (127, 128), (128, 128), (129, 128), (255, 128), (256, 256), (257, 256),
                                      (1000, 128), (1000, 512), (1024, 1024), (1025, 1024), (3000, 1024), (900, 4096)])
def test_attention_block_window(orc, P, window):
    """The drafter layer's block sliding window (src/flash_attn/src/flash_blockmask.h:32,43-46) pinned three ways:
    (1) torch's CPU scaled_dot_product_attention with the explicit visible set; (2) the windowed result equals
    the plain oracle on a cache cut down to the visible keys, bit for bit (same keys, same order of
    accumulation); (3) a window that covers the context changes nothing."""
    import torch
    g = synth.rng(77, P * 7 + window)
    k_, d_ = 6, 3
    T, R, Hq, Hkv, D = k_, k_ * d_, 4, 2, 32
    S = P + T
    q = g.standard_normal((T, Hq, D)).astype(np.float16)
    k = g.standard_normal((S, Hkv, D)).astype(np.float16)
    v = g.standard_normal((S, Hkv, D)).astype(np.float16)
    bits = g.integers(0, 2, size=(T, R)).astype(np.uint64)
    for i in range(T):
        bits[i, R - T + i] = 1
    mask = np.array([[sum(int(bits[i, j]) << j for j in range(R))] for i in range(T)], np.uint64)
    out = orc.tree_attention(q, k, v, mask, P, mask_k_range=R, block_window_size=window)
    first = _window_first_key(P, window)
    assert first % 128 == 0 and first <= P and P - first <= window
    vis = np.zeros((T, S), bool)
    for i in range(T):
        for c in range(S):
            vis[i, c] = c >= first and c <= P + i and (c < S - R or bool(bits[i, c - (S - R)]))
    qt = torch.from_numpy(q.astype(np.float32)).permute(1, 0, 2)
    kt = torch.from_numpy(k.astype(np.float32)).permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)
    vt = torch.from_numpy(v.astype(np.float32)).permute(1, 0, 2).repeat_interleave(Hq // Hkv, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=torch.from_numpy(vis)).permute(1, 0, 2).numpy()
    assert np.abs(out.astype(np.float32) - ref).max() < 5e-3
    if S - first >= R:  # the cut cache still holds every column the mask bits refer to
        cut = orc.tree_attention(q, k[first:], v[first:], mask, P - first, mask_k_range=R)
        assert np.array_equal(out.view(np.uint16), cut.view(np.uint16))
    if first == 0:
        plain = orc.tree_attention(q, k, v, mask, P, mask_k_range=R)
        assert np.array_equal(out.view(np.uint16), plain.view(np.uint16))
    else:
        assert not np.array_equal(out.view(np.uint16), orc.tree_attention(q, k, v, mask, P, mask_k_range=R).view(np.uint16))


def test_accept_commit_tail_against_numpy():
    """The oracle's restatement of verify() after the acceptance, pinned on what fixes it independently:
    the hidden gather is numpy fancy indexing, compaction is "rows P+path[d] land at P+d, nothing else
    moves" (checked on rows tagged with their own index), positions are an arange, ids are gt[path]."""
    import oracle as orc
    rng = np.random.default_rng(5)
    P, T, H, rows = 37, 20, 24, 80
    path = np.array([0, 3, 4, 9, 17], np.int32)  # increasing, path[d] >= d
    gt = rng.integers(0, 1000, T).astype(np.int32)
    hidden = rng.standard_normal((T, H)).astype(np.float16)
    caches = [np.repeat(np.arange(rows, dtype=np.float16)[:, None], 8, 1) + np.float16(c) * 0 for c in range(3)]
    before = [c.copy() for c in caches]
    out = orc.accept_commit(caches, P, path, gt, hidden)
    a = len(path)
    assert np.array_equal(out["prev_hidden"].view(np.uint16), hidden[path].view(np.uint16))
    assert np.array_equal(out["next_pos"], P + np.arange(a))
    assert np.array_equal(out["result"], np.concatenate([[a], gt[path]]))
    assert out["new_length"] == P + a and out["next_root"] == gt[path[-1]]
    for c, b in zip(caches, before):
        assert np.array_equal(c[:P], b[:P]) and np.array_equal(c[P + a:], b[P + a:])
        assert np.array_equal(c[P:P + a, 0], (P + path).astype(np.float16))  # the tag of the source row


def test_rope_against_complex_rotation():
    """Rotary embedding pinned on what the mathematics fixes: the pair (x[d], x[d+64]) is the complex number
    x[d] + i x[d+64] multiplied by exp(i * pos * inv_freq[d]) -- numpy complex128 here, so a swapped sign, a
    transposed pair or a wrong frequency index fails; position 0 is the identity; the norm of every pair is kept."""
    import oracle as orc
    rng = np.random.default_rng(11)
    T, Hq, Hkv, D = 7, 4, 2, 128
    half = D // 2
    q = rng.standard_normal((T, Hq, D)).astype(np.float16)
    k = rng.standard_normal((T, Hkv, D)).astype(np.float16)
    pos = np.array([0, 1, 2, 77, 4096, 40000, 131071], np.int32)
    inv_freq = (10000.0 ** (-np.arange(half) / half)).astype(np.float32)
    qr, kr = orc.rope(q, k, pos, inv_freq)
    for x, xr in ((q, qr), (k, kr)):
        z = x[..., :half].astype(np.float64) + 1j * x[..., half:].astype(np.float64)
        ang = (pos.astype(np.float32)[:, None] * inv_freq[None, :]).astype(np.float32).astype(np.float64)  # float32 product, as the kernel forms it
        w = z * np.exp(1j * ang)[:, None, :]
        want = np.concatenate([w.real, w.imag], -1)
        got = xr.astype(np.float64)
        assert np.max(np.abs(got - want)) <= 2e-3 * max(1.0, np.max(np.abs(want)))  # one fp16 rounding + float32 cos/sin
        assert np.array_equal(xr[0].view(np.uint16), x[0].view(np.uint16))          # position 0: identity
    # a given table is used as is: the quarter turn maps (a, b) to (-b, a) exactly
    table = np.zeros((T, half, 2), np.float32)
    table[..., 1] = 1.0
    qt, kt = orc.rope(q, k, table=table)
    assert np.array_equal(qt[..., :half], -q[..., half:]) and np.array_equal(qt[..., half:], q[..., :half])
    assert np.array_equal(kt[..., :half], -k[..., half:]) and np.array_equal(kt[..., half:], k[..., :half])


# ----------------------------------------------------------------------------- bfloat16 (torch_dtype = 1)
@pytest.fixture
def orc_bf16(orc):
    orc.set_dtype("bf16")
    yield orc
    orc.set_dtype("f16")


def test_bf16_conversions_against_torch(orc):
    """Every bfloat16 pattern to float32, and float32 to bfloat16 on random values over the whole exponent range, on the
    ties between neighbours and at the edges, against torch's CPU conversion (an independent implementation)."""
    import torch
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.bf16_to_f32(bits)
    ref = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy()
    nan = np.isnan(ref)
    assert np.array_equal(got.view(np.uint32)[~nan], ref.view(np.uint32)[~nan]) and np.all(np.isnan(got[nan]))
    g = synth.rng(1, 2)
    x = np.concatenate([
        g.standard_normal(300000).astype(np.float32) * np.float32(10.0) ** g.integers(-38, 38, 300000).astype(np.float32),
        np.array([0.0, -0.0, 3.3895314e38, 3.4e38, np.inf, -np.inf, 1e-40, 1.0, 1.00390625, 1.0078125], np.float32),
        # exact ties between adjacent bfloat16 values (round to even): 1 + (2i + 1) 2^-8
        1.0 + (2 * np.arange(0, 64, dtype=np.float32) + 1) * np.float32(2.0 ** -8),
    ])
    ref_bits = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(orc.f32_to_bf16(x), ref_bits)
    assert np.isnan(orc.bf16_to_f32(orc.f32_to_bf16(np.array([np.nan], np.float32)))).all()


def test_bf16_attention_closed_form(orc_bf16):
    orc = orc_bf16
    T, P, Hq, Hkv, seed = 60, 333, 32, 2, 1
    tree = synth.random_tree(T, seed, max_children=4, max_depth=9)
    enc = lambda shape, stream: orc.encode(synth.rng(seed, stream).standard_normal(shape, dtype=np.float32))
    q, k, v = enc((T, Hq, 128), 1), enc((P + T, Hkv, 128), 2), enc((P + T, Hkv, 128), 3)
    out, lse = orc.tree_attention(q, k, v, tree.mask, P, return_lse=True)
    ref, lse_ref = _attention_fp64(orc.decode(q), orc.decode(k), orc.decode(v), tree.mask, P)
    # bfloat16 output and bfloat16 P: a few ulps (2^-8 relative) of values that are O(1)
    assert np.abs(orc.decode(out).astype(np.float64) - ref).max() < 3e-2
    assert np.abs(lse - lse_ref).max() < 1e-3
    # and it is not the fp16 oracle on the same bits
    orc.set_dtype("f16")
    assert not np.array_equal(orc.tree_attention(q, k, v, tree.mask, P).view(np.uint16), out.view(np.uint16))
    orc.set_dtype("bf16")


def test_bf16_lm_head_log_softmax_and_rounding(orc_bf16):
    import torch
    orc = orc_bf16
    n, V, H = 7, 900, 256
    hid = orc.encode(synth.rng(6, 1).standard_normal((n, H), dtype=np.float32))
    w = orc.encode(synth.rng(6, 2).standard_normal((V, H), dtype=np.float32) * 0.05)
    z = orc.lm_head(hid, w)
    ref = orc.decode(hid).astype(np.float64) @ orc.decode(w).astype(np.float64).T
    assert np.abs(orc.decode(z).astype(np.float64) - ref).max() <= np.abs(ref).max() * 2.0 ** -7
    # the result is the correctly rounded bfloat16 of an fp32 sum that is within fp32 rounding of the fp64 one
    near = torch.from_numpy(ref.astype(np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (near == z.view(np.uint16)).mean() > 0.98
    # head_scale: the hidden rows are pre-scaled and ROUNDED to bfloat16 before the product, the scale itself rounded too
    sc = 0.3
    sc_r = orc.decode(orc.encode(np.array([sc], np.float32)))[0]
    pre = orc.encode(orc.decode(hid) * np.float32(sc_r))
    assert np.array_equal(orc.lm_head(hid, w, head_scale=sc).view(np.uint16), orc.lm_head(pre, w).view(np.uint16))
    # log-softmax: rounded once to bfloat16 from (x - m) - lse in fp32
    x = orc.encode(synth.rng(7, 1).standard_normal((4, 5000), dtype=np.float32) * 2)
    lp, m, lse = orc.log_softmax(x)
    xf = orc.decode(x)
    assert np.array_equal(m, xf.max(1))
    ref_lp = torch.from_numpy((xf - m[:, None]) - lse[:, None]).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(lp.view(np.uint16), ref_lp)
    assert np.allclose(lse, scipy.special.logsumexp(xf.astype(np.float64), axis=1) - m, atol=1e-5)
    # the ranking is on bit patterns: value descending, lower index first among equals, as for fp16
    val, pos = orc.topk(lp, 10)
    lpf = orc.decode(lp)
    ref_pos = np.stack([np.lexsort((np.arange(lpf.shape[1]), -r))[:10] for r in lpf]).astype(np.int32)
    assert np.array_equal(pos, ref_pos)


def test_bf16_rope_and_running_log_probs(orc_bf16):
    """Rotary pairs and the drafter's running sums are rounded to bfloat16 (torch's conversion as the independent rounding)."""
    import torch
    orc = orc_bf16
    T, Hq, Hkv, Dh = 5, 4, 2, 128
    q = orc.encode(synth.rng(9, 1).standard_normal((T, Hq, Dh), dtype=np.float32))
    k = orc.encode(synth.rng(9, 2).standard_normal((T, Hkv, Dh), dtype=np.float32))
    pos = np.arange(100, 100 + T, dtype=np.int32)
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, Dh, 2, dtype=np.float32) / Dh))).astype(np.float32)
    qr, kr = orc.rope(q, k, pos=pos, inv_freq=inv_freq)
    ang = pos[:, None].astype(np.float32) * inv_freq[None, :]
    c, s = np.cos(ang).astype(np.float32)[:, None, :], np.sin(ang).astype(np.float32)[:, None, :]
    qf = orc.decode(q)
    a, b = qf[..., :64], qf[..., 64:]
    ref = np.concatenate([a * c - b * s, a * s + b * c], axis=-1).astype(np.float32)
    ref_bits = torch.from_numpy(ref).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (ref_bits == qr.view(np.uint16)).mean() > 0.999  # (cos / sin of the host library may differ in their last bit)
    k_it = 4
    t = orc.DraftTree(k_it, 3)
    v0 = orc.encode(np.array([-0.11, -0.7, -1.3, -2.9], np.float32))
    t.begin(v0, np.arange(k_it, dtype=np.int32))
    rows = orc.encode(-np.abs(synth.rng(9, 3).standard_normal((k_it, k_it), dtype=np.float32)))
    rows = orc.encode(-np.sort(-orc.decode(rows), axis=1))
    _, _, summed = t.extend(1, rows, np.arange(k_it * k_it, dtype=np.int32).reshape(k_it, k_it))
    ref = torch.from_numpy(orc.decode(rows) + orc.decode(v0)[:, None]).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(summed.view(np.uint16), ref)
