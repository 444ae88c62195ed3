"""GPU parity of the tree-verify attention and KV append kernels against the CPU oracle.

Every call goes through the C-ABI (cpm.cu_amd.ops -> ctypes -> libcpmcu_amd.so).  Tolerance of the
path for fp16 outputs: max-abs 2e-2 and max-rel 1e-2 (see tests/util.py).
"""
import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 2, 128


@pytest.fixture(autouse=True, params=["2", "1"], ids=["groups2", "groups1"])
def kv_groups(request, set_option):
    """Every test of this module runs on both shapes of the split kernel (2 KV groups x 128 rows and
    1 x 256 rows per workgroup); without the override the library picks by context length."""
    set_option("attn_kv_groups", int(request.param))
    return request.param


def _case(torch, orc, tree, P, seed, page_perm=True, splits=0, use_mask=True, extra_pages=2, q_std=1.0):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    T = tree.T
    S = P + T
    q = synth.normal_f16((T, HQ, D), seed, 1, q_std)
    k = synth.normal_f16((S, HKV, D), seed, 2)
    v = synth.normal_f16((S, HKV, D), seed, 3)
    npages = (S + 255) // 256 + extra_pages
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32) if page_perm else np.arange(npages, dtype=np.int32)
    # stale garbage (incl. NaN bit patterns) in unused slots must not leak into the result
    cache = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
    cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    mask = tree.mask if use_mask else None
    out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, None if mask is None else to_dev(torch, mask),
                             num_splits=splits)
    torch.cuda.synchronize()
    ref_mask = tree.mask if use_mask else synth.chain_tree(T).mask
    ref = orc.tree_attention(q, k, v, ref_mask, P)
    return to_np(out), ref


@pytest.mark.parametrize("splits", [1, 2, 5, 0])
def test_c1_plumbing_case(gpu, orc, splits):
    """Config 1: 16-node tree (depth 4, top-k 4), 1024-token prefix, 32 q / 2 kv heads."""
    tree = synth.eagle_tree(4, 4, 16, seed=0)
    out, ref = _case(gpu, orc, tree, 1024, seed=0, splits=splits)
    assert_close_f16(out, ref, "attention c1 splits=%d" % splits)


@pytest.mark.parametrize("P,T,seed", [(0, 16, 1), (1, 7, 2), (63, 33, 3), (64, 64, 4), (255, 60, 5), (257, 60, 6),
                                      (700, 1, 7), (500, 128, 8), (2049, 100, 9)])
def test_ragged_shapes(gpu, orc, P, T, seed):
    """Prefix lengths around tile/page boundaries, empty prefix, one-node tree, two-word masks."""
    tree = synth.random_tree(T, seed, max_children=5, max_depth=10)
    for splits in (1, 3):
        out, ref = _case(gpu, orc, tree, P, seed, splits=splits)
        assert_close_f16(out, ref, "attention P=%d T=%d splits=%d" % (P, T, splits))


def test_chain_without_mask(gpu, orc):
    """mask == NULL means a causal chain (the reference's mask_2d = nullptr decode path)."""
    tree = synth.chain_tree(24)
    out, ref = _case(gpu, orc, tree, 300, seed=11, use_mask=False)
    assert_close_f16(out, ref, "attention chain")


def test_c2_shape_one_layer(gpu, orc):
    """Config 2 shape (60-node EAGLE tree, 4096-token prefix), one layer, default split choice."""
    tree = synth.eagle_tree(6, 10, 60, seed=0)
    out, ref = _case(gpu, orc, tree, 4096, seed=12)
    assert_close_f16(out, ref, "attention c2")


def test_split_count_invariance(gpu, orc):
    """The result may depend on the split count only through fp16 rounding of P."""
    tree = synth.eagle_tree(6, 10, 60, seed=3)
    outs = [_case(gpu, orc, tree, 1500, seed=13, splits=s)[0] for s in (1, 4, 24)]
    for o in outs[1:]:
        assert_close_f16(o, outs[0], "split invariance", atol=4e-3, rtol=4e-3)


def test_non_ancestor_perturbation(gpu, orc):
    """Row i must not change when K/V of a tree node outside its mask is perturbed."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    tree = synth.eagle_tree(6, 10, 60, seed=5)
    T, P = tree.T, 777
    S = P + T
    q = to_dev(torch, synth.normal_f16((T, HQ, D), 21, 1))
    k = to_dev(torch, synth.normal_f16((S, HKV, D), 21, 2))
    v = to_dev(torch, synth.normal_f16((S, HKV, D), 21, 3))
    npages = (S + 255) // 256
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    mask = to_dev(torch, tree.mask)
    cache = PagedKVCache(1, HKV, npages)
    cache.write_logical(0, 0, k, v)
    base = ops.tree_attention(q, cache, 0, kv_len, S, mask).clone()
    victim = 17
    k2, v2 = k.clone(), v.clone()
    k2[P + victim] += 3.0
    v2[P + victim] -= 5.0
    cache.write_logical(0, 0, k2, v2)
    pert = ops.tree_attention(q, cache, 0, kv_len, S, mask)
    torch.cuda.synchronize()
    sees = np.array([(int(tree.mask[i, victim // 64]) >> (victim % 64)) & 1 for i in range(T)], bool)
    base, pert = to_np(base), to_np(pert)
    assert np.array_equal(base[~sees], pert[~sees]), "rows that do not see the node changed"
    assert not np.array_equal(base[sees], pert[sees])


def test_kv_append_matches_logical_write(gpu):
    """copy_to_kvcache: the HIP append equals an index-based write, across a page boundary."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    T, P = 60, 4096 - 23
    npages = 20
    table = synth.rng(31, 4).permutation(npages).astype(np.int32)
    a = PagedKVCache(2, HKV, npages, block_table=table)
    b = PagedKVCache(2, HKV, npages, block_table=table)
    for layer in range(2):
        k = to_dev(torch, synth.normal_f16((T, HKV, D), 31, 10 + layer))
        v = to_dev(torch, synth.normal_f16((T, HKV, D), 31, 20 + layer))
        kv_len = torch.tensor([P + T], dtype=torch.int32, device="cuda")
        ops.kv_append(a, layer, k, v, kv_len)
        b.write_logical(layer, P, k, v)
    torch.cuda.synchronize()
    for layer in range(2):
        assert torch.equal(a.k[layer], b.k[layer])
        assert torch.equal(a.v[layer], b.v[layer])
        kk, vv = a.read_logical(layer, P, T)
        assert kk.abs().sum() > 0 and vv.abs().sum() > 0


@pytest.mark.parametrize("P,T,splits", [(1024, 16, 0), (4096 - 23, 60, 0), (250, 60, 1), (0, 16, 1), (700, 128, 3), (63, 64, 2)])
def test_fused_append_equals_append_then_attend(gpu, orc, P, T, splits):
    """Handing the tree rows' K/V to the attention kernel (fused copy_to_kvcache) must give the same
    output as appending first (up to the rounding of a different split partition), and must leave
    exactly the same cache behind -- stale garbage at [P, S) included."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    tree = synth.random_tree(T, P + T, max_children=5, max_depth=10)
    S = P + T
    seed = 41 + P
    q = synth.normal_f16((T, HQ, D), seed, 1)
    k = synth.normal_f16((S, HKV, D), seed, 2)
    v = synth.normal_f16((S, HKV, D), seed, 3)
    npages = (S + 255) // 256 + 1
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32)
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    mask = to_dev(torch, tree.mask)
    # reference path: append kernel, then attention
    a = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
    if P:
        a.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
    ops.kv_append(a, 0, to_dev(torch, k[P:]), to_dev(torch, v[P:]), kv_len)
    out_a = ops.tree_attention(to_dev(torch, q), a, 0, kv_len, S, mask, num_splits=splits)
    # fused path on a cache whose tree region holds NaN garbage
    b = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
    if P:
        b.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
    out_b = ops.tree_attention(to_dev(torch, q), b, 0, kv_len, S, mask, num_splits=splits,
                               k_new=to_dev(torch, k[P:]), v_new=to_dev(torch, v[P:]))
    torch.cuda.synchronize()
    # the fused call partitions the KV stream differently (the appending split gets fewer tiles), so the
    # two outputs agree to the fp16 rounding of the split partials, not bit for bit
    assert_close_f16(to_np(out_b), to_np(out_a), "fused vs unfused append", atol=4e-3, rtol=4e-3)
    assert_close_f16(to_np(out_b), orc.tree_attention(q, k, v, tree.mask, P), "fused append attention")
    kb, vb = b.read_logical(0, 0, S)
    assert np.array_equal(to_np(kb).view(np.uint16), k.view(np.uint16))
    assert np.array_equal(to_np(vb).view(np.uint16), v.view(np.uint16))


def _draft_layer_case(k, d, P0, seed):
    """Inputs of the drafter's own attention in round d (src/model/minicpm4/minicpm4_eagle.cuh:359):
    k queries (the newest k draft tokens) over P0 prefix tokens + k*d draft tokens, with
    Mask(eagle_mask_2d, k, k*d): bit j of row i refers to draft token j of the k*d."""
    import oracle
    vocab = 300
    t = oracle.DraftTree(k, d + 1)
    v, p = synth.draft_topk_rows(1, k, vocab, seed, 0)
    t.begin(v[0], p[0])
    for it in range(1, d):
        v, p = synth.draft_topk_rows(k, k, vocab, seed, it)
        t.extend(it, v, p)
    mask = t.mask.copy().reshape(k, 1)  # the mask the round-d attention uses: bits over k*d columns
    S = P0 + k * d
    q = synth.normal_f16((k, HQ, D), seed, 1)
    kk = synth.normal_f16((S, HKV, D), seed, 2)
    vv = synth.normal_f16((S, HKV, D), seed, 3)
    return mask, q, kk, vv, S


@pytest.mark.parametrize("k,d,P0,seed", [(10, 1, 500, 1), (10, 3, 500, 2), (10, 6, 4096, 3), (4, 5, 61, 4), (8, 8, 0, 5)])
def test_draft_layer_mask_range(gpu, orc, k, d, P0, seed):
    """mask_k_range = k*d > T = k: the mask bits cover more key columns than there are queries."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    mask, q, kk, vv, S = _draft_layer_case(k, d, P0, seed)
    npages = (S + 255) // 256 + 1
    cache = PagedKVCache(1, HKV, npages, fill=float("nan"))
    cache.write_logical(0, 0, to_dev(torch, kk[:S - k]), to_dev(torch, vv[:S - k]))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, mask), mask_k_range=k * d,
                             k_new=to_dev(torch, kk[S - k:]), v_new=to_dev(torch, vv[S - k:]))
    torch.cuda.synchronize()
    ref = orc.tree_attention(q, kk, vv, mask, S - k, mask_k_range=k * d)
    assert_close_f16(to_np(out), ref, "draft-layer attention k=%d d=%d" % (k, d))


@pytest.mark.parametrize("k,d,P0,window,splits,seed", [
    (10, 1, 100, 128, 0, 1), (10, 3, 127, 128, 0, 2), (10, 3, 128, 128, 1, 3), (10, 3, 129, 128, 0, 4),
    (10, 6, 1000, 128, 0, 5), (10, 6, 1000, 512, 3, 6), (10, 5, 1024, 1024, 0, 7), (10, 5, 1025, 1024, 0, 8),
    (10, 6, 5000, 1024, 0, 9), (10, 6, 5000, 1024, 5, 10), (4, 5, 61, 256, 0, 11), (8, 8, 2049, 2048, 0, 12),
    (10, 2, 9000, 8192, 0, 13), (10, 6, 300, 4096, 0, 14), (10, 3, 115, 128, 0, 15), (10, 6, 140, 128, 2, 16)])
def test_draft_layer_block_window(gpu, orc, k, d, P0, window, splits, seed):
    """The drafter's own layer with its block sliding window (eagle_window_size): only the key blocks of 128 from
    ceil(P/128) - window/128 on are visited.  Queries are the newest k draft tokens, the mask covers k*d
    columns, the new rows are appended by the kernel; the page table is a seeded permutation.  The last two
    cases put the first mask column below the window's first key: the window wins."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    mask, q, kk, vv, S = _draft_layer_case(k, d, P0, seed)
    max_len = S + [0, 1, 100, 300][seed % 4]
    npages = (max_len + 255) // 256 + 1
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32)
    cache = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
    cache.write_logical(0, 0, to_dev(torch, kk[:S - k]), to_dev(torch, vv[:S - k]))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, max_len, to_dev(torch, mask), mask_k_range=k * d,
                             k_new=to_dev(torch, kk[S - k:]), v_new=to_dev(torch, vv[S - k:]), num_splits=splits,
                             block_window_size=window)
    torch.cuda.synchronize()
    ref = orc.tree_attention(q, kk, vv, mask, S - k, mask_k_range=k * d, block_window_size=window)
    assert_close_f16(to_np(out), ref, "windowed draft-layer attention k=%d d=%d P0=%d window=%d" % (k, d, P0, window))
    kc, vc = cache.read_logical(0, 0, S)
    assert np.array_equal(to_np(kc).view(np.uint16), kk.view(np.uint16))
    assert np.array_equal(to_np(vc).view(np.uint16), vv.view(np.uint16))
    # the window must matter whenever it cuts keys off: compare with the full-context result
    P = S - k
    if (P + 127) // 128 - window // 128 > 0:
        full = orc.tree_attention(q, kk, vv, mask, P, mask_k_range=k * d)
        assert np.abs(ref.astype(np.float32) - full.astype(np.float32)).max() > 1e-3


@pytest.mark.parametrize("P,T,window,rope", [(4096, 60, 1024, False), (4097, 60, 1024, True), (700, 64, 256, True), (33000, 60, 2048, False)])
def test_tree_block_window_with_rope(gpu, orc, P, T, window, rope):
    """The window together with a verify-sized tree, the fused append and (optionally) the fused rotary
    embedding: the cost-relevant part is that the stream starts at the window's first block."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    tree = synth.random_tree(T, 900 + P, max_children=5, max_depth=10)
    S = P + T
    npages = (S + 255) // 256 + 1
    q = synth.normal_f16((T, HQ, D), P, 1)
    k = synth.normal_f16((S, HKV, D), P, 2)
    v = synth.normal_f16((S, HKV, D), P, 3)
    cache = PagedKVCache(1, HKV, npages, fill=float("nan"))
    cache.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    table, q_ref, k_ref = None, q, k
    if rope:
        inv_freq = (10000.0 ** (-np.arange(D // 2, dtype=np.float64) / (D // 2))).astype(np.float32)
        table = ops.rope_table(to_dev(torch, tree.positions(P)), to_dev(torch, inv_freq))
        q_ref, k_rot = orc.rope(q, k[P:], table=to_np(table))
        k_ref = np.concatenate([k[:P], k_rot], 0)
    out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, tree.mask), k_new=to_dev(torch, k[P:]),
                             v_new=to_dev(torch, v[P:]), rope=table, block_window_size=window)
    torch.cuda.synchronize()
    ref = orc.tree_attention(q_ref, k_ref, v, tree.mask, P, block_window_size=window)
    assert_close_f16(to_np(out), ref, "windowed tree attention P=%d T=%d window=%d rope=%s" % (P, T, window, rope))
    kc, _ = cache.read_logical(0, P, T)
    assert np.array_equal(to_np(kc).view(np.uint16), k_ref[P:].view(np.uint16))


def test_block_window_argument_checks(gpu):
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    cache = PagedKVCache(1, HKV, 2)
    q = torch.zeros((4, HQ, D), dtype=torch.float16, device="cuda")
    kv_len = torch.tensor([100], dtype=torch.int32, device="cuda")
    for bad in (64, 127, -128):
        with pytest.raises(Exception):
            ops.tree_attention(q, cache, 0, kv_len, 100, None, block_window_size=bad)
    # more than 64 rows: the reference would start the window per 64-row query block; rejected, not approximated
    q100 = torch.zeros((100, HQ, D), dtype=torch.float16, device="cuda")
    kv_len.fill_(300)
    with pytest.raises(ValueError, match="at most 64"):
        ops.tree_attention(q100, cache, 0, kv_len, 300, None, block_window_size=128)


@pytest.mark.parametrize("T,num_iter,topk", [(60, 6, 10), (128, 8, 16)])
def test_32k_context_one_layer_against_oracle(gpu, orc, T, num_iter, topk):
    """Configs 4 and 5 at their real size for one layer: 32768-token prefix, 60- and 128-node trees."""
    tree = synth.eagle_tree(num_iter, topk, T, seed=1)
    out, ref = _case(gpu, orc, tree, 32768, seed=40 + T)
    assert_close_f16(out, ref, "attention at 32K context, T=%d" % T)


def test_128k_context_closed_form_and_split_invariance(gpu):
    """Config 4 at 128K context, checked through properties that need no CPU pass over the keys:
    (1) with identical K rows every visible key weighs the same, so row i is the mean of its visible
    V rows -- prefix and ancestors -- which numpy computes in fp64 from running sums;
    (2) on random K the result must not depend on the split count beyond fp16 rounding."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    P, T = 131072, 60
    S = P + T
    tree = synth.eagle_tree(6, 10, T, seed=2)
    npages = (S + 255) // 256 + 1
    table = synth.rng(5, 4).permutation(npages).astype(np.int32)
    q = synth.normal_f16((T, HQ, D), 70, 1)
    v = synth.normal_f16((S, HKV, D), 70, 3)
    k_same = np.broadcast_to(synth.normal_f16((1, HKV, D), 70, 2), (S, HKV, D)).copy()
    cache = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
    cache.write_logical(0, 0, to_dev(torch, k_same), to_dev(torch, v))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    mask = to_dev(torch, tree.mask)
    out = to_np(ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, mask)).astype(np.float64)
    v64 = v.astype(np.float64)
    prefix_sum = v64[:P].sum(0)                                   # [Hkv, D]
    for i in range(T):
        anc = [j for j in range(T) if (int(tree.mask[i, j >> 6]) >> (j & 63)) & 1]
        mean = (prefix_sum + v64[P + np.array(anc)].sum(0)) / (P + len(anc))
        for h in range(HQ):
            assert np.abs(out[i, h] - mean[h // (HQ // HKV)]).max() < 2e-3, (i, h)
    # random keys: 32 (automatic), 16 and 64 splits agree
    k = synth.normal_f16((S, HKV, D), 71, 2)
    cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
    outs = [to_np(ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, mask, num_splits=s)) for s in (0, 16, 64)]
    for o in outs[1:]:
        assert_close_f16(o, outs[0], "split invariance at 128K", atol=4e-3, rtol=4e-3)


def test_one_million_token_context_closed_form(gpu):
    """A million-token prefix (not a multiple of anything) on a permuted page table: with identical K rows every visible key
    weighs the same, so a row's output is the mean of its visible V rows (fp64 running sums in numpy) -- nothing in the index
    arithmetic (page offsets beyond 2^32 bytes, split ranges, the merge of 32 splits) may lose a key on the way."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    P, T = 1000003, 60
    S = P + T
    tree = synth.eagle_tree(6, 10, T, seed=2)
    npages = (S + 255) // 256 + 1
    table = synth.rng(5, 4).permutation(npages).astype(np.int32)
    q = synth.normal_f16((T, HQ, D), 70, 1)
    v = synth.rng(70, 3).standard_normal((S, HKV, D), dtype=np.float32).astype(np.float16)
    k_row = synth.normal_f16((1, HKV, D), 70, 2)
    cache = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
    step = 1 << 18
    for a in range(0, S, step):
        b = min(S, a + step)
        cache.write_logical(0, a, to_dev(torch, np.ascontiguousarray(np.broadcast_to(k_row, (b - a, HKV, D)))), to_dev(torch, v[a:b]))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    out = to_np(ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, tree.mask))).astype(np.float64)
    v64 = v.astype(np.float64)
    prefix_sum = v64[:P].sum(0)
    for i in range(T):
        anc = [j for j in range(T) if (int(tree.mask[i, j >> 6]) >> (j & 63)) & 1]
        mean = (prefix_sum + v64[P + np.array(anc)].sum(0)) / (P + len(anc))
        for h in range(HQ):
            assert np.abs(out[i, h] - mean[h // (HQ // HKV)]).max() < 2e-5, (i, h)  # outputs are O(3e-3) at this length


def _sweep_configs():
    """Seeded random (P, T, mode, splits, slack) tuples, biased to tile (64), page (256) and wave-row (2, 16 nodes)
    boundaries; slack = how far the host-side bound on the KV length exceeds the true length."""
    g = synth.rng(2024, 7)
    edges_p = [0, 1, 2, 3, 62, 63, 64, 65, 127, 128, 129, 191, 192, 250, 255, 256, 257, 258, 319, 320, 511, 512, 513,
               1023, 1024, 1025, 4095, 4096, 4097]
    edges_t = [1, 2, 3, 8, 15, 16, 17, 31, 32, 33, 60, 63, 64, 65, 100, 127, 128]
    out = []
    for i in range(36):
        P = int(edges_p[g.integers(len(edges_p))]) if g.random() < 0.7 else int(g.integers(0, 9000))
        T = int(edges_t[g.integers(len(edges_t))]) if g.random() < 0.7 else int(g.integers(1, 129))
        mode = ["in_cache", "append", "append_rope"][int(g.integers(3))]
        splits = [0, 0, 1, 3][int(g.integers(4))]
        slack = [0, 0, 1, 63, 64, 200, 1000][int(g.integers(7))]
        out.append((P, T, mode, splits, slack, i))
    return out


@pytest.mark.parametrize("P,T,mode,splits,slack,seed", _sweep_configs())
def test_randomised_shape_sweep(gpu, orc, P, T, mode, splits, slack, seed):
    """Prefix lengths, tree sizes, split counts and bounds drawn around the kernel's tile, page and row-block
    boundaries, in each of its three input modes, against the oracle; appended rows are checked bit for bit."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    tree = synth.random_tree(T, 500 + seed, max_children=5, max_depth=10)
    S = P + T
    max_len = S + slack
    npages = (max_len + 255) // 256 + 1
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32)
    q = synth.normal_f16((T, HQ, D), seed, 1)
    k = synth.normal_f16((S, HKV, D), seed, 2)
    v = synth.normal_f16((S, HKV, D), seed, 3)
    cache = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    mask = to_dev(torch, tree.mask)
    q_ref, k_ref = q, k
    if mode == "in_cache":
        cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
        out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, max_len, mask, num_splits=splits)
    else:
        if P:
            cache.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
        rope = None
        if mode == "append_rope":
            inv_freq = (10000.0 ** (-np.arange(D // 2, dtype=np.float64) / (D // 2))).astype(np.float32)
            rope = ops.rope_table(to_dev(torch, tree.positions(P)), to_dev(torch, inv_freq))
            q_ref, k_rot = orc.rope(q, k[P:], table=to_np(rope))
            k_ref = np.concatenate([k[:P], k_rot], 0)
        out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, max_len, mask, num_splits=splits,
                                 k_new=to_dev(torch, k[P:]), v_new=to_dev(torch, v[P:]), rope=rope)
    torch.cuda.synchronize()
    ref = orc.tree_attention(q_ref, k_ref, v, tree.mask, P)
    assert_close_f16(to_np(out), ref, "P=%d T=%d %s splits=%d slack=%d" % (P, T, mode, splits, slack))
    if mode != "in_cache":
        kc, vc = cache.read_logical(0, 0, S)
        assert np.array_equal(to_np(kc).view(np.uint16), k_ref.view(np.uint16))
        assert np.array_equal(to_np(vc).view(np.uint16), v.view(np.uint16))


def _heads_case(torch, orc, HQ_, HKV_, P, T, mode, seed):
    """One attention call with HQ_ query heads on HKV_ KV heads (any ratio) against the oracle; appended rows bit for bit."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    tree = synth.random_tree(T, seed, max_children=5, max_depth=10)
    S = P + T
    npages = (S + 255) // 256 + 1
    table = synth.rng(seed, 4).permutation(npages).astype(np.int32)
    q = synth.normal_f16((T, HQ_, D), seed, 1)
    k = synth.normal_f16((S, HKV_, D), seed, 2)
    v = synth.normal_f16((S, HKV_, D), seed, 3)
    cache = PagedKVCache(1, HKV_, npages, block_table=table, fill=float("nan"))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    mask = to_dev(torch, tree.mask)
    q_ref, k_ref = q, k
    if mode == "in_cache":
        cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
        out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, mask)
    else:
        if P:
            cache.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
        rope = None
        if mode == "append_rope":
            inv_freq = (10000.0 ** (-np.arange(D // 2, dtype=np.float64) / (D // 2))).astype(np.float32)
            rope = ops.rope_table(to_dev(torch, tree.positions(P)), to_dev(torch, inv_freq))
            q_ref, k_rot = orc.rope(q, k[P:], table=to_np(rope))
            k_ref = np.concatenate([k[:P], k_rot], 0)
        out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, mask, k_new=to_dev(torch, k[P:]), v_new=to_dev(torch, v[P:]), rope=rope)
    torch.cuda.synchronize()
    ref = orc.tree_attention(q_ref, k_ref, v, tree.mask, P)
    assert_close_f16(to_np(out), ref, "Hq=%d Hkv=%d P=%d T=%d %s" % (HQ_, HKV_, P, T, mode))
    if mode != "in_cache":
        kc, vc = cache.read_logical(0, 0, S)
        assert np.array_equal(to_np(kc).view(np.uint16), k_ref.view(np.uint16))
        assert np.array_equal(to_np(vc).view(np.uint16), v.view(np.uint16))


@pytest.mark.parametrize("HQ_,HKV_", [(32, 8), (32, 32), (8, 1), (40, 8), (48, 16), (6, 2), (1, 1)])
@pytest.mark.parametrize("P,T,mode", [(1000, 16, "append"), (4096, 60, "append"), (300, 60, "in_cache"), (2049, 128, "append_rope"), (64, 1, "append")])
def test_other_head_counts(gpu, orc, HQ_, HKV_, P, T, mode):
    """Query / KV head counts other than the 32 / 2 of the configurations: 4, 1, 8, 5 (not a power of two), 3 and 1 query heads per
    KV head, one KV head and thirty-two -- the packing of rows into waves, the split counts and the merge all depend on them."""
    _heads_case(gpu, orc, HQ_, HKV_, P, T, mode, HQ_ * 1000 + P)


@pytest.mark.parametrize("P,T,splits,fused_append,rope", [
    (4096, 60, 0, True, False),    # the verify step's shape: 16 splits (two groups) / 32 splits (one group), 256 workgroups
    (4096, 60, 0, True, True),
    (33000, 60, 0, False, False),
    (700, 128, 3, True, False),
    (1500, 60, 7, False, False),   # a split count that does not divide the blocks of a unit evenly
    (250, 16, 2, True, False),
])
def test_merge_in_launch_equals_separate_merge(gpu, set_option, P, T, splits, fused_append, rope):
    """The split workgroups' own merge (device-scope partials, per-unit arrival counters) and the combine launch run the
    same arithmetic on the same partials: outputs must be bit-identical.  Each path is called three times in a row, then
    with another split count on the same workspace, so that the counters are seen to come back to rest."""
    torch = gpu
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    tree = synth.eagle_tree(6, 10, T, seed=P) if T > 16 else synth.eagle_tree(3, 4, T, seed=P)
    S = P + T
    q = to_dev(torch, synth.normal_f16((T, HQ, D), P, 1))
    k = synth.normal_f16((S, HKV, D), P, 2)
    v = synth.normal_f16((S, HKV, D), P, 3)
    npages = (S + 255) // 256 + 1
    table = synth.rng(P, 4).permutation(npages).astype(np.int32)
    mask = to_dev(torch, tree.mask)
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    table_rope = None
    if rope:
        pos = torch.arange(P, P + T, dtype=torch.int32, device="cuda")
        inv_freq = to_dev(torch, (1.0 / (10000.0 ** (np.arange(0, D, 2, dtype=np.float32) / D))).astype(np.float32))
        table_rope = ops.rope_table(pos, inv_freq)
    outs = {}
    for mode in (0, 1):
        set_option("attn_merge_in_launch", mode)
        got = []
        for rep, sp in enumerate((splits, splits, splits, 4, splits)):
            cache = PagedKVCache(1, HKV, npages, block_table=table, fill=float("nan"))
            n_cached = P if fused_append else S
            cache.write_logical(0, 0, to_dev(torch, k[:n_cached]), to_dev(torch, v[:n_cached]))
            kw = dict(k_new=to_dev(torch, k[P:]), v_new=to_dev(torch, v[P:])) if fused_append else {}
            out = ops.tree_attention(q, cache, 0, kv_len, S, mask, num_splits=sp, rope=table_rope, **kw)
            torch.cuda.synchronize()
            got.append(to_np(out))
        outs[mode] = got
    for a, b in zip(outs[0], outs[1]):
        assert np.all(np.isfinite(a.astype(np.float32)))
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_merge_counter_blocks_stay_with_their_workspaces(gpu):
    """The library hands a block of merge counters to each workspace pointer it meets (a fixed number per device) and
    never takes one back while the workspace may still be in use: workspaces beyond that number are merged by the
    separate launch.  Every call must give the same bits whichever way it was merged, and a launch captured early must
    still own its counters after many other workspaces have come and gone."""
    torch = gpu
    from cpm.cu_amd import lib, ops
    from cpm.cu_amd.kvcache import PagedKVCache
    T, P = 60, 2000
    tree = synth.eagle_tree(6, 10, T, seed=3)
    S = P + T
    q = to_dev(torch, synth.normal_f16((T, HQ, D), 7, 1))
    k = synth.normal_f16((S, HKV, D), 7, 2)
    v = synth.normal_f16((S, HKV, D), 7, 3)
    npages = (S + 255) // 256 + 1
    cache = PagedKVCache(1, HKV, npages)
    cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
    mask = to_dev(torch, tree.mask)
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    merge_mode = lib.get().raw.cpmcu_tree_attention_merge_mode
    # a graph captured on the current workspace (one eager call first: its counters are assigned outside the capture)
    out_g = torch.empty_like(q)
    ref = to_np(ops.tree_attention(q, cache, 0, kv_len, S, mask, out=out_g))
    ws_g = ops._workspaces[("attn", q.device)]
    in_launch = merge_mode(ws_g.data_ptr())
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            ops.tree_attention(q, cache, 0, kv_len, S, mask, out=out_g)
    keep, modes = [], []
    for i in range(40):  # more distinct workspaces than the library has counter blocks; each is used twice in a row
        ops._workspaces.pop(("attn", q.device), None)
        for rep in range(2):
            out = ops.tree_attention(q, cache, 0, kv_len, S, mask)
            torch.cuda.synchronize()
            assert np.array_equal(to_np(out).view(np.uint16), ref.view(np.uint16)), "call %d.%d" % (i, rep)
        keep.append(ops._workspaces[("attn", q.device)])  # kept alive: every call sees a new address
        modes.append(merge_mode(keep[-1].data_ptr()))
    assert len({t.data_ptr() for t in keep}) == 40
    assert modes[-1] == 0, "the library has 32 counter blocks per device: the last of 40 workspaces cannot have one"
    assert modes == sorted(modes, reverse=True), "a workspace met earlier lost its block to a later one: %s" % modes
    assert merge_mode(ws_g.data_ptr()) == in_launch
    # the captured launch replayed next to eager launches on another workspace: same bits
    for rep in range(5):
        out_g.fill_(float("nan"))
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            graph.replay()
        out = ops.tree_attention(q, cache, 0, kv_len, S, mask)
        torch.cuda.synchronize()
        assert np.array_equal(to_np(out_g).view(np.uint16), ref.view(np.uint16)), rep
        assert np.array_equal(to_np(out).view(np.uint16), ref.view(np.uint16)), rep
    del graph
    for t in keep:
        ops.release_attention_workspace(t)
    ops._workspaces[("attn", q.device)] = ws_g


@pytest.mark.parametrize("P,T", [(4096, 60), (33000, 60), (700, 128)])
def test_merge_wait_that_runs_out_leaves_the_share_to_the_last_arrival(gpu, set_option, P, T):
    """With the wait limit at zero every workgroup but the last of a unit gives up at once (unless everyone has
    arrived already), marks its share as abandoned and leaves; the last arrival merges those shares.  The output must be
    what the separate merge launch gives, bit for bit, the counter of abandoned waits must say so, and the next call must be whole again."""
    torch = gpu
    from cpm.cu_amd import lib, ops
    from cpm.cu_amd.kvcache import PagedKVCache
    tree = synth.eagle_tree(6, 10, T, seed=P)
    S = P + T
    q = to_dev(torch, synth.normal_f16((T, HQ, D), P, 1))
    k = synth.normal_f16((S, HKV, D), P, 2)
    v = synth.normal_f16((S, HKV, D), P, 3)
    npages = (S + 255) // 256 + 1
    cache = PagedKVCache(1, HKV, npages)
    cache.write_logical(0, 0, to_dev(torch, k), to_dev(torch, v))
    mask = to_dev(torch, tree.mask)
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    names, splits, _, _ = ops.attention_plan(T, HQ, HKV, S)  # the split count a self-merging launch of this shape takes
    assert "combine" not in names and splits > 1
    set_option("attn_merge_in_launch", 0)
    ref = to_np(ops.tree_attention(q, cache, 0, kv_len, S, mask, num_splits=splits))
    set_option("attn_merge_in_launch", 1)
    L = lib.get()
    L.synchronize()
    set_option("attn_merge_in_launch", 1)  # (also puts workspaces back on the in-launch merge after an earlier test's abandoned waits)
    ws = ops._workspaces[("attn", q.device)].data_ptr()
    if not L.raw.cpmcu_tree_attention_merge_mode(ws):
        pytest.skip("this process has used up the library's counter blocks: the workspace is merged by the separate launch")
    seen0 = L.raw.cpmcu_attention_abandoned_waits()
    for wait_us in (0, 0, 2000, 0):
        set_option("attn_merge_wait_us", wait_us)
        out = torch.full_like(q, float("nan"))  # a share nobody merged would stay NaN
        ops.tree_attention(q, cache, 0, kv_len, S, mask, num_splits=splits, out=out)
        torch.cuda.synchronize()
        assert np.array_equal(to_np(out).view(np.uint16), ref.view(np.uint16)), "wait %d us" % wait_us
    # the abandoned waits are counted at the next synchronising call of the library, and the device's workspaces go back
    # to the separate merge launch until the option is set again
    L.synchronize()
    assert L.raw.cpmcu_attention_abandoned_waits() > seen0
    assert L.raw.cpmcu_tree_attention_merge_mode(ws) == 0
    out = torch.full_like(q, float("nan"))
    ops.tree_attention(q, cache, 0, kv_len, S, mask, num_splits=splits, out=out)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(out).view(np.uint16), ref.view(np.uint16))
    L.synchronize()
    set_option("attn_merge_in_launch", 1)
    assert L.raw.cpmcu_tree_attention_merge_mode(ws) == 1


def test_two_self_merging_launches_side_by_side(gpu):
    """Attention calls on two streams with a workspace each (the condition under which calls may overlap on one GPU):
    whether the launches run one after the other or share the CUs, every output must carry the bits of the same call
    made alone."""
    torch = gpu
    from cpm.cu_amd import lib, ops
    from cpm.cu_amd.kvcache import PagedKVCache
    T, P, layers = 60, 4096, 3
    tree = synth.eagle_tree(6, 10, T, seed=11)
    S = P + T
    mask = to_dev(torch, tree.mask)
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    npages = (S + 255) // 256 + 1
    need = lib.get().raw.cpmcu_tree_attention_workspace_bytes(T, HQ, HKV, S)
    sides = []
    for i in range(2):
        cache = PagedKVCache(layers, HKV, npages)
        for l in range(layers):
            cache.write_logical(l, 0, to_dev(torch, synth.normal_f16((S, HKV, D), 20 + i, 2 + l)),
                                to_dev(torch, synth.normal_f16((S, HKV, D), 30 + i, 2 + l)))
        sides.append(dict(q=to_dev(torch, synth.normal_f16((T, HQ, D), 40 + i, 1)), cache=cache,
                          ws=torch.empty(need, dtype=torch.uint8, device="cuda"), stream=torch.cuda.Stream()))
    key = ("attn", sides[0]["q"].device)
    saved = ops._workspaces.get(key)

    def call(side, l, out):
        ops._workspaces[key] = side["ws"]
        ops.tree_attention(side["q"], side["cache"], l, kv_len, S, mask, out=out)
    try:
        refs = []
        for side in sides:
            row = []
            for l in range(layers):
                o = torch.empty_like(side["q"])
                call(side, l, o)
                torch.cuda.synchronize()
                row.append(to_np(o))
            refs.append(row)
        for rep in range(10):
            outs = [[torch.full_like(side["q"], float("nan")) for _ in range(layers)] for side in sides]
            torch.cuda.synchronize()
            for l in range(layers):
                for i, side in enumerate(sides):
                    with torch.cuda.stream(side["stream"]):
                        call(side, l, outs[i][l])
            torch.cuda.synchronize()
            for i in range(2):
                for l in range(layers):
                    assert np.array_equal(to_np(outs[i][l]).view(np.uint16), refs[i][l].view(np.uint16)), (rep, i, l)
    finally:
        for side in sides:
            ops.release_attention_workspace(side["ws"])
        if saved is None:
            ops._workspaces.pop(key, None)
        else:
            ops._workspaces[key] = saved
