"""The path in bfloat16 (torch_dtype = 1 of src/entry.cu:26-59) against the CPU oracle in bfloat16.

numpy has no bfloat16: host arrays are float16-typed containers whose 16 bits are bfloat16 patterns (`orc.encode` /
`orc.decode` convert to and from float32), and the same containers travel to the device.  Integer results are bit-exact as
in fp16; floating-point results are compared within max-abs 2e-2 and a normalised-max error of 2e-2 -- one bfloat16 ulp
is 2^-8 of the value, eight times an fp16 ulp, and a result that lands on the other side of a rounding boundary (the
fp32 sums are taken in another order on the device) is off by a whole one.
"""
import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 2, 128
RTOL_BF16 = 2e-2


@pytest.fixture
def bf16(gpu, orc, set_option):
    """Library and oracle in bfloat16 for one test."""
    set_option("dtype", 1)
    orc.set_dtype("bf16")
    yield
    orc.set_dtype("f16")


def normal_bf16(orc, shape, seed, stream, std=1.0):
    return orc.encode(synth.rng(seed, stream).standard_normal(shape, dtype=np.float32) * std)


@pytest.mark.parametrize("groups", [2, 1])
@pytest.mark.parametrize("P,T,rope", [(1024, 16, False), (4096, 60, False), (4096 - 37, 60, True), (700, 128, False)])
def test_bf16_tree_attention_with_fused_append(gpu, orc, bf16, set_option, groups, P, T, rope):
    torch = gpu
    from cpm.cu_amd import ops
    from cpm.cu_amd.kvcache import PagedKVCache
    set_option("attn_kv_groups", groups)
    tree = synth.eagle_tree(6, 10, T, seed=P) if T > 16 else synth.eagle_tree(4, 4, T, seed=P)
    S = P + T
    q = normal_bf16(orc, (T, HQ, D), P, 1)
    k = normal_bf16(orc, (S, HKV, D), P, 2)
    v = normal_bf16(orc, (S, HKV, D), P, 3)
    npages = (S + 255) // 256 + 1
    cache = PagedKVCache(1, HKV, npages, block_table=synth.rng(P, 4).permutation(npages).astype(np.int32))
    cache.write_logical(0, 0, to_dev(torch, k[:P]), to_dev(torch, v[:P]))
    kv_len = torch.tensor([S], dtype=torch.int32, device="cuda")
    table = None
    q_ref, k_ref = q, k
    if rope:
        pos = np.arange(P, P + T, dtype=np.int32)
        inv_freq = (1.0 / (10000.0 ** (np.arange(0, D, 2, dtype=np.float32) / D))).astype(np.float32)
        table = ops.rope_table(to_dev(torch, pos), to_dev(torch, inv_freq))
        q_ref, k_rot = orc.rope(q, k[P:], table=to_np(table))
        k_ref = np.concatenate([k[:P], k_rot])
    out = ops.tree_attention(to_dev(torch, q), cache, 0, kv_len, S, to_dev(torch, tree.mask), k_new=to_dev(torch, k[P:]),
                             v_new=to_dev(torch, v[P:]), rope=table)
    torch.cuda.synchronize()
    ref = orc.tree_attention(q_ref, k_ref, v, tree.mask, P)
    assert_close_f16(orc.decode(to_np(out)), orc.decode(ref), "bf16 attention P=%d T=%d" % (P, T), rtol=RTOL_BF16)
    kc, vc = cache.read_logical(0, 0, S)
    assert np.array_equal(to_np(kc).view(np.uint16), k_ref.view(np.uint16))
    assert np.array_equal(to_np(vc).view(np.uint16), v.view(np.uint16))


def assert_close_bf16(orc, got, ref, what):
    """got / ref: bfloat16 containers.  Normalised-max error within 2e-2; absolute error within 2e-2 or, where the values
    are larger than 2.5, one bfloat16 ulp of the largest magnitude (2^-7 of it)."""
    g, r = orc.decode(got), orc.decode(ref)
    top = float(np.abs(r).max())
    return assert_close_f16(g, r, what, atol=max(2e-2, top * 2.0 ** -7), rtol=RTOL_BF16)


@pytest.mark.parametrize("n,V,H,tiled,scale", [(60, 3001, 512, False, None), (16, 40000, 1024, True, 0.3125), (128, 36000, 512, True, None),
                                                (33, 2100, 6144, False, None)])
def test_bf16_target_head_and_argmax(gpu, orc, bf16, n, V, H, tiled, scale):
    torch = gpu
    from cpm.cu_amd import ops
    hid = normal_bf16(orc, (n, H), V, 1)
    w = normal_bf16(orc, (V, H), V, 2, std=0.02)
    d_w = ops.tile_head_weight(to_dev(torch, w)) if tiled else to_dev(torch, w)
    gt, logits = ops.lm_head_argmax(to_dev(torch, hid), d_w, head_scale=scale, want_logits=True)
    gt2 = ops.lm_head_argmax(to_dev(torch, hid), d_w, head_scale=scale)
    torch.cuda.synchronize()
    z_dev = to_np(logits)
    z_ref = orc.lm_head(hid, w, head_scale=scale)
    assert_close_bf16(orc, z_dev, z_ref, "bf16 target logits")
    assert np.array_equal(to_np(gt), to_np(gt2))
    assert np.array_equal(to_np(gt), orc.argmax(z_dev))  # staged: the device's own logits decide, lowest index on ties
    assert np.array_equal(orc.argmax(z_dev), np.argmax(orc.decode(z_dev), axis=1))


def test_bf16_target_head_full_size(gpu, orc, bf16):
    """Config 2's head in bfloat16: 60 rows against 73448 x 4096, tiled (the streaming kernel)."""
    torch = gpu
    from cpm.cu_amd import ops
    n, V, H = 60, 73448, 4096
    hid = normal_bf16(orc, (n, H), 0, 1)
    w = normal_bf16(orc, (V, H), 0, 2, std=0.02)
    wt = ops.tile_head_weight(to_dev(torch, w))
    assert "head_gemm_stream_kernel" in ops.head_plan(n, wt)[0]
    gt, logits = ops.lm_head_argmax(to_dev(torch, hid), wt, want_logits=True)
    torch.cuda.synchronize()
    z_dev = to_np(logits)
    assert_close_bf16(orc, z_dev, orc.lm_head(hid, w), "bf16 target logits, full size")
    assert np.array_equal(to_np(gt), orc.argmax(z_dev))


@pytest.mark.parametrize("n,V,Vs,H,k,tiled", [(10, 6000, 4096, 512, 10, False), (16, 9000, 4096 + 40, 2048, 10, True), (1, 3000, 2048, 1024, 10, False),
                                               (10, 73448, 32768, 4096, 10, True),
                                               # k beyond 16: the top-k bound is shared between the waves
                                               (7, 40000, 32768, 512, 32, True), (4, 9000, 8192, 512, 20, False), (3, 50000, 40960, 512, 24, True)])
def test_bf16_frspec_head_topk(gpu, orc, bf16, n, V, Vs, H, k, tiled):
    """The FR-Spec head in bfloat16: logits within tolerance, and the ranking of the rounded log-probabilities bit-exact
    when the oracle ranks the device's own logits and row statistics (bfloat16 keeps 8 bits: far more ties than fp16)."""
    torch = gpu
    from cpm.cu_amd import ops
    hid = normal_bf16(orc, (n, H), Vs, 1)
    w = normal_bf16(orc, (V, H), Vs, 2, std=0.02)
    remap = synth.frspec_remap(V, Vs, Vs % 13)
    d_w, d_remap = to_dev(torch, w), to_dev(torch, remap)
    sub = orc.gather_rows(w, remap)
    d_sub = ops.tile_head_weight(d_w, d_remap) if tiled else ops.gather_rows(d_w, d_remap)
    r = ops.frspec_head_topk(to_dev(torch, hid), d_sub, d_remap, k)
    torch.cuda.synchronize()
    z_dev = to_np(r["logits"])
    assert_close_bf16(orc, z_dev, orc.lm_head(hid, sub), "bf16 FR-Spec logits")
    stats = to_np(r["row_stats"])
    lp_staged = orc.log_softmax_apply(z_dev, stats[:, 0], stats[:, 1])
    val_s, pos_s = orc.topk(lp_staged, k)
    assert np.array_equal(to_np(r["pos"]), pos_s), "top-k positions differ from the staged oracle"
    assert np.array_equal(to_np(r["val"]).view(np.uint16), val_s.view(np.uint16))
    assert np.array_equal(to_np(r["ids"]), remap[pos_s])
    _, m_ref, lse_ref = orc.log_softmax(z_dev)
    assert np.allclose(stats[:, 0], m_ref, atol=1e-6) and np.allclose(stats[:, 1], lse_ref, atol=1e-3)


@pytest.mark.parametrize("n,dim", [(3, 32768), (2, 40001), (4, 510)])
def test_bf16_log_softmax_and_raw_topk(gpu, orc, bf16, n, dim):
    torch = gpu
    from cpm.cu_amd import ops
    x = orc.encode(synth.rng(dim, 5).standard_normal((n, dim)).astype(np.float32) * 1.3)
    d = to_dev(torch, x)
    stats = to_np(ops.log_softmax_(d))
    torch.cuda.synchronize()
    staged = orc.log_softmax_apply(x, stats[:, 0], stats[:, 1])
    assert np.array_equal(to_np(d).view(np.uint16), staged.view(np.uint16))
    lp_ref, m_ref, lse_ref = orc.log_softmax(x)
    assert np.array_equal(stats[:, 0], m_ref) and np.allclose(stats[:, 1], lse_ref, atol=1e-4)
    for top in (10, 59):  # the raw ranking works on bit patterns: same order for both element types
        val, pos = ops.topk(to_dev(torch, x), top)
        torch.cuda.synchronize()
        v_ref, p_ref = orc.topk(x, top)
        assert np.array_equal(to_np(pos), p_ref) and np.array_equal(to_np(val).view(np.uint16), v_ref.view(np.uint16))


@pytest.mark.parametrize("k,num_iter,T,seed", [(10, 6, 60, 4), (4, 4, 16, 3)])
def test_bf16_draft_tree(gpu, orc, bf16, k, num_iter, T, seed):
    """The drafter's running log-probs are added and rounded in the element type (cumsum_kernel of the reference on T):
    the tree built from bfloat16 rows equals the oracle's."""
    torch = gpu
    from test_draft_tree_cpu import run_oracle
    from test_gpu_draft_tree import run_gpu
    vocab, full = 500, 2000
    remap = synth.frspec_remap(full, vocab, seed)
    vals, poss = [], []
    for d in range(num_iter):
        v, p = synth.draft_topk_rows(1 if d == 0 else k, k, vocab, seed, stream=d, dyadic=False)
        vals.append(orc.encode(-np.sort(-orc.decode(orc.encode(v.astype(np.float32))), axis=1)))  # descending after the rounding too
        poss.append(p)
    P = 4096 + seed
    (o_ids, o_pos, o_mask, o_parent), o_trace = run_oracle(orc, k, num_iter, T, P, vals, poss, remap)
    (g_ids, g_pos, g_mask, g_parent), g_trace, _ = run_gpu(torch, k, num_iter, T, P, vals, poss, remap)
    assert np.array_equal(g_trace[0], o_trace[0])
    for d in range(1, num_iter):
        for a, b in zip(g_trace[d], o_trace[d]):
            assert np.array_equal(a, b), "iteration %d" % d
    assert np.array_equal(g_ids[1:], o_ids[1:]) and np.array_equal(g_pos, o_pos)
    assert np.array_equal(g_parent, o_parent) and np.array_equal(g_mask, o_mask)


def test_bf16_verify_step_on_the_library_graph(gpu, orc):
    """The model-level path with torch_dtype = 1 (cpmcu_init_base_model ... cpmcu_verify_step): 3 layers, a 1000-token prefix,
    24-node tree, steps replayed from the library's graph with lengths advancing on the device.  Accept length, ids, gathered
    hidden rows and the compacted caches bit-exact against the oracle's acceptance on the device's arg-max; the attention of
    the last layer and the head's arg-max against the bfloat16 oracle."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.model import PathModel
    torch = gpu
    V, H, LAYERS, T, P0, STEPS = 3000, 512, 3, 24, 1000, 4
    tree = synth.random_tree(T, 3, max_children=3, max_depth=6)
    mask, parent = to_dev(torch, tree.mask), to_dev(torch, tree.parent)
    orc.set_dtype("bf16")
    m = None
    try:
        w = normal_bf16(orc, (V, H), 3, 2, std=0.02)
        m = PathModel(V, LAYERS, H, HQ, HKV, memory_limit=0.01, scale_lmhead=0.5, tree_size=T, num_iter=6, topk=4, dtype=1)
        m.load_head(w)
        cache = m.cache()
        kp = [normal_bf16(orc, (P0, HKV, D), 3, 10 + l) for l in range(LAYERS)]
        vp = [normal_bf16(orc, (P0, HKV, D), 3, 50 + l) for l in range(LAYERS)]
        for l in range(LAYERS):
            cache.write_logical(l, 0, to_dev(torch, kp[l]), to_dev(torch, vp[l]))
        flat = [c.reshape(P0, -1).copy() for l in range(LAYERS) for c in (kp[l], vp[l])]
        pos = to_dev(torch, tree.positions(P0))
        clen = torch.tensor([P0], dtype=torch.int32, device="cuda")
        kvlen = torch.tensor([P0 + T], dtype=torch.int32, device="cuda")
        ids = torch.zeros(T, dtype=torch.int32, device="cuda")
        gt_out = torch.zeros(T, dtype=torch.int32, device="cuda")
        result = torch.zeros(1 + T, dtype=torch.int32).pin_memory()
        f16 = dict(dtype=torch.float16, device="cuda")
        prev = torch.zeros((T, H), **f16)
        bo = [torch.zeros((T, HQ, D), **f16) for _ in range(LAYERS)]
        P = P0
        rg = synth.rng(3, 8)
        for s in range(STEPS):
            q = [normal_bf16(orc, (T, HQ, D), 3, 1000 + 10 * s + l) for l in range(LAYERS)]
            kn = [normal_bf16(orc, (T, HKV, D), 3, 2000 + 10 * s + l) for l in range(LAYERS)]
            vn = [normal_bf16(orc, (T, HKV, D), 3, 3000 + 10 * s + l) for l in range(LAYERS)]
            hidden = normal_bf16(orc, (T, H), 3, 4000 + s)
            d_hidden = to_dev(torch, hidden)
            gt = orc.argmax(orc.lm_head(hidden, w, head_scale=0.5))
            gt_dev = to_np(ops.lm_head_argmax(d_hidden, ops.tile_head_weight(to_dev(torch, w)), head_scale=0.5))
            depth = int(rg.integers(0, int(tree.depth.max()) + 1))
            pred, leaf = synth.draft_ids_for_accept(tree, gt_dev, depth, V, 300 + s)
            padded = (P + T + 31) // 32 * 32
            torch.cuda.synchronize()
            m.verify_step(T, padded, [to_dev(torch, x) for x in q], [to_dev(torch, x) for x in kn], [to_dev(torch, x) for x in vn], bo,
                          d_hidden, to_dev(torch, pred), pos, clen, kvlen, mask, parent, ids, gt_out=gt_out, prev_hidden=prev,
                          result=result, advance_length=True, cuda_graph=True)
            m.synchronize()
            a = int(result[0])
            assert np.array_equal(to_np(gt_out), gt_dev)
            assert (to_np(gt_out) == gt).mean() > 0.8  # the same head on the host, up to near-ties
            a_ref, _, path = orc.tree_accept(pred, gt_dev, tree.positions(P), P, tree.mask, tree.parent)
            assert a == a_ref == depth + 1 and list(path) == tree.path_to(leaf)
            assert np.array_equal(result[1:1 + a].numpy(), gt_dev[path])
            assert np.array_equal(to_np(prev)[:a].view(np.uint16), hidden[path].view(np.uint16))
            # attention of the last layer on the caches as they stood before this step
            l = LAYERS - 1
            k_all = np.concatenate([flat[2 * l].reshape(P, HKV, D), kn[l]])
            v_all = np.concatenate([flat[2 * l + 1].reshape(P, HKV, D), vn[l]])
            ref = orc.tree_attention(q[l], k_all, v_all, tree.mask, P)
            assert_close_f16(orc.decode(to_np(bo[l])), orc.decode(ref), "bf16 step %d, attention of layer %d" % (s, l), rtol=RTOL_BF16)
            # compaction: the accepted rows follow the prefix in every cache
            for l in range(LAYERS):
                flat[2 * l] = np.concatenate([flat[2 * l], kn[l].reshape(T, -1)[path]])
                flat[2 * l + 1] = np.concatenate([flat[2 * l + 1], vn[l].reshape(T, -1)[path]])
            P += a
            assert int(to_np(clen)[0]) == P
        for l in range(LAYERS):
            kd, vd = cache.read_logical(l, 0, P)
            assert np.array_equal(to_np(kd).reshape(P, -1).view(np.uint16), flat[2 * l].view(np.uint16))
            assert np.array_equal(to_np(vd).reshape(P, -1).view(np.uint16), flat[2 * l + 1].view(np.uint16))
    finally:
        orc.set_dtype("f16")
        if m is not None:
            m.close()
