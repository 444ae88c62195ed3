"""Whole verify steps at the benchmark configurations' real sizes, and the same path driven through the pybind
module `C` (the names of the reference's src/entry.cu:510-534), against the CPU oracle.

  * config 5 as ONE step: 32 layers, 32768-token prefix, 128-node tree, target arg-max rigged so that the seeded
    paths accept 0..8 draft tokens; accept length, accepted ids and the compacted rows of all 64 caches bit-exact,
    attention of a sampled layer within the fp16 tolerance;
  * `C.init_base_model -> C.init_minicpm4_eagle_model -> C.init_storage -> C.load_model -> C.decode_attention ->
    C.decode_lm_head -> C.verify_and_fix`, the call sequence of cpmcu/llm.py and cpmcu/speculative/tree_drafter.py
    restricted to the path.
"""
import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu

HQ, HKV, D = 32, 2, 128


def test_c5_wide_tree_step_32_layers_every_depth(gpu, orc):
    from cpm.cu_amd import ops
    from cpm.cu_amd.driver import VerifyStep
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    cfg = synth.CONFIGS["c5_wide_32k"]
    L, P, T = cfg["layers"], cfg["prefix"], cfg["T"]
    V, H = 20000, 1024  # the head at full size has its own tests; the step needs a target arg-max, not 602 MB of weights
    S = P + T
    tree = synth.eagle_tree(cfg["num_iter"], cfg["topk"], T, seed=3)  # a seed whose tree reaches all 8 draft levels
    assert int(tree.depth.max()) == 8
    npages = (S + 255) // 256 + 1
    table = synth.rng(5, 4).permutation(npages).astype(np.int32)
    cache = PagedKVCache(L, HKV, npages, block_table=table)
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    for l in range(L):  # ~N(0,1) prefix, generated on the device in the pools' own layout
        cache.k[l].normal_(generator=g)
        cache.v[l].normal_(generator=g)
    rn = lambda *s, std=1.0: (torch.randn(*s, device="cuda", generator=g) * std).to(torch.float16)
    q = [rn(T, HQ, D) for _ in range(L)]
    k_new = [rn(T, HKV, D) for _ in range(L)]
    v_new = [rn(T, HKV, D) for _ in range(L)]
    hidden = rn(T, H)
    w = rn(V, H, std=0.02)
    w_t = ops.tile_head_weight(w)
    mask, parent, pos = to_dev(torch, tree.mask), to_dev(torch, tree.parent), to_dev(torch, tree.positions(P))
    attn_out = [torch.empty(T, HQ, D, dtype=torch.float16, device="cuda") for _ in range(L)]
    # what the step must leave alone: the prefix rows of every cache (checked through logical reads of a few
    # layers in full and of every layer's last prefix page)
    sampled = (0, 17, 31)
    before = {l: cache.read_logical(l, 0, P) for l in sampled}
    tail0 = P - 256
    before_tail = [cache.read_logical(l, tail0, 256) for l in range(L)]

    vs = VerifyStep(cache, w_t, mask, parent, pos, P)
    gt = to_np(ops.lm_head_argmax(hidden, w_t))
    assert np.array_equal(gt, orc.argmax(to_np(ops.lm_head_argmax(hidden, w_t, want_logits=True)[1])))
    k_new_np = [to_np(t).reshape(T, -1) for t in k_new]
    v_new_np = [to_np(t).reshape(T, -1) for t in v_new]
    for depth in range(9):
        pred, leaf = synth.draft_ids_for_accept(tree, gt, depth, V, 100 + depth)
        vs.enqueue(q, k_new, v_new, hidden, to_dev(torch, pred), attn_out=attn_out)
        a, ids = vs.result()
        a_ref, node_ref, path = orc.tree_accept(pred, gt, tree.positions(P), P, tree.mask, tree.parent)
        assert a == a_ref == depth + 1 and list(path) == tree.path_to(leaf)
        assert int(vs.best[1].item()) == node_ref
        assert np.array_equal(to_np(vs.gt), gt)
        # the oracle's compaction of the tree rows (prefix length 0 on the T appended rows of each cache)
        flat = []
        for l in range(L):
            flat += [k_new_np[l].copy(), v_new_np[l].copy()]
        ids_ref = orc.kv_compact(flat, 0, path, gt)
        assert np.array_equal(ids, ids_ref) and np.array_equal(ids, gt[path])
        for l in range(L):
            kd, vd = cache.read_logical(l, P, a)
            assert np.array_equal(to_np(kd).reshape(a, -1).view(np.uint16), flat[2 * l][:a].view(np.uint16)), (depth, l)
            assert np.array_equal(to_np(vd).reshape(a, -1).view(np.uint16), flat[2 * l + 1][:a].view(np.uint16)), (depth, l)
        if depth == 0:
            # attention of one sampled layer against the oracle (prefix read back from the pool + the tree rows)
            l = 17
            kp, vp = before[l]
            k_all = np.concatenate([to_np(kp), to_np(k_new[l])])
            v_all = np.concatenate([to_np(vp), to_np(v_new[l])])
            ref = orc.tree_attention(to_np(q[l]), k_all, v_all, tree.mask, P)
            assert_close_f16(to_np(attn_out[l]), ref, "config 5 step, attention of layer %d" % l)
    for l in sampled:
        kd, vd = cache.read_logical(l, 0, P)
        assert torch.equal(kd, before[l][0]) and torch.equal(vd, before[l][1]), "prefix of layer %d changed" % l
    for l in range(L):
        kd, vd = cache.read_logical(l, tail0, 256)
        assert torch.equal(kd, before_tail[l][0]) and torch.equal(vd, before_tail[l][1]), "last prefix page of layer %d changed" % l


def test_pybind_module_drives_the_path_end_to_end(gpu, orc):
    """The reference's own entry-point names, positional signatures and raw-address conventions
    (tensor.data_ptr(); host pointer for load_model), nothing else: what cpmcu/llm.py would call."""
    from cpm.cu_amd import C
    torch = gpu
    V, Vs, H, layers, T, P = 5000, 2048, 512, 2, 60, 333
    keep = []

    def dev(a):
        t = to_dev(torch, a)
        keep.append(t)
        return t.data_ptr()
    C.init_base_model(0.02, V, layers, H, 1024, HQ, HKV, D, 1e-5, 0, 2048, 1.0, 0.25, 1.0)
    C.init_minicpm4_eagle_model(1, 6, 10, T, 0, False, 128, 1024, Vs, 1.0, True, True)
    ctx = C.init_storage()
    assert isinstance(ctx, int) and ctx >= 4096
    w = synth.normal_f16((V, H), 21, 2, std=0.02)
    remap = synth.frspec_remap(V, Vs, 21)
    with pytest.raises(ValueError):
        C.load_model("model.embed_tokens.weight", w.ctypes.data)
    C.load_model("eagle.token_id_remap", remap.ctypes.data)
    C.load_model("lm_head.weight", w.ctypes.data)
    tree = synth.eagle_tree(6, 10, T, seed=4)
    S = P + T
    cl = torch.tensor([0], dtype=torch.int32, device="cuda")
    dummy = torch.empty((64, HQ, D), dtype=torch.float16, device="cuda")
    flat = []
    for layer in range(layers):
        k = synth.normal_f16((S, HKV, D), 22, 10 + layer)
        v = synth.normal_f16((S, HKV, D), 22, 50 + layer)
        q = synth.normal_f16((T, HQ, D), 22, 90 + layer)
        done = 0
        while done < P:  # the prefix goes in as causal chunks of <= 64 rows
            n = min(64, P - done)
            cl.fill_(done + n)
            C.decode_attention(layer, n, done + n, dev(np.repeat(q[:1], n, 0)), dev(k[done:done + n]), dev(v[done:done + n]),
                               cl.data_ptr(), 0, dummy.data_ptr())
            C.synchronize()
            done += n
        cl.fill_(S)
        out = torch.empty((T, HQ, D), dtype=torch.float16, device="cuda")
        C.decode_attention(layer, T, (S + 127) // 128 * 128, dev(q), dev(k[P:]), dev(v[P:]), cl.data_ptr(), dev(tree.mask), out.data_ptr())
        C.synchronize()
        assert_close_f16(to_np(out), orc.tree_attention(q, k, v, tree.mask, P), "C.decode_attention layer %d" % layer)
        flat += [k.reshape(S, -1).copy(), v.reshape(S, -1).copy()]
    hid = synth.normal_f16((T, H), 22, 200)
    logits = torch.empty((64, V), dtype=torch.float16, device="cuda")
    gt = torch.empty(T, dtype=torch.int32, device="cuda")
    C.decode_lm_head(T, dev(hid), logits.data_ptr(), gt.data_ptr())
    C.synchronize()
    assert_close_f16(to_np(logits[:T]), orc.lm_head(hid, w, head_scale=0.25), "C.decode_lm_head")
    gt_np = to_np(gt)
    assert np.array_equal(gt_np, orc.argmax(to_np(logits[:T])))
    # the draft head on the loaded FR-Spec sub-matrix
    val = torch.empty((10, 10), dtype=torch.float16, device="cuda")
    pos = torch.empty((10, 10), dtype=torch.int32, device="cuda")
    ids = torch.empty((10, 10), dtype=torch.int32, device="cuda")
    C.draft_head(10, dev(hid[:10]), val.data_ptr(), pos.data_ptr(), ids.data_ptr())
    C.synchronize()
    assert np.array_equal(to_np(ids), remap[to_np(pos)])
    # verify_and_fix returns the accept length; pred[:a] becomes the accepted ids; every cache is compacted
    pred, leaf = synth.draft_ids_for_accept(tree, gt_np, 4, V, 6)
    d_pred = to_dev(torch, pred)
    cl.fill_(P)
    a = C.verify_and_fix(T, d_pred.data_ptr(), gt.data_ptr(), dev(tree.positions(P)), cl.data_ptr(), dev(tree.mask), dev(tree.parent))
    a_ref, _, path = orc.tree_accept(pred, gt_np, tree.positions(P), P, tree.mask, tree.parent)
    ids_ref = orc.kv_compact(flat, P, path, gt_np)
    assert a == a_ref == 5
    assert np.array_equal(to_np(d_pred)[:a], ids_ref)
    # the compacted caches as the next decode step sees them
    S2 = P + a + 1
    one = synth.chain_tree(1)
    for layer in range(layers):
        kn = synth.normal_f16((1, HKV, D), 23, 10 + layer)
        vn = synth.normal_f16((1, HKV, D), 23, 50 + layer)
        qn = synth.normal_f16((1, HQ, D), 23, 90 + layer)
        cl.fill_(S2)
        out = torch.empty((1, HQ, D), dtype=torch.float16, device="cuda")
        C.decode_attention(layer, 1, (S2 + 127) // 128 * 128, dev(qn), dev(kn), dev(vn), cl.data_ptr(), 0, out.data_ptr())
        C.synchronize()
        k_flat = np.concatenate([flat[2 * layer][: P + a].reshape(-1, HKV, D), kn])
        v_flat = np.concatenate([flat[2 * layer + 1][: P + a].reshape(-1, HKV, D), vn])
        assert_close_f16(to_np(out), orc.tree_attention(qn, k_flat, v_flat, one.mask, P + a), "C: decode after compaction, layer %d" % layer)
    with pytest.raises(RuntimeError, match="outside the verify/draft path"):
        C.decode(T, 128, 0, 0, 0, 0, 0, False)
    C.shutdown()


def _graph_replays_equal_eager_steps(torch, orc, seed, T, P0, STEPS, LAYERS=3, V=3000, H=512, num_iter=6, topk=4, min_paddings=2):
    """cpmcu_verify_step on the library's own storage: the same sequence of steps enqueued eagerly and as replays of
    the library's HIP graphs (one per padded length, lengths and positions advancing on the device) must give the same
    accept lengths, ids, gathered hidden rows and caches, and both must match the oracle's acceptance on the device's
    own arg-max.  The second model instance reuses the process-global model after a shutdown."""
    from cpm.cu_amd import ops
    from cpm.cu_amd.model import PathModel
    tree = synth.random_tree(T, seed, max_children=3, max_depth=6)
    mask, parent = to_dev(torch, tree.mask), to_dev(torch, tree.parent)
    w = synth.normal_f16((V, H), seed, 2, std=0.02)
    w_dev = ops.tile_head_weight(to_dev(torch, w))
    rg = synth.rng(seed, 8)
    inputs = []
    for s in range(STEPS):
        x = dict(q=[to_dev(torch, synth.normal_f16((T, HQ, D), seed, 1000 + 10 * s + l)) for l in range(LAYERS)],
                 k=[to_dev(torch, synth.normal_f16((T, HKV, D), seed, 2000 + 10 * s + l)) for l in range(LAYERS)],
                 v=[to_dev(torch, synth.normal_f16((T, HKV, D), seed, 3000 + 10 * s + l)) for l in range(LAYERS)],
                 hidden=to_dev(torch, synth.normal_f16((T, H), seed, 4000 + s)))
        x["gt"] = to_np(ops.lm_head_argmax(x["hidden"], w_dev, head_scale=0.5))
        x["depth"] = int(rg.integers(0, int(tree.depth.max()) + 1))
        pred, leaf = synth.draft_ids_for_accept(tree, x["gt"], x["depth"], V, 300 + s)
        x["pred"], x["path"] = to_dev(torch, pred), tree.path_to(leaf)
        x["pred_np"] = pred
        inputs.append(x)
    del w_dev

    def run(graph):
        m = PathModel(V, LAYERS, H, HQ, HKV, memory_limit=0.01, scale_lmhead=0.5, tree_size=T, num_iter=num_iter, topk=topk)
        try:
            m.load_head(w)
            cache = m.cache()
            for layer in range(LAYERS):
                cache.write_logical(layer, 0, to_dev(torch, synth.normal_f16((P0, HKV, D), seed, 10 + layer)),
                                    to_dev(torch, synth.normal_f16((P0, HKV, D), seed, 50 + layer)))
            f16 = dict(dtype=torch.float16, device="cuda")
            bq = [torch.zeros((T, HQ, D), **f16) for _ in range(LAYERS)]
            bk = [torch.zeros((T, HKV, D), **f16) for _ in range(LAYERS)]
            bv = [torch.zeros((T, HKV, D), **f16) for _ in range(LAYERS)]
            bo = [torch.zeros((T, HQ, D), **f16) for _ in range(LAYERS)]
            bh, prev = torch.zeros((T, H), **f16), torch.zeros((T, H), **f16)
            bd = torch.zeros(T, dtype=torch.int32, device="cuda")
            pos = to_dev(torch, tree.positions(P0))
            clen = torch.tensor([P0], dtype=torch.int32, device="cuda")
            kvlen = torch.tensor([P0 + T], dtype=torch.int32, device="cuda")
            ids = torch.zeros(T, dtype=torch.int32, device="cuda")
            gt_out = torch.zeros(T, dtype=torch.int32, device="cuda")
            result = torch.zeros(1 + T, dtype=torch.int32).pin_memory()
            P, hist, paddings = P0, [], set()
            for x in inputs:
                for l in range(LAYERS):
                    bq[l].copy_(x["q"][l]); bk[l].copy_(x["k"][l]); bv[l].copy_(x["v"][l])
                bh.copy_(x["hidden"]); bd.copy_(x["pred"])
                torch.cuda.synchronize()  # the library's stream is not torch's
                padded = (P + T + 31) // 32 * 32
                paddings.add(padded)
                m.verify_step(T, padded, bq, bk, bv, bo, bh, bd, pos, clen, kvlen, mask, parent, ids, gt_out=gt_out, prev_hidden=prev,
                              result=result, advance_length=True, cuda_graph=graph)
                m.synchronize()
                a = int(result[0])
                a_ref, _, path = orc.tree_accept(x["pred_np"], x["gt"], tree.positions(P), P, tree.mask, tree.parent)
                assert a == a_ref == x["depth"] + 1 and list(path) == x["path"]
                assert np.array_equal(to_np(gt_out), x["gt"]) and np.array_equal(result[1:1 + a].numpy(), x["gt"][path])
                assert np.array_equal(to_np(ids)[:a], x["gt"][path])
                assert np.array_equal(to_np(prev)[:a].view(np.uint16), to_np(x["hidden"])[path].view(np.uint16))
                assert np.array_equal(to_np(bd), x["pred_np"]), "the draft ids are read only"
                P += a
                assert int(to_np(clen)[0]) == P and int(to_np(kvlen)[0]) == P + T and np.array_equal(to_np(pos), tree.positions(P))
                hist.append((a, result[1:1 + a].numpy().tolist(), to_np(bo[LAYERS - 1]).copy()))
            kv = [tuple(to_np(t) for t in cache.read_logical(layer, 0, P)) for layer in range(LAYERS)]
            return hist, kv, P, len(paddings)
        finally:
            m.close()

    hist_e, kv_e, P_e, _ = run(False)
    hist_g, kv_g, P_g, npad = run(True)
    assert P_e == P_g and npad >= min_paddings, "the run should cross a padded length (%d seen)" % npad
    for (a1, i1, o1), (a2, i2, o2) in zip(hist_e, hist_g):
        assert (a1, i1) == (a2, i2)
        assert np.array_equal(o1.view(np.uint16), o2.view(np.uint16))  # same launches, same split geometry: same bits
    for (k1, v1), (k2, v2) in zip(kv_e, kv_g):
        assert np.array_equal(k1.view(np.uint16), k2.view(np.uint16)) and np.array_equal(v1.view(np.uint16), v2.view(np.uint16))


def test_library_graph_replays_equal_eager_steps(gpu, orc):
    _graph_replays_equal_eager_steps(gpu, orc, seed=3, T=24, P0=1000, STEPS=10)


@pytest.mark.parametrize("T", [65, 100, 128])
def test_model_level_steps_with_trees_of_more_than_64_nodes(gpu, orc, T):
    """cpmcu_verify_step takes trees of up to 128 nodes, masks of two words per row: the same sequence of steps, eagerly and
    as graph replays, against the oracle."""
    _graph_replays_equal_eager_steps(gpu, orc, seed=T, T=T, P0=900, STEPS=6, LAYERS=2, min_paddings=1)


@pytest.mark.parametrize("hq,hkv", [(32, 8), (8, 1), (40, 8)])
def test_model_level_steps_with_other_head_counts(gpu, orc, monkeypatch, hq, hkv):
    """The same sequence of steps on models with 4, 8 and 5 query heads per KV head (the configurations all have 16)."""
    import sys
    me = sys.modules[__name__]
    monkeypatch.setattr(me, "HQ", hq)
    monkeypatch.setattr(me, "HKV", hkv)
    _graph_replays_equal_eager_steps(gpu, orc, seed=hq, T=20 + hkv, P0=700, STEPS=6, LAYERS=2, num_iter=8, topk=8, min_paddings=1)


def test_step_graph_cache_is_bounded(gpu, orc):
    """A caller whose buffers are not static makes cpmcu_verify_step capture a graph per set of addresses: the library keeps
    the 16 used most recently and frees the rest.  40 sets of addresses, revisited in a different order, give the results of
    the eager step every time; cpmcu_graph_destroy frees a caller-made graph and its id is handed out again."""
    from cpm.cu_amd.model import PathModel
    torch = gpu
    V, H, LAYERS, T, P = 3000, 512, 1, 12, 300
    tree = synth.random_tree(T, 5, max_children=3, max_depth=4)
    w = synth.normal_f16((V, H), 8, 2, std=0.02)
    m = PathModel(V, LAYERS, H, HQ, HKV, memory_limit=0.005, tree_size=T, num_iter=4, topk=3)
    try:
        m.load_head(w)
        cache = m.cache()
        cache.write_logical(0, 0, to_dev(torch, synth.normal_f16((P, HKV, D), 8, 10)), to_dev(torch, synth.normal_f16((P, HKV, D), 8, 50)))
        f16 = dict(dtype=torch.float16, device="cuda")
        q, kn, vn = [to_dev(torch, synth.normal_f16((T, HQ, D), 8, 3))], [to_dev(torch, synth.normal_f16((T, HKV, D), 8, 4))], \
            [to_dev(torch, synth.normal_f16((T, HKV, D), 8, 5))]
        out = [torch.zeros((T, HQ, D), **f16)]
        hiddens = [to_dev(torch, synth.normal_f16((T, H), 8, 100 + i)) for i in range(40)]
        draft = torch.zeros(T, dtype=torch.int32, device="cuda")
        pos, mask, parent = to_dev(torch, tree.positions(P)), to_dev(torch, tree.mask), to_dev(torch, tree.parent)
        clen = torch.tensor([P], dtype=torch.int32, device="cuda")
        kvlen = torch.tensor([P + T], dtype=torch.int32, device="cuda")
        ids = torch.zeros(T, dtype=torch.int32, device="cuda")
        gt = torch.zeros(T, dtype=torch.int32, device="cuda")
        result = torch.zeros(1 + T, dtype=torch.int32).pin_memory()
        padded = (P + T + 127) // 128 * 128

        def step(i, graph):
            m.verify_step(T, padded, q, kn, vn, out, hiddens[i], draft, pos, clen, kvlen, mask, parent, ids, gt_out=gt, result=result,
                          cuda_graph=graph)
            m.synchronize()
            return int(result[0]), result[1:1 + int(result[0])].numpy().copy(), to_np(gt).copy()
        count = m.L.raw.cpmcu_step_graph_count
        ref = [step(i, False) for i in range(40)]
        assert count() == 0
        for order in (range(40), reversed(range(40)), [3, 3, 17, 3, 39, 0]):
            for i in order:
                a, acc, g = step(i, True)
                assert a == ref[i][0] and np.array_equal(acc, ref[i][1]) and np.array_equal(g, ref[i][2]), i
                assert 1 <= count() <= 16
        assert count() == 16
        # caller-made graphs: destroy frees the slot, the id comes back
        g0 = m.capture(lambda: m.L.decode_lm_head(T, hiddens[0].data_ptr(), 0, gt.data_ptr()))
        g1 = m.capture(lambda: m.L.decode_lm_head(T, hiddens[1].data_ptr(), 0, gt.data_ptr()))
        m.replay(g0)
        m.synchronize()
        assert np.array_equal(to_np(gt), ref[0][2])
        m.L.graph_destroy(g0)
        with pytest.raises(ValueError, match="unknown graph"):
            m.replay(g0)
        g2 = m.capture(lambda: m.L.decode_lm_head(T, hiddens[2].data_ptr(), 0, gt.data_ptr()))
        assert g2 == g0 and g1 != g0
        m.replay(g2)
        m.synchronize()
        assert np.array_equal(to_np(gt), ref[2][2])
    finally:
        m.close()


@pytest.mark.parametrize("frspec", [True, False])
def test_model_level_draft_rounds(gpu, orc, frspec):
    """cpmcu_draft_round / cpmcu_draft_finish (the drafter's state owned by the library, driven through the pybind module)
    against (1) the operator-level chain on an independently built sub-matrix, bit for bit, and (2) the oracle's tree
    bookkeeping fed with the device's per-round top-k, which pins ids, positions, masks and parents of the final tree.
    Once as the FR-Spec drafter of MiniCPM4 (init_minicpm4_eagle_model: a frequency-ranked sub-vocabulary and its id table),
    once as the plain EAGLE drafter (init_eagle_model, src/entry.cu: the head on the whole vocabulary, no id table)."""
    from cpm.cu_amd import C, ops
    torch = gpu
    V, Vs, H, T, K, N, P = 5000, 2048, 512, 60, 10, 6, 777
    w = synth.normal_f16((V, H), 41, 2, std=0.05)
    C.init_base_model(0.01, V, 1, H, 1024, HQ, HKV, D, 1e-5, 0, 2048, 1.0, 1.0, 1.0)
    if frspec:
        remap = synth.frspec_remap(V, Vs, 41)
        C.init_minicpm4_eagle_model(1, N, K, T, 0, False, 128, 1024, Vs, 1.0, True, True)
    else:
        remap = np.arange(V, dtype=np.int32)
        C.init_eagle_model(1, N, K, T, 0)
    C.init_storage()
    if frspec:
        C.load_model("eagle.token_id_remap", remap.ctypes.data)
    C.load_model("lm_head.weight", w.ctypes.data)
    try:
        hid = [to_dev(torch, synth.normal_f16((1 if d == 0 else K, H), 41, 100 + d)) for d in range(N)]
        next_ids = torch.zeros(K, dtype=torch.int32, device="cuda")
        rows = torch.zeros(K, dtype=torch.int32, device="cuda")
        dmask = torch.zeros(K, dtype=torch.int64, device="cuda")
        with pytest.raises(ValueError, match="out of order"):
            C.draft_round(2, hid[2].data_ptr(), next_ids.data_ptr(), rows.data_ptr(), dmask.data_ptr())
        trace = []
        for d in range(N):
            C.draft_round(d, hid[d].data_ptr(), next_ids.data_ptr(), rows.data_ptr() if d else 0, dmask.data_ptr())
            C.synchronize()
            trace.append((to_np(next_ids).copy(), to_np(rows).copy(), to_np(dmask).view(np.uint64).copy()))
            if d == 1:
                with pytest.raises(ValueError, match="rounds have run"):
                    C.draft_finish(1, 1, 1, 1, 1)
        ids = torch.full((T,), -1, dtype=torch.int32, device="cuda")
        ids[0] = 4321  # the root token is the caller's
        tpos = torch.zeros(T, dtype=torch.int32, device="cuda")
        tmask = torch.zeros(T, dtype=torch.int64, device="cuda")
        tpar = torch.zeros(T, dtype=torch.int32, device="cuda")
        cl = torch.tensor([P], dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        C.draft_finish(ids.data_ptr(), tpos.data_ptr(), cl.data_ptr(), tmask.data_ptr(), tpar.data_ptr())
        C.synchronize()
    finally:
        C.shutdown()
    # (1) the operator-level chain
    d_remap = to_dev(torch, remap)
    sub = ops.tile_head_weight(to_dev(torch, w), d_remap)
    t = ops.DraftTree(K, N, d_remap)
    o_tree = orc.DraftTree(K, N, remap)
    for d in range(N):
        r = ops.frspec_head_topk(hid[d], sub, d_remap, K)
        torch.cuda.synchronize()
        val_np, pos_np = to_np(r["val"]).copy(), to_np(r["pos"]).copy()
        if d == 0:
            got = to_np(t.begin(r["val"][0], r["pos"][0])).copy()
            assert np.array_equal(trace[0][0], got)
            assert np.array_equal(got, o_tree.begin(val_np[0], pos_np[0]))
        else:
            g_ids, g_rows, g_mask = t.extend(d, r["val"], r["pos"])
            torch.cuda.synchronize()
            assert np.array_equal(trace[d][0], to_np(g_ids)) and np.array_equal(trace[d][1], to_np(g_rows))
            assert np.array_equal(trace[d][2], to_np(g_mask).view(np.uint64))
            o_ids, o_rows, _ = o_tree.extend(d, val_np, pos_np)  # (2) the oracle on the device's top-k of the round
            assert np.array_equal(trace[d][0], o_ids) and np.array_equal(trace[d][1], o_rows) and np.array_equal(trace[d][2], o_tree.mask)
    o_ids, o_pos, o_mask, o_par = o_tree.finish(T, P)
    assert int(to_np(ids)[0]) == 4321 and np.array_equal(to_np(ids)[1:], o_ids[1:])
    assert np.array_equal(to_np(tpos), o_pos) and np.array_equal(to_np(tpar), o_par)
    assert np.array_equal(to_np(tmask).view(np.uint64), o_mask[:, 0])


@pytest.mark.parametrize("config", ["c2_verify_4k", "c5_wide_32k"])
def test_full_size_step_on_the_library_graph(gpu, orc, config):
    """Config 2 as the benchmark runs it: 32 layers, 4096-token prefix, 60-node tree, the 73448 x 4096 head, one
    cpmcu_verify_step on the library's storage replayed from the library's graph.  Accept length, ids and the compacted
    rows of all 64 caches bit-exact against the oracle, the arg-max staged on the oracle's logits of the same head,
    attention of two sampled layers within the fp16 tolerance.  And config 5 the same way: a 128-node tree (two mask words
    per row, beyond the reference's 64 nodes) behind a 32768-token prefix."""
    from cpm.cu_amd.model import PathModel
    torch = gpu
    cfg, shp = synth.CONFIGS[config], synth.MINICPM4_8B
    L, P, T, V, H = cfg["layers"], cfg["prefix"], cfg["T"], shp["vocab"], shp["hidden"]
    S = P + T
    tree = synth.eagle_tree(cfg["num_iter"], cfg["topk"], T, cfg["seed"])
    g = torch.Generator(device="cuda")
    g.manual_seed(2)
    w = (torch.randn(V, H, device="cuda", generator=g) * 0.02).to(torch.float16).cpu().numpy()
    npages = (S + 255) // 256 + 1
    m = PathModel(V, L, H, HQ, HKV, memory_limit=0.02, tree_size=T, num_iter=cfg["num_iter"], topk=cfg["topk"])
    try:
        m.load_head(w)
        table = to_dev(torch, synth.rng(0, 4).permutation(npages).astype(np.int32))
        cache = m.cache(block_table=table)
        for l in range(L):
            m._k[l][:npages].normal_(generator=g)
            m._v[l][:npages].normal_(generator=g)
        rn = lambda *s: torch.randn(*s, device="cuda", generator=g).to(torch.float16)
        q, kn, vn = [rn(T, HQ, D) for _ in range(L)], [rn(T, HKV, D) for _ in range(L)], [rn(T, HKV, D) for _ in range(L)]
        out = [torch.zeros(T, HQ, D, dtype=torch.float16, device="cuda") for _ in range(L)]
        hidden = rn(T, H)
        sampled = (3, 30)
        before = {l: tuple(to_np(t) for t in cache.read_logical(l, 0, P)) for l in sampled}
        draft = torch.zeros(T, dtype=torch.int32, device="cuda")
        gt = torch.zeros(T, dtype=torch.int32, device="cuda")
        ids = torch.zeros(T, dtype=torch.int32, device="cuda")
        result = torch.zeros(1 + T, dtype=torch.int32).pin_memory()
        clen = torch.tensor([P], dtype=torch.int32, device="cuda")
        kvlen = torch.tensor([S], dtype=torch.int32, device="cuda")
        pos, mask, parent = to_dev(torch, tree.positions(P)), to_dev(torch, tree.mask), to_dev(torch, tree.parent)
        padded = (S + 127) // 128 * 128
        torch.cuda.synchronize()
        step = lambda: m.verify_step(T, padded, q, kn, vn, out, hidden, draft, pos, clen, kvlen, mask, parent, ids, gt_out=gt,
                                     result=result, block_table=table, cuda_graph=True)
        step()  # captures; the target arg-max of this pass rigs the draft ids
        m.synchronize()
        gt_np = to_np(gt)
        z_ref = orc.lm_head(to_np(hidden), w)
        gt_ref = orc.argmax(z_ref)
        for i in np.nonzero(gt_np != gt_ref)[0]:  # only inside the logit tolerance
            assert float(z_ref[i, gt_ref[i]]) - float(z_ref[i, gt_np[i]]) <= 4e-2
        for depth in (0, 3, int(tree.depth.max())):
            pred, leaf = synth.draft_ids_for_accept(tree, gt_np, depth, V, 7 + depth)
            draft.copy_(to_dev(torch, pred))
            torch.cuda.synchronize()
            step()  # a replay
            m.synchronize()
            a = int(result[0])
            a_ref, _, path = orc.tree_accept(pred, gt_np, tree.positions(P), P, tree.mask, tree.parent)
            assert a == a_ref == depth + 1 and np.array_equal(result[1:1 + a].numpy(), gt_np[path])
            for l in range(L):
                kd, vd = cache.read_logical(l, P, a)
                assert np.array_equal(to_np(kd).reshape(a, -1).view(np.uint16), to_np(kn[l]).reshape(T, -1)[path].view(np.uint16)), (depth, l)
                assert np.array_equal(to_np(vd).reshape(a, -1).view(np.uint16), to_np(vn[l]).reshape(T, -1)[path].view(np.uint16)), (depth, l)
        for l in sampled:
            kp, vp = before[l]
            ref = orc.tree_attention(to_np(q[l]), np.concatenate([kp, to_np(kn[l])]), np.concatenate([vp, to_np(vn[l])]), tree.mask, P)
            assert_close_f16(to_np(out[l]), ref, "%s step on the library graph, attention of layer %d" % (config, l))
            kd, vd = cache.read_logical(l, 0, P)
            assert np.array_equal(to_np(kd).view(np.uint16), kp.view(np.uint16)) and np.array_equal(to_np(vd).view(np.uint16), vp.view(np.uint16))
    finally:
        m.close()


def test_128k_step_integer_parity_on_the_library_graph(gpu, orc):
    """The longest context of the benchmark as a verify step whose results are checked: 3 layers, a 131072-token
    prefix behind a permuted page table (the tree rows land in logical pages 512-513), 60-node tree, cpmcu_verify_step
    replayed from the library's graph.  Accept length, ids and the compacted rows of every cache bit-exact against the
    oracle at three accept depths; the attention of one layer against the oracle's pass over all 131132 keys; the
    last prefix page of every cache untouched.  The head is reduced (the full-size heads have their own tests)."""
    from cpm.cu_amd.model import PathModel
    torch = gpu
    L, P, T, V, H = 3, 131072, 60, 20000, 1024
    S = P + T
    tree = synth.eagle_tree(6, 10, T, seed=11)
    g = torch.Generator(device="cuda")
    g.manual_seed(128)
    w = (torch.randn(V, H, device="cuda", generator=g) * 0.02).to(torch.float16).cpu().numpy()
    npages = (S + 255) // 256 + 1
    m = PathModel(V, L, H, HQ, HKV, memory_limit=0.01, tree_size=T, num_iter=6, topk=10)
    try:
        assert m.max_context >= S
        m.load_head(w)
        table = to_dev(torch, synth.rng(128, 4).permutation(npages).astype(np.int32))
        cache = m.cache(block_table=table)
        for l in range(L):
            m._k[l][:npages].normal_(generator=g)
            m._v[l][:npages].normal_(generator=g)
        rn = lambda *s: torch.randn(*s, device="cuda", generator=g).to(torch.float16)
        q, kn, vn = [rn(T, HQ, D) for _ in range(L)], [rn(T, HKV, D) for _ in range(L)], [rn(T, HKV, D) for _ in range(L)]
        out = [torch.zeros(T, HQ, D, dtype=torch.float16, device="cuda") for _ in range(L)]
        hidden = rn(T, H)
        tail0 = P - 256
        before_tail = [cache.read_logical(l, tail0, 256) for l in range(L)]
        kp, vp = (to_np(t) for t in cache.read_logical(1, 0, P))
        draft = torch.zeros(T, dtype=torch.int32, device="cuda")
        gt = torch.zeros(T, dtype=torch.int32, device="cuda")
        ids = torch.zeros(T, dtype=torch.int32, device="cuda")
        result = torch.zeros(1 + T, dtype=torch.int32).pin_memory()
        clen = torch.tensor([P], dtype=torch.int32, device="cuda")
        kvlen = torch.tensor([S], dtype=torch.int32, device="cuda")
        pos, mask, parent = to_dev(torch, tree.positions(P)), to_dev(torch, tree.mask), to_dev(torch, tree.parent)
        padded = (S + 127) // 128 * 128
        torch.cuda.synchronize()
        step = lambda: m.verify_step(T, padded, q, kn, vn, out, hidden, draft, pos, clen, kvlen, mask, parent, ids, gt_out=gt,
                                     result=result, block_table=table, cuda_graph=True)
        step()  # captures; the target arg-max of this pass rigs the draft ids
        m.synchronize()
        gt_np = to_np(gt)
        z_ref = orc.lm_head(to_np(hidden), w)
        gt_ref = orc.argmax(z_ref)
        for i in np.nonzero(gt_np != gt_ref)[0]:  # only inside the logit tolerance
            assert float(z_ref[i, gt_ref[i]]) - float(z_ref[i, gt_np[i]]) <= 4e-2
        for depth in (0, 2, int(tree.depth.max())):
            pred, leaf = synth.draft_ids_for_accept(tree, gt_np, depth, V, 70 + depth)
            draft.copy_(to_dev(torch, pred))
            torch.cuda.synchronize()
            step()  # a replay
            m.synchronize()
            a = int(result[0])
            a_ref, _, path = orc.tree_accept(pred, gt_np, tree.positions(P), P, tree.mask, tree.parent)
            assert a == a_ref == depth + 1 and list(path) == tree.path_to(leaf)
            flat = []
            for l in range(L):
                flat += [to_np(kn[l]).reshape(T, -1).copy(), to_np(vn[l]).reshape(T, -1).copy()]
            ids_ref = orc.kv_compact(flat, 0, path, gt_np)
            assert np.array_equal(result[1:1 + a].numpy(), ids_ref) and np.array_equal(to_np(ids)[:a], ids_ref)
            for l in range(L):
                kd, vd = cache.read_logical(l, P, a)
                assert np.array_equal(to_np(kd).reshape(a, -1).view(np.uint16), flat[2 * l][:a].view(np.uint16)), (depth, l)
                assert np.array_equal(to_np(vd).reshape(a, -1).view(np.uint16), flat[2 * l + 1][:a].view(np.uint16)), (depth, l)
        ref = orc.tree_attention(to_np(q[1]), np.concatenate([kp, to_np(kn[1])]), np.concatenate([vp, to_np(vn[1])]), tree.mask, P)
        assert_close_f16(to_np(out[1]), ref, "128K step on the library graph, attention of layer 1")
        for l in range(L):
            kd, vd = cache.read_logical(l, tail0, 256)
            assert torch.equal(kd, before_tail[l][0]) and torch.equal(vd, before_tail[l][1]), "last prefix page of layer %d changed" % l
    finally:
        m.close()


def test_device_side_length_outside_the_promised_bound_is_reported(gpu):
    """A KV length read from device memory that exceeds the call's max_kv_len (a stale padded length under a replayed
    graph, say) must not walk off the page table: the launch clamps it, and the next synchronising call says so."""
    from cpm.cu_amd import lib as libmod, ops
    from cpm.cu_amd.kvcache import PagedKVCache
    torch = gpu
    L = libmod.get()
    T, P = 8, 300
    cache = PagedKVCache(1, HKV, 3)
    q = torch.randn(T, HQ, D, device="cuda").to(torch.float16)
    L.synchronize()  # clears anything an earlier test left
    kv_len = torch.tensor([P + T + 200], dtype=torch.int32, device="cuda")  # beyond the max_kv_len promised below
    out = ops.tree_attention(q, cache, 0, kv_len, P + T, None)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    with pytest.raises(RuntimeError, match="KV length of 508"):
        L.synchronize()
    L.synchronize()  # reported once
    kv_len.fill_(4)  # shorter than the query rows
    ops.tree_attention(q, cache, 0, kv_len, P + T, None)
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="KV length of 4"):
        L.synchronize()


def test_init_storage_failure_leaves_nothing_behind(gpu):
    """An init_storage that cannot fit its budget fails with an error and frees what it had taken: the retry with a
    workable budget starts clean."""
    from cpm.cu_amd import lib as libmod
    import ctypes
    torch = gpu
    L = libmod.get()
    free0 = torch.cuda.mem_get_info()[0]
    total = torch.cuda.mem_get_info()[1]
    V, H = 40000, 2048
    L.init_base_model(ctypes.c_float(200e6 / total), V, 2, H, 4 * H, HQ, HKV, D, ctypes.c_float(1e-5), 0, 2048, ctypes.c_float(1.0),
                      ctypes.c_float(1.0), ctypes.c_float(1.0))  # 200 MB: the head fits, its staging buffer and the pools do not
    L.init_minicpm4_eagle_model(1, 6, 10, 60, 0, 0, 128, 1024, 0, ctypes.c_float(1.0), 1, 1)
    ctx = ctypes.c_int(0)
    with pytest.raises(RuntimeError, match="budget"):
        L.init_storage(ctypes.byref(ctx))
    free1 = torch.cuda.mem_get_info()[0]
    assert free0 - free1 < 64 << 20, "a failed init_storage kept %d MB" % ((free0 - free1) >> 20)
    L.shutdown()
    L.init_base_model(ctypes.c_float(2e9 / total), V, 2, H, 4 * H, HQ, HKV, D, ctypes.c_float(1e-5), 0, 2048, ctypes.c_float(1.0),
                      ctypes.c_float(1.0), ctypes.c_float(1.0))
    L.init_minicpm4_eagle_model(1, 6, 10, 60, 0, 0, 128, 1024, 0, ctypes.c_float(1.0), 1, 1)
    L.init_storage(ctypes.byref(ctx))
    assert ctx.value >= 4096
    L.shutdown()
