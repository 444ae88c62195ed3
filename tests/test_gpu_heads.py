"""GPU parity of the FR-Spec draft head (+ log-softmax, top-k, id map-back), the target head with
fused arg-max and the stand-alone top-k / log-softmax operators, all through the C-ABI.

Logits are fp16 with fp32 accumulation in a different order than the oracle's, so they are compared
within max-abs 2e-2 / max-rel 1e-2.  Integer results are bit-exact in two ways:
  * staged: the oracle re-ranks the DEVICE's fp16 logits (and row statistics) -- must match always;
  * end to end: the oracle's own logits -- must match whenever the decision margin exceeds the
    logit tolerance; a seed that fails only inside that margin is reported, not hidden.
"""
import numpy as np
import pytest

from cpm.cu_amd import synth
from util import assert_close_f16, to_dev, to_np

pytestmark = pytest.mark.gpu


def _frspec_check(torch, orc, n, V, Vs, H, k, seed, tiled=False):
    """tiled: the sub-matrix is built by tile_head_weight(w, remap) -- gather fused with the re-tiling, the layout
    the model-level loader and the benchmark keep -- instead of gather_rows into a row-major matrix."""
    from cpm.cu_amd import ops
    hid = synth.normal_f16((n, H), seed, 1)
    w = synth.normal_f16((V, H), seed, 2, std=0.02)
    remap = synth.frspec_remap(V, Vs, seed)
    d_w = to_dev(torch, w)
    d_remap = to_dev(torch, remap)
    sub = orc.gather_rows(w, remap)
    assert np.array_equal(sub.view(np.uint16), w[remap].view(np.uint16))
    if tiled:
        d_sub = ops.tile_head_weight(d_w, d_remap)
    else:
        d_sub = ops.gather_rows(d_w, d_remap)  # remap_copy
        assert np.array_equal(to_np(d_sub).view(np.uint16), sub.view(np.uint16))

    r = ops.frspec_head_topk(to_dev(torch, hid), d_sub, d_remap, k)
    torch.cuda.synchronize()
    z_dev = to_np(r["logits"])
    z_ref = orc.lm_head(hid, sub)
    assert_close_f16(z_dev, z_ref, "frspec logits")

    # row statistics vs the oracle's on the oracle's logits
    lp_ref, m_ref, lse_ref = orc.log_softmax(z_ref)
    stats = to_np(r["row_stats"])
    assert np.allclose(stats[:, 0], m_ref, atol=2e-2)
    assert np.allclose(stats[:, 1], lse_ref, atol=2e-2)

    # staged bit-exactness: device logits + device statistics -> oracle ranking
    lp_staged = orc.log_softmax_apply(z_dev, stats[:, 0], stats[:, 1])
    val_s, pos_s = orc.topk(lp_staged, k)
    assert np.array_equal(to_np(r["pos"]), pos_s), "top-k positions differ from the staged oracle"
    assert np.array_equal(to_np(r["val"]).view(np.uint16), val_s.view(np.uint16))
    assert np.array_equal(to_np(r["ids"]), orc.remap(pos_s, remap))
    assert np.array_equal(to_np(r["ids"]), remap[pos_s])

    # end to end against the pure oracle, margin-aware
    val_e, pos_e = orc.topk(lp_ref, k + 1)
    exact = np.array_equal(to_np(r["pos"]), pos_e[:, :k])
    if not exact:
        lpf = lp_ref.astype(np.float32)
        bad_rows = [i for i in range(n) if not np.array_equal(to_np(r["pos"])[i], pos_e[i, :k])]
        for i in bad_rows:
            top = np.take(lpf[i], pos_e[i]).astype(np.float64)
            gaps = -np.diff(top)
            assert gaps.min() <= 2 * 2e-2, "row %d differs from the oracle outside the logit tolerance" % i
    return exact


def test_frspec_small(gpu, orc):
    for seed in range(3):
        _frspec_check(gpu, orc, n=10, V=6000, Vs=4096, H=512, k=10, seed=seed)


def test_frspec_one_row_and_sixteen_rows(gpu, orc):
    _frspec_check(gpu, orc, n=1, V=3000, Vs=2048, H=1024, k=10, seed=5)
    _frspec_check(gpu, orc, n=16, V=5000, Vs=4100, H=512, k=7, seed=6)


def test_frspec_clustered_logits_merge_in_fp16(gpu, orc):
    """Nearly flat logits: z spreads over a few hundredths while log-probabilities sit near -ln(V), where an
    fp16 ulp is 2^-7, so hundreds of distinct z collapse onto each rounded log-probability and the ranking is
    decided by the lowest index among ties.  Both the candidate path of the row kernel (bound lowered by the
    rounding slack) and its many-candidates fallback have to reproduce the oracle's order exactly."""
    from cpm.cu_amd import ops
    torch = gpu
    for (n, Vs, H, k, std, seed) in [(4, 4096, 512, 10, 0.0005, 1), (10, 32768, 512, 10, 0.002, 2), (3, 2048, 1024, 32, 0.0002, 3),
                                     (2, 4096, 512, 5, 0.0, 4)]:
        hid = synth.normal_f16((n, H), seed, 1)
        w = synth.normal_f16((Vs, H), seed, 2, std=std) if std > 0 else np.zeros((Vs, H), np.float16)
        remap = synth.frspec_remap(Vs + 1000, Vs, seed)
        r = ops.frspec_head_topk(to_dev(torch, hid), to_dev(torch, w), to_dev(torch, remap), k)
        torch.cuda.synchronize()
        z_dev = to_np(r["logits"])
        stats = to_np(r["row_stats"])
        lp_staged = orc.log_softmax_apply(z_dev, stats[:, 0], stats[:, 1])
        distinct = len(np.unique(lp_staged[0]))
        val_s, pos_s = orc.topk(lp_staged, k)
        assert np.array_equal(to_np(r["pos"]), pos_s), "Vs=%d std=%g: %d distinct log-probs in row 0" % (Vs, std, distinct)
        assert np.array_equal(to_np(r["val"]).view(np.uint16), val_s.view(np.uint16))
        assert np.array_equal(to_np(r["ids"]), remap[pos_s])
        if std == 0.0:
            assert np.array_equal(pos_s, np.tile(np.arange(k, dtype=np.int32), (n, 1)))  # all equal: lowest indices


def test_frspec_c3_full_size(gpu, orc):
    """Config 3: 10 frontier rows, 73448x4096 head, 32768-row subset, top-10 mapped to full-vocab ids."""
    exact = _frspec_check(gpu, orc, n=10, V=73448, Vs=32768, H=4096, k=10, seed=0)
    print("c3 end-to-end ids bit-exact vs pure oracle:", exact)


@pytest.mark.parametrize("n", [10, 1])
def test_frspec_c3_full_size_tiled_layout(gpu, orc, n):
    """Config 3 through the layout the benchmark and the model-level loader use: the 32768-row sub-matrix gathered
    and tiled in one pass out of the 73448-row head, so the GEMM is the single-pass chunked shape (one 16-row block
    per wave, 8 K chunks of 512 rotated over the workgroups, 256 workgroups).  n = 1 is the first draft round."""
    exact = _frspec_check(gpu, orc, n=n, V=73448, Vs=32768, H=4096, k=10, seed=0, tiled=True)
    print("c3 tiled, n=%d: end-to-end ids bit-exact vs pure oracle: %s" % (n, exact))


def test_frspec_tiled_chunk_rotation_shapes(gpu, orc):
    """The single-pass tiled shape away from config 3: several K chunks with fewer workgroups than chunks' rotation
    period, a vocabulary that leaves the last row block partly filled, 16 rows."""
    _frspec_check(gpu, orc, n=16, V=9000, Vs=4096 + 40, H=2048, k=10, seed=11, tiled=True)
    _frspec_check(gpu, orc, n=7, V=40000, Vs=32768, H=1024, k=32, seed=12, tiled=True)


@pytest.mark.parametrize("n,V,Vs,H,k", [(10, 73448, 32768 + 16 * 300, 1024, 10), (16, 60000, 50000, 512, 10), (3, 73448, 70000, 512, 32),
                                        (12, 50000, 36000, 512, 5), (10, 200000, 180000, 512, 10),
                                        # sub-vocabularies whose rows of logits are not whole 16-byte pieces
                                        (5, 9000, 4099, 512, 10), (3, 40000, 33001, 512, 7), (16, 70000, 65537, 512, 16)])
def test_frspec_streaming_kernel_with_a_shared_last_pass(gpu, orc, n, V, Vs, H, k):
    """Sub-vocabularies that are not a whole number of passes: the streaming GEMM with its statistics epilogue, the
    last pass shared by 4, 1, 4 (behind two full passes) and 8 waves; 180000 rows: twice as many workgroups as CUs."""
    from cpm.cu_amd import ops
    if Vs >= 32768:
        assert "head_gemm_stream_kernel" in ops.head_plan(n, ops.tile_head_weight(to_dev(gpu, np.zeros((Vs, H), np.float16))))[0]
    _frspec_check(gpu, orc, n=n, V=V, Vs=Vs, H=H, k=k, seed=Vs % 97, tiled=True)


def test_frspec_subset_vs_full_head(gpu, orc):
    """If the full-vocab top-k ids all lie in the subset, the mapped subset top-k is the full-vocab top-k."""
    from cpm.cu_amd import ops
    torch = gpu
    n, V, H, k = 4, 8192, 512, 5
    hid = synth.normal_f16((n, H), 9, 1)
    w = synth.normal_f16((V, H), 9, 2, std=0.02)
    d_hid, d_w = to_dev(torch, hid), to_dev(torch, w)
    full = ops.frspec_head_topk(d_hid, d_w, None, k)
    torch.cuda.synchronize()
    full_ids = to_np(full["ids"])
    # subset = the winners plus filler rows, in shuffled order
    rest = np.setdiff1d(np.arange(V), np.unique(full_ids))
    remap = np.concatenate([np.unique(full_ids), rest[:3000]]).astype(np.int32)
    synth.rng(9, 7).shuffle(remap)
    d_remap = to_dev(torch, remap)
    sub = ops.frspec_head_topk(d_hid, ops.gather_rows(d_w, d_remap), d_remap, k)
    torch.cuda.synchronize()
    # Same raw logits for the winners, but log-probs are rounded to fp16 before ranking and ties go to
    # the lower index OF THE MATRIX BEING RANKED, so at the k-th place a subset row may legitimately
    # pick another member of a tie group (and the two normalisers round differently).  What must
    # hold, with one fp16 ulp of a log-prob (|lp| < 32 -> 2^-6) as slack on the raw logits: every id
    # the subset head returns is at least as good as the full head's k-th, and every clear winner of
    # the full head is returned.
    sub_ids = to_np(sub["ids"])
    z_full = to_np(full["logits"]).astype(np.float32)
    ulp = 2.0 ** -6
    for i in range(n):
        kth = z_full[i, full_ids[i]].min()
        assert np.all(z_full[i, sub_ids[i]] >= kth - 2 * ulp)
        clear = set(int(t) for t in full_ids[i] if z_full[i, t] > kth + 2 * ulp)
        assert clear <= set(int(t) for t in sub_ids[i])


def test_frspec_c3_full_size_against_the_full_vocabulary_head(gpu, orc):
    """Config 3 as stated: the 32768-row FR-Spec head (gathered and tiled out of the 73448 x 4096 head, the layout the
    benchmark runs) beside the full-vocabulary head on the same 10 hidden rows.  The subset's raw logits are the full
    head's logits of the remapped rows; log-probabilities are rounded to fp16 (one ulp = 2^-6 below 16 in magnitude)
    before ranking and the two heads normalise differently, so what must hold is: every id the subset returns is a
    member of the subset and ranks, among the subset's members, no lower than the k-th best of them in the full head's
    logits (within that rounding); every clear winner among the subset's members is returned; and a row whose
    full-vocabulary top-k all lie in the subset returns the full head's ids."""
    from cpm.cu_amd import ops
    torch = gpu
    n, V, Vs, H, k = 10, 73448, 32768, 4096, 10
    hid = synth.normal_f16((n, H), 0, 1)
    w = synth.normal_f16((V, H), 0, 2, std=0.02)
    remap = synth.frspec_remap(V, Vs, 0)
    d_hid, d_w, d_remap = to_dev(torch, hid), to_dev(torch, w), to_dev(torch, remap)
    full = ops.frspec_head_topk(d_hid, ops.tile_head_weight(d_w), None, k)
    sub = ops.frspec_head_topk(d_hid, ops.tile_head_weight(d_w, d_remap), d_remap, k)
    torch.cuda.synchronize()
    z_full, z_sub = to_np(full["logits"]), to_np(sub["logits"])
    assert_close_f16(z_full, orc.lm_head(hid, w), "full-vocabulary logits")
    # the two launches walk K in the same chunk order per row block, but in different kernels: logits to an fp16 ulp
    assert_close_f16(z_sub, z_full[:, remap], "subset logits vs the full head's remapped rows", atol=8e-3, rtol=2e-3)
    full_ids, sub_ids = to_np(full["ids"]), to_np(sub["ids"])
    assert np.array_equal(full_ids, to_np(full["pos"]))  # no map: ids are positions
    in_subset = np.zeros(V, bool)
    in_subset[remap] = True
    zf = z_full.astype(np.float32)
    ulp = 2.0 ** -6
    rows_inside = 0
    for i in range(n):
        assert in_subset[sub_ids[i]].all()
        members = np.where(in_subset, zf[i], -np.inf)
        kth = np.sort(members)[-k]
        assert np.all(zf[i, sub_ids[i]] >= kth - 2 * ulp), "row %d: a returned id ranks below the subset's k-th" % i
        clear = set(np.nonzero(members > kth + 2 * ulp)[0].tolist())
        assert clear <= set(sub_ids[i].tolist()), "row %d: a clear winner of the subset is missing" % i
        if in_subset[full_ids[i]].all():
            rows_inside += 1
            gaps = -np.diff(zf[i, full_ids[i]])
            if gaps.min() > 2 * ulp:
                assert np.array_equal(sub_ids[i], full_ids[i]), "row %d" % i
    print("c3: rows whose full-vocabulary top-%d lies inside the subset: %d of %d" % (k, rows_inside, n))
    # a subset that holds every row's full-vocabulary winners returns exactly the full head's ids
    winners = np.unique(full_ids)
    rest = np.setdiff1d(np.arange(V), winners)
    remap2 = np.concatenate([winners, rest[: Vs - len(winners)]]).astype(np.int32)
    synth.rng(0, 9).shuffle(remap2)
    d_remap2 = to_dev(torch, remap2)
    sub2 = ops.frspec_head_topk(d_hid, ops.tile_head_weight(d_w, d_remap2), d_remap2, k)
    torch.cuda.synchronize()
    sub2_ids = to_np(sub2["ids"])
    for i in range(n):
        kth = zf[i, full_ids[i]].min()
        assert np.all(zf[i, sub2_ids[i]] >= kth - 2 * ulp)
        clear = set(int(t) for t in full_ids[i] if zf[i, t] > kth + 2 * ulp)
        assert clear <= set(int(t) for t in sub2_ids[i])


def _argmax_check(torch, orc, n, V, H, seed, scale=None, plant=None, tiled=False):
    from cpm.cu_amd import ops
    hid = synth.normal_f16((n, H), seed, 1)
    w = synth.normal_f16((V, H), seed, 2, std=0.02)
    if plant is not None:
        plant(hid, w)
    d_w = ops.tile_head_weight(to_dev(torch, w)) if tiled else to_dev(torch, w)
    gt, logits = ops.lm_head_argmax(to_dev(torch, hid), d_w, head_scale=scale, want_logits=True)
    gt2 = ops.lm_head_argmax(to_dev(torch, hid), d_w, head_scale=scale)  # logits not materialised
    torch.cuda.synchronize()
    z_dev = to_np(logits)
    z_ref = orc.lm_head(hid, w, head_scale=scale)
    assert_close_f16(z_dev, z_ref, "target logits")
    assert np.array_equal(to_np(gt), to_np(gt2))
    # staged: arg-max of the device logits, lowest index on ties
    assert np.array_equal(to_np(gt), orc.argmax(z_dev))
    assert np.array_equal(orc.argmax(z_dev), np.argmax(z_dev.astype(np.float32), axis=1))
    # end to end, margin-aware
    gt_ref = orc.argmax(z_ref)
    for i in np.nonzero(to_np(gt) != gt_ref)[0]:
        zr = z_ref[i].astype(np.float32)
        assert zr[gt_ref[i]] - zr[to_np(gt)[i]] <= 2 * 2e-2, "row %d arg-max differs outside the logit tolerance" % i
    return to_np(gt), z_dev


@pytest.mark.parametrize("n", [1, 16, 17, 32, 60, 64, 100, 128])
def test_target_head_row_counts(gpu, orc, n):
    _argmax_check(gpu, orc, n, V=3001, H=512, seed=n)


@pytest.mark.parametrize("n,H", [(30, 4096), (128, 1024), (60, 2048), (16, 4096)])
def test_target_head_k_chunking(gpu, orc, n, H):
    """Hidden sizes that need several K chunks in LDS (double-buffered staging) for each row-block count."""
    _argmax_check(gpu, orc, n, V=1000, H=H, seed=100 + n)


def _head_sweep_configs():
    """Seeded random (rows, vocabulary, hidden, tiled, scale): row counts around the 16/32/64 thresholds of the
    kernel shapes, vocabularies around multiples of 16 (row blocks) and of 2048 * 16 (full passes of 256 x 8 waves)."""
    g = synth.rng(77, 3)
    rows = [1, 2, 15, 16, 17, 31, 32, 33, 59, 60, 63, 64, 65, 128]
    out = []
    for i in range(24):
        n = int(rows[g.integers(len(rows))])
        base = int([16, 2048 * 16, 2 * 2048 * 16, 4096, 12000][g.integers(5)])
        V = max(n, 1, base + int(g.integers(-20, 21))) if g.random() < 0.7 else int(g.integers(1, 40000))
        H = int([512, 1024, 2048, 4096][g.integers(4)])
        if V * H > 40000 * 2048:
            H = 512
        out.append((n, V, H, bool(g.integers(2)), [None, None, 0.3125, 2.0][int(g.integers(4))], i))
    return out


@pytest.mark.parametrize("n,V,H,tiled,scale,seed", _head_sweep_configs())
def test_target_head_randomised_sweep(gpu, orc, n, V, H, tiled, scale, seed):
    _argmax_check(gpu, orc, n, V=V, H=H, seed=900 + seed, scale=scale, tiled=tiled)


def test_target_head_scale(gpu, orc):
    _argmax_check(gpu, orc, 20, V=2048, H=1024, seed=3, scale=0.3125)


def test_target_head_planted_ties(gpu, orc):
    """Two identical weight rows give bit-identical logits: the lower index must win."""
    def plant(hid, w):
        w[1500] = w[700] = (hid[0].astype(np.float32) * 0.05).astype(np.float16)
        w[2999] = w[2998] = (hid[1].astype(np.float32) * 0.05).astype(np.float16)
    gt, z = _argmax_check(gpu, orc, 4, V=3000, H=512, seed=4, plant=plant)
    assert gt[0] == 700 and gt[1] == 2998


@pytest.mark.parametrize("tiled", [False, True])
def test_target_head_c1_full_size(gpu, orc, tiled):
    """Config 1 head: 16 tree rows against the 73448x4096 head, in both weight layouts."""
    _argmax_check(gpu, orc, 16, V=73448, H=4096, seed=1, tiled=tiled)


@pytest.mark.parametrize("n", [1, 10, 16])
@pytest.mark.parametrize("H", [6144, 8192])
def test_row_major_head_with_many_k_chunks(gpu, orc, n, H):
    """Up to 16 rows against a row-major matrix whose K range needs more than two LDS buffers: the row-walking
    kernel in its chunked form.  Arg-max and the FR-Spec statistics come from per-workgroup partials, whose row
    stride has to be the launched kernel's."""
    _argmax_check(gpu, orc, n, V=2100, H=H, seed=40 + n)
    _frspec_check(gpu, orc, n=n, V=2600, Vs=2048 + 24, H=H, k=10, seed=50 + n)


def test_target_head_c2_full_size(gpu, orc):
    """Config 2 head: 60 tree rows against the 73448x4096 head."""
    _argmax_check(gpu, orc, 60, V=73448, H=4096, seed=0)


def test_target_head_c5_full_size(gpu, orc):
    """Config 5 head: 128 tree rows against the 73448x4096 head in the tiled layout -- the 8-row-block streaming
    kernel at its real K depth (32 chunks of 128 columns, two full passes and a shared last pass)."""
    from cpm.cu_amd import ops
    wt = ops.tile_head_weight(to_dev(gpu, np.zeros((73448, 4096), np.float16)))
    assert "head_gemm_stream_kernel<8,2,128>" in ops.head_plan(128, wt)[0].replace(" ", "")
    del wt
    _argmax_check(gpu, orc, 128, V=73448, H=4096, seed=5, tiled=True)


@pytest.mark.parametrize("n,dim,top", [(1, 100, 10), (1, 510, 59), (10, 32768, 10), (3, 5000, 32), (2, 2048, 1),
                                        (2, 2049, 128), (4, 73448, 10), (1, 7, 7),
                                        # the row kernel's bounds: no bound (up to 1024 elements, also k = the whole row), k shared by
                                        # 2, 3, 4, 8 and 16 full waves, every lane of two waves needed, slices with k beyond 64
                                        (1, 64, 10), (3, 64, 64), (2, 1000, 128), (2, 1024, 17), (1, 1032, 128), (2, 1032, 100),
                                        (2, 1536, 128), (2, 2048, 128), (3, 4096, 64), (2, 4096, 17), (3, 32768, 64), (2, 32768, 128),
                                        (2, 20000, 33), (2, 73448, 100), (2, 151936, 128), (2, 32776, 128),
                                        # rows that are not whole 16-byte pieces (every row but the first starts off 16 bytes)
                                        (3, 510, 59), (4, 100, 10), (3, 1001, 128), (3, 4099, 59), (4, 32001, 59), (3, 32767, 10),
                                        (2, 50257, 64), (2, 151643, 59), (2, 65537, 128), (5, 9, 9), (3, 1025, 100)])
def test_topk_matches_oracle(gpu, orc, n, dim, top):
    from cpm.cu_amd import ops
    torch = gpu
    g = synth.rng(dim, top)
    x = g.standard_normal((n, dim)).astype(np.float16)
    val, pos = ops.topk(to_dev(torch, x), top)
    torch.cuda.synchronize()
    v_ref, p_ref = orc.topk(x, top)
    assert np.array_equal(to_np(pos), p_ref)
    assert np.array_equal(to_np(val).view(np.uint16), v_ref.view(np.uint16))


@pytest.mark.parametrize("n,dim,top,off", [(3, 512, 59, 1), (2, 32768, 10, 3), (2, 40960, 64, 5), (4, 104, 10, 7), (2, 8200, 128, 2)])
def test_topk_of_rows_that_start_off_16_bytes(gpu, orc, n, dim, top, off):
    """The input begins `off` elements into an aligned buffer: the row kernel reads such rows element by element."""
    from cpm.cu_amd import ops
    torch = gpu
    x = synth.rng(dim, off).standard_normal((n, dim)).astype(np.float16)
    buf = torch.zeros(n * dim + 8, dtype=torch.float16, device="cuda")
    d_x = buf[off:off + n * dim].view(n, dim)
    d_x.copy_(to_dev(torch, x))
    assert d_x.data_ptr() % 16 != 0
    val, pos = ops.topk(d_x, top)
    torch.cuda.synchronize()
    v_ref, p_ref = orc.topk(x, top)
    assert np.array_equal(to_np(pos), p_ref)
    assert np.array_equal(to_np(val).view(np.uint16), v_ref.view(np.uint16))


@pytest.mark.parametrize("n,dim,top,kind", [(3, 510, 59, "normal"), (10, 32768, 10, "normal"), (2, 32768, 64, "ties"), (4, 5000, 32, "ties"),
                                            (2, 73448, 25, "normal"), (3, 20000, 100, "normal"), (2, 32001, 63, "ties"), (5, 64, 64, "normal"),
                                            (2, 16384, 40, "neg_inf")])
def test_topk_row_kernel_equals_chunk_and_merge_form(gpu, orc, set_option, n, dim, top, kind):
    """The library's two top-k implementations (option topk_row_kernel): the one-launch row kernel, which bounds, extracts
    and ranks by counting, and k rounds of a maximum search per 2048-element chunk followed by a merge launch -- the same
    positions and value bits from both, and from the oracle."""
    from cpm.cu_amd import ops
    torch = gpu
    g = synth.rng(dim, top + 1)
    if kind == "ties":
        x = (g.integers(-3, 4, size=(n, dim)) * 0.5).astype(np.float16)
    else:
        x = g.standard_normal((n, dim)).astype(np.float16)
    if kind == "neg_inf":
        x[:, g.random(dim) < 0.97] = -np.inf
    d_x = to_dev(torch, x)
    got = []
    for form in (1, 0):
        set_option("topk_row_kernel", form)
        val, pos = ops.topk(d_x, top)
        torch.cuda.synchronize()
        got.append((to_np(val).view(np.uint16).copy(), to_np(pos).copy()))
    assert np.array_equal(got[0][0], got[1][0]) and np.array_equal(got[0][1], got[1][1])
    v_ref, p_ref = orc.topk(x, top)
    assert np.array_equal(got[0][1], p_ref) and np.array_equal(got[0][0], v_ref.view(np.uint16))


def test_frspec_head_with_the_chunk_and_merge_top_k(gpu, orc, set_option):
    """The FR-Spec head with the fused log-softmax statistics ranked by the chunk + merge form instead of the row kernel."""
    set_option("topk_row_kernel", 0)
    _frspec_check(gpu, orc, n=10, V=9000, Vs=4096, H=512, k=10, seed=31, tiled=True)
    _frspec_check(gpu, orc, n=3, V=70000, Vs=65536, H=512, k=16, seed=32, tiled=True)
    _frspec_check(gpu, orc, n=5, V=9000, Vs=4099, H=512, k=32, seed=33, tiled=False)


def test_topk_heavy_ties_and_neg_inf(gpu, orc):
    from cpm.cu_amd import ops
    torch = gpu
    g = synth.rng(77, 0)
    x = g.integers(-3, 3, size=(5, 6000)).astype(np.float16)  # few distinct values -> ties everywhere
    x[0, :] = 1.0
    x[1, 100:] = -np.inf
    x[2, ::2] = -0.0
    x[2, 1::2] = 0.0
    val, pos = ops.topk(to_dev(torch, x), 32)
    torch.cuda.synchronize()
    v_ref, p_ref = orc.topk(x, 32)
    assert np.array_equal(to_np(pos), p_ref)
    assert np.array_equal(to_np(val).view(np.uint16), v_ref.view(np.uint16))
    assert np.array_equal(p_ref[0], np.arange(32))


@pytest.mark.parametrize("case", ["two_values", "mostly_neg_inf", "descending", "ascending", "wide_range", "k64", "tiny_rows",
                                  "k128_descending", "k64_one_wave_neg_inf", "k100_two_values", "k40_few_finite"])
def test_topk_row_kernel_shapes_of_data(gpu, orc, case):
    """Inputs chosen against the one-launch row kernel's bound / candidate / fallback logic."""
    from cpm.cu_amd import ops
    torch = gpu
    g = synth.rng(len(case), 5)
    top = 10
    if case == "two_values":
        x = g.integers(0, 2, size=(4, 32768)).astype(np.float16)          # half the row ties for the top: fallback
    elif case == "mostly_neg_inf":
        x = np.full((3, 8192), -np.inf, np.float16)
        x[0, 5] = 1.0                                                      # fewer finite values than k
        x[1, ::700] = g.standard_normal(len(x[1, ::700])).astype(np.float16)
        x[2, :12] = np.arange(12, dtype=np.float16)
    elif case == "descending":
        x = np.tile(np.linspace(8, -8, 32768, dtype=np.float32).astype(np.float16), (2, 1))   # all of the top in one wave
    elif case == "ascending":
        x = np.tile(np.linspace(-8, 8, 16384, dtype=np.float32).astype(np.float16), (2, 1))
    elif case == "wide_range":
        x = (g.standard_normal((5, 24576)) * np.exp(g.standard_normal((5, 24576)) * 3)).astype(np.float16)
        x[0, 100] = np.float16(65504)
        x[1, 200] = np.float16(-65504)
        x[2, :64] = np.float16(6e-8)                                       # subnormals and signed zeros near the bound
        x[3, ::2] = 0.0
        x[3, 1::2] = -0.0
    elif case == "k64":
        x = g.standard_normal((3, 32768)).astype(np.float16)
        top = 64
    elif case == "k128_descending":
        x = np.tile(np.linspace(8, -8, 32768, dtype=np.float32).astype(np.float16), (2, 1))   # the waves' shares of k are far apart
        x[1] = x[1, ::-1]
        top = 128
    elif case == "k64_one_wave_neg_inf":
        x = g.standard_normal((3, 16384)).astype(np.float16)
        x[0, 8 * 64 * 3:8 * 64 * 4] = -np.inf                              # first piece of wave 3: that wave's share has no finite bound
        x[1].reshape(2, 16, 64, 8)[:, 5] = -np.inf                         # everything wave 5 holds (piece, wave, lane, element)
        x[2].reshape(2, 16, 64, 8)[:, 1:] = -np.inf                        # only wave 0 holds finite values
        top = 64
    elif case == "k100_two_values":
        x = g.integers(0, 2, size=(3, 8192)).astype(np.float16)
        x[1, 50:] = 0                                                      # fewer ones than k: the bound is the tie value
        top = 100
    elif case == "k40_few_finite":
        x = np.full((2, 4096), -np.inf, np.float16)
        x[0, ::128] = g.standard_normal(32).astype(np.float16)             # 32 finite values for k = 40
        x[1, 7::64] = g.standard_normal(64).astype(np.float16)
        top = 40
    else:
        x = g.standard_normal((6, 64)).astype(np.float16)                  # one wave holds everything
        top = 8
    val, pos = ops.topk(to_dev(torch, x), top)
    torch.cuda.synchronize()
    v_ref, p_ref = orc.topk(x, top)
    assert np.array_equal(to_np(pos), p_ref)
    assert np.array_equal(to_np(val).view(np.uint16), v_ref.view(np.uint16))


@pytest.mark.parametrize("n,dim,off", [(3, 32768, 0), (1, 7, 0), (5, 510, 0), (2, 32768 + 8, 0), (3, 73448, 0), (2, 151643, 0), (4, 4096, 3),
                                       (2, 40000, 5), (3, 33, 1), (16, 1000, 0)])
def test_log_softmax_operator(gpu, orc, n, dim, off):
    """Rows of whole 16-byte pieces, rows with single elements in front of and behind the pieces (odd lengths; a buffer that
    starts `off` elements off 16 bytes), rows shorter than a piece, rows longer than the registers hold."""
    from cpm.cu_amd import ops
    torch = gpu
    x = (synth.rng(dim, 5 + off).standard_normal((n, dim)) * 1.3).astype(np.float16)
    buf = torch.zeros(n * dim + 8, dtype=torch.float16, device="cuda")
    d = buf[off:off + n * dim].view(n, dim)
    d.copy_(to_dev(torch, x))
    stats = to_np(ops.log_softmax_(d))
    torch.cuda.synchronize()
    lp_ref, m_ref, lse_ref = orc.log_softmax(x)
    assert np.array_equal(stats[:, 0], m_ref)
    assert np.allclose(stats[:, 1], lse_ref, atol=1e-4)
    staged = orc.log_softmax_apply(x, stats[:, 0], stats[:, 1])
    assert np.array_equal(to_np(d).view(np.uint16), staged.view(np.uint16))
    assert_close_f16(to_np(d), lp_ref, "log_softmax", atol=2e-2, rtol=1e-2)
    assert not to_np(buf[:off]).any() and not to_np(buf[off + n * dim:]).any()  # nothing written outside the rows


@pytest.mark.parametrize("n,V,H", [(60, 1000 + 7, 512), (10, 4096, 1024), (24, 530, 2048), (128, 2000, 512), (1, 16, 512)])
def test_tiled_weight_layout_gives_the_same_logits(gpu, orc, n, V, H):
    """The tiled layout holds the same numbers in another order.  The kernels chosen for the two layouts
    may walk K in different chunk sizes, so the fp32 sums can differ in their last bits: logits agree
    to an fp16 ulp, the arg-max wherever the top two are further apart than that, both match the oracle."""
    from cpm.cu_amd import ops
    torch = gpu
    hid = synth.normal_f16((n, H), V + n, 1)
    w = synth.normal_f16((V, H), V + n, 2, std=0.05)
    d_hid, d_w = to_dev(torch, hid), to_dev(torch, w)
    gt_r, z_r = ops.lm_head_argmax(d_hid, d_w, want_logits=True)
    gt_t, z_t = ops.lm_head_argmax(d_hid, ops.tile_head_weight(d_w), want_logits=True)
    torch.cuda.synchronize()
    assert_close_f16(to_np(z_t), to_np(z_r), "tiled vs row-major logits", atol=8e-3, rtol=2e-3)
    ref = orc.lm_head(hid, w)
    assert_close_f16(to_np(z_t), ref, "tiled target logits")
    top2 = np.sort(ref.astype(np.float32), axis=1)[:, -2:]
    clear = (top2[:, 1] - top2[:, 0]) > 2e-2
    assert np.array_equal(to_np(gt_t)[clear], to_np(gt_r)[clear]) and np.array_equal(to_np(gt_t)[clear], orc.argmax(ref)[clear])


@pytest.mark.parametrize("n,V,H", [(60, 73448, 4096), (10, 40000, 1024), (33, 36000, 512), (64, 34000, 512), (5, 32768 + 16 * 300, 512)])
def test_shared_last_pass_equals_plain_mapping(gpu, orc, set_option, n, V, H):
    """Row-block counts that leave the last pass partly filled (1, 2 or more blocks per workgroup, with 2, 4 and 16
    K chunks): the waves that share a block add their partial sums in LDS.  Same logits as the plain mapping up to
    the fp32 summation order, same arg-max wherever the top two are apart, and both match the oracle."""
    from cpm.cu_amd import ops
    torch = gpu
    hid = synth.normal_f16((n, H), V, 1)
    w = synth.normal_f16((V, H), V, 2, std=0.02)
    d_hid = to_dev(torch, hid)
    wt = ops.tile_head_weight(to_dev(torch, w))
    gt_s, z_s = ops.lm_head_argmax(d_hid, wt, want_logits=True)
    torch.cuda.synchronize()
    set_option("head_share_last_pass", 0)
    gt_p, z_p = ops.lm_head_argmax(d_hid, wt, want_logits=True)
    torch.cuda.synchronize()
    assert_close_f16(to_np(z_s), to_np(z_p), "shared vs plain last pass", atol=8e-3, rtol=2e-3)
    z_ref = orc.lm_head(hid, w)
    assert_close_f16(to_np(z_s), z_ref, "shared last pass vs oracle")
    for z, gt in ((to_np(z_s), to_np(gt_s)), (to_np(z_p), to_np(gt_p))):
        assert np.array_equal(gt, orc.argmax(z))  # staged: the kernel's own logits decide


def test_tiled_frspec_head_with_fused_gather(gpu, orc):
    """tile_head_weight with a row map == gather_rows followed by tiling == the row-major sub-matrix."""
    from cpm.cu_amd import ops
    torch = gpu
    V, Vs, H, n, k = 3000, 1024 + 8, 512, 10, 10
    hid = synth.normal_f16((n, H), 91, 1)
    w = synth.normal_f16((V, H), 91, 2, std=0.05)
    remap = synth.frspec_remap(V, Vs, 91)
    d_hid, d_w, d_remap = to_dev(torch, hid), to_dev(torch, w), to_dev(torch, remap)
    a = ops.frspec_head_topk(d_hid, ops.gather_rows(d_w, d_remap), d_remap, k)
    b = ops.frspec_head_topk(d_hid, ops.tile_head_weight(d_w, d_remap), d_remap, k)
    torch.cuda.synchronize()
    ref = orc.lm_head(hid, orc.gather_rows(w, remap))
    assert_close_f16(to_np(b["logits"]), to_np(a["logits"]), "tiled vs row-major FR-Spec logits", atol=8e-3, rtol=2e-3)
    assert_close_f16(to_np(b["logits"]), ref, "tiled FR-Spec logits")
    # staged exactness of the tiled path: the oracle ranks the device's own logits and statistics
    st = to_np(b["row_stats"])
    lp = orc.log_softmax_apply(to_np(b["logits"]), st[:, 0], st[:, 1])
    val_s, pos_s = orc.topk(lp, k)
    assert np.array_equal(to_np(b["pos"]), pos_s) and np.array_equal(to_np(b["val"]).view(np.uint16), val_s.view(np.uint16))
    assert np.array_equal(to_np(b["ids"]), remap[pos_s])


# (rows, vocabulary, hidden, head_scale) -> streaming kernel <NB, FP, KC>, waves per shared last-pass block
_STREAM_SHAPES = [
    (60, 73448, 4096, None),      # <4,2,256>, 4
    (10, 32768, 4096, None),      # <1,1,512>, no last pass
    (1, 32768 + 16 * 300, 512, None),   # <1,1,512>, 4; a single K chunk
    (33, 36000, 512, 0.3125),     # <4,1,256>, 8
    (64, 50000, 512, None),       # <4,1,256>, 1 (five blocks of the last pass per workgroup)
    (20, 45000, 1024, None),      # <2,1,512>, 2
    (100, 40000, 512, None),      # <8,1,128>, 4
    (128, 70000, 512, 2.0),       # <8,2,128>, 4
    (16, 122753, 1024, None),     # <1,3,256>, 1
    (32, 110000, 512, None),      # <2,3,256>, 2
    (60, 100000, 512, None),      # <4,3,128>, 4
    (17, 151936, 512, None),      # <2,4,128>, 1
    (60, 140000, 512, 0.3125),    # <4,4,128>, 2
    (7, 140000, 512, None),       # <1,4,256>, 2
    (40, 65536, 512, None),       # <4,2,256>, no last pass
    (24, 65536 + 16 * 2047, 1024, None),  # <2,2,256>, 1: all but one wave slot of the last pass filled
    (128, 100000, 512, None),     # <8,1,128> on twice as many workgroups as CUs (three full passes would not fit the accumulators)
    (100, 151936, 512, 0.3125),   # <8,2,128> likewise
    (65, 220000, 512, None),      # <8,2,128> on three times as many
    (16, 200000, 512, None),      # <1,3,256> on twice as many (six passes over the CUs' wave slots)
    (40, 262144, 512, 2.0),       # <4,4,128> on twice as many, no last pass
    (20, 400000, 512, None),      # <2,4,128> on three times as many
]


@pytest.mark.parametrize("n,V,H,scale", _STREAM_SHAPES)
def test_streaming_head_kernel_equals_chunked_kernel(gpu, orc, set_option, n, V, H, scale):
    """Tiled weights of at least one full pass run the streaming kernel (register ring refilled fragment by
    fragment, last pass shared by K slices).  Every (row blocks, full passes) shape it is built for, with 1, 2,
    4 and 8 waves per last-pass block and without a last pass: same logits as the K-chunked kernel up to the
    fp32 summation order, both within tolerance of the oracle, arg-max exact on each kernel's own logits."""
    from cpm.cu_amd import ops
    torch = gpu
    hid = synth.normal_f16((n, H), V + n, 1)
    w = synth.normal_f16((V, H), V + n, 2, std=0.02)
    d_hid = to_dev(torch, hid)
    wt = ops.tile_head_weight(to_dev(torch, w))
    assert "head_gemm_stream_kernel" in ops.head_plan(n, wt)[0]
    gt_s, z_s = ops.lm_head_argmax(d_hid, wt, head_scale=scale, want_logits=True)
    gt_s2 = ops.lm_head_argmax(d_hid, wt, head_scale=scale)
    torch.cuda.synchronize()
    set_option("head_stream_kernel", 0)
    assert "head_gemm_stream_kernel" not in ops.head_plan(n, wt)[0]
    gt_c, z_c = ops.lm_head_argmax(d_hid, wt, head_scale=scale, want_logits=True)
    torch.cuda.synchronize()
    assert_close_f16(to_np(z_s), to_np(z_c), "streaming vs chunked kernel", atol=8e-3, rtol=2e-3)
    z_ref = orc.lm_head(hid, w, head_scale=scale)
    assert_close_f16(to_np(z_s), z_ref, "streaming kernel vs oracle")
    assert np.array_equal(to_np(gt_s), to_np(gt_s2))
    for z, gt in ((to_np(z_s), to_np(gt_s)), (to_np(z_c), to_np(gt_c))):
        assert np.array_equal(gt, orc.argmax(z))  # staged: the kernel's own logits decide


def test_streaming_head_kernel_plain_last_pass(gpu, orc, set_option):
    """head_share_last_pass = 0 on the streaming kernel: whole row blocks per wave in the last pass."""
    from cpm.cu_amd import ops
    torch = gpu
    n, V, H = 60, 73448, 512
    hid = synth.normal_f16((n, H), 5, 1)
    w = synth.normal_f16((V, H), 5, 2, std=0.02)
    d_hid = to_dev(torch, hid)
    wt = ops.tile_head_weight(to_dev(torch, w))
    gt_s, z_s = ops.lm_head_argmax(d_hid, wt, want_logits=True)
    torch.cuda.synchronize()
    set_option("head_share_last_pass", 0)
    assert "head_gemm_stream_kernel" in ops.head_plan(n, wt)[0]
    gt_p, z_p = ops.lm_head_argmax(d_hid, wt, want_logits=True)
    torch.cuda.synchronize()
    assert_close_f16(to_np(z_s), to_np(z_p), "shared vs plain last pass", atol=8e-3, rtol=2e-3)
    assert_close_f16(to_np(z_p), orc.lm_head(hid, w), "plain last pass vs oracle")
    assert np.array_equal(to_np(gt_p), orc.argmax(to_np(z_p)))
