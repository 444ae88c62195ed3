"""The FR-Spec head with its log-softmax, top-k and id map-back in ONE launch (cpmcu_frspec_head_topk on tiled weights,
k <= 16, option frspec_fused = 1) against the same call as two launches (the default) -- every output bit for bit -- and against the
oracle's ranking of the device logits.  The reference runs these steps as separate kernels
(src/model/minicpm4/minicpm4_eagle.cuh:366-372: Linear::prefill, log_softmax src/model/eagle.cuh:29-89, TopK::prefill
src/model/topk.cuh:255-288, remap src/model/tree_drafter.cuh:88-90).

Covered: one and two full passes of row blocks, a shared last pass, 1 / 10 / 16 hidden rows and changing row counts on
one workspace (the per-row generations of the published words), rows dominated by equal values (redone from the logits
in memory), token ids beyond 20 bits, bfloat16, replays of a captured graph, and a wait that is forced to run out from
the host (every kernel still exits; the rows hold -1 and the next synchronisation reports it)."""
import ctypes

import numpy as np
import pytest

from cpm.cu_amd import synth
from util import to_dev, to_np

pytestmark = pytest.mark.gpu


def _rows_seen(lib):
    f, s, t = ctypes.c_long(0), ctypes.c_long(0), ctypes.c_long(0)
    lib.get().frspec_fused_rows(ctypes.byref(f), ctypes.byref(s), ctypes.byref(t))
    return f.value, s.value, t.value


def _both_forms(torch, set_option, hid, d_w, d_remap, k):
    from cpm.cu_amd import ops
    d_hid = to_dev(torch, hid)
    set_option("frspec_fused", 1)
    one = ops.frspec_head_topk(d_hid, d_w, d_remap, k)
    torch.cuda.synchronize()
    one = {key: to_np(v).copy() for key, v in one.items()}
    set_option("frspec_fused", 0)
    two = ops.frspec_head_topk(d_hid, d_w, d_remap, k)
    torch.cuda.synchronize()
    two = {key: to_np(v).copy() for key, v in two.items()}
    return one, two


def _assert_same(one, two, what):
    """Bit for bit: the finisher of the one-launch form adds the workgroups' (max, sum exp) up in the order of the two-launch
    form's row kernel (which ranks rows beyond 32768 elements in slices, every slice reducing the statistics the same way)."""
    assert np.array_equal(one["logits"].view(np.uint16), two["logits"].view(np.uint16)), what + ": logits"
    assert np.array_equal(one["row_stats"].view(np.uint32), two["row_stats"].view(np.uint32)), what + ": row statistics"
    assert np.array_equal(one["pos"], two["pos"]), what + ": positions"
    assert np.array_equal(one["val"].view(np.uint16), two["val"].view(np.uint16)), what + ": values"
    assert np.array_equal(one["ids"], two["ids"]), what + ": ids"


@pytest.mark.parametrize("n,Vs,H,k", [(10, 32768, 4096, 10), (1, 32768, 4096, 10), (16, 32768, 512, 16), (10, 16384, 512, 10),
                                      (7, 4096, 1024, 10), (10, 32768 + 16 * 300, 512, 10), (5, 65536, 512, 8), (3, 50000, 512, 1),
                                      (16, 8192, 512, 3)])
def test_one_launch_equals_two_launches(gpu, orc, set_option, n, Vs, H, k):
    """Random data: every row is finished from the published candidates, and nothing differs from the two-launch form."""
    torch = gpu
    from cpm.cu_amd import lib, ops
    hid = synth.normal_f16((n, H), Vs % 89 + n, 1)
    w = synth.normal_f16((Vs, H), Vs % 89 + n, 2, std=0.02)
    remap = synth.frspec_remap(Vs + 3000, Vs, n)
    d_w = ops.tile_head_weight(to_dev(torch, w))
    d_remap = to_dev(torch, remap)
    ws = ops._workspace("head", lib.get().raw.cpmcu_head_workspace_bytes(n, Vs), d_remap.device)
    ops.release_head_workspace(ws)  # states that earlier tests' shapes hold on this workspace
    set_option("frspec_fused", 1)
    assert lib.get().raw.cpmcu_frspec_head_mode(ctypes.c_void_p(ws.data_ptr()), 1, n, Vs, H, k) == 1
    lib.get().synchronize()
    before = _rows_seen(lib)
    one, two = _both_forms(torch, set_option, hid, d_w, d_remap, k)
    lib.get().synchronize()
    after = _rows_seen(lib)
    _assert_same(one, two, "n=%d Vs=%d H=%d k=%d" % (n, Vs, H, k))
    assert after[0] - before[0] + after[1] - before[1] == n and after[2] == before[2]
    if Vs >= 16384:
        assert after[0] - before[0] == n, "rows of ordinary data are finished from the published candidates"
    # and the oracle's ranking of the device logits under the device statistics
    lp = orc.log_softmax_apply(one["logits"], one["row_stats"][:, 0], one["row_stats"][:, 1])
    val_s, pos_s = orc.topk(lp, k)
    assert np.array_equal(one["pos"], pos_s)
    assert np.array_equal(one["val"].view(np.uint16), val_s.view(np.uint16))
    assert np.array_equal(one["ids"], remap[pos_s])


@pytest.mark.parametrize("case", ["all_equal", "flat", "two_values", "one_workgroup_holds_the_top", "neg_inf"])
def test_rows_dominated_by_equal_values(gpu, orc, set_option, case):
    """Data on which a workgroup has more candidates than slots, or no bound exists: those rows are redone from the
    logits in memory and still match the two-launch form and the oracle."""
    torch = gpu
    from cpm.cu_amd import lib, ops
    n, Vs, H, k = 6, 32768, 512, 10
    rng = np.random.default_rng(7)
    hid = synth.normal_f16((n, H), 3, 1)
    if case == "all_equal":
        w = np.zeros((Vs, H), np.float16)
    elif case == "flat":
        w = synth.normal_f16((Vs, H), 3, 2, std=0.0003)
    elif case == "two_values":
        base = synth.normal_f16((2, H), 3, 2, std=0.02)
        w = base[rng.integers(0, 2, Vs)]
    elif case == "one_workgroup_holds_the_top":
        # the 16-row blocks of workgroup 5 (blocks 5, 261, 517, ... of 2048) all score high on every hidden row
        w = synth.normal_f16((Vs, H), 3, 2, std=0.01)
        boost = (hid.astype(np.float32).mean(axis=0) * 0.05).astype(np.float16)
        for blk in range(5, Vs // 16, 256):
            w[blk * 16:(blk + 1) * 16] += boost
    else:
        # most of every row overflows to -inf in fp16 (all-positive hidden rows against large negative weights)
        hid = (np.abs(hid.astype(np.float32)) + 8.0).astype(np.float16)
        w = synth.normal_f16((Vs, H), 3, 2, std=0.002)
        w[100:30000] = np.float16(-300.0)
    remap = synth.frspec_remap(Vs + 500, Vs, 1)
    d_w = ops.tile_head_weight(to_dev(torch, w))
    d_remap = to_dev(torch, remap)
    lib.get().synchronize()
    before = _rows_seen(lib)
    one, two = _both_forms(torch, set_option, hid, d_w, d_remap, k)
    lib.get().synchronize()
    after = _rows_seen(lib)
    _assert_same(one, two, case)
    assert after[0] - before[0] + after[1] - before[1] == n and after[2] == before[2]
    if case in ("all_equal", "flat", "two_values"):
        assert after[1] - before[1] > 0, "tie-heavy rows are expected to be redone from the logits"
    lp = orc.log_softmax_apply(one["logits"], one["row_stats"][:, 0], one["row_stats"][:, 1])
    val_s, pos_s = orc.topk(lp, k)
    assert np.array_equal(one["pos"], pos_s)
    assert np.array_equal(one["ids"], remap[pos_s])
    if case == "all_equal":
        assert np.array_equal(one["pos"], np.tile(np.arange(k, dtype=np.int32), (n, 1)))


def test_changing_row_counts_on_one_workspace(gpu, orc, set_option):
    """10, 1, 16, 3, 16 hidden rows in a row on one workspace and one matrix: words of rows that an earlier call wrote and
    a later one does not must never be taken for fresh ones."""
    torch = gpu
    from cpm.cu_amd import ops
    Vs, H, k = 32768, 512, 10
    w = synth.normal_f16((Vs, H), 21, 2, std=0.02)
    d_w = ops.tile_head_weight(to_dev(torch, w))
    d_remap = to_dev(torch, synth.frspec_remap(Vs + 100, Vs, 2))
    for i, n in enumerate([10, 1, 16, 3, 16, 1, 1, 10]):
        hid = synth.normal_f16((n, H), 100 + i, 1)
        one, two = _both_forms(torch, set_option, hid, d_w, d_remap, k)
        _assert_same(one, two, "call %d with %d rows" % (i, n))


def test_token_ids_beyond_twenty_bits(gpu, orc, set_option):
    """Published words carry 20 bits of token id; larger ids are looked up by the finisher instead."""
    torch = gpu
    from cpm.cu_amd import ops
    n, Vs, H, k = 4, 16384, 512, 10
    hid = synth.normal_f16((n, H), 5, 1)
    w = synth.normal_f16((Vs, H), 5, 2, std=0.02)
    remap = (np.arange(Vs, dtype=np.int64) * 131 + (1 << 21)).astype(np.int32)
    one, two = _both_forms(torch, set_option, hid, ops.tile_head_weight(to_dev(torch, w)), to_dev(torch, remap), k)
    _assert_same(one, two, "wide ids")
    assert np.array_equal(one["ids"], remap[one["pos"]])


def test_bfloat16(gpu, orc, set_option):
    torch = gpu
    from cpm.cu_amd import ops
    n, Vs, H, k = 10, 32768, 1024, 10
    orc.set_dtype(1)
    try:
        set_option("dtype", 1)
        hid = orc.encode(synth.normal_f16((n, H), 9, 1).astype(np.float32))
        w = orc.encode(synth.normal_f16((Vs, H), 9, 2, std=0.02).astype(np.float32))
        remap = synth.frspec_remap(Vs + 100, Vs, 3)
        d_w = ops.tile_head_weight(to_dev(torch, w))
        one, two = _both_forms(torch, set_option, hid, d_w, to_dev(torch, remap), k)
        _assert_same(one, two, "bf16")
        lp = orc.log_softmax_apply(one["logits"], one["row_stats"][:, 0], one["row_stats"][:, 1])
        val_s, pos_s = orc.topk(lp, k)
        assert np.array_equal(one["pos"], pos_s)
        assert np.array_equal(one["val"].view(np.uint16), val_s.view(np.uint16))
    finally:
        orc.set_dtype(0)


def test_replays_of_a_captured_graph(gpu, orc, set_option):
    """The launch inside a HIP graph: five replays with eager work in between, each equal to the eager result (the
    generations advance on the device, not in the launch arguments)."""
    torch = gpu
    from cpm.cu_amd import ops
    n, Vs, H, k = 10, 32768, 512, 10
    hid = synth.normal_f16((n, H), 31, 1)
    w = synth.normal_f16((Vs, H), 31, 2, std=0.02)
    d_w = ops.tile_head_weight(to_dev(torch, w))
    d_remap = to_dev(torch, synth.frspec_remap(Vs + 100, Vs, 4))
    d_hid = to_dev(torch, hid)
    set_option("frspec_fused", 1)
    eager = ops.frspec_head_topk(d_hid, d_w, d_remap, k)   # also assigns the state outside the capture
    torch.cuda.synchronize()
    ref = {key: to_np(v).copy() for key, v in eager.items()}
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            out = ops.frspec_head_topk(d_hid, d_w, d_remap, k)
    for i in range(5):
        for v in out.values():
            v.zero_()
        other = ops.frspec_head_topk(to_dev(torch, synth.normal_f16((3, H), 40 + i, 1)), d_w, d_remap, k)  # eager, same workspace
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = {key: to_np(v) for key, v in out.items()}
        _assert_same(got, ref, "replay %d" % i)
        del other


def test_a_wait_that_runs_out_is_reported(gpu, orc, set_option):
    """Wait limit zero: a finisher that does not find every word at its first look gives up.  Every kernel still exits;
    rows that were given up hold -1, the library's next synchronisation fails and says so, the device goes back to two
    launches, and switching the option on again restores the one-launch form."""
    torch = gpu
    from cpm.cu_amd import lib, ops
    n, Vs, H, k = 10, 32768, 4096, 10
    hid = synth.normal_f16((n, H), 51, 1)
    w = synth.normal_f16((Vs, H), 51, 2, std=0.02)
    d_w = ops.tile_head_weight(to_dev(torch, w))
    d_remap = to_dev(torch, synth.frspec_remap(Vs + 100, Vs, 5))
    ws = ops._workspace("head", lib.get().raw.cpmcu_head_workspace_bytes(n, Vs), d_remap.device)
    ops.release_head_workspace(ws)
    set_option("frspec_fused", 1)
    good = ops.frspec_head_topk(to_dev(torch, hid), d_w, d_remap, k)
    lib.get().synchronize()
    good = {key: to_np(v).copy() for key, v in good.items()}
    before = _rows_seen(lib)
    set_option("frspec_wait_us", 0)
    r = ops.frspec_head_topk(to_dev(torch, hid), d_w, d_remap, k)
    torch.cuda.synchronize()
    pos = to_np(r["pos"])
    given_up = [i for i in range(n) if (pos[i] == -1).all()]
    for i in range(n):
        if i not in given_up:
            assert np.array_equal(pos[i], good["pos"][i])
    if given_up:
        with pytest.raises(RuntimeError, match="not finished"):
            lib.get().synchronize()
        assert _rows_seen(lib)[2] - before[2] == len(given_up)
        assert lib.get().raw.cpmcu_frspec_head_mode(ctypes.c_void_p(ws.data_ptr()), 1, n, Vs, H, k) == 0
    else:
        lib.get().synchronize()
    set_option("frspec_wait_us", 50000)
    set_option("frspec_fused", 1)
    assert lib.get().raw.cpmcu_frspec_head_mode(ctypes.c_void_p(ws.data_ptr()), 1, n, Vs, H, k) == 1
    again = ops.frspec_head_topk(to_dev(torch, hid), d_w, d_remap, k)
    lib.get().synchronize()
    _assert_same({key: to_np(v) for key, v in again.items()}, good, "after the wait limit was restored")


def test_randomised_sweep(gpu, orc, set_option):
    """80 random shapes and data sets (1-16 rows, k 1-16, vocabularies of one and two passes with and without a last
    pass, weights from ordinary to flat to constant, a third of the rows duplicated): nothing differs from the
    two-launch form, whichever way a row was finished."""
    torch = gpu
    from cpm.cu_amd import lib, ops
    rng = np.random.default_rng(2024)
    H = 512
    weights = {}
    lib.get().synchronize()
    before = _rows_seen(lib)
    rows = 0
    for it in range(80):
        V = int(rng.choice([4096, 8192, 16384, 32768, 32768, 37568, 50000, 65536]))
        n, k = int(rng.integers(1, 17)), int(rng.integers(1, 17))
        std = float(rng.choice([0.02, 0.02, 0.002, 0.0003, 0.0]))
        if (V, std) not in weights:
            if len(weights) > 5:
                weights.clear()
            w = synth.normal_f16((V, H), it, 2, std=std) if std > 0 else np.zeros((V, H), np.float16)
            if rng.random() < 0.3:
                w[rng.integers(1, V, size=V // 3)] = w[0]
            weights[(V, std)] = ops.tile_head_weight(to_dev(torch, w))
        hid = (synth.normal_f16((n, H), it, 1).astype(np.float32) * float(rng.choice([1.0, 0.1, 4.0]))).astype(np.float16)
        remap = rng.permutation(V + 1000)[:V].astype(np.int32)
        one, two = _both_forms(torch, set_option, hid, weights[(V, std)], to_dev(torch, remap), k)
        _assert_same(one, two, "case %d: V=%d n=%d k=%d std=%g" % (it, V, n, k, std))
        rows += n
    lib.get().synchronize()
    after = _rows_seen(lib)
    assert after[2] == before[2]
    assert after[0] - before[0] > 0 and after[1] - before[1] > 0, "both ways of finishing a row are expected in the sweep"
