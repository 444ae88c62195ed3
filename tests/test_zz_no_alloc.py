"""The allocation-free target head (cpmcu_lm_head_argmax_static) against cpmcu_lm_head_argmax.

Both entry points launch the same kernels, one on a caller-provided workspace and one on the device array
built into the library, so their results must be identical bit for bit: the arg-max ids and the fp16
logits.  Two calls in a row share the built-in array; the second one is smaller (fewer rows, a smaller
vocabulary, fewer workgroups), so anything the first call left behind would show.
"""
import ctypes

import numpy as np
import pytest

from cpm.cu_amd import synth
from util import to_dev, to_np

pytestmark = pytest.mark.gpu


def _both(torch, hid, w, layout, V, H, scale):
    from cpm.cu_amd import lib, ops
    L = lib.get()
    n = hid.shape[0]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ws = torch.empty(L.raw.cpmcu_head_workspace_bytes(n, V), dtype=torch.uint8, device="cuda")
    out = []
    for static in (False, True):
        logits = torch.full((n, V), float("nan"), dtype=torch.float16, device="cuda")
        gt = torch.full((n,), -7, dtype=torch.int32, device="cuda")
        if static:
            L.lm_head_argmax_static(p(hid), p(w), layout, n, V, H, 1, ctypes.c_float(scale), p(logits), p(gt), st)
        else:
            L.lm_head_argmax(p(hid), p(w), layout, n, V, H, 1, ctypes.c_float(scale), p(logits), p(gt), p(ws), ws.numel(), st)
        torch.cuda.synchronize()
        out.append((to_np(gt), to_np(logits)))
    return out


def test_static_scratch_head_matches_workspace_head(gpu, orc):
    torch = gpu
    from cpm.cu_amd import lib, ops
    L = lib.get()
    assert L.raw.cpmcu_lm_head_argmax_static_scratch_bytes() == 1 << 20
    # first call: 60 rows on a 40000 x 1024 tiled head (every CU busy); second: 5 rows on 1000 x 512, row-major
    for (n, V, H, tiled, seed) in ((60, 40000, 1024, True, 1), (5, 1000, 512, False, 2)):
        hid = to_dev(torch, synth.normal_f16((n, H), seed, 1))
        w_np = synth.normal_f16((V, H), seed, 2, std=0.02)
        w = to_dev(torch, w_np)
        if tiled:
            tw = ops.tile_head_weight(w)
            wd, layout = tw.data, ops.W_TILED
        else:
            wd, layout = w, ops.W_ROW_MAJOR
        (gt_ws, z_ws), (gt_st, z_st) = _both(torch, hid, wd, layout, V, H, 0.5)
        assert np.array_equal(gt_st, gt_ws), (n, V, gt_st, gt_ws)
        assert np.array_equal(z_st.view(np.uint16), z_ws.view(np.uint16))
        # and the shared result is the oracle's arg-max of the device logits (lowest index on ties)
        assert np.array_equal(gt_st, orc.argmax(z_st))
    # what the entry point is for: it takes no device memory, and it can be part of a stream capture (its first call on the
    # device, above, was outside one)
    n, V, H = 60, 40000, 1024
    hid = to_dev(torch, synth.normal_f16((n, H), 1, 1))
    tw = ops.tile_head_weight(to_dev(torch, synth.normal_f16((V, H), 1, 2, std=0.02)))
    gt = torch.full((n,), -7, dtype=torch.int32, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    call = lambda: L.lm_head_argmax_static(p(hid), p(tw.data), ops.W_TILED, n, V, H, 1, ctypes.c_float(0.5), None, p(gt),
                                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the call took device memory"
    ref = to_np(gt).copy()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call()
    for rep in range(3):
        gt.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(to_np(gt), ref), rep
    # more rows than the built-in scratch holds: a clear error, nothing launched
    with pytest.raises(ValueError, match="outside \\[1, 128\\]"):
        q = ctypes.c_void_p(16)
        L.lm_head_argmax_static(q, q, 0, 129, 1000, 512, 0, ctypes.c_float(1.0), q, q, None)
