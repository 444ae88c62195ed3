"""Helpers shared by the tests: tolerances of the path and torch <-> numpy plumbing."""
import numpy as np

# fp16 results (attention outputs, logits): max-abs 2e-2 and max-rel 1e-2, where max-rel is the
# largest absolute error divided by the largest reference magnitude
ATOL_F16 = 2e-2
RTOL_F16 = 1e-2


def err_stats(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    d = np.abs(got - ref)
    max_abs = float(d.max()) if d.size else 0.0
    max_rel = max_abs / max(float(np.abs(ref).max()), 1e-30) if d.size else 0.0
    return max_abs, max_rel


def assert_close_f16(got, ref, what="", atol=ATOL_F16, rtol=RTOL_F16):
    assert np.all(np.isfinite(np.asarray(got, np.float32))), "%s: non-finite values" % what
    max_abs, max_rel = err_stats(got, ref)
    assert max_abs <= atol and max_rel <= rtol, "%s: max_abs=%.3e (limit %.1e) max_rel=%.3e (limit %.1e)" % (
        what, max_abs, atol, max_rel, rtol)
    return max_abs, max_rel


def to_dev(torch, a):
    """numpy -> cuda tensor (uint64 masks travel as int64 bit patterns)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint64:
        return torch.from_numpy(a.view(np.int64)).cuda()
    return torch.from_numpy(a).cuda()


def to_np(t):
    return t.detach().cpu().numpy()
