"""The MFMA-rate probe (bench.py's measurement helper, its own small library): it must do the arithmetic it claims."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_mfma_rate_probe_counts_its_flops(gpu):
    import bench_probes
    torch = gpu
    n = bench_probes.load().bench_mfma_rate_probe_operand_bytes() // 2
    assert n == 16 * 512 * 8
    ones = torch.ones(n, dtype=torch.float16, device="cuda")
    wgs, iters = 3, 10
    flops, out = bench_probes.mfma_rate_probe(ones, iters, wgs)
    torch.cuda.synchronize()
    # all-ones operands: every MFMA adds k = 16 to each of a lane's 16 accumulator values; 16 MFMAs per iteration
    assert np.array_equal(out.cpu().numpy(), np.full(wgs * 512, iters * 16 * 16 * 16, np.float32))
    assert flops == wgs * 8 * iters * 16 * 2.0 * 32 * 32 * 16
    with pytest.raises(ValueError):
        bench_probes.mfma_rate_probe(ones, 0, wgs)
