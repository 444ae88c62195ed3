"""The MFMA-rate probe (a measurement helper of the library): it must do the arithmetic it claims."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_mfma_rate_probe_counts_its_flops(gpu):
    from cpm.cu_amd import lib as libmod
    torch = gpu
    L = libmod.get()
    n = L.raw.cpmcu_mfma_rate_probe_operand_bytes() // 2
    assert n == 16 * 512 * 8
    ones = torch.ones(n, dtype=torch.float16, device="cuda")
    wgs, iters = 3, 10
    out = torch.zeros(wgs * 512, dtype=torch.float32, device="cuda")
    flops = ctypes.c_double(0.0)
    L.mfma_rate_probe(ones.data_ptr(), iters, wgs, out.data_ptr(), ctypes.byref(flops), None)
    torch.cuda.synchronize()
    # all-ones operands: every MFMA adds k = 16 to each of a lane's 16 accumulator values; 16 MFMAs per iteration
    assert np.array_equal(out.cpu().numpy(), np.full(wgs * 512, iters * 16 * 16 * 16, np.float32))
    assert flops.value == wgs * 8 * iters * 16 * 2.0 * 32 * 32 * 16
    with pytest.raises(ValueError):
        L.mfma_rate_probe(ones.data_ptr(), 0, wgs, out.data_ptr(), None, None)
