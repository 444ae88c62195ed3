"""Measurement helpers of bench.py that are not part of the product library.

``mfma_rate_probe``: a register-resident loop of v_mfma_f32_32x32x16_f16 (bench_probes/mfma_rate_probe.hip, built
into bench_probes/libbench_probes.so by ``cpm.cu_amd.build``): what the matrix pipes of this GPU sustain on
given operand data when a kernel does nothing else.
"""
import ctypes
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libbench_probes.so")
_lib = None


def load():
    global _lib
    if _lib is None:
        import torch  # noqa: F401  (one HIP runtime per process: the one torch loaded)
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is not built; run `python -m cpm.cu_amd.build`" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.bench_mfma_rate_probe_operand_bytes.restype = ctypes.c_size_t
        _lib.bench_mfma_rate_probe_operand_bytes.argtypes = []
        _lib.bench_mfma_rate_probe.restype = ctypes.c_int
        _lib.bench_mfma_rate_probe.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                               ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    return _lib


def mfma_rate_probe(operands, iters, workgroups=256, out=None):
    """Enqueue the probe on torch's current stream; returns (flops of the launch, out tensor)."""
    import torch
    lib = load()
    need = lib.bench_mfma_rate_probe_operand_bytes()
    assert operands.dtype == torch.float16 and operands.numel() * 2 >= need and operands.is_contiguous() and operands.is_cuda
    if out is None:
        out = torch.empty(workgroups * 512, dtype=torch.float32, device=operands.device)
    flops = ctypes.c_double(0.0)
    rc = lib.bench_mfma_rate_probe(operands.data_ptr(), int(iters), int(workgroups), out.data_ptr(), ctypes.byref(flops),
                                   torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise ValueError("bench_mfma_rate_probe failed with code %d" % rc)
    return flops.value, out
