"""cpm.cu_amd -- MI355X (gfx950) implementation of CPM.cu's speculative-decoding verify/draft path.

The compute lives in ``libcpmcu_amd.so`` (hand-written HIP kernels behind a C-ABI, see
``include/cpmcu_amd.h``); this package is the host-side mirror of the reference's Python/pybind
interface for that path:

* ``cpm.cu_amd.lib``     -- ctypes binding of the C-ABI (status codes -> Python exceptions)
* ``cpm.cu_amd.ops``     -- the operators on torch device tensors (torch only provides memory/streams)
* ``cpm.cu_amd.kvcache`` -- the paged KV-cache layout (K row-major pages, V transposed pages)
* ``cpm.cu_amd.synth``   -- seeded synthetic trees / workloads of the benchmark configurations
* ``cpm.cu_amd.driver``  -- the per-step loop of cpmcu/speculative/tree_drafter.py:222-250
* ``cpm.cu_amd.model``   -- the library's process-global model (its own paged cache, heads and HIP graphs) from Python
* ``cpm.cu_amd.C``       -- pybind11 module with the function names of the reference's src/entry.cu

There is no CPU fallback: importing ``lib`` without the built shared library raises.
"""
import torch  # noqa: F401,E402  -- first, so the shared library binds to the HIP runtime torch loads

__all__ = ["lib", "ops", "kvcache", "synth", "driver", "model"]
