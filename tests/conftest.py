import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure): built on demand with g++."""
    import oracle
    return oracle


@pytest.fixture(scope="session")
def gpu():
    """torch + the HIP library on cuda:0; skips (never falls back) when there is no GPU."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    from cpm.cu_amd import lib
    lib.get()  # raises ImportError if libcpmcu_amd.so is missing: no fallback
    torch.cuda.set_device(0)
    return torch


@pytest.fixture
def set_option():
    """Sets kernel-shape options of the library for one test and restores the defaults afterwards."""
    from cpm.cu_amd import lib
    defaults = {"dtype": 0, "attn_kv_groups": 0, "head_share_last_pass": 1, "head_stream_kernel": 1, "attn_merge_in_launch": 1, "attn_merge_wait_us": 2000,
                "frspec_fused": 0, "frspec_wait_us": 50000, "topk_row_kernel": 1}
    touched = []

    def setter(name, value):
        lib.get().set_option(name.encode(), int(value))
        touched.append(name)
    yield setter
    for name in touched:
        lib.get().set_option(name.encode(), defaults[name])
