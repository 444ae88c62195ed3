"""CPU-only checks of the boundary: the shared library loads without a GPU and exports every symbol
that include/cpmcu_amd.h declares; the ctypes table covers them all; argument validation that needs
no device works; the pybind11 module `C` exposes the reference's entry-point names."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cpmcu_amd.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cpmcu_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from cpm.cu_amd import lib
    raw = ctypes.CDLL(lib.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 30
    for name in names:
        assert hasattr(raw, name), "libcpmcu_amd.so does not export %s" % name


def test_timeline_library_is_the_product_plus_its_readers():
    """The build with the in-kernel stamps (csrc/timeline.h) exports everything the product library does, and the two
    functions that hand the records over; the product library has neither."""
    from cpm.cu_amd import build, lib
    tl = ctypes.CDLL(build.TIMELINE_LIB_PATH)
    for name in declared_symbols():
        assert hasattr(tl, name), "libcpmcu_amd_timeline.so does not export %s" % name
    product = ctypes.CDLL(lib.LIB_PATH)
    for name in ("cpmcu_timeline_read_attention", "cpmcu_timeline_read_head", "cpmcu_timeline_read_topk"):
        assert hasattr(tl, name)
        assert not hasattr(product, name)


def test_ctypes_table_matches_header():
    from cpm.cu_amd import lib
    assert sorted(lib.SIGNATURES) == declared_symbols()
    lib.load_raw()


def test_argument_validation_without_device():
    """Checks that run before any HIP call: status codes, messages, exception mapping."""
    from cpm.cu_amd import lib
    L = lib.get()
    assert b"gfx950" in L.raw.cpmcu_version()
    with pytest.raises(ValueError, match="null pointer"):
        L.tree_accept(60, None, None, None, None, None, 1, None, None, None)
    with pytest.raises(ValueError, match="tree size 129"):
        p = ctypes.c_void_p(16)
        L.tree_accept(129, p, p, p, p, p, 3, p, p, None)
    with pytest.raises(ValueError, match="mask_words"):
        p = ctypes.c_void_p(16)
        L.tree_accept(100, p, p, p, p, p, 1, p, p, None)
    with pytest.raises(ValueError, match="top=200"):
        p = ctypes.c_void_p(16)
        L.topk(p, 1, 1000, 200, p, p, None, 0, None)
    with pytest.raises(RuntimeError, match="outside the verify/draft path"):
        L.decode(1, 128, 0, 0, 0, 0, 0, 0)
    with pytest.raises(RuntimeError, match="no model"):
        L.load_model(b"lm_head.weight", 1)
    assert L.raw.cpmcu_tree_attention_workspace_bytes(60, 32, 2, 4156) > 0
    assert L.raw.cpmcu_head_workspace_bytes(60, 73448) > 0


def test_pybind_module_has_reference_names():
    """Names of src/entry.cu:510-534."""
    from cpm.cu_amd import C
    for name in ("init_base_model", "init_minicpm4_model", "init_w4a16_gptq_marlin_base_model",
                 "init_w4a16_gptq_marlin_minicpm4_model", "init_eagle_model", "init_minicpm4_eagle_model",
                 "init_w4a16_gm_spec_w4a16_gm_model", "init_hier_eagle_w4a16_gm_spec_w4a16_gm_model",
                 "init_hier_eagle_w4a16_gm_rot_spec_w4a16_gm_model", "init_storage", "load_model", "prefill",
                 "decode", "draft", "verify_and_fix", "print_perf_summary"):
        assert callable(getattr(C, name)), name
    with pytest.raises(RuntimeError, match="outside the verify/draft path"):
        C.decode(1, 128, 0, 0, 0, 0, 0, False)
    with pytest.raises(RuntimeError):
        C.init_minicpm4_model(0.9, 1, 1, 1, 1, 1, 1, 128, 1e-5, 0, 1, 1.0, 1.0, 1.0, 0, 0, 0, 0, False)
    with pytest.raises(RuntimeError, match="dtype"):
        C.init_base_model(0.5, 100, 1, 512, 1024, 32, 2, 128, 1e-5, 2, 2048, 1.0, 1.0, 1.0)
    with pytest.raises(ValueError, match="head_dim"):
        C.init_base_model(0.5, 100, 1, 512, 1024, 32, 2, 64, 1e-5, 0, 2048, 1.0, 1.0, 1.0)
