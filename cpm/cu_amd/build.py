"""Builds libcpmcu_amd.so (HIP kernels + C-ABI, gfx950) and the pybind11 module ``C`` in-tree.

    python -m cpm.cu_amd.build [--force]

hipcc cross-compiles for gfx950 without a GPU.  Every translation unit is compiled on each call of
``build_all(force=True)``; without ``force`` only stale objects are rebuilt.
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(os.path.dirname(HERE))
INCLUDE = os.path.join(ROOT, "include")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libcpmcu_amd.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

HIP_SOURCES = ["runtime.hip", "tree_attention.hip", "lm_head.hip", "topk.hip", "tree_accept.hip", "draft_tree.hip"]
TIMELINE_SOURCES = ["tree_attention.hip", "lm_head.hip", "topk.hip"]  # kernels with optional wall-clock stamps (csrc/timeline.h)
TIMELINE_LIB_PATH = os.path.join(HERE, "libcpmcu_amd_timeline.so")  # loaded only by `python -m cpm.cu_amd.timeline`
HEADERS = sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))

# packed fp32 VALU ops stay off for every device translation unit
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes", f"-I{INCLUDE}",
]


def pybind_module_path():
    return os.path.join(HERE, "C" + sysconfig.get_config_var("EXT_SUFFIX"))


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _run(cmd):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_all(force=False, verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    common_deps = [os.path.join(CSRC, h) for h in HEADERS] + [os.path.join(INCLUDE, "cpmcu_amd.h")]
    jobs = []
    objs = []
    for src in HIP_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        objs.append(o)
        if force or _stale(o, [s] + common_deps):
            jobs.append([HIPCC] + HIP_FLAGS + ["-c", s, "-o", o])
    # the same two kernels files once more with wall-clock stamps compiled in (csrc/timeline.h), for a library of their own
    tl_objs = []
    for src in HIP_SOURCES:
        if src in TIMELINE_SOURCES:
            s = os.path.join(CSRC, src)
            o = os.path.join(OBJ_DIR, src.replace(".hip", "_timeline.o"))
            tl_objs.append(o)
            if force or _stale(o, [s] + common_deps):
                jobs.append([HIPCC] + HIP_FLAGS + ["-DCPMCU_TIMELINE", "-c", s, "-o", o])
        else:
            tl_objs.append(os.path.join(OBJ_DIR, src.replace(".hip", ".o")))
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for out in ex.map(_run, jobs):
            if verbose and out.strip():
                print(out)
    if force or jobs or _stale(LIB_PATH, objs):
        _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH] + objs)
    if force or jobs or _stale(TIMELINE_LIB_PATH, tl_objs):
        _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", TIMELINE_LIB_PATH] + tl_objs)
    # pybind11 module `C`: the reference's entry-point names over the C-ABI
    import pybind11
    mod = pybind_module_path()
    entry = os.path.join(CSRC, "pybind_entry.cpp")
    if os.path.exists(entry) and (force or _stale(mod, [entry, LIB_PATH] + common_deps)):
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
              f"-I{pybind11.get_include()}", f"-I{sysconfig.get_paths()['include']}", f"-I{INCLUDE}",
              entry, "-o", mod, f"-L{HERE}", "-lcpmcu_amd", "-Wl,-rpath,$ORIGIN"])
    # bench.py's measurement helper: its own small library, outside the product
    probe_src = os.path.join(ROOT, "bench_probes", "mfma_rate_probe.hip")
    probe_lib = os.path.join(ROOT, "bench_probes", "libbench_probes.so")
    if os.path.exists(probe_src) and (force or _stale(probe_lib, [probe_src])):
        _run([HIPCC, f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared", "-Xclang", "-target-feature", "-Xclang",
              "-packed-fp32-ops", probe_src, "-o", probe_lib])
    return LIB_PATH


if __name__ == "__main__":
    print(build_all(force="--force" in sys.argv, verbose=True))
