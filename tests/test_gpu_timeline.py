"""The timeline tool (python -m cpm.cu_amd.timeline) on the stamped build of the kernels: it runs in a process of its own
-- it swaps the library under cpm.cu_amd.lib -- and what it prints must be a consistent sequence of stamps."""
import os
import re
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    res = subprocess.run([sys.executable, "-m", "cpm.cu_amd.timeline"] + list(args), cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True, timeout=300)
    assert res.returncode == 0, res.stdout
    return res.stdout


def _medians(out, names):
    vals = []
    for name in names:
        m = re.search(r"^\s+%s\s+min\s+([\d.]+)\s+median\s+([\d.]+)" % re.escape(name), out, flags=re.M)
        assert m, "no line for %r in:\n%s" % (name, out)
        vals.append(float(m.group(2)))
    return vals


def test_attention_timeline_is_ordered(gpu):
    out = _run("attention", "4096")
    v = _medians(out, ["start", "K loop entered", "K loop left", "KV groups merged", "partials issued", "partials acknowledged",
                       "all splits of the unit arrived", "end (own share merged, output stored)"])
    assert v == sorted(v) and 5.0 < v[-1] < 60.0, out
    assert "256 workgroups recorded" in out


def test_frspec_timeline_covers_both_forms(gpu):
    out = _run("frspec")
    assert "topk_row_kernel<true>" in out and "frspec_head_topk_kernel<1,512>" in out
    assert len(re.findall(r"finisher of row \d+:", out)) == 10, out
