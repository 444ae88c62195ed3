"""bench.py's command line: the part that needs no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def test_the_survey_tools_print_their_usage_without_a_gpu():
    """`python -m cpm.cu_amd.sweep` / `.timeline` with no operator named: the usage text, exit status 2, nothing touches the GPU."""
    import subprocess
    import sys
    for mod in ("cpm.cu_amd.sweep", "cpm.cu_amd.timeline"):
        r = subprocess.run([sys.executable, "-m", mod], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
        assert r.returncode == 2 and "python -m " + mod in r.stdout, r.stdout


def test_an_unknown_workload_is_refused_before_the_gpu_is_touched():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "nope"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 1 and "unknown workload" in res.stderr and res.stdout.strip() == "", (res.returncode, res.stderr)
