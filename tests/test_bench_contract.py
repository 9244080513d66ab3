"""bench.py's command-line contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode == 2
    assert "single-GPU" in p.stderr and p.stdout.strip() == ""


def test_recorded_traffic_covers_the_headline_ops():
    entries = {}
    with open(os.path.join(ROOT, "profiles", "hbm_traffic.txt")) as f:
        for line in f:
            if "=" in line and not line.startswith("#"):
                k, v = line.split("=")
                entries[k.strip()] = int(v)
    n = 1 << 28
    # measured HBM bytes per launch stay within 2% of the algorithmic bytes where the
    # kernel has to touch everything
    for op, per_elem in (("add", 12), ("gelu", 8), ("silu", 8), ("relu", 8), ("eq", 9)):
        got = entries[f"{op}@2^28"]
        assert abs(got - per_elem * n) <= 0.02 * per_elem * n, (op, got)
    assert entries["masked_select_p0.50@2^28"] <= 1.02 * (5 * n + 4 * (n // 2))


def test_recorded_traffic_is_not_older_than_the_kernels():
    # roofline.traffic in bench.py's line is a recorded figure; the file names the commit it
    # was measured at, and that commit must contain the last change to the kernel sources
    path = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    commit = None
    with open(path) as f:
        for line in f:
            if line.startswith("# measured at commit"):
                commit = line.split()[-1]
    assert commit, "profiles/hbm_traffic.txt does not say which commit it was measured at"

    def git(*args):
        return subprocess.run(["git", "-C", ROOT, *args], capture_output=True, text=True, timeout=60)

    if git("rev-parse", "--git-dir").returncode != 0:
        import pytest
        pytest.skip("not a git checkout")
    assert git("cat-file", "-e", commit + "^{commit}").returncode == 0, f"unknown commit {commit}"
    last = git("log", "-1", "--format=%H", "--", "torch-webgpu_amd/csrc/hip").stdout.strip()
    assert last, "no commit touches the kernel sources?"
    assert git("merge-base", "--is-ancestor", last, commit).returncode == 0, (
        f"profiles/hbm_traffic.txt was measured at {commit}, before the last change to "
        f"torch-webgpu_amd/csrc/hip ({last[:12]}): run the counter profiles again")
