"""Checks on the repository itself that need no GPU: bench.py's command line, the profile
summaries it reads, and the rule that the product never reaches into the test oracle."""
import glob
import importlib.util
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench_module():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)      # defines functions and constants; main() is not run
    return mod


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and "--gpus must be 1" in r.stderr
    assert r.stdout.strip() == ""      # no JSON line for a run that did not happen


def test_bench_rejects_unknown_section():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--section", "nonsense"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode != 0 and "nonsense" in r.stderr


def test_roofline_traffic_comes_from_the_committed_profile():
    bench = _bench_module()
    got = bench.measured_traffic("silu_and_mul_kernel")
    alg = bench.BYTES["silu_and_mul"]
    assert got is not None and 0.98 * alg <= got <= 1.10 * alg
    assert bench.measured_traffic("no_such_kernel") is None
    assert os.path.relpath(bench.TRAFFIC_PROFILE, ROOT).startswith("profiles" + os.sep)


def test_algorithmic_bytes_of_the_headline_ops():
    """Closed forms of the compulsory traffic at the 2304-token Llama-3-8B batch (bf16)."""
    bench = _bench_module()
    T, H, D, nq, nkv, dff = 2304, 4096, 128, 32, 8, 14336
    assert bench.BYTES["rms_norm"] == 2 * T * H * 2 + H * 2 == 37_756_928
    assert bench.BYTES["fused_add_rms_norm"] == 4 * T * H * 2 + H * 2 == 75_505_664
    assert bench.BYTES["silu_and_mul"] == 3 * T * dff * 2 == 198_180_864
    assert bench.BYTES["rotary_embedding"] == 2 * T * (nq + nkv) * D * 2 + T * 8 + T * D * 2 == 47_794_176
    assert bench.BYTES["append_paged_kv_cache"] == 4 * T * nkv * D * 2 + T * 16 == 18_911_232


def test_profile_summaries_name_committed_commands_only():
    files = sorted(glob.glob(os.path.join(ROOT, "profiles", "*")))
    assert files, "profiles/ holds the rocprofv3 summaries"
    for path in files:
        assert path.endswith((".txt", ".md")), path
        assert os.path.getsize(path) < 64 * 1024, path
        text = open(path).read()
        assert "rocprofv3" in text, path + " gives no command"
        assert "_work" not in text, path
        for script in re.findall(r"python3?\s+(\S+\.py)", text):
            rel = script.replace("$R/", "").replace("$GRAFT_REPO_ROOT/", "")
            assert os.path.exists(os.path.join(ROOT, rel)), "%s runs %s, which is not in the tree" % (path, script)


def test_product_never_touches_the_oracle():
    """Only tests/, __graft_entry__.smoke() and bench.py's CPU-baseline leg may use oracle/."""
    pkg = os.path.join(ROOT, "sarathi-serve_amd")
    offenders = []
    for base, dirs, names in os.walk(pkg):
        dirs[:] = [d for d in dirs if d not in ("build", "__pycache__")]
        for n in names:
            if n.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(base, n), errors="replace").read()
                if re.search(r"\boracle\b", text):
                    offenders.append(os.path.join(base, n))
    assert offenders == []
    for n in ("include/sarathi_ops.h",):
        assert "oracle" not in open(os.path.join(ROOT, n)).read()
