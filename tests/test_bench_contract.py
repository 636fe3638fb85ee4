"""Host-side contract of bench.py that needs no GPU: one GPU only, and the product path has no CPU fallback."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)


def test_product_sources_do_not_reach_into_the_oracle():
    """only tests, smoke() and bench.py's cpu_baseline leg may touch oracle/; the package never does"""
    pkg = os.path.join(ROOT, "llama.cpp_amd")
    for base, _, files in os.walk(pkg):
        if os.sep + "lib" in base:
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(base, f), errors="replace").read()
                assert "oracle/" not in text and "import orc" not in text and "oracle." not in text.replace("oracle.c:", ""), os.path.join(base, f)
