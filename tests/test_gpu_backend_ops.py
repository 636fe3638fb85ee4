"""Drop-in check: the reference's own acceptance harness, tests/test-backend-ops.cpp, built
unmodified from the reference sources (oracle/Makefile), loads libggml-mi355.so through
GGML_BACKEND_PATH and compares every operator the backend claims against the reference CPU
backend (NMSE thresholds of the harness: 5e-4 for MUL_MAT / MUL_MAT_ID / FLASH_ATTN_EXT,
1e-7 default).  Cases the backend declines in supports_op print "not supported"."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "oracle", "_ref", "test-backend-ops")
PLUGIN = os.path.join(ROOT, "llama.cpp_amd", "lib", "libggml-mi355.so")

OPS = ["MUL_MAT", "MUL_MAT_ID", "FLASH_ATTN_EXT", "RMS_NORM", "ADD", "MUL", "DIV", "SUB", "ROPE", "SOFT_MAX", "CPY", "CONT", "DUP",
       "GET_ROWS", "SCALE", "SUM_ROWS", "ARGSORT", "SILU", "GELU", "RELU", "TANH", "SIGMOID", "EXP", "NEG", "ABS"]


def _run(op, out_dir):
    env = dict(os.environ, GGML_BACKEND_PATH=PLUGIN)
    r = subprocess.run([HARNESS, "test", "-b", "MI355X0", "-o", op], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                       text=True, timeout=600, cwd=os.path.dirname(HARNESS))
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "backend_ops_%s.log" % op), "w") as f:
        f.write(r.stdout)
    return r


@pytest.mark.parametrize("op", OPS)
def test_backend_ops(dev, op):
    if not (os.path.exists(HARNESS) and os.path.exists(PLUGIN)):
        pytest.skip("reference harness or plug-in not built (needs the llama.cpp tree at build time)")
    r = _run(op, os.path.join(ROOT, "gpurun_out", "backend_ops"))
    text = re.sub(r"\x1b\[[0-9;]*m", "", r.stdout)
    assert "Backend 2/2: MI355X0" in text or "MI355X0" in text, "plug-in was not loaded:\n" + text[-2000:]
    m = re.search(r"(\d+)/(\d+) tests passed", text)
    assert m, text[-2000:]
    n_ok, n_all = int(m.group(1)), int(m.group(2))
    n_run = len(re.findall(r": OK$", text, flags=re.M))
    failed = [l for l in text.splitlines() if l.rstrip().endswith("FAIL")]
    assert r.returncode == 0 and n_ok == n_all and not failed, "\n".join(failed[:20]) + "\n" + text[-1500:]
    # the operators on the llama hot path must actually execute here, not be declined
    assert n_run > 0, "every %s case was declined by supports_op" % op
