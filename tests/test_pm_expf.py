"""The exponential the router kernels use must equal the C library's expf, which the CPU reference
calls, on every input. The host build of the same header is compared over a strided sweep of all
bit patterns here (stride 1 = exhaustive: PLOW_EXPF_STRIDE=1, about 10 s on 8 cores)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_pm_expf_equals_libm_expf(tmp_path):
    exe = str(tmp_path / "pm_expf_check")
    subprocess.check_call(["gcc", "-O2", "-ffp-contract=off", "-o", exe,
                           os.path.join(ROOT, "tests", "pm_expf_check.c"), "-lm", "-lpthread"])
    stride = os.environ.get("PLOW_EXPF_STRIDE", "7")
    out = subprocess.run([exe, stride], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "0", out.stdout
