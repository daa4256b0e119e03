"""The exponential the router kernels use must equal the C library's expf, which the CPU reference
calls, on every input. The host build of the same header is compared over a strided sweep of all
bit patterns here (stride 1 = exhaustive: PLOW_EXPF_STRIDE=1, about 10 s on 8 cores)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_pm_log1pf_equals_libm_log1pf_on_the_unit_interval(tmp_path):
    """Every float in [0, 1] (the range of expf(-|l|), the argument of the router's sqrt-softplus transform)."""
    exe = str(tmp_path / "pm_log1pf_check")
    subprocess.check_call(["gcc", "-O2", "-ffp-contract=off", "-o", exe,
                           os.path.join(ROOT, "tests", "pm_log1pf_check.c"), "-lm", "-lpthread"])
    out = subprocess.run([exe, "1"], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "0", out.stdout + out.stderr


def test_pm_expf_equals_libm_expf(tmp_path):
    exe = str(tmp_path / "pm_expf_check")
    subprocess.check_call(["gcc", "-O2", "-ffp-contract=off", "-o", exe,
                           os.path.join(ROOT, "tests", "pm_expf_check.c"), "-lm", "-lpthread"])
    stride = os.environ.get("PLOW_EXPF_STRIDE", "7")
    out = subprocess.run([exe, stride], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "0", out.stdout
