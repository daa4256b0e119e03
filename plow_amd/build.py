"""Builds the operator library ``plow_amd/libplow_moe_gfx950.so`` from ``plow_amd/csrc`` with hipcc.

gfx950 (MI355X, CDNA4) only. hipcc cross-compiles without a GPU, so this runs anywhere the ROCm
toolchain is installed. ``python -m plow_amd.build`` rebuilds unconditionally.
"""
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libplow_moe_gfx950.so")
# the device code object plowrt loads by this name (plow crates/plowrt/src/exec/amd.rs:11718-11760)
ELF = os.path.join(HERE, "moe_fp8_pf_gfx950.elf")
ELF_COMBINE = os.path.join(HERE, "moe_combine_gfx950.elf")   # amd.rs:11666-11716
ELF_DEC = os.path.join(HERE, "moe_w8a8_dec_gfx950.elf")      # amd.rs:10799-10852
ELF_ROUTER = os.path.join(HERE, "router_decode_gfx950.elf")  # amd.rs:10755-10800

COMMON = ["--offload-arch=gfx950", "-O3", *os.environ.get("PLOW_MOE_EXTRA_FLAGS", "").split(), "-std=c++17", "-fPIC", "-fno-fast-math",
          # packed-FP32 VALU forms are kept out of every kernel
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# Translation units whose floating-point results must match the CPU reference bit for bit are built
# without multiply-add contraction.
SOURCES = {
    "route.hip": ["-ffp-contract=off"],
    "quant.hip": ["-ffp-contract=off"],
    "experts_w8a8.hip": [],
    "experts_a16.hip": [],
    "experts_gemv.hip": [],
    "experts_w8a8_tiled.hip": [],
    "api.hip": [],
    "device.hip": [],
}


def _compile(src, extra):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = ["hipcc", *COMMON, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return obj, err


def _code_object(src="plowrt_obj.hip", out=None, extra=()):
    """One raw (unbundled) gfx950 ELF with plow's kernel names, built the way plow builds its own
    (hipcc -O3, device only; plow runtime/cmake/hipcc_hsaco.sh)."""
    out = out or ELF
    cmd = ["hipcc", *[f for f in COMMON if f != "-fPIC"], *extra, "--cuda-device-only", "--no-gpu-bundle-output",
           "-o", out, os.path.join(CSRC, src)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    return out, err


def build(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=8) as ex:
        elfs = [ex.submit(_code_object), ex.submit(_code_object, "plowrt_combine_obj.hip", ELF_COMBINE, ("-ffp-contract=off",)),
                ex.submit(_code_object, "plowrt_dec_obj.hip", ELF_DEC),
                ex.submit(_code_object, "plowrt_router_obj.hip", ELF_ROUTER, ("-ffp-contract=off",))]
        results = list(ex.map(lambda kv: _compile(*kv), SOURCES.items()))
        for f in elfs:
            _, elf_err = f.result()
            if verbose and elf_err.strip():
                print(elf_err, file=sys.stderr)
    objs = [o for o, _ in results]
    for _, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
        print("built", ELF)
        print("built", ELF_COMBINE)
        print("built", ELF_DEC)
        print("built", ELF_ROUTER)
    return LIB


if __name__ == "__main__":
    build()
