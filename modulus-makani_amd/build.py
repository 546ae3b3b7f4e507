"""Builds libsfno_spectral.so (HIP, gfx950) in-tree next to the Python package.

    python modulus-makani_amd/build.py            # compile only if sources are newer
    python modulus-makani_amd/build.py --force    # always compile
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "makani_amd", "libsfno_spectral.so")
SOURCES = ["tables.cpp", "capi.cpp", "dhconv.hip", "dhconv_wgrad.hip", "pointwise.hip", "diagonal.hip", "degree_power.hip", "legendre_fold.hip", "fft.hip", "fft_fast.hip", "layout.hip", "static_scratch.hip"]
HEADERS = [os.path.join(CSRC, "sfno_internal.h"), os.path.join(ROOT, "include", "sfno_spectral.h")]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def command():
    return [
        hipcc(), "-O3", "-std=c++17", "--offload-arch=gfx950",
        # packed fp32 VALU forms are kept out of the generated code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-fPIC", "-shared", "-Wno-unused-command-line-argument",
        "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
        "-o", OUT,
    ] + [os.path.join(CSRC, s) for s in SOURCES] + ["-lpthread"]


def up_to_date():
    if not os.path.exists(OUT):
        return False
    t = os.path.getmtime(OUT)
    deps = [os.path.join(CSRC, s) for s in SOURCES] + HEADERS
    return all(os.path.getmtime(d) <= t for d in deps)


def build(force=True, verbose=True):
    if not force and up_to_date():
        return OUT
    cmd = command()
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return OUT


if __name__ == "__main__":
    build(force="--force" in sys.argv or True)
    print("built", OUT)
