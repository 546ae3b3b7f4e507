"""Builds libsfno_spectral.so (HIP, gfx950) in-tree next to the Python package.

    python modulus-makani_amd/build.py            # compile what is out of date
    python modulus-makani_amd/build.py --force    # compile everything

Every source is compiled to an object under build/ (in parallel), then linked.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
OUT = os.path.join(HERE, "makani_amd", "libsfno_spectral.so")
SOURCES = ["tables.cpp", "capi.cpp", "dhconv.hip", "dhconv_f16.hip", "dhconv_wgrad.hip", "pointwise.hip", "pointwise_wgrad.hip", "diagonal.hip", "degree_power.hip", "legendre_fold.hip", "legendre_f16.hip", "fft.hip",
           "fft_fast.hip", "layout.hip", "static_scratch.hip"]
HEADERS = [os.path.join(CSRC, "sfno_internal.h"), os.path.join(CSRC, "dhconv_map.h"), os.path.join(ROOT, "include", "sfno_spectral.h")]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def flags():
    return [
        "-O3", "-std=c++17", "--offload-arch=gfx950",
        # packed fp32 VALU forms are kept out of the generated code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-fPIC", "-Wno-unused-command-line-argument",
        "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    ]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + log)
    if verbose and log.strip():
        print(log)


def compile_objects(csrc=CSRC, objdir=OBJ, force=True, verbose=True, sources=SOURCES, extra=()):
    """Compiles `sources` from `csrc` into `objdir`; returns the object paths."""
    os.makedirs(objdir, exist_ok=True)
    newest_header = max(os.path.getmtime(h) for h in HEADERS)
    jobs, objs = [], []
    for s in sources:
        src, obj = os.path.join(csrc, s), os.path.join(objdir, s + ".o")
        objs.append(obj)
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), newest_header):
            jobs.append([hipcc()] + flags() + list(extra) + ["-c", src, "-o", obj])
    workers = max(1, min(len(jobs), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    with ThreadPoolExecutor(workers) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    return objs


def link(objs, out=OUT, verbose=True):
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs + ["-lpthread"], verbose)
    return out


def up_to_date():
    if not os.path.exists(OUT):
        return False
    t = os.path.getmtime(OUT)
    deps = [os.path.join(CSRC, s) for s in SOURCES] + HEADERS
    return all(os.path.getmtime(d) <= t for d in deps)


def build(force=True, verbose=True):
    if not force and up_to_date():
        return OUT
    return link(compile_objects(force=force, verbose=verbose), verbose=verbose)


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    print("built", OUT)
