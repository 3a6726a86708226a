"""Build libmi355moe.so (HIP, gfx950) in-tree with hipcc: one object per source, compiled side by side, then linked."""
import glob
import os
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libmi355moe.so")
# the same sources with the timing hooks compiled in (-DMOE_TIMING_HOOKS): loaded by bench.py only, to time one
# launch of the decode path as the difference of two step loops
LIB_TIMING = os.path.join(HERE, "libmi355moe_timing.so")
SOURCES = sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))
CFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]
FLAGS = CFLAGS + ["-shared"]


def _clean(text):
    return "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l and "warning generated" not in l)


def build(verbose=False, out=LIB, extra=(), jobs=None):
    """Compile every HIP source of the package into one shared library (always recompiles).
    out / extra: another output path and additional compiler flags (-D switches of variants)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    jobs = jobs or min(8, os.cpu_count() or 1, len(SOURCES))
    tmp = tempfile.mkdtemp(prefix="mi355moe_build_")
    log = []
    try:
        def one(src):
            obj = os.path.join(tmp, os.path.basename(src) + ".o")
            cmd = [hipcc] + CFLAGS + list(extra) + ["-c", "-o", obj, src]
            if verbose:
                print(" ".join(cmd))
            r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            return obj, r.returncode, _clean(r.stdout)

        with ThreadPoolExecutor(max_workers=jobs) as ex:
            results = list(ex.map(one, SOURCES))
        failed = [t for _, rc, t in results if rc != 0]
        if failed:
            raise RuntimeError("hipcc failed:\n" + "\n".join(failed))
        log = [t for _, _, t in results if t.strip()]
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fvisibility=hidden", "-o", out + ".tmp"] + [o for o, _, _ in results]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + _clean(r.stdout))
        os.replace(out + ".tmp", out)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    text = "\n".join(log)
    if verbose and text.strip():
        print(text)
    return text


def build_all(verbose=False):
    """The library and its timing twin."""
    build(verbose=verbose)
    build(verbose=verbose, out=LIB_TIMING, extra=("-DMOE_TIMING_HOOKS=1",))


if __name__ == "__main__":
    build_all(verbose=True)
