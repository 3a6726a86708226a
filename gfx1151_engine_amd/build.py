"""Build libmi355moe.so (HIP, gfx950) in-tree with hipcc."""
import glob
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libmi355moe.so")
SOURCES = sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-result"]


def build(verbose=False, out=LIB, extra=()):
    """Compile every HIP source of the package into one shared library (always recompiles).
    out / extra: another output path and additional compiler flags (-D switches of experimental variants)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + list(extra) + ["-o", out] + SOURCES
    if verbose:
        print(" ".join(cmd))
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return out


if __name__ == "__main__":
    print(build(verbose=True))
