"""Build libferrotensor_hip.so for gfx950 with hipcc (in-tree).

    python -m ferrotensor_amd.build            # rebuild everything
    python -m ferrotensor_amd.build --if-stale # only when a source is newer
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(HERE, "libferrotensor_hip.so")

SOURCES = ["ft_runtime.cpp", "ft_rowops.hip", "ft_gemm.hip", "ft_thin.hip", "ft_attention.hip", "ft_attention16.hip", "ft_step.cpp"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src):
    path = os.path.join(CSRC, src)
    obj = os.path.join(OBJ_DIR, src + ".o")
    cmd = ["hipcc", "-x", "hip", *FLAGS, "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return obj


def build(force=True, sources=None):
    srcs = [s for s in (sources or SOURCES) if os.path.exists(os.path.join(CSRC, s))]
    headers = [os.path.join(CSRC, "ft_common.h"), os.path.join(CSRC, "ft_thin.h"), os.path.join(CSRC, "ft_attention.h"), os.path.join(ROOT, "include", "ferrotensor_hip.h")]
    deps = [os.path.join(CSRC, s) for s in srcs] + headers
    if not force and not _stale(LIB, deps):
        return LIB
    os.makedirs(OBJ_DIR, exist_ok=True)
    todo = [s for s in srcs
            if force or _stale(os.path.join(OBJ_DIR, s + ".o"), [os.path.join(CSRC, s)] + headers)]
    with ThreadPoolExecutor(max_workers=min(6, max(1, len(todo)))) as ex:
        list(ex.map(_compile, todo))
    objs = [os.path.join(OBJ_DIR, s + ".o") for s in srcs]
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    return LIB


if __name__ == "__main__":
    print(build(force="--if-stale" not in sys.argv))
