"""Builds libratchet_hip.so (gfx950 only) from ratchet_amd/csrc/*.hip with hipcc, in-tree.

    python -m ratchet_amd.build            # build if sources are newer than the library
    python -m ratchet_amd.build --force    # rebuild everything

Flags that matter for results:
  -ffp-contract=off   every float operation rounds on its own, as in ratchet's Rust CPU code (hipcc would
                      otherwise fuse a*b+c into v_fma / v_fmac and change the bits)
  -Xclang -target-feature -Xclang -packed-fp32-ops   no packed-fp32 instructions are generated
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libratchet_hip.so")
HOST_DIR = os.path.join(CSRC, "host")
HOST_LIB_PATH = os.path.join(HERE, "libratchet_host.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def headers():
    return sorted(glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(HERE, "..", "include", "*.h")))


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    if force or _newer(obj, [src] + headers()):
        cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr[-8000:]))
        warn = [l for l in r.stderr.splitlines() if "warning" in l and "packed-fp32-ops" not in l]
        if warn:
            sys.stderr.write("\n".join(warn[:20]) + "\n")
    return obj


def build_host(force=False, sanitize=False):
    """libratchet_host.so: the C++ mirror of ratchet's lazy Tensor API (host code only, g++), linked against
    libratchet_hip.so in the same directory.  sanitize=True builds the same sources with AddressSanitizer and
    UndefinedBehaviorSanitizer into csrc/build/asan/ instead (CPU only; loaded by tests/test_sanitizers.py)."""
    srcs = sorted(glob.glob(os.path.join(HOST_DIR, "*.cpp")))
    deps = srcs + glob.glob(os.path.join(HOST_DIR, "*.hpp")) + headers() + [LIB_PATH]
    if sanitize:
        out_dir = os.path.join(OBJ_DIR, "asan")
        os.makedirs(out_dir, exist_ok=True)
        out = os.path.join(out_dir, "libratchet_host.so")
        if force or _newer(out, deps):
            cmd = [os.environ.get("CXX", "g++"), "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-fsanitize=address,undefined",
                   "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-o", out] + srcs + [
                "-L" + HERE, "-lratchet_hip", "-Wl,-rpath," + HERE]
            r = subprocess.run(cmd, capture_output=True, text=True)
            if r.returncode != 0:
                raise RuntimeError("sanitizer build of the host library failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-8000:]))
        return out
    if force or _newer(HOST_LIB_PATH, deps):
        cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-o", HOST_LIB_PATH] + srcs + [
            "-L" + HERE, "-lratchet_hip", "-Wl,-rpath,$ORIGIN"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("host library build failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-8000:]))
        if r.stderr.strip():
            sys.stderr.write(r.stderr[-4000:])
    return HOST_LIB_PATH


STAMP_PATH = os.path.join(HERE, "built_from.txt")              # beside the library: it travels with it


def _stamp():
    """Record beside the objects which commit the library was linked from (and whether the kernel sources differed from
    it), so that a run on a machine that received the tree without its history can still say what it measured."""
    root = os.path.dirname(HERE)
    try:
        head = subprocess.run(["git", "-C", root, "rev-parse", "--short=12", "HEAD"], capture_output=True, text=True, timeout=20)
        dirty = subprocess.run(["git", "-C", root, "status", "--porcelain", "--", "ratchet_amd/csrc", "include"],
                               capture_output=True, text=True, timeout=20)
        if head.returncode != 0:
            return
        text = head.stdout.strip() + (" + uncommitted changes to the sources" if dirty.stdout.strip() else "")
    except (OSError, subprocess.SubprocessError):
        return
    with open(STAMP_PATH, "w") as f:
        f.write(text + "\n")


def built_from():
    """what _stamp() wrote at the last link, or None"""
    try:
        return open(STAMP_PATH).read().strip() or None
    except OSError:
        return None


def build(force=False, jobs=4):
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), sources()))
    if force or _newer(LIB_PATH, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-8000:]))
        _stamp()
    build_host(force)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
