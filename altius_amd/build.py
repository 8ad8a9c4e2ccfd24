"""Builds altius_amd/libaltius_hip.so (HIP kernels + C ABI + C++ host session) for gfx950.

Usage: python -m altius_amd.build [--force]
"""
import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libaltius_hip.so")
MODULE_SRC_DIR = os.path.join(CSRC, "modules")  # stand-alone code objects, not linked into the library
MODULE_DIR = os.path.join(HERE, "modules")

ARCH = "gfx950"

COMMON_FLAGS = [
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wextra",
    "-Wno-unused-parameter",
    # The reference never contracts a*b+c; fused multiply-adds are written out
    # as __builtin_fmaf where the reference uses mul_add.
    "-ffp-contract=off",
]

DEVICE_FLAGS = [
    f"--offload-arch={ARCH}",
    # IEEE-correct fp32 division and sqrt (bit-exact Div / Sqrt / 1/sum).
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # No packed-fp32 instructions.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libaltius_hip.so")
    return exe


def sources():
    src = sorted(glob.glob(os.path.join(CSRC, "**", "*.hip"), recursive=True))
    src += sorted(glob.glob(os.path.join(CSRC, "**", "*.cpp"), recursive=True))
    return [s for s in src if not s.startswith(MODULE_SRC_DIR + os.sep)]


def module_path(name):
    """Path of the code object built from csrc/modules/<name>.hip."""
    return os.path.join(MODULE_DIR, name + ".hsaco")


def _compile_module(src, force):
    out = module_path(os.path.splitext(os.path.basename(src))[0])
    if not force and os.path.exists(out) and os.path.getmtime(out) >= os.path.getmtime(src):
        return out
    cmd = [hipcc(), "--genco"] + COMMON_FLAGS + DEVICE_FLAGS + [src, "-o", out]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc --genco failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    return out


def _obj_path(src):
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    return os.path.join(OBJ_DIR, rel + ".o")


def _deps_newer(obj):
    """True if any source or header is newer than obj."""
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    files = glob.glob(os.path.join(CSRC, "**", "*.h"), recursive=True)
    files += glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    files.append(os.path.abspath(__file__))
    return any(os.path.getmtime(f) > t for f in files)


def _compile(src, force):
    obj = _obj_path(src)
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= os.path.getmtime(src) and not _deps_newer(obj):
        return obj
    cmd = [hipcc()] + COMMON_FLAGS
    if src.endswith(".hip"):
        cmd += DEVICE_FLAGS
    cmd += ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    noise = ("packed-fp32-ops", "is not a recognized feature")
    warn = "\n".join(l for l in r.stderr.splitlines() if l.strip() and not any(n in l for n in noise))
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(force=False, jobs=None):
    """Compiles every source and links the shared library.  Returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    src = sources()
    jobs = jobs or min(8, os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), src))
        os.makedirs(MODULE_DIR, exist_ok=True)
        list(ex.map(lambda s: _compile_module(s, force), sorted(glob.glob(os.path.join(MODULE_SRC_DIR, "*.hip")))))
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
