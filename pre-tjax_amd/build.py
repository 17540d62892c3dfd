"""Build recipe for libptj.so (gfx950 HIP kernels + C ABI).

Every ``csrc/*.hip`` file is compiled with hipcc for gfx950 and linked into
``libptj.so`` next to this file.  No GPU is needed to build.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "build")
LIB = os.path.join(HERE, "libptj.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wno-unused-command-line-argument",
         # packed-fp32 VALU forms are kept out of all device code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _fresh(src, obj):
    """True when `obj` is newer than `src` and every header beside it."""
    if not os.path.exists(obj):
        return False
    t = os.path.getmtime(obj)
    deps = [src, os.path.join(HERE, "..", "include", "ptj.h")]
    deps += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    return all(os.path.getmtime(d) < t for d in deps)


def _compile(src, only_changed=False):
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
    if only_changed and _fresh(src, obj):
        return obj, ""
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=False, jobs=None, only_changed=False):
    """Compile and link.  `only_changed` skips sources whose object file is newer than the
    source and the headers (a developer convenience; the default compiles everything)."""
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))
    jobs = jobs or min(8, len(srcs))
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        results = list(ex.map(lambda src: _compile(src, only_changed), srcs))
    for obj, err in results:
        if verbose and err.strip():
            print(err, file=sys.stderr)
    objs = [o for o, _ in results]
    r = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-o", LIB] + objs, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, only_changed="--changed" in sys.argv[1:]))
