"""Build of the HIP kernels under csrc/ into one shared library for gfx950.

The library's file name carries a hash of the sources and flags, so a library
that does not match the sources is never loaded: after a change the name
changes and the library is built again at the next load.  Objects are compiled
in parallel, one hipcc process per source.
"""
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(_PKG, "csrc")
LIB_DIR = os.path.join(_PKG, "lib")
ARCH = "gfx950"
HIPCC_FLAGS = [
    "--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
LINK_LIBS = ["-lhipblaslt"]          # the library matrix product for many rows (matmul_library.hip)


class BuildError(RuntimeError):
    pass


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def source_hash() -> str:
    h = hashlib.sha1()
    h.update(" ".join(HIPCC_FLAGS + LINK_LIBS).encode())
    for f in sorted(os.listdir(CSRC)):
        if f.endswith((".hip", ".h")):
            h.update(f.encode())
            with open(os.path.join(CSRC, f), "rb") as fh:
                h.update(fh.read())
    return h.hexdigest()[:12]


def library_name() -> str:
    return "libinfinicore_infer_hip-%s.so" % source_hash()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found: the HIP kernels cannot be built (looked at $HIPCC, PATH, /opt/rocm/bin)")


def _writable_dir(preferred: str) -> str:
    try:
        os.makedirs(preferred, exist_ok=True)
        probe = os.path.join(preferred, ".probe-%d" % os.getpid())
        with open(probe, "w"):
            pass
        os.remove(probe)
        return preferred
    except OSError:
        d = os.path.join(tempfile.gettempdir(), "infinicore_infer_amd-%d" % os.getuid())
        os.makedirs(d, exist_ok=True)
        return d


def find_library():
    """Path of a built library that matches the sources, or None."""
    name = library_name()
    for d in (LIB_DIR, os.path.join(tempfile.gettempdir(), "infinicore_infer_amd-%d" % os.getuid())):
        p = os.path.join(d, name)
        if os.path.isfile(p):
            return p
    return None


def build(force: bool = False, verbose: bool = True) -> str:
    """Compile every .hip source and link the library.  Returns its path."""
    if not force:
        p = find_library()
        if p:
            return p
    hipcc = _hipcc()
    out_dir = _writable_dir(LIB_DIR)
    obj_dir = _writable_dir(os.path.join(CSRC, "_build"))
    name = library_name()
    srcs = sources()
    t0 = time.time()

    def say(msg):
        if verbose:
            print("[infinicore_infer_amd build] " + msg, file=sys.stderr, flush=True)

    say("compiling %d HIP sources for %s with %s" % (len(srcs), ARCH, hipcc))

    def compile_one(src):
        obj = os.path.join(obj_dir, src[:-4] + "-" + name[-15:-3] + ".o")
        cmd = [hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise BuildError("hipcc failed on %s:\n%s" % (src, r.stdout))
        say("  %s done (%.0f s)" % (src, time.time() - t0))
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
    with ThreadPoolExecutor(max_workers=workers) as ex:
        objs = list(ex.map(compile_one, srcs))
    tmp = os.path.join(out_dir, ".%s.%d.tmp" % (name, os.getpid()))
    cmd = [hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs + LINK_LIBS
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise BuildError("link failed:\n%s" % r.stdout)
    final = os.path.join(out_dir, name)
    os.replace(tmp, final)
    for f in os.listdir(out_dir):          # drop libraries of older sources
        if f.startswith("libinfinicore_infer_hip-") and f != name:
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    for f in os.listdir(obj_dir):
        if f.endswith(".o") and name[-15:-3] not in f:
            try:
                os.remove(os.path.join(obj_dir, f))
            except OSError:
                pass
    say("linked %s (%.0f s)" % (final, time.time() - t0))
    return final


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
