"""Builds the gfx950 kernel library with hipcc (no torch headers, no pybind).

`library_path()` returns the built library, compiling it first if there is
none or if the one there was built from other sources (a digest of the .hip
and .h files and of the compiler flags is kept beside the library);
`build(force=True)` always compiles.  The library is placed in-tree
(`yalm_amd/lib/`); if the tree cannot be written, in a per-user folder under
the system's temporary directory.
"""
import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libyalm_hip.so"
ARCH = "gfx950"
# packed float32 operations are switched off for every device compile
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def sources():
    return sorted(f for f in os.listdir(HERE) if f.endswith(".hip"))


def sources_digest():
    """A digest of everything the library is built from: the .hip and .h files of this folder and the flags."""
    h = hashlib.sha256(" ".join(FLAGS).encode())
    for name in sorted(f for f in os.listdir(HERE) if f.endswith((".hip", ".h"))):
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _built_from(lib):
    """The digest recorded beside a built library, or None."""
    try:
        with open(lib + ".sources") as f:
            return f.read().strip()
    except OSError:
        return None


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found: the kernel library of yalm_amd cannot be built")


def _writable_dir():
    in_tree = os.path.join(os.path.dirname(HERE), "lib")
    try:
        os.makedirs(in_tree, exist_ok=True)
        probe = os.path.join(in_tree, ".probe_%d" % os.getpid())
        with open(probe, "w"):
            pass
        os.remove(probe)
        return in_tree
    except OSError:
        d = os.path.join(tempfile.gettempdir(), "yalm_amd_lib_%d" % os.getuid())
        os.makedirs(d, exist_ok=True)
        return d


def _candidates():
    return [os.path.join(os.path.dirname(HERE), "lib", LIB_NAME),
            os.path.join(tempfile.gettempdir(), "yalm_amd_lib_%d" % os.getuid(), LIB_NAME)]


def _say(msg):
    print("[yalm_amd build] " + msg, file=sys.stderr, flush=True)


def _compile_one(hipcc, src, obj):
    cmd = [hipcc] + FLAGS + ["-c", os.path.join(HERE, src), "-o", obj]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "packed-fp32-ops" not in l)
    return src, p.returncode, err


def build(force=True, jobs=None):
    """Compiles every .hip file of this folder and links the library."""
    digest = sources_digest()
    if not force:
        stale = []
        for c in _candidates():
            if os.path.exists(c):
                if _built_from(c) == digest:
                    return c
                stale.append(c)
        if stale:
            _say("%s was built from other sources than the ones here: building again" % stale[0])
    hipcc = _hipcc()
    out_dir = _writable_dir()
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), 8)
    t0 = time.time()
    _say("compiling %d files for %s into %s" % (len(srcs), ARCH, out_dir))
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futs = []
        for s in sorted(srcs, key=lambda f: -os.path.getsize(os.path.join(HERE, f))):     # the longest compilations first
            obj = os.path.join(obj_dir, s[:-4] + ".o")
            objs.append(obj)
            futs.append(pool.submit(_compile_one, hipcc, s, obj))
        pending = set(futs)
        while pending:
            done, pending = concurrent.futures.wait(pending, timeout=10, return_when=concurrent.futures.FIRST_COMPLETED)
            for f in done:
                src, rc, err = f.result()
                if rc != 0:
                    raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
                _say("compiled %s (%.0f s)" % (src, time.time() - t0))
            if pending and not done:
                _say("still compiling, %d files to go (%.0f s)" % (len(pending), time.time() - t0))
    tmp = os.path.join(out_dir, LIB_NAME + ".tmp%d" % os.getpid())
    p = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs,
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if p.returncode != 0:
        raise RuntimeError("linking the kernel library failed:\n" + p.stderr)
    lib = os.path.join(out_dir, LIB_NAME)
    os.replace(tmp, lib)
    with open(lib + ".sources.tmp%d" % os.getpid(), "w") as f:
        f.write(digest + "\n")
    os.replace(lib + ".sources.tmp%d" % os.getpid(), lib + ".sources")
    shutil.rmtree(obj_dir, ignore_errors=True)
    _say("built %s in %.0f s" % (lib, time.time() - t0))
    return lib


def build_kernel_bench():
    """Compiles kernel_bench.cpp (single kernels at 7B sizes, no Python) against the built library; returns the
    program's path (beside the library)."""
    lib = library_path()
    out = os.path.join(os.path.dirname(lib), "kernel_bench")
    cmd = [_hipcc(), "-O2", "-std=c++17", "-I" + HERE, os.path.join(HERE, "kernel_bench.cpp"), "-o", out,
           "-L" + os.path.dirname(lib), "-lyalm_hip", "-Wl,-rpath,$ORIGIN"]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if p.returncode != 0:
        raise RuntimeError("building kernel_bench failed:\n" + p.stderr)
    _say("built " + out)
    return out


def library_path():
    """The built library; compiled now if none exists."""
    return build(force=False)


if __name__ == "__main__":
    build(force=True)
    if len(sys.argv) > 1 and sys.argv[1] == "kernel_bench":
        build_kernel_bench()
