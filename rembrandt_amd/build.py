"""Builds librembrandt_hip.so (hand-written HIP for gfx950) in-tree with hipcc."""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.environ.get("RH_OBJ_DIR") or os.path.join(HERE, "build")
LIB = os.environ.get("RH_LIB_OUT") or os.path.join(HERE, "librembrandt_hip.so")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
         # packed fp32 instructions are not to be generated on this hardware pool
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"] + os.environ.get("RH_EXTRA_FLAGS", "").split()


def sources():
    out = []
    for root, _, files in os.walk(CSRC):
        for f in sorted(files):
            if f.endswith(".hip") or f.endswith(".cpp"):
                out.append(os.path.join(root, f))
    return sorted(out)


def source_hash():
    """sha1 (12 hex digits) over every source and header the library is built from, in path order."""
    import hashlib
    h = hashlib.sha1()
    files = []
    for root, _, names in os.walk(CSRC):
        files += [os.path.join(root, f) for f in names if f.endswith((".hip", ".cpp", ".h", ".hpp"))]
    inc = os.path.join(os.path.dirname(HERE), "include")
    files += [os.path.join(inc, f) for f in os.listdir(inc) if f.endswith(".h")]
    for f in sorted(files):
        h.update(os.path.relpath(f, os.path.dirname(HERE)).encode())
        h.update(open(f, "rb").read())
    return h.hexdigest()[:12]


def _compile(src):
    rel = os.path.relpath(src, CSRC).replace(os.sep, "_")
    obj = os.path.join(OBJ, rel + ".o")
    extra = ['-DRH_SOURCE_HASH="%s"' % source_hash()] if os.path.basename(src) == "ctx.hip" else []
    cmd = [HIPCC] + FLAGS + extra + ["-c", src, "-o", obj]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    return obj, log


def build(verbose=True, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, len(srcs))
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        results = list(ex.map(_compile, srcs))
    for obj, log in results:
        if verbose and log.strip():
            print(log)
    objs = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
