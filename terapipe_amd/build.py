"""Builds libterapipe_hip.so (gfx950) in-tree with hipcc.

Usage: ``python -m terapipe_amd.build`` (or ``build()`` from Python).  The shared library lands next to
this file so that it travels with the source tree; nothing is installed outside it.
"""
import os
import subprocess
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libterapipe_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["misc.hip", "layernorm.hip", "gemm.hip", "gemm_pipe.hip", "gemm_stream.hip", "attention.hip", "vocab.hip", "planner.hip", "optimizer.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-munsafe-fp-atomics",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-option-ignored",
]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _stale(src_path, obj):
    """True unless obj is newer than its source and every header the sources share."""
    if not os.path.exists(obj):
        return True
    deps = [src_path, os.path.join(CSRC, "common.h"), os.path.join(CSRC, "gemm_args.h"), os.path.join(CSRC, "gemm_epilogue.h"), os.path.join(CSRC, "gemm_tuned.inc"),
            os.path.join(os.path.dirname(HERE), "include", "terapipe_hip.h")]
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def build(verbose=True, jobs=7, incremental=False):
    """Compiles every source to an object (in parallel) and links the shared library.  incremental: leave
    objects alone that are newer than their source and the shared headers (a development convenience;
    the default compiles everything)."""
    hipcc = hipcc_path()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    t0 = time.time()
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        objs.append(obj)
        if incremental and not _stale(os.path.join(CSRC, src), obj):
            continue
        cmd = [hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        procs.append((src, cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        while sum(1 for _, _, p in procs if p.poll() is None) >= jobs:
            time.sleep(0.1)
    for src, cmd, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s\n%s" % (src, " ".join(cmd), text))
        if verbose and text.strip():
            lines = [l for l in text.splitlines() if "packed-fp32-ops" not in l and l.strip()]
            if lines:
                print("\n".join(lines))
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    subprocess.check_call(link)
    if verbose:
        print("built %s in %.1fs" % (LIB_PATH, time.time() - t0))
    return LIB_PATH


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv[1:])
    sys.exit(0)
