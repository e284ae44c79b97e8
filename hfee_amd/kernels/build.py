"""Compiling the HIP sources under hfee_amd/csrc for gfx950 into shared libraries.

Two kinds of library:
  * `core`: every kernel whose sizes are run-time arguments;
  * `attention_bf16_hd<N>`: the matrix-core attention kernels, compiled for one head
    size each, on demand (a model compiles only the head size it has).
Libraries are built in-tree (hfee_amd/_lib); if that folder cannot be written, in a
per-user folder under the system's temporary directory; $HFEE_BUILD_DIR, if set, comes
before both.  A library is rebuilt when its sources or flags no longer match the stamp
beside it.  $HFEE_EXTRA_FLAGS adds compiler flags (they are part of the stamp): together
with $HFEE_BUILD_DIR that builds a variant beside the in-tree libraries, to measure one
against the other.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
IN_TREE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "_lib")

ARCH = "gfx950"
FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]

CORE_SOURCES = ["elementwise.hip", "gemm_f32.hip", "attention_ref.hip", "gemm_bf16.hip", "gemm_skinny.hip",
                "sampling.hip", "random_fill.hip", "yardstick.hip"]
ATTENTION_SOURCE = "attention_bf16.hip"
HEAD_DIMS = tuple(range(16, 257, 16))


class BuildError(RuntimeError):
    pass


def _say(msg: str):
    print(f"[hfee_amd] {msg}", file=sys.stderr, flush=True)


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); "
                     "the HIP kernels cannot be built")


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".probe{os.getpid()}.{threading.get_ident()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False
    finally:
        pass


def extra_flags() -> list:
    return os.environ.get("HFEE_EXTRA_FLAGS", "").split()


def build_dirs() -> list:
    """Folders a library may live in, in the order they are searched."""
    dirs = []
    if os.environ.get("HFEE_BUILD_DIR"):
        dirs.append(os.path.abspath(os.environ["HFEE_BUILD_DIR"]))
    dirs.append(IN_TREE)
    dirs.append(os.path.join(tempfile.gettempdir(), f"hfee_amd-{os.getuid()}", "_lib"))
    return dirs


def _stamp(sources, defines) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + extra_flags() + sorted(defines)).encode())
    for name in sorted(set(sources) | {"common.h"} | {f for f in os.listdir(CSRC) if f.endswith(".h")}):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def library_spec(name: str):
    if name == "core":
        return CORE_SOURCES, []
    if name.startswith("attention_bf16_hd"):
        hd = int(name[len("attention_bf16_hd"):])
        if hd not in HEAD_DIMS:
            raise BuildError(f"attention kernels exist for head sizes {HEAD_DIMS[0]}..{HEAD_DIMS[-1]} "
                             f"in steps of 16, not {hd}")
        return [ATTENTION_SOURCE], [f"-DHFEE_HEAD_DIM={hd}"]
    raise BuildError(f"unknown kernel library {name!r}")


def find_built(name: str):
    """Path of an up-to-date built library, or None."""
    sources, defines = library_spec(name)
    want = _stamp(sources, defines)
    for d in build_dirs():
        so = os.path.join(d, f"libhfee_{name}.so")
        stamp = so + ".stamp"
        if os.path.isfile(so) and os.path.isfile(stamp):
            with open(stamp) as f:
                if f.read().strip() == want:
                    return so
    return None


def _run_with_heartbeat(cmds, what: str):
    """Runs the commands in parallel (at most 8 at a time), printing a line every
    ten seconds while they run."""
    procs, pending, failed = [], list(cmds), []
    start = last = time.time()
    limit = min(8, os.cpu_count() or 1)
    while pending or procs:
        while pending and len(procs) < limit:
            label, cmd = pending.pop(0)
            procs.append((label, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        for label, p in list(procs):
            if p.poll() is not None:
                out = p.stdout.read()
                procs.remove((label, p))
                if p.returncode != 0:
                    failed.append((label, out))
        if time.time() - last > 10:
            last = time.time()
            _say(f"still compiling {what} ({int(last - start)} s; {len(procs) + len(pending)} file(s) to go)")
        time.sleep(0.05)
    if failed:
        raise BuildError("hipcc failed:\n" + "\n".join(f"--- {l} ---\n{o}" for l, o in failed))


def build_library(name: str, force: bool = False) -> str:
    """Compiles one library (if needed) and returns its path."""
    if not force:
        so = find_built(name)
        if so:
            return so
    sources, defines = library_spec(name)
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError("no writable folder for the kernel library (set HFEE_BUILD_DIR)")
    cc = hipcc()
    obj_dir = os.path.join(out_dir, "obj", name)
    os.makedirs(obj_dir, exist_ok=True)
    _say(f"compiling kernel library '{name}' for {ARCH} ({len(sources)} source file(s)) into {out_dir}")
    t0 = time.time()
    cmds, objs = [], []
    for src in sources:
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        objs.append(obj)
        cmds.append((src, [cc, *FLAGS, *extra_flags(), *defines, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]))
    _run_with_heartbeat(cmds, name)
    so = os.path.join(out_dir, f"libhfee_{name}.so")
    tmp = so + f".{os.getpid()}.tmp"
    _run_with_heartbeat([("link", [cc, "--offload-arch=" + ARCH, "-shared", "-fPIC", *objs, "-o", tmp])], name)
    os.replace(tmp, so)
    with open(so + ".stamp", "w") as f:
        f.write(_stamp(sources, defines))
    shutil.rmtree(os.path.join(out_dir, "obj", name), ignore_errors=True)
    _say(f"built {os.path.basename(so)} in {time.time() - t0:.1f} s")
    return so


def build_all(head_dims=HEAD_DIMS, force: bool = True) -> list:
    """Compiles the core library and the attention library of every head size."""
    out = [build_library("core", force=force)]
    # the attention libraries are independent: build them side by side
    names = [f"attention_bf16_hd{hd}" for hd in head_dims]
    errors = []

    def work(n):
        try:
            out.append(build_library(n, force=force))
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append(e)

    threads = []
    for n in names:
        while sum(t.is_alive() for t in threads) >= 4:
            time.sleep(0.05)
        t = threading.Thread(target=work, args=(n,))
        t.start()
        threads.append(t)
    for t in threads:
        t.join()
    if errors:
        raise errors[0]
    return out
