"""Builds the gfx950 kernel library from ``csrc/*.hip`` with hipcc.

The library is one shared object with C entry points, kept in the tree under
``tffinfer_amd/lib`` (or, if the tree cannot be written, under the temporary
folder).  ``ensure_built`` builds only when there is no library for the present
sources; ``build`` always compiles.
"""
from __future__ import annotations

import hashlib
import json
import os
import re
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor

from .. import log

PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libtffinfer_hip.so"
ENGINE_LIB_NAME = "libtffinfer_engine.so"     # the engine's C interface (csrc/tffinfer_engine.h)
ENGINE_DEMO_NAME = "engine_demo"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",
    "-Rpass-analysis=kernel-resource-usage",     # read below: which kernels use scratch memory
]


class BuildError(RuntimeError):
    pass


def _sources() -> list[str]:
    return sorted(
        os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".hip")
    )


def _headers() -> list[str]:
    return sorted(os.path.join(CSRC_DIR, f) for f in os.listdir(CSRC_DIR) if f.endswith(".h"))


def source_digest() -> str:
    h = hashlib.sha256()
    for path in _sources() + _headers():
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe_{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dirs() -> list[str]:
    """Folders a library may live in, in order of preference."""
    fallback = os.path.join(tempfile.gettempdir(), f"tffinfer_amd_{os.getuid()}")
    return [os.path.join(PKG_DIR, "lib"), fallback]


def find_library() -> str | None:
    """Path of a library built from the present sources, or None."""
    digest = source_digest()
    for d in lib_dirs():
        info = os.path.join(d, "build_info.json")
        lib = os.path.join(d, LIB_NAME)
        if os.path.exists(lib) and os.path.exists(info):
            try:
                with open(info) as f:
                    if json.load(f).get("digest") == digest:
                        return lib
            except (OSError, ValueError):
                pass
    return None


def _scratch_users(remarks: str) -> dict[str, int]:
    """Kernels that use scratch memory, from hipcc's resource-usage remarks: name -> bytes a lane.
    A kernel that spills registers costs more than its spills: a launch that needs scratch
    memory takes some 15 us longer (measured: a product of 80 us took 96)."""
    out, name = {}, None
    for ln in remarks.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", ln)
        if m:
            name = m.group(1)
            continue
        m = re.search(r"remark:\s+ScratchSize \[bytes/lane\]: (\d+)", ln)
        if m and name and int(m.group(1)) > 0:
            out[name] = int(m.group(1))
    return out


def _masked_mfma(asm: str) -> dict[str, int]:
    """Kernels of a device assembly listing in which an MFMA stands under a mask of lanes with no
    branch round it: name -> number of such places.  Where the compiler takes a condition to
    differ between lanes it may, for a short body, only narrow the mask of active lanes and run
    the body (s_and_saveexec without an s_cbranch_execz).  An MFMA does not look at that mask: it
    runs for the whole wave and accumulates what the condition was meant to keep out.  The cure is
    a condition that is a scalar in the compiler's eyes (values derived from the wave's number
    go through readfirstlane)."""
    out: dict[str, int] = {}
    name, masked = None, False
    for ln in asm.splitlines():
        m = re.match(r"^(\S+):\s+; @", ln)
        if m:
            name, masked = m.group(1), False
            continue
        t = ln.strip()
        if name is None or not t:
            continue
        if re.match(r"s_\w+_saveexec_b64", t):
            masked = True
        elif masked:
            if t.startswith("s_cbranch_exec") or re.match(r"s_\w+_b64 exec,", t):
                masked = False      # the body is skipped when no lane is on, or the mask is restored
            elif t.startswith("v_mfma") or t.startswith("v_smfma"):
                out[name] = out.get(name, 0) + 1
                masked = False
    return out


def build(verbose: bool = True, check_masks: bool = True) -> str:
    """Compiles every source for gfx950 and links the library; returns its path.
    check_masks: also lists the device assembly of the sources that use the matrix cores and
    fails if an MFMA stands under a mask of lanes (see _masked_mfma): what the compiler makes of
    a condition is its choice, and another version may choose otherwise.  It runs beside the
    compilation and takes as long as the longest source."""
    hipcc = _hipcc()
    out_dir = next((d for d in lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError("no writable folder for the kernel library: " + ", ".join(lib_dirs()))
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    sources = _sources()
    t0 = time.time()
    done = threading.Event()

    scratch: dict[str, int] = {}

    def say(msg):
        if verbose:
            log.info("build: %s", msg)

    def ticker():
        while not done.wait(10.0):
            say(f"still compiling ... {time.time() - t0:.0f} s")

    def compile_one(src):
        obj = os.path.join(obj_dir, os.path.basename(src)[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", CSRC_DIR, "-c", src, "-o", obj]
        p = subprocess.run(cmd, capture_output=True, text=True)
        if p.returncode != 0:
            raise BuildError(f"hipcc failed on {os.path.basename(src)}:\n{p.stderr[-4000:]}")
        scratch.update(_scratch_users(p.stderr))
        say(f"compiled {os.path.basename(src)} ({time.time() - t0:.0f} s)")
        return obj

    masked: dict[str, int] = {}

    def list_one(src):
        flags = [f for f in HIPCC_FLAGS if not f.startswith("-Rpass")]
        p = subprocess.run([hipcc, *flags, "-I", CSRC_DIR, "-S", "--cuda-device-only", src, "-o", "-"],
                           capture_output=True, text=True)
        if p.returncode != 0:
            raise BuildError(f"hipcc -S failed on {os.path.basename(src)}:\n{p.stderr[-4000:]}")
        masked.update(_masked_mfma(p.stdout))
        say(f"checked the MFMAs of {os.path.basename(src)} ({time.time() - t0:.0f} s)")

    def uses_mfma(src):
        with open(src) as f:
            return "mfma" in f.read()

    say(f"compiling {len(sources)} files for gfx950 into {out_dir}")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    try:
        listed = [s for s in sources if uses_mfma(s)] if check_masks else []
        workers = max(1, min(len(sources) + len(listed), int(os.environ.get("MAX_JOBS", "8")), 16))
        with ThreadPoolExecutor(workers) as pool:
            checks = [pool.submit(list_one, s) for s in listed]
            objs = list(pool.map(compile_one, sources))
            for c in checks:
                c.result()
        if masked:
            raise BuildError("an MFMA under a mask of lanes, which it does not look at (make its condition a "
                             "scalar): " + ", ".join(f"{k} ({v})" for k, v in sorted(masked.items())))
        tmp_lib = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp_lib]
        p = subprocess.run(cmd, capture_output=True, text=True)
        if p.returncode != 0:
            raise BuildError(f"link failed:\n{p.stderr[-4000:]}")
        os.replace(tmp_lib, os.path.join(out_dir, LIB_NAME))
        with open(os.path.join(out_dir, "build_info.json"), "w") as f:
            info = {"digest": source_digest(), "flags": HIPCC_FLAGS, "scratch_bytes_per_lane": scratch}
            if check_masks:
                info["mfma_under_lane_mask"] = masked
            json.dump(info, f, indent=1)
    finally:
        done.set()
    for name, n in sorted(scratch.items()):
        log.warning("build: %s uses %d bytes of scratch memory a lane (registers spilled: some 15 us more at every launch)",
                    name, n)
    say(f"built {LIB_NAME} in {time.time() - t0:.0f} s")
    return os.path.join(out_dir, LIB_NAME)


def build_engine_capi(out_dir: str | None = None, verbose: bool = True) -> str:
    """Compiles the engine's C interface (csrc/engine_capi.c: an embedded interpreter around the
    package's engine) and the example program that uses it; returns the library's path."""
    import sysconfig
    cc = os.environ.get("CC") or shutil.which("gcc") or shutil.which("cc")
    if not cc:
        raise BuildError("no C compiler was found for the engine's C interface (looked at $CC, gcc, cc)")
    out_dir = out_dir or next((d for d in lib_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError("no writable folder for the engine library: " + ", ".join(lib_dirs()))
    inc, libdir = sysconfig.get_config_var("INCLUDEPY"), sysconfig.get_config_var("LIBDIR")
    pylib = "python" + (sysconfig.get_config_var("LDVERSION") or sysconfig.get_python_version())
    if not inc or not os.path.exists(os.path.join(inc, "Python.h")):
        raise BuildError(f"Python.h was not found in {inc}: the engine's C interface embeds the interpreter")
    lib = os.path.join(out_dir, ENGINE_LIB_NAME)
    cmd = [cc, "-O2", "-shared", "-fPIC", "-fvisibility=hidden", "-Wall", "-I", CSRC_DIR, "-I", inc,
           os.path.join(CSRC_DIR, "engine_capi.c"), "-L", libdir, "-l" + pylib, "-ldl", "-o", lib]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0:
        raise BuildError(f"{cc} failed on engine_capi.c:\n{p.stderr[-4000:]}")
    demo_src = os.path.join(os.path.dirname(PKG_DIR), "examples", "engine_demo.c")
    if os.path.exists(demo_src):
        cmd = [cc, "-O2", "-Wall", "-I", CSRC_DIR, demo_src, "-L", out_dir, "-ltffinfer_engine",
               "-Wl,-rpath,$ORIGIN", "-o", os.path.join(out_dir, ENGINE_DEMO_NAME)]
        p = subprocess.run(cmd, capture_output=True, text=True)
        if p.returncode != 0:
            raise BuildError(f"{cc} failed on engine_demo.c:\n{p.stderr[-4000:]}")
    if verbose:
        log.info("build: built %s", ENGINE_LIB_NAME)
    return lib


def find_engine_library() -> str | None:
    for d in lib_dirs():
        lib = os.path.join(d, ENGINE_LIB_NAME)
        if os.path.exists(lib):
            return lib
    return None


def ensure_built(verbose: bool = True) -> str:
    lib = find_library()
    if lib is None:
        lib = build(verbose=verbose)
    return lib


if __name__ == "__main__":
    print(build())
