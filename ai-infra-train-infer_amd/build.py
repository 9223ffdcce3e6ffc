"""Builds libpaged_attn.so (the C-ABI HIP library) for gfx950 with hipcc, and beside it the
measuring library csrc/probes/libpa_probes.so (csrc/probes/pa_probes.h: what bench.py times the
kernels against; never loaded by the package).

Usage:  python build.py

Each csrc/*.hip file is compiled to an object in csrc/_obj/ (in parallel) and the objects
are linked into libpaged_attn.so next to this file; csrc/probes/*.hip likewise into
libpa_probes.so.  hipcc cross-compiles for gfx950 without a GPU present.  The libraries depend
on the HIP runtime only (no torch symbols).
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OBJ = os.path.join(CSRC, "_obj")
LIB = os.path.join(HERE, "libpaged_attn.so")
PROBES = os.path.join(CSRC, "probes")
PROBES_LIB = os.path.join(PROBES, "libpa_probes.so")
ARCH = "gfx950"

# -packed-fp32-ops: keep hipcc from forming v_pk_{add,mul,fma}_f32 out of ordinary float code.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
CXXFLAGS = ["-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-ffp-contract=off",
            f"--offload-arch={ARCH}", "-Wall", "-Wno-unused-function",
            "-I", INCLUDE, "-I", CSRC, "-I", PROBES, "-Rpass-analysis=kernel-resource-usage"] + DEVICE_FLAGS
# extra compiler flags (e.g. -DNAME=value for a tuning macro of a kernel), space separated
CXXFLAGS += os.environ.get("PA_EXTRA_HIPCC_FLAGS", "").split()


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or put /opt/rocm/bin on PATH)")


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def probe_sources():
    return sorted(os.path.join(PROBES, f) for f in os.listdir(PROBES) if f.endswith(".hip"))


def _newest_input():
    files = sources() + probe_sources() + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    files += [os.path.join(PROBES, f) for f in os.listdir(PROBES) if f.endswith(".h")]
    files += [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)] + [os.path.abspath(__file__)]
    return max(os.path.getmtime(f) for f in files)


def is_current():
    newest = _newest_input()
    return all(os.path.exists(lib) and os.path.getmtime(lib) >= newest for lib in (LIB, PROBES_LIB))


def _compile(hipcc, src):
    prefix = "probes_" if os.path.dirname(src) == PROBES else ""
    obj = os.path.join(OBJ, prefix + os.path.basename(src)[:-4] + ".o")
    cmd = [hipcc] + CXXFLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr[-8000:]))
    # No kernel of the library may use scratch memory (register spills or arrays the compiler could not
    # keep in registers): such a kernel is several times slower than intended and nothing else says so.
    name, spilled = "?", []
    for ln in r.stderr.splitlines():
        if "Function Name:" in ln:
            name = ln.split("Function Name:")[1].split()[0]
        elif "ScratchSize [bytes/lane]:" in ln:
            size = int(ln.split("ScratchSize [bytes/lane]:")[1].split()[0])
            if size:
                spilled.append("%s: %d bytes of scratch per lane" % (name, size))
    if spilled and not os.environ.get("PA_ALLOW_SCRATCH"):      # the variable is for experiments with a kernel's shape
        raise RuntimeError("kernels of %s use scratch memory:\n%s" % (src, "\n".join(spilled)))
    # the host pass does not know the device-only target feature; that warning is expected
    noise = ("packed-fp32-ops", "is not a recognized feature")
    msgs, skip = [], 0
    for ln in r.stderr.splitlines():
        if "kernel-resource-usage" in ln:
            skip = 2          # the remark's source line and caret follow it
        elif skip and (ln.lstrip()[:1].isdigit() or ln.lstrip().startswith("|")):
            skip -= 1
        else:
            skip = 0
            if ln.strip() and not ln.startswith("In file included from") and not any(n in ln for n in noise):
                msgs.append(ln)
    return obj, "\n".join(msgs)


def build_library(force=True, verbose=False):
    """Compile and link the library. With force=False an up-to-date library is kept."""
    if not force and is_current():
        if not os.path.exists(FASTCALL_LIB):
            build_fastcall()
        return LIB
    hipcc = _hipcc()
    os.makedirs(OBJ, exist_ok=True)
    srcs, probes = sources(), probe_sources()
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as ex:
        results = list(ex.map(lambda s: _compile(hipcc, s), srcs + probes))
    for obj, msgs in results:
        if verbose and msgs:
            print(msgs, file=sys.stderr)
    objs = [o for o, _ in results]
    # -Bsymbolic: each library binds its own copy of the helpers both define (pa::fail, ...)
    for lib, members in ((LIB, objs[:len(srcs)]), (PROBES_LIB, objs[len(srcs):])):
        tmp = lib + ".tmp"
        cmd = [hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", "-Wl,-Bsymbolic", "-o", tmp] + members
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-8000:]))
        os.replace(tmp, lib)
    build_fastcall()
    return LIB


FASTCALL_SRC = os.path.join(CSRC, "fastcall", "pa_fastcall.c")
FASTCALL_LIB = os.path.join(HERE, "pa_fastcall.so")


def build_fastcall():
    """The CPython module the binding uses for its hottest calls instead of ctypes (csrc/fastcall): plain C
    for the host, no GPU code.  The binding works without it, only slower, so a host without a C compiler
    or Python's headers skips it with a note."""
    import sysconfig
    include = sysconfig.get_paths()["include"]
    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None or not os.path.exists(os.path.join(include, "Python.h")):
        print("build.py: no C compiler or no Python.h - pa_fastcall.so not built (the binding falls back to ctypes)",
              file=sys.stderr)
        return None
    tmp = FASTCALL_LIB + ".tmp"
    cmd = [cc, "-O2", "-Wall", "-shared", "-fPIC", "-I" + include, FASTCALL_SRC, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("compiling pa_fastcall failed:\n%s\n%s" % (" ".join(cmd), r.stderr[-4000:]))
    os.replace(tmp, FASTCALL_LIB)
    return FASTCALL_LIB


if __name__ == "__main__":
    path = build_library(force=True, verbose=True)
    print(path)
