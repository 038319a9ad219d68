"""Builds libdnatok_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc."""
from __future__ import annotations

import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libdnatok_hip.so")
SOURCES = ["errors.hip", "char_encode.hip", "kmer_encode.hip", "bpe_encode.hip", "pack.hip", "host_ingest.hip", "normalize.hip"]
# bench.py's memory-only kernels: a library of their own (include/dnatok_diag.h), not part of the product
DIAG_LIB_PATH = os.path.join(_HERE, "libdnatok_diag.so")
DIAG_SOURCES = ["diag.hip", "errors.hip"]
# the BPE engine with its per-phase cycle counters compiled in (-DDNATOK_BPE_PHASE_CYCLES): a whole
# library beside the product's, for bench.py --only-extra bpe_phase_cycles
PHASES_LIB_PATH = os.path.join(_HERE, "libdnatok_hip_phases.so")
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 instruction forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hostpack_path() -> str:
    import sysconfig
    return os.path.join(_HERE, "_hostpack" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_hostpack(verbose: bool = False) -> str:
    """The small CPython module that packs a list of str into a byte buffer (host code only)."""
    import sysconfig
    cc = os.environ.get("CC", "gcc")
    cmd = [cc, "-O2", "-shared", "-fPIC", "-Wall", "-I" + sysconfig.get_paths()["include"],
           os.path.join(CSRC, "hostpack.c"), "-o", hostpack_path()]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return hostpack_path()


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_extension(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 and link the shared library. Always rebuilds."""
    objs = []
    procs = []
    for src in SOURCES + [x for x in DIAG_SOURCES if x not in SOURCES]:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
        if src in SOURCES:
            objs.append(obj)
    phases_obj = os.path.join(CSRC, "bpe_encode_phases.o")
    cmd = [hipcc(), *HIPCC_FLAGS, "-DDNATOK_BPE_PHASE_CYCLES", "-c", os.path.join(CSRC, "bpe_encode.hip"), "-o", phases_obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    procs.append(("bpe_encode.hip (phase cycles)", subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        text = out.decode(errors="replace")
        # the host pass does not know the device-only target feature; that warning is harmless
        text = "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"--- {src} failed ---\n{text}\n")
        elif verbose and text.strip():
            print(text)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    subprocess.check_call(cmd)
    diag_objs = [os.path.join(CSRC, x.replace(".hip", ".o")) for x in DIAG_SOURCES]
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", DIAG_LIB_PATH, *diag_objs])
    phases_objs = [phases_obj if o.endswith("bpe_encode.o") else o for o in objs]
    subprocess.check_call([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PHASES_LIB_PATH, *phases_objs])
    build_hostpack(verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build_extension(verbose=True))
