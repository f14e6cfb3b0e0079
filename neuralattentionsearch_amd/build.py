"""Builds libnats_hip.so (gfx950) in-tree with hipcc.  Usage: python -m neuralattentionsearch_amd.build"""
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
LIB_PATH = os.path.join(PKG_DIR, "libnats_hip.so")
SOURCES = ["nats_roles.hip", "nats_rolestep.hip", "nats_prefill.hip", "nats_decode.hip", "nats_evict.hip", "nats_glue.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    # hipcc -O3 may otherwise form packed fp32 ops; keep them off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


# The packed-fp32 switch is a feature of the gfx950 target; hipcc hands -Xclang options to its x86 host pass as well,
# which answers with this line (three times per file) and ignores the option there.  Only that exact line is dropped.
_HOST_PASS_NOTE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"


def _run_hipcc(cmd):
    proc = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    rest = [ln for ln in proc.stderr.splitlines() if ln.strip() != _HOST_PASS_NOTE]
    if rest:
        print("\n".join(rest), file=sys.stderr, flush=True)
    if proc.returncode:
        raise subprocess.CalledProcessError(proc.returncode, cmd)


def build(verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        _run_hipcc(cmd)
        objs.append(obj)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-Wl,-z,defs", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
    print("built", LIB_PATH)
    sys.exit(0)
