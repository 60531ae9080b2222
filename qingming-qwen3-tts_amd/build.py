"""Builds libqm_attn.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python build.py            (from anywhere; also called by __graft_entry__.build())
hipcc cross-compiles without a GPU.  The flags are part of the product: fp contraction is
off so that the bf16 rounding chain is evaluated exactly as written, and packed-fp32
instruction selection is disabled.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libqm_attn.so")
ENGINE_LIB_PATH = os.path.join(LIB_DIR, "libqm_engine.so")

SOURCES = ["qm_lib.hip", "qm_norm_rope.hip", "qm_decode.hip", "qm_prefill.hip", "qm_predictor.hip", "qm_predictor_layout.hip", "qm_predictor_mfma.hip", "qm_predictor_frame.hip", "qm_talker_chain.hip", "qm_linear.hip", "qm_rmsnorm.hip", "qm_sampler.hip", "qm_linear_rows.hip", "qm_linear_rows_mfma.hip"]

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wextra", "-Wno-unused-parameter",
]


def build(verbose=True, jobs=4):
    os.makedirs(LIB_DIR, exist_ok=True)
    objs, procs = [], []
    for src in SOURCES:
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        objs.append(obj)
        cmd = ["hipcc", *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs, verbose)
    _drain(procs, verbose)
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.run(link, check=True)
    build_engine(verbose)
    return LIB_PATH


ENGINE_SOURCES = ["engine/qm_safetensors.cpp", "engine/qm_engine.cpp", "engine/qm_frame_engine.cpp"]


def build_engine(verbose=True):
    """libqm_engine.so: the host-side engine shell (C++ over the HIP runtime and libqm_attn.so, found
    next to it through an $ORIGIN run path)."""
    cmd = ["hipcc", "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
           "-Wno-unused-parameter", "-o", ENGINE_LIB_PATH,
           *[os.path.join(CSRC, src) for src in ENGINE_SOURCES],
           "-L" + LIB_DIR, "-lqm_attn", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(line for line in p.stdout.splitlines() if "packed-fp32-ops" not in line and line.strip())
    if verbose and out:
        print(out, flush=True)
    if p.returncode != 0:
        raise RuntimeError(f"hipcc failed on the engine library:\n{out}")
    return ENGINE_LIB_PATH


def _drain(procs, verbose):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        # hipcc's host pass does not know the packed-fp32 feature name; that warning is harmless.
        out = "\n".join(line for line in out.splitlines() if "packed-fp32-ops" not in line and line.strip())
        if verbose and out:
            print(out, flush=True)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")


if __name__ == "__main__":
    build()
    print(LIB_PATH)
