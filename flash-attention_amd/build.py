"""Builds libfa_mi355x.so in-tree with hipcc for gfx950 (no GPU needed: hipcc cross-compiles).

    python flash-attention_amd/build.py [-j N]

Counterpart of the reference's CUDAExtension build (setup.py:135-216), which compiles one
translation unit per (dtype, head-dim) with nvcc: here one hipcc invocation per unit, run in
parallel, then one link.
"""
import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "flash_attn")
OBJ_DIR = os.path.join(HERE, "build")
LIB = os.path.join(OUT_DIR, "libfa_mi355x.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU ops are kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def units():
    u = []
    for bf in (1, 0):
        for d in (64, 128, 256):
            u.append(("fa_prefill_inst.hip", "prefill_%s_%d.o" % ("bf16" if bf else "fp16", d),
                      ["-DFA_T_BF16=%d" % bf, "-DFA_D=%d" % d]))
            u.append(("fa_bwd_inst.hip", "bwd_%s_%d.o" % ("bf16" if bf else "fp16", d),
                      ["-DFA_T_BF16=%d" % bf, "-DFA_D=%d" % d]))
    u.append(("fa_decode.hip", "decode.o", []))
    u.append(("fa_aux.hip", "aux.o", []))
    u.append(("fa_rotary.hip", "rotary.o", []))
    u.append(("fa_peak.hip", "peak.o", []))
    u.append(("fa_api.hip", "api.o", []))
    return u


EXTRA = []


def compile_one(args):
    src, obj, defs = args
    cmd = [HIPCC] + FLAGS + EXTRA + defs + ["-c", os.path.join(CSRC, src), "-o", os.path.join(OBJ_DIR, obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    return r.returncode, obj, err


def build(jobs=None, verbose=True, out=None, defines=(), obj_dir=None):
    global OBJ_DIR, LIB
    EXTRA[:] = ["-D" + d for d in defines]
    if obj_dir:
        OBJ_DIR = obj_dir
    if out:
        LIB = out
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    us = units()
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(compile_one, us))
    for rc, obj, err in results:
        if err.strip() and verbose:
            print("[%s]\n%s" % (obj, err), file=sys.stderr)
        if rc != 0:
            raise RuntimeError("hipcc failed for %s" % obj)
    objs = [os.path.join(OBJ_DIR, o) for _, o, _ in us]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=None)
    ap.add_argument("--out", default=None, help="write the library here instead of the package dir")
    ap.add_argument("--obj-dir", default=None)
    ap.add_argument("-D", dest="defines", action="append", default=[], help="extra preprocessor define")
    a = ap.parse_args()
    build(a.j, out=a.out, defines=a.defines, obj_dir=a.obj_dir)
