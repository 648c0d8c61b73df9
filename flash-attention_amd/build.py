"""Builds libflash_attn_gfx950.so (the C-ABI attention library) with hipcc for gfx950.

Usage:  python flash-attention_amd/build.py [-j JOBS]
The translation units under csrc/ compile in parallel; objects go to build/ (git-ignored) and the
shared library next to the Python package that loads it.
"""
import argparse
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "flash_attn", "libflash_attn_gfx950.so")
# a caller of the C ABI without Python or torch (examples/c_abi_caller.cpp), run by the GPU tests
EXAMPLE_SRC = os.path.join(HERE, "examples", "c_abi_caller.cpp")
EXAMPLE_BIN = os.path.join(OBJ_DIR, "c_abi_caller")
INCLUDE_DIR = os.path.join(os.path.dirname(HERE), "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms (v_pk_*_f32) are switched off on purpose: some of their forms have produced silently
    # wrong results on this hardware; ordinary float code must not be compiled into them
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    "-Wno-inline-asm",  # fa_stage.h sets M0 inside an asm statement on purpose (direct-to-LDS loads need it)
] + os.environ.get("FA_EXTRA_HIPCC_FLAGS", "").split()  # measurement variants of a kernel: -DFA_FUSED_EXPERIMENTS, -DFA_ABLATE_FWD=<bits>, -DFA_ABLATE_DKDV=<bits>


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "not a recognized feature" not in l)
    return src, obj, r.returncode, out


def build(jobs=8, verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = []
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, obj, rc, out in ex.map(_compile, sources()):
            if rc != 0:
                raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
            if verbose and out.strip():
                print(out)
            objs.append(obj)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout)
    cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-I", INCLUDE_DIR, EXAMPLE_SRC, "-L", os.path.dirname(LIB_PATH),
           "-lflash_attn_gfx950", "-Wl,-rpath,$ORIGIN/../flash_attn", "-o", EXAMPLE_BIN]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("building %s failed:\n%s" % (EXAMPLE_SRC, r.stdout))
    return LIB_PATH


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("-v", action="store_true")
    a = ap.parse_args()
    print(build(a.j, a.v))
