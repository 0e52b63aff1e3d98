"""Builds libtritium_mi355x.so (the HIP kernel library + its C ABI) in-tree with hipcc for gfx950.

    python -m tritium_amd.build
"""
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtritium_mi355x.so")
SOURCES = ["tk_kernels.hip", "tk_gemm128.hip", "tk_base3.hip", "tk_salt_v2.hip", "tk_vjp.hip", "tk_api.hip", "tk_format.cpp", "tk_salt.cpp", "tk_gguf.cpp"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # packed-FP32 instructions are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_library(verbose=True):
    """Compile every translation unit and link the shared library. Always rebuilds. The device
    assembly of the kernel file is produced alongside and checked (check_isa) before linking."""
    objs = []
    procs = []
    asm_file = tempfile.NamedTemporaryFile(suffix=".s", delete=False)
    asm_file.close()
    asm_cmd = [hipcc(), *FLAGS, "--offload-device-only", "-S", "-x", "hip", os.path.join(CSRC, "tk_kernels.hip"),
               "-o", asm_file.name]
    if verbose:
        print(" ".join(asm_cmd), flush=True)
    asm_proc = subprocess.Popen(asm_cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # (the 128-row prefill kernel has a register budget too; its file compiles in seconds)
    asm128_file = tempfile.NamedTemporaryFile(suffix=".s", delete=False)
    asm128_file.close()
    asm128_proc = subprocess.Popen([hipcc(), *FLAGS, "--offload-device-only", "-S", "-x", "hip",
                                    os.path.join(CSRC, "tk_gemm128.hip"), "-o", asm128_file.name],
                                   stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc(), *FLAGS, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        # the host pass does not know the gfx-only target feature and says so; that is harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip() and (verbose or p.returncode):
            print(out, flush=True)
        failed |= p.returncode != 0
    asm_out, _ = asm_proc.communicate()
    try:
        if asm_proc.returncode:
            print(asm_out, flush=True)
            failed = True
        if failed:
            raise RuntimeError("hipcc failed")
        from . import check_isa
        with open(asm_file.name) as f:
            bad = check_isa.check_text(f.read())
        if bad:
            raise RuntimeError("generated code reads registers of loads still in flight:\n" + check_isa.report(bad))
        asm128_out, _ = asm128_proc.communicate()
        if asm128_proc.returncode:
            print(asm128_out, flush=True)
            raise RuntimeError("hipcc failed")
        with open(asm_file.name) as f, open(asm128_file.name) as f128:
            over = check_isa.check_budgets(f.read() + "\n" + f128.read())
        if over:
            raise RuntimeError("kernels over their register budget (kernel, registers [+10000 = spills], budget):\n" +
                               "\n".join(str(x) for x in over))
    finally:
        os.unlink(asm_file.name)
        if asm128_proc.poll() is None:
            asm128_proc.kill()
        os.unlink(asm128_file.name)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build_library()
    print(LIB)
    sys.exit(0)
