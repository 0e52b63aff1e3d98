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
SOURCES = ["tk_kernels.hip", "tk_flow_a8.hip", "tk_zskip.hip", "tk_gemm128.hip", "tk_gemm256.hip", "tk_base3.hip", "tk_salt_v2.hip", "tk_vjp.hip", "tk_api.hip", "tk_format.cpp", "tk_salt.cpp", "tk_gguf.cpp"]
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


# Translation units whose device assembly is emitted and checked before linking: in-flight registers of the
# hand-issued loads (the prefill kernels), register budgets, and kernels that need an empty static LDS segment.
ASM_SOURCES = ["tk_kernels.hip", "tk_flow_a8.hip", "tk_zskip.hip", "tk_gemm128.hip", "tk_gemm256.hip", "tk_base3.hip"]
HAZARD_SOURCES = ["tk_kernels.hip", "tk_gemm256.hip"]


def build_library(verbose=True):
    """Compile every translation unit and link the shared library. Always rebuilds. The device
    assembly of the kernel files is produced alongside and checked (check_isa) before linking."""
    objs = []
    procs = []
    asm = []
    for src in ASM_SOURCES:
        f = tempfile.NamedTemporaryFile(suffix=".s", delete=False)
        f.close()
        cmd = [hipcc(), *FLAGS, "--offload-device-only", "-S", "-x", "hip", os.path.join(CSRC, src), "-o", f.name]
        if verbose:
            print(" ".join(cmd), flush=True)
        asm.append((src, f.name, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
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
    try:
        texts = {}
        for src, path, p in asm:
            out, _ = p.communicate()
            if p.returncode:
                print(out, flush=True)
                failed = True
            else:
                with open(path) as f:
                    texts[src] = f.read()
        if failed:
            raise RuntimeError("hipcc failed")
        from . import check_isa
        for src in HAZARD_SOURCES:
            bad = check_isa.check_text(texts[src])
            if bad:
                raise RuntimeError("generated code reads registers of loads still in flight:\n" + check_isa.report(bad))
        everything = "\n".join(texts.values())
        over = check_isa.check_budgets(everything)
        if over:
            raise RuntimeError("kernels over their register budget (kernel, registers [+10000 = spills], budget):\n" +
                               "\n".join(str(x) for x in over))
        lds = check_isa.check_static_lds(everything)
        if lds:
            raise RuntimeError("kernels that address their dynamic LDS from 0 have static LDS in front of it "
                               "(kernel, bytes; None = kernel not found):\n" + "\n".join(str(x) for x in lds))
    finally:
        for _, path, p in asm:
            if p.poll() is None:
                p.kill()
            os.unlink(path)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build_library()
    print(LIB)
    sys.exit(0)
