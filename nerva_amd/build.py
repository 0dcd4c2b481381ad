"""Builds nerva_amd/libnerva_hip.so from nerva_amd/csrc/*.hip with hipcc for gfx950.

hipcc cross-compiles without a GPU, so this runs in CI as the "does it build" check.
"""
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(HERE, "libnerva_hip.so")

SOURCES = ["gemv_stream.hip", "fp8_gemv.hip", "attn_decode.hip", "attn_prompt.hip", "argmax.hip", "synth_fill.hip",
           "sampler.hip", "gemm_rows.hip", "gemm_block.hip", "op_entry.hip", "decode_session.hip"]

FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         # packed fp32 VALU ops are kept off for every device function of this library
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libnerva_hip.so cannot be built")
    return exe


def _spilling_kernels(remarks):
    """Kernels whose register allocation went to scratch memory, from hipcc's resource-usage remarks."""
    bad, name = [], None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line and name is not None:
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            if size != 0:
                bad.append("%s (%d bytes a lane)" % (name, size))
            name = None
    return bad


# Kernels that request their data with hand-written loads and wait for it with explicit counts. The compiler
# does not know that such a register is still being written, so a spill (or any copy) of it reads garbage:
# these kernels must compile without scratch memory, which every build checks.
HAND_ISSUED_LOADS = ("attn_step_kernel", "moe_gate_up_lean_kernel", "moe_down_lean_kernel", "fp8_gemv_lean_kernel",
                     "gemm_deep_kernel")


def _compile(src):
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc()] + FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    lines = (res.stdout + res.stderr).splitlines()
    log = "\n".join(l for l in lines if "packed-fp32-ops" not in l and "kernel-resource-usage" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    bad = [k for k in _spilling_kernels("\n".join(l for l in lines if "kernel-resource-usage" in l))
           if any(name in k for name in HAND_ISSUED_LOADS)]
    if bad:
        raise RuntimeError("%s: kernels that issue loads by hand must not spill registers:\n  %s" % (src, "\n  ".join(bad)))
    return obj, log


def build(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        results = list(pool.map(_compile, sources))
    for obj, log in results:
        if verbose and log.strip():
            print(log)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + [o for o, _ in results]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout + res.stderr)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
