"""Compile the HIP sources under csrc/ into proteusai_amd/libproteus_hip.so for gfx950, and the measurement probes
(csrc/probes.hip, which the benchmark and one test load, nothing else) into proteusai_amd/libproteus_probes.so.

Plain `hipcc -shared -fPIC`; no torch extension machinery (the library has a C
ABI and is loaded with ctypes).  hipcc cross-compiles without a GPU present.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB = os.path.join(HERE, "libproteus_hip.so")
SOURCES = ["abi.hip", "we_fwd.hip", "we_dropout_fwd.hip", "we_aniso_fwd.hip", "we_bwd.hip", "geo_attn_fwd.hip", "geo_attn_fwd_d32.hip", "geo_attn_fwd_d128.hip",
           "geo_attn_bwd.hip", "geo_attn_bwd_d32.hip", "geo_attn_bwd_d128.hip", "geo_attn_delta.hip", "add_layernorm.hip"]
PROBE_LIB = os.path.join(HERE, "libproteus_probes.so")
PROBE_SOURCES = ["probes.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 instructions are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core results stay in ordinary VGPRs: the softmax reads every accumulator element on
    # the vector ALU, and AGPR-resident accumulators would cost a v_accvgpr_read/write per access
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    "-Wall", "-Wno-unused-command-line-argument",
    "-I", INCLUDE,
]


def build(verbose: bool = False) -> str:
    """Compile every source (always; no up-to-date check) and link the two libraries.  Returns the product library."""
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in SOURCES + PROBE_SOURCES:
        obj = os.path.join(HERE, "build", src.replace(".hip", ".o"))
        cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        outp, _ = p.communicate()
        lines = [l for l in outp.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if p.returncode != 0:
            failed = True
            print(f"[build] {src} FAILED\n" + "\n".join(lines), file=sys.stderr)
        elif verbose and lines:
            print("\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")
    n = len(SOURCES)
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs[:n], check=True)
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", PROBE_LIB] + objs[n:], check=True)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
