"""Builds libpsn_hip.so: gfx950 code objects (hipcc --genco) linked into the host C-ABI library.

    python -m openagents_amd.build [--jobs N]

Everything is compiled in-tree into openagents_amd/lib/.  hipcc cross-compiles gfx950 without a
GPU present.  Device code is always built with packed-fp32 code generation switched off.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
ARCH = "gfx950"
LIB_NAME = "libpsn_hip.so"

DEVICE_FLAGS = ["-O3", "-std=c++17", f"--offload-arch={ARCH}", "--genco",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# (output stem, source, extra defines): one code object each, built in parallel
CODE_OBJECTS = [
    ("psn_quant", "psn_matvec.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_QUANT"]),
    ("psn_mv_q4_0", "psn_matvec.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_Q4_0"]),
    ("psn_mv_q8_0", "psn_matvec.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_Q8_0"]),
    ("psn_mv_q4_K", "psn_matvec.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_Q4_K"]),
    ("psn_mv_q5_K", "psn_matvec.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_Q5_K"]),
    ("psn_mv_q6_K", "psn_matvec.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_Q6_K"]),
    ("psn_mvm", "psn_matvec_mfma.hip", []),
    ("psn_pf_skinny", "psn_prefill.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_PF=0"]),
    ("psn_pf_wide", "psn_prefill.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_PF=2"]),
    ("psn_pf_dense", "psn_prefill.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_PF=5"]),
    *[(f"psn_pf_{fmt}_{fam}", "psn_prefill.hip", ["-DPSN_BUILD_ONLY", f"-DPSN_BUILD_PF={num}", f"-DPSN_BUILD_PF_{fmt.upper()}"])
      for fmt in ("q4_0", "q8_0") for num, fam in ((1, "ws"), (4, "base"))],
    *[(f"psn_pf_{fmt}_base", "psn_prefill.hip", ["-DPSN_BUILD_ONLY", "-DPSN_BUILD_PF=4", f"-DPSN_BUILD_PF_{fmt.upper()}"])
      for fmt in ("q4_K", "q5_K", "q6_K")],
    ("psn_decode", "psn_decode.hip", []),
    ("psn_calib", "psn_calib.hip", []),
]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), p.stdout))
    return p.stdout


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def lib_path() -> str:
    return os.path.join(LIB, LIB_NAME)


def code_object_paths():
    return [os.path.join(LIB, f"{stem}.{ARCH}.hsaco") for stem, src, _ in CODE_OBJECTS
            if os.path.exists(os.path.join(CSRC, src))]


def build(jobs: int = 0, verbose: bool = True, reuse_device: bool = False) -> str:
    """Compiles everything; with reuse_device a code object newer than its source and the device headers is kept."""
    os.makedirs(LIB, exist_ok=True)
    hipcc = _hipcc()
    jobs = jobs or min(8, os.cpu_count() or 1)
    todo = [(stem, src, defs) for stem, src, defs in CODE_OBJECTS if os.path.exists(os.path.join(CSRC, src))]

    device_headers = ["psn_args.h", "psn_device.h"]

    def compile_co(item):
        stem, src, defs = item
        out = os.path.join(LIB, f"{stem}.{ARCH}.hsaco")
        newest_src = max(os.path.getmtime(os.path.join(CSRC, f)) for f in [src, *device_headers])
        if reuse_device and os.path.exists(out) and os.path.getmtime(out) > newest_src:
            return out
        _run([hipcc, *DEVICE_FLAGS, *defs, "-I", CSRC, "-o", out, os.path.join(CSRC, src)])
        return out

    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        outs = list(ex.map(compile_co, todo))
    if verbose:
        for o in outs:
            print("built", os.path.relpath(o, os.path.dirname(HERE)), os.path.getsize(o), "bytes")

    # table of code objects: one .incbin per blob plus {begin, end} pairs the host walks
    asm = os.path.join(LIB, "psn_blobs.S")
    with open(asm, "w") as f:
        f.write("    .section .rodata\n")
        for i, o in enumerate(outs):
            f.write(f"    .balign 4096\npsn_blob_{i}_begin:\n    .incbin \"{o}\"\npsn_blob_{i}_end:\n")
        f.write("    .balign 16\n    .globl psn_builtin_blobs\npsn_builtin_blobs:\n")
        for i in range(len(outs)):
            f.write(f"    .quad psn_blob_{i}_begin\n    .quad psn_blob_{i}_end\n")
        f.write("    .balign 4\n    .globl psn_builtin_blob_count\npsn_builtin_blob_count:\n")
        f.write(f"    .long {len(outs)}\n")
        f.write("    .section .note.GNU-stack,\"\",@progbits\n")
    blob_o = os.path.join(LIB, "psn_blobs.o")
    _run(["gcc", "-c", "-fPIC", "-o", blob_o, asm])

    # the translation unit that owns the static device scratch: host + gfx950 device code in one object
    noalloc_o = os.path.join(LIB, "psn_noalloc.o")
    _run([hipcc, "-O2", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-I", CSRC, "-c", "-o", noalloc_o, os.path.join(CSRC, "psn_noalloc.hip")])

    host_o = os.path.join(LIB, "psn_host.o")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__",
          "-I", INCLUDE, "-I", CSRC, "-isystem", os.path.join(rocm, "include"),
          "-c", "-o", host_o, os.path.join(CSRC, "psn_host.cpp")])
    # the host quantizer keeps a*b+c as two roundings, like the reference quantizers it restates
    quant_o = os.path.join(LIB, "psn_quantize.o")
    _run(["g++", "-O3", "-march=x86-64-v3", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-ffp-contract=off", "-I", INCLUDE,
          "-c", "-o", quant_o, os.path.join(CSRC, "psn_quantize.cpp")])
    out = lib_path()
    _run(["g++", "-shared", "-fPIC", "-pthread", "-o", out, host_o, quant_o, noalloc_o, blob_o, "-Wl,--no-undefined",
          "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(rocm, "lib")])
    if verbose:
        print("built", os.path.relpath(out, os.path.dirname(HERE)), os.path.getsize(out), "bytes")
    return out


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=0)
    ap.add_argument("--reuse-device", action="store_true", help="keep code objects that are newer than every source file")
    args = ap.parse_args(argv)
    build(args.jobs, reuse_device=args.reuse_device)


if __name__ == "__main__":
    main(sys.argv[1:])
