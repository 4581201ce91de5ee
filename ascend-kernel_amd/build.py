"""Builds the gfx950 binaries of this package, in-tree.

  libmoe_gfx950.so          HIP kernels + the C ABI declared in include/moe_gfx950.h
  cinfer_ascendc.*.so       pybind11/torch module with the reference's Python API
  cabi_driver               torch-free C++ test driver of the C ABI (tests/cabi_driver.cpp)

Run as `python ascend-kernel_amd/build.py [--no-ext]`; hipcc cross-compiles for
gfx950 without a GPU.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmoe_gfx950.so")
KERNEL_SOURCES = ["moe_abi.cpp", "moe_dequant.hip", "moe_prepack.hip", "moe_route.hip", "moe_gemv.hip", "moe_gemm.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 from scalar float code
HIP_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


def ext_path() -> str:
    return os.path.join(HERE, "cinfer_ascendc" + sysconfig.get_config_var("EXT_SUFFIX"))


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_kernels(jobs: int = 4) -> str:
    objs, procs = [], []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in KERNEL_SOURCES:
        obj = os.path.join(HERE, "build", src + ".o")
        cmd = [HIPCC, *HIP_FLAGS, "-Rpass-analysis=kernel-resource-usage", "-x", "hip", "-I",
               os.path.join(ROOT, "include"), "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stderr=subprocess.PIPE, text=True)))
        objs.append(obj)
        if len(procs) >= jobs:
            _wait(procs)
    _wait(procs)
    _check_accumulator_moves("moe_gemm.hip")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB])
    return LIB


def _check_resources(src: str, remarks: list) -> None:
    """The GEMM accumulators are updated by inline-asm MFMAs whose latency the compiler does
    not track: they must stay in registers.  Any scratch use in a GEMM kernel means that
    they (or the loops around them) were not fully promoted -- refuse such a build."""
    name = None
    for line in remarks:
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split()[0]
        elif "ScratchSize [bytes/lane]:" in line and name and "grouped_gemm_kernel" in name:
            scratch = int(line.split("ScratchSize [bytes/lane]:")[1].split()[0])
            if scratch:
                raise RuntimeError(f"{src}: {name} uses {scratch} bytes of scratch per lane")


# instructions that must separate an ordinary write of an accumulator register from an MFMA on it
ACC_WRITE_GAP = 8


def _check_accumulator_moves(src: str) -> None:
    """Second guard for the inline-asm MFMAs of the GEMM: inside the k loops nothing but MFMAs may
    touch an accumulator register.  The compiler does not know the latency of the asm MFMAs, so a
    copy it inserted there (live-range split, spill to another register) would read a value that
    is not written yet.  Compiles the source to assembly and scans every innermost loop that
    contains MFMAs for any other instruction that names a register one of those MFMAs accumulates
    into (accumulators may be AGPRs or VGPRs)."""
    import re
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, src + ".s")
        cmd = [HIPCC, *HIP_FLAGS, "-x", "hip", "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-S",
               "--cuda-device-only", os.path.join(CSRC, src), "-o", asm]
        print("+", " ".join(cmd), flush=True)
        subprocess.run(cmd, check=True, stderr=subprocess.DEVNULL)
        text = open(asm).read()
    def regs(tok):
        out = []
        for mm in re.finditer(r"\b([av])\[(\d+):(\d+)\]|\b([av])(\d+)\b", tok):
            if mm.group(1):
                out += [(mm.group(1), r) for r in range(int(mm.group(2)), int(mm.group(3)) + 1)]
            else:
                out.append((mm.group(4), int(mm.group(5))))
        return out

    for m in re.finditer(r"^(\w*grouped_gemm_kernel\w*):", text, re.M):
        lines = text[m.end():text.index("s_endpgm", m.end())].split("\n")
        # Only the MFMAs of inline asm are invisible to the compiler; those it emitted itself (builtins)
        # get their wait states from it and are ordinary instructions here: rename them.
        in_asm = False
        for i, l in enumerate(lines):
            if "#ASMSTART" in l:
                in_asm = True
            elif "#ASMEND" in l:
                in_asm = False
            elif not in_asm and l.strip().startswith("v_mfma"):
                lines[i] = l.replace("v_mfma", "v_builtin_mfma", 1)
        labels = {mm.group(1): i for i, l in enumerate(lines) if (mm := re.match(r"^(\.LBB\d+_\d+):", l))}
        loops = []
        for i, l in enumerate(lines):
            mm = re.search(r"s_cbranch_\w+ (\.LBB\d+_\d+)", l)
            if mm and labels.get(mm.group(1), i) < i:
                loops.append((labels[mm.group(1)], i))
        for s0, e0 in loops:
            if any(s1 >= s0 and e1 <= e0 and (s1, e1) != (s0, e0) for s1, e1 in loops):
                continue  # not innermost
            body = [l.split(";")[0].strip() for l in lines[s0:e0 + 1]]
            # a k loop stores nothing to global memory; a backward branch around a whole tile (a steps' MFMAs
            # placed after their loop, then the epilogue) is not one
            if any(l.startswith(("buffer_store", "global_store")) for l in body):
                continue
            accs = set()
            for l in body:
                if l.startswith("v_mfma"):
                    accs.update(regs(l.split(None, 1)[1].split(",")[0]))
            for l in body:
                if not accs or not l or l.startswith("v_mfma") or l.endswith(":") or l.startswith("."):
                    continue
                parts = l.split(None, 1)
                if len(parts) == 2 and any(r in accs for r in regs(parts[1])):
                    raise RuntimeError(f"{src}: {m.group(1)} touches an accumulator inside a k loop: {l}")
        # Outside the loops too: an ordinary write of an MFMA's accumulator input needs wait states
        # before that MFMA (the compiler inserts them only for MFMAs it can see), e.g. zeros
        # re-materialized right in front of a peeled first k step.
        code = [l.split(";")[0].strip() for l in lines]
        code = [l for l in code if l and not l.endswith(":") and not l.startswith(".")]
        for i, l in enumerate(code):
            if not l.startswith("v_mfma"):
                continue
            accs = set(regs(l.split(None, 1)[1].split(",")[0]))
            for prev in code[max(0, i - ACC_WRITE_GAP):i]:
                parts = prev.split(None, 1)
                if prev.startswith("v_mfma") or prev.startswith("s_") or len(parts) < 2:
                    continue
                if any(r in accs for r in regs(parts[1].split(",")[0])):
                    raise RuntimeError(f"{src}: {m.group(1)} writes an accumulator right before its MFMA: {prev}")
            # ... and nothing but another MFMA may touch the result right behind it (the epilogues wait out the
            # latency with s_nop first); covers the k steps that sit outside the loops
            for nxt in code[i + 1:i + 1 + ACC_WRITE_GAP]:
                if nxt.startswith("s_nop 15"):
                    break
                parts = nxt.split(None, 1)
                if nxt.startswith("v_mfma") or nxt.startswith("s_") or len(parts) < 2:
                    continue
                if any(r in accs for r in regs(parts[1])):
                    raise RuntimeError(f"{src}: {m.group(1)} touches an accumulator right behind its MFMA: {nxt}")


def _wait(procs):
    for src, p in procs:
        _, err = p.communicate()
        lines = err.splitlines()
        remarks = [l for l in lines if "-Rpass-analysis" in l]
        err = "\n".join(l for l in lines if "packed-fp32-ops" not in l and "-Rpass-analysis" not in l)
        if err.strip():
            print(err, file=sys.stderr)
        if p.returncode:
            raise RuntimeError(f"hipcc failed on {src}")
        _check_resources(src, remarks)
    procs.clear()


def build_extension() -> str:
    import pybind11  # noqa: F401
    from torch.utils import cpp_extension as ce

    out = ext_path()
    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}",
                                                    f"-I{os.path.join(ROOT, 'include')}", "-I/opt/rocm/include"]
    libdirs = ce.library_paths()
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=cinfer_ascendc", "-D_GLIBCXX_USE_CXX11_ABI=1", *inc,
           os.path.join(CSRC, "cinfer_ascendc.cpp"), "-o", out, f"-L{HERE}", "-lmoe_gfx950",
           *[f"-L{d}" for d in libdirs], "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-ltorch_python",
           "-Wl,-rpath,$ORIGIN", *[f"-Wl,-rpath,{d}" for d in libdirs]]
    _run(cmd)
    return out


def build_cabi_driver() -> str:
    """tests/cabi_driver.cpp: the torch-free C++ caller of the C ABI (a test binary, kept beside the library so that it
    travels with it and finds it through its rpath)."""
    out = os.path.join(HERE, "cabi_driver")
    _run([HIPCC, "-O2", "-std=c++17", "--offload-arch=gfx950", "-I", os.path.join(ROOT, "include"),
          os.path.join(ROOT, "tests", "cabi_driver.cpp"), "-o", out, f"-L{HERE}", "-lmoe_gfx950", "-ldl", "-Wl,-rpath,$ORIGIN"])
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-ext", action="store_true", help="skip the torch/pybind11 module")
    args = ap.parse_args()
    build_kernels()
    build_cabi_driver()
    if not args.no_ext:
        build_extension()


if __name__ == "__main__":
    main()
