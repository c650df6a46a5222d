"""Build libspion_hip.so and the four drop-in libraries for gfx950, in-tree under spion_amd/lib/.

    python -m spion_amd.build

hipcc cross-compiles without a GPU.  Object files go to spion_amd/lib/obj/.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
OBJ = os.path.join(LIB, "obj")

HIP_SOURCES = ["capi.hip", "sparse_attn.hip", "dense_attn.hip", "pattern.hip"]
DROPINS = {1: "attn.so", 2: "attn_mask.so", 3: "block_attn.so", 4: "block_attn_mask.so"}

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    # packed-fp32 instruction selection is switched off on purpose for this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"command failed ({r.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out, flush=True)


def build_autograd_node(verbose: bool = False) -> str:
    """csrc/autograd_node.cpp -> lib/_spion_node.so: host code against libtorch and libspion_hip.so (g++, no HIP)."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    out = os.path.join(LIB, "_spion_node.so")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-DTORCH_EXTENSION_NAME=_spion_node",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for inc in cpp_extension.include_paths() + [sysconfig.get_paths()["include"]]:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "autograd_node.cpp"), "-o", out, f"-L{LIB}", "-lspion_hip", "-Wl,-rpath,$ORIGIN"]
    for d in cpp_extension.library_paths():
        cmd += [f"-L{d}", f"-Wl,-rpath,{d}"]
    cmd += ["-lc10", "-ltorch_cpu", "-ltorch", "-ltorch_python"]
    _run(cmd, verbose)
    return out


def emit_device_asm(src: str, out: str) -> str:
    """Device-only assembly of one HIP source (same flags as the library build)."""
    _run([HIPCC, *HIP_FLAGS, "--cuda-device-only", "-S", os.path.join(CSRC, src), "-o", out], False)
    return out


def scan_sgpr_hazards(asm_text: str):
    """Inline-assembly buffer instructions that read a scalar register fewer than five wait states after a vector
    instruction wrote it (v_readlane when the compiler restores a spilled scalar, v_readfirstlane, v_cmp into a scalar
    pair).  The compiler keeps that distance for the instructions it emits itself but does not look inside assembly
    blocks, so the loads into LDS (csrc/tile_kernels.h, csrc/bf16_kernels.h) have to carry it themselves.
    Returns (number of assembly blocks seen, list of findings)."""
    import re

    def sregs(tok):
        regs = set()
        for m in re.finditer(r"\bs\[(\d+):(\d+)\]", tok):
            regs.update(range(int(m.group(1)), int(m.group(2)) + 1))
        for m in re.finditer(r"\bs(\d+)\b", tok):
            regs.add(int(m.group(1)))
        return regs

    lines = asm_text.split("\n")
    kernel, in_asm, blocks, found = None, False, 0, []
    for idx, ln in enumerate(lines):
        t = ln.strip()
        if re.match(r"^_Z\w+:", ln):
            kernel = ln.split(":")[0]
        if t.startswith(";;#ASMSTART"):
            in_asm, blocks = True, blocks + 1
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not (in_asm and t.startswith("buffer_")):
            continue
        need = sregs(t.split(None, 1)[1] if " " in t else "")
        waited, j = 0, idx - 1
        while j >= 0 and waited < 5:
            u = lines[j].strip()
            j -= 1
            if not u or u.startswith(";"):
                continue
            if u.endswith(":") or u.startswith("."):
                break  # a label: what ran before is not known from the text
            m = re.match(r"(?:v_readlane_b32|v_readfirstlane_b32)\s+s(\d+)", u)
            hit = m is not None and int(m.group(1)) in need
            m = re.match(r"v_cmp\w*\s+(s\[\d+:\d+\])", u)
            hit = hit or (m is not None and bool(sregs(m.group(1)) & need))
            if hit:
                found.append(f"{kernel} line {idx + 1}: '{t}' {waited} wait states after '{u}'")
            m = re.match(r"s_nop\s+(\d+)", u)
            waited += int(m.group(1)) + 1 if m else 1
    return blocks, found


def build_all(verbose: bool = False, jobs: int = 4) -> str:
    os.makedirs(OBJ, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        _run([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj], verbose)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, HIP_SOURCES))
    main_lib = os.path.join(LIB, "libspion_hip.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", main_lib, *objs,
          "-Wl,-soname,libspion_hip.so"], verbose)
    for k, name in DROPINS.items():
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", f"-DSPION_DROPIN={k}",
              os.path.join(CSRC, "dropin.cpp"), "-o", os.path.join(LIB, name),
              f"-L{LIB}", "-lspion_hip", "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed", "-Wl,-z,defs"], verbose)
    build_autograd_node(verbose)
    return main_lib


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", sorted(f for f in os.listdir(LIB) if f.endswith(".so")))
    sys.exit(0)
