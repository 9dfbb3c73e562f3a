"""Builds ``libmsa_amd.so`` (the C-ABI library) from ``csrc/*.hip`` for gfx950 with hipcc.

``python -m msa_amd.build`` compiles in-tree; the library then travels with the source tree.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmsa_amd.so")
ARCH = "gfx950"
# packed fp32 VALU ops are switched off for all device code of this library
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wall", "-Wno-unused-function", "-Wno-inline-asm"]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src: str) -> str:
    obj = src[:-4] + ".o"
    cmd = ["hipcc", *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


# ---------------------------------------------------------------------------------------------------------------
# Contracts between hand-written asm statements and the compiler-allocated code around them, checked on the device
# assembly of every build:
#  * score_scan4_kernel (route_score.hip): its asm statements own v128-v255 and all accumulation registers across
#    statements.  The code the compiler generates for that kernel must therefore stay below v128, touch no
#    accumulation register (the compiler would only do so to spill), and use no scratch memory.
#  * flash_wide_kernel (flash_attn.hip): likewise, its statements own v56-v255 and all accumulation registers.
#  * flash_attn_kernel (flash_attn.hip): its direct-to-LDS loads are asm statements the compiler does not order
#    against LDS reads; a spill would add vector-memory waits in the middle of that ring.  No scratch, no spills.
# ---------------------------------------------------------------------------------------------------------------
CONTRACTS = {
    "route_score.hip": [("score_scan4_kernel", {"max_compiler_vgpr": 127, "no_agpr": True})],
    "flash_attn.hip": [("flash_attn_kernel", {}), ("flash_wide_kernel", {"max_compiler_vgpr": 55, "no_agpr": True})],
}


def _device_asm(src: str, extra=()) -> str:
    r = subprocess.run(["hipcc", *FLAGS, *extra, "--cuda-device-only", "-S", src, "-o", "-"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc -S failed for {src}:\n{r.stderr}")
    return r.stdout


def check_kernel_contracts(asm: str, kernel_substring: str, max_compiler_vgpr=None, no_agpr=False):
    """Returns the list of violations found in the device assembly `asm` for every kernel whose symbol contains
    `kernel_substring`: scratch use or spills (always), and, outside inline-asm regions, vector registers above
    `max_compiler_vgpr` / any accumulation register."""
    problems = []
    lines = asm.split("\n")
    # function bodies: from "<symbol>:" to s_endpgm
    i, found = 0, 0
    while i < len(lines):
        m = re.match(r"^(\S*%s\S*):" % re.escape(kernel_substring), lines[i])
        if not m or m.group(1).endswith(".kd"):
            i += 1
            continue
        name, found = m.group(1), found + 1
        in_asm = False
        i += 1
        while i < len(lines) and "s_endpgm" not in lines[i]:
            line = lines[i]
            i += 1
            if "#ASMSTART" in line:
                in_asm = True
                continue
            if "#ASMEND" in line:
                in_asm = False
                continue
            code = line.split(";")[0].strip()
            if not code or code.endswith(":") or code.startswith("."):
                continue
            if in_asm:
                continue
            if code.startswith("scratch_"):
                problems.append(f"{name}: scratch access: {code}")
            if no_agpr and re.search(r"\ba\d+\b|\ba\[\d+|accvgpr", code):
                problems.append(f"{name}: compiler-generated code touches an accumulation register: {code}")
            if max_compiler_vgpr is not None:
                for mm in re.finditer(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]", code):
                    hi = int(mm.group(1) or mm.group(3))
                    if hi > max_compiler_vgpr:
                        problems.append(f"{name}: compiler-generated code uses v{hi}: {code}")
    if found == 0:
        problems.append(f"no kernel matching {kernel_substring!r} in the assembly")
    # resource summary of the code object (YAML metadata at the end of the assembly)
    for m in re.finditer(r"\.name:\s+(\S*%s\S*)\n(.*?)\.wavefront_size" % re.escape(kernel_substring), asm, flags=re.S):
        meta = m.group(2)
        for key in ("private_segment_fixed_size", "vgpr_spill_count"):
            mm = re.search(r"\.%s:\s+(\d+)" % key, meta)
            if mm and int(mm.group(1)) != 0:
                problems.append(f"{m.group(1)}: {key} = {mm.group(1)}")
    return problems


def _check_contracts(src: str) -> None:
    rules = CONTRACTS.get(os.path.basename(src))
    if not rules:
        return
    asm = _device_asm(src)
    problems = []
    for kernel, kw in rules:
        problems += check_kernel_contracts(asm, kernel, **kw)
    if problems:
        raise RuntimeError("inline-asm contract broken in %s:\n  %s" % (src, "\n  ".join(problems[:20])))


def build(jobs: int = 8) -> str:
    """Compiles every source (always, even if the library exists), checks the inline-asm contracts on the device
    assembly and links the shared library."""
    srcs = sources()
    for gen, inc in (("gen_scan_asm.py", "scan_asm.inc"), ("gen_flash_asm.py", "flash_asm.inc")):
        if subprocess.run([sys.executable, os.path.join(CSRC, gen), "--check"]).returncode != 0:
            raise RuntimeError(f"csrc/{inc} is not what csrc/{gen} generates: run the generator")
    with ThreadPoolExecutor(max_workers=min(jobs, len(srcs) + len(CONTRACTS))) as ex:
        checks = [ex.submit(_check_contracts, s) for s in srcs if os.path.basename(s) in CONTRACTS]
        objs = list(ex.map(_compile, srcs))
        for c in checks:
            c.result()
    tmp = LIB + ".tmp"
    r = subprocess.run(["hipcc", "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build())
