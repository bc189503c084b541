"""Builds libbp_ternary_hip.so (the gfx950 kernels and their C ABI) in-tree with hipcc.

    python -m deepseekternarized_amd.build [--incremental]

The shared object lands next to this file; it is what ``deepseekternarized_amd.kernels.ternary_hip``
loads with ctypes. hipcc cross-compiles for gfx950 without a GPU present.
"""

from __future__ import annotations

import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libbp_ternary_hip.so"
SOURCES = ["bp_api.hip", "bp_general.hip", "bp_route.hip", "bp_gguf.hip", "bp_huffman.hip", "bp_moe.hip", "bp_mfma.hip", "bp_mfma_tq2.hip", "bp_gemm_tq2.hip", "bp_gemm_tq2f.hip", "bp_mfma_tq1.hip", "bp_gemm_tq1.hip", "bp_tq1_gemv.hip", "bp_tq1_gemv_fp4.hip", "bp_tq1_gemv_cw.hip", "bp_tq2_gemv_fp4.hip"]
# packed FP32 VALU ops are disabled for every device object of this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function", "-Wno-int-to-pointer-cast",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


# These kernels address LDS absolutely (their dynamic allocation must start at LDS address 0): a kernel of theirs
# with static LDS - e.g. a register array the compiler moved there because it was indexed dynamically - would
# compute on the wrong bytes, so the build refuses it.
NO_STATIC_LDS = {"bp_mfma_tq2.hip", "bp_gemm_tq2.hip", "bp_gemm_tq2f.hip", "bp_mfma_tq1.hip", "bp_gemm_tq1.hip", "bp_gemm_tq1.hip", "bp_tq1_gemv.hip", "bp_tq1_gemv_fp4.hip", "bp_tq1_gemv_cw.hip", "bp_tq2_gemv_fp4.hip"}
_REMARK = "[-Rpass-analysis=kernel-resource-usage]"


def _compile(src: str) -> Path:
    obj = CSRC / (src + ".o")
    check = src in NO_STATIC_LDS
    cmd = ["hipcc", *FLAGS, *(["-Rpass-analysis=kernel-resource-usage"] if check else []), "-c", str(CSRC / src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    lines = [l for l in res.stderr.splitlines() if noise not in l]
    if check:  # drop the resource remarks (and the source excerpts printed under them) after reading the LDS sizes
        kept, name, skip = [], "?", 0
        for l in lines:
            if _REMARK in l:
                if "Function Name:" in l:
                    name = l.split("Function Name:")[1].split()[0]
                if "LDS Size [bytes/block]:" in l and int(l.split("LDS Size [bytes/block]:")[1].split()[0]) != 0:
                    raise RuntimeError(f"{src}: kernel {name} uses static LDS; these kernels address LDS absolutely")
                skip = 2
            elif skip and (l.lstrip().startswith("|") or l.lstrip()[:1].isdigit()):
                skip -= 1
            else:
                kept.append(l)
        lines = kept
    err = "\n".join(lines)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def _fresh(src: str) -> bool:
    """The object of `src` is newer than the source and every header (used by --incremental only)."""
    obj = CSRC / (src + ".o")
    if not obj.exists():
        return False
    deps = [CSRC / src, *CSRC.glob("*.h"), HERE.parent / "include" / "bp_ternary.h", Path(__file__)]
    return all(obj.stat().st_mtime > d.stat().st_mtime for d in deps)


def build(verbose: bool = True, incremental: bool = False) -> Path:
    """Compiles every source (``incremental``: only those older than their inputs) and links the library."""
    todo = [s for s in SOURCES if not (incremental and _fresh(s))]
    with ThreadPoolExecutor(max_workers=7) as pool:
        list(pool.map(_compile, todo))
    objs = [CSRC / (s + ".o") for s in SOURCES]
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,--no-undefined", *map(str, objs), "-o", str(LIB)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv[1:])
