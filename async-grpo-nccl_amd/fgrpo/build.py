"""Builds ``csrc/libfgrpo.so`` for gfx950 with hipcc.

The library is a handful of translation units (``*.hip`` under ``csrc/``) compiled side by side and linked into one
shared object.  Every compile also asks the compiler for its per-kernel resource report
(``-Rpass-analysis=kernel-resource-usage``); the report is written to ``csrc/resource_usage.json`` and the build
FAILS when a kernel of the guarded families reports scratch memory, register spills or more than 256 VGPRs
(``check_resource_usage``): the tile kernels issue their LDS fragment reads as inline assembly with hand-counted
waits, which is only correct while no fragment register is spilled or copied between the read and its wait."""
from __future__ import annotations

import concurrent.futures
import json
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
LIB_PATH = os.environ.get("FGRPO_LIB", os.path.join(CSRC, "libfgrpo.so"))
# an alternative output (FGRPO_LIB, for side-by-side builds) keeps its own objects and report
_ALT = "" if LIB_PATH == os.path.join(CSRC, "libfgrpo.so") else "_" + os.path.splitext(os.path.basename(LIB_PATH))[0]
USAGE_PATH = os.path.join(CSRC, f"resource_usage{_ALT}.json")
OBJ_DIR = os.path.join(CSRC, "build" + _ALT)

SOURCES = ["fgrpo_api.hip", "launch_lmhead.hip", "launch_gemm.hip", "launch_attn.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Rpass-analysis=kernel-resource-usage",
]

# What the compiler's report must show before the library may ship.
#  * Kernels that read their MFMA operands from LDS through inline assembly (the two-buffer direct-to-LDS loops:
#    tile configurations <..., 2, true>) must not spill a single vector register: a fragment register that is
#    spilled or copied between the `ds_read` and the hand-placed wait would be read before the data has landed.
#  * The kernels on the default path (tile ids 4, 7, 8 and the attention kernels) must stay at the occupancy they
#    were tuned for: at most 256 VGPRs and no AGPRs where two wavefronts share a SIMD.
ASM_READ_CFG = re.compile(r"TileCfgILi\d+ELi\d+ELi\d+ELi\d+ELi\d+ELi\d+ELi2ELb1EE")
TILE_KERNELS = ("lmhead_fwd_kernel", "lmhead_ds_kernel", "gemm_store_kernel")
TWO_PER_SIMD = ("TileCfgILi256ELi256ELi64ELi2ELi4ELi2ELi2ELb1EE",      # id 8
                "TileCfgILi256ELi128ELi32ELi2ELi2ELi2ELi3ELb1EE",      # id 7
                "TileCfgILi128ELi128ELi64ELi2ELi2ELi2ELi2ELb0EE",      # id 4
                "varlen_attn_fwd_kernel", "varlen_attn_dq_kernel",
                "varlen_attn_fwd2_kernel", "varlen_attn_dq2_kernel", "varlen_attn_dkv2_kernel")
# attention kernels whose LDS reads are inline assembly: a spilled register could be one whose data is still on its way
ASM_READ_ATTN = ("varlen_attn_fwd2_kernel", "varlen_attn_dq2_kernel", "varlen_attn_dkv2_kernel")
MUST_EXIST = TILE_KERNELS + ("varlen_attn_fwd_kernel", "varlen_attn_dq_kernel", "varlen_attn_dkv_kernel") + ASM_READ_ATTN

_FIELDS = {
    "TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch",
    "Occupancy [waves/SIMD]": "occupancy", "SGPRs Spill": "sgpr_spill", "VGPRs Spill": "vgpr_spill",
    "LDS Size [bytes/block]": "lds",
}


def parse_resource_usage(text: str) -> dict:
    """{mangled kernel name: {vgprs, agprs, sgprs, scratch, occupancy, sgpr_spill, vgpr_spill, lds}} from the
    compiler's kernel-resource-usage remarks."""
    out, cur = {}, None
    for line in text.splitlines():
        m = re.search(r"remark:\s+Function Name:\s+(\S+)", line)
        if m:
            cur = out.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z][A-Za-z \[\]/]*?):\s+(\d+)\s+\[-Rpass-analysis", line)
        if m and cur is not None and m.group(1).strip() in _FIELDS:
            cur[_FIELDS[m.group(1).strip()]] = int(m.group(2))
    return out


def check_resource_usage(usage: dict) -> list:
    """Problems (strings) that forbid shipping the build; an empty list means it may ship."""
    bad = []
    seen = {key: 0 for key in MUST_EXIST}
    for name, u in sorted(usage.items()):
        for key in MUST_EXIST:
            if key in name:
                seen[key] += 1
        tile = any(k in name for k in TILE_KERNELS)
        if tile and ASM_READ_CFG.search(name) and (u.get("scratch", 0) or u.get("vgpr_spill", 0)):
            bad.append(f"{name}: inline-assembly fragment reads with {u.get('vgpr_spill')} spilled VGPRs "
                       f"({u.get('scratch')} B/lane of scratch)")
        if any(k in name for k in ASM_READ_ATTN) and (u.get("scratch", 0) or u.get("vgpr_spill", 0)):
            bad.append(f"{name}: inline-assembly fragment reads with {u.get('vgpr_spill')} spilled VGPRs "
                       f"({u.get('scratch')} B/lane of scratch)")
        if any(k in name for k in TWO_PER_SIMD) and (tile or "varlen" in name):
            if u.get("vgprs", 0) > 256 or u.get("agprs", 0) or u.get("scratch", 0):
                bad.append(f"{name}: {u.get('vgprs')} VGPRs, {u.get('agprs')} AGPRs, {u.get('scratch')} B/lane of "
                           "scratch do not fit two wavefronts per SIMD")
    for key, n in seen.items():
        if n == 0:
            bad.append(f"no kernel named *{key}* in the compiler's report (guard out of date?)")
    return bad


def _compile(src: str, verbose: bool):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc, *HIPCC_FLAGS, *os.environ.get("FGRPO_EXTRA_FLAGS", "").split(), "-c", os.path.join(CSRC, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return src, obj, res.returncode, res.stdout


def _is_noise(line: str) -> bool:
    return "packed-fp32-ops" in line or "kernel-resource-usage" in line or line.startswith("In file included from")


def build(verbose: bool = True, only=None) -> str:
    """Compile every translation unit (or those named in ``only``, reusing the other objects) and link."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    todo = [s for s in SOURCES if only is None or s in only]
    by_source = {}
    if only is not None and os.path.exists(USAGE_PATH):
        by_source = json.load(open(USAGE_PATH)).get("sources", {})
    with concurrent.futures.ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        results = list(pool.map(lambda s: _compile(s, verbose), todo))
    for src, obj, rc, out in results:
        # remarks carry source excerpts on the following lines ("  2 | ..." and "    | ^"): drop those too
        keep, skip = [], 0
        for line in out.splitlines():
            if _is_noise(line):
                skip = 2
                continue
            if skip and re.match(r"^\s+(\d+\s+)?\|", line):
                skip -= 1
                continue
            skip = 0
            keep.append(line)
        shown = "\n".join(keep)
        if rc != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n" + shown)
        if verbose and shown.strip():
            print(shown)
        by_source[src] = parse_resource_usage(out)
    objs = [os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    missing = [o for o in objs if not os.path.exists(o)]
    if missing:
        raise RuntimeError(f"objects missing (build everything first): {missing}")
    # The guard decides before anything is linked: a build it refuses leaves no library behind (a stale one from an
    # earlier build is removed too), so nothing can load the kernels it exists to block.
    usage = {k: v for src in SOURCES for k, v in by_source.get(src, {}).items()}
    problems = check_resource_usage(usage)
    json.dump({"sources": by_source, "kernels": usage, "problems": problems}, open(USAGE_PATH, "w"), indent=1,
              sort_keys=True)
    if problems:
        if os.path.exists(LIB_PATH):
            os.remove(LIB_PATH)
        raise RuntimeError("kernel resource guard failed (no library written):\n  " + "\n  ".join(problems))
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    tmp = LIB_PATH + ".linking"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise RuntimeError("link failed:\n" + res.stdout)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build(only=sys.argv[1:] or None)
    sys.exit(0)
