"""Builds libfdattn.so (the HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

Usage: python -m fastdeploy_amd.build
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libfdattn.so")

# -ffp-contract=off: the cache writer's bytes are defined by separately rounded fp32
# operations; the attention kernels lose nothing measurable from it.
# packed-fp32 instructions are switched off for every kernel.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fvisibility=hidden", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
] + os.environ.get("FDATTN_EXTRA_FLAGS", "").split()

# prefill_v2.hip: the compiler's sinking of common code out of two branches turns "this branch fills staging registers
# 0 and 1, that one 0 .. 3" into one store with a run-time register index, i.e. an array in scratch memory
SOURCE_FLAGS = {"prefill_v2.hip": ["-mllvm", "-simplifycfg-sink-common=false"]}

SOURCES = ["api.hip", "cache_writer.hip", "decode_generic.hip", "decode_tiles.hip", "decode_c8.hip", "decode_api.hip",
           "sqattn.hip", "prefill.hip", "prefill_v2.hip", "prefill_tiles.hip", "append_api.hip", "block_pool.hip",
           "kv_wire.hip"]


def _compile(src):
    """One source to its object.  The compiler's resource report rides along: a kernel that keeps private arrays in
    scratch memory (an array index the compiler could not resolve, or registers that ran out) fails the build - every
    kernel here is written to live in registers, and one that silently does not is several times slower."""
    import re
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = ["hipcc", *FLAGS, *SOURCE_FLAGS.get(src, []), "-Rpass-analysis=kernel-resource-usage", "-c",
           os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    report = [l for l in r.stderr.splitlines() if "-Rpass-analysis=kernel-resource-usage" in l]
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    # (a remark is followed by the source line it points at and a caret line)
    err = "\n".join(l for l in r.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "-Rpass-analysis=kernel-resource-usage" not in l
                    and not re.match(r"^\s*(\d+\s*)?\|", l))
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    name, spilled = None, []
    for l in report:
        m = re.search(r"Function Name: (\S+)", l)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", l)
        if m and int(m.group(1)) > 0:
            spilled.append("%s: %s bytes per lane" % (name, m.group(1)))
    if spilled:
        raise RuntimeError("%s: kernels that use scratch memory:\n  %s" % (src, "\n  ".join(spilled)))
    return obj


def highest_agpr(line):
    """Highest accumulation register an assembly line names, -1 if none: both ends of a tuple count (`a[28:43]` reaches
    a43 although it starts below a32), as do single registers (`a7`); whatever follows a `;` is a comment."""
    import re
    code, top = line.split(";")[0], -1
    for lo, hi in re.findall(r"\ba\[(\d+):(\d+)\]", code):
        top = max(top, int(lo), int(hi))
    for reg in re.findall(r"\ba\[?(\d+)\b", code):
        top = max(top, int(reg))
    return top


# What the hand-written register plan of prefill_v2.hip assumes of the compiler's resource report: every kernel owns
# the whole register file of its SIMD - 256 VGPRs (the accumulation registers start right behind them) and 256 AGPRs.
PLAN_AGPRS, PLAN_ACCUM_OFFSET = 256, 256


def _check_register_plan():
    """prefill_v2.hip addresses the upper AGPRs by name from asm statements, behind the compiler's back; what the
    compiler itself allocates must stay in the VGPRs and the lowest AGPRs (a[0:31]; a[0:63] for the kernels of the formats
    with one scale per stored row) and nothing may be spilled to scratch.  Checked on the device assembly of the same
    compile; a violation fails the build."""
    import re
    cmd = ["hipcc", *FLAGS, *SOURCE_FLAGS["prefill_v2.hip"], "-S", "--cuda-device-only",
           os.path.join(CSRC, "prefill_v2.hip"), "-o", "-"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc -S failed on prefill_v2.hip:\n" + r.stderr)
    kernel, in_asm, worst, scratch = None, False, {}, {}
    for line in r.stdout.splitlines():
        m = re.match(r"^(_ZN6fdattn17prefill_v2_kernelILi\d+ELb([01])ELb[01]EEEvNS_11PrefillArgsE):", line)
        if m:
            kernel, dyn = m.group(1), m.group(2) == "1"
            worst[kernel], scratch[kernel] = (-1, 64 if dyn else 32), 0
            continue
        if kernel is None:
            continue
        if re.match(r"^\.Lfunc_end\d+:", line):  # (not s_endpgm: a kernel with early returns has several)
            kernel = None
            continue
        if "#ASMSTART" in line:
            in_asm = True
        elif "#ASMEND" in line:
            in_asm = False
        elif not in_asm and not re.match(r"^\s*[;.]", line):
            if "scratch_" in line:
                scratch[kernel] += 1
            worst[kernel] = (max(worst[kernel][0], highest_agpr(line)), worst[kernel][1])
    # the kernel descriptors of the same assembly: `.amdhsa_accum_offset` / `.amdhsa_next_free_vgpr` follow each
    # kernel's `.amdhsa_kernel <name>` line
    desc, cur = {}, None
    for line in r.stdout.splitlines():
        m = re.match(r"^\s*\.amdhsa_kernel\s+(\S+)", line)
        if m:
            cur = m.group(1)
            continue
        m = re.match(r"^\s*\.amdhsa_(accum_offset|next_free_vgpr)\s+(\d+)", line)
        if m and cur in worst:
            desc.setdefault(cur, {})[m.group(1)] = int(m.group(2))
    for k in worst:
        d = desc.get(k, {})
        if d.get("accum_offset") != PLAN_ACCUM_OFFSET or d.get("next_free_vgpr") != PLAN_ACCUM_OFFSET + PLAN_AGPRS:
            raise RuntimeError("register-plan check failed for %s: the kernel descriptor says accum_offset %s, "
                               "next_free_vgpr %s; the hand-written plan needs %d and %d" %
                               (k, d.get("accum_offset"), d.get("next_free_vgpr"), PLAN_ACCUM_OFFSET,
                                PLAN_ACCUM_OFFSET + PLAN_AGPRS))
    if len(worst) != 6:
        raise RuntimeError("register-plan check: expected 6 prefill_v2 kernels in the assembly, found %d" % len(worst))
    for k, (hi, limit) in worst.items():
        if hi >= limit or scratch[k]:
            raise RuntimeError("register-plan check failed for %s: the compiler allocated a%d (limit a%d), %d scratch "
                               "accesses" % (k, hi, limit - 1, scratch[k]))


def build(verbose=True):
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=4) as ex:
        check = ex.submit(_check_register_plan)
        objs = list(ex.map(_compile, srcs))
        check.result()
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
