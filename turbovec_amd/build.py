"""Builds libturbovec_hip.so for gfx950 with hipcc (in-tree, next to this file)."""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libturbovec_hip.so")

SOURCES = ["tv_kernels.hip", "tv_kernels2.hip", "tv_kernels3.hip", "tv_kernels4.hip", "tv_encode.hip", "tv_api.hip", "host_tables.cpp", "tv_snapshot.cpp"]

# -ffp-contract=off: the parity contract is bit-exact float arithmetic, fused
# only where the code says fmaf.  The packed-FP32 feature is switched off for
# device code on purpose.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    # the direct-to-LDS loads set M0 by hand and say so in their clobber list; clang notes that M0
    # is a reserved register once per instantiation
    "-Wno-inline-asm",
    # per-kernel register, scratch and LDS figures, checked below
    "-Rpass-analysis=kernel-resource-usage",
]

# The scan kernels request LDS and global loads through inline assembly the compiler's wait-count
# bookkeeping does not see, and wait for them by hand: a register spilled or reloaded between such
# a request and its wait would be read stale, silently.  So none of them may touch scratch memory.
# (k_scan_p4, k_scan_p4_multi, k_scan_p4_wide, k_scan_lut16 and the matrix-unit probe;
# k_scan_p4_batched and the other LUT scans leave every wait to the compiler.)
NO_SCRATCH = re.compile(r"k_scan_p4I|k_scan_p4_multiI|k_scan_p4_wideI|k_scan_lut16I|k_probe_mfma")
# These address their byte -> levels table by the byte's value alone: the table must sit at LDS
# address 0, i.e. the kernel may have no static LDS allocation in front of its dynamic one
# (k_scan_p4, k_scan_p4_multi, and the instances of k_scan_p4_wide whose last template argument,
# the split decode, is true).
NO_STATIC_LDS = re.compile(r"k_scan_p4(_multi)?I|k_scan_p4_wideI.*Lb1EEEv")


def check_resources(src, remarks):
    """Raises if a kernel of `src` breaks what its hand-written waits and addresses assume."""
    name = None
    problems = []
    for line in remarks.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            continue
        m = re.search(r"remark:\s+(ScratchSize \[bytes/lane\]|SGPRs Spill|VGPRs Spill|LDS Size \[bytes/block\]): (\d+)", line)
        if not m or name is None:
            continue
        what, value = m.group(1), int(m.group(2))
        if what.startswith("LDS"):
            if value and NO_STATIC_LDS.search(name):
                problems.append(f"{name}: {value} bytes of static LDS in front of the byte table")
        elif value and NO_SCRATCH.search(name):
            problems.append(f"{name}: {what} = {value}")
    if problems:
        raise RuntimeError(f"{src}: kernels with hand-placed waits must not spill or use scratch:\n  " + "\n  ".join(problems))


def build(verbose=False, jobs=4):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc] + FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if out.returncode != 0:
        raise RuntimeError("link failed:\n" + out.stdout)
    return OUT


def _drain(procs):
    while procs:
        src, p = procs.pop(0)
        out, _ = p.communicate()
        lines, skip = [], 0
        for l in out.splitlines():
            if skip:                      # the two source-echo lines under a remark
                skip -= 1
                continue
            if "is not a recognized feature for this target" in l:
                continue
            if "[-Rpass-analysis=kernel-resource-usage]" in l:
                skip = 2 if "Function Name" in l else 0
                continue
            if re.match(r"^\d+ warnings? generated", l):
                continue
            lines.append(l)
        text = "\n".join(lines)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{text}")
        check_resources(src, out)
        if text.strip():
            print(text, file=sys.stderr)


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
