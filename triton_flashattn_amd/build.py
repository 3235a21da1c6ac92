"""Builds libfa_mi355.so (HIP kernels + C ABI) for gfx950 next to this file.

Usage: python -m triton_flashattn_amd.build [-j N]
hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libfa_mi355.so")
HEAD_DIMS = (128, 64, 256, 32, 16)  # longest compiles first
# (source, head dim or None): the kernel files are compiled once per head dimension
UNITS = [("fa_bwd.hip", d) for d in HEAD_DIMS] + [("fa_fwd.hip", d) for d in HEAD_DIMS] + [("fa_api.hip", None)]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
    # packed fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # one remark block per kernel with its register, scratch and LDS use; read by _scratch_users
    "-Rpass-analysis=kernel-resource-usage",
]


def _compile(unit):
    src, d = unit
    obj = os.path.join(CSRC, src.replace(".hip", ".o" if d is None else "_d%d.o" % d))
    defs = [] if d is None else ["-DFA_HEAD_DIM=%d" % d]
    cmd = [HIPCC] + FLAGS + defs + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (res.stdout + res.stderr).splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s (D=%s):\n%s" % (src, d, log))
    return obj, log, d


def _scratch_users(log):
    """(kernel, VGPRs, scratch bytes per lane) of every kernel in a compile log that spills."""
    out, name, vgprs = [], None, None
    for line in log.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name, vgprs = m.group(1), None
        m = re.search(r" VGPRs: (\d+)", line)
        if m:
            vgprs = int(m.group(1))
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name and int(m.group(1)) > 0:
            out.append((name, vgprs, int(m.group(1))))
    return out


def build(jobs=8, verbose=False):
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        results = list(ex.map(_compile, UNITS))
    objs = [o for o, _, _ in results]
    # A kernel that spills registers to scratch runs its spill traffic through the same queue as
    # the hand-counted direct-to-LDS copies (every reload drains that queue): no kernel of any head
    # dim may do that.
    spills = [(d, k, v, b) for _, log, d in results for k, v, b in _scratch_users(log)]
    bad = [x for x in spills if x[0] is not None]
    if verbose:
        for d, k, v, b in spills:
            print("scratch: D=%s %s: %d VGPRs, %d bytes/lane" % (d, k, v, b))
    if bad:
        raise RuntimeError("kernels that spill registers:\n" + "\n".join(
            "  D=%s %s: %s VGPRs, %d bytes/lane of scratch" % x for x in bad))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout + res.stderr)
    return LIB


if __name__ == "__main__":
    j = 8
    if "-j" in sys.argv:
        j = int(sys.argv[sys.argv.index("-j") + 1])
    print(build(jobs=j, verbose=True))
