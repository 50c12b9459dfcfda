"""Builds libbitdecode.so (hand-written HIP for gfx950) in-tree with hipcc."""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libbitdecode.so")
# measurement aid of the benchmark (read-only kernels); not part of the decode path, loaded by bench.py only
PROBE_LIB_PATH = os.path.join(_HERE, "libbitdecode_probe.so")

ARCH = "gfx950"
COMMON = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
          # packed-FP32 VALU forms are kept out of the generated code on purpose
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          # per-kernel register / scratch report, checked below
          "-Rpass-analysis=kernel-resource-usage"]
# the quantizer must be IEEE fp32: no contraction, correctly rounded division;
# the decode kernel is scheduled for instruction-level parallelism rather than for occupancy (its
# occupancy is fixed by LDS): 2-3 % faster on the long-context workloads, same register counts
PER_FILE = {
    "qpack.hip": ["-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt"],
    "decode.hip": ["-mllvm", "-amdgpu-sched-strategy=gcn-max-ilp", "-fhip-fp32-correctly-rounded-divide-sqrt"],
    "api.hip": [],
}
PROBE_SRC = "probe.hip"


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def check_no_scratch(src: str, report: str) -> None:
    """No kernel of the library may spill registers: a kernel with a scratch segment pays for its set-up
    at every launch (about 1 us on the decode kernel), whether or not the spilling path runs."""
    name = None
    for line in report.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and int(m.group(1)) > 0:
            raise RuntimeError(f"{src}: kernel {name} needs {m.group(1)} bytes of scratch per lane (register spills)")


def build(verbose: bool = False) -> str:
    """Compile every HIP source and link the shared library (and the benchmark's probe library); returns the
    path of the former."""
    cc = hipcc()
    objdir = os.path.join(_HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    procs = []
    probe_cmd = [cc, *COMMON, "-shared", os.path.join(CSRC, PROBE_SRC), "-o", PROBE_LIB_PATH]
    if verbose:
        print(" ".join(probe_cmd), flush=True)
    probe_proc = subprocess.Popen(probe_cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    for src, extra in PER_FILE.items():
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [cc, *COMMON, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        check_no_scratch(src, out)
    out, _ = probe_proc.communicate()
    if probe_proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {PROBE_SRC}:\n{out}")
    cmd = [cc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
