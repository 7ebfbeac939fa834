"""Compile the gfx950 HIP sources into ``lib/libmts_moe.so`` with hipcc.

``python -m minitrain_amd.build`` (or ``build_library()``) always recompiles.  The
library is linked against the HIP runtime by soname only, with no run path, so a
process that has already imported torch resolves it to the runtime torch loaded.
"""

from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys
import tempfile

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(PKG_DIR), "csrc")
INCLUDE = os.path.join(os.path.dirname(os.path.dirname(PKG_DIR)), "include")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmts_moe.so")
SOURCES = ("mts_router.hip", "mts_router_linear.hip", "mts_route.hip", "mts_capacity.hip", "mts_combine.hip", "mts_gemm.hip", "mts_gemm_f16.hip", "mts_gemm_f32.hip", "mts_probe.hip", "mts_tuning.hip")

FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-fPIC",
    "-shared",
    "-std=c++17",
    # packed fp32 arithmetic is kept off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def build_library(verbose: bool = False, resource_report: bool = False, out: str | None = None,
                  defines: tuple = ()) -> str:
    """Compile every source (one hipcc process each, side by side) and link the shared library."""
    out = out or LIB_PATH
    os.makedirs(os.path.dirname(out), exist_ok=True)
    hipcc = find_hipcc()
    objdir = tempfile.mkdtemp(prefix="mts_build_")
    try:
        base = [hipcc, *[f for f in FLAGS if f != "-shared"], f"-I{INCLUDE}", f"-I{CSRC}", *[f"-D{d}" for d in defines]]
        if resource_report:
            base.append("-Rpass-analysis=kernel-resource-usage")
        procs = []
        for src in SOURCES:
            obj = os.path.join(objdir, src.replace(".hip", ".o"))
            procs.append((obj, subprocess.Popen(base + ["-c", os.path.join(CSRC, src), "-o", obj],
                                                stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)))
        stderr = ""
        failure = None
        for obj, proc in procs:
            if failure is not None:
                # one compile has failed: the others are ended and reaped before their directory goes away
                proc.kill()
                proc.communicate()
                continue
            _, err = proc.communicate()
            stderr += err
            if proc.returncode != 0:
                failure = f"hipcc failed ({proc.returncode}):\n{_quiet(err)}"
        if failure is not None:
            raise RuntimeError(failure)
        tmp = out + ".tmp"
        link = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *[o for o, _ in procs], "-o", tmp],
                              capture_output=True, text=True)
        if link.returncode != 0:
            raise RuntimeError(f"link failed ({link.returncode}):\n{_quiet(link.stderr)}")
        os.replace(tmp, out)
    finally:
        shutil.rmtree(objdir, ignore_errors=True)
    if resource_report:
        print(summarise_resources(stderr))
    elif verbose and _quiet(stderr).strip():
        print(_quiet(stderr))
    return out


def _quiet(err: str) -> str:
    return "\n".join(l for l in err.splitlines() if "packed-fp32-ops" not in l)


def summarise_resources(text: str) -> str:
    rows, cur = [], {}
    for line in text.splitlines():
        m = re.search(r"remark: .*?:\d+:\d+: (.*) \[-Rpass", line) or re.search(r"remark:\s+(.*) \[-Rpass", line)
        if not m:
            continue
        item = m.group(1).strip()
        if item.startswith("Function Name:"):
            cur = {"name": item.split(":", 1)[1].strip()}
            rows.append(cur)
        elif ":" in item and cur is not None:
            k, v = item.split(":", 1)
            cur[k.strip()] = v.strip()
    out = []
    for r in rows:
        name = subprocess.run(["c++filt", r["name"]], capture_output=True, text=True).stdout.strip()
        name = re.sub(r"\(anonymous namespace\)::", "", name).split("(")[0]
        out.append(
            f"{name[:90]:<90} vgpr={r.get('VGPRs', '?'):>4} agpr={r.get('AGPRs', '?'):>4} "
            f"spill={r.get('VGPRs Spill', r.get('VGPR Spill', '?')):>3} scratch={r.get('ScratchSize [bytes/lane]', '?'):>4} "
            f"occ={r.get('Occupancy [waves/SIMD]', '?'):>2} lds={r.get('LDS Size [bytes/block]', '?')}"
        )
    return "\n".join(out)


if __name__ == "__main__":
    path = build_library(verbose=True, resource_report="--resources" in sys.argv)
    print("built", path)
