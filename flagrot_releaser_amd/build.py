"""Builds the gfx950 shared libraries of this package with hipcc (cross-compiles without a GPU).

    python -m flagrot_releaser_amd.build            # all libraries
    python -m flagrot_releaser_amd.build kernels    # one of: kernels, kivi, mq, probe (a measurement aid for bench.py)

Libraries land in flagrot_releaser_amd/lib/ (in-tree, git-ignored).  Counterpart of the reference's
integrations/vllm_flagrot/csrc/build.sh / build_kivi.sh / build_mq.sh.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIBDIR = HERE / "lib"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed fp32 instructions are disabled for every device translation unit
COMMON = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
          "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]
# bit-exact translation units: every fp32 operation rounded on its own
STRICT = ["-ffp-contract=off", "-fno-fast-math"]
# FLAGROT_STRICT_MERGE=1 in the environment of the build: memory-model-strict split merge in the decode kernels (decode.hip)
if os.environ.get("FLAGROT_STRICT_MERGE", "0") not in ("", "0"):
    COMMON = COMMON + ["-DFLAGROT_STRICT_MERGE=1"]

# library -> [(source, extra flags)]
LIBS = {
    "kernels": ("libflagrot_kernels.so", [("writer.hip", STRICT), ("decode.hip", []), ("decode_gqa8.hip", []), ("decode_wide.hip", []), ("decode_wide_mma.hip", []), ("capi.hip", [])]),
    "kivi": ("libflagrot_kivi.so", [("kivi_write.hip", STRICT), ("kivi_wide.hip", STRICT), ("kivi_attn.hip", []), ("kivi_decode.hip", []), ("kivi_decode_wide.hip", [])]),
    "mq": ("libflagrot_mq.so", [("mq_prefill.hip", []), ("mq_wide.hip", [])]),
    "probe": ("libflagrot_probe.so", [("probe_read.hip", []), ("probe_mfma.hip", [])]),      # measurement aid (bench.py), not a boundary library
}


def lib_path(name: str) -> Path:
    return LIBDIR / LIBS[name][0]


def sources(name: str) -> list:
    return [CSRC / s for s, _ in LIBS[name][1]] + sorted(CSRC.glob("*.hpp")) + [Path(__file__)]


def _compile(args):
    """one translation unit -> object file; the compiler's per-kernel register report goes to <object>.usage.txt"""
    src, flags, obj = args
    cmd = [HIPCC, *COMMON, *flags, "-Rpass-analysis=kernel-resource-usage", "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stdout}\n{r.stderr}")
    Path(str(obj) + ".usage.txt").write_text(r.stderr)
    return obj


def spills(name: str) -> dict:
    """kernel (mangled name) -> spilled vector registers, from the register reports of the library's last build"""
    out = {}
    for s, _ in LIBS[name][1]:
        rep = LIBDIR / "obj" / (Path(s).stem + ".o.usage.txt")
        if not rep.exists():
            continue
        kernel = None
        for line in rep.read_text().splitlines():
            if "Function Name:" in line:
                kernel = line.split("Function Name:")[1].split()[0]
            elif "VGPRs Spill:" in line and kernel:
                out[kernel] = int(line.split("VGPRs Spill:")[1].split()[0])
    return out


def build(name: str, verbose: bool = True) -> Path:
    out, units = LIBS[name]
    units = [(CSRC / s, f) for s, f in units if (CSRC / s).exists()]
    if not units:
        raise FileNotFoundError(f"no sources for library {name}")
    LIBDIR.mkdir(exist_ok=True)
    objdir = LIBDIR / "obj"
    objdir.mkdir(exist_ok=True)
    jobs = [(s, f, objdir / (s.stem + ".o")) for s, f in units]
    with ThreadPoolExecutor(max_workers=min(4, len(jobs))) as ex:
        objs = list(ex.map(_compile, jobs))
    target = LIBDIR / out
    tmp = target.with_suffix(".so.tmp")
    r = subprocess.run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed for {out}:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, target)
    if verbose:
        print(f"built {target}")
    return target


def build_all(verbose: bool = True) -> list:
    return [build(n, verbose) for n in LIBS if all((CSRC / s).exists() for s, _ in LIBS[n][1])]


if __name__ == "__main__":
    names = sys.argv[1:] or None
    if names:
        for n in names:
            build(n)
    else:
        build_all()
