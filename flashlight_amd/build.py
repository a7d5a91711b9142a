"""Builds libflashlight_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

One translation unit per kernel instance (rows of csrc/instance_list.inc) so the instances compile in parallel;
objects are cached under csrc/build/ keyed by a hash of the sources and flags.
"""
from __future__ import annotations

import concurrent.futures as cf
import hashlib
import os
import re
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
INCLUDE = PKG_DIR.parent / "include"
BUILD_DIR = CSRC / "build"
LIB_PATH = PKG_DIR / "libflashlight_amd.so"

ARCH = "gfx950"
# -packed-fp32-ops: keep hipcc from forming v_pk_*_f32; the kernels are written for scalar fp32 VALU ops.
HIPCC_FLAGS = [
    "-O3", f"--offload-arch={ARCH}", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm", "-Wno-ignored-optimization-argument",
    "-Wno-pass-failed", "-Rpass-analysis=kernel-resource-usage",
    f"-I{INCLUDE}", f"-I{CSRC}",
]


# Development knobs: extra hipcc flags (e.g. -DFL_SCHED=2) and an alternative output path for side-by-side builds.
HIPCC_FLAGS += os.environ.get("FL_HIPCC_EXTRA", "").split()
LIB_PATH = Path(os.environ.get("FL_LIB", str(LIB_PATH)))
PROBE_LIB_PATH = LIB_PATH.with_name("libflashlight_amd_probe.so")


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def instance_rows() -> list[tuple[str, str]]:
    rows = []
    for line in (CSRC / "instance_list.inc").read_text().splitlines():
        m = re.match(r"\s*X\(\s*(\w+)\s*,\s*(.*)\)\s*$", line)
        if m:
            rows.append((m.group(1), m.group(2).replace(" ", "")))
    if not rows:
        raise RuntimeError("instance_list.inc holds no instances")
    return rows


def _sources_digest() -> str:
    h = hashlib.sha256()
    for f in sorted(list(CSRC.glob("*.h")) + list(CSRC.glob("*.hip")) + list(CSRC.glob("*.inc")) + list(INCLUDE.glob("*.h"))):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _resource_usage(log: str) -> list[str]:
    """'kernel: VGPRs n, scratch n bytes/lane, occupancy n' lines from hipcc's kernel-resource-usage remarks."""
    out, cur = [], {}
    for line in log.splitlines():
        m = re.search(r"remark:\s+(Function Name|VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]): (\S+)", line)
        if not m:
            continue
        key, val = m.group(1), m.group(2)
        if key == "Function Name":
            cur = {"name": val}
        cur[key] = val
        if key.startswith("Occupancy"):
            out.append(f"{cur.get('name')}: VGPRs {cur.get('VGPRs')} AGPRs {cur.get('AGPRs')} "
                       f"scratch {cur.get('ScratchSize [bytes/lane]')} B/lane occupancy {val}")
    return out


def _compile(args: tuple[list[str], Path]) -> str:
    cmd, out = args
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        log = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l and "remark:" not in l)
        raise RuntimeError(f"hipcc failed for {out.name}:\n{' '.join(cmd)}\n{log}")
    usage = _resource_usage(r.stdout)
    if usage:
        out.with_suffix(".resources.txt").write_text("\n".join(usage) + "\n")
    return "\n".join(usage)


def build(force: bool = True, jobs: int | None = None, verbose: bool = False) -> Path:
    """Compiles every kernel instance and links the shared library.  force=False reuses cached objects."""
    cc = hipcc()
    digest = _sources_digest()
    objdir = BUILD_DIR / digest
    if force and BUILD_DIR.exists():
        shutil.rmtree(BUILD_DIR)
    objdir.mkdir(parents=True, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)

    tasks: list[tuple[list[str], Path]] = []
    objs: list[Path] = []
    for name, args in instance_rows():
        for f16 in (0, 1):  # every instance once for bf16 and once for fp16 elements
            o = objdir / f"inst_{name}{'_f16' if f16 else ''}.o"
            objs.append(o)
            if not o.exists():
                tasks.append(([cc, *HIPCC_FLAGS, f"-DFL_INST_NAME={name}", f"-DFL_INST_ARGS={args}", f"-DFL_INST_F16={f16}",
                               "-c", str(CSRC / "instance_unit.hip"), "-o", str(o)], o))
    # backward kernels: one unit per (head dim, feature bits) of FL_BWD_LIST in bwd_instances.h
    bwd_list = re.search(r"#define FL_BWD_LIST\(X\)(.*)", (CSRC / "bwd_instances.h").read_text()).group(1)
    for d, feat in re.findall(r"X\((\d+),\s*(\d+)\)", bwd_list):
        for f16 in (0, 1):
            o = objdir / f"bwd_{d}_{feat}{'_f16' if f16 else ''}.o"
            objs.append(o)
            if not o.exists():
                tasks.append(([cc, *HIPCC_FLAGS, f"-DFL_BWD_D={d}", f"-DFL_BWD_FEAT={feat}", f"-DFL_INST_F16={f16}", "-c",
                               str(CSRC / "bwd_unit.hip"), "-o", str(o)], o))
    # the shared-bias streaming forward: one unit per element type
    for f16 in (0, 1):
        o = objdir / f"pairbias{'_f16' if f16 else ''}.o"
        objs.append(o)
        if not o.exists():
            tasks.append(([cc, *HIPCC_FLAGS, f"-DFL_INST_F16={f16}", "-c", str(CSRC / "pairbias_unit.hip"), "-o", str(o)], o))
    # the instance tables are host data only: compiling them for the device would reference the host launchers
    for src, extra in (("instances_table.hip", ["--cuda-host-only"]), ("bwd_table.hip", ["--cuda-host-only"]),
                       ("api.hip", []), ("ipa_pack.hip", []), ("merge_chunks.hip", [])):
        o = objdir / (Path(src).stem + ".o")
        objs.append(o)
        if not o.exists():
            tasks.append(([cc, *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(o)], o))
    # the measurement probes go into a library of their own, which only the benchmark loads
    probe_obj = objdir / "probe.o"
    if not probe_obj.exists():
        tasks.append(([cc, *HIPCC_FLAGS, "-c", str(CSRC / "probe.hip"), "-o", str(probe_obj)], probe_obj))
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        for log in ex.map(_compile, tasks):
            if verbose and log.strip():
                print(log, file=sys.stderr)
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _compile(([cc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", *map(str, objs), "-o", str(tmp)], tmp))
    os.replace(tmp, LIB_PATH)
    tmp = PROBE_LIB_PATH.with_suffix(".so.tmp")
    _compile(([cc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", str(probe_obj), "-o", str(tmp)], tmp))
    os.replace(tmp, PROBE_LIB_PATH)
    build_c_host()
    return LIB_PATH


C_HOST_SRC = PKG_DIR.parent / "tests" / "c_host" / "attn_host.c"
C_HOST_BIN = C_HOST_SRC.with_suffix("")


def build_c_host() -> Path | None:
    """The plain-C host program of the test suite (tests/c_host/attn_host.c): C99, gcc, linked against the library just
    built and the HIP runtime.  Skipped when the source is not there (a copy of the package alone)."""
    if not C_HOST_SRC.exists() or LIB_PATH.parent != PKG_DIR:
        return None
    rocm = Path(hipcc()).resolve().parent.parent
    cmd = [shutil.which("gcc") or "gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__",
           f"-I{rocm / 'include'}", f"-I{INCLUDE}", str(C_HOST_SRC), "-o", str(C_HOST_BIN), f"-L{PKG_DIR}", "-lflashlight_amd",
           f"-L{rocm / 'lib'}", "-lamdhip64", "-lm", "-Wl,-rpath,$ORIGIN/../../flashlight_amd", f"-Wl,-rpath,{rocm / 'lib'}"]
    _compile((cmd, C_HOST_BIN))
    return C_HOST_BIN


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--incremental", action="store_true", help="reuse cached objects when sources are unchanged")
    ap.add_argument("-j", "--jobs", type=int, default=None)
    a = ap.parse_args()
    print(build(force=not a.incremental, jobs=a.jobs, verbose=True))
