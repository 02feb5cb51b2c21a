"""Compile the HIP sources in ``forgeminds_amd/csrc`` into ``forgeminds_amd/_lib/libfmhip.so``.

    python -m forgeminds_amd.build            # build (always recompiles)
    python -m forgeminds_amd.build --check    # exit 0 if an up-to-date library exists

gfx950 only. hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.
Packed-fp32 instruction selection is switched off for the device pass (plain fp32 FMAs are
what the kernels are tuned and validated with).
"""

from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libfmhip.so")
OBJ_DIR = os.path.join(LIB_DIR, "obj")

ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unused-command-line-argument",
    "-Wno-unknown-attributes",
]


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def headers() -> list[str]:
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(os.path.dirname(HERE), "include", "fm_hip.h"))
    return sorted(hs)


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build libfmhip.so")
    return exe


def up_to_date() -> bool:
    if not os.path.exists(LIB_PATH):
        return False
    t = os.path.getmtime(LIB_PATH)
    return all(os.path.getmtime(p) <= t for p in sources() + headers())


def _compile(src: str) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    cmd = [hipcc(), *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only target feature; that note is harmless
    err = "\n".join(l for l in r.stderr.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True, jobs: int | None = None) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(8, os.cpu_count() or 1)))
    with cf.ThreadPoolExecutor(jobs) as ex:
        objs = list(ex.map(_compile, srcs))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(srcs)} sources")
    return LIB_PATH


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--check", action="store_true", help="only report whether the library is current")
    ap.add_argument("-j", "--jobs", type=int, default=None)
    a = ap.parse_args(argv)
    if a.check:
        ok = up_to_date()
        print("up to date" if ok else "stale or missing")
        return 0 if ok else 1
    build(jobs=a.jobs)
    return 0


if __name__ == "__main__":
    sys.exit(main())
