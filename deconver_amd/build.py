"""In-tree build of the HIP library (and, on request, of the host checker).

    python -m deconver_amd.build            # libdeconver_ndc.so for gfx950
    python -m deconver_amd.build --hostcheck  # + libndc_hostcheck.so (CPU test-suite)
"""

from __future__ import annotations

import argparse
import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=fast",
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # LLVM's VectorCombine widens scalar loads of the per-thread state into overlapping
    # two-element loads, which pins that state in private memory instead of registers
    "-mllvm", "-disable-vector-combine",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if proc.returncode != 0:
        sys.stderr.write(out + "\n")
        raise RuntimeError("build failed: " + " ".join(cmd))
    return out


def build_hip(extra_flags=()) -> str:
    out = os.path.join(_HERE, "libdeconver_ndc.so")
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-o", out, os.path.join(CSRC, "ndc_capi.hip")])
    return out


def build_hostcheck(sanitize: bool = False) -> str:
    out = os.path.join(_HERE, "libndc_hostcheck.so")
    flags = ["-O1", "-g", "-fsanitize=address,undefined"] if sanitize else ["-O2"]
    _run(["g++", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unknown-pragmas", *flags, "-o", out,
          os.path.join(CSRC, "ndc_hostcheck.cpp")])
    return out


def main(argv=None) -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--hostcheck", action="store_true")
    ap.add_argument("--no-hip", action="store_true")
    args = ap.parse_args(argv)
    if not args.no_hip:
        print(build_hip())
    if args.hostcheck:
        print(build_hostcheck())


if __name__ == "__main__":
    main()
