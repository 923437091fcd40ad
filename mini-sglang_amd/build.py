"""Build recipe for the gfx950 shared objects (no cmake, no JIT cache).

    python mini-sglang_amd/build.py            # build what is stale
    python mini-sglang_amd/build.py --force

Outputs (git-ignored, shipped to the GPU box by gpurun because they are in-tree):
    mini-sglang_amd/lib/libmsgl_hip.so    every kernel + host helpers   (include/msgl_hip.h)
    mini-sglang_amd/lib/libmsgl_comm.so   RCCL communicator             (links librccl)
    mini-sglang_amd/lib/libmsgl_gemm.so   projection GEMMs + tuner      (links libhipblaslt)
    mini-sglang_amd/lib/libmsgl_mix.so    sequence-mixing kernels       (include/msgl_mix.h; no library dependency)

`build_all(only=("mix", "gemm"))` builds a subset: a model needs the libraries its layers call, not all of them.

hipcc cross-compiles for gfx950 without a GPU, so this also runs in the build container.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
LIB = ROOT / "lib"
OBJ = ROOT / "build"
INCLUDE = ROOT.parent / "include"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
HIPCC = os.environ.get("HIPCC", str(ROCM / "bin" / "hipcc"))
ARCH = "gfx950"

HIP_SOURCES = [
    "host.cpp",
    "radix.cpp",
    "store_index.hip",
    "norm_rope_act.hip",
    "attn_decode.hip",
    "attn_prefill.hip",
    "sampling.hip",
    "gemm_skinny.hip",
    "gemm_rowstream.hip",
    "gemm_wstream.hip",
    "gemm_m256.hip",
    "gemm_g3.hip",
    "gemm_ro.hip",
    "comm_p2p.hip",
]
MIX_SOURCES = ["seqmix.hip", "mix_delta.hip", "mix_par.hip", "mix_scan.hip"]
COMM_SOURCES = ["comm.cpp"]
GEMM_SOURCES = ["gemm.cpp"]

COMMON_FLAGS = [
    "-O3",
    "-std=c++17",
    "-fPIC",
    f"--offload-arch={ARCH}",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-inline-asm",
    "-I",
    str(INCLUDE),
]
if os.environ.get("MSGL_PREFILL_DIAG") == "1":  # timing-only ablation variants of the prefill kernels (tools/prefill_ablate.py)
    COMMON_FLAGS.append("-DMSGL_PREFILL_DIAG")


def _stale(out: Path, deps: list[Path]) -> bool:
    if not out.exists():
        return True
    t = out.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps if d.exists())


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + proc.stderr)
        raise RuntimeError(f"build step failed: {cmd[-1]}")
    if proc.stderr.strip():
        sys.stderr.write(proc.stderr)


# fp32 arithmetic stays scalar in the sequence-mixing kernels: no packed two-lane fp32 instructions (a device-pass flag;
# the host pass says it does not know the feature, which is harmless)
MIX_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ / (src.name + ".o")
    headers = list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h"))
    if force or _stale(obj, [src] + headers):
        extra = MIX_FLAGS if src.name in MIX_SOURCES else []
        _run([HIPCC, *COMMON_FLAGS, *extra, "-x", "hip", "-c", str(src), "-o", str(obj)])
    return obj


def build_all(force: bool = False, verbose: bool = True, only=None) -> dict[str, Path]:
    """Build the shared objects named in `only` (default: all of "hip", "mix", "comm", "gemm")."""
    want = set(only) if only else {"hip", "mix", "comm", "gemm"}
    LIB.mkdir(exist_ok=True)
    OBJ.mkdir(exist_ok=True)

    def srcs(key, names):
        return [CSRC / s for s in names if (CSRC / s).exists()] if key in want else []

    hip_srcs, mix_srcs = srcs("hip", HIP_SOURCES), srcs("mix", MIX_SOURCES)
    comm_srcs, gemm_srcs = srcs("comm", COMM_SOURCES), srcs("gemm", GEMM_SOURCES)
    groups = [hip_srcs, mix_srcs, comm_srcs, gemm_srcs]
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), [s for g in groups for s in g]))
    cut = [0]
    for g in groups:
        cut.append(cut[-1] + len(g))
    hip_objs, mix_objs, comm_objs, gemm_objs = (objs[cut[i]: cut[i + 1]] for i in range(4))
    out = {}
    # --no-undefined: a kernel whose host-side launch stub went missing must fail HERE, not at dlopen on the GPU box
    if hip_objs:
        lib_hip = LIB / "libmsgl_hip.so"
        if force or _stale(lib_hip, hip_objs):
            _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wl,--no-undefined", *map(str, hip_objs), "-o", str(lib_hip)])
        out["hip"] = lib_hip
    if mix_objs:
        lib_mix = LIB / "libmsgl_mix.so"
        if force or _stale(lib_mix, mix_objs):
            _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-Wl,--no-undefined", *map(str, mix_objs), "-o", str(lib_mix)])
        out["mix"] = lib_mix
    if comm_objs:
        lib_comm = LIB / "libmsgl_comm.so"
        if force or _stale(lib_comm, comm_objs):
            _run([HIPCC, "-shared", "-fPIC", *map(str, comm_objs), "-L", str(ROCM / "lib"), "-lrccl",
                  f"-Wl,-rpath,{ROCM / 'lib'}", "-o", str(lib_comm)])
        out["comm"] = lib_comm
    if gemm_objs:
        lib_gemm = LIB / "libmsgl_gemm.so"
        if force or _stale(lib_gemm, gemm_objs):
            _run([HIPCC, "-shared", "-fPIC", *map(str, gemm_objs), "-L", str(ROCM / "lib"), "-lhipblaslt",
                  f"-Wl,-rpath,{ROCM / 'lib'}", "-o", str(lib_gemm)])
        out["gemm"] = lib_gemm
    if verbose:
        for k, v in out.items():
            print(f"[build] {k}: {v} ({v.stat().st_size >> 10} KiB)")
    return out


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
