"""Builds libratchet_hip.so for gfx950 with hipcc, in-tree.

    python -m ratchet_amd.build            # build if sources are newer than the library
    python -m ratchet_amd.build --force    # always rebuild

Objects go to ratchet_amd/_build/, the library to ratchet_amd/libratchet_hip.so.
hipcc cross-compiles without a GPU, so this runs anywhere ROCm is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "_build")
LIB = os.path.join(HERE, "libratchet_hip.so")
# measurement probes of bench.py --read-calibration: their own library, not part of the product
PROBES_SRC = "bench_probes.hip"
PROBES_LIB = os.path.join(HERE, "libratchet_probes.so")
ARCH = "gfx950"
# timing-only builds of the f16 tiled GEMM (bit mask: 1 no tile loads, 2 no MFMAs, 4 no fragment reads, 8 no output)
NT_ABLATIONS = (4, 7, 8, 9, 13, 14, 15)

SOURCES = ["api.cpp", "spec.cpp", "gguf.cpp", "kernels_blocks.hip", "kernels_softmax.hip", "kernels_unary.hip", "kernels_attention.hip", "kernels_gemv.hip", "kernels_gemv_mfma.hip", "kernels_gemv_rowdot.hip", "kernels_gemv_quad.hip", "kernels_gemv_rowfloat.hip",
    "kernels_gemv_q4k_mfma.hip", "kernels_gemv_q4k_rowdot.hip", "kernels_gemm.hip", "kernels_gemm_f32.hip", "kernels_gemm_q4k.hip",
    "kernels_gemm_nt.hip", "kernels_gemm_nn.hip", "kernels_gemm_stream.hip"]
HEADERS = ["spec.h", "device_common.h", os.path.join("..", "..", "include", "ratchet_hip.h")]

# -packed-fp32-ops is switched off on purpose: the compiler then never forms
# v_pk_{add,mul,fma}_f32 from scalar float code.
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators stay in ordinary VGPRs: with the AGPR form the register allocator
    # rotates the loop-carried accumulators of the tiled GEMMs through dozens of
    # v_accvgpr_mov per iteration.
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wall", "-Wno-unused-function", "-x", "hip",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, h) for h in HEADERS] + [os.path.abspath(__file__)]
    if force or _stale(obj, deps):
        cmd = [hipcc(), *FLAGS, "-DRT_BUILDING_LIB", "-c", os.path.join(CSRC, src), "-o", obj]
        res = subprocess.run(cmd, capture_output=True, text=True)
        # the host pass does not know the packed-fp32 feature and says so once per file
        err = "\n".join(l for l in res.stderr.splitlines() if "is not a recognized feature" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if err.strip():
            sys.stderr.write(err + "\n")
    return obj


def build_probes(force: bool = False) -> str:
    """libratchet_probes.so: bench_probes.hip plus one timing-only build of kernels_gemm_nt.hip per entry of
    NT_ABLATIONS (its namespace renamed, so the builds do not collide), for bench.py's calibration flags."""
    os.makedirs(OBJ, exist_ok=True)
    probes_src, nt_src = os.path.join(CSRC, PROBES_SRC), os.path.join(CSRC, "kernels_gemm_nt.hip")
    deps = [probes_src, nt_src, os.path.abspath(__file__)] + [os.path.join(CSRC, h) for h in HEADERS]
    if not (force or _stale(PROBES_LIB, deps)):
        return PROBES_LIB

    def one(job):
        src, obj, extra = job
        res = subprocess.run([hipcc(), *FLAGS, *extra, "-c", src, "-o", obj], capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {os.path.basename(src)} {' '.join(extra)}:\n{res.stderr}")
        return obj

    jobs = [(probes_src, os.path.join(OBJ, "bench_probes.o"), [])]
    for mask in NT_ABLATIONS:
        jobs.append((nt_src, os.path.join(OBJ, f"nt_ablation_{mask}.o"),
                     [f"-DRT_NT_ABLATION={mask}", f"-Drt=rt_nt_ablation_{mask}", f"-DRT_NT_ABL_ENTRY=probe_gemm_nt_ablation_{mask}"]))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        objs = list(ex.map(one, jobs))
    res = subprocess.run([hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", PROBES_LIB, *objs], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link of the probes failed:\n{res.stderr}")
    return PROBES_LIB


def build(force: bool = False, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    if force or _stale(LIB, objs):
        cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB, *objs]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stderr}")
    try:
        build_probes(force)
    except RuntimeError as e:  # measurement probes only: the product does not depend on them
        sys.stderr.write(f"warning: {e}\n")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
