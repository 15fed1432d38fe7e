"""Builds ``tannic_amd/csrc/libtannic_hip.so`` with hipcc for gfx950.

``python -m tannic_amd.build`` compiles every translation unit (in parallel)
and links the shared library in-tree, next to the sources.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(CSRC, "libtannic_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# Elementwise results are compared bit for bit with a CPU that does not fuse
# multiply-add, so those units are compiled without contraction.
EXACT = ["-ffp-contract=off"]

# (source, object name, extra flags)
UNITS = [
    ("runtime.hip", "runtime.o", []),
    ("unary.hip", "unary.o", EXACT),
    ("binary.hip", "binary_add.o", EXACT + ["-DTH_BINARY_ONLY=0"]),
    ("binary.hip", "binary_sub.o", EXACT + ["-DTH_BINARY_ONLY=1"]),
    ("binary.hip", "binary_mul.o", EXACT + ["-DTH_BINARY_ONLY=2"]),
    ("binary.hip", "binary_pow.o", EXACT + ["-DTH_BINARY_ONLY=3"]),
    ("misc.hip", "misc.o", EXACT),
    ("extended.hip", "extended_pairs.o", EXACT + ["-DTH_EXTENDED_ONLY=0"]),
    ("extended.hip", "extended_cast.o", EXACT + ["-DTH_EXTENDED_ONLY=1"]),
    ("rows.hip", "rows.o", []),
    ("reduce.hip", "reduce.o", []),
    ("shape_ops.hip", "shape_ops.o", []),
    ("gemm.hip", "gemm.o", []),
    ("gemm_mfma.hip", "gemm_mfma.o", []),
    ("gemm_skinny.hip", "gemm_skinny.o", []),
    ("gemm_small.hip", "gemm_small.o", []),
    ("gemm_f64.hip", "gemm_f64.o", []),
    ("gemm_rows_nn.hip", "gemm_rows_nn.o", []),
    ("gemm_repack.hip", "gemm_repack.o", []),
    ("gemm_dtl.hip", "gemm_dtl.o", ["-DTH_DTL_PART=0"]),
    ("gemm_dtl.hip", "gemm_dtl_krows_f16.o", ["-DTH_DTL_PART=1"]),
    ("gemm_dtl.hip", "gemm_dtl_krows_bf16.o", ["-DTH_DTL_PART=2"]),
    ("probes.hip", "probes.o", []),
    ("conv2d.hip", "conv2d.o", []),
    ("conv2d_mfma.hip", "conv2d_mfma.o", []),
    ("conv2d_patch.hip", "conv2d_patch.o", []),
    ("conv2d_resident.hip", "conv2d_resident.o", []),
    ("conv2d_k3.hip", "conv2d_k3.o", ["-DTH_K3_PART=0"]),
    ("conv2d_k3.hip", "conv2d_k5.o", ["-DTH_K3_PART=1"]),
    ("conv2d_k1.hip", "conv2d_k1.o", []),
    ("conv2d_pointwise.hip", "conv2d_pointwise.o", []),
    ("conv2d_stem.hip", "conv2d_stem.o", []),
    ("conv2d_gather32.hip", "conv2d_gather32.o", []),
    ("conv2d_unfold.hip", "conv2d_unfold.o", []),
    ("conv2d_unfold_batch.hip", "conv2d_unfold_batch.o", []),
]


def _headers():
    found = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    found.append(os.path.join(HERE, "..", "include", "tannic_hip.h"))
    return found


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def _compile(unit, force):
    src, obj, extra = unit
    src_path, obj_path = os.path.join(CSRC, src), os.path.join(OBJ, obj)
    if not force and not _stale(obj_path, [src_path] + _headers()):
        return obj_path, ""
    cmd = [HIPCC] + FLAGS + extra + ["-c", src_path, "-o", obj_path]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{log}")
    return obj_path, log


def build(force=True, jobs=None, verbose=False):
    """Compiles all units (``force`` recompiles even up-to-date objects) and links."""
    os.makedirs(OBJ, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda u: _compile(u, force), UNITS))
    for _, log in results:
        if verbose and log.strip():
            print(log)
    objects = [o for o, _ in results]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objects
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stdout + proc.stderr)
    return LIB


if __name__ == "__main__":
    print(build(force="--incremental" not in sys.argv, verbose=True))
