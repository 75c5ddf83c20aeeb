"""Build driver: hipcc --offload-arch=gfx950 only, everything in-tree.

Artefacts (all under vq_gemm_amd/lib/):
  libvqgemm.so        the C-ABI library (HIP kernels + dispatch), no torch dependency
  libvqgemm_ref.so    hipBLASLt fp16 baseline
  mfma_ceiling        stand-alone program: what a register-only MFMA loop sustains on the device
  launch_floor        stand-alone program: what an empty kernel costs per launch in a replayed graph
  vq_gemm_cuda_<k>.so one torch extension module per variant, named as the reference's
                      harness imports them (reference compile_kernels.py:55-68, bench.py:6-11)

The torch modules are built from one host-only C++ file (csrc/bind.cpp) with the host
compiler and linked against libvqgemm.so; no source passes through hipify.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(REPO_ROOT, "build", "obj")

ARCH = "gfx950"
HIPCC = os.environ.get("HIPCC", shutil.which("hipcc") or "/opt/rocm/bin/hipcc")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

KERNEL_SOURCES = ["vq_api.hip", "vq_dequant.hip", "vq_encode.hip", "vq_generic.hip", "vq_decode.hip", "vq_decode_gemv.hip", "vq_decode_stream.hip", "vq_decode_general.hip", "vq_prefill.hip",
                  "vq_prefill_small.hip", "vq_gemm_plain.hip", "vq_gemm_tiled.hip", "vq_epilogue.hip", "vq_check.hip", "vq_noalloc.hip"]

# sources with no kernel of their own (argument validation and dispatch)
HOST_ONLY_SOURCES = {"vq_api.hip", "vq_noalloc.hip"}

# -packed-fp32-ops: keep the compiler from forming packed fp32 VALU ops.
HIP_FLAGS = ["-O3", f"--offload-arch={ARCH}", "-fPIC", "-std=c++17", "-fno-gpu-rdc",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]

# The decode kernels are short launches, and a wave's first instruction there is a fetch of its kernel arguments from a
# cold scalar cache: gfx950 can hand the first arguments to a wave in scalar registers at launch (at most 14 dwords beside
# the two of the argument pointer).  The kernels of these sources take their arguments in the order they need them.
KERNARG_PRELOAD_SOURCES = {"vq_decode_gemv.hip"}
KERNARG_PRELOAD_FLAGS = ["-mllvm", "-amdgpu-kernarg-preload-count=14"]

# variant key -> (VQGEMM_VARIANT_* value, is the hipBLASLt baseline module)
# The keys are the reference's strategy names: s1 is its two-pass strategy
# (strategy_1/src.cu:323-399); s2_*/s3_* are its fused strategies, all served here by the
# shape-selected fused kernels.
VARIANTS = {
    "cublas_gemm": (0, True),
    "s1": (4, False),
    "s2_128": (0, False),
    "s2_512": (0, False),
    "s3_naive": (0, False),
    "s3_wasp": (0, False),
}


def module_name(key: str) -> str:
    return f"vq_gemm_cuda_{key}"


def _run(cmd, quiet=True):
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    if out.strip() and not quiet:
        print(out)
    return out


def _newer(target: str, deps) -> bool:
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps)


# Several kernels issue loads by inline assembly and wait for them by hand: they keep values in
# registers that the hardware is still writing; the compiler does not know, so a register it spills
# in that window would save stale data.  The MFMA kernels pin their accumulators in AGPRs and
# budget the rest by hand; a spill there means the budget was missed.  No kernel of this library
# has a reason to spill or to use scratch memory, so every kernel of every source is checked:
# zero VGPR spills and zero bytes of private segment.  (A scalar register that the compiler parks in a lane
# of a vector register - an "SGPR spill" that never touches memory - is tolerated in small numbers: it costs
# one lane write and read outside the hand-scheduled loops.)
MAX_SGPR_SPILLS = 4


def _check_no_spills(asm_path: str) -> None:
    name, bad, seen = None, [], 0
    with open(asm_path) as f:
        for line in f:
            line = line.strip()
            if line.startswith(".name:"):
                name = line.split(":", 1)[1].strip()
                seen += 1
            elif name and line.startswith((".vgpr_spill_count:", ".private_segment_fixed_size:")):
                if int(line.split(":")[1]) != 0:
                    bad.append(f"{name}: {line}")
            elif name and line.startswith(".sgpr_spill_count:"):
                if int(line.split(":")[1]) > MAX_SGPR_SPILLS:
                    bad.append(f"{name}: {line}")
    if seen == 0:
        raise RuntimeError(f"{asm_path}: no kernel metadata found, the spill check did not run")
    if bad:
        raise RuntimeError("register spills / scratch in a kernel that must have none:\n" + "\n".join(bad))


def _headers():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    inc = os.path.join(REPO_ROOT, "include")
    hs += [os.path.join(inc, f) for f in os.listdir(inc) if f.endswith(".h")]
    return hs


def build_lib(force: bool = True, jobs: int = 6) -> str:
    """Compile the HIP kernels and link libvqgemm.so."""
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    hdrs = _headers()
    objs = []

    def compile_one(src):
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
        if force or not _newer(o, [s] + hdrs):
            extra = KERNARG_PRELOAD_FLAGS if src in KERNARG_PRELOAD_SOURCES else []
            _run([HIPCC] + HIP_FLAGS + extra + ["--save-temps=obj", "-c", s, "-o", o])
            if src not in HOST_ONLY_SOURCES:
                _check_no_spills(o.replace(".o", f"-hip-amdgcn-amd-amdhsa-{ARCH}.s"))
        return o

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, KERNEL_SOURCES))
    out = os.path.join(LIB_DIR, "libvqgemm.so")
    _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc", "-o", out] + objs)
    return out


def build_ref(force: bool = True) -> str:
    """hipBLASLt baseline library."""
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(CSRC, "ref_gemm_hipblaslt.cpp")
    out = os.path.join(LIB_DIR, "libvqgemm_ref.so")
    if force or not _newer(out, [src] + _headers()):
        _run([HIPCC, "-O2", "-fPIC", "-std=c++17", "-shared", "-D__HIP_PLATFORM_AMD__", src, "-o", out,
              f"-L{ROCM}/lib", "-lhipblaslt", "-lamdhip64", f"-Wl,-rpath,{ROCM}/lib"])
    return out


def build_ceiling(force: bool = True) -> str:
    """Register-only MFMA loop (csrc/mfma_ceiling.hip), run by `bench.py --mfma-ceiling`."""
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(CSRC, "mfma_ceiling.hip")
    out = os.path.join(LIB_DIR, "mfma_ceiling")
    if force or not _newer(out, [src]):
        _run([HIPCC] + [f for f in HIP_FLAGS if f != "-fPIC"] + [src, "-o", out])
    return out


def build_launch_floor(force: bool = True) -> str:
    """Empty-kernel launch cost in a replayed graph (csrc/launch_floor.hip), run by `bench.py --launch-floor`."""
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(CSRC, "launch_floor.hip")
    out = os.path.join(LIB_DIR, "launch_floor")
    if force or not _newer(out, [src]):
        _run([HIPCC] + [f for f in HIP_FLAGS if f != "-fPIC"] + [src, "-o", out])
    return out


def build_ext(keys=None, force: bool = True, jobs: int = 6):
    """Torch extension modules, one per variant key (host C++ only)."""
    import torch  # noqa: F401  (needed for its include/lib paths)
    from torch.utils import cpp_extension as ce

    keys = list(VARIANTS) if keys is None else list(keys)
    for k in keys:
        if k not in VARIANTS:
            raise KeyError(f"unknown kernel variant {k!r}; known: {', '.join(VARIANTS)}")
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(CSRC, "bind.cpp")
    cxx = os.environ.get("CXX", "g++")
    torch_lib = ce.library_paths()[0]
    incs = [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}", f"-I{ROCM}/include"]
    abi = int(getattr(__import__("torch")._C, "_GLIBCXX_USE_CXX11_ABI", True))
    hdrs = _headers()

    def one(k):
        variant, is_ref = VARIANTS[k]
        name = module_name(k)
        out = os.path.join(LIB_DIR, name + ".so")
        if not force and _newer(out, [src] + hdrs):
            return out
        cmd = [cxx, "-O2", "-fPIC", "-shared", "-std=c++17", "-Wall", "-Wno-unused-function",
               "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
               f"-DTORCH_EXTENSION_NAME={name}", "-DTORCH_API_INCLUDE_EXTENSION_H", f"-DVQ_VARIANT={variant}"]
        if is_ref:
            cmd.append("-DVQ_REF_MODULE=1")
        cmd += incs + [src, "-o", out, f"-L{LIB_DIR}"] + (["-lvqgemm_ref"] if is_ref else ["-lvqgemm"]) + [
                       f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python",
                       "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
        _run(cmd)
        return out

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        return list(ex.map(one, keys))


def build_all(keys=None, force: bool = True):
    lib = build_lib(force=force)
    ref = build_ref(force=force)
    ceiling = build_ceiling(force=force)
    floor = build_launch_floor(force=force)
    exts = build_ext(keys, force=force)
    return [lib, ref, ceiling, floor] + exts


if __name__ == "__main__":
    for path in build_all(force="--incremental" not in sys.argv):
        print(path)
