"""Builds the extension modules, one per kernel variant, with hipcc --offload-arch=gfx950 only.

Counterpart of the reference's compile_kernels.py:9-68: the KERNELS environment variable
("all" or a comma list of cublas_gemm, s1, s2_128, s2_512, s3_naive, s3_wasp) selects which
vq_gemm_cuda_<k> modules are produced; setuptools-style arguments such as
`build_ext --inplace` are accepted and ignored (everything is always built in-tree, under
vq_gemm_amd/lib/).  The HIP kernels are compiled directly by hipcc and the host binding by
the host C++ compiler: no source passes through hipify.

    KERNELS=s2_128 python compile_kernels.py build_ext --inplace
"""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from vq_gemm_amd import build  # noqa: E402


def main():
    sel = os.getenv("KERNELS", "all")
    keys = list(build.VARIANTS) if sel == "all" else [k.strip() for k in sel.split(",") if k.strip()]
    unknown = [k for k in keys if k not in build.VARIANTS]
    if unknown:
        raise SystemExit(f"unknown KERNELS entries {unknown}; known: {', '.join(build.VARIANTS)}")
    incremental = "--incremental" in sys.argv
    print(build.build_lib(force=not incremental))
    print(build.build_ref(force=not incremental))
    for path in build.build_ext(keys, force=not incremental):
        print(path)


if __name__ == "__main__":
    main()
