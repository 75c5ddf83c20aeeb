"""Benchmark of the VQ-GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu] [--skip-traffic] [--only-main]
    python bench.py --launch-floor | --mfma-ceiling | --probe CONFIG     (measurement aids, no JSON)

One "step" is one fused VQ-GEMM launch over one weight matrix.  The headline workload is the
decode GEMV (M=1, K=4096, N=4096, 8-vectors, uint8 codes, one 256x8 codebook).  So that the
2 MB of codes really stream from HBM, the steps rotate over a pool of distinct code matrices
larger than the L2 and the 256 MB Infinity Cache; the launches are captured in HIP graphs so that
host launch overhead does not pace a microsecond-scale kernel, and timed with HIP events recorded
on the stream the kernels run on.  Inputs are resident in HBM before the timed region.  Whatever
--steps says, a cold configuration's timed region covers at least two full rotations of its pool
(`timed_launches` in the output; `ms_per_step` is per launch), and a device copy larger than the
caches runs between the untimed replay that uploads the graphs and the timed one.

Printed: ONE JSON line (rank 0).  `value` is the decode configuration's effective bandwidth:
the bytes an uncompressed fp16 GEMV would have had to stream (fp16 weights + X + Y) per
second.  `roofline` prices the same kernel against HBM peak on its *algorithmic* bytes (codes
+ codebook + X + Y); its `traffic` is what two `rocprofv3 --pmc` child runs of `--probe C2` count
after the timed region (FETCH_SIZE and WRITE_SIZE, scaled by a 256 MiB copy; `--skip-traffic`
leaves them out and reports the committed summary's figure).  Next to it: the hipBLASLt fp16 GEMM on the dequantised weights timed by
the same loop, the other measured configurations, and the reference math on the host CPU
(torch gather + fp32 matmul, all cores) on a bounded sample.

Counterpart of the reference harness bench.py:62-171 (same operator call, the accuracy and
determinism reports), with timing moved out of the kernel wrappers into the harness.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
FP16_MFMA_PEAK_TFLOPS = 2500.0
from vq_gemm_amd.timing import MIN_TIMED_LAUNCHES, POOL_BYTES  # the cold-HBM protocol's pool size and minimum count
# HBM bytes one cold decode launch moves: NOT measured by this program.  From rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE of `bench.py --probe C2`, scaled by a 256 MiB copy in the same run
# (1104.1 KiB x 2.0 read + 8 KiB written); the summary and its command are in the file named here.
PROFILED_C2_HBM_BYTES_PER_LAUNCH = 2_228_224
PROFILED_C2_TRAFFIC_SOURCE = "profiles/decode_gemv_wide_kernel_c2_decode_gemv.md"
# The same for the other configurations (name in `other_configs` -> bytes per launch, summary file): what the
# per-configuration `roofline` objects carry as `traffic`.  None where no counter run exists.
PROFILED_TRAFFIC = {
    "C3": (24_371_000, "profiles/decode_batched_kernel_c3_m16_mlp_up.md"),
    "decode_m1_k4096_n28672": (14_921_700, "profiles/decode_gemv_wide_kernel_m1_n28672.md"),
    "decode_m1_k8192_n28672": (29_657_000, "profiles/decode_gemv_wide_kernel_m1_n28672.md"),
    "decode_qkv_m1_k4096_n12288": (6_578_000, "profiles/decode_gemv_wide_kernel_m1_n28672.md"),
    "decode_m2_k4096_n28672": (15_187_968, "profiles/decode_gemv_wide_kernel_m2_two_rows_of_x.md"),
    "decode_down_m1_k14336_n4096": (7_692_288, "profiles/decode_gemv_wide_kernel_long_k_down_projection.md"),
    "decode_down_m1_k28672_n8192": (29_952_000, "profiles/decode_gemv_wide_kernel_long_k_down_projection.md"),
    "decode_down_m16_k14336_n4096": (11_270_000, "profiles/decode_stream_kernel_m16_k14336_n4096.md"),
    "C4": (85_373_000, "profiles/prefill_kernel_c4_prefill_gemm.md"),
    "C5": (489_400_000, "profiles/prefill_kernel_c5_m2048_k8192_n28672.md"),
}


def measured_traffic_bytes(probe: str = "C2", kernel: str = "decode_gemv", steps: int = 200):
    """HBM bytes per launch of `kernel` from two counter runs in child processes (FETCH_SIZE, WRITE_SIZE: KiB per dispatch),
    each scaled by what the same counter reads for the 256 MiB device copy at the end of the probe.  `kernel` = a piece of
    the kernel's name, or "vq" for every kernel of this library that the probe launches (a launch of several kernels:
    their sum per launch).  None when a run fails."""
    import csv, glob, shutil, statistics, subprocess, tempfile
    # (not under a profiler: its preloaded library would be inherited by the children)
    if any("rocprof" in v.lower() for k, v in os.environ.items() if k in ("LD_PRELOAD", "HSA_TOOLS_LIB", "ROCP_TOOL_LIBRARIES")) or \
            any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ):
        return None
    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    here = os.path.abspath(__file__)
    total = 0.0
    detail = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        out = tempfile.mkdtemp(prefix="vq_traffic_", dir="/tmp")
        try:
            cmd = [rocprof, "--pmc", counter, "--output-format", "csv", "-d", out, "-o", "p", "--", sys.executable, here,
                   "--probe", probe, "--steps", str(steps)]
            res = subprocess.run(cmd, cwd="/tmp", env=dict(os.environ, TMPDIR="/tmp"), stdout=subprocess.PIPE,
                                 stderr=subprocess.STDOUT, timeout=90)
            files = glob.glob(os.path.join(out, "**", "*counter_collection.csv"), recursive=True)
            if res.returncode != 0 or not files:
                return None
            kern, copy, by_name = [], [], {}
            with open(files[0]) as f:
                for row in csv.DictReader(f):
                    if row["Counter_Name"] != counter:
                        continue
                    name = row["Kernel_Name"]
                    if "copyBuffer" in name:
                        copy.append(float(row["Counter_Value"]))
                    elif kernel in name and "pack_codes" not in name:
                        kern.append(float(row["Counter_Value"]))
                        by_name.setdefault(name, []).append(float(row["Counter_Value"]))
            if not kern or not copy or max(copy) <= 0:
                return None
            factor = 262144.0 / max(copy)     # the copy moves 256 MiB each way: what one counted KiB stands for
            # one kernel per launch: the median dispatch; several: each kernel's median times its dispatches per launch
            kib = sum(statistics.median(v) * max(1, round(len(v) / steps)) for v in by_name.values())
            detail[counter] = {"kib_per_dispatch": kib, "copy_256MiB_reads": max(copy), "factor": factor, "dispatches": len(kern)}
            total += kib * factor * 1024.0
        except (OSError, subprocess.SubprocessError):
            return None
        finally:
            shutil.rmtree(out, ignore_errors=True)
    return int(total), detail


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-main", action="store_true", help="time only the headline decode configuration")
    ap.add_argument("--skip-traffic", action="store_true",
                    help="do not measure the roofline objects' traffic in this run (per configuration two child runs of "
                         "`rocprofv3 --pmc`, FETCH_SIZE and then WRITE_SIZE, on `bench.py --probe <configuration>`, each scaled by "
                         "the 256 MiB copy of the same run: about half a minute in all); the figures of the committed counter "
                         "summaries are reported instead, as they are when a child run fails or this command itself runs "
                         "under a profiler")
    ap.add_argument("--probe", metavar="CONFIG", default=None,
                    help="profiling aid (BLAS,C4 = hipBLASLt on the dequantised weights of C4): launch CONFIG (C1..C5, REF = the reference's own shape in its native layout, "
                         "a geometry-B shape M,K,N,vec,entries,code_bits, or GEMM,M,K,N = the plain fp16 GEMM) "
                         "--steps times, cold-HBM rotation for the decode configs, followed by one 256 MiB "
                         "device copy as a counter yardstick; prints no JSON")
    ap.add_argument("--probe-variant", type=int, default=0,
                    help="with --probe on a geometry-B shape: the VQGEMM_VARIANT_* value to launch (0 = automatic choice)")
    ap.add_argument("--probe-set", action="append", default=[], metavar="NAME=VALUE",
                    help="with --probe: set a constant of the tuning table first (a kernel parameter candidate, e.g. "
                         "gemv_wide_groups_in_flight=3), for counter runs on one candidate")
    ap.add_argument("--probe-skew", type=float, default=1.0,
                    help="with --probe on a geometry-B shape: codes = floor(entries * u^P) for uniform u; 1 = uniform codes (the "
                         "measured configurations), larger P concentrates the codes on few 'hot' entries (P = 4: half of all "
                         "codes fall on 6 %% of the entries) - for counter runs on what a skewed code distribution does to the gathers")
    ap.add_argument("--study", choices=["gated", "split-k", "code-usage"], default=None,
                    help="print one JSON report instead of the benchmark line: 'gated' times gate/up projection pairs as the "
                         "plain product + element-wise pass and as the gated entry point; 'split-k' times C3 whole and as "
                         "K slices with a summing pass behind them; 'code-usage' quantises Gaussian and heavy-tailed "
                         "weights with the package's k-means and reports how unevenly the entries are used")
    ap.add_argument("--probe-workspace", action="store_true",
                    help="with --probe on a geometry-B shape: launch through the entry point with a sized workspace "
                         "(vqgemm_e2e_gemm_b_ws), so that the automatic choice may split K")
    ap.add_argument("--probe-flat-codebook", action="store_true",
                    help="with --probe on a geometry-B shape: every entry of a codebook is a copy of its first entry, so that W is "
                         "constant whatever the codes are (the control for --probe-skew 1000: same W, but the gathers still go to "
                         "random entries)")
    ap.add_argument("--launch-floor", action="store_true",
                    help="run the empty-kernel launch probe (vq_gemm_amd/lib/launch_floor): what one launch of a replayed "
                         "HIP graph costs on this device when the kernel does nothing; prints no JSON")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="run the register-only MFMA loop (vq_gemm_amd/lib/mfma_ceiling): what the matrix cores "
                         "sustain on this device with random and with zero operands; prints no JSON")
    return ap.parse_args()


def mfma_ceiling_tflops():
    """TFLOP/s of the register-only v_mfma_f32_16x16x32_f16 loop with random operands (None if the tool is not built)."""
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vq_gemm_amd", "lib", "mfma_ceiling")
    if not os.path.exists(exe):
        return None
    try:
        text = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True, timeout=60).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    m = re.search(r"random operands, v_mfma_f32_16x16x32_f16: [\d.]+ us per launch, (\d+) TFLOP/s", text)
    return float(m.group(1)) if m else None


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures the single-GPU VQ-GEMM path; this build has no multi-GPU leg "
              "(the path shards along N without any exchange). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    if args.mfma_ceiling or args.launch_floor:
        import subprocess
        exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vq_gemm_amd", "lib",
                           "mfma_ceiling" if args.mfma_ceiling else "launch_floor")
        if not os.path.exists(exe):
            print(f"{exe} is not built (python -m vq_gemm_amd.build)", file=sys.stderr)
            sys.exit(2)
        sys.exit(subprocess.run([exe]).returncode)

    import torch

    from vq_gemm_amd import cabi
    from vq_gemm_amd.problems import CONFIGS, GEOM_B, ProblemSpec, make_problem

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = "cuda:0"
    torch.cuda.set_device(0)
    cabi.lib()      # fail loudly if the HIP library is missing
    cabi.ref_lib()

    def barrier():
        torch.cuda.synchronize()

    if args.probe:
        from vq_gemm_amd.problems import GEOM_A, GEOM_B, ProblemSpec
        for item in args.probe_set:
            name, value = item.split("=", 1)
            cabi.set_tuning(**{name: float(value)})
        if args.probe.startswith("GEMM,"):
            m, k, n = (int(v) for v in args.probe.split(",")[1:])
            g = torch.Generator().manual_seed(42)
            xa = torch.randn(m, k, generator=g).half().to(dev)
            wa = (torch.randn(k, n, generator=g) * 0.02).half().to(dev)
            ya = torch.empty(m, n, dtype=torch.float16, device=dev)
            barrier()
            for _ in range(args.steps):
                cabi.gemm_f16(xa, wa, out=ya)
            barrier()
            print(f"probe {args.probe}: {args.steps} launches of the plain GEMM", file=sys.stderr)
            return
        if args.probe.startswith("BLAS,"):
            # the hipBLASLt baseline on the dequantised weights of a configuration, for counter runs beside the fused kernel
            spec = CONFIGS[args.probe.split(",")[1]]
            x, codes, cb = make_problem(spec, seed=42, device=dev)
            wd = cabi.dequant_b(codes, cb)
            y = torch.empty(spec.M, spec.N, dtype=torch.float16, device=dev)
            cabi.ref_gemm_f16(x, wd, w_is_nk=True, out=y)   # (picks its algorithm)
            barrier()
            for _ in range(args.steps):
                cabi.ref_gemm_f16(x, wd, w_is_nk=True, out=y)
            barrier()
            print(f"probe {args.probe}: {args.steps} launches of hipBLASLt on the dequantised weights", file=sys.stderr)
            return
        if args.probe in CONFIGS:
            spec = CONFIGS[args.probe]
        else:
            fields = [int(v) for v in args.probe.split(",")]
            m, k, n, vec, entries, bits = fields[:6]
            spec = ProblemSpec("probe", GEOM_B, m, k, n, vec, entries, fields[6] if len(fields) > 6 else 1, bits)
        x, codes, cb = make_problem(spec, seed=42, device=dev)
        if args.probe_flat_codebook and spec.geometry == GEOM_B:
            cb3 = cb.view(-1, spec.entries, spec.vec)
            cb3.copy_(cb3[:, :1, :].expand_as(cb3).clone())
        if spec.geometry == GEOM_A:
            y = torch.empty(spec.M, spec.N, dtype=torch.float16, device=dev)
            barrier()
            for _ in range(args.steps):
                cabi.e2e_gemm_a(x, codes, cb, out=y)
            barrier()
            print(f"probe {args.probe}: {args.steps} launches, reference-native layout", file=sys.stderr)
            return
        n_bufs = max(1, min(512, POOL_BYTES // spec.code_bytes)) if spec.M <= 16 else 1
        gen = torch.Generator(device=dev).manual_seed(1234)
        def draw_codes():
            if args.probe_skew == 1.0:
                return torch.randint(0, spec.entries, spec.codes_shape, generator=gen, device=dev, dtype=torch.int32).to(spec.code_dtype)
            u = torch.rand(spec.codes_shape, generator=gen, device=dev)
            return (u.pow(args.probe_skew) * spec.entries).to(torch.int32).clamp_(0, spec.entries - 1).to(spec.code_dtype)
        pool = [codes if args.probe_skew == 1.0 else draw_codes()] + [draw_codes() for _ in range(n_bufs - 1)]
        if args.probe_variant == cabi.VARIANT_DECODE_PACKED:   # that variant reads code matrices re-laid offline
            pool = [cabi.pack_codes_b(c, spec.vec) for c in pool]
        y = torch.empty(spec.M, spec.N, dtype=torch.float16, device=dev)
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_()
        dst = torch.empty_like(src)
        barrier()
        if args.probe_workspace:
            need = cabi.workspace_bytes_b(spec.M, spec.K, spec.N, spec.vec, spec.entries, spec.n_codebooks, spec.code_bits)
            ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
            barrier()
            for i in range(args.steps):
                cabi.e2e_gemm_b_ws(x, pool[i % n_bufs], cb, out=y, workspace=ws)
        else:
            for i in range(args.steps):
                cabi.e2e_gemm_b(x, pool[i % n_bufs], cb, out=y, variant=args.probe_variant)
        barrier()
        dst.copy_(src)   # yardstick: reads 256 MiB, writes 256 MiB
        barrier()
        print(f"probe {args.probe}: {args.steps} launches over {n_bufs} code matrices, then one 256 MiB copy",
              file=sys.stderr)
        return

    # the cold-HBM timing protocol (rotating pool, graphs, events on the launch stream) lives in the package
    from vq_gemm_amd.timing import time_launches

    def bench_config(name, steps, warmup, cold_pool):
        spec = CONFIGS[name] if isinstance(name, str) else name
        x, codes, cb = make_problem(spec, seed=42, device=dev)
        n_bufs = max(1, min(512, POOL_BYTES // max(spec.code_bytes, 1))) if cold_pool else 1
        pool = [codes]
        gen = torch.Generator(device=dev).manual_seed(1234)
        for _ in range(n_bufs - 1):
            c = torch.randint(0, spec.entries, spec.codes_shape, generator=gen, device=dev, dtype=torch.int32)
            pool.append(c.to(spec.code_dtype))
        y = torch.empty(spec.M, spec.N, dtype=torch.float16, device=dev)
        # launches above ~50 us need no minimum count: --steps of them are a long enough region
        min_l = MIN_TIMED_LAUNCHES if spec.flops < 5e10 else 1
        t_cold, n_timed = time_launches(lambda i: cabi.e2e_gemm_b(x, pool[i], cb, out=y), n_bufs, steps, warmup, min_launches=min_l)
        t_warm = time_launches(lambda i: cabi.e2e_gemm_b(x, pool[0], cb, out=y), 1, steps, warmup, min_launches=min_l)[0] if cold_pool else t_cold
        # Baselines on the dequantised weights (a pool of them for the cold protocol), same loop:
        # hipBLASLt fp16 with the fastest of its heuristic answers for the shape, and torch's own linear.
        n_wbufs = max(1, min(n_bufs, POOL_BYTES * 2 // spec.dense_weight_bytes)) if cold_pool else 1
        wpool = [cabi.dequant_b(pool[i], cb) for i in range(n_wbufs)]
        t_blas = time_launches(lambda i: cabi.ref_gemm_f16(x, wpool[i], w_is_nk=True, out=y), n_wbufs, steps, warmup, min_launches=min_l)[0]
        t_torch = time_launches(lambda i: torch.nn.functional.linear(x, wpool[i]), n_wbufs, steps, warmup, min_launches=min_l)[0]
        t_base = min(t_blas, t_torch)
        res = {
            "M": spec.M, "K": spec.K, "N": spec.N, "vec": spec.vec, "code_bits": spec.code_bits,
            "entries": spec.entries, "n_codebooks": spec.n_codebooks,
            "variant": cabi.VARIANT_NAMES[cabi.select_variant_b(spec.M, spec.K, spec.N, spec.vec, spec.entries,
                                                                 spec.n_codebooks, spec.code_bits)],
            "us": t_cold * 1e6, "us_warm_cache": t_warm * 1e6,
            "tflops": spec.flops / t_cold / 1e12,
            "tflops_2p40": spec.flops / t_cold / 1024 ** 4,   # the reference's own divisor (strategy_1/src.cu:396)
            "algorithmic_gbps": spec.algorithmic_bytes / t_cold / 1e9,
            "effective_gbps": (spec.dense_weight_bytes + 2 * spec.M * (spec.K + spec.N)) / t_cold / 1e9,
            "hbm_roofline_frac": spec.algorithmic_bytes / t_cold / 1e9 / HBM_PEAK_GBPS,
            "mfma_roofline_frac": spec.flops / t_cold / 1e12 / FP16_MFMA_PEAK_TFLOPS,
            "hipblaslt_us": t_blas * 1e6, "hipblaslt_tflops": spec.flops / t_blas / 1e12,
            "hipblaslt_tuning": cabi.ref_tuning_info(spec.M, spec.K, spec.N, w_is_nk=True),
            "torch_linear_us": t_torch * 1e6,
            "speedup_vs_hipblaslt": t_blas / t_cold,
            "speedup_vs_fastest_baseline": t_base / t_cold,
            "code_buffers_rotated": n_bufs, "weight_buffers_rotated_by_baselines": n_wbufs,
            "steps": steps, "timed_launches": n_timed,
        }
        # The same launches on code matrices re-laid offline in the order the decode kernel's lanes
        # load them (vqgemm_pack_codes_b): beside the figures above, which stay on the plain
        # [N, K/vec] tensor of the reference's call.  (Where the K-sliced MFMA kernel is the one that
        # runs: the GEMV kernel of short single-row launches reads the plain matrix in whole runs.)
        dims = (spec.M, spec.K, spec.N, spec.vec, spec.entries, spec.n_codebooks, spec.code_bits)
        if cold_pool and res["variant"] == "decode" and cabi.decode_packed_supports(*dims):
            ppool = [cabi.pack_codes_b(c, spec.vec) for c in pool]
            launch_p = lambda i: cabi.e2e_gemm_b(x, ppool[i], cb, out=y, variant=cabi.VARIANT_DECODE_PACKED)
            tp_cold = time_launches(launch_p, n_bufs, steps, warmup)[0]
            tp_warm = time_launches(lambda i: launch_p(0), 1, steps, warmup)[0]
            y_plain = cabi.e2e_gemm_b(x, pool[0], cb, variant=cabi.VARIANT_DECODE).clone()
            res["prepacked_codes"] = {
                "us": tp_cold * 1e6, "us_warm_cache": tp_warm * 1e6,
                "algorithmic_gbps": spec.algorithmic_bytes / tp_cold / 1e9,
                "hbm_roofline_frac": spec.algorithmic_bytes / tp_cold / 1e9 / HBM_PEAK_GBPS,
                "speedup_vs_hipblaslt": t_blas / tp_cold,
                "bit_identical_to_plain_layout": bool(torch.equal(launch_p(0), y_plain)),
            }
            del ppool
        # run-to-run determinism, as the reference harness reports it (bench.py:118-132)
        y0 = cabi.e2e_gemm_b(x, codes, cb).clone()
        res["deterministic_5_runs"] = all(torch.equal(cabi.e2e_gemm_b(x, codes, cb), y0) for _ in range(4))
        del pool, wpool
        torch.cuda.empty_cache()
        return res, (x, codes, cb, y0)

    if args.study == "gated":
        # A gate/up pair of an MLP, H outputs each: before = one product [M, 2H] written to HBM, then the element-wise
        # pass reads it back; after = the gated entry point (epilogue inside the GEMM kernel where one applies).
        report = {}
        for name, M, K, H, G in (("prefill_m2048_k8192_h14336", 2048, 8192, 14336, 56), ("prefill_m2048_k4096_h11008", 2048, 4096, 11008, 43),
                                 ("prefill_m512_k4096_h11008", 512, 4096, 11008, 43), ("decode_m16_k4096_h11008", 16, 4096, 11008, 1),
                                 ("decode_m1_k4096_h14336", 1, 4096, 14336, 1), ("decode_m1_k8192_h14336", 1, 8192, 14336, 1),
                                 ("decode_m1_k4096_h11008", 1, 4096, 11008, 1)):
            spec = ProblemSpec(name, GEOM_B, M, K, 2 * H, 8, 256, G, 8)
            x, codes, cb = make_problem(spec, seed=42, device=dev)
            cold = M <= 16
            n_bufs = max(1, min(512, POOL_BYTES // spec.code_bytes)) if cold else 1
            gen = torch.Generator(device=dev).manual_seed(1234)
            pool = [codes] + [torch.randint(0, 256, spec.codes_shape, generator=gen, device=dev, dtype=torch.int32).to(torch.uint8)
                              for _ in range(n_bufs - 1)]
            prod = torch.empty(M, 2 * H, dtype=torch.float16, device=dev)
            y = torch.empty(M, H, dtype=torch.float16, device=dev)
            steps, warm, min_l = (200, 20, MIN_TIMED_LAUNCHES) if cold else (10, 3, 1)
            t_before = time_launches(lambda i: (cabi.e2e_gemm_b(x, pool[i], cb, out=prod), cabi.silu_mul(prod, out=y)),
                                     n_bufs, steps, warm, min_launches=min_l)[0]
            t_plain = time_launches(lambda i: cabi.e2e_gemm_b(x, pool[i], cb, out=prod), n_bufs, steps, warm, min_launches=min_l)[0]
            t_after = time_launches(lambda i: cabi.e2e_gemm_b_gated(x, pool[i], cb, out=y, workspace=prod), n_bufs, steps, warm,
                                    min_launches=min_l)[0]
            report[name] = {"M": M, "K": K, "H": H, "n_codebooks": G,
                            "product_then_elementwise_us": t_before * 1e6, "product_alone_us": t_plain * 1e6,
                            "gated_entry_point_us": t_after * 1e6, "speedup": t_before / t_after,
                            "plain_variant": cabi.VARIANT_NAMES[cabi.select_variant_b(M, K, 2 * H, 8, 256, G, 8)],
                            "cold_code_buffers": n_bufs}
            del pool, prod, y
            torch.cuda.empty_cache()
        print(json.dumps({"study": "gated", "shapes": report}))
        return

    if args.study == "split-k":
        # Would splitting K across workgroups pay on C3?  A split-K launch of S slices reads the same code bytes, gives every
        # workgroup 1/S of X to pull, and leaves S partial products to sum.  The slices are timed as what they are to the kernel,
        # an [M, K/S] x [S*N, K/S] problem (same code bytes, same number of row tiles x S), plus the summing pass over [S, M, N].
        spec = CONFIGS["C3"]
        report = {}
        for S in (1, 2, 4):
            sspec = ProblemSpec(f"C3/{S}", GEOM_B, spec.M, spec.K // S, spec.N * S, spec.vec, spec.entries, 1, spec.code_bits)
            x, codes, cb = make_problem(sspec, seed=42, device=dev)
            n_bufs = max(1, min(512, POOL_BYTES // sspec.code_bytes))
            gen = torch.Generator(device=dev).manual_seed(1234)
            pool = [codes] + [torch.randint(0, spec.entries, sspec.codes_shape, generator=gen, device=dev, dtype=torch.int32).to(sspec.code_dtype)
                              for _ in range(n_bufs - 1)]
            part = torch.empty(spec.M, spec.N * S, dtype=torch.float16, device=dev)
            ysum = torch.empty(spec.M, spec.N, dtype=torch.float16, device=dev)
            t_prod = time_launches(lambda i: cabi.e2e_gemm_b(x, pool[i], cb, out=part), n_bufs, 200, 20)[0]
            if S > 1:
                view = part.view(spec.M, S, spec.N)
                t_both = time_launches(lambda i: (cabi.e2e_gemm_b(x, pool[i], cb, out=part), torch.sum(view, dim=1, out=ysum)),
                                       n_bufs, 200, 20)[0]
            else:
                t_both = t_prod
            report[f"slices_{S}"] = {"K_per_slice": spec.K // S, "rows": spec.N * S, "product_us": t_prod * 1e6,
                                     "with_summing_pass_us": t_both * 1e6,
                                     "variant": cabi.VARIANT_NAMES[cabi.select_variant_b(spec.M, spec.K // S, spec.N * S, spec.vec,
                                                                                         spec.entries, 1, spec.code_bits)]}
            del pool, part, ysum
            torch.cuda.empty_cache()
        # The tiles of medium M: split K is built there (vqgemm_e2e_gemm_b_ws: 128x128 tiles, 2-8 workgroups per tile, the
        # last one sums the partial products).  The automatic choice without and with a workspace, and the baselines.
        tiles = {}
        for M, K, N, G in ((256, 4096, 4096, 32), (384, 4096, 4096, 32), (512, 4096, 4096, 32), (768, 4096, 4096, 32),
                           (256, 8192, 8192, 1), (512, 8192, 8192, 1), (256, 11008, 4096, 1), (2048, 4096, 1024, 8),
                           (128, 8192, 4096, 1), (512, 4096, 11008, 1)):
            tspec = ProblemSpec(f"m{M}_k{K}_n{N}", GEOM_B, M, K, N, 8, 256, G, 8)
            x, codes, cb = make_problem(tspec, seed=42, device=dev)
            y = torch.empty(M, N, dtype=torch.float16, device=dev)
            need = cabi.workspace_bytes_b(M, K, N, 8, 256, G, 8)
            ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
            wd = cabi.dequant_b(codes, cb)
            t_plain = time_launches(lambda i: cabi.e2e_gemm_b(x, codes, cb, out=y), 1, 40, 10, min_launches=1)[0]
            t_ws = time_launches(lambda i: cabi.e2e_gemm_b_ws(x, codes, cb, out=y, workspace=ws), 1, 40, 10, min_launches=1)[0]
            t_blas = time_launches(lambda i: cabi.ref_gemm_f16(x, wd, w_is_nk=True, out=y), 1, 40, 10, min_launches=1)[0]
            t_torch = time_launches(lambda i: torch.nn.functional.linear(x, wd), 1, 40, 10, min_launches=1)[0]
            tiles[tspec.name] = {"n_codebooks": G, "without_workspace_us": t_plain * 1e6,
                                 "without_workspace_variant": cabi.VARIANT_NAMES[cabi.select_variant_b(M, K, N, 8, 256, G, 8)],
                                 "workspace_bytes_wanted": need, "with_workspace_us": t_ws * 1e6,
                                 "hipblaslt_us": t_blas * 1e6, "torch_linear_us": t_torch * 1e6}
            del x, codes, cb, y, ws, wd
            torch.cuda.empty_cache()
        print(json.dumps({"study": "split-k", "decode_C3_emulated": report, "tiles_medium_m": tiles}))
        return

    if args.study == "code-usage":
        # How unevenly does a trained codebook use its entries?  A "hot entry" table only pays when few entries carry most codes.
        import numpy as np

        from vq_gemm_amd.quantize import kmeans_quantize
        torch.manual_seed(0)
        report = {}
        for name, w in (("gaussian", torch.randn(1024, 4096)),
                        ("student_t_3dof", torch.distributions.StudentT(3.0).sample((1024, 4096)))):
            q = kmeans_quantize(w.half().to(dev), 8, 256, 1, iters=10)
            h = np.bincount(q[0].cpu().numpy().astype(np.int64).ravel(), minlength=256).astype(np.float64)
            h = np.sort(h)[::-1] / h.sum()
            report[name] = {"share_of_16_most_used": h[:16].sum(), "share_of_32": h[:32].sum(), "share_of_64": h[:64].sum(),
                            "most_used_over_mean": h[0] * 256, "entropy_bits": float(-(h[h > 0] * np.log2(h[h > 0])).sum())}
        print(json.dumps({"study": "code-usage", "format": "8-vectors, 256 entries, 1024x4096 weights", "weights": report}))
        return

    # ---- headline: decode GEMV ---------------------------------------------------------------
    main_name = "C2"
    main_res, (x, codes, cb, y_gpu) = bench_config(main_name, args.steps, args.warmup, cold_pool=True)
    spec = CONFIGS[main_name]

    others = {}
    if not args.only_main:
        others["C3"], _ = bench_config("C3", max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        # a long run of tiles per workgroup: one token through a 70B-class MLP up-projection
        others["decode_m1_k8192_n28672"], _ = bench_config(
            ProblemSpec("decode_m1_k8192_n28672", GEOM_B, 1, 8192, 28672, 8, 256, 1, 8),
            max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        # a medium run of rows with one row of X: the streaming form of the GEMV kernel
        others["decode_m1_k4096_n28672"], _ = bench_config(
            ProblemSpec("decode_m1_k4096_n28672", GEOM_B, 1, 4096, 28672, 8, 256, 1, 8),
            max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        # what a decode stack launches for attention: q, k and v projections in one launch, one codebook each
        others["decode_qkv_m1_k4096_n12288"], _ = bench_config(
            ProblemSpec("decode_qkv_m1_k4096_n12288", GEOM_B, 1, 4096, 12288, 8, 256, 3, 8),
            max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        # two tokens through the same up-projection: the wide GEMV form with two rows of X
        others["decode_m2_k4096_n28672"], _ = bench_config(
            ProblemSpec("decode_m2_k4096_n28672", GEOM_B, 2, 4096, 28672, 8, 256, 1, 8),
            max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        # the down-projection behind such an MLP (K beyond what a lane's registers hold of x: rows worked through in pieces)
        others["decode_down_m1_k14336_n4096"], _ = bench_config(
            ProblemSpec("decode_down_m1_k14336_n4096", GEOM_B, 1, 14336, 4096, 8, 256, 1, 8),
            max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        others["decode_down_m1_k28672_n8192"], _ = bench_config(
            ProblemSpec("decode_down_m1_k28672_n8192", GEOM_B, 1, 28672, 8192, 8, 256, 1, 8),
            max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        # the same down-projection at a batch of sixteen: the streaming kernel of the K-sliced path
        others["decode_down_m16_k14336_n4096"], _ = bench_config(
            ProblemSpec("decode_down_m16_k14336_n4096", GEOM_B, 16, 14336, 4096, 8, 256, 1, 8),
            max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=True)
        others["C1"], _ = bench_config("C1", max(200, args.steps // 5), max(20, args.warmup // 5), cold_pool=False)
        others["C4"], _ = bench_config("C4", 40, 10, cold_pool=False)
        others["C5"], _ = bench_config("C5", 10, 3, cold_pool=False)

    # ---- the reference's own shape in its native layout, and the plain GEMM control ---------------
    native = None
    if not args.only_main:
        rspec = CONFIGS["REF"]
        xr_, wr_, cbr_ = make_problem(rspec, seed=42, device=dev)
        yr_ = torch.empty(rspec.M, rspec.N, dtype=torch.float16, device=dev)
        dec_ = torch.empty(rspec.K, rspec.N, dtype=torch.float16, device=dev)
        t_fused = time_launches(lambda i: cabi.e2e_gemm_a(xr_, wr_, cbr_, out=yr_), 1, 100, 50, min_launches=1)[0]
        t_two = time_launches(lambda i: cabi.e2e_gemm_a(xr_, wr_, cbr_, variant=cabi.VARIANT_TWOPASS, out=yr_,
                                                        workspace=dec_), 1, 100, 50, min_launches=1)[0]
        cabi.ref_gemm_f16(xr_, cabi.dequant_a(wr_, cbr_, out=dec_), out=yr_)   # (the baseline picks its algorithm outside the loop)
        t_lib = time_launches(lambda i: (cabi.dequant_a(wr_, cbr_, out=dec_), cabi.ref_gemm_f16(xr_, dec_, out=yr_)), 1, 100, 50,
                              min_launches=1)[0]
        g = torch.Generator().manual_seed(7)
        xa = torch.randn(4096, 4096, generator=g).half().to(dev)
        wa = (torch.randn(4096, 4096, generator=g) * 0.02).half().to(dev)
        ya = torch.empty(4096, 4096, dtype=torch.float16, device=dev)
        t_gemm = time_launches(lambda i: cabi.gemm_f16(xa, wa, out=ya), 1, 40, 10, min_launches=1)[0]
        t_gemm_lib = time_launches(lambda i: cabi.ref_gemm_f16(xa, wa, out=ya), 1, 40, 10, min_launches=1)[0]
        native = {
            "reference_shape": {"M": rspec.M, "K": rspec.K, "code_columns": rspec.N // 2, "layout": "w[K,Nc] uint8, codebook[Nc/4,256,2]",
                                "variant": cabi.VARIANT_NAMES[cabi.select_variant_a(rspec.M, rspec.K, rspec.N // 2)],
                                "us": t_fused * 1e6, "tflops": rspec.flops / t_fused / 1e12,
                                "two_pass_us": t_two * 1e6, "dequant_plus_hipblaslt_us": t_lib * 1e6},
            "plain_gemm_4096": {"us": t_gemm * 1e6, "tflops": 2 * 4096 ** 3 / t_gemm / 1e12,
                                "hipblaslt_us": t_gemm_lib * 1e6, "hipblaslt_tflops": 2 * 4096 ** 3 / t_gemm_lib / 1e12},
        }
        del xr_, wr_, cbr_, yr_, dec_, xa, wa, ya
        torch.cuda.empty_cache()

    # ---- CPU baseline: the reference math (gather + fp32 matmul) on the host cores -------------
    cpu = None
    if not args.skip_cpu:
        import numpy as np

        from oracle import torch_baseline
        from oracle import vq_oracle as vo

        xc, cc, cbc = x.cpu(), codes.cpu(), cb.cpu()
        budget_s, reps, t_total = 12.0, 0, 0.0   # about 12 s of CPU work
        best = float("inf")
        y_cpu = None
        while t_total < budget_s and reps < 5000:
            t0 = time.perf_counter()
            y_cpu = torch_baseline.vq_gemm_b(xc, cc, cbc)
            dt = time.perf_counter() - t0
            best = min(best, dt)
            t_total += dt
            reps += 1
        mean = t_total / reps
        e1, e2 = vo.rel_err(y_gpu.cpu().numpy(), y_cpu.numpy().astype(np.float64))
        cpu = {
            "value": (spec.dense_weight_bytes + 2 * spec.M * (spec.K + spec.N)) / mean / 1e9, "unit": "GB/s",
            "cores": torch.get_num_threads(), "host_cpu_count": os.cpu_count(), "kind": "port",
            "sample": f"{reps} full {main_name} GEMVs (dequant gather + fp32 matmul, torch CPU), {t_total:.1f} s; mean per step",
            "ms_per_step": mean * 1e3, "best_ms_per_step": best * 1e3,
            "gpu_vs_cpu_max_rel_err": e1, "gpu_vs_cpu_max_err_over_max": e2,
        }

    t = main_res["us"] * 1e-6
    out = {
        "metric": "vq_gemm_decode_effective_bandwidth",
        "value": main_res["effective_gbps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": t * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "timed_launches": main_res["timed_launches"],
        "config": {"workload": "C2 decode GEMV: M=1 K=4096 N=4096, vec 8, uint8 codes [4096,512], one fp16 codebook [256,8]; "
                               f"cold HBM: {main_res['timed_launches']} timed launches rotating over "
                               f"{main_res['code_buffers_rotated']} distinct code matrices "
                               f"({main_res['code_buffers_rotated'] * spec.code_bytes >> 20} MiB, every one read "
                               f"{main_res['timed_launches'] // main_res['code_buffers_rotated']} times or more, a pool apart), "
                               "caches emptied before the timed region, fp32 accumulate",
                   "kernel": main_res["variant"]},
        "roofline": {"bound": "hbm", "achieved": spec.algorithmic_bytes / t / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": spec.algorithmic_bytes / t / 1e9 / HBM_PEAK_GBPS,
                     "traffic": PROFILED_C2_HBM_BYTES_PER_LAUNCH, "traffic_from": PROFILED_C2_TRAFFIC_SOURCE,
                     "traffic_measured_in_this_run": False,
                     # the fraction rests on this run's launch time: HIP events on the launch stream around replayed
                     # graphs, not on a tracer's per-dispatch durations (those serialise the replay and read 6-20 % more)
                     "timing": "hip events around replayed hip graphs, cold code matrices",
                     "algorithmic_bytes_per_launch": spec.algorithmic_bytes,
                     "kernel_us": main_res["us"], "kernel_us_warm_cache": main_res["us_warm_cache"]},
        "cpu_baseline": cpu,
        "tflops": main_res["tflops"],
        "hipblaslt": {"us": main_res["hipblaslt_us"], "tflops": main_res["hipblaslt_tflops"],
                      "speedup_vs_hipblaslt": main_res["speedup_vs_hipblaslt"], "tuning": main_res["hipblaslt_tuning"],
                      "torch_linear_us": main_res["torch_linear_us"],
                      "speedup_vs_fastest_baseline": main_res["speedup_vs_fastest_baseline"]},
        "deterministic_5_runs": main_res["deterministic_5_runs"],
        "prepacked_codes": main_res.get("prepacked_codes"),
        "other_configs": others,
        "reference_layout_and_control": native,
        # the file of cost-model constants behind the automatic kernel choice (None: the compiled-in table)
        "tuning_file": cabi.tuning_file(),
    }
    # Every configuration carries the same evidence as the headline: which roofline bounds it, what it achieves against
    # the published peak on its algorithmic bytes or flops (the launch time is this run's, HIP events around replayed
    # graphs), and the HBM traffic a counter run measured (not this run: the summary file is named).
    if not args.skip_traffic:
        measured = measured_traffic_bytes()
        if measured:
            out["roofline"].update({"traffic": measured[0], "traffic_from": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, child runs of this command",
                                    "traffic_measured_in_this_run": True, "traffic_counters": measured[1]})
    for name, res in others.items():
        mfma_bound = res["variant"].startswith("prefill")
        traffic = PROFILED_TRAFFIC.get(name)
        res["roofline"] = {
            "bound": "mfma" if mfma_bound else "hbm",
            "achieved": res["tflops"] if mfma_bound else res["algorithmic_gbps"],
            "peak": FP16_MFMA_PEAK_TFLOPS if mfma_bound else HBM_PEAK_GBPS,
            "unit": "TFLOP/s" if mfma_bound else "GB/s",
            "frac": res["mfma_roofline_frac"] if mfma_bound else res["hbm_roofline_frac"],
            "traffic": traffic[0] if traffic else None, "traffic_from": traffic[1] if traffic else None,
            "traffic_measured_in_this_run": False, "kernel_us": res["us"],
        }
        if not args.skip_traffic:
            probe = name if name in CONFIGS else ",".join(str(v) for v in (res["M"], res["K"], res["N"], res["vec"], res["entries"],
                                                                            res["code_bits"], res["n_codebooks"]))
            measured = measured_traffic_bytes(probe, "vq", 20 if mfma_bound else 100)
            if measured:
                res["roofline"].update({"traffic": measured[0], "traffic_measured_in_this_run": True, "traffic_counters": measured[1],
                                        "traffic_from": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, child runs of this command"})
    if others:
        # what the matrix cores sustain on this device with random operands (register-only MFMA loop):
        # the ceiling the MFMA-bound configurations are to be read against, next to the nominal peak
        ceiling = mfma_ceiling_tflops()
        if ceiling:
            out["mfma_ceiling_random_operands_tflops"] = ceiling
            for res in others.values():
                if res["variant"].startswith("prefill"):
                    res["frac_of_mfma_ceiling"] = res["tflops"] / ceiling
    print(json.dumps(out))


if __name__ == "__main__":
    main()
