"""Times every kernel variant on one geometry-B shape and shows what the automatic choice picks:

    python -m vq_gemm_amd.tune [--cold] M K N [vec entries codebooks code_bits]

(`--cold`: every launch reads a code matrix that comes from HBM - the rotating pool of `vq_gemm_amd.timing` - instead
of one that sits in the caches)

or measures the box at hand and refits the constants of the cost models behind the automatic choice:

    python -m vq_gemm_amd.tune --fit [--search] [--write [PATH]]
    python -m vq_gemm_amd.tune --search [--write [PATH]]

`--search` tries the candidates of the kernels' run-time parameters - rows per group and groups of codes in flight
of the wide GEMV kernel, plain against bank-replicated table, the limits between the GEMV kernels and the K-sliced
decode kernels, the tile count from which the batched decode kernel replicates its table - on codes that come from
HBM (the rotating-pool protocol of `vq_gemm_amd.timing`, the one `bench.py` times with), and keeps the winners.
A counter run on one candidate: `rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_WAIT_ANY -- python3 bench.py --probe
M,K,N,vec,entries,bits --probe-set name=value` launches the shape with that constant set.

`--fit` times forced variants on a fixed set of shapes (per-stage and per-tile times come out of pairs of
shapes that differ in K or in the number of tiles), prints the fitted constants next to the compiled-in
ones, and with `--write` stores them as a flat JSON object (default: vq_gemm_amd/tuning.json) that
`vq_gemm_amd.cabi` hands to the library at its next load (`VQGEMM_TUNING_FILE`, `vqgemm_tuning_load`).
The same run under `rocprofv3 --kernel-trace --stats -- python3 -m vq_gemm_amd.tune --fit` gives the
per-kernel durations behind every figure.

The choice between the kernels rests on cost models fitted to measurements on one MI355X; this
prints, for the box at hand, the time of each variant that accepts the shape (launches replayed
from a HIP graph), the variant `VQGEMM_VARIANT_AUTO` resolves to, its distance from the fastest,
and the hipBLASLt fp16 GEMM on the dequantised weights beside them.  Inputs are synthetic
(X ~ N(0,1), uniform codes, codebooks ~ N(0, 0.02)), as in the bench.
"""
from __future__ import annotations

import sys

import torch

from . import cabi
from .problems import GEOM_B, ProblemSpec, make_problem


def time_graph(fn, launches: int = 20, repeats: int = 3) -> float:
    """Microseconds per launch of `fn`, replayed from a HIP graph on a side stream (default priority)."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(3):
            fn()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(launches):
                fn()
        graph.replay()
        stream.synchronize()
        best = float("inf")
        for _ in range(repeats):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            e1.synchronize()
            best = min(best, e0.elapsed_time(e1) / launches * 1e3)
    return best


def tune_cold(M: int, K: int, N: int, vec: int = 8, entries: int = 256, n_codebooks: int = 1, code_bits: int = 8,
              device: str = "cuda:0", verbose: bool = True) -> dict:
    """Microseconds per launch of every variant that takes the shape, on codes that come from HBM."""
    times = {}
    for variant in (cabi.VARIANT_AUTO, cabi.VARIANT_DECODE, cabi.VARIANT_DECODE_GEMV, cabi.VARIANT_PREFILL, cabi.VARIANT_PREFILL_NARROW,
                    cabi.VARIANT_PREFILL_SMALL):
        t = _cold_us(M, K, N, variant, vec=vec, entries=entries, n_codebooks=n_codebooks, code_bits=code_bits, device=device)
        if t is not None:
            times[cabi.VARIANT_NAMES[variant]] = t
    picked = cabi.VARIANT_NAMES[cabi.select_variant_b(M, K, N, vec, entries, n_codebooks, code_bits)]
    if verbose:
        print(f"M={M} K={K} N={N} vec={vec} entries={entries} codebooks={n_codebooks} code_bits={code_bits}, cold code matrices")
        for v, t in times.items():
            print(f"  {v:15s} {t:9.2f} us")
        print(f"  automatic choice: {picked}")
    return {"times_us": times, "auto_picks": picked}


def tune(M: int, K: int, N: int, vec: int = 8, entries: int = 256, n_codebooks: int = 1, code_bits: int = 8,
         device: str = "cuda:0", verbose: bool = True) -> dict:
    spec = ProblemSpec("tune", GEOM_B, M, K, N, vec, entries, n_codebooks, code_bits)
    x, codes, cb = make_problem(spec, seed=1, device=device)
    y = torch.empty(M, N, dtype=torch.float16, device=device)
    workspace = torch.empty(N, K, dtype=torch.float16, device=device)
    times = {}
    # a first untimed pass of the heaviest variant brings the device out of its idle clocks
    cabi.e2e_gemm_b(x, codes, cb, out=y, variant=cabi.VARIANT_TWOPASS, workspace=workspace)
    torch.cuda.synchronize()
    for variant in (cabi.VARIANT_DECODE, cabi.VARIANT_DECODE_GEMV, cabi.VARIANT_PREFILL, cabi.VARIANT_PREFILL_NARROW, cabi.VARIANT_PREFILL_SMALL,
                    cabi.VARIANT_TWOPASS, cabi.VARIANT_AUTO):
        try:
            times[variant] = time_graph(lambda: cabi.e2e_gemm_b(x, codes, cb, out=y, variant=variant, workspace=workspace))
        except cabi.VqGemmError as e:
            if e.code != -4:   # anything but "this variant does not take the shape"
                raise
    # split K over the 128x128 tiles, and the automatic choice when it is given a workspace to split K with
    need = cabi.workspace_bytes_b(M, K, N, vec, entries, n_codebooks, code_bits, cabi.VARIANT_PREFILL_SPLITK)
    if need > 0:
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        times[cabi.VARIANT_PREFILL_SPLITK] = time_graph(
            lambda: cabi.e2e_gemm_b_ws(x, codes, cb, out=y, variant=cabi.VARIANT_PREFILL_SPLITK, workspace=ws))
    auto_need = cabi.workspace_bytes_b(M, K, N, vec, entries, n_codebooks, code_bits)
    w = cabi.dequant_b(codes, cb)
    t_lib = time_graph(lambda: cabi.ref_gemm_f16(x, w, w_is_nk=True, out=y))
    picked = cabi.select_variant_b(M, K, N, vec, entries, n_codebooks, code_bits)
    forced = {v: t for v, t in times.items() if v != cabi.VARIANT_AUTO}
    fastest = min(forced, key=forced.get)
    if auto_need > 0:   # with a workspace the automatic choice splits K here
        picked = cabi.VARIANT_PREFILL_SPLITK
        times[cabi.VARIANT_AUTO] = times[cabi.VARIANT_PREFILL_SPLITK]
    result = {"times_us": {cabi.VARIANT_NAMES[v]: t for v, t in times.items()}, "auto_picks": cabi.VARIANT_NAMES[picked],
              "fastest": cabi.VARIANT_NAMES[fastest], "auto_over_fastest": times[cabi.VARIANT_AUTO] / forced[fastest],
              "hipblaslt_us": t_lib}
    if verbose:
        print(f"M={M} K={K} N={N} vec={vec} entries={entries} codebooks={n_codebooks} code_bits={code_bits}")
        for v, t in times.items():
            print(f"  {cabi.VARIANT_NAMES[v]:15s} {t:9.1f} us  {spec.flops / t / 1e6:8.1f} TFLOP/s")
        print(f"  {'hipBLASLt fp16':15s} {t_lib:9.1f} us  (on the dequantised weights)")
        print(f"  automatic choice: {result['auto_picks']} (the prefill variant chooses its tile itself); fastest forced "
              f"variant: {result['fastest']}; automatic / fastest = {result['auto_over_fastest']:.2f}")
    return result


def _t(M, K, N, variant, vec=8, entries=256, n_codebooks=1, code_bits=8, device="cuda:0"):
    """Microseconds of one forced variant on one shape (None when the variant refuses it)."""
    spec = ProblemSpec("fit", GEOM_B, M, K, N, vec, entries, n_codebooks, code_bits)
    x, codes, cb = make_problem(spec, seed=1, device=device)
    y = torch.empty(M, N, dtype=torch.float16, device=device)
    try:
        return time_graph(lambda: cabi.e2e_gemm_b(x, codes, cb, out=y, variant=variant))
    except cabi.VqGemmError as e:
        if e.code != -4:
            raise
        return None


def fit(device: str = "cuda:0", verbose: bool = True) -> dict:
    """Measures forced variants on shape pairs and returns the cost-model constants they imply for this box.
    Constants whose measurement fails (a variant that refuses the shape) keep their current value."""
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    cur = cabi.tuning()
    out = dict(cur)
    say = print if verbose else (lambda *a, **k: None)

    def pair(variant, M, N, k1, k2, **kw):
        """(fixed microseconds, microseconds per 64-k stage) out of two K."""
        t1, t2 = _t(M, k1, N, variant, **kw), _t(M, k2, N, variant, **kw)
        if t1 is None or t2 is None:
            return None
        stage = (t2 - t1) / ((k2 - k1) / 64.0)
        return t1 - stage * k1 / 64.0, stage

    # prefill, 256x256 tiles on a full device (one tile per unit): fixed part and per-stage time
    n_side = 256 * int(cus ** 0.5)
    r = pair(cabi.VARIANT_PREFILL, n_side, n_side, 2048, 4096, n_codebooks=n_side // 128)
    if r:
        fixed, stage_full = r
        factor = cur["prefill_full_device_factor"]
        out["prefill_tile_fixed_us"] = max(fixed, 0.5)
        out["prefill_stage_us_256x256"] = stage_full / factor
        say(f"prefill 256x256, {n_side}x{n_side}: fixed {fixed:.2f} us, stage {stage_full:.3f} us on a full device")
    r = pair(cabi.VARIANT_PREFILL_NARROW, n_side, n_side // 2, 2048, 4096, n_codebooks=n_side // 256)
    if r:
        out["prefill_stage_us_256x128"] = r[1] / cur["prefill_full_device_factor"]
        say(f"prefill 256x128: fixed {r[0]:.2f} us, stage {r[1]:.3f} us on a full device")
    # 128x128 tiles: a busy device (one tile per unit) and an idle one (a sixteenth of that)
    rb = pair(cabi.VARIANT_PREFILL_SMALL, 128 * int(cus ** 0.5), 128 * int(cus ** 0.5), 2048, 4096)
    ri = pair(cabi.VARIANT_PREFILL_SMALL, 512, 512, 2048, 4096)
    if rb and ri:
        out["prefill_small_tile_fixed_us"] = max(0.5 * (rb[0] + ri[0]), 0.5)
        out["prefill_small_stage_us_busy"] = rb[1]
        out["prefill_small_stage_us_idle"] = min(ri[1], rb[1])
        say(f"prefill 128x128: fixed {rb[0]:.2f} / {ri[0]:.2f} us, stage {rb[1]:.3f} us busy, {ri[1]:.3f} us idle")
    # batched decode kernel, 16 rows of X: one and eight tiles of 16 rows per unit
    t1 = _t(16, 4096, 16 * cus, cabi.VARIANT_DECODE)
    t8 = _t(16, 4096, 128 * cus, cabi.VARIANT_DECODE)
    if t1 and t8:
        tile = (t8 - t1) / 7.0
        out["decode_tile_us"] = tile
        out["decode_prologue_us"] = max(t1 - tile, 0.5)
        say(f"decode, K=4096: {t1:.2f} us at one tile per unit, {t8:.2f} us at eight: {tile:.3f} us per tile")
    # (the batched kernel's chunks of K: its streaming sibling, which would take the first of these shapes, is switched off)
    stream_was = {k: cabi.tuning()[k] for k in ("decode_stream_min_k", "decode_stream_min_k_few_rows")}
    cabi.set_tuning(decode_stream_min_k=1e8, decode_stream_min_k_few_rows=1e8)
    try:
        t1c = _t(16, 8192, 16 * cus, cabi.VARIANT_DECODE)
        t8c = _t(16, 8192, 128 * cus, cabi.VARIANT_DECODE)
    finally:
        cabi.set_tuning(**stream_was)
    if t1c and t8c:
        out["decode_tile_chunked_us"] = (t8c - t1c) / 7.0 / 2.0   # per 4096 k
        say(f"decode, K=8192 (two chunks): {(t8c - t1c) / 7.0:.3f} us per tile")
    # four-wave GEMV kernel against the batched kernel, one row of X in a format the wide form does not take
    best = 0.0
    for tiles in (1, 2, 4, 8, 16):
        tg = _t(1, 4096, 16 * cus * tiles, cabi.VARIANT_DECODE_GEMV, vec=4)
        td = _t(1, 4096, 16 * cus * tiles, cabi.VARIANT_DECODE, vec=4)
        if tg is None or td is None:
            break
        say(f"one row of X, 4-vectors, {tiles} tile(s) per unit: GEMV {tg:.2f} us, batched {td:.2f} us")
        if tg <= td:
            best = float(tiles)
        else:
            break
    out["gemv_max_tiles_per_cu"] = best
    # split K over the 128x128 tiles: what two slices cost beyond their multiplying (the same tiles as an unsplit problem
    # of half the K and twice the columns), at two sizes of partial sums
    def split_extra(M, K, N):
        cabi.set_tuning(splitk_force_splits=2)
        try:
            need = cabi.workspace_bytes_b(M, K, N, 8, 256, 1, 8, cabi.VARIANT_PREFILL_SPLITK)
            if need <= 0:
                return None
            spec = ProblemSpec("fit", GEOM_B, M, K, N, 8, 256, 1, 8)
            x, codes, cb = make_problem(spec, seed=1, device=device)
            y = torch.empty(M, N, dtype=torch.float16, device=device)
            ws = torch.empty(need, dtype=torch.uint8, device=device)
            t_split = time_graph(lambda: cabi.e2e_gemm_b_ws(x, codes, cb, out=y, variant=cabi.VARIANT_PREFILL_SPLITK, workspace=ws))
        finally:
            cabi.set_tuning(splitk_force_splits=cur["splitk_force_splits"])
        t_main = _t(M, K // 2, 2 * N, cabi.VARIANT_PREFILL_SMALL)
        return None if t_main is None else (t_split - t_main, need / 1e6)
    small, large = split_extra(128, 4096, 4096), split_extra(512, 4096, 4096)
    if small and large and large[1] > small[1]:
        per_mb = max((large[0] - small[0]) / (large[1] - small[1]), 0.05)
        out["splitk_us_per_partial_mb"] = per_mb
        out["splitk_fixed_us"] = max(small[0] - per_mb * small[1], 0.5)
        say(f"split K, two slices: {small[0]:.2f} us beyond the multiplying at {small[1]:.1f} MB of partial sums, {large[0]:.2f} us at {large[1]:.1f} MB")
    # (the limits between the GEMV kernels and the kernels' run-time parameters are decided by launches on codes that
    # come from HBM - the wide form wins its short launches cold and loses them warm - and this function times warm
    # launches: `search` below covers them)
    if verbose:
        print("constant                          compiled-in / current -> fitted")
        for k in out:
            print(f"  {k:32s} {cur[k]:8.3f} -> {out[k]:8.3f}")
    return out


def _cold_us(M, K, N, variant=None, vec=8, entries=256, n_codebooks=1, code_bits=8, device="cuda:0", steps=50, repeats=3,
             **constants):
    """Microseconds per launch on codes from HBM (rotating pool; the median of `repeats` timed regions), with
    `constants` set in the tuning table for the duration; None when the variant refuses the shape."""
    from . import timing
    variant = cabi.VARIANT_AUTO if variant is None else variant
    spec = ProblemSpec("search", GEOM_B, M, K, N, vec, entries, n_codebooks, code_bits)
    x, codes, cb = make_problem(spec, seed=1, device=device)
    pool = timing.code_pool(spec, timing.pool_size(spec.code_bytes), first=codes, device=device)
    y = torch.empty(M, N, dtype=torch.float16, device=device)
    before = cabi.tuning()
    try:
        cabi.set_tuning(**constants)
        try:
            cabi.e2e_gemm_b(x, pool[0], cb, out=y, variant=variant)
        except cabi.VqGemmError as e:
            if e.code != -4:
                raise
            return None
        ts = sorted(timing.time_launches(lambda i: cabi.e2e_gemm_b(x, pool[i], cb, out=y, variant=variant), len(pool), steps, 20,
                                         device=device)[0] for _ in range(repeats))
        return ts[len(ts) // 2] * 1e6
    finally:
        cabi.set_tuning(**{k: before[k] for k in constants})
        del pool


def search(device: str = "cuda:0", verbose: bool = True, quick: bool = False, margin: float = 0.02) -> dict:
    """Times the candidates of the kernels' run-time parameters on cold code matrices and returns the table with the
    winners in it.  `quick` leaves out the largest shapes (for tests).  A candidate replaces the value in force only
    when it is ahead by more than `margin` (as a share of the time): differences inside the noise change nothing."""
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    waves = 16 * cus  # the wide GEMV kernel's waves on the device
    cur = cabi.tuning()
    out = dict(cur)
    report = {}
    say = print if verbose else (lambda *a, **k: None)
    GEMV, DEC = cabi.VARIANT_DECODE_GEMV, cabi.VARIANT_DECODE
    force_wide = dict(gemv_wide_min_rows_per_wave=0.0)

    # 1. the wide form's loop: (rows per group, groups in flight), K up to 4096 and beyond
    def loop_search(tag, names, shapes):
        totals = {}
        for g in (1, 2):
            for nbuf in (2, 3):
                if g * nbuf > 4 and any(K > 4096 for (K, _, _) in shapes):
                    continue   # (not built: two rows per group with three groups in flight beyond K = 4096)
                ts = [_cold_us(1, K, N, GEMV, n_codebooks=G, device=device, **force_wide, **{names[0]: g, names[1]: nbuf})
                      for (K, N, G) in shapes]
                if all(t is not None for t in ts):
                    totals[(g, nbuf)] = ts
        if not totals:
            return
        # each shape counts alike: sum of times relative to the shape's best candidate
        best_of = [min(ts[i] for ts in totals.values()) for i in range(len(shapes))]
        score = {c: sum(t / b for t, b in zip(ts, best_of)) for c, ts in totals.items()}
        win = min(score, key=score.get)
        now = (int(cur[names[0]]), int(cur[names[1]]))
        if now in score and score[now] <= score[win] * (1.0 + margin):
            win = now
        out[names[0]], out[names[1]] = float(win[0]), float(win[1])
        report[tag] = {f"g{c[0]}_nbuf{c[1]}": [round(t, 3) for t in ts] for c, ts in totals.items()}
        say(f"wide GEMV loop, {tag}: " + "; ".join(f"G={c[0]} NBUF={c[1]}: " + "/".join(f"{t:.2f}" for t in ts) for c, ts in totals.items())
            + f" us on {shapes} -> G={win[0]} NBUF={win[1]}")
    # (a wave with one or two rows takes them one by one whatever these say: shapes of three rows per wave and more)
    loop_search("K<=4096", ("gemv_wide_rows_per_group", "gemv_wide_groups_in_flight"),
                [(4096, 4 * waves, 1), (4096, 3 * waves, 3)] + ([] if quick else [(4096, 7 * waves, 1), (2048, 4 * waves, 1)]))
    loop_search("K>4096", ("gemv_wide_rows_per_group_long_k", "gemv_wide_groups_in_flight_long_k"),
                [(8192, 3 * waves, 1)] + ([] if quick else [(8192, 7 * waves, 1), (6144, 4 * waves, 1), (14336, waves, 1)]))
    loop_now = {k: out[k] for k in ("gemv_wide_rows_per_group", "gemv_wide_groups_in_flight", "gemv_wide_rows_per_group_long_k",
                                    "gemv_wide_groups_in_flight_long_k")}

    # 1b. the waves of a SIMD taking turns at the issue priority
    rot_shapes = [(4096, 7 * waves), (8192, 7 * waves)] + ([] if quick else [(4096, 16 * waves), (2048, 8 * waves), (4096, 3 * waves)])
    rot = {r: [_cold_us(1, K, N, GEMV, device=device, **force_wide, **loop_now, gemv_wide_rotate_priority=r) for (K, N) in rot_shapes] for r in (0, 1)}
    if all(t is not None for ts in rot.values() for t in ts):
        score = {r: sum(t / min(a, b) for t, a, b in zip(ts, rot[0], rot[1])) for r, ts in rot.items()}
        now = int(cur["gemv_wide_rotate_priority"] >= 1.0)
        win = min(score, key=score.get)
        if score[now] <= score[win] * (1.0 + margin):
            win = now
        out["gemv_wide_rotate_priority"] = float(win)
        report["rotate_priority"] = {r: [round(t, 3) for t in ts] for r, ts in rot.items()}
        say("wide GEMV, issue priority: " + "; ".join(("rotating: " if r else "left alone: ") + "/".join(f"{t:.2f}" for t in ts) for r, ts in rot.items())
            + f" us on {rot_shapes} -> {win}")
    loop_now["gemv_wide_rotate_priority"] = out["gemv_wide_rotate_priority"]

    # 1c. several codebooks: how many compute units may go without a workgroup so that no workgroup's rows cross a codebook
    book_shapes = [(4096, 48 * cus, 3), (4096, 112 * cus, 56)] + ([] if quick else [(8192, 112 * cus, 56), (4096, 24 * cus, 3)])
    shares = {}
    for share in (1.0, 0.85, 0.7, 0.5):
        ts = [_cold_us(1, K, N, GEMV, n_codebooks=G, device=device, **force_wide, **loop_now, gemv_wide_min_units_share=share)
              for (K, N, G) in book_shapes]
        if all(t is not None for t in ts):
            shares[share] = ts
    if shares:
        best_of = [min(ts[i] for ts in shares.values()) for i in range(len(book_shapes))]
        score = {c: sum(t / b for t, b in zip(ts, best_of)) for c, ts in shares.items()}
        win = min(score, key=score.get)
        now = cur["gemv_wide_min_units_share"]
        if now in score and score[now] <= score[win] * (1.0 + margin):
            win = now
        out["gemv_wide_min_units_share"] = float(win)
        report["min_units_share"] = {c: [round(t, 3) for t in ts] for c, ts in shares.items()}
        say("wide GEMV, units left idle for whole codebooks: " + "; ".join(f"share {c}: " + "/".join(f"{t:.2f}" for t in ts) for c, ts in shares.items())
            + f" us on {book_shapes} -> {win}")

    # 2. plain against bank-replicated table: the threshold in gathers per lane (rows per wave x runs of 2048 k)
    rows = []
    for (K, N) in [(2048, waves), (4096, waves), (4096, 2 * waves), (8192, waves)] + ([] if quick else [(2048, 2 * waves), (8192, 2 * waves)]):
        runs = (N // waves) * (K // 2048)
        tp = _cold_us(1, K, N, GEMV, device=device, **force_wide, **loop_now, gemv_wide_plain_table_max_runs=1e6)
        tr = _cold_us(1, K, N, GEMV, device=device, **force_wide, **loop_now, gemv_wide_plain_table_max_runs=0.0)
        if tp is not None and tr is not None:
            rows.append((runs, tp, tr))
            say(f"wide GEMV table, K={K} N={N} ({runs} runs per wave): plain {tp:.2f} us, replicated {tr:.2f} us")
    if rows:
        cands = sorted({0.0} | {float(r[0]) for r in rows})
        cost = {c: sum(tp if runs <= c else tr for runs, tp, tr in rows) for c in cands}
        out["gemv_wide_plain_table_max_runs"] = min(cost, key=cost.get)
        report["plain_table"] = [(r, round(a, 3), round(b, 3)) for r, a, b in rows]

    # 3. wide form against the four-wave form: from how many rows per wave on the wide form wins
    limit = None
    fracs = (0.0625, 0.125, 0.25, 0.5, 0.75, 1.0)
    wins = []
    for f in fracs:
        N = int(waves * f) // 16 * 16
        tw = _cold_us(1, 4096, N, GEMV, device=device, **loop_now, gemv_wide_plain_table_max_runs=out["gemv_wide_plain_table_max_runs"],
                      gemv_wide_min_rows_per_wave=0.0)
        t4 = _cold_us(1, 4096, N, GEMV, device=device, gemv_wide_min_rows_per_wave=1e6)
        if tw is None or t4 is None:
            continue
        say(f"one row of X, K=4096, N={N} ({f} rows per wave): wide {tw:.2f} us, four-wave {t4:.2f} us")
        wins.append((f, tw <= t4 * (1.0 - margin)))
    for f, won in reversed(wins):   # the smallest share from which the wide form wins all the way up
        if not won:
            break
        limit = f
    if wins and all(won for _, won in wins):
        limit = 0.0   # ahead down to the smallest launch tried: every launch the wide form supports
    if limit is not None:
        out["gemv_wide_min_rows_per_wave"] = limit
    report["wide_vs_four_wave"] = wins

    # 3b. two rows of X: the wide form against the K-sliced kernel, by the runs of 2048 k a wave's rows make (K = 4096)
    best_runs = None
    for rows in ((8, 11, 14) if quick else (6, 8, 10, 11, 12, 14)):
        N = rows * waves
        tw = _cold_us(2, 4096, N, GEMV, device=device, gemv_wide_two_rows_max_runs=1e6, gemv_wide_max_m=2.0)
        td = _cold_us(2, 4096, N, DEC, device=device)
        if tw is None or td is None:
            continue
        say(f"two rows of X, K=4096, {rows} rows per wave: wide {tw:.2f} us, K-sliced {td:.2f} us")
        if tw <= td:
            best_runs = 2.0 * rows
        else:
            break
    if best_runs is not None:
        out["gemv_wide_two_rows_max_runs"] = best_runs
    report["wide_two_rows"] = best_runs

    # 4. four-wave GEMV against the batched K-sliced kernel in a format the wide form does not take: tiles per unit, K
    best_tiles = 0.0
    for tiles in (1, 2, 4, 8) if not quick else (1, 2):
        tg = _cold_us(1, 4096, 16 * cus * tiles, GEMV, vec=4, device=device)
        td = _cold_us(1, 4096, 16 * cus * tiles, DEC, vec=4, device=device)
        if tg is None or td is None:
            break
        say(f"one row of X, 4-vectors, {tiles} tile(s) per unit: four-wave GEMV {tg:.2f} us, batched {td:.2f} us")
        if tg > td:
            break
        best_tiles = float(tiles)
    out["gemv_max_tiles_per_cu"] = best_tiles
    best_k = 0.0
    for K in (2048, 4096, 6144, 8192):
        won = []
        for tiles in (1, 2):
            tg = _cold_us(1, K, 16 * cus * tiles, GEMV, vec=4, device=device)
            td = _cold_us(1, K, 16 * cus * tiles, DEC, vec=4, device=device)
            if tg is None or td is None:
                continue
            say(f"one row of X, 4-vectors, {tiles} tile(s) per unit, K={K}: four-wave GEMV {tg:.2f} us, batched {td:.2f} us")
            won.append(tg <= td)
        if won and all(won):
            best_k = float(K)
    if best_k:
        out["gemv_max_k"] = best_k

    # 5. batched decode kernel: from how many tiles per workgroup the replicated table pays (16 rows of X)
    rows = []
    for tiles in (1, 2, 3, 4):
        tp = _cold_us(16, 4096, 16 * cus * tiles, DEC, device=device, decode_replicated_table_min_tiles=1e6)
        tr = _cold_us(16, 4096, 16 * cus * tiles, DEC, device=device, decode_replicated_table_min_tiles=0.0)
        if tp is None or tr is None:
            continue
        say(f"batched decode, {tiles} tile(s) per workgroup: plain table {tp:.2f} us, replicated {tr:.2f} us")
        rows.append((tiles, tp, tr))
    if rows:
        cands = [1.0, 2.0, 3.0, 4.0, 5.0]
        cost = {c: sum(tr if tiles >= c else tp for tiles, tp, tr in rows) for c in cands}
        out["decode_replicated_table_min_tiles"] = min(cost, key=cost.get)
        report["decode_table"] = [(t, round(a, 3), round(b, 3)) for t, a, b in rows]

    # 6. the streaming kernel of the K-sliced path against the batched kernel's chunks of K: from which K on it is ahead,
    #    for sixteen and for four rows of X (one tile per unit)
    stream_on = dict(decode_stream_min_k=0.0, decode_stream_min_k_few_rows=0.0, decode_stream_min_m=0.0, decode_stream_max_m=16.0)
    stream_off = dict(decode_stream_min_k=1e8, decode_stream_min_k_few_rows=1e8)
    for rows_x, name in ((16, "decode_stream_min_k"), (4, "decode_stream_min_k_few_rows")):
        first = None
        ks = (8192, 14336) if quick else (8192, 12288, 14336, 16384)
        for K in reversed(ks):
            ts = _cold_us(rows_x, K, 16 * cus, DEC, device=device, **stream_on)
            tb = _cold_us(rows_x, K, 16 * cus, DEC, device=device, **stream_off)
            if ts is None or tb is None:
                break
            say(f"{rows_x} rows of X, K={K}, one tile per unit: streaming {ts:.2f} us, batched {tb:.2f} us")
            report.setdefault("decode_stream", []).append((rows_x, K, round(ts, 3), round(tb, 3)))
            if ts > tb * (1.0 - margin):
                break
            first = K
        out[name] = float(first) if first else 1e8

    if verbose:
        print("constant                          current -> searched")
        for k in out:
            if out[k] != cur[k]:
                print(f"  {k:36s} {cur[k]:8.3f} -> {out[k]:8.3f}")
    out_report = dict(out)
    search.last_report = report
    return out_report


search.last_report = {}


def main(argv) -> int:
    if argv and argv[0] in ("--fit", "--search"):
        import json
        fitted = fit() if "--fit" in argv else cabi.tuning()
        if "--search" in argv:
            cabi.set_tuning(**fitted)
            fitted = search()
        if "--write" in argv:
            i = argv.index("--write")
            path = argv[i + 1] if len(argv) > i + 1 else cabi.TUNING_FILE
            with open(path, "w") as f:
                json.dump({"device": torch.cuda.get_device_name(0), **fitted}, f, indent=1)
            print("wrote", path)
        return 0
    cold = "--cold" in argv
    argv = [a for a in argv if a != "--cold"]
    if len(argv) not in (3, 7):
        print(__doc__)
        return 2
    vals = [int(a) for a in argv]
    (tune_cold if cold else tune)(*vals)
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
