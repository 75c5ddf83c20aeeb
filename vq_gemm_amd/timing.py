"""Timing of microsecond-scale launches on codes that really come from HBM.

The protocol behind every per-launch figure of `bench.py` and behind `python -m vq_gemm_amd.tune --search`:

  * launches are captured in HIP graphs and replayed, so that host launch overhead does not pace the kernel,
    and timed with HIP events recorded on the stream the kernels run on;
  * launch i reads buffer i % n_bufs of a pool of distinct code matrices larger than the L2 and the Infinity
    Cache together, so that two reads of one matrix lie a whole pool apart;
  * the timed region is `steps` launches repeated until it covers two full rotations of the pool and at least
    `min_launches` launches: what is measured does not depend on `steps`;
  * every graph is replayed once untimed (the first replay uploads it), then a device copy larger than the
    caches runs, then all graphs are replayed between two events.
"""
from __future__ import annotations

import torch

POOL_BYTES = 640 << 20   # distinct code matrices rotated through by the bandwidth-bound configurations
EVICT_BYTES = 512 << 20  # source and destination of the device copy that empties the caches
MIN_TIMED_LAUNCHES = 200  # a microsecond-scale kernel is never timed over fewer launches than this

_evict = {}


def evict_caches(stream, device="cuda:0"):
    """A device copy larger than L2 + Infinity Cache on `stream`: what was cached before it is gone after."""
    if device not in _evict:
        _evict[device] = (torch.empty(EVICT_BYTES, dtype=torch.uint8, device=device).random_(),
                          torch.empty(EVICT_BYTES, dtype=torch.uint8, device=device))
    src, dst = _evict[device]
    with torch.cuda.stream(stream):
        dst.copy_(src)


def release():
    """Give the eviction buffers back (1 GiB of device memory)."""
    _evict.clear()


def pool_size(code_bytes: int, cold: bool = True) -> int:
    """How many distinct code matrices of `code_bytes` each the rotating pool holds."""
    return max(1, min(512, POOL_BYTES // max(code_bytes, 1))) if cold else 1


def time_launches(launch, n_bufs, steps, warmup, chunk=500, min_launches=MIN_TIMED_LAUNCHES, device="cuda:0"):
    """(average seconds per launch, launches timed) of `launch(i)`, i rotating over n_bufs buffers."""
    n_timed = steps * max(1, -(-max(2 * n_bufs if n_bufs > 1 else 0, min_launches) // steps))
    stream = torch.cuda.Stream()   # default priority
    with torch.cuda.stream(stream):
        for i in range(max(warmup, 1)):
            launch(i % n_bufs)
        stream.synchronize()
        graphs = []
        done = 0
        while done < n_timed:
            c = min(chunk, n_timed - done)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(c):
                    launch((done + i) % n_bufs)
            graphs.append(g)
            done += c
        for g in graphs:            # first replay uploads a graph: keep it out of the timing
            g.replay()
        stream.synchronize()
        if n_bufs > 1:
            evict_caches(stream, device)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        for g in graphs:
            g.replay()
        e1.record(stream)
        e1.synchronize()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / n_timed, n_timed


def code_pool(spec, n_bufs, first=None, device="cuda:0", seed=1234):
    """`n_bufs` code matrices of a geometry-B problem with uniformly random codes (`first`, if given, is the first)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    pool = [] if first is None else [first]
    while len(pool) < n_bufs:
        c = torch.randint(0, spec.entries, spec.codes_shape, generator=gen, device=device, dtype=torch.int32)
        pool.append(c.to(spec.code_dtype))
    return pool
