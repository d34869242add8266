"""Measured denominators for `bench.py`: what one launch costs, how fast a launch can stream a
buffer of a given size, and what the matrix unit issues, on the card the benchmark runs on.

Everything is timed as HIP-graph replays of back-to-back launches between two events on the
replaying stream, the way the mat-vec launches themselves are timed.

`python -m loken_amd.probes` prints one JSON object with the full sweep.
"""
from __future__ import annotations

import ctypes as C
import json
from pathlib import Path

import numpy as np
import torch

from . import lib

PROBES_PATH = Path(__file__).resolve().parent / "libloken_probes.so"
_probes = None


def load() -> C.CDLL:
    """The measurement library (include/loken_probes.h): a library of its own, not the product's."""
    global _probes
    if _probes is None:
        if not PROBES_PATH.exists():
            raise ImportError(f"{PROBES_PATH} is missing: build it with `python -m loken_amd.build`")
        L = C.CDLL(str(PROBES_PATH))
        vp, i, i64 = C.c_void_p, C.c_int, C.c_int64
        for name, args in {"lk_probe_empty": [i, vp], "lk_probe_read": [vp, i64, i, i, vp, vp],
                           "lk_probe_mfma": [i, i, i, i, i, vp, vp, vp],
                           "lk_probe_overlap": [i, i, i, i, i, i, vp, vp]}.items():
            fn = getattr(L, name)
            fn.restype = i
            fn.argtypes = args
        _probes = L
    return _probes

HBM_PEAK_GBS = 8000.0
PEAK_TOPS = {0: 5000.0, 1: 2500.0, 2: 5000.0, 3: 5000.0}
MFMA_NAMES = {0: "v_mfma_i32_32x32x32_i8", 1: "v_mfma_f32_32x32x16_f16", 2: "v_mfma_i32_16x16x64_i8",
              3: "v_mfma_i32_32x32x16_i8"}


def _check(rc, what):
    if rc:
        raise lib.LokenError(what, rc)


def _graph_us(record, launches_in_graph, replays=20, warm=3):
    """Median microseconds per launch of a graph that `record(stream)` fills with launches."""
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        record(side.cuda_stream)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            record(side.cuda_stream)
    torch.cuda.synchronize()
    for _ in range(warm):
        graph.replay()
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(replays)]
    for a, b in pairs:
        a.record()
        graph.replay()
        b.record()
    torch.cuda.synchronize()
    us = np.array([a.elapsed_time(b) * 1e3 for a, b in pairs]) / launches_in_graph
    return float(np.median(us))


def launch_floor(workgroups=512, launches=256):
    """Microseconds per launch of a graph of empty 256-thread kernels of `workgroups` workgroups."""
    L = load()

    def record(s):
        for _ in range(launches):
            _check(L.lk_probe_empty(workgroups, s), "lk_probe_empty")

    return _graph_us(record, launches)


class ReadBuffers:
    """Device memory for the streaming-read probes: one allocation, sliced into rotating copies."""

    def __init__(self, total_bytes=1 << 30):
        self.buf = torch.empty(total_bytes, dtype=torch.uint8, device="cuda")
        self.buf.fill_(1)
        self.sink = torch.zeros(4, dtype=torch.uint8, device="cuda")
        self.total = total_bytes

    def rate(self, nbytes, workgroups, pattern, launches=None):
        """(microseconds per launch, GB/s) of launches that each read `nbytes`, walking through the
        allocation so that a launch never re-reads what the last-level cache may still hold."""
        L = load()
        nbytes -= nbytes % 16
        copies = max(1, self.total // nbytes)
        if launches is None:
            launches = max(1, min(64, copies))
        base = self.buf.data_ptr()

        def record(s):
            for i in range(launches):
                _check(L.lk_probe_read(base + (i % copies) * nbytes, nbytes, workgroups, pattern, self.sink.data_ptr(), s),
                       "lk_probe_read")

        us = _graph_us(record, launches, replays=10 if nbytes >= 1 << 28 else 20)
        return us, nbytes / us / 1e3


def mfma_rate(kind=0, workgroups=2048, iters=2000, valu_per_mfma=0, mode=0):
    """TOP/s of the register-resident matrix-unit loop (and microseconds per launch)."""
    L = load()
    sink = torch.zeros(4, dtype=torch.uint8, device="cuda")
    ops = C.c_double(0)

    def record(s):
        _check(L.lk_probe_mfma(kind, workgroups, iters, valu_per_mfma, mode, sink.data_ptr(), C.byref(ops), s), "lk_probe_mfma")

    us = _graph_us(record, 1, replays=10)
    return ops.value / us / 1e6, us


def overlap_ns(kind, valu, dep=0, waves_per_simd=1, iters=20000):
    """Nanoseconds per slot of one wave of lk_probe_overlap (a SIMD runs `waves_per_simd` of them): one
    matrix instruction and `valu` fmas; kind 4: the chained item, two instructions and 2 x valu fmas."""
    L = load()
    sink = torch.zeros(64, dtype=torch.uint8, device="cuda")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    s = torch.cuda.current_stream().cuda_stream
    _check(L.lk_probe_overlap(kind, valu, dep, waves_per_simd, cus, 200, sink.data_ptr(), s), "lk_probe_overlap")
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    _check(L.lk_probe_overlap(kind, valu, dep, waves_per_simd, cus, iters, sink.data_ptr(), s), "lk_probe_overlap")
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e6 / (iters * 4.0)


def overlap_table():
    """Vector work beside matrix work, with nothing waiting on an instruction in flight."""
    names = {0: "v_mfma_f32_32x32x16_f16", 1: "v_mfma_i32_32x32x32_i8", 2: "v_mfma_i32_16x16x64_i8", 3: "no matrix instruction",
             4: "item: 2 chained f16 + fmas of the previous item"}
    out = {}
    for kind in (3, 0, 1, 2):
        for dep in ((0, 1) if kind in (0, 1) else (0,)):
            row = {}
            for valu in (0, 4, 8, 12, 16, 24, 32):
                row[f"V{valu}"] = {f"{w}_wave_per_simd_ns": round(overlap_ns(kind, valu, dep, w), 2) for w in (1, 2)}
            out[f"{names[kind]}, fmas {'read an older result tile' if dep else 'on their own registers'}"] = row
    out[names[4]] = {f"V{2 * v}": {f"{w}_wave_per_simd_ns": round(overlap_ns(4, v, 0, w), 2) for w in (1, 2)} for v in (4, 8, 12, 16)}
    return out


def ceilings(quick=True):
    """The denominators bench.py reports: streaming read over 1 GiB and the int8 matrix loop."""
    rb = ReadBuffers()
    best = max(rb.rate(1 << 30, wgs, pat)[1] for wgs, pat in ((2048, 1), (4096, 1), (1024, 2)))
    tops, _ = mfma_rate(0)
    f16, _ = mfma_rate(1)
    return {"hbm_read_1gib_gbs": round(best, 1), "hbm_read_frac_of_8tbs": round(best / HBM_PEAK_GBS, 4),
            "mfma_i8_32x32x32_tops": round(tops, 1), "mfma_i8_frac_of_5pops": round(tops / PEAK_TOPS[0], 4),
            "mfma_f16_32x32x16_tflops": round(f16, 1),
            "empty_launch_us": round(launch_floor(512), 3)}, rb


def sweep():
    out = {"launch_floor_us": {str(w): round(launch_floor(w), 3) for w in (1, 256, 512, 1024, 2048, 8192)}}
    rb = ReadBuffers()
    out["read_1gib_gbs"] = {f"wgs{w}_u{p}": round(rb.rate(1 << 30, w, p)[1], 1)
                            for w in (1024, 2048, 4096, 16384) for p in (0, 1, 2, 4, 8)}
    sizes = {"k_or_v 2.36MB": 2359296, "q_or_o 9.44MB": 9437184, "q+k+v 14.2MB": 14155776, "mix mean 29.9MB": 29884416,
             "gate 33MB": 33030144, "down 48.2MB": 48168960, "gate+up 66MB": 66060288, "lm_head 558MB": 558170112}
    out["read_launch_us_by_size"] = {}
    for name, nbytes in sizes.items():
        best = None
        for wgs in (256, 512, 1024, 2048):
            for pat in (0, 2, 4, 8):
                us, gbs = rb.rate(nbytes, wgs, pat)
                if best is None or us < best[0]:
                    best = (us, gbs, wgs, pat)
        out["read_launch_us_by_size"][name] = {"us": round(best[0], 3), "gbs": round(best[1], 1), "workgroups": best[2],
                                               "pattern": best[3], "frac_of_8tbs": round(best[1] / HBM_PEAK_GBS, 4)}
    del rb
    out["mfma"] = {}
    for kind in (0, 1, 2, 3):
        tops, us = mfma_rate(kind)
        out["mfma"][MFMA_NAMES[kind]] = {"tops": round(tops, 1), "frac_of_nominal": round(tops / PEAK_TOPS[kind], 4), "us": round(us, 1)}
    # vector work beside matrix work: the same wave, or a second wave on the same SIMD
    ov = {}
    for valu in (0, 8, 16, 32):
        for mode in (0, 1):
            tops, us = mfma_rate(0, valu_per_mfma=valu, mode=mode)
            ov[f"i8_valu{valu}_{'same_wave' if mode == 0 else 'other_wave'}"] = {"tops": round(tops, 1), "us": round(us, 1)}
    out["mfma_with_vector_work_old_probe"] = ov
    out["overlap_ns_per_slot"] = overlap_table()
    return out


if __name__ == "__main__":
    torch.cuda.set_device(0)
    print(json.dumps(sweep(), indent=1))
