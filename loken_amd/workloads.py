"""The other measured workloads of `bench.py` (`--workload ...`): one JSON line each.

  gemv        one mat-vec of any served format (`--wtype`, `--rows-n`, `--cols-k`, `--batch`) over rotating
              copies of the weight, as one graph
  gemv-4096   one Q4_K 4096x4096 mat-vec at one row, over rotating copies of the weight (more
              than twice the 256 MB last-level cache) and over one hot copy; the Q8_1 quantizer
              launch timed by itself and the two-launch call timed as a whole
  mmq         the tiled int8-MFMA matmul: `--shape 2a` = 512 rows x 4096 -> 14336 in Q4_K,
              `--shape 2b` = 2048 rows x 14336 -> 4096 in Q6_K; quantizer + matmul per step
  moe         one Qwen3-30B-A3B-shaped expert block (128 experts, 2048 -> 768 -> 2048, top-8,
              Q4_K) at `--tokens` rows, path chosen as the layer code chooses it
  decode-1p7b every quantized linear of a Qwen3-1.7B-shaped decode step at `--batch` rows:
              mat-vec launches up to 8 rows, the tiled matmul above

Timing: 20 warm-up launches, then `--launches` (default 200) launches each bracketed by its own
pair of events on the launch stream; median, p10, p90, min and max are reported (the protocol of
the reference's own kernel benchmark, src/tensor/cuda/quant.rs:3940-3957).
"""
from __future__ import annotations

import json

import numpy as np
import torch

from . import lib, moe, ops, synth

HBM_PEAK_GBS = 8000.0
INT8_PEAK_TOPS = 5000.0
F16_PEAK_TFLOPS = 2500.0
Q4K, Q6K, Q80 = lib.TYPE_Q4_K, lib.TYPE_Q6_K, lib.TYPE_Q8_0
NAMES = {Q4K: "Q4_K", Q6K: "Q6_K", Q80: "Q8_0", lib.TYPE_Q5_K: "Q5_K", lib.TYPE_Q2_K: "Q2_K", lib.TYPE_Q3_K: "Q3_K",
         lib.TYPE_Q4_0: "Q4_0", lib.TYPE_Q4_1: "Q4_1", lib.TYPE_Q5_0: "Q5_0", lib.TYPE_Q5_1: "Q5_1"}


# ---------------------------------------------------------------------------- synthetic blocks
class Maker:
    """Random blocks generated on the device (field distributions of the seeded host generator
    in synth.py, which would take minutes for gigabytes)."""

    def __init__(self, dev, seed=0):
        self.dev = dev
        self.gen = torch.Generator(device=dev)
        self.gen.manual_seed(seed)

    def halfs(self, n, scale):
        v = torch.randn(n, device=self.dev, generator=self.gen).abs() * scale
        return v.to(torch.float16).view(torch.uint8).reshape(n, 2)

    def q4k(self, n, k):
        nb = n * (k // 256)
        w = torch.randint(0, 256, (nb, 144), dtype=torch.uint8, device=self.dev, generator=self.gen)
        w[:, 0:2] = self.halfs(nb, 1e-3)
        w[:, 2:4] = self.halfs(nb, 5e-4)
        return w.reshape(-1)

    def q6k(self, n, k):
        nb = n * (k // 256)
        w = torch.randint(0, 256, (nb, 210), dtype=torch.uint8, device=self.dev, generator=self.gen)
        sc = torch.randint(-64, 64, (nb, 16), dtype=torch.int8, device=self.dev, generator=self.gen)
        w[:, 192:208] = sc.view(torch.uint8)
        w[:, 208:210] = self.halfs(nb, 1e-3)
        return w.reshape(-1)

    def q80(self, n, k):
        nb = n * (k // 32)
        w = torch.empty((nb, 34), dtype=torch.uint8, device=self.dev)
        w[:, 0:2] = self.halfs(nb, 1e-3)
        w[:, 2:] = torch.randint(-127, 128, (nb, 32), dtype=torch.int8, device=self.dev,
                                 generator=self.gen).view(torch.uint8)
        return w.reshape(-1)

    def make(self, wtype, n, k):
        if wtype in (Q4K, Q6K, Q80):
            return {Q4K: self.q4k, Q6K: self.q6k, Q80: self.q80}[wtype](n, k)
        # any other format: 256 rows of the seeded host generator, repeated (the kernels do not care what
        # the blocks hold)
        base = torch.from_numpy(synth.weight(wtype, 256, k, seed=0, stream=wtype)).to(self.dev).reshape(256, -1)
        return base.repeat((n + 255) // 256, 1)[:n].contiguous().reshape(-1)

    def randn(self, *shape):
        return torch.randn(shape, device=self.dev, generator=self.gen)


# ---------------------------------------------------------------------------- timing
def time_launches(fn, launches, warm=20):
    """Per-launch durations in microseconds; `fn(i)` issues launch i on the current stream."""
    for i in range(warm):
        fn(i)
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
    for i, (a, b) in enumerate(pairs):
        a.record()
        fn(i)
        b.record()
    torch.cuda.synchronize()
    return np.array([a.elapsed_time(b) * 1e3 for a, b in pairs])


def time_back_to_back(fn, launches, warm=20):
    """Average microseconds per launch with the launches issued back to back between two events."""
    for i in range(warm):
        fn(i)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for i in range(launches):
        fn(i)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / launches


def capture(fn):
    """`fn()` (launches on the current stream) recorded once into a HIP graph on a side stream."""
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        fn()                                  # first-launch set-up happens outside the capture
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            fn()
    torch.cuda.synchronize()
    return graph


def time_replays(graph, launches, warm=20):
    """Per-replay durations in microseconds of a captured graph."""
    return time_launches(lambda i: graph.replay(), launches, warm)


def spread(us):
    return {"median_us": round(float(np.median(us)), 3), "p10_us": round(float(np.percentile(us, 10)), 3),
            "p90_us": round(float(np.percentile(us, 90)), 3), "min_us": round(float(us.min()), 3),
            "max_us": round(float(us.max()), 3), "launches": int(us.size)}


def line(args, metric_value, unit, ms_per_step, dtype, config, roofline, extra=None):
    out = {"metric": "Q4_K GEMV weight GB/s (% HBM peak); prefill MMQ int8 TOPS (% MFMA peak)",
           "value": round(metric_value, 1), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": dtype, "data": "synthetic", "config": config, "roofline": roofline, "cpu_baseline": None}
    if extra:
        out.update(extra)
    print(json.dumps(out))
    return 0


def check(rc, what):
    if rc:
        raise lib.LokenError(what, rc)


# ---------------------------------------------------------------------------- gemv (any format)
WTYPES = {"q4_0": lib.TYPE_Q4_0, "q4_1": lib.TYPE_Q4_1, "q5_0": lib.TYPE_Q5_0, "q5_1": lib.TYPE_Q5_1,
          "iq4_nl": lib.TYPE_IQ4_NL, "mxfp4": lib.TYPE_MXFP4, "q8_0": lib.TYPE_Q8_0, "q4_k": lib.TYPE_Q4_K,
          "q5_k": lib.TYPE_Q5_K, "q6_k": lib.TYPE_Q6_K, "q2_k": lib.TYPE_Q2_K, "q3_k": lib.TYPE_Q3_K, "iq4_xs": lib.TYPE_IQ4_XS,
          "iq2_xxs": lib.TYPE_IQ2_XXS, "iq3_xxs": lib.TYPE_IQ3_XXS, "iq3_s": lib.TYPE_IQ3_S, "iq2_s": lib.TYPE_IQ2_S, "q2_0": lib.TYPE_Q2_0}


def gemv(args, dev):
    """One `--wtype` mat-vec of `--rows-n` x `--cols-k` at `--batch` rows through lk_mmvq, over rotating
    copies of the weight (together past twice the last-level cache), replayed as one HIP graph."""
    L = lib.load()
    wtype, n, k, b = WTYPES[args.wtype], args.rows_n, args.cols_k, args.batch
    nbytes = synth.weight_bytes(wtype, n, k)
    n_copies = max(2, min(64, int(600e6 // nbytes) + 1))
    seed_rows = min(n, 256)   # a few generated rows repeated: the kernels do not care what the blocks hold
    base = torch.from_numpy(synth.weight(wtype, seed_rows, k, seed=0)).to(dev).reshape(seed_rows, -1)
    base = base.repeat((n + seed_rows - 1) // seed_rows, 1)[:n].contiguous().reshape(-1)
    copies = [base.clone() for _ in range(n_copies)]
    q = ops.quantize_q8_1_rows(torch.from_numpy(synth.activation(b, k, seed=0)).to(dev))
    out = torch.empty((b, n), device=dev)

    def all_copies():
        s2 = torch.cuda.current_stream().cuda_stream
        for w in copies:
            check(L.lk_mmvq(wtype, w.data_ptr(), q.data_ptr(), out.data_ptr(), lib.TYPE_F32, k, n, b, q.shape[1], n,
                            None, 0, s2), "lk_mmvq")

    us = time_replays(capture(all_copies), max(20, -(-args.launches // n_copies))) / n_copies
    med = float(np.median(us))
    value = nbytes / med / 1e3
    roofline = {"bound": "hbm", "achieved": round(value, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(value / HBM_PEAK_GBS, 4), "traffic": None, "kernel": f"lk_mmvq, {args.wtype}",
                "avg_launch_us": round(float(us.mean()), 3), "algorithmic_bytes_per_launch": nbytes}
    return line(args, value, "GB/s", med / 1e3, "int8",
                {"workload": f"{args.wtype} mat-vec {n} x {k}, {b} activation row(s), graph of {n_copies} launches over "
                             f"{n_copies} rotating copies ({n_copies * nbytes / 1e6:.0f} MB)", "hip_graph": True}, roofline,
                {"per_launch": spread(us)})


# ---------------------------------------------------------------------------- gemv-4096
def gemv_4096(args, dev):
    L = lib.load()
    n = k = 4096
    nbytes = synth.weight_bytes(Q4K, n, k)
    base = torch.from_numpy(synth.weight(Q4K, n, k, seed=0, stream=0)).to(dev).reshape(-1)
    copies = [base.clone() for _ in range(64)]           # 604 MB > 2 x 256 MB of last-level cache
    x = torch.from_numpy(synth.activation(1, k, seed=0)).to(dev)
    q = ops.quantize_q8_1_rows(x)
    out = torch.empty((1, n), device=dev)
    s = torch.cuda.current_stream().cuda_stream

    def mv(w):
        check(L.lk_mmvq(Q4K, w.data_ptr(), q.data_ptr(), out.data_ptr(), lib.TYPE_F32, k, n, 1, q.shape[1], n, None,
                        0, s), "lk_mmvq")

    def quant():
        check(L.lk_quantize_q8_1(x.data_ptr(), lib.TYPE_F32, q.data_ptr(), k, q.shape[1] * 32, 1, s), "lk_quantize_q8_1")

    vx = (lib.C.c_void_p * 1)()
    dst = (lib.C.c_void_p * 1)(out.data_ptr())
    nn = (lib.C.c_int * 1)(n)

    def fused(w):
        vx[0] = w.data_ptr()
        check(L.lk_mmvq_fused(Q4K, 1, vx, x.data_ptr(), x.stride(0), dst, lib.TYPE_F32, k, nn, 1, n, None, s),
              "lk_mmvq_fused")

    launches = args.launches
    rotated = time_launches(lambda i: mv(copies[i % 64]), launches)
    hot = time_launches(lambda i: mv(copies[0]), launches)
    quant_us = time_launches(lambda i: quant(), launches)
    two = time_launches(lambda i: (quant(), mv(copies[i % 64])), launches)
    one = time_launches(lambda i: fused(copies[i % 64]), launches)
    stream_us = time_back_to_back(lambda i: mv(copies[i % 64]), launches)
    # GPU-side rate without the host's per-launch cost: the 64 rotating launches as one graph
    side_calls = {}

    def sixty_four():
        s2 = torch.cuda.current_stream().cuda_stream
        for w in copies:
            check(L.lk_mmvq(Q4K, w.data_ptr(), q.data_ptr(), out.data_ptr(), lib.TYPE_F32, k, n, 1, q.shape[1], n,
                            None, 0, s2), "lk_mmvq")

    def sixty_four_fused():
        s2 = torch.cuda.current_stream().cuda_stream
        for j, w in enumerate(copies):
            vxs = side_calls.setdefault(j, (lib.C.c_void_p * 1)(w.data_ptr()))
            check(L.lk_mmvq_fused(Q4K, 1, vxs, x.data_ptr(), x.stride(0), dst, lib.TYPE_F32, k, nn, 1, n, None, s2),
                  "lk_mmvq_fused")

    graph_us = time_replays(capture(sixty_four), 50) / 64.0
    graph_fused_us = time_replays(capture(sixty_four_fused), 50) / 64.0
    gbs = lambda us: nbytes / us / 1e3
    med = float(np.median(rotated))
    roofline = {"bound": "hbm", "achieved": round(gbs(med), 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs(med) / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "mmvq_kernel<EngQ4K,1,2,float>",
                "avg_launch_us": round(float(rotated.mean()), 3), "algorithmic_bytes_per_launch": nbytes,
                "launches_timed": launches}
    extra = {"rotated_64_copies": dict(spread(rotated), gbs_median=round(gbs(med), 1)),
             "hot_one_copy": dict(spread(hot), gbs_median=round(gbs(float(np.median(hot))), 1)),
             "quantizer_launch": spread(quant_us),
             "call_two_launches": dict(spread(two), gbs_median=round(gbs(float(np.median(two))), 1)),
             "call_fused_one_launch": dict(spread(one), gbs_median=round(gbs(float(np.median(one))), 1)),
             "back_to_back_us_per_launch": round(stream_us, 3), "back_to_back_gbs": round(gbs(stream_us), 1),
             "graph_of_64_rotating_launches": dict(spread(graph_us), us_per_launch_median=round(float(np.median(graph_us)), 3),
                                                   gbs_median=round(gbs(float(np.median(graph_us))), 1), launches=50 * 64),
             "graph_of_64_fused_launches": dict(spread(graph_fused_us), us_per_launch_median=round(float(np.median(graph_fused_us)), 3),
                                                gbs_median=round(gbs(float(np.median(graph_fused_us))), 1), launches=50 * 64),
             "note": "per-launch event pairs and back-to-back eager launches are bounded by the host's launch cost; "
                     "the graph figures are the GPU-side rate, cache-cold (604 MB of rotating copies)"}
    g_med = float(np.median(graph_us))
    roofline.update({"achieved": round(gbs(g_med), 1), "frac": round(gbs(g_med) / HBM_PEAK_GBS, 4),
                     "avg_launch_us": round(float(graph_us.mean()), 3), "launches_timed": 50 * 64,
                     "timed_as": "graph of 64 launches over rotating copies"})
    med = g_med
    return line(args, gbs(med), "GB/s", med * 1e-3, "int8",
                {"workload": "Q4_K mat-vec 4096x4096, one row, 64 rotating weight copies", "weight_bytes": nbytes},
                roofline, extra)


# ---------------------------------------------------------------------------- mmq
def mmq(args, dev):
    L = lib.load()
    wtype, m, k, n = {"2a": (Q4K, 512, 4096, 14336), "2b": (Q6K, 2048, 14336, 4096)}[args.shape]
    if args.mmq_wtype:   # the same shape in another format of the tiled matmul's table
        wtype = WTYPES[args.mmq_wtype]
        if wtype not in ops.MMQ_LAUNCHER:
            raise SystemExit(f"--mmq-wtype {args.mmq_wtype}: no dense tiled matmul for this format")
    mk = Maker(dev)
    w = mk.make(wtype, n, k)
    x = mk.randn(m, k)
    out = torch.empty((m, n), device=dev)
    ws = ops.mmq_quantize(wtype, x)
    quantizer = getattr(L, ops.MMQ_QUANTIZER[wtype])
    launcher = getattr(L, ops.MMQ_LAUNCHER[wtype])
    info = ops.MMQ_DEVICE_INFO
    s = torch.cuda.current_stream().cuda_stream
    k_padded = ops.pad_to(ops.pad_to(k, 512), 128)

    def quant():
        quantizer(x.data_ptr(), None, ws.data_ptr(), 0, k, x.stride(0), 0, 0, k_padded, m, 1, 1, s)

    def matmul():
        if launcher(ops.mmq_fixup(dev).data_ptr(), w.data_ptr(), ws.data_ptr(), out.data_ptr(), k, n, m, k // synth.BLOCK_LEN[wtype], n,
                    info["cc"], info["nsm"], info["smpbo"], info["warp_size"], s) == 0:
            raise lib.LokenError(ops.MMQ_LAUNCHER[wtype], lib.LK_ERR_ARG)

    launches = args.launches
    mm = time_launches(lambda i: matmul(), launches)
    qu = time_launches(lambda i: quant(), launches)
    both = time_launches(lambda i: (quant(), matmul()), launches)
    op_count = 2.0 * m * k * n
    tops = lambda us: op_count / us / 1e6
    med = float(np.median(both))
    kern = float(np.median(mm))
    # Q4_K above 64 rows forms its exact integer dots on the f16 matrix unit (scale folded into
    # the weight operand), so that unit's dense peak prices it; the int8 fraction is kept beside
    # it because the target is quoted on the int8 peak.
    if wtype == Q4K:
        kernel = "q4k_wide_dense_kernel (+ q4k_tokens_f16_kernel once per call)" if m > 128 else "q4k_f16_dense_kernel"
        peak, dtype = F16_PEAK_TFLOPS, "f16 operands (exact integers), f32 accumulate"
    elif wtype == Q6K:
        kernel, peak, dtype = "mmq_dense_kernel<MmqQ6K,128,1>", INT8_PEAK_TOPS, "int8"
    else:
        kernel, peak, dtype = f"mmq_dense_kernel<{NAMES[wtype]} tile policy,128,1>", INT8_PEAK_TOPS, "int8"
    roofline = {"bound": "mfma", "achieved": round(tops(kern), 1), "peak": peak, "unit": "TOP/s",
                "frac": round(tops(kern) / peak, 4), "frac_of_int8_peak": round(tops(kern) / INT8_PEAK_TOPS, 4),
                "traffic": None, "kernel": kernel, "avg_launch_us": round(float(mm.mean()), 3),
                "algorithmic_ops_per_launch": int(op_count), "launches_timed": launches}
    extra = {"matmul_launch": dict(spread(mm), tops_median=round(tops(kern), 1)), "quantizer_launch": spread(qu),
             "call_two_launches": dict(spread(both), tops_median=round(tops(med), 1))}
    return line(args, tops(med), "TOP/s", med * 1e-3, dtype,
                {"workload": f"tiled matmul {m} rows x {k} -> {n}, {NAMES[wtype]} weights, quantizer + matmul",
                 "ops": int(op_count)}, roofline, extra)


# ---------------------------------------------------------------------------- moe
def moe_block(args, dev):
    experts, hidden, ffn, topk, tokens = 128, 2048, 768, 8, args.tokens
    mk = Maker(dev)
    # `--moe-wtype` other than q4_k: the same block with every expert matrix in that format
    name = args.moe_wtype
    wt = WTYPES[name]
    if wt == Q4K:
        gate = mk.q4k(experts * ffn, hidden)
        up = mk.q4k(experts * ffn, hidden)
        down = mk.q4k(experts * hidden, ffn)
    else:
        def stack(n, k, stream):   # a few generated rows repeated: the kernels do not care what the blocks hold
            base = torch.from_numpy(synth.weight(wt, 256, k, seed=0, stream=stream)).to(dev).reshape(256, -1)
            return base.repeat(n // 256, 1).contiguous().reshape(-1)
        gate, up, down = stack(experts * ffn, hidden, 1), stack(experts * ffn, hidden, 2), stack(experts * hidden, ffn, 3)
    x = mk.randn(tokens, hidden)
    logits = mk.randn(tokens, experts)
    probs = torch.softmax(logits, dim=-1)
    weights, choices = torch.topk(probs, topk, dim=-1)
    weights = (weights / weights.sum(dim=-1, keepdim=True)).contiguous()
    choices = choices.to(torch.int32).contiguous()

    pairs = tokens * topk
    tiled = moe.moe_mmq_pays(pairs, experts, wt) if args.moe_path == "auto" else args.moe_path in ("tiled", "rows")
    tiled = tiled and moe.moe_mmq_serves(wt, hidden) and moe.moe_mmq_serves(wt, ffn)
    # The routing (the router's side of the boundary) is built once; the timed block is what the
    # expert launchers do with it, recorded into a graph so that the host's cost stays outside.
    rows_launch = False

    def block_of(gate, up, down, choices, weights):
        nonlocal rows_launch
        flat_w = weights.reshape(-1)
        if tiled:
            plan = moe.MmqRouting.from_choices(choices, experts).with_path(args.moe_path if args.moe_path in ("tiled", "rows") else "auto")
            rows_launch = plan.takes_rows_launch(wt, hidden)

            def block():
                h = plan.gate_up_silu(wt, x, gate, up, ffn)
                return plan.down_fold(wt, h, down, hidden, flat_w)
        else:
            routing = moe.ExpertRouting(choices)

            def block():   # x + experts(x): the residual enters where the fold writes its sum
                h = moe.moe_gemm_gguf_gate_up_silu_mul(wt, x, gate, up, routing, experts, ffn)
                return moe.moe_gemm_gguf_down_reduce(wt, h, down, routing, flat_w, experts, hidden, add_after=x)
        return block

    block = block_of(gate, up, down, choices, weights)
    eager = time_launches(lambda i: block(), args.launches)
    single = time_replays(capture(block), args.launches)
    # The block as a decode step holds it: one graph of `layers` blocks, each layer with its own copy of
    # the expert tensors and its own routing, so that no replay finds a layer's experts in a cache (a
    # graph of one block also carries the whole cost of starting a graph, some microseconds, which a
    # step of many layers pays once). More layers at few tokens: a layer then touches few experts.
    layers = 24 if pairs <= 512 else 4
    blocks, layer_choices = [block], [choices]
    for layer in range(1, layers):
        lg = mk.randn(tokens, experts)
        lw, lc = torch.topk(torch.softmax(lg, dim=-1), topk, dim=-1)
        lw = (lw / lw.sum(dim=-1, keepdim=True)).contiguous()
        layer_choices.append(lc.to(torch.int32).contiguous())
        blocks.append(block_of(gate.clone(), up.clone(), down.clone(), layer_choices[-1], lw))

    def step():
        for b in blocks:
            b()

    us = time_replays(capture(step), max(10, args.launches // 4)) / layers
    med = float(np.median(us))
    load = torch.bincount(choices.reshape(-1).to(torch.int64), minlength=experts).cpu().numpy()
    distinct = float(np.mean([int((torch.bincount(c.reshape(-1).to(torch.int64), minlength=experts) > 0).sum())
                              for c in layer_choices]))   # experts a layer's block reads, mean over the layers
    one_matrix = synth.weight_bytes(wt, ffn, hidden)
    # Both floors of the block: the bytes of the experts it reads at the HBM peak, and its multiply-adds
    # at the int8 matrix peak. The larger one binds (at 256 tokens every expert is read: 340 MB is
    # 42 us at 8 TB/s against 4 us of matrix work), and the block is reported against that one.
    nbytes = 3 * one_matrix * distinct
    op_count = 6.0 * pairs * ffn * hidden
    hbm_floor_us, mfma_floor_us = nbytes / HBM_PEAK_GBS / 1e3, op_count / INT8_PEAK_TOPS / 1e6
    gbs, tops = nbytes / med / 1e3, op_count / med / 1e6
    if tiled:
        kernel = f"q4k_rows_moe_kernel, {name}" if rows_launch else f"mmq_moe_kernel, {name}"
        note = ("whole expert block (quantize, two grouped matmuls with the activation in the first, fold)" if rows_launch
                else "whole expert block (plan, route, quantize, two grouped matmuls, activation, fold)")
    else:
        kernel = f"moe_rows_kernel / moe_rows_legacy_kernel, {name}"
        note = "whole expert block (quantize, gate/up pairs, down pairs, weighted sum)"
    note += "; bytes = 3 matrices per distinct expert read, ops = 6 x pairs x ffn x hidden"
    if hbm_floor_us >= mfma_floor_us:
        value, unit = gbs, "GB/s"
        roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": kernel, "note": note,
                    "algorithmic_bytes_per_launch": int(nbytes), "avg_launch_us": round(float(us.mean()), 3),
                    "other_floor": {"bound": "mfma", "achieved": round(tops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                    "frac": round(tops / INT8_PEAK_TOPS, 4)}}
    else:
        value, unit = tops, "TOP/s"
        roofline = {"bound": "mfma", "achieved": round(tops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                    "frac": round(tops / INT8_PEAK_TOPS, 4), "traffic": None, "kernel": kernel, "note": note,
                    "algorithmic_ops_per_launch": int(op_count), "avg_launch_us": round(float(us.mean()), 3),
                    "other_floor": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                    "frac": round(gbs / HBM_PEAK_GBS, 4)}}
    extra = {"block_in_step_graph": dict(spread(us), blocks_per_graph=layers), "block_graph_replay": spread(single),
             "block_eager_from_python": spread(eager), "path": ("expert-batched rows on the matrix unit" if rows_launch else "expert-batched tiled matmul") if tiled else "mat-vec per routed pair",
             "routed_pairs": pairs, "distinct_experts": distinct,
             "expert_load_histogram": {"max": int(load.max()), "mean": round(float(load.mean()), 2),
                                       "rows_per_expert_sorted_top8": sorted(load.tolist(), reverse=True)[:8]}}
    return line(args, value, unit, med * 1e-3, "int8",
                {"workload": f"MoE expert block, 128 experts 2048->768->2048 {name}, top-8, {tokens} tokens"}, roofline,
                extra)


# ---------------------------------------------------------------------------- decode-1p7b
def decode_1p7b(args, dev):
    L = lib.load()
    b = args.batch
    hidden, kv, ffn, vocab, layers = 2048, 1024, 6144, 151936, 28
    mk = Maker(dev)
    s = torch.cuda.current_stream().cuda_stream
    info = ops.MMQ_DEVICE_INFO
    groups = [("x", hidden, Q4K, [hidden, kv, kv]), ("attn", hidden, Q4K, [hidden]), ("x2", hidden, Q4K, [ffn, ffn]),
              ("h", ffn, Q6K, [hidden])]
    acts = {g: mk.randn(b, k) for g, k, _, _ in groups}
    acts["final"] = mk.randn(b, hidden)
    keep, plan, total_bytes = [], [], 0
    matvec = b <= 8
    used = {"rows": 0, "matvec": 0, "tiled": 0}

    def rows_kernel_serves(wtype, n, k, rows):   # the rule of host_qmatmul.hip
        if wtype != Q6K and 8 < rows <= 16 and k >= 8192 and n >= 2048:
            return False
        return rows <= 16 or n * rows * max(k, 4096) <= 450000 * 4096 * (2048 // max(n, 1) if n < 2048 else 1)

    # 3 to 16 rows: the 16-row-tile kernels on the matrix unit, the matrices that share an activation in
    # one launch (q + k + v; gate + up with the activation on top, as dense_q4k_imma_m8_act_mul of the
    # reference does)
    fused_rows = 3 <= b <= 16 and args.mid_rows == "auto"
    matvec = matvec and not fused_rows

    rows_h_q81 = torch.empty((b, ffn // 32, 36), dtype=torch.uint8, device=dev) if fused_rows else None
    # above 16 rows, while the rows kernels serve gate + up and down: the same hand-over
    mid_h_q81 = (torch.empty((b, ffn // 32, 36), dtype=torch.uint8, device=dev)
                 if (not fused_rows and not matvec and args.mid_rows == "auto" and rows_kernel_serves(Q4K, ffn, hidden, b)
                     and rows_kernel_serves(Q6K, hidden, ffn, b)) else None)

    def quantize_or_take(g, x, q, k):
        """The Q8_1 rows of group `g`: a quantizer launch of the step, or (--acts norm-q8_1, the groups a norm
        feeds) written once here, as the model's RMSNorm launch that also quantizes would leave them."""
        item = ("status", L.lk_quantize_q8_1, (x.data_ptr(), lib.TYPE_F32, q.data_ptr(), k, k, b, s))
        if getattr(args, "acts", "f32") == "norm-q8_1" and g in ("x", "x2"):
            check(item[1](*item[2]), "lk_quantize_q8_1")
            return
        plan.append(item)

    def add_fused_rows(g, k, wtype, ns):
        nonlocal total_bytes
        weights = [mk.make(wtype, n, k) for n in ns]
        keep.extend(weights)
        total_bytes += sum(synth.weight_bytes(wtype, n, k) for n in ns)
        x = acts[g]
        used["rows"] += len(ns)
        if g == "h":   # `down` reads the Q8_1 rows the gate + up launch wrote
            out = torch.empty((b, ns[0]), device=dev)
            keep.append(out)
            if b <= 6 and ns[0] * k < (48 << 20):   # a small matrix at few rows: the mat-vec (host_qmatmul.hip's rule)
                plan.append(("status", L.lk_mmvq, (wtype, weights[0].data_ptr(), rows_h_q81.data_ptr(), out.data_ptr(), lib.TYPE_F32,
                                                   k, ns[0], b, k // 32, ns[0], None, 0, s)))
                used["rows"] -= 1
                used["matvec"] += 1
            else:
                plan.append(("status", L.lk_dense_q6k_rows, (weights[0].data_ptr(), rows_h_q81.data_ptr(), out.data_ptr(), b, ns[0], k, s)))
            return
        q = torch.empty((b, k // 32, 36), dtype=torch.uint8, device=dev)
        keep.append(q)
        quantize_or_take(g, x, q, k)
        if wtype == Q6K:
            for w, n in zip(weights, ns):
                out = torch.empty((b, n), device=dev)
                keep.append(out)
                plan.append(("status", L.lk_dense_q6k_rows, (w.data_ptr(), q.data_ptr(), out.data_ptr(), b, n, k, s)))
        elif g == "x2":
            plan.append(("status", L.lk_dense_q4k_rows_actmul_q8_1,
                         (weights[0].data_ptr(), weights[1].data_ptr(), q.data_ptr(), rows_h_q81.data_ptr(), b, ns[0], k, 0, 0, s)))
        else:
            outs = [torch.empty((b, n), device=dev) for n in ns]
            vx = (lib.C.c_void_p * len(ns))(*[w.data_ptr() for w in weights])
            dst = (lib.C.c_void_p * len(ns))(*[o.data_ptr() for o in outs])
            nn = (lib.C.c_int * len(ns))(*ns)
            keep.extend(outs + [vx, dst, nn])
            plan.append(("status", L.lk_dense_q4k_rows_multi, (vx, dst, nn, len(ns), q.data_ptr(), b, k, 0, s)))

    # one or two rows: gate + up as the pair launch that applies SiLU and writes the Q8_1 rows `down`
    # reads (the default plan of the Llama step), so `down` needs neither the f32 rows nor a quantizer
    paired = matvec and b <= 2
    h_q81 = torch.empty((b, ops.pad_to(ffn, 512) // 32, 36), dtype=torch.uint8, device=dev) if paired else None

    def add_group(g, k, wtype, ns):
        nonlocal total_bytes
        if fused_rows:
            return add_fused_rows(g, k, wtype, ns)
        weights = [mk.make(wtype, n, k) for n in ns]
        keep.extend(weights)
        total_bytes += sum(synth.weight_bytes(wtype, n, k) for n in ns)
        x = acts[g]
        from_norm = getattr(args, "acts", "f32") == "norm-q8_1" and g in ("x", "x2") and k <= 8192
        if from_norm and matvec:
            # the group's rows arrive as Q8_1, as the model's quantizing norm leaves them: written once here
            qn = torch.empty((b, ops.pad_to(k, 512) // 32, 36), dtype=torch.uint8, device=dev)
            keep.append(qn)
            check(L.lk_quantize_q8_1(x.data_ptr(), lib.TYPE_F32, qn.data_ptr(), k, qn.shape[1] * 32, b, s), "lk_quantize_q8_1")
        if paired and g == "x2" and from_norm:
            plan.append(("status", L.lk_mmvq_pair_act_q8_1, (wtype, weights[0].data_ptr(), weights[1].data_ptr(), qn.data_ptr(), 0,
                                                              qn.shape[1], h_q81.data_ptr(), h_q81.shape[1], k, ns[0], b, 0, s)))
        elif paired and g == "x2":
            plan.append(("status", L.lk_mmvq_pair_act_q8_1, (wtype, weights[0].data_ptr(), weights[1].data_ptr(), x.data_ptr(), 1,
                                                              x.stride(0), h_q81.data_ptr(), h_q81.shape[1], k, ns[0], b, 0, s)))
        elif paired and g == "h":
            out = torch.empty((b, ns[0]), device=dev)
            keep.append(out)
            plan.append(("status", L.lk_mmvq, (wtype, weights[0].data_ptr(), h_q81.data_ptr(), out.data_ptr(), lib.TYPE_F32, k,
                                               ns[0], b, h_q81.shape[1], ns[0], None, 0, s)))
        elif matvec and k <= 8192:
            stride = max(ns)
            outs = [torch.empty((b, stride), device=dev) for _ in ns]
            vx = (lib.C.c_void_p * len(ns))(*[w.data_ptr() for w in weights])
            dst = (lib.C.c_void_p * len(ns))(*[o.data_ptr() for o in outs])
            nn = (lib.C.c_int * len(ns))(*ns)
            keep.extend(outs + [vx, dst, nn])
            if from_norm:
                plan.append(("status", L.lk_mmvq_multi, (wtype, len(ns), vx, qn.data_ptr(), dst, lib.TYPE_F32, k, nn, b, qn.shape[1],
                                                          stride, None, s)))
            else:
                plan.append(("status", L.lk_mmvq_fused, (wtype, len(ns), vx, x.data_ptr(), x.stride(0), dst, lib.TYPE_F32, k, nn, b,
                                                          stride, None, s)))
        elif matvec:
            q = torch.empty((b, ops.pad_to(k, 512) // 32, 36), dtype=torch.uint8, device=dev)
            keep.append(q)
            plan.append(("status", L.lk_quantize_q8_1, (x.data_ptr(), lib.TYPE_F32, q.data_ptr(), k, q.shape[1] * 32, b, s)))
            for w, n in zip(weights, ns):
                out = torch.empty((b, n), device=dev)
                keep.append(out)
                plan.append(("status", L.lk_mmvq, (wtype, w.data_ptr(), q.data_ptr(), out.data_ptr(), lib.TYPE_F32, k, n, b,
                                         q.shape[1], n, None, 0, s)))
        elif args.mid_rows == "auto" and all(rows_kernel_serves(wtype, n, k, b) for n in ns):
            # the host mirror's choice (host_qmatmul.hip): the matrix-unit rows kernels, no weight staging
            if g == "h" and mid_h_q81 is not None:   # `down` reads the Q8_1 rows the gate + up launch wrote
                out = torch.empty((b, ns[0]), device=dev)
                keep.append(out)
                plan.append(("status", L.lk_dense_q6k_rows, (weights[0].data_ptr(), mid_h_q81.data_ptr(), out.data_ptr(), b, ns[0], k, s)))
                used["rows"] += 1
                return
            q = torch.empty((b, k // 32, 36), dtype=torch.uint8, device=dev)
            keep.append(q)
            quantize_or_take(g, x, q, k)
            if g == "x2" and wtype == Q4K:
                # gate and up with the activation on top in one launch (dense_q4k_imma_m8_act_mul of the reference),
                # its result handed on as the Q8_1 rows `down` reads
                plan.append(("status", L.lk_dense_q4k_rows_actmul_q8_1,
                             (weights[0].data_ptr(), weights[1].data_ptr(), q.data_ptr(), mid_h_q81.data_ptr(), b, ns[0], k, 0, 0, s)))
                used["rows"] += 2
                return
            if wtype == Q4K and len(ns) > 1:   # q + k + v: one launch over the three matrices
                outs = [torch.empty((b, n), device=dev) for n in ns]
                vx = (lib.C.c_void_p * len(ns))(*[w.data_ptr() for w in weights])
                dst = (lib.C.c_void_p * len(ns))(*[o.data_ptr() for o in outs])
                nn = (lib.C.c_int * len(ns))(*ns)
                keep.extend(outs + [vx, dst, nn])
                plan.append(("status", L.lk_dense_q4k_rows_multi, (vx, dst, nn, len(ns), q.data_ptr(), b, k, 0, s)))
                used["rows"] += len(ns)
                return
            for w, n in zip(weights, ns):
                out = torch.empty((b, n), device=dev)
                keep.append(out)
                plan.append(("status", L.lk_dense_q4k_rows if wtype == Q4K else L.lk_dense_q6k_rows,
                             (w.data_ptr(), q.data_ptr(), out.data_ptr(), b, n, k, s)))
                used["rows"] += 1
        elif b <= 32 and args.mid_rows == "matvec":
            # mat-vec launches over slices of eight rows
            used["matvec"] += len(ns)
            q = torch.empty((b, ops.pad_to(k, 512) // 32, 36), dtype=torch.uint8, device=dev)
            keep.append(q)
            plan.append(("status", L.lk_quantize_q8_1, (x.data_ptr(), lib.TYPE_F32, q.data_ptr(), k, q.shape[1] * 32, b, s)))
            for w, n in zip(weights, ns):
                out = torch.empty((b, n), device=dev)
                keep.append(out)
                for r0 in range(0, b, 8):
                    rows = min(8, b - r0)
                    plan.append(("status", L.lk_mmvq, (wtype, w.data_ptr(), q[r0].data_ptr(), out[r0].data_ptr(),
                                                        lib.TYPE_F32, k, n, rows, q.shape[1], n, None, 0, s)))
        else:
            used["tiled"] += len(ns)
            k_padded = ops.pad_to(ops.pad_to(k, 512), 128)
            ws = torch.empty(ops.mmq_workspace_bytes(b, k), dtype=torch.uint8, device=dev)
            keep.append(ws)
            plan.append(("void", getattr(L, ops.MMQ_QUANTIZER[wtype]),
                         (x.data_ptr(), None, ws.data_ptr(), 0, k, x.stride(0), 0, 0, k_padded, b, 1, 1, s)))
            for w, n in zip(weights, ns):
                out = torch.empty((b, n), device=dev)
                keep.append(out)
                plan.append(("tile", getattr(L, ops.MMQ_LAUNCHER[wtype]),
                             (ops.mmq_fixup(dev).data_ptr(), w.data_ptr(), ws.data_ptr(), out.data_ptr(), k, n, b, k // 256, n, info["cc"],
                              info["nsm"], info["smpbo"], info["warp_size"], s)))

    for _ in range(layers):
        for g, k, wtype, ns in groups:
            add_group(g, k, wtype, ns)
    add_group("final", hidden, Q6K, [vocab])
    def run(items):
        for kind, fn, a in items:
            rc = fn(*a)
            if kind == "tile" and rc == 0:      # tile width launched; 0 = nothing ran
                raise lib.LokenError("tiled matmul launcher", lib.LK_ERR_ARG)
            if kind == "status" and rc:
                raise lib.LokenError("mat-vec launcher", rc)

    run(plan)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        cap = [(kind, fn, a[:-1] + (side.cuda_stream,)) for kind, fn, a in plan]
        run(cap)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            run(cap)
    torch.cuda.synchronize()
    # at least 20 warm-up replays and 200 timed ones, each replay between its own pair of events
    us = time_replays(graph, max(200, args.steps), warm=max(20, args.warmup))
    ms = float(np.median(us)) * 1e-3
    value = total_bytes / (ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "achieved": round(value, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(value / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel": "whole step (all launches of the graph)", "launches_per_step": len(plan)}
    return line(args, value, "GB/s", ms, "int8",
                {"workload": f"qwen3-1.7b decode-step quantized linears (Q4_K attention and gate/up, Q6_K down and "
                             f"lm_head), batch {b}, 28 layers",
                 "path": "mat-vec (fused: q + k + v, o from f32 rows; gate + up as the pair launch that writes down's Q8_1 rows)" if paired
                         else "mat-vec (fused; own quantizer launch for rows over 8192 values)" if matvec
                         else "16-row tiles on the matrix unit: q + k + v in one launch, o, gate + up with SiLU in one launch that writes "
                              "the Q8_1 rows down reads, down, lm_head; a Q8_1 quantizer launch before the others" if fused_rows
                         else f"linears on the matrix-unit rows kernels: {used['rows']}, as mat-vec slices of eight rows: "
                              f"{used['matvec']}, on the tiled matmul: {used['tiled']}",
                 "acts": "f32 rows into every group" if getattr(args, "acts", "f32") == "f32"
                         else "q + k + v and gate + up read Q8_1 rows as the model's RMSNorm launches that also quantize leave them "
                              "(those launches are not timed); o and lm_head from f32 rows",
                 "weight_bytes_per_step": total_bytes, "launches_per_step": len(plan), "hip_graph": True}, roofline,
                {"step_spread": spread(us), "ms_per_step_is": "median of the timed replays"})


# ---------------------------------------------------------------------------- short forms for the default line
def brief_gemv_4096(launches=64, replays=50):
    """Config 0 for the default benchmark line: the Q4_K 4096 x 4096 mat-vec at one row as a graph of
    `launches` launches over that many rotating copies (604 MB at 64: past twice the last-level
    cache), from a Q8_1 row and from the f32 row quantized in the kernel."""
    L = lib.load()
    dev = torch.device("cuda:0")
    n = k = 4096
    nbytes = synth.weight_bytes(Q4K, n, k)
    base = torch.from_numpy(synth.weight(Q4K, n, k, seed=0, stream=0)).to(dev).reshape(-1)
    copies = [base.clone() for _ in range(launches)]
    x = torch.from_numpy(synth.activation(1, k, seed=0)).to(dev)
    q = ops.quantize_q8_1_rows(x)
    out = torch.empty((1, n), device=dev)
    keep = []

    def plain():
        s2 = torch.cuda.current_stream().cuda_stream
        for w in copies:
            check(L.lk_mmvq(Q4K, w.data_ptr(), q.data_ptr(), out.data_ptr(), lib.TYPE_F32, k, n, 1, q.shape[1], n, None, 0,
                            s2), "lk_mmvq")

    def fused():
        s2 = torch.cuda.current_stream().cuda_stream
        dst = (lib.C.c_void_p * 1)(out.data_ptr())
        nn = (lib.C.c_int * 1)(n)
        for w in copies:
            vx = (lib.C.c_void_p * 1)(w.data_ptr())
            keep.append(vx)
            check(L.lk_mmvq_fused(Q4K, 1, vx, x.data_ptr(), x.stride(0), dst, lib.TYPE_F32, k, nn, 1, n, None, s2),
                  "lk_mmvq_fused")

    all_us = time_replays(capture(plain), replays) / launches
    all_fused = time_replays(capture(fused), replays) / launches
    us, us_fused = float(np.median(all_us)), float(np.median(all_fused))
    return {"workload": "Q4_K 4096x4096 mat-vec, one row, seed 0, graph of %d launches over %d rotating copies" % (launches, launches),
            "weight_bytes": nbytes, "us_per_launch": round(us, 3), "gbs": round(nbytes / us / 1e3, 1),
            "frac_of_8tbs": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
            "per_launch": dict(spread(all_us), launches=replays * launches),
            "f32_activation_quantized_in_kernel": {"us_per_launch": round(us_fused, 3),
                                                   "gbs": round(nbytes / us_fused / 1e3, 1),
                                                   "per_launch": dict(spread(all_fused), launches=replays * launches)}}


def brief_mmq(shape, launches=200):
    """Configs 2a / 2b for the default benchmark line: median of event-bracketed launches of the tiled
    matmul alone and of quantizer + matmul."""
    L = lib.load()
    dev = torch.device("cuda:0")
    wtype, m, k, n = {"2a": (Q4K, 512, 4096, 14336), "2b": (Q6K, 2048, 14336, 4096)}[shape]
    mk = Maker(dev)
    w = mk.make(wtype, n, k)
    x = mk.randn(m, k)
    out = torch.empty((m, n), device=dev)
    ws = ops.mmq_quantize(wtype, x)
    quantizer = getattr(L, ops.MMQ_QUANTIZER[wtype])
    launcher = getattr(L, ops.MMQ_LAUNCHER[wtype])
    info = ops.MMQ_DEVICE_INFO
    s = torch.cuda.current_stream().cuda_stream
    k_padded = ops.pad_to(ops.pad_to(k, 512), 128)

    def quant():
        quantizer(x.data_ptr(), None, ws.data_ptr(), 0, k, x.stride(0), 0, 0, k_padded, m, 1, 1, s)

    def matmul():
        if launcher(ops.mmq_fixup(dev).data_ptr(), w.data_ptr(), ws.data_ptr(), out.data_ptr(), k, n, m, k // synth.BLOCK_LEN[wtype], n,
                    info["cc"], info["nsm"], info["smpbo"], info["warp_size"], s) == 0:
            raise lib.LokenError(ops.MMQ_LAUNCHER[wtype], lib.LK_ERR_ARG)

    mm_all = time_launches(lambda i: matmul(), launches)
    both_all = time_launches(lambda i: (quant(), matmul()), launches)
    mm, both = float(np.median(mm_all)), float(np.median(both_all))
    op_count = 2.0 * m * k * n
    return {"workload": f"tiled matmul {m} rows x {k} -> {n}, {NAMES[wtype]}", "ops": int(op_count),
            "kernel": "q4k_wide_dense_kernel after q4k_tokens_f16_kernel (exact integers on f16 operands)" if wtype == Q4K else "mmq_dense_kernel<MmqQ6K,128,1>",
            "matmul_us": round(mm, 2), "tops": round(op_count / mm / 1e6, 1), "matmul_launch": spread(mm_all),
            "call_two_launches": spread(both_all),
            "frac_of_int8_peak": round(op_count / mm / 1e6 / INT8_PEAK_TOPS, 4),
            "quantize_plus_matmul_us": round(both, 2), "tops_with_quantizer": round(op_count / both / 1e6, 1)}


# ---------------------------------------------------------------------------- rows kernels against tiles
def rows_sweep(args, dev):
    """One weight matrix at a ladder of row counts: quantizer + matrix-unit rows kernel against
    quantizer + tiled matmul, each as a graph replay of the two launches, and the path the host
    mirror of QKernelMatMul::forward takes. The crossover constants in host_qmatmul.hip come from
    these tables."""
    L = lib.load()
    wtype = {"q4_k": Q4K, "q5_k": WTYPES["q5_k"], "q6_k": Q6K}.get(args.wtype)
    if wtype is None:
        raise SystemExit("--workload rows-sweep: --wtype q4_k, q5_k or q6_k")
    n, k = args.rows_n, args.cols_k
    mk = Maker(dev)
    w = mk.make(wtype, n, k)
    quantizer = getattr(L, ops.MMQ_QUANTIZER[wtype])
    launcher = getattr(L, ops.MMQ_LAUNCHER[wtype])
    rows_fn = {Q4K: L.lk_dense_q4k_rows, Q6K: L.lk_dense_q6k_rows}.get(wtype, L.lk_dense_q5k_rows)
    info = ops.MMQ_DEVICE_INFO
    k_padded = ops.pad_to(ops.pad_to(k, 512), 128)
    handle = L.lkh_qkernel_matmul_new(wtype, n, k, w.data_ptr(), dev.index or 0)
    paths = {1: "matvec-fused", 2: "matvec", 3: "rows-on-matrix-unit", 4: "tiled"}
    table = []
    for m in (16, 32, 64, 128, 256, 512, 1024, 2048):
        x = mk.randn(m, k)
        out = torch.empty((m, n), device=dev)
        ws = torch.empty(ops.mmq_workspace_bytes(m, k), dtype=torch.uint8, device=dev)
        q = torch.empty((m, k // 32, 36), dtype=torch.uint8, device=dev)

        def tiled():
            s = torch.cuda.current_stream().cuda_stream
            quantizer(x.data_ptr(), None, ws.data_ptr(), 0, k, x.stride(0), 0, 0, k_padded, m, 1, 1, s)
            if launcher(ops.mmq_fixup(dev).data_ptr(), w.data_ptr(), ws.data_ptr(), out.data_ptr(), k, n, m, k // synth.BLOCK_LEN[wtype], n,
                        info["cc"], info["nsm"], info["smpbo"], info["warp_size"], s) == 0:
                raise lib.LokenError(ops.MMQ_LAUNCHER[wtype], lib.LK_ERR_ARG)

        def rows():
            s = torch.cuda.current_stream().cuda_stream
            check(L.lk_quantize_q8_1(x.data_ptr(), lib.TYPE_F32, q.data_ptr(), k, k, m, s), "lk_quantize_q8_1")
            check(rows_fn(w.data_ptr(), q.data_ptr(), out.data_ptr(), m, n, k, s), "rows kernel")

        t_tiled = float(np.median(time_replays(capture(tiled), args.launches)))
        t_rows = float(np.median(time_replays(capture(rows), args.launches)))
        check(L.lkh_qkernel_matmul_forward(handle, x.data_ptr(), lib.TYPE_F32, m, out.data_ptr(),
                                           torch.cuda.current_stream().cuda_stream, 0), "lkh_qkernel_matmul_forward")
        table.append({"rows": m, "rows_kernel_us": round(t_rows, 1), "tiled_us": round(t_tiled, 1),
                      "forward_takes": paths.get(L.lkh_qkernel_matmul_last_path(handle), "none")})
    L.lkh_qkernel_matmul_free(handle)
    best = min(table, key=lambda r: min(r["rows_kernel_us"], r["tiled_us"]) / r["rows"])
    op_count = 2.0 * best["rows"] * k * n
    us = min(best["rows_kernel_us"], best["tiled_us"])
    return line(args, op_count / us / 1e6, "TOP/s", us * 1e-3, "int8",
                {"workload": f"{NAMES[wtype]} {n} x {k}: quantizer + rows kernel against quantizer + tiled matmul, graph replays"},
                None, {"table": table})


# ---------------------------------------------------------------------------- prefill-layer
def prefill_layer(args, dev):
    """The quantized linears of one Llama-3-8B layer (Q4_K_M: q, k, v, o, gate, up Q4_K; down Q6_K) at
    `--tokens` rows, each through the host mirror of QKernelMatMul::forward (which picks the kernel
    family by row count), over `--layers` layers with their own weights, as one HIP graph."""
    L = lib.load()
    m = args.tokens
    hidden, kv, ffn = 4096, 1024, 14336
    linears = [("q", Q4K, hidden, hidden, "x"), ("k", Q4K, kv, hidden, "x"), ("v", Q4K, kv, hidden, "x"),
               ("o", Q4K, hidden, hidden, "attn"), ("gate", Q4K, ffn, hidden, "x2"), ("up", Q4K, ffn, hidden, "x2"),
               ("down", Q6K, hidden, ffn, "h")]
    layers = max(1, args.layers)
    mk = Maker(dev)
    acts = {"x": mk.randn(m, hidden), "attn": mk.randn(m, hidden), "x2": mk.randn(m, hidden), "h": mk.randn(m, ffn)}
    paths = {1: "matvec-fused", 2: "matvec", 3: "rows-on-matrix-unit", 4: "tiled"}
    keep, handles, per_layer = [], [], []
    for _ in range(layers):
        row = []
        for name, wtype, n, k, src in linears:
            w = mk.make(wtype, n, k)
            out = torch.empty((m, n), device=dev)
            h = L.lkh_qkernel_matmul_new(wtype, n, k, w.data_ptr(), dev.index or 0)
            keep.extend([w, out])
            handles.append(h)
            row.append((name, h, acts[src], out, wtype, n, k))
        per_layer.append(row)

    def one(h, x, out):
        check(L.lkh_qkernel_matmul_forward(h, x.data_ptr(), lib.TYPE_F32, m, out.data_ptr(),
                                           torch.cuda.current_stream().cuda_stream, 0), "lkh_qkernel_matmul_forward")

    def step():
        for row in per_layer:
            for _, h, x, out, *_ in row:
                one(h, x, out)

    us = time_replays(capture(step), max(20, args.launches))
    table = []
    for name, h, x, out, wtype, n, k in per_layer[0]:
        t = float(np.median(time_replays(capture(lambda: one(h, x, out)), 50)))
        table.append({"linear": name, "wtype": NAMES[wtype], "n": n, "k": k, "us": round(t, 1),
                      "path": paths.get(L.lkh_qkernel_matmul_last_path(h), "none"),
                      "tops": round(2.0 * m * n * k / t / 1e6, 1)})
    for h in handles:
        L.lkh_qkernel_matmul_free(h)
    ops_layer = sum(2.0 * m * n * k for _, _, n, k, _ in linears)
    med = float(np.median(us)) / layers
    return line(args, ops_layer / med / 1e6, "TOP/s", med * 1e-3, "int8 / f16 operands (exact integers), f32 accumulate",
                {"workload": f"Llama-3-8B layer, quantized linears at {m} rows through forward(), {layers} layers a graph replay"},
                None, {"per_layer_us": spread(us / layers), "ops_per_layer": ops_layer, "linears": table})


def run(args) -> int:
    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible")
    lib.load()  # raises if the HIP library is missing: there is no other path
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    return {"gemv": gemv, "gemv-4096": gemv_4096, "mmq": mmq, "moe": moe_block, "decode-1p7b": decode_1p7b,
            "rows-sweep": rows_sweep, "prefill-layer": prefill_layer}[args.workload](args, dev)
