#!/usr/bin/env python3
"""Benchmark of the GGUF block-quantized matmul hot path on one MI355X.

One *step* = every quantized linear of one Llama-3-8B-shaped decode step at batch `--batch`
(default 1): per layer q, o 4096->4096, k, v 4096->1024, gate, up 4096->14336 in Q4_K and down
14336->4096 in Q6_K, 32 layers, then lm_head 4096->128256 in Q8_0: 225 weight matrices,
4.97 GB of blocks. Launch plans: `--plan fused`: the linears that share an activation go out as
one launch (q,k,v; gate,up) and every launch quantizes its f32 activation to Q8_1 in LDS itself,
4 launches per layer; `--plan split`: the two-launch form per linear (Q8_1 quantizer, then
mat-vec); `--plan rows`: the matrices on the matrix-unit kernels of 16-row tiles (q + k + v in one
launch, o, gate + up with SiLU in one launch, down, each after a Q8_1 quantizer launch); `--plan auto`
(default): at 1 and 2 rows fused, the gate,up launch applying SiLU(gate)*up and writing the Q8_1 rows
that `down` reads (4 launches per layer, no quantizer launch); from 3 rows `rows`, as measured on MI355X.
Distinct weights per layer, so the step is cache-cold by construction.
Weights and activations are synthetic (seeded, generated on the device) and resident in HBM
before the timed region.

`value` = the figure the metric names: Q4_K weight bytes of the step / time of the step's Q4_K mat-vec
launches (the reference's mat-vec convention: weight bytes only, src/tensor/cuda/quant.rs:3905,
3959-3961 of loken), whole job, one GPU; it is the roofline leg's `achieved`. `ms_per_step` and
`whole_step` are the whole step (Q4_K, Q6_K down, Q8_0 lm_head): EXACTLY `--steps` replays after
`--warmup` untimed ones between two synchronizations, and, beside that, 200 replays after 20 warm-ups
each between its own pair of events (median, p10, p90, min, max).

Two more measurements ride in the same JSON line:
  roofline      the dominant kernel (Q4_K mat-vec): average launch duration over the step's own
                mix of Q4_K launches, timed with HIP events on the launch stream, against the
                algorithmic weight bytes per launch and MI355X's 8 TB/s HBM peak.
  cpu_baseline  loken's served CPU decode path for Q4_K, restated (Q8_K activation, weights repacked
                eight rows at a time, persistent worker pool), on a bounded sample of the same
                workload, on this host's cores, over copies that together exceed twice the host's
                last-level cache (its size is printed); `legs` adds the served CPU prefill path on
                configuration 2a and the expert block of configuration 3 on the pool.
  gemv_4096     the benchmark set's configuration 0 (Q4_K 4096 x 4096, one row) over rotating copies.
  mmq           configurations 2a / 2b, the tiled matmul, against the int8 matrix peak.
  rows-sweep    one --wtype q4_k|q5_k|q6_k matrix (--rows-n x --cols-k) at 16..2048 rows: the matrix-unit
                rows kernel against the tiled matmul, and the path QKernelMatMul::forward's mirror takes.
  prefill-layer the quantized linears of one Llama-3-8B layer at --tokens rows, each through the host mirror of
                QKernelMatMul::forward (--layers of them, each with its own weights, a graph replay).
  other_configs the step at 4 and 8 rows, the MoE block at 1 / 16 / 256 tokens, the Qwen3-1.7B step at
                1 / 16 / 64 rows (configurations 1, 3, 4) and a Llama-3-8B layer's linears at 128 / 512 rows
                through forward(), each from a child run of this file.
  roofline.peak_measured / mmq.peak_measured: what a read-only launch and a register-resident
                matrix-instruction loop reach on this card (loken_amd/probes.py).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel's launch mix, from the two rocprofv3 counter runs
# (FETCH_SIZE, then WRITE_SIZE, scaled by a plain 1 GiB copy) summarized in
# profiles/mmvq_llama3_8b_decode_b1_hbm_traffic.md. Counters cannot be read from inside this
# process, so the figure is carried here for the configuration it was taken on:
# (launch plan, batch, layers) -> bytes.
MEASURED_TRAFFIC = {("auto", 1, 32): 30120755}
LAYERS = 32
HIDDEN, KV, FFN, VOCAB = 4096, 1024, 14336, 128256


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=1, help="activation rows per mat-vec (1..8)")
    ap.add_argument("--layers", type=int, default=LAYERS)
    ap.add_argument("--plan", choices=["auto", "fused", "split", "rows"], default="auto",
                    help="fused: shared-activation linears per launch, Q8_1 quantized in-kernel; split: quantize + "
                         "mat-vec per linear; rows: the Q4_K matrices on the matrix-unit rows kernel (q + k + v in one "
                         "launch, gate + up in one); auto: fused at one or two rows, except that rows longer than 8192 "
                         "values are quantized by their own launch (every workgroup of a fused launch quantizes the "
                         "whole row), and rows from three rows on")
    ap.add_argument("--acts", choices=["f32", "norm-q8_1"], default="f32",
                    help="the step (plans auto, fused, rows) and --workload decode-1p7b from three rows: f32 rows into every group "
                         "(a Q8_1 quantizer launch each), or q + k + v and gate + up reading Q8_1 rows as a model's "
                         "RMSNorm launches that also quantize (lk_rmsnorm_q8_1, lk_add_rmsnorm_q8_1) leave them: those "
                         "launches are the norms' and are not timed, o keeps its quantizer")
    ap.add_argument("--no-graph", action="store_true", help="launch the step eagerly instead of replaying a HIP graph")
    ap.add_argument("--cpu-seconds", type=float, default=20.0,
                    help="wall-clock budget of the CPU baseline samples together (mat-vec 40 %, prefill 30 %, expert block 30 %)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--brief", action="store_true",
                    help="the decode step and its roofline leg only: no config 0, tiled-matmul or ceiling measurements")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one plain device copy of 1 GiB before the steps: the dispatch of known size that "
                         "scales the FETCH_SIZE / WRITE_SIZE counters of a profiled run")
    ap.add_argument("--workload", choices=["decode", "gemv", "gemv-4096", "mmq", "moe", "decode-1p7b", "rows-sweep", "prefill-layer"], default="decode",
                    help="decode (default): the Llama-3-8B step described above; the others are the further measured "
                         "workloads of loken_amd/workloads.py, one JSON line each")
    ap.add_argument("--shape", choices=["2a", "2b"], default="2a", help="--workload mmq: 512x4096->14336 Q4_K or 2048x14336->4096 Q6_K")
    ap.add_argument("--mmq-wtype", default=None, help="--workload mmq: the shape in another format of the tiled matmul "
                    "(q8_0 q4_0 q4_1 q5_0 q5_1 q2_k q3_k q5_k)")
    ap.add_argument("--wtype", default="q4_0", help="--workload gemv: q4_0 q4_1 q5_0 q5_1 iq4_nl mxfp4 q8_0 q2_k q3_k q4_k q5_k q6_k iq4_xs iq2_xxs iq3_xxs iq3_s iq2_s q2_0")
    ap.add_argument("--rows-n", type=int, default=14336, help="--workload gemv: weight rows")
    ap.add_argument("--cols-k", type=int, default=4096, help="--workload gemv: values per row")
    ap.add_argument("--tokens", type=int, default=256, help="--workload moe / prefill-layer: rows through the expert block / the layer")
    ap.add_argument("--moe-wtype", default="q4_k", help="--workload moe: the experts' format (as --wtype)")
    ap.add_argument("--moe-path", choices=["auto", "tiled", "rows", "pairs"], default="auto",
                    help="--workload moe: expert-batched tiled matmul, expert-batched rows on the matrix unit, mat-vec per "
                         "routed pair, or the library's choice")
    ap.add_argument("--mid-rows", choices=["auto", "matvec", "tiled"], default="auto",
                    help="--workload decode-1p7b above 8 rows: auto = the host mirror's choice between the matrix-unit "
                         "rows kernels and the tiled matmul; matvec = mat-vec launches over slices of eight rows up to "
                         "32 rows; tiled = the tiled matmul")
    ap.add_argument("--launches", type=int, default=200, help="timed launches of the per-launch workloads")
    return ap.parse_args()


def other_configs():
    """ms per step (or per block) of the other configured workloads, from child runs of this file."""
    import subprocess

    def child(flags):
        # a child that hangs, dies or prints something else costs its own entry, never the parent's line
        try:
            r = subprocess.run([sys.executable, os.path.abspath(__file__), "--no-cpu-baseline", "--steps", "20", *flags],
                               capture_output=True, text=True, timeout=300)
            for ln in reversed(r.stdout.splitlines()):
                if ln.startswith("{"):
                    d = json.loads(ln)
                    out = {"ms_per_step": d["ms_per_step"], "value": d["value"], "unit": d["unit"]}
                    if "whole_step" in d:
                        out["whole_step_gbs"] = d["whole_step"]["gbs"]
                        out["spread"] = d["whole_step"]["per_step"]
                    for key in ("step_spread", "block_in_step_graph", "per_layer_us"):
                        if key in d:
                            out["spread"] = d[key]
                    if "linears" in d:
                        out["linears_us"] = {r["linear"]: [r["us"], r["path"]] for r in d["linears"]}
                    if d.get("roofline"):
                        out["roofline"] = {k: d["roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac") if k in d["roofline"]}
                    return out
            return {"error": (r.stderr or r.stdout)[-200:]}
        except subprocess.TimeoutExpired:
            return {"error": "child run exceeded 300 s and was ended"}
        except (OSError, ValueError, KeyError) as e:
            return {"error": f"{type(e).__name__}: {e}"[:200]}

    return {
        "llama3_8b_step_by_rows": {str(b): child(["--brief", "--batch", str(b)]) for b in (4, 8)},
        "moe_block_128x2048x768_top8_by_tokens": {str(t): child(["--workload", "moe", "--tokens", str(t)]) for t in (1, 16, 256)},
        "qwen3_1p7b_step_by_rows": {str(b): child(["--workload", "decode-1p7b", "--batch", str(b)]) for b in (1, 16, 64)},
        "same_steps_with_q8_1_rows_from_the_norms": {
            "llama3_8b_1_row": child(["--brief", "--acts", "norm-q8_1"]),
            "llama3_8b_8_rows": child(["--brief", "--batch", "8", "--acts", "norm-q8_1"]),
            "qwen3_1p7b_1_row": child(["--workload", "decode-1p7b", "--batch", "1", "--acts", "norm-q8_1"]),
            "qwen3_1p7b_16_rows": child(["--workload", "decode-1p7b", "--batch", "16", "--acts", "norm-q8_1"]),
            "qwen3_1p7b_64_rows": child(["--workload", "decode-1p7b", "--batch", "64", "--acts", "norm-q8_1"])},
        "llama3_8b_layer_linears_through_forward_by_rows": {
            str(t): child(["--workload", "prefill-layer", "--tokens", str(t), "--layers", "4"]) for t in (128, 512)},
    }


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus > 1 is not supported "
              "(no collectives or sharding are part of it).", file=sys.stderr)
        return 2

    if args.workload != "decode":
        from loken_amd import workloads
        return workloads.run(args)

    import torch
    from loken_amd import lib, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    L = lib.load()  # raises if the HIP library is missing: there is no other path
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev)
    gen.manual_seed(0)
    b = args.batch
    # `auto` from three rows on (measured on MI355X: 2.03 against 2.10 ms at 3 rows, 2.70 against 3.44 at 8):
    # the Q4_K matrices on the matrix-unit rows kernel, q + k + v in one launch and gate + up in one
    kind = args.plan if args.plan != "auto" or b <= 2 else "rows"

    # ------------------------------------------------------------------ synthetic blocks
    def halfs(n, scale):
        v = torch.randn(n, device=dev, generator=gen).abs() * scale
        return v.to(torch.float16).view(torch.uint8).reshape(n, 2)

    def make_q4k(n, k):
        nb = n * (k // 256)
        w = torch.randint(0, 256, (nb, 144), dtype=torch.uint8, device=dev, generator=gen)
        w[:, 0:2] = halfs(nb, 1e-3)
        w[:, 2:4] = halfs(nb, 5e-4)
        return w.reshape(-1)

    def make_q6k(n, k):
        nb = n * (k // 256)
        w = torch.randint(0, 256, (nb, 210), dtype=torch.uint8, device=dev, generator=gen)
        sc = torch.randint(-64, 64, (nb, 16), dtype=torch.int8, device=dev, generator=gen)
        w[:, 192:208] = sc.view(torch.uint8)
        w[:, 208:210] = halfs(nb, 1e-3)
        return w.reshape(-1)

    def make_q80(n, k):
        nb = n * (k // 32)
        w = torch.empty((nb, 34), dtype=torch.uint8, device=dev)
        w[:, 0:2] = halfs(nb, 1e-3)
        w[:, 2:] = torch.randint(-127, 128, (nb, 32), dtype=torch.int8, device=dev, generator=gen).view(torch.uint8)
        return w.reshape(-1)

    Q4K, Q6K, Q80 = lib.TYPE_Q4_K, lib.TYPE_Q6_K, lib.TYPE_Q8_0
    shapes = [  # (name, wtype, n, k, maker, activation group)
        ("q", Q4K, HIDDEN, HIDDEN, make_q4k, "x"), ("k", Q4K, KV, HIDDEN, make_q4k, "x"),
        ("v", Q4K, KV, HIDDEN, make_q4k, "x"), ("o", Q4K, HIDDEN, HIDDEN, make_q4k, "attn"),
        ("gate", Q4K, FFN, HIDDEN, make_q4k, "x2"), ("up", Q4K, FFN, HIDDEN, make_q4k, "x2"),
        ("down", Q6K, HIDDEN, FFN, make_q6k, "h"),
    ]
    stream = torch.cuda.current_stream().cuda_stream
    acts = {g: torch.randn((b, k), device=dev, generator=gen) for g, k in
            (("x", HIDDEN), ("attn", HIDDEN), ("x2", HIDDEN), ("h", FFN), ("final", HIDDEN))}
    q81 = {g: torch.empty((b, -(-a.shape[1] // 512) * 512 // 32, 36), dtype=torch.uint8, device=dev)
           for g, a in acts.items()}

    plan = []       # (fn, args) in launch order: one step
    q4k_plan = []   # the Q4_K mat-vec launches of a step
    q4k_launch_sizes = []   # their weight bytes, launch by launch
    total_bytes = 0
    q4k_bytes = 0
    keep = []

    def add_quant(g, from_norm=False):
        a, q = acts[g], q81[g]
        item = (L.lk_quantize_q8_1, (a.data_ptr(), lib.TYPE_F32, q.data_ptr(), a.shape[1], q.shape[1] * 32, b, stream))
        if from_norm and args.acts == "norm-q8_1":
            # the rows arrive quantized: written once here, outside the step
            rc = item[0](*item[1])
            if rc:
                raise lib.LokenError("lk_quantize_q8_1", rc)
            return
        plan.append(item)

    def add_gemv(wtype, w, g, n, k):
        nonlocal total_bytes, q4k_bytes
        out = torch.empty((b, n), dtype=torch.float32, device=dev)
        keep.append(out)
        q = q81[g]
        item = (L.lk_mmvq, (wtype, w.data_ptr(), q.data_ptr(), out.data_ptr(), lib.TYPE_F32, k, n, b,
                            q.shape[1], n, None, 0, stream))
        plan.append(item)
        nbytes = synth.weight_bytes(wtype, n, k)
        total_bytes += nbytes
        if wtype == Q4K:
            q4k_plan.append(item)
            q4k_bytes += nbytes
            q4k_launch_sizes.append(nbytes)
        return out

    import ctypes as C

    def add_fused(wtype, ws, g, ns, k):
        """One launch: the matrices `ws` (ns rows each) over activation group `g`, quantized in-kernel."""
        nonlocal total_bytes, q4k_bytes
        a = acts[g]
        stride = max(ns)
        outs = [torch.empty((b, stride), dtype=torch.float32, device=dev) for _ in ns]
        vx = (C.c_void_p * len(ws))(*[w.data_ptr() for w in ws])
        dst = (C.c_void_p * len(ws))(*[o.data_ptr() for o in outs])
        nn = (C.c_int * len(ws))(*ns)
        keep.extend(outs + [vx, dst, nn])
        if args.acts == "norm-q8_1" and g in ("x", "x2") and k <= 8192:
            # the group's rows arrive as Q8_1 (written once here, outside the step): the same launch over them
            add_quant(g, from_norm=True)
            q = q81[g]
            item = (L.lk_mmvq_multi, (wtype, len(ws), vx, q.data_ptr(), dst, lib.TYPE_F32, k, nn, b, q.shape[1], stride, None, stream))
        else:
            item = (L.lk_mmvq_fused, (wtype, len(ws), vx, a.data_ptr(), a.stride(0), dst, lib.TYPE_F32, k, nn, b,
                                      stride, None, stream))
        plan.append(item)
        nbytes = sum(synth.weight_bytes(wtype, n, k) for n in ns)
        total_bytes += nbytes
        if wtype == Q4K:
            q4k_plan.append(item)
            q4k_bytes += nbytes
            q4k_launch_sizes.append(nbytes)
        return outs[0]

    def add_pair(wtype, gate, up, g, n, k):
        """One launch: silu(gate . x) * (up . x) as Q8_1 rows in q81["h"] (which `down` then reads)."""
        nonlocal total_bytes, q4k_bytes
        a, q = acts[g], q81["h"]
        if args.acts == "norm-q8_1":
            add_quant(g, from_norm=True)
            item = (L.lk_mmvq_pair_act_q8_1, (wtype, gate.data_ptr(), up.data_ptr(), q81[g].data_ptr(), 0, q81[g].shape[1],
                                              q.data_ptr(), q.shape[1], k, n, b, 0, stream))
        else:
            item = (L.lk_mmvq_pair_act_q8_1, (wtype, gate.data_ptr(), up.data_ptr(), a.data_ptr(), 1, a.stride(0),
                                              q.data_ptr(), q.shape[1], k, n, b, 0, stream))
        plan.append(item)
        nbytes = 2 * synth.weight_bytes(wtype, n, k)
        total_bytes += nbytes
        if wtype == Q4K:
            q4k_plan.append(item)
            q4k_bytes += nbytes
            q4k_launch_sizes.append(nbytes)

    def add_rows(w, g, n, k):
        """Q4_K x the Q8_1 rows of group `g` on the matrix unit (the activation staged in LDS up to 8 rows)."""
        nonlocal total_bytes, q4k_bytes
        out = torch.empty((b, n), dtype=torch.float32, device=dev)
        keep.append(out)
        q = q81[g]
        assert q.shape[1] * 32 == k
        item = (L.loken_dense_q4k_imma_m8_plain, (w.data_ptr(), q.data_ptr(), out.data_ptr(), b, n, k, stream))
        plan.append(item)
        nbytes = synth.weight_bytes(Q4K, n, k)
        total_bytes += nbytes
        q4k_plan.append(item)
        q4k_bytes += nbytes
        q4k_launch_sizes.append(nbytes)
        return out

    def count_q4k(item, nbytes):
        nonlocal total_bytes, q4k_bytes
        plan.append(item)
        total_bytes += nbytes
        q4k_plan.append(item)
        q4k_bytes += nbytes
        q4k_launch_sizes.append(nbytes)

    def add_rows_multi(ws, g, ns, k):
        """Q4_K matrices sharing the Q8_1 rows of group `g`, one launch on the matrix unit."""
        outs = [torch.empty((b, n), dtype=torch.float32, device=dev) for n in ns]
        q = q81[g]
        assert q.shape[1] * 32 == k
        vx = (C.c_void_p * len(ws))(*[w.data_ptr() for w in ws])
        dst = (C.c_void_p * len(ws))(*[o.data_ptr() for o in outs])
        nn = (C.c_int * len(ws))(*ns)
        keep.extend(outs + [vx, dst, nn])
        count_q4k((L.lk_dense_q4k_rows_multi, (vx, dst, nn, len(ws), q.data_ptr(), b, k, 0, stream)),
                  sum(synth.weight_bytes(Q4K, n, k) for n in ns))
        return outs[0]

    def add_rows_actmul(gate, up, g, n, k):
        """silu(gate . x) * (up . x) over the Q8_1 rows of group `g`, one launch on the matrix unit; f32
        out into the rows the next quantizer launch reads."""
        q = q81[g]
        assert q.shape[1] * 32 == k
        count_q4k((L.lk_dense_q4k_rows_actmul, (gate.data_ptr(), up.data_ptr(), q.data_ptr(), acts["h"].data_ptr(), b, n, k, 0,
                                                stream)), 2 * synth.weight_bytes(Q4K, n, k))

    def add_rows_q6k(w, g, n, k):
        """Q6_K x the Q8_1 rows of group `g` on the matrix unit."""
        nonlocal total_bytes
        out = torch.empty((b, n), dtype=torch.float32, device=dev)
        keep.append(out)
        q = q81[g]
        assert q.shape[1] * 32 == k
        plan.append((L.lk_dense_q6k_rows, (w.data_ptr(), q.data_ptr(), out.data_ptr(), b, n, k, stream)))
        total_bytes += synth.weight_bytes(Q6K, n, k)

    first_out = None
    first_w = None
    for layer in range(args.layers):
        if kind in ("fused", "auto"):
            made = {name: (maker(n, k), wtype, n, k, g) for name, wtype, n, k, maker, g in shapes}
            keep.extend(v[0] for v in made.values())
            paired = kind == "auto" and b <= 4
            for group in (("q", "k", "v"), ("o",), ("gate", "up"), ("down",)):
                wtype, k, g = made[group[0]][1], made[group[0]][3], made[group[0]][4]
                if paired and group == ("gate", "up"):
                    # act(gate . x) * (up . x) written as the Q8_1 rows `down` reads
                    add_pair(wtype, made["gate"][0], made["up"][0], g, made["gate"][2], k)
                    continue
                if paired and group == ("down",):
                    add_gemv(wtype, made["down"][0], "h", made["down"][2], k)
                    continue
                if kind == "auto" and k > 8192:
                    add_quant(g)
                    for nm in group:
                        add_gemv(wtype, made[nm][0], g, made[nm][2], k)
                    continue
                out = add_fused(wtype, [made[nm][0] for nm in group], g, [made[nm][2] for nm in group], k)
                if first_out is None:
                    first_out, first_w = out, made["q"][0]
            continue
        if kind == "rows":
            # a handful of rows on the matrix unit: q + k + v in one launch, o, gate + up with the
            # activation in one launch, `down` (Q6_K) on the matrix unit too, each over Q8_1 rows a
            # quantizer launch wrote
            made = {name: (maker(n, k), wtype, n, k, g) for name, wtype, n, k, maker, g in shapes}
            keep.extend(v[0] for v in made.values())
            add_quant("x", from_norm=True)
            out = add_rows_multi([made[nm][0] for nm in ("q", "k", "v")], "x", [made[nm][2] for nm in ("q", "k", "v")], HIDDEN)
            if first_out is None:
                first_out, first_w = out, made["q"][0]
            add_quant("attn")
            add_rows(made["o"][0], "attn", HIDDEN, HIDDEN)
            add_quant("x2", from_norm=True)
            if b <= 16:
                # gate + up hands its result on as the Q8_1 rows `down` reads: no f32 round trip, no quantizer launch
                count_q4k((L.lk_dense_q4k_rows_actmul_q8_1, (made["gate"][0].data_ptr(), made["up"][0].data_ptr(), q81["x2"].data_ptr(),
                                                             q81["h"].data_ptr(), b, FFN, HIDDEN, 0, 0, stream)),
                          2 * synth.weight_bytes(Q4K, FFN, HIDDEN))
            else:
                add_rows_actmul(made["gate"][0], made["up"][0], "x2", FFN, HIDDEN)
                add_quant("h")
            add_rows_q6k(made["down"][0], "h", HIDDEN, FFN)
            continue
        last_group = None
        for name, wtype, n, k, maker, g in shapes:
            w = maker(n, k)
            keep.append(w)
            if g != last_group:
                add_quant(g)
                last_group = g
            out = add_gemv(wtype, w, g, n, k)
            if first_out is None:
                first_out, first_w = out, w
    lm_head = make_q80(VOCAB, HIDDEN)
    keep.append(lm_head)
    if kind in ("fused", "auto"):
        add_fused(Q80, [lm_head], "final", [VOCAB], HIDDEN)
    else:
        add_quant("final")
        add_gemv(Q80, lm_head, "final", VOCAB, HIDDEN)
    torch.cuda.synchronize()

    def run(items):
        for fn, a in items:
            rc = fn(*a)
            if rc:
                raise lib.LokenError(fn.__name__, rc)

    run(plan)  # eager once: first-launch set-up happens outside any capture
    torch.cuda.synchronize()
    if args.copy_probe:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev)
        src.fill_(1.0)
        dstc = torch.empty_like(src)
        dstc.copy_(src)   # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dstc

    graph = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        # the launch stream is an argument of every planned call: rebuild the plans on `side`
        def on_stream(items, s):
            return [(fn, a[:-1] + (s,)) for fn, a in items]
        with torch.cuda.stream(side):
            cap_plan = on_stream(plan, side.cuda_stream)
            run(cap_plan)
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                run(cap_plan)
        torch.cuda.synchronize()

    def step():
        if graph is not None:
            graph.replay()
        else:
            run(plan)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    step_gbs = total_bytes / (ms_per_step * 1e-3) / 1e9
    from loken_amd import workloads as wl
    # beside the K-step wall clock: 200 steps after 20 warm-ups, each between its own events
    step_us = wl.time_launches(lambda i: step(), 200, warm=20)

    # ------------------------------------------------------------------ roofline leg
    # The step's own mix of Q4_K mat-vec launches, nothing else, recorded into one graph and
    # replayed between two events on the replaying stream (the stream the kernels run on).
    reps = 200
    run(q4k_plan)
    torch.cuda.synchronize()
    q4k_graph = None
    if not args.no_graph:
        side2 = torch.cuda.Stream()
        q4k_graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side2):
            cap_q4k = [(fn, a[:-1] + (side2.cuda_stream,)) for fn, a in q4k_plan]
            run(cap_q4k)
            side2.synchronize()
            with torch.cuda.graph(q4k_graph, stream=side2):
                run(cap_q4k)
        torch.cuda.synchronize()
        q4k_graph.replay()
        torch.cuda.synchronize()
    # 20 warm-up passes over the mix, then 200 timed ones, each between its own pair of events on the
    # stream the kernels run on; the average launch duration is the mean over all of them
    mix_us = wl.time_launches(lambda i: q4k_graph.replay() if q4k_graph is not None else run(q4k_plan), reps, warm=20) / len(q4k_plan)
    launches = reps * len(q4k_plan)
    avg_us = float(mix_us.mean())
    bytes_per_launch = q4k_bytes / len(q4k_plan)
    achieved = bytes_per_launch / (avg_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": MEASURED_TRAFFIC.get((args.plan, b, args.layers)),
                "kernel": (f"Q4_K mat-vec launches of a layer: q4k_reg_kernel<1,1,true,1> (q+k+v, 512 workgroups), q4k_reg_kernel<2,1,true,1> (o, 256), "
                           f"q4k_reg_pair_kernel<1,true,true,1> (gate+up)") if kind == "auto" and b == 1
                          else (f"Q4_K mat-vec launches of a layer: q4k_reg_kernel<1,1,true,2> (q+k+v), q4k_reg_kernel<2,1,true,2> (o), "
                                f"mmvq_pair_q8_1_kernel<EngQ4K,{b},1,0> (gate+up)") if kind == "auto"
                          else ("Q4_K launches of a layer on the matrix unit, 16-row tiles: q4k_rows16_kernel<false,false,4,2> (q+k+v; o), "
                                "q4k_rows16_kernel<true,false,4,4> (gate+up)") if kind == "rows"
                          else f"mmvq_kernel<EngQ4K,{b},2,float>", "avg_launch_us": round(avg_us, 3),
                "algorithmic_bytes_per_launch": int(bytes_per_launch), "launches_timed": launches,
                "per_launch": wl.spread(mix_us),
                "timed_as": (f"{reps} graph replays of the mix of {len(q4k_plan)} launches, each replay between its own events; "
                             f"per-launch figures are a replay's time over its launches") if q4k_graph is not None else "eager launches"}
    q4k_launch_bytes = sorted({int(a_bytes) for a_bytes in q4k_launch_sizes})
    # The mix kernel by kernel: the launches of one size (q + k + v; o; gate + up) over the layers' own weights
    # as a graph of their own, timed the same way. The gate + up launch is the step's largest share of time.
    if q4k_graph is not None and not args.brief:
        by_kernel = {}
        for nbytes in q4k_launch_bytes:
            items = [it for it, sz in zip(q4k_plan, q4k_launch_sizes) if int(sz) == nbytes]
            side3 = torch.cuda.Stream()
            g3 = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side3):
                cap = [(fn, a[:-1] + (side3.cuda_stream,)) for fn, a in items]
                run(cap)
                side3.synchronize()
                with torch.cuda.graph(g3, stream=side3):
                    run(cap)
            torch.cuda.synchronize()
            us3 = wl.time_launches(lambda i: g3.replay(), 200, warm=20) / len(items)
            gbs3 = nbytes / float(us3.mean()) / 1e3
            by_kernel[str(nbytes)] = dict(wl.spread(us3), launches_per_replay=len(items), avg_launch_us=round(float(us3.mean()), 3),
                                          achieved_gbs=round(gbs3, 1), frac=round(gbs3 / HBM_PEAK_GBS, 4))
            del g3
        roofline["by_launch_size"] = by_kernel

    # ------------------------------------------------------------------ the rest of the metric, and measured denominators
    extras = {}
    used_graph = graph is not None
    if not args.brief:
        from loken_amd import probes, workloads
        used_graph = graph is not None
        graph = q4k_graph = None   # the step's 5 GB of weights make room for the other workloads
        keep.clear()
        torch.cuda.empty_cache()
        ceil, rb = probes.ceilings()
        # what a launch that only READS as many bytes as each Q4_K launch of the mix takes (best of a
        # few grid shapes): the floor a dependent launch of that size has on this card
        floors = {}
        for nbytes in q4k_launch_bytes:
            floors[str(nbytes)] = round(min(rb.rate(nbytes, wgs, pat)[0] for wgs, pat in ((1024, 2), (2048, 4), (2048, 8), (1024, 4))), 3)
        del rb
        torch.cuda.empty_cache()
        mix_floor_us = sum(floors[str(int(sz))] for sz in q4k_launch_sizes) / len(q4k_launch_sizes)
        roofline["peak_measured"] = {"hbm_read_1gib_gbs": ceil["hbm_read_1gib_gbs"], "empty_launch_us": ceil["empty_launch_us"],
                                     "read_only_launch_us_by_bytes": floors,
                                     "read_only_mix_avg_us": round(mix_floor_us, 3),
                                     "read_only_mix_gbs": round(bytes_per_launch / mix_floor_us / 1e3, 1),
                                     "frac_of_read_only_mix": round(mix_floor_us / avg_us, 4)}
        extras["gemv_4096"] = workloads.brief_gemv_4096()
        extras["mmq"] = {"2a": workloads.brief_mmq("2a"), "2b": workloads.brief_mmq("2b"),
                         "peak": 5000.0, "unit": "TOP/s",
                         "peak_measured": {"mfma_i8_32x32x32_tops": ceil["mfma_i8_32x32x32_tops"],
                                           "mfma_f16_32x32x16_tflops": ceil["mfma_f16_32x32x16_tflops"]}}

        # The other configured workloads, each as a child process running this file (their weights
        # do not fit beside one another's): the step at 4 and 8 rows, the MoE block, the Qwen3-1.7B step.
        del ceil
        torch.cuda.empty_cache()
        extras["other_configs"] = other_configs()

    # ------------------------------------------------------------------ CPU baseline leg
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(args, torch, synth, lib, first_w, first_out, acts["x"], b)

    line = {
        "metric": "Q4_K GEMV weight GB/s (% HBM peak); prefill MMQ int8 TOPS (% MFMA peak)",
        "value": round(achieved, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"llama3-8b decode-step quantized linears (Q4_K q,k,v,o,gate,up; Q6_K down; "
                               f"Q8_0 lm_head), batch {b}, {args.layers} layers",
                   "launch_plan": args.plan if kind == args.plan else f"{args.plan} -> {kind}",
                   "acts": "f32 rows into every group" if args.acts == "f32" or kind not in ("rows", "auto", "fused")
                           else "q + k + v and gate + up read Q8_1 rows as the model's RMSNorm launches that also quantize "
                                "leave them (those launches are not timed); o from f32 rows",
                   "weight_bytes_per_step": total_bytes, "launches_per_step": len(plan),
                   "hip_graph": used_graph},
        "value_is": "Q4_K weight bytes of the step over the time of its Q4_K mat-vec launches (the roofline leg); "
                    "ms_per_step and whole_step are the whole step, Q6_K and Q8_0 matrices included",
        "pct_hbm_peak": round(100.0 * achieved / HBM_PEAK_GBS, 2),
        "whole_step": {"gbs": round(step_gbs, 1), "pct_hbm_peak": round(100.0 * step_gbs / HBM_PEAK_GBS, 2),
                       "ms_per_step": round(ms_per_step, 4), "weight_bytes": total_bytes,
                       "per_step": wl.spread(step_us),
                       "gbs_at_median": round(total_bytes / float(__import__("numpy").median(step_us)) / 1e3, 1)},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    line.update(extras)
    print(json.dumps(line))
    return 0


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def host_last_level_cache():
    """(bytes, domains) of the L3 slices the CPUs of this process's affinity set sit under, from sysfs;
    (0, 0) when the host does not say."""
    seen = {}
    try:
        cpus = sorted(os.sched_getaffinity(0))
    except AttributeError:
        cpus = list(range(os.cpu_count() or 1))
    for c in cpus:
        base = f"/sys/devices/system/cpu/cpu{c}/cache/index3/"
        try:
            shared = open(base + "shared_cpu_list").read().strip()
            size = open(base + "size").read().strip()
        except OSError:
            continue
        mult = {"K": 1 << 10, "M": 1 << 20, "G": 1 << 30}.get(size[-1:].upper(), 1)
        seen[shared] = int(size.rstrip("KMGkmg")) * mult
    return sum(seen.values()), len(seen)


def rotating_copies(arr, llc_bytes, cap_bytes=3 << 30):
    """Copies of `arr` that together exceed twice the last-level cache (512 MB assumed when the host
    does not say), at least 2 and at most `cap_bytes` in all."""
    want = 2 * (llc_bytes or (256 << 20)) + arr.nbytes
    count = max(2, min(-(-want // arr.nbytes), max(2, cap_bytes // arr.nbytes)))
    return [arr.copy() for _ in range(count)]


def timed_calls(fn, copies, seconds):
    """Calls `fn(copy)` over the copies in turn for about `seconds`; returns (calls, elapsed, per-call seconds)."""
    import numpy as np
    fn(copies[0])
    per = []
    t0 = time.perf_counter()
    i = 0
    while True:
        a = time.perf_counter()
        fn(copies[i % len(copies)])
        bnow = time.perf_counter()
        per.append(bnow - a)
        i += 1
        if bnow - t0 >= seconds and i >= 3:
            break
    return i, bnow - t0, np.array(per)


def cpu_spread(per_s):
    import numpy as np
    us = per_s * 1e6
    return {"median_us": round(float(np.median(us)), 1), "p10_us": round(float(np.percentile(us, 10)), 1),
            "p90_us": round(float(np.percentile(us, 90)), 1), "min_us": round(float(us.min()), 1),
            "max_us": round(float(us.max()), 1), "calls": int(us.size)}


def cpu_baseline(args, torch, synth, lib, w_dev, out_dev, x_dev, b):
    """loken's served CPU paths, restated (oracle/cpu_baseline.c), on a persistent pool of one worker
    per physical core of this process's CPU set (or OMP_NUM_THREADS when the host sets it: the GPU
    box gives a job a share of its cores):
      * decode: Q8_K activation, weights repacked eight rows at a time, one group dot per eight
        columns, on layer 0's q_proj-shaped sample (the headline leg);
      * prefill (configuration 2a, 512 rows x 4096 -> 14336 Q4_K): the tiled driver over the same
        repacked weights (matmul_q4k_repacked_tiled, src/tensor/quant_cpu/drivers.rs:231-339);
      * the expert block of configuration 3 (128 experts 2048 -> 768 -> 2048 Q4_K, top-8, 256 tokens):
        the scalar oracle's block with the tokens spread over the pool.
    Every leg rotates copies of its weights that together exceed twice the host's last-level cache."""
    import numpy as np

    import oracle

    physical, logical = oracle.cpu_counts()
    asked = int(os.environ.get("OMP_NUM_THREADS", "0"))
    threads = oracle.pool_start(min(asked, physical) if asked > 0 else 0)
    llc, llc_domains = host_last_level_cache()
    budget = max(args.cpu_seconds, 1.0)
    n, k = HIDDEN, HIDDEN
    w = w_dev.cpu().numpy()
    x = x_dev.cpu().numpy()
    # parity of the benchmarked path on this very matrix, against the same-codes oracle
    want = oracle.ob_matmul(oracle.Q4_K, x, w, n)
    got = out_dev.cpu().numpy()
    ok = bool((np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-4).all())
    x8 = oracle.repack_q4k_x8(w, n, k)
    scalar = oracle.oa_matmul(oracle.Q4_K, x, w, n)
    served_ok = bool((np.abs(oracle.oa_matmul_q4k_x8(x, x8, n) - scalar) <= 1e-3 * np.maximum(np.abs(scalar), 1.0)).all())
    copies = rotating_copies(x8, llc)
    calls, dt, per = timed_calls(lambda c: oracle.oa_matmul_q4k_x8(x, c, n), copies, 0.4 * budget)
    nbytes = synth.weight_bytes(lib.TYPE_Q4_K, n, k)
    gbs = calls * nbytes / dt / 1e9
    rotated = len(copies) * x8.nbytes
    del copies
    legs = {}

    # ---- prefill, configuration 2a
    m2, k2, n2 = 512, 4096, 14336
    w2 = synth.weight(lib.TYPE_Q4_K, 256, k2, seed=1).reshape(256, -1)
    w2 = np.ascontiguousarray(np.tile(w2, (n2 // 256, 1)))          # a few generated rows repeated
    x2 = synth.activation(m2, k2, seed=1)
    x82 = oracle.repack_q4k_x8(w2, n2, k2)
    sample = oracle.oa_matmul_q4k_x8_tiled(x2[:8], x82[:(256 // 8) * (k2 // 256) * 1152], 256)
    ref2 = oracle.oa_matmul(oracle.Q4_K, x2[:8], w2[:256], 256)
    tiled_ok = bool((np.abs(sample - ref2) <= 1e-3 * np.maximum(np.abs(ref2), 1.0)).all())
    copies = rotating_copies(x82, llc)
    calls2, dt2, per2 = timed_calls(lambda c: oracle.oa_matmul_q4k_x8_tiled(x2, c, n2), copies, 0.3 * budget)
    ops2 = 2.0 * m2 * k2 * n2
    legs["prefill_2a"] = {"value": round(calls2 * ops2 / dt2 / 1e12, 3), "unit": "TOP/s", "cores": threads, "kind": "port",
                          "per_call": cpu_spread(per2), "rotated_bytes": len(copies) * x82.nbytes,
                          "tiled_path_vs_scalar_oracle": "ok" if tiled_ok else "FAILED",
                          "sample": f"tiled matmul {m2} rows x {k2} -> {n2} Q4_K, {calls2} calls ({dt2:.1f} s): Q8_K rows quantized on "
                                    f"the pool, one chunk per eight columns, rows in tiles of eight (loken's served CPU prefill "
                                    f"path, restated in C with AVX2)"}
    del copies, x82, w2

    # ---- the expert block of configuration 3
    experts, hidden, ffn, topk, tokens = 128, 2048, 768, 8, 256
    rng = np.random.default_rng(3)

    def stack(rows, cols, stream):
        base = synth.weight(lib.TYPE_Q4_K, 256, cols, seed=3, stream=stream).reshape(256, -1)
        return np.ascontiguousarray(np.tile(base, (rows // 256, 1))).reshape(-1)
    gate, up, down = stack(experts * ffn, hidden, 1), stack(experts * ffn, hidden, 2), stack(experts * hidden, ffn, 3)
    xm = synth.activation(tokens, hidden, seed=3)
    ids = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    wts = rng.random((tokens, topk)).astype(np.float32)
    wts /= wts.sum(axis=1, keepdims=True)
    block = np.concatenate([gate, up, down])
    g_end, u_end = gate.size, gate.size + up.size
    copies = rotating_copies(block, llc)
    del gate, up, down

    def run_block(c):
        return oracle.moe_forward_pool(0, oracle.Q4_K, oracle.Q4_K, xm, c[:g_end], c[g_end:u_end], c[u_end:], ids, wts, experts, ffn)
    calls3, dt3, per3 = timed_calls(run_block, copies, 0.3 * budget)
    ops3 = 6.0 * tokens * topk * ffn * hidden
    legs["moe_block_256_tokens"] = {"value": round(calls3 * block.nbytes / dt3 / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
                                    "tops": round(calls3 * ops3 / dt3 / 1e12, 4), "per_call": cpu_spread(per3),
                                    "rotated_bytes": len(copies) * block.nbytes,
                                    "sample": f"expert block, {experts} experts {hidden} -> {ffn} -> {hidden} Q4_K, top-{topk}, {tokens} tokens, "
                                              f"{calls3} calls ({dt3:.1f} s): the scalar block per routed pair (gate and up dots over "
                                              f"Q8_K rows, SiLU, down dot, weighted sum), chunks of tokens on the pool"}
    del copies, block
    oracle.pool_start(1)   # joins the workers: no thread of the pool outlives the measurement
    return {"value": round(gbs, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "cpu_model": cpu_model(), "physical_cores": physical, "logical_cpus": logical,
            "last_level_cache_bytes": llc, "last_level_cache_domains": llc_domains, "rotated_bytes": rotated,
            "threads_source": "OMP_NUM_THREADS" if asked > 0 else "one per physical core",
            "per_call": cpu_spread(per),
            "sample": f"Q4_K mat-vec {n}x{k}, batch {b}, {calls} calls over {rotated // x8.nbytes} rotating copies of the repacked weights "
                      f"({rotated / 1e6:.0f} MB against {llc / 1e6:.0f} MB of last-level cache; {dt:.1f} s): Q8_K activation, eight-row "
                      f"repacked weights, group dot per eight columns (loken's served decode path, restated in C with AVX2), "
                      f"persistent pool of {threads} threads",
            "served_path_vs_scalar_oracle": "ok" if served_ok else "FAILED",
            "gpu_parity_on_sample": "ok" if ok else "FAILED",
            "legs": legs}


if __name__ == "__main__":
    sys.exit(main())
