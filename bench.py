#!/usr/bin/env python3
"""Benchmark of the quantized-SDPA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 2] [--skip-cpu-baseline]

A step is one pass of the whole path (K mean, INT8 Q/K quantization, V repack,
attention, bf16 output) over one synthetic batch that is already resident in
HBM.  The workload is the Flux/Klein joint text+image attention shape
B=1, H=24, S=4608, D=128 (INT8 QK^T, FP16 PV).  One JSON line is printed:

  value          effective attention TOPS = 4*B*H*S^2*D / step time
  roofline       the attention kernel alone (the dominant kernel), timed with
                 HIP events on the launch stream, against the dense INT8 MFMA peak
  cpu_baseline   the CPU checker's implementation of the same path, timed on
                 this machine's host cores (a reported baseline, not a target)

This path runs on a single GPU; --gpus above 1 is refused.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "effective attention TOPS at H=24,S=4608,D=128; % of INT8/FP8 MFMA peak"
PEAK_INT8_TOPS = 5000.0      # MI355X dense INT8 MFMA, published
PEAK_FP8_TOPS = 5000.0       # MI355X dense FP8 MFMA, published
PEAK_HBM_GBS = 8000.0
K_FLAGS = 3                  # K mean smoothing + per-channel Q/K balancing (the default recipe)

# HBM bytes per launch of the attention kernel, from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE
# (KiB per dispatch, one run each) scaled by the readings of the same counters for a 256 MiB
# device copy (--copy-calibration): fetch 54 520 KiB x 2.000, write 76 390 KiB x 1.000.
# Keyed by (workload id, variant); other workloads have not been measured.
MEASURED_ATTN_TRAFFIC_BYTES = {(2, 0): int(54520 * 1024 * 2.0 + 76390 * 1024 * 1.0)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", type=int, default=2)
    ap.add_argument("--skip-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain device copy of 256 MiB (read 256 MiB, write 256 MiB) five times: "
                         "the known-size kernel the HBM traffic counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this hot path is measured on ONE GPU (heads are independent and would shard "
              "without any exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from mojodiffusion_amd import _lib
    from mojodiffusion_amd.workloads import WORKLOADS, make_inputs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the library has no CPU path", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        src = torch.full((256 << 20,), 7, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_each_way": src.numel(), "launches": 5}))
        return
    L = _lib.lib()
    w = WORKLOADS[args.workload]
    q, k, v = make_inputs(w)
    up = lambda x: torch.from_numpy(x.view(np.int16)).to(dev).view(torch.bfloat16)
    qd, kd, vd = up(q), up(k), up(v)
    o = torch.empty_like(qd)
    B, S, H, D = w.B, w.S, w.H, w.D
    st = _lib.strides_bhnd(S, H, D)
    nws = L.mi355_sage_workspace_bytes(B, H, S, S, D, w.variant)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        rc = L.mi355_sage_sdpa_bf16_ex(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(),
                                       B, H, S, S, D, w.scale, st, st, st, st, 0, 0, 0, 0, 0, stream,
                                       w.variant, w.blkq, w.blkk, K_FLAGS, ws.data_ptr(), nws)
        if rc != 0:
            raise RuntimeError("mi355_sage_sdpa_bf16_ex rc=%d" % rc)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    tops = w.ops / (ms_per_step * 1e-3) / 1e12

    # ---- stage timings with HIP events on the launch stream -------------------------
    nqp, nkp = L.mi355_sage_pad_q(S), L.mi355_sage_pad_kv(S)
    q8 = torch.empty((B, H, nqp, D), dtype=torch.int8, device=dev)
    k8 = torch.empty((B, H, nkp, D), dtype=torch.int8, device=dev)
    qs = torch.empty((B, H, nqp // w.blkq), dtype=torch.float32, device=dev)
    ks = torch.empty((B, H, nkp // w.blkk), dtype=torch.float32, device=dev)
    km, qm, kmu = (torch.empty((B, H, D), dtype=torch.float32, device=dev) for _ in range(3))
    vsc = torch.empty((B, H, D), dtype=torch.float32, device=dev)
    vq = torch.empty((B, H, nkp // 64, D, 64), dtype=torch.int16 if w.variant == 0 else torch.uint8, device=dev)
    scr = torch.empty(max(L.mi355_sage_quant_scratch_bytes(B, H, S, D), 8), dtype=torch.uint8, device=dev)

    def stage_quant_qk():
        return L.mi355_sage_quant_qk_bf16(qd.data_ptr(), kd.data_ptr(), B, H, S, S, D, w.scale, st, st, 0, 0,
                                          w.blkq, w.blkk, K_FLAGS, 0, 0, q8.data_ptr(), qs.data_ptr(), k8.data_ptr(),
                                          ks.data_ptr(), km.data_ptr(), qm.data_ptr(), kmu.data_ptr(),
                                          scr.data_ptr(), scr.numel(), stream)

    def stage_quant_v():
        if w.variant == 0:
            return L.mi355_sage_quant_v_f16(vd.data_ptr(), B, H, S, D, st, 0, 0, 0, vq.data_ptr(), stream)
        return L.mi355_sage_quant_v_fp8(vd.data_ptr(), B, H, S, D, st, 0, 0, 0, vq.data_ptr(), vsc.data_ptr(),
                                        scr.data_ptr(), scr.numel(), stream)

    def stage_attn():
        return L.mi355_sage_attn_fwd(q8.data_ptr(), qs.data_ptr(), w.blkq, k8.data_ptr(), ks.data_ptr(), w.blkk,
                                     vq.data_ptr(), vsc.data_ptr(), w.variant, B, H, S, S, S, 0, 0, D,
                                     o.data_ptr(), st, 0, None, None, stream)

    def time_stage(fn, n):
        assert fn() == 0
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for a, b in evs:
            a.record()
            assert fn() == 0
            b.record()
        torch.cuda.synchronize()
        ts = sorted(a.elapsed_time(b) for a, b in evs)
        return sum(ts) / len(ts), ts[len(ts) // 2], ts[0]

    n_ev = max(args.steps, 20)
    qk_avg, qk_med, _ = time_stage(stage_quant_qk, n_ev)
    v_avg, v_med, _ = time_stage(stage_quant_v, n_ev)
    at_avg, at_med, at_min = time_stage(stage_attn, n_ev)
    attn_tops = w.ops / (at_avg * 1e-3) / 1e12
    peak = PEAK_INT8_TOPS if w.variant == 0 else PEAK_FP8_TOPS
    # algorithmic HBM bytes of the quantize stage: Q,K,V read once as bf16; int8 Q/K and fp16/e4m3 V written
    elems = B * H * S * D
    quant_bytes = 3 * elems * 2 + 2 * elems + elems * (2 if w.variant == 0 else 1)
    quant_gbs = quant_bytes / ((qk_avg + v_avg) * 1e-3) / 1e9

    out = {
        "metric": METRIC,
        "value": round(tops, 2),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8/f16" if w.variant == 0 else "int8/f8e4m3",
        "data": "synthetic",
        "config": {
            "workload": w.name,
            "B": B, "H": H, "S": S, "D": D,
            "recipe": "K mean-smoothed, Q/K channel-balanced; Q int8 per %d tokens; K int8 per %d tokens; PV %s" % (
                w.blkq, w.blkk, "fp16" if w.variant == 0 else "fp8-e4m3 with per-channel V scales"),
            "ops_per_step": w.ops,
            "pct_of_peak": round(100.0 * tops / peak, 2),
            "peak_tops_used": peak,
            # the stage entry points, each timed on its own (the one-shot call fuses the quantizers
            # into two launches, so its quantize share is about ms_per_step - attn)
            "stage_ms": {"quant_qk": round(qk_avg, 5), "quant_v": round(v_avg, 5), "attn": round(at_avg, 5)},
            "one_shot_quant_ms": round(ms_per_step - at_avg, 5),
            "quant_stage_hbm": {"algorithmic_bytes": quant_bytes, "GB/s": round(quant_gbs, 1),
                                "frac_of_8TB/s": round(quant_gbs / PEAK_HBM_GBS, 4)},
            "device": torch.cuda.get_device_name(0),
        },
        "roofline": {
            "kernel": "sage_attn_kernel<%d,%d>" % (D, w.variant),
            "bound": "mfma",
            "achieved": round(attn_tops, 2),
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": round(attn_tops / peak, 4),
            "traffic": MEASURED_ATTN_TRAFFIC_BYTES.get((args.workload, w.variant)),
            # int8 Q and K read once, V^T tiles (fp16 or e4m3) read once, bf16 O written once
            "algorithmic_bytes_per_launch": 2 * elems + elems * (2 if w.variant == 0 else 1) + 2 * elems,
            "avg_ms": round(at_avg, 5), "median_ms": round(at_med, 5), "min_ms": round(at_min, 5),
            "algorithmic_ops_per_launch": w.ops,
        },
    }

    if not args.skip_cpu_baseline:
        from oracle import sage_oracle
        # bounded sample: a subset of heads at the full sequence length
        # bounded sample: whole passes over a subset of heads at the full sequence length, repeated
        # until about ten seconds of CPU work have been timed
        heads = min(H, 8)
        qh, kh, vh = (np.ascontiguousarray(x[:, :, :heads]) for x in (q, k, v))
        sage_oracle.sdpa_bf16(qh[:, :256], kh[:, :256], vh[:, :256], w.scale, w.variant, w.blkq, w.blkk)   # warm
        passes, c0 = 0, time.perf_counter()
        while True:
            sage_oracle.sdpa_bf16(qh, kh, vh, w.scale, variant=w.variant, blkq=w.blkq, blkk=w.blkk)
            passes += 1
            c1 = time.perf_counter()
            if c1 - c0 >= 10.0 or passes >= 64:
                break
        sample_ops = 4 * B * heads * S * S * D * passes
        out["cpu_baseline"] = {
            "value": round(sample_ops / (c1 - c0) / 1e12, 5),
            "unit": "TOPS",
            "cores": sage_oracle.num_threads(),
            "kind": "port",
            "sample": "%d of %d heads of the same workload at full S=%d, %d passes, %.2f s (C + OpenMP restatement; "
                      "the reference's own path is Mojo/cuDNN and cannot run here)" % (heads, H, S, passes, c1 - c0),
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
