#!/usr/bin/env python3
"""Benchmark of the pipeline-stage hot path on one MI355X.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload codec]

Workloads
  codec   boundary activation codec alone: hidden state [4096, 4096] f32 -> q8_0 blocks (pack), inputs
          resident in HBM; value = algorithmic GB/s of pack_q8_0 (5.0625 B/element).

The kernel's launch duration is measured with HIP events recorded on the stream the kernels are queued on.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def codec_input(T, h=4096):
    rng = np.random.Generator(np.random.PCG64(1234 + T))
    x = rng.standard_normal((T, h)).astype(np.float32)
    ch = np.random.Generator(np.random.PCG64(1234)).choice(h, size=int(np.ceil(h * 0.001)), replace=False)
    x[:, ch] *= 50
    return x


def time_events(torch, fn, steps, warmup):
    """Average milliseconds per call of fn() over `steps` calls, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall_ms


def cpu_codec_baseline(sample_T):
    """The oracle's quantize_row_q8_0 restatement on the host, one thread, on `sample_T` rows of the workload."""
    import oracle
    x = codec_input(sample_T).reshape(-1)
    oracle.quantize_q8_0(x[:32 * 1024])  # warm
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 10.0:
        oracle.quantize_q8_0(x)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(x.size * 5.0625 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "pack_q8_0 of [%d,4096] f32, %d repeats, scalar C restatement of quantize_row_q8_0_ref" % (sample_T, reps)}


def bench_codec(args):
    import torch
    import __graft_entry__ as graft
    m = graft.load_package()
    m.lib()
    T, h = 4096, 4096
    n = T * h
    x = torch.from_numpy(codec_input(T)).cuda()
    packed = torch.empty(m.act_packed_size(m.Q8_0, T, h), dtype=torch.uint8, device="cuda")
    half = torch.empty(n, dtype=torch.float16, device="cuda")
    back = torch.empty(n, dtype=torch.float32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    ops = {
        "pack_q8_0": (lambda: m.act_pack_dev(m.Q8_0, x.data_ptr(), packed.data_ptr(), n, s), 5.0625),
        "unpack_q8_0": (lambda: m.act_unpack_dev(m.Q8_0, packed.data_ptr(), back.data_ptr(), n, s), 5.0625),
        "pack_f16": (lambda: m.act_pack_dev(m.F16, x.data_ptr(), half.data_ptr(), n, s), 6.0),
        "unpack_f16": (lambda: m.act_unpack_dev(m.F16, half.data_ptr(), back.data_ptr(), n, s), 6.0),
    }
    res = {}
    for name, (fn, bpe) in ops.items():
        ms, wall = time_events(torch, fn, args.steps, args.warmup)
        res[name] = {"ms": round(ms, 5), "GBps": round(n * bpe / ms / 1e6, 1), "frac_hbm": round(n * bpe / ms / 1e6 / HBM_PEAK_GBS, 4)}
    ms = res["pack_q8_0"]["ms"]
    gbs = res["pack_q8_0"]["GBps"]
    out = {
        "metric": "activation pack GB/s (q8_0, [4096,4096] f32)", "value": gbs, "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32->i8+f16", "data": "synthetic",
        "config": {"workload": "codec: pack_q8_0 of hidden state [4096,4096] f32, N(0,1) with 0.1% channels x50"},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
        "codec": res,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_codec_baseline(512)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="codec", choices=["codec"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the stage path; --gpus %d is not supported (one GPU per box)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    out = bench_codec(args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
