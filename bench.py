#!/usr/bin/env python3
"""Benchmark of the pipeline-stage hot path on one MI355X.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload stage|codec] [--batches 1,4,16]

Workloads
  stage   (default) Llama-3-8B-shaped stage, layers 0-15 of 32 (hidden 4096, 32/8 heads, head_dim 128, FFN 14336,
          RoPE theta 5e5), random Q4_K_M weights generated in the block domain, 4096-token f16 KV context, input
          hidden state resident in HBM, output the q8_0 boundary activation.  A step = one decode call of the
          whole stage at batch 1; value = tokens/s.  Batch 4 and 16 and the boundary codec are reported beside it.
  codec   boundary activation codec alone on [4096, 4096] f32; value = algorithmic GB/s of pack_q8_0.
  c4      Qwen2.5-32B-shaped stage, layers 0-31 of 64 (hidden 5120, 40/8 heads, FFN 27648, q/k/v biases), 8192-token
          KV context in the cache tier the reference picks for a 20 GB model (K q8_0 / V q4_0; --kv f16 for the f16
          tier), decode batch 1/8/32 and a 4096-token prefill.  value = batch-1 tokens/s.
  c5      Qwen3-30B-A3B-shaped expert shard: all 48 layers, 64 of the 128 experts per layer (top-8 routing, expert FFN
          768, per-head q/k norms), decode batch 16 at a 4096-token context.  value = tokens/s at batch 16.

Timing uses HIP events recorded on the stream the kernels run on (the session's own stream for the stage).
The cpu_baseline leg times the CPU oracle (a restatement of ggml's reference routines, NOT llama.cpp) on the
host cores, on a bounded sample.
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

# algorithmic bytes per element of the codec (f32 in + packed out)
Q8_BPE, F16_BPE = 4 + 34 / 32, 6.0


def codec_input(T, h=4096):
    rng = np.random.Generator(np.random.PCG64(1234 + T))
    x = rng.standard_normal((T, h)).astype(np.float32)
    ch = np.random.Generator(np.random.PCG64(1234)).choice(h, size=int(np.ceil(h * 0.001)), replace=False)
    x[:, ch] *= 50
    return x


def kernel_sources_digest(files):
    """sha256 over the named files of mesh-llm_amd/csrc (the sources of one kernel family), first 16 hex digits."""
    import hashlib
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(ROOT, "mesh-llm_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


GEMV_SOURCES = ("gemv.hip", "gemv_body.inc", "gemv_device.hpp", "gemv.hpp")
CODEC_SOURCES = ("codec.hip",)


def profiled_ratio(fname, key, sources):
    """(ratio, note): the number on the line `<key> = <number>` of profiles/<fname> (HBM traffic measured with rocprofv3
    counters, as a multiple of the algorithmic bytes).  The profile names the digest of the kernel sources it was taken
    with (`sources_sha256 = ...`); when the sources have changed since, the ratio describes another kernel and is not
    used: (None, "stale ...").  (None, "absent") when the file or the line is not there."""
    ratio = digest = None
    try:
        with open(os.path.join(ROOT, "profiles", fname)) as f:
            for line in f:
                if line.startswith(key + " ="):
                    ratio = float(line.split("=", 1)[1].split()[0])
                if line.startswith("sources_sha256 ="):
                    digest = line.split("=", 1)[1].split()[0]
    except (OSError, ValueError):
        return None, "absent"
    if ratio is None:
        return None, "absent"
    now = kernel_sources_digest(sources)
    if digest != now:
        return None, "stale: profiles/%s was taken with kernel sources %s, the tree holds %s" % (fname, digest, now)
    return ratio, "profiles/" + fname


def time_on_stream(torch, stream, fn, steps, warmup):
    """Average ms per call of fn(i) over `steps` calls: events recorded on `stream`, host clock beside it."""
    for i in range(warmup):
        fn(i)
    stream.synchronize()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record(stream)
    for i in range(steps):
        fn(i)
    stop.record(stream)
    stream.synchronize()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return start.elapsed_time(stop) / steps, wall_ms


def hbm_probe(m):
    """Streaming-read bandwidth of this GPU: 512 MiB, 3 warm-up + 20 timed passes, the protocol of the reference's
    mesh-llm/benchmarks/membench-fingerprint.hip; quoted beside the nominal 8 TB/s."""
    g = m.hbm_read_probe(512 << 20, 3, 20)
    return {"p50": round(g[len(g) // 2], 1), "p90": round(g[int(len(g) * 0.9)], 1), "bytes": 512 << 20, "runs": len(g)}


# ------------------------------------------------------------------------------------------------ codec
def run_codec(torch, m, steps, warmup, T=4096, h=4096):
    """Each op cycles through enough distinct buffers (> 256 MiB in total) that no pass is served by the
    memory-side cache."""
    n = T * h
    nbuf = 6
    base = torch.from_numpy(codec_input(T, h)).cuda()
    xs = [base.clone() if i else base for i in range(nbuf)]
    packed = [torch.empty(m.act_packed_size(m.Q8_0, T, h), dtype=torch.uint8, device="cuda") for _ in range(nbuf)]
    halves = [torch.empty(n, dtype=torch.float16, device="cuda") for _ in range(nbuf)]
    backs = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(nbuf)]
    stream = torch.cuda.current_stream()
    s = stream.cuda_stream
    for i in range(nbuf):   # valid packed inputs for the unpack runs
        m.act_pack_dev(m.Q8_0, xs[i].data_ptr(), packed[i].data_ptr(), n, s)
        m.act_pack_dev(m.F16, xs[i].data_ptr(), halves[i].data_ptr(), n, s)
    ops = {
        "pack_q8_0": (lambda i: m.act_pack_dev(m.Q8_0, xs[i % nbuf].data_ptr(), packed[i % nbuf].data_ptr(), n, s), Q8_BPE),
        "unpack_q8_0": (lambda i: m.act_unpack_dev(m.Q8_0, packed[i % nbuf].data_ptr(), backs[i % nbuf].data_ptr(), n, s), Q8_BPE),
        "pack_f16": (lambda i: m.act_pack_dev(m.F16, xs[i % nbuf].data_ptr(), halves[i % nbuf].data_ptr(), n, s), F16_BPE),
        "unpack_f16": (lambda i: m.act_unpack_dev(m.F16, halves[i % nbuf].data_ptr(), backs[i % nbuf].data_ptr(), n, s), F16_BPE),
    }
    res = {}
    for name, (fn, bpe) in ops.items():
        ms, _ = time_on_stream(torch, stream, fn, steps, warmup)
        gbs = n * bpe / ms / 1e6
        res[name] = {"ms": round(ms, 5), "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4)}
    # yardstick: a plain streaming kernel of the same traffic shape over the same buffers, timed the same way (f32 side
    # n * 4 bytes; the other side a quarter of that for q8_0, whose packed side is really 0.266 of it, half for f16)
    big = n * 4
    plain = {
        "pack_q8_0": lambda i: m.hbm_mix_probe_dev(xs[i % nbuf].data_ptr(), packed[i % nbuf].data_ptr(), big, 4, True, s),
        "unpack_q8_0": lambda i: m.hbm_mix_probe_dev(packed[i % nbuf].data_ptr(), backs[i % nbuf].data_ptr(), big, 4, False, s),
        "pack_f16": lambda i: m.hbm_mix_probe_dev(xs[i % nbuf].data_ptr(), halves[i % nbuf].data_ptr(), big, 2, True, s),
        "unpack_f16": lambda i: m.hbm_mix_probe_dev(halves[i % nbuf].data_ptr(), backs[i % nbuf].data_ptr(), big, 2, False, s),
    }
    for name, fn in plain.items():
        ms, _ = time_on_stream(torch, stream, fn, steps, warmup)
        ratio = 4 if "q8_0" in name else 2
        gbs = (big + big // ratio) / ms / 1e6
        res[name]["plain_stream_ms"] = round(ms, 5)
        res[name]["plain_stream_GBps"] = round(gbs, 1)
        res[name]["frac_of_plain_stream"] = round(res[name]["GBps"] / gbs, 4)
    return res


def cpu_codec_baseline(sample_T):
    import oracle
    x = codec_input(sample_T).reshape(-1)
    oracle.quantize_q8_0(x[:32 * 1024])
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 8.0:
        oracle.quantize_q8_0(x)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(x.size * Q8_BPE / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "pack_q8_0 of [%d,4096] f32, %d repeats, scalar C restatement of quantize_row_q8_0_ref" % (sample_T, reps)}


def bench_codec(args):
    import torch
    import __graft_entry__ as graft
    m = graft.load_package()
    m.lib()
    res = run_codec(torch, m, args.steps, args.warmup)
    gbs, ms = res["pack_q8_0"]["GBps"], res["pack_q8_0"]["ms"]
    codec_ratio, codec_src = profiled_ratio(CODEC_TRAFFIC_PROFILE, "pack_q8_0_traffic_over_algorithmic", CODEC_SOURCES)
    out = {
        "metric": "activation pack GB/s (q8_0, [4096,4096] f32)", "value": gbs, "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32->i8+f16", "data": "synthetic",
        "config": {"workload": "codec: pack_q8_0 of hidden state [4096,4096] f32, N(0,1) with 0.1% channels x50"},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": int(round(codec_ratio * 4096 * 4096 * Q8_BPE)) if codec_ratio else None,
                     "traffic_source": codec_src,
                     "plain_stream_GBps": res["pack_q8_0"]["plain_stream_GBps"], "frac_of_plain_stream": res["pack_q8_0"]["frac_of_plain_stream"],
                     "measured_stream_read_GBps": hbm_probe(m)},
        "codec": res,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_codec_baseline(512)
    return out


# ------------------------------------------------------------------------------------------------ stage
N_CTX = 4096
STAGE_LAYERS = 16
# bytes of one head_dim-128 cache row: f16, q8_0 (32 x 34-byte blocks' worth: 128 quants + 4 scales), q4_0 (64 + 8)
HD_BYTES_F16, HD_BYTES_Q8_0, HD_BYTES_Q4_0 = 256, 136, 72
PREFILL_T = 2048
TRAFFIC_PROFILE = "stage_decode_llama3_8b_l0_15_hbm_traffic.txt"
CODEC_TRAFFIC_PROFILE = "codec_4096x4096_hbm_traffic.txt"
BURN_IN_SECONDS = 2.0


def build_stage_model(models, path):
    cfg = models.CONFIGS["llama3-8b"]
    t0 = time.perf_counter()
    tensors = models.write_model(path, cfg, range(STAGE_LAYERS), seed=42, fast=True)
    return cfg, tensors, time.perf_counter() - t0


def cpu_stage_baseline(cfg, tensors, n_layers=2):
    """One decode token through the first `n_layers` layers of the same stage on the host cores (all of them,
    OpenMP), at KV depth 4095; scaled to the 16-layer stage."""
    import oracle
    from oracle.stage import StageOracle
    orc = StageOracle(cfg, tensors, 0, n_layers, N_CTX)
    rng = np.random.Generator(np.random.PCG64(5))
    kv = (rng.standard_normal((cfg["n_head_kv"], N_CTX - 1, cfg["head_dim"])) * 0.1).astype(np.float16).view(np.uint16)
    for li in range(n_layers):
        orc.k[li, 0, :, :N_CTX - 1] = kv
        orc.v[li, 0, :, :N_CTX - 1] = kv
    x = rng.standard_normal((1, cfg["n_embd"])).astype(np.float32)
    orc.forward(x, [N_CTX - 1])
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 10.0:
        orc.forward(x, [N_CTX - 1])
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(1.0 / (dt * STAGE_LAYERS / n_layers), 3), "unit": "tok/s", "cores": oracle.get_threads(), "kind": "port",
            "sample": "batch-1 decode of layers 0-%d of the same stage at KV depth 4095, %d repeats, time scaled x%d to 16 layers; "
                      "CPU restatement of ggml's reference routines (f32 activations), not llama.cpp" % (n_layers - 1, reps, STAGE_LAYERS // n_layers)}


def vendor_f16_matvec(torch, cfg):
    """The vendor library's mat-vec (torch.matmul of an f16 matrix and a vector) on the four projection shapes of a
    layer, launched back to back with no dependence between launches: what a plain f16 kernel of that size costs on
    this GPU, next to the average launch of the dequant-fused mat-vec in `roofline`."""
    E, FF = cfg["n_embd"], cfg["n_ff"]
    QKV = (cfg["n_head"] + 2 * cfg["n_head_kv"]) * cfg["head_dim"]
    out = {}
    for name, (M, K) in (("qkv", (QKV, E)), ("o", (E, cfg["n_head"] * cfg["head_dim"])), ("gate_up", (2 * FF, E)), ("down", (E, FF))):
        w = torch.randn(M, K, device="cuda", dtype=torch.float16)
        x = torch.randn(K, 1, device="cuda", dtype=torch.float16)
        for _ in range(5):
            y = w @ x
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(50):
            y = w @ x
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / 50 * 1e3
        out[name] = {"rows": M, "k": K, "MB": round(M * K * 2 / 1e6, 1), "us": round(us, 2), "GBps": round(M * K * 2 / us / 1e3, 1)}
        del w, x, y
    return out


def bench_stage(args):
    import torch
    import __graft_entry__ as graft
    import models
    m = graft.load_package()
    m.lib()
    tmp = models.tmp_dir()
    path = os.path.join(tmp, "mesh_bench_llama3_8b_l0_15.gguf")
    cfg, tensors, t_gen = build_stage_model(models, path)
    batches = sorted(set(int(b) for b in (args.batches or "1,4,16").split(",")))
    bmax = max(batches)
    t0 = time.perf_counter()
    kv_types = {"f16": (m.F16, m.F16), "q8_0/q4_0": (m.Q8_0, m.Q4_0), "q4_0/q4_0": (m.Q4_0, m.Q4_0)}[args.kv]
    kv_row = {m.F16: HD_BYTES_F16, m.Q8_0: HD_BYTES_Q8_0, m.Q4_0: HD_BYTES_Q4_0}
    st = m.Stage(path, 0, STAGE_LAYERS, n_ctx=N_CTX, n_seq_max=bmax, n_batch_max=max(bmax, 16, PREFILL_T if args.prefill else 0),
                 kv_types=kv_types)
    t_load = time.perf_counter() - t0
    os.unlink(path)
    weight_bytes = st.weight_bytes
    ses = st.session()
    E, HK, HD = cfg["n_embd"], cfg["n_head_kv"], cfg["head_dim"]
    # KV context: 4095 cached positions per sequence, f16 N(0,1)*0.1
    rng = np.random.Generator(np.random.PCG64(99))
    kv = (rng.standard_normal((N_CTX - 1, HK, HD)) * 0.1).astype(np.float16).view(np.uint16)
    for il in range(STAGE_LAYERS):
        for s in range(bmax):
            ses.kv_write(il, s, 0, kv, kv)
    kv_bytes_per_seq = STAGE_LAYERS * N_CTX * HK * (kv_row[kv_types[0]] + kv_row[kv_types[1]])
    stream = torch.cuda.ExternalStream(ses.stream)
    # Burn-in, outside every timed region: the first second or so of a process's decode work contains a one-time
    # stall of ~35 ms (whatever kernel is running; its position follows elapsed time rather than the launch count),
    # which would otherwise land in whichever batch size happens to be measured at that moment.  Every batch size
    # runs --burn-in steps, and the whole burn-in lasts at least BURN_IN_SECONDS.
    burn = [(B, torch.from_numpy(rng.standard_normal((B, E)).astype(np.float32)).cuda(),
             torch.empty(m.act_packed_size(m.Q8_0, B, E), dtype=torch.uint8, device="cuda")) for B in batches]
    t_burn = time.perf_counter()
    rounds = 0
    while rounds < 1 or (args.burn_in > 0 and time.perf_counter() - t_burn < BURN_IN_SECONDS):
        for B, xb, ob in burn:
            for _ in range(args.burn_in):
                ses.decode_dev(xb.data_ptr(), np.full(B, N_CTX - 1, np.int32), ob.data_ptr(), ob.numel(), seq=np.arange(B, dtype=np.int32),
                               in_fmt=m.F32, out_fmt=m.Q8_0)
        stream.synchronize()
        rounds += 1
    del burn
    results = {}
    for B in batches:
        x = torch.from_numpy(rng.standard_normal((B, E)).astype(np.float32)).cuda()
        out = torch.empty(m.act_packed_size(m.Q8_0, B, E), dtype=torch.uint8, device="cuda")
        torch.cuda.synchronize()
        pos = np.full(B, N_CTX - 1, np.int32)
        seq = np.arange(B, dtype=np.int32)

        def step(i):
            ses.decode_dev(x.data_ptr(), pos, out.data_ptr(), out.numel(), seq=seq, in_fmt=m.F32, out_fmt=m.Q8_0)

        ms, wall = time_on_stream(torch, stream, step, args.steps, args.warmup)
        # per-kernel-class durations over a few extra steps: every launch carries its own start / stop stamps
        ses.profile(True)
        for i in range(5):
            step(i)
        prof = ses.profile_read()
        ses.profile(False)
        step_bytes = weight_bytes + kv_bytes_per_seq * B
        results[B] = {"ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall, 4), "tok_s": round(B * 1e3 / ms, 1),
                      "algorithmic_GB_per_step": round(step_bytes / 1e9, 4),
                      "GBps": round(step_bytes / ms / 1e6, 1), "frac_hbm": round(step_bytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                      "kernel_ms_per_step": {k: round(v["ms"] / 5, 4) for k, v in prof.items()},
                      "kernel_launches_per_step": {k: v["launches"] // 5 for k, v in prof.items()}}
    prefill = None
    if args.prefill:
        # prompt ingestion: 2048 tokens of sequence 0 in one call (MFMA GEMM path); done last, it overwrites the KV context
        xp = torch.from_numpy(rng.standard_normal((PREFILL_T, E)).astype(np.float32)).cuda()
        outp = torch.empty(m.act_packed_size(m.Q8_0, PREFILL_T, E), dtype=torch.uint8, device="cuda")
        ppos = np.arange(PREFILL_T, dtype=np.int32)

        def pstep(i):
            ses.decode_dev(xp.data_ptr(), ppos, outp.data_ptr(), outp.numel(), in_fmt=m.F32, out_fmt=m.Q8_0)

        pms, _ = time_on_stream(torch, stream, pstep, 3, 1)
        ses.profile(True)
        pstep(0)
        pprof = ses.profile_read()
        ses.profile(False)
        H, HD, FF = cfg["n_head"], cfg["head_dim"], cfg["n_ff"]
        mm_flop = 2.0 * PREFILL_T * STAGE_LAYERS * (E * H * HD * 2 + E * HK * HD * 2 + 3 * E * FF)
        at_flop = 4.0 * STAGE_LAYERS * H * HD * PREFILL_T * (PREFILL_T + 1) / 2
        gemm_ms = pprof["gemv"]["ms"]
        # what the matrix pipes sustain from registers alone on this GPU (20 launches of ~15 ms each, median)
        mp = m.mfma_f16_probe(20000, 2, 20)
        mfma_probe = mp[len(mp) // 2]
        # and what the vendor library's plain f16 GEMM reaches on the largest projection's shape (gate + up: tokens x
        # 2 n_ff x n_embd) with weights that are already f16: no dequantisation, no epilogue, 2 bytes per weight
        va = torch.randn(PREFILL_T, E, device="cuda", dtype=torch.float16)
        vb = torch.randn(2 * FF, E, device="cuda", dtype=torch.float16)
        for _ in range(3):
            vc = va @ vb.t()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        ev0.record()
        for _ in range(10):
            vc = va @ vb.t()
        ev1.record()
        torch.cuda.synchronize()
        vendor_tflops = 2.0 * PREFILL_T * 2 * FF * E * 10 / ev0.elapsed_time(ev1) / 1e9
        del va, vb, vc
        prefill = {"tokens": PREFILL_T, "ms": round(pms, 2), "tok_s": round(PREFILL_T * 1e3 / pms, 1),
                   "matmul_TFLOP": round(mm_flop / 1e12, 3), "attention_TFLOP": round(at_flop / 1e12, 3),
                   "stage_TFLOPs": round((mm_flop + at_flop) / pms / 1e9, 1),
                   "gemm_ms": round(gemm_ms, 2), "gemm_TFLOPs": round(mm_flop / gemm_ms / 1e9, 1),
                   "gemm_frac_mfma_f16_peak": round(mm_flop / gemm_ms / 1e9 / 2500.0, 4),
                   "vendor_plain_f16_gemm_TFLOPs_gate_up_shape": round(vendor_tflops, 1),
                   "mfma_f16_probe_TFLOPs": round(mfma_probe, 1), "gemm_frac_of_mfma_probe": round(mm_flop / gemm_ms / 1e9 / mfma_probe, 4),
                   "kernel_ms": {k: round(v["ms"], 2) for k, v in pprof.items()}}
    b1 = results[batches[0]]
    # roofline of the dominant kernel (the dequant-fused GEMV): all of a step's weight bytes pass through its
    # launches, so the average launch moves weight_bytes / launches in kernel_ms / launches
    g_ms = b1["kernel_ms_per_step"]["gemv"]
    g_n = b1["kernel_launches_per_step"]["gemv"]
    gemv_gbs = weight_bytes / g_ms / 1e6
    traffic_ratio, traffic_src = profiled_ratio(TRAFFIC_PROFILE, "gemv_batch1_traffic_over_algorithmic", GEMV_SOURCES)
    codec = run_codec(torch, m, max(10, args.steps // 2), args.warmup)
    probe = hbm_probe(m)
    vendor_matvec = vendor_f16_matvec(torch, cfg)
    out = {
        "metric": "stage decode tok/s @8B Q4_K_M", "value": b1["tok_s"], "unit": "tok/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": b1["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 activations x q4_K/q6_K weights, %s KV" % args.kv, "data": "synthetic",
        "config": {"workload": "Llama-3-8B-shaped stage, layers 0-15 of 32, Q4_K_M block-domain random weights, decode batch %d, "
                               "4096-token %s KV context, f32 hidden state in HBM -> q8_0 boundary activation out" % (batches[0], args.kv),
                   "weight_bytes": weight_bytes, "kv_bytes_per_seq": kv_bytes_per_seq},
        "roofline": {"bound": "hbm", "kernel": "gemv_dot_kernel<type,1,NU> (q4_K/q6_K dequant-fused mat-vec, all instantiations)",
                     "achieved": round(gemv_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gemv_gbs / HBM_PEAK_GBS, 4),
                     # HBM bytes per average launch: the ratio of counted (rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated
                     # on a copy of known size) to algorithmic bytes recorded in the committed profile summary
                     "traffic": int(round(traffic_ratio * weight_bytes / g_n)) if traffic_ratio else None,
                     "traffic_source": traffic_src, "launches_per_step": g_n, "avg_launch_us": round(g_ms / g_n * 1e3, 2),
                     "algorithmic_bytes_per_launch": weight_bytes // g_n,
                     "measured_stream_read_GBps": probe, "frac_of_measured_p90": round(gemv_gbs / probe["p90"], 4),
                     "vendor_f16_matvec_same_shapes": vendor_matvec},
        "stage_frac_hbm": b1["frac_hbm"],
        "decode": {str(k): v for k, v in results.items()},
        "prefill": prefill,
        "codec": codec,
        "setup_s": {"generate_gguf": round(t_gen, 1), "open_stage": round(t_load, 1)},
    }
    ses.close()
    st.close()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_stage_baseline(cfg, tensors)
    return out


# ------------------------------------------------------------------------------------------------ other shapes
SHAPES = {
    # (the reference's table quotes this shape on an f16 cache and its launcher picks q8_0 / q4_0 for a 32B model: both are measured)
    "c4": dict(model="qwen2.5-32b", layers=32, n_ctx=8192, batches=[1, 8, 32], prefill=4096, n_expert_local=None, kv="q8_0/q4_0", also_kv="f16",
               metric="stage decode tok/s @32B Q4_K_M, layers 0-31 of 64"),
    "c5": dict(model="qwen3-30b-a3b", layers=48, n_ctx=4096, batches=[16], prefill=1024, n_expert_local=64, kv="q8_0/q4_0", router="zipf",
               metric="expert-shard decode tok/s @Qwen3-30B-A3B Q4_K_M, 64 of 128 experts, batch 16"),
}


def bench_shape(args):
    """The larger configurations (32B dense stage, 64-expert shard) at full size on one GPU: same timing as the default workload, fewer extras."""
    import torch
    import __graft_entry__ as graft
    import models
    m = graft.load_package()
    m.lib()
    sp = SHAPES[args.workload]
    cfg = models.CONFIGS[sp["model"]]
    kv_name = args.kv if args.kv_given else sp["kv"]
    kv_types = {"f16": (m.F16, m.F16), "q8_0/q4_0": (m.Q8_0, m.Q4_0), "q4_0/q4_0": (m.Q4_0, m.Q4_0)}[kv_name]
    kv_row = {m.F16: HD_BYTES_F16, m.Q8_0: HD_BYTES_Q8_0, m.Q4_0: HD_BYTES_Q4_0}
    path = os.path.join(models.tmp_dir(), "mesh_bench_%s.gguf" % args.workload)
    t0 = time.perf_counter()
    zipf = sp.get("router") == "zipf"
    tensors = models.write_model(path, cfg, range(sp["layers"]), seed=42, fast=True, n_expert_local=sp["n_expert_local"],
                                 router=sp.get("router"))
    t_gen = time.perf_counter() - t0
    expert_bytes = sum(d.nbytes for n, (_, _, d) in tensors.items() if "_exps." in n)
    del tensors
    print("[bench] model file written in %.1f s" % t_gen, file=sys.stderr, flush=True)
    batches = sorted(set(int(b) for b in args.batches.split(","))) if args.batches else sp["batches"]
    bmax = max(batches)
    n_ctx, L = sp["n_ctx"], sp["layers"]
    t0 = time.perf_counter()
    st = m.Stage(path, 0, L, n_ctx=n_ctx, n_seq_max=bmax, n_batch_max=max(bmax, 16, sp["prefill"]), kv_types=kv_types)
    t_load = time.perf_counter() - t0
    os.unlink(path)
    ses = st.session()
    E, HK, HD = cfg["n_embd"], cfg["n_head_kv"], cfg["head_dim"]
    rng = np.random.Generator(np.random.PCG64(99))
    kv = (rng.standard_normal((n_ctx - 1, HK, HD)) * 0.1).astype(np.float16).view(np.uint16)
    t0 = time.perf_counter()
    for il in range(L):
        for s in range(bmax):
            ses.kv_write(il, s, 0, kv, kv)
    t_kv = time.perf_counter() - t0
    print("[bench] stage open %.1f s, KV context filled in %.1f s" % (t_load, t_kv), file=sys.stderr, flush=True)
    kv_bytes_per_seq = L * n_ctx * HK * (kv_row[kv_types[0]] + kv_row[kv_types[1]])
    stream = torch.cuda.ExternalStream(ses.stream)
    if args.burn_in > 0:
        # untimed decode work for BURN_IN_SECONDS: the one-time ~35 ms stall early in a process's life (see bench_stage)
        B0 = batches[0]
        xb = torch.from_numpy(rng.standard_normal((B0, E)).astype(np.float32)).cuda()
        ob = torch.empty(m.act_packed_size(m.Q8_0, B0, E), dtype=torch.uint8, device="cuda")
        t_burn = time.perf_counter()
        while time.perf_counter() - t_burn < BURN_IN_SECONDS:
            for _ in range(20):
                ses.decode_dev(xb.data_ptr(), np.full(B0, n_ctx - 1, np.int32), ob.data_ptr(), ob.numel(), seq=np.arange(B0, dtype=np.int32),
                               in_fmt=m.F32, out_fmt=m.Q8_0)
            stream.synchronize()
    results = {}
    for B in batches:
        print("[bench] decode batch %d" % B, file=sys.stderr, flush=True)
        # router="zipf": the expert bias rides on a constant channel of the hidden state (tests/models.py)
        x = torch.from_numpy(models.zipf_hidden_state(rng, B, E) if zipf else rng.standard_normal((B, E)).astype(np.float32)).cuda()
        out = torch.empty(m.act_packed_size(m.Q8_0, B, E), dtype=torch.uint8, device="cuda")
        pos = np.full(B, n_ctx - 1, np.int32)
        seq = np.arange(B, dtype=np.int32)

        def step(i):
            ses.decode_dev(x.data_ptr(), pos, out.data_ptr(), out.numel(), seq=seq, in_fmt=m.F32, out_fmt=m.Q8_0)

        ms, wall = time_on_stream(torch, stream, step, args.steps, args.warmup)
        ses.profile(True)
        for i in range(3):
            step(i)
        prof = ses.profile_read()
        ses.profile(False)
        r = {"ms_per_step": round(ms, 4), "wall_ms_per_step": round(wall, 4), "tok_s": round(B * 1e3 / ms, 1),
             "kernel_ms_per_step": {k: round(v["ms"] / 3, 4) for k, v in prof.items()}}
        if sp["n_expert_local"]:
            # bytes a step must read: attention + router + the DISTINCT experts the batch selected (last layer's count)
            ids = ses.moe_last_ids(B)
            distinct = int(np.unique(ids).size)
            r["distinct_experts_last_layer"] = distinct
            if zipf:
                # how much of the carrier channel's level survives 48 layers of residual updates
                back = torch.empty(B * E, dtype=torch.float32, device="cuda")
                m.act_unpack_dev(m.Q8_0, out.data_ptr(), back.data_ptr(), B * E, stream.cuda_stream)
                stream.synchronize()
                h = back.cpu().numpy().reshape(B, E)
                r["carrier_channel_over_rms_in_out"] = [round(float(models.ZIPF_LEVEL / np.sqrt(((E - 1) + models.ZIPF_LEVEL ** 2) / E)), 3),
                                                        round(float(np.mean(h[:, models.ZIPF_CHANNEL] / np.sqrt(np.mean(h * h, axis=1)))), 3)]
            step_bytes = (st.weight_bytes - expert_bytes) + expert_bytes * distinct / sp["n_expert_local"] + kv_bytes_per_seq * B
        else:
            step_bytes = st.weight_bytes + kv_bytes_per_seq * B
        r["algorithmic_GB_per_step"] = round(step_bytes / 1e9, 3)
        r["GBps"] = round(step_bytes / ms / 1e6, 1)
        r["frac_hbm"] = round(step_bytes / ms / 1e6 / HBM_PEAK_GBS, 4)
        results[B] = r
    prefill = None
    if sp["prefill"] and args.prefill:
        T = sp["prefill"]
        xp = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).cuda()
        outp = torch.empty(m.act_packed_size(m.Q8_0, T, E), dtype=torch.uint8, device="cuda")
        ppos = np.arange(T, dtype=np.int32)

        def pstep(i):
            ses.decode_dev(xp.data_ptr(), ppos, outp.data_ptr(), outp.numel(), in_fmt=m.F32, out_fmt=m.Q8_0)

        pms, _ = time_on_stream(torch, stream, pstep, 2, 1)
        H = cfg["n_head"]
        FF = cfg["n_ff_exp"] * cfg["n_expert_used"] if cfg.get("n_expert") else cfg["n_ff"]      # FFN rows a token passes through
        mm_flop = 2.0 * T * L * (E * H * HD * 2 + E * HK * HD * 2 + 3 * E * FF)
        ses.profile(True)
        pstep(0)
        pprof = ses.profile_read()
        ses.profile(False)
        prefill = {"tokens": T, "ms": round(pms, 2), "tok_s": round(T * 1e3 / pms, 1), "matmul_TFLOP": round(mm_flop / 1e12, 2),
                   "matmul_TFLOPs_over_whole_step": round(mm_flop / pms / 1e9, 1),
                   "kernel_ms": {k: round(v["ms"], 2) for k, v in pprof.items()}}
    head = results[batches[0]]
    out = {"metric": sp["metric"], "value": head["tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "f32 activations x q4_K/q6_K weights, %s KV" % kv_name, "data": "synthetic",
           "config": {"workload": "%s-shaped stage, %d layers, Q4_K_M block-domain random weights, %d-token %s KV context, decode batch %d"
                                  % (sp["model"], L, n_ctx, kv_name, batches[0]),
                      "weight_bytes": st.weight_bytes, "kv_bytes_per_seq": kv_bytes_per_seq},
           "decode": {str(k): v for k, v in results.items()}, "prefill": prefill,
           "setup_s": {"generate_gguf": round(t_gen, 1), "open_stage": round(t_load, 1), "fill_kv": round(t_kv, 1)}}
    ses.close()
    st.close()
    del ses, st
    if sp.get("also_kv") and not args.kv_given:
        # the same decode batches once more on the other cache type (a stage of its own: the cache rows are fixed at open)
        import copy
        a2 = copy.copy(args)
        a2.kv, a2.kv_given, a2.prefill = sp["also_kv"], True, False
        torch.cuda.empty_cache()
        second = bench_shape(a2)
        out["decode_%s_kv" % sp["also_kv"].replace("/", "_")] = {"kv_bytes_per_seq": second["config"]["kv_bytes_per_seq"], **second["decode"]}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="stage", choices=["stage", "codec", "c4", "c5"])
    ap.add_argument("--batches", default=None, help="decode batch sizes; the first is the headline value (default 1,4,16 for the stage workload, the shape's own list for c4 / c5)")
    ap.add_argument("--kv", default="f16", choices=["f16", "q8_0/q4_0", "q4_0/q4_0"],
                    help="KV cache row types K/V (default f16: the tier the reference picks for an 8B Q4_K_M model)")
    ap.add_argument("--burn-in", type=int, default=80, help="untimed decode steps per batch size before anything is timed")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-prefill", dest="prefill", action="store_false", help="skip the 2048-token prefill measurement")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the stage path (one GPU per box); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    args.kv_given = any(a == "--kv" or a.startswith("--kv=") for a in sys.argv[1:])
    out = bench_stage(args) if args.workload == "stage" else bench_codec(args) if args.workload == "codec" else bench_shape(args)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
