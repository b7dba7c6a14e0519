#!/usr/bin/env python3
"""Benchmark of the E.T. encoder hot path on one MI355X.

Workload (config.workload): one BERT-base-shape encoder layer, six tile-pruned
linears at 80 % tile sparsity (16x16 tiles, seeded), on-the-fly fused attention,
batch 16 x seq 512, fp16 storage / fp32 accumulate, all sequences full length,
additive mask supplied (all zeros), base-2 softmax as in the reference.  A
"step" is one Encoder_tile::run over that batch with inputs resident in HBM.

Prints ONE JSON line: throughput in sequences/s (batch / layer time), the
roofline figures of the dominant kernel measured live with HIP events around
every launch of the layer sequence, a per-kernel table, and the CPU oracle
timed on this box's host cores as a reported baseline.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--extras]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
MFMA_F16_PEAK_TF = 2500.0   # MI355X dense fp16 MFMA, published

D, H, DFF = 768, 12, 3072

# HBM bytes per launch come from profiles/encoder_layer_b16_s512_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE, scaled by the 64 MiB copy kernel launched below).  The summary records a fingerprint of the kernel
# sources it was measured on; when the sources have changed since, `traffic` is null rather than a stale figure.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "encoder_layer_b16_s512_hbm_traffic.txt")
KERNEL_SOURCES = ("tile_linear.hip", "tile_tail.hip", "tile_plan.h", "attention.hip", "skip_layernorm.hip", "common.h")
TRAFFIC_KERNELS = {  # bench line -> kernel instance in the profile summary (the default workload's launches)
    "tile_linear qkv (3 x 768->768, one launch)": "et::tile_linear_resident_kernel<2, false, 12, false, 64>",
    "attention (on-the-fly)": "et::attention_kernel<64, 2, 4, false, false, true, 64, false>",
    "layer tail: o + skip + LayerNorm + feed-forward (gelu) + skip + LayerNorm, fused": "et::tile_ffn_fused_kernel<3, true>",
}


def kernel_source_fingerprint():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "et_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic_mib():
    """{kernel instance: fetch + write MiB per launch} from the profile summary, or {} when it is stale or absent"""
    import re
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return {}
    m = re.search(r"kernel sources fingerprint:\s*([0-9a-f]+)", text)
    if not m or m.group(1) != kernel_source_fingerprint():
        return {}
    out = {}
    for line in text.splitlines():
        m = re.match(r"(\S.*?)\s+n=\s*\d+\s+fetch avg\s+([0-9.]+) MiB\s+write avg\s+([0-9.]+) MiB", line)
        if m:
            out[m.group(1)] = float(m.group(2)) + float(m.group(3))
    return out


def tile_bytes(T, N, K, ntile):
    return 2 * T * K + 512 * ntile + 4 * ntile + 4 * (N // 16 + 1) + 2 * N + 2 * T * N


def tile_flops(T, ntile):
    return 512 * ntile * T


def product_tile_linear(r, N, K, sparsity, seed, std=0.02):
    """dense W ~ N(0, std) -> seeded tile_mat through the library's own generator and packer
    (et_gen_sparse_tile_mat / et_tile_pack); same dictionary as tests/helpers.make_tile_linear"""
    from et_amd import formats
    from et_amd.synthetic import randn_h
    W = randn_h(r, (N, K), std)
    row_ptr, row_offset = formats.gen_sparse_tile_mat(N, K, sparsity, seed)
    return dict(W=W, row_ptr=row_ptr, row_offset=row_offset, data=formats.tile_pack(W, row_ptr, row_offset),
                bias=np.zeros(N, np.float16), N=N, K=K)


def build_layer(orc, r, sparsity, seed):
    shapes = [(D, D)] * 4 + [(DFF, D), (D, DFF)]
    lins = [product_tile_linear(r, n, k, sparsity, seed=seed + j) for j, (n, k) in enumerate(shapes)]
    ln = [np.ones(D, np.float16), np.zeros(D, np.float16), np.ones(D, np.float16), np.zeros(D, np.float16)]
    return lins, ln


SPIN_UP_S = 0.2  # untimed run of the measured launches before every measurement (see main)


def spin_up(fn, seconds=SPIN_UP_S):
    """keep the GPU busy with fn for `seconds` (batches of 20 calls, each batch waited for, so the host never
    queues more than one batch ahead)"""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--seq", type=int, default=512)
    ap.add_argument("--sparsity", type=float, default=0.8)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--extras", action="store_true", help="also time the other BASELINE configurations")
    ap.add_argument("--one-stream", action="store_true",
                    help="skip the two-batches-in-flight figure (for profiler runs: launches that overlap on two "
                         "streams would mix into the per-kernel averages)")
    ap.add_argument("--micro", action="store_true",
                    help="only run the delivery-path microbenchmarks (LDS reads, weight stream, MFMA / vector-ALU "
                         "co-execution) and print their figures")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU (the path needs no collectives; it shards by "
              "batch). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    if args.micro:
        print(json.dumps(run_micro()))
        return

    import torch
    import oracle.et_oracle as orc          # checker / CPU baseline only
    from et_amd import kernels as K
    from et_amd.encoder import Encoder_tile, Linear_tile, run_multi
    from et_amd.synthetic import randn_h, rng

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    B, S = args.batch, args.seq
    T = B * S
    r = rng(2025)
    lins, ln = build_layer(orc, r, args.sparsity, seed=3000)
    x_h = randn_h(r, (T, D))
    mask_h = np.zeros((S, S), np.float16)
    x = torch.from_numpy(x_h).to(dev)

    def mk_linears():
        return [Linear_tile(l["K"], l["N"], T, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"],
                            l["bias"], j == 4) for j, l in enumerate(lins)]

    ws = torch.empty(Encoder_tile.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
    enc = Encoder_tile(D, S, H, ws, *mk_linears(), *ln, mask_h, B)
    out = torch.empty_like(x)

    # ---- a plain copy kernel of known size (64 MiB read + 64 MiB written):
    # the reference that rocprofv3's FETCH_SIZE / WRITE_SIZE are scaled against
    from et_amd._lib import check, lib
    cal_src = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    cal_dst = torch.empty_like(cal_src)
    cal_src.zero_()
    check(lib().et_copy(cal_dst.data_ptr(), cal_src.data_ptr(), cal_src.numel(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    del cal_src, cal_dst

    # ---- whole layer: W warm-up steps, then exactly K timed steps.  A GPU that comes out of idle runs its
    # first milliseconds at lower clocks (20 steps behind 5 warm-up steps read 5 % slower than behind 2000), so
    # the layer first runs untimed for SPIN_UP_S seconds: the timed steps see the clocks of a loop that has been
    # running, whatever W is.
    spin_up(lambda: enc.run(out, x))
    for _ in range(args.warmup):
        enc.run(out, x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        enc.run(out, x)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    seqs_per_s = B / (wall / args.steps)

    # ---- same launch sequence with HIP events around every kernel
    L = mk_linears()
    mask = torch.from_numpy(mask_h).to(dev)
    # as Encoder_base does at construction: let the launcher skip the mask's all-zero tiles
    mask_summary = K.attention_mask_summary(mask, S)
    K.attention_mask_summary_attach(mask, S, mask_summary)
    gam = [torch.from_numpy(t).to(dev) for t in ln]
    b = [torch.empty((T, D), dtype=torch.float16, device=dev) for _ in range(4)]
    ffn = torch.empty((T, DFF), dtype=torch.float16, device=dev)
    y = torch.empty((T, D), dtype=torch.float16, device=dev)
    nt = [l["row_offset"].size for l in lins]
    steps_def = [
        ("tile_linear qkv (3 x 768->768, one launch)", lambda: run_multi(L[:3], x, b[:3]),
         3 * tile_flops(T, nt[0]), sum(tile_bytes(T, D, D, nt[j]) for j in range(3)) - 2 * 2 * T * D, "hbm"),
        ("attention (on-the-fly)", lambda: K.OTF_attention(b[0], b[1], b[2], mask, S, H, B, None, 1.0, out=b[3]),
         4 * B * S * S * D, 8 * B * S * D + 2 * S * S, "mfma"),
        ("tile_linear o (768->768) + skip + LayerNorm", lambda: L[3].run_ln(b[3], x, gam[0], gam[1], out=b[0]),
         tile_flops(T, nt[3]), tile_bytes(T, D, D, nt[3]) + 2 * T * D + 4 * D, "hbm"),
        # the feed-forward block in one launch: X in, Y out, both weights once; the hidden activations stay in LDS
        ("feed-forward 768->3072->768 (gelu) + skip + LayerNorm, fused", lambda: Linear_tile.run_ffn_ln(L[4], L[5], b[0], b[0], gam[2], gam[3], out=y),
         tile_flops(T, nt[4]) + tile_flops(T, nt[5]),
         tile_bytes(T, DFF, D, nt[4]) + tile_bytes(T, D, DFF, nt[5]) - 2 * 2 * T * DFF + 4 * D, "mfma"),
    ]
    if Linear_tile.tail_fusable(L[3], L[4], L[5]):
        # steps 6-10 in one launch: attention output and layer input in, Y out, three weights once
        steps_def[-2:] = [
            ("layer tail: o + skip + LayerNorm + feed-forward (gelu) + skip + LayerNorm, fused",
             lambda: Linear_tile.run_tail(L[3], L[4], L[5], b[3], x, gam[0], gam[1], gam[2], gam[3], out=y),
             tile_flops(T, nt[3]) + tile_flops(T, nt[4]) + tile_flops(T, nt[5]),
             tile_bytes(T, D, D, nt[3]) + 2 * T * D + tile_bytes(T, DFF, D, nt[4]) + tile_bytes(T, D, DFF, nt[5])
             - 2 * 2 * T * DFF - 2 * 2 * T * D + 8 * D, "mfma"),
        ]
    elif not Linear_tile.ffn_fusable(L[4], L[5]):  # (tuning override): the two launches through a hidden buffer
        steps_def[-1:] = [
            ("tile_linear ffn1+gelu (768->3072)", lambda: L[4].run(b[0], out=ffn), tile_flops(T, nt[4]), tile_bytes(T, DFF, D, nt[4]), "hbm"),
            ("tile_linear ffn2 (3072->768) + skip + LayerNorm", lambda: L[5].run_ln(ffn, b[0], gam[2], gam[3], out=y),
             tile_flops(T, nt[5]), tile_bytes(T, D, DFF, nt[5]) + 2 * T * D + 4 * D, "hbm"),
        ]
    nk = len(steps_def)
    reps = max(20, min(args.steps, 100))

    def all_steps():
        for _, fn, *_ in steps_def:
            fn()
    spin_up(all_steps)
    for _ in range(5):
        all_steps()
    # (the first passes after the events are created are not counted: the first launch behind a fresh
    # batch of event records has been seen to block the host for tens of milliseconds)
    skip = 3
    ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(nk)]
          for _ in range(reps + skip)]
    torch.cuda.synchronize()
    for i in range(reps + skip):
        for j, (_, fn, *_r) in enumerate(steps_def):
            ev[i][j][0].record()
            fn()
            ev[i][j][1].record()
    torch.cuda.synchronize()
    ev = ev[skip:]
    kern = []
    for j, (name, _, flops, nbytes, bound) in enumerate(steps_def):
        us = float(np.mean([ev[i][j][0].elapsed_time(ev[i][j][1]) for i in range(reps)])) * 1e3
        kern.append({"kernel": name, "us": round(us, 2), "algo_MB": round(nbytes / 1e6, 2), "GFLOP": round(flops / 1e9, 3),
                     "GBps": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                     "TFLOPs": round(flops / us / 1e6, 1), "mfma_frac": round(flops / us / 1e6 / MFMA_F16_PEAK_TF, 4),
                     "bound": bound})
    default_cfg = (B, S, args.sparsity) == (16, 512, 0.8)
    traffic = measured_traffic_mib() if default_cfg else {}
    for k in kern:
        mib = traffic.get(TRAFFIC_KERNELS.get(k["kernel"], ""))
        k["traffic_MB"] = None if mib is None else round(mib * 1.048576, 2)
    dom = max(kern, key=lambda k: k["us"])
    if dom["bound"] == "hbm":
        roof = {"kernel": dom["kernel"], "bound": "hbm", "achieved": dom["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": dom["hbm_frac"], "traffic": dom["traffic_MB"], "traffic_unit": "MB/launch",
                "mfma_frac": dom["mfma_frac"]}
    else:
        roof = {"kernel": dom["kernel"], "bound": "mfma", "achieved": dom["TFLOPs"], "peak": MFMA_F16_PEAK_TF,
                "unit": "TFLOP/s", "frac": dom["mfma_frac"], "traffic": dom["traffic_MB"],
                "traffic_unit": "MB/launch", "hbm_frac": dom["hbm_frac"]}
    layer_flops = sum(k["GFLOP"] for k in kern)
    total_us = sum(k["us"] for k in kern)

    # ---- parity spot check of the timed configuration: three sequences from across the batch (sequences do
    # not interact, so the oracle runs them as a batch of their own)
    sample = sorted({0, B // 2, B - 1})
    srows = np.concatenate([np.arange(b * S, (b + 1) * S) for b in sample])
    got = out.float().cpu().numpy()[srows]
    want = orc.encoder_tile_layer(x_h[srows], lins, ln, mask_h, S, H, len(sample), None, 1.0).astype(np.float32)
    max_abs = float(np.abs(got - want).max())
    mean_rel = float(np.abs(got - want).mean() / np.abs(want).mean())

    # ---- CPU baseline: the fp32 host-loop oracle on a bounded sample of the same workload, with all host
    # threads and with one
    cpu = cpu1 = None
    if not args.no_cpu:
        import ctypes
        cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        orc.encoder_tile_layer(x_h[:S], lins, ln, mask_h, S, H, 1, None, 1.0)  # warm
        passes, t0 = 0, time.perf_counter()
        while passes < 40:  # whole batches of the same workload until about 10 s of CPU work
            orc.encoder_tile_layer(x_h, lins, ln, mask_h, S, H, B, None, 1.0)
            passes += 1
            dt = time.perf_counter() - t0
            if dt >= 10.0:
                break
        model = ""
        try:
            with open("/proc/cpuinfo") as f:
                model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "")
        except OSError:
            pass
        cpu = {"value": round(passes * B / dt, 3), "unit": "seqs/s", "cores": cores, "cpu_model": model, "kind": "port",
               "sample": f"{passes} passes over all {B} sequences (seq {S}) through the fp32 host-loop oracle layer, {dt:.1f} s",
               "ms_per_seq": round(dt / (passes * B) * 1e3, 2)}
        # one thread: single sequences of the same workload for about 8 s (the oracle's loops are OpenMP;
        # the thread count is set through the OpenMP runtime that the oracle library has loaded)
        try:
            gomp = ctypes.CDLL("libgomp.so.1")
            gomp.omp_set_num_threads(1)
            n1, t0 = 0, time.perf_counter()
            while n1 < B:
                orc.encoder_tile_layer(x_h[n1 * S:(n1 + 1) * S], lins, ln, mask_h, S, H, 1, None, 1.0)
                n1 += 1
                dt1 = time.perf_counter() - t0
                if dt1 >= 8.0:
                    break
            gomp.omp_set_num_threads(cores)
            cpu1 = {"value": round(n1 / dt1, 3), "unit": "seqs/s", "cores": 1, "cpu_model": model, "kind": "port",
                    "sample": f"{n1} single sequences (seq {S}) through the same oracle layer with one thread, {dt1:.1f} s"}
        except OSError:
            cpu1 = None

    extras = {}
    if args.extras:
        extras = run_extras(torch, orc, K, dev)

    res = {
        "metric": "encoder_layer_seqs_per_s", "value": round(seqs_per_s, 1), "unit": "seqs/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "spin_up_s": SPIN_UP_S, "ms_per_step": round(ms_per_step, 4),
        "latency_us": round(ms_per_step * 1e3, 1), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 storage, f32 accumulate", "data": "synthetic",
        "config": {"workload": f"BERT-base encoder layer, {int(args.sparsity * 100)}% tile-pruned linears (16x16), "
                               f"on-the-fly attention, batch {B} x seq {S}, all full length (BASELINE config 3)",
                   "batch": B, "seq_len": S, "d_model": D, "heads": H, "d_ff": DFF, "sparsity": args.sparsity,
                   "softmax_base": 2, "mask": "additive zeros"},
        "layer_GFLOP_surviving": round(layer_flops, 2),
        "layer_mfma_frac": round(layer_flops / (ms_per_step * 1e3) * 1e3 / MFMA_F16_PEAK_TF, 4),  # GFLOP/us = PFLOP/s
        "sum_kernel_us": round(total_us, 1),
        "parity_vs_oracle": {"max_abs": round(max_abs, 5), "mean_rel": round(mean_rel, 6), "rows": int(srows.size),
                             "sequences": sample},
        "roofline": roof, "kernels": kern, "cpu_baseline": cpu, "cpu_baseline_1thread": cpu1,
    }
    res.update(second_targets(torch, K, dev, enc, out, x, B, S, mask_h, lins, ln, two_streams=not args.one_stream))
    if extras:
        res["extras"] = extras
    print(json.dumps(res))


def run_micro():
    """Delivery-path microbenchmarks (et_microbench).  Rates are per CU; "clk" figures use the clock that the
    MFMA-only loop implies (a v_mfma_f32_16x16x32_f16 occupies its SIMD's matrix unit for 16 cycles)."""
    import ctypes as C
    from et_amd._lib import check, lib
    from et_amd.build import MICROBENCH_LIB

    lib()                                        # (the microbenchmark library links against the main one)
    if not os.path.exists(MICROBENCH_LIB):
        raise ImportError(f"{MICROBENCH_LIB} is missing: build it with `python -m et_amd.build`")
    mbl = C.CDLL(MICROBENCH_LIB)
    mbl.et_microbench.restype = C.c_int
    mbl.et_microbench.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]

    def mb(what, p0, p1):
        sec, units = C.c_double(), C.c_double()
        check(mbl.et_microbench(what, p0, p1, C.byref(sec), C.byref(units)))
        return sec.value, units.value

    res = {}
    t_m, n_m = mb(2, 0, 4)                       # one MFMA wave per SIMD
    clk_ghz = n_m * 16 / t_m / 1e9               # 16 cycles per MFMA
    res["clock_GHz_from_mfma_loop"] = round(clk_ghz, 3)
    lds = {}
    for stride, name in ((0, "linear"), (1568, "x_panel_stride_1568"), (160, "k_tile_stride_160"), (1552, "stride_1552"),
                         (1536, "stride_1536")):
        t, b = mb(0, stride, 16)
        lds[name] = {"GBps_per_CU": round(b / t / 1e9, 1), "bytes_per_clk_per_CU": round(b / t / 1e9 / clk_ghz, 1)}
    res["lds_ds_read_b128"] = lds
    ws = {}
    for waves in (4, 8, 16):
        t, b = mb(1, 0, waves)
        ws[f"{waves}_waves"] = {"GBps_per_CU": round(b / t / 1e9, 1), "bytes_per_clk_per_CU": round(b / t / 1e9 / clk_ghz, 1)}
    res["weight_stream_1KB_requests_from_L2"] = ws
    co = {}
    t_v, _ = mb(2, 1, 4)
    t_x, _ = mb(2, 2, 4)
    t_s, _ = mb(2, 3, 8)
    co["mfma_only_1_wave_per_simd_ms"] = round(t_m * 1e3, 4)
    co["fma_only_1_wave_per_simd_ms"] = round(t_v * 1e3, 4)
    co["alternating_in_one_wave_ms"] = round(t_x * 1e3, 4)
    co["mfma_wave_and_fma_wave_on_one_simd_ms"] = round(t_s * 1e3, 4)
    co["same_wave_overlap"] = round(1.0 - (t_x - max(t_m, t_v)) / min(t_m, t_v), 3)   # 1 = fully hidden, 0 = added
    co["two_wave_overlap"] = round(1.0 - (t_s - max(t_m, t_v)) / min(t_m, t_v), 3)
    res["mfma_valu_coexecution"] = co
    return res


def event_time(torch, fn, reps=100, warm=10):
    spin_up(fn)
    for _ in range(warm):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps * 1e3  # us


def second_targets(torch, K, dev, enc, out, x, B, S, mask_h, lins, ln, two_streams=True):
    """Figures that belong in the default line next to the headline: the stand-alone skip + LayerNorm on
    operands beyond the 256 MB last-level cache (an HBM figure, not a cache figure), BASELINE config 1
    (dense layer, batch 1 x seq 128) and the headline layer with a padding mask instead of the all-zero one."""
    from et_amd.encoder import Encoder_tile, Linear_tile
    from et_amd.synthetic import randn_h, rng
    res = {}
    rows = 131072
    gam = torch.ones(D, dtype=torch.float16, device=dev)
    bet = torch.zeros(D, dtype=torch.float16, device=dev)
    a_ = torch.randn((rows, D), device=dev).to(torch.float16)
    s_ = torch.randn((rows, D), device=dev).to(torch.float16)
    us = event_time(torch, lambda: K.skip_layernorm(a_, s_, gam, bet), reps=30, warm=3)
    nbytes = 6.0 * rows * D + 4 * D
    res["skip_layernorm"] = {"rows": rows, "width": D, "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                             "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                             "operand_MB": round(4.0 * rows * D / 1e6, 1)}
    del a_, s_
    # config 1: dense layer, batch 1 x seq 128
    r = rng(8)
    S1 = 128
    lins1, ln1 = build_layer(None, r, 0.0, seed=50)
    x1 = torch.from_numpy(randn_h(r, (S1, D))).to(dev)
    ws1 = torch.empty(Encoder_tile.buffer_size(D, S1, H, 1) // 2, dtype=torch.float16, device=dev)
    L1 = [Linear_tile(l["K"], l["N"], S1, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], j == 4)
          for j, l in enumerate(lins1)]
    enc1 = Encoder_tile(D, S1, H, ws1, *L1, *ln1, np.zeros((S1, S1), np.float16), 1)
    o1 = torch.empty_like(x1)
    res["config1_us"] = round(event_time(torch, lambda: enc1.run(o1, x1)), 2)
    # the headline layer with a padding mask (the last 64 keys masked out): the attention launch then runs
    # the form that reads and adds mask tiles, which the all-zero mask of the headline skips
    pm = np.zeros((S, S), np.float16)
    pm[:, S - 64:] = -30000.0
    T = B * S
    Lp = [Linear_tile(l["K"], l["N"], T, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], j == 4)
          for j, l in enumerate(lins)]
    wsp = torch.empty(Encoder_tile.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
    encp = Encoder_tile(D, S, H, wsp, *Lp, *ln, pm, B)
    res["latency_us_padding_mask"] = round(event_time(torch, lambda: encp.run(out, x), reps=50), 1)
    # ... and checked: its first and last sequence against the oracle with the same mask
    import oracle.et_oracle as orc          # checker only
    x_h = x.cpu().numpy()
    sample = sorted({0, B - 1})
    srows = np.concatenate([np.arange(b * S, (b + 1) * S) for b in sample])
    got = out.float().cpu().numpy()[srows]
    want = orc.encoder_tile_layer(x_h[srows], lins, ln, pm, S, H, len(sample), None, 1.0).astype(np.float32)
    res["parity_vs_oracle_padding_mask"] = {"max_abs": round(float(np.abs(got - want).max()), 5),
                                            "mean_rel": round(float(np.abs(got - want).mean() / np.abs(want).mean()), 6),
                                            "rows": int(srows.size), "sequences": sample}
    # two batches in flight: the same layer on a second set of buffers, steps alternating between two streams (a
    # server with more than one request queue).  A launch's start-up and drain then overlap the other stream's
    # kernel; `value` above stays the one-stream figure.
    if two_streams:
        L2_ = [Linear_tile(l["K"], l["N"], T, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], j == 4)
               for j, l in enumerate(lins)]
        ws2 = torch.empty(Encoder_tile.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
        enc2 = Encoder_tile(D, S, H, ws2, *L2_, *ln, mask_h, B)
        x2, out2 = x.clone(), torch.empty_like(x)
        st = [torch.cuda.Stream(), torch.cuda.Stream()]

        def pair_of_steps():
            with torch.cuda.stream(st[0]):
                enc.run(out, x)
            with torch.cuda.stream(st[1]):
                enc2.run(out2, x2)
        torch.cuda.synchronize()
        spin_up(pair_of_steps)
        npairs = 100
        t0 = time.perf_counter()
        for _ in range(npairs):
            pair_of_steps()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        res["two_batches_in_flight"] = {"seqs_per_s": round(2 * npairs * B / dt, 1),
                                        "us_per_batch": round(dt / (2 * npairs) * 1e6, 1), "steps": 2 * npairs, "streams": 2}
        del enc2, ws2, L2_
    # the headline layer replayed from a HIP graph of twenty runs (Encoder_tile::run only launches kernels, so a
    # caller can capture it: a 12-layer model is such a graph); replays repeated with eager work in between
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enc.run(out, x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for _ in range(20):
            enc.run(out, x)
    res["latency_us_hip_graph_of_20"] = round(event_time(torch, graph.replay, reps=10, warm=2) / 20, 1)
    return res


def run_extras(torch, orc, K, dev):
    """Other BASELINE configurations, timed with HIP events (reported, not the headline)."""
    from et_amd.encoder import Encoder_tile, Linear_tile
    from et_amd.synthetic import randn_h, rng
    out = {}

    def timeit(fn, reps=100, warm=10):
        spin_up(fn)
        for _ in range(warm):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps * 1e3  # us

    def timeit_graph(fn, reps=100, warm=3):
        """the same calls captured once in a HIP graph and replayed (no per-kernel launch work on the host)"""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            fn()
        return timeit(graph.replay, reps=reps, warm=warm)

    # config 2: tile linear 4096x768 -> 3072 at 0/50/80/90 %
    r = rng(7)
    M, N, Kd = 4096, 3072, 768
    X = torch.from_numpy(randn_h(r, (M, Kd))).to(dev)
    Y = torch.empty((M, N), dtype=torch.float16, device=dev)
    sweep = []
    for sp in (0.0, 0.5, 0.8, 0.9):
        lin = product_tile_linear(r, N, Kd, sp, seed=11)
        nt = lin["row_offset"].size
        lt = Linear_tile(Kd, N, M, nt, lin["data"], lin["row_ptr"], lin["row_offset"], lin["bias"])
        us = timeit(lambda: lt.run(X, out=Y))
        fl, by = tile_flops(M, nt), tile_bytes(M, N, Kd, nt)
        sweep.append({"sparsity": sp, "ntile": nt, "us": round(us, 2), "mfma_frac": round(fl / us / 1e6 / MFMA_F16_PEAK_TF, 4),
                      "hbm_frac": round(by / us / 1e3 / HBM_PEAK_GBS, 4)})
    out["config2_tile_linear_4096x768x3072"] = sweep

    # config 1: dense layer, batch 1 x seq 128
    r = rng(8)
    S, B = 128, 1
    lins, ln = build_layer(orc, r, 0.0, seed=50)
    x = torch.from_numpy(randn_h(r, (S, D))).to(dev)
    ws = torch.empty(Encoder_tile.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
    L = [Linear_tile(l["K"], l["N"], S, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], j == 4)
         for j, l in enumerate(lins)]
    enc = Encoder_tile(D, S, H, ws, *L, *ln, np.zeros((S, S), np.float16), B)
    o = torch.empty_like(x)
    us = timeit(lambda: enc.run(o, x))
    us_g = timeit_graph(lambda: enc.run(o, x))
    out["config1_dense_layer_b1_s128"] = {"us": round(us, 2), "seqs_per_s": round(1e6 / us, 1),
                                          "us_as_hip_graph": round(us_g, 2)}

    # stand-alone skip + LayerNorm (the launcher replacement; the layer itself runs the fused form):
    # 6 bytes per element moved.  The 38 MB of 8192 rows (config 3's count) stay in the last-level
    # cache between launches; the larger counts stream from HBM.
    ln_rows = []
    gam = torch.ones(D, dtype=torch.float16, device=dev)
    bet = torch.zeros(D, dtype=torch.float16, device=dev)
    for rows in (8192, 32768, 131072, 524288):
        a_ = torch.randn((rows, D), device=dev).to(torch.float16)
        s_ = torch.randn((rows, D), device=dev).to(torch.float16)
        us = timeit(lambda: K.skip_layernorm(a_, s_, gam, bet), reps=100 if rows <= 32768 else 30)
        if rows <= 32768:
            # a launch this short is issued no faster than the Python wrapper returns: twenty of them
            # captured in one HIP graph take the host out of the figure
            us = min(us, timeit_graph(lambda: [K.skip_layernorm(a_, s_, gam, bet) for _ in range(20)], reps=20) / 20)
        nbytes = 6.0 * rows * D + 4 * D
        ln_rows.append({"rows": rows, "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                        "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
        del a_, s_
    out["skip_layernorm_768_wide"] = ln_rows

    # the headline layer (80 % tile-pruned) at seq 128: batch 64, the same number of rows
    r = rng(12)
    S, B = 128, 64
    lins, ln = build_layer(orc, r, 0.8, seed=60)
    x = torch.from_numpy(randn_h(r, (S * B, D))).to(dev)
    ws = torch.empty(Encoder_tile.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
    L = [Linear_tile(l["K"], l["N"], S * B, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], j == 4)
         for j, l in enumerate(lins)]
    enc128 = Encoder_tile(D, S, H, ws, *L, *ln, np.zeros((S, S), np.float16), B)
    o = torch.empty_like(x)
    us = timeit(lambda: enc128.run(o, x))
    out["pruned_layer_80pct_b64_s128"] = {"us": round(us, 2), "seqs_per_s": round(B * 1e6 / us, 1)}
    del enc128, ws

    # the reference's own pruned wiring (test/prune_test.cu: tile-pruned Q, K, O, FFN; row-pruned V,
    # pruned attention), batch 16 x seq 512, 80 % tiles, V keeps 230 of 768 rows
    from et_amd.encoder import Encoder_prune, Linear_row
    r = rng(13)
    S, B = 512, 16
    lins, ln = build_layer(orc, r, 0.8, seed=70)
    v_id = orc.gen_sparse_row_mat(D, 0.7, seed=16)
    mk = lambda l, g=False: Linear_tile(l["K"], l["N"], S * B, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], g)
    Lv = Linear_row(D, D, S * B, randn_h(r, (v_id.size, D), 0.02), v_id, v_id.size, np.zeros(v_id.size, np.float16), H)
    ws = torch.empty(Encoder_prune.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
    encp = Encoder_prune(D, S, H, ws, mk(lins[0]), mk(lins[1]), Lv, mk(lins[3]), mk(lins[4], True), mk(lins[5]), *ln,
                         np.zeros((S, S), np.float16), B)
    x = torch.from_numpy(randn_h(r, (S * B, D))).to(dev)
    o = torch.empty_like(x)
    us = timeit(lambda: encp.run(o, x))
    out["reference_prune_wiring_b16_s512"] = {"us": round(us, 2), "seqs_per_s": round(B * 1e6 / us, 1)}
    del encp, ws

    # config 4: attention-aware pruned layer, batch 32 x seq 256 (Q/K keep 32 of 64 columns per head,
    # O/FFN1/FFN2 row-pruned at 70 %)
    from et_amd.encoder import Encoder_attnaware, Linear_row
    r = rng(9)
    S, B = 256, 32
    T = S * B
    pad16 = lambda n: (n + 15) // 16 * 16
    qk_id = orc.gen_head_balanced_rows(H, D // H, 32, seed=11)
    o_id, m1_id, m2_id = (orc.gen_sparse_row_mat(n, 0.7, seed=s) for n, s in ((D, 12), (DFF, 13), (D, 14)))
    rw = lambda n, k: randn_h(r, (n, k), 0.02)
    zb = lambda n: np.zeros(n, np.float16)
    vt = product_tile_linear(r, D, D, 0.0, seed=15)
    Lq, Lk = (Linear_row(D, D, T, rw(qk_id.size, D), qk_id, qk_id.size, zb(qk_id.size), H) for _ in range(2))
    Lv = Linear_tile(D, D, T, vt["row_offset"].size, vt["data"], vt["row_ptr"], vt["row_offset"], vt["bias"])
    Lo = Linear_row(D, D, T, rw(o_id.size, D), o_id, o_id.size, zb(o_id.size), H)
    L1 = Linear_row(D, DFF, T, rw(m1_id.size, D), m1_id, m1_id.size, zb(m1_id.size), H, is_gelu=True)
    L2 = Linear_row(pad16(m1_id.size), D, T, rw(m2_id.size, pad16(m1_id.size)), m2_id, m2_id.size, zb(m2_id.size), H)
    ws = torch.empty(Encoder_attnaware.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
    ln1 = [np.ones(D, np.float16), np.zeros(D, np.float16)] * 2
    enc4 = Encoder_attnaware(D, S, H, ws, Lq, Lk, Lv, Lo, L1, L2, *ln1, np.zeros((S, S), np.float16), B)
    x = torch.from_numpy(randn_h(r, (T, D))).to(dev)
    o = torch.empty_like(x)
    us = timeit(lambda: enc4.run(o, x), reps=50)
    out["config4_attention_aware_pruned_layer_b32_s256"] = {"us": round(us, 2), "seqs_per_s": round(B * 1e6 / us, 1)}
    del enc4, ws

    # config 5: 12-layer stack, batch 64, lengths ~ U{32..512} padded to 512: packed (length-aware) vs padded
    from et_amd.encoder import Encoder_length, Encoder_stack
    r = rng(10)
    S, B, NL = 512, 64, 12
    lens = r.integers(32, 513, size=B).astype(np.int32)
    layers = []
    for li in range(NL):
        lins, ln = build_layer(orc, r, 0.8, seed=200 + 10 * li)
        ws = torch.empty(Encoder_length.buffer_size(D, S, H, B) // 2, dtype=torch.float16, device=dev)
        L = [Linear_tile(l["K"], l["N"], S * B, l["row_offset"].size, l["data"], l["row_ptr"], l["row_offset"], l["bias"], j == 4)
             for j, l in enumerate(lins)]
        layers.append((Encoder_length(D, S, H, ws, *L, *ln, np.zeros((S, S), np.float16), B), ws))
    x = torch.from_numpy(randn_h(r, (S * B, D))).to(dev)
    o = torch.empty_like(x)
    stack = Encoder_stack([l for l, _ in layers], D, S, B)
    res5 = {"lengths_sum": int(lens.sum()), "padded_rows": S * B}
    for name, ll in (("padded", None), ("length_aware", lens)):
        for l, _ in layers:
            l.set_seq_lens(ll)
        us = timeit(lambda: stack.run(o, x), reps=10, warm=3)
        res5[name] = {"us_12_layers": round(us, 1), "seqs_per_s": round(B * 1e6 / us, 1)}
        if ll is not None:
            res5[name]["us_12_layers_as_hip_graph"] = round(timeit_graph(lambda: stack.run(o, x), reps=10), 1)
    res5["padding_skip_speedup"] = round(res5["padded"]["us_12_layers"] / res5["length_aware"]["us_12_layers"], 3)
    out["config5_length_aware_12_layer_stack_b64"] = res5
    return out


if __name__ == "__main__":
    main()
