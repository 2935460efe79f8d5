#!/usr/bin/env python3
"""Benchmark of the W4A4 linear hot path on one MI355X.

A step is one pass over the W4A4 linears of one Wan-2.1 14B transformer block
at 720p x 81 frames (M = 21*45*80 = 75600 tokens): fused QKV 5120->15360,
O-proj 5120->5120, FFN-up 5120->13824, FFN-down 13824->5120; every linear is
the dynamic per-token A4 quantizer followed by the W4A4 GEMM with its fused
scale/bias epilogue.  Inputs and packed weights are resident in HBM before the
timed region.  Prints ONE JSON line.

  value      effective TOPS of the whole step: sum(2*M*N*K) / step time
             (quantizer time included)
  roofline   the GEMM kernel alone (HIP events around its launches):
             algorithmic ops 2*M*N*K per launch / average launch duration,
             against the peak of the matrix instructions it runs on: the bf6
             path (v_mfma_f32_32x32x64_f8f6f4, what the library picks for
             shapes this large) 10.1 PFLOP/s dense FP6, --matrix-path int8
             (v_mfma_i32_32x32x32_i8) 5.0 POP/s dense INT8; the fraction of the
             INT8 peak is reported next to it in either case
  quantizer  the A4 quantizer alone: algorithmic bytes per launch (fp16 in,
             int4 rows or 6-bit blocks + one fp16 scale per row out) / average
             launch duration, against the 8 TB/s HBM3E peak
  cpu_baseline  the torch QuantLinear floating-point path (oracle/quantlinear_torch.py,
             a restatement of the reference's CPU-runnable path) on config 0
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

INT8_PEAK_TOPS = 5000.0  # MI355X dense INT8 MFMA, published
FP6_PEAK_TOPS = 10100.0  # MI355X dense FP6 MFMA, published
# HBM bytes per launch of the dominant kernels on the default workload, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this program (mean over the four launches of a step; the summary with the scaling by
# the copy kernel's readings is profiles/gemm_w4a4_kernel+quantize_rows_kernel.wan14b_720p_block.md for the int8
# path and profiles/gemm_bf6_persistent_kernel+quantize_rows_kernel.wan14b_720p_block.md for the bf6 path)
# gemm: (FETCH_SIZE 1377438 KiB x 2.0 + WRITE_SIZE 1455495 KiB x 1.0) x 1024; the reads are requests leaving L2
# (Infinity Cache or HBM), 9x the operand bytes because every XCD fetches most of its super-tile's slabs once.
# quant: (FETCH_SIZE 538736 KiB x 2.0 + WRITE_SIZE 269920 KiB x 1.0) x 1024 = 1.0005 x the algorithmic bytes.
# bf6 path, same method: gemm (FETCH_SIZE 2692746 KiB x 2.0 + WRITE_SIZE 1456313 KiB x 1.0) x 1024 (6-bit operands and
# little slab re-use between super-tiles: 12x the operand bytes); quant (538745 x 2.0 + 404284 x 1.0) x 1024 = 1.0002 x
# the algorithmic bytes.
MEASURED_TRAFFIC = {("wan14b_720p_block", "int8"): {"gemm": 4311418572, "quant": 1379729408},
                    ("wan14b_720p_block", "bf6"): {"gemm": 7006008524, "quant": 1517336576}}
HBM_PEAK_GBS = 8000.0    # MI355X HBM3E, published

# (name, K, N) at M tokens
WAN14B_720P = dict(M=75600, linears=[("qkv", 5120, 15360), ("o", 5120, 5120), ("ffn_up", 5120, 13824), ("ffn_down", 13824, 5120)])
WAN13B_480P = dict(M=32760, linears=[("qkv", 1536, 4608), ("o", 1536, 1536), ("ffn_up", 1536, 8960), ("ffn_down", 8960, 1536)])
WAN5B = dict(M=27280, linears=[("qkv", 3072, 9216), ("o", 3072, 3072), ("ffn_up", 3072, 14336), ("ffn_down", 14336, 3072)])
WORKLOADS = {"wan14b_720p_block": WAN14B_720P, "wan1.3b_480p_block": WAN13B_480P, "wan5b_704x1280_block": WAN5B}


def quant_bytes(M, K, bf6=False):
    if bf6:  # 6-bit codes, K padded to 128
        return 2 * M * K + M * (-(-K // 128) * 128) * 3 // 4 + 2 * M
    return 2 * M * K + M * K // 2 + 2 * M


def synth_inputs(torch, M, K, N, seed, dev):
    """X fp16 ~ N(0,1) with 1% of channels x20; int4 weights uniform in [-7,7]
    packed straight into the native layout; fp16 scales ~U(1e-3,1e-2); bias ~N(0,0.02)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn((M, K), generator=g, device=dev, dtype=torch.float32)
    cols = torch.randperm(K, generator=g, device=dev)[: -(-K // 100)]
    x[:, cols] *= 20
    x = x.half()
    q = torch.randint(-7, 8, (N, K), generator=g, device=dev, dtype=torch.int32)
    nib = (q & 0xF).to(torch.uint8)
    wq = (nib[:, 0::2] | (nib[:, 1::2] << 4)).contiguous()
    ws = (1e-3 + 9e-3 * torch.rand(N, generator=g, device=dev)).half()
    bias = (0.02 * torch.randn(N, generator=g, device=dev)).half()
    return x, wq, ws, bias


def cpu_baseline(torch, budget_s=16.0):
    """Reference torch QuantLinear fp path on config 0, on the host cores: repeated
    forwards for about budget_s seconds in all (half per dtype), median time."""
    from oracle.quantlinear_torch import QuantLinearTorchPath

    M, K, N = 4096, 1536, 4608
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    x = torch.randn((M, K), generator=g)
    x[:, torch.randperm(K, generator=g)[:16]] *= 20
    w = torch.randint(-7, 8, (N, K), generator=g).float() * (1e-3 + 9e-3 * torch.rand(N, 1, generator=g))
    b = 0.02 * torch.randn(N, generator=g)
    out, reps = {}, {}
    for name, dt in (("fp32", torch.float32), ("fp16", torch.float16)):
        layer = QuantLinearTorchPath(w.to(dt), b.to(dt))
        xs = x.to(dt)
        layer(xs)  # warm-up
        times = []
        t_start = time.perf_counter()
        while len(times) < 3 or time.perf_counter() - t_start < budget_s / 2:
            t0 = time.perf_counter()
            layer(xs)
            times.append(time.perf_counter() - t0)
        out[name], reps[name] = statistics.median(times), len(times)
    best = min(out.values())
    return {
        "value": round(2.0 * M * N * K / best / 1e12, 5), "unit": "TOPS", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"config 0 (M={M}, K={K}, N={N}; 0.058 TOP per forward), torch {torch.__version__} restatement of the reference's "
                  f"QuantLinear fp path (fake-quant W and X per forward + F.linear), ~{budget_s:.0f} s of repeated forwards, median s per forward: "
                  + ", ".join(f"{k}={v:.4f} ({reps[k]} reps)" for k, v in out.items()),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="wan14b_720p_block", choices=sorted(WORKLOADS))
    ap.add_argument("--matrix-path", default="auto", choices=["auto", "int8", "bf6"],
                    help="matrix instructions of the GEMM: auto = what the library picks for the shape")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run the library's plain 1 GiB copy kernel three times first, so that a rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                         "run holds a copy kernel of known size to scale the counters by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path shards by token rows with no exchange; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from dsaquant_amd import _lib
    from dsaquant_amd.kernels import vdm_w4a4 as v

    assert v.is_available(), f"libvdmq / GPU not available: {v.load_error()}"
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    wl = WORKLOADS[args.workload]
    M = wl["M"]

    if args.calibrate_copy:
        # the library's plain 128-bit copy kernel: reads 1 GiB, writes 1 GiB
        src = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(lib.vdmq_copy_u128(src.data_ptr(), dst.data_ptr(), src.numel(), torch.cuda.current_stream(dev).cuda_stream))
        torch.cuda.synchronize()
        del src, dst

    v.set_matrix_path(args.matrix_path)
    stream = torch.cuda.current_stream(dev)
    s = stream.cuda_stream
    layers = []
    for i, (name, K, N) in enumerate(wl["linears"]):
        x, wq, ws, bias = synth_inputs(torch, M, K, N, seed=i, dev=dev)
        Kp = v.k_padded(K)
        assert Kp == K
        bf6 = v._use_bf6(M, N, K)
        if bf6:  # operands of the bf6 path: 6-bit blocks (weights converted once, like a module's cache does)
            wblocks = torch.empty(int(lib.vdmq_bf6_bytes(N, K)), dtype=torch.uint8, device=dev)
            _lib.check(lib.vdmq_native_to_bf6(wq.data_ptr(), N, K, wblocks.data_ptr(), s))
            wq = wblocks
            qact = torch.empty(int(lib.vdmq_bf6_bytes(M, K)), dtype=torch.uint8, device=dev)
        else:
            qact = torch.empty((M, Kp // 2), dtype=torch.uint8, device=dev)
        layers.append(dict(name=name, K=K, N=N, x=x, wq=wq, ws=ws, bias=bias, bf6=bf6, qact=qact,
                           scale=torch.empty((M,), dtype=torch.float16, device=dev),
                           out=torch.empty((M, N), dtype=torch.float16, device=dev)))
    torch.cuda.synchronize()

    def run_step(events=None):
        for li, L in enumerate(layers):
            if events is not None:
                events[li][0].record(stream)
            if L["bf6"]:
                _lib.check(lib.vdmq_quantize_act_bf6(L["x"].data_ptr(), M, L["K"], L["K"], 1.0, 0, L["qact"].data_ptr(), L["scale"].data_ptr(), s))
            else:
                _lib.check(lib.vdmq_quantize_act(L["x"].data_ptr(), M, L["K"], L["K"], 1.0, L["qact"].data_ptr(), L["scale"].data_ptr(), s))
            if events is not None:
                events[li][1].record(stream)
            if L["bf6"]:
                _lib.check(lib.vdmq_gemm_w4a4_bf6(L["qact"].data_ptr(), L["scale"].data_ptr(), L["wq"].data_ptr(), L["ws"].data_ptr(),
                                                  L["bias"].data_ptr(), L["out"].data_ptr(), M, L["N"], L["K"], L["N"], s))
            else:
                _lib.check(lib.vdmq_gemm_w4a4(L["qact"].data_ptr(), L["scale"].data_ptr(), L["wq"].data_ptr(), L["ws"].data_ptr(),
                                              L["bias"].data_ptr(), L["out"].data_ptr(), _lib.VDMQ_OUT_F16, M, L["N"], L["K"], L["N"], s))
            if events is not None:
                events[li][2].record(stream)

    for _ in range(args.warmup):
        run_step()
    torch.cuda.synchronize()

    evs = [[[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in layers] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        run_step(evs[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    ms_per_step = wall * 1e3 / args.steps
    total_ops = sum(2.0 * M * L["N"] * L["K"] for L in layers)
    per_layer = {}
    gemm_ms_sum = quant_ms_sum = 0.0
    for li, L in enumerate(layers):
        q_ms = statistics.mean(evs[k][li][0].elapsed_time(evs[k][li][1]) for k in range(args.steps))
        g_ms = statistics.mean(evs[k][li][1].elapsed_time(evs[k][li][2]) for k in range(args.steps))
        gemm_ms_sum += g_ms
        quant_ms_sum += q_ms
        per_layer[L["name"]] = {
            "K": L["K"], "N": L["N"], "gemm_ms": round(g_ms, 4), "gemm_tops": round(2.0 * M * L["N"] * L["K"] / g_ms / 1e9, 1),
            "quant_ms": round(q_ms, 4), "quant_gbs": round(quant_bytes(M, L["K"], L["bf6"]) / q_ms / 1e6, 1),
            "matrix_path": "bf6" if L["bf6"] else "int8",
        }
    gemm_tops = total_ops / gemm_ms_sum / 1e9
    quant_gbs = sum(quant_bytes(M, L["K"], L["bf6"]) for L in layers) / quant_ms_sum / 1e6
    paths = sorted({"bf6" if L["bf6"] else "int8" for L in layers})
    path = paths[0] if len(paths) == 1 else "mixed"
    # a step that mixes both kinds of launches is priced against the higher peak
    peak = INT8_PEAK_TOPS if path == "int8" else FP6_PEAK_TOPS
    gemm_kernel = {"int8": "gemm_w4a4_kernel", "bf6": "gemm_bf6_persistent_kernel"}.get(path, "gemm_w4a4_kernel + gemm_bf6_persistent_kernel")
    traffic = MEASURED_TRAFFIC.get((args.workload, path), {})
    value = total_ops / (ms_per_step * 1e-3) / 1e12

    result = {
        "metric": "W4A4 GEMM TOPS (% INT8-MFMA peak) at Wan-14B 720p shapes; A4-quant GB/s",
        "value": round(value, 1), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("int4 x int4 -> int32 (int8 MFMA), fp16 in/out" if path == "int8" else
                  "int4 x int4 as exact E3M2 floats -> fp32 accumulator holding the exact integer (FP6 MFMA), fp16 in/out"),
        "data": "synthetic", "matrix_path": path,
        "config": {"workload": f"{args.workload}: M={M} tokens, linears " + ", ".join(f"{n} {k}->{o}" for n, k, o in wl["linears"])
                               + "; each = A4 quantizer + W4A4 GEMM + scale/bias epilogue, clip 1.0"},
        "roofline": {"bound": "mfma", "achieved": round(gemm_tops, 1), "peak": peak, "unit": "TOP/s",
                     "frac": round(gemm_tops / peak, 4), "frac_of_int8_peak": round(gemm_tops / INT8_PEAK_TOPS, 4),
                     "traffic": traffic.get("gemm"),
                     "traffic_unit": "HBM bytes per launch (mean of the step's four launches)", "kernel": gemm_kernel,
                     "algorithmic_ops_per_launch": total_ops / len(layers),
                     "avg_launch_ms": round(gemm_ms_sum / len(layers), 4)},
        "quantizer": {"bound": "hbm", "achieved": round(quant_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                      "frac": round(quant_gbs / HBM_PEAK_GBS, 4), "traffic": traffic.get("quant"),
                      "traffic_unit": "HBM bytes per launch (mean of the step's four launches)", "kernel": "quantize_rows_kernel",
                      "algorithmic_bytes_per_launch": sum(quant_bytes(M, L["K"], L["bf6"]) for L in layers) / len(layers),
                      "avg_launch_ms": round(quant_ms_sum / len(layers), 4)},
        "per_linear": per_layer,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
