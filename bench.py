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

Beside the headline fields the line carries, all measured in the same run (the figures a reader needs are repeated
as flat numbers inside the `roofline` object: int8_path_*, quantizer_*, <workload>_gemm_*, <case>_*, config4_*):
  int8_path     the same workload with the GEMM forced onto the int8 matrix instructions (gemm_w4a4_kernel), with its
                own roofline object against the 5.0 POP/s INT8 peak
  workloads     whole-step TOPS of the other block workloads (Wan-2.1 1.3B at 480p, Wan-2.2 5B) on the path the
                library picks
  cases         single linears: config 0's fused QKV at M = 4096 (the shape the CPU baseline is timed on), the 14B
                model's cross-attention K/V projection (M = 512 text tokens) and its fused QKV with a ragged last tile
                (M = 75600 + 37)
  config4       the end-to-end Wan-2.1 1.3B DiT harness (30 blocks, 32760 tokens, cond + uncond, 5 steps; bench_dit.py):
                ms per step and the shares of the W4A4 calls and of attention
  stream_ceiling  what a kernel that only streams sustains with the quantizer's mix of reads and writes over the same
                volumes (vdmq_stream_probe), the memory system's ceiling for that mix: the quantizer is read against it
  mfma_ceiling  what the two MFMA instructions sustain in a loop with nothing else (vdmq_mfma_probe) on all-zero
                operands, on int4-valued operands and on operands with the workload's statistics: the published peaks
                assume the top clock, which the part does not hold under matrix load
--per-linear adds the per-launch table of every workload.  --ubench prints only the probe (longer runs), for counter
collection with rocprofv3.

Weights start as a checkpoint holds them -- int4 in the v1 byte order, scales replicated per 64-deep k-group -- and go
through the library's own load-time relayout (vdmq_weight_v1_to_bf6 / vdmq_weight_v1_to_native, vdmq_wscale_v1_to_plain),
untimed, as a loaded module's do.
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
# Bytes that left the XCDs' L2 caches per launch of the dominant kernels on the default workload (mean over the four
# launches of a step).  NOT measured by this program: hardware counters need the profiler.  The figures are copied
# from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summaries named below (each reading scaled by what the same counter
# shows for the library's plain copy kernel of known size in the same run) and belong to the library build those
# files name; the line says so ("traffic_source").  Requests that leave an L2 are served by the 256 MB Infinity Cache
# or by HBM -- no counter available here separates the two -- so for the GEMM, whose operands fit that cache, this is
# an upper bound of its HBM bytes; for the quantizer (a stream far larger than the cache) it is the HBM traffic.
TRAFFIC_FROM_PROFILES = {
    ("wan14b_720p_block", "int8"): {"gemm": 4315445555, "quant": 1379725133,
                                    "source": "profiles/gemm_w4a4_kernel+quantize_rows_kernel.wan14b_720p_block.md"},
    ("wan14b_720p_block", "bf6"): {"gemm": 6434431309, "quant": 1517356237,
                                   "source": "profiles/gemm_bf6_persistent_kernel+quantize_rows_kernel.wan14b_720p_block.md"},
}
TRAFFIC_UNIT = "bytes leaving L2 per launch, mean of the step's 4 launches; from traffic_source, not from this run"
HBM_PEAK_GBS = 8000.0    # MI355X HBM3E, published

# (name, K, N) at M tokens
WAN14B_720P = dict(M=75600, linears=[("qkv", 5120, 15360), ("o", 5120, 5120), ("ffn_up", 5120, 13824), ("ffn_down", 13824, 5120)])
WAN13B_480P = dict(M=32760, linears=[("qkv", 1536, 4608), ("o", 1536, 1536), ("ffn_up", 1536, 8960), ("ffn_down", 8960, 1536)])
WAN5B = dict(M=27280, linears=[("qkv", 3072, 9216), ("o", 3072, 3072), ("ffn_up", 3072, 14336), ("ffn_down", 14336, 3072)])
WORKLOADS = {"wan14b_720p_block": WAN14B_720P, "wan1.3b_480p_block": WAN13B_480P, "wan5b_704x1280_block": WAN5B}
# single linears (benchmark configurations 0 and 3), timed next to the blocks
CASES = {"cfg0_qkv_m4096": dict(M=4096, linears=[("qkv", 1536, 4608)]),
         "cfg3_cross_kv_m512": dict(M=512, linears=[("cross_kv", 5120, 10240)]),
         "cfg3_qkv_ragged_m75637": dict(M=75637, linears=[("qkv", 5120, 15360)])}
SHORT = {"wan1.3b_480p_block": "wan1p3b", "wan5b_704x1280_block": "wan5b", "wan14b_720p_block": "wan14b"}


def quant_bytes(M, K, bf6=False):
    if bf6:  # 6-bit codes, K padded to 128
        return 2 * M * K + M * (-(-K // 128) * 128) * 3 // 4 + 2 * M
    return 2 * M * K + M * K // 2 + 2 * M


def synth_inputs(torch, lib, check, M, K, N, seed, dev, stream):
    """X fp16 ~ N(0,1) with 1% of channels x20; int4 weights uniform in [-7,7] and fp16 scales ~U(1e-3,1e-2) as a
    packed checkpoint holds them (v1 byte order, scales repeated per k-group); bias ~N(0,0.02)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn((M, K), generator=g, device=dev, dtype=torch.float32)
    cols = torch.randperm(K, generator=g, device=dev)[: -(-K // 100)]
    x[:, cols] *= 20
    x = x.half()
    q = torch.randint(-7, 8, (N, K), generator=g, device=dev, dtype=torch.int32)
    nib = (q & 0xF).to(torch.uint8)
    rows = (nib[:, 0::2] | (nib[:, 1::2] << 4)).contiguous()
    ws = (1e-3 + 9e-3 * torch.rand(N, generator=g, device=dev)).half()
    bias = (0.02 * torch.randn(N, generator=g, device=dev)).half()
    wq_v1 = torch.empty((N, K // 2), dtype=torch.uint8, device=dev)
    ws_v1 = torch.empty((N, K // 64), dtype=torch.float16, device=dev)
    check(lib.vdmq_weight_native_to_v1(rows.data_ptr(), wq_v1.data_ptr(), N, K, stream))
    check(lib.vdmq_wscale_plain_to_v1(ws.data_ptr(), ws_v1.data_ptr(), N, K, stream))
    return x, wq_v1, ws_v1, bias


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

class Workload:
    """The linears of one block with inputs, packed weights and outputs resident on the device."""

    def __init__(self, torch, lib, v, name, path, dev):
        from dsaquant_amd import _lib

        self.torch, self.lib, self._lib, self.name, self.dev = torch, lib, _lib, name, dev
        wl = WORKLOADS.get(name) or CASES[name]
        self.M = M = wl["M"]
        self.stream = torch.cuda.current_stream(dev)
        s = self.stream.cuda_stream
        self.layers = []
        for i, (lname, K, N) in enumerate(wl["linears"]):
            x, wq_v1, ws_v1, bias = synth_inputs(torch, lib, _lib.check, M, K, N, seed=i, dev=dev, stream=s)
            assert v.k_padded(K) == K
            bf6 = v._use_bf6(M, N, K, path=path)
            # the load-time relayout of a packed checkpoint's buffers into the one form the chosen kernels stream
            ws = torch.empty((N,), dtype=torch.float16, device=dev)
            _lib.check(lib.vdmq_wscale_v1_to_plain(ws_v1.data_ptr(), ws.data_ptr(), N, K, s))
            if bf6:
                wq = torch.empty(int(lib.vdmq_bf6_bytes(N, K)), dtype=torch.uint8, device=dev)
                _lib.check(lib.vdmq_weight_v1_to_bf6(wq_v1.data_ptr(), wq.data_ptr(), N, K, s))
                qact = torch.empty(int(lib.vdmq_bf6_bytes(M, K)), dtype=torch.uint8, device=dev)
            else:
                wq = torch.empty((N, K // 2), dtype=torch.uint8, device=dev)
                _lib.check(lib.vdmq_weight_v1_to_native(wq_v1.data_ptr(), wq.data_ptr(), N, K, s))
                qact = torch.empty((M, K // 2), dtype=torch.uint8, device=dev)
            del wq_v1, ws_v1
            self.layers.append(dict(name=lname, K=K, N=N, x=x, wq=wq, ws=ws, bias=bias, bf6=bf6, qact=qact,
                                    scale=torch.empty((M,), dtype=torch.float16, device=dev),
                                    out=torch.empty((M, N), dtype=torch.float16, device=dev)))
        torch.cuda.synchronize()

    def step(self, events=None):
        lib, _lib, M, s = self.lib, self._lib, self.M, self.stream.cuda_stream
        # events[2 * li] .. [2 * li + 1] bracket layer li's quantizer, [2 * li + 1] .. [2 * li + 2] its GEMM: a GEMM's
        # end is the next quantizer's start (an event record costs the stream 2...3 us)
        if events is not None:
            events[0].record(self.stream)
        for li, L in enumerate(self.layers):
            if L["bf6"]:
                _lib.check(lib.vdmq_quantize_act_bf6(L["x"].data_ptr(), M, L["K"], L["K"], 1.0, 0, L["qact"].data_ptr(), L["scale"].data_ptr(), s))
            else:
                _lib.check(lib.vdmq_quantize_act(L["x"].data_ptr(), M, L["K"], L["K"], 1.0, L["qact"].data_ptr(), L["scale"].data_ptr(), s))
            if events is not None:
                events[2 * li + 1].record(self.stream)
            if L["bf6"]:
                _lib.check(lib.vdmq_gemm_w4a4_bf6(L["qact"].data_ptr(), L["scale"].data_ptr(), L["wq"].data_ptr(), L["ws"].data_ptr(),
                                                  L["bias"].data_ptr(), L["out"].data_ptr(), _lib.VDMQ_OUT_F16, M, L["N"], L["K"], L["N"], s))
            else:
                _lib.check(lib.vdmq_gemm_w4a4(L["qact"].data_ptr(), L["scale"].data_ptr(), L["wq"].data_ptr(), L["ws"].data_ptr(),
                                              L["bias"].data_ptr(), L["out"].data_ptr(), _lib.VDMQ_OUT_F16, M, L["N"], L["K"], L["N"], s))
            if events is not None:
                events[2 * li + 2].record(self.stream)
            if events is not None and "kernel" not in L:
                L["kernel"] = {1: "gemm_w4a4_kernel", 2: "gemm_bf6_kernel", 3: "gemm_bf6_persistent_kernel"}[_lib.last_gemm_launch().kernel]

    def measure(self, steps, warmup):
        """W untimed steps, then exactly K timed steps between synchronisations; per-launch times from HIP events
        recorded on the stream the kernels run on."""
        torch, M = self.torch, self.M
        for _ in range(warmup):
            self.step()
        torch.cuda.synchronize()
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(2 * len(self.layers) + 1)] for _ in range(steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(steps):
            self.step(evs[k])
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms_per_step = wall * 1e3 / steps
        total_ops = sum(2.0 * M * L["N"] * L["K"] for L in self.layers)
        per_layer, gemm_ms, quant_ms = {}, 0.0, 0.0
        for li, L in enumerate(self.layers):
            q_ms = statistics.mean(evs[k][2 * li].elapsed_time(evs[k][2 * li + 1]) for k in range(steps))
            g_ms = statistics.mean(evs[k][2 * li + 1].elapsed_time(evs[k][2 * li + 2]) for k in range(steps))
            gemm_ms += g_ms
            quant_ms += q_ms
            per_layer[L["name"]] = {
                "K": L["K"], "N": L["N"], "gemm_ms": round(g_ms, 4), "gemm_tops": round(2.0 * M * L["N"] * L["K"] / g_ms / 1e9, 1),
                "quant_ms": round(q_ms, 4), "quant_gbs": round(quant_bytes(M, L["K"], L["bf6"]) / q_ms / 1e6, 1),
                "quant_gbs_int4_bytes": round(quant_bytes(M, L["K"]) / q_ms / 1e6, 1),
                "matrix_path": "bf6" if L["bf6"] else "int8", "kernel": L["kernel"],
            }
        n = len(self.layers)
        paths = sorted({"bf6" if L["bf6"] else "int8" for L in self.layers})
        kernels = sorted({L["kernel"] for L in self.layers})
        path = paths[0] if len(paths) == 1 else "mixed"
        # a step that mixes both kinds of launches is priced against the higher peak
        peak = INT8_PEAK_TOPS if path == "int8" else FP6_PEAK_TOPS
        gemm_tops = total_ops / gemm_ms / 1e9
        block_bytes = sum(quant_bytes(M, L["K"], L["bf6"]) for L in self.layers)
        int4_bytes = sum(quant_bytes(M, L["K"]) for L in self.layers)
        traffic = TRAFFIC_FROM_PROFILES.get((self.name, path), {})
        return {
            "path": path, "ms_per_step": ms_per_step, "step_tops": total_ops / (ms_per_step * 1e-3) / 1e12, "total_ops": total_ops,
            "roofline": {"bound": "mfma", "achieved": round(gemm_tops, 1), "peak": peak, "unit": "TOP/s", "frac": round(gemm_tops / peak, 4),
                         "frac_of_int8_peak": round(gemm_tops / INT8_PEAK_TOPS, 4), "traffic": traffic.get("gemm"),
                         "traffic_unit": TRAFFIC_UNIT if traffic else None, "traffic_source": traffic.get("source"), "kernel": " + ".join(kernels),
                         "algorithmic_ops_per_launch": total_ops / n, "avg_launch_ms": round(gemm_ms / n, 4)},
            "quantizer": {"bound": "hbm", "achieved": round(block_bytes / quant_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(block_bytes / quant_ms / 1e6 / HBM_PEAK_GBS, 4),
                          "achieved_int4_bytes": round(int4_bytes / quant_ms / 1e6, 1),
                          "frac_int4_bytes": round(int4_bytes / quant_ms / 1e6 / HBM_PEAK_GBS, 4),
                          "traffic": traffic.get("quant"),
                          "kernel": "quantize_rows_kernel", "algorithmic_bytes_per_launch": block_bytes / n,
                          "avg_launch_ms": round(quant_ms / n, 4)},
            "per_linear": per_layer,
        }


BF6_CODES = [0, 1, 2, 3, 4, 5, 6, 7, 8]  # E3M2 codes of |q| / 16, |q| = 0..8, as the operand blocks hold them; the sign is bit 5


def probe_operands(np, kind, data, rng):
    """Register images for vdmq_mfma_probe: [8 waves][12 operands][64 lanes] x 32 bytes.  ``data``: "zeros"; "int4"
    = both sides uniform in [-8, 7]; "workload" = weight side uniform in [-7, 7], token side with the statistics of
    the benchmark activations (N(0,1) with 1 % of the channels x 20, per-token scale absmax / 7: mostly 0 and +-1);
    "bytes" (int8 only) = uniformly random bytes."""
    per = 32 if kind == "bf6" else 16  # int4 values one lane holds per operand: a 192-bit string of codes / 16 bytes
    shape = (8, 12, 64, per)
    if data == "zeros":
        q = np.zeros(shape, np.int64)
    elif data == "int4":
        q = rng.integers(-8, 8, shape)
    elif data == "workload":
        q = rng.integers(-7, 8, shape)
        K = 5120
        x = rng.standard_normal((8 * 8 * 64, K)).astype(np.float32)
        x[:, rng.permutation(K)[: -(-K // 100)]] *= 20.0
        scale = np.abs(x).max(axis=1, keepdims=True) / 7.0
        qx = np.clip(np.rint(x / scale), -8, 7).astype(np.int64)  # one token row per lane; the lane takes `per` consecutive k
        start = rng.integers(0, K - per, 8 * 8 * 64)
        tok = np.stack([qx[i, st:st + per] for i, st in enumerate(start)]).reshape(8, 8, 64, per)
        for side, o in enumerate((2, 3, 4, 5, 8, 9, 10, 11)):  # the token-side operands
            q[:, o] = tok[:, side]
    elif data == "bytes" and kind == "int8":
        q = None
    else:
        raise ValueError(data)
    img = np.zeros((8, 12, 64, 32), np.uint8)
    if kind == "int8":
        img[..., :16] = rng.integers(0, 256, shape, dtype=np.uint8) if q is None else ((q & 0xF) << 4).astype(np.uint8)  # bytes 16 * q
    else:
        codes = np.asarray(BF6_CODES, np.uint8)[np.abs(q)] | np.where(q < 0, 0x20, 0).astype(np.uint8)
        bits = (codes[..., None] >> np.arange(6, dtype=np.uint8)) & 1  # code e at bits [6e, 6e + 6)
        img[..., :24] = np.packbits(bits.reshape(*shape[:3], 192), axis=-1, bitorder="little")
    return img


def stream_ceiling(torch, lib, dev, M, Ks, bf6, repeats=10):
    """What a kernel that only streams sustains with the quantizer's mix of reads and writes (vdmq_stream_probe:
    8 : 3 for 6-bit operand blocks, 4 : 1 for int4 rows; a wave reads consecutive kilobytes and writes fewer
    consecutive ones) over the byte volumes of the workload's quantizer launches; also a plain copy and reads alone
    at the largest volume.  GB/s of bytes moved (read + written)."""
    from dsaquant_amd import _lib

    stream = torch.cuda.current_stream(dev)
    reads, writes = (8, 3) if bf6 else (4, 1)
    biggest = max(M * K * 2 for K in Ks)
    src = torch.zeros(biggest, dtype=torch.uint8, device=dev)
    dst = torch.empty(biggest, dtype=torch.uint8, device=dev)

    def timed(threads, r, w):
        run = lambda: _lib.check(lib.vdmq_stream_probe(src.data_ptr(), dst.data_ptr(), threads, r, w, stream.cuda_stream))
        for _ in range(2):
            run()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        for _ in range(repeats):
            run()
        b.record(stream)
        torch.cuda.synchronize()
        return a.elapsed_time(b) / repeats  # ms

    moved, ms, per_k = 0.0, 0.0, {}
    for K in Ks:
        threads = M * K * 2 // (reads * 16) // 64 * 64
        t = timed(threads, reads, writes)
        per_k[str(K)] = round(threads * (reads + writes) * 16 / t / 1e6, 1)
        moved += threads * (reads + writes) * 16
        ms += t
    threads = biggest // 16 // 64 * 64
    res = {"mix": f"{reads}:{writes}", "gbs": round(moved / ms / 1e6, 1), "gbs_by_row_length": per_k,
           "copy_gbs": round(threads * 32 / timed(threads, 1, 1) / 1e6, 1), "read_only_gbs": round(threads // 4 * 64 / timed(threads // 4, 4, 0) / 1e6, 1)}
    del src, dst
    torch.cuda.empty_cache()
    return res


def quantizers_alone(torch, lib, dev, M, Ks, repeats=20):
    """The two A4 quantizers (6-bit operand blocks, int4 rows) on the workload's row lengths, back to back launches
    timed with HIP events: GB/s of the bytes each really moves.  For reading next to stream_ceiling in one run."""
    from dsaquant_amd import _lib

    stream = torch.cuda.current_stream(dev)
    s = stream.cuda_stream
    out = {"bf6_blocks": {}, "int4_rows": {}}
    for K in Ks:
        x = synth_inputs(torch, lib, _lib.check, M, K, 128, 7, dev, s)[0]
        scale = torch.empty((M,), dtype=torch.float16, device=dev)
        blocks = torch.empty((int(lib.vdmq_bf6_bytes(M, K)),), dtype=torch.uint8, device=dev)
        rows = torch.empty((M, int(lib.vdmq_k_padded(K)) // 2), dtype=torch.uint8, device=dev)
        forms = {"bf6_blocks": (lambda: _lib.check(lib.vdmq_quantize_act_bf6(x.data_ptr(), M, K, K, 1.0, 0, blocks.data_ptr(), scale.data_ptr(), s)),
                                M * (2 * K + 3 * K // 4 + 2)),
                 "int4_rows": (lambda: _lib.check(lib.vdmq_quantize_act(x.data_ptr(), M, K, K, 1.0, rows.data_ptr(), scale.data_ptr(), s)),
                               M * (2 * K + K // 2 + 2))}
        for name, (run, nbytes) in forms.items():
            for _ in range(2):
                run()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            for _ in range(repeats):
                run()
            b.record(stream)
            torch.cuda.synchronize()
            out[name][str(K)] = round(nbytes / (a.elapsed_time(b) / repeats) / 1e6, 1)
        del x, scale, blocks, rows
        torch.cuda.empty_cache()
    return out


def mfma_ceiling(torch, lib, dev, ms_target=30.0, repeats=3):
    """TOP/s of the MFMA-only loop per instruction and operand data, HIP events around each launch."""
    import ctypes

    import numpy as np

    from dsaquant_amd import _lib

    stream = torch.cuda.current_stream(dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    out = torch.empty(cus * 512, dtype=torch.int32, device=dev)
    rng = np.random.default_rng(0)
    res = {"workgroups": cus, "waves_per_workgroup": 8, "mfma_per_wave_and_iteration": 16}
    for kind, code, datas in (("int8", 0, ("zeros", "int4", "workload", "bytes")), ("bf6", 1, ("zeros", "int4", "workload"))):
        res[kind] = {}
        for data in datas:
            ops = ctypes.c_double()
            operands = torch.from_numpy(probe_operands(np, kind, data, rng)).to(dev)
            assert operands.numel() == lib.vdmq_mfma_probe_operand_bytes()

            def launch(iters):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(stream)
                _lib.check(lib.vdmq_mfma_probe(code, operands.data_ptr(), iters, cus, out.data_ptr(), ctypes.byref(ops), stream.cuda_stream))
                b.record(stream)
                torch.cuda.synchronize()
                return a.elapsed_time(b)

            iters = 2000
            ms = launch(iters)
            iters = max(2000, int(iters * ms_target / max(ms, 1e-3)))
            times = [launch(iters) for _ in range(repeats)]
            res[kind][data] = {"tops": round(ops.value / (statistics.median(times) * 1e-3) / 1e12, 1), "ms": round(statistics.median(times), 3)}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="wan14b_720p_block", choices=sorted(WORKLOADS))
    ap.add_argument("--matrix-path", default="auto", choices=["auto", "int8", "bf6"],
                    help="matrix instructions of the GEMM: auto = what the library picks for the shape")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the int8-path run, the other workloads, the single-linear cases, the config-4 harness and the MFMA probe")
    ap.add_argument("--no-config4", action="store_true", help="skip the end-to-end DiT harness (about 15 s)")
    ap.add_argument("--per-linear", action="store_true", help="add the per-launch table of every workload to the line")
    ap.add_argument("--details", action="store_true",
                    help="add the full objects behind the flat figures of `roofline` (int8_path, workloads, cases, stream_ceiling, "
                         "mfma_ceiling, config4); without it the line stays short")
    ap.add_argument("--ubench", action="store_true", help="only the MFMA-only probe, 200 ms per case (for counter collection)")
    ap.add_argument("--stream-probe", action="store_true",
                    help="only the streaming probe (reads and writes in the quantizer's proportion, nothing else) over the byte volumes "
                         "of the workload's quantizer launches, then the quantizers themselves on the same volumes (for counter collection)")
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

    if args.ubench:
        print(json.dumps({"metric": "MFMA-only loop, TOP/s", "unit": "TOP/s", "peaks": {"int8": INT8_PEAK_TOPS, "bf6": FP6_PEAK_TOPS},
                          "mfma_ceiling": mfma_ceiling(torch, lib, dev, ms_target=200.0, repeats=3)}))
        return

    if args.stream_probe:
        wl = WORKLOADS[args.workload]
        Ks = sorted({k for _, k, _ in wl["linears"]})
        print(json.dumps({"metric": "streaming probe, GB/s of bytes read + written", "unit": "GB/s", "peak": HBM_PEAK_GBS,
                          "workload": args.workload, "M": wl["M"], "row_lengths": Ks,
                          "bf6_blocks": stream_ceiling(torch, lib, dev, wl["M"], Ks, True, repeats=20),
                          "int4_rows": stream_ceiling(torch, lib, dev, wl["M"], Ks, False, repeats=20),
                          "quantizers_gbs_by_row_length": quantizers_alone(torch, lib, dev, wl["M"], Ks)}))
        return

    if args.calibrate_copy:
        # the library's plain 128-bit copy kernel: reads 1 GiB, writes 1 GiB
        src = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(lib.vdmq_copy_u128(src.data_ptr(), dst.data_ptr(), src.numel(), torch.cuda.current_stream(dev).cuda_stream))
        torch.cuda.synchronize()
        del src, dst

    def run(name, path, steps, warmup):
        w = Workload(torch, lib, v, name, path, dev)
        r = w.measure(steps, warmup)
        del w
        torch.cuda.empty_cache()
        return r

    wl = WORKLOADS[args.workload]
    r = run(args.workload, args.matrix_path, args.steps, args.warmup)
    path = r["path"]
    roof = r["roofline"]
    # the quantizer's figures next to the GEMM's, where a reader of the roofline object finds them
    roof.update({"quantizer_achieved_gbs": r["quantizer"]["achieved"], "quantizer_frac": r["quantizer"]["frac"],
                 "quantizer_achieved_gbs_int4_bytes": r["quantizer"]["achieved_int4_bytes"],
                 "quantizer_frac_int4_bytes": r["quantizer"]["frac_int4_bytes"], "quantizer_peak_gbs": HBM_PEAK_GBS})
    result = {
        "metric": "W4A4 GEMM TOPS (% INT8-MFMA peak) at Wan-14B 720p shapes; A4-quant GB/s",
        "value": round(r["step_tops"], 1), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("int4 x int4 -> int32 (int8 MFMA), fp16 in/out" if path == "int8" else
                  "int4 x int4 as exact E3M2 floats (q / 16) -> fp32 accumulator holding the exact integer / 256 (FP6 MFMA), fp16 in/out"),
        "data": "synthetic", "matrix_path": path,
        "config": {"workload": f"{args.workload}: M={wl['M']} tokens, linears " + ", ".join(f"{n} {k}->{o}" for n, k, o in wl["linears"])
                               + "; each = A4 quantizer + W4A4 GEMM + scale/bias epilogue, clip 1.0"},
        "roofline": roof, "quantizer": r["quantizer"],
    }
    per_linear = {args.workload: r["per_linear"]}
    if not args.no_extras:
        extra_steps, extra_warmup = max(10, args.steps // 4), 3

        # The measurements beside the headline: each in a section of its own, so that a failure in one (out of memory on a
        # smaller part, a missing package for the harness) is named in the line instead of costing the line.  The
        # headline above is not guarded: without it there is nothing to report.
        def section(name, body):
            try:
                body()
            except Exception as e:  # noqa: BLE001 -- reported, not swallowed
                roof[f"{name}_error"] = f"{type(e).__name__}: {e}"[:300]
                print(f"bench.py: section {name} failed: {e!r}", file=sys.stderr)

        def int8_section():  # the instruction the path was specified on: the same workload on the int8 matrix path
            r8 = run(args.workload, "int8", extra_steps, extra_warmup)
            result["int8_path"] = {"steps": extra_steps, "warmup": extra_warmup, "step_tops": round(r8["step_tops"], 1),
                                   "ms_per_step": round(r8["ms_per_step"], 4), "roofline": r8["roofline"], "quantizer": r8["quantizer"]}
            per_linear[args.workload + " (int8 path)"] = r8["per_linear"]
            roof.update({"int8_path_achieved": r8["roofline"]["achieved"], "int8_path_peak": INT8_PEAK_TOPS,
                         "int8_path_frac": r8["roofline"]["frac"], "int8_path_kernel": r8["roofline"]["kernel"],
                         "int8_path_quantizer_frac": r8["quantizer"]["frac"], "int8_path_step_tops": round(r8["step_tops"], 1)})

        def workload_section(other):
            ro = run(other, args.matrix_path, extra_steps, extra_warmup)
            result.setdefault("workloads", {})[other] = {
                "M": WORKLOADS[other]["M"], "steps": extra_steps, "warmup": extra_warmup,
                "step_tops": round(ro["step_tops"], 1), "ms_per_step": round(ro["ms_per_step"], 4),
                "gemm_tops": ro["roofline"]["achieved"], "gemm_frac": ro["roofline"]["frac"],
                "gemm_frac_of_int8_peak": ro["roofline"]["frac_of_int8_peak"],
                "quant_gbs": ro["quantizer"]["achieved"], "quant_gbs_int4_bytes": ro["quantizer"]["achieved_int4_bytes"]}
            per_linear[other] = ro["per_linear"]
            k = SHORT[other]
            roof.update({f"{k}_gemm_achieved": ro["roofline"]["achieved"], f"{k}_gemm_frac": ro["roofline"]["frac"],
                         f"{k}_gemm_frac_of_int8_peak": ro["roofline"]["frac_of_int8_peak"], f"{k}_step_tops": round(ro["step_tops"], 1),
                         f"{k}_quantizer_frac_int4_bytes": ro["quantizer"]["frac_int4_bytes"]})

        def case_section(case, spec):  # single linears: launches of 15 ... 2400 us, so more repetitions for the short ones
            steps_c = 200 if spec["M"] <= 4096 else extra_steps
            rc = run(case, args.matrix_path, steps_c, 5)
            lin = next(iter(rc["per_linear"].values()))
            result.setdefault("cases", {})[case] = {
                "M": spec["M"], "K": lin["K"], "N": lin["N"], "steps": steps_c, "kernel": lin["kernel"],
                "gemm_us": round(lin["gemm_ms"] * 1e3, 2), "gemm_tops": lin["gemm_tops"],
                "quant_us": round(lin["quant_ms"] * 1e3, 2), "quant_gbs_int4_bytes": lin["quant_gbs_int4_bytes"],
                "linear_tops": round(rc["step_tops"], 1), "linear_us": round(rc["ms_per_step"] * 1e3, 2)}
            roof.update({f"{case}_gemm_achieved": lin["gemm_tops"], f"{case}_gemm_frac": round(lin["gemm_tops"] / rc["roofline"]["peak"], 4),
                         f"{case}_linear_tops": round(rc["step_tops"], 1), f"{case}_kernel": lin["kernel"]})

        def stream_section():  # the quantizer against a kernel that only streams the same mix of reads and writes over the same volumes
            sc = stream_ceiling(torch, lib, dev, wl["M"], [k for _, k, _ in wl["linears"]], path != "int8")
            result["stream_ceiling"] = sc
            roof.update({"quantizer_stream_ceiling_gbs": sc["gbs"], "quantizer_stream_mix": sc["mix"],
                         "quantizer_frac_of_stream_ceiling": round(r["quantizer"]["achieved"] / sc["gbs"], 4),
                         "stream_copy_gbs": sc["copy_gbs"], "stream_read_only_gbs": sc["read_only_gbs"]})

        def mfma_section():
            ceiling = mfma_ceiling(torch, lib, dev)
            result["mfma_ceiling"] = ceiling
            roof.update({"mfma_only_loop_bf6_workload_data": ceiling["bf6"]["workload"]["tops"],
                         "mfma_only_loop_int8_workload_data": ceiling["int8"]["workload"]["tops"]})

        def config4_section():
            import contextlib

            import bench_dit

            with contextlib.redirect_stdout(sys.stderr):  # (the loader reports what it loaded; this program prints one line)
                c4 = bench_dit.measure(torch, steps=5, warmup_steps=1, fuse_ln=True, fuse_gelu=True, fuse_residual=True, reuse_context=True)
                c4_plain = bench_dit.measure(torch, steps=2, warmup_steps=0)
            result["config4"] = {"workload": "Wan-2.1 1.3B DiT, 30 blocks, 32760 tokens, cond + uncond, 5 steps after 1 warm-up step; LayerNorm, GELU and "
                                             "residual updates fused into the W4A4 kernels, context quantized once",
                                 "ms_per_step": c4["ms_per_step"], "w4a4_share": c4["value"], "attention_share": c4["attention_share"],
                                 "w4a4_ms_per_forward": c4["w4a4_ms_per_forward"], "attention_ms_per_forward": c4["attention_ms_per_forward"],
                                 "w4a4_calls_per_forward": c4["w4a4_calls_per_forward"], "forwards": c4["forwards"],
                                 "unfused": {"steps": 2, "ms_per_step": c4_plain["ms_per_step"], "w4a4_share": c4_plain["value"],
                                             "w4a4_ms_per_forward": c4_plain["w4a4_ms_per_forward"],
                                             "w4a4_calls_per_forward": c4_plain["w4a4_calls_per_forward"]}}
            roof.update({"config4_ms_per_step": c4["ms_per_step"], "config4_w4a4_share": c4["value"], "config4_attention_share": c4["attention_share"],
                         "config4_w4a4_calls_per_forward": c4["w4a4_calls_per_forward"], "config4_unfused_ms_per_step": c4_plain["ms_per_step"],
                         "config4_unfused_w4a4_share": c4_plain["value"]})

        if path != "int8":
            section("int8_path", int8_section)
        for other in sorted(WORKLOADS):
            if other != args.workload:
                section(SHORT[other], lambda other=other: workload_section(other))
        for case, spec in CASES.items():
            section(case, lambda case=case, spec=spec: case_section(case, spec))
        section("stream_ceiling", stream_section)
        section("mfma_only_loop", mfma_section)
        if not args.no_config4:
            section("config4", config4_section)
    if not args.details:  # every figure of these objects that matters is a flat key of `roofline`
        for key in ("int8_path", "workloads", "cases", "stream_ceiling", "mfma_ceiling", "config4"):
            result.pop(key, None)
    if args.per_linear:
        result["per_linear"] = per_linear
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
