#!/usr/bin/env python3
"""Benchmark of the MixedQLinear forward path on one MI355X.

A step is one forward of the layer: the per-token asymmetric quantize kernel followed by the
fused GEMM kernel (int4 x int4 + fp16 outlier GEMM + dequantize epilogue), on synthetic inputs
already resident in HBM.  W4A4 layers with more than 32 token rows take the path MixedQLinear takes:
the int4 products run on the 6-bit (E2M3) matrix-core instructions, exactly (--int8-mfma forces the
int8 MFMA path, which has the same output bits).  The default workload is the one the headline
metric is quoted on: Llama-2-70B gate_proj, 8192 -> 28672, 2048 tokens, 256 fp16 outlier
columns, W4A4 asymmetric activations.

Prints ONE JSON line.  value = 2*M*N*K / t_step in TOPS (the integer GEMM's operations over the
whole forward time; the outlier GEMM's 2*M*N*F flops are not counted).  `roofline` is for the
dominant kernel (the fused GEMM, priced against the peak of the MFMA instructions it issues: 10.1 POP/s
for the 6-bit path, 5.0 POP/s for int8; for the workloads of at most 32 token rows the weight-streaming
kernel, priced against the HBM peak); `roofline_quantize` for the
quantize kernel (bounded by HBM).  Kernel durations are measured with HIP events recorded on
the stream the kernels run on, inside the timed region.  `cpu_baseline` times the CPU
restatement of the reference's fake-quant path (oracle/sim_path.py) on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (tokens M, in_features, out_features N, outliers F, bits)
    "llama2-70b.gate_proj": (2048, 8192, 28672, 256, 4),
    "llama2-70b.q_proj": (2048, 8192, 8192, 256, 4),
    "llama2-70b.k_proj": (2048, 8192, 1024, 256, 4),
    "llama2-70b.qkv_fused": (2048, 8192, 10240, 256, 4),       # q + k + v as one GEMM (FusedMixedQLinearGroup)
    "llama2-70b.down_proj.int8": (2048, 28672, 8192, 256, 8),
    "llama2-7b.gate_proj": (2048, 4096, 11008, 256, 4),
    "llama2-7b.q_proj": (2048, 4096, 4096, 256, 4),
    "llama2-7b.down_proj.int8": (2048, 11008, 4096, 256, 8),
    "config1": (512, 4096, 4096, 128, 4),
    "llama2-13b.gate_proj": (2048, 5120, 13824, 256, 4),
    "llama2-13b.gate_proj.t128": (128, 5120, 13824, 256, 4),
    "llama2-13b.gate_proj.t16": (16, 5120, 13824, 256, 4),
    "llama2-13b.gate_proj.t1": (1, 5120, 13824, 256, 4),
    "llama2-13b.gate_proj.t2": (2, 5120, 13824, 256, 4),
    "llama2-13b.gate_proj.t4": (4, 5120, 13824, 256, 4),
    "llama2-70b.gate_proj.t1": (1, 8192, 28672, 256, 4),
    "llama2-70b.down_proj.int8.t1": (1, 28672, 8192, 256, 8),
    "llama2-13b.down_proj.int8.t16": (16, 13824, 5120, 256, 8),
    "llama2-70b.gate_proj.t64": (64, 8192, 28672, 256, 4),
    "llama2-70b.gate_proj.t32": (32, 8192, 28672, 256, 4),          # weight-streaming kernel, token rows in LDS
    "llama2-70b.down_proj.int8.t64": (64, 28672, 8192, 256, 8),     # 64 tiles, K = 28416: split over K
}

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, published
PEAK_FP6_TOPS = 10100.0   # MI355X dense fp6 / fp4 MFMA, published
PEAK_HBM_GBPS = 8000.0    # MI355X HBM3E, published

# HBM/fabric bytes per launch from rocprofv3 counter runs of this file (FETCH_SIZE and WRITE_SIZE, each
# scaled by what the same counter reads for a plain 256 MiB copy).  OFFLINE figures: they come from the profiler
# summaries named beside them, not from the run that prints them, and are labelled so in the JSON line
# (`traffic_source`).  (gemm6 / quantize6: the kernels of the 6-bit matrix-core path, the default; gemm / quantize:
# --int8-mfma)
MEASURED_TRAFFIC_BYTES = {
    "llama2-70b.gate_proj": {"gemm": 809.4e6, "quantize": 43.0e6, "gemm6": 754.7e6, "quantize6": 47.1e6},
}
TRAFFIC_SOURCE = {
    "gemm6": "offline: profiles/gemm_fused6_split_kernel__llama2-70b.gate_proj.md (rocprofv3 --pmc FETCH_SIZE / "
             "WRITE_SIZE, scaled by profiles/copy_calibration__256MiB.md)",
    "quantize6": "offline: profiles/quantize_fp6_wave_kernel__llama2-70b.gate_proj.md",
    "gemm": "offline: profiles/gemm_fused_split_kernel__llama2-70b.gate_proj.md",
    "quantize": "offline: profiles/asym_quantize_stream_kernel__llama2-70b.gate_proj.md",
}


def make_layer(name, device, seed=0):
    import torch

    from quik_amd.qlinear import MixedQLinear
    M, n_in, N, F, bits = WORKLOADS[name]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, n_in, generator=g)
    fp_idx = torch.randperm(n_in, generator=g)[:F]
    x[:, fp_idx] *= 50
    x = x.half()
    K = n_in - F
    lo, hi = (-8, 8) if bits == 4 else (-127, 128)
    s_w = (torch.rand(N, 1, generator=g) * 0.009 + 0.001).half()
    int_idx = torch.arange(n_in)
    int_idx = int_idx[~torch.isin(int_idx, fp_idx)]
    W = torch.empty(N, n_in, dtype=torch.float16)
    # fill in column blocks to bound host memory
    for s in range(0, N, 4096):
        e = min(N, s + 4096)
        codes = torch.randint(lo, hi, (e - s, K), generator=g).float()
        W[s:e, int_idx] = (codes * s_w[s:e].float()).half()
        W[s:e, fp_idx] = (0.02 * torch.randn(e - s, F, generator=g)).half()
    lin = torch.nn.Linear(n_in, N, bias=False, dtype=torch.float16, device="meta")
    mod = MixedQLinear.from_float(lin, W, s_w, None, fp_idx, bits=bits).to(device)
    return mod, x, W, int_idx, fp_idx


def verify_spot_tile(name, out, x_cpu, W_cpu, fp_idx, mod, rows=48, cols=64):
    """Three spot tiles of the layer output (first, middle straddling a tile boundary, last) against the CPU oracle's
    MixedQLinear forward (oracle/quik_oracle.py), tolerance 1e-2 x output RMS: the check of the exact configuration
    that is timed.  Runs once, before the warm-up; returns the largest error relative to the RMS."""
    import numpy as np

    from oracle import quik_oracle as qo
    M, n_in, N, F, bits = WORKLOADS[name]
    th, tw = min(rows, M), min(cols, N)
    mid_c = min(N - tw, (N // 2 // 256) * 256 + 200)
    worst = 0.0
    for r0, c0 in ((0, 0), ((M - th) // 2, mid_c), (M - th, N - tw)):
        r, c = slice(r0, r0 + th), slice(c0, c0 + tw)
        omod = qo.from_float(W_cpu[c].numpy(), mod.weights_scales[c].cpu().numpy(), fp_idx.numpy(), bits)
        want, _ = qo.mixed_qlinear_forward(x_cpu[r].numpy(), omod, bits)
        got = out[r, c].float().cpu().numpy().astype(np.float64)
        w64 = want.astype(np.float64)
        rel = float(np.abs(got - w64).max() / np.sqrt((w64 ** 2).mean()))
        assert rel <= 1e-2, f"bench.py: output differs from the oracle on tile ({r0}, {c0}): {rel:.3e} x RMS"
        worst = max(worst, rel)
    return worst


def spread(block_ms, int_ops):
    """Per-step times of the timed blocks (the first one is the block `value` comes from) -> median, mean and
    1.96 sigma (the reference's confidence interval, experiments/layer_benchmark.py:29-31), in ms and TOPS."""
    import statistics
    n = len(block_ms)
    mean = sum(block_ms) / n
    sd = statistics.stdev(block_ms) if n > 1 else 0.0
    med = statistics.median(block_ms)
    tops = lambda ms: round(int_ops / (ms * 1e-3) / 1e12, 1)
    return {"blocks": n, "ms_per_step_each": [round(b, 4) for b in block_ms], "median_ms": round(med, 4),
            "mean_ms": round(mean, 4), "ci95_ms": round(1.96 * sd, 4), "median_tops": tops(med), "mean_tops": tops(mean),
            "pct_int8_mfma_peak_median": round(100.0 * int_ops / (med * 1e-3) / 1e12 / PEAK_INT8_TOPS, 2)}


def cpu_baseline(name, x, W, int_idx, fp_idx, budget_s=25.0):
    """CPU restatement of the reference's simulated path on the host cores (oracle/sim_path.py)."""
    import torch

    from oracle import sim_path
    M, n_in, N, F, bits = WORKLOADS[name]
    K = n_in - F
    cores = torch.get_num_threads()
    times = []
    t_all = time.perf_counter()
    w32 = W.float()                                                             # widened once, not timed
    sim_path.sim_mixed_linear(x[:64], W[:256], int_idx, fp_idx, bits)          # warm the BLAS threads
    while len(times) < 5 and (time.perf_counter() - t_all) < budget_s:
        t0 = time.perf_counter()
        sim_path.sim_mixed_linear(x, W, int_idx, fp_idx, bits, weight_f32=w32)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": 2.0 * M * N * K / med / 1e12, "unit": "TOPS", "cores": cores, "kind": "port",
            "sample": f"full layer {name} (M={M}, in={n_in}, N={N}), median of {len(times)} runs, "
                      f"{med * 1e3:.0f} ms each, torch CPU fp32 compute on fp16 storage",
            "ms_per_step": med * 1e3}


# ---------------------------------------------------------------------------------------------------
# Full decoder block at Llama-2-70B dims (hidden 8192, 64 heads, 8 KV heads, MLP 28672): the seven
# linears are MixedQLinear (q/k/v/o/gate/up W4A4, down_proj W8A8, 256 fp16 outlier columns each, q/k/v and
# gate/up sharing their quantized input as experiments/llama.py:394-440 sets them up); RMSNorm, rotary-free
# attention (torch SDPA, causal for prefill) and SiLU stay in PyTorch.  Random-init weights made on the device.
BLOCK_WORKLOADS = {
    # name: (batch, new tokens per sequence, tokens already in the KV cache)
    "llama2-70b.decoder_block.prefill": (16, 512, 0),
    "llama2-70b.decoder_block.decode": (64, 1, 512),
    "llama2-70b.decoder_block.decode1": (1, 1, 512),     # single-stream decode: every linear is one launch
}
BLOCK_DIMS = dict(hidden=8192, heads=64, kv_heads=8, head_dim=128, mlp=28672, F=256)


def make_device_layer(n_in, N, F, bits, fp_idx, shared, gen, device):
    """A MixedQLinear with random codes and scales written straight into its buffers on the device (what
    from_float would store for W = codes * scale; the distributions of make_layer)."""
    import torch

    from quik_amd.qlinear import MixedQLinear, pack_to_i4
    K = n_in - F
    mod = MixedQLinear(n_in, N, shared, fp_features_num=F, symm=False, bits=bits, dtype=torch.float16).to(device)
    lo, hi = (-8, 8) if bits == 4 else (-127, 128)
    s_w = (torch.rand(N, 1, generator=gen, device=device) * 0.009 + 0.001).half()
    int_idx = torch.arange(n_in, device=device)
    int_idx = int_idx[~torch.isin(int_idx, fp_idx)]
    red = torch.empty(N, dtype=torch.float32, device=device)
    for s in range(0, N, 4096):
        e = min(N, s + 4096)
        codes = torch.randint(lo, hi, (e - s, K), generator=gen, device=device, dtype=torch.int8)
        mod.int_weight[s:e] = pack_to_i4(codes) if bits == 4 else codes
        red[s:e] = (codes.float() * s_w[s:e].float()).half().float().sum(1)
    mod.weights_scales.copy_(s_w)
    mod.reduced_w.copy_(red.half().reshape(1, N))
    mod.fp_weight.copy_((0.02 * torch.randn(N, F, generator=gen, device=device)).half())
    mod.int_indices.copy_(int_idx)
    mod.fp_indices.copy_(fp_idx)
    mod.bias = None
    return mod


class DecoderBlock:
    """One Llama-2-70B-sized decoder block whose seven linears are MixedQLinear (q/k/v/o/gate/up W4A4, down_proj
    W8A8, 256 fp16 outlier columns each; q/k/v and gate/up share their quantized input as experiments/llama.py:394-440
    sets them up).  The same weights also exist as two fused groups (one quantize and ONE GEMM for q/k/v and for
    gate/up).  RMSNorm, attention (torch SDPA, causal for prefill, no rotary embedding) and SiLU stay in PyTorch.
    `hook(name, module, x, out)`, when given, is called after every linear with the tensors it consumed and produced."""

    def __init__(self, dev, dims=None, seed=0):
        import copy

        import torch

        from quik_amd.qlinear import FusedMixedQLinearGroup, SharedQuantizedInput
        d = dict(BLOCK_DIMS if dims is None else dims)
        self.dims, self.dev = d, dev
        H, heads, kvh, hd, mlp, F = d["hidden"], d["heads"], d["kv_heads"], d["head_dim"], d["mlp"], d["F"]
        gen = torch.Generator(device=dev).manual_seed(seed)
        self.gen = gen
        self.fp_h = torch.randperm(H, generator=gen, device=dev)[:F]
        self.fp_m = torch.randperm(mlp, generator=gen, device=dev)[:F]
        sh_qkv, sh_mlp = SharedQuantizedInput(3), SharedQuantizedInput(2)
        self.L = {
            "q": make_device_layer(H, heads * hd, F, 4, self.fp_h, sh_qkv, gen, dev),
            "k": make_device_layer(H, kvh * hd, F, 4, self.fp_h, sh_qkv, gen, dev),
            "v": make_device_layer(H, kvh * hd, F, 4, self.fp_h, sh_qkv, gen, dev),
            "o": make_device_layer(heads * hd, H, F, 4, self.fp_h, None, gen, dev),
            "gate": make_device_layer(H, mlp, F, 4, self.fp_h, sh_mlp, gen, dev),
            "up": make_device_layer(H, mlp, F, 4, self.fp_h, sh_mlp, gen, dev),
            "down": make_device_layer(mlp, H, F, 8, self.fp_m, None, gen, dev),
        }
        members = {n: copy.copy(self.L[n]) for n in ("q", "k", "v", "gate", "up")}
        for m in members.values():
            m.shared_input = None
        self.g_qkv = FusedMixedQLinearGroup([members["q"], members["k"], members["v"]])
        self.g_mlp = FusedMixedQLinearGroup([members["gate"], members["up"]])
        self.norm1 = torch.ones(H, dtype=torch.float16, device=dev)
        self.norm2 = torch.ones(H, dtype=torch.float16, device=dev)

    def inputs(self, B, S, past):
        """Hidden states with the outlier columns scaled up, and a KV cache of `past` tokens (or None)."""
        import torch
        d, dev, gen = self.dims, self.dev, self.gen
        x = torch.randn(B, S, d["hidden"], generator=gen, device=dev)
        x[..., self.fp_h] *= 50
        cache = None
        if past:
            cache = tuple(torch.randn(B, d["kv_heads"], past, d["head_dim"], generator=gen, device=dev).half()
                          for _ in range(2))
        return x.half(), cache

    @staticmethod
    def rmsnorm(t, w):
        import torch
        v = t.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5)).half() * w

    def attention(self, q, k, v, cache):
        import torch
        import torch.nn.functional as Fn
        d = self.dims
        B, S = q.shape[:2]
        heads, kvh, hd = d["heads"], d["kv_heads"], d["head_dim"]
        q = q.view(B, S, heads, hd).transpose(1, 2)
        k = k.view(B, S, kvh, hd).transpose(1, 2)
        v = v.view(B, S, kvh, hd).transpose(1, 2)
        if cache is not None:
            k, v = torch.cat([cache[0], k], 2), torch.cat([cache[1], v], 2)
        k = k.repeat_interleave(heads // kvh, 1)
        v = v.repeat_interleave(heads // kvh, 1)
        o = Fn.scaled_dot_product_attention(q, k, v, is_causal=(cache is None and S > 1))
        return o.transpose(1, 2).reshape(B, S, heads * hd)

    def forward(self, t, fused_groups, cache=None, hook=None):
        import torch.nn.functional as Fn

        def lin(name, x):
            out = self.L[name](x)
            if hook is not None:
                hook(name, self.L[name], x, out)
            return out

        h = self.rmsnorm(t, self.norm1)
        if fused_groups:
            q, k, v = self.g_qkv(h)
        else:
            q, k, v = lin("q", h), lin("k", h), lin("v", h)
        t = t + lin("o", self.attention(q, k, v, cache))
        h = self.rmsnorm(t, self.norm2)
        if fused_groups:
            g, u = self.g_mlp(h)
        else:
            g, u = lin("gate", h), lin("up", h)
        return t + lin("down", Fn.silu(g) * u)


def bench_block(args):
    import torch

    dev = torch.device("cuda:0")
    B, S, past = BLOCK_WORKLOADS[args.workload]
    blk = DecoderBlock(dev)
    d, L, gen = blk.dims, blk.L, blk.gen
    heads, hd, mlp = d["heads"], d["head_dim"], d["mlp"]
    x, cache = blk.inputs(B, S, past)

    # inputs of realistic scale for timing the seven linears alone
    h_in = blk.rmsnorm(x, blk.norm1)
    a_in = torch.randn(B, S, heads * hd, generator=gen, device=dev).half()
    m_in = torch.randn(B, S, mlp, generator=gen, device=dev)
    m_in[..., blk.fp_m] *= 50
    m_in = m_in.half()

    def linears(fused_groups):
        if fused_groups:
            blk.g_qkv(h_in)
        else:
            L["q"](h_in), L["k"](h_in), L["v"](h_in)
        L["o"](a_in)
        if fused_groups:
            blk.g_mlp(h_in)
        else:
            L["gate"](h_in), L["up"](h_in)
        L["down"](m_in)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    out = blk.forward(x, False, cache)
    out_f = blk.forward(x, True, cache)
    assert torch.isfinite(out).all() and torch.equal(out, out_f)       # the fused groups give the same bits
    block_ms = timed(lambda: blk.forward(x, False, cache))
    block_f_ms = timed(lambda: blk.forward(x, True, cache))
    lin_ms = timed(lambda: linears(False))
    lin_f_ms = timed(lambda: linears(True))
    # the linears of the block (fused groups) replayed from a HIP graph: what a serving loop that captures the
    # layer sees; every replay is checked against the eager outputs
    lin_graph_ms = None
    try:
        outs = {}

        def linears_out():
            outs["qkv"] = blk.g_qkv(h_in)
            outs["o"] = L["o"](a_in)
            outs["mlp"] = blk.g_mlp(h_in)
            outs["down"] = L["down"](m_in)

        linears_out()
        want = {k: [t.clone() for t in (v if isinstance(v, (tuple, list)) else [v])] for k, v in outs.items()}
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            linears_out()
        torch.cuda.current_stream().wait_stream(side)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            linears_out()
        for _ in range(3):
            g.replay()
            torch.cuda.synchronize()
            for k, v in outs.items():
                for t, w in zip(v if isinstance(v, (tuple, list)) else [v], want[k]):
                    assert torch.equal(t, w), f"graph replay of {k} differs from the eager result"
        for _ in range(max(20, args.warmup)):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        lin_graph_ms = e0.elapsed_time(e1) / args.steps
    except Exception as exc:   # noqa: BLE001  (an extra figure)
        print(f"bench.py: graph replay of the linears skipped: {exc}", file=sys.stderr)
    M = B * S
    ops = sum(2.0 * M * m.out_features * m.int_features_num for m in L.values())
    weight_bytes = sum(m.out_features * (m.int_features_num * m.bits // 8 + m.fp_features_num * 2) for m in L.values())
    res = {
        "metric": "decoder block latency, Llama-2-70B dims, 7 MixedQLinear + PyTorch norm/attention, 1 GPU",
        "value": round(block_f_ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(block_f_ms, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 / int8 (down_proj) codes, fp16 activations", "data": "synthetic",
        "config": {"workload": f"{args.workload}: batch {B} x {S} new tokens, {past} cached; q/k/v and gate/up as "
                               f"one GEMM each (FusedMixedQLinearGroup)", "tokens": M, **d},
        "block_ms_seven_modules_shared_input": round(block_ms, 4),
        "linears_only_ms": {"seven_modules_shared_input": round(lin_ms, 4), "fused_groups": round(lin_f_ms, 4),
                            "fused_groups_graph_replay": None if lin_graph_ms is None else round(lin_graph_ms, 4)},
        "linears_weight_bytes_reference_layout": weight_bytes,
        "linears_weight_stream_gbps": round(weight_bytes / (min(lin_graph_ms or lin_f_ms, lin_f_ms) * 1e-3) / 1e9, 1),
        "linears_int_tops": round(ops / (lin_f_ms * 1e-3) / 1e12, 1),
        "linears_pct_int8_mfma_peak": round(100.0 * ops / (lin_f_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS, 2),
    }
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="llama2-70b.gate_proj", choices=sorted(WORKLOADS) + sorted(BLOCK_WORKLOADS))
    ap.add_argument("--repeats", type=int, default=5,
                    help="further timed blocks of --steps forwards each, run after the block that gives `value` "
                         "(the reference's protocol repeats its timed block and reports mean +- 1.96 sigma, "
                         "experiments/layer_benchmark.py:19-31); their spread is printed as `repeats` (0: none)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--event-every", type=int, default=1,
                    help="record the HIP events that time the two kernels on every N-th timed step (default: every step)")
    ap.add_argument("--no-verify", action="store_true", help="skip the spot check of the output against the CPU oracle")
    ap.add_argument("--unfused", action="store_true", help="run the reference's three-op sequence instead")
    ap.add_argument("--int8-mfma", action="store_true",
                    help="row-major operands on the int8 MFMA kernels instead of the tile-ordered paths (same output bits)")
    ap.add_argument("--cold-weights", action="store_true",
                    help="extra figure cold_ms_per_forward: the forward of the layer rotating over enough copies of "
                         "its weights (>= 700 MB) that none of them stays in the 256 MB Infinity Cache, as in a model "
                         "with many layers; one HIP graph over all copies, replayed")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only plain device-to-device copies of a 256 MiB buffer (known traffic: 256 MiB read, "
                         "256 MiB written per launch) to scale the FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only; run with --gpus 1 (no multi-GPU path exists)",
              file=sys.stderr)
        sys.exit(2)

    import torch

    from quik_amd import _lib
    _lib.load()  # fails loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        src = torch.randn(128 * 1024 * 1024, device=dev).half()       # 256 MiB
        dst = torch.empty_like(src)
        for _ in range(max(args.steps, 1)):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": True, "bytes_read_per_launch": src.numel() * 2,
                          "bytes_written_per_launch": src.numel() * 2, "launches": max(args.steps, 1)}))
        return

    if args.workload in BLOCK_WORKLOADS:
        bench_block(args)
        return

    name = args.workload
    M, n_in, N, F, bits = WORKLOADS[name]
    K = n_in - F
    mod, x_cpu, W_cpu, int_idx, fp_idx = make_layer(name, dev)
    mod.fused = not args.unfused
    x = x_cpu.to(dev)

    from quik_amd import asymmetric, matmul
    colmap = mod._column_map()
    # the path MixedQLinear.forward takes: tile-ordered operands (4 bits: 6-bit matrix-core GEMM, 8 bits: int8 MFMA)
    if args.int8_mfma:
        mod.six_bit_path = False          # row-major operands on the int8 MFMA kernels
    six = mod._six_bit_ok(M)
    quantize6 = asymmetric.quantize_mapped_fp6 if bits == 4 else asymmetric.quantize_mapped_tile8

    def quantize_only():
        if six:
            return quantize6(x, colmap, K, F)
        return asymmetric.quantize_mapped(x, colmap, K, F, bits)

    def step(ev=None, before=True):
        """One forward of the layer.  Fused (the default): ONE call of the module, mod(x) -> quik_layer_forward, which
        launches the quantize kernel and the fused GEMM.  --unfused: the reference's op sequence through the stand-alone
        ops.  ev = (before, between, after): events on the launch stream; in the fused form the library records the
        middle one between its two launches.  before=False: the step in front of this one recorded its `after` event,
        which then serves as this step's `before` (one event record per step less)."""
        if ev is not None and before:
            ev[0].record()
        if mod.fused:
            if ev is not None:
                mod.mid_event = ev[1]
            out = mod(x)[0]
            if ev is not None:
                assert mod.mid_event is None, "the forward did not go through the one-call path"
                ev[2].record()
            return out
        q, meta, fp = asymmetric.quantize_mapped(x, colmap, K, F, bits)
        if ev is not None:
            ev[1].record()
        from quik_amd.qlinear import SharedQuantizedInput
        sh = SharedQuantizedInput(1)
        sh.qint_x, sh.meta, sh.fp_x = q, meta, fp
        out = mod._forward_unfused(sh)
        if ev is not None:
            ev[2].record()
        return out

    # One spot tile of what the timed step computes, against the CPU oracle, outside the timed region.
    spot = None if (args.no_verify or args.unfused) else verify_spot_tile(name, step(), x_cpu, W_cpu, fp_idx, mod)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # Kernel durations from HIP events inside the timed region: between the two launches (recorded by the library) and
    # after the forward; the event after one forward is the event before the next.  An event record between two
    # launches costs 3 - 4 us on the GPU's timeline, which ms_per_step includes (--event-every N records them on
    # every N-th step only).
    every = max(1, args.event_every)
    events = {i: [torch.cuda.Event(enable_timing=True) for _ in range(3)] for i in range(0, args.steps, every)}
    for evs in events.values():        # an event has a handle only once it has been recorded
        for e in evs:
            e.record()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(events.get(i), before=(i - 1) not in events)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_step = (t1 - t0) * 1e3 / args.steps
    q_ms = sorted((events[i - 1][2] if (i - 1) in events else e[0]).elapsed_time(e[1]) for i, e in events.items())
    g_ms = sorted(e[1].elapsed_time(e[2]) for e in events.values())
    q_avg, g_avg = sum(q_ms) / len(q_ms), sum(g_ms) / len(g_ms)

    # the quantize kernel alone, launched back to back (outside the timed region)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(50):
        quantize_only()
    e1.record()
    torch.cuda.synchronize()
    q_b2b = e0.elapsed_time(e1) / 50
    # ... and the same 20 launches replayed from a HIP graph: no host time and no event records between them, so
    # the period per launch is the kernel plus the gap between two dependent launches
    q_graph = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            quantize_only()
        torch.cuda.current_stream().wait_stream(side)
        qg = torch.cuda.CUDAGraph()
        with torch.cuda.graph(qg):
            for _ in range(20):
                quantize_only()
        for _ in range(3):
            qg.replay()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            qg.replay()
        e1.record()
        torch.cuda.synchronize()
        q_graph = e0.elapsed_time(e1) / 100
        del qg
    except Exception as exc:   # noqa: BLE001  (an extra figure: the benchmark does not depend on it)
        print(f"bench: quantize graph timing skipped: {exc}", file=sys.stderr)
    traffic = MEASURED_TRAFFIC_BYTES.get(name, {})

    # the same forward without the two event records per step: the figure a caller of the module sees
    module_ms = None
    if mod.fused:
        for _ in range(3):
            mod(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            mod(x)
        torch.cuda.synchronize()
        module_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # Spread of the headline: `value` comes from the one timed block above (exactly --steps forwards after --warmup
    # warm-up forwards).  The same block (with its event records) is timed --repeats more times, back to back, as the
    # reference's layer benchmark repeats its timed block; median, mean and 1.96 sigma of the per-step time over ALL
    # blocks, the first included, go into `repeats`.  On this part the first block after an idle period runs in the
    # window in which the power management has just pulled the clock down, so it is usually the slowest.
    block_ms = [ms_step]
    for _ in range(max(0, args.repeats)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(events.get(i), before=(i - 1) not in events)
        torch.cuda.synchronize()
        block_ms.append((time.perf_counter() - t0) * 1e3 / args.steps)

    # the same step replayed from a HIP graph (extra figure: what a serving loop that captures the layer sees;
    # for small token counts the eager step is bound by Python launch overhead, not by the kernels)
    graph_ms = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for _ in range(max(60, args.warmup)):   # past the clock transient (about 12 ms) that follows the idle gap of the capture
            graph.replay()
        torch.cuda.synchronize()
        g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        g0.record()
        for _ in range(args.steps):
            graph.replay()
        g1.record()
        torch.cuda.synchronize()
        graph_ms = g0.elapsed_time(g1) / args.steps
    except Exception as exc:  # the figure is optional
        print(f"bench.py: graph replay skipped: {exc}", file=sys.stderr)

    cold_ms = None
    if args.cold_weights:
        import copy
        n_copies = max(2, int(700e6 / (N * K * bits / 8)) + 1)
        mods = [mod] + [copy.deepcopy(mod) for _ in range(n_copies - 1)]
        if args.int8_mfma:
            for m in mods:
                m.six_bit_path = False

        def all_layers():
            for m in mods:
                m(x)

        all_layers()                       # operand copies and the split-K workspace exist before the capture
        torch.cuda.synchronize()
        cold_graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cold_graph):
            all_layers()
        cold_graph.replay()
        torch.cuda.synchronize()
        c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        c0.record()
        for _ in range(10):
            cold_graph.replay()
        c1.record()
        torch.cuda.synchronize()
        cold_ms = c0.elapsed_time(c1) / 10 / n_copies
        del mods, cold_graph

    int_ops = 2.0 * M * N * K
    tops = int_ops / (ms_step * 1e-3) / 1e12
    gemm_tops = int_ops / (g_avg * 1e-3) / 1e12
    # read the row once; write the codes (6 bits each in the operand format of the 6-bit path, plus a 4-byte
    # level sum per row), the outlier values and the (scale, zero) pair
    quant_bytes = M * n_in * 2 + (M * K * 6 // 8 + M * 4 if six and bits == 4 else M * K * bits // 8) + M * F * 2 + M * 4
    quant_gbps = quant_bytes / (q_avg * 1e-3) / 1e9
    peak = PEAK_FP6_TOPS if six and bits == 4 else PEAK_INT8_TOPS
    split_k = six and matmul.split_k and _lib.load().quik_splitk_workspace_bytes(M, N, K, bits) > 0
    if six and bits == 4:
        gemm_kernel = "gemm_fused6_splitk_kernel (K split over several workgroups per tile)" if split_k else \
            "gemm_fused6_split_kernel / gemm_fused6_kernel (one launch per step)"
        dtype = "int4 (exact, as E2M3 on the 6-bit MFMA path)"
    elif six:
        gemm_kernel = "gemm_fused8t_splitk_kernel (tile-ordered int8 operands, K split over several workgroups per " \
            "tile)" if split_k else \
            "gemm_fused8t_split_kernel / gemm_fused8t_kernel (tile-ordered int8 operands, one launch per step)"
        dtype = "int8"
    elif mod.fused:
        gemm_kernel = "gemv_decode_kernel (one or two token rows: quantize and weight-streaming matrix-vector product " \
            "in ONE launch)" \
            if M <= 2 else "gemm_decode_kernel (weight streaming, one launch per step)" if M <= 32 else \
            "gemm_fused_split_kernel / gemm_fused_kernel (one launch per step)"
        dtype = "int8" if bits == 8 else "int4 (dot-product instructions)" if M <= 2 else "int4 (on int8 MFMA)"
    else:
        gemm_kernel = "gemm_i32_split_kernel + dequantize + F.linear"
        dtype = "int8" if bits == 8 else "int4 (on int8 MFMA)"

    roofline = {"kernel": gemm_kernel,
                "bound": "mfma", "achieved": round(gemm_tops, 2), "peak": peak,
                "unit": "TOP/s", "frac": round(gemm_tops / peak, 4),
                "frac_of_int8_peak": round(gemm_tops / PEAK_INT8_TOPS, 4),
                "traffic": traffic.get("gemm6" if six else "gemm") if mod.fused else None,
                "traffic_source": TRAFFIC_SOURCE["gemm6" if six else "gemm"]
                if mod.fused and traffic.get("gemm6" if six else "gemm") else None,
                "avg_ms": round(g_avg, 4), "median_ms": round(g_ms[len(g_ms) // 2], 4),
                "timed_launches": len(g_ms), "algorithmic_ops": int_ops}
    one_launch = mod.fused and not six and M <= 2
    if mod.fused and not six and M <= 32:
        # the weight-streaming kernels are bound by HBM: every weight byte once, plus the small operands
        stream_bytes = N * K * bits // 8 + N * F * 2 + 3 * N * 2 + M * n_in * 2 + M * N * 2
        launch_ms = q_avg if one_launch else g_avg       # (one launch: it ends at the event the library records)
        launch_med = (q_ms if one_launch else g_ms)[len(g_ms) // 2]
        gbps = stream_bytes / (launch_ms * 1e-3) / 1e9
        roofline = {"kernel": gemm_kernel, "bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS,
                    "unit": "GB/s", "frac": round(gbps / PEAK_HBM_GBPS, 4), "traffic": None,
                    "avg_ms": round(launch_ms, 4), "median_ms": round(launch_med, 4), "timed_launches": len(g_ms),
                    "algorithmic_bytes": stream_bytes,
                    "note": "avg_ms includes the cost of one event record (several us); kernel-trace durations of "
                            "the launch alone: profiles/"}

    res = {
        "metric": "MixedQLinear fwd TOPS (2*M*N*K / forward time), 1 GPU",
        "value": round(tops, 2), "unit": "TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": f"{name}: MixedQLinear fwd, tokens={M}, in={n_in}, out={N}, fp16 outliers={F}, "
                               f"W{bits}A{bits} asymmetric per-token, fp16 activations, "
                               f"{'fused GEMM+dequant' if mod.fused else 'unfused three-op sequence'}"
                               f"{', 6-bit matrix-core path' if six and bits == 4 else ', tile-ordered operands' if six else ''}",
                   "M": M, "in_features": n_in, "K": K, "N": N, "F": F, "bits": bits},
        "pct_int8_mfma_peak": round(100.0 * tops / PEAK_INT8_TOPS, 2),
        "repeats": spread(block_ms, int_ops),
        "module_forward_ms_per_step": None if module_ms is None else round(module_ms, 4),
        "graph_replay_ms_per_step": None if graph_ms is None else round(graph_ms, 4),
        "cold_ms_per_forward": None if cold_ms is None else round(cold_ms, 4),
        # weight storage of this layer on the GPU: the reference's buffers and the tile-ordered copy the prefill GEMM
        # reads (MixedQLinear.release_row_major_weights() / release_tiled_weights() keep one of them)
        "resident_weight_bytes": mod.weight_bytes(),
        "verified_vs_oracle": None if spot is None else {"tiles": 3, "max_abs_err_over_rms": round(spot, 6),
                                                         "tolerance": 1e-2},
        "roofline": roofline,
        "roofline_quantize": None if one_launch else {"kernel": (f"quantize_fp6_wave_kernel (one wave per token row, {'two' if M <= 1536 else 'eight'} rows per workgroup, 6-bit operand output)" if six and bits == 4
                                         else "quantize_tile8_ring_kernel (row copied into an LDS ring, int8 operand output in tile order)"
                                         if six and bits == 8 and n_in > 8192 and str(x.dtype) == "torch.float16"
                                         else "asym_quantize_stream_kernel" + (" (tile-ordered operand output)" if six else "")),
                              "bound": "hbm",
                              "achieved": round(quant_gbps, 1),
                              "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": round(quant_gbps / PEAK_HBM_GBPS, 4),
                              "traffic": traffic.get("quantize6" if six else "quantize"),
                              "traffic_source": TRAFFIC_SOURCE["quantize6" if six else "quantize"]
                              if traffic.get("quantize6" if six else "quantize") else None,
                              "avg_ms": round(q_avg, 5),
                              "median_ms": round(q_ms[len(q_ms) // 2], 5), "algorithmic_bytes": quant_bytes,
                              "back_to_back_ms": round(q_b2b, 5),
                              "graph_back_to_back_ms": None if q_graph is None else round(q_graph, 5),
                              "frac_by_graph_period": None if q_graph is None
                              else round(quant_bytes / (q_graph * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                              "note": "avg_ms: from the event behind the previous forward to the event the library "
                                      "records between the quantize launch and the GEMM launch (the launch plus the "
                                      "cost of one event record, several us); back_to_back_ms: per launch over 50 consecutive "
                                      "launches after the timed region (bound by the host: ~14 us of Python per "
                                      "call); graph_back_to_back_ms: period per launch of 20 launches replayed from a "
                                      "HIP graph (kernel + the gap between dependent launches); kernel-trace durations of the launch alone: profiles/"},
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(name, x_cpu, W_cpu, int_idx, fp_idx)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
