#!/usr/bin/env python3
"""Benchmark of the mi355x hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME]

Prints one JSON line.  The headline workload is BASELINE config 2, the
memory-bound residual-add + LayerNorm fusion in bf16 on [8192, 4096]; a "step"
is one launch of the fused op over one batch of seeded synthetic input that is
already resident in HBM.  `value` is algorithmic bytes moved per second through
the product path (torch.ops.xpu_ops -> C ABI -> HIP kernel).  `roofline` is the
same kernel launched back-to-back straight through the C ABI, timed with HIP
events on the launch stream.  `cpu_baseline` is the same eager function on the
host cores (through this package's default, non-vendor compile path when it is
available).  `configs` carries the same three figures for the other benchmark
configurations.

Every GPU figure is taken on warm clocks: before a timed region the same call
runs for at least WARM_SECONDS (the first ~100 ms of work after an idle spell,
e.g. after a CPU baseline, run visibly slower), then the --warmup launches,
then the timed ones.  `roofline.traffic` is not measured by this run: it is
read from profiles/traffic.json, which the rocprofv3 --pmc recipe printed in
that file produces, and the top-level `traffic_source` names it (once for every
workload of the line).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
FP8_PEAK_TFLOPS = 5000.0
FP32_PEAK_TFLOPS = 157.3
N_SETS = 6  # rotating buffer sets so that timed launches stream from HBM, not from the 256 MB last-level cache
WARM_SECONDS = 0.15  # GPU work of the same kind in front of every timed region
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def _traffic_table():
    try:
        with open(TRAFFIC_FILE) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def _warm(torch, fn, n_sets):
    """Run fn for WARM_SECONDS of wall clock so that the timed region starts on warm clocks."""
    torch.cuda.synchronize()
    t_end = time.perf_counter() + WARM_SECONDS
    i = 0
    while time.perf_counter() < t_end:
        for _ in range(4):
            fn(i % n_sets)
            i += 1
        torch.cuda.synchronize()


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _events_time(torch, fn, n_sets, steps, warmup):
    """Average seconds per call of fn(i) over `steps` back-to-back calls, by HIP events on the current stream."""
    _warm(torch, fn, n_sets)
    for i in range(warmup):
        fn(i % n_sets)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fn(i % n_sets)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def _wall_time(torch, fn, n_sets, steps, warmup):
    _warm(torch, fn, n_sets)
    for i in range(warmup):
        fn(i % n_sets)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i % n_sets)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


NOMINAL_CLOCK_GHZ = 2.4  # MI355X peak engine clock: the published MFMA peaks are quoted at it


def _shader_clock_ghz(torch, fn, n_sets, t_call, label=""):
    """Median engine clock while `fn` runs back to back: a one-wave probe kernel on a second stream samples the shader
    clock against the constant-rate wall clock in 20 us windows for 8 ms (xg_clock_probe); the second half counts, by
    which the power management has settled on this load."""
    from xpu_graph_amd import _lib

    lib = _lib.lib()
    khz = int(lib.xg_wall_clock_khz())
    if khz <= 0:
        return None
    n_win, win_us = 400, 20
    buf = torch.zeros(2 * n_win, dtype=torch.int64, device="cuda")
    side = torch.cuda.Stream()
    warm = min(2000, max(3, int(0.02 / t_call)))                      # ~20 ms of this load first
    reps = max(3, int(1.5 * n_win * win_us * 1e-6 / t_call) + 2)      # outlasts the probe
    for i in range(warm):
        fn(i % n_sets)
    torch.cuda.synchronize()
    fn(0)
    _lib.check(lib.xg_clock_probe(_p(buf), n_win, win_us * khz // 1000, ctypes.c_void_p(side.cuda_stream)), "xg_clock_probe")
    for i in range(reps):
        fn(i % n_sets)
    torch.cuda.synchronize()
    d = buf.view(n_win, 2).double()
    ghz = d[:, 0] / d[:, 1].clamp(min=1) * khz / 1e6
    quarters = [float(ghz[i * n_win // 4:(i + 1) * n_win // 4].median().item()) for i in range(4)]
    print(f"[bench] shader clock under {label}: median GHz per 2 ms quarter {' '.join(f'{q:.2f}' for q in quarters)}", file=sys.stderr)
    return float(ghz[n_win // 2:].median().item())


def _cpu_time(fn, min_iters=3, budget_s=12.0, max_iters=30, warmups=2):
    for _ in range(warmups):  # also compiles the default path
        fn()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < min_iters or (time.perf_counter() < t_end and len(times) < max_iters):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], len(times)


def _default_path_compile(fn):
    """The reference's non-vendor path: XpuGraph(XpuGraphConfig(is_training=False)) on CPU tensors."""
    import torch

    try:
        from xpu_graph_amd import XpuGraph, XpuGraphConfig

        return torch.compile(fn, backend=XpuGraph(XpuGraphConfig(is_training=False)), dynamic=False), "XpuGraph default path (target=none, level1)"
    except ImportError:
        return fn, "eager"


class Workload:
    name = ""
    bound = "hbm"
    dtype = ""
    unit = "GB/s"

    def setup(self, torch, dev):
        raise NotImplementedError

    def op_call(self, i):  # product path
        raise NotImplementedError

    def abi_call(self, i):  # straight C ABI
        raise NotImplementedError

    def check(self, torch):
        raise NotImplementedError

    def cpu_fn(self, torch):
        raise NotImplementedError

    work = 0  # algorithmic bytes (hbm) or flops (mfma) per launch


class AddLayerNormC2(Workload):
    name = "C2 residual-add + LayerNorm bf16 [8192,4096] -> (y, h)"
    dtype = "bf16"
    kernel = "norm_rows_kernel<bf16,bf16,LAYER>"
    work = 4 * 8192 * 4096 * 2 + 2 * 4096 * 2
    traffic_key = "c2_add_layernorm"

    def setup(self, torch, dev):
        from oracle import inputs

        self.torch = torch
        self.sets = [inputs.c2_add_layernorm(device=dev, seed=i) for i in range(N_SETS)]
        self.y = [torch.empty_like(s[0]) for s in self.sets]
        self.h = [torch.empty_like(s[0]) for s in self.sets]
        from xpu_graph_amd import _lib

        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x, r, g, b = self.sets[i]
        return self.torch.ops.xpu_ops.add_layer_norm(x, r, g, b, 1e-5)

    def abi_call(self, i):
        x, r, g, b = self.sets[i]
        self.lib.xg_add_layer_norm(_p(x), _p(r), _p(g), _p(b), _p(self.y[i]), _p(self.h[i]), 8192, 4096, 4096, 4096, 1e-5, 2, 2, self.st)

    def check(self, torch):
        from oracle import eager

        x, r, g, b = self.sets[0]
        y, h = self.op_call(0)
        y_ref, h_ref = eager.add_layernorm_eager(x, r, g, b, 1e-5)
        assert torch.equal(h, h_ref)
        torch.testing.assert_close(y, y_ref, rtol=1.6e-2, atol=1e-5)

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        x, r, g, b = inputs.c2_add_layernorm(device="cpu", seed=0)
        fn, how = _default_path_compile(lambda x, r, g, b: eager.add_layernorm_eager(x, r, g, b, 1e-5))
        return (lambda: fn(x, r, g, b)), how


class RmsNormC1(Workload):
    name = "C1 RMSNorm fp32 [2048,4096]"
    dtype = "f32"
    kernel = "norm_rows_kernel<f32,f32,RMS>"
    work = 2 * 2048 * 4096 * 4 + 4096 * 4
    traffic_key = "c1_rmsnorm"

    def setup(self, torch, dev):
        from oracle import inputs
        from xpu_graph_amd import _lib

        self.torch = torch
        self.sets = [inputs.c1_rmsnorm(device=dev, seed=i) for i in range(N_SETS)]
        self.y = [torch.empty_like(s[0]) for s in self.sets]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x, w = self.sets[i]
        return self.torch.ops.xpu_ops.rms_norm(x, w, 1e-6)

    def abi_call(self, i):
        x, w = self.sets[i]
        self.lib.xg_rms_norm(_p(x), _p(w), _p(self.y[i]), 2048, 4096, 4096, 1e-6, 0, 0, self.st)

    def check(self, torch):
        from oracle import eager

        x, w = self.sets[0]
        torch.testing.assert_close(self.op_call(0), eager.rmsnorm_eager(x, w, 1e-6), rtol=1e-5, atol=1e-5)

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        x, w = inputs.c1_rmsnorm(device="cpu", seed=0)
        fn, how = _default_path_compile(lambda x, w: eager.rmsnorm_eager(x, w, 1e-6))
        return (lambda: fn(x, w)), how


class SliceCatC3a(Workload):
    name = "C3a slice/cat fp32 [4096,8192] -> 64x32 -> [4096,2048]"
    dtype = "b32"
    kernel = "slice_cat_kernel<16>"
    work = 2 * 4096 * 2048 * 4 + 64 * 8
    traffic_key = "c3a_slice_cat"

    def setup(self, torch, dev):
        from oracle import inputs
        from xpu_graph_amd import _lib, ops

        self.torch = torch
        self.srcs = []
        for i in range(N_SETS):
            src, self.slices = inputs.c3_slice_cat(device=dev, seed=i)
            self.srcs.append(src)
        table, self.chunk, self.out_cols = ops.build_slice_table([self.slices], 8192, 4, 8192)
        self.table = table.to(dev)
        self.outs = [torch.empty(4096, 2048, device=dev) for _ in range(N_SETS)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.ptrs = [(ctypes.c_void_p * 1)(o.data_ptr()) for o in self.outs]
        self.rbs = (ctypes.c_int64 * 1)(2048 * 4)

    def op_call(self, i):
        return self.torch.ops.xpu_ops.slice_cat(self.srcs[i], self.table, self.chunk, self.out_cols[0])

    def abi_call(self, i):
        self.lib.xg_slice_cat(_p(self.srcs[i]), 8192 * 4, 4096, self.ptrs[i], self.rbs, 1, _p(self.table), self.table.shape[0], self.chunk, self.st)

    def check(self, torch):
        from oracle import eager

        assert torch.equal(self.op_call(0), eager.slice_cat_eager(self.srcs[0], self.slices))

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        src, slices = inputs.c3_slice_cat(device="cpu", seed=0)
        fn, how = _default_path_compile(lambda s: eager.slice_cat_eager(s, slices))
        return (lambda: fn(src)), how


class AddNC3b(Workload):
    name = "C3b sum of 32 x [4096,256] fp32"
    dtype = "f32"
    kernel = "addn_kernel<f32>"
    work = 33 * 4096 * 256 * 4
    traffic_key = "c3b_addn"

    def setup(self, torch, dev):
        from oracle import inputs
        from xpu_graph_amd import _lib

        self.torch = torch
        self.sets = [inputs.c3_addn(device=dev, seed=i) for i in range(N_SETS)]
        self.outs = [torch.empty(4096, 256, device=dev) for _ in range(N_SETS)]
        self.arrs = [(ctypes.c_void_p * 32)(*[t.data_ptr() for t in s]) for s in self.sets]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        return self.torch.ops.xpu_ops.addn(self.sets[i])

    def abi_call(self, i):
        self.lib.xg_addn(self.arrs[i], 32, _p(self.outs[i]), 4096 * 256, 0, self.st)

    def check(self, torch):
        from oracle import eager

        assert torch.equal(self.op_call(0), eager.addn_eager(self.sets[0]))

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        ts = inputs.c3_addn(device="cpu", seed=0)
        fn, how = _default_path_compile(lambda *t: eager.addn_eager(list(t)))
        return (lambda: fn(*ts)), how


class DenseC4(Workload):
    zero_operands = True
    name = "C4 dense + bias + SiLU bf16 M8192 K4096 N11008"
    bound = "mfma"
    dtype = "bf16"
    unit = "TFLOP/s"
    kernel = "gemm_dma_split_kernel<bf16,[K,N]>"
    work = 2 * 8192 * 4096 * 11008
    traffic_key = "c4_dense_bf16"
    n_sets = 3
    cpu_warmups = 1

    def setup(self, torch, dev):
        from oracle import inputs
        from xpu_graph_amd import _lib

        self.torch = torch
        self.sets = [inputs.c4_dense(device=dev, seed=i) for i in range(self.n_sets)]
        self.outs = [torch.empty(8192, 11008, device=dev, dtype=torch.bfloat16) for _ in range(self.n_sets)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x, W, b = self.sets[i]
        return self.torch.ops.xpu_ops.dense(x, W, False, b, None, "silu")

    def abi_call(self, i):
        x, W, b = self.sets[i]
        self.lib.xg_dense(_p(x), _p(W), _p(b), None, _p(self.outs[i]), 8192, 11008, 4096, 4096, 11008, 0, 0, 3, 2, 2, self.st)

    def check(self, torch):
        x, W, b = self.sets[0]
        rows = torch.arange(0, 8192, 97, device=x.device)
        want = torch.nn.functional.silu(x[rows].float() @ W.float() + b.float())
        torch.testing.assert_close(self.op_call(0)[rows].float(), want, rtol=1.6e-2, atol=2e-2)

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        x, W, b = inputs.c4_dense(device="cpu", seed=0)
        fn, how = _default_path_compile(eager.dense_silu_eager)
        return (lambda: fn(x, W, b)), how


class DenseFp32(Workload):
    name = "dense + bias + SiLU fp32 M4096 K4096 N4096"
    bound = "mfma"
    dtype = "f32"
    unit = "TFLOP/s"
    kernel = "gemm_dma_kernel<f32,[K,N]>"
    work = 2 * 4096 * 4096 * 4096
    traffic_key = None
    n_sets = 3
    cpu_warmups = 1

    def setup(self, torch, dev):
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(0)
        self.sets = [(torch.randn(4096, 4096, generator=g).to(dev), (0.02 * torch.randn(4096, 4096, generator=g)).to(dev),
                      (0.02 * torch.randn(4096, generator=g)).to(dev)) for _ in range(self.n_sets)]
        self.outs = [torch.empty(4096, 4096, device=dev) for _ in range(self.n_sets)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x, W, b = self.sets[i]
        return self.torch.ops.xpu_ops.dense(x, W, False, b, None, "silu")

    def abi_call(self, i):
        x, W, b = self.sets[i]
        self.lib.xg_dense(_p(x), _p(W), _p(b), None, _p(self.outs[i]), 4096, 4096, 4096, 4096, 4096, 0, 0, 3, 0, 0, self.st)

    def check(self, torch):
        x, W, b = self.sets[0]
        rows = torch.arange(0, 4096, 97, device=x.device)
        z = x[rows].double() @ W.double() + b.double()
        want = torch.nn.functional.silu(z)
        torch.testing.assert_close(self.op_call(0)[rows].double(), want, rtol=1e-5, atol=1.1 * z.abs().max().item() * 64 * 2.0**-24)

    def cpu_fn(self, torch):
        g = torch.Generator().manual_seed(0)
        x, W, b = torch.randn(4096, 4096, generator=g), 0.02 * torch.randn(4096, 4096, generator=g), 0.02 * torch.randn(4096, generator=g)
        return (lambda: torch.nn.functional.silu(x @ W + b)), "eager fp32 matmul + bias + SiLU"


class DenseFp8C4(DenseC4):
    name = "C4 dense + bias + SiLU fp8 e4m3 M8192 K4096 N11008"
    dtype = "fp8"
    kernel = "gemm_dma_split_kernel<e4m3,[N,K]>"
    traffic_key = "c4_dense_fp8"

    def setup(self, torch, dev):
        from oracle import eager, inputs
        from xpu_graph_amd import _lib

        self.torch = torch
        self.sets = []
        for i in range(self.n_sets):
            x, W, b = inputs.c4_dense(device=dev, seed=i)
            x_q, s_x = eager.quantize_fp8_per_tensor(x)
            W_q, s_w = eager.quantize_fp8_per_out_channel(W)
            self.sets.append((x_q, W_q.t().contiguous(), s_x, s_w.contiguous(), b))
            if i == 0:
                self.W_q0 = W_q
        self.outs = [torch.empty(8192, 11008, device=dev, dtype=torch.bfloat16) for _ in range(self.n_sets)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x_q, w_nk, s_x, s_w, b = self.sets[i]
        return self.torch.ops.xpu_ops.dense_fp8(x_q, w_nk, True, s_x, s_w, b, "silu", self.torch.bfloat16)

    def abi_call(self, i):
        x_q, w_nk, s_x, s_w, b = self.sets[i]
        self.lib.xg_dense_fp8(_p(x_q), _p(w_nk), _p(s_x), _p(s_w), _p(b), _p(self.outs[i]), 8192, 11008, 4096, 4096, 4096, 1, 3, 2, 2, self.st)

    def check(self, torch):
        from oracle import eager

        x_q, w_nk, s_x, s_w, b = self.sets[0]
        rows = torch.arange(0, 8192, 97, device=x_q.device)
        want = eager.dense_fp8_silu_eager(x_q[rows], self.W_q0, s_x, s_w, b)
        torch.testing.assert_close(self.op_call(0)[rows].float(), want, rtol=1.6e-2, atol=2e-3)
        del self.W_q0

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        x, W, b = inputs.c4_dense(device="cpu", seed=0)
        x_q, s_x = eager.quantize_fp8_per_tensor(x)
        W_q, s_w = eager.quantize_fp8_per_out_channel(W)
        return (lambda: eager.dense_fp8_silu_eager(x_q, W_q, s_x, s_w, b)), "eager dequantise + fp32 matmul"


class DenseGluC5(Workload):
    zero_operands = True
    name = "C5 MLP gate+up gated dense bf16 M8192 K4096 N11008"
    bound = "mfma"
    dtype = "bf16"
    unit = "TFLOP/s"
    kernel = "gemm_glu_kernel<bf16>"
    work = 4 * 8192 * 4096 * 11008
    traffic_key = "c5_dense_glu"
    n_sets = 3
    cpu_warmups = 1

    def setup(self, torch, dev):
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(5)
        self.sets = [
            (
                torch.randn(8192, 4096, generator=g).bfloat16().to(dev),
                (0.02 * torch.randn(11008, 4096, generator=g)).bfloat16().to(dev),
                (0.02 * torch.randn(11008, 4096, generator=g)).bfloat16().to(dev),
            )
            for _ in range(self.n_sets)
        ]
        self.outs = [torch.empty(8192, 11008, device=dev, dtype=torch.bfloat16) for _ in range(self.n_sets)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x, wg, wu = self.sets[i]
        return self.torch.ops.xpu_ops.dense_glu(x, wg, wu)

    def abi_call(self, i):
        x, wg, wu = self.sets[i]
        self.lib.xg_dense_glu(_p(x), _p(wg), _p(wu), _p(self.outs[i]), 8192, 11008, 4096, 4096, 4096, 2, self.st)

    def check(self, torch):
        x, wg, wu = self.sets[0]
        rows = torch.arange(0, 8192, 97, device=x.device)
        xf = x[rows].float()
        want = torch.nn.functional.silu(xf @ wg.float().t()) * (xf @ wu.float().t())
        torch.testing.assert_close(self.op_call(0)[rows].float(), want, rtol=1.6e-2, atol=2e-2)

    def cpu_fn(self, torch):
        from oracle import eager

        x, wg, wu = (t.cpu() for t in self.sets[0])
        fn, how = _default_path_compile(lambda x, wg, wu: torch.nn.functional.silu(torch.nn.functional.linear(x, wg)) * torch.nn.functional.linear(x, wu))
        return (lambda: fn(x, wg, wu)), how


class SdpaC5(Workload):
    zero_operands = True
    name = "C5 causal attention bf16 B4 H32 S2048 D128"
    bound = "mfma"
    dtype = "bf16"
    unit = "TFLOP/s"
    kernel = "sdpa_fwd_kernel<bf16,128>"
    work = 4 * 4 * 32 * 2048 * 2048 * 128 // 2  # two matmuls, lower triangle only
    traffic_key = "c5_sdpa"
    n_sets = 3
    cpu_warmups = 1

    def setup(self, torch, dev):
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(0)
        self.sets = [tuple(torch.randn(4, 32, 2048, 128, generator=g).bfloat16().to(dev) for _ in range(3)) for _ in range(self.n_sets)]
        self.outs = [torch.empty_like(s[0]) for s in self.sets]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.strides = (ctypes.c_int64 * 3)(32 * 2048 * 128, 2048 * 128, 128)
        self.scale = ctypes.c_float(128**-0.5)

    def op_call(self, i):
        q, k, v = self.sets[i]
        return self.torch.ops.xpu_ops.sdpa(q, k, v, True, 128**-0.5)

    def abi_call(self, i):
        q, k, v = self.sets[i]
        s = self.strides
        self.lib.xg_sdpa(_p(q), _p(k), _p(v), _p(self.outs[i]), 4, 32, 32, 2048, 2048, 128, s, s, s, s, self.scale, 1, 2, self.st)

    def check(self, torch):
        from oracle import eager

        q, k, v = (t[:1, :4] for t in self.sets[0])
        got = self.op_call(0)[:1, :4]
        torch.testing.assert_close(got.float(), eager.causal_sdpa_eager(q.float(), k.float(), v.float()), rtol=1.6e-2, atol=8e-3)

    def cpu_fn(self, torch):
        from oracle import eager

        g = torch.Generator().manual_seed(0)
        q, k, v = (torch.randn(4, 32, 2048, 128, generator=g).bfloat16() for _ in range(3))
        fn, how = _default_path_compile(eager.causal_sdpa_eager)
        return (lambda: fn(q, k, v)), how


class SdpaBackwardC5(Workload):
    name = "C5 causal attention backward bf16 B4 H32 S2048 D128"
    bound = "mfma"
    dtype = "bf16"
    unit = "TFLOP/s"
    kernel = "sdpa_bwd_dq_kernel + sdpa_bwd_dkv_kernel"
    work = 10 * 4 * 32 * 2048 * 2048 * 128 // 2  # five matmuls (S, dP, dV, dK, dQ), lower triangle only
    cpu_work = work // 4  # the CPU leg runs one of the four batch entries
    traffic_key = None
    n_sets = 2
    cpu_warmups = 0

    def setup(self, torch, dev):
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(0)
        mk = lambda: torch.randn(4, 32, 2048, 128, generator=g).bfloat16().to(dev)  # noqa: E731
        self.sets = []
        for _ in range(self.n_sets):
            q, k, v, do = mk(), mk(), mk(), mk()
            out, lse = torch.ops.xpu_ops.sdpa_lse(q, k, v, True, 128**-0.5)
            self.sets.append((q, k, v, out, do, lse))
        self.grads = [tuple(torch.empty_like(s[0]) for _ in range(3)) for s in self.sets]
        self.delta = torch.empty(4, 32, 2048, dtype=torch.float32, device=dev)
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.strides = (ctypes.c_int64 * 3)(32 * 2048 * 128, 2048 * 128, 128)
        self.scale = ctypes.c_float(128**-0.5)

    def op_call(self, i):
        q, k, v, out, do, lse = self.sets[i]
        return self.torch.ops.xpu_ops.sdpa_bwd(q, k, v, out, do, lse, True, 128**-0.5)

    def abi_call(self, i):
        q, k, v, out, do, lse = self.sets[i]
        dq, dk, dv = self.grads[i]
        s = self.strides
        self.lib.xg_sdpa_backward(_p(q), _p(k), _p(v), _p(out), _p(do), _p(lse), _p(dq), _p(dk), _p(dv), _p(self.delta), 4, 32, 32, 2048, 2048,
                                  128, s, s, s, s, s, s, s, s, self.scale, 1, 2, self.st)

    def check(self, torch):
        from oracle import eager

        q, k, v, _, do, _ = (t[:1, :2] for t in self.sets[0])
        leaves = [t.float().requires_grad_(True) for t in (q, k, v)]
        want = torch.autograd.grad(eager.causal_sdpa_eager(*leaves), leaves, do.float())
        got = self.op_call(0)
        for a, b in zip(got, want):
            torch.testing.assert_close(a[:1, :2].float(), b, rtol=1.6e-2, atol=b.abs().max().item() * 2.0**-7)

    def cpu_fn(self, torch):
        from oracle import eager

        g = torch.Generator().manual_seed(0)
        q, k, v = (torch.randn(1, 32, 2048, 128, generator=g).bfloat16().requires_grad_(True) for _ in range(3))
        do = torch.randn(1, 32, 2048, 128, generator=g).bfloat16()

        def run():
            return torch.autograd.grad(eager.causal_sdpa_eager(q, k, v), (q, k, v), do)

        return run, "eager autograd on one batch entry (B1 H32 S2048 D128; forward and backward, the forward's flops not counted)"


class DenseDecode(Workload):
    name = "decode dense + bias bf16 M1 K4096 N11008, [N,K] weights"
    dtype = "bf16"
    kernel = "gemm_skinny_kernel<bf16,1>"
    work = 11008 * 4096 * 2 + (4096 + 2 * 11008) * 2  # the weights once, x, bias and the output row
    n_sets = 3  # 270 MB of weights in rotation: more than the last-level cache holds

    def setup(self, torch, dev):
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(0)
        self.sets = [
            (torch.randn(1, 4096, generator=g).bfloat16().to(dev), (torch.randn(11008, 4096, generator=g) * 0.02).bfloat16().to(dev),
             (torch.randn(11008, generator=g) * 0.02).bfloat16().to(dev))
            for _ in range(self.n_sets)
        ]
        self.outs = [torch.empty(1, 11008, device=dev, dtype=torch.bfloat16) for _ in range(self.n_sets)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x, W, b = self.sets[i]
        return self.torch.ops.xpu_ops.dense(x, W, True, b, None, "none")

    def abi_call(self, i):
        x, W, b = self.sets[i]
        self.lib.xg_dense(_p(x), _p(W), _p(b), None, _p(self.outs[i]), 1, 11008, 4096, 4096, 4096, 0, 1, 0, 2, 2, self.st)

    def check(self, torch):
        from oracle import eager

        x, W, b = self.sets[0]
        want = eager.dense_eager(x.float(), W.float(), True, b.float(), "none")
        torch.testing.assert_close(self.op_call(0).float(), want, rtol=1.6e-2, atol=2e-2)

    def cpu_fn(self, torch):
        from oracle import eager

        x, W, b = (t.cpu() for t in self.sets[0])
        fn, how = _default_path_compile(lambda x, W, b: eager.dense_eager(x, W, True, b, "none"))
        return (lambda: fn(x, W, b)), how


class DenseDecodeFp8(DenseDecode):
    name = "decode dense + bias fp8 e4m3 M1 K4096 N11008, [N,K] weights"
    dtype = "fp8"
    kernel = "gemm_skinny_fp8_kernel<bf16,1>"
    work = 11008 * 4096 + 4096 + 11008 * 4 + 2 * 11008 * 2  # the weights once, x, the weight scales, bias and the output row
    n_sets = 6  # 270 MB of weights in rotation

    def setup(self, torch, dev):
        from oracle import eager
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(0)
        self.sets = []
        for _ in range(self.n_sets):
            x_q, s_x = eager.quantize_fp8_per_tensor(torch.randn(1, 4096, generator=g))
            W_q, s_w = eager.quantize_fp8_per_out_channel(torch.randn(4096, 11008, generator=g) * 0.02)
            b = (torch.randn(11008, generator=g) * 0.02).bfloat16()
            self.sets.append((x_q.to(dev), W_q.t().contiguous().to(dev), s_x.to(dev), s_w.contiguous().to(dev), b.to(dev)))
        self.outs = [torch.empty(1, 11008, device=dev, dtype=torch.bfloat16) for _ in range(self.n_sets)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x_q, w_nk, s_x, s_w, b = self.sets[i]
        return self.torch.ops.xpu_ops.dense_fp8(x_q, w_nk, True, s_x, s_w, b, "none", self.torch.bfloat16)

    def abi_call(self, i):
        x_q, w_nk, s_x, s_w, b = self.sets[i]
        self.lib.xg_dense_fp8(_p(x_q), _p(w_nk), _p(s_x), _p(s_w), _p(b), _p(self.outs[i]), 1, 11008, 4096, 4096, 4096, 1, 0, 2, 2, self.st)

    def check(self, torch):
        x_q, w_nk, s_x, s_w, b = self.sets[0]
        want = (x_q.float() @ w_nk.float().t()) * s_x * s_w + b.float()
        torch.testing.assert_close(self.op_call(0).float(), want, rtol=1.6e-2, atol=2e-3)

    def cpu_fn(self, torch):
        x_q, w_nk, s_x, s_w, b = (t.cpu() for t in self.sets[0])
        return (lambda: (x_q.float() @ w_nk.float().t()) * s_x * s_w + b.float()), "eager dequantise + fp32 matmul"


class SdpaDecode(Workload):
    name = "decode attention bf16 B8 H32 Hkv8 Sq1 Skv8192 D128"
    dtype = "bf16"
    kernel = "sdpa_decode_kernel<bf16,128> + sdpa_decode_merge_kernel (kernel_us covers both launches)"
    work = 2 * 8 * 8 * 8192 * 128 * 2 + 2 * 8 * 32 * 128 * 2  # K and V once, q and the output
    n_sets = 3

    def setup(self, torch, dev):
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(0)
        self.sets = [
            (torch.randn(8, 32, 1, 128, generator=g).bfloat16().to(dev), torch.randn(8, 8, 8192, 128, generator=g).bfloat16().to(dev),
             torch.randn(8, 8, 8192, 128, generator=g).bfloat16().to(dev))
            for _ in range(self.n_sets)
        ]
        self.outs = [torch.empty_like(s[0]) for s in self.sets]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        S3 = ctypes.c_int64 * 3
        self.qs, self.ks = S3(32 * 128, 128, 128), S3(8 * 8192 * 128, 8192 * 128, 128)
        self.n_ws = self.lib.xg_sdpa_decode_workspace_floats(8, 32, 8, 1, 8192, 128)
        self.ws = torch.empty(max(self.n_ws, 1), device=dev)
        self.scale = ctypes.c_float(128**-0.5)

    def op_call(self, i):
        q, k, v = self.sets[i]
        return self.torch.ops.xpu_ops.sdpa(q, k, v, False, 128**-0.5)

    def abi_call(self, i):
        q, k, v = self.sets[i]
        self.lib.xg_sdpa_decode(_p(q), _p(k), _p(v), _p(self.outs[i]), None, None, None, 2, None, _p(self.ws), self.n_ws, 8, 32, 8, 1, 8192, 128,
                                self.qs, self.ks, self.ks, self.qs, self.scale, 2, self.st)

    def check(self, torch):
        from oracle import eager

        q, k, v = (t[:1] for t in self.sets[0])
        want = eager.sdpa_eager(q.float(), k.float(), v.float())
        torch.testing.assert_close(self.op_call(0)[:1].float(), want, rtol=1.6e-2, atol=2e-3)

    def cpu_fn(self, torch):
        from oracle import eager

        q, k, v = (t.cpu() for t in self.sets[0])
        fn, how = _default_path_compile(eager.sdpa_eager)
        return (lambda: fn(q, k, v)), how


class DenseWeightGradC4(Workload):
    zero_operands = True
    name = "C4 dense weight gradient bf16 x[8192,4096]^T g[8192,11008]"
    bound = "mfma"
    dtype = "bf16"
    unit = "TFLOP/s"
    kernel = "gemm_dma_kernel<bf16,[K,N],A[K,M]>"
    work = 2 * 8192 * 4096 * 11008
    traffic_key = "c4_dense_at"
    n_sets = 3
    cpu_warmups = 1

    def setup(self, torch, dev):
        from xpu_graph_amd import _lib

        self.torch = torch
        g = torch.Generator().manual_seed(0)
        self.sets = [(torch.randn(8192, 4096, generator=g).bfloat16().to(dev), (0.02 * torch.randn(8192, 11008, generator=g)).bfloat16().to(dev))
                     for _ in range(self.n_sets)]
        self.outs = [torch.empty(4096, 11008, device=dev, dtype=torch.bfloat16) for _ in range(self.n_sets)]
        self.lib = _lib.lib()
        self.st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def op_call(self, i):
        x, g = self.sets[i]
        return self.torch.ops.xpu_ops.dense_at(x, g, None)

    def abi_call(self, i):
        x, g = self.sets[i]
        self.lib.xg_dense_at(_p(x), _p(g), None, _p(self.outs[i]), 4096, 11008, 8192, 4096, 11008, 0, 2, self.st)

    def check(self, torch):
        x, g = self.sets[0]
        rows = torch.arange(0, 4096, 97, device=x.device)
        want = x[:, rows].float().t() @ g.float()
        torch.testing.assert_close(self.op_call(0)[rows].float(), want, rtol=1.6e-2, atol=want.abs().max().item() * 2.0**-8)

    def cpu_fn(self, torch):
        g = torch.Generator().manual_seed(0)
        x = torch.randn(8192, 4096, generator=g).bfloat16()
        gz = (0.02 * torch.randn(8192, 11008, generator=g)).bfloat16()
        return (lambda: x.t() @ gz), "eager bf16 matmul (x.t() @ g)"


class LlamaBlockC5(Workload):
    name = "C5 Llama decoder block bf16 B4 S2048 compiled"
    bound = "mfma"
    dtype = "bf16"
    unit = "TFLOP/s"
    kernel = "compiled block"
    traffic_key = None
    work = 2 * 8192 * (4 * 4096 * 4096 + 3 * 4096 * 11008) + 4 * 4 * 32 * 2048 * 2048 * 128 // 2
    n_sets = 1
    cpu_warmups = 1

    def setup(self, torch, dev):
        from oracle import eager, inputs
        from xpu_graph_amd import mi355x_compiler

        self.torch = torch
        self.x, self.p = inputs.c5_llama_block(device=dev)
        self.names = sorted(self.p)
        names = self.names

        def block(x, *ws):
            return eager.llama_block_eager(x, dict(zip(names, ws)), n_heads=32)

        self.eager_fn = block
        self.fn = torch.compile(block, backend=mi355x_compiler(), dynamic=False)
        self.ws = [self.p[n] for n in names]

    def op_call(self, i):
        with self.torch.no_grad():
            return self.fn(self.x, *self.ws)

    abi_call = op_call

    def check(self, torch):
        got = self.op_call(0)
        with torch.no_grad():
            want = self.eager_fn(self.x, *self.ws)
            self.eager_ms = _events_time(torch, lambda i: self.eager_fn(self.x, *self.ws), 1, 5, 2) * 1e3
        assert (got.float() - want.float()).abs().mean().item() < 2e-2

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        x, p = inputs.c5_llama_block(device="cpu")
        fn, how = _default_path_compile(lambda x: eager.llama_block_eager(x, p, n_heads=32))

        def run():
            with torch.no_grad():
                return fn(x)

        return run, how


class LlamaBlockDecode(Workload):
    name = "Llama block decode step bf16 B8, one token against 4096 cached positions, compiled + HIP graph"
    dtype = "bf16"
    kernel = "compiled decode step (norms, rotary, 7 row-streaming dense launches incl. the gated one, key-split attention)"
    traffic_key = None
    # what one step must read: the seven weight matrices and the two caches (activations are a few KB)
    work = 2 * (4 * 4096 * 4096 + 3 * 4096 * 11008) + 2 * 8 * 32 * 4096 * 128 * 2
    n_sets = 1
    cpu_warmups = 1
    B, S = 8, 4096

    def _inputs(self, torch, dev):
        from oracle import eager, inputs

        _, p = inputs.c5_llama_block(B=1, S=1, device=dev)
        g = torch.Generator().manual_seed(1)
        x = torch.randn(self.B, 1, 4096, generator=g).bfloat16().to(dev)
        kc, vc = (torch.randn(self.B, 32, self.S, 128, generator=g).bfloat16().to(dev) for _ in range(2))
        cos, sin = eager.rope_tables(self.S, 128, device=dev, dtype=torch.bfloat16)
        return x, p, kc, vc, cos[-1].contiguous(), sin[-1].contiguous()

    def setup(self, torch, dev):
        from oracle import eager
        from xpu_graph_amd import HIPGraphRunner, mi355x_compiler

        self.torch = torch
        x, p, kc, vc, cos, sin = self._inputs(torch, dev)
        names = sorted(p)

        def step(x, kc, vc, cos, sin, *ws):
            return eager.llama_block_decode_eager(x, dict(zip(names, ws)), kc, vc, cos, sin, n_heads=32)

        self.eager_fn = step
        self.args = (x, kc, vc, cos, sin, *[p[n] for n in names])
        compiled = torch.compile(step, backend=mi355x_compiler(), dynamic=False)
        with torch.no_grad():
            compiled(*self.args)  # compile outside the capture
        self.runner = HIPGraphRunner(compiled)
        self.runner.capture(*self.args, clone_args=False)

    def op_call(self, i):
        return self.runner(*self.args)

    abi_call = op_call

    def check(self, torch):
        got = [t.clone() for t in self.op_call(0)]
        with torch.no_grad():
            want = self.eager_fn(*self.args)
            self.eager_ms = _events_time(torch, lambda i: self.eager_fn(*self.args), 1, 20, 5) * 1e3
        for a, b in zip(got, want):
            assert (a.float() - b.float()).abs().mean().item() < 2e-2

    def cpu_fn(self, torch):
        from oracle import eager

        x, p, kc, vc, cos, sin = self._inputs(torch, "cpu")
        fn, how = _default_path_compile(lambda x, kc, vc: eager.llama_block_decode_eager(x, p, kc, vc, cos, sin, n_heads=32))

        def run():
            with torch.no_grad():
                return fn(x, kc, vc)

        return run, how


class LlamaBlockTrainC5(LlamaBlockC5):
    name = "C5 Llama decoder block bf16 B4 S2048 compiled training step"
    kernel = "compiled training step"
    work = 3 * LlamaBlockC5.work  # one forward, two products per forward product in the backward
    cpu_work = work // 4            # the CPU leg runs one of the four batch entries
    cpu_warmups = 0

    def setup(self, torch, dev):
        from oracle import eager, inputs
        from xpu_graph_amd import OptLevel, Target, XpuGraph, XpuGraphConfig

        self.torch = torch
        x, p = inputs.c5_llama_block(device=dev)
        names = sorted(p)

        def block(x, *ws):
            return eager.llama_block_eager(x, dict(zip(names, ws)), n_heads=32)

        self.eager_fn = block
        self.args = [x.requires_grad_(True)] + [p[n].requires_grad_(True) for n in names]
        backend = XpuGraph(XpuGraphConfig(is_training=True, target=Target.mi355x, opt_level=OptLevel.level2, enable_cache=False))
        self.fn = torch.compile(block, backend=backend, dynamic=False)

    def _step(self, fn):
        return self.torch.autograd.grad(fn(*self.args).float().pow(2).mean(), self.args)

    def op_call(self, i):
        return self._step(self.fn)

    abi_call = op_call

    def check(self, torch):
        got = self.op_call(0)
        want = self._step(self.eager_fn)
        self.eager_ms = _events_time(torch, lambda i: self._step(self.eager_fn), 1, 3, 1) * 1e3
        for a, b in zip(got, want):  # eager bf16 is the yardstick here; tests/test_gpu_training.py compares both with fp32 autograd
            assert (a.float() - b.float()).abs().mean().item() <= 0.1 * b.float().abs().mean().item() + 1e-6

    def cpu_fn(self, torch):
        from oracle import eager, inputs

        x, p = inputs.c5_llama_block(B=1, device="cpu")
        names = sorted(p)
        args = [x.requires_grad_(True)] + [p[n].requires_grad_(True) for n in names]

        def run():
            return torch.autograd.grad(eager.llama_block_eager(args[0], dict(zip(names, args[1:])), n_heads=32).float().pow(2).mean(), args)

        return run, "eager autograd on one batch entry (B1 S2048)"


# ---- roofline.traffic: HBM bytes per launch from two rocprofv3 --pmc runs of this file -------------------------
# kernel of each workload as it appears in rocprofv3's Kernel_Name column (mangled or demangled): all of `has`, and
# any of `any` when given
TRAFFIC_KERNELS = {
    "c2_add_layernorm": {"has": ["norm_rows_kernel"], "any": ["Lb1EEE", "true>"]},
    "c1_rmsnorm": {"has": ["norm_rows_kernel"], "any": ["IffLi", "<float, float"]},
    "c3a_slice_cat": {"has": ["slice_cat_kernel"]},
    "c3b_addn": {"has": ["addn_kernel"]},
    "c4_dense_bf16": {"has": ["gemm_dma_split_kernel"], "any": ["IDF16bDF16b", "<__bf16", "<__hip_bfloat16"]},
    "c4_dense_fp8": {"has": ["gemm_dma_split_kernel"], "any": ["IhDF16b", "<unsigned char"]},
    "c5_dense_glu": {"has": ["gemm_glu_"]},
    "c5_sdpa": {"has": ["sdpa_fwd_kernel"]},
    "c4_dense_at": {"has": ["gemm_dma_kernel"], "any": ["ALayoutE1", "ALayout)1"]},
}
COPY_YARDSTICK_BYTES = 64 << 20


def copy_yardstick(torch, dev):
    """A few launches of the plain copy kernel over 64 MiB: the known-size dispatch that tells what one unit of
    FETCH_SIZE / WRITE_SIZE is worth on this box."""
    from xpu_graph_amd import _lib

    a = torch.empty(COPY_YARDSTICK_BYTES, dtype=torch.uint8, device=dev)
    b = torch.empty_like(a)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(5):
        _lib.check(_lib.lib().xg_copy_bytes(_p(a), _p(b), COPY_YARDSTICK_BYTES, st), "xg_copy_bytes")
    torch.cuda.synchronize()


def _median_counter(csv_dir, counter):
    """kernel name -> median `counter` per dispatch, from the *_counter_collection.csv files under csv_dir."""
    import csv
    import glob

    vals = {}
    for path in glob.glob(os.path.join(csv_dir, "**", "*counter_collection.csv"), recursive=True):
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] == counter:
                    vals.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
    out = {}
    for k, v in vals.items():
        v.sort()
        out[k] = (v[len(v) // 2], len(v))
    return out


def traffic_from(fetch_dir, write_dir, out_path=TRAFFIC_FILE):
    """Turns `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` runs of this file into profiles/traffic.json:
    bytes per launch = counter x (64 MiB / what the same counter reads for the 64 MiB copy kernel)."""
    fetch, write = _median_counter(fetch_dir, "FETCH_SIZE"), _median_counter(write_dir, "WRITE_SIZE")

    def pick(table, spec):
        hits = [(v, k) for k, v in table.items() if all(h in k for h in spec["has"]) and ("any" not in spec or any(a in k for a in spec["any"]))]
        return max(hits, key=lambda h: h[0][1]) if hits else None  # the variant with the most dispatches is the benchmark's

    copy_spec = {"has": ["xg", "copy_kernel"]}
    cf, cw = pick(fetch, copy_spec), pick(write, copy_spec)
    if cf is None or cw is None:
        raise SystemExit("the counter runs hold no xg copy_kernel dispatch: run bench.py itself under rocprofv3")
    unit_f, unit_w = COPY_YARDSTICK_BYTES / cf[0][0], COPY_YARDSTICK_BYTES / cw[0][0]
    table = {}
    for key, spec in TRAFFIC_KERNELS.items():
        f, w = pick(fetch, spec), pick(write, spec)
        if f is None or w is None:
            continue
        table[key] = {
            "bytes_per_launch": round(f[0][0] * unit_f + w[0][0] * unit_w),
            "fetch_bytes": round(f[0][0] * unit_f),
            "write_bytes": round(w[0][0] * unit_w),
            "dispatches": [f[0][1], w[0][1]],
            "kernel": f[1][:120],
            "from": f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, median per dispatch; one counter unit = {unit_f:.0f} / {unit_w:.0f} bytes by the 64 MiB copy kernel",
        }
    with open(out_path, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"wrote {out_path}: {sorted(table)}")


HEADLINE = AddLayerNormC2
OTHERS = [RmsNormC1, SliceCatC3a, AddNC3b, DenseC4, DenseFp32, DenseFp8C4, DenseGluC5, SdpaC5, SdpaBackwardC5, DenseWeightGradC4, DenseDecode, DenseDecodeFp8, SdpaDecode,
          LlamaBlockDecode, LlamaBlockC5, LlamaBlockTrainC5]


def run_workload(torch, dev, wl, steps, warmup, with_cpu=True):
    wl.setup(torch, dev)
    wl.check(torch)
    peak = HBM_PEAK_GBPS if wl.bound == "hbm" else {"fp8": FP8_PEAK_TFLOPS, "f32": FP32_PEAK_TFLOPS}.get(wl.dtype, BF16_PEAK_TFLOPS)
    scale = 1e9 if wl.bound == "hbm" else 1e12
    n_sets = getattr(wl, "n_sets", N_SETS)
    entry = _traffic_table().get(getattr(wl, "traffic_key", None) or "", None)
    traffic = entry["bytes_per_launch"] if entry else None
    t_op = _wall_time(torch, wl.op_call, n_sets, steps, warmup)
    t_k = _events_time(torch, wl.abi_call, n_sets, max(steps, 100), max(warmup, 20))
    res = {
        "workload": wl.name,
        "dtype": wl.dtype,
        "value": wl.work / t_op / scale,
        "unit": "GB/s" if wl.bound == "hbm" else "TFLOP/s",
        "ms_per_step": t_op * 1e3,
        "roofline": {
            "bound": wl.bound,
            "kernel": wl.kernel,
            "achieved": wl.work / t_k / scale,
            "peak": peak,
            "unit": "GB/s" if wl.bound == "hbm" else "TFLOP/s",
            "frac": wl.work / t_k / scale / peak,
            "kernel_us": t_k * 1e6,
            "traffic": traffic,
        },
    }
    clock = _shader_clock_ghz(torch, wl.abi_call, n_sets, t_k, wl.name)
    if clock:
        # the engine clock the GPU held under this kernel; for an MFMA kernel also the fraction of the peak scaled to that
        # clock (`frac` prices against the published peak, which assumes the nominal clock)
        res["roofline"]["clock_ghz"] = clock
        if wl.bound == "mfma":
            res["roofline"]["frac_at_clock"] = res["roofline"]["frac"] * NOMINAL_CLOCK_GHZ / clock
    if getattr(wl, "zero_operands", False):
        # The same launches with every matrix operand zeroed: the identical instruction stream at the power of operands
        # that toggle no bits.  Beside `frac` it tells how much of the gap to the peak is the engine clock the GPU gives
        # this kernel on random data, and how much is the kernel's own.
        for group in wl.sets:
            for t in group:
                if t.dim() >= 2:
                    t.zero_()
        t_z = _events_time(torch, wl.abi_call, n_sets, max(steps, 100), max(warmup, 20))
        res["roofline"]["zero_operands"] = {
            "kernel_us": t_z * 1e6,
            "frac": wl.work / t_z / scale / peak,
            "clock_ghz": _shader_clock_ghz(torch, wl.abi_call, n_sets, t_z, wl.name + " (zero operands)"),
        }
    if traffic and wl.bound == "hbm":
        # what the bytes that really moved (whole 128-byte lines) amount to per second: beside `frac`, which prices the
        # algorithmic bytes only
        res["roofline"]["traffic_gbps"] = traffic / t_k / 1e9
    if with_cpu:
        fn, how = wl.cpu_fn(torch)
        t_cpu, n = _cpu_time(fn, warmups=getattr(wl, "cpu_warmups", 2))
        res["cpu_baseline"] = {
            "value": getattr(wl, "cpu_work", wl.work) / t_cpu / scale,
            "unit": res["unit"],
            "cores": torch.get_num_threads(),
            "host_cpu_count": os.cpu_count(),
            "kind": "port",
            "sample": f"{'bounded sample' if hasattr(wl, 'cpu_work') else 'full size'}, {n} runs, median {t_cpu * 1e3:.1f} ms",
        }
        print(f"[bench] cpu baseline of {wl.name}: {how}", file=sys.stderr)
    if hasattr(wl, "eager_ms"):
        res["eager_gpu_ms"] = wl.eager_ms
    return res


def _rounded(obj):
    """Floats to six significant digits: the line is read by people and by a log tail of bounded length."""
    if isinstance(obj, float):
        return float(f"{obj:.6g}")
    if isinstance(obj, dict):
        return {k: _rounded(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return [_rounded(v) for v in obj]
    return obj


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", default=None, help="headline only, or a substring of another workload's name")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"), default=None,
                    help="no GPU work: read two rocprofv3 --pmc output folders of earlier runs of this file and write profiles/traffic.json")
    args = ap.parse_args()
    if args.traffic_from:
        traffic_from(*args.traffic_from)
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the hot path has no cross-GPU part; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the mi355x path has no CPU fallback)", file=sys.stderr)
        sys.exit(1)
    import logging

    import xpu_graph_amd.ops  # noqa: F401

    for handler in logging.getLogger("xpu_graph").handlers:  # stdout carries the one JSON line only
        if isinstance(handler, logging.StreamHandler):
            handler.setStream(sys.stderr)

    # The CPU baseline uses the cores this job owns: OMP_NUM_THREADS when the launcher sets it (a GPU box hands one job
    # a share of a larger host, and more threads than that share only fight each other), else every core.  Both
    # counts are reported: cpu_baseline.cores (threads used) and cpu_baseline.host_cpu_count.
    torch.set_num_threads(min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))))
    dev = torch.device("cuda:0")
    copy_yardstick(torch, dev)
    head = run_workload(torch, dev, HEADLINE(), args.steps, args.warmup, with_cpu=not args.no_cpu)
    out = {
        "metric": "fused-op GB/s (residual-add + LayerNorm, % of HBM peak in roofline.frac)",
        "value": head["value"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic",
        "config": {"workload": head["workload"], "buffer_sets": N_SETS},
        "roofline": head["roofline"],
    }
    if "cpu_baseline" in head:
        out["cpu_baseline"] = head["cpu_baseline"]
    others = []
    if args.only != "headline":
        for cls in OTHERS:
            wl = cls()
            if args.only and args.only.lower() not in wl.name.lower():
                continue
            others.append(run_workload(torch, dev, wl, args.steps, args.warmup, with_cpu=not args.no_cpu))
            del wl
            torch.cuda.empty_cache()
    out["configs"] = others
    entries = [e for e in _traffic_table().values() if e.get("from")]
    # said once for every roofline.traffic in the line (the whole line has to stay well under the 16 000 characters a log tail keeps)
    out["traffic_source"] = f"profiles/traffic.json ({entries[0]['from']})" if entries else None
    print(json.dumps(_rounded(out), separators=(",", ":")))


if __name__ == "__main__":
    main()
