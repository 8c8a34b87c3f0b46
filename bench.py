#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of a random-init Llama-3-8B-architecture model with
int4 weight-only (group 64) quantization on every nn.Linear, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decoded token (one pass of every quantized linear over one activation row).  The timed
region is K replays of the HIP graph of the decode step with all weights resident in HBM, bracketed by
torch.cuda.synchronize().  One JSON line is printed with:
  value        tokens/s
  roofline     the int4wo GEMV kernel over the 129 linear launches of one decoded token: algorithmic bytes
               (N*K*(1/2 + 4/g) + 2*M*K + 2*M*N per launch) / kernel time, kernel time taken from HIP events
               that carry each kernel's own begin / end timestamps
  cpu_baseline the C oracle (dequantize_affine + fp32 linear, 1 thread) timed on one transformer layer's
               linears and scaled to a whole token
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def int4wo_bytes(N, K, g, M=1):
    return N * K * (0.5 + 4.0 / g) + 2 * M * K + 2 * M * N


def _hip():
    for name in ("libamdhip64.so.7", "libamdhip64.so"):
        try:
            return ctypes.CDLL(name)
        except OSError:
            continue
    raise RuntimeError("HIP runtime not found")


class KernelTimer:
    """HIP event pairs armed on the linear launch: elapsed time = the kernel's own duration."""

    def __init__(self, n):
        self.hip = _hip()
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.pairs = []
        for _ in range(n):
            a, b = ctypes.c_void_p(), ctypes.c_void_p()
            assert self.hip.hipEventCreate(ctypes.byref(a)) == 0
            assert self.hip.hipEventCreate(ctypes.byref(b)) == 0
            self.pairs.append((a, b))

    def elapsed_us(self, i):
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), self.pairs[i][0], self.pairs[i][1])
        assert rc == 0, f"hipEventElapsedTime failed: {rc}"
        return ms.value * 1e3

    def close(self):
        for a, b in self.pairs:
            self.hip.hipEventDestroy(a)
            self.hip.hipEventDestroy(b)


def roofline_leg(model, passes=3):
    """Time the GEMV kernel alone over the linear launches of one decoded token (M=1), `passes` times: per layer
    norm + wqkv, wo + residual, norm + gate/up SwiGLU over the interleaved pair, w2 + residual, then norm + head:
    the same entry points, weights and order as the decode step, 4 * n_layer + 1 launches."""
    import torch

    from ao_amd import _lib

    L = _lib.lib()
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    cfg = model.config
    x = torch.randn(1, cfg.dim, device=dev).bfloat16()
    xf = torch.randn(1, cfg.intermediate_size, device=dev).bfloat16()
    res = torch.randn(1, cfg.dim, device=dev).bfloat16()
    launches = []  # (callable, algorithmic bytes)

    def add(fn, nbytes):
        launches.append((fn, nbytes))

    def plain(lay, xin, residual=None, norm=None):
        y = torch.empty(1, lay.N, dtype=torch.bfloat16, device=dev)
        common = (lay.packed_weight.data_ptr(), lay.scale_and_zero.data_ptr(), lay.N, lay.group_size, None)
        if norm is not None:
            return lambda: L.ao_amd_int4wo_rmsnorm_linear(xin.data_ptr(), 1, lay.K, lay.K, norm.weight.data_ptr(),
                                                          float(norm.eps), *common, y.data_ptr(), _lib.BF16, lay.N, st), y
        if residual is not None:
            return lambda: L.ao_amd_int4wo_linear_residual(xin.data_ptr(), 1, lay.K, lay.K, *common, residual.data_ptr(),
                                                           lay.N, y.data_ptr(), lay.N, st), y
        return lambda: L.ao_amd_int4wo_linear(xin.data_ptr(), 1, lay.K, lay.K, *common, y.data_ptr(), _lib.BF16,
                                              lay.N, st), y

    keep = []
    for b in model.layers:
        lay = b.attention.wqkv.weight.layout_tensor
        ks = model.qkv_ksplit(lay.N)
        if ks > 1:  # as the decode step launches it: fp32 partial rows over `ks` runs of K
            yp = torch.empty(ks, 1, lay.N, dtype=torch.float32, device=dev)
            norm = b.attention_norm
            fn = (lambda lay=lay, norm=norm, yp=yp, ks=ks: L.ao_amd_int4wo_linear_partials(
                x.data_ptr(), 1, lay.K, lay.K, norm.weight.data_ptr(), float(norm.eps), lay.packed_weight.data_ptr(),
                lay.scale_and_zero.data_ptr(), lay.N, lay.group_size, ks, yp.data_ptr(), lay.N, st))
            add(fn, int4wo_bytes(lay.N, lay.K, lay.group_size)); keep.append(yp)
        else:
            fn, y = plain(lay, x, norm=b.attention_norm)
            add(fn, int4wo_bytes(lay.N, lay.K, lay.group_size)); keep.append(y)
        lay = b.attention.wo.weight.layout_tensor
        fn, y = plain(lay, x, residual=res)
        add(fn, int4wo_bytes(lay.N, lay.K, lay.group_size)); keep.append(y)
        pair, pair_q, group, n_ff = model._gate_up_pair(b.feed_forward)
        yff = torch.empty(1, n_ff, dtype=torch.bfloat16, device=dev)
        norm = b.ffn_norm
        add(lambda pair=pair, pair_q=pair_q, group=group, n_ff=n_ff, norm=norm, yff=yff:
            L.ao_amd_int4wo_swiglu_interleaved(x.data_ptr(), 1, cfg.dim, cfg.dim, norm.weight.data_ptr(), float(norm.eps),
                                               pair.data_ptr(), pair_q.data_ptr(), n_ff, group, yff.data_ptr(), n_ff, st),
            int4wo_bytes(2 * n_ff, cfg.dim, group) - 2 * n_ff)
        keep.append(yff)
        lay = b.feed_forward.w2.weight.layout_tensor
        fn, y = plain(lay, xf, residual=res)
        add(fn, int4wo_bytes(lay.N, lay.K, lay.group_size)); keep.append(y)
    lay = model.output.weight.layout_tensor
    fn, y = plain(lay, x, norm=model.norm)
    add(fn, int4wo_bytes(lay.N, lay.K, lay.group_size)); keep.append(y)

    timer = KernelTimer(len(launches))
    total_bytes = sum(nb for _, nb in launches)
    # the average launch duration over the passes (every pass streams all 4.2 GB of weights: no launch finds its weight cached)
    best = [0.0] * len(launches)
    for _ in range(passes):
        for i, (fn, _) in enumerate(launches):
            L.ao_amd_profile_next_linear(timer.pairs[i][0], timer.pairs[i][1])
            _lib.check(fn())
        torch.cuda.synchronize()
        for i in range(len(launches)):
            best[i] += timer.elapsed_us(i) / passes
    timer.close()
    total_us = sum(best)
    achieved = total_bytes / total_us / 1e3  # GB/s
    return {
        "bound": "hbm",
        "kernel": "ao::int4wo_gemv1_kernel / int4wo_gemv2_kernel (M=1, g=64)",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "launches": len(launches),
        "bytes_per_launch": round(total_bytes / len(launches)),
        "avg_launch_us": round(total_us / len(launches), 3),
        "us_by_linear": {k: round(sum(best[i] for i in range(j, len(launches) - 1, 4)) / len(model.layers), 2)
                         for j, k in enumerate(("norm_wqkv", "wo_residual", "norm_w1w3_swiglu", "w2_residual"))}
        | {"output": round(best[-1], 2)},
        "traffic": _traffic_from_profile(),
        # the counters need rocprofv3 --pmc runs of their own: this figure is read from the committed summary of
        # those runs, it is not measured by this invocation
        "traffic_source": "profiles/int4wo_gemv_llama3_8b_decode_pmc.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                          "scaled by a copy kernel of known size; not measured in this run)",
    }


def _traffic_from_profile():
    """HBM bytes per launch of the GEMV kernel from the committed rocprofv3 --pmc summary (its
    'traffic_bytes_per_launch:' line), if one exists."""
    path = os.path.join(ROOT, "profiles", "int4wo_gemv_llama3_8b_decode_pmc.txt")
    if os.path.exists(path):
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return int(float(line.split(":", 1)[1]))
    return None


def copy_calibration(mib=256):
    """One elementwise copy kernel of known size (reads and writes `mib` MiB) for scaling the FETCH_SIZE /
    WRITE_SIZE counters of a rocprofv3 --pmc run of this script."""
    import torch

    src = torch.ones(mib << 18, dtype=torch.float32, device="cuda:0")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    torch.add(src, 1.0, out=dst)
    torch.cuda.synchronize()


def cpu_baseline_leg(config, group=64, min_seconds=10.0):
    """C oracle on one layer's linears (M=1): dequantize_affine + fp32 linear, one thread."""
    import numpy as np

    import oracle as O

    O.lib()
    rng = np.random.default_rng(1234)
    dim, ffn = config.dim, config.intermediate_size
    qkv = (config.n_head + 2 * config.n_local_heads) * config.head_dim
    shapes = [(qkv, dim), (dim, dim), (ffn, dim), (ffn, dim), (dim, ffn)]  # (N, K)
    prepared = []
    for N, K in shapes:
        w = O.f32_to_bf16_bits((rng.standard_normal((N, K), dtype=np.float32) * 0.02))
        codes, scale, zero = O.int4wo_quantize(w, O.BF16, group, N, K)
        x = O.f32_to_bf16_bits(rng.standard_normal((1, K), dtype=np.float32))
        prepared.append((codes, scale, zero, x))
    layer_params = sum(n * k for n, k in shapes)
    t_layer, reps = 0.0, 0
    while t_layer < min_seconds and reps < 50:
        t0 = time.perf_counter()
        for codes, scale, zero, x in prepared:
            dq = O.dequantize_affine(codes, O.I32, (1, group), scale, O.BF16, zero, O.BF16, 0, 15, 1, O.BF16)
            O.linear(x, O.BF16, dq, O.BF16)
        t_layer += time.perf_counter() - t0
        reps += 1
    per_layer = t_layer / reps
    # the reference's CPU-runnable case step by step: one bf16 weight [4096, 4096], g = 128, x [1, 4096]
    w = O.f32_to_bf16_bits((rng.standard_normal((4096, 4096), dtype=np.float32) * 0.02))
    x = O.f32_to_bf16_bits(rng.standard_normal((1, 4096), dtype=np.float32))
    c1 = {}
    t0 = time.perf_counter()
    codes, scale, zero = O.int4wo_quantize(w, O.BF16, 128, 4096, 4096)
    c1["choose_qparams+quantize"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    O.int4wo_pack(codes, scale, zero, 128)
    c1["pack"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    dq = O.dequantize_affine(codes, O.I32, (1, 128), scale, O.BF16, zero, O.BF16, 0, 15, 1, O.BF16)
    c1["dequantize"] = time.perf_counter() - t0
    t0 = time.perf_counter()
    O.linear(x, O.BF16, dq, O.BF16)
    c1["linear"] = time.perf_counter() - t0
    head_params = config.vocab_size * dim
    per_token = per_layer * config.n_layer + per_layer * head_params / layer_params
    torch_leg = _torch_cpu_leg(config, group, shapes, layer_params, head_params)
    port = {
        "value": round(1.0 / per_token, 4),
        "unit": "tokens/s",
        "cores": 1,
        "kind": "port",
        "sample": (f"C oracle dequantize_affine+fp32 linear (M=1, g={group}) on one transformer layer's five linears "
                   f"({layer_params / 1e6:.0f}M weights), {reps} repetitions, {per_layer:.2f} s per layer; scaled to "
                   f"{config.n_layer} layers + vocabulary head"),
        "config0_steps_ms": {k: round(v * 1e3, 1) for k, v in c1.items()},
    }
    # headline: the reference's CPU route for a quantized weight with every host thread (the oracle's arithmetic run by
    # torch's CPU kernels op by op); the one-thread C port and the fused CPU kernel of the aten operator beside it
    fused = torch_leg.pop("aten_int4pack_mm", None)
    out = dict(torch_leg)
    out["c_port_one_thread"] = port
    if fused is not None:
        out["aten_int4pack_mm"] = fused
    return out


def _torch_cpu_leg(config, group, shapes, layer_params, head_params, min_seconds=5.0):
    """The same linears on the host with torch's own CPU kernels and every thread torch is configured with, beside the
    scalar port.  `value`: the reference's CPU route for a quantized weight, op by op in bf16 as its tensor subclass
    does it (dequantize_affine: (q - 8) * scale, + zero, then F.linear; torchao/dtypes/affine_quantized_tensor.py:
    dequantize() fallback of _quantized_linear_op).  `aten_int4pack_mm`: the fused CPU kernel of the operator the
    reference dispatches to on a GPU (aten._weight_int4pack_mm; its CPU build is _weight_int4pack_mm_for_cpu here),
    the fastest CPU execution of these linears this image offers."""
    import torch
    import torch.nn.functional as F

    gen = torch.Generator().manual_seed(1234)
    prepared = []
    for N, K in shapes:
        q = torch.randint(0, 16, (N, K), dtype=torch.int32, generator=gen)
        scale = (torch.rand(N, K // group, generator=gen) * 0.01 + 1e-3).bfloat16()
        zero = (torch.randn(N, K // group, generator=gen) * 0.01).bfloat16()
        prepared.append((torch.randn(1, K, generator=gen).bfloat16(), q, scale, zero))

    def eager_layer():
        for x, q, scale, zero in prepared:
            N, K = q.shape
            w = ((q.view(N, K // group, group) - 8).to(torch.bfloat16) * scale.unsqueeze(-1) + zero.unsqueeze(-1)).view(N, K)
            F.linear(x, w)

    def timed(fn, max_reps):
        fn()
        total, reps = 0.0, 0
        while total < min_seconds and reps < max_reps:
            t0 = time.perf_counter()
            fn()
            total += time.perf_counter() - t0
            reps += 1
        return total / reps, reps

    scale_up = config.n_layer + head_params / layer_params
    per_layer, reps = timed(eager_layer, 50)
    out = {
        "value": round(1.0 / (per_layer * scale_up), 4),
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": (f"torch eager on the host, all threads: dequantize_affine op by op in bf16 ((q - 8) * scale + zero), then "
                   f"F.linear (M=1, g={group}) on one transformer layer's five linears ({layer_params / 1e6:.0f}M weights, "
                   f"1.7 GB of int32 codes and bf16 weights per pass: not cache resident), {reps} repetitions, "
                   f"{per_layer * 1e3:.1f} ms per layer; scaled to {config.n_layer} layers + vocabulary head"),
    }
    if hasattr(torch.ops.aten, "_weight_int4pack_mm_for_cpu"):
        packed = [(x, torch.ops.aten._convert_weight_to_int4pack_for_cpu(q, 2),
                   torch.stack([scale.t(), zero.t()], dim=-1).contiguous()) for x, q, scale, zero in prepared]
        # distinct copies of the layer (12 x 123 MB), walked in turn, so that a pass streams its weights from memory as a
        # decode step over 32 different layers does, instead of re-reading one layer from the last-level cache
        n_copies = 12
        layers = [packed] + [[(x, p.clone(), sz.clone()) for x, p, sz in packed] for _ in range(n_copies - 1)]

        def fused_layers():
            for layer in layers:
                for x, p, sz in layer:
                    torch.ops.aten._weight_int4pack_mm_for_cpu(x, p, group, sz)

        per_pass, reps_f = timed(fused_layers, 200)
        per_layer_f = per_pass / n_copies
        out["aten_int4pack_mm"] = {"value": round(1.0 / (per_layer_f * scale_up), 3), "unit": "tokens/s",
                                   "cores": torch.get_num_threads(), "kind": "aten._weight_int4pack_mm_for_cpu (fused CPU kernel of the operator the reference dispatches to)",
                                   "sample": (f"{n_copies} distinct copies of one layer's five linears walked in turn ({n_copies * 123} MB "
                                              f"of packed weights per pass), {reps_f} passes, {per_layer_f * 1e3:.2f} ms per layer")}
    return out


MFMA_PEAK_TFLOPS = 2500.0  # dense bf16 / fp16 MFMA, published

SWEEP_ROTATE_BYTES = 640 << 20  # the sweeps rotate over weight copies totalling at least this much
LLAMA3_8B_SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096)]  # (N, K)


def _time_linear(L, launch, iters, armed=True):
    """Median of the kernel's own duration (us) over `iters` launches; launch(i) is given the iteration number so
    that it can rotate over copies of the weight (each launch then reads HBM, not the last-level cache).  Linear
    kernels are timed by events armed on the launch itself; entry points without that hook (`armed=False`) by
    stream events recorded around the launch."""
    import torch

    for i in range(10):
        launch(i)
    if not armed:
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        for i in range(iters):
            evs[i][0].record()
            launch(i + 10)
            evs[i][1].record()
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) * 1e3 for a, b in evs)[iters // 2]
    timer = KernelTimer(iters)
    for i in range(iters):
        L.ao_amd_profile_next_linear(timer.pairs[i][0], timer.pairs[i][1])
        launch(i + 10)
    torch.cuda.synchronize()
    durs = sorted(timer.elapsed_us(i) for i in range(iters))
    timer.close()
    return durs[len(durs) // 2]


def replayed_us(fn, n, reps):
    """Device time per call of fn(0) .. fn(n - 1) from a replayed HIP graph of the n calls (no host dispatch in the figure)."""
    import torch

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for i in range(n):
            fn(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(n):
                fn(i)
    for _ in range(2):
        graph.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        graph.replay()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / (reps * n)


def sweep(kind, iters=100):
    """Per-kernel lines for the shapes of the other benchmark configurations: int4 GEMV (M in 1, 4; g in 64, 128),
    int4 GEMM (M in 16 .. 2048, g=64), the FP6 e3m2 linear (M in 1, 16, 128, 512) and the int8 weight-only linear
    (M in 1, 4, 16); one JSON line per case.  `tinygemm` times PyTorch's own int4 matmul operator beside this library's."""
    import torch

    from ao_amd import _lib

    L = _lib.lib()
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator(device=dev).manual_seed(0)
    if kind in ("gemv", "gemm"):
        cases = ([(N, K, M, g) for (N, K) in LLAMA3_8B_SHAPES for g in (64, 128) for M in (1, 4)] if kind == "gemv" else
                 [(N, K, M, 64) for (N, K) in LLAMA3_8B_SHAPES for M in (16, 128, 512, 2048) if N * M < 1 << 28])
        for N, K, M, g in cases:
            _, _, pb, qb = _lib.packed_shape(N, K, g)
            w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).bfloat16()
            copies = max(2, -(-SWEEP_ROTATE_BYTES // pb))
            packed = torch.empty(copies, pb // 4, dtype=torch.int32, device=dev)
            qp = torch.empty(copies, qb // 4, dtype=torch.int32, device=dev)
            _lib.check(L.ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, K, g, packed.data_ptr(), qp.data_ptr(), st))
            packed[1:] = packed[0]
            qp[1:] = qp[0]
            x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
            y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            us = _time_linear(L, lambda i: _lib.check(L.ao_amd_int4wo_linear(
                x.data_ptr(), M, K, K, packed[i % copies].data_ptr(), qp[i % copies].data_ptr(), N, g, None,
                y.data_ptr(), _lib.BF16, N, st)), iters)
            gbs = int4wo_bytes(N, K, g, M) / us / 1e3
            tfs = 2.0 * M * N * K / us / 1e6
            line = {"kernel": "int4wo_linear", "N": N, "K": K, "M": M, "group": g, "us": round(us, 2),
                    "GBs": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 4),
                    "TFLOPs": round(tfs, 2), "mfma_frac": round(tfs / MFMA_PEAK_TFLOPS, 4)}
            if kind == "gemv":
                # for information: the same launch on one copy of the weight (served from the 256 MB last-level
                # cache when it fits); every other figure is the cold one above
                line["us_warm"] = round(_time_linear(L, lambda i: _lib.check(L.ao_amd_int4wo_linear(
                    x.data_ptr(), M, K, K, packed[0].data_ptr(), qp[0].data_ptr(), N, g, None, y.data_ptr(), _lib.BF16,
                    N, st)), iters), 2)
            print(json.dumps(line), flush=True)
            if kind == "gemm":
                from ao_amd import ops

                if ops.int4wo_two_pass(M, N, K):
                    # what torch.ops.torchao.int4wo_linear runs at this size: the dequantize kernel into a bf16
                    # scratch weight, then the library bf16 GEMM; timed with stream events around the op
                    shp_p, shp_q = ops.int4wo_packed_shapes(N, K, g)
                    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
                    for i in range(iters + 10):
                        pi, qi = packed[i % copies].view(shp_p), qp[i % copies].view(shp_q)
                        if i >= 10:
                            evs[i - 10][0].record()
                        ops.int4wo_linear(x, pi, qi, g, N)
                        if i >= 10:
                            evs[i - 10][1].record()
                    torch.cuda.synchronize()
                    us2 = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)[iters // 2]
                    tfs2 = 2.0 * M * N * K / us2 / 1e6
                    print(json.dumps({"kernel": "int4wo_linear op: int4wo_dequantize + library bf16 GEMM", "N": N, "K": K,
                                      "M": M, "group": g, "us": round(us2, 2), "TFLOPs": round(tfs2, 2),
                                      "mfma_frac": round(tfs2 / MFMA_PEAK_TFLOPS, 4)}), flush=True)
                if M == 2048 or (M == 512 and N * 2048 >= 1 << 28):
                    wd = torch.empty(N, K, dtype=torch.bfloat16, device=dev)
                    usd = _time_linear(L, lambda i: _lib.check(L.ao_amd_int4wo_dequantize(
                        packed[i % copies].data_ptr(), qp[i % copies].data_ptr(), N, K, g, wd.data_ptr(), st)), iters,
                        armed=False)
                    gbd = (N * K * (0.5 + 4.0 / g) + 2.0 * N * K) / usd / 1e3
                    print(json.dumps({"kernel": "int4wo_dequantize", "N": N, "K": K, "group": g, "us": round(usd, 2),
                                      "GBs": round(gbd, 1), "hbm_frac": round(gbd / HBM_PEAK_GBS, 4)}), flush=True)
                    del wd
            del w, packed, qp, x, y
    elif kind == "fp6":
        for N, K in [(4096, 4096), (14336, 4096), (4096, 14336)]:
            w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).half()
            tc = torch.empty(N * K * 3 // 4, dtype=torch.uint8, device=dev)
            sc = torch.empty(N, dtype=torch.float16, device=dev)
            _lib.check(L.ao_amd_fp6_quantize_pack(w.data_ptr(), _lib.F16, N, K, 3, 2, tc.data_ptr(), sc.data_ptr(), st))
            nbytes = ctypes.c_int64()
            _lib.check(L.ao_amd_fp6_native_bytes(N, K, ctypes.byref(nbytes)))
            copies = max(2, -(-SWEEP_ROTATE_BYTES // nbytes.value))
            native = torch.empty(copies, nbytes.value, dtype=torch.uint8, device=dev)
            _lib.check(L.ao_amd_fp6_repack(tc.data_ptr(), N, K, 6, native.data_ptr(), st))
            native[1:] = native[0]
            for M in (1, 16, 128, 512):
                x = torch.randn(M, K, device=dev, generator=gen).half()
                y = torch.empty(M, N, dtype=torch.float16, device=dev)
                us = _time_linear(L, lambda i: _lib.check(L.ao_amd_fp6_linear(
                    x.data_ptr(), M, K, native[i % copies].data_ptr(), sc.data_ptr(), N, 3, 2, y.data_ptr(), st)), iters)
                gbs = (N * K * 0.75 + 2 * N + 2 * M * K + 2 * M * N) / us / 1e3
                tfs = 2.0 * M * N * K / us / 1e6
                print(json.dumps({"kernel": "fp6_linear_e3m2", "N": N, "K": K, "M": M, "us": round(us, 2),
                                  "GBs": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 4),
                                  "TFLOPs": round(tfs, 2), "mfma_frac": round(tfs / MFMA_PEAK_TFLOPS, 4)}), flush=True)
            del w, tc, native
    elif kind == "int8":
        for N, K in LLAMA3_8B_SHAPES:
            copies = max(2, -(-SWEEP_ROTATE_BYTES // (N * K)))
            wq = torch.randint(-127, 128, (copies, N, K), device=dev, dtype=torch.int8, generator=gen)
            sc = (torch.rand(N, device=dev, generator=gen) * 1e-3 + 1e-4).bfloat16()
            for M in (1, 4, 16):
                x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
                y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
                us = _time_linear(L, lambda i: _lib.check(L.ao_amd_int8wo_linear(
                    x.data_ptr(), M, K, K, wq[i % copies].data_ptr(), K, sc.data_ptr(), N, None, y.data_ptr(), _lib.BF16,
                    N, st)), iters)
                gbs = (N * K + 2 * N + 2 * M * K + 2 * M * N) / us / 1e3
                tfs = 2.0 * M * N * K / us / 1e6
                print(json.dumps({"kernel": "int8wo_linear", "N": N, "K": K, "M": M, "us": round(us, 2),
                                  "GBs": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 4),
                                  "TFLOPs": round(tfs, 2), "mfma_frac": round(tfs / MFMA_PEAK_TFLOPS, 4)}), flush=True)
            del wq
    elif kind == "ws":
        # The linears with a caller-owned workspace beside the plain entry points on the shapes where the library splits K
        # over workgroups (two launches: tiles + finish), both from replayed HIP graphs over rotating weight copies.
        def stream():
            return torch.cuda.current_stream().cuda_stream

        for N, K in [(4096, 4096), (6144, 4096), (4096, 14336), (1024, 4096)]:
            g = 64
            _, _, pb, qb = _lib.packed_shape(N, K, g)
            w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).bfloat16()
            copies = max(2, -(-SWEEP_ROTATE_BYTES // pb))
            packed = torch.empty(copies, pb // 4, dtype=torch.int32, device=dev)
            qp = torch.empty(copies, qb // 4, dtype=torch.int32, device=dev)
            _lib.check(L.ao_amd_int4wo_quantize_pack(w.data_ptr(), N, K, K, g, packed.data_ptr(), qp.data_ptr(), st))
            packed[1:] = packed[0]
            qp[1:] = qp[0]
            wh = w.half()
            tc = torch.empty(N * K * 3 // 4, dtype=torch.uint8, device=dev)
            sc = torch.empty(N, dtype=torch.float16, device=dev)
            _lib.check(L.ao_amd_fp6_quantize_pack(wh.data_ptr(), _lib.F16, N, K, 3, 2, tc.data_ptr(), sc.data_ptr(), st))
            nbytes = ctypes.c_int64()
            _lib.check(L.ao_amd_fp6_native_bytes(N, K, ctypes.byref(nbytes)))
            copies6 = max(2, -(-SWEEP_ROTATE_BYTES // nbytes.value))
            native = torch.empty(copies6, nbytes.value, dtype=torch.uint8, device=dev)
            _lib.check(L.ao_amd_fp6_repack(tc.data_ptr(), N, K, 6, native.data_ptr(), st))
            native[1:] = native[0]
            for M in (16, 32, 64, 128):
                x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
                y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
                parts = L.ao_amd_int4wo_linear_ws_parts(M, K, N, g)
                if parts > 1:
                    ws = torch.empty(parts * M * N, dtype=torch.float32, device=dev)
                    plain = replayed_us(lambda i: _lib.check(L.ao_amd_int4wo_linear(
                        x.data_ptr(), M, K, K, packed[i % copies].data_ptr(), qp[i % copies].data_ptr(), N, g, None, y.data_ptr(),
                        _lib.BF16, N, stream())), copies, 4)
                    split = replayed_us(lambda i: _lib.check(L.ao_amd_int4wo_linear_ws(
                        x.data_ptr(), M, K, K, packed[i % copies].data_ptr(), qp[i % copies].data_ptr(), N, g, None, y.data_ptr(),
                        _lib.BF16, N, ws.data_ptr(), ws.numel() * 4, stream())), copies, 4)
                    tfs = 2.0 * M * N * K / split / 1e6
                    print(json.dumps({"kernel": "int4wo_linear_ws", "N": N, "K": K, "M": M, "group": g, "parts": parts,
                                      "us": round(split, 2), "us_plain": round(plain, 2), "TFLOPs": round(tfs, 2),
                                      "mfma_frac": round(tfs / MFMA_PEAK_TFLOPS, 4)}), flush=True)
                parts6 = L.ao_amd_fp6_linear_ws_parts(M, K, N)
                if parts6 > 1:
                    xh = x.half()
                    yh = torch.empty(M, N, dtype=torch.float16, device=dev)
                    ws = torch.empty(parts6 * M * N, dtype=torch.float32, device=dev)
                    plain = replayed_us(lambda i: _lib.check(L.ao_amd_fp6_linear(
                        xh.data_ptr(), M, K, native[i % copies6].data_ptr(), sc.data_ptr(), N, 3, 2, yh.data_ptr(), stream())),
                        copies6, 4)
                    split = replayed_us(lambda i: _lib.check(L.ao_amd_fp6_linear_ws(
                        xh.data_ptr(), M, K, native[i % copies6].data_ptr(), sc.data_ptr(), N, 3, 2, yh.data_ptr(), ws.data_ptr(),
                        ws.numel() * 4, stream())), copies6, 4)
                    tfs = 2.0 * M * N * K / split / 1e6
                    print(json.dumps({"kernel": "fp6_linear_ws_e3m2", "N": N, "K": K, "M": M, "parts": parts6,
                                      "us": round(split, 2), "us_plain": round(plain, 2), "TFLOPs": round(tfs, 2),
                                      "mfma_frac": round(tfs / MFMA_PEAK_TFLOPS, 4)}), flush=True)
            del w, wh, packed, qp, tc, native
    elif kind == "tinygemm":
        # The operator the reference's int4 weight-only linear dispatches to (torchao/dtypes/affine_quantized_tensor.py:631 ->
        # aten._weight_int4pack_mm), as this PyTorch-ROCm build implements it, beside torch.ops.torchao.int4wo_linear
        # on the same codes and qparams.  Both run from a replayed HIP graph of one launch per weight copy, so the
        # figure is device time per launch with cold weights and no host dispatch in it.
        from ao_amd import ops
        from ao_amd.quantization.utils import groupwise_affine_quantize_tensor

        g = 64
        for N, K in [(4096, 4096), (6144, 4096), (14336, 4096), (4096, 14336), (128256, 4096)]:
            w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).bfloat16()
            codes, sz = groupwise_affine_quantize_tensor(w, 4, g)
            try:
                theirs = torch.ops.aten._convert_weight_to_int4pack(
                    ((codes[:, ::2] << 4) | codes[:, 1::2]).to(torch.uint8), 8)
            except (RuntimeError, NotImplementedError) as e:
                sys.exit(f"aten._convert_weight_to_int4pack is not available on this device: {e}")
            mine, mine_q = ops.int4wo_pack(codes, sz[:, :, 0].t().contiguous(), sz[:, :, 1].t().contiguous(), g)
            copies = max(2, -(-SWEEP_ROTATE_BYTES // (N * K // 2)))
            theirs_c, sz_c = [theirs.clone() for _ in range(copies)], [sz.clone() for _ in range(copies)]
            mine_c, mine_qc = [mine.clone() for _ in range(copies)], [mine_q.clone() for _ in range(copies)]
            for M in (1, 4, 16, 512, 2048):
                if M * N >= 1 << 28:
                    continue
                x = torch.randn(M, K, device=dev, generator=gen).bfloat16()
                reps = 20 if M <= 16 else 2
                t_us = replayed_us(lambda i: torch.ops.aten._weight_int4pack_mm(x, theirs_c[i % copies], g,
                                                                                 sz_c[i % copies]), copies, reps)
                m_us = replayed_us(lambda i: ops.int4wo_linear(x, mine_c[i % copies], mine_qc[i % copies], g, N),
                                   copies, reps)
                y_t = torch.ops.aten._weight_int4pack_mm(x, theirs, g, sz).float()
                y_m = ops.int4wo_linear(x, mine, mine_q, g, N).float()
                print(json.dumps({"N": N, "K": K, "M": M, "group": g, "aten_weight_int4pack_mm_us": round(t_us, 2),
                                  "int4wo_linear_us": round(m_us, 2), "speedup": round(t_us / m_us, 2),
                                  "rel_l2_between_outputs": float(f"{float((y_t - y_m).norm() / y_m.norm()):.3e}")}),
                      flush=True)
            del w, codes, theirs_c, sz_c, mine_c, mine_qc
    elif kind == "quantize":
        # the one-time quantize side at its reference call (quant_api.py:376-385: asymmetric, (1, g) blocks, int32 codes
        # in 0..15, bf16 scale and zero point in the float domain): the three primitives and the fused quantize + pack
        for N, K, g in [(4096, 4096, 128), (4096, 4096, 64), (14336, 4096, 64), (4096, 14336, 64)]:
            copies = max(2, -(-SWEEP_ROTATE_BYTES // (N * K * 2)))
            w = (torch.randn(copies, N, K, device=dev, generator=gen) * 0.02).bfloat16()
            scale = torch.empty(N, K // g, dtype=torch.bfloat16, device=dev)
            zero = torch.empty_like(scale)
            codes = torch.empty(copies, N, K, dtype=torch.int32, device=dev)
            deq = torch.empty(N, K, dtype=torch.bfloat16, device=dev)
            _, _, pb, qb = _lib.packed_shape(N, K, g)
            packed = torch.empty(pb // 4, dtype=torch.int32, device=dev)
            qp = torch.empty(qb // 4, dtype=torch.int32, device=dev)
            BF16, I32, ASYM, ZP_FLOAT = 1, 3, 1, 1
            tc = torch.empty(N * K * 3 // 4, dtype=torch.uint8, device=dev)
            sc16 = torch.empty(N, dtype=torch.float16, device=dev)
            qparam_bytes = 4 * N * K // g
            steps = [
                ("choose_qparams_affine", N * K * 2 + qparam_bytes, lambda i: _lib.check(L.ao_amd_choose_qparams_affine(
                    w[i % copies].data_ptr(), BF16, N, K, K, 1, g, ASYM, 0, 15, 1e-6, 0, ZP_FLOAT, BF16, BF16,
                    scale.data_ptr(), zero.data_ptr(), st))),
                ("quantize_affine", N * K * 6 + qparam_bytes, lambda i: _lib.check(L.ao_amd_quantize_affine(
                    w[i % copies].data_ptr(), BF16, N, K, K, 1, g, scale.data_ptr(), BF16, zero.data_ptr(), BF16, 0, 15,
                    ZP_FLOAT, codes[i % copies].data_ptr(), I32, st))),
                ("dequantize_affine", N * K * 6 + qparam_bytes, lambda i: _lib.check(L.ao_amd_dequantize_affine(
                    codes[i % copies].data_ptr(), I32, N, K, 1, g, scale.data_ptr(), BF16, zero.data_ptr(), BF16, 0, 15,
                    ZP_FLOAT, deq.data_ptr(), BF16, st))),
                ("int4wo_quantize_pack", N * K * 2 + N * K // 2 + qparam_bytes, lambda i: _lib.check(
                    L.ao_amd_int4wo_quantize_pack(w[i % copies].data_ptr(), N, K, K, g, packed.data_ptr(), qp.data_ptr(),
                                                  st))),
                ("fp6_quantize_pack_e3m2", N * K * 2 + N * K * 3 // 4 + 2 * N, lambda i: _lib.check(
                    L.ao_amd_fp6_quantize_pack(w[i % copies].data_ptr(), BF16, N, K, 3, 2, tc.data_ptr(), sc16.data_ptr(),
                                               st))),
            ]
            if g == 64:
                # the int8 weight-only call (quant_api.py:390-405): symmetric, one block per row, int8 codes, int64 zeros
                I64, I8, SYM, ZP_INT = 4, 5, 0, 0
                srow = torch.empty(N, dtype=torch.bfloat16, device=dev)
                zrow = torch.zeros(N, dtype=torch.int64, device=dev)
                codes8 = codes.view(torch.int8).view(copies, -1)[:, : N * K].view(copies, N, K)
                steps += [
                    ("choose_qparams_i8_row", N * K * 2 + 10 * N, lambda i: _lib.check(
                        L.ao_amd_choose_qparams_affine(w[i % copies].data_ptr(), BF16, N, K, K, 1, K, SYM, -128, 127,
                                                       float(torch.finfo(torch.float32).eps), 1, ZP_INT, BF16, I64,
                                                       srow.data_ptr(), zrow.data_ptr(), st))),
                    ("quantize_affine_i8_row", N * K * 3 + 10 * N, lambda i: _lib.check(L.ao_amd_quantize_affine(
                        w[i % copies].data_ptr(), BF16, N, K, K, 1, K, srow.data_ptr(), BF16, zrow.data_ptr(), I64, -128,
                        127, ZP_INT, codes8[i % copies].data_ptr(), I8, st))),
                    ("dequant_affine_i8_row", N * K * 3 + 10 * N, lambda i: _lib.check(L.ao_amd_dequantize_affine(
                        codes8[i % copies].data_ptr(), I8, N, K, 1, K, srow.data_ptr(), BF16, zrow.data_ptr(), I64, -128,
                        127, ZP_INT, deq.data_ptr(), BF16, st))),
                ]
            for name, nbytes, launch in steps:
                us = _time_linear(L, launch, iters, armed=False)
                print(json.dumps({"kernel": name, "N": N, "K": K, "group": g, "us": round(us, 2),
                                  "GBs": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / 8000.0, 4)}),
                      flush=True)
            del w, codes
    else:
        sys.exit(f"unknown sweep {kind}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="Llama-3-8B")
    ap.add_argument("--group", type=int, default=64)
    ap.add_argument("--prompt-len", type=int, default=128)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--roofline-only", action="store_true",
                    help="build the model, run one pass of the roofline leg and a copy kernel of known size, no decode "
                         "loop: the command to put under rocprofv3 --pmc")
    ap.add_argument("--quantization", default=None,
                    help="int4wo-<group> (default: int4wo-<--group>, the headline configuration), int8wo or fp6 (e3m2 on an "
                         "fp16 model): the decode loop of the reference's other weight-only configurations, reported "
                         "without the int4 roofline leg")
    ap.add_argument("--sweep", choices=("gemv", "gemm", "fp6", "int8", "ws", "tinygemm", "quantize"), default=None,
                    help="instead of the decode benchmark, print one line per kernel case of the named sweep")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if args.sweep:
        import torch

        assert torch.cuda.is_available(), "bench.py needs the GPU"
        torch.cuda.set_device(0)
        sweep(args.sweep)
        return

    import torch

    from ao_amd._models.llama.generate import GraphedDecoder, build_random_model, prefill
    from ao_amd._models.llama.model import prepare_inputs_for_model
    from ao_amd.utils import get_model_size_in_bytes

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    quant = args.quantization or f"int4wo-{args.group}"
    if not quant.startswith("int4wo-"):
        args.no_roofline = args.no_cpu_baseline = True  # both legs describe the int4 kernels
    model = build_random_model(args.model, device, quant)
    cfg = model.config
    model_size = get_model_size_in_bytes(model, ignore_embeddings=True)

    if args.roofline_only:
        copy_calibration()
        print(json.dumps({"roofline": roofline_leg(model, passes=1)}), flush=True)
        return

    gen = torch.Generator(device=device).manual_seed(0)
    prompt = torch.randint(0, cfg.vocab_size, (args.prompt_len,), device=device, dtype=torch.int, generator=gen)
    total_len = args.prompt_len + args.warmup + args.steps + 8
    with torch.no_grad():
        model.setup_caches(max_batch_size=1, max_seq_length=total_len)
        x, input_pos = prepare_inputs_for_model(prompt)
        first = prefill(model, x, input_pos, greedy=True).clone()
        dec = GraphedDecoder(model, device, greedy=True)
        dec.capture(first, args.prompt_len)
        for _ in range(args.warmup):
            dec.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            dec.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0

    tok_s = args.steps / elapsed
    line = {
        "metric": ("tok/s Llama-3-8B-arch int4wo-64 bs=1; int4 GEMV HBM GB/s vs peak" if quant.startswith("int4wo-")
                   else f"tok/s Llama-3-8B-arch {quant} bs=1"),
        "value": round(tok_s, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp16" if quant == "fp6" else "bf16",
        "data": "synthetic",
        "config": {
            "workload": (f"{args.model}-architecture random-init (weights ~N(0,0.02), seed 1234), {quant} on every "
                         f"nn.Linear, greedy batch-1 decode after a {args.prompt_len}-token uniform-random prompt, "
                         "HIP-graph replay per token"),
            "model_size_bytes": model_size,
            "model_bandwidth_GBs": round(model_size * tok_s / 1e9, 1),
        },
    }
    if not args.no_roofline:
        line["roofline"] = roofline_leg(model)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_leg(cfg, args.group)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
