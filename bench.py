#!/usr/bin/env python3
"""Benchmark of the MX quantization hot path on one MI355X.

One "step" = one `_quantize_mx` pass (MXFP8 e4m3, block 32 along the last axis, scale_bits 8,
round 'nearest') over a seeded fp32 [8192, 8192] tensor that is already resident in HBM.
Prints ONE JSON line: whole-job throughput in GB/s of algorithmic bytes (8 B per element: fp32 in,
fp32 out), the roofline position of the kernel from HIP events around the timed launches, and the CPU
baseline (the torch op-sequence oracle timed on this box's host cores).  The metric has a second half,
the fused MX linear layer in TFLOP/s: without --workload the same line carries it as "secondary"
(workload mx_linear timed for the same steps: whole-step TFLOP/s, the GEMM kernel's own launch time
against the dense fp8 MFMA peak, its CPU baseline).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

Workloads (config N = the N-th benchmark configuration of this build's baseline file):
    mxfp8_fp32_8192      headline (default)
    mxfp8_fp32_4096      config 1 (fits in the 256 MB Infinity Cache -- not an HBM figure)
    mxfp6_e3m2_bf16_m1 / mxfp6_e2m3_bf16_m1 / mxfp4_bf16_m1      config 2, axis -1
    mxfp6_e3m2_bf16_m2 / mxfp6_e2m3_bf16_m2 / mxfp4_bf16_m2      config 2, axis -2
    elem_bf16_fp32 / elem_fp16_fp32                              config 3, elementwise
    reduce_sum_m1 / reduce_max_m1 / reduce_sum_0 / reduce_max_0  config 3, reductions
    mx_linear / mx_linear_fp4 / mx_linear_fp6 / mx_linear_bfloat16  config 4: mx.Linear forward (TFLOP/s)
    mx_linear_train                                              ... forward + backward
    mx_linear_prequantized                                       ... as an inference layer that keeps its weight's MX codes
    mx_bmm_softmax (_two_kernels: product and softmax separately) config 5: mx.bmm + bfloat16 softmax
    softmax_bf16 / layernorm_bf16 / gelu_bf16 / silu_bf16 (+ _train), norm_param_grads_bf16, pack_t_bf16,
    mxfp8_fp32_8192_tiles                                        single kernels of the layers around the path
    (suffix _unfused where it exists: the same step as separate tensor passes)
    copy_fp32_8192       torch copy_ of the headline tensor (calibrates the rocprof byte counters)
"""
import argparse
import json
import os
import sys
import time

import torch

HBM_PEAK_GBPS = 8000.0          # MI355X published HBM3E peak


def outlier_bf16(rows, cols, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    idx = torch.randperm(cols, generator=g)[: cols // 100]
    scale = torch.ones(cols)
    scale[idx] = torch.exp(2.0 * torch.randn(idx.numel(), generator=g))
    return (x * scale).to(torch.bfloat16)


def wide_fp32(rows, cols, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g) .double()
    x = x * 10.0 ** (torch.rand(rows, cols, generator=g).double() * 80 - 40)
    x = x.to(torch.float32).reshape(-1)
    n = x.numel()
    sp = torch.randperm(n, generator=g)
    k = n // 1000
    x[sp[:k]] = torch.tensor([float("inf"), -float("inf"), float("nan")]).repeat(k // 3 + 1)[:k]
    m = n // 100
    sub = torch.randint(1, 1 << 23, (m,), generator=g, dtype=torch.int32)
    sub |= torch.randint(0, 2, (m,), generator=g, dtype=torch.int32) << 31
    x[sp[k:k + m]] = sub.view(torch.float32)
    return x.reshape(rows, cols)


def make_workload(name):
    """-> dict(x=cpu tensor, gpu=callable(xd), cpu=callable(x_rows), bytes=algorithmic bytes per
    step, dtype=..., desc=...)"""
    from microxcaling_amd.mx_ops import _quantize_mx
    from microxcaling_amd.elemwise_ops import _quantize_elemwise_core
    from microxcaling_amd.custom_extensions import funcs
    from oracle import mx_oracle as O

    def mx(fmt, axis, rnd="nearest"):
        return (lambda t: _quantize_mx(t, 8, fmt, axes=[axis], block_size=32, round=rnd),
                lambda t: O.quantize_mx(t, 8, fmt, axes=[axis], block_size=32, round=rnd))

    if name in ("mxfp8_fp32_8192", "mxfp8_fp32_4096"):
        n = 8192 if name.endswith("8192") else 4096
        x = torch.randn(n, n, generator=torch.Generator().manual_seed(0))
        g, c = mx("fp8_e4m3", -1)
        return dict(x=x, gpu=g, cpu=c, bytes=x.numel() * 8, dtype="f32", sample_axis=0,
                    desc="_quantize_mx fp8_e4m3 block 32 axis -1 nearest, fp32 [%d,%d] N(0,1)" % (n, n))
    if name.startswith("mxfp") and "_bf16_m" in name:
        fmt = {"mxfp6_e3m2": "fp6_e3m2", "mxfp6_e2m3": "fp6_e2m3", "mxfp4": "fp4_e2m1"}[name.split("_bf16_")[0]]
        axis = -1 if name.endswith("m1") else -2
        x = outlier_bf16(8192, 8192, 7)
        g, c = mx(fmt, axis)
        return dict(x=x, gpu=g, cpu=c, bytes=x.numel() * 4, dtype="bf16", sample_axis=0 if axis == -1 else 1,
                    desc="_quantize_mx %s block 32 axis %d nearest, bf16 [8192,8192] with outlier columns" % (fmt, axis))
    if name in ("elem_bf16_fp32", "elem_fp16_fp32"):
        bits, eb, mn = (9, 8, 2 ** 127 * 255 / 128) if "bf16" in name else (12, 5, 65504.0)
        x = wide_fp32(16384, 8192, 11)
        return dict(x=x, gpu=lambda t: _quantize_elemwise_core(t, bits, eb, mn, round="nearest"),
                    cpu=lambda t: O.quantize_elemwise_core(t, bits, eb, mn, round="nearest"),
                    bytes=x.numel() * 8, dtype="f32", sample_axis=0,
                    desc="_quantize_elemwise_core bits=%d exp_bits=%d nearest, fp32 [16384,8192] wide range" % (bits, eb))
    if name.startswith("reduce_"):
        x = wide_fp32(16384, 8192, 13)
        x[~torch.isfinite(x)] = 1.0
        op, ax = name.split("_")[1], name.split("_")[2]
        fn = {("sum", "m1"): funcs.reduce_sum_inner_dim, ("max", "m1"): funcs.reduce_max_inner_dim,
              ("sum", "0"): funcs.reduce_sum_outer_dim, ("max", "0"): funcs.reduce_max_outer_dim}[(op, ax)]
        dim = -1 if ax == "m1" else 0
        cpu = (lambda t: t.sum(dim)) if op == "sum" else (lambda t: t.max(dim).values)
        return dict(x=x, gpu=fn, cpu=cpu, bytes=x.numel() * 4, dtype="f32", sample_axis=0 if dim == -1 else 1,
                    launches=1 if dim == -1 else 2,
                    desc="reduce %s over axis %d, fp32 [16384,8192]" % (op, dim))
    if name in ("mx_linear", "mx_linear_unfused", "mx_linear_fp4", "mx_linear_fp4_unfused",
                "mx_linear_fp6", "mx_linear_fp6_unfused", "mx_linear_bfloat16", "mx_linear_bfloat16_unfused"):
        # config 4: mx.Linear forward, MXFP8 e4m3 (or MXFP4 e2m1) both operands, block 32 along K, bias
        from microxcaling_amd import gemm
        from microxcaling_amd.linear import linear
        from microxcaling_amd.specs import finalize_mx_specs
        g = torch.Generator().manual_seed(4)
        M, N, K = 16384, 14336, 4096
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
        b = torch.randn(N, generator=g).to(torch.bfloat16)
        ef = "fp4_e2m1" if "fp4" in name else "fp6_e2m3" if "fp6" in name else "fp8_e4m3"
        spec_dict = {"w_elem_format": ef, "a_elem_format": ef, "block_size": 32}
        if "bfloat16" in name:                   # the same layer with bfloat16 vector quantization as well:
            spec_dict["bfloat"] = 16             # operands, product and bias sum go through it
        specs = finalize_mx_specs(spec_dict)
        dev_extra = {}
        fused = not name.endswith("_unfused")

        def run(xd):
            if "w" not in dev_extra:
                dev_extra["w"], dev_extra["b"] = w.to(xd.device), b.to(xd.device)
            gemm.set_fused(fused)
            return linear(xd, dev_extra["w"], dev_extra["b"], mx_specs=specs)
        bf = 16 if "bfloat16" in name else 0

        def gemm_only(xd):
            # the GEMM kernel on its own: both operands packed once, as the layer packs them
            from microxcaling_amd import fused
            nib = ef == "fp4_e2m1"
            pre = bool(bf)
            pa = fused.pack_mx(xd, ef, 8, "nearest", False, nib, pre)
            pb = fused.pack_mx(w.to(xd.device), ef, 8, "nearest", False, nib, pre)
            bd = b.to(xd.device)
            return lambda: fused.gemm_nt(pa, pb, out_dtype=torch.bfloat16, bias=bd, epilogue_quant=bool(bf))
        extra = dict(gemm_only=gemm_only, gemm_flops=2.0 * M * N * K,
                     gemm_kernel="mx_gemm_nt_kernel_256p") if fused else {}
        return dict(x=x, gpu=run, cpu=lambda t: O.mx_linear_forward(t, w, b, ef, ef, bfloat=bf), **extra,
                    tolerance="vs the oracle's quantize-then-fp32-matmul on sampled rows (tests/test_gpu_baseline_shapes.py): "
                              "fp32 tensors max|diff| / RMS < 1e-3; bf16 tensors (this run) |diff| <= 2^-6 (|out| + |bias|) "
                              "+ 2e-3 RMS, i.e. one bf16 rounding step of the product and of the bias sum on top",
                    flops=2.0 * M * N * K, bytes=0, dtype="%s x %s -> f32 acc" % (ef, ef), sample_axis=0,
                    cpu_rows=1024, launches=5, peak="fp4" if ef == "fp4_e2m1" else "fp8",   # fp6 runs on byte codes: fp8 rate
                    desc="mx.Linear forward: x bf16 [16384,4096], W bf16 [14336,4096] ~N(0,0.02), bias; %s "
                         "block 32 along K, %s" % ({"fp4_e2m1": "MXFP4 e2m1", "fp6_e2m3": "MXFP6 e2m3"}.get(ef, "MXFP8 e4m3"),
                                                   ("packed codes + scaled-MFMA GEMM" if fused else
                                                    "fake-quantize kernels + torch (hipBLASLt) bf16 GEMM")))
    if name == "mx_linear_prequantized":
        # config 4 as an inference layer: mx.Linear.prequantize_weights() keeps the weight's MX codes, a
        # forward pass packs the activations only
        from microxcaling_amd.linear import Linear
        from microxcaling_amd.specs import finalize_mx_specs
        g = torch.Generator().manual_seed(4)
        M, N, K = 16384, 14336, 4096
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
        b = torch.randn(N, generator=g).to(torch.bfloat16)
        specs = finalize_mx_specs({"w_elem_format": "fp8_e4m3", "a_elem_format": "fp8_e4m3", "block_size": 32,
                                   "bfloat": 16, "round": "even"})
        st = {}

        def run(xd):
            if "m" not in st:
                m = Linear(K, N, mx_specs=specs)
                with torch.no_grad():
                    m.weight.copy_(w)
                    m.bias.copy_(b)
                m.to(xd.device).eval()
                m.prequantize_weights(keep_dense=False)
                st["m"] = m
            with torch.no_grad():
                return st["m"](xd)
        return dict(x=x, gpu=run, cpu=lambda t: O.mx_linear_forward(t, w, b, "fp8_e4m3", "fp8_e4m3", bfloat=16, round="even"),
                    flops=2.0 * M * N * K, bytes=0, dtype="fp8_e4m3 x fp8_e4m3 -> f32 acc", sample_axis=0,
                    cpu_rows=1024, launches=2,
                    desc="mx.Linear forward with prequantized weights (MX codes + scales kept, 1 + 1/32 B per weight): "
                         "x bf16 [16384,4096] packed per step, W [14336,4096] packed once; MXFP8 e4m3, bias")
    if name in ("mx_linear_train", "mx_linear_train_unfused"):
        # forward + backward of the same layer (three GEMMs: output, grad_input, grad_weight), every
        # operand MX-quantized along its contraction axis (mx/linear.py:20-198)
        from microxcaling_amd import gemm
        from microxcaling_amd.linear import linear
        from microxcaling_amd.specs import finalize_mx_specs
        g = torch.Generator().manual_seed(4)
        M, N, K = 16384, 14336, 4096
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
        b = torch.randn(N, generator=g).to(torch.bfloat16)
        specs = finalize_mx_specs({"w_elem_format": "fp8_e4m3", "a_elem_format": "fp8_e4m3", "block_size": 32,
                                   "quantize_backprop": True})
        st = {}
        fused = name == "mx_linear_train"

        def run(xd):
            if "w" not in st:
                st["w"] = w.to(xd.device).requires_grad_(True)
                st["b"] = b.to(xd.device).requires_grad_(True)
                st["x"] = xd.clone().requires_grad_(True)
                st["go"] = torch.randn(M, N, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(xd.device)
            gemm.set_fused(fused)
            for t in (st["w"], st["b"], st["x"]):
                t.grad = None
            out = linear(st["x"], st["w"], st["b"], mx_specs=specs)
            out.backward(st["go"])
            return out
        return dict(x=x, gpu=run, cpu=lambda t: O.mx_linear_forward(t, w, b, "fp8_e4m3", "fp8_e4m3"),
                    flops=6.0 * M * N * K, bytes=0, dtype="fp8_e4m3 x fp8_e4m3 -> f32 acc", sample_axis=0,
                    cpu_rows=1024, launches=20,
                    desc="mx.Linear forward + backward: x bf16 [16384,4096], W bf16 [14336,4096], bias; MXFP8 "
                         "e4m3 block 32 along every contraction axis, %s" %
                         ("packed codes + scaled-MFMA GEMMs" if fused else "fake-quantize kernels + torch GEMMs"))
    if name in ("mx_bmm_softmax", "mx_bmm_softmax_two_kernels", "mx_bmm_softmax_unfused"):
        # config 5: mx.bmm Q.K^T, MXFP6 e2m3 along head_dim, then the bfloat16 softmax chain
        from microxcaling_amd import gemm
        from microxcaling_amd.bmm import bmm
        from microxcaling_amd.softmax import softmax
        from microxcaling_amd.specs import finalize_mx_specs
        g = torch.Generator().manual_seed(5)
        B, S, D = 128, 2048, 128
        q = torch.randn(B, S, D, generator=g).to(torch.bfloat16)
        k = torch.randn(B, S, D, generator=g).to(torch.bfloat16)
        specs = finalize_mx_specs({"a_elem_format": "fp6_e2m3", "block_size": 32, "bfloat": 16})
        dev_extra = {}
        fused = name != "mx_bmm_softmax_unfused"

        def run(qd):
            if "k" not in dev_extra:
                dev_extra["k"] = k.to(qd.device)
            gemm.set_fused(fused)
            # The reference's own call sequence, mx.softmax(mx.bmm(q, k^T)).  mx.bmm hands back its product
            # unevaluated and the softmax runs product and softmax as one launch (+ two packs); with that
            # switched off the same two calls are the GEMM kernel and the softmax kernel.
            gemm.set_deferred_scores(name == "mx_bmm_softmax")
            try:
                logits = bmm(qd, dev_extra["k"].transpose(-1, -2), mx_specs=specs)
                return softmax(logits, dim=-1, mx_specs=specs)
            finally:
                gemm.set_deferred_scores(True)

        def cpu(t):
            n = t.shape[0]
            return O.softmax_forward(O.mx_bmm_forward(t, k[:n].transpose(-1, -2), "fp6_e2m3", bfloat=16), -1)
        tol = ("vs the oracle's bfloat16 softmax chain on the logits the GPU produced, sampled batch entries "
               "(tests/test_gpu_baseline_shapes.py): %s; the logits themselves within one bf16 step of the oracle's "
               "quantize-then-fp32-bmm" %
               ("|diff| <= 2^-6 p, one step of the bfloat16 quantizer's grid on at most 2 % of the elements (looser than "
                "abs 2^-8 for probabilities from 0.25 up, which the two-kernel form meets)" if name == "mx_bmm_softmax"
                else "abs 2^-8, at most 2 % of the elements differing"))
        return dict(x=q, gpu=run, cpu=cpu, flops=2.0 * B * S * S * D, bytes=0, tolerance=tol,
                    dtype="fp6_e2m3 x fp6_e2m3 -> f32 acc", sample_axis=0, cpu_rows=8, launches=20,
                    desc="mx.bmm Q.K^T bf16 [128,2048,128] MXFP6 e2m3 along head_dim + bfloat16 softmax, %s"
                         % ("mx.softmax(mx.bmm(q, k^T)): packed codes, product and softmax in one kernel (logits in registers)" if name == "mx_bmm_softmax"
                            else "packed codes + scaled-MFMA GEMM, softmax kernel" if fused else "fake-quantize + torch.bmm"))
    if name in ("softmax_bf16", "softmax_bf16_unfused", "layernorm_bf16", "layernorm_bf16_unfused"):
        # the fused row kernels on their own: bfloat16 softmax over [128*2048, 2048] (the logits of
        # config 5) and bfloat16 LayerNorm over [32768, 4096]
        from microxcaling_amd import gemm
        from microxcaling_amd.layernorm import LayerNorm
        from microxcaling_amd.softmax import softmax
        from microxcaling_amd.specs import finalize_mx_specs
        specs = finalize_mx_specs({"bfloat": 16})
        fused = not name.endswith("unfused")
        g = torch.Generator().manual_seed(6)
        extra = {}
        if name.startswith("softmax"):
            x = (torch.randn(16384, 2048, generator=g) * 3).to(torch.bfloat16).repeat(16, 1)
            per_elem, what = 4, "softmax over the last axis, bf16 [262144,2048]"

            def run(xd):
                gemm.set_fused(fused)
                return softmax(xd, dim=-1, mx_specs=specs)
            cpu = lambda t: O.softmax_forward(t, -1, bfloat=16)
        else:
            x = (torch.randn(32768, 4096, generator=g) * 2 + 0.5).to(torch.bfloat16)
            per_elem, what = 6, "LayerNorm (output + saved normalized input), bf16 [32768,4096]"
            ln = {}

            def run(xd):
                if "m" not in ln:
                    ln["m"] = LayerNorm(4096, eps=1e-5, mx_specs=specs).to(torch.bfloat16).to(xd.device)
                gemm.set_fused(fused)
                with torch.no_grad():
                    return ln["m"](xd)
            cpu_ln = LayerNorm(4096, eps=1e-5, mx_specs=specs).to(torch.bfloat16)
            cpu = lambda t: cpu_ln(t)
            extra["cpu_what"] = "this package's LayerNorm on CPU tensors (host-library quantizers)"
        return dict(x=x, gpu=run, cpu=cpu, bytes=x.numel() * per_elem, dtype="bf16", sample_axis=0, **extra,
                    launches=1 if fused else 12,
                    desc="%s, bfloat16 quantization after every step, %s" % (what, "one kernel" if fused else
                                                                             "separate tensor passes"))
    if name in ("layernorm_bf16_train", "layernorm_bf16_train_unfused"):
        # LayerNorm forward + backward over bf16 [32768, 4096]: two row kernels + the column-sum
        # kernels of the parameter gradients.  Algorithmic bytes per element: forward 2 in + 4 out
        # (output, saved normalized input), input gradient 4 in + 2 out, parameter gradients 4 in
        from microxcaling_amd import gemm
        from microxcaling_amd.layernorm import LayerNorm
        from microxcaling_amd.specs import finalize_mx_specs
        specs = finalize_mx_specs({"bfloat": 16})
        fused = not name.endswith("unfused")
        x = (torch.randn(32768, 4096, generator=torch.Generator().manual_seed(6)) * 2 + 0.5).to(torch.bfloat16)
        ln = {}

        def run(xd):
            if "m" not in ln:
                ln["m"] = LayerNorm(4096, eps=1e-5, mx_specs=specs).to(torch.bfloat16).to(xd.device)
                ln["g"] = torch.randn(xd.shape, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(xd.device)
            gemm.set_fused(fused)
            xi = xd.requires_grad_(True)
            xi.grad = None
            ln["m"](xi).backward(ln["g"])
            return xi.grad
        cpu_ln = LayerNorm(4096, eps=1e-5, mx_specs=specs).to(torch.bfloat16)
        return dict(x=x, gpu=run, cpu=lambda t: cpu_ln(t), bytes=x.numel() * (6 + 6 + 4), dtype="bf16", sample_axis=0,
                    cpu_what="this package's LayerNorm forward on CPU tensors (host-library quantizers)",
                    launches=8 if fused else 50,
                    desc="LayerNorm forward + backward, bf16 [32768,4096], bfloat16 quantization after every step, %s"
                         % ("two row kernels + column-sum kernels for the parameter gradients" if fused else "separate tensor passes"))
    if name in ("gelu_bf16_train", "gelu_bf16_train_unfused", "softmax_bf16_train", "softmax_bf16_train_unfused"):
        # forward + backward of one bfloat16 layer: the fused forward kernel writes what the fused
        # backward kernel reads
        from microxcaling_amd import activations, gemm
        from microxcaling_amd.softmax import softmax
        from microxcaling_amd.specs import finalize_mx_specs
        specs = finalize_mx_specs({"bfloat": 16})
        fused = not name.endswith("unfused")
        is_gelu = name.startswith("gelu")
        gen = torch.Generator().manual_seed(8)
        if is_gelu:
            x = (torch.randn(4096, 8192, generator=gen) * 2).to(torch.bfloat16).repeat(4, 1)
            per_elem = 8 + 8                              # fwd: 1 read, 3 writes; bwd: 3 reads, 1 write
        else:
            x = (torch.randn(16384, 2048, generator=gen) * 3).to(torch.bfloat16).repeat(8, 1)
            per_elem = 4 + 6                              # fwd: read, write; bwd: 2 reads, 1 write
        extra = {}

        def run(xd):
            if "g" not in extra:
                extra["g"] = torch.randn(xd.shape, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(xd.device)
            gemm.set_fused(fused)
            xi = xd.requires_grad_(True)
            xi.grad = None
            y = activations.gelu(xi, mx_specs=specs) if is_gelu else softmax(xi, dim=-1, mx_specs=specs)
            y.backward(extra["g"])
            return xi.grad
        cpu = (lambda t: activations.gelu(t, mx_specs=specs)) if is_gelu else (lambda t: O.softmax_forward(t, -1, bfloat=16))
        return dict(x=x, gpu=run, cpu=cpu, bytes=x.numel() * per_elem, dtype="bf16", sample_axis=0,
                    launches=2 if fused else 40,
                    desc="%s forward + backward, bf16 %s, bfloat16 quantization after every step, %s"
                         % ("GELU (cubic)" if is_gelu else "softmax over the last axis", list(x.shape),
                            "two kernels" if fused else "separate tensor passes"))
    if name in ("gelu_bf16", "gelu_bf16_unfused", "silu_bf16", "silu_bf16_unfused"):
        # fused activation kernels: GELU (writes the result, phi and the quantized input: what the
        # layer saves for its backward pass) and SiLU (result and sigmoid) over bf16 [16384, 8192]
        from microxcaling_amd import activations, gemm
        from microxcaling_amd.specs import finalize_mx_specs
        specs = finalize_mx_specs({"bfloat": 16})
        fused = not name.endswith("unfused")
        is_gelu = name.startswith("gelu")
        x = (torch.randn(4096, 8192, generator=torch.Generator().manual_seed(7)) * 2).to(torch.bfloat16).repeat(4, 1)

        def run(xd):
            gemm.set_fused(fused)
            xi = xd.requires_grad_(True)                # the layers only save tensors when a gradient is wanted
            return activations.gelu(xi, mx_specs=specs) if is_gelu else activations.silu(xi, mx_specs=specs)
        cpu = (lambda t: activations.gelu(t, mx_specs=specs)) if is_gelu else (lambda t: activations.silu(t, mx_specs=specs))
        return dict(x=x, gpu=run, cpu=cpu, bytes=x.numel() * (8 if is_gelu else 6), dtype="bf16", sample_axis=0,
                    launches=1 if fused else (22 if is_gelu else 12),
                    desc="%s forward, bf16 [16384,8192], bfloat16 quantization after every step, %s"
                         % ("GELU (cubic)" if is_gelu else "SiLU", "one kernel" if fused else "separate tensor passes"))
    if name == "norm_param_grads_bf16":
        # weight and bias gradients of LayerNorm over bf16 [32768, 4096] on their own: column sums of
        # Q(g z) and of g; algorithmic bytes = g and z read once
        from microxcaling_amd.layernorm import _fused_param_grads, _param_grads
        from microxcaling_amd.specs import apply_mx_specs, finalize_mx_specs
        specs = apply_mx_specs(finalize_mx_specs({"bfloat": 16}))
        g = torch.Generator().manual_seed(9)
        x = torch.randn(32768, 4096, generator=g).to(torch.bfloat16)
        z = {}

        def run(xd):
            if "z" not in z:
                z["z"] = (torch.randn(xd.shape, generator=torch.Generator().manual_seed(10)) * 1.5).to(torch.bfloat16).to(xd.device)
            return _fused_param_grads(xd, z["z"], specs)
        zc = (torch.randn(x.shape, generator=torch.Generator().manual_seed(10)) * 1.5).to(torch.bfloat16)
        return dict(x=x, gpu=run, cpu=lambda t: _param_grads(t, zc[:t.shape[0], :t.shape[1]].contiguous(), specs), bytes=x.numel() * 4,
                    dtype="bf16", sample_axis=0, launches=2,
                    cpu_what="this package's separate steps on CPU tensors (host-library quantizers)",
                    desc="LayerNorm weight and bias gradients, bf16 [32768,4096], bfloat16 quantization: "
                         "two column-sum launches (CPU leg: this package's separate steps on CPU tensors)")
    if name == "pack_t_bf16":
        # quantize along axis -2 + transpose + pack: the operand form of grad_output^T in a linear layer's
        # weight gradient; algorithmic bytes = input + codes + scales
        from microxcaling_amd.fused import pack_mx_t
        x = torch.randn(16384, 14336, generator=torch.Generator().manual_seed(12)).to(torch.bfloat16)
        return dict(x=x, gpu=lambda t: pack_mx_t(t, "fp8_e4m3"),
                    cpu=lambda t: O.quantize_mx(t, 8, "fp8_e4m3", axes=[-2], block_size=32).t().contiguous(),
                    bytes=x.numel() * 3 + x.numel() // 32, dtype="bf16", sample_axis=1,
                    desc="MXFP8 e4m3 transposing pack (blocks of 32 along axis -2), bf16 [16384,14336] -> "
                         "codes [14336,16384] + scale bytes (CPU leg: fake quantization + transpose)")
    if name == "mxfp8_fp32_8192_tiles":
        # one exponent per 32 x 32 tile (two shared axes): the general-shape kernel
        x = torch.randn(8192, 8192, generator=torch.Generator().manual_seed(0))
        return dict(x=x, gpu=lambda t: _quantize_mx(t, 8, "fp8_e4m3", axes=[-2, -1], block_size=32),
                    cpu=lambda t: O.quantize_mx(t, 8, "fp8_e4m3", axes=[-2, -1], block_size=32),
                    bytes=x.numel() * 8, dtype="f32", sample_axis=0,
                    desc="_quantize_mx fp8_e4m3, one exponent per 32 x 32 tile (axes -2 and -1), fp32 [8192,8192]")
    if name == "copy_fp32_8192":
        # a plain device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters
        x = torch.randn(8192, 8192, generator=torch.Generator().manual_seed(0))
        buf = {}

        def copy(t):
            if "y" not in buf:
                buf["y"] = torch.empty_like(t)
            return buf["y"].copy_(t)
        return dict(x=x, gpu=copy, cpu=lambda t: t.clone(), bytes=x.numel() * 8, dtype="f32", sample_axis=0,
                    desc="torch copy_ of fp32 [8192,8192] (counter calibration)")
    raise SystemExit("unknown workload %r" % name)


def cpu_baseline(wl, budget_s=15.0):
    """Time the oracle on the host cores: repeated passes over the FULL workload tensor (so caches
    do not flatter it) until about `budget_s` seconds of CPU work are spent; median pass."""
    x = wl["x"]
    cores = min(os.cpu_count() or 1, 16)      # the box's CPU share for one GPU
    torch.set_num_threads(cores)
    wl["cpu"](x[:64, :64].contiguous())       # warm up the op sequence
    times = []
    t_all = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_all < budget_s and len(times) < 25):
        t0 = time.perf_counter()
        wl["cpu"](x)
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_all > 4 * budget_s:
            break
    times.sort()
    t = times[len(times) // 2]
    return {"value": round(wl["bytes"] / t / 1e9, 4), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "the full workload tensor (%s), %d passes in %.1f s, median pass %.3f s; torch %s "
                      "%s, %d threads"
                      % ("x".join(str(n) for n in x.shape), len(times), time.perf_counter() - t_all, t,
                         torch.__version__, wl.get("cpu_what", "op-by-op oracle (oracle/mx_oracle.py)"), cores)}


# MI355X dense MFMA peaks, published: fp8 (e4m3 / e5m2 byte codes, which also carry fp6 elements) and
# fp4 (e2m1 nibble codes)
MFMA_PEAK_TFLOPS = {"fp8": 5000.0, "fp4": 10100.0}


def measured_traffic(workload):
    """HBM bytes per launch of the workload's dominant kernel, measured separately with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE (the summaries are in profiles/) -- but only while the kernel's source files
    are the ones that summary was taken with, or ones for which the kernel's generated code has been compared
    with that of the measured build and found identical (profiles/traffic.json says which): a figure from
    another build of the kernel is not this build's traffic.
    -> (bytes or None, where the last measurement is and whether it is current)"""
    import hashlib
    here = os.path.dirname(os.path.abspath(__file__))
    tfile = os.path.join(here, "profiles", "traffic.json")
    if not os.path.exists(tfile):
        return None, None
    with open(tfile) as f:
        entry = json.load(f).get(workload)
    if not isinstance(entry, dict):
        return None, None
    h = hashlib.sha256()
    for name in entry["sources"]:
        with open(os.path.join(here, "microxcaling_amd", "csrc", name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read() + b"\0")
    unchanged = not entry["sources"] or h.hexdigest() == entry["sources_sha256"]
    # ... or the files are in the state for which the measured kernel's generated code was compared with the
    # code of the measurement's sources and found identical
    same_code = h.hexdigest() == entry.get("same_code_checked", {}).get("sources_sha256")
    note = {"last_measured_bytes": entry["bytes"], "summary": entry["profile"],
            "kernel_sources_unchanged_since": unchanged, "kernel_code_compared_identical": same_code}
    return (entry["bytes"] if unchanged or same_code else None), note


METRIC = "MX quantize GB/s + % HBM peak (8192² fp32 MXFP8); fused MX-linear TFLOP/s"


def time_steps(fn, xd, steps, warmup):
    """W untimed steps, then exactly K steps bracketed by a synchronize on both sides (wall clock) and
    by one pair of HIP events recorded on the stream the kernels are launched on, torch's current
    stream (GPU time of the K back-to-back steps).  Events between the launches would each cost a
    ~10 us bubble on the queue, so there are none.  -> (wall ms per step, GPU ms per step)"""
    for _ in range(warmup):
        fn(xd)
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        y = fn(xd)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    del y
    return wall * 1e3 / steps, ev0.elapsed_time(ev1) / steps


def gemm_kernel_ms(wl, xd, steps, warmup):
    """Average duration of the GEMM kernel alone at the workload's shape: the operands are packed once,
    then K back-to-back launches of mxq_gemm_mx_nt are timed with one pair of HIP events."""
    g = wl["gemm_only"](xd)
    return time_steps(lambda _: g(), xd, steps, warmup)[1]


def flops_report(name, wl, steps, warmup, ms_per_step, step_gpu_ms, kernel_ms, cpu):
    """GEMM-shaped workloads.  value: whole-step TFLOP/s (quantize + pack of both operands, GEMM, bias
    and epilogue all inside the step).  roofline: the dominant kernel, the scaled-MFMA GEMM --
    2 M N K flop per launch over its average launch duration -- against the dense MFMA peak of its
    operand format."""
    peak = MFMA_PEAK_TFLOPS[wl.get("peak", "fp8")]
    value = wl["flops"] / (ms_per_step * 1e-3) / 1e12
    if kernel_ms is not None:
        achieved = wl["gemm_flops"] / (kernel_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": measured_traffic(name)[0], "traffic_source": measured_traffic(name)[1],
                "kernel": wl["gemm_kernel"], "launch_ms_avg": round(kernel_ms, 5),
                "step_gpu_ms_avg": round(step_gpu_ms, 5),
                "note": "GEMM kernel alone (operands packed beforehand) over the dense %s MFMA peak; the whole "
                        "step runs at %.1f TFLOP/s = %.4f of it" % (wl.get("peak", "fp8"),
                                                                    wl["flops"] / (step_gpu_ms * 1e-3) / 1e12,
                                                                    wl["flops"] / (step_gpu_ms * 1e-3) / 1e12 / peak)}
    else:
        achieved = wl["flops"] / (step_gpu_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": measured_traffic(name)[0], "traffic_source": measured_traffic(name)[1],
                "step_gpu_ms_avg": round(step_gpu_ms, 5),
                "note": "whole step (all launches) over the dense %s MFMA peak" % wl.get("peak", "fp8")}
    out = {"metric": METRIC, "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": steps,
           "warmup": warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": wl["dtype"], "data": "synthetic",
           "config": {"workload": name, "detail": wl["desc"], "flop_per_step": wl["flops"],
                      "tolerance": wl.get("tolerance")},
           "roofline": roof}
    if cpu:
        x = wl["x"]
        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        rows = wl["cpu_rows"]
        xs = x[:rows].contiguous()
        t0 = time.perf_counter()
        wl["cpu"](xs)
        t = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(wl["flops"] * rows / x.shape[0] / t / 1e12, 5), "unit": "TFLOP/s",
                               "cores": cores, "kind": "port",
                               "sample": "first %d of %d rows/batches of the first operand, one pass, %.1f s; "
                                         "torch op-by-op oracle" % (rows, x.shape[0], t)}
    return out


def bytes_report(name, wl, steps, warmup, ms_per_step, kern_avg_ms, cpu):
    value = wl["bytes"] / (ms_per_step * 1e-3) / 1e9
    achieved = wl["bytes"] / (kern_avg_ms * 1e-3) / 1e9
    out = {
        "metric": METRIC,
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": wl["dtype"], "data": "synthetic",
        "config": {"workload": name, "detail": wl["desc"],
                   "algorithmic_bytes_per_step": wl["bytes"],
                   "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(name)[0], "traffic_source": measured_traffic(name)[1],
                     "launch_ms_avg": round(kern_avg_ms, 5),
                     "launches_per_step": wl.get("launches", 1)},
    }
    if cpu:
        out["cpu_baseline"] = cpu_baseline(wl)
    return out


def run_workload(name, steps, warmup, cpu):
    """One workload, inputs resident in HBM before the timed region -> its report (a dict)."""
    wl = make_workload(name)
    dev = torch.device("cuda:0")
    xd = wl["x"].to(dev)
    torch.cuda.synchronize()
    ms_per_step, gpu_ms = time_steps(wl["gpu"], xd, steps, warmup)
    if "flops" in wl:
        kernel_ms = gemm_kernel_ms(wl, xd, steps, warmup) if "gemm_only" in wl else None
        return flops_report(name, wl, steps, warmup, ms_per_step, gpu_ms, kernel_ms, cpu)
    return bytes_report(name, wl, steps, warmup, ms_per_step, gpu_ms, cpu)


HEADLINE, SECONDARY = "mxfp8_fp32_8192", "mx_linear"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)     # the clocks need a few ms to ramp up
    ap.add_argument("--workload", default=None,
                    help="one workload only; default: the headline quantization, then the fused MX linear "
                         "layer of the same metric as \"secondary\" in the same JSON line")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: the quantization path has no multi-GPU part "
                         "(blocks are independent, so sharding needs no exchange step); run with --gpus 1")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU (torch.cuda.is_available() is False)")

    cpu = not args.no_cpu_baseline
    if args.workload is not None:
        out = run_workload(args.workload, args.steps, args.warmup, cpu)
    else:
        # both halves of the metric: the headline fields are the quantization throughput; the fused MX
        # linear layer (config 4), timed for the same number of steps, rides along as "secondary"
        out = run_workload(HEADLINE, args.steps, args.warmup, cpu)
        sec = run_workload(SECONDARY, args.steps, args.warmup, cpu)
        out["secondary"] = {k: sec[k] for k in ("value", "unit", "steps", "warmup", "ms_per_step", "dtype",
                                                "config", "roofline", "cpu_baseline") if k in sec}
        out["secondary"]["metric"] = "fused MX-linear TFLOP/s"
    print(json.dumps(out, ensure_ascii=False), flush=True)


if __name__ == "__main__":
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    main()
