#!/usr/bin/env python3
"""Benchmark of the MoE-layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2|C3] [--no-cpu-baseline]

One "step" is one forward + backward pass of the whole layer (router GEMM, top-K softmax, routing metadata, the two
forward grouped GEMMs, combine, the four backward grouped GEMMs, dx reduction, router backward) on seeded synthetic
inputs that are resident in HBM before the timed region.  FLOPs are counted as the reference's benchmark does
(benchmarks/moe-cute.py:231-232, :297-298): 18 * T*K * I * H for forward + backward with a gated activation; the
router GEMM and the routing kernels are in the time but not in the FLOPs.

Prints ONE JSON line on stdout; a per-kernel breakdown goes to stderr.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "sonic-moe_amd"))
sys.path.insert(0, str(ROOT))

import torch  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0
PEAK_FP8_TFLOPS = 5000.0   # MI355X dense fp8 MFMA peak

CONFIGS = {
    "C2": dict(T=32768, H=4096, I=1024, E=128, K=8, zipf=False),
    # the reference's published shapes with short down-projection contractions (its tput.png: I = 256 / 512)
    "I256": dict(T=32768, H=4096, I=256, E=256, K=16, zipf=False),
    "I512": dict(T=32768, H=4096, I=512, E=128, K=8, zipf=False),
    "C3": dict(T=32768, H=4096, I=1536, E=128, K=8, zipf=True),
    "C4": dict(T=16384, H=4096, I=1024, E=256, K=8, zipf=False, rounding="nr", tile=128),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_inputs(cfg, dev, seed=0, dtype=torch.bfloat16):
    g = torch.Generator(device=dev).manual_seed(seed)
    T, H, I, E = cfg["T"], cfg["H"], cfg["I"], cfg["E"]
    bf = dtype
    x = torch.randn(T, H, generator=g, device=dev, dtype=torch.float32).to(bf).requires_grad_()
    wr = (0.02 * torch.randn(E, H, generator=g, device=dev)).to(bf).requires_grad_()
    w1 = (0.02 * torch.randn(E, 2 * I, H, generator=g, device=dev)).to(bf).requires_grad_()
    w2 = (0.02 * torch.randn(E, H, I, generator=g, device=dev)).to(bf).requires_grad_()
    dout = torch.randn(T, H, generator=g, device=dev, dtype=torch.float32).to(bf)
    return x, wr, w1, w2, dout


def time_region(fn, steps, warmup, per_step=False):
    """ms per call: `warmup` untimed calls, then `steps` calls between two events on the current stream.  With
    per_step=True an event is recorded between the calls as well and the list of per-call times is returned too."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1 if per_step else 2)]
    t0 = time.perf_counter()
    marks[0].record()
    for k in range(steps):
        fn()
        if per_step:
            marks[k + 1].record()
    if not per_step:
        marks[1].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    mean = marks[0].elapsed_time(marks[-1]) / steps
    if per_step:
        return mean, wall, [marks[k].elapsed_time(marks[k + 1]) for k in range(steps)]
    return mean, wall


def kernel_breakdown(cfg, x, wr, w1, w2, dout, steps, only=None, gemms_only=False):
    """Time every operator of the path on its own (events on the launch stream) and return a list of dicts with
    algorithmic FLOPs / bytes.  The grouped GEMM ops launch a tile-map builder (~5 us) next to the GEMM kernel."""
    from sonicmoe.functional import _build_metadata, backward, forward

    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    TK = T * K
    dev = x.device
    bf = x.dtype
    stream = torch.cuda.current_stream().cuda_stream
    with torch.no_grad():
        logits = torch.nn.functional.linear(x, wr)
        if cfg["zipf"]:
            logits = logits + zipf_bias(E, dev).to(logits.dtype)
        scores = torch.empty(T, K, dtype=torch.float32, device=dev)
        idx = torch.empty(T, K, dtype=torch.int32, device=dev)
        forward._topk_fwd(logits, K, scores, idx, True)
        freq, off, gidx, sidx, ridx, tok_off = _build_metadata(idx.view(-1), None, T, E, K)
        z = torch.empty(TK, 2 * I, dtype=bf, device=dev)
        y1 = torch.empty(TK, I, dtype=bf, device=dev)
        y2 = torch.empty(TK, H, dtype=bf, device=dev)
        o = torch.empty(T, H, dtype=bf, device=dev)
        dz = torch.empty_like(z)
        ds = torch.empty(TK, dtype=torch.float32, device=dev)
        dw1 = torch.empty_like(w1).permute(1, 2, 0)
        dw2 = torch.empty_like(w2).permute(1, 2, 0)
        dxe = torch.empty(TK, H, dtype=bf, device=dev)
        dx = torch.empty(T, H, dtype=bf, device=dev)
        dlog = torch.zeros(T, E, dtype=bf, device=dev)
        sl_acc = torch.empty(E, dtype=torch.float32, device=dev)
        sl_aux = torch.empty(1, dtype=torch.float32, device=dev)
        sl_g = torch.ones(1, dtype=torch.float32, device=dev)
        w1v, w2v = w1.detach().permute(1, 2, 0), w2.detach().permute(1, 2, 0)
        xd = x.detach()
        sflat = scores.view(-1)
        gemm = 2.0 * TK * I * H
        ops = [
            ("router_gemm(hipBLASLt)", lambda: torch.nn.functional.linear(xd, wr.detach()), 2.0 * T * H * E, None),
            ("topk_softmax", lambda: forward._topk_fwd(logits, K, scores, idx, True), None, T * E * 2 + T * K * 8),
            ("routing_metadata", lambda: _build_metadata(idx.view(-1), None, T, E, K), None, TK * 4 * 4),
            ("up_projection_forward", lambda: forward._up_projection_forward(xd, w1v, z, y1, None, off, None, gidx, stream, "swiglu", True, False), 2 * gemm, None),
            ("down_projection_forward", lambda: forward._down_projection_forward(w2v, y1, y2, None, off, None, gidx, stream), gemm, None),
            ("router_forward(combine)", lambda: forward._router_forward(y2, o, sflat, ridx, tok_off, K, H, False), None, TK * H * 2 + T * H * 2 + TK * 8),
            ("down_projection_backward(dz only)", lambda: backward._down_projection_backward(dout, z, w2v, None, dz, ds, None, None, sflat, off, None, gidx, sidx, stream, True, "swiglu"), gemm, None),
            ("down_projection_backward(dz+dW2)", lambda: backward._down_projection_backward(dout, z, w2v, dw2, dz, ds, None, None, sflat, off, None, gidx, sidx, stream, True, "swiglu"), 2 * gemm, None),
            ("up_projection_backward(dW1 only)", lambda: backward._up_projection_backward(xd, w1v, None, dw1, dz, None, off, None, gidx, sidx, True, stream), 2 * gemm, None),
            ("up_projection_backward(dx only)", lambda: backward._up_projection_backward(xd, w1v, dxe, None, dz, None, off, None, gidx, sidx, True, stream), 2 * gemm, None),
            ("token_broadcast_backward", lambda: backward._token_broadcast_backward(dx, dxe, ridx, tok_off, K, H, False), None, TK * H * 2 + T * H * 2 + TK * 4),
            ("softmax_topk_bwd", lambda: backward._softmax_topk_bwd(dlog, None, ds.view(T, K), scores, idx, K), None, T * K * 12 + T * E * 2),
            # auxiliary (switch) loss of MoE.forward: not part of the timed layer step, listed for completeness
            ("switch_loss_fwd", lambda: forward._switch_loss_fwd(logits, freq, sl_acc, sl_aux), None, T * E * 2),
            ("switch_loss_bwd", lambda: backward._switch_loss_bwd(logits, freq, sl_acc, sl_g, dlog), None, T * E * 4),
        ]
        if forward.router_fused_supported(xd, wr.detach()):
            # the router in one kernel (opt-in, sonicmoe.functional.fused_router): replaces router_gemm + topk_softmax and
            # the column-sum pass of switch_loss_fwd
            rf_logits = torch.empty(T, E, dtype=bf, device=dev)
            rf_part = torch.empty(forward.router_fused_partials(T, E), E, dtype=torch.float32, device=dev)
            ops.append(("router_forward_fused(gemm+topk+colsum)",
                        lambda: forward._router_forward_fused(xd, wr.detach(), rf_logits, scores, idx, rf_part),
                        2.0 * T * H * E, T * H * 2 + T * E * 2 + T * K * 8))
        # the down projection fused with the combine (opt-in, sonicmoe.functional.fused_combine): zero-fill of the output
        # + one kernel with atomic adds, against down_projection_forward + router_forward(combine) above
        o_fused = torch.empty(T, H, dtype=bf, device=dev)

        def down_combine_fused():
            o_fused.zero_()
            forward._down_projection_forward_combine(w2v, y1, o_fused, None, sflat, off, None, gidx, sidx, stream)

        ops.append(("down_projection_forward_fused_combine(atomics)", down_combine_fused, gemm, None))
        if gemms_only:
            ops = [o for o in ops if o[2] and "router_gemm" not in o[0] and "fused_combine" not in o[0]]
        if H % 128 == 0 and I % 128 == 0 and (only is None or only.startswith("fp8:")) and not gemms_only:
            # fp8 forward (config 5 = this shape with block-scaled e4m3 operands): quantisers and the two fp8 GEMMs
            from sonicmoe.functional import fp8

            xq, xs = fp8.mx_quantize(xd)
            w1q, w1s = fp8.quantize_expert_weight(w1v)
            w2q, w2s = fp8.quantize_expert_weight(w2v)
            y1q, y1s = fp8.mx_quantize(y1)
            w1_2d, w2_2d = w1.detach().view(E * 2 * I, H), w2.detach().view(E * H, I)
            ops += [
                ("fp8:quantize(x)", lambda: fp8._mx_quantize(xd, xq, xs), None, T * H * 3 + T * H // 32),
                ("fp8:quantize(W1)", lambda: fp8._mx_quantize(w1_2d, w1q, w1s), None, E * 2 * I * H * 3 + E * 2 * I * H // 32),
                ("fp8:up_projection_forward(+quantised y1)", lambda: fp8._up_projection_forward_fp8(xq, xs, w1q, w1s, z, None, None, off, gidx, E, stream, "swiglu", True, y1q, y1s), 2 * gemm, None),
                ("fp8:quantize(W2)", lambda: fp8._mx_quantize(w2_2d, w2q, w2s), None, E * H * I * 3 + E * H * I // 32),
                ("fp8:down_projection_forward", lambda: fp8._down_projection_forward_fp8(y1q, y1s, w2q, w2s, y2, None, off, E, stream), gemm, None),
            ]
            # fp8 activation gradients: dout and the transposed weights quantised, dz (+ its quantised copy), dx
            doq, dos = fp8.mx_quantize(dout)
            w2tq, w2ts = fp8.quantize_expert_weight_transposed(w2v)
            w1tq, w1ts = fp8.quantize_expert_weight_transposed(w1v)
            w2t3, w1t3 = w2tq.view(E, I, H), w1tq.view(E, H, 2 * I)
            dzq = torch.empty(TK, 2 * I, dtype=torch.uint8, device=dev)
            dzs = torch.empty(2 * I // 128, TK, dtype=torch.int32, device=dev)
            y1sc = torch.empty(TK, I, dtype=bf, device=dev)
            ops += [
                ("fp8:quantize(dout)", lambda: fp8._mx_quantize(dout, doq, dos), None, T * H * 3 + T * H // 32),
                ("fp8:quantize_transposed(W2)", lambda: fp8._mx_quantize_transposed(w2.detach(), w2t3, w2ts), None, E * H * I * 3 + E * H * I // 32),
                ("fp8:down_projection_backward(dz, +quantised dz)", lambda: fp8._down_projection_backward_fp8(doq, dos, w2tq, w2ts, z, dz, dzq, dzs, y1sc, ds, sflat, off, gidx, sidx, E, stream, "swiglu", True), gemm, None),
                ("fp8:quantize_transposed(W1)", lambda: fp8._mx_quantize_transposed(w1.detach(), w1t3, w1ts), None, E * 2 * I * H * 3 + E * 2 * I * H // 32),
                ("fp8:up_projection_backward(dx)", lambda: fp8._down_projection_forward_fp8(dzq, dzs, w1tq, w1ts, dxe, None, off, E, stream), 2 * gemm, None),
                # what a training step runs instead of the four weight quantisers above: both copies from one read
                ("fp8:quantize_both(W1)", lambda: fp8._mx_quantize_both(w1.detach(), w1q, w1s, w1t3, w1ts), None, E * 2 * I * H * 4 + E * 2 * I * H // 16),
                ("fp8:quantize_both(W2)", lambda: fp8._mx_quantize_both(w2.detach(), w2q, w2s, w2t3, w2ts), None, E * H * I * 4 + E * H * I // 16),
            ]
        rows = []
        for name, fn, flops, nbytes in ops:
            if only is not None and name != only:
                continue
            ms, _ = time_region(fn, steps, 2)
            row = dict(op=name, ms=round(ms, 4))
            if flops and name.startswith("fp8:"):
                row["tflops"] = round(flops / ms / 1e9, 1)
                row["frac_fp8_mfma_peak"] = round(flops / ms / 1e9 / PEAK_FP8_TFLOPS, 4)
                row["frac_mfma_peak"] = row["frac_fp8_mfma_peak"]
                row["flops"] = flops
            elif flops:
                row["tflops"] = round(flops / ms / 1e9, 1)
                row["frac_mfma_peak"] = round(flops / ms / 1e9 / PEAK_BF16_TFLOPS, 4)
                row["flops"] = flops
            if nbytes:
                row["gbs"] = round(nbytes / ms / 1e6, 1)
                row["frac_hbm_peak"] = round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)
            rows.append(row)
            log(f"  {name:36s} {ms:9.4f} ms" + (f"  {row['tflops']:8.1f} TFLOP/s ({100*row['frac_mfma_peak']:.1f}% peak)" if flops else "")
                + (f"  {row['gbs']:8.1f} GB/s ({100*row['frac_hbm_peak']:.1f}% HBM)" if nbytes else ""))
    return rows


def vendor_dense(cfg, dev, steps=5):
    """The vendor library (hipBLASLt through torch.matmul) on the dense GEMM of the same shape as each grouped GEMM, same
    process, warm, random bf16 data: what the machine's own best GEMM kernel does with these FLOPs when there is no
    gather, no expert boundary and no fused epilogue.  The two weight-gradient GEMMs are E separate (N x tokens) @
    (tokens x M) products with TK / E tokens each, launched back to back."""
    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    TK = T * K
    bf = torch.bfloat16
    res = {}

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, device=dev, dtype=torch.float32) * scale).to(bf)

    with torch.no_grad():
        for name, (m, k, n) in {
            "up_projection_forward": (TK, H, 2 * I),
            "down_projection_forward": (TK, I, H),
            "down_projection_backward(dz only)": (TK, H, I),
            "up_projection_backward(dx only)": (TK, 2 * I, H),
        }.items():
            a, b = rnd(m, k), rnd(n, k, scale=0.02)
            c = torch.empty(m, n, dtype=bf, device=dev)
            ms, _ = time_region(lambda: torch.matmul(a, b.t(), out=c), steps, 2)
            res[name] = round(2.0 * m * k * n / ms / 1e9, 1)
            del a, b, c
        tok = TK // E
        for name, (n, m) in {"up_projection_backward(dW1 only)": (2 * I, H), "dW2": (H, I)}.items():
            a, b = rnd(TK, n), rnd(TK, m)
            c = torch.empty(E, n, m, dtype=bf, device=dev)

            def per_expert():
                for e in range(E):
                    torch.matmul(a[e * tok:(e + 1) * tok].t(), b[e * tok:(e + 1) * tok], out=c[e])

            ms, _ = time_region(per_expert, max(2, steps // 2), 1)
            res[name] = round(2.0 * TK * n * m / ms / 1e9, 1)
            del a, b, c
    torch.cuda.empty_cache()
    return res


# operators that are one grouped-GEMM kernel launch (plus a ~5 us tile-map builder), and the kernel they launch
SINGLE_KERNEL_OPS = {
    "up_projection_forward": "varlen_m_asm_kernel<up-projection forward>",
    "down_projection_forward": "varlen_m_asm_kernel<down-projection forward>",
    "down_projection_backward(dz only)": "varlen_m_asm_kernel<dz>",
    "up_projection_backward(dW1 only)": "varlen_k_stream_kernel<dW1>",
    "up_projection_backward(dx only)": "varlen_m_asm_kernel<dx_expanded>",
    "fp8:up_projection_forward(+quantised y1)": "fp8_stream_kernel<up-projection forward>",
    "fp8:down_projection_forward": "fp8_stream_kernel<down-projection forward>",
    "fp8:down_projection_backward(dz, +quantised dz)": "fp8_varlen_m_kernel<dz>",
    "fp8:up_projection_backward(dx)": "fp8_stream_kernel<dx_expanded>",
}


def recorded_traffic(kernel: str, config: str):
    """HBM bytes per launch of `kernel`, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and calibrated against
    a copy of known size; recorded in profiles/hbm_traffic.json (None if that kernel has no record)."""
    f = ROOT / "profiles" / "hbm_traffic.json"
    if not f.exists():
        return None
    try:
        return json.loads(f.read_text()).get(config, {}).get(kernel)
    except (ValueError, OSError):
        return None


def pmc_target(cfg, op_name, dev, dtype=torch.bfloat16):
    """Workload for the counter passes: 3 launches of one operator's kernel and one 1 GiB device-to-device copy whose
    FETCH_SIZE / WRITE_SIZE readings calibrate the counters."""
    x, wr, w1, w2, dout = make_inputs(cfg, dev, dtype=dtype)
    a = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    b = torch.empty_like(a)
    b.copy_(a)
    torch.cuda.synchronize()
    import contextlib, io

    with contextlib.redirect_stderr(io.StringIO()):
        rows = kernel_breakdown(cfg, x, wr, w1, w2, dout, 1, only=op_name)
    torch.cuda.synchronize()
    print(json.dumps(dict(pmc_target=op_name, copy_bytes=a.numel() * 4, rows=rows)))


def zipf_bias(E, dev):
    e = torch.arange(E, device=dev, dtype=torch.float32)
    return 2.0 * torch.log(1.0 / (e + 1.0))


def cpu_baseline(cfg, budget_s=20.0):
    """The oracle's restated torch backend (fp32, torch.autograd backward) on the host cores, on a bounded sample of the
    same workload: same H, I, E, K, tokens scaled down so that one forward+backward pass takes seconds."""
    from oracle import moe_math as M

    H, I, E, K = cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    T = 1024
    torch.manual_seed(0)
    x = torch.randn(T, H, requires_grad=True)
    wr = (0.02 * torch.randn(E, H)).requires_grad_()
    w1 = (0.02 * torch.randn(E, 2 * I, H)).requires_grad_()
    w2 = (0.02 * torch.randn(E, H, I)).requires_grad_()
    dout = torch.randn(T, H)
    flops = 18.0 * T * K * I * H

    def step():
        out, _, _ = M.moe_torch_backend(x, wr, w1, w2, K)
        torch.autograd.grad(out, [x, wr, w1, w2], grad_outputs=dout)

    step()  # warm-up (thread pool, allocator)
    times = []
    t_start = time.perf_counter()
    while len(times) < 5 and (time.perf_counter() - t_start) < budget_s:
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    best = sorted(times)[len(times) // 2]

    # the reference's own CPU-runnable case, whole: fp32, T=1024 H=512 I=256 E=8 K=2, loss = sum(out * g), seed 0
    c1 = dict(T=1024, H=512, I=256, E=8, K=2)
    torch.manual_seed(0)
    x1 = torch.randn(c1["T"], c1["H"], requires_grad=True)
    wr1 = (0.02 * torch.randn(c1["E"], c1["H"])).requires_grad_()
    w11 = (0.02 * torch.randn(c1["E"], 2 * c1["I"], c1["H"])).requires_grad_()
    w21 = (0.02 * torch.randn(c1["E"], c1["H"], c1["I"])).requires_grad_()
    g1 = torch.randn(c1["T"], c1["H"])

    def step1():
        out, _, _ = M.moe_torch_backend(x1, wr1, w11, w21, c1["K"])
        (out * g1).sum().backward()
        for t in (x1, wr1, w11, w21):
            t.grad = None

    step1()
    times1 = []
    for _ in range(7):
        t0 = time.perf_counter()
        step1()
        times1.append(time.perf_counter() - t0)
    best1 = sorted(times1)[len(times1) // 2]
    flops1 = 18.0 * c1["T"] * c1["K"] * c1["I"] * c1["H"]
    return dict(
        value=round(flops / best / 1e12, 4),
        unit="TFLOP/s",
        cores=torch.get_num_threads(),
        kind="port",
        sample=f"oracle.moe_torch_backend fp32 fwd+bwd, T={T} tokens (1/{cfg['T'] // T} of the workload's tokens), "
        f"H={H} I={I} E={E} K={K}; median of {len(times)} passes, {best * 1e3:.0f} ms per pass",
        config1=dict(
            workload="C1: fp32 fwd+bwd on the host, T=1024 H=512 I=256 E=8 K=2, SwiGLU, no bias, loss = sum(out * g), seed 0",
            ms_per_step=round(best1 * 1e3, 3),
            tflops=round(flops1 / best1 / 1e12, 4),
            passes=len(times1),
        ),
    )


def measure_layer(cfg, name, dev, steps, warmup, dtype=torch.bfloat16):
    """Forward and forward+backward of the whole layer at one configuration.  Returns (record, tensors) where tensors are
    the inputs, kept for the per-kernel breakdown of the headline configuration."""
    from sonicmoe.enums import ActivationType
    from sonicmoe.functional import (
        TC_Softmax_Topk_Router_Function,
        _build_metadata,
        _ExpertsFunction,
        moe_general_routing_inputs,
        moe_TC_softmax_topk_layer,
    )

    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    x, wr, w1, w2, dout = make_inputs(cfg, dev, dtype=dtype)
    stream = torch.cuda.current_stream().cuda_stream
    w1v, w2v = w1.permute(1, 2, 0), w2.permute(1, 2, 0)
    bias = zipf_bias(E, dev).to(dtype) if cfg["zipf"] else None

    rounding = cfg.get("rounding")
    if rounding:
        from sonicmoe.routing import token_choice_rounding

        with torch.no_grad():  # the rounding router is outside the timed region, as in the reference's benchmark
            r_scores, r_tok, r_exp = token_choice_rounding(torch.nn.functional.linear(x, wr), K, cfg["tile"], rounding)
        r_scores = r_scores.float().requires_grad_()

    def layer():
        if rounding:
            o, _ = moe_general_routing_inputs(x, r_scores, r_tok, r_exp, w1v, None, w2v, None, E, stream,
                                              ActivationType.SWIGLU, False)
            return o
        if bias is None:
            o, _, _ = moe_TC_softmax_topk_layer(x, wr, w1v, None, w2v, None, K, stream, ActivationType.SWIGLU, False)
            return o
        logits = torch.nn.functional.linear(x, wr) + bias
        s, i = TC_Softmax_Topk_Router_Function.apply(logits, E, K)
        _, off, gidx, sidx, ridx, tok_off = _build_metadata(i.view(-1), None, T, E, K)
        return _ExpertsFunction.apply(x, w1v, None, w2v, None, s.view(-1), off, gidx, sidx, ridx, tok_off, K, False,
                                      ActivationType.SWIGLU, stream, False)

    def fwd_only():
        with torch.no_grad():
            layer()

    def fwd_bwd():
        o = layer()
        torch.autograd.grad(o, [x, r_scores, w1, w2] if rounding else [x, wr, w1, w2], grad_outputs=dout)

    TK = r_tok.numel() if rounding else T * K
    flops_fwd, flops_all = 6.0 * TK * I * H, 18.0 * TK * I * H
    fwd_ms, _ = time_region(fwd_only, steps, warmup)
    ms, wall_ms, per_step = time_region(fwd_bwd, steps, warmup, per_step=True)
    per_step.sort()
    # peak memory of one step above what is resident between steps (inputs, weights): activations kept for the backward
    # pass, transient buffers and the gradients while they are being produced
    torch.cuda.synchronize()
    resident = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    o = layer()
    torch.cuda.synchronize()
    held_for_backward = torch.cuda.memory_allocated() - resident - o.numel() * o.element_size()
    peak_forward = torch.cuda.max_memory_allocated() - resident
    torch.autograd.grad(o, [x, r_scores, w1, w2] if rounding else [x, wr, w1, w2], grad_outputs=dout)
    torch.cuda.synchronize()
    peak_step = torch.cuda.max_memory_allocated() - resident
    del o
    tflops = flops_all / ms / 1e9
    rec = dict(
        workload=f"{name}: MoE layer fwd+bwd, T={T} H={H} I={I} E={E} K={K}, SwiGLU, no bias, token-choice softmax "
        f"top-k router{' with Zipf logit bias' if cfg['zipf'] else ''}"
        f"{' then token rounding (' + rounding + ', tile 128), ' + str(TK) + ' routed pairs, general-routing entry' if rounding else ''}"
        f"; x,dout~N(0,1), weights~N(0,0.02), seed 0",
        flops_per_step=flops_all,
        ms_per_step=round(ms, 4),
        ms_per_step_median=round(per_step[len(per_step) // 2], 4),
        ms_per_step_min=round(per_step[0], 4),
        tflops=round(tflops, 2),
        frac_of_peak=round(tflops / PEAK_BF16_TFLOPS, 4),
        fwd_ms=round(fwd_ms, 4),
        fwd_tflops=round(flops_fwd / fwd_ms / 1e9, 2),
        host_wall_ms_per_step=round(wall_ms, 4),
        activation_bytes_held_for_backward=int(held_for_backward),
        peak_bytes_forward=int(peak_forward),
        peak_bytes_step=int(peak_step),
    )
    log(f"{name}: fwd {fwd_ms:.3f} ms ({flops_fwd / fwd_ms / 1e9:.1f} TFLOP/s), fwd+bwd {ms:.3f} ms mean / "
        f"{rec['ms_per_step_median']:.3f} median / {rec['ms_per_step_min']:.3f} min ({tflops:.1f} TFLOP/s = "
        f"{100 * tflops / PEAK_BF16_TFLOPS:.1f}% of bf16 MFMA peak); kept for backward "
        f"{held_for_backward / 2**30:.2f} GiB, peak of a step {peak_step / 2**30:.2f} GiB above the resident tensors")
    return rec, dict(x=x, wr=wr, w1=w1, w2=w2, dout=dout, layer=layer, fwd_only=fwd_only, fwd_bwd=fwd_bwd,
                     flops_fwd=flops_fwd, flops_all=flops_all)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="C2", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the extra lines (C3, C4 layer times; per-kernel rows of the short-contraction shapes)")
    ap.add_argument("--pmc-dtype", default="bf16", choices=["bf16", "fp16"],
                    help="element type of the --pmc-target workload (fp16 = the second build of the library)")
    ap.add_argument("--pmc-target", default=None, choices=sorted(SINGLE_KERNEL_OPS),
                    help="run only this operator (3 launches) and a 1 GiB copy: the workload of the rocprofv3 --pmc passes")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one MI355X: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    cfg = CONFIGS[a.config]
    dev = torch.device("cuda:0")
    if a.pmc_target:
        pmc_target(cfg, a.pmc_target, dev, torch.float16 if a.pmc_dtype == "fp16" else torch.bfloat16)
        return
    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    rec, t = measure_layer(cfg, a.config, dev, a.steps, a.warmup)
    rounding = cfg.get("rounding")

    fp8_info = fp8_step = None
    if not rounding and not cfg["zipf"] and H % 128 == 0 and I % 128 == 0:
        from sonicmoe import enable_fp8_backward, enable_fp8_forward
        from sonicmoe.functional.fp8 import cache_quantized_weights

        with torch.no_grad():
            ref_out = t["layer"]()
            with enable_fp8_forward():
                fp8_out = t["layer"]()
                with cache_quantized_weights(False):
                    fp8_ms, _ = time_region(t["fwd_only"], a.steps, a.warmup)
                fp8_cached_ms, _ = time_region(t["fwd_only"], a.steps, a.warmup)
        rel = float((fp8_out.float() - ref_out.float()).norm() / ref_out.float().norm())
        fp8_info = dict(
            what="forward with block-scaled e4m3 operands (x, W1, y1, W2 quantised inside the timed region), bf16 outputs; "
            "fwd_ms_weights_quantised_once: W1, W2 quantised before the timed region (inference)",
            fwd_ms=round(fp8_ms, 4),
            fwd_ms_weights_quantised_once=round(fp8_cached_ms, 4),
            fwd_tflops=round(t["flops_fwd"] / fp8_ms / 1e9, 2),
            frac_of_fp8_peak=round(t["flops_fwd"] / fp8_ms / 1e9 / PEAK_FP8_TFLOPS, 4),
            rel_l2_vs_bf16_forward=round(rel, 4),
        )
        log(f"fp8 forward: {fp8_ms:.3f} ms ({fp8_info['fwd_tflops']:.1f} TFLOP/s), rel-L2 vs bf16 forward {rel:.4f}")
        del ref_out, fp8_out
        # the whole step with the four activation-side GEMMs on fp8 operands (weights quantised inside the timed region,
        # twice each: along either index); the two weight-gradient GEMMs are the bf16 ones
        with enable_fp8_forward(), enable_fp8_backward(), cache_quantized_weights(False):
            ms8, _, per8 = time_region(t["fwd_bwd"], a.steps, a.warmup, per_step=True)
        per8.sort()
        fp8_step = dict(
            what="fwd+bwd with x, W1, y1, W2 (forward) and dout, W2^T, dz, W1^T (activation gradients) as block-scaled "
            "e4m3, every quantisation inside the timed region; dW1, dW2 are bf16 GEMMs",
            ms_per_step=round(ms8, 4),
            ms_per_step_median=round(per8[len(per8) // 2], 4),
            ms_per_step_min=round(per8[0], 4),
            tflops=round(t["flops_all"] / ms8 / 1e9, 2),
            frac_of_bf16_peak=round(t["flops_all"] / ms8 / 1e9 / PEAK_BF16_TFLOPS, 4),
        )
        log(f"fp8 fwd+bwd: {ms8:.3f} ms ({fp8_step['tflops']:.1f} TFLOP/s of useful work)")

    rows = [] if (a.no_breakdown or rounding) else kernel_breakdown(cfg, t["x"], t["wr"], t["w1"], t["w2"], t["dout"],
                                                                    max(5, a.steps // 2))
    if rows and not a.no_other_configs:
        # the vendor library's dense rate on each grouped GEMM's shape: a same-box, same-run ceiling per kernel
        ceil = vendor_dense(cfg, dev)
        for r in rows:
            if r["op"] in ceil:
                r["vendor_dense_tflops"] = ceil[r["op"]]
            elif r["op"] == "down_projection_backward(dz+dW2)":
                r["vendor_dense_tflops_dW2"] = ceil["dW2"]
        log("vendor dense GEMM (hipBLASLt) on the same shapes: " + ", ".join(f"{k} {v:.0f}" for k, v in ceil.items()))
    # dominant kernel = the single grouped-GEMM launch with the largest average duration
    single = [r for r in rows if r["op"] in SINGLE_KERNEL_OPS and not r["op"].startswith("fp8:")]
    roofline = None
    if single:
        dom = max(single, key=lambda r: r["ms"])
        roofline = dict(
            bound="mfma",
            kernel=SINGLE_KERNEL_OPS[dom["op"]],
            op=dom["op"],
            avg_launch_ms=dom["ms"],
            achieved=dom["tflops"],
            peak=PEAK_BF16_TFLOPS,
            unit="TFLOP/s",
            frac=dom["frac_mfma_peak"],
            traffic=recorded_traffic(SINGLE_KERNEL_OPS[dom["op"]], a.config),
        )

    out = dict(
        metric=f"MoE fwd+bwd TFLOP/s (% bf16 MFMA peak), T={T} H={H} I={I} E={E} K={K}",
        value=rec["tflops"],
        unit="TFLOP/s",
        n_gpus=1,
        steps=a.steps,
        warmup=a.warmup,
        ms_per_step=rec["ms_per_step"],
        ms_per_step_median=rec["ms_per_step_median"],
        ms_per_step_min=rec["ms_per_step_min"],
        higher_is_better=True,
        scaling="weak",
        vs_baseline=None,
        dtype="bf16",
        data="synthetic",
        config=dict(workload=rec["workload"], flops_per_step=rec["flops_per_step"]),
        frac_of_peak=rec["frac_of_peak"],
        fwd_ms=rec["fwd_ms"],
        fwd_tflops=rec["fwd_tflops"],
        activation_bytes_held_for_backward=rec["activation_bytes_held_for_backward"],
        peak_activation_bytes=rec["peak_bytes_forward"],
        peak_bytes_step=rec["peak_bytes_step"],
        roofline=roofline,
        fp8_forward=fp8_info,
        fp8_fwd_bwd=fp8_step,
        kernels=[{k: v for k, v in r.items() if k != "flops"} for r in rows],
    )
    del t
    torch.cuda.empty_cache()

    if not a.no_other_configs and a.config == "C2":
        # the other benchmark configurations (whole layer) and the reference's short-contraction shapes (per kernel):
        # extra keys, not the headline
        others = {}
        for name in ("C3", "C4"):
            r, tt = measure_layer(CONFIGS[name], name, dev, max(5, a.steps // 2), 2)
            others[name] = r
            del tt
            torch.cuda.empty_cache()
        out["other_configs"] = others
        # the headline configuration on fp16 tensors (the second build of the library; same kernels, f16 MFMA)
        try:
            r16, tt = measure_layer(CONFIGS["C2"], "C2 on fp16 tensors", dev, max(5, a.steps // 2), 2,
                                    dtype=torch.float16)
            out["fp16_fwd_bwd"] = {k: r16[k] for k in ("ms_per_step", "tflops", "frac_of_peak", "fwd_ms", "fwd_tflops")}
            del tt
        except RuntimeError as e:  # an extra line must not cost the headline (e.g. the fp16 library was not built)
            out["fp16_fwd_bwd"] = {"error": str(e)}
        torch.cuda.empty_cache()
        shapes = {}
        for name in ("I512", "I256"):
            c = CONFIGS[name]
            xs, wrs, w1s, w2s, ds = make_inputs(c, dev)
            log(f"{name}: T={c['T']} H={c['H']} I={c['I']} E={c['E']} K={c['K']}")
            shapes[name] = [{k: v for k, v in r.items() if k != "flops"}
                            for r in kernel_breakdown(c, xs, wrs, w1s, w2s, ds, 5, gemms_only=True)]
            del xs, wrs, w1s, w2s, ds
            torch.cuda.empty_cache()
        out["short_contraction_shapes"] = shapes

    if not a.no_cpu_baseline:
        torch.cuda.empty_cache()
        out["cpu_baseline"] = cpu_baseline(cfg)
        log("cpu baseline:", out["cpu_baseline"])
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
