#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--extra]

One "step" is one pass of the FLUX DiT MLP FP8 chain over one batch of synthetic tokens
(BASELINE.json configs[2], M=4608 tokens = 4096 image + 512 text at 1024^2):

    x bf16 [4608,3072]  --fp8 amax+cast-->  e4m3
        --FP8 GEMM 3072->12288, bias fused, bf16 out, the largest output left beside it-->  u [4608,12288]
    u --tanh-GELU, dynamic scale max|h|/448 (from the largest output: GELU is monotone there) and e4m3 cast, one pass--> e4m3
      --FP8 GEMM 12288->3072, bias, bf16 out-->  y [4608,3072]

(The activation sits in the memory-bound cast pass, where the vector ALU is idle, instead of the GEMM's epilogue, where it
costs 19-26 us: the GEMM then runs as the persistent one-wavefront-per-SIMD kernel.  `kernels` also times the up projection
with bias + GELU + output maximum in its epilogue, the form this chain used before.)

Inputs and (pre-quantised, rows32-repacked) weights are resident in HBM before the timed region.
`value` is the GEMM work of the step (2*M*N*K summed over both GEMMs) divided by the wall time of
the whole step, quant kernels included.  The JSON line also carries:
  roofline      the dominant kernel (up-projection FP8 GEMM) priced against the dense FP8 MFMA peak
                from HIP-event timings taken inside the timed steps, on the launch stream (every
                --event-every-th step brackets one kernel: markers are not free, see --help); beside it, measured after the
                timed region: the same kernel on all-zero operands, the shader clock under it, under the vendor library's
                FP8 GEMM and idle, the vendor GEMM's time on both shapes, and `matrix_pipes_alone`: the FP8 MFMA stream
                of a 128x128 wavefront tile on register operands without any memory traffic (what the part's power
                limit leaves of the published peak before a GEMM has moved a byte);
  cpu_baseline  the same math (dequantise e4m3 -> fp32 matmul -> scale/bias/GELU) through PyTorch
                CPU on the host cores (oracle port; a reported baseline only);
  kernels       per-kernel averages of the same timed steps (GEMM TFLOP/s, act-quant GB/s);
  extra         (with --extra) INT8 / W4A4 / SDXL-shape kernels, measured after the timed region.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP8_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 MFMA (2.5 PFLOP/s bf16 x 2)
INT8_PEAK_TOPS = 5000.0
HBM_PEAK_GBS = 8000.0

M, D, H = 4608, 3072, 12288


def make_inputs(torch, dev, seed=1002):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, D, generator=g).to(torch.bfloat16)
    w_up = (torch.randn(H, D, generator=g) * 0.02).to(torch.bfloat16)
    w_dn = (torch.randn(D, H, generator=g) * 0.02).to(torch.bfloat16)
    b_up = (torch.randn(H, generator=g) * 0.02).to(torch.bfloat16)
    b_dn = (torch.randn(D, generator=g) * 0.02).to(torch.bfloat16)
    return x, w_up, w_dn, b_up, b_dn


def cpu_baseline(torch, x, w_up, w_dn, b_up, b_dn, rows):
    """Oracle port on the host cores: e4m3 quantise, dequantise to fp32, torch.matmul, epilogue."""
    import numpy as np

    from oracle import oracle as O

    nthreads = os.cpu_count() or 1
    torch.set_num_threads(nthreads)
    xs = x[:rows].float().numpy()
    qwu, swu = O.fp8_amax_cast(w_up.float().numpy())
    qwd, swd = O.fp8_amax_cast(w_dn.float().numpy())
    wu = torch.from_numpy(O.e4m3_decode(qwu))
    wd = torch.from_numpy(O.e4m3_decode(qwd))
    t0 = time.perf_counter()
    qa, sa = O.fp8_amax_cast(xs)
    a = torch.from_numpy(O.e4m3_decode(qa))
    h = ((a @ wu.t()) * float(np.float32(sa) * np.float32(swu)) + b_up.float()).to(torch.bfloat16)  # the GEMM stores bf16
    h = torch.nn.functional.gelu(h.float(), approximate="tanh").to(torch.bfloat16)
    qh, sh = O.fp8_amax_cast(h.float().numpy())
    hh = torch.from_numpy(O.e4m3_decode(qh))
    y = ((hh @ wd.t()) * float(np.float32(sh) * np.float32(swd)) + b_dn.float()).to(torch.bfloat16)
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * (D * H + H * D)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first {rows} of {M} token rows, both GEMMs + both act-quant passes, PyTorch CPU fp32 matmul "
                      f"on dequantised e4m3 ({dt:.1f} s)"}, y


def profiled_traffic():
    """HBM-side bytes per launch of the roofline kernel from the committed rocprofv3 --pmc summary (a line
    `roofline.traffic_bytes_per_launch = <number>`); (None, None) when the summary is not there."""
    import re

    rel = "profiles/bench_flux_mlp_fp8_hbm_traffic.md"
    try:
        with open(os.path.join(ROOT, rel)) as f:
            m = re.search(r"roofline\.traffic_bytes_per_launch\s*=\s*([0-9.eE+]+)", f.read())
        return (float(m.group(1)), rel) if m else (None, None)
    except OSError:
        return None, None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=M)
    ap.add_argument("--extra", action="store_true", help="also time the INT8 / W4A4 / SDXL-shape kernels")
    ap.add_argument("--chain-only", action="store_true",
                    help="time the chain and its four kernels only: no zero-operand, row-major, vendor, clock or matrix-pipe launches")
    ap.add_argument("--row-major", action="store_true",
                    help="run the chain on row-major quantised activations (the reference's layout) instead of k-panels")
    ap.add_argument("--event-every", type=int, default=2,
                    help="on every N-th timed step ONE kernel is bracketed by a pair of HIP events (the up GEMM on every other "
                         "such step, the three others in turn); markers are not free -- five of them in one step cost the "
                         "GPU 15-20 us -- so a marked step carries two and the per-kernel figures come from a sample")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path shards by token rows without "
              "collectives, so N GPUs are N independent copies of this run). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the quantized-linear path has no CPU fallback.", file=sys.stderr)
        sys.exit(3)
    from lyradiff_amd import ops

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    x, w_up, w_dn, b_up, b_dn = make_inputs(torch, dev)

    # ---- one-time weight preparation (offline in a deployment): per-tensor e4m3 + rows32 repack ----
    xd = x.to(dev)
    wq_up, s_up = ops.fp8_quant(w_up.to(dev))
    wq_dn, s_dn = ops.fp8_quant(w_dn.to(dev))
    wp_up, wp_dn = ops.repack_weight(wq_up), ops.repack_weight(wq_dn)
    bu, bd = b_up.to(dev), b_dn.to(dev)
    del wq_up, wq_dn
    # rotating activation copies (> 256 MB in total) so that the first quant kernel reads HBM, not cache
    n_rot = 12
    xs = [xd.clone() for _ in range(n_rot)]

    # set-up-time tile-configuration search for the two GEMM shapes, as the reference's GemmPluginProfiler does at
    # initialisation (outside the timed region; the winners are cached inside the library by shape)
    tactics = {f"{n}x{k}": ops.gemm_profile("fp8", M, n, k, dev)[0] for (n, k) in ((H, D), (D, H))}

    s_h = [torch.zeros(1, dtype=torch.float32, device=dev) for _ in range(2)]
    ev = lambda: torch.cuda.Event(enable_timing=True)
    names = ["quant_x", "gemm_up", "quant_h", "gemm_down"]
    marks = {n: [] for n in names}

    calls = [0]

    # The four kernels of a step.  Quantised activations travel between them as k-panels [K/64, M, 64] (written by the
    # quantisers in the same pass, read by the GEMMs in whole cache lines; codes, scales and outputs are bit for bit those
    # of the row-major calls, which --row-major times instead).
    if args.row_major:
        quant_x = ops.fp8_quant
        gemm_up = lambda q, s, um: ops.fp8_linear_max(q, wp_up, s, s_up, bu, um, torch.bfloat16)
        quant_h = lambda u, um, nxt: ops.fp8_gelu_quant(u, um, clear_max=nxt)
        gemm_down = lambda q, s: ops.fp8_linear(q, wp_dn, s, s_dn, bd, False, None, 0.0, torch.bfloat16)
    else:
        quant_x = ops.fp8_quant_panels
        gemm_up = lambda q, s, um: ops.fp8_linear_panels(q, wp_up, s, s_up, bu, um, torch.bfloat16)
        quant_h = lambda u, um, nxt: ops.fp8_gelu_quant_panels(u, um, clear_max=nxt)
        gemm_down = lambda q, s: ops.fp8_linear_panels(q, wp_dn, s, s_dn, bd, None, torch.bfloat16)

    def step(i, record=None):
        """One pass of the chain; record = index into `names` of the one kernel to bracket with a pair of events."""
        xi = xs[i % n_rot]
        e = (ev(), ev()) if record is not None else None
        if record == 0:
            e[0].record()
        qx, sx = quant_x(xi)
        if record == 0:
            e[1].record()
        # the up projection's epilogue also leaves its largest output, from which the next pass derives max|gelu(u)|/448,
        # the dynamic scale of h: activation and quantisation are a single pass (the same numbers as GELU, an amax pass over
        # h and the cast)
        # zeroed by the previous step's activation pass (the two slots alternate from call to call), so no fill launch here
        um, um_next = s_h[calls[0] % 2], s_h[(calls[0] + 1) % 2]
        calls[0] += 1
        if record == 1:
            e[0].record()
        u = gemm_up(qx, sx, um)
        if record == 1:
            e[1].record()
        if record == 2:
            e[0].record()
        qh, sh = quant_h(u, um, um_next)
        if record == 2:
            e[1].record()
        if record == 3:
            e[0].record()
        y = gemm_down(qh, sh)
        if record == 3:
            e[1].record()
        if record is not None:
            marks[names[record]].append(e)
        return y

    # Set-up, before the W warm-up steps: bring the device out of idle.  From an idle start the power management needs about
    # 30 ms of load before it gives the compute units their sustained clock (the same GEMM takes 198 us on its first launches
    # and 163 us from the 150th on); a serving process is past that point after its first image, a 25-step benchmark that
    # starts cold would measure the ramp.  The chain is run until two consecutive groups of ten steps agree to 1.5 % (at
    # most 400 steps); what it took is reported as `settle_ms`.
    settle_t0 = time.perf_counter()
    prev, settled_after = None, 0
    for grp in range(40):
        a, b = ev(), ev()
        a.record()
        for i in range(10):
            step(i)
        b.record()
        torch.cuda.synchronize()
        cur = a.elapsed_time(b)
        settled_after = (grp + 1) * 10
        if prev is not None and abs(cur - prev) <= 0.015 * prev:
            break
        prev = cur
    settle_ms = (time.perf_counter() - settle_t0) * 1e3

    for i in range(args.warmup):
        y = step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    every = max(1, args.event_every)
    turn = (1, 0, 1, 2, 1, 3)  # which kernel a marked step brackets: the roofline kernel every other time
    for i in range(args.steps):
        y = step(i, record=turn[(i // every) % len(turn)] if i % every == 0 else None)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0

    ms_per_step = dt / args.steps * 1e3
    flops_step = 2.0 * M * (D * H + H * D)
    value = flops_step / (dt / args.steps) / 1e12
    per = {n: (sum(a.elapsed_time(b) for a, b in marks[n]) / len(marks[n]) * 1e3 if marks[n] else None) for n in names}  # us
    gemm_flops = 2.0 * M * D * H

    # ---- after the timed region: each kernel alone, launched back to back between ONE pair of events (no marker
    # between launches, so no launch gap inside the figure), on the same rotating inputs
    def batched(fn, n=20):
        # first at least 40 ms of this kernel's own load, and on until two groups of ten launches agree to 1.5 %: after
        # any pause the device needs some 30 ms of load before its power management settles, a figure taken during that
        # ramp is up to 20 % too slow, and two neighbouring groups can agree to 1.5 % half way up the ramp
        prev, busy_ms = None, 0.0
        for _ in range(120):
            a, b = ev(), ev()
            a.record()
            for i in range(10):
                fn(i)
            b.record()
            torch.cuda.synchronize()
            cur = a.elapsed_time(b)
            busy_ms += cur
            if busy_ms >= 40.0 and prev is not None and abs(cur - prev) <= 0.015 * prev:
                break
            prev = cur
        a, b = ev(), ev()
        a.record()
        for i in range(n):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n * 1e3

    qx0, sx0 = ops.fp8_quant(xs[0])  # row-major codes for the comparison kernels below
    um0 = torch.zeros(1, dtype=torch.float32, device=dev)
    qxc, sxc = quant_x(xs[0])
    u0 = gemm_up(qxc, sxc, um0)
    qh0, sh0 = quant_h(u0, um0, None)
    alone = {
        "quant_x": batched(lambda i: quant_x(xs[i % n_rot])),
        "gemm_up": batched(lambda i: gemm_up(qxc, sxc, um0)),
        "quant_h": batched(lambda i: quant_h(u0, um0, None)),
        "gemm_down": batched(lambda i: gemm_down(qh0, sh0)),
    }
    # ---- comparisons and diagnostics around the chain's kernels (skipped with --chain-only, so that a kernel trace of the run
    # holds the chain's GEMM kernels in the benchmarked configuration only: several of the launches below are the same
    # kernels on other operands -- zeros, row-major activations)
    rows_cmp = up_gelu_us = zeros_us = vendor = pipe_only = clocks = None
    if not args.chain_only:
        # the same two GEMMs on row-major activations (every line of the activation is then requested from L2 twice)
        if not args.row_major:
            qhr, shr = ops.fp8_gelu_quant(u0, um0)
            rows_cmp = {"gemm_up_us_back_to_back": round(batched(lambda i: ops.fp8_linear_max(qx0, wp_up, sx0, s_up, bu, um0, torch.bfloat16)), 2),
                        "gemm_down_us_back_to_back": round(batched(lambda i: ops.fp8_linear(qhr, wp_dn, shr, s_dn, bd, False, None, 0.0, torch.bfloat16)), 2)}
            del qhr
        # the up projection with the activation and the output maximum in its epilogue (not part of the timed chain)
        sg0 = torch.zeros(1, dtype=torch.float32, device=dev)
        up_gelu_us = batched(lambda i: ops.fp8_linear(qx0, wp_up, sx0, s_up, bu, True, None, 0.0, torch.bfloat16, out_scale=sg0))
        # the power argument, checkable from this line: the SAME up-projection kernel on all-zero operands (no switching in
        # the matrix pipe, so the clock is not pulled down), and the shader clock a probe on a second stream sees while the
        # kernel runs on random and on zero operands (idle clock for reference)
        zq, zw = torch.zeros_like(qxc), torch.zeros_like(wp_up)
        if args.row_major:
            gemm_up_on = lambda q, w: ops.fp8_linear_max(q, w, sx0, s_up, bu, um0, torch.bfloat16)
        else:
            gemm_up_on = lambda q, w: ops.fp8_linear_panels(q, w, sx0, s_up, bu, um0, torch.bfloat16)
        zeros_us = batched(lambda i: gemm_up_on(zq, zw))

        def clock_under(fn, per_launch_us=None, n=6):
            side = torch.cuda.Stream()
            torch.cuda.synchronize()
            for i in range(20):
                fn(i)  # the kernel under study is running, and has been for a while, before the probe starts
            with torch.cuda.stream(side):
                t = ops.shader_clock_probe(int(0.6 * n * (per_launch_us or alone["gemm_up"])), 8, side)
            for i in range(n):
                fn(i)
            torch.cuda.synchronize()
            t = t.cpu().double()
            return round(float((0.1 * t[:, 0] / t[:, 1]).median()), 3)

        vendor = None
        try:  # the vendor library's plain FP8 GEMM on the same operands (no bias, GELU or amax), for scale only
            a8, one = qx0.view(torch.float8_e4m3fn), torch.ones((), device=dev)
            w8 = ops.unpack_weight(wp_up).view(torch.float8_e4m3fn)
            vendor = {"up_4608x12288x3072": round(batched(lambda i: torch._scaled_mm(a8, w8.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)), 2)}
            del w8
            h8 = (qh0 if args.row_major else ops.fp8_panels_to_rows(qh0)).view(torch.float8_e4m3fn)
            wd8 = ops.unpack_weight(wp_dn).view(torch.float8_e4m3fn)
            vendor["down_4608x3072x12288"] = round(batched(lambda i: torch._scaled_mm(h8, wd8.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)), 2)
            del wd8
        except Exception:  # not every PyTorch build exposes it
            pass
        # what the matrix pipes alone sustain on this part: 16 x 1000 FP8 MFMAs per wavefront on register operands, no memory or
        # LDS traffic, one wavefront per SIMD (the layout of the down projection's kernel), on the chain's input codes and on zeros
        pipe_only = {}
        for name, codes in (("random_operands", qx0.view(-1)[: 1 << 22]), ("zero_operands", None)):
            flop = [0.0]

            def probe(i, codes=codes):
                flop[0] = ops.mfma_fp8_probe(codes, 1000)

            us = batched(probe)
            pipe_only[name] = {"us": round(us, 2), "TFLOP/s": round(flop[0] / us / 1e6, 1)}
        pipe_only["random_operands"]["shader_clock_ghz"] = clock_under(lambda i: ops.mfma_fp8_probe(qx0.view(-1)[: 1 << 22], 1000), pipe_only["random_operands"]["us"])
        pipe_only["zero_operands"]["shader_clock_ghz"] = clock_under(lambda i: ops.mfma_fp8_probe(None, 1000), pipe_only["zero_operands"]["us"])
        clocks = {
            "idle": clock_under(lambda i: None),
            "up_gemm_random_operands": clock_under(lambda i: gemm_up_on(qxc, wp_up)),
            "up_gemm_zero_operands": clock_under(lambda i: gemm_up_on(zq, zw)),
        }
        if vendor is not None:
            w8 = ops.unpack_weight(wp_up).view(torch.float8_e4m3fn)
            clocks["vendor_up_gemm_random_operands"] = clock_under(lambda i: torch._scaled_mm(a8, w8.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16))
            del w8
        del zq, zw

    # the other two GEMMs the metric names, at their FLUX 1024^2 shapes, timed like `alone` above (after the timed region):
    # W8A8 = INT8 up projection with per-token x per-channel dequant + bias, fp16 out; W4A4 = attention projection with
    # 16-bit group scales (BASELINE.json configs[3]), bf16 out.  Both are priced against the dense int8 MFMA peak (there
    # is no int4 matrix instruction; the W4A4 kernel widens nibbles to int8).
    other = other_metric_gemms(torch, ops, dev, batched)

    for n_ in names:  # a kernel that no marked step bracketed (very few --steps): its back-to-back time stands in
        if per[n_] is None:
            per[n_] = alone[n_]
    kernels = {
        "gemm_up_fp8_4608x12288x3072": {"us_in_step_incl_launch_gap": round(per["gemm_up"], 2), "us_back_to_back": round(alone["gemm_up"], 2),
                                        "TFLOP/s": round(gemm_flops / alone["gemm_up"] / 1e6, 1)},
        "gemm_down_fp8_4608x3072x12288": {"us_in_step_incl_launch_gap": round(per["gemm_down"], 2), "us_back_to_back": round(alone["gemm_down"], 2),
                                          "TFLOP/s": round(gemm_flops / alone["gemm_down"] / 1e6, 1)},
        "fp8_amax_cast_4608x3072": {"us_in_step_incl_launch_gap": round(per["quant_x"], 2), "us_back_to_back": round(alone["quant_x"], 2),
                                    "GB/s": round(3.0 * M * D / alone["quant_x"] / 1e3, 1)},
        "fp8_gelu_cast_with_gemm_max_4608x12288": {"us_in_step_incl_launch_gap": round(per["quant_h"], 2), "us_back_to_back": round(alone["quant_h"], 2),
                                                   "GB/s": round(3.0 * M * H / alone["quant_h"] / 1e3, 1)},
    }
    if up_gelu_us is not None:
        kernels["gemm_up_fp8_with_gelu_and_amax_epilogue_4608x12288x3072"] = {
            "us_back_to_back": round(up_gelu_us, 2), "TFLOP/s": round(gemm_flops / up_gelu_us / 1e6, 1),
            "note": "not in the timed chain: the activation in the GEMM's epilogue"}
    if rows_cmp is not None:
        kernels["same_gemms_on_row_major_activations"] = rows_cmp
    kernels.update(other)
    achieved = gemm_flops / per["gemm_up"] / 1e6
    traffic, traffic_src = profiled_traffic()
    roofline = {"bound": "mfma", "kernel": "lq::gemm_persist_kernel<fp8> 4608x12288x3072 (bias, running maximum, bf16 out)",
                "achieved": round(achieved, 1), "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / FP8_PEAK_TFLOPS, 4),
                "timing": f"a pair of HIP events around the kernel on {len(marks['gemm_up'])} of the {args.steps} timed steps, on the launch stream",
                # HBM-side bytes per launch of this kernel: not measured in this run -- taken from the committed rocprofv3
                # --pmc summary (FETCH_SIZE x2.0, the factor a plain copy of known size gives on this part, + WRITE_SIZE)
                "traffic": traffic, "traffic_unit": "bytes per launch (algorithmic: 1.65e8)", "traffic_source": traffic_src,
                "same_kernel_all_zero_operands": None if zeros_us is None else {
                    "us": round(zeros_us, 2), "TFLOP/s": round(gemm_flops / zeros_us / 1e6, 1),
                    "frac": round(gemm_flops / zeros_us / 1e6 / FP8_PEAK_TFLOPS, 4)},
                # the same instruction stream without any memory or LDS traffic (lq_mfma_fp8_probe): on real operands the part is
                # power limited below the published peak before a GEMM has moved a byte
                "matrix_pipes_alone": pipe_only,
                "shader_clock_ghz": clocks,
                "vendor_fp8_gemm_same_operands_us": vendor}  # plain GEMMs of the vendor library, no bias / GELU / amax
    # what the matrix pipes can deliver at the clock the device sustains under this kernel: CUs x 8192 FP8 FLOP per clock
    # (the published 5.0 PFLOP/s is 256 CUs at 2.4 GHz); `frac` above stays relative to the published peak
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    ghz = (clocks or {}).get("up_gemm_random_operands") if isinstance(clocks, dict) else None
    if ghz:
        at_clock = cus * 8192 * ghz / 1e3
        roofline["peak_at_sustained_clock"] = {"compute_units": cus, "TFLOP/s": round(at_clock, 1), "frac": round(achieved / at_clock, 4)}

    out = {
        "metric": "W8A8/FP8 GEMM TOPS at FLUX shapes (% MFMA peak); act-quant HBM GB/s",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3", "data": "synthetic",
        "config": {"workload": "FLUX DiT MLP FP8 e4m3 per-tensor, M=4608: act-quant -> GEMM 3072->12288 (+bias) "
                               "-> GELU + act-quant -> GEMM 12288->3072 (+bias), bf16 in/out (BASELINE.json configs[2])",
                   "quantised_activation_layout": "row-major [M, K]" if args.row_major else "k-panels [K/64, M, 64] written by the quantisers",
                   "tokens": M, "d_model": D, "d_ff": H, "profiled_tactics": tactics,
                   "settle_steps_before_warmup": settled_after, "settle_ms": round(settle_ms, 1)},
        "roofline": roofline, "kernels": kernels,
        "kernel_timing": f"us_in_step_incl_launch_gap: a pair of HIP events around one kernel on {sum(len(v) for v in marks.values())} of the "
                         f"{args.steps} timed steps ({', '.join(f'{n}: {len(v)}' for n, v in marks.items())}; the markers "
                         "themselves and the gap to the next launch are inside); us_back_to_back: 20 launches of the "
                         "kernel alone between one pair of events, after the timed region (rates are computed from these)",
    }
    if not args.no_cpu:
        cb, y_cpu = cpu_baseline(torch, x, w_up, w_dn, b_up, b_dn, args.cpu_rows)
        out["cpu_baseline"] = cb
        # sanity: the GPU chain on the same rows agrees with the CPU port (bf16 outputs; the two differ
        # by the GELU flavour of the fused epilogue and by bf16/e4m3 rounding flips, so a loose bound)
        xr = xd[: args.cpu_rows].contiguous()
        qx, sx = ops.fp8_quant(xr)
        ug = ops.fp8_linear(qx, wp_up, sx, s_up, bu, False, None, 0.0, torch.bfloat16)
        um = ug.float().max().clamp(min=0).reshape(1)
        qh, sh = ops.fp8_gelu_quant(ug, um)  # the scale is checked equal to an amax pass over gelu(u) in tests/
        y_gpu = ops.fp8_linear(qh, wp_dn, sh, s_dn, bd, False, None, 0.0, torch.bfloat16).float().cpu()
        out["cpu_gpu_max_abs_diff"] = round((y_gpu - y_cpu.float()).abs().max().item(), 4)
    if args.extra:
        out["extra"] = extra_kernels(torch, ops, dev)
    print(json.dumps(out))


def other_metric_gemms(torch, ops, dev, batched):
    """INT8 W8A8 GEMM 4608x12288x3072 and W4A4 GEMM 4608x3072x3072 (16-bit group scales), random codes, back to back."""
    g = torch.Generator().manual_seed(1003)
    out = {}
    m, n, k = M, H, D
    ops.gemm_profile("int8", m, n, k, dev)
    a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8).to(dev)
    w = ops.repack_weight(torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8).to(dev))
    ac = (torch.rand(n, generator=g) * 9e-3 + 1e-3).to(dev)
    ar = (torch.rand(m, generator=g) * 0.05).to(dev)
    b = (torch.randn(n, generator=g) * 0.02).half().to(dev)
    # the activation as k-panels [K/64, M, 64], the layout lq_sq_dynamic_quant_panels writes (random codes: any arrangement of
    # them is a valid activation); the row-major time beside it
    a_p = a.view(k // 64, m, 64)
    us = batched(lambda i: ops.int8_linear_panels(a_p, w, ac, ar, b, torch.float16))
    us_rows = batched(lambda i: ops.int8_linear(a, w, ac, ar, b, torch.float16))
    tops = 2.0 * m * n * k / us / 1e6
    out[f"gemm_int8_w8a8_{m}x{n}x{k}"] = {"us_back_to_back": round(us, 2), "TOP/s": round(tops, 1),
                                          "frac_of_int8_peak": round(tops / INT8_PEAK_TOPS, 4),
                                          "activation_layout": "k-panels [K/64, M, 64]",
                                          "us_back_to_back_row_major_activation": round(us_rows, 2)}
    del a, w
    m, n, k = M, D, D
    aw = torch.randint(-2 ** 31, 2 ** 31 - 1, (m, k // 8), generator=g, dtype=torch.int32).to(dev)
    ww = ops.repack_weight(torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.int32).to(torch.uint8).to(dev))
    sa = torch.rand(m, k // 64, generator=g).half().to(dev)
    sb = torch.rand(n, k // 64, generator=g).half().to(dev)
    us = batched(lambda i: ops.w4a4_linear(aw, ww, sa, sb, None, torch.bfloat16))
    tops = 2.0 * m * n * k / us / 1e6
    out[f"gemm_w4a4_f16scales_{m}x{n}x{k}"] = {"us_back_to_back": round(us, 2), "TOP/s": round(tops, 1),
                                               "frac_of_int8_peak": round(tops / INT8_PEAK_TOPS, 4)}
    return out


def extra_kernels(torch, ops, dev):
    """INT8 / W4A4 / SDXL-shape kernels (parity-test configurations), HIP-event timed, informative only."""
    res = {}

    def timeit(fn, iters=30, warm=5):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        # a kernel of 50 us and more is power limited: give it at least 40 ms of its own load and run it on until two
        # groups of ten launches agree to 1.5 % (the device needs about 30 ms of load to settle from idle)
        prev, busy_ms = None, 0.0
        for _ in range(120):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(10):
                fn()
            b.record()
            torch.cuda.synchronize()
            cur = a.elapsed_time(b)
            busy_ms += cur
            if cur < 0.5 or (busy_ms >= 40.0 and prev is not None and abs(cur - prev) <= 0.015 * prev):
                break
            prev = cur
        es = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        for a, b in es:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in es) / iters * 1e3

    def rotating(x, total_bytes=320 << 20, cap=24):
        """Copies of x totalling more than the 256 MB Infinity Cache, handed out in turn: the quantisation kernels are
        timed on inputs that no earlier launch left in a cache."""
        n = max(1, min(cap, -(-total_bytes // (x.numel() * x.element_size()))))
        xs = [x] + [x.clone() for _ in range(n - 1)]
        state = [0]

        def nxt():
            state[0] = (state[0] + 1) % n
            return xs[state[0]]

        return nxt

    g = torch.Generator().manual_seed(1001)
    for (m, n, k) in [(1024, 1280, 1280), (4096, 5120, 640), (4096, 640, 2560), (4608, 12288, 3072)]:
        a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8).to(dev)
        w = ops.repack_weight(torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8).to(dev))
        ac = (torch.rand(n, generator=g) * 9e-3 + 1e-3).to(dev)
        ar = (torch.rand(m, generator=g) * 0.05).to(dev)
        b = (torch.randn(n, generator=g) * 0.02).half().to(dev)
        us = timeit(lambda: ops.int8_linear(a, w, ac, ar, b, torch.float16))
        res[f"gemm_int8_{m}x{n}x{k}"] = {"us": round(us, 2), "TOP/s": round(2.0 * m * n * k / us / 1e6, 1)}
    m, n, k = 4608, 3072, 3072
    aw = torch.randint(-2 ** 31, 2 ** 31 - 1, (m, k // 8), generator=g, dtype=torch.int32).to(dev)
    ww = ops.repack_weight(torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.int32).to(torch.uint8).to(dev))
    sA = torch.rand(m, k // 64, generator=g).to(dev)
    sB = torch.rand(n, k // 64, generator=g).to(dev)
    us = timeit(lambda: ops.w4a4_linear(aw, ww, sA, sB, None, torch.bfloat16))
    res[f"gemm_w4a4_f32scales_{m}x{n}x{k}"] = {"us": round(us, 2), "TOP/s": round(2.0 * m * n * k / us / 1e6, 1)}
    sAh, sBh = sA.half(), sB.half()
    us = timeit(lambda: ops.w4a4_linear(aw, ww, sAh, sBh, None, torch.bfloat16))
    res[f"gemm_w4a4_f16scales_{m}x{n}x{k}"] = {"us": round(us, 2), "TOP/s": round(2.0 * m * n * k / us / 1e6, 1)}
    la = torch.randn(m, 32, generator=g).bfloat16().to(dev)
    lu = torch.randn(n, 32, generator=g).bfloat16().to(dev)
    us = timeit(lambda: ops.w4a4_linear(aw, ww, sAh, sBh, None, torch.bfloat16, 64, la, lu))
    res[f"gemm_w4a4_f16scales_lora32_{m}x{n}x{k}"] = {"us": round(us, 2), "TOP/s": round(2.0 * m * n * k / us / 1e6, 1)}
    x = torch.randn(m, k, generator=g).bfloat16().to(dev)
    dn = torch.randn(32, k, generator=g).bfloat16().to(dev)
    xr = rotating(x)
    us = timeit(lambda: ops.lora_down(xr(), dn))
    res[f"lora_down_rank32_{m}x{k}"] = {"us": round(us, 2), "GB/s": round(2.0 * m * k / us / 1e3, 1)}
    mod = torch.randn(1, k, generator=g).bfloat16().to(dev)
    one = torch.tensor([0.01], dtype=torch.float32, device=dev)
    us = timeit(lambda: ops.layernorm_mod_fp8(xr().view(1, m, k), mod, mod, one))
    res[f"layernorm_mod_fp8_{m}x{k}"] = {"us": round(us, 2), "GB/s": round(3.0 * m * k / us / 1e3, 1)}
    sm = (torch.rand(k, generator=g) + 0.5).to(dev)
    us = timeit(lambda: ops.w4a4_quant(xr(), sm))
    res[f"w4a4_quant_{m}x{k}"] = {"us": round(us, 2), "GB/s": round((2.5 * m * k + 4.0 * m * k / 64) / us / 1e3, 1)}
    us = timeit(lambda: ops.w4a4_quant_lora_down(xr(), sm, dn))  # both of the above from one read of x
    res[f"w4a4_quant_and_lora_down_rank32_{m}x{k}"] = {"us": round(us, 2), "GB/s": round((2.5 * m * k + 4.0 * m * k / 64 + 64.0 * m) / us / 1e3, 1)}
    y16 = torch.randn(m, 4 * k, generator=g).bfloat16().to(dev)
    ymx = y16.float().max().clamp(min=0).reshape(1)
    us = timeit(lambda: ops.fp8_gelu_quant(y16, ymx))
    res[f"fp8_gelu_cast_{m}x{4 * k}"] = {"us": round(us, 2), "GB/s": round(3.0 * m * 4 * k / us / 1e3, 1)}
    del y16
    for (m, k) in [(4608, 3072), (6912, 3072)]:
        # where the one-launch quantiser's time goes: device time stamps of every workgroup, medians over 20 launches (us from the
        # first workgroup's start)
        xr = rotating(torch.randn(m, k, generator=g).bfloat16().to(dev))
        rows = []
        for _ in range(25):
            q, s_, st = ops.fp8_quant_timeline(xr())
            t = (st - st[:, 0].min()).double().cpu() * 0.01
            rows.append([t[:, 0].max().item(), t[:, 1].max().item(), t[:, 2].max().item(), t[:, 3].max().item(),
                         (t[:, 1] - t[:, 0]).mean().item(), (t[:, 2] - t[:, 1]).mean().item(), (t[:, 3] - t[:, 2]).mean().item()])
        med = torch.tensor(rows[5:]).median(dim=0).values.tolist()
        res[f"fp8_amax_cast_timeline_{m}x{k}"] = dict(zip(
            ["last_workgroup_started_us", "last_loads_back_us", "last_released_from_exchange_us", "last_stores_acknowledged_us",
             "mean_load_phase_us", "mean_exchange_us", "mean_cast_and_store_us"], [round(v, 2) for v in med]))
    for (m, k) in [(4608, 3072), (4608, 12288)]:
        xr = rotating(torch.randn(m, k, generator=g).bfloat16().to(dev))
        us = timeit(lambda: ops.fp8_quant(xr()))
        res[f"fp8_amax_cast_{m}x{k}"] = {"us": round(us, 2), "GB/s": round(3.0 * m * k / us / 1e3, 1)}
        us = timeit(lambda: ops.fp8_quant_panels(xr()))
        res[f"fp8_amax_cast_panels_{m}x{k}"] = {"us": round(us, 2), "GB/s": round(3.0 * m * k / us / 1e3, 1)}
        us = timeit(lambda: ops.fp8_scale_cast(xr(), one))
        res[f"fp8_scale_cast_{m}x{k}"] = {"us": round(us, 2), "GB/s": round(3.0 * m * k / us / 1e3, 1)}
    for (m, k) in [(1024, 1280), (4096, 640), (4608, 3072), (4608, 12288)]:
        x = torch.randn(m, k, generator=g).half().to(dev)
        pre = (torch.rand(k, generator=g) + 0.5).to(dev)
        xr = rotating(x)
        us = timeit(lambda: ops.sq_quant_dynamic(xr(), pre))
        res[f"sq_dynamic_quant_{m}x{k}"] = {"us": round(us, 2), "GB/s": round((3.0 * m * k + 4 * m + 4 * k) / us / 1e3, 1)}
        if k >= 3072:  # the same quantiser writing k-panels [K/64, M, 64]
            us = timeit(lambda: ops.sq_quant_dynamic_panels(xr(), pre))
            res[f"sq_dynamic_quant_panels_{m}x{k}"] = {"us": round(us, 2), "GB/s": round((3.0 * m * k + 4 * m + 4 * k) / us / 1e3, 1)}
    for (m, k) in [(4096, 1280), (4096, 640), (4608, 3072)]:
        x = torch.randn(m, k, generator=g).half().to(dev)
        gb = torch.randn(k, generator=g).half().to(dev)
        xr = rotating(x)
        us = timeit(lambda: ops.layernorm_int8(xr(), gb, gb, None, None))
        res[f"layernorm_int8_dynamic_{m}x{k}"] = {"us": round(us, 2), "GB/s": round(3.0 * m * k / us / 1e3, 1)}
    m, d = 4096, 2560
    x = torch.randn(m, 2 * d, generator=g).half().to(dev)
    b = torch.randn(2 * d, generator=g).half().to(dev)
    pre = (torch.rand(d, generator=g) + 0.5).to(dev)
    xr = rotating(x)
    us = timeit(lambda: ops.geglu_int8_dynamic(xr(), b, pre))
    res[f"geglu_int8_{m}x{d}"] = {"us": round(us, 2), "GB/s": round(5.0 * m * d / us / 1e3, 1)}
    # weight-only GEMM (16-bit activations, int8 / int4 weights) at the FLUX up-projection shape
    m, n, k = 4608, 12288, 3072
    for dt, name in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
        x = torch.randn(m, k, generator=g).to(dt).to(dev)
        sc = (torch.rand(n, generator=g) * 0.01).to(dt).to(dev)
        for kind in ("int8", "int4"):
            q = torch.randint(-128, 128, (k, n if kind == "int8" else n // 2), generator=g, dtype=torch.int8).to(dev)
            wp = ops.repack_weight_only(q, kind)
            us = timeit(lambda: ops.weight_only_linear(x, wp, sc, None, kind), iters=20, warm=3)
            res[f"gemm_weight_only_{kind}_{name}_{m}x{n}x{k}"] = {"us": round(us, 2), "TFLOP/s": round(2.0 * m * n * k / us / 1e6, 1)}
            if kind == "int4":  # group-wise scales and zero points (group 128), dequantised per weight in the main loop
                gs = (torch.rand(k // 128, n, generator=g) * 0.01).to(dt).to(dev)
                gz = (torch.randn(k // 128, n, generator=g) * 0.01).to(dt).to(dev)
                us = timeit(lambda: ops.weight_only_linear_grouped(x, wp, gs, gz, None, kind, 128), iters=20, warm=3)
                res[f"gemm_weight_only_{kind}_g128_zeros_{name}_{m}x{n}x{k}"] = {"us": round(us, 2), "TFLOP/s": round(2.0 * m * n * k / us / 1e6, 1)}
    res.update(flux_block_times(torch, ops, dev, timeit))
    res.update(flux_linear_chain_1280(torch, ops, dev, timeit))
    res.update(flux_mlp_chain_graph(torch, ops, dev, timeit))
    res.update(sdxl_geglu_ffn_chain(torch, ops, dev, timeit))
    res.update(flux_whole_blocks(torch, dev, timeit))
    return res


def flux_whole_blocks(torch, dev, timeit):
    """Whole FLUX blocks at 1024x1024 (4096 image + 512 text tokens, d = 3072, 24 heads) through the block classes with the
    reference's interface, FP8 level: every linear, adaLN, gate and residual on this library's kernels, the attention core
    (q/k RMSNorm, rotary embedding, softmax attention) in PyTorch.  Random weights; informative only."""
    from lyradiff_amd import flux_ops as FO

    d, heads, dh, s, sc = 3072, 24, 128, 4096, 512
    g = torch.Generator().manual_seed(88)

    def state(prefix, names, norms):
        sd = {}
        for name, (n, k) in names.items():
            sd[f"{prefix}{name}.weight"] = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
            sd[f"{prefix}{name}.bias"] = (torch.randn(n, generator=g) * 0.02).bfloat16()
            sd[f"{prefix}{name}_input_scale"] = torch.tensor([6.0 / 448])
        for n in norms:
            sd[f"{prefix}attn.{n}.weight"] = torch.ones(dh).bfloat16()
        return sd

    dbl = {"norm1.linear": (6 * d, d), "norm1_context.linear": (6 * d, d), "attn.to_qkv": (3 * d, d), "attn.to_added_qkv": (3 * d, d),
           "attn.to_out.0": (d, d), "attn.to_add_out": (d, d), "ff.net.0.proj": (4 * d, d), "ff.net.2": (d, 4 * d),
           "ff_context.net.0.proj": (4 * d, d), "ff_context.net.2": (d, 4 * d)}
    sgl = {"norm.linear": (3 * d, d), "attn.to_qkv": (3 * d, d), "proj_mlp": (4 * d, d), "proj_out": (d, 5 * d)}
    x = torch.randn(1, s, d, generator=g).bfloat16().to(dev)
    ctx = torch.randn(1, sc, d, generator=g).bfloat16().to(dev)
    temb = torch.randn(1, d, generator=g).bfloat16().to(dev)
    ang = torch.rand(1, sc + s, dh // 2, generator=g) * 6.28
    rope = torch.stack([ang.cos(), -ang.sin(), ang.sin(), ang.cos()], dim=-1).reshape(1, sc + s, dh // 2, 2, 2).bfloat16().to(dev)
    res = {}
    from lyradiff_amd import ops as _ops
    qkv = torch.randn(1, s, 3 * d, generator=g).bfloat16().to(dev)
    cqkv = torch.randn(1, sc, 3 * d, generator=g).bfloat16().to(dev)
    nqk = torch.ones(2 * dh).bfloat16().to(dev)
    us = timeit(lambda: _ops.rmsnorm_rope(qkv, nqk, rope, heads, cqkv, nqk))
    res["rmsnorm_rope_cat_4608x72x128"] = {"us": round(us, 2), "GB/s": round(2 * 2.0 * (s + sc) * 3 * d / us / 1e3, 1)}
    op = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 6, FO.LyraQuantLevel.FP8_W8A8.value)
    op.reload_model_from_state_dict("b.", state("b.", dbl, ("norm_q", "norm_k", "norm_added_q", "norm_added_k")), "cpu")
    us = timeit(lambda: op.forward(x, ctx, rope, temb), iters=10, warm=3)
    lin = 2.0 * d * d * ((s + sc) * (3 + 1 + 8))
    res["flux_double_block_fp8_whole_1024"] = {"us": round(us, 1), "linear_TFLOP/s": round(lin / us / 1e6, 1)}
    del op
    sop = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, FO.LyraQuantLevel.FP8_W8A8.value)
    sop.reload_model_from_state_dict("b.", state("b.", sgl, ("norm_q", "norm_k")), "cpu")
    xs = torch.cat([ctx, x], dim=1).contiguous()
    us = timeit(lambda: sop.forward(xs, rope, temb), iters=10, warm=3)
    lin = 2.0 * d * d * (s + sc) * (3 + 4 + 5)
    res["flux_single_block_fp8_whole_1024"] = {"us": round(us, 1), "linear_TFLOP/s": round(lin / us / 1e6, 1)}
    del sop

    # The same blocks at level INT4_W4A4_FULL: W4A4 linears with their rank-32 low-rank branch (random codes and scales in
    # the reference's container layout), FP8 adaLN and ff.net.2 linears.
    def w4(prefix, n, k, bias=True):
        sd = {prefix + "packed_weight": torch.randint(-128, 128, (n, k // 2), generator=g, dtype=torch.int8),
              prefix + "weight_scale": torch.rand(n, k // 64, generator=g) * 4e-3 + 1e-3,
              prefix + "smooth": torch.rand(k, generator=g) + 0.5,
              prefix + "lora_up": (0.05 * torch.randn(n, 32, generator=g)).bfloat16(),
              prefix + "lora_down": (0.05 * torch.randn(32, k, generator=g)).bfloat16()}
        if bias:
            sd[prefix + "bias"] = (0.02 * torch.randn(n, generator=g)).bfloat16()
        return sd

    level = FO.LyraQuantLevel.INT4_W4A4_FULL.value
    sd = state("b.", {k: v for k, v in dbl.items() if k.startswith("norm1") or k.endswith("net.2")},
               ("norm_q", "norm_k", "norm_added_q", "norm_added_k"))
    for name, n in (("attn.to_qkv.", 3 * d), ("attn.to_added_qkv.", 3 * d), ("attn.to_out.0.", d), ("attn.to_add_out.", d),
                    ("ff.net.0.proj.", 4 * d), ("ff_context.net.0.proj.", 4 * d)):
        sd.update(w4("b." + name, n, d))
    op = FO.FluxTransformerBlockOp("bf16", d, heads, dh, 6, level)
    op.reload_model_from_state_dict("b.", sd, "cpu")
    us = timeit(lambda: op.forward(x, ctx, rope, temb), iters=10, warm=3)
    lin = 2.0 * d * d * ((s + sc) * (3 + 1 + 8))
    res["flux_double_block_int4_whole_1024"] = {"us": round(us, 1), "linear_TOP/s": round(lin / us / 1e6, 1)}
    del op, sd
    sd = state("b.", {"norm.linear": (3 * d, d)}, ("norm_q", "norm_k"))
    sd.update(w4("b.attn.to_qkv.", 3 * d, d))
    sd.update(w4("b.proj_mlp.", 4 * d, d))
    sd.update(w4("b.proj_out.linears.0.", d, d))
    sd.update(w4("b.proj_out.linears.1.linear.", d, 4 * d, bias=False))
    sop = FO.FluxSingleTransformerBlockOp("bf16", d, heads, dh, 4, level)
    sop.reload_model_from_state_dict("b.", sd, "cpu")
    us = timeit(lambda: sop.forward(xs, rope, temb), iters=10, warm=3)
    lin = 2.0 * d * d * (s + sc) * (3 + 4 + 5)
    res["flux_single_block_int4_whole_1024"] = {"us": round(us, 1), "linear_TOP/s": round(lin / us / 1e6, 1)}
    return res


def sdxl_geglu_ffn_chain(torch, ops, dev, timeit):
    """BASELINE.json configs[1]: the SDXL GEGLU feed-forward with INT8 W8A8 linears at 1024x1024 (M = 4096 tokens of the
    64x64 latent stage): per-token quantisation, up GEMM 640 -> 5120, bias + GEGLU -> per-token INT8, down GEMM 2560 -> 640."""
    m, d = 4096, 640
    g = torch.Generator().manual_seed(1002)
    x = torch.randn(m, d, generator=g).half()
    x[:, torch.randperm(d, generator=g)[:6]] *= 15.0
    x = x.to(dev)
    w_up = ops.repack_weight(torch.randint(-127, 128, (8 * d, d), generator=g, dtype=torch.int8).to(dev))
    w_dn = ops.repack_weight(torch.randint(-127, 128, (d, 4 * d), generator=g, dtype=torch.int8).to(dev))
    s_up = (torch.rand(8 * d, generator=g) * 9e-3 + 1e-3).to(dev)
    s_dn = (torch.rand(d, generator=g) * 9e-3 + 1e-3).to(dev)
    b_up = (torch.randn(8 * d, generator=g) * 0.02).half().to(dev)
    b_dn = (torch.randn(d, generator=g) * 0.02).half().to(dev)
    pre1 = (torch.rand(d, generator=g) + 0.5).to(dev)
    pre2 = (torch.rand(4 * d, generator=g) + 0.5).to(dev)
    for (n, k) in ((8 * d, d), (d, 4 * d)):
        ops.gemm_profile("int8", m, n, k, dev)

    def chain():
        q, s = ops.sq_quant_dynamic(x, pre1)
        up = ops.int8_linear(q, w_up, s_up, s, None, torch.float16)
        q2, s2 = ops.geglu_int8_dynamic(up, b_up, pre2)
        return ops.int8_linear(q2, w_dn, s_dn, s2, b_dn, torch.float16)

    us = timeit(chain, iters=30, warm=5)
    ops_total = 2.0 * m * (8 * d * d + d * 4 * d)
    res = {"sdxl_geglu_ffn_int8_chain_4096": {"us": round(us, 2), "TOP/s": round(ops_total / us / 1e6, 1)}}
    # The same five launches replayed from a HIP graph: the eager figure above is bounded by the host's per-launch cost
    # (the kernels take 3-10 us each), the replay shows what the kernels themselves need.
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        chain()
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        y_static = chain()
    torch.cuda.synchronize()
    us_g = timeit(graph.replay, iters=50, warm=5)
    if not torch.equal(y_static, chain()):
        raise RuntimeError("graph replay of the SDXL INT8 chain differs from the eager result")
    res["sdxl_geglu_ffn_int8_chain_4096_graph_replay"] = {"us": round(us_g, 2), "TOP/s": round(ops_total / us_g / 1e6, 1)}
    return res


def flux_mlp_chain_graph(torch, ops, dev, timeit):
    """The headline chain (BASELINE.json configs[2]) replayed from a HIP graph, next to the same chain launched eagerly: what the
    four launch gaps of a step cost.  Under capture the input quantiser takes its exchange-free three-kernel route."""
    m, d, h = 4608, 3072, 12288
    g = torch.Generator().manual_seed(1003)
    x = torch.randn(m, d, generator=g).bfloat16().to(dev)
    wu, su = ops.fp8_quant((torch.randn(h, d, generator=g) * 0.02).bfloat16().to(dev))
    wd, sd = ops.fp8_quant((torch.randn(d, h, generator=g) * 0.02).bfloat16().to(dev))
    wu, wd = ops.repack_weight(wu), ops.repack_weight(wd)
    bu = (torch.randn(h, generator=g) * 0.1).bfloat16().to(dev)
    bd = (torch.randn(d, generator=g) * 0.1).bfloat16().to(dev)
    um = torch.zeros(1, dtype=torch.float32, device=dev)

    def chain():  # quantised activations as k-panels, as in the headline step
        qx, sx = ops.fp8_quant_panels(x)
        um.zero_()
        u = ops.fp8_linear_panels(qx, wu, sx, su, bu, um, torch.bfloat16)
        qh, sh = ops.fp8_gelu_quant_panels(u, um)
        return ops.fp8_linear_panels(qh, wd, sh, sd, bd, None, torch.bfloat16)

    us = timeit(chain, iters=30, warm=20)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        chain()
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        y_static = chain()
    torch.cuda.synchronize()
    for _ in range(3):  # every replay against the eager result, with eager work and synchronisations between the replays
        ref = chain()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        if not torch.equal(y_static, ref):
            raise RuntimeError("graph replay of the FLUX MLP chain differs from the eager result")
    us_g = timeit(graph.replay, iters=30, warm=20)
    flop = 2.0 * m * (d * h + h * d)
    return {"flux_mlp_fp8_chain_eager_same_input": {"us": round(us, 2), "TFLOP/s": round(flop / us / 1e6, 1)},
            "flux_mlp_fp8_chain_graph_replay": {"us": round(us_g, 2), "TFLOP/s": round(flop / us_g / 1e6, 1)}}


def flux_linear_chain_1280(torch, ops, dev, timeit):
    """BASELINE.json configs[4]: the FP8 linears of a FLUX double-stream block at 1280x1280 (M = 6912 tokens), each preceded
    by the fused amax + cast of its bf16 input: QKV 3072->9216, out-proj 3072->3072, MLP 3072->12288 (GELU) ->3072.  The
    four linears run on independent synthetic inputs of the right shapes (the attention between them is not part of the
    path); the MLP pair is chained through the up projection's largest output as in the headline step."""
    m, d = 6912, 3072
    g = torch.Generator().manual_seed(1005)
    lin = {}
    for name, n, k in (("qkv", 3 * d, d), ("out", d, d), ("up", 4 * d, d), ("down", d, 4 * d)):
        wq, sw = ops.fp8_quant((torch.randn(n, k, generator=g) * 0.02).bfloat16().to(dev))
        lin[name] = (ops.repack_weight(wq), sw, (torch.randn(n, generator=g) * 0.02).bfloat16().to(dev))
        ops.gemm_profile("fp8", m, n, k, dev)
    xs = [torch.randn(m, d, generator=g).bfloat16().to(dev) for _ in range(3)]
    sh = torch.zeros(1, dtype=torch.float32, device=dev)

    def chain():
        for name, x in (("qkv", xs[0]), ("out", xs[1])):
            q, s = ops.fp8_quant_panels(x)
            ops.fp8_linear_panels(q, lin[name][0], s, lin[name][1], lin[name][2])
        q, s = ops.fp8_quant_panels(xs[2])
        sh.zero_()
        u = ops.fp8_linear_panels(q, lin["up"][0], s, lin["up"][1], lin["up"][2], sh, torch.bfloat16)
        qh, s2 = ops.fp8_gelu_quant_panels(u, sh)
        return ops.fp8_linear_panels(qh, lin["down"][0], s2, lin["down"][1], lin["down"][2])

    us = timeit(chain, iters=20, warm=3)
    flop = 2.0 * m * d * (3 * d + d + 4 * d + 4 * d)
    return {"flux_double_block_fp8_linear_chain_6912": {"us": round(us, 2), "TFLOP/s": round(flop / us / 1e6, 1)}}


def flux_block_times(torch, ops, dev, timeit):
    """FP8 feed-forward halves of the FLUX blocks at 1024x1024 (4608 tokens, d=3072): the fused three-launch forms
    against the reference's launch sequence run step by step with this library's unfused kernels (torch for the two
    elementwise gate/residual steps), same operands, bit-identical outputs."""
    from lyradiff_amd import flux_fp8 as F

    g = torch.Generator().manual_seed(77)
    b, s, d = 1, 4608, 3072
    bf = lambda *shape, sc=1.0: (sc * torch.randn(*shape, generator=g)).bfloat16()
    sd = {"p.net.0.proj.weight": bf(4 * d, d, sc=0.02), "p.net.0.proj.bias": bf(4 * d, sc=0.1),
          "p.net.2.weight": bf(d, 4 * d, sc=0.02), "p.net.2.bias": bf(d, sc=0.1),
          "p.net.0.proj_input_scale": torch.tensor([5.0 / 448]), "p.net.2_input_scale": torch.tensor([2.0 / 448]),
          "p.proj_mlp.weight": bf(4 * d, d, sc=0.02), "p.proj_mlp.bias": bf(4 * d, sc=0.1),
          "p.proj_out.weight": bf(d, 5 * d, sc=0.02), "p.proj_out.bias": bf(d, sc=0.1),
          "p.proj_mlp_input_scale": torch.tensor([5.0 / 448]), "p.proj_out_input_scale": torch.tensor([4.0 / 448])}
    wp = F.load_flux_attn_post_fp8(sd, "p.", d, torch.bfloat16, dev)
    ws = F.load_flux_single_mlp_fp8(sd, "p.", d, 4, torch.bfloat16, dev)
    x, attn, norm = bf(b, s, d).to(dev), bf(b, s, d).to(dev), bf(b, s, d).to(dev)
    msa = bf(6, b, d, sc=0.5).to(dev)
    for kind, (n, k) in (("fp8", (4 * d, d)), ("fp8", (d, 4 * d)), ("fp8", (d, 5 * d))):
        ops.gemm_profile(kind, b * s, n, k, dev)

    def post_unfused():
        hidden = x + msa[2][:, None, :] * attn
        q1 = ops.layernorm_mod_fp8(hidden, msa[4], msa[3], wp.gelu_proj.input_scale)
        inner = ops.fp8_linear(q1.view(b * s, d), wp.gelu_proj.weight_rows32, wp.gelu_proj.input_scale, wp.gelu_proj.weight_scale,
                               wp.gelu_proj.bias, True, None, 0.0, torch.bfloat16)
        q2 = ops.fp8_scale_cast(inner, wp.ff_linear.input_scale)
        ff = ops.fp8_linear(q2, wp.ff_linear.weight_rows32, wp.ff_linear.input_scale, wp.ff_linear.weight_scale, wp.ff_linear.bias,
                            False, None, 0.0, torch.bfloat16)
        return hidden + msa[5][:, None, :] * ff.view(b, s, d)

    def single_unfused():
        q1 = ops.fp8_scale_cast(norm, ws.proj_mlp.input_scale)
        mlp = ops.fp8_linear(q1.view(b * s, d), ws.proj_mlp.weight_rows32, ws.proj_mlp.input_scale, ws.proj_mlp.weight_scale,
                             ws.proj_mlp.bias, False, None, 0.0, torch.bfloat16)
        cat = torch.cat([attn.view(b * s, d), torch.nn.functional.gelu(mlp.float(), approximate="tanh").bfloat16()], dim=1)
        q2 = ops.fp8_scale_cast(cat, ws.proj_out.input_scale)
        o = ops.fp8_linear(q2, ws.proj_out.weight_rows32, ws.proj_out.input_scale, ws.proj_out.weight_scale, ws.proj_out.bias,
                           False, None, 0.0, torch.bfloat16)
        return x + msa[2][:, None, :] * o.view(b, s, d)

    same = bool(torch.equal(F.flux_attn_post_fp8(x, attn, msa, wp), post_unfused()))
    flops_post, flops_single = 2.0 * b * s * 8 * d * d, 2.0 * b * s * 9 * d * d
    out = {}
    for name, fn, fl in (("flux_attn_post_fp8_fused_3_launches", lambda: F.flux_attn_post_fp8(x, attn, msa, wp), flops_post),
                         ("flux_attn_post_fp8_reference_sequence_7_launches", post_unfused, flops_post),
                         ("flux_single_mlp_fp8_fused_3_launches", lambda: F.flux_single_mlp_fp8(x, norm, attn, msa[2], ws), flops_single),
                         ("flux_single_mlp_fp8_reference_sequence_7_launches", single_unfused, flops_single)):
        us = timeit(fn, iters=20, warm=3)
        out[name] = {"us": round(us, 2), "TFLOP/s": round(fl / us / 1e6, 1)}
    out["flux_attn_post_fp8_fused_equals_sequence"] = same
    return out


if __name__ == "__main__":
    main()
