#!/usr/bin/env python3
"""Benchmark of the tensorized conv2d / GEMM path on one MI355X.

A step is one pass over the 53 convolutions of ResNet-50 v1 at batch 32 (20 unique layer shapes x
their multiplicity), int8 u8 x s8 -> i32 in NCHW16c / NCHW4c, through the C ABI with operands and
outputs already resident in HBM.  `value` is the whole-step throughput in TOP/s (2 x logical MACs /
time).  The same line also carries the 4096^3 int8 and fp16 GEMMs, a per-layer table, the roofline
of the layer that takes the largest share of the step, and the CPU baseline (the VNNI oracle on
the host cores, same tensors, also used to check every GPU layer output bit for bit).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5033.0   # MI355X dense int8 MFMA, published
PEAK_F16_TFLOPS = 2516.0  # MI355X dense fp16 MFMA, published
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, published
BATCH = 32
# HBM bytes per launch (read + written) from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of
# `bench.py --profile <layer>`, scaled by the plain-copy calibration; the summaries are
# profiles/conv_i8_resnet50_b32_<layer>.txt and profiles/hbm_copy_calibration_128MiB.txt
MEASURED_HBM_BYTES = {
    "3x3_256_256@14": 13072331,   # algorithmic 8617984
    "1x1_64_256@56": 115840483,   # algorithmic 109199360 (two 64-channel tiles per panel: the input is read twice)
    "3x3_512_512@7": 14772236,    # algorithmic 6373376
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / bit-exactness leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only (no HIP graph replay)")
    ap.add_argument("--weights", default="prepared", choices=["prepared", "reference"],
                    help="headline convolutions on weights prepared once with unit_conv2d_prepare_weight (default), "
                         "or on the reference's blocked layout in every call")
    ap.add_argument("--profile", default=None, metavar="WHAT",
                    help="launch one kernel 20 times and exit (for rocprofv3): a ResNet-50 layer name such as "
                         "3x3_256_256@14, or gemm_i8 / gemm_f16 / gemm_f16_prepared / copy")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus must be 1 "
              "(nothing here shards across devices)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import unit_amd as U
    from unit_amd import _lib, rng
    from unit_amd import workloads as WL

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    L = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream

    def dev_t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def time_us(fn, iters, warm=3, bursts=1, median=False):
        """Mean launch-to-launch time of `iters` back-to-back launches; with bursts > 1 the fastest burst (the
        clocks of this part follow the load of whatever ran just before), or the median one."""
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        seen = []
        for _ in range(bursts):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(iters):
                fn()
            e.record()
            torch.cuda.synchronize()
            seen.append(s.elapsed_time(e) * 1e3 / iters)
        return sorted(seen)[len(seen) // 2] if median else min(seen)

    if args.profile in ("gemm_i8", "gemm_f16", "gemm_f16_prepared", "copy"):
        n = 4096
        if args.profile == "gemm_i8":
            a = dev_t(rng.uniform_u8((n, n), 11))
            w = dev_t(rng.uniform_s8((n, n), 12))
            fn = lambda: U.dense(a, w)
        elif args.profile == "gemm_f16":
            a = dev_t(rng.normal_f16((n, n), 13, 1.0 / 64))
            b = dev_t(rng.normal_f16((n, n), 14))
            fn = lambda: U.gemm_fp16(a, b)
        elif args.profile == "gemm_f16_prepared":
            a = dev_t(rng.normal_f16((n, n), 13, 1.0 / 64))
            pb = U.prepare_gemm_b(dev_t(rng.normal_f16((n, n), 14)))
            fn = lambda: U.gemm_fp16(a, pb)
        else:  # plain 128 MiB device-to-device copy: the calibration point for FETCH_SIZE / WRITE_SIZE
            a = torch.empty(128 * 1024 * 1024, dtype=torch.uint8, device=dev)
            b = torch.empty_like(a)
            fn = lambda: b.copy_(a)
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        print(json.dumps({"profiled": args.profile, "launches": 20}))
        return

    # ------------------------------------------------------------------ ResNet-50 b32 int8 conv stack
    layers = []
    for idx, s in enumerate(WL.RESNET50):
        if args.profile and s.name != args.profile:
            continue
        cb = WL.channel_block(s.C)
        cp = -(-s.C // cb) * cb
        data_np = rng.uniform_u8((BATCH, cp // cb, s.H, s.W, cb), 1000 + idx)
        if cp != s.C:  # padded input channels hold zeros
            data_np[..., s.C % cb:] = 0
        w_oihw = rng.uniform_s8((s.K, s.C, s.KH, s.KW), 2000 + idx)
        data = dev_t(data_np)
        wt = U.prepack_conv_weight(dev_t(w_oihw), cb)
        oh, ow = WL.out_hw(s)
        out = torch.empty((BATCH, s.K // 16, oh, ow, 16), dtype=torch.int32, device=dev)
        desc = _lib.ConvDesc(BATCH, cp, s.H, s.W, s.K, s.KH, s.KW, s.stride, s.stride, s.pad, s.pad, s.pad,
                             s.pad, 1, 1, cb)
        call_ref = (lambda d=desc, x=data, w=wt, o=out: _lib.check(
            L.unit_conv2d_nchwc_u8s8s32(ctypes.byref(d), x.data_ptr(), w.data_ptr(), o.data_ptr(),
                                        torch.cuda.current_stream().cuda_stream)))
        call, prep = call_ref, None
        if args.weights == "prepared" and (cb == 16 or s.KW <= 8):
            # the constant weight is re-ordered once, before the timed region, as the reference's compiled
            # graphs fold the weight layout chain and sum(w) (apps/cpu/relay/result.log:8-16)
            prep = U.prepare_conv2d_weight(wt)
            call = (lambda d=desc, x=data, w=prep.buf, o=out: _lib.check(
                L.unit_conv2d_nchwc_u8s8s32_prepared(ctypes.byref(d), x.data_ptr(), w.data_ptr(), o.data_ptr(),
                                                     torch.cuda.current_stream().cuda_stream)))
        call()
        layers.append(dict(shape=s, cb=cb, data=data, data_np=data_np, wt=wt, prep=prep, out=out, call=call,
                           call_ref=call_ref, variant=U.last_variant(), ops=2 * WL.macs(s, BATCH),
                           bytes=WL.algorithmic_bytes(s, BATCH)))
    torch.cuda.synchronize()
    if args.profile:
        if not layers:
            print(f"bench.py: unknown --profile target {args.profile!r}", file=sys.stderr)
            sys.exit(2)
        for _ in range(19):
            layers[0]["call"]()
        torch.cuda.synchronize()
        print(json.dumps({"profiled": args.profile, "launches": 20, "kernel": layers[0]["variant"]}))
        return

    def step():
        for ly in layers:
            for _ in range(ly["shape"].count):
                ly["call"]()

    def step_ref():  # the same stack on the reference's weight layout
        for ly in layers:
            for _ in range(ly["shape"].count):
                ly["call_ref"]()

    def timed(run):
        for _ in range(args.warmup):
            run()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record()
        for _ in range(args.steps):
            run()
        ev1.record()
        torch.cuda.synchronize()
        return ev0.elapsed_time(ev1) / args.steps, (time.perf_counter() - t0) * 1e3 / args.steps

    # eager: 53 C-ABI calls per step; graph: the same 53 launches captured once in a HIP graph
    # and replayed (the library enqueues plain kernels only, so a step is capturable as is)
    eager_ms, eager_wall_ms = timed(step)
    launch_mode = "eager"
    ms_per_step, wall_ms = eager_ms, eager_wall_ms
    graph_ms = None
    if not args.no_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            graph_ms, graph_wall_ms = timed(graph.replay)
            # replays must reproduce the eager outputs bit for bit
            keep = [ly["out"].clone() for ly in layers]
            for ly in layers:
                ly["out"].fill_(-1)
            graph.replay()
            torch.cuda.synchronize()
            same = all(torch.equal(k, ly["out"]) for k, ly in zip(keep, layers))
            if same and graph_ms < eager_ms:
                launch_mode, ms_per_step, wall_ms = "hipgraph", graph_ms, graph_wall_ms
            elif not same:
                print("bench.py: graph replay differs from eager launches; reporting eager", file=sys.stderr)
        except Exception as ex:  # graph capture unavailable: the eager figure stands
            print(f"bench.py: HIP graph capture failed ({ex}); reporting eager", file=sys.stderr)
    step_ops = sum(ly["ops"] * ly["shape"].count for ly in layers)
    value = step_ops / (ms_per_step * 1e-3) / 1e12
    ref_weights = None
    if args.weights == "prepared":
        ref_ms = timed(step_ref)[0]
        if not args.no_graph:
            try:
                graph_ref = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph_ref):
                    step_ref()
                ref_ms = min(ref_ms, timed(graph_ref.replay)[0])
            except Exception as ex:
                print(f"bench.py: HIP graph capture failed ({ex})", file=sys.stderr)
        ref_weights = dict(workload="the same step with every convolution on the reference's blocked weight layout",
                           ms_per_step=round(ref_ms, 4), tops=round(step_ops / (ref_ms * 1e-3) / 1e12, 2))

    # per-layer launch duration (HIP events on the launch stream, back-to-back launches; the median of three bursts of
    # 30 launches: a single burst now and then lands 20 % high on the write-bound layers)
    ridge = PEAK_INT8_TOPS * 1e12 / (PEAK_HBM_GBS * 1e9)
    table = []
    for ly in layers:
        us = time_us(ly["call"], 30, bursts=3, median=True)
        ai = ly["ops"] / ly["bytes"]
        bound = "mfma" if ai >= ridge else "hbm"
        tops, gbs = ly["ops"] / us / 1e6, ly["bytes"] / us / 1e3
        frac = tops / PEAK_INT8_TOPS if bound == "mfma" else gbs / PEAK_HBM_GBS
        ly["us"] = us
        table.append(dict(layer=ly["shape"].name, count=ly["shape"].count, us=round(us, 2), tops=round(tops, 1),
                          pct_int8_peak=round(100 * tops / PEAK_INT8_TOPS, 2), gbs=round(gbs, 1), bound=bound,
                          frac=round(frac, 4), kernel=ly["variant"]))
    dom = max(layers, key=lambda ly: ly["us"] * ly["shape"].count)
    dom_row = table[layers.index(dom)]
    if dom_row["bound"] == "mfma":
        roofline = dict(bound="mfma", achieved=dom_row["tops"], peak=PEAK_INT8_TOPS, unit="TFLOP/s")
    else:
        roofline = dict(bound="hbm", achieved=dom_row["gbs"], peak=PEAK_HBM_GBS, unit="GB/s")
    roofline.update(frac=dom_row["frac"], traffic=None, kernel=dom_row["kernel"], layer=dom_row["layer"],
                    launch_us=dom_row["us"])

    # ------------------------------------------------------------------ 4096^3 GEMMs
    M = N = K = 4096
    a8 = dev_t(rng.uniform_u8((M, K), 11))
    w8_np = rng.uniform_s8((N, K), 12)
    w8 = dev_t(w8_np)
    wp8 = U.prepack_dense_weight(w8)
    c8 = torch.empty((M, N), dtype=torch.int32, device=dev)
    g_rm = lambda: _lib.check(L.unit_dense_u8s8s32(a8.data_ptr(), w8.data_ptr(), c8.data_ptr(), M, N, K, stream))
    g_pk = lambda: _lib.check(L.unit_dense_dotprod_u8s8s32(a8.data_ptr(), wp8.data_ptr(), c8.data_ptr(), M, N, K,
                                                            stream))
    us_rm = time_us(g_rm, 30, bursts=3)
    v_rm = U.last_variant()
    us_pk = time_us(g_pk, 30, bursts=3)
    v_pk = U.last_variant()
    gemm_ops = 2.0 * M * N * K
    gemm_i8 = dict(workload="int8 GEMM 4096^3 u8 x s8 -> i32", timing="fastest of 3 bursts of 30 launches",
                   row_major=dict(us=round(us_rm, 2), tops=round(gemm_ops / us_rm / 1e6, 1),
                                  pct_int8_peak=round(100 * gemm_ops / us_rm / 1e6 / PEAK_INT8_TOPS, 2), kernel=v_rm),
                   vnni_packed=dict(us=round(us_pk, 2), tops=round(gemm_ops / us_pk / 1e6, 1),
                                    pct_int8_peak=round(100 * gemm_ops / us_pk / 1e6 / PEAK_INT8_TOPS, 2),
                                    kernel=v_pk))
    ah_np = rng.normal_f16((M, K), 13, 1.0 / np.sqrt(K))
    bh_np = rng.normal_f16((K, N), 14)
    ah, bh = dev_t(ah_np), dev_t(bh_np)
    cf = torch.empty((M, N), dtype=torch.float32, device=dev)
    g_f = lambda: _lib.check(L.unit_gemm_f16(ah.data_ptr(), bh.data_ptr(), cf.data_ptr(), M, N, K, 0, stream))
    us_f = time_us(g_f, 30, bursts=3)
    v_f = U.last_variant()
    # the same product with b re-laid once as (N, K) before the timed region (a constant operand, as the
    # reference pre-packs b in apps/gpu/gemm-pack.py)
    pb = U.prepare_gemm_b(bh)
    g_fp = lambda: _lib.check(L.unit_gemm_f16_prepared(ah.data_ptr(), pb.bt.data_ptr(), cf.data_ptr(), M, N, K, 0, stream))
    us_fp = time_us(g_fp, 30, bursts=3)
    v_fp = U.last_variant()
    g_f()
    v_f = U.last_variant()
    # fp16 check on a 256 x 256 corner against float64
    ref = ah_np[:256].astype(np.float64) @ bh_np[:, :256].astype(np.float64)
    got = cf[:256, :256].cpu().numpy().astype(np.float64)
    f16_err = float((np.abs(got - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max())).max())
    gemm_f16 = dict(workload="fp16 GEMM 4096^3, fp32 accumulate, fp32 out", timing="fastest of 3 bursts of 30 launches",
                    us=round(us_f, 2),
                    tflops=round(gemm_ops / us_f / 1e6, 1),
                    pct_f16_peak=round(100 * gemm_ops / us_f / 1e6 / PEAK_F16_TFLOPS, 2), kernel=v_f,
                    max_rel_err=f16_err, tolerance=1e-2)
    g_fp()
    torch.cuda.synchronize()
    got = cf[:256, :256].cpu().numpy().astype(np.float64)
    gemm_f16["prepared_b"] = dict(us=round(us_fp, 2), tflops=round(gemm_ops / us_fp / 1e6, 1),
                                  pct_f16_peak=round(100 * gemm_ops / us_fp / 1e6 / PEAK_F16_TFLOPS, 2), kernel=v_fp,
                                  max_rel_err=float((np.abs(got - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max())).max()))

    # the reference's own GEMM sizes (its drivers' constants): few output tiles, so the reduction is split between workgroups
    ra = torch.randint(0, 256, (128, 768), dtype=torch.uint8, device=dev)
    rw = torch.randint(-128, 128, (3072, 768), dtype=torch.int8, device=dev)
    rc = torch.empty((128, 3072), dtype=torch.int32, device=dev)
    us_r8 = time_us(lambda: _lib.check(L.unit_dense_u8s8s32(ra.data_ptr(), rw.data_ptr(), rc.data_ptr(), 128, 3072, 768, stream)),
                    50, bursts=3)
    v_r8 = U.last_variant()
    rha = torch.randn((128, 3072), dtype=torch.float16, device=dev) / 55
    rhb = torch.randn((3072, 768), dtype=torch.float16, device=dev)
    rhc = torch.empty((128, 768), dtype=torch.float32, device=dev)
    us_r16 = time_us(lambda: _lib.check(L.unit_gemm_f16(rha.data_ptr(), rhb.data_ptr(), rhc.data_ptr(), 128, 768, 3072, 0, stream)),
                     50, bursts=3)
    v_r16 = U.last_variant()
    torch.cuda.synchronize()
    want = rha.float() @ rhb.float()
    gemm_ref_sizes = dict(
        int8_dense_128x3072x768=dict(us=round(us_r8, 2), kernel=v_r8, source="apps/cpu/kernel/int8-gemm.py:9, apps/cpu/relay/int8-gemm.py:14-16"),
        fp16_gemm_128x768x3072=dict(us=round(us_r16, 2), kernel=v_r16, source="apps/gpu/gemm.py:6",
                                    max_rel_err=float(((rhc - want).abs() / want.abs().clamp_min(1e-3 * float(want.abs().max()))).max())))
    del ra, rw, rc, rha, rhb, rhc, want

    # ------------------------------------------------------------------ secondary legs (BASELINE.json configs 0, 3, 4-fp16; layouts)
    def conv_i8_leg(shapes, batch, iters, fused=False, prepared=False, requant=False, device_data=False):
        rows, tot_us, tot_ops = [], 0.0, 0.0
        for i, s in enumerate(shapes):
            cb = WL.channel_block(s.C)
            cp = -(-s.C // cb) * cb
            if device_data:  # large batches: uniform bytes drawn on the GPU (seeded)
                gen = torch.Generator(device=dev)
                gen.manual_seed(3000 + i)
                d = torch.randint(0, 256, (batch, cp // cb, s.H, s.W, cb), dtype=torch.uint8, device=dev, generator=gen)
            else:
                d = dev_t(rng.uniform_u8((batch, cp // cb, s.H, s.W, cb), 3000 + i))
            w = dev_t(rng.uniform_s8((s.K // 16, cp // cb, s.KH, s.KW, cb // 4, 16, 4), 4000 + i))
            oh, ow = WL.out_hw(s)
            o = torch.empty((batch, s.K // 16, oh, ow, 16), dtype=torch.int32, device=dev)
            desc = _lib.ConvDesc(batch, cp, s.H, s.W, s.K, s.KH, s.KW, s.stride, s.stride, s.pad, s.pad, s.pad, s.pad,
                                 1, 1, cb)
            prep = (prepared or requant) and (s.KH * s.KW <= 31 if cb == 16 else s.KW <= 8)
            if prep:
                w = U.prepare_conv2d_weight(w).buf
            if requant:  # u8 output in the layout the next convolution reads: 4 x less output traffic
                o = torch.empty((batch, s.K // 16, oh, ow, 16), dtype=torch.uint8, device=dev)
                bias = dev_t(rng.uniform_s8((s.K,), 5000 + i).astype(np.int32) * 1000)
                f = lambda: _lib.check(L.unit_conv2d_nchwc_u8s8u8_requant_prepared(
                    ctypes.byref(desc), d.data_ptr(), w.data_ptr(), bias.data_ptr(), 3, 14, o.data_ptr(), stream))
            elif fused:  # signed activations, bias and scale: the form the reference's quantized graphs run
                d = d.view(torch.int8)
                bias = dev_t(rng.uniform_s8((s.K,), 5000 + i).astype(np.int32) * 1000)
                fn = L.unit_conv2d_nchwc_s8s8s32_fused_prepared if prep else L.unit_conv2d_nchwc_s8s8s32_fused
                f = lambda: _lib.check(fn(ctypes.byref(desc), d.data_ptr(), w.data_ptr(), bias.data_ptr(), 11,
                                          o.data_ptr(), stream))
            else:
                fn = L.unit_conv2d_nchwc_u8s8s32_prepared if prep else L.unit_conv2d_nchwc_u8s8s32
                f = lambda: _lib.check(fn(ctypes.byref(desc), d.data_ptr(), w.data_ptr(), o.data_ptr(), stream))
            us = time_us(f, iters)
            ops = 2 * WL.macs(s, batch)
            rows.append(dict(layer=s.name, us=round(us, 2), tops=round(ops / us / 1e6, 2), kernel=U.last_variant()))
            tot_us += us * s.count
            tot_ops += ops * s.count
        return rows, tot_us, tot_ops

    use_prep = args.weights == "prepared"
    r18_rows, r18_us, r18_ops = conv_i8_leg(WL.RESNET18, 1, 30, prepared=use_prep)
    resnet18_b1 = dict(workload="ResNet-18 v1 conv layers, batch 1, int8 (BASELINE.json configs[3])",
                       stack_us=round(r18_us, 1), tops=round(r18_ops / r18_us / 1e6, 2), layers=r18_rows)
    single_rows, _, _ = conv_i8_leg((WL.SINGLE_CONV,), 1, 50, prepared=use_prep)
    single_conv = dict(workload="N=1 C=64 56x56 K=64 3x3 s1 p1 NCHW16c (BASELINE.json configs[0])", **single_rows[0],
                       reference_us=24.27, reference_source="cpu-tune.log:160 (x86 VNNI, hardware unstated)")

    # the same sweep at batch 256: what the kernels reach once the 3.5 us launch-to-launch floor no longer counts
    lb_rows, lb_us, lb_ops = conv_i8_leg(WL.RESNET50, 256, 10, prepared=use_prep, device_data=True)
    for r in lb_rows:
        r["pct_int8_mfma_peak"] = round(100 * r["tops"] / 5000.0, 1)
    large_batch = dict(workload="ResNet-50 v1 conv layers, batch 256, int8 u8 x s8 -> i32 (the sweep of configs[4] at 8 x the "
                                "batch; per-layer rate against the 5 POP/s dense int8 MFMA peak)",
                       stack_us=round(lb_us, 1), tops=round(lb_ops / lb_us / 1e6, 2),
                       pct_int8_mfma_peak=round(100 * lb_ops / lb_us / 1e6 / 5000.0, 1), layers=lb_rows)
    torch.cuda.empty_cache()

    fu_rows, fu_us, fu_ops = conv_i8_leg(WL.RESNET50, BATCH, 20, fused=True, prepared=use_prep)
    fused_s8 = dict(workload="ResNet-50 v1 conv stack, batch 32, fused signed form (conv + bias) * scale of "
                             "apps/cpu/relay/result.log:3-26 (s8 x s8 -> i32)",
                    stack_us=round(fu_us, 1), tops=round(fu_ops / fu_us / 1e6, 2), layers=fu_rows)
    if use_prep:
        _, fr_us, _ = conv_i8_leg(WL.RESNET50, BATCH, 20, fused=True)
        fused_s8["reference_layout_weights_stack_us"] = round(fr_us, 1)
    rq_rows, rq_us, rq_ops = conv_i8_leg(WL.RESNET50, BATCH, 20, requant=True)
    requant_u8 = dict(workload="ResNet-50 v1 conv stack, batch 32, u8 x s8 with the output requantised to u8 NCHW16c "
                               "(clamp(((conv + bias) * scale + half) >> shift, 0, 255)); an extension, not in the "
                               "reference's graphs",
                      stack_us=round(rq_us, 1), tops=round(rq_ops / rq_us / 1e6, 2), layers=rq_rows)

    # The same network as a chain: the 52 convolutions behind the stem, each reading the u8 NCHW16c output of the one
    # before it (projection shortcuts as side branches), buffers owned by the runner, replayed as one HIP graph.
    from unit_amd import chain as CH
    ch_layers = CH.resnet50_layers(lambda oc, ic, k: torch.randint(-128, 128, (oc, ic, k, k), dtype=torch.int8, device=dev),
                                   lambda oc: torch.randint(-1000, 1000, (oc,), dtype=torch.int32, device=dev))
    ch = CH.ConvChain(ch_layers, (BATCH, 4, 56, 56, 16))
    ch_x = torch.randint(0, 256, (BATCH, 4, 56, 56, 16), dtype=torch.uint8, device=dev)
    for i, ly in enumerate(ch_layers):  # per-layer shift from the layer's own int32 sums: activations stay spread over 0..255
        acc = U.conv2d_NCHWc_int8(ch.source_of(i, ch_x), ch.weights[i], ly.stride, ly.padding)
        p95 = float(torch.quantile(acc.flatten()[::61][:1 << 20].float(), 0.95))
        ch.consts[i] = (3, max(1, int(np.ceil(np.log2(max(p95, 1.0) * 3 / 200)))))
        ch.launch_layer(i, ch_x)
        del acc
    ch_alive = min(float((o[:1] > 0).float().mean()) for o in ch.outputs)
    ch_iso = sum(time_us(lambda i=i: ch.launch_layer(i, ch_x), 20) for i in range(len(ch_layers)))
    ch_eager = time_us(lambda: ch.run(ch_x), 10)
    ch_replay = ch.graph(ch_x)
    ch_graph = time_us(ch_replay, 10)
    ch_ops = sum(2 * WL.macs(s_, BATCH) * s_.count for s_ in WL.RESNET50[1:])
    conv_chain = dict(workload="ResNet-50 v1 behind the stem as a chain: 52 requantising convolutions, batch 32, each reading the "
                               "u8 NCHW16c output of the one before it (projection shortcuts as side branches; residual additions "
                               "are not part of the path); an extension like the requantised output itself",
                      hipgraph_us=round(ch_graph, 1), eager_us=round(ch_eager, 1), sum_of_isolated_layers_us=round(ch_iso, 1),
                      tops=round(ch_ops / ch_graph / 1e6, 2), min_fraction_of_nonzero_activations=round(ch_alive, 3))
    del ch, ch_replay

    # The Relay-level graph of apps/cpu/relay/conv2d.py:15-27, NCHW int8 in -> NCHW int32 out, as it runs per call
    # (result.log:30-36): Op #0 data layout transform, Op #5 fused convolution, Op #6 output layout transform --
    # folded into the convolution's store, and as a kernel of its own.  Weight-side ops #1-#4 are constants.
    def relay_leg(shapes, batch, iters):
        rows, tot_f, tot_u, same = [], 0.0, 0.0, True
        for i, (s, n) in enumerate(shapes):
            cb = WL.channel_block(s.C)
            cp = -(-s.C // cb) * cb
            oh, ow = WL.out_hw(s)
            x = torch.randint(-128, 128, (n, s.C, s.H, s.W), dtype=torch.int8, device=dev)
            wt = torch.randint(-128, 128, (s.K, s.C, s.KH, s.KW), dtype=torch.int8, device=dev)
            bias = dev_t(rng.uniform_s8((s.K,), 6000 + i).astype(np.int32) * 1000)
            wp = U.prepare_conv2d_weight(U.prepack_conv_weight(wt, cb)).buf
            data = torch.empty((n, cp // cb, s.H, s.W, cb), dtype=torch.int8, device=dev)
            o5 = torch.empty((n, s.K // 16, oh, ow, 16), dtype=torch.int32, device=dev)
            o4 = torch.empty((n, s.K, oh, ow), dtype=torch.int32, device=dev)
            desc = _lib.ConvDesc(n, cp, s.H, s.W, s.K, s.KH, s.KW, s.stride, s.stride, s.pad, s.pad, s.pad, s.pad, 1, 1, cb)

            def op0():
                _lib.check(L.unit_pack_nchwc(x.data_ptr(), data.data_ptr(), n, s.C, s.H, s.W, cb, 1, stream))

            def folded():
                op0()
                _lib.check(L.unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(
                    ctypes.byref(desc), data.data_ptr(), wp.data_ptr(), bias.data_ptr(), 11, o4.data_ptr(), s.K, stream))

            def unfolded():
                op0()
                _lib.check(L.unit_conv2d_nchwc_s8s8s32_fused_prepared(
                    ctypes.byref(desc), data.data_ptr(), wp.data_ptr(), bias.data_ptr(), 11, o5.data_ptr(), stream))
                _lib.check(L.unit_unpack_nchwc(o5.data_ptr(), o4.data_ptr(), n, s.K, oh, ow, 16, 4, stream))

            unfolded()
            torch.cuda.synchronize()
            want = o4.clone()
            o4.zero_()
            us_f = time_us(folded, iters)
            kern = U.last_variant()
            same = same and torch.equal(o4, want)
            us_u = time_us(unfolded, iters)
            rows.append(dict(layer=s.name, batch=n, graph_us=round(us_f, 2), unfolded_us=round(us_u, 2), kernel=kern))
            tot_f += us_f * s.count
            tot_u += us_u * s.count
        return rows, tot_f, tot_u, same

    logged = WL.ConvShape("1x1_1024_2048@16", 1024, 16, 16, 2048, 1, 1, 1, 0, 1)
    rl_rows, _, _, rl_same0 = relay_leg(((logged, 1),), 1, 30)
    rl_rows[0].update(reference_us=234.7, reference_source="sum of the seven operators at apps/cpu/relay/result.log:30-36 "
                                                         "(x86 VNNI, -mcpu=cascadelake; 206.0 us without the weight-side operators #1-#4)")
    r50_rows, r50_f, r50_u, rl_same = relay_leg(tuple((s, BATCH) for s in WL.RESNET50), BATCH, 20)
    relay_graph = dict(workload="(conv2d(x, w) + b) * 11, x int8 NCHW -> int32 NCHW (apps/cpu/relay/conv2d.py:15-27): data layout "
                                "transform + fused convolution storing NCHW; `unfolded` runs the output layout transform as its own kernel",
                       logged_graph=rl_rows[0], resnet50_b32_stack_us=round(r50_f, 1),
                       resnet50_b32_unfolded_stack_us=round(r50_u, 1), folded_equals_unfolded=bool(rl_same and rl_same0),
                       layers=r50_rows)

    # 3-D convolution workloads of apps/cpu/kernel/conv3d.py:13-25 (depth 16, batch 1)
    c3_rows = []
    for i, (ic, h, w_, oc, ks, st) in enumerate(((256, 16, 16, 256, 3, 1), (512, 9, 9, 512, 3, 1), (128, 30, 30, 128, 3, 1),
                                                   (64, 56, 56, 128, 1, 2), (64, 58, 58, 64, 3, 1), (128, 28, 28, 256, 1, 2),
                                                   (256, 16, 16, 512, 3, 2), (64, 58, 58, 128, 3, 2), (4, 230, 230, 64, 7, 2),
                                                   (128, 30, 30, 256, 3, 2), (256, 14, 14, 512, 1, 2))):
        cb3 = 4 if ic % 16 else 16   # conv3d.py:39-56
        a3 = torch.randint(-128, 128, (1, ic // cb3, 16, h, w_, cb3), dtype=torch.int8, device=dev)
        w3 = torch.randint(-128, 128, (oc // 16, ic // cb3, ks, ks, ks, cb3 // 4, 16, 4), dtype=torch.int8, device=dev)
        od, oh, ow = (16 - ks) // st + 1, (h - ks) // st + 1, (w_ - ks) // st + 1
        o3 = torch.empty((1, oc // 16, od, oh, ow, 16), dtype=torch.int32, device=dev)
        d3 = _lib.Conv3dDesc(1, ic, 16, h, w_, oc, ks, ks, ks, st)
        f = lambda: _lib.check(L.unit_conv3d_ncdhwc_s8s8s32(ctypes.byref(d3), a3.data_ptr(), w3.data_ptr(), o3.data_ptr(),
                                                            stream))
        us = time_us(f, 20)
        ops = 2.0 * od * oh * ow * oc * ic * ks ** 3
        c3_rows.append(dict(workload=f"{ic}x16x{h}x{w_} -> {oc}, {ks}^3 s{st}", us=round(us, 2),
                            tops=round(ops / us / 1e6, 1), kernel=U.last_variant()))
    conv3d = dict(workload="3-D int8 convolutions of apps/cpu/kernel/conv3d.py:13-25, NCDHW16c / NCDHW4c, s8 x s8 -> i32",
                  layers=c3_rows)

    # fp16 variant of the ResNet-50 b32 sweep: valid convolution on pre-padded NCHW16c inputs
    f16_rows, f16_us, f16_flops, f16_ref_us = [], 0.0, 0.0, 0.0
    for i, s in enumerate(WL.RESNET50):
        if s.C % 16:
            continue  # the fp16 operator needs C % 16 == 0 (the 3-channel stem has no NCHW16c form)
        hp, wp_ = s.H + 2 * s.pad, s.W + 2 * s.pad
        a = torch.randn((BATCH, s.C // 16, hp, wp_, 16), dtype=torch.float16, device=dev)
        b = torch.randn((s.K // 16, s.C // 16, s.KH, s.KW, 16, 16), dtype=torch.float16, device=dev) * 0.05
        oh, ow = WL.out_hw(s)
        o = torch.empty((BATCH, s.K // 16, oh, ow, 16), dtype=torch.float32, device=dev)
        desc = _lib.ConvDesc(BATCH, s.C, hp, wp_, s.K, s.KH, s.KW, s.stride, s.stride, 0, 0, 0, 0, 1, 1, 16)
        f = lambda: _lib.check(L.unit_conv2d_nchw16c_f16f32(ctypes.byref(desc), a.data_ptr(), b.data_ptr(),
                                                            o.data_ptr(), stream))
        if use_prep:
            f16_ref_us += time_us(f, 20) * s.count
            bp = U.prepare_conv2d_weight(b).buf
            f = lambda: _lib.check(L.unit_conv2d_nchw16c_f16f32_prepared(ctypes.byref(desc), a.data_ptr(), bp.data_ptr(),
                                                                         o.data_ptr(), stream))
        us = time_us(f, 20)
        flops = 2 * WL.macs(s, BATCH)
        f16_rows.append(dict(layer=s.name, us=round(us, 2), tflops=round(flops / us / 1e6, 1),
                             pct_f16_peak=round(100 * flops / us / 1e6 / PEAK_F16_TFLOPS, 2), kernel=U.last_variant()))
        f16_us += us * s.count
        f16_flops += flops * s.count
    conv_fp16 = dict(workload="ResNet-50 v1 conv layers except the stem, batch 32, fp16 -> fp32 (BASELINE.json configs[4], "
                              "fp16 variant)", stack_us=round(f16_us, 1), tflops=round(f16_flops / f16_us / 1e6, 1),
                     layers=f16_rows)
    if use_prep:
        conv_fp16["reference_layout_weights_stack_us"] = round(f16_ref_us, 1)

    # layout transforms / pre-packs: bytes read + written over time
    x8 = torch.randint(0, 256, (BATCH, 256, 56, 56), dtype=torch.uint8, device=dev)
    o32 = torch.empty((BATCH, 16, 56, 56, 16), dtype=torch.int32, device=dev)
    w33 = torch.randint(-128, 128, (512, 512, 3, 3), dtype=torch.int8, device=dev)
    layout = {}
    us = time_us(lambda: U.pack_nchwc(x8, 16), 20)
    layout["pack_nchw16c_u8_32x256x56x56"] = dict(us=round(us, 2), gbs=round(2 * x8.numel() / us / 1e3, 1))
    p8 = U.pack_nchwc(x8, 16)
    us = time_us(lambda: U.unpack_nchwc(p8), 20)
    layout["unpack_nchw16c_u8_32x256x56x56"] = dict(us=round(us, 2), gbs=round(2 * x8.numel() / us / 1e3, 1))
    del p8
    us = time_us(lambda: U.unpack_nchwc(o32), 20)
    layout["unpack_nchw16c_i32_32x256x56x56"] = dict(us=round(us, 2), gbs=round(2 * o32.numel() * 4 / us / 1e3, 1))
    us = time_us(lambda: U.prepack_conv_weight(w33, 16), 20)
    layout["prepack_conv_weight_512x512x3x3"] = dict(us=round(us, 2), gbs=round(2 * w33.numel() / us / 1e3, 1))
    us = time_us(lambda: U.prepack_dense_weight(w8), 20)
    layout["prepack_dense_weight_4096x4096"] = dict(us=round(us, 2), gbs=round(2 * w8.numel() / us / 1e3, 1))
    # plain device-to-device copy of known size: the HBM calibration point for the counters
    src = torch.empty(128 * 1024 * 1024, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    us = time_us(lambda: dst.copy_(src), 10)
    layout["plain_copy_128MiB"] = dict(us=round(us, 2), gbs=round(2 * src.numel() / us / 1e3, 1))
    del src, dst

    # register-only MFMA throughput of this box (no memory traffic): what the silicon sustains
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    probe = {}
    # (constant operands, then operands whose bits change from one MFMA to the next: clocks follow
    # power, and the bench data is uniform random)
    for f16, key, per in ((0, "int8_tops", 65536.0), (1, "fp16_tflops", 32768.0),
                          (2, "int8_tops_random_operands", 65536.0), (3, "fp16_tflops_random_operands", 32768.0)):
        blocks, iters = 512, 4000
        L.unit_mfma_peak(f16, blocks, 200, sink.data_ptr(), stream)
        us = time_us(lambda: _lib.check(L.unit_mfma_peak(f16, blocks, iters, sink.data_ptr(), stream)), 3, warm=1)
        probe[key] = round(blocks * 16 * iters * per / us / 1e6, 1)

    # HBM traffic of the dominant kernel, when a counter run has been recorded for that layer
    roofline["traffic"] = MEASURED_HBM_BYTES.get(roofline["layer"])

    # ------------------------------------------------------------------ CPU baseline + bit-exactness
    cpu_baseline = None
    bit_exact = None
    if not args.no_cpu:
        from oracle import oracle as O  # the checker; also the timed CPU baseline ("port")
        cores = len(os.sched_getaffinity(0))
        cpu_s = 0.0
        bit_exact = True
        for ly in layers:
            s = ly["shape"]
            w_np = ly["wt"].cpu().numpy()
            O.c_conv2d_nchwc(ly["data_np"][:1], w_np, s.stride, s.pad, 1)  # warm the thread pool
            # repeated for about 0.5 s per layer shape (about 10 s of CPU work in all); the mean counts
            reps, t1 = 0, time.perf_counter()
            while reps < 3 or time.perf_counter() - t1 < 0.5:
                ref = O.c_conv2d_nchwc(ly["data_np"], w_np, s.stride, s.pad, 1, impl="vnni", nthreads=cores)
                reps += 1
            cpu_s += (time.perf_counter() - t1) / reps * s.count
            ly["call"]()
            torch.cuda.synchronize()
            if not np.array_equal(ly["out"].cpu().numpy(), ref):
                bit_exact = False
                print(f"bench.py: MISMATCH vs oracle in layer {s.name}", file=sys.stderr)
        g_rm()
        torch.cuda.synchronize()
        rows = 512
        a8_rows, wp8_np = a8[:rows].cpu().numpy(), O.prepack_dense_weight(w8_np)
        ref = O.c_dense(a8_rows, wp8_np, nthreads=cores)
        if not np.array_equal(c8[:rows].cpu().numpy(), ref):
            bit_exact = False
            print("bench.py: MISMATCH vs oracle in int8 GEMM", file=sys.stderr)
        # the GEMM configs on the host, on a bounded sample (512 of the 4096 rows of a, all of b), the reference's
        # number=10 protocol (apps/cpu/kernel/int8-gemm.py:34): int8 by the VNNI oracle, fp16 as an fp32 GEMM of the
        # fp16-rounded operands (torch CPU matmul); and the host's vpdpbusd peak, as poc/vnni/micro.cc measures it
        t1 = time.perf_counter()
        for _ in range(10):
            O.c_dense(a8_rows, wp8_np, nthreads=cores)
        cpu_i8_s = (time.perf_counter() - t1) / 10
        af32, bf32 = torch.from_numpy(ah_np[:rows].astype(np.float32)), torch.from_numpy(bh_np.astype(np.float32))
        torch.matmul(af32, bf32)
        t1 = time.perf_counter()
        for _ in range(10):
            torch.matmul(af32, bf32)
        cpu_f16_s = (time.perf_counter() - t1) / 10
        vnni_peak = O.vnni_peak_gops(nthreads=cores) / 1e3 if O.has_vnni() else None
        cpu_baseline = dict(value=round(step_ops / cpu_s / 1e12, 4), unit="TOP/s", cores=cores, kind="port",
                            vnni=bool(O.has_vnni()),
                            sample="the same step (53 convolutions, batch 32) by the AVX-512 VNNI oracle: each of "
                                   "the 20 unique layers repeated for about 0.5 s, mean time x its multiplicity",
                            seconds=round(cpu_s, 3),
                            host_vnni_peak_tops=None if vnni_peak is None else round(vnni_peak, 3),
                            pct_of_host_vnni_peak=None if not vnni_peak else round(100 * step_ops / cpu_s / 1e12 / vnni_peak, 1),
                            gemm_int8_4096=dict(tops=round(2.0 * rows * N * K / cpu_i8_s / 1e12, 3),
                                                sample=f"{rows} of the 4096 rows of a, mean of 10 runs, VNNI oracle"),
                            gemm_fp16_4096=dict(tflops=round(2.0 * rows * N * K / cpu_f16_s / 1e12, 3),
                                                sample=f"{rows} of the 4096 rows of a, mean of 10 runs, torch CPU fp32 matmul "
                                                       "of the fp16-rounded operands"))
        gemm_i8["bit_exact_rows_checked"] = rows

    line = {
        "metric": "int8 conv2d TOPS & % int8 MFMA peak (ResNet-50 b32); fp16 GEMM TFLOPS",
        "value": round(value, 2),
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": "ResNet-50 v1 conv stack (53 convolutions, 20 unique shapes), batch 32, int8 "
                               "u8 x s8 -> i32, NCHW16c / NCHW4c stem (BASELINE.json configs[4])",
                   "batch": BATCH, "ops_per_step": step_ops,
                   "weights": ("prepared once before the timed region (unit_conv2d_prepare_weight: MFMA fragment "
                               "order + 128 * sum(w)), as the reference folds its weight layout chain and sum(w) "
                               "into constants" if args.weights == "prepared"
                               else "the reference's blocked layout in every call")},
        "pct_int8_mfma_peak": round(100 * value / PEAK_INT8_TOPS, 2),
        "host_wall_ms_per_step": round(wall_ms, 4),
        "launch": launch_mode,
        "eager_ms_per_step": round(eager_ms, 4),
        "hipgraph_ms_per_step": None if graph_ms is None else round(graph_ms, 4),
        "bit_exact_vs_oracle": bit_exact,
        "reference_layout_weights": ref_weights,
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "gemm_int8_4096": gemm_i8,
        "gemm_fp16_4096": gemm_f16,
        "gemm_reference_sizes": gemm_ref_sizes,
        "mfma_probe": probe,
        "single_conv": single_conv,
        "resnet18_b1": resnet18_b1,
        "conv_i8_resnet50_b256": large_batch,
        "conv_fp16_resnet50_b32": conv_fp16,
        "conv_fused_s8_resnet50_b32": fused_s8,
        "conv_requant_u8_resnet50_b32": requant_u8,
        "conv_chain_u8_resnet50_b32": conv_chain,
        "relay_graph_s8": relay_graph,
        "conv3d_s8": conv3d,
        "layout_kernels": layout,
        "layers": table,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
