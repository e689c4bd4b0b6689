#!/usr/bin/env python3
"""Benchmark of the tensorized conv2d / GEMM path on one MI355X.

A step is one pass over the 53 convolutions of ResNet-50 v1 at batch 32 (20 unique layer shapes x
their multiplicity), int8 u8 x s8 -> i32 in NCHW16c / NCHW4c, through the C ABI with operands and
outputs already resident in HBM.  `value` is the whole-step throughput in TOP/s (2 x logical MACs /
time).

Output: every leg prints one `DETAIL {json}` line as soon as it is done (per-layer tables, the
4096^3 GEMMs, the fp16 sweep, ...); the LAST line of stdout is one compact JSON object (under
2 KiB) with the headline, the roofline of the layer that takes the largest share of the step, the
CPU baseline and the GEMM scalars.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--full]
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
COLD_BYTES = 640 << 20    # the cold legs cycle through this many bytes of operand copies (memory-side cache: 256 MB)
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_table.txt")
FINAL_LINE_BUDGET = 2048


def detail(leg, **fields):
    print("DETAIL " + json.dumps(dict(leg=leg, **fields)), flush=True)


def read_traffic_table(path=TRAFFIC_TABLE):
    """Rows `layer kernel bytes_per_launch profile_file` measured with rocprofv3 FETCH_SIZE / WRITE_SIZE runs."""
    table = {}
    try:
        with open(path) as f:
            for ln in f:
                parts = ln.split()
                if len(parts) >= 4 and not ln.startswith("#"):
                    table[(parts[0], parts[1])] = (int(parts[2]), parts[3])
    except OSError:
        pass
    return table


def compact_line(line, budget=FINAL_LINE_BUDGET):
    """The final line must survive a tail of a few KiB: drop optional keys until it fits."""
    optional = ["probe", "fp16_conv", "launch", "config_note"]
    s = json.dumps(line, separators=(",", ":"))
    while len(s) > budget and optional:
        line.pop(optional.pop(0), None)
        s = json.dumps(line, separators=(",", ":"))
    return s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / bit-exactness leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only (no HIP graph replay)")
    ap.add_argument("--full", action="store_true",
                    help="also run the secondary legs (fused / requantised stacks, layer chain, conv3d, layouts of every size)")
    ap.add_argument("--weights", default="prepared", choices=["prepared", "reference"],
                    help="headline convolutions on weights prepared once with unit_conv2d_prepare_weight (default), "
                         "or on the reference's blocked layout in every call")
    ap.add_argument("--profile", default=None, metavar="WHAT",
                    help="launch one kernel 20 times and exit (for rocprofv3): a ResNet-50 layer name such as "
                         "3x3_256_256@14 (append :f16 for the fp16 convolution, :cold to cycle operand copies), "
                         "or gemm_i8 / gemm_i8_prepared / gemm_f16 / gemm_f16_prepared / gemm_f16_2048 / copy / pack_u8")
    ap.add_argument("--profile-launches", type=int, default=20, metavar="N",
                    help="launches of the --profile kernel (default 20; the 4096^3 GEMMs reach their steady-state clocks "
                         "after ~300 launches: profile 500 and read the last ones)")
    ap.add_argument("--profile-batch", type=int, default=None, metavar="N",
                    help="batch of the --profile launches of a layer (default: the benchmark's 32)")
    args = ap.parse_args()
    if args.profile_batch:
        if not args.profile:
            ap.error("--profile-batch goes with --profile")
        global BATCH
        BATCH = args.profile_batch
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

    last_min = [0.0]

    def time_us(fn, iters, warm=3, bursts=1, median=True):
        """Mean launch-to-launch time of `iters` back-to-back launches (HIP events on the launch stream); with
        bursts > 1 the median burst -- one protocol for every leg.  The fastest burst is left in last_min[0].
        `warm` untimed launches come first: the clocks of this part follow the load of whatever ran just before
        (launch by launch the 4096^3 int8 GEMM runs 69, 82 around the 50th, then 65 us from the ~300th launch on), so the
        GEMM legs warm up with sustained launches and report the steady state."""
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
        last_min[0] = min(seen)
        return sorted(seen)[len(seen) // 2] if median else min(seen)

    prof, prof_mode = (args.profile.split(":") + [""])[:2] if args.profile else (None, "")
    if prof in ("gemm_i8", "gemm_i8_prepared", "gemm_f16", "gemm_f16_prepared", "gemm_f16_2048", "copy", "pack_u8"):
        n = 2048 if prof.endswith("_2048") else 4096
        if prof == "gemm_i8":
            a = dev_t(rng.uniform_u8((n, n), 11))
            w = dev_t(rng.uniform_s8((n, n), 12))
            fn = lambda: U.dense(a, w)
        elif prof == "gemm_i8_prepared":
            a = dev_t(rng.uniform_u8((n, n), 11))
            pw = U.prepare_dense_weight(dev_t(rng.uniform_s8((n, n), 12)))
            fn = lambda: U.dense(a, pw)
        elif prof in ("gemm_f16", "gemm_f16_2048"):
            a = dev_t(rng.normal_f16((n, n), 13, 1.0 / 64))
            b = dev_t(rng.normal_f16((n, n), 14))
            fn = lambda: U.gemm_fp16(a, b)
        elif prof == "gemm_f16_prepared":
            a = dev_t(rng.normal_f16((n, n), 13, 1.0 / 64))
            pb = U.prepare_gemm_b(dev_t(rng.normal_f16((n, n), 14)))
            fn = lambda: U.gemm_fp16(a, pb)
        elif prof == "pack_u8":
            x8 = torch.randint(0, 256, (BATCH, 256, 56, 56), dtype=torch.uint8, device=dev)
            fn = lambda: U.pack_nchwc(x8, 16)
        else:  # plain 1 GiB device-to-device copy (larger than the 256 MB memory-side cache): the calibration
            a = torch.empty(1 << 30, dtype=torch.uint8, device=dev)   # point for FETCH_SIZE / WRITE_SIZE
            b = torch.empty_like(a)
            fn = lambda: b.copy_(a)
        for _ in range(args.profile_launches):
            fn()
        torch.cuda.synchronize()
        print(json.dumps({"profiled": prof, "launches": args.profile_launches, "kernel": U.last_variant()}))
        return

    def cold_copies(tensors, per_bytes):
        """As many copies of a launch's tensors as fill COLD_BYTES (at most 96): a launch then finds its operands
        the way a layer of a running network does, not in the caches its own previous launch filled."""
        n_inst = max(2, min(96, COLD_BYTES // per_bytes + 1))
        return [tensors] + [tuple(t.clone() for t in tensors) for _ in range(n_inst - 1)]

    # ------------------------------------------------------------------ ResNet-50 b32 int8 conv stack
    layers = []
    for idx, s in enumerate(WL.RESNET50):
        if prof and s.name != prof:
            continue
        if prof_mode == "f16":
            break
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
            L.unit_conv2d_nchwc_u8s8s32(ctypes.byref(d), x.data_ptr(), w.data_ptr(), o.data_ptr(), stream)))
        call, prep, entry, wbuf = call_ref, None, L.unit_conv2d_nchwc_u8s8s32, wt
        if args.weights == "prepared" and (cb == 16 or s.KW <= 8):
            # the constant weight is re-ordered once, before the timed region, as the reference's compiled
            # graphs fold the weight layout chain and sum(w) (apps/cpu/relay/result.log:8-16)
            prep = U.prepare_conv2d_weight(wt)
            entry, wbuf = L.unit_conv2d_nchwc_u8s8s32_prepared, prep.buf
            call = (lambda d=desc, x=data, w=prep.buf, o=out: _lib.check(
                L.unit_conv2d_nchwc_u8s8s32_prepared(ctypes.byref(d), x.data_ptr(), w.data_ptr(), o.data_ptr(), stream)))
        call()
        layers.append(dict(shape=s, cb=cb, data=data, data_np=data_np, wt=wt, wbuf=wbuf, prep=prep, out=out, call=call,
                           call_ref=call_ref, entry=entry, desc=desc, variant=U.last_variant(),
                           ops=2 * WL.macs(s, BATCH), bytes=WL.algorithmic_bytes(s, BATCH)))
    torch.cuda.synchronize()

    def cold_call(ly):
        per = sum(t.numel() * t.element_size() for t in (ly["data"], ly["wbuf"], ly["out"]))
        copies = cold_copies((ly["data"], ly["wbuf"], ly["out"]), per)
        turn = [0]

        def call():
            d_, w_, o_ = copies[turn[0] % len(copies)]
            turn[0] += 1
            _lib.check(ly["entry"](ctypes.byref(ly["desc"]), d_.data_ptr(), w_.data_ptr(), o_.data_ptr(), stream))
        return call, len(copies)

    if prof and prof_mode != "f16":
        if not layers:
            print(f"bench.py: unknown --profile target {args.profile!r}", file=sys.stderr)
            sys.exit(2)
        fn = layers[0]["call"]
        if prof_mode == "cold":
            fn, _ = cold_call(layers[0])
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        print(json.dumps({"profiled": args.profile, "launches": 20 + (prof_mode != "cold"), "kernel": layers[0]["variant"]}))
        return

    def f16_layer(s, prepared=True):
        hp, wp_ = s.H + 2 * s.pad, s.W + 2 * s.pad
        a = torch.randn((BATCH, s.C // 16, hp, wp_, 16), dtype=torch.float16, device=dev)
        b = torch.randn((s.K // 16, s.C // 16, s.KH, s.KW, 16, 16), dtype=torch.float16, device=dev) * 0.05
        oh, ow = WL.out_hw(s)
        o = torch.empty((BATCH, s.K // 16, oh, ow, 16), dtype=torch.float32, device=dev)
        desc = _lib.ConvDesc(BATCH, s.C, hp, wp_, s.K, s.KH, s.KW, s.stride, s.stride, 0, 0, 0, 0, 1, 1, 16)
        f_ref = lambda: _lib.check(L.unit_conv2d_nchw16c_f16f32(ctypes.byref(desc), a.data_ptr(), b.data_ptr(),
                                                                o.data_ptr(), stream))
        if not prepared:
            return f_ref, f_ref
        bp = U.prepare_conv2d_weight(b).buf
        f = lambda: _lib.check(L.unit_conv2d_nchw16c_f16f32_prepared(ctypes.byref(desc), a.data_ptr(), bp.data_ptr(),
                                                                     o.data_ptr(), stream))
        return f, f_ref

    if prof:  # <layer>:f16
        match = [s for s in WL.RESNET50 if s.name == prof and s.C % 16 == 0]
        if not match:
            print(f"bench.py: unknown --profile target {args.profile!r}", file=sys.stderr)
            sys.exit(2)
        f, _ = f16_layer(match[0])
        for _ in range(20):
            f()
        torch.cuda.synchronize()
        print(json.dumps({"profiled": args.profile, "launches": 20, "kernel": U.last_variant()}))
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
                stream = torch.cuda.current_stream().cuda_stream  # the launches go to the capturing stream
                step()
            stream = torch.cuda.current_stream().cuda_stream
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
            del keep
        except Exception as ex:  # graph capture unavailable: the eager figure stands
            print(f"bench.py: HIP graph capture failed ({ex}); reporting eager", file=sys.stderr)
    step_ops = sum(ly["ops"] * ly["shape"].count for ly in layers)
    value = step_ops / (ms_per_step * 1e-3) / 1e12
    ref_ms = None
    if args.weights == "prepared":
        ref_ms = timed(step_ref)[0]
    detail("headline", ms_per_step=round(ms_per_step, 4), tops=round(value, 2), launch=launch_mode,
           eager_ms=round(eager_ms, 4), hipgraph_ms=None if graph_ms is None else round(graph_ms, 4),
           host_wall_ms_per_step=round(wall_ms, 4),
           reference_layout_weights_ms=None if ref_ms is None else round(ref_ms, 4))

    # per-layer launch duration (HIP events on the launch stream, back-to-back launches; the median of three bursts
    # of 30 launches) on hot operands (the same buffers every launch), and on cold ones (the launches cycle through
    # more copies of the layer's tensors than the 256 MB memory-side cache holds)
    ridge = PEAK_INT8_TOPS * 1e12 / (PEAK_HBM_GBS * 1e9)
    table = []
    for ly in layers:
        us = time_us(ly["call"], 30, bursts=3, median=True)
        cfn, n_inst = cold_call(ly)
        us_cold = time_us(cfn, max(30, n_inst), warm=n_inst, bursts=3, median=True)
        del cfn
        torch.cuda.empty_cache()
        ai = ly["ops"] / ly["bytes"]
        bound = "mfma" if ai >= ridge else "hbm"
        tops, gbs = ly["ops"] / us / 1e6, ly["bytes"] / us / 1e3
        frac = tops / PEAK_INT8_TOPS if bound == "mfma" else gbs / PEAK_HBM_GBS
        frac_cold = frac * us / us_cold
        ly["us"], ly["us_cold"] = us, us_cold
        table.append(dict(layer=ly["shape"].name, count=ly["shape"].count, us=round(us, 2), us_cold=round(us_cold, 2),
                          tops=round(tops, 1), pct_int8_peak=round(100 * tops / PEAK_INT8_TOPS, 2), gbs=round(gbs, 1),
                          bound=bound, frac=round(frac, 4), frac_cold=round(frac_cold, 4), kernel=ly["variant"]))
    detail("layers_int8_resnet50_b32", rows=table,
           sum_hot_us=round(sum(ly["us"] * ly["shape"].count for ly in layers), 1),
           sum_cold_us=round(sum(ly["us_cold"] * ly["shape"].count for ly in layers), 1))
    dom = max(layers, key=lambda ly: ly["us"] * ly["shape"].count)
    dom_row = table[layers.index(dom)]
    if dom_row["bound"] == "mfma":
        roofline = dict(bound="mfma", achieved=dom_row["tops"], peak=PEAK_INT8_TOPS, unit="TOP/s")
    else:
        roofline = dict(bound="hbm", achieved=dom_row["gbs"], peak=PEAK_HBM_GBS, unit="GB/s")
    traffic = read_traffic_table().get((dom_row["layer"], dom_row["kernel"]))
    roofline.update(frac=dom_row["frac"], frac_cold=dom_row["frac_cold"], traffic=None if traffic is None else traffic[0],
                    traffic_source=None if traffic is None else traffic[1], kernel=dom_row["kernel"],
                    layer=dom_row["layer"], launch_us=dom_row["us"], launch_us_cold=dom_row["us_cold"])
    # the whole step against its composite roof: every launch at max(bytes / HBM peak, ops / int8 MFMA peak)
    ideal_us = sum(max(ly["bytes"] / (PEAK_HBM_GBS * 1e3), ly["ops"] / (PEAK_INT8_TOPS * 1e6)) * ly["shape"].count
                   for ly in layers)
    roofline_step = dict(ideal_us=round(ideal_us, 1), frac=round(ideal_us / (ms_per_step * 1e3), 3),
                         bytes=int(sum(ly["bytes"] * ly["shape"].count for ly in layers)), ops=int(step_ops),
                         launches=sum(ly["shape"].count for ly in layers))
    mfma_rows = [r for r in table if r["bound"] == "mfma"]
    best_mfma = max(mfma_rows, key=lambda r: r["pct_int8_peak"]) if mfma_rows else None

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
    GEMM_WARM = 400  # sustained launches before the timed bursts (25-50 ms): a 4096^3 GEMM starts at boost clocks,
    # is throttled ~15 % around its 50th launch and settles only after ~300 launches
    us_rm = time_us(g_rm, 30, warm=GEMM_WARM, bursts=3)
    v_rm, min_rm = U.last_variant(), last_min[0]
    us_pk = time_us(g_pk, 30, warm=GEMM_WARM, bursts=3)
    v_pk = U.last_variant()
    # the same dense with the weight's row sums folded once before the timed region (a constant operand, as the
    # reference's graphs fold sum(w) next to their u8 x s8 operators): both tiles global -> LDS directly
    wsum8 = torch.empty((N,), dtype=torch.int32, device=dev)
    _lib.check(L.unit_dense_prepare_weight(w8.data_ptr(), wsum8.data_ptr(), N, K, stream))
    g_pp = lambda: _lib.check(L.unit_dense_u8s8s32_prepared(a8.data_ptr(), w8.data_ptr(), wsum8.data_ptr(), c8.data_ptr(),
                                                            M, N, K, stream))
    us_pp = time_us(g_pp, 30, warm=GEMM_WARM, bursts=3)
    v_pp, min_pp = U.last_variant(), last_min[0]
    torch.cuda.synchronize()
    c8_pp = c8.clone()
    gemm_ops = 2.0 * M * N * K
    gemm_timing = f"median of 3 bursts of 30 launches after {GEMM_WARM} warm-up launches (us_min: the fastest burst)"
    gemm_i8 = dict(workload="int8 GEMM 4096^3 u8 x s8 -> i32", timing=gemm_timing,
                   prepared_weight=dict(us=round(us_pp, 2), us_min=round(min_pp, 2), tops=round(gemm_ops / us_pp / 1e6, 1),
                                        pct_int8_peak=round(100 * gemm_ops / us_pp / 1e6 / PEAK_INT8_TOPS, 2), kernel=v_pp),
                   row_major=dict(us=round(us_rm, 2), us_min=round(min_rm, 2), tops=round(gemm_ops / us_rm / 1e6, 1),
                                  pct_int8_peak=round(100 * gemm_ops / us_rm / 1e6 / PEAK_INT8_TOPS, 2), kernel=v_rm),
                   vnni_packed=dict(us=round(us_pk, 2), tops=round(gemm_ops / us_pk / 1e6, 1),
                                    pct_int8_peak=round(100 * gemm_ops / us_pk / 1e6 / PEAK_INT8_TOPS, 2),
                                    kernel=v_pk))
    ah_np = rng.normal_f16((M, K), 13, 1.0 / np.sqrt(K))
    bh_np = rng.normal_f16((K, N), 14)
    ah, bh = dev_t(ah_np), dev_t(bh_np)
    cf = torch.empty((M, N), dtype=torch.float32, device=dev)
    g_f = lambda: _lib.check(L.unit_gemm_f16(ah.data_ptr(), bh.data_ptr(), cf.data_ptr(), M, N, K, 0, stream))
    us_f = time_us(g_f, 30, warm=GEMM_WARM, bursts=3)
    v_f, min_f = U.last_variant(), last_min[0]
    # the same product with b re-laid once as (N, K) before the timed region (a constant operand, as the
    # reference pre-packs b in apps/gpu/gemm-pack.py)
    pb = U.prepare_gemm_b(bh)
    g_fp = lambda: _lib.check(L.unit_gemm_f16_prepared(ah.data_ptr(), pb.bt.data_ptr(), cf.data_ptr(), M, N, K, 0, stream))
    us_fp = time_us(g_fp, 30, warm=GEMM_WARM, bursts=3)
    v_fp, min_fp = U.last_variant(), last_min[0]

    # fp16 output (BASELINE.json configs[2] names both output types; the reference script's own result is fp32,
    # apps/gpu/gemm.py:14-20): half the bytes to write back
    ch = torch.empty((M, N), dtype=torch.float16, device=dev)
    g_fh = lambda: _lib.check(L.unit_gemm_f16(ah.data_ptr(), bh.data_ptr(), ch.data_ptr(), M, N, K, 1, stream))
    us_fh = time_us(g_fh, 30, warm=GEMM_WARM, bursts=3)
    v_fh, min_fh = U.last_variant(), last_min[0]

    def f16_err():  # every 16th row of the result against float64
        torch.cuda.synchronize()
        ref = ah_np[::16].astype(np.float64) @ bh_np.astype(np.float64)
        got = cf[::16].cpu().numpy().astype(np.float64)
        return float((np.abs(got - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max())).max())
    g_f()
    err_f = f16_err()
    g_fp()
    err_fp = f16_err()
    g_fh()
    torch.cuda.synchronize()
    ref_h = ah_np[::16].astype(np.float64) @ bh_np.astype(np.float64)
    got_h = ch[::16].float().cpu().numpy().astype(np.float64)
    err_fh = float((np.abs(got_h - ref_h) / np.maximum(np.abs(ref_h), 1e-3 * np.abs(ref_h).max())).max())
    del ch, ref_h, got_h
    gemm_f16 = dict(workload="fp16 GEMM 4096^3, fp32 accumulate, fp32 out", timing=gemm_timing,
                    us=round(us_f, 2), us_min=round(min_f, 2), tflops=round(gemm_ops / us_f / 1e6, 1),
                    pct_f16_peak=round(100 * gemm_ops / us_f / 1e6 / PEAK_F16_TFLOPS, 2), kernel=v_f,
                    max_rel_err=err_f, tolerance=1e-2, rows_checked=M // 16,
                    prepared_b=dict(us=round(us_fp, 2), us_min=round(min_fp, 2), tflops=round(gemm_ops / us_fp / 1e6, 1),
                                    pct_f16_peak=round(100 * gemm_ops / us_fp / 1e6 / PEAK_F16_TFLOPS, 2), kernel=v_fp,
                                    max_rel_err=err_fp),
                    f16_out=dict(us=round(us_fh, 2), us_min=round(min_fh, 2), tflops=round(gemm_ops / us_fh / 1e6, 1),
                                 pct_f16_peak=round(100 * gemm_ops / us_fh / 1e6 / PEAK_F16_TFLOPS, 2), kernel=v_fh,
                                 max_rel_err=err_fh))

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
    # the same product with the k-splits' partial tiles in a workspace, added in split order (deterministic)
    ws_bytes = ctypes.c_size_t()
    _lib.check(L.unit_gemm_f16_ws_bytes(128, 768, 3072, ctypes.byref(ws_bytes)))
    rws = torch.empty((max(ws_bytes.value, 16),), dtype=torch.uint8, device=dev)
    rhc2 = torch.empty((128, 768), dtype=torch.float32, device=dev)
    us_r16w = time_us(lambda: _lib.check(L.unit_gemm_f16_ws(rha.data_ptr(), rhb.data_ptr(), rhc2.data_ptr(), 128, 768, 3072, 0,
                                                            rws.data_ptr(), rws.numel(), stream)), 50, bursts=3)
    v_r16w = U.last_variant()
    torch.cuda.synchronize()
    want = rha.float() @ rhb.float()
    gemm_ref_sizes = dict(
        int8_dense_128x3072x768=dict(us=round(us_r8, 2), kernel=v_r8, source="apps/cpu/kernel/int8-gemm.py:9, apps/cpu/relay/int8-gemm.py:14-16"),
        fp16_gemm_128x768x3072=dict(us=round(us_r16, 2), kernel=v_r16, source="apps/gpu/gemm.py:6",
                                    max_rel_err=float(((rhc - want).abs() / want.abs().clamp_min(1e-3 * float(want.abs().max()))).max())),
        fp16_gemm_128x768x3072_workspace=dict(us=round(us_r16w, 2), kernel=v_r16w, workspace_bytes=ws_bytes.value,
                                              max_rel_err=float(((rhc2 - want).abs() / want.abs().clamp_min(1e-3 * float(want.abs().max()))).max())))
    del ra, rw, rc, rha, rhb, rhc, rhc2, rws, want
    detail("gemm_int8_4096", **gemm_i8)
    detail("gemm_fp16_4096", **gemm_f16)
    detail("gemm_reference_sizes", **gemm_ref_sizes)

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
    detail("resnet18_b1", workload="ResNet-18 v1 conv layers, batch 1, int8 (BASELINE.json configs[3])",
           stack_us=round(r18_us, 1), tops=round(r18_ops / r18_us / 1e6, 2), layers=r18_rows)
    single_rows, _, _ = conv_i8_leg((WL.SINGLE_CONV,), 1, 50, prepared=use_prep)
    detail("single_conv", workload="N=1 C=64 56x56 K=64 3x3 s1 p1 NCHW16c (BASELINE.json configs[0])", **single_rows[0],
           reference_us=24.27, reference_source="cpu-tune.log:160 (x86 VNNI, hardware unstated)")

    # fp16 variant of the ResNet-50 b32 sweep: valid convolution on pre-padded NCHW16c inputs
    f16_rows, f16_us, f16_flops, f16_ref_us = [], 0.0, 0.0, 0.0
    for i, s in enumerate(WL.RESNET50):
        if s.C % 16:
            continue  # the fp16 operator needs C % 16 == 0 (the 3-channel stem has no NCHW16c form)
        f, f_ref = f16_layer(s, use_prep)
        if use_prep:
            f16_ref_us += time_us(f_ref, 20) * s.count
        us = time_us(f, 20)
        flops = 2 * WL.macs(s, BATCH)
        f16_rows.append(dict(layer=s.name, us=round(us, 2), tflops=round(flops / us / 1e6, 1),
                             pct_f16_peak=round(100 * flops / us / 1e6 / PEAK_F16_TFLOPS, 2), kernel=U.last_variant()))
        f16_us += us * s.count
        f16_flops += flops * s.count
        del f, f_ref
    conv_fp16 = dict(workload="ResNet-50 v1 conv layers except the stem, batch 32, fp16 -> fp32 (BASELINE.json configs[4], "
                              "fp16 variant)", stack_us=round(f16_us, 1), tflops=round(f16_flops / f16_us / 1e6, 1),
                     layers=f16_rows)
    if use_prep:
        conv_fp16["reference_layout_weights_stack_us"] = round(f16_ref_us, 1)
    detail("conv_fp16_resnet50_b32", **conv_fp16)
    torch.cuda.empty_cache()

    # layout transforms / pre-packs: bytes read + written over time; operands cycle through cold copies
    x8 = torch.randint(0, 256, (BATCH, 256, 56, 56), dtype=torch.uint8, device=dev)
    layout = {}
    xs = cold_copies((x8,), 2 * x8.numel())
    turn = [0]

    def nxt(seq):
        turn[0] += 1
        return seq[turn[0] % len(seq)][0]
    us = time_us(lambda: U.pack_nchwc(nxt(xs), 16), 30, warm=len(xs))
    layout["pack_nchw16c_u8_32x256x56x56"] = dict(us=round(us, 2), gbs=round(2 * x8.numel() / us / 1e3, 1))
    ps = [(U.pack_nchwc(x[0], 16),) for x in xs]
    us = time_us(lambda: U.unpack_nchwc(nxt(ps)), 30, warm=len(ps))
    layout["unpack_nchw16c_u8_32x256x56x56"] = dict(us=round(us, 2), gbs=round(2 * x8.numel() / us / 1e3, 1))
    del ps, xs
    o32s = [(torch.empty((BATCH, 16, 56, 56, 16), dtype=torch.int32, device=dev),) for _ in range(4)]
    us = time_us(lambda: U.unpack_nchwc(nxt(o32s)), 20, warm=4)
    layout["unpack_nchw16c_i32_32x256x56x56"] = dict(us=round(us, 2), gbs=round(2 * o32s[0][0].numel() * 4 / us / 1e3, 1))
    del o32s
    w33 = torch.randint(-128, 128, (512, 512, 3, 3), dtype=torch.int8, device=dev)
    us = time_us(lambda: U.prepack_conv_weight(w33, 16), 20)
    layout["prepack_conv_weight_512x512x3x3"] = dict(us=round(us, 2), gbs=round(2 * w33.numel() / us / 1e3, 1))
    us = time_us(lambda: U.prepack_dense_weight(w8), 20)
    layout["prepack_dense_weight_4096x4096"] = dict(us=round(us, 2), gbs=round(2 * w8.numel() / us / 1e3, 1))
    # plain device-to-device copy larger than the memory-side cache: what HBM sustains on this box
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    us = time_us(lambda: dst.copy_(src), 5)
    layout["plain_copy_1GiB"] = dict(us=round(us, 2), gbs=round(2 * src.numel() / us / 1e3, 1))
    del src, dst, x8, w33
    torch.cuda.empty_cache()
    detail("layout_kernels", note="bytes read + written over time, operands cycling through more copies than the "
                                  "memory-side cache holds", **layout)

    # register-only MFMA throughput of this box (no memory traffic): what the silicon sustains
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    probe = {}
    # (constant operands, then operands whose bits change from one MFMA to the next: clocks follow
    # power, and the bench data is uniform random)
    # int8: the random operands are uniform bytes, i.e. the int8 GEMM benchmark's own distribution; fp16 has a leg of
    # its own with operands drawn like the fp16 benchmark's (N(0,1)/64 against N(0,1))
    for f16, key, per in ((0, "int8_tops", 65536.0), (1, "fp16_tflops", 32768.0),
                          (2, "int8_tops_random_operands", 65536.0), (3, "fp16_tflops_random_operands", 32768.0),
                          (5, "fp16_tflops_bench_operands", 32768.0)):
        blocks, iters = 2048, 2000
        us = time_us(lambda: _lib.check(L.unit_mfma_peak(f16, blocks, iters, sink.data_ptr(), stream)), 3, warm=8, bursts=3)
        probe[key] = round(blocks * 16 * iters * per / us / 1e6, 1)
    probe["int8_tops_bench_operands"] = probe["int8_tops_random_operands"]
    probe["gemm_int8_frac_of_probe"] = round(gemm_i8["row_major"]["tops"] / probe["int8_tops_bench_operands"], 3)
    probe["gemm_int8_prepared_w_frac_of_probe"] = round(gemm_i8["prepared_weight"]["tops"] / probe["int8_tops_bench_operands"], 3)
    probe["gemm_fp16_frac_of_probe"] = round(gemm_f16["tflops"] / probe["fp16_tflops_bench_operands"], 3)
    probe["gemm_fp16_prepared_b_frac_of_probe"] = round(gemm_f16["prepared_b"]["tflops"] / probe["fp16_tflops_bench_operands"], 3)
    detail("mfma_probe", **probe)

    if args.full:
        fu_rows, fu_us, fu_ops = conv_i8_leg(WL.RESNET50, BATCH, 20, fused=True, prepared=use_prep)
        detail("conv_fused_s8_resnet50_b32",
               workload="ResNet-50 v1 conv stack, batch 32, fused signed form (conv + bias) * scale of "
                        "apps/cpu/relay/result.log:3-26 (s8 x s8 -> i32)",
               stack_us=round(fu_us, 1), tops=round(fu_ops / fu_us / 1e6, 2), layers=fu_rows)
        rq_rows, rq_us, rq_ops = conv_i8_leg(WL.RESNET50, BATCH, 20, requant=True)
        detail("conv_requant_u8_resnet50_b32",
               workload="ResNet-50 v1 conv stack, batch 32, u8 x s8 with the output requantised to u8 NCHW16c "
                        "(clamp(((conv + bias) * scale + half) >> shift, 0, 255)); an extension, not in the reference's graphs",
               stack_us=round(rq_us, 1), tops=round(rq_ops / rq_us / 1e6, 2), layers=rq_rows)

        # The same network as a chain: the 52 convolutions behind the stem, each reading the u8 NCHW16c output of the
        # one before it (projection shortcuts as side branches), buffers owned by the runner, replayed as one HIP graph.
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
        detail("conv_chain_u8_resnet50_b32",
               workload="ResNet-50 v1 behind the stem as a chain: 52 requantising convolutions, batch 32, each reading the "
                        "u8 NCHW16c output of the one before it (projection shortcuts as side branches; residual additions "
                        "are not part of the path); an extension like the requantised output itself",
               hipgraph_us=round(ch_graph, 1), eager_us=round(ch_eager, 1), sum_of_isolated_layers_us=round(ch_iso, 1),
               tops=round(ch_ops / ch_graph / 1e6, 2), min_fraction_of_nonzero_activations=round(ch_alive, 3))
        del ch, ch_replay

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
        detail("conv3d_s8", workload="3-D int8 convolutions of apps/cpu/kernel/conv3d.py:13-25, NCDHW16c / NCDHW4c, s8 x s8 -> i32",
               layers=c3_rows)

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
            # the reference's protocol (apps/cpu/kernel/conv2d.py:61): a warm-up run, then repeat=10 x number=3, mean
            ref = O.c_conv2d_nchwc(ly["data_np"], w_np, s.stride, s.pad, 1, impl="vnni", nthreads=cores)
            t1 = time.perf_counter()
            for _ in range(30):
                O.c_conv2d_nchwc(ly["data_np"], w_np, s.stride, s.pad, 1, impl="vnni", nthreads=cores)
            cpu_s += (time.perf_counter() - t1) / 30 * s.count
            ly["out"].fill_(-1)
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
        if not np.array_equal(c8[:rows].cpu().numpy(), ref) or not torch.equal(c8, c8_pp):
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
        cpu_baseline = dict(value=round(step_ops / cpu_s / 1e12, 3), unit="TOP/s", cores=cores, kind="port",
                            vnni=bool(O.has_vnni()),
                            sample="same step by the AVX-512 VNNI oracle: 20 unique layers, warm-up + repeat=10 x "
                                   "number=3 each, mean x multiplicity",
                            seconds=round(cpu_s, 3),
                            gemm_int8_tops=round(2.0 * rows * N * K / cpu_i8_s / 1e12, 2),
                            gemm_fp16_tflops=round(2.0 * rows * N * K / cpu_f16_s / 1e12, 2))
        detail("cpu_baseline", **cpu_baseline,
               host_vnni_peak_tops=None if vnni_peak is None else round(vnni_peak, 3),
               pct_of_host_vnni_peak=None if not vnni_peak else round(100 * step_ops / cpu_s / 1e12 / vnni_peak, 1),
               gemm_sample=f"{rows} of the 4096 rows of a, mean of 10 runs (apps/cpu/kernel/int8-gemm.py:34); fp16 as a "
                           "torch CPU fp32 matmul of the fp16-rounded operands",
               gemm_int8_rows_bit_exact=rows)

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
        "config": {"workload": "ResNet-50 v1 conv stack (53 convs, 20 shapes), batch 32, int8 u8 x s8 -> i32, "
                               "NCHW16c / NCHW4c stem (BASELINE.json configs[4])",
                   "batch": BATCH, "ops_per_step": step_ops, "weights": args.weights},
        "pct_int8_mfma_peak": round(100 * value / PEAK_INT8_TOPS, 2),
        "bit_exact_vs_oracle": bit_exact,
        "roofline": roofline,
        "roofline_step": roofline_step,
        "cpu_baseline": cpu_baseline,
        "best_mfma_bound_layer": None if best_mfma is None else dict(
            layer=best_mfma["layer"], us=best_mfma["us"], pct_int8_peak=best_mfma["pct_int8_peak"]),
        "gemm_int8_us": gemm_i8["row_major"]["us"],
        "gemm_int8_pct_peak": gemm_i8["row_major"]["pct_int8_peak"],
        "gemm_int8_prepared_w_us": gemm_i8["prepared_weight"]["us"],
        "gemm_int8_prepared_w_pct_peak": gemm_i8["prepared_weight"]["pct_int8_peak"],
        "gemm_fp16_us": gemm_f16["us"],
        "gemm_fp16_tflops": gemm_f16["tflops"],
        "gemm_fp16_pct_peak": gemm_f16["pct_f16_peak"],
        "gemm_fp16_prepared_b_us": gemm_f16["prepared_b"]["us"],
        "gemm_fp16_prepared_b_pct_peak": gemm_f16["prepared_b"]["pct_f16_peak"],
        "gemm_fp16_f16_out_us": gemm_f16["f16_out"]["us"],
        "gemm_fp16_max_rel_err": round(max(err_f, err_fp, err_fh), 6),
        "sum_layers_cold_us": round(sum(ly["us_cold"] * ly["shape"].count for ly in layers), 1),
        "launch": launch_mode,
        "fp16_conv": dict(stack_us=conv_fp16["stack_us"], tflops=conv_fp16["tflops"]),
        "gemm_int8_frac_of_probe": probe["gemm_int8_frac_of_probe"],
        "gemm_fp16_frac_of_probe": probe["gemm_fp16_frac_of_probe"],
        "probe": {k: probe[k] for k in ("int8_tops", "fp16_tflops", "int8_tops_bench_operands", "fp16_tflops_bench_operands")},
    }
    sys.stdout.flush()
    print(compact_line(line), flush=True)


if __name__ == "__main__":
    main()
