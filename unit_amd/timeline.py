"""Wave timelines of the GEMM and direct convolution kernels.

    make -C unit_amd/csrc trace            # libunit_amd_trace.so: the library with stamps compiled in
    python -m unit_amd.timeline gemm_i8_prepared gemm_i8 gemm_f16 gemm_f16_prepared
    python -m unit_amd.timeline 3x3_256_256@14 1x1_64_256@56      # ResNet-50 layers, batch 32, prepared weights

Every wave of an instrumented kernel records s_memrealtime stamps (100 MHz, common to the device) at the points
the kernel names, plus shader-clock tick counts; this tool runs the workload in steady state (sustained
launches first: the clocks of the part follow the load), reads the stamps of the last launch and prints, per
point, the distribution over the waves relative to the first wave's entry.  The GEMM shapes and operand
distributions are those of bench.py (4096^3; u8 / s8 uniform, fp16 N(0,1)/64 against N(0,1)).
UNIT_AMD_TIMELINE_DUMP=<folder> also saves the raw stamps (one row per wave) as <workload>.npy.
"""
import ctypes
import os
import sys

import numpy as np

GEMM_POINTS = ["entry", "ring issued", "stage 0 landed", "last MFMA done", "stores issued", "stores acknowledged"]
CONV_POINTS = ["entry", "arguments fetched", "weight loads issued", "window state built", "pixel loads issued",
               "reduction done", "k-groups summed", "stores acknowledged"]


def _percentiles(v):
    v = np.sort(v)
    return "min %7.2f  p10 %7.2f  median %7.2f  p90 %7.2f  max %7.2f" % (
        v[0], v[len(v) // 10], v[len(v) // 2], v[len(v) * 9 // 10], v[-1])


def main(argv):
    import torch

    from . import _lib
    here = os.path.dirname(os.path.abspath(__file__))
    _lib.LIB_PATH = os.path.join(here, "libunit_amd_trace.so")
    if not os.path.exists(_lib.LIB_PATH):
        sys.exit(f"{_lib.LIB_PATH} is not built: make -C {os.path.join(here, 'csrc')} trace")
    import unit_amd as U
    from . import rng
    from . import workloads as WL
    L = _lib.load()
    L.unit_trace_set.argtypes = [ctypes.c_void_p]
    L.unit_trace_set.restype = None
    words, waves = L.unit_trace_words(), L.unit_trace_waves()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    buf = torch.zeros((waves, words), dtype=torch.int64, device=dev)
    L.unit_trace_set(buf.data_ptr())
    batch = int(os.environ.get("BATCH", "32"))

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def timed(fn, warm, iters=30, bursts=3):
        for _ in range(warm):
            fn()
        seen = []
        for _ in range(bursts):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            e1.synchronize()
            seen.append(e0.elapsed_time(e1) * 1e3 / iters)
        return sorted(seen)[len(seen) // 2]

    for what in argv or ["gemm_i8_prepared"]:
        buf.zero_()
        if what.startswith("gemm"):
            n = 4096
            if what.startswith("gemm_i8"):
                a, w = t(rng.uniform_u8((n, n), 11)), t(rng.uniform_s8((n, n), 12))
                wop = U.prepare_dense_weight(w) if what.endswith("prepared") else w
                fn = lambda: U.dense(a, wop)
                ideal_ticks = (n // 32) * 8 * 32 * 2  # k-steps x 8 MFMAs of a 64 x 128 wave tile x 32 clocks x 2 waves per SIMD
            else:
                a, b = t(rng.normal_f16((n, n), 13, 1.0 / 64)), t(rng.normal_f16((n, n), 14))
                bop = U.prepare_gemm_b(b) if what.endswith("prepared") else b
                fn = lambda: U.gemm_fp16(a, bop)
                ideal_ticks = (2 * n // 32) * 8 * 32 * 2
            us = timed(fn, 400)  # the clocks settle after ~300 sustained launches
            points = GEMM_POINTS
        else:
            match = [s for s in WL.RESNET50 if s.name == what]
            if not match:
                sys.exit(f"unknown workload {what!r}")
            s = match[0]
            cb = WL.channel_block(s.C)  # 4 for the three-channel stem (padded input channels hold zeros)
            cp = -(-s.C // cb) * cb
            data_np = rng.uniform_u8((batch, cp // cb, s.H, s.W, cb), 1)
            if cp != s.C:
                data_np[..., s.C % cb:] = 0
            data = t(data_np)
            wt = U.prepack_conv_weight(t(rng.uniform_s8((s.K, s.C, s.KH, s.KW), 2)), cb)
            prep = U.prepare_conv2d_weight(wt)
            oh, ow = WL.out_hw(s)
            out = torch.empty((batch, s.K // 16, oh, ow, 16), dtype=torch.int32, device=dev)
            desc = _lib.ConvDesc(batch, cp, s.H, s.W, s.K, s.KH, s.KW, s.stride, s.stride, s.pad, s.pad, s.pad, s.pad,
                                 1, 1, cb)
            fn = lambda: _lib.check(L.unit_conv2d_nchwc_u8s8s32_prepared(ctypes.byref(desc), data.data_ptr(),
                                                                         prep.buf.data_ptr(), out.data_ptr(), stream))
            us = timed(fn, 10)
            points, ideal_ticks = CONV_POINTS, 0
        torch.cuda.synchronize()
        h = buf.cpu().numpy().astype(np.uint64)
        h = h[h[:, 0] > 0]
        print(f"{what}: {U.last_variant()}, {us:.2f} us launch to launch (median of 3 bursts of 30), {len(h)} waves traced")
        if len(h) == 0:
            print("   no stamps: this kernel is not instrumented")
            continue
        if os.environ.get("UNIT_AMD_TIMELINE_DUMP"):  # the raw stamps, one row per wave
            os.makedirs(os.environ["UNIT_AMD_TIMELINE_DUMP"], exist_ok=True)
            np.save(os.path.join(os.environ["UNIT_AMD_TIMELINE_DUMP"], what.replace("@", "_at_") + ".npy"), h)
        base = h[:, 0].min()
        last = 0
        for k, name in enumerate(points):
            col = h[:, k]
            col = col[col > 0]
            if len(col) == 0:
                continue
            rel = (col - base).astype(np.float64) * 0.01
            last = max(last, rel.max())
            print(f"   {name:28s} {_percentiles(rel)}")
        print(f"   kernel span (first entry to last stamp) {last:.2f} us")
        if points is GEMM_POINTS:
            loop_us = (h[:, 3] - h[:, 2]).astype(np.float64) * 0.01
            ticks = h[:, 8].astype(np.float64)
            print(f"   reduction loop: {np.median(loop_us):.2f} us = {np.median(ticks):.0f} shader clocks "
                  f"({np.median(ticks / loop_us) / 1e3:.3f} GHz); MFMA pipe busy {100 * ideal_ticks / np.median(ticks):.1f} % of them; "
                  f"waiting for direct loads {100 * np.median(h[:, 9] / ticks):.2f} %, at lgkmcnt + barrier "
                  f"{100 * np.median(h[:, 10] / ticks):.1f} % (min {100 * (h[:, 10] / ticks).min():.1f}, max {100 * (h[:, 10] / ticks).max():.1f})")
            xcc = h[:, 15] & 15
            for x in sorted(set(xcc.tolist())):
                e = (h[xcc == x, 3] - base).astype(np.float64) * 0.01
                print(f"   XCD {x}: {len(e)} waves, last MFMA done min {e.min():.2f} median {np.median(e):.2f} max {e.max():.2f}")
        else:
            ph = [(h[:, k + 1].astype(np.int64) - h[:, k].astype(np.int64)) * 0.01 for k in range(7)]
            names = ["argument fetch", "place + weight loads", "window decode", "tap entries + pixel loads",
                     "tables, barrier, reduction", "k-group sum", "stores"]
            valid = h[:, 6] > 0
            parts = []
            for k, nm in enumerate(names):
                a_, b_ = h[:, k], h[:, k + 1]
                if nm == "k-group sum" and not valid.any():
                    continue
                if nm == "stores" and not valid.any():
                    d = (h[:, 7].astype(np.int64) - h[:, 5].astype(np.int64)) * 0.01
                else:
                    ok = (a_ > 0) & (b_ > 0)
                    if not ok.any():
                        continue
                    d = (b_[ok].astype(np.int64) - a_[ok].astype(np.int64)) * 0.01
                parts.append(f"{nm} {np.median(d):.2f}")
            life = (h[:, 7].astype(np.int64) - h[:, 0].astype(np.int64)) * 0.01
            print(f"   per wave (median us): {', '.join(parts)}; lifetime median {np.median(life):.2f} max {life.max():.2f}")


if __name__ == "__main__":
    main(sys.argv[1:])
