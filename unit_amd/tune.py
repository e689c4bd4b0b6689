"""Kernel-variant tuner for the int8 convolution: the counterpart of the reference's tuning loop
(apps/cpu/kernel/conv2d.py:37-83 tries schedule candidates one by one, keeps the fastest and
appends it to cpu-tune.log; python/tensorizer/tune.py:20-31 reads that log back into a table
keyed by (ashape, bshape, strides)).

Here the candidates are the tile variants compiled into libunit_amd.so.  For every layer shape
each variant is run through the C ABI, checked bit for bit against the library's default choice,
and timed with HIP events; the fastest goes into unit_amd/csrc/tuned_conv_{i8,f16}.inc, which the
library's planner consults first (rebuild after tuning).  Needs an MI355X.  With --prepared the
convolutions on prepared weights are tuned (direct variants only) into
tuned_conv_{i8,f16}_prepared.inc.

    python -m unit_amd.tune [--dtype i8|f16] [--prepared] [--nets resnet50:32,resnet18:1] [--iters 20] [--instances 8] [--write]
"""
import argparse
import ctypes
import json
import os
import sys


def _shapes(spec):
    from . import workloads as WL
    nets = {"resnet50": WL.RESNET50, "resnet18": WL.RESNET18, "single": (WL.SINGLE_CONV,)}
    out = []
    for item in spec.split(","):
        name, batch = item.split(":")
        for s in nets[name]:
            out.append((name, int(batch), s))
    return out


def tune(spec, iters=20, verbose=True, dtype="i8", prepared=False, instances=1):
    import torch

    from . import _lib, last_variant
    from . import workloads as WL

    dev = torch.device("cuda:0")
    L = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    num_variants = L.unit_conv_variant_count()

    def time_us(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):  # best of three bursts: one burst next to a clock ramp misleads the choice
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) * 1e3 / iters)
        return best

    saved = {k: os.environ.get(k) for k in ("UNIT_AMD_CONV_VARIANT", "UNIT_AMD_CONV_SPLITK", "UNIT_AMD_CONV_PANEL",
                                             "UNIT_AMD_CONV_NOTABLE")}
    os.environ["UNIT_AMD_CONV_NOTABLE"] = "1"  # "default" below = the heuristic, not an older table
    results = []
    seen = set()
    try:
        for net, batch, s in _shapes(spec):
            cb = WL.channel_block(s.C) if dtype == "i8" else 16
            if s.C % cb and dtype != "i8":
                continue  # the fp16 operator needs C % 16 == 0
            if prepared and ((cb == 16 and dtype == "i8" and s.KH * s.KW > 31) or (cb == 4 and s.KW > 8)):
                continue  # no prepared form
            cp = -(-s.C // cb) * cb
            oh, ow = WL.out_hw(s)
            key = (batch * oh * ow, s.K, cp, s.KH, s.KW, s.stride)
            if key in seen:
                continue
            seen.add(key)
            if dtype == "i8":
                data = torch.randint(0, 256, (batch, cp // cb, s.H, s.W, cb), dtype=torch.uint8, device=dev)
                wt = torch.randint(-128, 128, (s.K // 16, cp // cb, s.KH, s.KW, cb // 4, 16, 4), dtype=torch.int8,
                                   device=dev)
                out = torch.empty((batch, s.K // 16, oh, ow, 16), dtype=torch.int32, device=dev)
                desc = _lib.ConvDesc(batch, cp, s.H, s.W, s.K, s.KH, s.KW, s.stride, s.stride, s.pad, s.pad, s.pad,
                                     s.pad, 1, 1, cb)
                entry = L.unit_conv2d_nchwc_u8s8s32
            else:  # valid convolution on the pre-padded input, integer-valued data: every variant is exact
                hp, wp = s.H + 2 * s.pad, s.W + 2 * s.pad
                data = torch.randint(-3, 4, (batch, cp // 16, hp, wp, 16), device=dev).to(torch.float16)
                wt = torch.randint(-3, 4, (s.K // 16, cp // 16, s.KH, s.KW, 16, 16), device=dev).to(torch.float16)
                out = torch.empty((batch, s.K // 16, oh, ow, 16), dtype=torch.float32, device=dev)
                desc = _lib.ConvDesc(batch, cp, hp, wp, s.K, s.KH, s.KW, s.stride, s.stride, 0, 0, 0, 0, 1, 1, 16)
                entry = L.unit_conv2d_nchw16c_f16f32
                wt_timed = (torch.randn(wt.shape, device=dev) * 0.05).to(torch.float16)  # see the timed copies below
            if prepared:
                from .ops import prepare_conv2d_weight
                if dtype == "f16":
                    wt_timed = prepare_conv2d_weight(wt_timed).buf
                wt = prepare_conv2d_weight(wt).buf
                entry = L.unit_conv2d_nchwc_u8s8s32_prepared if dtype == "i8" else L.unit_conv2d_nchw16c_f16f32_prepared

            # instances > 1: the launches cycle through that many copies of the layer's tensors, so that a launch
            # finds its operands the way a layer of a running network does (last touched many launches ago), not
            # in the caches its own previous launch filled
            if instances < 0:  # as many copies as fill -instances MiB (at most 64): more than the memory-side cache holds
                per = data.numel() * data.element_size() + wt.numel() * wt.element_size() + out.numel() * out.element_size()
                n_inst = max(1, min(64, -(instances * (1 << 20)) // per + 1))
            else:
                n_inst = instances
            if dtype == "f16":
                # copy 0 (integer-valued) is the one checked for exactness; the timed launches run on the other copies,
                # which hold normally distributed values: the clock follows the bit activity of the operands, and on
                # small integers an MFMA-bound layer runs up to a quarter faster than on real activations
                n_inst = max(2, n_inst)
                copies = [(data, wt, out)]
                for _ in range(n_inst - 1):
                    copies.append((torch.randn(data.shape, device=dev).to(torch.float16), wt_timed.clone(),
                                   torch.empty_like(out)))
                first_timed = 1
            else:
                copies = [(data, wt, out)] + [(data.clone(), wt.clone(), torch.empty_like(out)) for _ in range(n_inst - 1)]
                first_timed = 0
            turn = [0]
            timed = [False]

            def call():
                if timed[0]:
                    d_, w_, o_ = copies[first_timed + turn[0] % (n_inst - first_timed)]
                else:
                    d_, w_, o_ = copies[turn[0] % n_inst]
                turn[0] += 1
                return entry(ctypes.byref(desc), d_.data_ptr(), w_.data_ptr(), o_.data_ptr(), stream)

            def timed_us():
                timed[0] = True
                try:
                    return time_us(call)
                finally:
                    timed[0] = False

            os.environ["UNIT_AMD_CONV_VARIANT"] = "0"
            os.environ["UNIT_AMD_CONV_SPLITK"] = "0"
            os.environ["UNIT_AMD_CONV_PANEL"] = "0"
            turn[0] = 0
            _lib.check(call())
            torch.cuda.synchronize()
            ref = out.clone()
            for _ in range(n_inst):  # touch every copy once: the first launch on fresh memory is not what is being compared
                call()
            torch.cuda.synchronize()
            best = (timed_us(), -1, last_variant())
            default_us = best[0]
            timings = {}  # kernel name -> us, every candidate (kept in the --json dump)
            combos = [(1, 0), (1, 1), (1, 2), (1, 4)]  # (k-splits, channel tiles per panel)
            if dtype == "i8" and not prepared:
                combos += [(n, 0) for n in (2, 4, 8, 16, 32)]
            for v in range(num_variants):
                kind = L.unit_conv_variant_is_direct(v)  # 1 direct, 2 LDS-shared (prepared weights, 16-channel blocks), 0 staged
                if prepared and not (kind == 1 or (kind == 2 and cb == 16)):
                    continue
                if not prepared and kind == 2:
                    continue
                for splits, panel in combos:
                    if splits > 1 and (splits // 2) * key[0] * s.K > 256 * 256 * 256:
                        break  # the grid already covers the chip: more k-splits only add atomics
                    os.environ["UNIT_AMD_CONV_VARIANT"] = str(v + 1)
                    os.environ["UNIT_AMD_CONV_SPLITK"] = str(splits)
                    os.environ["UNIT_AMD_CONV_PANEL"] = str(panel)
                    out.fill_(-7)
                    turn[0] = 0  # the checked launch writes `out`
                    if call() != 0:  # variant cannot run this shape (LDS budget)
                        break
                    torch.cuda.synchronize()
                    name = last_variant()
                    if dtype == "i8" and int(name.rsplit("_s", 1)[1]) != splits:
                        break  # clamped to the number of stages: already measured
                    if panel and f"_r{panel}" not in name:
                        continue  # fewer channel tiles than the panel: same as panel 0
                    if not torch.equal(out, ref):
                        raise RuntimeError(f"variant {v} ({name}) disagrees with the default on {s.name}")
                    us = timed_us()
                    timings[name] = round(us, 2)
                    if us < best[0]:
                        best = (us, v, name, splits, panel)
            results.append(dict(net=net, batch=batch, layer=s.name, key=key, variant=best[1], us=best[0],
                                default_us=default_us, kernel=best[2], splits=best[3] if len(best) > 3 else 1,
                                panel=best[4] if len(best) > 4 else 0, timings=timings))
            if verbose:
                print(f"{net:9s} b{batch:<3d} {s.name:22s} default {default_us:7.1f} us  best {best[0]:7.1f} us  {best[2]}",
                      flush=True)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    return results


def write_table(results, path):
    lines = []
    for r in results:
        if r["variant"] < 0:
            continue  # the heuristic's own choice was the fastest
        npix, k, c, kh, kw, sh = r["key"]
        lines.append(f"    {{{npix}, {k}, {c}, {kh}, {kw}, {sh}, {r['variant']}, {r['splits']}, {r['panel']}}},  // {r['net']} b{r['batch']} "
                     f"{r['layer']}: {r['us']:.1f} us ({r['kernel']})\n")
    with open(path, "w") as f:
        f.writelines(lines)
    return len(lines)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--nets", default="resnet50:32,resnet18:1,single:1")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--dtype", default="i8", choices=["i8", "f16"])
    ap.add_argument("--prepared", action="store_true", help="tune the convolutions on prepared weights")
    ap.add_argument("--instances", type=int, default=1,
                    help="cycle the timed launches through this many copies of each layer's tensors (cold operands); "
                         "-M: as many copies as fill M MiB, at most 64")
    ap.add_argument("--write", action="store_true", help="rewrite csrc/tuned_conv_<dtype>[_prepared].inc")
    ap.add_argument("--table", default=None, help="write the table here instead of csrc/tuned_conv_i8.inc")
    ap.add_argument("--json", default=None, help="also dump the raw results here")
    args = ap.parse_args()
    results = tune(args.nets, args.iters, dtype=args.dtype, prepared=args.prepared, instances=args.instances)
    if args.json:
        json.dump(results, open(args.json, "w"), indent=1)
    if args.write or args.table:
        path = args.table or os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc",
                                          f"tuned_conv_{args.dtype}{'_prepared' if args.prepared else ''}.inc")
        n = write_table(results, path)
        print(f"wrote {n} entries to {path}; rebuild with `make -C {os.path.dirname(path)}`")


if __name__ == "__main__":
    sys.exit(main())
