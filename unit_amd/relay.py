"""The reference's Relay-level convolution graph on the GPU, NCHW in and NCHW out.

apps/cpu/relay/conv2d.py:15-27 builds, from ten integers `n c h w oc ic kh kw sh sw`,

    y = (nn.conv2d(x, w, strides=(sh, sw), out_dtype='int32') + b) * 11      x, w int8, b int32

and TVM legalises it to the graph printed at apps/cpu/relay/result.log:3-26 (16-channel blocks)
and :6803-6828 (the 3-channel stem: channels padded to 4, NCHW4c), which runs as seven operators
(result.log:30-36):

    #0 fused_cast_add_cast[_nn_pad]_layout_transform   x + 128 as u8, NCHW -> NCHW{cb}c
    #1 fused_[nn_pad_]transpose_reshape_...            weight OIHW -> OIHW{cb/4}i16o4i
    #2 fused_cast_sum, #3 ..., #4 ...                  128 * sum(w) and the bias as NCHW16c
    #5 fused_nn_contrib_conv2d_NCHWc_subtract_add_multiply
    #6 fused_layout_transform                          NCHW16c -> NCHW

Here #1-#4 depend on constants only and run once, when the graph object is built (weights end up
in the kernels' prepared form, which carries 128 * sum(w)); a call runs #0 as the layout kernel on
the signed data (the +128 shift is the convolution kernel's sign flip of the operand), #5 as the
fused convolution and, by default, #6 inside its store.
"""
import sys

import torch

from . import ops
from .workloads import channel_block


class Conv2dBiasMultiply:
    """(conv2d(x, w, strides, padding) + b) * multiplier with x (N, IC, H, W) int8, w (OC, IC, KH, KW)
    int8, b int32 with OC elements; returns int32 (N, OC, OH, OW).

    The channel block follows the reference's rule (apps/cpu/kernel/conv2d.py:18-30): input channels
    are padded to a multiple of 4 and blocked by 16 if that is a multiple of 16, else by 4; output
    channels are padded to a multiple of 16 and the padding is not written back.
    """

    def __init__(self, weight, bias=None, multiplier=11, strides=1, padding=0, dilation=1):
        weight = ops._dev(weight, "weight", torch.int8, 4)
        self.oc, self.ic, self.kh, self.kw = weight.shape
        self.cb = channel_block(self.ic)
        self.strides, self.padding, self.dilation = strides, padding, dilation
        self.multiplier = int(multiplier)
        blocked = ops.prepack_conv_weight(weight, self.cb)        # Op #1
        self.weight = ops.prepare_conv2d_weight(blocked)          # + Ops #2, #3 (128 * sum(w) behind the fragments)
        self._L = ops._lib.load()
        self._plans = {}
        self.bias = None
        if bias is not None:                                      # Op #4: the bias per padded output channel
            if bias.dtype != torch.int32 or bias.numel() != self.oc or bias.device != weight.device:
                raise ValueError(f"bias: expected {self.oc} int32 values on {weight.device}")
            self.bias = torch.zeros(self.weight.K, dtype=torch.int32, device=weight.device)
            self.bias[:self.oc] = bias.reshape(-1)

    def __call__(self, x, fold_output_transform=True):
        """Run the graph.  The result tensor belongs to the graph object and is overwritten by the next call on an
        input of the same shape (as a graph runtime's output buffers are); clone it to keep it."""
        x = ops._dev(x, "x", torch.int8, 4)
        if x.shape[1] != self.ic:
            raise ValueError(f"x: {x.shape[1]} channels, the weights take {self.ic}")
        if not fold_output_transform:
            data = ops.pack_nchwc(x, self.cb)                     # Op #0
            out = ops.conv2d_NCHWc_int8_fused(data, self.weight, self.bias, self.multiplier, self.strides, self.padding,
                                              self.dilation)      # Op #5
            return ops.unpack_nchwc(out, self.oc)                 # Op #6
        plan = self._plans.get(tuple(x.shape))
        if plan is None:  # buffers and descriptor of this input shape: the per-call path only launches kernels
            import ctypes
            from ._lib import ConvDesc
            n, c, h, w = x.shape
            cp = -(-c // self.cb) * self.cb
            sh, sw = ops._pair(self.strides, "strides")
            dh, dw = ops._pair(self.dilation, "dilation")
            pt, pl, pb, pr = ops._pad4(self.padding)
            desc = ConvDesc(n, cp, h, w, self.weight.K, self.kh, self.kw, sh, sw, pt, pl, pb, pr, dh, dw, self.cb)
            oh, ow = ctypes.c_int32(), ctypes.c_int32()
            ops.check(self._L.unit_conv_out_hw(ctypes.byref(desc), ctypes.byref(oh), ctypes.byref(ow)))
            data = torch.empty((n, cp // self.cb, h, w, self.cb), dtype=torch.int8, device=x.device)
            out = torch.empty((n, self.oc, oh.value, ow.value), dtype=torch.int32, device=x.device)
            plan = self._plans[tuple(x.shape)] = (desc, ctypes.byref(desc), data, out)
        desc, desc_ref, data, out = plan
        stream = ops._stream()
        n, c, h, w = x.shape
        ops.check(self._L.unit_pack_nchwc(x.data_ptr(), data.data_ptr(), n, c, h, w, self.cb, 1, stream))     # Op #0
        ops.check(self._L.unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(                                       # Ops #5 + #6
            desc_ref, data.data_ptr(), self.weight.buf.data_ptr(), self.bias.data_ptr() if self.bias is not None else None,
            self.multiplier, out.data_ptr(), self.oc, stream))
        return out


    def graph(self, x):
        """Capture a run on x into a HIP graph; returns a callable that replays it and returns the result tensor
        (x's storage is the graph's input)."""
        self(x)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            out = self(x)

        def replay():
            g.replay()
            return out

        replay.graph = g
        return replay


def time_evaluator(fn, number=3, repeat=10):
    """Mean seconds per run over `repeat` measurements of `number` back-to-back runs, the protocol of
    the reference's drivers (time_evaluator('run', number=3, repeat=10), apps/cpu/relay/conv2d.py:56)."""
    fn()
    torch.cuda.synchronize()
    total = 0.0
    for _ in range(repeat):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(number):
            fn()
        e1.record()
        torch.cuda.synchronize()
        total += e0.elapsed_time(e1) * 1e-3 / number
    return total / repeat


def main(argv=None):
    """python -m unit_amd.relay N C H W OC IC KH KW SH SW   (or the ten integers on stdin, as the
    reference's driver reads them): builds the graph on random operands drawn as the reference
    draws them (randn * 128 cast to int8 / int32) and prints the mean time of a run in us (two kernel
    launches from Python per run; replaying so short a sequence as a HIP graph measured slower, 35 against 17 us)."""
    import numpy as np
    argv = sys.argv[1:] if argv is None else argv
    fields = argv if argv else sys.stdin.readline().split()
    if len(fields) != 10:
        raise SystemExit("usage: python -m unit_amd.relay N C H W OC IC KH KW SH SW")
    n, c, h, w, oc, ic, kh, kw, sh, sw = map(int, fields)
    if c != ic:
        raise SystemExit(f"C ({c}) and IC ({ic}) differ")
    dev = torch.device("cuda:0")
    w_ = torch.from_numpy((np.random.randn(oc, ic, kh, kw) * 128).astype("int8")).to(dev)
    b_ = torch.from_numpy((np.random.randn(1, oc, 1, 1) * 128).astype("int32")).to(dev)
    x_ = torch.from_numpy((np.random.randn(n, c, h, w) * 128).astype("int8")).to(dev)
    graph = Conv2dBiasMultiply(w_, b_, 11, (sh, sw))
    mean = time_evaluator(lambda: graph(x_))
    print(f"{mean * 1e6:.3f} us per run  ({ops.last_variant()})")
    return 0


if __name__ == "__main__":
    sys.exit(main())
