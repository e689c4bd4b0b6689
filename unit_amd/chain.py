"""Layer-chain runner: a network's convolutions back to back with the activations kept in the blocked
u8 layout (N, C/16, H, W, 16) from one layer to the next, the way the reference's compiled graphs keep
NCHW16c between consecutive convolutions after AlterOpLayout (layout_transform only at the graph's
ends: apps/cpu/relay/result.log:7,25).  The layer shapes of its ResNet-50 are the ones logged at
cpu-shapes.log:388-420.

Every layer is the requantising convolution (ops.conv2d_NCHWc_int8_requant): u8 in, u8 out, so a layer's
output is the next layer's input as it lies in memory.  The runner owns all activation buffers and
prepared weights, issues nothing but kernel launches through the C ABI (no allocation per call), and
can therefore be captured into a HIP graph.
"""
import ctypes
from collections import namedtuple

import torch

from . import _lib, ops
from ._lib import ConvDesc, check

# source: index of the layer whose output this layer reads; -1 = the chain's input; None = the layer before
ChainLayer = namedtuple("ChainLayer", "weight bias scale shift stride padding source", defaults=(None,))


class ConvChain:
    """layers: ChainLayer items with `weight` an int8 OIHW tensor (IC, OC multiples of 16) or a
    PreparedConvWeight, `bias` int32 (OC,) or None, integer `scale`, `shift` in 1..62, `stride`, `padding`.
    input_shape: (N, C/16, H, W, 16) of the u8 chain input.

    run(x) launches every layer on the current stream and returns the last layer's output buffer (owned by
    the chain and overwritten by the next run); outputs[i] is layer i's.  graph(x) captures run(x) once and
    returns a callable that replays it (x's storage is the graph's input)."""

    def __init__(self, layers, input_shape):
        if len(input_shape) != 5 or input_shape[4] != 16:
            raise ValueError(f"input_shape: expected (N, C/16, H, W, 16), got {tuple(input_shape)}")
        self.input_shape = tuple(int(v) for v in input_shape)
        self._L = _lib.load()
        self.weights, self.biases, self.descs, self.outputs, self.sources, self.consts = [], [], [], [], [], []
        shapes = []
        for i, ly in enumerate(layers):
            src = i - 1 if ly.source is None else int(ly.source)
            if not -1 <= src < i:
                raise ValueError(f"layer {i}: source {src} is not an earlier layer")
            n, cc, h, w, _ = self.input_shape if src < 0 else shapes[src]
            wt = ly.weight
            if not isinstance(wt, ops.PreparedConvWeight):
                wt = ops._dev(wt, f"layer {i} weight", torch.int8, 4)
                if wt.shape[0] % 16 or wt.shape[1] % 16:
                    raise ValueError(f"layer {i}: OC and IC must be multiples of 16, got {tuple(wt.shape)}")
                wt = ops.prepare_conv2d_weight(ops.prepack_conv_weight(wt, 16))
            if wt.cb != 16 or wt.dtype != torch.int8 or wt.C != cc * 16:
                raise ValueError(f"layer {i}: {wt!r} does not take {cc * 16} channels in 16-channel blocks")
            bias = ly.bias
            if bias is not None:
                if bias.dtype != torch.int32 or bias.numel() != wt.K or bias.device != wt.buf.device:
                    raise ValueError(f"layer {i} bias: expected {wt.K} int32 values on {wt.buf.device}")
                bias = bias.contiguous()
            scale, shift = int(ly.scale), int(ly.shift)
            if not -2 ** 31 <= scale < 2 ** 31 or not 1 <= shift <= 62:
                raise ValueError(f"layer {i}: scale must fit int32 and shift lie in 1..62")
            sh, sw = ops._pair(ly.stride, "stride")
            pt, pl, pb, pr = ops._pad4(ly.padding)
            d = ConvDesc(n, cc * 16, h, w, wt.K, wt.KH, wt.KW, sh, sw, pt, pl, pb, pr, 1, 1, 16)
            oh, ow = ctypes.c_int32(), ctypes.c_int32()
            check(self._L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
            shapes.append((n, wt.K // 16, oh.value, ow.value, 16))
            self.weights.append(wt)
            self.biases.append(bias)
            self.descs.append(d)
            self.sources.append(src)
            self.consts.append((scale, shift))
            self.outputs.append(torch.empty(shapes[-1], dtype=torch.uint8, device=wt.buf.device))
        if not self.outputs:
            raise ValueError("layers: empty chain")
        self.variants = [None] * len(self.outputs)

    def run(self, x):
        x = ops._dev(x, "x", torch.uint8, 5)
        if tuple(x.shape) != self.input_shape:
            raise ValueError(f"x: expected {self.input_shape}, got {tuple(x.shape)}")
        for i in range(len(self.outputs)):
            self.launch_layer(i, x)
        return self.outputs[-1]

    def source_of(self, i, x):
        """The tensor layer i reads: the chain input x or an earlier layer's output buffer."""
        return x if self.sources[i] < 0 else self.outputs[self.sources[i]]

    def launch_layer(self, i, x):
        """Launch layer i alone (its source must hold the data it is to read); returns its output buffer."""
        bias = self.biases[i]
        check(self._L.unit_conv2d_nchwc_u8s8u8_requant_prepared(
            ctypes.byref(self.descs[i]), self.source_of(i, x).data_ptr(), self.weights[i].buf.data_ptr(),
            bias.data_ptr() if bias is not None else None, self.consts[i][0], self.consts[i][1],
            self.outputs[i].data_ptr(), ops._stream()))
        if self.variants[i] is None:
            self.variants[i] = ops.last_variant()
        return self.outputs[i]

    __call__ = run

    def graph(self, x):
        """Capture run(x) into a HIP graph (after one eager run, which also leaves the results in place)."""
        self.run(x)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.run(x)

        def replay():
            g.replay()
            return self.outputs[-1]

        replay.graph = g
        return replay


def resnet50_layers(make_weight, make_bias=None, scale=3, shift=14):
    """The 52 convolutions of ResNet-50 v1 behind the stem and its pooling (cpu-shapes.log:388-420: 16 bottleneck
    blocks in stages of 3, 4, 6, 3; the stride sits on a block's first 1x1) as ChainLayer items.  The main
    path is chained (a block reads the last 1x1 of the block before it); the projection shortcut of a
    stage's first block is a side branch on the block's input.  The element-wise residual additions are not
    part of the convolution path and are left out: a block's output is its last 1x1.

    make_weight(oc, ic, k) -> int8 OIHW tensor (or PreparedConvWeight); make_bias(oc) -> int32 tensor or None.
    Input of the chain: (N, 4, 56, 56, 16) u8 (64 channels)."""
    layers = []
    block_in, c_in = -1, 64

    def add(oc, ic, k, stride, pad, source):
        layers.append(ChainLayer(make_weight(oc, ic, k), make_bias(oc) if make_bias else None, scale, shift, stride, pad,
                                 source))
        return len(layers) - 1

    for stage, (mid, blocks) in enumerate(((64, 3), (128, 4), (256, 6), (512, 3))):
        for b in range(blocks):
            stride = 2 if (b == 0 and stage > 0) else 1
            a = add(mid, c_in, 1, stride, 0, block_in)
            a = add(mid, mid, 3, 1, 1, a)
            last = add(4 * mid, mid, 1, 1, 0, a)
            if b == 0:
                add(4 * mid, c_in, 1, stride, 0, block_in)  # projection shortcut
            block_in, c_in = last, 4 * mid
    return layers


def resnet18_layers(make_weight, make_bias=None, scale=3, shift=14):
    """The 19 convolutions of ResNet-18 v1 behind the stem and its pooling (cpu-shapes.log:368-386: 8 basic blocks of
    two 3x3 convolutions in stages of 2, 2, 2, 2; a stage's first block has stride 2 on its first 3x3 and a 1x1
    stride-2 projection shortcut, taken here as a side branch on the block's input).  Residual additions are
    left out as in resnet50_layers.  Input of the chain: (N, 4, 56, 56, 16) u8 (64 channels)."""
    layers = []
    block_in, c_in = -1, 64

    def add(oc, ic, k, stride, pad, source):
        layers.append(ChainLayer(make_weight(oc, ic, k), make_bias(oc) if make_bias else None, scale, shift, stride, pad,
                                 source))
        return len(layers) - 1

    for stage, width in enumerate((64, 128, 256, 512)):
        for b in range(2):
            stride = 2 if (b == 0 and stage > 0) else 1
            a = add(width, c_in, 3, stride, 1, block_in)
            last = add(width, width, 3, 1, 1, a)
            if stride == 2:
                add(width, c_in, 1, 2, 0, block_in)  # projection shortcut
            block_in, c_in = last, width
    return layers
