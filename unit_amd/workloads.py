"""Layer-shape lists for the benchmark / parity sweeps.

The shapes are the conv2d workloads the reference logs for its quantized ResNets
(cpu-shapes.log:368-386 for resnet18_v1, :388-420 for resnet50_v1; the log holds the
already-padded input extents, e.g. 58x58 for a 56x56 pad-1 layer).  `count` is how often the
layer occurs in the network (stage depths [2,2,2,2] / [3,4,6,3]); the log itself de-duplicates
repeated shapes.  v1 networks put the stride on the first 1x1 of a bottleneck.
"""
from collections import namedtuple

ConvShape = namedtuple("ConvShape", "name C H W K KH KW stride pad count")


def _c(name, c, hw, k, ks, stride, pad, count):
    return ConvShape(name, c, hw, hw, k, ks, ks, stride, pad, count)


# 11 unique conv shapes, batch 1 in the reference
RESNET18 = (
    _c("stem7x7s2_3_64@224", 3, 224, 64, 7, 2, 3, 1),
    _c("3x3_64_64@56", 64, 56, 64, 3, 1, 1, 4),
    _c("3x3s2_64_128@56", 64, 56, 128, 3, 2, 1, 1),
    _c("1x1s2_64_128@56", 64, 56, 128, 1, 2, 0, 1),
    _c("3x3_128_128@28", 128, 28, 128, 3, 1, 1, 3),
    _c("3x3s2_128_256@28", 128, 28, 256, 3, 2, 1, 1),
    _c("1x1s2_128_256@28", 128, 28, 256, 1, 2, 0, 1),
    _c("3x3_256_256@14", 256, 14, 256, 3, 1, 1, 3),
    _c("3x3s2_256_512@14", 256, 14, 512, 3, 2, 1, 1),
    _c("1x1s2_256_512@14", 256, 14, 512, 1, 2, 0, 1),
    _c("3x3_512_512@7", 512, 7, 512, 3, 1, 1, 3),
)

# 20 unique conv shapes (53 convolutions)
RESNET50 = (
    _c("stem7x7s2_3_64@224", 3, 224, 64, 7, 2, 3, 1),
    _c("1x1_64_64@56", 64, 56, 64, 1, 1, 0, 1),
    _c("3x3_64_64@56", 64, 56, 64, 3, 1, 1, 3),
    _c("1x1_64_256@56", 64, 56, 256, 1, 1, 0, 4),
    _c("1x1_256_64@56", 256, 56, 64, 1, 1, 0, 2),
    _c("1x1s2_256_128@56", 256, 56, 128, 1, 2, 0, 1),
    _c("1x1s2_256_512@56", 256, 56, 512, 1, 2, 0, 1),
    _c("3x3_128_128@28", 128, 28, 128, 3, 1, 1, 4),
    _c("1x1_128_512@28", 128, 28, 512, 1, 1, 0, 4),
    _c("1x1_512_128@28", 512, 28, 128, 1, 1, 0, 3),
    _c("1x1s2_512_256@28", 512, 28, 256, 1, 2, 0, 1),
    _c("1x1s2_512_1024@28", 512, 28, 1024, 1, 2, 0, 1),
    _c("3x3_256_256@14", 256, 14, 256, 3, 1, 1, 6),
    _c("1x1_256_1024@14", 256, 14, 1024, 1, 1, 0, 6),
    _c("1x1_1024_256@14", 1024, 14, 256, 1, 1, 0, 5),
    _c("1x1s2_1024_512@14", 1024, 14, 512, 1, 2, 0, 1),
    _c("1x1s2_1024_2048@14", 1024, 14, 2048, 1, 2, 0, 1),
    _c("3x3_512_512@7", 512, 7, 512, 3, 1, 1, 3),
    _c("1x1_512_2048@7", 512, 7, 2048, 1, 1, 0, 3),
    _c("1x1_2048_512@7", 2048, 7, 512, 1, 1, 0, 2),
)

# the reference's single-conv case (cpu-tune.log:160): N=1, C=64, 56x56, K=64, 3x3, s1, p1
SINGLE_CONV = _c("3x3_64_64@56", 64, 56, 64, 3, 1, 1, 1)


def channel_block(c):
    """Input-channel block the reference picks: 16 when the (x4-padded) channel count is a
    multiple of 16, else 4 (apps/cpu/kernel/conv2d.py:18-30)."""
    c4 = -(-c // 4) * 4
    return 16 if c4 % 16 == 0 else 4


def out_hw(s):
    return ((s.H + 2 * s.pad - s.KH) // s.stride + 1, (s.W + 2 * s.pad - s.KW) // s.stride + 1)


def macs(s, batch, logical=True):
    """Multiply-accumulates of one layer; `logical` counts the unpadded channel count (3 for the
    stem), otherwise the executed one (4)."""
    oh, ow = out_hw(s)
    c = s.C if logical else -(-s.C // channel_block(s.C)) * channel_block(s.C)
    return batch * oh * ow * s.K * c * s.KH * s.KW


def algorithmic_bytes(s, batch, in_size=1, w_size=1, out_size=4):
    """Unpadded input + packed weights + output, each touched once."""
    oh, ow = out_hw(s)
    return batch * s.C * s.H * s.W * in_size + s.K * s.C * s.KH * s.KW * w_size + batch * s.K * oh * ow * out_size
