"""Operator entry points of the tensorized conv2d / dense / GEMM path, on torch tensors that live
on the MI355X.  Same names, argument order and argument meaning as the reference operators they
replace; every one hands raw device pointers to the C ABI in libunit_amd.so (hand-written gfx950
kernels).  torch is used to allocate the result and to read shapes / pointers, nothing else.

Reference call sites:
  conv2d_NCHWc_int8        apps/cpu/kernel/conv2d.py:50-51   (topi.nn.conv2d_NCHWc_int8)
  dense_dotprod            apps/cpu/kernel/int8-gemm.py:13-16 (topi.x86.dense_dotprod)
  dense                    apps/cpu/relay/int8-gemm.py:14-16  (relay.nn.dense)
  conv2d_NCHW16c_OHWI16o   python/tensorizer/ops/gpu.py:8-53  (_conv2d_NCHW16c_OHWI16o_impl)
  gemm_fp16                apps/gpu/gemm.py:8-20
"""
import ctypes
import re

import torch

from . import _lib
from ._lib import ConvDesc, check

__all__ = [
    "conv2d_NCHWc_int8", "dense_dotprod", "dense", "conv2d_NCHW16c_OHWI16o", "gemm_fp16", "gemm_fp16_workspace_bytes",
    "pack_nchwc", "unpack_nchwc", "prepack_conv_weight", "prepack_dense_weight", "prepare_dense_weight", "PreparedDenseWeight",
    "prepack_conv_weight_f16", "conv_out_hw", "last_variant",
    "PreparedConvWeight", "prepare_conv2d_weight", "PreparedGemmB", "prepare_gemm_b",
    "conv2d_NCHWc_int8_requant",
]


# ------------------------------------------------------------------------------- helpers
def _stream():
    return torch.cuda.current_stream().cuda_stream


def _dev(t, name, dtype=None, ndim=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise ValueError(f"{name}: tensor must live on the GPU (there is no CPU implementation)")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() not in (ndim if isinstance(ndim, tuple) else (ndim,)):
        raise ValueError(f"{name}: expected {ndim}-D tensor, got shape {tuple(t.shape)}")
    return t if t.is_contiguous() else t.contiguous()


def _pair(v, name):
    if isinstance(v, int):
        return v, v
    v = tuple(int(x) for x in v)
    if len(v) != 2:
        raise ValueError(f"{name}: expected an int or a pair, got {v}")
    return v


def _pad4(padding):
    """TVM's get_pad_tuple: int -> all sides; (ph, pw) -> symmetric; (pt, pl, pb, pr)."""
    if isinstance(padding, int):
        return padding, padding, padding, padding
    p = tuple(int(x) for x in padding)
    if len(p) == 2:
        return p[0], p[1], p[0], p[1]
    if len(p) == 4:
        return p
    raise ValueError(f"padding: expected an int, (ph, pw) or (pt, pl, pb, pr), got {p}")


def _layout_block(layout, name):
    m = re.fullmatch(r"NCHW(\d+)c", layout)
    if not m:
        raise ValueError(f"{name}: expected a layout of the form NCHW<x>c, got {layout!r}")
    return int(m.group(1))


def conv_out_hw(h, w, kh, kw, stride, padding=0, dilation=1):
    """Output height / width of a convolution, as the library computes it."""
    sh, sw = _pair(stride, "stride")
    dh, dw = _pair(dilation, "dilation")
    pt, pl, pb, pr = _pad4(padding)
    d = ConvDesc(1, 16, h, w, 16, kh, kw, sh, sw, pt, pl, pb, pr, dh, dw, 16)
    import ctypes
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    check(_lib.load().unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
    return oh.value, ow.value


def last_variant():
    """Kernel variant chosen by the last compute call (the analogue of the tuned-schedule index
    the reference records per shape, python/tensorizer/tune.py:20-31)."""
    return _lib.last_variant()


# ------------------------------------------------------------------------------- prepared weights
class PreparedConvWeight:
    """Convolution weights in the MFMA fragment order of the kernels (see prepare_conv2d_weight).
    Accepted wherever conv2d_NCHWc_int8, conv2d_NCHWc_int8_fused and conv2d_NCHW16c_OHWI16o take
    a kernel."""

    def __init__(self, buf, K, C, KH, KW, cb, dtype):
        self.buf, self.K, self.C, self.KH, self.KW, self.cb, self.dtype = buf, K, C, KH, KW, cb, dtype

    def __repr__(self):
        return (f"PreparedConvWeight(K={self.K}, C={self.C}, KH={self.KH}, KW={self.KW}, cb={self.cb}, "
                f"dtype={self.dtype})")


def prepare_conv2d_weight(kernel):
    """Re-order a blocked convolution weight once for the direct kernels: the counterpart of the
    constant sub-graphs the reference's compiled models keep next to each convolution (weight
    layout chain apps/cpu/relay/result.log:8-13, sum(w) result.log:15-16).

    kernel int8 (K/16, C/16, KH, KW, 4, 16, 4), int8 (K/16, C/4, KH, KW, 1, 16, 4) with KW <= 8 (the stem's
           4-channel blocks), or fp16 (K/16, C/16, KH, KW, 16 in, 16 out)
    returns a PreparedConvWeight; convolutions on it give the same results as on `kernel`.
    """
    import ctypes
    if isinstance(kernel, torch.Tensor) and kernel.dtype == torch.float16:
        kernel = _dev(kernel, "kernel", torch.float16, 6)
        ko, cc, kh, kw, ic, ob = kernel.shape
        if (ic, ob) != (16, 16):
            raise ValueError(f"kernel: expected (K/16, C/16, KH, KW, 16, 16), got {tuple(kernel.shape)}")
        eb, cb = 2, 16
    else:
        kernel = _dev(kernel, "kernel", torch.int8, 7)
        ko, cc, kh, kw, e, kb, i4 = kernel.shape
        if e not in (1, 4) or (kb, i4) != (16, 4):
            raise ValueError(f"kernel: expected (K/16, C/cb, KH, KW, cb/4, 16, 4) with cb 16 or 4, got {tuple(kernel.shape)}")
        eb, cb = 1, 4 * e
    L = _lib.load()
    nbytes = ctypes.c_size_t()
    check(L.unit_conv2d_prepared_weight_bytes(ko * 16, cc * cb, kh, kw, cb, eb, ctypes.byref(nbytes)))
    buf = torch.empty(nbytes.value, dtype=torch.uint8, device=kernel.device)
    check(L.unit_conv2d_prepare_weight(ko * 16, cc * cb, kh, kw, cb, eb, kernel.data_ptr(), buf.data_ptr(), _stream()))
    return PreparedConvWeight(buf, ko * 16, cc * cb, kh, kw, cb, kernel.dtype)


def _prepared_dims(kernel, data, want_dtype):
    """(K/16, C/16, KH, KW) of a PreparedConvWeight after checking it against the data tensor."""
    n, cc, h, w, cb = data.shape
    if kernel.dtype != want_dtype:
        raise TypeError(f"kernel: prepared from {kernel.dtype}, this operator takes {want_dtype}")
    if cb != kernel.cb or kernel.C != cc * cb:
        raise ValueError(f"kernel: {kernel!r} does not match data {tuple(data.shape)}")
    if kernel.buf.device != data.device:
        raise ValueError("kernel: prepared on another device")
    return kernel.K // 16, cc, kernel.KH, kernel.KW


# ------------------------------------------------------------------------------- int8
def conv2d_NCHWc_int8(data, kernel, stride, padding, dilation=1, out_dtype="int32", layout="NCHW16c",
                      out_layout="NCHW16c"):
    """u8 x s8 -> i32 convolution on blocked layouts.

    data   uint8 (N, C/cb, H, W, cb), cb in {16, 4}
    kernel int8  (K/16, C/cb, KH, KW, cb/4, 16, 4)
    returns int32 (N, K/16, OH, OW, 16)

    As in TVM the channel block is taken from the tensor shapes; `layout` / `out_layout` are
    checked for form only (the reference's driver passes 'NCHW4c' for 16-channel blocks too).
    """
    import ctypes
    data = _dev(data, "data", torch.uint8, 5)
    prepared = isinstance(kernel, PreparedConvWeight)
    if not prepared:
        kernel = _dev(kernel, "kernel", torch.int8, 7)
    if out_dtype != "int32":
        raise ValueError(f"out_dtype: only 'int32' is supported, got {out_dtype!r}")
    _layout_block(layout, "layout")
    if _layout_block(out_layout, "out_layout") != 16:
        raise ValueError("out_layout: the output channel block is 16 (NCHW16c)")
    n, cc, h, w, cb = data.shape
    if cb not in (4, 16):
        raise ValueError(f"data: channel block must be 16 or 4, got {cb}")
    if prepared:
        ko, cc2, kh, kw = _prepared_dims(kernel, data, torch.int8)
    else:
        ko, cc2, kh, kw, e, kb, i4 = kernel.shape
        if (cc2, e, kb, i4) != (cc, cb // 4, 16, 4):
            raise ValueError(f"kernel: shape {tuple(kernel.shape)} does not match data {tuple(data.shape)}; "
                             f"expected (K/16, {cc}, KH, KW, {cb // 4}, 16, 4)")
    sh, sw = _pair(stride, "stride")
    dh, dw = _pair(dilation, "dilation")
    pt, pl, pb, pr = _pad4(padding)
    d = ConvDesc(n, cc * cb, h, w, ko * 16, kh, kw, sh, sw, pt, pl, pb, pr, dh, dw, cb)
    L = _lib.load()
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    check(L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
    out = torch.empty((n, ko, oh.value, ow.value, 16), dtype=torch.int32, device=data.device)
    if prepared:
        check(L.unit_conv2d_nchwc_u8s8s32_prepared(ctypes.byref(d), data.data_ptr(), kernel.buf.data_ptr(),
                                                   out.data_ptr(), _stream()))
    else:
        check(L.unit_conv2d_nchwc_u8s8s32(ctypes.byref(d), data.data_ptr(), kernel.data_ptr(), out.data_ptr(),
                                          _stream()))
    return out


def conv2d_NCHWc_int8_fused(data, kernel, bias, scale, stride, padding, dilation=1, out_dtype="int32",
                            layout="NCHW16c", out_layout="NCHW16c", out_channels=None):
    """The quantized model form of the convolution,
    fused_nn_contrib_conv2d_NCHWc_subtract_add_multiply (apps/cpu/relay/result.log:3-26,35):

        out = (conv2d_NCHWc_int8(data + 128, kernel) - 128 * sum(kernel per out channel) + bias) * scale

    on signed activations, in int32.

    data   int8  (N, C/cb, H, W, cb), cb in {16, 4}
    kernel int8  (K/16, C/cb, KH, KW, cb/4, 16, 4)
    bias   int32 (K,) / any shape with K elements, or None
    scale  Python int
    returns int32 (N, K/16, OH, OW, 16)

    out_layout='NCHW' (prepared weights only) folds the graph's closing layout_transform
    (result.log:25) into the store: returns int32 (N, out_channels, OH, OW), out_channels
    (default K) being the channel count before the caller padded it up to a multiple of 16.
    """
    import ctypes
    data = _dev(data, "data", torch.int8, 5)
    prepared = isinstance(kernel, PreparedConvWeight)
    if not prepared:
        kernel = _dev(kernel, "kernel", torch.int8, 7)
    if out_dtype != "int32":
        raise ValueError(f"out_dtype: only 'int32' is supported, got {out_dtype!r}")
    _layout_block(layout, "layout")
    planar = out_layout == "NCHW"
    if planar and not prepared:
        raise ValueError("out_layout: 'NCHW' needs prepared weights (prepare_conv2d_weight)")
    if not planar and out_channels is not None:
        raise ValueError("out_channels: only with out_layout='NCHW'")
    if not planar and _layout_block(out_layout, "out_layout") != 16:
        raise ValueError("out_layout: the output channel block is 16 (NCHW16c), or 'NCHW'")
    n, cc, h, w, cb = data.shape
    if cb not in (4, 16):
        raise ValueError(f"data: channel block must be 16 or 4, got {cb}")
    if prepared:
        ko, cc2, kh, kw = _prepared_dims(kernel, data, torch.int8)
    else:
        ko, cc2, kh, kw, e, kb, i4 = kernel.shape
        if (cc2, e, kb, i4) != (cc, cb // 4, 16, 4):
            raise ValueError(f"kernel: shape {tuple(kernel.shape)} does not match data {tuple(data.shape)}; "
                             f"expected (K/16, {cc}, KH, KW, {cb // 4}, 16, 4)")
    if bias is not None:
        if bias.dtype != torch.int32 or bias.numel() != ko * 16 or bias.device != data.device:
            raise ValueError(f"bias: expected {ko * 16} int32 values on {data.device}")
        bias = bias.contiguous()
    scale = int(scale)
    if not -2 ** 31 <= scale < 2 ** 31:
        raise ValueError("scale: must fit int32")
    sh, sw = _pair(stride, "stride")
    dh, dw = _pair(dilation, "dilation")
    pt, pl, pb, pr = _pad4(padding)
    d = ConvDesc(n, cc * cb, h, w, ko * 16, kh, kw, sh, sw, pt, pl, pb, pr, dh, dw, cb)
    L = _lib.load()
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    check(L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
    if planar:
        oc = ko * 16 if out_channels is None else int(out_channels)
        if not ko * 16 - 16 < oc <= ko * 16:
            raise ValueError(f"out_channels: {oc} does not round up to K = {ko * 16}")
        out = torch.empty((n, oc, oh.value, ow.value), dtype=torch.int32, device=data.device)
        check(L.unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw(
            ctypes.byref(d), data.data_ptr(), kernel.buf.data_ptr(), bias.data_ptr() if bias is not None else None,
            scale, out.data_ptr(), oc, _stream()))
        return out
    out = torch.empty((n, ko, oh.value, ow.value, 16), dtype=torch.int32, device=data.device)
    fn = L.unit_conv2d_nchwc_s8s8s32_fused_prepared if prepared else L.unit_conv2d_nchwc_s8s8s32_fused
    check(fn(ctypes.byref(d), data.data_ptr(), kernel.buf.data_ptr() if prepared else kernel.data_ptr(),
             bias.data_ptr() if bias is not None else None, scale, out.data_ptr(), _stream()))
    return out


def conv2d_NCHWc_int8_requant(data, kernel, bias, scale, shift, stride, padding, dilation=1):
    """u8 x s8 convolution whose output is requantised to u8 in the blocked layout the next
    convolution reads (four times less output traffic than int32):

        q = clamp(((conv(data, kernel)[k] + bias[k]) * scale + 2**(shift - 1)) >> shift, 0, 255)

    data   uint8 (N, C/cb, H, W, cb)
    kernel a PreparedConvWeight (prepare_conv2d_weight), or the blocked int8 kernel (prepared here)
    bias   int32 (K,) or None;  scale int32;  shift 1..62
    returns uint8 (N, K/16, OH, OW, 16)

    The reference's graphs stop at the int32 subtract / add / multiply
    (apps/cpu/relay/result.log:15-24); this is the integer requantisation that follows it in a
    quantised network.
    """
    import ctypes
    data = _dev(data, "data", torch.uint8, 5)
    if not isinstance(kernel, PreparedConvWeight):
        kernel = prepare_conv2d_weight(kernel)
    n, cc, h, w, cb = data.shape
    ko, _, kh, kw = _prepared_dims(kernel, data, torch.int8)
    if bias is not None:
        if bias.dtype != torch.int32 or bias.numel() != ko * 16 or bias.device != data.device:
            raise ValueError(f"bias: expected {ko * 16} int32 values on {data.device}")
        bias = bias.contiguous()
    scale, shift = int(scale), int(shift)
    if not -2 ** 31 <= scale < 2 ** 31:
        raise ValueError("scale: must fit int32")
    sh, sw = _pair(stride, "stride")
    dh, dw = _pair(dilation, "dilation")
    pt, pl, pb, pr = _pad4(padding)
    d = ConvDesc(n, cc * cb, h, w, ko * 16, kh, kw, sh, sw, pt, pl, pb, pr, dh, dw, cb)
    L = _lib.load()
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    check(L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
    out = torch.empty((n, ko, oh.value, ow.value, 16), dtype=torch.uint8, device=data.device)
    check(L.unit_conv2d_nchwc_u8s8u8_requant_prepared(ctypes.byref(d), data.data_ptr(), kernel.buf.data_ptr(),
                                                      bias.data_ptr() if bias is not None else None, scale, shift,
                                                      out.data_ptr(), _stream()))
    return out


def conv3d_NCDHWc_int8(data, kernel, stride=1):
    """The 3-D blocked convolution of apps/cpu/kernel/conv3d.py:39-64: valid, one stride for depth,
    height and width, int8 x int8 -> int32 (its te.compute casts both placeholders from int8).

    data   int8  (N, C/cb, D, H, W, cb), cb = 16, or 4 with KW <= 8 (the file's 3 -> 4 channel workload)
    kernel int8  (K/16, C/cb, KD, KH, KW, cb/4, 16, 4)
    returns int32 (N, K/16, OD, OH, OW, 16)
    """
    import ctypes
    data = _dev(data, "data", torch.int8, 6)
    kernel = _dev(kernel, "kernel", torch.int8, 8)
    n, cc, dd, h, w, cb = data.shape
    ko, cc2, kd, kh, kw, e, kb, i4 = kernel.shape
    if cb not in (4, 16) or (cb == 4 and (cc * cb) % 16 == 0):
        raise ValueError(f"data: channel block must be 16, or 4 when C is not a multiple of 16 (got {cb}, C = {cc * cb})")
    if (cc2, e, kb, i4) != (cc, cb // 4, 16, 4):
        raise ValueError(f"kernel: shape {tuple(kernel.shape)} does not match data {tuple(data.shape)}; "
                         f"expected (K/16, {cc}, KD, KH, KW, {cb // 4}, 16, 4)")
    stride = int(stride)
    if stride <= 0 or kd > dd or kh > h or kw > w:
        raise ValueError("stride must be positive and the kernel window must fit the input")
    d = _lib.Conv3dDesc(n, cc * cb, dd, h, w, ko * 16, kd, kh, kw, stride)
    od, oh, ow = (dd - kd) // stride + 1, (h - kh) // stride + 1, (w - kw) // stride + 1
    out = torch.empty((n, ko, od, oh, ow, 16), dtype=torch.int32, device=data.device)
    check(_lib.load().unit_conv3d_ncdhwc_s8s8s32(ctypes.byref(d), data.data_ptr(), kernel.data_ptr(), out.data_ptr(),
                                                  _stream()))
    return out


def dense_dotprod(data, weight, bias=None, out_dtype="int32"):
    """u8 (M, K) x s8 packed (N/128, K/4, 128, 4) -> i32 (M, N) = data . W^T.
    A 2-D weight (N, K) is taken as the un-packed relay.nn.dense operand."""
    data = _dev(data, "data", torch.uint8, 2)
    weight = _dev(weight, "weight", torch.int8, (2, 4))
    if out_dtype != "int32":
        raise ValueError(f"out_dtype: only 'int32' is supported, got {out_dtype!r}")
    m, k = data.shape
    L = _lib.load()
    if weight.dim() == 4:
        nb, kg, t, four = weight.shape
        if (t, four) != (128, 4) or kg * 4 != k:
            raise ValueError(f"weight: expected (N/128, {k // 4}, 128, 4), got {tuple(weight.shape)}")
        n = nb * 128
        out = torch.empty((m, n), dtype=torch.int32, device=data.device)
        check(L.unit_dense_dotprod_u8s8s32(data.data_ptr(), weight.data_ptr(), out.data_ptr(), m, n, k, _stream()))
    else:
        n, k2 = weight.shape
        if k2 != k:
            raise ValueError(f"weight: expected (N, {k}), got {tuple(weight.shape)}")
        out = torch.empty((m, n), dtype=torch.int32, device=data.device)
        check(L.unit_dense_u8s8s32(data.data_ptr(), weight.data_ptr(), out.data_ptr(), m, n, k, _stream()))
    if bias is not None:
        out += _dev(bias, "bias", torch.int32)
    return out


class PreparedDenseWeight:
    """A dense weight (N, K) s8 with its row sums, computed once by `prepare_dense_weight`: the constant part of the
    u8 -> s8 shift, which the reference's compiled graphs fold the same way (apps/cpu/relay/result.log:15-16)."""

    def __init__(self, w, wsum):
        self.w, self.wsum = w, wsum
        self.shape = tuple(w.shape)


def prepare_dense_weight(weight):
    """(N, K) s8 -> PreparedDenseWeight, accepted by `dense`."""
    weight = _dev(weight, "weight", torch.int8, 2)
    n, k = weight.shape
    wsum = torch.empty((n,), dtype=torch.int32, device=weight.device)
    check(_lib.load().unit_dense_prepare_weight(weight.data_ptr(), wsum.data_ptr(), n, k, _stream()))
    return PreparedDenseWeight(weight, wsum)


def dense(data, weight, out_dtype="int32"):
    """relay.nn.dense(x u8 (M, K), w s8 (N, K)) -> i32 (M, N); `weight` may be a PreparedDenseWeight."""
    if isinstance(weight, PreparedDenseWeight):
        data = _dev(data, "data", torch.uint8, 2)
        if out_dtype != "int32":
            raise ValueError(f"out_dtype: only 'int32' is supported, got {out_dtype!r}")
        m, k = data.shape
        n, k2 = weight.shape
        if k2 != k:
            raise ValueError(f"weight: expected (N, {k}), got {weight.shape}")
        out = torch.empty((m, n), dtype=torch.int32, device=data.device)
        check(_lib.load().unit_dense_u8s8s32_prepared(data.data_ptr(), weight.w.data_ptr(), weight.wsum.data_ptr(),
                                                      out.data_ptr(), m, n, k, _stream()))
        return out
    weight = _dev(weight, "weight", torch.int8, 2)
    return dense_dotprod(data, weight, None, out_dtype)


# ------------------------------------------------------------------------------- fp16
class PreparedGemmB:
    """The b operand of gemm_fp16 re-laid once as (N, K) (see prepare_gemm_b)."""

    def __init__(self, bt, K, N):
        self.bt, self.K, self.N = bt, K, N

    def __repr__(self):
        return f"PreparedGemmB(K={self.K}, N={self.N})"


def prepare_gemm_b(b):
    """Re-lay the constant operand b (K, N) of gemm_fp16 once as (N, K), the counterpart of the one-time
    packing of b in apps/gpu/gemm-pack.py:9,17; gemm_fp16 accepts the result in place of b.  A 4-D b is taken
    as that file's packed operand (N/32, K/32, 32, 32)."""
    b = _dev(b, "b", torch.float16, (2, 4))
    if b.dim() == 4:  # already packed as the reference packs it: (N/32, K/32, 32, 32), [y/32][k/32][k%32][y%32]
        nb, kb, k32, n32 = b.shape
        if (k32, n32) != (32, 32):
            raise ValueError(f"b: a packed operand is (N/32, K/32, 32, 32), got {tuple(b.shape)}")
        k, n = kb * 32, nb * 32
        bt = torch.empty((n, k), dtype=torch.float16, device=b.device)
        check(_lib.load().unit_gemm_f16_prepare_b_packed32(b.data_ptr(), bt.data_ptr(), k, n, _stream()))
        return PreparedGemmB(bt, k, n)
    k, n = b.shape
    bt = torch.empty((n, k), dtype=torch.float16, device=b.device)
    check(_lib.load().unit_gemm_f16_prepare_b(b.data_ptr(), bt.data_ptr(), k, n, _stream()))
    return PreparedGemmB(bt, k, n)


def gemm_fp16(a, b, out_dtype="float32", workspace=None):
    """c[x, y] = sum_k f32(a[x, k]) * f32(b[k, y]); a (M, K), b (K, N) fp16 row-major, or b a
    PreparedGemmB, or b packed (N/32, K/32, 32, 32) with b4[y/32][k/32][k%32][y%32] = b[k][y] as
    apps/gpu/gemm-pack.py:9,14-18 takes it (re-laid on every call: prepare it once instead).
    workspace (b (K, N) only): True, or a uint8 tensor of `gemm_fp16_workspace_bytes(M, N, K)` bytes: k-splits keep
    their partial tiles in it and are added in split order (run-to-run identical results, also for float16 output)."""
    a = _dev(a, "a", torch.float16, 2)
    if out_dtype not in ("float32", "float16"):
        raise ValueError(f"out_dtype: expected 'float32' or 'float16', got {out_dtype!r}")
    m, k = a.shape
    half = out_dtype == "float16"
    if isinstance(b, torch.Tensor) and b.dim() == 4:
        b = prepare_gemm_b(b)
    if isinstance(b, PreparedGemmB):
        if b.K != k or b.bt.device != a.device:
            raise ValueError(f"b: {b!r} does not match a {tuple(a.shape)} on {a.device}")
        out = torch.empty((m, b.N), dtype=torch.float16 if half else torch.float32, device=a.device)
        check(_lib.load().unit_gemm_f16_prepared(a.data_ptr(), b.bt.data_ptr(), out.data_ptr(), m, b.N, k, int(half),
                                                 _stream()))
        return out
    b = _dev(b, "b", torch.float16, 2)
    k2, n = b.shape
    if k2 != k:
        raise ValueError(f"b: expected ({k}, N), got {tuple(b.shape)}")
    out = torch.empty((m, n), dtype=torch.float16 if half else torch.float32, device=a.device)
    if workspace is not None and workspace is not False:
        need = gemm_fp16_workspace_bytes(m, n, k)
        if workspace is True:
            workspace = torch.empty((max(need, 16),), dtype=torch.uint8, device=a.device)
        workspace = _dev(workspace, "workspace", torch.uint8)
        check(_lib.load().unit_gemm_f16_ws(a.data_ptr(), b.data_ptr(), out.data_ptr(), m, n, k, int(half),
                                           workspace.data_ptr(), workspace.numel(), _stream()))
        return out
    check(_lib.load().unit_gemm_f16(a.data_ptr(), b.data_ptr(), out.data_ptr(), m, n, k, int(half), _stream()))
    return out


def gemm_fp16_workspace_bytes(m, n, k):
    """Bytes `gemm_fp16(..., workspace=...)` needs for this shape (0: the shape runs without k-splits)."""
    nbytes = ctypes.c_size_t()
    check(_lib.load().unit_gemm_f16_ws_bytes(m, n, k, ctypes.byref(nbytes)))
    return nbytes.value


def conv2d_NCHW16c_OHWI16o(a, b, stride_h, stride_w, out_type="float32"):
    """fp16 valid convolution (no padding argument: callers pre-pad), fp32 accumulate.

    Either a (N, C, H, W) + b (K, C, KH, KW), packed here exactly as the reference operator packs
    them in-op, or a (N, C/16, H, W, 16) + b (K/16, C/16, KH, KW, 16 in, 16 out).
    Returns float32 (N, K/16, OH, OW, 16)."""
    import ctypes
    if out_type != "float32":
        raise ValueError(f"out_type: only 'float32' is supported, got {out_type!r}")
    a = _dev(a, "a", torch.float16, (4, 5))
    if isinstance(b, PreparedConvWeight):
        if a.dim() != 5:
            raise ValueError("a: prepared weights take the blocked (N, C/16, H, W, 16) operand")
        ko, cc, kh, kw = _prepared_dims(b, a, torch.float16)
        n, _, h, w, _ = a.shape
        d = ConvDesc(n, cc * 16, h, w, ko * 16, kh, kw, int(stride_h), int(stride_w), 0, 0, 0, 0, 1, 1, 16)
        L = _lib.load()
        oh, ow = ctypes.c_int32(), ctypes.c_int32()
        check(L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
        out = torch.empty((n, ko, oh.value, ow.value, 16), dtype=torch.float32, device=a.device)
        check(L.unit_conv2d_nchw16c_f16f32_prepared(ctypes.byref(d), a.data_ptr(), b.buf.data_ptr(), out.data_ptr(),
                                                    _stream()))
        return out
    b = _dev(b, "b", torch.float16, (4, 6))
    if a.dim() == 4 and b.dim() == 4:
        if a.shape[1] % 16 or b.shape[0] % 16 or b.shape[1] != a.shape[1]:
            raise ValueError("a, b: channel counts must match and be multiples of 16")
        a = pack_nchwc(a, 16)
        b = prepack_conv_weight_f16(b)
    elif not (a.dim() == 5 and b.dim() == 6):
        raise ValueError("a, b: expected 4-D + 4-D or 5-D + 6-D operands")
    n, cc, h, w, cb = a.shape
    ko, ib, kh, kw, ic, ob = b.shape
    if cb != 16 or ic != 16 or ob != 16 or ib != cc:
        raise ValueError(f"a {tuple(a.shape)} / b {tuple(b.shape)}: expected (N, C/16, H, W, 16) and "
                         f"(K/16, C/16, KH, KW, 16, 16)")
    d = ConvDesc(n, cc * 16, h, w, ko * 16, kh, kw, int(stride_h), int(stride_w), 0, 0, 0, 0, 1, 1, 16)
    L = _lib.load()
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    check(L.unit_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
    out = torch.empty((n, ko, oh.value, ow.value, 16), dtype=torch.float32, device=a.device)
    check(L.unit_conv2d_nchw16c_f16f32(ctypes.byref(d), a.data_ptr(), b.data_ptr(), out.data_ptr(), _stream()))
    return out


# ------------------------------------------------------------------------------- layouts
_ELEM = {torch.uint8: 1, torch.int8: 1, torch.float16: 2, torch.int32: 4, torch.float32: 4}


def _elem(t, name):
    if t.dtype not in _ELEM:
        raise TypeError(f"{name}: unsupported dtype {t.dtype}")
    return _ELEM[t.dtype]


def pack_nchwc(x, cb):
    """layout_transform NCHW -> NCHW{cb}c; channels are zero-padded up to a multiple of cb."""
    x = _dev(x, "x", None, 4)
    n, c, h, w = x.shape
    out = torch.empty((n, -(-c // cb), h, w, cb), dtype=x.dtype, device=x.device)
    check(_lib.load().unit_pack_nchwc(x.data_ptr(), out.data_ptr(), n, c, h, w, cb, _elem(x, "x"), _stream()))
    return out


def unpack_nchwc(x, channels=None):
    """layout_transform NCHW{cb}c -> NCHW, keeping the first `channels` channels."""
    x = _dev(x, "x", None, 5)
    n, cc, h, w, cb = x.shape
    c = cc * cb if channels is None else int(channels)
    if not 0 < c <= cc * cb or -(-c // cb) != cc:
        raise ValueError(f"channels: {c} does not fit {cc} blocks of {cb}")
    out = torch.empty((n, c, h, w), dtype=x.dtype, device=x.device)
    check(_lib.load().unit_unpack_nchwc(x.data_ptr(), out.data_ptr(), n, c, h, w, cb, _elem(x, "x"), _stream()))
    return out


def prepack_conv_weight(w, cb):
    """int8 OIHW -> (ceil(O/16), ceil(I/cb), KH, KW, cb/4, 16, 4), zero-padded."""
    w = _dev(w, "w", torch.int8, 4)
    o, i, kh, kw = w.shape
    if cb not in (4, 16):
        raise ValueError(f"cb: must be 16 or 4, got {cb}")
    out = torch.empty((-(-o // 16), -(-i // cb), kh, kw, cb // 4, 16, 4), dtype=torch.int8, device=w.device)
    check(_lib.load().unit_prepack_conv_weight_s8(w.data_ptr(), out.data_ptr(), o, i, kh, kw, cb, _stream()))
    return out


def prepack_dense_weight(w):
    """int8 (N, K) -> (N/128, K/4, 128, 4)."""
    w = _dev(w, "w", torch.int8, 2)
    n, k = w.shape
    if n % 128 or k % 4:
        raise ValueError(f"w: N must be a multiple of 128 and K of 4, got {tuple(w.shape)}")
    out = torch.empty((n // 128, k // 4, 128, 4), dtype=torch.int8, device=w.device)
    check(_lib.load().unit_prepack_dense_weight_s8(w.data_ptr(), out.data_ptr(), n, k, _stream()))
    return out


def prepack_conv_weight_f16(w):
    """fp16 OIHW -> (O/16, I/16, KH, KW, 16 in, 16 out)."""
    w = _dev(w, "w", torch.float16, 4)
    o, i, kh, kw = w.shape
    if o % 16 or i % 16:
        raise ValueError(f"w: O and I must be multiples of 16, got {tuple(w.shape)}")
    out = torch.empty((o // 16, i // 16, kh, kw, 16, 16), dtype=torch.float16, device=w.device)
    check(_lib.load().unit_prepack_conv_weight_f16(w.data_ptr(), out.data_ptr(), o, i, kh, kw, _stream()))
    return out
