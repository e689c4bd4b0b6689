"""CPU oracle for the tensorized conv2d / dense / GEMM path -- numpy half + ctypes bindings.

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` -- always as the checker, never as the thing that is
measured or shipped.  The product package must not import this module.

Each function cites the reference file:line it restates (paths relative to the reference
tree).  What pins each function is listed in the header of tests/test_oracle.py.

Parity status:
  * conv2d / stencil / layouts / pre-pack / fp16: pinned (known-answer vector, brute force,
    independent library routine, printed transform chain).
  * dense packed-weight *index order*: pinned at tile 16 by the reference's own literal index
    lambda (poc/vnni/vnni_dense.py:10-11, checked element by element); for the 128-row tile the
    reference gives only the placeholder shape (N/128, K/4, 128, 4) (apps/cpu/kernel/
    int8-gemm.py:14), read here as the same rule with 128 in place of 16 -- that reading stays
    PARITY UNPINNED.  The logical product a . W^T is pinned.
  * fused signed form with spatial padding: PARITY UNPINNED (the reference's printed graphs have
    padding 0; zero padding of the signed data follows upstream TVM).
  * conv2d_nchwc_u8_requant: PARITY UNPINNED -- an extension with no counterpart in the
    reference (its graphs stop at the int32 subtract / add / multiply); the convolution inside is
    the pinned one, the requantisation is checked against exact Python integers.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


# --------------------------------------------------------------------------- RNG
def _splitmix64(x):
    with np.errstate(over="ignore"):
        z = x + _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def random_bytes(n, seed):
    """Byte i = byte (i % 8), little-endian, of splitmix64(seed * GOLDEN + i // 8).

    Same stream as ``oracle_fill_u8`` in unit_oracle.c and ``unit_amd.rng.random_bytes``.
    """
    n = int(n)
    words = (n + 7) // 8
    with np.errstate(over="ignore"):
        base = np.uint64(seed) * _GOLDEN
        ctr = base + np.arange(words, dtype=np.uint64)
    out = _splitmix64(ctr).astype("<u8").view(np.uint8)
    return out[:n].copy()


def fill_u8(shape, seed):
    return random_bytes(int(np.prod(shape)), seed).reshape(shape)


def fill_s8(shape, seed):
    return random_bytes(int(np.prod(shape)), seed).view(np.int8).reshape(shape)


# --------------------------------------------------------------------------- a1 stencil
def vpdpbusd(acc, a, b):
    """python/tensorizer/intrinsics/pattern.py:3-16 with (out_lanes, reduce_lanes) = (16, 4):
    c[x] = acc[x] + sum_{r<4} i32(u8 a[4x+r]) * i32(s8 b[4x+r]), wrapping mod 2^32."""
    a = np.asarray(a, dtype=np.uint8).astype(np.int64).reshape(16, 4)
    b = np.asarray(b, dtype=np.int8).astype(np.int64).reshape(16, 4)
    s = np.asarray(acc, dtype=np.int32).astype(np.int64) + (a * b).sum(axis=1)
    return (s & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


# --------------------------------------------------------------------------- layouts
def pack_nchwc(x, cb):
    """NCHW -> NCHW[cb]c (apps/cpu/relay/result.log:7 layout_transform; in-op form
    python/tensorizer/ops/gpu.py:26-28): A5[n,ci,h,w,c] = A[n, cb*ci+c, h, w]; channels are
    zero-padded up to a multiple of cb (apps/cpu/kernel/conv2d.py:18-22, result.log:6807)."""
    n, c, h, w = x.shape
    cp = -(-c // cb) * cb
    if cp != c:
        x = np.concatenate([x, np.zeros((n, cp - c, h, w), dtype=x.dtype)], axis=1)
    return np.ascontiguousarray(x.reshape(n, cp // cb, cb, h, w).transpose(0, 1, 3, 4, 2))


def unpack_nchwc(x5, channels=None):
    """NCHW[cb]c -> NCHW (apps/cpu/relay/result.log:25), dropping padded channels."""
    n, cc, h, w, cb = x5.shape
    x = x5.transpose(0, 1, 4, 2, 3).reshape(n, cc * cb, h, w)
    if channels is not None:
        x = x[:, :channels]
    return np.ascontiguousarray(x)


def prepack_conv_weight_chain(w, cb):
    """OIHW -> (O/16, I/cb, KH, KW, cb/4, 16, 4) by replaying the transform chain the
    reference prints: apps/cpu/relay/result.log:8-13 (cb=16) and :6809-6815 (cb=4, with the
    nn.pad of the input channels).  O % 16 == 0 required (result.log never pads O)."""
    o, i, kh, kw = w.shape
    ip = -(-i // cb) * cb
    if ip != i:  # %5 = nn.pad(%w, pad_width=[[0,0],[0,1],[0,0],[0,0]])
        w = np.concatenate([w, np.zeros((o, ip - i, kh, kw), dtype=w.dtype)], axis=1)
    t = w.transpose(1, 2, 3, 0)  # %4  (I, KH, KW, O)
    t = t.reshape(ip, kh, kw, o // 16, 16)  # %5
    t = t.transpose(3, 1, 2, 4, 0)  # %6  (O/16, KH, KW, 16, I)
    t = t.reshape(o // 16, kh, kw, 16, ip // cb, cb)  # %7
    t = t.reshape(o // 16, kh, kw, 16, ip // cb, cb // 4, 4)  # %8
    t = t.transpose(0, 4, 1, 2, 5, 3, 6)  # %9  (O/16, I/cb, KH, KW, cb/4, 16, 4)
    return np.ascontiguousarray(t)


def prepack_conv_weight(w, cb):
    """Same result from the one-line index formula
    W7[ko,ci,kh,kw,e,kb,i] = W[16ko+kb, cb*ci+4e+i, kh, kw]; O padded to x16, I to x cb."""
    o, i, kh, kw = w.shape
    op, ip = -(-o // 16) * 16, -(-i // cb) * cb
    wp = np.zeros((op, ip, kh, kw), dtype=w.dtype)
    wp[:o, :i] = w
    t = wp.reshape(op // 16, 16, ip // cb, cb // 4, 4, kh, kw)  # ko kb ci e i kh kw
    return np.ascontiguousarray(t.transpose(0, 2, 5, 6, 3, 1, 4))


def prepack_dense_weight(w, tile=128):
    """(N, K) -> (N/tile, K/4, tile, 4), Wp[n/tile, k/4, n%tile, k%4] = W[n, k]
    (tile 128: shape from apps/cpu/kernel/int8-gemm.py:14; tile 16: the reference's own statement of the order,
    poc/vnni/vnni_dense.py:10-11 `packed[w, x, y, z] = b[w * 16 + y, x * 4 + z]`)."""
    n, k = w.shape
    assert n % tile == 0 and k % 4 == 0
    return np.ascontiguousarray(w.reshape(n // tile, tile, k // 4, 4).transpose(0, 2, 1, 3))


def prepack_conv_weight_f16(w):
    """OIHW -> (O/16, I/16, KH, KW, 16i, 16o) (python/tensorizer/ops/gpu.py:29-31):
    B6[oc,ic,x,y,ib,ob] = B[16oc+ob, 16ic+ib, x, y]."""
    o, i, kh, kw = w.shape
    assert o % 16 == 0 and i % 16 == 0
    t = w.reshape(o // 16, 16, i // 16, 16, kh, kw)  # oc ob ic ib x y
    return np.ascontiguousarray(t.transpose(0, 2, 4, 5, 3, 1))


# --------------------------------------------------------------------------- a2 conv (int8)
def _pad_tuple(padding):
    if isinstance(padding, int):
        return padding, padding, padding, padding
    padding = tuple(int(p) for p in padding)
    if len(padding) == 2:
        return padding[0], padding[1], padding[0], padding[1]
    if len(padding) == 4:
        return padding
    raise ValueError("padding must be an int, (ph, pw) or (pt, pl, pb, pr)")


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


def conv_out_hw(h, w, kh, kw, stride, padding, dilation):
    sh, sw = _pair(stride)
    dh, dw = _pair(dilation)
    pt, pl, pb, pr = _pad_tuple(padding)
    return ((h + pt + pb - dh * (kh - 1) - 1) // sh + 1, (w + pl + pr - dw * (kw - 1) - 1) // sw + 1)


def conv2d_nchwc_int8(data, weight, stride=1, padding=0, dilation=1):
    """apps/cpu/kernel/conv3d.py:60-64 (2-D case) / topi.nn.conv2d_NCHWc_int8 call at
    apps/cpu/kernel/conv2d.py:50-51, in int64 then wrapped to int32:

    O[n,ko,oh,ow,kb] = sum_{ci,kh,kw,e,i} A[n,ci,sh*oh+dh*kh,sw*ow+dw*kw,4e+i] * W[ko,ci,kh,kw,e,kb,i]
    over the zero-padded data."""
    data = np.asarray(data)
    weight = np.asarray(weight)
    assert data.dtype == np.uint8 and weight.dtype == np.int8
    n, cc, h, w, cb = data.shape
    ko, cc2, kh, kw, e, kb, i4 = weight.shape
    assert cc == cc2 and kb == 16 and i4 == 4 and e * 4 == cb
    sh, sw = _pair(stride)
    dh, dw = _pair(dilation)
    pt, pl, pb, pr = _pad_tuple(padding)
    oh, ow = conv_out_hw(h, w, kh, kw, stride, padding, dilation)
    a = np.zeros((n, cc, h + pt + pb, w + pl + pr, cb), dtype=np.int64)
    a[:, :, pt:pt + h, pl:pl + w, :] = data
    wt = weight.astype(np.int64).transpose(0, 5, 1, 2, 3, 4, 6).reshape(ko * 16, cc, kh, kw, cb)
    out = np.zeros((n, ko * 16, oh, ow), dtype=np.int64)
    for y in range(kh):
        for x in range(kw):
            win = a[:, :, y * dh:y * dh + (oh - 1) * sh + 1:sh, x * dw:x * dw + (ow - 1) * sw + 1:sw, :]
            out += np.einsum("nchwi,kci->nkhw", win, wt[:, :, y, x, :], optimize=True)
    out = out.reshape(n, ko, 16, oh, ow).transpose(0, 1, 3, 4, 2)
    return np.ascontiguousarray((out & 0xFFFFFFFF).astype(np.uint32).view(np.int32))


def conv2d_nchwc_int8_loops(data, weight, stride=1, padding=0, dilation=1):
    """The same closed form as seven nested Python loops (tiny shapes only) -- shares no
    vectorised code with conv2d_nchwc_int8, so an index slip in either shows up."""
    n, cc, h, w, cb = data.shape
    ko, _, kh, kw, e, _, _ = weight.shape
    sh, sw = _pair(stride)
    dh, dw = _pair(dilation)
    pt, pl, pb, pr = _pad_tuple(padding)
    oh, ow = conv_out_hw(h, w, kh, kw, stride, padding, dilation)
    out = np.zeros((n, ko, oh, ow, 16), dtype=np.int64)
    for b in range(n):
        for o in range(ko):
            for y in range(oh):
                for x in range(ow):
                    for c in range(cc):
                        for r in range(kh):
                            for s in range(kw):
                                iy, ix = y * sh + r * dh - pt, x * sw + s * dw - pl
                                if iy < 0 or iy >= h or ix < 0 or ix >= w:
                                    continue
                                av = data[b, c, iy, ix].astype(np.int64).reshape(e, 1, 4)
                                out[b, o, y, x] += (av * weight[o, c, r, s].astype(np.int64)).sum(axis=(0, 2))
    return (out & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


def conv2d_nchwc_int8_fused(data_s8, weight, bias, scale, stride=1, padding=0, dilation=1, conv=None):
    """fused_nn_contrib_conv2d_NCHWc_subtract_add_multiply, op by op as the reference prints it
    (apps/cpu/relay/result.log:3-26): x + 128 cast to u8 (:4-6), the u8 x s8 convolution (:14),
    minus 128 * sum of the weights over (in-channel, kh, kw) per out channel (:15-21), plus the bias
    (:22-23), times the scale (:24), in wrapping int32.  The printed graphs carry no spatial padding;
    a padded convolution is taken as upstream TVM legalises it: zero-pad the signed data first,
    then shift, so the correction stays exact at the borders.  `conv` is the u8 convolution to use
    (default: the vectorised numpy restatement)."""
    data_s8 = np.asarray(data_s8)
    weight = np.asarray(weight)
    assert data_s8.dtype == np.int8 and weight.dtype == np.int8
    pt, pl, pb, pr = _pad_tuple(padding)
    xp = np.pad(data_s8, ((0, 0), (0, 0), (pt, pb), (pl, pr), (0, 0)))
    xu = (xp.astype(np.int32) + 128).astype(np.uint8)
    conv = conv or conv2d_nchwc_int8
    acc = conv(xu, weight, stride, 0, dilation).astype(np.int64)             # (N, K/16, OH, OW, 16)
    wsum = weight.astype(np.int64).sum(axis=(1, 2, 3, 4, 6))                  # (K/16, 16)
    out = acc - 128 * wsum[None, :, None, None, :]
    if bias is not None:
        out = out + np.asarray(bias, dtype=np.int64).reshape(1, -1, 1, 1, 16)
    out = out * int(scale)
    return np.ascontiguousarray((out & 0xFFFFFFFF).astype(np.uint32).view(np.int32))


def conv2d_nchwc_u8_requant(data_u8, weight, bias, scale, shift, stride=1, padding=0, dilation=1, conv=None):
    """u8 x s8 convolution with requantised u8 output (no counterpart in the reference's files: its
    graphs stop at the int32 subtract / add / multiply, apps/cpu/relay/result.log:15-24; parity
    unpinned beyond the convolution itself, which is pinned):

        q = clamp(((conv_u8(x, w)[k] + bias[k]) * scale + 2**(shift - 1)) >> shift, 0, 255)

    conv + bias in wrapping int32, product and arithmetic shift in 64 bits.  Output u8
    (N, K/16, OH, OW, 16)."""
    conv = conv or conv2d_nchwc_int8
    acc = conv(np.asarray(data_u8), np.asarray(weight), stride, padding, dilation).astype(np.int64)
    if bias is not None:
        acc = acc + np.asarray(bias, dtype=np.int64).reshape(1, -1, 1, 1, 16)
    acc = (acc & 0xFFFFFFFF).astype(np.uint32).view(np.int32).astype(np.int64)   # the int32 the device holds
    assert 1 <= int(shift) <= 62
    t = (acc * int(scale) + (1 << (int(shift) - 1))) >> int(shift)
    return np.ascontiguousarray(np.clip(t, 0, 255).astype(np.uint8))


def conv3d_ncdhwc_int8(data, weight, stride=1):
    """apps/cpu/kernel/conv3d.py:39-64, the reference's own te.compute: valid 3-D convolution, one
    stride, both operands int8 cast to int32:

    O[n,ko,x,y,z,kb] = sum_{rco,rd,rh,rw,rcm,rci} A[n,rco,s*x+rd,s*y+rh,s*z+rw,4*rcm+rci] * B[ko,rco,rd,rh,rw,rcm,kb,rci]
    """
    data = np.asarray(data)
    weight = np.asarray(weight)
    assert data.dtype == np.int8 and weight.dtype == np.int8
    n, cc, dd, h, w, cb = data.shape
    ko, cc2, kd, kh, kw, e, kb, i4 = weight.shape
    assert cc == cc2 and kb == 16 and i4 == 4 and e * 4 == cb
    s = int(stride)
    od, oh, ow = (dd - kd) // s + 1, (h - kh) // s + 1, (w - kw) // s + 1
    a = data.astype(np.int64)
    wt = weight.astype(np.int64).transpose(0, 6, 1, 2, 3, 4, 5, 7).reshape(ko * 16, cc, kd, kh, kw, cb)
    out = np.zeros((n, ko * 16, od, oh, ow), dtype=np.int64)
    for z in range(kd):
        for y in range(kh):
            for x in range(kw):
                win = a[:, :, z:z + (od - 1) * s + 1:s, y:y + (oh - 1) * s + 1:s, x:x + (ow - 1) * s + 1:s, :]
                out += np.einsum("ncdhwi,kci->nkdhw", win, wt[:, :, z, y, x, :], optimize=True)
    out = out.reshape(n, ko, 16, od, oh, ow).transpose(0, 1, 3, 4, 5, 2)
    return np.ascontiguousarray((out & 0xFFFFFFFF).astype(np.uint32).view(np.int32))


# --------------------------------------------------------------------------- a3 dense
def dense_logical(a, w):
    """relay.nn.dense(x, w) of apps/cpu/relay/int8-gemm.py:14-16: C = A . W^T, A u8 (M,K), W s8 (N,K)."""
    c = a.astype(np.int64) @ w.astype(np.int64).T
    return (c & 0xFFFFFFFF).astype(np.uint32).view(np.int32)


def dense_dotprod(a, wp):
    """topi.x86.dense_dotprod call at apps/cpu/kernel/int8-gemm.py:13-16 on the packed weight:
    C[m,n] = sum_k A[m,k] * Wp[n/128, k/4, n%128, k%4]."""
    nb, kg, t, four = wp.shape
    assert t == 128 and four == 4
    w = wp.transpose(0, 2, 1, 3).reshape(nb * 128, kg * 4)
    return dense_logical(a, w)


# --------------------------------------------------------------------------- a8 / a9 fp16
def gemm_f16(a, b):
    """apps/gpu/gemm.py:8-20: c[x,y] = sum_k f32(a[x,k]) * f32(b[k,y]); evaluated in float64 on the
    fp16-rounded inputs (the tolerance test compares against this)."""
    return a.astype(np.float64) @ b.astype(np.float64)


def pack_gemm_b32(b):
    """The packed operand of apps/gpu/gemm-pack.py:9,17: bp[y/32][k/32][k%32][y%32] = b[k][y], b (K, N)."""
    k, n = b.shape
    assert k % 32 == 0 and n % 32 == 0
    return np.ascontiguousarray(b.reshape(k // 32, 32, n // 32, 32).transpose(2, 0, 1, 3))


def gemm_f16_packed(a, bp):
    """apps/gpu/gemm-pack.py:14-18: c[x,y] = sum_k f32(a[x,k]) * f32(bp[y/32, k/32, k%32, y%32]), in float64 on the
    fp16-rounded inputs, as explicit index arithmetic (no reshape shared with pack_gemm_b32)."""
    m, k = a.shape
    nb, kb, k32, n32 = bp.shape
    assert (k32, n32) == (32, 32) and kb * 32 == k
    ks = np.arange(k)
    out = np.empty((m, nb * 32), dtype=np.float64)
    a64 = a.astype(np.float64)
    for y in range(nb * 32):
        out[:, y] = a64 @ bp[y // 32, ks // 32, ks % 32, y % 32].astype(np.float64)
    return out


def conv2d_nchw16c_f16(a, b, stride_h=1, stride_w=1):
    """python/tensorizer/ops/gpu.py:35-53: valid conv (no padding argument),
    O[n,ko,x,y,ob] = sum_{rc,rh,rw} a[n,rc/16,sh*x+rh,sw*y+rw,rc%16] * b[ko,rc/16,rh,rw,rc%16,ob],
    a (N,C/16,H,W,16), b (K/16,C/16,KH,KW,16,16); float64 on the fp16-rounded inputs."""
    n, cc, h, w, _ = a.shape
    ko, cc2, kh, kw, ib, ob = b.shape
    assert cc == cc2 and ib == 16 and ob == 16
    oh, ow = (h - kh) // stride_h + 1, (w - kw) // stride_w + 1
    a64 = a.astype(np.float64)
    b64 = b.astype(np.float64)
    out = np.zeros((n, ko, oh, ow, 16), dtype=np.float64)
    for y in range(kh):
        for x in range(kw):
            win = a64[:, :, y:y + (oh - 1) * stride_h + 1:stride_h, x:x + (ow - 1) * stride_w + 1:stride_w, :]
            out += np.einsum("nchwi,kcio->nkhwo", win, b64[:, :, y, x], optimize=True)
    return out


# --------------------------------------------------------------------------- C library
class _ConvT(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int) for k in
                ("N", "C", "H", "W", "K", "KH", "KW", "sh", "sw", "pt", "pl", "pb", "pr", "dh", "dw", "cb")]


def build_lib():
    """Compile liboracle.so (and oracle/_ref when the reference tree is mounted)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "all", "ref"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build_lib()
        L = ctypes.CDLL(path)
        vp = ctypes.c_void_p
        L.oracle_has_vnni.restype = ctypes.c_int
        L.oracle_default_threads.restype = ctypes.c_int
        L.oracle_fill_u8.argtypes = [vp, ctypes.c_size_t, ctypes.c_uint64]
        L.oracle_vpdpbusd_scalar.argtypes = [vp, vp, vp]
        L.oracle_vpdpbusd_hw.argtypes = [vp, vp, vp]
        L.oracle_vpdpbusd_hw.restype = ctypes.c_int
        L.oracle_conv2d_nchwc_scalar.argtypes = [ctypes.POINTER(_ConvT), vp, vp, vp]
        L.oracle_conv2d_nchwc_scalar.restype = ctypes.c_int
        L.oracle_conv2d_nchwc_vnni.argtypes = [ctypes.POINTER(_ConvT), vp, vp, vp, ctypes.c_int]
        L.oracle_conv2d_nchwc_vnni.restype = ctypes.c_int
        L.oracle_dense_scalar.argtypes = [vp, vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.oracle_dense_scalar.restype = ctypes.c_int
        L.oracle_dense_vnni.argtypes = [vp, vp, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.oracle_dense_vnni.restype = ctypes.c_int
        L.oracle_vnni_peak.argtypes = [ctypes.c_long, ctypes.c_int]
        L.oracle_vnni_peak.restype = ctypes.c_double
        _LIB = L
    return _LIB


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def c_fill_u8(n, seed):
    out = np.empty(int(n), dtype=np.uint8)
    lib().oracle_fill_u8(_ptr(out), out.size, seed)
    return out


def c_vpdpbusd(acc, a, b, hw=False):
    acc = np.ascontiguousarray(acc, dtype=np.int32).copy()
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.int8)
    if hw:
        if lib().oracle_vpdpbusd_hw(_ptr(acc), _ptr(a), _ptr(b)) != 0:
            return None
    else:
        lib().oracle_vpdpbusd_scalar(_ptr(acc), _ptr(a), _ptr(b))
    return acc


def _conv_desc(data, weight, stride, padding, dilation):
    n, cc, h, w, cb = data.shape
    ko, _, kh, kw, _, _, _ = weight.shape
    sh, sw = _pair(stride)
    dh, dw = _pair(dilation)
    pt, pl, pb, pr = _pad_tuple(padding)
    return _ConvT(n, cc * cb, h, w, ko * 16, kh, kw, sh, sw, pt, pl, pb, pr, dh, dw, cb)


def c_conv2d_nchwc(data, weight, stride=1, padding=0, dilation=1, impl="vnni", nthreads=0):
    """C oracle: impl 'scalar' (closed-form loops) or 'vnni' (vpdpbusd, reference loop nest)."""
    data = np.ascontiguousarray(data, dtype=np.uint8)
    weight = np.ascontiguousarray(weight, dtype=np.int8)
    d = _conv_desc(data, weight, stride, padding, dilation)
    oh, ow = conv_out_hw(d.H, d.W, d.KH, d.KW, stride, padding, dilation)
    out = np.empty((d.N, d.K // 16, oh, ow, 16), dtype=np.int32)
    if impl == "scalar":
        rc = lib().oracle_conv2d_nchwc_scalar(ctypes.byref(d), _ptr(data), _ptr(weight), _ptr(out))
    else:
        rc = lib().oracle_conv2d_nchwc_vnni(ctypes.byref(d), _ptr(data), _ptr(weight), _ptr(out), nthreads)
    if rc != 0:
        raise ValueError("oracle conv2d: bad arguments")
    return out


def c_dense(a, wp, impl="vnni", nthreads=0):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    wp = np.ascontiguousarray(wp, dtype=np.int8)
    m, k = a.shape
    n = wp.shape[0] * 128
    out = np.empty((m, n), dtype=np.int32)
    if impl == "scalar":
        rc = lib().oracle_dense_scalar(_ptr(a), _ptr(wp), _ptr(out), m, n, k)
    else:
        rc = lib().oracle_dense_vnni(_ptr(a), _ptr(wp), _ptr(out), m, n, k, nthreads)
    if rc != 0:
        raise ValueError("oracle dense: bad arguments")
    return out


def has_vnni():
    return bool(lib().oracle_has_vnni())


def default_threads():
    return int(lib().oracle_default_threads())


def vnni_peak_gops(iters=20_000_000, nthreads=0):
    """Host vpdpbusd peak in Gop/s (2 ops per MAC, 64 MACs per instruction)."""
    return lib().oracle_vnni_peak(iters, nthreads) * 128.0
