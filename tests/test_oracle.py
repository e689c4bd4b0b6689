"""Pins the CPU oracle (runs without a GPU).

What pins what:
  stencil (a1)      the reference's known-answer vector (poc/vnni/poc.cc:17-38, committed as
                    golden/vpdpbusd_poc.json), the reference program itself when oracle/_ref is built,
                    the hardware vpdpbusd on random + extreme operands, the 4-term closed form.
  conv (a2)         three independent restatements agree (scalar C, VNNI C with the reference loop nest,
                    vectorised numpy) with a fourth (pure-Python loops) on the golden cases; then what
                    the mathematics fixes: all-ones -> tap count, one-hot weight -> shifted copy,
                    1x1 == dense, stride 2 == sub-sampled stride 1, padding == explicit zero pad,
                    linearity in W, torch float64 conv2d as an independent library routine.
  dense (a3)        numpy int64 A @ W.T; the packed index order is this build's reading of the
                    placeholder shape (parity unpinned for that order, pinned for the product).
  layouts (a5/a6)   the transpose/reshape chain printed at apps/cpu/relay/result.log:8-13 and
                    :6809-6815 vs the one-line index formula; pack/unpack round trip;
                    conv(packed) == textbook NCHW/OIHW conv.
  u8->s8 shift (a7) conv(x ^ 0x80 as s8, w) + 128 * sum(w) == conv(x as u8, w) in int64.
  fp16 (a8/a9)      integer-valued operands make the float64 reference exact; torch conv2d double.
"""
import glob
import json
import os
import subprocess

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
GOLD = os.path.join(HERE, "golden")


# ------------------------------------------------------------------ RNG
def test_rng_c_and_numpy_agree(oracle):
    from unit_amd import rng
    for n, seed in [(1, 0), (7, 1), (8, 2), (1003, 7), (4096, 123456789)]:
        a = oracle.c_fill_u8(n, seed)
        assert np.array_equal(a, oracle.random_bytes(n, seed))
        assert np.array_equal(a, rng.random_bytes(n, seed))
    # splitmix64(0 + GOLDEN) first output, published test vector of the generator
    assert oracle.random_bytes(8, 0).view("<u8")[0] == 0xE220A8397B1DCDAF


# ------------------------------------------------------------------ a1
def test_vpdpbusd_reference_known_answer(oracle):
    g = json.load(open(os.path.join(GOLD, "vpdpbusd_poc.json")))
    a, b = np.array(g["a"], np.uint8), np.array(g["b"], np.int8)
    acc = np.array(g["acc_in"], np.int32)
    want = np.array(g["lanes"], np.int32)
    assert want.tolist() == [620, 1516, 2284, 2924, 3436, 3820, 4076, 4204, 4204, 4076, 3820, 3436, 2924, 2284,
                             1516, 620]
    assert np.array_equal(oracle.vpdpbusd(acc, a, b), want)
    assert np.array_equal(oracle.c_vpdpbusd(acc, a, b), want)
    hw = oracle.c_vpdpbusd(acc, a, b, hw=True)
    if hw is not None:
        assert np.array_equal(hw, want)


def test_vpdpbusd_reference_program_if_built(oracle):
    exe = os.path.join(ROOT, "oracle", "_ref", "poc_vnni")
    if not os.path.exists(exe) or not oracle.has_vnni():
        pytest.skip("oracle/_ref/poc_vnni not built or host lacks AVX-512 VNNI")
    lines = subprocess.run([exe], capture_output=True, text=True, check=True).stdout.strip().split("\n")
    g = json.load(open(os.path.join(GOLD, "vpdpbusd_poc.json")))
    assert [int(x) for x in lines[0].split()] == g["lanes"]  # the instruction
    assert [int(x) for x in lines[1].split()] == g["lanes"]  # the reference's scalar loop


def test_vpdpbusd_random_and_extremes(oracle):
    rs = np.random.RandomState(0)
    cases = [(rs.randint(0, 256, 64), rs.randint(-128, 128, 64), rs.randint(-2**31, 2**31 - 1, 16)) for _ in range(50)]
    cases.append((np.full(64, 255), np.full(64, -128), np.zeros(16)))
    cases.append((np.full(64, 255), np.full(64, 127), np.full(16, 2**31 - 1)))  # wraps, does not saturate
    cases.append((np.full(64, 255), np.full(64, -128), np.full(16, -2**31)))
    for a, b, acc in cases:
        a, b, acc = a.astype(np.uint8), b.astype(np.int8), acc.astype(np.int32)
        want = acc.astype(np.int64) + (a.astype(np.int64).reshape(16, 4) * b.astype(np.int64).reshape(16, 4)).sum(1)
        want = ((want + 2**31) % 2**32 - 2**31).astype(np.int32)
        assert np.array_equal(oracle.vpdpbusd(acc, a, b), want)
        assert np.array_equal(oracle.c_vpdpbusd(acc, a, b), want)
        hw = oracle.c_vpdpbusd(acc, a, b, hw=True)
        if hw is not None:
            assert np.array_equal(hw, want)


# ------------------------------------------------------------------ a2
@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "conv_*.npz"))))
def test_conv_golden(oracle, path):
    g = np.load(path)
    st, pad, dil, cb = (int(x) for x in g["params"])
    data, wt, want = g["data"], g["weight"], g["out"]
    assert data.shape[-1] == cb
    assert np.array_equal(oracle.conv2d_nchwc_int8(data, wt, st, pad, dil), want)
    assert np.array_equal(oracle.conv2d_nchwc_int8_loops(data, wt, st, pad, dil), want)
    assert np.array_equal(oracle.c_conv2d_nchwc(data, wt, st, pad, dil, "scalar"), want)
    assert np.array_equal(oracle.c_conv2d_nchwc(data, wt, st, pad, dil, "vnni"), want)


def _rand_conv(oracle, n, c, h, w, k, ks, cb, seed):
    data = oracle.fill_u8((n, c // cb, h, w, cb), seed)
    wt = oracle.fill_s8((k // 16, c // cb, ks, ks, cb // 4, 16, 4), seed + 1)
    return data, wt


def test_conv_all_ones_counts_taps(oracle):
    data = np.ones((1, 2, 6, 5, 16), np.uint8)
    wt = np.ones((1, 2, 3, 3, 4, 16, 4), np.int8)
    out = oracle.c_conv2d_nchwc(data, wt, 1, 1)
    assert out[0, 0, 2, 2, 0] == 32 * 9          # interior: C * KH * KW
    assert out[0, 0, 0, 0, 0] == 32 * 4          # corner: only 2x2 taps fall inside the image
    assert out[0, 0, 0, 2, 5] == 32 * 6          # top edge


def test_conv_one_hot_weight_is_a_shifted_copy(oracle):
    data, _ = _rand_conv(oracle, 1, 32, 7, 6, 16, 3, 16, 5)
    wt = np.zeros((1, 2, 3, 3, 4, 16, 4), np.int8)
    # output channel 3 picks input channel 21 (= block 1, e 1, i 1) at tap (kh, kw) = (0, 2)
    wt[0, 1, 0, 2, 1, 3, 1] = 1
    out = oracle.c_conv2d_nchwc(data, wt, 1, 0)
    assert np.array_equal(out[0, 0, :, :, 3], data[0, 1, 0:5, 2:6, 5].astype(np.int32))
    assert not out[..., [i for i in range(16) if i != 3]].any()


def test_conv_1x1_equals_dense(oracle):
    n, c, h, w, k = 2, 48, 5, 6, 128
    data, wt = _rand_conv(oracle, n, c, h, w, k, 1, 16, 9)
    out = oracle.c_conv2d_nchwc(data, wt, 1, 0)
    a = oracle.unpack_nchwc(data).transpose(0, 2, 3, 1).reshape(n * h * w, c)
    wmat = wt.transpose(0, 5, 1, 4, 6, 2, 3).reshape(k, c)  # (ko,kb) x (ci,e,i)
    ref = oracle.dense_logical(a, wmat).reshape(n, h, w, k).transpose(0, 3, 1, 2)
    assert np.array_equal(oracle.unpack_nchwc(out), ref)
    assert np.array_equal(oracle.c_dense(a, oracle.prepack_dense_weight(wmat)), ref.transpose(0, 2, 3, 1).reshape(-1, k))


def test_conv_stride2_is_subsampled_stride1(oracle):
    data, wt = _rand_conv(oracle, 1, 16, 9, 11, 32, 3, 16, 13)
    s1 = oracle.c_conv2d_nchwc(data, wt, 1, 1)
    s2 = oracle.c_conv2d_nchwc(data, wt, 2, 1)
    assert np.array_equal(s2, s1[:, :, ::2, ::2])


def test_conv_padding_is_explicit_zero_padding(oracle):
    data, wt = _rand_conv(oracle, 2, 16, 6, 7, 16, 3, 16, 17)
    padded = np.zeros((2, 1, 6 + 1 + 2, 7 + 3 + 0, 16), np.uint8)
    padded[:, :, 1:7, 3:10] = data
    assert np.array_equal(oracle.c_conv2d_nchwc(data, wt, 1, (1, 3, 2, 0)), oracle.c_conv2d_nchwc(padded, wt, 1, 0))


def test_conv_linear_in_weights(oracle):
    data, w1 = _rand_conv(oracle, 1, 16, 6, 6, 16, 3, 16, 21)
    w2 = oracle.fill_s8(w1.shape, 99)
    w1, w2 = (w1 // 2).astype(np.int8), (w2 // 2).astype(np.int8)
    lhs = oracle.c_conv2d_nchwc(data, (w1 + w2).astype(np.int8), 1, 1)
    assert np.array_equal(lhs, oracle.c_conv2d_nchwc(data, w1, 1, 1) + oracle.c_conv2d_nchwc(data, w2, 1, 1))


@pytest.mark.parametrize("c,k,hw,ks,st,pad,dil", [(35, 40, 9, 3, 1, 1, 1), (3, 64, 20, 7, 2, 3, 1), (64, 32, 8, 1, 2, 0, 1),
                                                  (16, 16, 9, 3, 1, 2, 2), (128, 128, 7, 3, 1, 1, 1)])
def test_conv_matches_torch_float64_on_nchw(oracle, c, k, hw, ks, st, pad, dil):
    """pack -> oracle conv -> unpack against torch.nn.functional.conv2d in double (exact: |sum| < 2^53)."""
    cb = 16 if (-(-c // 4) * 4) % 16 == 0 else 4
    x = oracle.fill_u8((2, c, hw, hw), c)
    w = oracle.fill_s8((k, c, ks, ks), k)
    out5 = oracle.c_conv2d_nchwc(oracle.pack_nchwc(x, cb), oracle.prepack_conv_weight(w, cb), st, pad, dil)
    ref = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), stride=st,
                                     padding=pad, dilation=dil).numpy()
    assert np.array_equal(oracle.unpack_nchwc(out5, k).astype(np.float64), ref)
    assert np.array_equal(oracle.conv2d_nchwc_int8(oracle.pack_nchwc(x, cb), oracle.prepack_conv_weight(w, cb), st, pad, dil),
                          out5)


def test_conv_rejects_bad_arguments(oracle):
    data = np.zeros((1, 1, 4, 4, 16), np.uint8)
    wt = np.zeros((1, 1, 5, 5, 4, 16, 4), np.int8)
    with pytest.raises(ValueError):
        oracle.c_conv2d_nchwc(data, wt, 1, 0)  # window larger than the input


# ------------------------------------------------------------------ a3
@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLD, "dense_*.npz"))))
def test_dense_golden(oracle, path):
    g = np.load(path)
    assert np.array_equal(oracle.c_dense(g["a"], g["wp"], "scalar"), g["out"])
    assert np.array_equal(oracle.c_dense(g["a"], g["wp"], "vnni"), g["out"])
    assert np.array_equal(oracle.dense_dotprod(g["a"], g["wp"]), g["out"])
    assert np.array_equal(oracle.dense_logical(g["a"], g["w"]), g["out"])
    assert np.array_equal(oracle.prepack_dense_weight(g["w"]), g["wp"])


def test_dense_reference_sizes(oracle):
    for m, n, k in [(128, 3072, 768), (1, 1024, 512), (29, 128, 20)]:  # int8-gemm.py:9, cpu-shapes.log:367
        a, w = oracle.fill_u8((m, k), m), oracle.fill_s8((n, k), n)
        assert np.array_equal(oracle.c_dense(a, oracle.prepack_dense_weight(w)), oracle.dense_logical(a, w))


# ------------------------------------------------------------------ a5 / a6
@pytest.mark.parametrize("o,i,ks,cb", [(32, 16, 1, 16), (64, 64, 3, 16), (2048, 1024, 1, 16), (64, 3, 7, 4), (16, 8, 3, 4)])
def test_prepack_formula_matches_printed_relay_chain(oracle, o, i, ks, cb):
    w = oracle.fill_s8((o, i, ks, ks), o + i)
    assert np.array_equal(oracle.prepack_conv_weight(w, cb), oracle.prepack_conv_weight_chain(w, cb))


def test_prepack_shapes_match_the_reference_logs(oracle):
    # result.log:13 (128, 64, 1, 1, 4, 16, 4) and :6815 (4, 1, 7, 7, 1, 16, 4)
    assert oracle.prepack_conv_weight(np.zeros((2048, 1024, 1, 1), np.int8), 16).shape == (128, 64, 1, 1, 4, 16, 4)
    assert oracle.prepack_conv_weight(np.zeros((64, 3, 7, 7), np.int8), 4).shape == (4, 1, 7, 7, 1, 16, 4)
    assert oracle.pack_nchwc(np.zeros((1, 3, 8, 8), np.uint8), 4).shape == (1, 1, 8, 8, 4)


def test_pack_round_trip_and_padding(oracle):
    x = oracle.fill_u8((2, 35, 5, 6), 3)
    p = oracle.pack_nchwc(x, 16)
    assert p.shape == (2, 3, 5, 6, 16) and not p[:, 2, :, :, 3:].any()
    assert p[1, 2, 4, 5, 2] == x[1, 34, 4, 5]
    assert np.array_equal(oracle.unpack_nchwc(p, 35), x)


# ------------------------------------------------------------------ a7
def test_unsigned_to_signed_shift_identity(oracle):
    """conv(u8 x, w) == conv((x ^ 0x80) as s8, w) + 128 * sum(w): the identity the MFMA kernels use
    (MFMA int8 is signed x signed) and the mirror image of the reference's own legalisation
    (apps/cpu/relay/result.log:4-6,15-21).  Zero-padded pixels are u8 0, i.e. s8 -128 after the shift."""
    n, c, hw, k = 1, 32, 6, 16
    x = oracle.fill_u8((n, c, hw, hw), 31)
    w = oracle.fill_s8((k, c, 3, 3), 32)
    xs = (x ^ 0x80).view(np.int8)
    xt = torch.nn.functional.pad(torch.from_numpy(xs).double(), (1, 1, 1, 1), value=-128.0)
    signed = torch.nn.functional.conv2d(xt, torch.from_numpy(w).double()).numpy()
    corr = 128.0 * w.astype(np.float64).sum(axis=(1, 2, 3)).reshape(1, k, 1, 1)
    ref = oracle.unpack_nchwc(oracle.c_conv2d_nchwc(oracle.pack_nchwc(x, 16), oracle.prepack_conv_weight(w, 16), 1, 1), k)
    assert np.array_equal(signed + corr, ref.astype(np.float64))


@pytest.mark.parametrize("cb,ks,stride,pad", [(16, 1, 1, 0), (16, 3, 1, 1), (4, 7, 2, 3), (16, 3, 2, (0, 1, 1, 0))])
def test_fused_form_is_the_signed_convolution(oracle, cb, ks, stride, pad):
    """The reference's fused graph (x + 128 -> u8 conv -> - 128 sum(w) -> + bias -> * scale,
    apps/cpu/relay/result.log:3-26) equals (signed conv + bias) * scale, computed here by an
    independent routine (torch float64 conv2d on the un-blocked tensors, exact at these sizes)."""
    n, c, hw, k = 2, 2 * cb, 9, 32
    x = oracle.fill_s8((n, c, hw, hw), 41)
    w = oracle.fill_s8((k, c, ks, ks), 42)
    b = (oracle.fill_s8((k,), 43).astype(np.int32) * 1000)
    pt, pl, pb, pr = (pad,) * 4 if isinstance(pad, int) else pad
    xt = torch.nn.functional.pad(torch.from_numpy(x).double(), (pl, pr, pt, pb))
    signed = torch.nn.functional.conv2d(xt, torch.from_numpy(w).double(), stride=stride).numpy()
    want = ((signed + b.reshape(1, k, 1, 1)) * 11).astype(np.int64)
    for conv in (None, oracle.c_conv2d_nchwc):
        got = oracle.conv2d_nchwc_int8_fused(oracle.pack_nchwc(x, cb), oracle.prepack_conv_weight(w, cb), b, 11,
                                             stride, pad, 1, conv=conv)
        assert np.array_equal(oracle.unpack_nchwc(got, k).astype(np.int64), want)


def test_fused_form_printed_shapes(oracle):
    """The two graphs the reference prints: 1x1 1024 -> 2048 on 16x16 (result.log:3-26) and the 7x7
    stride-2 stem 3 -> 64 on 224x224 with the input channels padded to 4 (result.log:6803-6828),
    scale 11; reduced in size here (same structure), checked against int64 loops on the signed data."""
    for (c, k, hw, ks, stride, cb) in ((32, 32, 5, 1, 1, 16), (3, 16, 19, 7, 2, 4)):
        x = oracle.fill_s8((1, c, hw, hw), 51)
        w = oracle.fill_s8((k, c, ks, ks), 52)
        b = oracle.fill_s8((k,), 53).astype(np.int32)
        got = oracle.unpack_nchwc(oracle.conv2d_nchwc_int8_fused(oracle.pack_nchwc(x, cb), oracle.prepack_conv_weight(w, cb),
                                                                  b, 11, stride, 0, 1), k)
        oh = (hw - ks) // stride + 1
        want = np.zeros((1, k, oh, oh), dtype=np.int64)
        for o in range(k):
            for y in range(oh):
                for z in range(oh):
                    win = x[0, :, y * stride:y * stride + ks, z * stride:z * stride + ks].astype(np.int64)
                    want[0, o, y, z] = ((win * w[o].astype(np.int64)).sum() + b[o]) * 11
        assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("c,k,d,hw,ks,stride", [(32, 32, 5, 6, 3, 1), (16, 48, 6, 7, 3, 2), (32, 16, 4, 5, 1, 2),
                                                 (4, 16, 9, 12, 7, 2), (8, 32, 4, 6, 3, 1)])
def test_conv3d_closed_form(oracle, c, k, d, hw, ks, stride):
    """The restatement of apps/cpu/kernel/conv3d.py:60-64 against torch's float64 conv3d on the
    un-blocked tensors (an independent library routine; exact at these magnitudes).  Channel block 16,
    or 4 when C is not a multiple of 16 (conv3d.py:39-56)."""
    cb = 4 if c % 16 else 16
    x = oracle.fill_s8((2, c, d, hw, hw), 61)
    w = oracle.fill_s8((k, c, ks, ks, ks), 62)
    xb = np.ascontiguousarray(x.reshape(2, c // cb, cb, d, hw, hw).transpose(0, 1, 3, 4, 5, 2))
    # (K, C, kd, kh, kw) -> (K/16, C/cb, kd, kh, kw, cb/4, 16, 4): the conv2d pre-pack with one more window axis
    wb = np.ascontiguousarray(w.reshape(k // 16, 16, c // cb, cb // 4, 4, ks, ks, ks).transpose(0, 2, 5, 6, 7, 3, 1, 4))
    got = oracle.conv3d_ncdhwc_int8(xb, wb, stride)
    want = torch.nn.functional.conv3d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), stride=stride).numpy()
    got_ncdhw = got.transpose(0, 1, 5, 2, 3, 4).reshape(2, k, *got.shape[2:5])
    assert np.array_equal(got_ncdhw.astype(np.float64), want)


# ------------------------------------------------------------------ a8 / a9
def test_fp16_golden_and_integer_exact(oracle):
    g = np.load(os.path.join(GOLD, "fp16_gemm_24x36x40.npz"))
    assert np.allclose(oracle.gemm_f16(g["a"], g["b"]), g["out"], rtol=0, atol=0)
    a = (np.arange(6 * 8).reshape(6, 8) % 7).astype(np.float16)
    b = (np.arange(8 * 5).reshape(8, 5) % 5).astype(np.float16)
    assert np.array_equal(oracle.gemm_f16(a, b), (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float64))


def test_fp16_gemm_packed_b(oracle):
    """The packed operand of apps/gpu/gemm-pack.py:9,17 against its defining index formula, element by element,
    and the packed GEMM against the plain one on the same b (integer-valued operands: exact)."""
    k, n = 64, 96
    b = (np.arange(k * n).reshape(k, n) % 11 - 5).astype(np.float16)
    bp = oracle.pack_gemm_b32(b)
    assert bp.shape == (n // 32, k // 32, 32, 32)
    for y in range(n):
        for kk in range(k):
            assert bp[y // 32, kk // 32, kk % 32, y % 32] == b[kk, y]
    a = (np.arange(5 * k).reshape(5, k) % 7).astype(np.float16)
    assert np.array_equal(oracle.gemm_f16_packed(a, bp), oracle.gemm_f16(a, b))


def test_fp16_conv_matches_torch_double(oracle):
    g = np.load(os.path.join(GOLD, "fp16_conv_3x3_c32_k32.npz"))
    assert np.array_equal(oracle.conv2d_nchw16c_f16(g["a"], g["b"], 1, 1), g["out"])
    rs = np.random.RandomState(3)
    x = rs.randn(2, 32, 9, 8).astype(np.float16)
    w = rs.randn(48, 32, 3, 3).astype(np.float16)
    for st in (1, 2):
        out5 = oracle.conv2d_nchw16c_f16(oracle.pack_nchwc(x, 16), oracle.prepack_conv_weight_f16(w), st, st)
        ref = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), stride=st).numpy()
        assert np.allclose(oracle.unpack_nchwc(out5), ref, rtol=1e-12, atol=1e-12)


def test_requant_definition_small_cases(oracle):
    """The integer requantisation, spelled out scalar by scalar with Python integers on a tiny case
    (floor shift of the 64-bit product plus half, both clamps), and the identities that fix its
    corners: shift s with scale 2**s gives round-half-up of conv + bias clamped; a negative
    accumulator always gives 0."""
    x = oracle.fill_u8((1, 1, 5, 5, 16), 71)
    w = oracle.fill_s8((1, 1, 3, 3, 4, 16, 4), 72)
    bias = (np.arange(16, dtype=np.int32) - 8) * 3000
    acc = oracle.conv2d_nchwc_int8(x, w, 1, 1, 1).astype(np.int64) + bias.reshape(1, 1, 1, 1, 16)
    for scale, shift in ((3, 10), (-2, 7), (1 << 20, 36), (1, 1)):
        got = oracle.conv2d_nchwc_u8_requant(x, w, bias, scale, shift, 1, 1, 1)
        want = np.zeros(acc.shape, np.uint8)
        for idx in np.ndindex(*acc.shape):
            t = (int(acc[idx]) * scale + (1 << (shift - 1))) >> shift   # Python ints: exact, floor shift
            want[idx] = min(255, max(0, t))
        assert np.array_equal(got, want)
    ident = oracle.conv2d_nchwc_u8_requant(x, w, bias, 1 << 8, 16, 1, 1, 1)   # (acc * 256 + 2**15) >> 16 = round(acc / 256)
    assert np.array_equal(ident, np.clip(np.floor(acc / 256.0 + 0.5), 0, 255).astype(np.uint8))
    assert (oracle.conv2d_nchwc_u8_requant(x, w, bias, 5, 3, 1, 1, 1)[acc < -1] == 0).all()


def test_dense_pack_order_is_the_reference_lambda_at_tile_16(oracle):
    """poc/vnni/vnni_dense.py:10-11 states the packed order literally, for 16-row tiles:
    packed[w, x, y, z] = b[w * 16 + y, x * 4 + z]; and :17-19 the product through it:
    c[x, y] = sum_k packed_a[x // 16, k // 4, x % 16, k % 4] * packed_b[y // 16, k // 4, y % 16, k % 4].
    The oracle's pack at tile 16 must be that lambda, element by element; tile 128 is the same rule."""
    from unit_amd import rng
    n, k = 48, 24
    b = rng.uniform_s8((n, k), 77)
    got = oracle.prepack_dense_weight(b, tile=16)
    assert got.shape == (n // 16, k // 4, 16, 4)
    for w in range(n // 16):
        for x in range(k // 4):
            for y in range(16):
                for z in range(4):
                    assert got[w, x, y, z] == b[w * 16 + y, x * 4 + z]
    a = rng.uniform_s8((32, k), 78)
    pa = oracle.prepack_dense_weight(a, tile=16)
    c = np.zeros((32, n), np.int64)
    for x in range(32):
        for y in range(n):
            c[x, y] = sum(int(pa[x // 16, r // 4, x % 16, r % 4]) * int(got[y // 16, r // 4, y % 16, r % 4]) for r in range(k))
    assert np.array_equal(c, a.astype(np.int64) @ b.astype(np.int64).T)
    # the 128-row form follows the same rule
    b2 = rng.uniform_s8((256, 8), 79)
    g2 = oracle.prepack_dense_weight(b2)
    assert all(g2[w, x, y, z] == b2[w * 128 + y, x * 4 + z] for w in range(2) for x in range(2) for y in (0, 5, 127) for z in range(4))
