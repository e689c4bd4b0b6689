"""Random shapes through every entry point against the oracle: convolutions (16- and 4-channel blocks, strides,
asymmetric padding, dilation, ragged sizes; reference layout, prepared weights, the fused form, its NCHW store, the
requantised form, the fp16 operator), conv3d, the int8 dense and the fp16 GEMM (every layout of the constant operand,
both output types) and the layout kernels.  Every fourth case runs with the tuned tables switched off.  int8 is compared
bit for bit, fp16 within the stated tolerance.  A failure names its case by (block, index, shape, seed)."""
import numpy as np
import pytest
import torch

import unit_amd as U

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2  # fp16: max relative error against float64 on the fp16-rounded inputs
CASES_PER_BLOCK = 40


def _rel(got, ref):
    return float((np.abs(got - ref) / np.maximum(np.abs(ref), 1e-3 * np.abs(ref).max() + 1e-30)).max())


def _conv_case(r):
    cb = 16 if r.rand() < 0.8 else 4
    c = 16 * int(r.randint(1, 41)) if cb == 16 else 4 * int(r.choice([1, 2, 3, 5]))
    n = int(r.choice([1, 1, 2, 3, 5, 8]))
    h, w = int(r.randint(1, 41)), int(r.randint(1, 41))
    k = 16 * int(r.randint(1, 33))
    kh, kw = int(r.randint(1, 6)), int(r.randint(1, 6))
    if r.rand() < 0.3:
        kh = kw = 1
    stride = (int(r.randint(1, 4)), int(r.randint(1, 4)))
    dil = (int(r.randint(1, 3)), int(r.randint(1, 3))) if r.rand() < 0.2 else (1, 1)
    pad = tuple(int(v) for v in r.randint(0, 3, 4)) if r.rand() < 0.6 else (0, 0, 0, 0)
    if h + pad[0] + pad[2] < dil[0] * (kh - 1) + 1 or w + pad[1] + pad[3] < dil[1] * (kw - 1) + 1:
        return None
    oh = (h + pad[0] + pad[2] - dil[0] * (kh - 1) - 1) // stride[0] + 1
    ow = (w + pad[1] + pad[3] - dil[1] * (kw - 1) - 1) // stride[1] + 1
    macs = n * oh * ow * k * c * kh * kw
    if macs > 3e9:
        return None
    return dict(cb=cb, c=c, n=n, h=h, w=w, k=k, kh=kh, kw=kw, stride=stride, dil=dil, pad=pad, macs=macs)


def _run_conv(O, dev, cs, seed):
    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    cb, c, n, h, w, k, kh, kw = (cs[x] for x in ("cb", "c", "n", "h", "w", "k", "kh", "kw"))
    stride, dil, pad = cs["stride"], cs["dil"], cs["pad"]
    g = np.random.RandomState(seed)
    data = g.randint(0, 256, (n, c // cb, h, w, cb)).astype(np.uint8)
    wt = g.randint(-128, 128, (k // 16, c // cb, kh, kw, cb // 4, 16, 4)).astype(np.int8)
    bias = (g.randint(-128, 128, (k,)) * 1000).astype(np.int32)
    ref = O.c_conv2d_nchwc(data, wt, stride, pad, dil)
    td, tw, tb = t(data), t(wt), t(bias)
    out = U.conv2d_NCHWc_int8(td, tw, stride, pad, dil)
    assert np.array_equal(out.cpu().numpy(), ref), ("reference layout", U.last_variant())
    # prepared weights serve the direct kernels: windows of at most 31 positions; 4-channel blocks: KW <= 8, no dilation along W
    prepared = U.prepare_conv2d_weight(tw) if (kh * kw <= 31 if cb == 16 else kw <= 8 and dil[1] == 1) else None
    if prepared is not None:
        out = U.conv2d_NCHWc_int8(td, prepared, stride, pad, dil)
        assert np.array_equal(out.cpu().numpy(), ref), ("prepared", U.last_variant())
    signed = data.view(np.int8)
    ts = t(signed)
    fused_ref = O.conv2d_nchwc_int8_fused(signed, wt, bias, 11, stride, pad, dil, conv=O.c_conv2d_nchwc)
    out = U.conv2d_NCHWc_int8_fused(ts, tw, tb, 11, stride, pad, dil)
    assert np.array_equal(out.cpu().numpy(), fused_ref), ("fused", U.last_variant())
    if prepared is not None:
        out = U.conv2d_NCHWc_int8_fused(ts, prepared, tb, 11, stride, pad, dil)
        assert np.array_equal(out.cpu().numpy(), fused_ref), ("fused, prepared", U.last_variant())
        oc = k - int(g.randint(0, 16))
        out = U.conv2d_NCHWc_int8_fused(ts, prepared, tb, 11, stride, pad, dil, out_layout="NCHW", out_channels=oc)
        assert np.array_equal(out.cpu().numpy(), O.unpack_nchwc(fused_ref, oc)), ("fused, NCHW", oc, U.last_variant())
        if cb == 16:
            shift, scale = int(g.randint(1, 30)), int(g.randint(-5, 2000))
            q_ref = O.conv2d_nchwc_u8_requant(data, wt, bias, scale, shift, stride, pad, dil, conv=O.c_conv2d_nchwc)
            q = U.conv2d_NCHWc_int8_requant(td, prepared, tb, scale, shift, stride, pad, dil)
            assert np.array_equal(q.cpu().numpy(), q_ref), ("requantised", scale, shift, U.last_variant())
    # the fp16 operator on the same geometry where it exists: 16-channel blocks, no padding argument, no dilation
    if cb == 16 and pad == (0, 0, 0, 0) and dil == (1, 1) and cs["macs"] <= 3e8:
        a = g.randn(n, c // 16, h, w, 16).astype(np.float16)
        b = (g.randn(k // 16, c // 16, kh, kw, 16, 16) / np.sqrt(c * kh * kw)).astype(np.float16)
        ref16 = O.conv2d_nchw16c_f16(a, b, stride[0], stride[1])
        ta, tb16 = t(a), t(b)
        out = U.conv2d_NCHW16c_OHWI16o(ta, tb16, stride[0], stride[1], "float32")
        assert _rel(out.cpu().numpy(), ref16) <= REL_TOL, ("fp16", U.last_variant())
        if kh * kw <= 31:
            out = U.conv2d_NCHW16c_OHWI16o(ta, U.prepare_conv2d_weight(tb16), stride[0], stride[1], "float32")
            assert _rel(out.cpu().numpy(), ref16) <= REL_TOL, ("fp16, prepared", U.last_variant())


def _gemm_case(r):
    m = int(r.choice([1, 3, 17, 64, 100, 128, 129, 255, 256, 300, 512, 777, 1024, 1500, 2048]))
    n = 4 * int(r.randint(1, 600))
    k = 16 * int(r.randint(1, 300))
    return dict(m=m, n=n, k=k) if m * n * k <= 4e9 else None


def _run_gemm(O, dev, cs, seed):
    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    m, n, k = cs["m"], cs["n"], cs["k"]
    g = np.random.RandomState(seed)
    a = g.randint(0, 256, (m, k)).astype(np.uint8)
    w = g.randint(-128, 128, (n, k)).astype(np.int8)
    ref = O.dense_logical(a, w)
    assert np.array_equal(U.dense(t(a), t(w)).cpu().numpy(), ref), ("dense", U.last_variant())
    if n % 128 == 0:
        out = U.dense_dotprod(t(a), t(O.prepack_dense_weight(w)))
        assert np.array_equal(out.cpu().numpy(), ref), ("dense, packed", U.last_variant())
    a16 = g.randn(m, k).astype(np.float16)
    b16 = (g.randn(k, n) / np.sqrt(k)).astype(np.float16)
    ref16 = O.gemm_f16(a16, b16)
    ta, tb = t(a16), t(b16)
    for out_dtype in ("float32", "float16"):
        out = U.gemm_fp16(ta, tb, out_dtype)
        assert _rel(out.float().cpu().numpy(), ref16) <= REL_TOL, ("gemm", out_dtype, U.last_variant())
        out = U.gemm_fp16(ta, U.prepare_gemm_b(tb), out_dtype)
        assert _rel(out.float().cpu().numpy(), ref16) <= REL_TOL, ("gemm, prepared b", out_dtype, U.last_variant())
    if n % 32 == 0 and k % 32 == 0:  # b as the reference packs it, (N/32, K/32, 32, 32)
        out = U.gemm_fp16(ta, t(O.pack_gemm_b32(b16)))
        assert _rel(out.cpu().numpy(), ref16) <= REL_TOL, ("gemm, packed b", U.last_variant())


def _conv3d_case(r):
    cb = 16 if r.rand() < 0.75 else 4
    c = 16 * int(r.randint(1, 9)) if cb == 16 else 4 * int(r.choice([1, 2, 3]))
    n = int(r.choice([1, 2, 3]))
    d, h, w = int(r.randint(1, 9)), int(r.randint(1, 15)), int(r.randint(1, 15))
    k = 16 * int(r.randint(1, 9))
    kd, kh, kw = int(r.randint(1, 4)), int(r.randint(1, 4)), int(r.randint(1, 4))
    if kd > d or kh > h or kw > w or (cb == 16 and kd * kh * kw > 31):
        return None
    return dict(cb=cb, c=c, n=n, d=d, h=h, w=w, k=k, kd=kd, kh=kh, kw=kw, stride=int(r.randint(1, 3)))


def _run_conv3d(O, dev, cs, seed):
    g = np.random.RandomState(seed)
    cb = cs["cb"]
    data = g.randint(-128, 128, (cs["n"], cs["c"] // cb, cs["d"], cs["h"], cs["w"], cb)).astype(np.int8)
    wt = g.randint(-128, 128, (cs["k"] // 16, cs["c"] // cb, cs["kd"], cs["kh"], cs["kw"], cb // 4, 16, 4)).astype(np.int8)
    out = U.conv3d_NCDHWc_int8(torch.from_numpy(data).to(dev), torch.from_numpy(wt).to(dev), cs["stride"])
    assert np.array_equal(out.cpu().numpy(), O.conv3d_ncdhwc_int8(data, wt, cs["stride"])), ("conv3d", U.last_variant())


def _layout_case(r):
    return dict(n=int(r.randint(1, 5)), c=int(r.randint(1, 200)), h=int(r.randint(1, 60)), w=int(r.randint(1, 60)),
                cb=int(r.choice([16, 16, 4])), es=int(r.choice([1, 1, 2, 4])))


def _run_layout(O, dev, cs, seed):
    g = np.random.RandomState(seed)
    x = g.randint(-100, 100, (cs["n"], cs["c"], cs["h"], cs["w"])).astype({1: np.int8, 2: np.float16, 4: np.int32}[cs["es"]])
    packed = U.pack_nchwc(torch.from_numpy(x).to(dev), cs["cb"])
    assert np.array_equal(packed.cpu().numpy(), O.pack_nchwc(x, cs["cb"])), "pack"
    assert np.array_equal(U.unpack_nchwc(packed, cs["c"]).cpu().numpy(), x), "unpack"


@pytest.mark.parametrize("block", range(8))
def test_random_cases(dev, oracle, block, monkeypatch):
    r = np.random.RandomState(52000 + block)
    make = {"conv": _conv_case, "gemm": _gemm_case, "layout": _layout_case, "conv3d": _conv3d_case}
    run = {"conv": _run_conv, "gemm": _run_gemm, "layout": _run_layout, "conv3d": _run_conv3d}
    done = 0
    while done < CASES_PER_BLOCK:
        kind = str(r.choice(["conv", "conv", "conv", "conv", "gemm", "layout", "conv3d"]))
        cs = make[kind](r)
        if cs is None:
            continue
        seed = int(r.randint(1, 1 << 30))
        if done % 4 == 0:
            monkeypatch.setenv("UNIT_AMD_CONV_NOTABLE", "1")
        else:
            monkeypatch.delenv("UNIT_AMD_CONV_NOTABLE", raising=False)
        try:
            run[kind](oracle, dev, cs, seed)
        except AssertionError as e:
            raise AssertionError(f"block {block} case {done} {kind} {cs} seed {seed}: {e}") from e
        done += 1
