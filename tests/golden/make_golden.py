#!/usr/bin/env python3
"""Writes the golden fixtures under tests/golden/ (run from the repository root).

  vpdpbusd_poc.json   the reference's only known-answer vector: inputs and expected lanes of
                      poc/vnni/poc.cc:17-38.  The expected lanes are what that program prints and
                      self-asserts (it is compiled from the reference tree by `make -C oracle ref`
                      and run here when present; the values are also checked against the closed form).
  conv_*.npz          small u8 x s8 -> i32 convolutions: operands + expected output.
  dense_*.npz         small dense cases.
  fp16_*.npz          small fp16 GEMM / conv cases with float64 expected output.

Expected outputs come from the scalar C oracle and are cross-checked, before writing, against the
independent pure-Python-loop restatement and the VNNI build of the oracle.
"""
import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CONV_CASES = {
    # name: (N, C, H, W, K, ks, stride, pad, dilation, cb)
    "conv_3x3_s1_p1_c32": (1, 32, 6, 6, 32, 3, 1, 1, 1, 16),
    "conv_1x1_s1_c16": (2, 16, 5, 4, 16, 1, 1, 0, 1, 16),
    "conv_1x1_s2_c32": (1, 32, 6, 6, 16, 1, 2, 0, 1, 16),
    "conv_3x3_s2_p1_c16": (1, 16, 7, 7, 32, 3, 2, 1, 1, 16),
    "conv_7x7_s2_p3_c4": (1, 4, 12, 12, 16, 7, 2, 3, 1, 4),
    "conv_3x3_s1_p0_c8_cb4": (1, 8, 5, 5, 16, 3, 1, 0, 1, 4),
    "conv_3x3_d2_p2_c16": (1, 16, 7, 7, 16, 3, 1, 2, 2, 16),
}


def main():
    # --- the reference's known-answer vector
    a = (np.arange(64) + 1).astype(np.uint8)
    b = (64 - np.arange(64)).astype(np.int8)
    lanes = O.vpdpbusd(np.zeros(16, np.int32), a, b).tolist()
    ref_bin = os.path.join(ROOT, "oracle", "_ref", "poc_vnni")
    source = "closed form"
    if os.path.exists(ref_bin) and O.has_vnni():
        out = subprocess.run([ref_bin], capture_output=True, text=True, check=True).stdout.split("\n")
        printed = [int(x) for x in out[0].split()]
        assert printed == lanes, (printed, lanes)
        source = "printed by the reference's poc/vnni/poc.cc compiled with g++ and run on an AVX-512 VNNI host"
    json.dump({"a": a.tolist(), "b": b.tolist(), "acc_in": [0] * 16, "lanes": lanes, "source": source},
              open(os.path.join(HERE, "vpdpbusd_poc.json"), "w"), indent=1)

    # --- conv
    for seed, (name, (n, c, h, w, k, ks, st, pad, dil, cb)) in enumerate(sorted(CONV_CASES.items())):
        data = O.fill_u8((n, c // cb, h, w, cb), 100 + seed)
        wt = O.fill_s8((k // 16, c // cb, ks, ks, cb // 4, 16, 4), 200 + seed)
        out = O.c_conv2d_nchwc(data, wt, st, pad, dil, impl="scalar")
        assert np.array_equal(out, O.conv2d_nchwc_int8_loops(data, wt, st, pad, dil))
        assert np.array_equal(out, O.c_conv2d_nchwc(data, wt, st, pad, dil, impl="vnni"))
        np.savez_compressed(os.path.join(HERE, name + ".npz"), data=data, weight=wt, out=out,
                            params=np.array([st, pad, dil, cb], dtype=np.int32))

    # --- dense
    for seed, (m, n, k) in enumerate([(5, 128, 32), (33, 256, 48)]):
        a = O.fill_u8((m, k), 300 + seed)
        w = O.fill_s8((n, k), 400 + seed)
        wp = O.prepack_dense_weight(w)
        out = O.c_dense(a, wp, impl="scalar")
        assert np.array_equal(out, O.dense_logical(a, w))
        np.savez_compressed(os.path.join(HERE, f"dense_{m}x{n}x{k}.npz"), a=a, w=w, wp=wp, out=out)

    # --- fp16 (float64 expected values on the fp16-rounded operands)
    rs = np.random.RandomState(7)
    a = (rs.randn(24, 40) / 6).astype(np.float16)
    b = rs.randn(40, 36).astype(np.float16)
    np.savez_compressed(os.path.join(HERE, "fp16_gemm_24x36x40.npz"), a=a, b=b, out=O.gemm_f16(a, b))
    a5 = rs.randn(1, 2, 6, 7, 16).astype(np.float16)
    b6 = (rs.randn(2, 2, 3, 3, 16, 16) / 17).astype(np.float16)
    np.savez_compressed(os.path.join(HERE, "fp16_conv_3x3_c32_k32.npz"), a=a5, b=b6,
                        out=O.conv2d_nchw16c_f16(a5, b6, 1, 1), params=np.array([1, 1], dtype=np.int32))
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith((".npz", ".json"))))


if __name__ == "__main__":
    main()
