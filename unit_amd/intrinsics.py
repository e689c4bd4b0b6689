"""Registry of the instruction back ends, keyed by name like the reference's INTRINSICS dict
(python/tensorizer/intrinsics/intrinsics.py:7-40).

The reference maps a name ('vnni', 'vdot', 'tensorcore', ...) to the callbacks its TIR rewrite
pass splices in (pattern / operands / write / init / schedule / cleanup).  Here there is no
compiler pass: a name maps to the stencil it stands for and to the operator entry points that
run on it, so "select the implementation by name" keeps working.

  'mfma.i8'   v_mfma_i32_32x32x32_i8   u8 x s8 -> i32   (takes the place of 'vnni':
              llvm.x86.avx512.vpdpbusd.512, intrinsics/cpu.py:189-193)
  'mfma.f16'  v_mfma_f32_32x32x16_f16  f16 x f16 -> f32 (takes the place of 'tensorcore':
              wmma.m16n16k16, intrinsics/gpu.py:104-216)
"""
from . import ops

INTRINSICS = {
    "mfma.i8": {
        "pattern": {"instruction": "v_mfma_i32_32x32x32_i8", "tile": (32, 32, 32),
                    "a_dtype": "uint8", "b_dtype": "int8", "out_dtype": "int32"},
        "replaces": "vnni",
        "conv2d": ops.conv2d_NCHWc_int8,
        "dense": ops.dense_dotprod,
    },
    "mfma.f16": {
        "pattern": {"instruction": "v_mfma_f32_32x32x16_f16", "tile": (32, 32, 16),
                    "a_dtype": "float16", "b_dtype": "float16", "out_dtype": "float32"},
        "replaces": "tensorcore",
        "conv2d": ops.conv2d_NCHW16c_OHWI16o,
        "gemm": ops.gemm_fp16,
    },
}
# the reference's own keys resolve to the back end that took their place
INTRINSICS["vnni"] = INTRINSICS["mfma.i8"]
INTRINSICS["tensorcore"] = INTRINSICS["mfma.f16"]
