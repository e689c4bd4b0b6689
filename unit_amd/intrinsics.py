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
# The reference registers the wmma fragment moves as intrinsics of their own ('tensorcore.load_a', '.load_b',
# '.store_c': intrinsics.py:28-39, emitters intrinsics/gpu.py:104-113,197-216).  Here they are steps inside the
# kernels, not callable operators; the keys stay so that a lookup by the reference's names says what took their place.
INTRINSICS["tensorcore.load_a"] = {
    "pattern": {"instruction": "global_load_lds_dwordx4 + ds_read_b128", "tile": (32, 16), "dtype": "float16"},
    "replaces": "llvm.nvvm.wmma.m16n16k16.load.a.row.stride.f16", "part_of": INTRINSICS["mfma.f16"]}
INTRINSICS["tensorcore.load_b"] = {
    "pattern": {"instruction": "global_load_lds_dwordx4 + ds_read_b128", "tile": (32, 16), "dtype": "float16"},
    "replaces": "llvm.nvvm.wmma.m16n16k16.load.b.row.stride.f16", "part_of": INTRINSICS["mfma.f16"]}
INTRINSICS["tensorcore.store_c"] = {
    "pattern": {"instruction": "global_store_dwordx4 (non-temporal) from the accumulators", "tile": (32, 32),
                "dtype": "float32"},
    "replaces": "llvm.nvvm.wmma.m16n16k16.store.d.row.stride.f32", "part_of": INTRINSICS["mfma.f16"]}
