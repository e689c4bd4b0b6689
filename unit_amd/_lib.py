"""ctypes binding of libunit_amd.so (the C ABI declared in include/unit_amd.h).

The library is the product: there is no fallback.  If it has not been built, loading raises
with the build command; nothing in this package computes on the CPU.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libunit_amd.so")

# every symbol include/unit_amd.h declares
SYMBOLS = (
    "unit_version",
    "unit_last_error",
    "unit_last_variant",
    "unit_conv_variant_count",
    "unit_conv_variant_is_direct",
    "unit_conv_out_hw",
    "unit_conv2d_nchwc_u8s8s32",
    "unit_conv2d_nchwc_s8s8s32_fused",
    "unit_conv3d_ncdhwc_s8s8s32",
    "unit_dense_dotprod_u8s8s32",
    "unit_dense_u8s8s32",
    "unit_dense_prepare_weight",
    "unit_dense_u8s8s32_prepared",
    "unit_gemm_f16",
    "unit_gemm_f16_ws_bytes",
    "unit_gemm_f16_ws",
    "unit_gemm_f16_static",
    "unit_gemm_f16_prepare_b",
    "unit_gemm_f16_prepare_b_packed32",
    "unit_gemm_f16_prepared",
    "unit_conv2d_nchw16c_f16f32",
    "unit_pack_nchwc",
    "unit_unpack_nchwc",
    "unit_prepack_conv_weight_s8",
    "unit_prepack_dense_weight_s8",
    "unit_prepack_conv_weight_f16",
    "unit_conv2d_prepared_weight_bytes",
    "unit_conv2d_prepare_weight",
    "unit_conv2d_nchwc_u8s8s32_prepared",
    "unit_conv2d_nchwc_s8s8s32_fused_prepared",
    "unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw",
    "unit_conv2d_nchw16c_f16f32_prepared",
    "unit_conv2d_nchwc_u8s8u8_requant_prepared",
    "unit_mfma_tile_i8",
    "unit_mfma_tile_f16",
    "unit_mfma_peak",
)


class ConvDesc(ctypes.Structure):
    """struct unit_conv_desc"""
    _fields_ = [(k, ctypes.c_int32) for k in
                ("N", "C", "H", "W", "K", "KH", "KW", "sh", "sw", "pt", "pl", "pb", "pr", "dh", "dw", "cb")]


class Conv3dDesc(ctypes.Structure):
    """struct unit_conv3d_desc"""
    _fields_ = [(k, ctypes.c_int32) for k in ("N", "C", "D", "H", "W", "K", "KD", "KH", "KW", "stride")]


class UnitError(RuntimeError):
    pass


_lib = None


def load():
    """Load libunit_amd.so and declare its prototypes.  Raises if the library is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise UnitError(
            f"{LIB_PATH} is not built. Build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no CPU fallback.")
    L = ctypes.CDLL(LIB_PATH)
    vp, i32 = ctypes.c_void_p, ctypes.c_int32
    dp = ctypes.POINTER(ConvDesc)
    L.unit_version.restype = ctypes.c_int
    L.unit_last_error.restype = ctypes.c_char_p
    L.unit_last_variant.restype = ctypes.c_char_p
    L.unit_conv_variant_is_direct.argtypes = [i32]
    L.unit_conv_out_hw.argtypes = [dp, ctypes.POINTER(i32), ctypes.POINTER(i32)]
    L.unit_conv2d_nchwc_u8s8s32.argtypes = [dp, vp, vp, vp, vp]
    L.unit_conv2d_nchwc_s8s8s32_fused.argtypes = [dp, vp, vp, vp, i32, vp, vp]
    L.unit_conv3d_ncdhwc_s8s8s32.argtypes = [ctypes.POINTER(Conv3dDesc), vp, vp, vp, vp]
    L.unit_dense_dotprod_u8s8s32.argtypes = [vp, vp, vp, i32, i32, i32, vp]
    L.unit_dense_u8s8s32.argtypes = [vp, vp, vp, i32, i32, i32, vp]
    L.unit_dense_prepare_weight.argtypes = [vp, vp, i32, i32, vp]
    L.unit_gemm_f16_ws_bytes.argtypes = [i32, i32, i32, ctypes.POINTER(ctypes.c_size_t)]
    L.unit_gemm_f16_ws.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp, ctypes.c_size_t, vp]
    L.unit_gemm_f16_static.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
    L.unit_dense_u8s8s32_prepared.argtypes = [vp, vp, vp, vp, i32, i32, i32, vp]
    L.unit_gemm_f16.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
    L.unit_gemm_f16_prepare_b.argtypes = [vp, vp, i32, i32, vp]
    L.unit_gemm_f16_prepare_b_packed32.argtypes = [vp, vp, i32, i32, vp]
    L.unit_gemm_f16_prepared.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
    L.unit_conv2d_nchw16c_f16f32.argtypes = [dp, vp, vp, vp, vp]
    L.unit_pack_nchwc.argtypes = [vp, vp, i32, i32, i32, i32, i32, i32, vp]
    L.unit_unpack_nchwc.argtypes = [vp, vp, i32, i32, i32, i32, i32, i32, vp]
    L.unit_prepack_conv_weight_s8.argtypes = [vp, vp, i32, i32, i32, i32, i32, vp]
    L.unit_prepack_dense_weight_s8.argtypes = [vp, vp, i32, i32, vp]
    L.unit_prepack_conv_weight_f16.argtypes = [vp, vp, i32, i32, i32, i32, vp]
    L.unit_conv2d_prepared_weight_bytes.argtypes = [i32, i32, i32, i32, i32, i32, ctypes.POINTER(ctypes.c_size_t)]
    L.unit_conv2d_prepare_weight.argtypes = [i32, i32, i32, i32, i32, i32, vp, vp, vp]
    L.unit_conv2d_nchwc_u8s8s32_prepared.argtypes = [dp, vp, vp, vp, vp]
    L.unit_conv2d_nchwc_s8s8s32_fused_prepared.argtypes = [dp, vp, vp, vp, i32, vp, vp]
    L.unit_conv2d_nchwc_s8s8s32_fused_prepared_nchw.argtypes = [dp, vp, vp, vp, i32, vp, i32, vp]
    L.unit_conv2d_nchw16c_f16f32_prepared.argtypes = [dp, vp, vp, vp, vp]
    L.unit_conv2d_nchwc_u8s8u8_requant_prepared.argtypes = [dp, vp, vp, vp, i32, i32, vp, vp]
    L.unit_mfma_tile_i8.argtypes = [vp, vp, vp, vp]
    L.unit_mfma_tile_f16.argtypes = [vp, vp, vp, vp]
    L.unit_mfma_peak.argtypes = [i32, i32, i32, vp, vp]
    for name in SYMBOLS:
        fn = getattr(L, name)
        if name not in ("unit_last_error", "unit_last_variant"):
            fn.restype = ctypes.c_int
    _lib = L
    return L


def check(rc):
    """Raise the library's message for a non-zero return: ValueError for rejected arguments,
    UnitError for launch / device failures."""
    if rc == 0:
        return
    msg = load().unit_last_error().decode()
    if rc == -1:
        raise ValueError(msg)
    raise UnitError(f"{msg} (code {rc})")


def last_variant():
    return load().unit_last_variant().decode()
