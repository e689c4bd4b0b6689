"""unit_amd -- the tensorized u8 x s8 -> i32 and fp16 -> fp32 conv2d / dense / GEMM path of
were/UNIT as hand-written gfx950 (MI355X) kernels behind the reference's operator entry points."""
from .ops import (conv2d_NCHWc_int8, conv2d_NCHWc_int8_fused, conv2d_NCHWc_int8_requant, conv3d_NCDHWc_int8, conv2d_NCHW16c_OHWI16o, conv_out_hw, dense, dense_dotprod, gemm_fp16, gemm_fp16_workspace_bytes,
                  last_variant, pack_nchwc, prepack_conv_weight, prepack_conv_weight_f16,
                  prepack_dense_weight, unpack_nchwc, PreparedConvWeight, prepare_conv2d_weight,
                  PreparedGemmB, prepare_gemm_b, PreparedDenseWeight, prepare_dense_weight)
from .intrinsics import INTRINSICS
from . import rng, workloads

__version__ = "0.1.0"
