"""MI355X (gfx950) backend for the kxc compiler's lowered-operator hot path.

The product is the C-ABI library ``lib/libkxc_hip.so`` (declared in ``include/kxc_hip.h``) and the
C++ host layer in ``host/``.  This Python package is a thin ctypes binding of that ABI, used by the
tests and the benchmark; PyTorch appears only as a provider of device memory and streams.

The directory name carries a hyphen, so import it with
``importlib.import_module("hdkx-aicompiler_amd")``.
"""
from . import synth  # noqa: F401
from .hipabi import (  # noqa: F401
    KxcHipError, lib, library_path, conv2d, relu, binary, bias_add, pool2d, global_avg_pool2d, gemm,
    flatten, quantize, qconv2d, qdense, maxpool2d_i8, global_avg_pool2d_i8, conv2d_variant, conv2d_pair, conv2d_pair_supported, conv2d_pair_variant,
    conv2d_winograd_supported, conv2d_winograd_preferred, conv2d_winograd_weight_bytes, conv2d_winograd_variant, conv2d_winograd_transform_weights, conv2d_winograd,
    absmax, quantize_to_c4, qconv2d_c4_pack_weights, qconv2d_c4, qconv2d_c4_maxpool, qconv2d_c4_maxpool_supported, i8_nchw_to_c16, i8_c16_to_nchw, quantize_to_c16, qconv_desc, qconv2d_c16_variant, qconv2d_c16_pack_weights, qconv2d_c16_pair_supported, qconv2d_c16_pair_pack_weights, qconv2d_c16_pair,
    qconv2d_c16, maxpool2d_c16_i8, global_avg_pool2d_c16_i8, c16_shape, pool_desc, pool_out_shape,
    device_attributes, set_select_lanes, Plan, Buf, ConvDesc, PoolDesc, QConvDesc, conv_desc, conv_out_shape,
    CONV_BIAS, CONV_RESIDUAL, CONV_RELU, CONV_HPOOL, CONV_FORCE_DIRECT, conv2d_hpool_supported, QPACK_C16, QPACK_C4, QPACK_C16_PAIR,
)
