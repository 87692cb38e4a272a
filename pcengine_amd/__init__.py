"""pcengine_amd — sparse 3-D convolution engine for AMD MI355X (gfx950).

Front end with the names of PCEngine's ``script`` package (conv3d, spTensor, BatchNorm, ReLU,
LeakyReLU, cat, sparse_collate, sparse_quantize, ...) over a hand-written HIP backend reached
through the C ABI of include/pcengine_amd.h.
"""
from .sptensor import spTensor
from .spconv import conv3d, conv_func
from .batchnorm import BatchNorm
from .activation import ReLU, LeakyReLU
from .utils import (cat, fapply, sparse_collate, sparse_collate_fn, sparse_quantize, ravel_hash, conv_info_encoder,
                    conv_info_decoder, output_stride_compute, build_conv_buffer, init_layer_scheduler, make_ntuple)
from . import backend

__all__ = ["spTensor", "conv3d", "conv_func", "BatchNorm", "ReLU", "LeakyReLU", "cat", "fapply", "sparse_collate",
           "sparse_collate_fn", "sparse_quantize", "ravel_hash", "conv_info_encoder", "conv_info_decoder",
           "output_stride_compute", "build_conv_buffer", "init_layer_scheduler", "make_ntuple", "backend"]
