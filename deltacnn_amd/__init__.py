"""deltacnn_amd: DeltaCNN's sparse delta-propagation inference path on MI355X (gfx950).

Export list mirrors ``src/deltacnn/__init__.py`` of the reference.
"""
from .hip_kernels import (sparse_conv, sparse_deconv, sparse_pooling, sparse_activation, sparsify,
                          sparse_add_tensors, sparse_add_to_dense_tensor, sparse_upsample,
                          sparse_concatenate, sparse_mul_add, sparse_conv_activation, pack_filter)
from .sparse_layers import (DCConv2d, DCConvTranspose2d, DCMaxPooling, DCAdaptiveAveragePooling,
                            DCDensify, DCAdd, DCActivation, DCUpsamplingNearest2d, DCSparsify,
                            DCThreshold, DCBackend, DCModule, DCBatchNorm2d, DCConcatenate,
                            DCTruncation)

__all__ = [
    "sparse_conv", "sparse_deconv", "sparse_pooling", "sparse_activation", "sparsify",
    "sparse_add_tensors", "sparse_add_to_dense_tensor", "sparse_upsample", "sparse_concatenate",
    "sparse_mul_add", "sparse_conv_activation", "pack_filter",
    "DCConv2d", "DCConvTranspose2d", "DCMaxPooling", "DCAdaptiveAveragePooling", "DCDensify",
    "DCAdd", "DCActivation", "DCUpsamplingNearest2d", "DCSparsify", "DCThreshold", "DCBackend",
    "DCModule", "DCBatchNorm2d", "DCConcatenate", "DCTruncation",
]
