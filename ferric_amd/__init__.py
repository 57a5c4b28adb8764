"""ferric_amd -- MI355X (gfx950) implementation of Ferric's quantized-GGUF matmul path.

The product is libferric_hip.so (C ABI in include/ferric_hip.h); this package is the host-side
mirror of the reference's quantized-linear interface on top of it.
"""
from .qmatrix import (BATCH_AUTO, BATCH_F32_MATVEC, BATCH_ORDERED, BF16, F16, F32, IQ4_NL, IQ4_XS, MXFP4, Q4_0, Q4_1, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, DeviceBuffer, Graph, Iq4NlWeights, Iq4XsWeights,
                      Mxfp4Weights, Q4_0Weights, Q4_1Weights, Q4_KWeights, Q5_0Weights, Q5_1Weights, Q5_KWeights, Q6_KWeights, Q8_0Weights,
                      Pool, QMatrix, Stream, Tensor, deq_raw, f16_to_f32, matvec_q8_0, matvec_q8_0_pooled, matvec_q8_0_span,
                      matvec_q8_0_threaded, type_size)
from .gguf import Gguf, GgufFile, Proj, TensorInfo

__all__ = ["BATCH_AUTO", "BATCH_F32_MATVEC", "BATCH_ORDERED", "BF16", "F16", "F32", "IQ4_NL", "IQ4_XS", "MXFP4", "Q4_0", "Q4_1", "Q5_0", "Q5_1", "Q5_K", "Q4_K", "Q6_K", "Q8_0", "DeviceBuffer", "Graph",
           "Iq4NlWeights", "Iq4XsWeights", "Mxfp4Weights", "Q4_0Weights", "Q4_1Weights", "Q5_0Weights", "Q5_1Weights", "Q5_KWeights",
           "Q4_KWeights", "Q6_KWeights", "Q8_0Weights", "QMatrix", "Stream",
           "Tensor", "deq_raw", "f16_to_f32", "matvec_q8_0", "matvec_q8_0_pooled", "Pool", "matvec_q8_0_span", "matvec_q8_0_threaded", "type_size",
           "Proj", "Gguf", "GgufFile", "TensorInfo"]
