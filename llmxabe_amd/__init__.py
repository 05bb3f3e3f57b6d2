"""llmxabe_amd: the MI355X (gfx950) quantized MoE feed-forward block behind the reference's launch API."""
from .moe import (BLOCK_Q6_K_DEVICE_BYTES, BufferScope, ExpertQuant, LayerOpsKernels, MmaKernels, MoeBuffers,  # noqa: F401
                  MoeError, MoeGeometry, MoeKernels, QuantTensor, calibrate_hbm_read, calibrate_mfma_f16, dequantize, moe_block_size,
                  synth_normal_f32, synth_quant, to_device_layout, zipf_logit_bias)
from .block import (DEFAULT_RMS_EPS, DenseFfnBlock, DenseFfnLayerWeights, FfnBlock, FfnConfig, FfnKind,  # noqa: F401
                    FfnLayerWeights, MoeBlock, MoeLayerWeights, moe_block_forward_noalloc)
from .gguf import GgmlType, GgufError, GgufFile, TensorInfo, UploadedDenseFfnLayer, UploadedMoeLayer  # noqa: F401
from .lm_head import ARGMAX_BLOCKS, MAX_BATCH_TILE, HeadFormat, HeadTensor, LmHeadGeometry, LmHeadKernels  # noqa: F401
