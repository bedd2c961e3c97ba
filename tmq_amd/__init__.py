"""tmq_amd -- MI355X-native implementation of TMQ's GPU hot path behind TMQ's Python API.

    from tmq_amd import quantize_model, QuantizationControl, ...     # same names as the reference's `tmq`
"""
from .tmq import *  # noqa: F401,F403
from .tmq import (QuantMode, TensorType, QuantizationScheduleBuilder, QuantizationControl, SoftStep,  # noqa: F401
                  SoftStepDerivative, TMQLayer, Linear, Conv2d, ConvTranspose2d, quantize_weights, quantize_model,
                  compressed_state_dict, prepare_compressed_load, load_compressed_state_dict, expand_compact_layers, fold_batchnorm, set_compact_output_dtype, use_native_pooling, fuse_epilogues, GraphedForward,
                  CUDA_EXT_AVAILABLE, NATIVE_EXT_AVAILABLE)
from .inference import FoldedConv, FoldedStem, ResNetRunner, InferenceSession, optimize_for_inference  # noqa: F401,E402
