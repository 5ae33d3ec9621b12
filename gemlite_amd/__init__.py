"""MI355X-native quantized matmul behind the GemLite ``GemLiteLinear`` API.

Public names follow the reference package (reference: gemlite/__init__.py:5-29).
"""
__version__ = "0.1.0"

from . import _ext, helper
from .bitpack import (
    pack_weights_over_cols,
    pack_weights_over_cols_torch,
    unpack_over_cols,
    unpack_over_cols_torch,
)
from .core import (
    GEMLITE_ACC_DTYPE,
    GEMLITE_CONFIG_CACHE,
    GEMLITE_MATMUL_TYPES,
    GEMLITE_MATMUL_TYPES_MAPPING,
    GEMLITE_TRITON_MAPPING,
    GemLiteLinear,
    GemLiteLinearTriton,
    config_key,
    forward_functional,
    forward_functional_op,
    get_closest_m,
    get_default_gemv,
    get_matmul_type,
    get_type_id,
    set_acc_dtype,
    set_packing_bitwidth,
)
from .dtypes import DTYPE_TO_TORCH, TORCH_TO_DTYPE, DType, is_mx_dtype
from .quant_utils import (
    WeightQuantizerMXFP,
    quantize_weights_per_channel,
    scale_activations_mxfp4,
    scale_activations_mxfp8,
    scale_activations_per_block,
    scale_activations_per_token,
)

load_config = GemLiteLinear.load_config
cache_config = GemLiteLinear.cache_config
reset_config = GemLiteLinear.reset_config
from . import tune  # noqa: E402,F401  (offline tile tuner)
