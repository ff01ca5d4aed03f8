"""Quantized-linear host code: the reference's function and module names over PyTorch-ROCm tensors.

Every forward runs through the HIP library (``tensorplay_amd.ops``); there is no CPU path here.
"""
from .bitnet import (  # noqa: F401
    BitNetPacked2bitLinear,
    bitnet_linear_packed,
    get_bitnet_scale,
    pack_ternary,
    quantize_bitnet_weight,
    quantize_int8_rowwise,
    unpack_ternary,
)
from .binary import (  # noqa: F401
    BinaryWeightOnlyConfig,
    WeightOnlyBinaryLinear,
    _binary_mm,
    _quantize_binary_weight,
    binary_weight_only,
    pack_binary,
    quantize_binary_weight_only,
    unpack_binary,
)
from .int2_weight_only import (  # noqa: F401
    Int2WeightOnlyConfig,
    WeightOnlyInt2Linear,
    _int2_mm,
    _quantize_int2_groupwise,
    int2_weight_only,
    pack_int2,
    quantize_int2_weight_only,
    unpack_int2,
)
from .int4_weight_only import (  # noqa: F401
    Int4WeightOnlyConfig,
    WeightOnlyInt4Linear,
    _int4_mm,
    _pack_int4_weight,
    _quantize_int4_groupwise,
    int4_weight_only,
)
from .int8_dyn_act_lowbit import (  # noqa: F401
    Int8DynActBinaryWeightLinear,
    Int8DynActInt2WeightLinear,
    Int8DynActInt4WeightLinear,
    Int8DynamicActivationBinaryWeightConfig,
    Int8DynamicActivationInt2WeightConfig,
    Int8DynamicActivationInt4WeightConfig,
    int8_dynamic_activation_binary_weight,
    int8_dynamic_activation_int2_weight,
    int8_dynamic_activation_int4_weight,
)
from .int8_mixed_precision import (  # noqa: F401
    Int8DynamicLinear,
    Int8DynamicLinearConfig,
    _dynamic_int8_mm,
    _int8_mm,
    int8_dynamic_linear,
    scaled_int8_mm,
)
from .intx_weight_only import (  # noqa: F401
    IntxWeightOnlyConfig,
    WeightOnlyIntxLinear,
    _intx_mm,
    _quantize_intx_groupwise,
    intx_weight_only,
    pack_intx,
    quantize_intx_weight_only,
    unpack_intx,
)
from .quantize_api import quantize_, register_quantize_module_handler  # noqa: F401
