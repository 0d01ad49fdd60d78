"""ARCQ packed on-the-fly quantized linear for AMD MI355X (gfx950): hand-written HIP kernels
behind the reference's Python packed-linear API and packed-checkpoint layout."""
from . import _lib, ops, synth  # noqa: F401
from .ops import (  # noqa: F401
    arcq_linear_forward,
    arcq_linear_forward_u8,
    dequant_activation_hip,
    linear_fused,
    linear_otf,
    pack_codes,
    quantize_activation,
    quantize_activation_dequant,
    quantize_activation_u8,
    unpack_codes,
    unpack_codes_u8,
    unpack_weight_hip,
)
from .pack_py import pack_codes_py, unpack_codes_py  # noqa: F401
from .packed_conv import ARCQPackedPatchConv  # noqa: F401
from .packed_convert import (  # noqa: F401
    convert_arcq_conv_to_packed,
    convert_arcq_linear_to_packed,
    count_packed_linear,
    load_packed_state_dict,
    set_fp8_operands,
    share_buffers,
    to_on_the_fly,
)
from .packed_fast_linear import ARCQPackedLinearFast  # noqa: F401
from .packed_linear import ARCQPackedLinear, _quantize_weight_reference, infer_packed_hparams  # noqa: F401
from .packed_on_the_fly import ARCQPackedLinearOnTheFly, clear_workspaces  # noqa: F401
from .quant_source import (  # noqa: F401
    FrozenARCQQuantizer,
    LSQQuantizer,
    QuantConv2dPCARCQ,
    QuantLinearLSQ,
    QuantLinearPCARCQ,
)

__all__ = [
    "pack_codes", "unpack_codes", "unpack_codes_u8", "quantize_activation", "quantize_activation_dequant",
    "quantize_activation_u8", "arcq_linear_forward", "arcq_linear_forward_u8", "dequant_activation_hip",
    "unpack_weight_hip", "linear_fused", "linear_otf", "pack_codes_py", "unpack_codes_py",
    "ARCQPackedLinear", "ARCQPackedLinearOnTheFly", "ARCQPackedLinearFast", "QuantLinearPCARCQ",
    "FrozenARCQQuantizer", "convert_arcq_linear_to_packed", "count_packed_linear", "to_on_the_fly",
    "load_packed_state_dict", "infer_packed_hparams", "share_buffers", "clear_workspaces",
    "ARCQPackedPatchConv", "convert_arcq_conv_to_packed", "QuantConv2dPCARCQ", "QuantLinearLSQ", "LSQQuantizer",
    "set_fp8_operands",
]
