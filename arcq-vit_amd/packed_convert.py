"""Model-level conversion and packed-checkpoint I/O.

``convert_arcq_linear_to_packed`` / ``count_packed_linear`` mirror FQ/arcq_packed_convert.py:8-28.
``to_on_the_fly`` is the second swap the reference benchmark performs
(scripts/benchmark_arcq_on_the_fly.py:151-170).  ``load_packed_state_dict`` fills a model from the
flat ``state_dict`` the reference converter saves (scripts/convert_arcq_to_packed.py:86-95), for
which the reference itself has no loader: hyper-parameters are inferred from tensor shapes.
"""
from __future__ import annotations

from typing import Dict, List

import torch
import torch.nn as nn

from .packed_conv import ARCQPackedPatchConv
from .packed_linear import ARCQPackedLinear
from .packed_on_the_fly import ARCQPackedLinearOnTheFly
from .quant_source import QuantConv2dPCARCQ, QuantLinearLSQ


def _is_pcarcq_linear(module: nn.Module) -> bool:
    # matched by class NAME so that modules from the reference's own code base convert too
    return (module.__class__.__name__ == "QuantLinearPCARCQ" and hasattr(module, "linear")
            and hasattr(module, "act_quant") and hasattr(module, "weight_quant"))


def convert_arcq_linear_to_packed(model: nn.Module, runtime_code_format: str = "packed") -> nn.Module:
    """Recursively (and in place) replace every ``QuantLinearPCARCQ`` by an ``ARCQPackedLinear``."""
    for name, child in list(model.named_children()):
        if _is_pcarcq_linear(child):
            setattr(model, name, ARCQPackedLinear(child, runtime_code_format=runtime_code_format))
        else:
            convert_arcq_linear_to_packed(child, runtime_code_format=runtime_code_format)
    return model


def _is_pcarcq_conv(module: nn.Module) -> bool:
    return (module.__class__.__name__ == "QuantConv2dPCARCQ" and hasattr(module, "conv")
            and hasattr(module, "act_quant") and hasattr(module, "weight_quant"))


def convert_arcq_conv_to_packed(model: nn.Module) -> int:
    """Replace (in place) every ``QuantConv2dPCARCQ`` that is a patch convolution by an ``ARCQPackedPatchConv``;
    other geometries stay as they are.  Returns the number replaced.  The reference has no counterpart: its
    converter leaves convolutions as fake quantization (FQ/arcq_packed_convert.py:8-14)."""
    done = 0
    for name, child in list(model.named_children()):
        if _is_pcarcq_conv(child):
            c = child.conv
            if (tuple(c.stride) == tuple(c.kernel_size) and tuple(int(p) for p in c.padding) == (0, 0)
                    and tuple(c.dilation) == (1, 1) and c.groups == 1):
                setattr(model, name, ARCQPackedPatchConv(child))
                done += 1
        else:
            done += convert_arcq_conv_to_packed(child)
    return done


def count_packed_linear(model: nn.Module) -> int:
    return sum(1 for m in model.modules() if isinstance(m, ARCQPackedLinear))


def to_on_the_fly(model: nn.Module) -> nn.Module:
    """Replace every ``ARCQPackedLinear`` by an ``ARCQPackedLinearOnTheFly`` sharing its buffers."""
    for name, child in list(model.named_children()):
        if isinstance(child, ARCQPackedLinear):
            setattr(model, name, ARCQPackedLinearOnTheFly.from_packed(child))
        else:
            to_on_the_fly(child)
    return model


def set_fp8_operands(model: nn.Module, enabled: bool = True) -> int:
    """Switch every ``ARCQPackedLinearOnTheFly`` of ``model`` to (or back from) FP8 operands: stage 1 and stage 2 as
    always, their fp32 reconstructions rounded to FP8 (OCP E4M3) and the product on FP8 matrix units.  About 1.5 x the
    speed on ViT-L shapes and 4-6 % away from the fp16 path's layer outputs; no counterpart in the reference.
    Returns the number of layers switched."""
    count = 0
    for module in model.modules():
        if isinstance(module, ARCQPackedLinearOnTheFly):
            module.fp8_operands = bool(enabled)
            count += 1
    return count


def share_buffers(model: nn.Module, max_rows: int = 0) -> nn.Module:
    """Give every on-the-fly layer of ``model`` (already on its device) the two scratch buffers its forward uses,
    shared by all layers: ``_weight_buffer``, one flat fp16 tensor for the largest ``out_features * in_features``
    (what scripts/benchmark_arcq_on_the_fly.py:182-191 sets up), and, when ``max_rows`` is given, ``_x_hat_buffer``
    for ``max_rows`` tokens of the widest input (so that forwards allocate nothing and the buffer's lifetime is
    the model's).  Layers run one after another on a stream, which makes the sharing safe."""
    layers = [m for m in model.modules() if isinstance(m, ARCQPackedLinearOnTheFly)]
    if not layers:
        return model
    dev = layers[0].packed_weight_codes.device
    w = torch.zeros(max(m.out_features * m.in_features for m in layers), dtype=torch.float16, device=dev)
    xh = None
    if max_rows > 0:
        xh = torch.zeros(int(max_rows) * max(m.in_features for m in layers), dtype=torch.float16, device=dev)
    for m in layers:
        m._weight_buffer = w
        if xh is not None:
            m._x_hat_buffer = xh
    return model


def packed_layer_prefixes(state_dict: Dict[str, torch.Tensor]) -> List[str]:
    """Prefixes (with trailing dot) of all packed layers in a flat state dict."""
    tail = "packed_weight_codes"
    return sorted(k[: -len(tail)] for k in state_dict if k.endswith(tail))


def load_packed_state_dict(model: nn.Module, state_dict: Dict[str, torch.Tensor],
                           on_the_fly: bool = True, runtime_code_format: str = "hip_fused") -> nn.Module:
    """Install packed layers found in ``state_dict`` into ``model`` (whose block linears may be
    anything, e.g. ``nn.Linear``), then load every remaining key normally.

    Accepts ``bias`` and ``bias_tensor`` spellings; raises ``KeyError`` for a packed prefix that
    names no submodule of ``model``.
    """
    state_dict = {k.replace("module.", "", 1) if k.startswith("module.") else k: v for k, v in state_dict.items()}
    consumed = set()
    installed = []

    def install(prefix: str, layer: nn.Module) -> None:
        installed.append(prefix)
        path = prefix[:-1].split(".") if prefix else []
        if not path:
            raise KeyError("a packed layer cannot be the model root")
        parent = model
        for part in path[:-1]:
            if not hasattr(parent, part):
                raise KeyError(f"packed checkpoint names '{prefix[:-1]}', which the model does not have")
            parent = getattr(parent, part)
        if not hasattr(parent, path[-1]):
            raise KeyError(f"packed checkpoint names '{prefix[:-1]}', which the model does not have")
        setattr(parent, path[-1], layer)

    for prefix in packed_layer_prefixes(state_dict):
        if prefix + "conv_geometry" in state_dict:
            install(prefix, ARCQPackedPatchConv.from_packed_state(state_dict, prefix))
        else:
            layer = ARCQPackedLinear.from_packed_state(state_dict, prefix, runtime_code_format)
            install(prefix, ARCQPackedLinearOnTheFly.from_packed(layer) if on_the_fly else layer)
        consumed.update(k for k in state_dict if k.startswith(prefix))
    # Layers the reference's converter leaves as fake quantization: the patch-embedding convolution
    # (keys conv.weight + ARCQ quantizer buffers) and the LSQ classifier head (linear.weight + step parameters).
    for key in list(state_dict):
        if key.endswith("conv.weight") and key[: -len("conv.weight")] + "act_quant._pc_cb" in state_dict:
            prefix = key[: -len("conv.weight")]
            w = state_dict[key]
            bits = int(state_dict[prefix + "weight_quant._pc_cb"].numel()).bit_length() - 1
            a_bits = int(state_dict[prefix + "act_quant._pc_cb"].numel()).bit_length() - 1
            layer = QuantConv2dPCARCQ(w.shape[1], w.shape[0], tuple(w.shape[2:]), tuple(w.shape[2:]), 0,
                                      prefix + "conv.bias" in state_dict, bits, a_bits)
            for q in (layer.act_quant, layer.weight_quant):
                q._pc_ready = True
        elif key.endswith("linear.weight") and key[: -len("linear.weight")] + "act_quant.step" in state_dict:
            prefix = key[: -len("linear.weight")]
            w = state_dict[key]
            layer = QuantLinearLSQ(w.shape[1], w.shape[0], prefix + "linear.bias" in state_dict)
        else:
            continue
        for name, _ in list(layer.named_buffers()) + list(layer.named_parameters()):
            stored = state_dict.get(prefix + name)
            if stored is not None:      # buffers registered empty / step sizes of another shape take the stored shape
                owner = layer.get_submodule(name.rsplit(".", 1)[0]) if "." in name else layer
                attr = name.rsplit(".", 1)[-1]
                if attr in owner._buffers:
                    owner._buffers[attr] = stored.detach().clone()
                else:
                    owner._parameters[attr] = nn.Parameter(stored.detach().clone(), requires_grad=False)
        install(prefix, layer.eval())
        consumed.update(k for k in state_dict if k.startswith(prefix))
    rest = {k: v for k, v in state_dict.items() if k not in consumed}
    missing, unexpected = model.load_state_dict(rest, strict=False)
    missing = [k for k in missing if not any(k.startswith(p) for p in installed)]
    if missing or unexpected:
        raise KeyError(f"packed checkpoint mismatch: missing={missing[:8]} unexpected={list(unexpected)[:8]}")
    return model
