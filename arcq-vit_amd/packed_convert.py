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

from .packed_linear import ARCQPackedLinear
from .packed_on_the_fly import ARCQPackedLinearOnTheFly


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
    for prefix in packed_layer_prefixes(state_dict):
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
        layer = ARCQPackedLinear.from_packed_state(state_dict, prefix, runtime_code_format)
        setattr(parent, path[-1], ARCQPackedLinearOnTheFly.from_packed(layer) if on_the_fly else layer)
        consumed.update(k for k in state_dict if k.startswith(prefix))
    rest = {k: v for k, v in state_dict.items() if k not in consumed}
    missing, unexpected = model.load_state_dict(rest, strict=False)
    packed_keys = {k for k, _ in model.state_dict().items()
                   if any(k.startswith(p) for p in packed_layer_prefixes(state_dict))}
    missing = [k for k in missing if k not in packed_keys]
    if missing or unexpected:
        raise KeyError(f"packed checkpoint mismatch: missing={missing[:8]} unexpected={list(unexpected)[:8]}")
    return model
