"""Training checkpoint -> packed checkpoint, and the loader for training checkpoints.

``python -m arcq_vit_amd.convert --model deit_small --bits 4 --config CFG.yaml --checkpoint best.pt --output-dir OUT``
takes the arguments of the reference's converter (scripts/convert_arcq_to_packed.py:97-105) and does what it does
(:29-95): build the fake-quant model the config describes on the CPU, load the checkpoint into it, mark the codebooks
ready, replace every ``QuantLinearPCARCQ`` by an ``ARCQPackedLinear``, and save the ``state_dict`` once per runtime
format as ``<model>_w<bits>a<bits>_packed_<format>.pt`` (``deit_small_w4a4_packed_packed.pt`` /
``..._dequant_gemm.pt`` for the reference's defaults, whose file name is fixed at :88).

Two differences, both deliberate: (i) the reference converts the one model object in place for each format in turn,
so its second pass finds nothing left to convert and both files hold the first format; here each format is converted
from its own copy of the loaded model.  (ii) checkpoints are read with ``torch.load(weights_only=True)``.

The model skeleton is this package's own (``vit.VisionTransformer``, submodule names as timm's), since timm is not
available; the quantization scope follows FQ/timm_quant_models.py:63-121: every block linear and the patch-embedding
convolution get the ARCQ wrappers, the classifier head the W8A8 LSQ wrapper unless ``head_quant: fp32``.

The checkpoint loader follows scripts/benchmark_arcq_packed_inference.py:71-140: accept the ``model`` /
``state_dict`` / ``model_state_dict`` wrappers or a bare state dict, strip ``module.``, load what matches in shape,
then overwrite buffers whose registered shape differs from the stored one (the codebooks ``_pc_cb`` /
``_pc_thresholds`` are registered empty) and ``step`` parameters with the stored tensors.
"""
from __future__ import annotations

import argparse
import copy
import sys
from pathlib import Path
from typing import Dict, List, NamedTuple, Optional, Tuple, Union

import torch
import torch.nn as nn

from .packed_convert import convert_arcq_conv_to_packed, convert_arcq_linear_to_packed, count_packed_linear
from .quant_source import QuantConv2dPCARCQ, QuantLinearLSQ, QuantLinearPCARCQ
from .synth import MODEL_DIMS
from .vit import VisionTransformer

CONVERT_FORMATS = ("packed", "dequant_gemm")


class LoadReport(NamedTuple):
    missing: int
    unexpected: int
    skipped_shape: int
    restored_dynamic: int


def read_checkpoint_state(path: Union[str, Path]) -> Dict[str, torch.Tensor]:
    """State dict of a training checkpoint, keys without ``module.``
    (scripts/benchmark_arcq_packed_inference.py:71-79).  Nothing in the file is executed."""
    path = Path(path)
    if not path.is_file():
        raise FileNotFoundError(str(path))
    checkpoint = torch.load(str(path), map_location="cpu", weights_only=True)
    return unwrap_checkpoint(checkpoint)


def unwrap_checkpoint(checkpoint) -> Dict[str, torch.Tensor]:
    state = checkpoint
    if isinstance(checkpoint, dict):
        for key in ("model", "state_dict", "model_state_dict"):
            if key in checkpoint and isinstance(checkpoint[key], dict):
                state = checkpoint[key]
                break
    if not isinstance(state, dict):
        raise TypeError(f"checkpoint holds no state dict (got {type(state).__name__})")
    return {key.replace("module.", ""): value for key, value in state.items()}


def restore_dynamic_state_tensors(model: nn.Module, state: Dict[str, torch.Tensor]) -> int:
    """Put stored tensors in place of buffers (any shape) and of parameters named ``step``, which
    ``load_state_dict`` cannot do when the registered shape differs (what
    scripts/benchmark_arcq_packed_inference.py:82-98 does after its ordinary load).  Returns how many were placed."""
    owners = dict(model.named_modules())
    placed = 0
    for key, tensor in state.items():
        owner_name, dot, leaf = key.rpartition(".")
        owner = owners.get(owner_name) if dot else None
        if owner is None or not isinstance(tensor, torch.Tensor):
            continue
        fresh = tensor.detach().clone()
        if leaf in owner._buffers:
            owner._buffers[leaf] = fresh
        elif leaf == "step" and leaf in owner._parameters:
            owner._parameters[leaf] = nn.Parameter(fresh)
        else:
            continue
        placed += 1
    return placed


def load_training_checkpoint(model: nn.Module, source: Union[str, Path, Dict]) -> LoadReport:
    """Load a training checkpoint (path, wrapper dict or state dict) into a fake-quant model
    (scripts/benchmark_arcq_packed_inference.py:101-113)."""
    state = read_checkpoint_state(source) if isinstance(source, (str, Path)) else unwrap_checkpoint(source)
    # Entries whose name the model knows are split by whether the shapes agree; only those go through
    # load_state_dict, the rest (the quantizers' dynamically sized tensors among them) is handled below.
    own_shapes = {name: tuple(t.shape) for name, t in model.state_dict().items()}
    known = [name for name in state if name in own_shapes]
    fitting = {name: state[name] for name in known if tuple(state[name].shape) == own_shapes[name]}
    skipped_shape = len(known) - len(fitting)
    missing, unexpected = model.load_state_dict(fitting, strict=False)
    restored = restore_dynamic_state_tensors(model, state)
    return LoadReport(len(missing), len(unexpected), skipped_shape, restored)


def _filled(value) -> bool:
    return isinstance(value, torch.Tensor) and value.numel() > 0


def mark_arcq_codebooks_ready(model: nn.Module) -> Tuple[int, int]:
    """Flag every quantizer that holds a non-empty codebook and thresholds as compiled and stop recompilation
    (scripts/benchmark_arcq_packed_inference.py:116-140).  Returns ``(ready, missing)``."""
    counts = {True: 0, False: 0}
    for module in model.modules():
        if hasattr(module, "_pc_cb") and hasattr(module, "_pc_thresholds"):
            ok = _filled(module._pc_cb) and _filled(module._pc_thresholds)
            if ok:
                module._pc_ready = True
            counts[ok] += 1
        # quantizers of the training code base recompile at scheduled steps: none are left
        if hasattr(module, "phase_compile"):
            module.phase_compile = True
        if hasattr(module, "compile_steps"):
            try:
                module.compile_steps = set()
            except (AttributeError, TypeError):
                pass
    return counts[True], counts[False]


def model_key_of(config: Dict, fallback: Optional[str] = None) -> str:
    """``deit_small`` from ``model_key`` or from a timm name such as ``deit_small_patch16_224``."""
    for cand in (config.get("model_key"), config.get("model_name"), fallback):
        if not cand:
            continue
        for key in sorted(MODEL_DIMS, key=len, reverse=True):
            if str(cand) == key or str(cand).startswith(key + "_"):
                return key
    raise ValueError(f"config names no known model (model_key={config.get('model_key')!r}, "
                     f"model_name={config.get('model_name')!r}); known: {sorted(MODEL_DIMS)}")


def build_source_model(config: Dict, model_key: Optional[str] = None, group_size: int = 64,
                       depth: Optional[int] = None) -> VisionTransformer:
    """The fake-quant model a training config describes, codebooks still empty
    (FQ/timm_quant_models.py:155-182 with the ``pcarcq_nodc`` backend, FQ/quant_backends.py:392-421)."""
    key = model_key_of(config, model_key)
    dims = dict(MODEL_DIMS[key])
    if depth is not None:
        dims["depth"] = int(depth)
    w_bits = int(config.get("w_bits", config.get("bits", 4)))
    a_bits = int(config.get("a_bits", config.get("bits", 4)))
    head_quant = config.get("head_quant", "w8a8")
    num_classes = int(config.get("num_classes", 1000))
    img = int(config.get("image_size", 224))
    vit = VisionTransformer(dims["dim"], dims["depth"], dims["heads"], dims["mlp"], num_classes, img=img,
                            linear=lambda i, o, b: QuantLinearPCARCQ(i, o, b, w_bits, a_bits, group_size))
    conv = vit.patch_embed.proj
    vit.patch_embed.proj = QuantConv2dPCARCQ(conv.in_channels, conv.out_channels, conv.kernel_size, conv.stride,
                                             conv.padding, conv.bias is not None, w_bits, a_bits, group_size)
    if head_quant != "fp32":
        vit.head = QuantLinearLSQ(dims["dim"], num_classes, True, w_bits=8, a_bits=8)
    vit.quant_scope_stats = {"linear": 4 * dims["depth"], "conv2d": 1, "head": int(head_quant != "fp32"),
                             "skipped_linear": 0}
    return vit.eval()


def _size_mb(tensors) -> float:
    return sum(t.numel() * t.element_size() for t in tensors) / 1024 / 1024


def convert(args: argparse.Namespace) -> List[Path]:
    import yaml

    with open(args.config, "r") as f:
        config = yaml.safe_load(f) or {}
    if "w_bits" not in config and "bits" not in config:
        config["bits"] = int(args.bits)
    print("[BUILD] Creating ARCQ model on CPU...")
    model = build_source_model(config, args.model)
    print(f"[QUANT_SCOPE] {model.quant_scope_stats}")
    print(f"[LOAD] Loading checkpoint: {args.checkpoint}")
    report = load_training_checkpoint(model, args.checkpoint)
    ready, not_ready = mark_arcq_codebooks_ready(model)
    print(f"  missing={report.missing} unexpected={report.unexpected} skipped_shape={report.skipped_shape} "
          f"restored={report.restored_dynamic}")
    print(f"  ready_codebooks={ready}")
    if not_ready:
        print(f"  WARNING: {not_ready} quantizers have no codebook in this checkpoint")
    print(f"\n[ORIG] parameters={_size_mb(model.parameters()):.1f}MB buffers={_size_mb(model.buffers()):.1f}MB")

    key = model_key_of(config, args.model)
    bits = int(config.get("w_bits", config.get("bits", args.bits)))
    out_dir = Path(args.output_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    written = []
    for fmt in CONVERT_FORMATS:
        print(f"\n[CONVERT] Format: {fmt}")
        packed = convert_arcq_linear_to_packed(copy.deepcopy(model), runtime_code_format=fmt)
        convs = convert_arcq_conv_to_packed(packed) if args.pack_patch_embed else 0
        params, buffers = _size_mb(packed.parameters()), _size_mb(packed.buffers())
        print(f"  packed_layers={count_packed_linear(packed)} packed_convs={convs} params={params:.1f}MB "
              f"buffers={buffers:.1f}MB total={params + buffers:.1f}MB")
        out_path = out_dir / f"{key}_w{bits}a{bits}_packed_{fmt}.pt"
        torch.save(packed.state_dict(), out_path)
        print(f"[SAVE] {out_path}\n  File size: {out_path.stat().st_size / 1024 / 1024:.1f} MB")
        written.append(out_path)
    print("\n[DONE]")
    return written


def main(argv: Optional[List[str]] = None) -> int:
    parser = argparse.ArgumentParser(prog="python -m arcq_vit_amd.convert", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", default="deit_small")
    parser.add_argument("--bits", type=int, default=4)
    parser.add_argument("--config", required=True, help="training YAML (model_name, num_classes, w_bits, a_bits, "
                                                        "head_quant are read)")
    parser.add_argument("--checkpoint", required=True, help="training checkpoint (best.pt / latest.pt)")
    parser.add_argument("--output-dir", required=True)
    parser.add_argument("--pack-patch-embed", action="store_true",
                        help="also pack the patch-embedding convolution (the reference leaves it as fake quantization)")
    convert(parser.parse_args(argv))
    return 0


if __name__ == "__main__":
    sys.exit(main())
