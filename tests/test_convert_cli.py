"""Converter command line and training-checkpoint loader (host logic, CPU only).

The "training checkpoint" is synthetic and written by the test: a fake-quant DeiT-Tiny in the reference's full
quantization scope (ARCQ wrappers on block linears and the patch convolution, LSQ head), saved the way the training
script saves it (``{epoch, model_state_dict, optimizer_state_dict, best_top1}``, FW/utils.py:27-38) with DDP's
``module.`` prefix.  Its codebooks are stored with 16 entries while a freshly built model registers them empty, and
its per-channel LSQ step has ``[classes]`` entries against a registered ``[1]``: the two cases
``restore_dynamic_state_tensors`` exists for."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F
import yaml

import arcq_vit_amd as A
from arcq_vit_amd import convert, synth
from arcq_vit_amd.packed_linear import _quantize_weight_reference
from arcq_vit_amd.vit import VisionTransformer, build_fakequant_vit

CLASSES = 10
BUFFERS = {"packed_weight_codes", "weight_codes_u8", "weight_dequant", "weight_center", "weight_scale",
           "weight_code_sum", "weight_codebook", "activation_codebook", "activation_thresholds", "product_table", "bias"}


@pytest.fixture(scope="module")
def trained(tmp_path_factory):
    """(source model, checkpoint path, config path)."""
    d = tmp_path_factory.mktemp("train")
    model = build_fakequant_vit("deit_tiny", 4, num_classes=CLASSES, quantize_patch_embed=True, head_quant="w8a8")
    state = {"module." + k: v.clone() for k, v in model.state_dict().items()}
    ckpt = d / "best.pt"
    torch.save({"epoch": 3, "model_state_dict": state, "optimizer_state_dict": {}, "best_top1": 12.5}, ckpt)
    cfg = d / "cfg.yaml"
    cfg.write_text(yaml.safe_dump({"model_key": "deit_tiny", "model_name": "deit_tiny_patch16_224",
                                   "num_classes": CLASSES, "w_bits": 4, "a_bits": 4, "head_quant": "w8a8",
                                   "image_size": 224, "method": "pcarcq_nodc"}))
    return model, ckpt, cfg


def test_loader_restores_codebooks_and_steps(trained):
    model, ckpt, cfg = trained
    fresh = convert.build_source_model(yaml.safe_load(cfg.read_text()))
    assert fresh.quant_scope_stats == {"linear": 48, "conv2d": 1, "head": 1, "skipped_linear": 0}
    assert fresh.blocks[0].attn.qkv.act_quant._pc_cb.numel() == 0
    rep = convert.load_training_checkpoint(fresh, ckpt)
    quantizers = 2 * 49                                  # act + weight quantizer of 48 linears and the convolution
    assert rep.missing == 2 * quantizers + 1             # the empty-registered buffers and the per-channel step
    assert rep.unexpected == 0 and rep.skipped_shape == 2 * quantizers + 1
    assert rep.restored_dynamic == 2 * quantizers + 2    # every buffer, and both step parameters
    assert convert.mark_arcq_codebooks_ready(fresh) == (quantizers, 0)
    assert fresh.head.weight_quant.step.shape == (CLASSES,)
    for (k1, v1), (k2, v2) in zip(sorted(model.state_dict().items()), sorted(fresh.state_dict().items())):
        assert k1 == k2 and torch.equal(v1, v2), k1
    x = synth.make_images(2, 1)
    with torch.no_grad():
        assert torch.equal(fresh(x), model(x))           # same tensors, same code: same logits


@pytest.mark.parametrize("wrapper", ["model", "state_dict", "model_state_dict", None])
def test_checkpoint_wrappers(trained, tmp_path, wrapper):
    model = trained[0]
    state = {"module." + k: v for k, v in model.state_dict().items()}
    path = tmp_path / "c.pt"
    torch.save({wrapper: state, "epoch": 1} if wrapper else state, path)
    got = convert.read_checkpoint_state(path)
    assert set(got) == set(model.state_dict()) and all(not k.startswith("module.") for k in got)
    with pytest.raises(FileNotFoundError):
        convert.read_checkpoint_state(tmp_path / "absent.pt")


def test_unready_quantizers_are_counted():
    fresh = convert.build_source_model({"model_name": "deit_tiny_patch16_224", "bits": 3, "head_quant": "fp32"}, depth=1)
    assert isinstance(fresh.head, torch.nn.Linear)
    assert convert.mark_arcq_codebooks_ready(fresh) == (0, 2 * 5)
    with pytest.raises(ValueError, match="missing"):
        A.convert_arcq_linear_to_packed(fresh)
    with pytest.raises(ValueError, match="no known model"):
        convert.model_key_of({"model_name": "swin_tiny_patch4_window7_224"})
    assert convert.model_key_of({"model_name": "vit_large_patch16_224"}) == "vit_large"
    assert convert.model_key_of({}, "deit_base") == "deit_base"


@pytest.fixture(scope="module")
def converted(trained, tmp_path_factory):
    model, ckpt, cfg = trained
    out = tmp_path_factory.mktemp("packed")
    assert convert.main(["--model", "deit_tiny", "--bits", "4", "--config", str(cfg), "--checkpoint", str(ckpt),
                         "--output-dir", str(out / "nested" / "dir")]) == 0
    return out / "nested" / "dir"


def test_cli_writes_one_file_per_format(trained, converted):
    model = trained[0]
    files = sorted(p.name for p in converted.iterdir())
    assert files == ["deit_tiny_w4a4_packed_dequant_gemm.pt", "deit_tiny_w4a4_packed_packed.pt"]
    states = {f: torch.load(converted / f, map_location="cpu", weights_only=True) for f in files}
    cb = synth.quantile_codebook(4)
    thr = synth.midpoint_thresholds(cb)
    for f, st in states.items():
        prefixes = A.packed_convert.packed_layer_prefixes(st)
        assert len(prefixes) == 48
        for p in prefixes:
            assert {k[len(p):] for k in st if k.startswith(p)} == BUFFERS, p
            assert not any(k.startswith(p + "linear") for k in st)      # no floating-point weight is kept
        # the convolution and the head stay as the reference's converter leaves them
        assert "patch_embed.proj.conv.weight" in st and "head.weight_quant.step" in st
        src = dict(model.named_modules())["blocks.7.mlp.fc2"]
        codes, c, s, cs = _quantize_weight_reference(src.linear.weight, thr, cb, 64, 1e-6)
        p = "blocks.7.mlp.fc2."
        assert torch.equal(st[p + "packed_weight_codes"], A.pack_codes_py(codes, 4))
        assert torch.equal(st[p + "weight_center"], c) and torch.equal(st[p + "weight_scale"], s)
        assert torch.equal(st[p + "weight_code_sum"], cs) and torch.equal(st[p + "bias"], src.linear.bias.detach())
        assert st[p + "weight_codes_u8"].numel() == 0
        assert torch.equal(st[p + "product_table"], cb.view(-1, 1) * cb.view(1, -1))
    # each format is converted from its own copy of the model, so the second file really is the second format
    assert states[files[1]]["blocks.0.attn.qkv.weight_dequant"].numel() == 0
    wd = states[files[0]]["blocks.0.attn.qkv.weight_dequant"]
    assert wd.dtype == torch.float16 and tuple(wd.shape) == (576, 192)
    fq = model.blocks[0].attn.qkv
    ref = fq.weight_quant(fq.linear.weight).detach().to(torch.float16)      # same values up to the order of the
    differ = wd != ref                                                       # mean subtraction: rare one-ulp cases
    assert float(differ.float().mean()) < 1e-3
    assert float((wd.float() - ref.float()).abs().max()) <= 2.0 ** -10 * float(ref.abs().max())


def test_packed_checkpoint_loads_into_plain_skeleton(trained, converted):
    model = trained[0]
    st = torch.load(converted / "deit_tiny_w4a4_packed_packed.pt", map_location="cpu", weights_only=True)
    d = synth.MODEL_DIMS["deit_tiny"]
    skeleton = VisionTransformer(d["dim"], d["depth"], d["heads"], d["mlp"], CLASSES)
    A.load_packed_state_dict(skeleton, st)
    assert sum(isinstance(m, A.ARCQPackedLinearOnTheFly) for m in skeleton.modules()) == 48
    assert isinstance(skeleton.patch_embed.proj, A.QuantConv2dPCARCQ) and isinstance(skeleton.head, A.QuantLinearLSQ)
    assert skeleton.patch_embed.proj.act_quant.group_size == 3 and skeleton.patch_embed.proj.act_quant._pc_ready
    assert skeleton.head.weight_quant.step.shape == (CLASSES,)
    x = synth.make_images(2, 3)
    with torch.no_grad():           # the floating-point parts and the two fake-quant layers run on the CPU
        assert torch.equal(skeleton.patch_embed(x), model.patch_embed(x))
        t = torch.randn(4, d["dim"])
        assert torch.equal(skeleton.head(t), model.head(t))
        assert torch.equal(skeleton.pos_embed, model.pos_embed)
    lay = skeleton.blocks[11].mlp.fc1
    assert (lay.in_features, lay.out_features, lay.bits, lay.group_size) == (192, 768, 4, 64)


def test_cli_can_pack_the_patch_convolution(trained, tmp_path):
    model, ckpt, cfg = trained
    convert.main(["--config", str(cfg), "--checkpoint", str(ckpt), "--output-dir", str(tmp_path),
                  "--pack-patch-embed"])
    st = torch.load(tmp_path / "deit_tiny_w4a4_packed_packed.pt", map_location="cpu", weights_only=True)
    assert st["patch_embed.proj.conv_geometry"].tolist() == [3, 16, 16, 3]
    assert "patch_embed.proj.conv.weight" not in st
    d = synth.MODEL_DIMS["deit_tiny"]
    skeleton = VisionTransformer(d["dim"], d["depth"], d["heads"], d["mlp"], CLASSES)
    A.load_packed_state_dict(skeleton, st)
    pc = skeleton.patch_embed.proj
    assert isinstance(pc, A.ARCQPackedPatchConv)
    assert (pc.in_channels, pc.out_channels, pc.kernel_size, pc.act_group_size, pc.group_size, pc.bits) == \
        (3, 192, (16, 16), 3, 64, 4)
    cb = synth.quantile_codebook(4)
    w = model.patch_embed.proj.conv.weight.detach()
    codes, c, s, cs = _quantize_weight_reference(w.reshape(192, 768), synth.midpoint_thresholds(cb), cb, 64, 1e-6)
    assert torch.equal(pc.packed_weight_codes, A.pack_codes_py(codes, 4)) and torch.equal(pc.weight_scale, s)
    with pytest.raises(RuntimeError):          # no CPU forward
        pc(synth.make_images(1, 1))
    half = pc.half()
    assert half.weight_scale.dtype == torch.float32 and half.bias.dtype == torch.float32


def test_patch_rows_match_unfold():
    conv = A.QuantConv2dPCARCQ(3, 8, 4, 4, 0, True, 4, 4, group_size=16)
    cb = synth.quantile_codebook(4)
    conv.act_quant.set_codebook(cb)
    conv.weight_quant.set_codebook(cb)
    pc = A.ARCQPackedPatchConv(conv)
    x = torch.randn(2, 3, 8, 12)
    rows = pc.patch_rows(x.permute(0, 2, 3, 1).contiguous())
    ref = F.unfold(x, kernel_size=4, stride=4).transpose(1, 2).reshape(-1, 48)      # columns in (c, i, j) order
    assert torch.equal(rows, ref)
    for bad in (dict(s=2), dict(p=1)):
        c2 = A.QuantConv2dPCARCQ(3, 8, 4, bad.get("s", 4), bad.get("p", 0), True, 4, 4, group_size=16)
        c2.act_quant.set_codebook(cb)
        c2.weight_quant.set_codebook(cb)
        with pytest.raises(ValueError, match="patch convolutions"):
            A.ARCQPackedPatchConv(c2)
        holder = torch.nn.Sequential(c2)
        assert A.convert_arcq_conv_to_packed(holder) == 0 and isinstance(holder[0], A.QuantConv2dPCARCQ)


def test_fakequant_conv_groups_channels_of_one_pixel(oracle):
    """QuantConv2dPCARCQ against the oracle's quantizer applied the way FQ/quant_backends.py:366-376 says: pixels as
    rows of three channels (one group each), the weight as [out, in*kh*kw] rows in groups of 64; then a plain
    convolution.  A grouping along the wrong axis (NCHW rows, or groups over kh*kw only) fails this."""
    bits = 3
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    conv = A.QuantConv2dPCARCQ(3, 16, 8, 8, 0, True, bits, bits)
    conv.act_quant.set_codebook(cb)
    conv.weight_quant.set_codebook(cb)
    assert conv.act_quant.group_size == 3 and conv.weight_quant.group_size == 64
    x = torch.randn(2, 3, 16, 24, generator=torch.Generator().manual_seed(5))
    with torch.no_grad():
        y = conv(x)
    pix = x.permute(0, 2, 3, 1).reshape(-1, 3).contiguous().numpy()
    xh = oracle.act_quant_c(pix, thr, cb, bits, 3, fma=False)["x_hat"].reshape(2, 16, 24, 3)
    w2 = conv.conv.weight.detach().reshape(16, 192)
    codes, c, s, cs = oracle.quantize_weight_torch(w2, thr, cb, 64, 1e-6)
    wh = oracle.weight_dequant_c(A.pack_codes_py(codes, bits).numpy(), cb, c, s, cs, bits, 64, fma=False)
    ref = F.conv2d(torch.from_numpy(xh).permute(0, 3, 1, 2), torch.from_numpy(wh).reshape(16, 3, 8, 8),
                   conv.conv.bias.detach(), stride=8)
    assert float((y - ref).abs().max()) <= 1e-5 * float(ref.abs().max()) + 1e-6


def test_lsq_quantizer_known_answers():
    q = A.LSQQuantizer(bits=8, signed=True)
    q.step = torch.nn.Parameter(torch.tensor([0.5]))
    x = torch.tensor([0.26, -0.24, 100.0, -100.0, 0.75, 1.25])
    #                 0.52->1  -0.48->-0  clamp 127  clamp -128  1.5->2 (ties to even)  2.5->2
    assert q(x).tolist() == [0.5, -0.0, 63.5, -64.0, 1.0, 1.0]
    u = A.LSQQuantizer(bits=2, signed=False)
    assert u(torch.tensor([-1.0, 0.4, 2.6, 9.0])).tolist() == [0.0, 0.0, 3.0, 3.0]
    pc = A.LSQQuantizer(bits=8, signed=True, per_channel=True, ch_axis=0)
    pc.step = torch.nn.Parameter(torch.tensor([1.0, 0.25]))
    w = torch.tensor([[0.6, -0.6], [0.6, -0.6]])
    assert pc(w).tolist() == [[1.0, -1.0], [0.5, -0.5]]
    head = A.QuantLinearLSQ(2, 2, True)
    head.weight_quant.init_from(torch.tensor([[1.0, -3.0], [0.5, 0.5]]))
    assert np.allclose(head.weight_quant.step.tolist(), [2 * 2.0 / 127 ** 0.5, 2 * 0.5 / 127 ** 0.5])
