"""CPU-side tests: golden fixtures vs the oracle, the C-ABI library's exports, the module layer
(buffer layout, conversion, checkpoint loading, error behaviour) and the synthetic generators.
Nothing here launches a kernel."""
import ctypes
import json
import os
import re

import numpy as np
import pytest
import torch
import torch.nn as nn

import arcq_vit_amd as A
from arcq_vit_amd import synth
from arcq_vit_amd.vit import build_fakequant_vit

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


# ------------------------------------------------------------------------------------------------
# golden fixtures
# ------------------------------------------------------------------------------------------------
def test_layout_vectors(oracle):
    vecs = json.load(open(os.path.join(GOLDEN, "layout_vectors.json")))["vectors"]
    for v in vecs:
        codes = np.array([v["codes"]], dtype=np.int64)
        assert oracle.pack_codes_c(codes, v["bits"]).tolist() == [v["bytes"]]
        assert oracle.pack_codes_np(codes, v["bits"]).tolist() == [v["bytes"]]
        assert A.pack_codes_py(torch.from_numpy(codes), v["bits"]).tolist() == [v["bytes"]]
        assert oracle.unpack_codes_c(np.array([v["bytes"]], dtype=np.uint8), v["bits"], len(v["codes"])).tolist() == [v["codes"]]


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_oracle_reproduces_golden(oracle, bits):
    g = np.load(os.path.join(GOLDEN, f"arcq_w{bits}a{bits}_g64.npz"))
    a32 = oracle.act_quant_c(g["x"], g["thresholds"], g["codebook"], bits, 64)
    for k in ("packed", "codes", "center", "scale", "code_sum", "x_hat"):
        assert np.array_equal(a32[k], g[f"a32_{k}"]), k
    a16 = oracle.act_quant_c(g["x_f16"].astype(np.float32), g["thresholds"], g["codebook"], bits, 64)
    assert np.array_equal(a16["packed"], g["a16_packed"])
    assert np.array_equal(a16["x_hat"].astype(np.float16).view(np.uint16), g["a16_x_hat_f16"].view(np.uint16))
    wd = oracle.weight_dequant_c(g["w_packed"], g["codebook"], g["w_center"], g["w_scale"], g["w_code_sum"], bits, 64)
    assert np.array_equal(wd.astype(np.float16).view(np.uint16), g["w_dequant_f16"].view(np.uint16))
    y64, mag = oracle.linear_f64_c(g["a16_x_hat_f16"], g["w_dequant_f16"], g["bias"])
    assert np.array_equal(y64, g["y_f64"]) and np.array_equal(mag, g["y_abs_sum"])
    yp = oracle.linear_forward_packed_c(g["a32_packed"], g["a32_center"], g["a32_scale"], g["a32_code_sum"],
                                        g["w_packed"], g["w_center"], g["w_scale"], g["w_code_sum"],
                                        g["product_table"], g["bias"], bits, 64, 128, 16)
    assert np.array_equal(yp, g["y_index_packed"])
    yu = oracle.linear_forward_u8_c(g["a32_codes"], g["a32_center"], g["a32_scale"], g["a32_code_sum"], g["w_codes"],
                                    g["w_center"], g["w_scale"], g["w_code_sum"], g["product_table"], g["bias"], 64)
    assert np.array_equal(yu, g["y_index_u8"])
    # the fixture's first group is constant: s = sqrt(eps)
    assert g["a32_scale"][0, 0] == np.sqrt(np.float32(1e-6))


# ------------------------------------------------------------------------------------------------
# C ABI
# ------------------------------------------------------------------------------------------------
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "arcq_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(arcq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 11 and "arcq_linear_fused" in names and "arcq_act_quant" in names
    lib = A._lib.load()
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/arcq_hip.h but not exported"
    assert sorted(A._lib.EXPORTED_SYMBOLS) == names
    assert lib.arcq_version() == 100
    # no torch / pybind types leak into the ABI: the library links against the HIP runtime only
    deps = os.popen(f"ldd {A._lib.LIB_PATH}").read()
    assert "libtorch" not in deps and "libc10" not in deps and "python" not in deps.lower()


def test_abi_argument_errors_need_no_gpu():
    """Validation happens before any HIP call, so these are safe on a machine without a GPU."""
    lib = A._lib.load()
    assert lib.arcq_pack_codes(0, 0, 4, 4, 7, 0) == -1
    assert b"bits must be 2, 3, or 4" in lib.arcq_last_error()
    assert lib.arcq_unpack_codes(0, 0, -1, 4, 4, 0) == -4
    assert lib.arcq_pack_codes(0, 0, 4, 4, 4, 0) == -3                       # NULL tensors, non-empty shape
    assert lib.arcq_pack_codes(0, 0, 0, 4, 4, 0) == 0                        # empty is fine
    assert lib.arcq_act_quant(8, 0, 8, 8, 0, 0, 0, 0, 0, 0, 0, 4, 128, 4, 48, 1e-6, 0) == -2
    assert b"in_features must be divisible by group_size" in lib.arcq_last_error()
    assert lib.arcq_act_quant(8, 7, 8, 8, 0, 0, 0, 0, 0, 0, 0, 4, 128, 4, 64, 1e-6, 0) == -5
    assert lib.arcq_weight_dequant(8, 8, 8, 8, 8, 8, 9, 4, 128, 4, 64, 0) == -5
    assert lib.arcq_linear_fused(16, 16, 8, 8, 8, 8, 0, 16, 1, 4, 4, 128, 4, 32, 0) == -6
    assert b"group_size 64" in lib.arcq_last_error()
    assert lib.arcq_linear_fused(8, 16, 8, 8, 8, 8, 0, 16, 1, 4, 4, 128, 4, 64, 0) == -7  # misaligned x_hat
    assert lib.arcq_linear_forward_packed(*([8] * 11), 4, 4, 128, 4, 64, 8, 0) == -4      # 8 levels < 2^4
    assert lib.arcq_linear_forward_packed(*([8] * 11), 4, 4, 128, 4, 64, 200, 0) == -4    # a 200 x 200 table does not fit LDS
    assert b"levels <= 128" in lib.arcq_last_error()
    assert lib.arcq_linear_forward_u8(*([8] * 11), 4, 4, 128, 64, 129, 0) == -4
    assert lib.arcq_linear_otf(8, 0, 8, 8, 8, 8, 8, 8, 8, 0, 8, 16, 1, 4, 4, 128, 4, 64, 0) == -5  # fp32 x aliasing ws
    with pytest.raises(RuntimeError, match="aliasing|alias"):
        A._lib.check(-5)


# ------------------------------------------------------------------------------------------------
# module layer
# ------------------------------------------------------------------------------------------------
def _source(in_f=128, out_f=24, bias=True, bits=4, gs=64, seed=1):
    torch.manual_seed(seed)
    src = A.QuantLinearPCARCQ(in_f, out_f, bias, bits, bits, gs)
    cb = synth.quantile_codebook(bits)
    src.act_quant.set_codebook(cb * 1.1)
    src.weight_quant.set_codebook(cb)
    with torch.no_grad():
        src.linear.weight.copy_(synth.make_weight(out_f, in_f, seed))
        if bias:
            src.linear.bias.copy_(synth.make_bias(out_f, seed))
    return src.eval()


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("fmt", ["packed", "u8", "dequant_gemm", "hip_fused"])
def test_packed_linear_buffers(oracle, bits, fmt):
    """Buffer names, shapes, dtypes and contents (FQ/arcq_packed_linear.py:106-151)."""
    src = _source(bits=bits)
    layer = A.ARCQPackedLinear(src, runtime_code_format=fmt)
    n, k, g, L = 24, 128, 2, 1 << bits
    sd = layer.state_dict()
    assert list(sd) == ["packed_weight_codes", "weight_codes_u8", "weight_dequant", "weight_center", "weight_scale",
                        "weight_code_sum", "weight_codebook", "activation_codebook", "activation_thresholds",
                        "product_table", "bias"]
    want_shapes = {"packed_weight_codes": (n, k * bits // 8), "weight_center": (n, g), "weight_scale": (n, g),
                   "weight_code_sum": (n, g), "weight_codebook": (L,), "activation_codebook": (L,),
                   "activation_thresholds": (L - 1,), "product_table": (L, L), "bias": (n,),
                   "weight_codes_u8": (n, k) if fmt == "u8" else (0,),
                   "weight_dequant": (n, k) if fmt == "dequant_gemm" else (0,)}
    for name, shape in want_shapes.items():
        assert tuple(sd[name].shape) == shape, name
    assert sd["packed_weight_codes"].dtype == torch.uint8 and sd["weight_codes_u8"].dtype == torch.uint8
    assert sd["weight_dequant"].dtype == torch.float16
    assert all(sd[k_].dtype == torch.float32 for k_ in ("weight_center", "weight_scale", "weight_code_sum",
                                                        "weight_codebook", "product_table", "bias"))
    # contents: the oracle's restatement of the offline encoder + packer
    w_thr = src.weight_quant._pc_thresholds
    codes, center, scale, code_sum = oracle.quantize_weight_torch(src.linear.weight, w_thr, src.weight_quant._pc_cb,
                                                                 64, 1e-6)
    assert np.array_equal(sd["packed_weight_codes"].numpy(), oracle.pack_codes_np(codes.numpy(), bits))
    assert torch.equal(sd["weight_center"], center) and torch.equal(sd["weight_scale"], scale)
    assert torch.equal(sd["weight_code_sum"], code_sum)
    assert torch.equal(sd["product_table"], src.act_quant._pc_cb.view(-1, 1) * src.weight_quant._pc_cb.view(1, -1))
    assert torch.equal(sd["activation_thresholds"], src.act_quant._pc_thresholds)
    assert torch.equal(sd["bias"], src.linear.bias.detach())
    if fmt == "u8":
        assert np.array_equal(sd["weight_codes_u8"].numpy(), codes.numpy().astype(np.uint8))
    if fmt == "dequant_gemm":
        want = oracle.unpack_weight_torch(sd["packed_weight_codes"], sd["weight_codebook"], center, scale, code_sum,
                                          bits, 64)
        assert torch.equal(sd["weight_dequant"], want)
    # attributes and accounting (:148-151, :224-241)
    assert (layer.in_features, layer.out_features, layer.group_size, layer.bits, layer.act_bits) == (k, n, 64, bits, bits)
    assert layer.packed_weight_bytes == n * k * bits // 8 and layer.weight_meta_floats == 3 * n * g
    assert layer.estimated_storage_bytes() == n * k * bits // 8 + 4 * (3 * n * g + 3 * L - 1 + L * L + n)
    assert layer.runtime_cache_bytes() == (n * k if fmt == "u8" else 2 * n * k if fmt == "dequant_gemm" else 0)
    assert f"bits={bits}" in layer.extra_repr() and f"runtime_code_format={fmt}" in layer.extra_repr()


def test_packed_linear_no_bias_and_errors():
    layer = A.ARCQPackedLinear(_source(bias=False))
    assert layer.bias.numel() == 0 and layer.bias.dtype == torch.float32
    with pytest.raises(ValueError, match="runtime_code_format"):
        A.ARCQPackedLinear(_source(), "int8")
    with pytest.raises(TypeError, match="source.linear.weight"):
        A.ARCQPackedLinear(nn.Identity())
    no_q = nn.Module()
    no_q.linear = nn.Linear(64, 8)
    with pytest.raises(TypeError, match="act_quant and weight_quant"):
        A.ARCQPackedLinear(no_q)
    mixed = A.QuantLinearPCARCQ(64, 8, True, 4, 3)
    mixed.act_quant.set_codebook(synth.quantile_codebook(3))
    mixed.weight_quant.set_codebook(synth.quantile_codebook(4))
    with pytest.raises(ValueError, match="W bits == A bits"):
        A.ARCQPackedLinear(mixed)
    five = A.QuantLinearPCARCQ(64, 8, True, 5, 5)
    with pytest.raises(ValueError, match="supports bits 2/3/4"):
        A.ARCQPackedLinear(five)
    with pytest.raises(ValueError, match="divisible by group_size"):
        A.ARCQPackedLinear(A.QuantLinearPCARCQ(100, 8, True, 4, 4))
    empty = A.QuantLinearPCARCQ(64, 8, True, 4, 4)
    with pytest.raises(ValueError, match="is missing; load a checkpoint"):
        A.ARCQPackedLinear(empty)
    wrong = A.QuantLinearPCARCQ(64, 8, True, 4, 4)
    wrong.act_quant._pc_cb = torch.zeros(8)
    wrong.act_quant._pc_thresholds = torch.zeros(7)
    wrong.weight_quant.set_codebook(synth.quantile_codebook(4))
    with pytest.raises(ValueError, match="codebook size must be 16"):
        A.ARCQPackedLinear(wrong)
    with pytest.raises(ValueError, match="expected last dim"):
        layer(torch.zeros(2, 3))


def test_forward_has_no_cpu_fallback():
    """On CPU tensors every forward must fail loudly rather than compute something else."""
    x = torch.zeros(2, 128)
    for fmt in ("packed", "u8", "dequant_gemm", "hip_fused"):
        with pytest.raises(RuntimeError, match="CUDA tensor"):
            A.ARCQPackedLinear(_source(), fmt)(x)
    otf = A.ARCQPackedLinearOnTheFly.from_packed(A.ARCQPackedLinear(_source()))
    with pytest.raises(RuntimeError, match="CUDA"):
        otf(x)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        A.pack_codes(torch.zeros(2, 8, dtype=torch.int64), 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        A.quantize_activation(x, torch.zeros(15), torch.zeros(16), 4, 64)


def test_on_the_fly_module():
    packed = A.ARCQPackedLinear(_source())
    otf = A.ARCQPackedLinearOnTheFly.from_packed(packed)
    assert list(otf.state_dict()) == ["packed_weight_codes", "weight_codebook", "weight_center", "weight_scale",
                                      "weight_code_sum", "activation_codebook", "activation_thresholds", "bias_tensor"]
    assert otf.groups == 2 and otf.bits == 4 and otf.group_size == 64
    assert otf.packed_weight_codes.data_ptr() == packed.packed_weight_codes.data_ptr()     # shared, not copied
    want_mb = sum(b.numel() * b.element_size() for b in otf.buffers()) / 1024 / 1024
    assert abs(otf.estimated_persistent_mb() - want_mb) < 1e-12
    otf.half()                                                                            # half-chain cast
    assert all(b.dtype == torch.float32 for n, b in otf.named_buffers() if n != "packed_weight_codes")
    nb = A.ARCQPackedLinearOnTheFly(128, 24, False, packed.packed_weight_codes, packed.weight_codebook,
                                    packed.weight_center, packed.weight_scale, packed.weight_code_sum,
                                    packed.activation_codebook, packed.activation_thresholds, 4, 64, None)
    assert nb.bias_tensor.numel() == 0
    with pytest.raises(ValueError, match="packed_weight_codes has shape"):
        A.ARCQPackedLinearOnTheFly(256, 24, False, packed.packed_weight_codes, packed.weight_codebook,
                                   packed.weight_center, packed.weight_scale, packed.weight_code_sum,
                                   packed.activation_codebook, packed.activation_thresholds, 4, 64, None)


def test_convert_model_and_checkpoint_roundtrip(tmp_path, oracle):
    vit = build_fakequant_vit("deit_tiny", 4, num_classes=10)
    assert sum(m.__class__.__name__ == "QuantLinearPCARCQ" for m in vit.modules()) == 48
    A.convert_arcq_linear_to_packed(vit, "packed")
    assert A.count_packed_linear(vit) == 48
    assert A.count_packed_linear(A.convert_arcq_linear_to_packed(vit, "dequant_gemm")) == 48   # 2nd pass: nothing left
    assert all(m.runtime_code_format == "packed" for m in vit.modules() if isinstance(m, A.ARCQPackedLinear))
    sd = vit.state_dict()
    assert "blocks.3.mlp.fc1.packed_weight_codes" in sd and "blocks.0.attn.qkv.product_table" in sd
    assert tuple(sd["blocks.3.mlp.fc1.packed_weight_codes"].shape) == (768, 96)
    path = tmp_path / "deit_tiny_w4a4_packed.pt"
    torch.save({"module." + k: v for k, v in sd.items()}, path)                # DDP-style prefix

    hp = A.infer_packed_hparams(sd["blocks.3.mlp.fc2.packed_weight_codes"], sd["blocks.3.mlp.fc2.weight_center"],
                                sd["blocks.3.mlp.fc2.weight_codebook"])
    assert hp == {"in_features": 768, "out_features": 192, "bits": 4, "group_size": 64}

    from arcq_vit_amd.vit import VisionTransformer
    fresh = VisionTransformer(192, 12, 3, 768, num_classes=10)
    loaded = torch.load(path, weights_only=True)
    A.load_packed_state_dict(fresh, loaded, on_the_fly=True)
    otf = fresh.blocks[3].mlp.fc1
    assert isinstance(otf, A.ARCQPackedLinearOnTheFly) and (otf.in_features, otf.out_features) == (192, 768)
    assert torch.equal(otf.packed_weight_codes, sd["blocks.3.mlp.fc1.packed_weight_codes"])
    assert torch.equal(otf.bias_tensor, sd["blocks.3.mlp.fc1.bias"])
    assert torch.equal(fresh.pos_embed, vit.pos_embed) and torch.equal(fresh.head.weight, vit.head.weight)
    # the on-the-fly spelling (bias_tensor) loads too, into either module kind
    fresh2 = VisionTransformer(192, 12, 3, 768, num_classes=10)
    A.load_packed_state_dict(fresh2, fresh.state_dict(), on_the_fly=False, runtime_code_format="u8")
    pl = fresh2.blocks[0].attn.qkv
    assert isinstance(pl, A.ARCQPackedLinear) and pl.weight_codes_u8.shape == (576, 192)
    assert torch.equal(pl.bias, sd["blocks.0.attn.qkv.bias"])
    bad = dict(sd)
    bad["blocks.99.attn.qkv.packed_weight_codes"] = sd["blocks.0.attn.qkv.packed_weight_codes"]
    with pytest.raises(KeyError, match="blocks.99"):
        A.load_packed_state_dict(VisionTransformer(192, 12, 3, 768, num_classes=10), bad)


def test_three_bit_conversion_sizes():
    layer = A.ARCQPackedLinear(_source(in_f=384, out_f=16, bits=3))
    assert tuple(layer.packed_weight_codes.shape) == (16, 144)
    hp = A.infer_packed_hparams(layer.packed_weight_codes, layer.weight_center, layer.weight_codebook)
    assert hp == {"in_features": 384, "out_features": 16, "bits": 3, "group_size": 64}
    with pytest.raises(ValueError):
        A.infer_packed_hparams(layer.packed_weight_codes, layer.weight_center, torch.zeros(5))
    # 3-bit rows that end inside a byte: K = 35 in groups of 7 packs into ceil(105 / 8) = 14 bytes, and so would 36 and
    # 37 (the number of groups decides); K = 6, 7 or 8 in ONE group all pack into 3 bytes and cannot be told apart
    cb8 = torch.zeros(8)
    hp = A.infer_packed_hparams(torch.zeros(4, 14, dtype=torch.uint8), torch.zeros(4, 5), cb8)
    assert hp == {"in_features": 35, "out_features": 4, "bits": 3, "group_size": 7}
    with pytest.raises(ValueError, match="ambiguous"):
        A.infer_packed_hparams(torch.zeros(4, 3, dtype=torch.uint8), torch.zeros(4, 1), cb8)
    with pytest.raises(ValueError, match="inconsistent"):
        A.infer_packed_hparams(torch.zeros(4, 14, dtype=torch.uint8), torch.zeros(4, 11), cb8)


def test_fake_quant_source_matches_oracle(oracle):
    src = _source(in_f=192, out_f=32, bits=4)
    x = synth.make_activation(50, 192, 2)
    want = oracle.fake_quant_linear(x, src.linear.weight.detach(), src.linear.bias.detach(),
                                    src.act_quant._pc_thresholds, src.act_quant._pc_cb,
                                    src.weight_quant._pc_thresholds, src.weight_quant._pc_cb, 64, 1e-6)
    assert torch.equal(src(x), want)
    x3 = x.reshape(5, 10, 192)
    assert torch.equal(src(x3).reshape(50, 32), want)            # any leading dims
    q = A.FrozenARCQQuantizer(4, 64)
    with pytest.raises(RuntimeError, match="no compiled codebook"):
        q(x)
    q8 = A.FrozenARCQQuantizer(8, 64)
    assert q8(x) is x                                              # bits >= 8 is a pass-through (Q/dcarcq.py:513-514)


# ------------------------------------------------------------------------------------------------
# synthetic generators and work accounting
# ------------------------------------------------------------------------------------------------
def test_synth():
    for bits in (2, 3, 4):
        cb = synth.quantile_codebook(bits)
        thr = synth.midpoint_thresholds(cb)
        assert cb.dtype == torch.float32 and cb.numel() == 1 << bits and bool((cb[1:] > cb[:-1]).all())
        assert torch.allclose(cb, -cb.flip(0), atol=1e-6) and thr.numel() == cb.numel() - 1
    assert abs(float(synth.quantile_codebook(4)[-1]) - 1.8627) < 1e-3
    x = synth.make_activation(2000, 384, 0)
    frac = float((x.abs() == 8.0).float().mean())
    assert 0.003 < frac < 0.007 and torch.equal(x, synth.make_activation(2000, 384, 0))
    g = synth.make_activation(2000, 384, 0, "gelu")
    assert float(g.min()) > -0.2 and float(g.mean()) > 0.2
    w = synth.make_weight(256, 256, 0)
    assert abs(float(w.std()) - 0.02) < 1e-3
    img = synth.make_images(2, 0)
    assert tuple(img.shape) == (2, 3, 224, 224) and -2.2 < float(img.min()) and float(img.max()) < 2.7
    # algorithmic bytes/flops of the DeiT-S qkv shape at batch 1 and batch 64
    assert synth.algorithmic_bytes(197, 1152, 384, 4) == 914108
    assert synth.algorithmic_bytes(12608, 1152, 384, 4) == 39040700
    assert synth.algorithmic_bytes(197, 384, 1536, 4) == 1163708
    assert synth.algorithmic_bytes(197, 1152, 384, 3) == 858716
    assert synth.algorithmic_flops(12608, 1536, 384) == 2 * 12608 * 1536 * 384
    assert [s[1:] for s in synth.block_linear_shapes("deit_small")] == [(384, 1152), (384, 384), (384, 1536), (1536, 384)]


def test_fused_kernel_choice_is_reported_without_a_gpu(monkeypatch):
    """arcq_linear_fused_kernel is a pure function of the shape (and of the ARCQ_GEMM_KERNEL override)."""
    lib = A._lib.load()
    monkeypatch.delenv("ARCQ_GEMM_KERNEL", raising=False)
    assert lib.arcq_linear_fused_kernel(197, 1152, 384) == b"gemm_splitk_kernel"
    assert lib.arcq_linear_fused_kernel(12608, 1152, 384) == b"gemm_stream_kernel"      # wide N, one round of tiles
    assert lib.arcq_linear_fused_kernel(12608, 384, 1536) == b"gemm_slab_kernel"        # few slabs, many row ranges
    assert lib.arcq_linear_fused_kernel(12608, 1536, 384) == b"gemm_slab_kernel"        # K in one slab slice
    assert lib.arcq_linear_fused_kernel(50432, 4096, 1024) == b"gemm_stream_kernel"
    assert lib.arcq_linear_fused_kernel(5, 5, 0) == b"gemm_fused_kernel"                # K = 0: bias only
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "slab")
    assert lib.arcq_linear_fused_kernel(12608, 1152, 384) == b"gemm_slab_kernel"
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "stream")
    assert lib.arcq_linear_fused_kernel(12608, 384, 384) == b"gemm_stream_kernel"
    # With a weight workspace: long K and few slabs rebuild the weights once, everything else is unchanged.
    both = b"weight_dequant8_kernel+gemm_slab_kernel"
    assert lib.arcq_linear_fused_ws_kernel(12608, 384, 1536, 1) == b"gemm_stream_kernel"   # a pinned kernel wins
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    assert lib.arcq_linear_fused_ws_kernel(12608, 384, 1536, 1) == both
    assert lib.arcq_linear_fused_ws_kernel(12608, 384, 1536, 0) == b"gemm_slab_kernel"
    assert lib.arcq_linear_fused_ws_kernel(12608, 1536, 384, 1) == b"gemm_slab_kernel"     # K in one slice
    assert lib.arcq_linear_fused_ws_kernel(50432, 4096, 1024, 1) == b"gemm_stream_kernel"  # 32 slabs
    assert lib.arcq_linear_fused_ws_kernel(50432, 1024, 4096, 1) == both
    assert lib.arcq_linear_fused_ws_kernel(197, 384, 1536, 1) == b"gemm_splitk_kernel"     # below 512 rows
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "prebuilt")
    assert lib.arcq_linear_fused_ws_kernel(12608, 1152, 384, 1) == both
    assert lib.arcq_linear_fused_ws_kernel(12608, 1152, 384, 0) == b"gemm_stream_kernel"
    # The whole-layer entry point with scratch workspaces: whole 32-row blocks from 512 rows on take the block layout.
    monkeypatch.delenv("ARCQ_GEMM_KERNEL")
    both8 = b"gemm_slab8_kernel<copy>"
    rows = b"otf_rows_kernel"         # rows that fit LDS whole (K = 192 / 256 / 384 / 768) and both workspaces: one launch
    assert lib.arcq_linear_otf_ws_kernel(12608, 1152, 384, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(12608, 576, 192, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(512, 576, 192, 1) == rows                          # few weights: from 512 rows on
    assert lib.arcq_linear_otf_ws_kernel(1024, 384, 384, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(6304, 1152, 384, 1) == rows                        # many weights: where it beats two launches
    assert lib.arcq_linear_otf_ws_kernel(6144, 1152, 384, 1) == both8
    assert lib.arcq_linear_otf_ws_kernel(6976, 1536, 384, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(6720, 1536, 384, 1) == both8
    assert lib.arcq_linear_otf_ws_kernel(4480, 1024, 256, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(12608, 1152, 320, 1) == both8                     # (no instance for five groups)
    assert lib.arcq_linear_otf_ws_kernel(12608, 1000, 384, 1) == both8                     # (N must be whole 32-column blocks)
    monkeypatch.setenv("ARCQ_ROWS", "0")
    assert lib.arcq_linear_otf_ws_kernel(12608, 1152, 384, 1) == both8                     # the rebuild rides in stage 1
    monkeypatch.delenv("ARCQ_ROWS")
    assert lib.arcq_linear_otf_ws_kernel(12608, 1152, 384, 0) == b"gemm_slab8_kernel"
    # One workgroup per 64 rows must be resident at once (256 compute units; two workgroups each for K = 192).
    assert lib.arcq_linear_otf_ws_kernel(16384, 1152, 384, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(16448, 1152, 384, 1) == both8
    assert lib.arcq_linear_otf_ws_kernel(32768, 576, 192, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(32832, 576, 192, 1) == both8
    # Long rows and at most 384 outputs (fc2 of the small models): one launch, the row taken in slices of 384 values,
    # from the number of row tiles on at which it beats the two launches.
    phased = b"otf_rows_phased_kernel"
    assert lib.arcq_linear_otf_ws_kernel(12608, 384, 1536, 1) == phased
    assert lib.arcq_linear_otf_ws_kernel(12608, 192, 768, 1) == phased
    assert lib.arcq_linear_otf_ws_kernel(8192, 384, 1536, 1) == phased                     # 128 row tiles
    assert lib.arcq_linear_otf_ws_kernel(8128, 384, 1536, 1) == both8
    assert lib.arcq_linear_otf_ws_kernel(5504, 384, 768, 1) == phased                      # 86 row tiles
    assert lib.arcq_linear_otf_ws_kernel(5440, 384, 768, 1) != phased
    assert lib.arcq_linear_otf_ws_kernel(16448, 384, 1536, 1) == both8                     # (not resident at once)
    assert lib.arcq_linear_otf_ws_kernel(12608, 416, 1536, 1) == both8                     # (more than twelve column blocks)
    monkeypatch.setenv("ARCQ_ROWS", "0")
    assert lib.arcq_linear_otf_ws_kernel(12608, 384, 1536, 1) == both8
    monkeypatch.delenv("ARCQ_ROWS")
    assert lib.arcq_linear_otf_ws_kernel(12608, 384, 1536, 0) == b"gemm_slab8_kernel"
    # K = 768 with more than 384 outputs (the DeiT-B widths): the whole-row kernel, two stage-1 tiles per wave
    assert lib.arcq_linear_otf_ws_kernel(12608, 768, 768, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(12608, 2304, 768, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(12608, 3072, 768, 1) == rows
    assert lib.arcq_linear_otf_ws_kernel(16448, 2304, 768, 1) != rows                      # (not resident at once)
    assert lib.arcq_linear_otf_ws_kernel(4096, 2304, 768, 1) != rows                       # (few rows: two launches are faster)
    assert lib.arcq_linear_otf_ws_kernel(12608, 768, 3072, 1) == phased                    # K = 3072: up to 768 outputs
    assert lib.arcq_linear_otf_ws_kernel(8192, 768, 3072, 1) == phased                     # 128 row tiles
    assert lib.arcq_linear_otf_ws_kernel(8128, 768, 3072, 1) != phased
    assert lib.arcq_linear_otf_ws_kernel(12608, 800, 3072, 1) != phased
    pair = b"gemm_pair_kernel"        # several slices and at least eight row blocks per workgroup: two blocks per wave
    assert lib.arcq_linear_otf_ws_kernel(12608, 1024, 3072, 1) == pair                     # sixteen slices, eight slabs
    assert lib.arcq_linear_otf_ws_kernel(50432, 4096, 1024, 1) == pair                     # three slices
    monkeypatch.setenv("ARCQ_ROWS", "0")
    assert lib.arcq_linear_otf_ws_kernel(12608, 2304, 768, 1) == pair
    assert lib.arcq_linear_otf_ws_kernel(12608, 2304, 768, 0) == b"gemm_slab8_kernel"      # (needs the weights ready)
    monkeypatch.setenv("ARCQ_PAIR", "0")
    assert lib.arcq_linear_otf_ws_kernel(12608, 2304, 768, 1) == both8
    monkeypatch.delenv("ARCQ_PAIR")
    monkeypatch.delenv("ARCQ_ROWS")
    assert lib.arcq_linear_otf_ws_kernel(1576, 384, 1536, 1) == both8                      # a ragged last block is fine
    assert lib.arcq_linear_otf_ws_kernel(197, 1152, 384, 1) == b"gemm_splitk_kernel"
    monkeypatch.setenv("ARCQ_GEMM_KERNEL", "stream")
    assert lib.arcq_linear_otf_ws_kernel(12608, 1152, 384, 1) == b"gemm_stream_kernel"


def test_block_layout_entry_points_validate_before_launching():
    """Argument errors of the block-layout entry points come back as codes without touching a GPU."""
    import ctypes
    lib = A._lib.load()
    buf = (ctypes.c_char * 256)()
    p = ctypes.addressof(buf) & ~15
    F16 = A._lib.ARCQ_F16
    assert lib.arcq_act_quant_blocked(p, F16, p, p, p + 64, -1, 64, 4, 1e-6, None) == -4
    assert lib.arcq_act_quant_blocked(p, F16, p, p, p + 64, 32, 96, 4, 1e-6, None) == -2       # cols % 64
    assert lib.arcq_act_quant_blocked(p, F16, p, p, p + 64, 32, 64, 5, 1e-6, None) == -1       # bits
    assert lib.arcq_act_quant_blocked(p, F16, p, p, None, 32, 64, 4, 1e-6, None) == -3         # NULL output
    assert lib.arcq_act_quant_blocked(p, F16, p, p, p, 32, 64, 4, 1e-6, None) == -6            # in place is not possible
    assert lib.arcq_act_quant_blocked(p, F16, p, p, p + 64, 0, 64, 4, 1e-6, None) == 0         # empty
    args = lambda m, n, k, bits=4, gs=64, ready=0: (p, p, p, p, p, p, None, None, ready, p + 64, F16, m, n, k, bits, gs, None)
    assert lib.arcq_linear_fused_blocked(*args(-1, 8, 64)) == -4
    assert lib.arcq_linear_fused_blocked(*args(32, 8, 96)) == -2
    assert lib.arcq_linear_fused_blocked(*args(32, 8, 64, gs=32)) == -6
    assert lib.arcq_linear_fused_blocked(*args(32, 8, 64, bits=1)) == -1
    assert lib.arcq_linear_fused_blocked(*args(0, 8, 64)) == 0
    assert lib.arcq_linear_fused_blocked(*args(32, 8, 64, ready=1)) == -3                      # ready without a buffer
    wargs = lambda n, w_hat=p + 128: (p, F16, p, p, p + 64, 32, 64, 4, 1e-6, p, p, p, p, p, w_hat, n, None)
    assert lib.arcq_act_quant_blocked_with_weights(*wargs(8, None)) == -3
    assert lib.arcq_act_quant_blocked_with_weights(*wargs(8, p + 130)) == -7
    assert lib.arcq_act_quant_blocked_with_weights(*wargs(-1)) == -4


def test_bench_host_side_contract():
    """bench.py without a GPU: more than one GPU is refused with a message, and the committed rocprofv3 summaries
    hold a traffic line for the kernel that dominates each benchmarked configuration (bench.py's roofline.traffic
    is read from them, so a renamed kernel must not turn it into null unnoticed)."""
    import subprocess
    import sys
    from pathlib import Path
    root = Path(__file__).resolve().parents[1]
    proc = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2 and "one GPU" in proc.stderr and not proc.stdout.strip()
    sys.path.insert(0, str(root))
    try:
        import bench
    finally:
        sys.path.pop(0)
    for (model, bits, batch), kernels in {("deit_small", 4, 64): ("otf_rows_kernel", "otf_rows_phased_kernel"),
                                          ("deit_base", 4, 64): ("gemm_pair_kernel",),
                                          ("vit_large", 3, 256): ("gemm_pair_kernel",)}.items():
        for kernel in kernels:
            traffic = bench.profiled_traffic(model, bits, batch, kernel)
            assert traffic is not None and traffic > 1e6, (model, kernel)
    assert bench.profiled_traffic("deit_small", 4, 64, "no_such_kernel") is None


def test_rows_counter_slot_logic():
    """The table that gives every weight workspace its own counter word: a key keeps its slot, distinct keys never
    share one, a full table refuses further keys, and a collision moves on along the probe sequence."""
    import ctypes
    from arcq_vit_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("library not built")
    lib = _lib.load()
    slots = 64
    table = (ctypes.c_void_p * slots)()
    keys = [0x7f0000000000 + 256 * i * 4099 for i in range(slots)]
    got = [lib.arcq_rows_counter_slot(table, slots, k) for k in keys]
    assert sorted(got) == list(range(slots))                      # all distinct, table now full
    assert [lib.arcq_rows_counter_slot(table, slots, k) for k in keys] == got      # stable
    assert lib.arcq_rows_counter_slot(table, slots, 0x7e0000000100) == -1           # full: the caller falls back
    assert lib.arcq_rows_counter_slot(table, slots, None) == -1
    small = (ctypes.c_void_p * 2)()
    a = lib.arcq_rows_counter_slot(small, 2, 0x1000)
    b = lib.arcq_rows_counter_slot(small, 2, 0x2000)
    assert {a, b} == {0, 1} and lib.arcq_rows_counter_slot(small, 2, 0x3000) == -1


def test_linear_ex_args_mirror_the_header():
    """``_lib.LinearExArgs`` must list the fields of ``arcq_linear_ex_args`` (include/arcq_hip.h) in the header's order
    with the header's types: all the 32-bit fields are the same size, so a swapped pair would not show anywhere else."""
    import ctypes
    import re
    from arcq_vit_amd import _lib
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "include", "arcq_hip.h")).read()
    body = re.search(r"typedef struct arcq_linear_ex_args \{(.*?)\} arcq_linear_ex_args;", text, re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    want = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        m = re.match(r"(const )?(uint32_t|int32_t|int64_t|float|void|uint8_t) (.*)", decl)
        assert m, decl
        base = m.group(2)
        for name in m.group(3).split(","):
            name = name.strip()
            pointer = name.startswith("*")
            ctype = ctypes.c_void_p if pointer else {"uint32_t": ctypes.c_uint32, "int32_t": ctypes.c_int32,
                                                     "int64_t": ctypes.c_int64, "float": ctypes.c_float}[base]
            want.append((name.lstrip("*"), ctype))
    assert [(n, t) for n, t in _lib.LinearExArgs._fields_] == want
