"""arcq_linear_otf_static -- the whole on-the-fly layer with both scratch buffers in the library's static device
array, for callers that cannot allocate -- against arcq_linear_otf_ws, through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

import arcq_vit_amd as A
from arcq_vit_amd import _lib, synth
from arcq_vit_amd._lib import ARCQ_F16, ARCQ_F32, ARCQ_STATIC_SCRATCH_BYTES

pytestmark = pytest.mark.gpu


def _layer(oracle, n, k, bits, seed, dev):
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    codes, wc, ws, wcs = oracle.quantize_weight_torch(synth.make_weight(n, k, seed), thr, cb, 64, 1e-6)
    t = {"thr": thr, "cb": cb, "pw": A.pack_codes_py(codes, bits), "wc": wc, "ws": ws, "wcs": wcs,
         "bias": synth.make_bias(n, seed)}
    return {name: v.to(dev) for name, v in t.items()}


def _free_bytes():
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    hip = ctypes.CDLL("libamdhip64.so")
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _call(lib, static, x, L, y, m, n, k, bits, x_ws=None, w_ws=None):
    st = torch.cuda.current_stream().cuda_stream
    xd = ARCQ_F16 if x.dtype == torch.float16 else ARCQ_F32
    yd = ARCQ_F16 if y.dtype == torch.float16 else ARCQ_F32
    head = (x.data_ptr(), xd, L["thr"].data_ptr(), L["cb"].data_ptr(), L["pw"].data_ptr(), L["cb"].data_ptr(),
            L["wc"].data_ptr(), L["ws"].data_ptr(), L["wcs"].data_ptr(), L["bias"].data_ptr())
    tail = (y.data_ptr(), yd, m, n, k, bits, 64, st)
    if static:
        return lib.arcq_linear_otf_static(*head, *tail)
    return lib.arcq_linear_otf_ws(*head, x_ws.data_ptr(), w_ws.data_ptr(), *tail)


def test_static_scratch_layer_matches_workspace_layer(cuda, oracle):
    lib = _lib.load()
    # two calls in a row on one stream; the second is smaller (it reuses the front of the array, whose rest still
    # holds the first call's data) and takes the single-launch path; then a ragged large one with fp32 in and out
    cases = [(12608, 384, 1536, 4, torch.float16, torch.float16),
             (197, 1152, 384, 3, torch.float16, torch.float16),
             (1576, 768, 192, 2, torch.float32, torch.float32)]
    layers = [_layer(oracle, n, k, bits, 60 + i, cuda) for i, (m, n, k, bits, _, _) in enumerate(cases)]
    xs = [synth.make_activation(m, k, 70 + i, "gelu" if k > n else "ln").to(dt).to(cuda)
          for i, (m, n, k, bits, dt, _) in enumerate(cases)]
    ys = [torch.zeros((m, n), dtype=odt, device=cuda) for (m, n, k, bits, _, odt) in cases]
    wants = [torch.zeros_like(y) for y in ys]
    # reference results from the entry point that takes caller-owned workspaces
    for (m, n, k, bits, _, _), L, x, want in zip(cases, layers, xs, wants):
        x_ws = torch.empty(m * k, dtype=torch.float16, device=cuda)
        w_ws = torch.empty(n * k, dtype=torch.float16, device=cuda)
        assert _call(lib, False, x, L, want, m, n, k, bits, x_ws, w_ws) == 0
    torch.cuda.synchronize()
    # first call resolves the array's address on this device; after it, calls must not change device memory use
    m, n, k, bits, _, _ = cases[1]
    assert _call(lib, True, xs[1], layers[1], ys[1], m, n, k, bits) == 0, lib.arcq_last_error()
    torch.cuda.synchronize()
    ys[1].zero_()
    free0, alloc0 = _free_bytes(), torch.cuda.memory_allocated()
    for (m, n, k, bits, _, _), L, x, y in zip(cases, layers, xs, ys):          # back to back, no sync in between
        assert _call(lib, True, x, L, y, m, n, k, bits) == 0, lib.arcq_last_error()
    torch.cuda.synchronize()
    assert _free_bytes() == free0 and torch.cuda.memory_allocated() == alloc0
    for y, want, case in zip(ys, wants, cases):
        assert torch.equal(y, want), case
    # and against the oracle on sampled rows of the large case
    m, n, k, bits, _, _ = cases[0]
    L = layers[0]
    rows = torch.randint(0, m, (32,), generator=torch.Generator().manual_seed(1))
    a = oracle.act_quant_c(xs[0][rows.to(cuda)].float().cpu().numpy(), L["thr"].cpu(), L["cb"].cpu(), bits, 64)["x_hat"]
    w16 = oracle.weight_dequant_c(L["pw"].cpu().numpy(), L["cb"].cpu(), L["wc"].cpu(), L["ws"].cpu(), L["wcs"].cpu(),
                                  bits, 64, fma=True).astype(np.float16)
    y64, mag = oracle.linear_f64_c(a.astype(np.float16), w16, L["bias"].cpu().numpy())
    tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * 2.0 ** -11 + 2.0 ** -25
    assert np.all(np.abs(ys[0][rows.to(cuda)].cpu().numpy().astype(np.float64) - y64) <= tol)


def test_static_scratch_limit_and_errors(cuda, oracle):
    lib = _lib.load()
    L = _layer(oracle, 64, 64, 4, 1, cuda)
    x = torch.zeros((1, 64), dtype=torch.float16, device=cuda)
    y = torch.zeros((1, 64), dtype=torch.float16, device=cuda)
    # DeiT-B fc2 at batch 64 needs 77 MB of x_hat: rejected with an argument error, nothing launched
    m, n, k = 12608, 768, 3072
    assert 2 * m * k > ARCQ_STATIC_SCRATCH_BYTES
    rc = _call(lib, True, x, L, y, m, n, k, 4)
    assert rc == -4 and b"static scratch" in lib.arcq_last_error()
    assert _call(lib, True, x, L, y, -1, 64, 64, 4) == -4
    assert _call(lib, True, x, L, y, 1, 64, 64, 5) == -1          # argument checks of the layer itself still apply
    assert _call(lib, True, x, L, y, 0, 64, 64, 4) == 0           # empty input: nothing to do
    # the largest DeiT-S layer at batch 64 fits
    assert (1536 * 384 * 2 + 255) // 256 * 256 + 12608 * 1536 * 2 <= ARCQ_STATIC_SCRATCH_BYTES
