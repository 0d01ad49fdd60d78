"""GPU tests of the one-launch row-stationary layer kernels (``otf_rows_kernel``: stage 1 into LDS, weights rebuilt
cooperatively into the workspace in 32-column blocks, product from there; ``otf_rows_phased_kernel``: the same for
rows of 768 / 1536 values, quantized in slices of 384 while the previous slice is multiplied)."""
import numpy as np
import pytest
import torch

import arcq_vit_amd as A
from arcq_vit_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def _np(t):
    return t.detach().cpu().numpy()


def _layer(oracle, n, k, bits, seed):
    cb = synth.quantile_codebook(bits)
    thr = synth.midpoint_thresholds(cb)
    w = synth.make_weight(n, k, seed)
    codes, wc, ws, wcs = oracle.quantize_weight_torch(w, thr, cb, 64, 1e-6)
    return cb, thr, A.pack_codes_py(codes, bits), wc, ws, wcs, synth.make_bias(n, seed + 1)


def _w_blocked(w16):
    """Row-major [N, K] -> the 32-column block layout of the weight workspace, flat: [N/32][K/8][32][8]."""
    n, k = w16.shape
    return np.ascontiguousarray(w16.reshape(n // 32, 32, k // 8, 8).transpose(0, 2, 1, 3)).reshape(-1)


@pytest.mark.parametrize("m,n,k,bits,out", [(12608, 1152, 384, 4, torch.float16), (12608, 384, 384, 4, torch.float16),
                                            (12608, 1536, 384, 3, torch.float16), (12608, 576, 192, 4, torch.float16),
                                            (1001, 96, 192, 2, torch.float32), (5000, 1024, 256, 3, torch.float16),
                                            (577, 32, 384, 4, torch.float32),
                                            (12608, 384, 1536, 4, torch.float16), (12608, 192, 768, 3, torch.float32),
                                            (9000, 96, 1536, 2, torch.float16), (6001, 384, 768, 4, torch.float32),
                                            (12608, 2304, 768, 4, torch.float16), (12608, 768, 768, 3, torch.float16),
                                            (9001, 3072, 768, 2, torch.float16),
                                            (12608, 768, 3072, 4, torch.float16), (8200, 416, 3072, 3, torch.float32)])
def test_rows_kernel_against_oracle_and_two_launch_path(cuda, oracle, monkeypatch, m, n, k, bits, out):
    """The kernel's y against the fp64 oracle on sampled rows (fp32-accumulation bound plus the output rounding),
    the weight workspace against the oracle's w_hat bit for bit (block layout), and y bit for bit against the
    two-launch path (stage 1 into the block layout, weight-stationary GEMM)."""
    cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, bits, 31)
    x = synth.make_activation(m, k, 33, "ln").to(torch.float16)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    # (K = 768 with more than 384 outputs: the whole-row kernel with two stage-1 tiles per wave, fp16 outputs only;
    # K = 3072 with up to 768 outputs: the phased kernel with three column blocks per wave)
    kernel = b"otf_rows_kernel" if k <= 384 or (k == 768 and n > 384) else b"otf_rows_phased_kernel"
    assert _lib.load().arcq_linear_otf_ws_kernel(m, n, k, 1) == kernel
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    y = ops.linear_otf(d(x), *args, out_dtype=out, w_hat_ws=w_ws)
    torch.cuda.synchronize()
    w16 = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True).astype(np.float16)
    assert np.array_equal(_np(w_ws).view(np.uint16), _w_blocked(w16).view(np.uint16))
    rows = torch.randint(0, m, (64,), generator=torch.Generator().manual_seed(3))
    rows[0], rows[1] = 0, m - 1
    a = oracle.act_quant_c(x[rows].float().numpy(), thr, cb, bits, 64)["x_hat"].astype(np.float16)
    y64, mag = oracle.linear_f64_c(a, w16, bias.numpy())
    ulp = 2.0 ** -11 if out == torch.float16 else 2.0 ** -24
    tol = (k + 2) * 2.0 ** -24 * mag + np.abs(y64) * ulp + 2.0 ** -25
    err = np.abs(_np(y[rows.to(cuda)]).astype(np.float64) - y64)
    assert np.all(err <= tol), float((err / tol).max())
    # a weight workspace that is not 128-byte aligned (a view 16 bytes into a buffer) takes the two-launch path
    off = torch.zeros(n * k + 8, dtype=torch.float16, device=cuda)[8:]
    y1 = ops.linear_otf(d(x), *args, out_dtype=out, w_hat_ws=off)
    assert torch.equal(y, y1) and np.array_equal(_np(off).view(np.uint16), w16.reshape(-1).view(np.uint16))
    monkeypatch.setenv("ARCQ_ROWS", "0")
    assert _lib.load().arcq_linear_otf_ws_kernel(m, n, k, 1) != kernel
    y2 = ops.linear_otf(d(x), *args, out_dtype=out, w_hat_ws=torch.zeros_like(w_ws))
    assert torch.equal(y, y2)


@pytest.mark.parametrize("m,n,k", [(16448, 384, 384), (20032, 384, 1536)])
def test_more_row_tiles_than_the_device_holds_take_the_two_launch_path(cuda, oracle, monkeypatch, m, n, k):
    """A workgroup of the one-launch kernels waits for the weight shares of all the others, so a launch larger than
    the device holds at once would stall until the wait gives up.  Such calls must take the two-launch path: the
    weight workspace then comes back row-major, and y has the bits of the call with the one-launch kernels off."""
    cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, 4, 71)
    x = synth.make_activation(m, k, 73, "ln").to(torch.float16).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), 4, 64)
    assert not _lib.load().arcq_linear_otf_ws_kernel(m, n, k, 1).startswith(b"otf_rows")
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    y = ops.linear_otf(x, *args, out_dtype=torch.float16, w_hat_ws=w_ws)
    w16 = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, 4, 64, fma=True).astype(np.float16)
    assert np.array_equal(_np(w_ws).view(np.uint16), w16.reshape(-1).view(np.uint16))
    monkeypatch.setenv("ARCQ_ROWS", "0")
    assert torch.equal(y, ops.linear_otf(x, *args, out_dtype=torch.float16, w_hat_ws=w_ws))


@pytest.mark.parametrize("m,n,k,bits,out", [(6016, 768, 384, 4, torch.float16), (6016, 768, 384, 3, torch.float32),
                                            (12608, 2304, 768, 4, torch.float16), (9000, 1536, 768, 3, torch.float16)])
def test_rows_kernel_with_layernorm_gelu_residual(cuda, oracle, monkeypatch, m, n, k, bits, out):
    """arcq_linear_otf_ex through the one-launch kernel: LayerNorm in front, GELU and the skip connection behind,
    bit for bit what the two-launch path gives (whose parts are checked against the oracle elsewhere) and what the
    separate torch operations give around the plain layer."""
    assert _lib.load().arcq_linear_otf_ws_kernel(m, n, k, 1) == b"otf_rows_kernel"
    cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, bits, 41)
    g = torch.Generator().manual_seed(9)
    x = (synth.make_activation(m, k, 43, "ln") * 1.7 + 0.3).to(torch.float16).to(cuda)
    lw = (1 + 0.1 * torch.randn(k, generator=g)).to(cuda)
    lb = (0.1 * torch.randn(k, generator=g)).to(cuda)
    res = torch.randn(m, n, generator=g).to(out).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    kw = dict(out_dtype=out, layernorm=(lw, lb, 1e-6), gelu=True, residual=res, w_hat_ws=w_ws)
    y = ops.linear_otf_ex(x, *args, **kw)
    monkeypatch.setenv("ARCQ_ROWS", "0")
    y2 = ops.linear_otf_ex(x, *args, **kw)
    assert torch.equal(y, y2)
    # the unfused sequence in torch around the plain layer (LayerNorm in fp32 arithmetic on fp16 data, as the kernel)
    ln = torch.nn.functional.layer_norm(x.float(), (k,), lw, lb, 1e-6).to(torch.float16)
    plain = ops.linear_otf(ln, *args, out_dtype=out, w_hat_ws=w_ws)
    ref = torch.nn.functional.gelu(plain).to(out) + res
    close = (y.float() - ref.float()).abs() <= 2.0 ** -9 * ref.float().abs() + 1e-3
    assert float(close.float().mean()) > 0.999        # torch's LayerNorm may round a value differently: rare code flips


@pytest.mark.parametrize("n,k,bits,out", [(384, 1536, 4, torch.float16), (192, 768, 3, torch.float32),
                                          (768, 3072, 4, torch.float16)])
def test_phased_kernel_with_gelu_and_residual(cuda, oracle, monkeypatch, n, k, bits, out):
    """arcq_linear_otf_ex on the fc2 shapes: GELU and the skip connection in the one-launch kernel's epilogue give the
    bits of the two-launch path and of the separate torch operations behind the plain layer; a LayerNorm in front is
    not something the kernel does, so that call takes the two-launch path (and still agrees)."""
    m = 12608
    cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, bits, 81)
    g = torch.Generator().manual_seed(19)
    x = synth.make_activation(m, k, 83, "gelu").to(torch.float16).to(cuda)
    res = torch.randn(m, n, generator=g).to(out).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    assert _lib.load().arcq_linear_otf_ws_kernel(m, n, k, 1) == b"otf_rows_phased_kernel"
    y = ops.linear_otf_ex(x, *args, out_dtype=out, gelu=True, residual=res, w_hat_ws=w_ws)
    plain = ops.linear_otf(x, *args, out_dtype=out, w_hat_ws=w_ws)
    near = lambda a, b: bool(((a.float() - b.float()).abs() <= 2.0 ** -9 * b.float().abs() + 1e-3).all())
    assert near(y, torch.nn.functional.gelu(plain).to(out) + res)
    assert near(ops.linear_otf_ex(x, *args, out_dtype=out, residual=res, w_hat_ws=w_ws), plain + res)
    lw = (1 + 0.1 * torch.randn(k, generator=g)).to(cuda)
    lb = (0.1 * torch.randn(k, generator=g)).to(cuda)
    kw = dict(out_dtype=out, gelu=True, residual=res, w_hat_ws=w_ws)
    y_ln = ops.linear_otf_ex(x, *args, layernorm=(lw, lb, 1e-6), **kw) if k <= 1024 else None
    monkeypatch.setenv("ARCQ_ROWS", "0")
    assert torch.equal(y, ops.linear_otf_ex(x, *args, **kw))
    if y_ln is not None:
        assert torch.equal(y_ln, ops.linear_otf_ex(x, *args, layernorm=(lw, lb, 1e-6), **kw))


def test_rows_kernel_counter_protocol(cuda, oracle):
    """The cooperative weight reconstruction counts per weight workspace and never resets: many calls in a row, layers of
    different sizes sharing one weight workspace (every call must find the other layer's weights replaced), two
    streams at once, and HIP graph replays with eager calls in between all give the first call's bits."""
    shapes = [(12608, 1152, 384), (12608, 384, 384), (2000, 576, 192), (12608, 384, 1536)]
    layers = []
    for i, (m, n, k) in enumerate(shapes):
        cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, 4, 50 + i)
        d = lambda t: t.to(cuda)
        x = synth.make_activation(m, k, 60 + i, "ln").to(torch.float16).to(cuda)
        layers.append((x, (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), 4, 64)))
    shared = torch.zeros(max(n * k for _, n, k in shapes), dtype=torch.float16, device=cuda)
    first = [ops.linear_otf(x, *a, out_dtype=torch.float16, w_hat_ws=shared.clone()) for x, a in layers]
    for rep in range(6):
        for (x, a), want in zip(layers, first):
            assert torch.equal(ops.linear_otf(x, *a, out_dtype=torch.float16, w_hat_ws=shared), want), rep
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    outs = []
    for rep in range(4):
        for s, (x, a) in ((s1, layers[0]), (s2, layers[1])):
            with torch.cuda.stream(s):
                outs.append((ops.linear_otf(x, *a, out_dtype=torch.float16,
                                            w_hat_ws=torch.zeros(shared.numel(), dtype=torch.float16, device=cuda)),
                             first[0] if s is s1 else first[1]))
    torch.cuda.synchronize()
    assert all(torch.equal(got, want) for got, want in outs)
    # graph replays: the counter's state is whatever the calls before left, also between replays
    x, a = layers[0]
    y = torch.zeros_like(first[0])
    w_ws, x_ws = shared.clone(), torch.zeros(x.numel(), dtype=torch.float16, device=cuda)
    lib = _lib.load()
    F16 = _lib.ARCQ_F16
    sg = torch.cuda.Stream()
    with torch.cuda.stream(sg):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=sg):
            sp = torch.cuda.current_stream().cuda_stream
            thr, cb, pw, wcb, wc, ws, wcs, bias = a[:8]
            for _ in range(3):
                rc = lib.arcq_linear_otf_ws(x.data_ptr(), F16, thr.data_ptr(), cb.data_ptr(), pw.data_ptr(), wcb.data_ptr(),
                                            wc.data_ptr(), ws.data_ptr(), wcs.data_ptr(), bias.data_ptr(), x_ws.data_ptr(),
                                            w_ws.data_ptr(), y.data_ptr(), F16, x.shape[0], 1152, 384, 4, 64, sp)
                assert rc == 0
    for rep in range(3):
        y.zero_()
        w_ws.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, first[0]), rep
        assert torch.equal(ops.linear_otf(layers[1][0], *layers[1][1], out_dtype=torch.float16, w_hat_ws=shared), first[1])
        torch.cuda.synchronize()


@pytest.mark.parametrize("m,n,k,bits", [(12608, 1152, 384, 4), (3000, 576, 192, 3), (12608, 384, 1536, 4),
                                        (12608, 768, 768, 4), (12608, 768, 3072, 3)])
def test_rows_kernels_when_nobody_waits(cuda, oracle, monkeypatch, m, n, k, bits):
    """The wait for the other workgroups' weight shares is bounded; with the bound set to zero every workgroup gives
    up at once and reconstructs all the weights itself (what happens, later, when part of a launch is not resident).
    Same y, same weight workspace, and the calls that follow with the normal bound find the counter in order."""
    cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, bits, 91)
    x = synth.make_activation(m, k, 93, "ln").to(torch.float16).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    assert _lib.load().arcq_linear_otf_ws_kernel(m, n, k, 1).startswith(b"otf_rows")
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    want = ops.linear_otf(x, *args, out_dtype=torch.float16, w_hat_ws=w_ws)
    w_want = w_ws.clone()
    torch.cuda.synchronize()
    timeouts0 = _lib.load().arcq_rows_wait_timeouts()
    assert timeouts0 >= 0
    monkeypatch.setenv("ARCQ_ROWS_WAIT_TICKS", "0")
    for _ in range(3):
        w_ws.zero_()
        assert torch.equal(ops.linear_otf(x, *args, out_dtype=torch.float16, w_hat_ws=w_ws), want)
        assert torch.equal(w_ws, w_want)
    # the diagnostic counter saw the workgroups that gave up (nearly all of them: one that finds the shares complete
    # at its first look does not count), and stands still again under the normal bound
    timeouts1 = _lib.load().arcq_rows_wait_timeouts()
    assert timeouts1 > timeouts0
    monkeypatch.delenv("ARCQ_ROWS_WAIT_TICKS")
    w_ws.zero_()
    assert torch.equal(ops.linear_otf(x, *args, out_dtype=torch.float16, w_hat_ws=w_ws), want)
    assert torch.equal(w_ws, w_want)
    assert _lib.load().arcq_rows_wait_timeouts() == timeouts1


def test_k768_fp32_output_takes_the_two_launch_path(cuda, oracle, monkeypatch):
    """The whole-row kernel for K = 768 has LDS for fp16 staging tiles only: with fp32 outputs the call runs as two
    launches (the weight workspace then holds w_hat row-major) and gives the bits of the call with the one-launch
    kernels switched off."""
    m, n, k, bits = 12608, 1536, 768, 4
    cb, thr, pw, wc, ws, wcs, bias = _layer(oracle, n, k, bits, 51)
    x = synth.make_activation(m, k, 53, "ln").to(torch.float16).to(cuda)
    d = lambda t: t.to(cuda)
    args = (d(thr), d(cb), d(pw), d(cb), d(wc), d(ws), d(wcs), d(bias), bits, 64)
    w_ws = torch.zeros(n * k, dtype=torch.float16, device=cuda)
    y = ops.linear_otf(x, *args, out_dtype=torch.float32, w_hat_ws=w_ws)
    w16 = oracle.weight_dequant_c(pw.numpy(), cb, wc, ws, wcs, bits, 64, fma=True).astype(np.float16)
    assert np.array_equal(_np(w_ws).view(np.uint16), w16.reshape(-1).view(np.uint16))
    y16 = ops.linear_otf(x, *args, out_dtype=torch.float16, w_hat_ws=w_ws)
    assert np.array_equal(_np(w_ws).view(np.uint16), _w_blocked(w16).view(np.uint16))      # (one launch: block layout)
    assert torch.equal(y.to(torch.float16), y16)
    monkeypatch.setenv("ARCQ_ROWS", "0")
    assert torch.equal(y, ops.linear_otf(x, *args, out_dtype=torch.float32, w_hat_ws=torch.zeros_like(w_ws)))
