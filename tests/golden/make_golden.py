#!/usr/bin/env python3
"""Writes the golden fixtures in this directory.  Run from the repo root:
    python tests/golden/make_golden.py

The reference ships no test vectors for this path (it has no tests at all), and nothing of the
reference is imported here.  The vectors are produced by the CPU oracle AFTER tests/test_oracle_*.py
have pinned it, and frozen so that (a) any later drift of the oracle is caught and (b) the GPU
parity tests have a host-independent target.  Only serial-order / integer results go in: they do
not depend on the host's torch build.  layout_vectors.json is derived by hand (see the comments in
tests/test_oracle_layout.py), not by any code.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from arcq_vit_amd import synth  # noqa: E402
from oracle import arcq_ref  # noqa: E402


def main():
    json.dump({
        "comment": "hand-derived: code j occupies bits [j*bits,(j+1)*bits) of the row's little-endian bit string",
        "vectors": [
            {"bits": 4, "codes": [1, 2, 3, 4], "bytes": [0x21, 0x43]},
            {"bits": 3, "codes": [1, 2, 3, 4, 5, 6, 7, 0], "bytes": [0xD1, 0x58, 0x1F]},
            {"bits": 2, "codes": [3, 0, 1, 2], "bytes": [0x93]},
            {"bits": 3, "codes": [7, 7, 7], "bytes": [0xFF, 0x01]},
            {"bits": 4, "codes": [15, 0, 0, 15, 9], "bytes": [0x0F, 0xF0, 0x09]},
            {"bits": 3, "codes": [0, 0, 5, 0, 0, 6], "bytes": [0x40, 0x01, 0x03]},
        ]}, open(os.path.join(HERE, "layout_vectors.json"), "w"), indent=1)

    for bits in (2, 3, 4):
        cb = synth.quantile_codebook(bits)
        thr = synth.midpoint_thresholds(cb)
        x = synth.make_activation(12, 128, 7000 + bits)
        x[0, :64] = 1.5                      # constant group
        x[1] = synth.make_activation(1, 128, 1, "gelu")[0]
        x16 = x.to(torch.float16)
        a32 = arcq_ref.act_quant_c(x.numpy(), thr, cb, bits, 64)
        a16 = arcq_ref.act_quant_c(x16.float().numpy(), thr, cb, bits, 64)
        w = synth.make_weight(16, 128, 7100 + bits)
        wq = arcq_ref.act_quant_c(w.numpy(), thr, cb, bits, 64)      # weight encoded in serial order
        wd = arcq_ref.weight_dequant_c(wq["packed"], cb, wq["center"], wq["scale"], wq["code_sum"], bits, 64)
        bias = synth.make_bias(16, 7100 + bits)
        y64, mag = arcq_ref.linear_f64_c(a16["x_hat"].astype(np.float16), wd.astype(np.float16), bias.numpy())
        table = np.outer(cb.numpy(), cb.numpy() * 1.25).astype(np.float32)
        y_packed = arcq_ref.linear_forward_packed_c(a32["packed"], a32["center"], a32["scale"], a32["code_sum"],
                                                    wq["packed"], wq["center"], wq["scale"], wq["code_sum"], table,
                                                    bias.numpy(), bits, 64, 128, 16)
        y_u8 = arcq_ref.linear_forward_u8_c(a32["codes"], a32["center"], a32["scale"], a32["code_sum"], wq["codes"],
                                            wq["center"], wq["scale"], wq["code_sum"], table, bias.numpy(), 64)
        np.savez_compressed(
            os.path.join(HERE, f"arcq_w{bits}a{bits}_g64.npz"),
            codebook=cb.numpy(), thresholds=thr.numpy(), x=x.numpy(), x_f16=x16.numpy(),
            a32_packed=a32["packed"], a32_codes=a32["codes"], a32_center=a32["center"], a32_scale=a32["scale"],
            a32_code_sum=a32["code_sum"], a32_x_hat=a32["x_hat"],
            a16_packed=a16["packed"], a16_x_hat_f16=a16["x_hat"].astype(np.float16),
            w_packed=wq["packed"], w_codes=wq["codes"], w_center=wq["center"], w_scale=wq["scale"],
            w_code_sum=wq["code_sum"], w_dequant_f16=wd.astype(np.float16), bias=bias.numpy(),
            y_f64=y64, y_abs_sum=mag, product_table=table, y_index_packed=y_packed, y_index_u8=y_u8)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
