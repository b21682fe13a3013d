#!/usr/bin/env python3
"""Writes tests/golden/kat_small.npz: small known-answer cases for the bit-matmul / bit-convolution path.

The reference holds no golden vectors for this path and cannot be run here, so the expected outputs are
computed from what the mathematics fixes, with numpy / torch only (tests/refmath.py and the loops below):
+-1 dot products by integer matmul and zero-padded cross-correlation, thresholds by fp32 compare, pooling
by max, residual rules by direct restatement of kernel.cuh:770-794,818-824.  Nothing is imported from
oracle/ or from the product, so the fixture checks both of them.

    python tests/golden/make_golden.py        # rewrites the fixture (seeded: the file is reproducible)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import refmath as rm  # noqa: E402


def main():
    r = np.random.default_rng(20240229)
    out = {}

    # ---- 1. bit-GEMM (tensorcore_kernel.cu:38-57): C = A.B over +-1, K a multiple of 32
    a = rm.pm1(r, (9, 96))
    b = rm.pm1(r, (96, 32))
    out["bmm_a"], out["bmm_b"] = a, b
    out["bmm_c"] = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.int32)

    # ---- 2. bit-convolution, int32 output [N][P][Q][O] (bmma_kernel.cu:101-165), stride 1 and 2
    x = rm.pm1(r, (3, 5, 5, 64))
    f = rm.pm1(r, (3, 3, 64, 32))
    out["bconv_x"], out["bconv_f"] = x, f
    out["bconv_s1"] = rm.xcorr_pm1(x, f, 1, 1, 1, 5, 5).astype(np.int32)
    out["bconv_s2"] = rm.xcorr_pm1(x, f, 2, 1, 1, 3, 3).astype(np.int32)

    # ---- 3. FC with threshold and output layer (kernel.cuh:174-280)
    xf = r.standard_normal((6, 200)).astype(np.float32)
    w = rm.pm1(r, (200, 40))
    s = np.where(xf >= 0, 1.0, -1.0)
    dot = (s.astype(np.int64) @ w.astype(np.int64))
    bn = r.normal(0, 10, 40).astype(np.float32)
    bn[:5] = dot[0, :5]  # ties
    out["fc_x"], out["fc_w"], out["fc_bn"] = xf, w, bn
    out["fc_bits"] = (dot.astype(np.float32) >= bn[None, :])
    scale = r.normal(1, 0.1, 40).astype(np.float32)
    bias = r.normal(0, 1, 40).astype(np.float32)
    out["out_scale"], out["out_bias"] = scale, bias
    out["out_y"] = (dot.astype(np.float32) * scale[None, :]).astype(np.float32) + bias[None, :]

    # ---- 4. Conv128 layer: residual injected as the 2x2 max of a source twice the size into the first
    #         residual_channels channels, saved, thresholded, then OR-pooled (kernel.cuh:676-827).
    #         (The reference pools only without residuals; the two halves are separate cases here.)
    xc = rm.pm1(r, (4, 6, 6, 64))
    fc_ = rm.pm1(r, (3, 3, 64, 48))
    conv = rm.xcorr_pm1(xc, fc_, 1, 1, 1, 6, 6)                      # [B][P][Q][O]
    src = r.integers(-900, 900, size=(4, 12, 12, 40)).astype(np.int64)  # [B][2P][2Q][Csrc]
    pooled = rm.maxpool_nhwc(src.astype(np.float64), 2, 2).astype(np.int64)
    lim = 24                                                          # residual_channels
    res = conv.copy()
    res[..., :lim] += pooled[..., :lim]
    bnc = r.normal(0, 25, 48).astype(np.float32)
    bnc[:6] = res[1, 2, 3, :6]
    out["conv_x"], out["conv_f"], out["conv_bn"], out["conv_src"] = xc, fc_, bnc, src.astype(np.int32)
    out["conv_res"] = res.astype(np.int32)
    out["conv_bits"] = ~(res.astype(np.float32) < bnc)                 # bit = !(res < bn)
    plain_bits = ~(conv.astype(np.float32) < bnc)
    out["conv_pool2_bits"] = rm.maxpool_nhwc(np.where(plain_bits, 1.0, -1.0), 2, 2) > 0

    # ---- 5. first layer with +-1.0f input: every partial sum is an exact small integer, so the result does
    #         not depend on the summation order (kernel.cuh:578-672)
    xi = rm.pm1(r, (5, 9, 9, 3))                                      # NHWC here, fed as NCHW
    fi = rm.pm1(r, (3, 3, 3, 32))
    acc = rm.xcorr_pm1(xi, fi, 2, 1, 1, 5, 5)
    bni = r.normal(0, 4, 32).astype(np.float32)
    bni[:4] = acc[0, 0, 0, :4]
    out["inconv_x_nchw"] = np.ascontiguousarray(xi.transpose(0, 3, 1, 2))
    out["inconv_f"], out["inconv_bn"] = fi, bni
    out["inconv_res"] = acc.astype(np.int32)
    out["inconv_bits"] = ~(acc.astype(np.float32) < bni)

    np.savez_compressed(os.path.join(HERE, "kat_small.npz"), **out)
    print("wrote", os.path.join(HERE, "kat_small.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
