#!/usr/bin/env python3
"""Writes the golden fixtures of this folder.

The reference ships no golden vectors, known-answer tests or data files for the convolution path, and neither its CUDA code
nor Avocado's CPU backend can be built or run here, so these vectors come from this repository's own CPU oracle
(oracle/avocado_oracle.c) AFTER it has been pinned by tests/test_oracle.py against torch fp64 conv2d, numpy and closed
forms.  They freeze the oracle's answers: a later change of the oracle, or of the HIP path, that alters any result shows up
against files that did not change with it.  Inputs are seeded (0xA70CAD0 + case index), rounded to the tensor dtype before
the oracle sees them, and stored next to the expected outputs in small .npz files (numpy arrays only, no pickles).

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle as orc  # noqa: E402

SEED = 0xA70CAD0


def he(g, shape):
    K, R, S, C = shape
    return g.standard_normal(shape) * np.sqrt(2.0 / (R * S * C))


def conv_case(index, dtype, xs, ws, pad, stride=(1, 1), dilation=(1, 1), mode=0, act=orc.RELU, residual=False):
    g = np.random.default_rng(SEED + index)
    x = orc.round_to(g.standard_normal(xs), dtype)
    w = orc.round_to(he(g, ws), dtype)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    Ho, Wo = orc.conv_output_shape(xs[1], xs[2], ws[1], ws[2], pad, stride, dilation)
    z = orc.round_to(g.standard_normal((xs[0], Ho, Wo, ws[0])), dtype) if residual else None
    y = orc.conv2d(x, w, b, z, pad=pad, stride=stride, dilation=dilation, mode=mode, activation=act)
    out = dict(x=x.astype(np.float32), w=w.astype(np.float32), bias=b.astype(np.float32), y=y, pad=np.array(pad), stride=np.array(stride),
               dilation=np.array(dilation), mode=np.array(mode), activation=np.array(act), dtype=np.array(dtype))
    if residual:
        out["z"] = z.astype(np.float32)
    return out


def int8_case(index, xs, ws, pad, stride=(1, 1), mode=0):
    g = np.random.default_rng(SEED + index)
    x = g.integers(-127, 128, xs, dtype=np.int8)
    w = g.integers(-127, 128, ws, dtype=np.int8)
    b = g.integers(-2 ** 15, 2 ** 15, ws[0]).astype(np.int32)
    scale = g.uniform(1e-4, 1e-3, ws[0]).astype(np.float32)
    acc = orc.conv2d_i8(x, w, b, pad=pad, stride=stride, mode=mode, activation=orc.RELU)
    q = orc.requant_i8(acc, scale)
    return dict(x=x, w=w, bias=b, scale=scale, y_i32=acc, y_i8=q, pad=np.array(pad), stride=np.array(stride), mode=np.array(mode))


def winograd_case(index, m, xs, ws, pad):
    g = np.random.default_rng(SEED + index)
    x = orc.round_to(g.standard_normal(xs), "f32")
    w = orc.round_to(he(g, ws), "f32")
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    U = orc.winograd_weight_transform(w, m)
    V = orc.winograd_input_transform(x, m, ws[1], pad)
    M = orc.gemm_batched(V, U, opB=True)
    y = orc.winograd_output_transform(M, (xs[0], xs[1], xs[2], ws[0]), m, ws[1], bias=b, activation=orc.RELU)
    return dict(x=x.astype(np.float32), w=w.astype(np.float32), bias=b.astype(np.float32), U=U, V=V, M=M, y=y, m=np.array(m), pad=np.array(pad))


def main():
    cases = {
        "conv_f32_3x3_same": conv_case(1, "f32", (2, 7, 6, 12), (10, 3, 3, 12), (-1, -1), residual=True),
        "conv_f32_5x5_flipped_stride2": conv_case(2, "f32", (1, 11, 12, 8), (6, 5, 5, 8), (-2, -2), stride=(2, 2), mode=1, act=orc.LINEAR),
        "conv_bf16_3x3_dilated": conv_case(3, "bf16", (2, 9, 9, 16), (8, 3, 3, 16), (-2, -2), dilation=(2, 2)),
        "conv_f16_1x1": conv_case(4, "f16", (2, 5, 7, 24), (12, 1, 1, 24), (0, 0), act=orc.LINEAR),
        "conv_bf16_stem_4_planes": conv_case(5, "bf16", (2, 15, 15, 4), (32, 3, 3, 4), (-1, -1)),
        "int8_3x3": int8_case(6, (2, 10, 10, 32), (16, 3, 3, 32), (-1, -1)),
        "int8_1x1": int8_case(7, (2, 6, 5, 64), (24, 1, 1, 64), (0, 0)),
        "int8_3x3_stride2_flipped": int8_case(8, (1, 9, 9, 20), (8, 3, 3, 20), (-1, -1), stride=(2, 2), mode=1),
        "winograd_f4_nonfused": winograd_case(9, 4, (2, 9, 10, 8), (6, 3, 3, 8), (-1, -1)),
        "winograd_f2_nonfused": winograd_case(10, 2, (1, 7, 7, 8), (4, 3, 3, 8), (-1, -1)),
    }
    for name, arrays in cases.items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **arrays)
        print("%-36s %7d bytes" % (name + ".npz", os.path.getsize(path)))


if __name__ == "__main__":
    main()
