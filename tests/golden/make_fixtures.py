#!/usr/bin/env python3
"""Writes the regression vectors in this directory from the CPU oracle (oracle/), on seeded inputs.

The oracle itself is pinned by tests/test_oracle_*.py against the reference tests' closed forms, tables and
independent arithmetic engines; these files freeze its answers so that a later change to the oracle or to the HIP
kernels that alters a single bit shows up against data that is under version control.  Nothing here was produced
by running the reference.  Usage: python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
sys.path.insert(0, os.path.join(HERE, ".."))

import oracle as O  # noqa: E402
from _util import bits16, make_weight  # noqa: E402


def int4wo(name, N, K, g, seed):
    w = make_weight(N, K, seed=seed)
    Np, Kp = O.int4wo_padded_shape(N, K, g)
    codes, scale, zero = O.int4wo_quantize(bits16(w), O.BF16, g, Np, Kp)
    packed, qparams = O.int4wo_pack(codes, scale, zero, g)
    dq = O.dequantize_affine(codes, O.I32, (1, g), scale, O.BF16, zero, O.BF16, 0, 15, 1, O.BF16)
    x = (torch.randn(3, K, generator=torch.Generator().manual_seed(seed + 1))).bfloat16()
    y = O.linear(bits16(x), O.BF16, np.ascontiguousarray(dq[:N, :K]), O.BF16)
    np.savez_compressed(os.path.join(HERE, name), w_bits=bits16(w), group=np.int64(g), codes=codes.astype(np.uint8),
                        scale_bits=scale, zero_bits=zero, packed=packed, qparams=qparams, dequant_bits=dq[:N, :K],
                        x_bits=bits16(x), y_f32=y)


def fpx(name, N, K, ebits, mbits, seed):
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(seed)) * 0.05).half()
    codes, scale = O.fpx_quantize(bits16(w), O.F16, ebits, mbits)
    packed = O.pack_tc_fp6(codes) if ebits + mbits == 5 else O.pack_tc_fpx_generic(codes, 1 + ebits + mbits)
    x = (torch.rand(2, K, generator=torch.Generator().manual_seed(seed + 1)) + 0.5).half()
    y = O.fpx_linear(bits16(x), codes, scale, ebits, mbits)
    np.savez_compressed(os.path.join(HERE, name), w_bits=bits16(w), ebits=np.int64(ebits), mbits=np.int64(mbits),
                        codes=codes, scale_bits=scale, packed=packed, x_bits=bits16(x), y_f32=y)


def hqq(name, N, K, g, seed):
    gen = torch.Generator().manual_seed(seed)
    codes = torch.randint(0, 16, (K, N), generator=gen, dtype=torch.uint8).numpy()
    packed = (codes[0::2] & 15) | (codes[1::2] << 4)
    out = {}
    for tag, dt, code in (("bf16", torch.bfloat16, O.BF16), ("f16", torch.float16, O.F16)):
        s = (torch.rand(K // g, N, generator=gen) * 0.02 + 1e-3).to(dt)
        z = (torch.rand(K // g, N, generator=gen) * 6 + 5).to(dt)
        out[f"scale_{tag}"], out[f"zero_{tag}"] = bits16(s), bits16(z)
        out[f"dequant_{tag}"] = O.hqq_dequantize(packed, bits16(s), bits16(z), g, code)
    np.savez_compressed(os.path.join(HERE, name), packed=packed, group=np.int64(g), **out)


if __name__ == "__main__":
    int4wo("int4wo_48x192_g64.npz", 48, 192, 64, seed=1234)      # K padded to 256, ragged rows, planted outliers
    int4wo("int4wo_64x512_g128.npz", 64, 512, 128, seed=1235)
    int4wo("int4wo_32x256_g32.npz", 32, 256, 32, seed=1236)
    int4wo("int4wo_16x512_g256.npz", 16, 512, 256, seed=1237)
    fpx("fp6_e3m2_64x128.npz", 64, 128, 3, 2, seed=21)
    fpx("fp6_e2m3_64x64.npz", 64, 64, 2, 3, seed=22)
    fpx("fp5_e2m2_64x64.npz", 64, 64, 2, 2, seed=23)
    fpx("fp5_e3m1_64x64.npz", 64, 64, 3, 1, seed=24)
    hqq("hqq_128x64_g32.npz", 64, 128, 32, seed=31)
    print("written:", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
