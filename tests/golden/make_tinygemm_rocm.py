"""Writes tests/golden/tinygemm_rocm_int4pack.npz: 4-bit codes and the words `aten._convert_weight_to_int4pack` of
the installed PyTorch-ROCm build makes of them on the GPU, for inner_k_tiles 2, 4 and 8, plus the output of
`aten._weight_int4pack_mm` for one activation matrix.  Needs a GPU and PyTorch only:

    python tests/golden/make_tinygemm_rocm.py <output directory>
"""
import os
import sys

import numpy as np
import torch


def main(out_dir):
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(20240731)
    N, K, g = 48, 256, 64
    codes = rng.integers(0, 16, (N, K)).astype(np.int32)
    c = torch.from_numpy(codes).to(dev)
    two_per_byte = ((c[:, ::2] << 4) | c[:, 1::2]).to(torch.uint8)
    out = {"codes": codes, "torch_version": np.array(torch.__version__),
           "device": np.array(torch.cuda.get_device_properties(0).gcnArchName)}
    for ikt in (2, 4, 8):
        out[f"packed_ikt{ikt}"] = torch.ops.aten._convert_weight_to_int4pack(two_per_byte, ikt).cpu().numpy()
    scales = torch.from_numpy(rng.uniform(0.002, 0.02, (K // g, N)).astype(np.float32)).bfloat16()
    zeros = torch.from_numpy(rng.uniform(-0.05, 0.05, (K // g, N)).astype(np.float32)).bfloat16()
    x = torch.from_numpy(rng.standard_normal((5, K)).astype(np.float32)).bfloat16()
    sz = torch.stack([scales, zeros], -1).contiguous().to(dev)
    y = torch.ops.aten._weight_int4pack_mm(x.to(dev), torch.from_numpy(out["packed_ikt8"]).to(dev), g, sz)
    out["scales_bits"] = scales.view(torch.int16).numpy()
    out["zeros_bits"] = zeros.view(torch.int16).numpy()
    out["x_bits"] = x.view(torch.int16).numpy()
    out["mm_bits"] = y.cpu().view(torch.int16).numpy()
    np.savez_compressed(os.path.join(out_dir, "tinygemm_rocm_int4pack.npz"), **out)
    print("wrote", os.path.join(out_dir, "tinygemm_rocm_int4pack.npz"), flush=True)


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else os.path.dirname(os.path.abspath(__file__)))
