"""Module-swap int4 weight-only quantization (reference torchao/quantization/GPTQ.py:521-673).

`Int4WeightOnlyQuantizer.quantize(model)` replaces every eligible `nn.Linear` by a `WeightOnlyInt4Linear` whose
state is two buffers, as in the reference:

* `scales_and_zeros`, bf16 `[in_features / groupsize, out_features, 2]`: the same tensor, bit for bit, as the
  reference's (`pack_tinygemm_scales_and_zeros`);
* `weight`, int32: the 4-bit codes.  The reference stores them in the layout of
  `aten._convert_weight_to_int4pack` (`[N/8, K/(16*inner_k_tiles), 32, inner_k_tiles/2]`), which only its CUDA kernel
  reads; here they are stored in the gfx950 wave-tiled layout `[ceil(N/16), Kp/128, 64, 4]`
  (`ops.int4wo_packed_shapes`) that the HIP kernels read with one 16-byte load per lane.  The codes themselves are
  identical; `torch.ops.torchao.int4wo_unpack` recovers them.  State dicts written by the reference's quantizer
  therefore do not load into this module (and vice versa); quantize from the float checkpoint instead.

`inner_k_tiles` keeps its role in the eligibility rule (`in_features % (16 * inner_k_tiles) == 0`, else pad the
input features to a multiple of 1024 or skip the layer) so the same layers are swapped as in the reference; it does
not change the stored layout.  The calibrated GPTQ flow of the same file (`Int4WeightOnlyGPTQQuantizer`,
:675-720) is a different code path and is not provided.
"""
from typing import Any, Dict, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from .unified import Quantizer
from ..utils import find_multiple
from .utils import groupwise_affine_quantize_tensor

__all__ = ["Int4WeightOnlyQuantizer", "WeightOnlyInt4Linear", "linear_forward_int4", "replace_linear_int4",
           "interleave_scales_and_zeros"]


def _check_linear_int4_k(k, groupsize=1, inner_k_tiles=None):
    """Eligibility of an input-feature count (reference :521-526)."""
    k_divisible_by_groupsize = k % groupsize == 0
    if inner_k_tiles is not None:
        return k_divisible_by_groupsize and k % (inner_k_tiles * 16) == 0
    return k_divisible_by_groupsize


def interleave_scales_and_zeros(scales_and_zeros: torch.Tensor, groupsize: int) -> torch.Tensor:
    """`[K/g, N, 2]` bf16 (scale, zero) pairs -> the kernels' `[ceil(N/16), Kp/g, 16]` int32 words
    `scale | zero << 16`, the 16 rows of a row block adjacent.  Rows and groups past the logical shape get the
    neutral pair (scale bf16(1e-6), zero 0), as `torch.ops.torchao.int4wo_pack` writes them."""
    assert scales_and_zeros.dim() == 3 and scales_and_zeros.shape[2] == 2 and scales_and_zeros.dtype is torch.bfloat16
    groups, N, _ = scales_and_zeros.shape
    _, qshape = ops.int4wo_packed_shapes(N, groups * groupsize, groupsize)
    # a (scale, zero) pair of bf16 is, little-endian, exactly the 32-bit word the kernels read
    words = scales_and_zeros.contiguous().view(torch.int32).reshape(groups, N)
    out = torch.full((qshape[1], qshape[0] * 16), 0x3586, dtype=torch.int32, device=words.device)
    out[:groups, :N] = words
    return out.reshape(qshape[1], qshape[0], 16).permute(1, 0, 2).contiguous()


def linear_forward_int4(x, weight_int4pack, scales_and_zeros, out_features, groupsize, qparams=None):
    """`x @ dequant(W)^T` in bf16, cast back to `x.dtype` (reference :528-539).  `qparams` is the interleaved form of
    `scales_and_zeros` (`interleave_scales_and_zeros`); it is built here when the caller has not cached it."""
    origin_x_size = x.size()
    x = x.reshape(-1, origin_x_size[-1])
    if qparams is None:
        qparams = interleave_scales_and_zeros(scales_and_zeros.to(torch.bfloat16), groupsize)
    c = torch.ops.torchao.int4wo_linear(x.to(torch.bfloat16), weight_int4pack, qparams, groupsize, out_features,
                                        None, False).to(dtype=x.dtype)
    return c.reshape(origin_x_size[:-1] + (out_features,))


class WeightOnlyInt4Linear(nn.Module):
    """Linear layer over packed int4 codes and per-group (scale, zero) pairs (reference :541-582)."""
    __constants__ = ["in_features", "out_features"]
    in_features: int
    out_features: int
    weight: torch.Tensor

    def __init__(self, in_features: int, out_features: int, bias=False, device=None, dtype=None,
                 groupsize: int = 128, inner_k_tiles: int = 8) -> None:
        super().__init__()
        self.padding = not _check_linear_int4_k(in_features, groupsize, inner_k_tiles)
        if self.padding:
            self.origin_in_features = in_features
            in_features = find_multiple(in_features, 1024)
        self.in_features = in_features
        self.out_features = out_features
        assert not bias, "require bias=False"
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles
        assert out_features % 8 == 0, "require out_features % 8 == 0"
        assert in_features % (inner_k_tiles * 16) == 0, "require in_features % (innerKTiles * 16) == 0"
        pshape, _ = ops.int4wo_packed_shapes(out_features, in_features, groupsize)
        self.register_buffer("weight", torch.empty(pshape, dtype=torch.int32, device=device))
        self.register_buffer("scales_and_zeros",
                             torch.empty((in_features // groupsize, out_features, 2), dtype=torch.bfloat16, device=device))
        self._qparams = None
        self._qparams_key = None

    def _interleaved_qparams(self):
        # rebuilt whenever the buffer was replaced (module.to) or written in place (load_state_dict)
        sz = self.scales_and_zeros
        key = (sz.data_ptr(), sz._version, sz.device)
        if self._qparams is None or self._qparams_key != key:
            self._qparams = interleave_scales_and_zeros(sz, self.groupsize)
            self._qparams_key = key
        return self._qparams

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if self.padding:
            input = F.pad(input, pad=(0, self.in_features - self.origin_in_features))
        return linear_forward_int4(input, self.weight, self.scales_and_zeros, self.out_features, self.groupsize,
                                   qparams=self._interleaved_qparams())

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, groupsize={self.groupsize}"


def replace_linear_int4(module, groupsize, inner_k_tiles, padding_allowed, skip_layer_func=None):
    """Swap eligible `nn.Linear` children, recursively (reference :584-594)."""
    for name, child in module.named_children():
        if isinstance(child, nn.Linear) and (skip_layer_func is None or not skip_layer_func(child.weight)):
            if _check_linear_int4_k(child.in_features, groupsize, inner_k_tiles) or padding_allowed:
                setattr(module, name, WeightOnlyInt4Linear(
                    child.in_features, child.out_features, bias=False, device=child.weight.device,
                    groupsize=groupsize, inner_k_tiles=inner_k_tiles))
        else:
            replace_linear_int4(child, groupsize, inner_k_tiles, padding_allowed, skip_layer_func)


class Int4WeightOnlyQuantizer(Quantizer):
    """Round-to-nearest groupwise int4 quantizer by module swap (reference :596-673)."""

    def __init__(self, groupsize: int = 256, padding_allowed: bool = True, inner_k_tiles: Optional[int] = 8,
                 device: torch.device = torch.device("cuda")) -> None:
        super().__init__()
        assert inner_k_tiles in [2, 4, 8]
        assert groupsize in [32, 64, 128, 256]
        self.inner_k_tiles = inner_k_tiles
        self.groupsize: int = groupsize
        self.padding_allowed: bool = padding_allowed
        self.device: torch.device = torch.device(device)

    @torch.no_grad()
    def _create_quantized_state_dict(self, model: torch.nn.Module) -> Dict[str, torch.Tensor]:
        cur_state_dict = model.state_dict()
        for fqn, mod in model.named_modules():
            if not isinstance(mod, torch.nn.Linear):
                continue
            assert mod.bias is None, f"{fqn}: int4 module swap requires bias=False"
            in_features = mod.in_features
            assert in_features % self.groupsize == 0, \
                f"require in_features:{in_features} % self.groupsize:{self.groupsize} == 0"
            weight = mod.weight.data.to(self.device)
            if not _check_linear_int4_k(in_features, self.groupsize, self.inner_k_tiles):
                if not self.padding_allowed:
                    continue  # the layer stays an nn.Linear
                weight = F.pad(weight, pad=(0, find_multiple(in_features, 1024) - in_features))
            w_int4x8, scales_and_zeros = groupwise_affine_quantize_tensor(weight, 4, self.groupsize)
            # [K/g, N, 2] -> the [N, K/g] scales and zeros the packer takes
            scales = scales_and_zeros[:, :, 0].t().contiguous()
            zeros = scales_and_zeros[:, :, 1].t().contiguous()
            packed, _ = torch.ops.torchao.int4wo_pack(w_int4x8, scales, zeros, self.groupsize)
            cur_state_dict[f"{fqn}.weight"] = packed
            cur_state_dict[f"{fqn}.scales_and_zeros"] = scales_and_zeros
        return cur_state_dict

    def _convert_for_runtime(self, model: torch.nn.Module) -> torch.nn.Module:
        replace_linear_int4(model, self.groupsize, self.inner_k_tiles, self.padding_allowed)
        return model

    def quantize(self, model: torch.nn.Module, *args: Any, **kwargs: Any) -> torch.nn.Module:
        state_dict = self._create_quantized_state_dict(model)
        model = self._convert_for_runtime(model)
        model.load_state_dict(state_dict, strict=False)
        return model
