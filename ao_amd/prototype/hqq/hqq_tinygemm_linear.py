"""HQQ-quantized weights on the int4 weight-only kernels (interface of the reference's
torchao/prototype/hqq/hqq_tinygemm_linear.py).

HQQ reconstructs a group as (W_q - zero) * scale; the int4 kernels compute (q - 8) * scale + zero'.
`hqq_to_affine_int4` converts between the two conventions the way the reference does (:172-208): the scale is kept,
zero' = scale * 2^(nbits-1) - zero * scale, and the codes are re-derived by quantizing the HQQ reconstruction with
(scale, zero'), every step rounded in the compute dtype.  The module then packs codes and parameters into the gfx950
layout (`torch.ops.torchao.int4wo_pack`, where the reference calls `aten._convert_weight_to_int4pack`) and runs
`torch.ops.torchao.int4wo_linear`; `scales_and_zeros` keeps the reference's [K/g, N, 2] form.

Quantizing a float layer needs the `hqq` package's solver, as in the reference; without it, already quantized weights
go through `initialize_with_hqq_quants`.
"""
import copy

import torch
import torch.nn.functional as F

from ... import ops
from ...quantization.utils import pack_tinygemm_scales_and_zeros
from ...utils import find_multiple

_GROUP_SIZES = (None, 32, 64, 128, 256)


@torch.no_grad()
def hqq_to_affine_int4(W_q, scale, zero, shape, nbits=4, dtype=torch.bfloat16, device="cuda"):
    """HQQ (codes, scale, zero), each broadcastable as [groups, group_size] / [groups, 1], to the affine form
    (int32 codes [N, K], scale [N, K/g], zero' [N, K/g]) of the int4 weight-only kernels."""
    half = 2 ** (nbits - 1)
    q = W_q.to(dtype=dtype, device=device)
    s = scale.to(dtype=dtype, device=device)
    z = zero.to(dtype=dtype, device=device)
    zero_affine = s * half - z * s
    lowest = zero_affine - s * half          # value the code 0 stands for
    recon = (q - z) * s                      # what HQQ would dequantize to
    codes = ((recon - lowest) / s).round_().clamp_(0, 2 ** nbits - 1).to(torch.int32).reshape(shape).contiguous()
    n_out = shape[0]
    return codes, s.contiguous().reshape(n_out, -1), zero_affine.contiguous().reshape(n_out, -1)


def _regroup_channelwise(meta_tensor, group_size, shape):
    """Per-row HQQ parameter [N, 1] -> one value per group of `group_size` consecutive in-features."""
    per_element = meta_tensor.repeat([1, shape[1]]).reshape(shape)
    return per_element.reshape(-1, group_size).mean(dim=1, keepdim=True)


class HQQLinearTorchWeightOnlyInt4(torch.nn.Module):
    def __init__(self, linear_layer, quant_config, del_orig=True, compute_dtype=torch.bfloat16, device="cuda",
                 initialize=True, inner_k_tiles=8, padding=True):
        super().__init__()
        wq_params = quant_config["weight_quant_params"]
        if wq_params["nbits"] not in (1, 2, 4):
            raise AssertionError("Unsupported nbits")
        if wq_params["group_size"] not in _GROUP_SIZES:
            raise AssertionError("Unsupported groupsize")
        if inner_k_tiles not in (2, 4, 8):
            raise AssertionError("Unsupported tile")
        if compute_dtype is not torch.bfloat16:
            raise AssertionError("the int4 kernels compute in bfloat16")
        self.quant_config = copy.deepcopy(quant_config)
        self.nbits, self.groupsize = wq_params["nbits"], wq_params["group_size"]
        self.inner_k_tiles, self.padding = inner_k_tiles, padding
        self.compute_dtype, self.device = compute_dtype, device
        self.del_orig = del_orig
        self.linear_layer = linear_layer
        self.bias = None
        self.ready = self.in_gpu = False
        if initialize:
            self.initialize()

    # ---- construction -------------------------------------------------------------------------------------
    def _set_shape(self, shape, pad):
        self.shape = shape
        self.out_features, self.origin_in_features = shape[0], shape[1]
        self.in_features = find_multiple(shape[1], 1024) if pad else shape[1]
        self.in_features_diff = self.in_features - self.origin_in_features

    def initialize_with_hqq_quants(self, W_q, meta, bias=None):
        """Take weights that HQQ already quantized.  No input-feature padding here: padding after the grouping
        would cut through groups."""
        self.padding = False
        self._set_shape(meta["shape"], pad=False)
        self._ingest(W_q, meta)
        self.bias = bias
        self.ready = self.in_gpu = True
        return self

    def initialize(self):
        layer = self.linear_layer
        if layer is not None:
            self._set_shape(layer.weight.shape, pad=self.padding)
            W = layer.weight.data
            if self.in_features_diff:
                W = F.pad(W, (0, self.in_features_diff))
            self._ingest(*self.quantize(W, **self.quant_config))
            if layer.bias is not None:
                self.bias = layer.bias.to(dtype=self.compute_dtype, device=self.device)
        if self.del_orig:
            self.linear_layer = None
        self.ready = self.in_gpu = True
        return self

    def quantize(self, W, weight_quant_params, scale_quant_params=None, zero_quant_params=None, offload_meta=False):
        try:
            from hqq.core.quantize import Quantizer
        except ImportError as e:
            raise ImportError("quantizing a float layer the HQQ way needs the `hqq` package; pass already quantized "
                              "weights to initialize_with_hqq_quants instead") from e
        return Quantizer.quantize(W, **weight_quant_params, device=self.device, compute_dtype=self.compute_dtype,
                                  bitpack=False)

    def _ingest(self, W_q, meta):
        scale, zero, shape = meta["scale"], meta["zero"], meta["shape"]
        if meta.get("packing") is not None:
            from hqq.core.quantize import Quantizer

            W_q = Quantizer.unpack[meta["packing"]](W_q)
        if self.groupsize is None:  # channel-wise HQQ parameters: spread over groups of 128
            self.groupsize = 128
            W_q = W_q.reshape(-1, self.groupsize)
            scale = _regroup_channelwise(scale, self.groupsize, shape)
            zero = _regroup_channelwise(zero, self.groupsize, shape)
        codes, s, z = hqq_to_affine_int4(W_q, scale, zero, shape, self.nbits, self.compute_dtype, self.device)
        self.weight_int4pack, self._qparams = ops.int4wo_pack(codes, s, z, self.groupsize)
        self.scales_and_zeros = pack_tinygemm_scales_and_zeros(s, z)

    # ---- use ----------------------------------------------------------------------------------------------
    def matmul(self, x):
        lead = x.shape[:-1]
        y = ops.int4wo_linear(x.reshape(-1, x.shape[-1]), self.weight_int4pack, self._qparams, self.groupsize,
                              self.out_features)
        return y.reshape(*lead, self.out_features)

    def dequantize(self):
        """The [out_features, original in_features] weight the kernels multiply with."""
        w = ops.int4wo_dequantize(self.weight_int4pack, self._qparams, self.out_features, self.in_features,
                                  self.groupsize)
        return w[:, : self.origin_in_features]

    def forward(self, x):
        x = x.to(self.compute_dtype)
        if self.in_features_diff:
            x = F.pad(x, (0, self.in_features_diff))
        y = self.matmul(x)
        return y if self.bias is None else y + self.bias
