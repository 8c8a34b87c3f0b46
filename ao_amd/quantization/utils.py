"""tinygemm-flavoured helpers over the affine primitives (torchao/quantization/utils.py:274-392)."""
import torch

from .quant_primitives import (
    MappingType,
    ZeroPointDomain,
    choose_qparams_affine,
    dequantize_affine,
    quantize_affine,
)

__all__ = [
    "compute_error",
    "get_groupwise_affine_qparams",
    "pack_tinygemm_scales_and_zeros",
    "unpack_tinygemm_scales_and_zeros",
    "groupwise_affine_quantize_tensor_from_qparams",
    "groupwise_affine_dequantize_tensor_from_qparams",
    "groupwise_affine_quantize_tensor",
    "groupwise_affine_dequantize_tensor",
    "recommended_inductor_config_setter",
    "unpack_tinygemm_int4pack",
    "_MultiInput",
]


def compute_error(x, y):
    """Signal to quantization noise ratio in dB (reference :50-53)."""
    signal, noise = torch.linalg.norm(x), torch.linalg.norm(x - y)
    return 20 * torch.log10(signal / noise)


def guard_dtype_size(tensor_arg, arg_name, dtype=None, size=None):
    """ValueError unless the tensor has the given dtype / size (reference :125-129, same messages)."""
    for what, want, got in (("dtype", dtype, tensor_arg.dtype), ("size", size, tensor_arg.size())):
        if want is not None and got != want:
            raise ValueError(f"Expected Tensor argument {arg_name} to have {what} {want}, but got {got} instead.")


def _row_groups(t, groupsize, qparams=None):
    """Block size (1, g) of a groupwise operation on the 2-d tensor `t`, with the reference's argument checks.
    A group larger than the row means one group per row: always when choosing qparams (`qparams` None), and for the
    GPTQ loop's single-column slices when the qparams passed in have one column."""
    if qparams is not None:
        assert groupsize > 1   # as asked for; the single-column slice below then is its own group of one
    if groupsize > t.shape[-1] and (qparams is None or qparams.shape[-1] == 1):
        groupsize = t.shape[-1]
    if qparams is None:
        assert groupsize > 1
    assert t.shape[-1] % groupsize == 0
    assert t.dim() == 2
    return (1, groupsize)


def _uint_range(n_bit):
    return 0, 2**n_bit - 1


def get_groupwise_affine_qparams(w, n_bit=4, groupsize=128, dtype=torch.bfloat16):
    """Per-group (scale, zero) of an asymmetric uint`n_bit` quantization, float zero point (reference :274-308)."""
    block = _row_groups(w, groupsize)
    assert n_bit <= 8, f"only n_bit smaller than 8 is supported, got: {n_bit}"
    scale, zero_point = choose_qparams_affine(
        w, MappingType.ASYMMETRIC, block, torch.int32, *_uint_range(n_bit), 1e-6, scale_dtype=dtype,
        zero_point_dtype=dtype, preserve_zero=False, zero_point_domain=ZeroPointDomain.FLOAT)
    rows = w.shape[0]
    return scale.to(dtype=dtype).reshape(rows, -1), zero_point.to(dtype=dtype).reshape(rows, -1)


def pack_tinygemm_scales_and_zeros(scales, zeros):
    """[N, K/g] x 2 -> [K/g, N, 2] bf16, the tinygemm interchange form of the qparams (reference :310-322)."""
    guard_dtype_size(scales, "scales", dtype=torch.bfloat16, size=zeros.size())
    guard_dtype_size(zeros, "zeros", dtype=torch.bfloat16)
    return torch.stack([scales, zeros], dim=2).transpose(0, 1).contiguous()


def unpack_tinygemm_scales_and_zeros(scales_and_zeros):
    assert scales_and_zeros.dim() == 3 and scales_and_zeros.shape[2] == 2
    return torch.split(scales_and_zeros.transpose(0, 1), 1, 2)


def groupwise_affine_quantize_tensor_from_qparams(w, scales, zeros, n_bit=4, groupsize=128):
    return quantize_affine(w, _row_groups(w, groupsize, scales), scales, zeros, torch.int32, *_uint_range(n_bit),
                           zero_point_domain=ZeroPointDomain.FLOAT)


def groupwise_affine_dequantize_tensor_from_qparams(w_int4x8, scales, zeros, n_bit=4, groupsize=128):
    return dequantize_affine(w_int4x8, _row_groups(w_int4x8, groupsize, scales), scales, zeros, torch.int32,
                             *_uint_range(n_bit), zero_point_domain=ZeroPointDomain.FLOAT, output_dtype=scales.dtype)


def groupwise_affine_quantize_tensor(w, n_bit=4, groupsize=128, dtype=torch.bfloat16):
    qparams = get_groupwise_affine_qparams(w, n_bit, groupsize, dtype)
    codes = groupwise_affine_quantize_tensor_from_qparams(w, *qparams, n_bit, groupsize)
    return codes, pack_tinygemm_scales_and_zeros(*qparams)


def groupwise_affine_dequantize_tensor(w_int4x8, scales_and_zeros, n_bit=4, groupsize=128):
    return groupwise_affine_dequantize_tensor_from_qparams(
        w_int4x8, *unpack_tinygemm_scales_and_zeros(scales_and_zeros), n_bit, groupsize)


def recommended_inductor_config_setter():
    """The reference tunes torch.compile here (:461-476).  This library does not go through inductor:
    kernels are launched directly and decode loops are captured in HIP graphs, so there is nothing to set."""
    return None


# Position, inside a 32-wide span of k (two 16-wide k tiles), of nibble p of a tinygemm word held by the lane with
# t % 4 == 0; lane t adds 2 * (t % 4).  Nibbles 0..3 (low half-word) are the even k of the lane's four pairs, nibbles
# 4..7 the odd ones, so that `(word >> 4i) & 0x000F000F` is one (k, k + 1) pair.
_TINYGEMM_NIBBLE_K = (0, 8, 16, 24, 1, 9, 17, 25)


# The same for a word packed by a ROCm build: the packed tensor, read flat, is [N/16, K/(16*inner_k_tiles), 64,
# inner_k_tiles/2] (one 64-lane wavefront per 16 rows); the lane with t // 16 == 0 holds these positions of the 32-wide
# span and lane t adds 4 * (t // 16).
_TINYGEMM_NIBBLE_K_ROCM = (0, 2, 16, 18, 1, 3, 17, 19)


def unpack_tinygemm_int4pack(weight_int4pack: torch.Tensor, inner_k_tiles: int, packed_by: str = "cuda") -> torch.Tensor:
    """The 4-bit codes `[N, K]` (int32, 0..15) of a weight packed by `aten._convert_weight_to_int4pack`
    (`[N/8, K/(16*inner_k_tiles), 32, inner_k_tiles/2]` int32), the `weight` entry of state dicts written by the
    reference's module-swap quantizers (torchao/quantization/GPTQ.py:566-569, :737).  The words depend on the
    PyTorch build that packed them:

    `packed_by="cuda"`: the B fragment of `mma.m16n8k16`, as published in PyTorch's int4mm.cu (v2.3): word
    `[nt][ko][t][j]` belongs to row `8*nt + t//4` and to the two k tiles starting at `16*(ko*inner_k_tiles + 2j)`;
    its nibbles hold k offsets `2*(t%4) + {0, 8, 16, 24, 1, 9, 17, 25}` in order from the low nibble.  The reference
    repository holds no packed vectors of this format (the packer lives in PyTorch core), so this restatement is
    checked against a loop transcription of the same published kernel only.

    `packed_by="rocm"`: what the same operator of a PyTorch-ROCm build writes on a 64-lane device.  The tensor has
    the same shape but, read flat, is `[N/16][ko][t in 0..63][j]`: the word belongs to row `16*nt + t%16` and to the
    32-wide span of k starting at `16*inner_k_tiles*ko + 32*j`; its nibbles hold k offsets
    `4*(t//16) + {0, 2, 16, 18, 1, 3, 17, 19}`.  This one is checked on the GPU against the operator itself."""
    assert weight_int4pack.dtype is torch.int32 and weight_int4pack.dim() == 4, "expected the 4-d int32 tinygemm weight"
    n_tiles, k_outer, lanes, halves = weight_int4pack.shape
    assert inner_k_tiles in (2, 4, 8) and lanes == 32 and halves * 2 == inner_k_tiles, \
        f"shape {tuple(weight_int4pack.shape)} is not a tinygemm weight of inner_k_tiles={inner_k_tiles}"
    if packed_by not in ("cuda", "rocm"):
        raise ValueError(f"packed_by must be 'cuda' or 'rocm', got {packed_by!r}")
    dev = weight_int4pack.device
    shifts = torch.arange(0, 32, 4, device=dev, dtype=torch.int32)
    src = torch.empty(32, dtype=torch.long)
    if packed_by == "cuda":
        rows, lane_groups, lane_step, nibble_k = 8, 4, 2, _TINYGEMM_NIBBLE_K
        words = weight_int4pack
    else:
        assert n_tiles % 2 == 0, "a ROCm-packed tinygemm weight has a multiple of 16 rows"
        rows, lane_groups, lane_step, nibble_k = 16, 4, 4, _TINYGEMM_NIBBLE_K_ROCM
        words = weight_int4pack.reshape(n_tiles // 2, k_outer, 64, halves)
    nib = (words.unsqueeze(-1) >> shifts) & 0xF  # [nt, ko, t, j, p]
    if packed_by == "cuda":
        nib = nib.reshape(-1, k_outer, rows, lane_groups, halves, 8)  # t -> (row in tile, t % 4)
        nib = nib.permute(0, 2, 1, 4, 3, 5)
    else:
        nib = nib.reshape(-1, k_outer, lane_groups, rows, halves, 8)  # t -> (t // 16, row in tile)
        nib = nib.permute(0, 3, 1, 4, 2, 5)
    # now [nt, row, ko, j, lane group, p]; gather (lane group, p) into the 32 positions of the span
    nib = nib.reshape(-1, rows, k_outer, halves, 32)
    for lg in range(lane_groups):
        for p, koff in enumerate(nibble_k):
            src[koff + lane_step * lg] = 8 * lg + p
    codes = nib.index_select(-1, src.to(dev))
    return codes.reshape(n_tiles * 8, k_outer * inner_k_tiles * 16).contiguous()


class _MultiInput:
    """The values one positional argument of a model takes over the calibration samples (reference
    torchao/quantization/utils.py:106-122)."""

    def __init__(self, inputs):
        self.values = list(inputs)

    def add_input(self, input):
        self.values.append(input)
        return self

    def __getitem__(self, slice):
        return _MultiInput(self.values[slice])

    def cuda(self):
        self.values = [v.cuda() if isinstance(v, torch.Tensor) else v for v in self.values]
