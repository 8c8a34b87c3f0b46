"""Module-swap int4 weight-only quantization (reference torchao/quantization/GPTQ.py:521-673).

`Int4WeightOnlyQuantizer.quantize(model)` replaces every eligible `nn.Linear` by a `WeightOnlyInt4Linear` whose
state is two buffers, as in the reference:

* `scales_and_zeros`, bf16 `[in_features / groupsize, out_features, 2]`: the same tensor, bit for bit, as the
  reference's (`pack_tinygemm_scales_and_zeros`);
* `weight`, int32: the 4-bit codes.  The reference stores them in the layout of
  `aten._convert_weight_to_int4pack` (`[N/8, K/(16*inner_k_tiles), 32, inner_k_tiles/2]`), which only its CUDA kernel
  reads; here they are stored in the gfx950 wave-tiled layout `[ceil(N/16), Kp/128, 64, 4]`
  (`ops.int4wo_packed_shapes`) that the HIP kernels read with one 16-byte load per lane.  The codes themselves are
  identical; `torch.ops.torchao.int4wo_unpack` recovers them.  `load_state_dict` also accepts a `weight` entry in the
  reference's layout as packed by a CUDA build of PyTorch (state dicts written by the reference's quantizers) and
  repacks it on load (`utils.unpack_tinygemm_int4pack`).

`inner_k_tiles` keeps its role in the eligibility rule (`in_features % (16 * inner_k_tiles) == 0`, else pad the
input features to a multiple of 1024 or skip the layer) so the same layers are swapped as in the reference; it does
not change the stored layout.

`Int4WeightOnlyGPTQQuantizer` (reference :675-758) is the calibrated variant: each linear is quantized column by column
with the error of every column pushed onto the columns not yet quantized, weighted by the inverse Hessian of the
layer's calibration inputs (`gptq_quantize_weight`, reference `faster_quant` :300-398).  Where the reference traces
the model with torch._dynamo.export and interprets the graph over all samples, this module runs the model itself:
one thread per calibration sample, advanced in lock step from linear to linear by forward pre-hooks
(`_LockStepCalibration`), so that every linear sees the inputs produced by its already quantized predecessors, as in
the reference.
"""
import threading
from typing import Any, Callable, Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from .unified import Quantizer
from ..utils import find_multiple
from .utils import (
    _MultiInput,
    get_groupwise_affine_qparams,
    groupwise_affine_dequantize_tensor_from_qparams,
    groupwise_affine_quantize_tensor,
    groupwise_affine_quantize_tensor_from_qparams,
    pack_tinygemm_scales_and_zeros,
    unpack_tinygemm_int4pack,
)

__all__ = ["Int4WeightOnlyQuantizer", "Int4WeightOnlyGPTQQuantizer", "GPTQQuantizer", "WeightOnlyInt4Linear",
           "linear_forward_int4", "replace_linear_int4", "interleave_scales_and_zeros", "gptq_quantize_weight"]


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
    # which PyTorch build packed the `weight` of a reference-format state dict given to load_state_dict: "cuda" or
    # "rocm" (the two write different words into the same shape; see unpack_tinygemm_int4pack).  Set it on the class
    # or on a module before loading.
    tinygemm_packed_by: str = "cuda"

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

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # a `weight` in the reference's tinygemm layout [N/8, K/(16*inner_k_tiles), 32, inner_k_tiles/2] is
        # repacked into the layout of this module before the regular copy
        key = prefix + "weight"
        w = state_dict.get(key)
        tinygemm_shape = (self.out_features // 8, self.in_features // (self.inner_k_tiles * 16), 32,
                          self.inner_k_tiles // 2)
        if w is not None and w.dim() == 4 and tuple(w.shape) == tinygemm_shape and tuple(w.shape) != tuple(self.weight.shape):
            sz = state_dict.get(prefix + "scales_and_zeros", self.scales_and_zeros)
            dev = self.weight.device
            codes = unpack_tinygemm_int4pack(w.to(dev), self.inner_k_tiles, self.tinygemm_packed_by)
            scales = sz[:, :, 0].t().contiguous().to(device=dev, dtype=torch.bfloat16)
            zeros = sz[:, :, 1].t().contiguous().to(device=dev, dtype=torch.bfloat16)
            state_dict[key], _ = torch.ops.torchao.int4wo_pack(codes, scales, zeros, self.groupsize)
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

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


@torch.no_grad()
def gptq_quantize_weight(H: torch.Tensor, W: torch.Tensor, get_qparams_func: Callable, quantize_func: Callable,
                         dequantize_func: Callable, combine_qparams_list_func: Callable, blocksize: int = 128,
                         percdamp: float = 0.01, groupsize: int = 128):
    """GPTQ of one weight `W [N, K]` under the input Hessian `H [K, K]` (modified in place); returns
    `(Q, DQ, qparams)` = codes, dequantized weight in `W.dtype`, combined per-group qparams.

    Same recurrence as the reference's `faster_quant` (:300-398): dead inputs (zero diagonal) are pinned, the
    diagonal is damped by `percdamp` of its mean, and with U = the upper Cholesky factor of H^-1 every column i is
    quantized in turn and `(w_i - dq_i) / U[i, i] * U[i, j]` is subtracted from the columns j > i, inside a block of
    `blocksize` columns immediately and on the rest of the matrix once per block.  Qparams are taken at each group
    start from the weights as compensated by the completed blocks (a group that starts inside a block does not see
    the corrections of that block's earlier columns, as in the reference, :361-365).  The three callbacks work on a
    whole matrix, a group or one column."""
    orig_dtype = W.dtype
    W = W.detach().float().clone()
    columns = W.shape[1]
    idx = torch.arange(columns, device=W.device)
    dead = torch.diag(H) == 0
    H[dead, dead] = 1
    W[:, dead] = 0
    H[idx, idx] += percdamp * torch.mean(torch.diag(H))
    U = torch.linalg.cholesky(torch.cholesky_inverse(torch.linalg.cholesky(H)), upper=True)

    DQ = torch.zeros_like(W)
    group_qparams = []
    cur = get_qparams_func(W) if groupsize == -1 else None
    for start in range(0, columns, blocksize):
        stop = min(start + blocksize, columns)
        Wb = W[:, start:stop].clone()
        Eb = torch.zeros_like(Wb)
        Ub = U[start:stop, start:stop]
        for j in range(stop - start):
            col = start + j
            if groupsize != -1 and col % groupsize == 0:
                cur = get_qparams_func(W[:, col:col + groupsize])
                group_qparams.append(cur)
            w = Wb[:, j]
            dq = dequantize_func(quantize_func(w.unsqueeze(1), cur), cur).flatten().to(w.dtype)
            DQ[:, col] = dq
            e = (w - dq) / Ub[j, j]
            Wb[:, j:] -= e.unsqueeze(1) * Ub[j, j:].unsqueeze(0)
            Eb[:, j] = e
        # the block's accumulated error reaches the columns right of the block in one product
        W[:, stop:] -= Eb @ U[start:stop, stop:]
    if not group_qparams:
        group_qparams.append(cur)
    qparams = combine_qparams_list_func(group_qparams)
    return quantize_func(DQ, qparams), DQ.to(orig_dtype), qparams


class _LockStepCalibration:
    """Runs `model` over all calibration samples at once, one thread per sample, in lock step.

    Exactly one thread runs at any time.  A forward pre-hook on every watched linear parks the thread and hands its
    input to the scheduler; once every sample is parked at the same linear the scheduler folds the inputs into the
    Hessian `2/n * sum x x^T`, calls `on_linear(module, H)` (which rewrites `module.weight`) and releases the
    threads one by one to the next linear.  No sample therefore passes a linear before it has been quantized, and
    state a forward pass keeps in the model between two linears (a KV cache written and read inside one attention
    block) is never interleaved between samples."""

    def __init__(self, model: nn.Module, watched: Dict[nn.Module, str], on_linear: Callable, act_func=None):
        self.model = model
        self.watched = watched
        self.on_linear = on_linear
        self.act_func = act_func
        self._local = threading.local()

    def _pre_hook(self, module, args):
        worker = getattr(self._local, "worker", None)
        if worker is None:  # a forward outside the calibration threads passes through
            return None
        worker["at"] = (module, args[0])
        worker["parked"].set()
        worker["go"].wait()
        worker["go"].clear()
        if worker["abort"]:
            raise RuntimeError("calibration aborted")
        return None

    def _run_sample(self, worker, args):
        self._local.worker = worker
        worker["go"].wait()
        worker["go"].clear()
        try:
            with torch.no_grad():
                self.model(*args)
        except BaseException as e:  # surfaced by the scheduler
            worker["error"] = e
        worker["at"] = None
        worker["done"] = True
        worker["parked"].set()

    @staticmethod
    def _advance(worker):
        """Let one thread run to its next watched linear (or to the end of its forward pass)."""
        worker["parked"].clear()
        worker["go"].set()
        worker["parked"].wait()
        if worker.get("error") is not None:
            raise worker["error"]

    def run(self, inputs: List[_MultiInput]) -> None:
        n_samples = max(len(m.values) for m in inputs)
        per_sample = [[m.values[i] if len(m.values) > 1 else m.values[0] for m in inputs] for i in range(n_samples)]
        handles = [m.register_forward_pre_hook(self._pre_hook) for m in self.watched]
        workers = []
        try:
            for args in per_sample:
                w = {"go": threading.Event(), "parked": threading.Event(), "at": None, "done": False, "error": None,
                     "abort": False}
                w["thread"] = threading.Thread(target=self._run_sample, args=(w, args), daemon=True)
                w["thread"].start()
                workers.append(w)
            while True:
                for w in workers:
                    if not w["done"]:
                        self._advance(w)
                stops = [w["at"] for w in workers]
                if all(s is None for s in stops):
                    break
                module = stops[0][0] if stops[0] is not None else None
                if any(s is None or s[0] is not module for s in stops):
                    raise RuntimeError("calibration samples took different paths through the model")
                H, seen = None, 0
                for _, x in stops:
                    x = x.float()
                    if self.act_func is not None:
                        x = self.act_func(x)
                    n = 1 if x.dim() == 2 else x.shape[0]
                    x = x.reshape(-1, x.shape[-1])
                    if H is None:
                        H = torch.zeros((x.shape[1], x.shape[1]), dtype=torch.float32, device=x.device)
                    # running mean of 2 x^T x over the batches seen (reference :229-236)
                    H *= seen / (seen + n)
                    seen += n
                    x = x * (2.0 / seen) ** 0.5
                    H.addmm_(x.t(), x)
                for w in workers:
                    w["at"] = None
                self.on_linear(module, H)
        finally:
            for h in handles:
                h.remove()
            for w in workers:  # after an error: threads still parked leave their forward pass with an exception
                if not w["done"]:
                    w["abort"] = True
                    w["go"].set()
            for w in workers:
                w["thread"].join(timeout=60)


class GPTQQuantizer(Quantizer):
    """Base of the calibrated quantizers (reference :400-519).  A subclass sets, before calling `super().__init__()`:
    `get_qparams_func(w)`, `quantize_func(w, qparams)`, `dequantize_func(q, qparams)` (each for a whole weight, one
    group or one column), `combine_qparams_list_func(list)`, `skip_layer_func(weight) -> bool`,
    `make_names_and_values_dict_func(q, qparams) -> {buffer name: tensor}`, optionally `act_fake_quant_func(x)`."""

    def __init__(self):
        for name in ("get_qparams_func", "quantize_func", "dequantize_func", "combine_qparams_list_func",
                     "make_names_and_values_dict_func"):
            assert getattr(self, name, None) is not None, f"{type(self).__name__} must define {name}"

    @torch.no_grad()
    def _create_quantized_state_dict(self, model, inputs, blocksize, percdamp, groupsize) -> Dict[str, torch.Tensor]:
        """Calibrate and quantize every eligible `nn.Linear` of `model` in execution order.  The model is left with
        the dequantized GPTQ weights in place of the originals; the returned state dict holds, for each quantized
        linear, the entries of `make_names_and_values_dict_func` instead of `weight`."""
        skip = getattr(self, "skip_layer_func", None)
        watched = {m: fqn for fqn, m in model.named_modules()
                   if isinstance(m, nn.Linear) and not (skip is not None and skip(m.weight))}
        new_entries: Dict[str, Dict[str, torch.Tensor]] = {}

        def on_linear(module, H):
            if module in new_entries:  # a linear called twice in one pass keeps its first quantization
                return
            Q, DQ, qparams = gptq_quantize_weight(H, module.weight.data.to(H.device), self.get_qparams_func,
                                                  self.quantize_func, self.dequantize_func,
                                                  self.combine_qparams_list_func, blocksize, percdamp, groupsize)
            module.weight.data.copy_(DQ.to(module.weight.device))
            new_entries[module] = self.make_names_and_values_dict_func(Q, qparams)

        _LockStepCalibration(model, watched, on_linear, getattr(self, "act_fake_quant_func", None)).run(inputs)
        state_dict = {k: v for k, v in model.state_dict().items() if "kv_cache" not in k}
        for module, entries in new_entries.items():
            fqn = watched[module]
            state_dict.pop(f"{fqn}.weight", None)
            for name, value in entries.items():
                state_dict[f"{fqn}.{name}"] = value
        return state_dict

    def _convert_for_runtime(self, model: nn.Module) -> nn.Module:
        raise NotImplementedError("_convert_for_runtime not implemented")

    def quantize(self, model: nn.Module, inputs: List[_MultiInput], **kwargs: Any) -> nn.Module:
        raise NotImplementedError


class Int4WeightOnlyGPTQQuantizer(GPTQQuantizer):
    """GPTQ-calibrated groupwise int4 weight-only quantizer by module swap (reference :675-758).

    `quantize(model, inputs)` takes one `_MultiInput` per positional argument of `model.forward`, each holding that
    argument's value for every calibration sample (a single value is shared by all samples)."""

    def __init__(self, blocksize=128, percdamp=0.01, groupsize=64, inner_k_tiles=8, padding_allowed=True,
                 device: torch.device = torch.device("cuda")):
        self.blocksize = blocksize
        self.percdamp = percdamp
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles
        self.padding_allowed = padding_allowed
        self.device = torch.device(device)
        self.act_fake_quant_func = None
        n_bit = 4
        self.get_qparams_func = lambda w: get_groupwise_affine_qparams(w, n_bit, groupsize)
        self.quantize_func = lambda w, qparams: groupwise_affine_quantize_tensor_from_qparams(
            w, qparams[0], qparams[1], n_bit, groupsize)
        self.dequantize_func = lambda q, qparams: groupwise_affine_dequantize_tensor_from_qparams(
            q, qparams[0], qparams[1], n_bit, groupsize)
        self.combine_qparams_list_func = lambda qparams_list: [torch.cat(x, dim=1) for x in zip(*qparams_list)]
        self.skip_layer_func = lambda weight: not (_check_linear_int4_k(weight.shape[-1], groupsize) or padding_allowed)
        self.make_names_and_values_dict_func = self._pack
        super().__init__()

    def _pack(self, q: torch.Tensor, qparams) -> Dict[str, torch.Tensor]:
        """Codes `[N, K]` + (scales, zeros) `[N, K/g]` -> the two buffers of `WeightOnlyInt4Linear`, with the input
        features padded to a multiple of 1024 where the layer needs it (padding groups: scale 1, zero 1, code 0, as
        the reference pads them, :733-743)."""
        k = q.shape[1]
        new_k = k if _check_linear_int4_k(k, self.groupsize, self.inner_k_tiles) else find_multiple(k, 1024)
        q = F.pad(q.to(torch.int32).to(self.device), pad=(0, new_k - k))
        scales = qparams[0].to(torch.bfloat16).to(self.device)
        zeros = qparams[1].to(torch.bfloat16).to(self.device)
        scales_and_zeros = pack_tinygemm_scales_and_zeros(scales, zeros)
        extra_groups = new_k // self.groupsize - scales_and_zeros.shape[0]
        scales_and_zeros = F.pad(scales_and_zeros, pad=(0, 0, 0, 0, 0, extra_groups), value=1)
        packed, _ = torch.ops.torchao.int4wo_pack(q, scales_and_zeros[:, :, 0].t().contiguous(),
                                                  scales_and_zeros[:, :, 1].t().contiguous(), self.groupsize)
        return {"weight": packed, "scales_and_zeros": scales_and_zeros}

    def _convert_for_runtime(self, model: nn.Module) -> nn.Module:
        replace_linear_int4(model, self.groupsize, self.inner_k_tiles, self.padding_allowed,
                            skip_layer_func=self.skip_layer_func)
        return model

    def quantize(self, model: nn.Module, inputs: List[_MultiInput], **kwargs: Any) -> nn.Module:
        state_dict = self._create_quantized_state_dict(model, inputs, self.blocksize, self.percdamp, self.groupsize)
        model = self._convert_for_runtime(model)
        model.load_state_dict(state_dict, strict=False)
        return model
