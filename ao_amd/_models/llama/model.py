"""Llama-architecture decoder used by the decode benchmark.

Same architecture, module names and cache semantics as torchao/_models/llama/model.py:78-266
(gpt-fast): fused `wqkv` projection, grouped-query attention over a static KV cache, RMSNorm,
interleaved-pair RoPE, SwiGLU feed-forward.  State-dict keys are identical, so a checkpoint written for
the reference model loads here.
"""
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn import functional as F

from ...utils import find_multiple

__all__ = ["ModelArgs", "Transformer", "transformer_configs", "prepare_inputs_for_model"]


transformer_configs = {
    "7B": dict(n_layer=32, n_head=32, dim=4096),
    "13B": dict(n_layer=40, n_head=40, dim=5120),
    "70B": dict(n_layer=80, n_head=64, dim=8192, n_local_heads=8, intermediate_size=28672),
    "Mistral-7B": dict(n_layer=32, n_head=32, n_local_heads=8, dim=4096, intermediate_size=14336, vocab_size=32000),
    "stories15M": dict(n_layer=6, n_head=6, dim=288),
    "Llama-3-8B": dict(block_size=8192, n_layer=32, n_head=32, n_local_heads=8, dim=4096, intermediate_size=14336,
                       vocab_size=128256),
    # two-layer model of Llama-3-8B width for smoke tests
    "Llama-3-8B-2L": dict(block_size=8192, n_layer=2, n_head=32, n_local_heads=8, dim=4096, intermediate_size=14336,
                          vocab_size=128256),
    # small model with the head size of the fused decode kernels
    "tiny128": dict(block_size=512, n_layer=2, n_head=4, n_local_heads=2, dim=512, intermediate_size=1024,
                    vocab_size=1024),
    "tiny": dict(block_size=256, n_layer=2, n_head=4, n_local_heads=2, dim=256, intermediate_size=512, vocab_size=512),
}


@dataclass
class ModelArgs:
    block_size: int = 2048
    vocab_size: int = 32000
    n_layer: int = 32
    n_head: int = 32
    dim: int = 4096
    intermediate_size: Optional[int] = None
    n_local_heads: int = -1
    head_dim: int = 64
    rope_base: float = 10000
    norm_eps: float = 1e-5

    def __post_init__(self):
        if self.n_local_heads == -1:
            self.n_local_heads = self.n_head
        if self.intermediate_size is None:
            self.intermediate_size = find_multiple(int(2 * 4 * self.dim / 3), 256)
        self.head_dim = self.dim // self.n_head

    @classmethod
    def from_name(cls, name: str):
        if name in transformer_configs:
            return cls(**transformer_configs[name])
        matches = sorted((c for c in transformer_configs if c in str(name)), key=len, reverse=True)
        if not matches:
            raise KeyError(f"unknown model name {name}")
        return cls(**transformer_configs[matches[0]])


def prepare_inputs_for_model(inps: Tensor, max_new_tokens: int = 1):
    if inps.dim() > 2:
        raise ValueError(f"Expected input to be of dim 1 or 2, but got {inps.dim()}")
    return inps.view(1, -1), torch.arange(0, inps.numel(), device=inps.device)


def precompute_freqs_cis(seq_len: int, n_elem: int, base: float = 10000, dtype=torch.bfloat16, device=None) -> Tensor:
    """[seq_len, n_elem/2, 2] table of (cos, sin) of position * base^(-2i/n_elem)."""
    inv = 1.0 / (base ** (torch.arange(0, n_elem, 2, device=device)[: n_elem // 2].float() / n_elem))
    ang = torch.outer(torch.arange(seq_len, device=device).float(), inv)
    return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(dtype)


def apply_rotary_emb(x: Tensor, freqs_cis: Tensor) -> Tensor:
    """Rotate consecutive pairs (x[2i], x[2i+1]) of the head dimension; x: [B, S, H, D]."""
    xs = x.float().reshape(*x.shape[:-1], -1, 2)
    fc = freqs_cis.view(1, xs.size(1), 1, xs.size(3), 2)
    out = torch.stack([xs[..., 0] * fc[..., 0] - xs[..., 1] * fc[..., 1],
                       xs[..., 1] * fc[..., 0] + xs[..., 0] * fc[..., 1]], -1)
    return out.flatten(3).type_as(x)


class KVCache(nn.Module):
    def __init__(self, max_batch_size, max_seq_length, n_heads, head_dim, dtype=torch.bfloat16, device=None):
        super().__init__()
        shape = (max_batch_size, n_heads, max_seq_length, head_dim)
        self.register_buffer("k_cache", torch.zeros(shape, dtype=dtype, device=device), persistent=False)
        self.register_buffer("v_cache", torch.zeros(shape, dtype=dtype, device=device), persistent=False)

    def update(self, input_pos, k_val, v_val):
        """input_pos: [S]; k_val, v_val: [B, H, S, D].  Returns the full caches."""
        assert input_pos.shape[0] == k_val.shape[2]
        self.k_cache[:, :, input_pos] = k_val
        self.v_cache[:, :, input_pos] = v_val
        return self.k_cache, self.v_cache


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: Tensor) -> Tensor:
        xf = x.float()
        normed = (xf * torch.rsqrt(torch.mean(xf * xf, dim=-1, keepdim=True) + self.eps)).type_as(x)
        return normed * self.weight


class Attention(nn.Module):
    def __init__(self, config: ModelArgs):
        super().__init__()
        assert config.dim % config.n_head == 0
        total_head_dim = (config.n_head + 2 * config.n_local_heads) * config.head_dim
        self.wqkv = nn.Linear(config.dim, total_head_dim, bias=False)
        self.wo = nn.Linear(config.dim, config.dim, bias=False)
        self.kv_cache: Optional[KVCache] = None
        self.n_head = config.n_head
        self.head_dim = config.head_dim
        self.n_local_heads = config.n_local_heads
        self.dim = config.dim
        self._register_load_state_dict_pre_hook(self._fuse_qkv_hook)

    def _fuse_qkv_hook(self, state_dict, prefix, *args):
        if prefix + "wq.weight" in state_dict:
            parts = [state_dict.pop(prefix + n + ".weight") for n in ("wq", "wk", "wv")]
            state_dict[prefix + "wqkv.weight"] = torch.cat(parts)

    def forward(self, x: Tensor, freqs_cis: Tensor, mask: Tensor, input_pos: Optional[Tensor] = None) -> Tensor:
        bsz, seqlen, _ = x.shape
        kv_size = self.n_local_heads * self.head_dim
        q, k, v = self.wqkv(x).split([self.dim, kv_size, kv_size], dim=-1)
        q = apply_rotary_emb(q.view(bsz, seqlen, self.n_head, self.head_dim), freqs_cis).transpose(1, 2)
        k = apply_rotary_emb(k.view(bsz, seqlen, self.n_local_heads, self.head_dim), freqs_cis).transpose(1, 2)
        v = v.view(bsz, seqlen, self.n_local_heads, self.head_dim).transpose(1, 2)
        if self.kv_cache is not None:
            k, v = self.kv_cache.update(input_pos, k, v)
        rep = self.n_head // self.n_local_heads
        k = k.repeat_interleave(rep, dim=1)
        v = v.repeat_interleave(rep, dim=1)
        y = F.scaled_dot_product_attention(q, k, v, attn_mask=mask, dropout_p=0.0)
        return self.wo(y.transpose(1, 2).contiguous().view(bsz, seqlen, self.dim))


class FeedForward(nn.Module):
    def __init__(self, config: ModelArgs):
        super().__init__()
        self.w1 = nn.Linear(config.dim, config.intermediate_size, bias=False)
        self.w3 = nn.Linear(config.dim, config.intermediate_size, bias=False)
        self.w2 = nn.Linear(config.intermediate_size, config.dim, bias=False)

    def forward(self, x: Tensor) -> Tensor:
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


class TransformerBlock(nn.Module):
    def __init__(self, config: ModelArgs):
        super().__init__()
        self.attention = Attention(config)
        self.feed_forward = FeedForward(config)
        self.ffn_norm = RMSNorm(config.dim, config.norm_eps)
        self.attention_norm = RMSNorm(config.dim, config.norm_eps)

    def forward(self, x: Tensor, input_pos: Tensor, freqs_cis: Tensor, mask: Tensor) -> Tensor:
        h = x + self.attention(self.attention_norm(x), freqs_cis, mask, input_pos)
        return h + self.feed_forward(self.ffn_norm(h))


class Transformer(nn.Module):
    def __init__(self, config: ModelArgs):
        super().__init__()
        self.config = config
        self.tok_embeddings = nn.Embedding(config.vocab_size, config.dim)
        self.layers = nn.ModuleList(TransformerBlock(config) for _ in range(config.n_layer))
        self.norm = RMSNorm(config.dim, eps=config.norm_eps)
        self.output = nn.Linear(config.dim, config.vocab_size, bias=False)
        self.freqs_cis: Optional[Tensor] = None
        self.causal_mask: Optional[Tensor] = None
        self.max_batch_size = -1
        self.max_seq_length = -1
        # single-token batch-1 steps go through the fused HIP decode path whenever the model qualifies
        self.use_fused_decode = True

    @classmethod
    def from_name(cls, name: str):
        return cls(ModelArgs.from_name(name))

    def setup_caches(self, max_batch_size: int, max_seq_length: int):
        if self.max_seq_length >= max_seq_length and self.max_batch_size >= max_batch_size:
            return
        max_seq_length = find_multiple(max_seq_length, 8)
        self.max_seq_length, self.max_batch_size = max_seq_length, max_batch_size
        dtype = self.output.weight.dtype
        for name in ("scales", "scales_and_zeros"):  # module-swapped head: the compute dtype is that of its scales
            if hasattr(self.output, name):
                dtype = getattr(self.output, name).dtype
        w_scale = getattr(self.output.weight, "scale", None)  # FPx weight subclass: reports float32, computes in fp16
        if torch.is_tensor(w_scale) and dtype is torch.float32:
            dtype = w_scale.dtype
        device = self.tok_embeddings.weight.device
        for b in self.layers:
            b.attention.kv_cache = KVCache(max_batch_size, max_seq_length, self.config.n_local_heads,
                                           self.config.head_dim, dtype, device)
        self.freqs_cis = precompute_freqs_cis(self.config.block_size, self.config.head_dim, self.config.rope_base,
                                              dtype, device)
        self.causal_mask = torch.tril(torch.ones(max_seq_length, max_seq_length, dtype=torch.bool, device=device))

    def _decode_linears(self):
        return [self.output] + [m for b in self.layers for m in (b.attention.wqkv, b.attention.wo, b.feed_forward.w1,
                                                                 b.feed_forward.w3, b.feed_forward.w2)]

    def fused_decode_kind(self) -> Optional[str]:
        """"int4" / "int8" / "fp6" when a batch-1 single-token step can run on the HIP decode path, else None.  int4:
        every linear an int4 weight in the gfx950 layout with one group size; int8: every linear a per-channel int8
        weight in the plain layout with in_features a multiple of 128, both with bf16 everywhere; fp6: every linear an
        FPx weight on an fp16 model; in all cases head_dim 128 and caches set up for batch 1."""
        from ...dtypes.affine_quantized_tensor import AffineQuantizedTensor, Gfx950WaveTiledAQTLayout, PlainAQTLayout

        if self.freqs_cis is None or self.max_batch_size != 1 or self.config.head_dim != 128 \
                or self.max_seq_length > 16384:
            return None
        if self.tok_embeddings.weight.dtype is torch.float16:
            return "fp6" if self._fp6_decode_ready() else None
        if self.tok_embeddings.weight.dtype is not torch.bfloat16:
            return None
        kinds, groups = set(), set()
        for lin in self._decode_linears():
            if not isinstance(lin, nn.Linear):  # module-swapped layers (WeightOnlyInt4Linear, ...) run as modules
                return None
            w = lin.weight
            if lin.bias is not None or not isinstance(w, AffineQuantizedTensor) or w.dtype is not torch.bfloat16 \
                    or not w.is_cuda:
                return None
            lay = w.layout_tensor
            if isinstance(lay, Gfx950WaveTiledAQTLayout) and not lay.transposed:
                kinds.add("int4")
                groups.add(lay.group_size)
            elif isinstance(lay, PlainAQTLayout) and lay.int_data.dtype is torch.int8 and lay.int_data.dim() == 2 \
                    and lay.int_data.is_contiguous() and lay.int_data.shape[1] % 128 == 0 \
                    and lay.scale.numel() == lay.int_data.shape[0] and lay.scale.dtype is torch.bfloat16:
                kinds.add("int8")
            else:
                return None
        if kinds == {"int4"} and len(groups) == 1 and self.config.intermediate_size % 16 == 0:
            return "int4"
        return "int8" if kinds == {"int8"} else None

    def _fp6_decode_ready(self) -> bool:
        from ...prototype.quant_llm import QuantLlmLinearWeight

        for lin in self._decode_linears():
            if not isinstance(lin, nn.Linear) or lin.bias is not None or not isinstance(lin.weight, QuantLlmLinearWeight) \
                    or not lin.weight.fpx_data.is_cuda or lin.weight.scale.dtype is not torch.float16:
                return False
        return self.freqs_cis.dtype is torch.float16

    def fused_decode_ready(self) -> bool:
        return self.fused_decode_kind() is not None

    @staticmethod
    def qkv_ksplit(n_rows: int, n_cu: int = 256) -> int:
        """2 when the fused qkv weight's 16-row blocks would leave half of the CUs with one workgroup more than the
        others (Llama-3-8B: 384 blocks on 256 CUs), else 1."""
        blocks = (n_rows + 15) // 16
        frac = (blocks % n_cu) / n_cu
        return 2 if blocks < 4 * n_cu and 0.25 <= frac <= 0.75 else 1

    @staticmethod
    def _gate_up_pair(ff):
        """w1 and w3 of a feed-forward block as one packed weight with gate and up rows interleaved in eights, built
        on first use and rebuilt when either weight is replaced.  One launch of twice the row blocks, half the work
        each, spreads evenly over the CUs where two row-block streams per workgroup do not."""
        from ... import ops

        g, u = ff.w1.weight.layout_tensor, ff.w3.weight.layout_tensor
        srcs = (g.packed_weight, u.packed_weight, g.scale_and_zero, u.scale_and_zero)
        key = tuple((t.data_ptr(), t._version) for t in srcs)
        cached = getattr(ff, "_gate_up_pair_cache", None)
        if cached is None or cached[0] != key:
            pair, pair_q = ops.int4wo_interleave_pair(g.packed_weight, g.scale_and_zero, u.packed_weight,
                                                      u.scale_and_zero, g.N, g.K, g.group_size)
            cached = (key, pair, pair_q, g.group_size, g.N)
            ff._gate_up_pair_cache = cached
        return cached[1:]

    def _fused_layer(self, b, x: Tensor, pos: Tensor) -> Tensor:
        """One transformer block of the int4 decode step on the hidden state x [1, dim]: five launches (norm + qkv,
        attention, wo + residual, norm + gate/up + SwiGLU over the interleaved pair, down + residual)."""
        from ... import ops

        cfg = self.config

        def lin(x, layer, residual):
            lay = layer.weight.layout_tensor
            return ops.int4wo_linear_residual(x, lay.packed_weight, lay.scale_and_zero, lay.group_size, lay.N, residual)

        att = b.attention
        qw = att.wqkv.weight.layout_tensor
        if self.qkv_ksplit(qw.N) > 1:
            # fp32 partial rows over two halves of K; the attention kernel adds and rounds them
            qkv = ops.int4wo_linear_partials(x, qw.packed_weight, qw.scale_and_zero, qw.group_size, qw.N,
                                             self.qkv_ksplit(qw.N), b.attention_norm.weight, b.attention_norm.eps)
        else:
            qkv = ops.int4wo_rmsnorm_linear(x, b.attention_norm.weight, b.attention_norm.eps, qw.packed_weight,
                                            qw.scale_and_zero, qw.group_size, qw.N)
        y = ops.llama_decode_attention(qkv, self.freqs_cis, pos, att.kv_cache.k_cache, att.kv_cache.v_cache,
                                       cfg.n_head, cfg.n_local_heads)
        h = lin(y, att.wo, x)
        pair, pair_q, group, n_ff = self._gate_up_pair(b.feed_forward)
        ff = ops.int4wo_swiglu_interleaved(h, pair, pair_q, group, n_ff, b.ffn_norm.weight, b.ffn_norm.eps)
        return lin(ff, b.feed_forward.w2, h)

    def _fused_decode(self, idx: Tensor, input_pos: Tensor) -> Tensor:
        """One token, batch 1: five launches per layer, then norm + head.  Same roundings as the module-by-module
        path."""
        from ... import ops

        cfg = self.config
        x = self.tok_embeddings(idx).view(1, cfg.dim)
        pos = input_pos.to(torch.int32) if input_pos.dtype is not torch.int32 else input_pos
        for b in self.layers:
            x = self._fused_layer(b, x, pos)
        ow = self.output.weight.layout_tensor
        logits = ops.int4wo_rmsnorm_linear(x, self.norm.weight, self.norm.eps, ow.packed_weight, ow.scale_and_zero,
                                           ow.group_size, ow.N)
        return logits.view(1, 1, cfg.vocab_size)

    def _fused_decode_int8(self, idx: Tensor, input_pos: Tensor) -> Tensor:
        """The same step over int8 weight-only linears: the streaming int8 kernel per linear and the decode attention
        kernel, with each RMSNorm fused into the linears it feeds and the residual add and the SiLU(gate) * up product
        fused into the linear that precedes them; w1 and w3 stream in one launch (5 launches per layer)."""
        from ... import ops

        cfg = self.config

        def lin(x, layer, residual=None, gate=None, norm=None):
            lay = layer.weight.layout_tensor
            if norm is not None:
                return ops.int8wo_rmsnorm_linear(x, norm.weight, norm.eps, lay.int_data, lay.scale.reshape(-1), gate)
            if residual is not None:
                return ops.int8wo_linear_residual(x, lay.int_data, lay.scale.reshape(-1), residual)
            if gate is not None:
                return ops.int8wo_linear_gated(x, lay.int_data, lay.scale.reshape(-1), gate)
            return ops.int8wo_linear(x, lay.int_data, lay.scale.reshape(-1))

        x = self.tok_embeddings(idx).view(1, cfg.dim)
        pos = input_pos.to(torch.int32) if input_pos.dtype is not torch.int32 else input_pos
        for b in self.layers:
            att, ffn = b.attention, b.feed_forward
            qkv = lin(x, att.wqkv, norm=b.attention_norm)
            y = ops.llama_decode_attention(qkv, self.freqs_cis, pos, att.kv_cache.k_cache, att.kv_cache.v_cache,
                                           cfg.n_head, cfg.n_local_heads)
            h = lin(y, att.wo, residual=x)
            g, u = ffn.w1.weight.layout_tensor, ffn.w3.weight.layout_tensor
            act = ops.int8wo_swiglu(h, g.int_data, g.scale.reshape(-1), u.int_data, u.scale.reshape(-1),
                                    b.ffn_norm.weight, b.ffn_norm.eps)
            x = lin(act, ffn.w2, residual=h)
        return lin(x, self.output, norm=self.norm).view(1, 1, cfg.vocab_size)

    def _fused_decode_fp6(self, idx: Tensor, input_pos: Tensor) -> Tensor:
        """The same step over FPx weights on an fp16 model: the fp6 GEMV per linear with each RMSNorm fused into the
        staging of the linear it feeds, the residual add in the epilogue, w1 and w3 in one launch with the
        SiLU(gate) * up product, and the fp16 instance of the decode attention kernel (5 launches per layer)."""
        from ... import ops

        cfg = self.config

        def lin(x, layer, residual=None, norm=None):
            w = layer.weight
            if norm is not None:
                return ops.fp6_rmsnorm_linear(w.ebits, w.mbits, x, norm.weight, norm.eps, w.native(), w.scale)
            return ops.fp6_linear_native_fused(w.ebits, w.mbits, x, w.native(), w.scale, residual, False)

        x = self.tok_embeddings(idx).view(1, cfg.dim)
        pos = input_pos.to(torch.int32) if input_pos.dtype is not torch.int32 else input_pos
        for b in self.layers:
            att, ffn = b.attention, b.feed_forward
            qkv = lin(x, att.wqkv, norm=b.attention_norm)
            y = ops.llama_decode_attention(qkv, self.freqs_cis, pos, att.kv_cache.k_cache, att.kv_cache.v_cache,
                                           cfg.n_head, cfg.n_local_heads)
            h = lin(y, att.wo, residual=x)
            g, u = ffn.w1.weight, ffn.w3.weight
            act = ops.fp6_swiglu(g.ebits, g.mbits, h, g.native(), g.scale, u.native(), u.scale, b.ffn_norm.weight,
                                 b.ffn_norm.eps)
            x = lin(act, ffn.w2, residual=h)
        return lin(x, self.output, norm=self.norm).view(1, 1, cfg.vocab_size)

    def forward(self, idx: Tensor, input_pos: Optional[Tensor] = None) -> Tensor:
        assert self.freqs_cis is not None, "Caches must be initialized first"
        if self.use_fused_decode and idx.numel() == 1 and input_pos is not None and input_pos.numel() == 1:
            kind = self.fused_decode_kind()
            if kind == "int4":
                return self._fused_decode(idx, input_pos)
            if kind == "int8":
                return self._fused_decode_int8(idx, input_pos)
            if kind == "fp6":
                return self._fused_decode_fp6(idx, input_pos)
        mask = self.causal_mask[None, None, input_pos]
        freqs_cis = self.freqs_cis[input_pos]
        x = self.tok_embeddings(idx)
        for layer in self.layers:
            x = layer(x, input_pos, freqs_cis, mask)
        return self.output(self.norm(x))
