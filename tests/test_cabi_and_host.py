"""CPU-only checks: the C-ABI library exports every symbol the header declares, and the host logic
(module walk, layout registry, shape helpers, meta-device quantization, error paths) behaves like the
reference's.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "ao_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ao_amd_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(cabi):
    names = _declared_functions()
    assert len(names) >= 10
    handle = ctypes.CDLL(cabi.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f"{n} declared in include/ao_amd.h but not exported"
    assert cabi.lib().ao_amd_abi_version() == 1
    assert set(cabi._SIGNATURES) == set(names)


def test_packed_shape_host_entry(cabi):
    from ao_amd.ops import int4wo_packed_shapes

    for (N, K, g) in [(4096, 4096, 64), (17, 64, 32), (128256, 4096, 64), (48, 192, 256), (4096, 14336, 128)]:
        Np, Kp, pb, qb = cabi.packed_shape(N, K, g)
        assert Np % 16 == 0 and Np >= N and Kp % max(128, g) == 0 and Kp >= K
        assert pb == Np * Kp // 2 and qb == Np * (Kp // g) * 4
        ps, qs = int4wo_packed_shapes(N, K, g)
        assert ps == (Np // 16, Kp // 128, 64, 4) and qs == (Np // 16, Kp // g, 16)
    L = cabi.lib()
    assert L.ao_amd_int4wo_packed_shape(16, 128, 48, None, None, None, None) != 0
    assert b"group_size" in L.ao_amd_last_error()


def test_argument_errors_without_launch(cabi):
    L = cabi.lib()
    assert L.ao_amd_int4wo_linear(None, 1, 128, 128, None, None, 16, 64, None, None, cabi.BF16, 16, None) != 0
    assert b"null" in L.ao_amd_last_error()
    assert L.ao_amd_choose_qparams_affine(None, 0, 4, 4, 4, 1, 4, 1, 0, 15, -1.0, 1, 0, 0, 0, None, None, None) != 0


def test_cpu_tensors_are_rejected():
    """There is no CPU fallback: a CPU tensor raises instead of silently computing somewhere else."""
    import ao_amd
    from ao_amd import ops
    from ao_amd.quantization import MappingType, choose_qparams_affine

    w = torch.randn(32, 128).bfloat16()
    with pytest.raises(RuntimeError):
        ops.int4wo_quantize_pack(w, 64)
    with pytest.raises(RuntimeError):
        choose_qparams_affine(w, MappingType.ASYMMETRIC, (1, 64), torch.int32, 0, 15)
    lin = torch.nn.Linear(128, 32, bias=False).bfloat16()
    with pytest.raises(RuntimeError):
        ao_amd.quantize_(lin, ao_amd.int4_weight_only(64))


def test_quantize_walks_modules_and_respects_filter():
    import ao_amd
    from ao_amd.dtypes import AffineQuantizedTensor

    class Toy(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Linear(256, 64, bias=False)
            self.inner = torch.nn.Sequential(torch.nn.Linear(64, 128), torch.nn.ReLU(), torch.nn.Linear(128, 32))
            self.emb = torch.nn.Embedding(10, 256)

    m = Toy().to(device="meta", dtype=torch.bfloat16)
    out = ao_amd.quantize(m, ao_amd.int4_weight_only(group_size=32))
    assert out is m
    assert isinstance(m.a.weight, AffineQuantizedTensor)
    assert isinstance(m.inner[0].weight, AffineQuantizedTensor) and isinstance(m.inner[2].weight, AffineQuantizedTensor)
    assert not isinstance(m.emb.weight, AffineQuantizedTensor)
    assert m.a.weight.shape == (64, 256) and m.a.weight.dtype is torch.bfloat16
    assert m.a.weight.extended_layout == "gfx950_wave_tiled" and m.a.weight.block_size == (1, 32)
    assert not m.a.weight.requires_grad
    lay = m.inner[2].weight.layout_tensor
    assert lay.packed_weight.shape == (2, 1, 64, 4) and lay.scale_and_zero.shape == (2, 4, 16)
    # second call: already-quantized weights are skipped
    before = m.a.weight
    ao_amd.quantize_(m, ao_amd.int4_weight_only(group_size=32))
    assert m.a.weight is before

    m2 = Toy().to(device="meta", dtype=torch.bfloat16)
    ao_amd.quantize_(m2, ao_amd.int4_weight_only(64), filter_fn=lambda mod, fqn: isinstance(mod, torch.nn.Linear) and fqn == "inner.0")
    assert isinstance(m2.inner[0].weight, AffineQuantizedTensor) and not isinstance(m2.a.weight, AffineQuantizedTensor)


def test_subclass_protocol_on_meta():
    from ao_amd import int4_weight_only
    from ao_amd.dtypes import AffineQuantizedTensor

    w = torch.empty(64, 256, dtype=torch.bfloat16, device="meta")
    q = int4_weight_only(64)(w)
    names, attrs = q.__tensor_flatten__()
    assert names == ["layout_tensor"]
    inner_names, inner_attrs = q.layout_tensor.__tensor_flatten__()
    assert inner_names == ["packed_weight", "scale_and_zero"] and inner_attrs == [64, 256, 64, False]
    rebuilt_layout = type(q.layout_tensor).__tensor_unflatten__(
        {n: getattr(q.layout_tensor, n) for n in inner_names}, inner_attrs, None, None)
    rebuilt = AffineQuantizedTensor.__tensor_unflatten__({"layout_tensor": rebuilt_layout}, attrs, None, None)
    assert rebuilt.shape == q.shape and rebuilt.block_size == q.block_size
    # repeated transposes keep the shape bookkeeping right (test/dtypes/test_affine_quantized.py:11-26)
    t = q.t()
    assert t.shape == (256, 64) and t.layout_tensor.transposed and t.block_size == (64, 1)
    tt = t.t()
    assert tt.shape == (64, 256) and not tt.layout_tensor.transposed
    d = q.detach()
    assert isinstance(d, AffineQuantizedTensor) and d.shape == q.shape


def test_layout_registry_and_errors():
    from ao_amd.dtypes.affine_quantized_tensor import (Gfx950WaveTiledAQTLayout, PlainAQTLayout,
                                                       get_layout_tensor_constructor)

    assert get_layout_tensor_constructor("plain") == PlainAQTLayout.from_plain
    assert get_layout_tensor_constructor("gfx950_wave_tiled") == Gfx950WaveTiledAQTLayout.from_plain
    assert get_layout_tensor_constructor("tensor_core_tiled") == Gfx950WaveTiledAQTLayout.from_plain
    with pytest.raises(ValueError, match="is not supported yet"):
        get_layout_tensor_constructor("no_such_layout")
    import ao_amd

    with pytest.raises(ValueError):
        ao_amd.int4_weight_only(group_size=48)


def test_primitive_argument_checks():
    """Error behaviour of the primitives (test_quant_primitives.py:405-448)."""
    from ao_amd.quantization import MappingType, ZeroPointDomain, choose_qparams_affine, quantize_affine

    x = torch.empty(10, 256, device="meta")
    with pytest.raises(ValueError, match="preserve_zero == False is not supported for symmetric quantization"):
        choose_qparams_affine(x, MappingType.SYMMETRIC, (1, 128), torch.int8, 0, 15, 1e-6, scale_dtype=torch.bfloat16,
                              zero_point_dtype=torch.bfloat16, preserve_zero=False)
    s, z = choose_qparams_affine(x, MappingType.ASYMMETRIC, (1, 128), torch.int8)
    assert s.shape == (10, 2) and z.shape == (10, 2)
    with pytest.raises(AssertionError, match="Unsupported input dtype:"):
        quantize_affine(x.to(torch.int32), (1, 128), s, z, torch.int8)
    with pytest.raises(RuntimeError, match="is invalid for input of size 20"):
        quantize_affine(x, (1, 1), s, z, torch.int8)
    with pytest.raises(ValueError, match="Unsupported dtype"):
        choose_qparams_affine(x, MappingType.ASYMMETRIC, (1, 128), torch.float64)
    with pytest.raises(AssertionError, match="quant_max out of bound"):
        choose_qparams_affine(x, MappingType.ASYMMETRIC, (1, 128), torch.int8, 0, 1000)
    q = quantize_affine(x, (1, 128), s, z, torch.int8, zero_point_domain=ZeroPointDomain.INT)
    assert q.shape == x.shape and q.dtype is torch.int8


def test_block_mapping_and_helpers():
    from ao_amd.quantization.quant_primitives import _as_2d_blocks, _get_reduction_params, _qparam_shape
    from ao_amd.utils import find_multiple, get_model_size_in_bytes

    assert _get_reduction_params((3, 3, 2, 10), (3, 3, 10, 10)) == ([3, 3, 5, 2, 10], [0, 1, 3, 4])
    assert _qparam_shape((1, 64), (8, 256)) == [8, 4]
    assert _as_2d_blocks((1, 64), (8, 256)) == (8, 256, 1, 64)
    assert _as_2d_blocks((8, 256), (8, 256)) == (8, 256, 8, 256)
    assert _as_2d_blocks((1, 1, 32), (2, 4, 64)) == (16, 32, 1, 32)
    assert _as_2d_blocks((1, 4, 64), (2, 4, 64)) == (2, 256, 1, 256)
    assert _as_2d_blocks((2, 4, 64), (2, 4, 64)) == (1, 512, 1, 512)
    with pytest.raises(NotImplementedError):
        _as_2d_blocks((2, 1, 64), (2, 4, 64))
    assert find_multiple(4096, 1024) == 4096 and find_multiple(100, 8) == 104 and find_multiple(3, 2, 5) == 10
    m = torch.nn.Sequential(torch.nn.Embedding(10, 8), torch.nn.Linear(8, 4, bias=False))
    assert get_model_size_in_bytes(m) == (80 + 32) * 4 and get_model_size_in_bytes(m, ignore_embeddings=True) == 32 * 4


def test_llama_model_shapes_on_meta():
    from ao_amd._models.llama.model import ModelArgs, Transformer

    cfg = ModelArgs.from_name("Llama-3-8B")
    assert (cfg.n_layer, cfg.dim, cfg.n_head, cfg.n_local_heads, cfg.intermediate_size, cfg.vocab_size,
            cfg.head_dim) == (32, 4096, 32, 8, 14336, 128256, 128)
    with torch.device("meta"):
        m = Transformer(cfg)
    n_lin = sum(p.numel() for name, p in m.named_parameters() if p.dim() == 2 and "tok_embeddings" not in name)
    assert n_lin == 7_504_658_432  # linear weights per decoded token
    assert m.layers[0].attention.wqkv.weight.shape == (6144, 4096)


def test_module_swap_host_logic(oracle):
    """Eligibility rule, module replacement on the meta device and the torch-side interleaving of the reference's
    [K/g, N, 2] qparams into the kernels' words (checked against the oracle's packer, pads included)."""
    import numpy as np
    from ao_amd.quantization.GPTQ import (WeightOnlyInt4Linear, _check_linear_int4_k, interleave_scales_and_zeros,
                                          replace_linear_int4)

    assert _check_linear_int4_k(4096, 128, 8) and not _check_linear_int4_k(192, 64, 8) and _check_linear_int4_k(192, 64, 2)
    assert not _check_linear_int4_k(4096 + 64, 128) and _check_linear_int4_k(4096 + 64, 64)

    with torch.device("meta"):
        m = torch.nn.Sequential(torch.nn.Linear(256, 64, bias=False), torch.nn.ReLU(),
                                torch.nn.Sequential(torch.nn.Linear(192, 24, bias=False)))
    replace_linear_int4(m, 64, 8, padding_allowed=False)
    assert isinstance(m[0], WeightOnlyInt4Linear) and type(m[2][0]) is torch.nn.Linear
    assert m[0].weight.shape == (4, 2, 64, 4) and m[0].scales_and_zeros.shape == (4, 64, 2)
    replace_linear_int4(m, 64, 8, padding_allowed=True, skip_layer_func=lambda w: w.shape[0] == 24)
    assert type(m[2][0]) is torch.nn.Linear
    replace_linear_int4(m, 64, 8, padding_allowed=True)
    assert isinstance(m[2][0], WeightOnlyInt4Linear) and m[2][0].in_features == 1024 and m[2][0].origin_in_features == 192

    for (N, K, g) in [(20, 96, 32), (64, 256, 64), (33, 256, 256), (16, 384, 128)]:
        gen = torch.Generator().manual_seed(N + K)
        sz = torch.randn(K // g, N, 2, generator=gen).bfloat16()
        words = interleave_scales_and_zeros(sz, g).numpy().view(np.uint32)
        Np, Kp = oracle.int4wo_padded_shape(N, K, g)
        bits = sz.view(torch.int16).numpy().view(np.uint16)
        spad = np.full((Np, Kp // g), 0x3586, np.uint16)
        zpad = np.zeros((Np, Kp // g), np.uint16)
        spad[:N, :K // g] = bits[:, :, 0].T
        zpad[:N, :K // g] = bits[:, :, 1].T
        _, q_ref = oracle.int4wo_pack(np.full((Np, Kp), 8, np.int32), spad, zpad, g)
        assert words.shape == q_ref.shape and np.array_equal(words, q_ref)


def test_dispatch_rules_are_pure_host_functions():
    """The shape rules that pick a kernel path need no GPU: prefill two-pass thresholds, context splits of the
    decode attention, K split of the fused qkv projection."""
    from ao_amd import ops
    from ao_amd._models.llama.model import Transformer

    assert ops.int4wo_two_pass(4096, 14336, 4096) and not ops.int4wo_two_pass(4095, 14336, 4096)
    assert not ops.int4wo_two_pass(2048, 4096, 4096) and ops.int4wo_two_pass(4096, 128256, 4096)
    assert not ops.int4wo_two_pass(4096, 1024, 4096) and ops.int4wo_two_pass(8192, 1024, 4096)
    assert [ops.decode_attention_splits(s) for s in (8, 1024, 1025, 4096, 4097, 8192, 8193, 16384)] == [1, 1, 4, 4, 8, 8, 16, 16]
    assert Transformer.qkv_ksplit(6144) == 2 and Transformer.qkv_ksplit(4096) == 1 and Transformer.qkv_ksplit(2048) == 2
    assert ops.int4wo_packed_shapes(48, 192, 64) == ((3, 2, 64, 4), (3, 4, 16))
    with pytest.raises(ValueError):
        ops.int4wo_packed_shapes(48, 192, 48)


def test_decode_loop_refuses_positions_past_the_kv_cache():
    """The graphed decode loop advances its position on the device; the host mirror must stop it at the end of the
    cache (the attention kernel itself only degrades to NaN there), and generate() must refuse a request that cannot fit."""
    from types import SimpleNamespace

    import torch

    from ao_amd._models.llama.generate import GraphedDecoder, generate

    gd = GraphedDecoder(SimpleNamespace(max_seq_length=4), "cpu", greedy=True)
    gd.host_pos = 4
    with pytest.raises(IndexError, match="past the KV cache"):
        gd.step()
    with pytest.raises(IndexError, match="past the KV cache"):
        gd.capture(torch.zeros(1, dtype=torch.int), pos=4)
    model = SimpleNamespace(config=SimpleNamespace(block_size=16))
    with pytest.raises(ValueError, match="do not fit"):
        generate(model, torch.zeros(10, dtype=torch.int), 10)
    with pytest.raises(ValueError, match="interactive"):
        generate(model, torch.zeros(300, dtype=torch.int), 100, interactive=True)


def test_torchao_alias_package_resolves_to_this_library():
    """`import torchao` from the repository root gives the reference's import paths for this path (torchao/__init__.py:
    31-41): the modules are the ao_amd modules themselves."""
    import ao_amd
    import torchao
    from torchao.dtypes import AffineQuantizedTensor
    from torchao.prototype.quant_llm import QuantLlmLinearWeight  # noqa: F401
    from torchao.quantization import int4_weight_only, quantize_
    from torchao.quantization.quant_api import quantize_ as quantize_again

    assert torchao.quantization is ao_amd.quantization and quantize_ is quantize_again is ao_amd.quantize_
    assert int4_weight_only is ao_amd.int4_weight_only and AffineQuantizedTensor is ao_amd.dtypes.AffineQuantizedTensor
    assert torchao.ops.quant_llm_linear is ao_amd.ops.quant_llm_linear
    import torchao._models.llama.model as m

    assert m is ao_amd._models.llama.model
    # the legacy subclass through both import paths is one class object (isinstance checks on weights made by
    # change_linear_weights_to_int4_woqtensors hold whichever path the caller imported), and no module of the library
    # is loaded a second time under the torchao name
    import sys

    from torchao.quantization.subclass import Int4WeightOnlyQuantizedLinearWeight as via_alias

    from ao_amd.quantization.subclass import Int4WeightOnlyQuantizedLinearWeight as direct

    assert via_alias is direct is torchao.quantization.Int4WeightOnlyQuantizedLinearWeight
    for name, mod in list(sys.modules.items()):
        if name.startswith("torchao.") and mod is not None:
            twin = sys.modules.get("ao_amd." + name[len("torchao."):])
            assert twin is None or twin is mod, name
