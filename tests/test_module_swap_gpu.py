"""GPU tests of the module-swap int4 quantizer (`Int4WeightOnlyQuantizer` / `WeightOnlyInt4Linear`, reference
torchao/quantization/GPTQ.py:521-673): buffers bit-exact against the oracle (codes, and `scales_and_zeros` in the
reference's own [K/g, N, 2] form), forward within 1e-3 relative L2 of the fp32-accumulated dequantize-then-linear
oracle and identical to the tensor-subclass path, padding / skipping rules as in the reference."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

from _util import bits16, make_act, make_weight, rel_l2

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


class _Toy(nn.Module):
    def __init__(self, k=256, h=512, n=64):
        super().__init__()
        self.l1 = nn.Linear(k, h, bias=False)
        self.inner = nn.Sequential(nn.Linear(h, n, bias=False))

    def forward(self, x):
        return self.inner(self.l1(x))


def _oracle_layer(oracle, w, g):
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, g, w.shape[0], w.shape[1])
    dq = oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero, oracle.BF16, 0, 15, 1, oracle.BF16)
    return codes, scale, zero, dq


@pytest.mark.parametrize("g", [32, 64, 128, 256])
def test_buffers_and_forward_match_oracle(oracle, g):
    from ao_amd.quantization.GPTQ import Int4WeightOnlyQuantizer, WeightOnlyInt4Linear

    print(f"case module swap g={g}", flush=True)
    dev = _dev()
    m = _Toy().bfloat16()
    w1 = make_weight(512, 256, seed=5 + g)
    w2 = make_weight(64, 512, seed=6 + g)
    m.l1.weight.data.copy_(w1)
    m.inner[0].weight.data.copy_(w2)
    m = Int4WeightOnlyQuantizer(groupsize=g).quantize(m.to(dev))
    assert isinstance(m.l1, WeightOnlyInt4Linear) and isinstance(m.inner[0], WeightOnlyInt4Linear)
    assert set(m.state_dict()) == {"l1.weight", "l1.scales_and_zeros", "inner.0.weight", "inner.0.scales_and_zeros"}

    h_ref = None
    for mod, w in ((m.l1, w1), (m.inner[0], w2)):
        N, K = w.shape
        codes, scale, zero, _ = _oracle_layer(oracle, w, g)
        assert mod.scales_and_zeros.shape == (K // g, N, 2) and mod.scales_and_zeros.dtype is torch.bfloat16
        sz = bits16(mod.scales_and_zeros)
        assert np.array_equal(sz[:, :, 0].T, scale) and np.array_equal(sz[:, :, 1].T, zero)
        c, s, z = torch.ops.torchao.int4wo_unpack(mod.weight, mod._interleaved_qparams(), N, K, g)
        assert np.array_equal(c.cpu().numpy(), codes)
        assert np.array_equal(bits16(s), scale) and np.array_equal(bits16(z), zero)

    for M in (1, 7, 33):
        x = make_act(M, 256, seed=M)
        with torch.no_grad():
            h = m.l1(x.to(dev))
            y = m(x.to(dev))
        assert y.dtype is torch.bfloat16 and y.shape == (M, 64)
        _, _, _, dq1 = _oracle_layer(oracle, w1, g)
        _, _, _, dq2 = _oracle_layer(oracle, w2, g)
        h_ref = oracle.linear(bits16(x), oracle.BF16, dq1, oracle.BF16)
        assert rel_l2(h.float().cpu().numpy(), h_ref) <= 1e-3 + 2.0 ** -8  # bf16 output rounding on top of the kernel's 1e-3
        y_ref = oracle.linear(bits16(h), oracle.BF16, dq2, oracle.BF16)
        assert rel_l2(y.float().cpu().numpy(), y_ref) <= 1e-3 + 2.0 ** -8


def test_same_result_as_tensor_subclass_path():
    """The module-swap layer and `quantize_(model, int4_weight_only())` hold the same codes and qparams and call the
    same kernel: outputs are identical bit for bit."""
    import ao_amd
    from ao_amd.quantization.GPTQ import Int4WeightOnlyQuantizer

    dev = _dev()
    torch.manual_seed(3)
    base = _Toy(512, 1024, 256).bfloat16().to(dev)
    a = Int4WeightOnlyQuantizer(groupsize=64).quantize(copy.deepcopy(base))
    b = copy.deepcopy(base)
    ao_amd.quantize_(b, ao_amd.int4_weight_only(group_size=64))
    for shape in [(1, 512), (5, 512), (2, 40, 512)]:
        x = torch.randn(*shape, device=dev).bfloat16()
        with torch.no_grad():
            assert torch.equal(a(x), b(x))


def test_state_dict_round_trip_and_device_move():
    from ao_amd.quantization.GPTQ import Int4WeightOnlyQuantizer

    dev = _dev()
    torch.manual_seed(4)
    base = _Toy().bfloat16()
    q = Int4WeightOnlyQuantizer(groupsize=128)
    m = q.quantize(copy.deepcopy(base).to(dev))
    x = torch.randn(3, 256, device=dev).bfloat16()
    with torch.no_grad():
        y = m(x)
    sd = {k: v.cpu() for k, v in m.state_dict().items()}
    # quantizing a CPU-resident model works too: the weights are quantized on the quantizer's device, the swapped
    # modules are created where the float modules lived and moved afterwards, as in the reference's tests
    m2 = q.quantize(copy.deepcopy(base)).to(dev)
    with torch.no_grad():
        assert torch.equal(m2(x), y)
    m3 = q._convert_for_runtime(copy.deepcopy(base)).to(dev)
    m3.load_state_dict(sd)
    with torch.no_grad():
        assert torch.equal(m3(x), y)
        # overwriting the qparams in place must be picked up by the cached interleaved copy
        m3.l1.scales_and_zeros.mul_(2)
        assert not torch.equal(m3(x), y)
        m3.load_state_dict(sd)
        assert torch.equal(m3(x), y)


def test_input_dtype_is_restored_and_leading_dims():
    from ao_amd.quantization.GPTQ import Int4WeightOnlyQuantizer

    dev = _dev()
    torch.manual_seed(5)
    m = Int4WeightOnlyQuantizer(groupsize=32).quantize(_Toy().bfloat16().to(dev))
    x = torch.randn(2, 3, 256, device=dev)
    with torch.no_grad():
        y32 = m.l1(x)
        y16 = m.l1(x.half())
        ybf = m.l1(x.bfloat16())
    assert y32.dtype is torch.float32 and y16.dtype is torch.float16 and y32.shape == (2, 3, 512)
    assert torch.equal(y32, ybf.float())


def test_padding_and_skipping_rules(oracle):
    """in_features = 192 is a multiple of the group size but not of 16 * inner_k_tiles: padded to 1024 input
    features with zero weights when padding is allowed (reference :623-632, :547-551), left as nn.Linear otherwise."""
    from ao_amd.quantization.GPTQ import Int4WeightOnlyQuantizer, WeightOnlyInt4Linear

    dev = _dev()
    lin = nn.Sequential(nn.Linear(192, 128, bias=False)).bfloat16()
    w = make_weight(128, 192, seed=9)
    lin[0].weight.data.copy_(w)
    kept = Int4WeightOnlyQuantizer(groupsize=64, padding_allowed=False).quantize(copy.deepcopy(lin).to(dev))
    assert type(kept[0]) is nn.Linear and torch.equal(kept[0].weight.cpu(), w)

    padded = Int4WeightOnlyQuantizer(groupsize=64, padding_allowed=True).quantize(copy.deepcopy(lin).to(dev))
    mod = padded[0]
    assert isinstance(mod, WeightOnlyInt4Linear) and mod.padding and mod.in_features == 1024 and mod.origin_in_features == 192
    assert mod.scales_and_zeros.shape == (16, 128, 2)
    wp = torch.zeros(128, 1024).bfloat16()
    wp[:, :192] = w
    codes, scale, zero, dq = _oracle_layer(oracle, wp, 64)
    sz = bits16(mod.scales_and_zeros)
    assert np.array_equal(sz[:, :, 0].T, scale) and np.array_equal(sz[:, :, 1].T, zero)
    x = make_act(4, 192, seed=2)
    with torch.no_grad():
        y = mod(x.to(dev))
    xp = torch.zeros(4, 1024).bfloat16()
    xp[:, :192] = x
    y_ref = oracle.linear(bits16(xp), oracle.BF16, dq, oracle.BF16)
    assert rel_l2(y.float().cpu().numpy(), y_ref) <= 1e-3 + 2.0 ** -8

    # inner_k_tiles = 2 makes 192 eligible without padding
    direct = Int4WeightOnlyQuantizer(groupsize=64, padding_allowed=False, inner_k_tiles=2).quantize(copy.deepcopy(lin).to(dev))
    assert isinstance(direct[0], WeightOnlyInt4Linear) and not direct[0].padding and direct[0].in_features == 192


def test_constructor_checks():
    from ao_amd.quantization.GPTQ import Int4WeightOnlyQuantizer, WeightOnlyInt4Linear

    with pytest.raises(AssertionError):
        Int4WeightOnlyQuantizer(groupsize=48)
    with pytest.raises(AssertionError):
        Int4WeightOnlyQuantizer(inner_k_tiles=3)
    with pytest.raises(AssertionError, match="bias=False"):
        WeightOnlyInt4Linear(256, 64, bias=True)
    with pytest.raises(AssertionError, match="out_features % 8"):
        WeightOnlyInt4Linear(256, 36)
    biased = nn.Sequential(nn.Linear(256, 64, bias=True)).bfloat16().to(_dev())
    with pytest.raises(AssertionError, match="bias=False"):
        Int4WeightOnlyQuantizer(groupsize=64).quantize(biased)


def test_module_swapped_llama_decodes_token_by_token():
    """A Llama-architecture model whose linears were swapped for `WeightOnlyInt4Linear` modules is not a candidate for
    the fused decode step (that one reads tensor-subclass weights); it decodes through the modules, eagerly and under
    graph capture, with the same tokens."""
    from ao_amd._models.llama.generate import build_random_model, generate
    from ao_amd.quantization.GPTQ import Int4WeightOnlyQuantizer, WeightOnlyInt4Linear

    print("case module swap llama decode", flush=True)
    dev = _dev()
    model = Int4WeightOnlyQuantizer(groupsize=64).quantize(build_random_model("tiny128", dev))
    assert isinstance(model.output, WeightOnlyInt4Linear)
    prompt = torch.arange(3, 19, dtype=torch.int, device=dev)
    eager = generate(model, prompt, 8, greedy=True)
    assert model.fused_decode_kind() is None
    graphed = generate(model, prompt, 8, greedy=True, use_graph=True)
    assert eager.shape == (24,) and torch.equal(eager, graphed)
