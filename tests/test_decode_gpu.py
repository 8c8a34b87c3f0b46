"""GPU tests of the decode-loop kernels: fused epilogues of the int4 linear (bit-exact against the
plain kernel + the module's rounding chain), RMSNorm and decode attention (floating point: compared with a
plain PyTorch fp32 restatement of the module, tolerances stated per test), and the fused decode step
against the module-by-module forward."""
import numpy as np
import pytest
import torch

from _util import bits16, make_act, make_weight, rel_l2

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _rb(a):
    """numpy fp32 -> bf16 (round to nearest even) -> fp32."""
    import oracle as O

    return O.bf16_bits_to_f32(O.f32_to_bf16_bits(a))


@pytest.mark.parametrize("M", [1, 3])
def test_linear_residual_epilogue(M):
    from ao_amd import ops

    dev = _dev()
    N, K, g = 256, 1024, 64
    w = make_weight(N, K, seed=21).to(dev)
    x = make_act(M, K, seed=22).to(dev)
    res = make_act(M, N, seed=23).to(dev)
    bias = (torch.randn(N) * 0.1).bfloat16().to(dev)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    y32 = ops.int4wo_linear(x, packed, qp, g, N, bias, True).cpu().numpy()
    y = ops.int4wo_linear_residual(x, packed, qp, g, N, res, bias)
    expect = _rb(_rb(y32) + res.float().cpu().numpy())
    assert np.array_equal(y.float().cpu().numpy(), expect)


@pytest.mark.parametrize("M", [1, 5])
def test_swiglu_epilogue(M):
    from ao_amd import ops

    dev = _dev()
    N, K, g = 512, 1024, 64
    wg = make_weight(N, K, seed=31).to(dev)
    wu = make_weight(N, K, seed=32).to(dev)
    x = make_act(M, K, seed=33).to(dev)
    pg, qg = ops.int4wo_quantize_pack(wg, g)
    pu, qu = ops.int4wo_quantize_pack(wu, g)
    a = ops.int4wo_linear(x, pg, qg, g, N, None, False)   # bf16, as the module chain produces
    b = ops.int4wo_linear(x, pu, qu, g, N, None, False)
    expect = (torch.nn.functional.silu(a) * b).float().cpu().numpy()
    y = ops.int4wo_swiglu(x, pg, qg, pu, qu, g, N).float().cpu().numpy()
    # same roundings as the chain; expf on the device may differ from torch's by an ulp on rare elements
    mism = np.count_nonzero(y != expect)
    assert mism <= 0.002 * y.size, f"{mism} of {y.size} elements differ"
    assert rel_l2(y, expect) <= 1e-3


def test_rmsnorm_matches_module():
    from ao_amd import ops
    from ao_amd._models.llama.model import RMSNorm

    dev = _dev()
    torch.manual_seed(3)
    x = (torch.randn(3, 4096) * 2).bfloat16().to(dev)
    norm = RMSNorm(4096, 1e-5).to(dev).bfloat16()
    norm.weight.data = (1 + 0.1 * torch.randn(4096)).bfloat16().to(dev)
    with torch.no_grad():
        ref = norm(x).float().cpu().numpy()
        out = ops.rmsnorm(x, norm.weight, norm.eps).float().cpu().numpy()
    # fp32 statistics summed in a different order: at most one bf16 ulp on a few elements
    assert rel_l2(out, ref) <= 2e-3
    assert np.count_nonzero(out != ref) <= 0.02 * out.size


@pytest.mark.parametrize("M,N,K,g", [(1, 6144, 4096, 64), (1, 512, 1024, 128), (3, 256, 2048, 32), (16, 64, 512, 256)])
def test_rmsnorm_linear_fused(M, N, K, g):
    """linear(rmsnorm(x)) in one launch against the two separate launches.  The statistics are summed in a
    different order, which can move the normalised activation by one bf16 ulp on rare elements: the outputs agree
    to 1e-3 relative L2 (fp32 comparison of bf16 results) and most are identical."""
    from ao_amd import ops

    dev = _dev()
    w = make_weight(N, K, seed=41).to(dev)
    x = (make_act(M, K, seed=42) * 3).to(dev)
    nw = (1 + 0.1 * torch.randn(K, generator=torch.Generator().manual_seed(43))).bfloat16().to(dev)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    xn = ops.rmsnorm(x, nw, 1e-5)
    ref = ops.int4wo_linear(xn, packed, qp, g, N).float().cpu().numpy()
    out = ops.int4wo_rmsnorm_linear(x, nw, 1e-5, packed, qp, g, N).float().cpu().numpy()
    assert rel_l2(out, ref) <= 1e-3
    assert np.count_nonzero(out != ref) <= 0.05 * out.size


@pytest.mark.parametrize("M", [1, 4])
def test_rmsnorm_swiglu_fused(M):
    from ao_amd import ops

    dev = _dev()
    N, K, g = 1024, 4096, 64
    wg = make_weight(N, K, seed=51).to(dev)
    wu = make_weight(N, K, seed=52).to(dev)
    x = (make_act(M, K, seed=53) * 0.5).to(dev)
    nw = (1 + 0.1 * torch.randn(K, generator=torch.Generator().manual_seed(54))).bfloat16().to(dev)
    pg, qg = ops.int4wo_quantize_pack(wg, g)
    pu, qu = ops.int4wo_quantize_pack(wu, g)
    xn = ops.rmsnorm(x, nw, 1e-5)
    ref = ops.int4wo_swiglu(xn, pg, qg, pu, qu, g, N).float().cpu().numpy()
    out = ops.int4wo_rmsnorm_swiglu(x, nw, 1e-5, pg, qg, pu, qu, g, N).float().cpu().numpy()
    assert rel_l2(out, ref) <= 1e-3
    assert np.count_nonzero(out != ref) <= 0.05 * out.size


@pytest.mark.parametrize("N,K,g", [(512, 1024, 64), (48, 256, 32), (1024, 4096, 128), (32, 512, 256)])
def test_interleave_pair_is_the_row_permutation(N, K, g):
    """Unpacking the interleaved weight gives, in every 16-row block, 8 gate rows then the 8 up rows of the same
    outputs: codes, scales and zeros bit for bit."""
    from ao_amd import ops

    dev = _dev()
    wg = make_weight(N, K, seed=71 + N).to(dev)
    wu = make_weight(N, K, seed=72 + N).to(dev)
    pg, qg = ops.int4wo_quantize_pack(wg, g)
    pu, qu = ops.int4wo_quantize_pack(wu, g)
    pp, qq = ops.int4wo_interleave_pair(pg, qg, pu, qu, N, K, g)
    got = [t.cpu() for t in ops.int4wo_unpack(pp, qq, 2 * N, K, g)]
    gate = [t.cpu() for t in ops.int4wo_unpack(pg, qg, N, K, g)]
    up = [t.cpu() for t in ops.int4wo_unpack(pu, qu, N, K, g)]
    for t, a, b in zip(got, gate, up):
        expect = torch.stack([a.reshape(N // 8, 8, -1), b.reshape(N // 8, 8, -1)], dim=1).reshape(2 * N, -1)
        assert torch.equal(t.view(torch.int16) if t.dtype is torch.bfloat16 else t,
                           expect.view(torch.int16) if expect.dtype is torch.bfloat16 else expect)


@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("N,K,g", [(1024, 4096, 64), (48, 256, 32), (14336, 4096, 64)])
def test_swiglu_interleaved_matches_two_weight_kernel(M, N, K, g):
    """Same products, same roundings as the two-weight SwiGLU kernel; the K tiles may be split over a different
    number of waves, which reorders the fp32 sums (1e-3 relative L2, nearly all elements identical).  With the
    RMSNorm fused as well."""
    from ao_amd import ops

    print(f"case swiglu interleaved M={M} N={N} K={K} g={g}", flush=True)
    dev = _dev()
    wg = make_weight(N, K, seed=81).to(dev)
    wu = make_weight(N, K, seed=82).to(dev)
    x = (make_act(M, K, seed=83) * 0.5).to(dev)
    nw = (1 + 0.1 * torch.randn(K, generator=torch.Generator().manual_seed(84))).bfloat16().to(dev)
    pg, qg = ops.int4wo_quantize_pack(wg, g)
    pu, qu = ops.int4wo_quantize_pack(wu, g)
    pp, qq = ops.int4wo_interleave_pair(pg, qg, pu, qu, N, K, g)
    ref = ops.int4wo_swiglu(x, pg, qg, pu, qu, g, N).float().cpu().numpy()
    out = ops.int4wo_swiglu_interleaved(x, pp, qq, g, N).float().cpu().numpy()
    assert rel_l2(out, ref) <= 1e-3
    assert np.count_nonzero(out != ref) <= 0.02 * out.size
    # norm fused into the staging against the two-launch chain (statistics summed in another order: an ulp of the
    # normalised activation on rare elements)
    ref_n = ops.int4wo_swiglu(ops.rmsnorm(x, nw, 1e-5), pg, qg, pu, qu, g, N).float().cpu().numpy()
    out_n = ops.int4wo_swiglu_interleaved(x, pp, qq, g, N, nw, 1e-5).float().cpu().numpy()
    assert rel_l2(out_n, ref_n) <= 1e-3
    assert np.count_nonzero(out_n != ref_n) <= 0.05 * out_n.size


def test_two_weight_swiglu_at_16_rows_of_4096():
    """16 activation rows of 4096 fill 128 KB of LDS; with two weights the cross-wave reduction arrays no longer fit
    beside them, so the launch must take the path that reads activations from global memory (and the fused-norm
    variant, which only exists on the LDS path, must say so)."""
    from ao_amd import ops

    dev = _dev()
    N, K, g, M = 256, 4096, 64, 16
    pg, qg = ops.int4wo_quantize_pack(make_weight(N, K, seed=95).to(dev), g)
    pu, qu = ops.int4wo_quantize_pack(make_weight(N, K, seed=96).to(dev), g)
    x = (make_act(M, K, seed=97) * 0.5).to(dev)
    a = ops.int4wo_linear(x, pg, qg, g, N, None, False)
    b = ops.int4wo_linear(x, pu, qu, g, N, None, False)
    expect = (torch.nn.functional.silu(a) * b).float().cpu().numpy()
    y = ops.int4wo_swiglu(x, pg, qg, pu, qu, g, N).float().cpu().numpy()
    assert rel_l2(y, expect) <= 1e-3
    nw = torch.ones(K, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="fused rmsnorm"):
        ops.int4wo_rmsnorm_swiglu(x, nw, 1e-5, pg, qg, pu, qu, g, N)


def test_swiglu_interleaved_rejects_what_it_cannot_take():
    from ao_amd import ops

    dev = _dev()
    N, K, g = 64, 512, 64
    pg, qg = ops.int4wo_quantize_pack(make_weight(N, K, seed=91).to(dev), g)
    pp, qq = ops.int4wo_interleave_pair(pg, qg, pg, qg, N, K, g)
    with pytest.raises(RuntimeError, match="interleaved swiglu"):
        ops.int4wo_swiglu_interleaved(make_act(17, K, seed=92).to(dev), pp, qq, g, N)
    p24, q24 = ops.int4wo_quantize_pack(make_weight(24, K, seed=93).to(dev), g)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        ops.int4wo_interleave_pair(p24, q24, p24, q24, 24, K, g)


def test_rmsnorm_linear_rejects_prefill_shapes():
    from ao_amd import ops

    dev = _dev()
    N, K, g = 64, 512, 64
    packed, qp = ops.int4wo_quantize_pack(make_weight(N, K, seed=61).to(dev), g)
    nw = torch.ones(K, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="fused rmsnorm"):
        ops.int4wo_rmsnorm_linear(make_act(17, K, seed=62).to(dev), nw, 1e-5, packed, qp, g, N)


@pytest.mark.parametrize("pos,S", [(0, 256), (5, 256), (130, 256), (511, 1024), (512, 1024), (700, 1024), (1023, 1024),
                                   (3, 2048), (700, 2048), (1500, 2048), (2047, 2048), (100, 8192), (5000, 8192),
                                   (8191, 8192), (12345, 16384)])
def test_decode_attention_matches_module_math(pos, S):
    """fp32 restatement of Attention.forward for one token (RoPE on interleaved pairs, cache update,
    GQA softmax attention); tolerance 1e-2 relative L2 (bf16 inputs and output).  Caches above 1024 positions run
    with 4, 8 or 16 workgroups per head and the merge launch, whatever the position."""
    from ao_amd import ops
    from ao_amd._models.llama.model import apply_rotary_emb, precompute_freqs_cis

    dev = _dev()
    torch.manual_seed(pos)
    n_head, n_kv, hd = 8, 2, 128
    assert ops.decode_attention_splits(S) == {256: 1, 1024: 1, 2048: 4, 8192: 8, 16384: 16}[S]
    qkv = torch.randn(1, (n_head + 2 * n_kv) * hd).bfloat16().to(dev)
    freqs = precompute_freqs_cis(S, hd, 10000, torch.bfloat16, dev)
    k_cache = torch.randn(1, n_kv, S, hd).bfloat16().to(dev)
    v_cache = torch.randn(1, n_kv, S, hd).bfloat16().to(dev)
    kc, vc = k_cache.clone(), v_cache.clone()
    p = torch.tensor([pos], dtype=torch.int32, device=dev)
    out = ops.llama_decode_attention(qkv, freqs, p, kc, vc, n_head, n_kv)

    q, k, v = qkv.view(1, 1, -1).split([n_head * hd, n_kv * hd, n_kv * hd], dim=-1)
    fc = freqs[p.long()]
    q = apply_rotary_emb(q.view(1, 1, n_head, hd), fc).transpose(1, 2)
    k = apply_rotary_emb(k.view(1, 1, n_kv, hd), fc).transpose(1, 2)
    v = v.view(1, 1, n_kv, hd).transpose(1, 2)
    k_ref, v_ref = k_cache.clone(), v_cache.clone()
    k_ref[:, :, pos] = k[:, :, 0]
    v_ref[:, :, pos] = v[:, :, 0]
    assert torch.equal(kc, k_ref) and torch.equal(vc, v_ref), "cache rows written by the kernel differ"
    kk = k_ref[:, :, : pos + 1].repeat_interleave(n_head // n_kv, dim=1).float()
    vv = v_ref[:, :, : pos + 1].repeat_interleave(n_head // n_kv, dim=1).float()
    att = torch.softmax((q.float() @ kk.transpose(-1, -2)) / hd**0.5, dim=-1) @ vv
    ref = att.transpose(1, 2).reshape(1, n_head * hd).cpu().numpy()
    assert rel_l2(out.float().cpu().numpy(), ref) <= 1e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 128256])
def test_argmax_bf16(n, dtype):
    from ao_amd import ops

    dev = _dev()
    g = torch.Generator().manual_seed(n)
    x = torch.randn(n, generator=g).to(dtype)
    if n >= 1000:
        x[n // 3] = x[n - 5] = x.max() + 1   # a tie: the lower index wins
    out = ops.argmax_bf16(x.to(dev))
    assert out.dtype is torch.int32 and out.shape == (1,)
    xf = x.float()
    expect = int((xf == xf.max()).nonzero()[0, 0])
    assert int(out.item()) == expect
    if n >= 8:
        x[n - 2] = float("nan")   # a NaN counts as the largest value, like torch.argmax
        x[n // 2] = float("nan")
        assert int(ops.argmax_bf16(x.to(dev)).item()) == n // 2
        assert int(ops.argmax_bf16(torch.full((n,), float("-inf")).to(dtype).to(dev)).item()) == 0


def test_fused_decode_step_matches_module_path():
    """One decode step of a small quantized model: fused HIP path vs module-by-module forward, same cache
    state.  bf16 model, different summation orders: logits agree to 3e-2 relative L2 and pick the same token."""
    from ao_amd._models.llama.generate import build_random_model, generate

    dev = _dev()
    model = build_random_model("tiny128", dev, "int4wo-64")
    prompt = torch.randint(0, model.config.vocab_size, (12,), device=dev, dtype=torch.int)
    with torch.no_grad():
        model.setup_caches(1, 64)
        assert model.fused_decode_ready()
        pos = torch.arange(12, device=dev)
        model(prompt.view(1, -1), pos)  # prefill fills the caches
        tok = torch.tensor([[7]], device=dev, dtype=torch.int)
        p = torch.tensor([12], device=dev, dtype=torch.int)
        model.use_fused_decode = False
        ref = model(tok, p).float()
        model.use_fused_decode = True
        out = model(tok, p).float()
    assert out.shape == ref.shape == (1, 1, model.config.vocab_size)
    assert rel_l2(out.cpu().numpy(), ref.cpu().numpy()) <= 3e-2
    # whole generation: graph replay of the fused path vs eager fused path
    a = generate(model, prompt, 10, use_graph=True, greedy=True)
    b = generate(model, prompt, 10, use_graph=False, greedy=True)
    assert torch.equal(a, b)


def test_fused_decode_step_int8_weight_only():
    """The same comparison for an int8 weight-only model: streaming int8 kernel + RMSNorm / attention kernels
    against the module-by-module forward; then graph replay against the eager loop."""
    from ao_amd._models.llama.generate import build_random_model, generate

    dev = _dev()
    model = build_random_model("tiny128", dev, "int8wo")
    prompt = torch.randint(0, model.config.vocab_size, (12,), device=dev, dtype=torch.int)
    with torch.no_grad():
        model.setup_caches(1, 64)
        assert model.fused_decode_kind() == "int8"
        model(prompt.view(1, -1), torch.arange(12, device=dev))
        tok = torch.tensor([[7]], device=dev, dtype=torch.int)
        p = torch.tensor([12], device=dev, dtype=torch.int)
        model.use_fused_decode = False
        ref = model(tok, p).float()
        model.use_fused_decode = True
        out = model(tok, p).float()
    assert rel_l2(out.cpu().numpy(), ref.cpu().numpy()) <= 3e-2
    a = generate(model, prompt, 10, use_graph=True, greedy=True)
    b = generate(model, prompt, 10, use_graph=False, greedy=True)
    assert torch.equal(a, b)


@pytest.mark.parametrize("ksplit", [1, 2, 3])
@pytest.mark.parametrize("M,N,K,g", [(1, 6144, 4096, 64), (1, 512, 1024, 128), (5, 256, 2048, 32)])
def test_linear_partials_sum_to_the_linear(M, N, K, g, ksplit):
    """K split over workgroups: the fp32 partial rows add up to the unsplit fp32 result (another summation order:
    1e-5 relative), with and without the fused RMSNorm; an uneven split (3 over 8 or 32 tiles) included."""
    from ao_amd import ops

    dev = _dev()
    w = make_weight(N, K, seed=101).to(dev)
    x = (make_act(M, K, seed=102) * 2).to(dev)
    nw = (1 + 0.1 * torch.randn(K, generator=torch.Generator().manual_seed(103))).bfloat16().to(dev)
    packed, qp = ops.int4wo_quantize_pack(w, g)
    parts = ops.int4wo_linear_partials(x, packed, qp, g, N, ksplit)
    assert parts.shape == (ksplit, M, N) and parts.dtype is torch.float32
    full = ops.int4wo_linear(x, packed, qp, g, N, None, True)
    assert rel_l2(parts.sum(0).cpu().numpy(), full.cpu().numpy()) <= 1e-5
    parts_n = ops.int4wo_linear_partials(x, packed, qp, g, N, ksplit, nw, 1e-5)
    full_n = ops.int4wo_linear(ops.rmsnorm(x, nw, 1e-5), packed, qp, g, N, None, True)
    assert rel_l2(parts_n.sum(0).cpu().numpy(), full_n.cpu().numpy()) <= 1e-3


@pytest.mark.parametrize("S", [64, 4096])
def test_decode_attention_from_partial_rows(S):
    """fp32 partial qkv rows are added and rounded to bf16 inside the attention kernel: same result as handing it the
    rounded sum."""
    from ao_amd import ops

    dev = _dev()
    n_head, n_kv, hd = 8, 2, 128
    gen = torch.Generator().manual_seed(5)
    parts = torch.randn(2, 1, (n_head + 2 * n_kv) * hd, generator=gen).to(dev)
    qkv = parts.sum(0).bfloat16()
    freqs = torch.randn(S, hd // 2, 2, generator=gen).bfloat16().to(dev)
    pos = torch.tensor([9], dtype=torch.int32, device=dev)
    caches = [torch.randn(1, n_kv, S, hd, generator=gen).bfloat16().to(dev) for _ in range(2)]
    k1, v1 = caches[0].clone(), caches[1].clone()
    k2, v2 = caches[0].clone(), caches[1].clone()
    a = ops.llama_decode_attention(qkv, freqs, pos, k1, v1, n_head, n_kv)
    b = ops.llama_decode_attention(parts, freqs, pos, k2, v2, n_head, n_kv)
    assert torch.equal(a, b) and torch.equal(k1, k2) and torch.equal(v1, v2)


def test_qkv_split_rule():
    from ao_amd._models.llama.model import Transformer

    assert Transformer.qkv_ksplit(6144) == 2       # Llama-3-8B: 384 row blocks on 256 CUs
    assert Transformer.qkv_ksplit(4096) == 1 and Transformer.qkv_ksplit(12288) == 1 and Transformer.qkv_ksplit(512) == 1
    assert Transformer.qkv_ksplit(2048) == 2       # half of the CUs idle otherwise


@pytest.mark.parametrize("g", [32, 64, 128, 256])
@pytest.mark.parametrize("N,K", [(8192, 512), (8192 + 16, 1024), (28672, 4096), (16384 + 48, 256)])
def test_single_row_over_many_row_blocks(N, K, g):
    """Large row counts (two and more row blocks per CU, ragged last block) at M = 1 against the same product at
    M = 2, whose second row takes another staging path and wave count: 1e-5 relative in fp32; bf16 outputs with bias
    and residual identical but for rare boundary roundings."""
    from ao_amd import ops

    if K % max(128, g):
        pytest.skip("K must be a multiple of max(128, group)")
    print(f"case many row blocks N={N} K={K} g={g}", flush=True)
    dev = _dev()
    w = make_weight(N, K, seed=111 + g).to(dev)
    x = make_act(2, K, seed=112).to(dev)
    x[1] = x[0]
    packed, qp = ops.int4wo_quantize_pack(w, g)
    y1 = ops.int4wo_linear(x[:1], packed, qp, g, N, None, True)
    y2 = ops.int4wo_linear(x, packed, qp, g, N, None, True)
    assert rel_l2(y1.cpu().numpy(), y2[:1].cpu().numpy()) <= 1e-5
    bias = (torch.randn(N, generator=torch.Generator().manual_seed(113)) * 0.1).bfloat16().to(dev)
    res = make_act(2, N, seed=114).to(dev)
    res[1] = res[0]
    z1 = ops.int4wo_linear_residual(x[:1], packed, qp, g, N, res[:1], bias).float().cpu().numpy()
    z2 = ops.int4wo_linear_residual(x, packed, qp, g, N, res, bias)[:1].float().cpu().numpy()
    assert rel_l2(z1, z2) <= 1e-3 and np.count_nonzero(z1 != z2) <= 0.01 * z1.size


def test_single_row_many_row_blocks_one_hot_is_exact(oracle):
    """One-hot activation over a weight with many row blocks: every output is a single dequantized weight, bit for
    bit the oracle's dequantize_affine."""
    from ao_amd import ops

    dev = _dev()
    N, K, g = 8192 + 32, 512, 64
    w = make_weight(N, K, seed=121)
    packed, qp = ops.int4wo_quantize_pack(w.to(dev), g)
    codes, scale, zero = oracle.int4wo_quantize(bits16(w), oracle.BF16, g, N, K)
    dq = oracle.bf16_bits_to_f32(oracle.dequantize_affine(codes, oracle.I32, (1, g), scale, oracle.BF16, zero,
                                                          oracle.BF16, 0, 15, 1, oracle.BF16))
    for k in (0, 33, 127, 128, 300, 511):
        x = torch.zeros(1, K, dtype=torch.bfloat16)
        x[0, k] = 1.0
        y = ops.int4wo_linear(x.to(dev), packed, qp, g, N, None, True).cpu().numpy()
        assert np.array_equal(y[0], dq[:, k]), k


def test_fp6_model_decodes_eagerly_and_under_graph_capture():
    """FP6-LLM e3m2 weights on an fp16 Llama-architecture model (the flow of torchao/prototype/quant_llm/README.md:9-20):
    the KV cache takes the model's fp16; the fused fp16 decode step (fp6 GEMVs with fused epilogues, fp16 RMSNorm and
    attention kernels) against the module-by-module forward; the same tokens eagerly and from a HIP graph; logits close
    to the fp16 model's."""
    from ao_amd._models.llama.generate import build_random_model, generate
    from ao_amd.prototype.quant_llm import QuantLlmLinearWeight

    dev = _dev()
    model = build_random_model("tiny128", dev, "fp6")
    ref = build_random_model("tiny128", dev).half()
    assert isinstance(model.output.weight, QuantLlmLinearWeight) and model.tok_embeddings.weight.dtype is torch.float16
    prompt = torch.randint(0, model.config.vocab_size, (12,), device=dev, dtype=torch.int)
    with torch.no_grad():
        for m in (model, ref):
            m.setup_caches(1, 64)
        assert model.layers[0].attention.kv_cache.k_cache.dtype is torch.float16
        assert model.fused_decode_kind() == "fp6" and ref.fused_decode_kind() is None
        pos = torch.arange(12, device=dev)
        got, want = model(prompt.view(1, -1), pos).float(), ref(prompt.view(1, -1), pos).float()
        assert rel_l2(got.cpu().numpy(), want.cpu().numpy()) <= 0.15
        tok = torch.tensor([[7]], device=dev, dtype=torch.int)
        p = torch.tensor([12], device=dev, dtype=torch.int)
        model.use_fused_decode = False
        unfused = model(tok, p).float()
        k_unfused = model.layers[1].attention.kv_cache.k_cache[0, :, 12].clone()
        model.use_fused_decode = True
        fused = model(tok, p).float()
        assert torch.equal(model.layers[1].attention.kv_cache.k_cache[0, :, 12], k_unfused) or rel_l2(
            model.layers[1].attention.kv_cache.k_cache[0, :, 12].float().cpu().numpy(), k_unfused.float().cpu().numpy()) <= 5e-3
    assert rel_l2(fused.cpu().numpy(), unfused.cpu().numpy()) <= 2e-2
    a = generate(model, prompt, 8, use_graph=True, greedy=True)
    b = generate(model, prompt, 8, use_graph=False, greedy=True)
    assert torch.equal(a, b)


@pytest.mark.parametrize("rows,dim", [(1, 4096), (3, 512), (2, 1000)])
def test_rmsnorm_fp16_matches_the_module_formula(rows, dim):
    """bit for bit `(x.float() * rsqrt(mean(x^2) + eps)).half() * w` (RMSNorm.forward on an fp16 model), up to elements
    where the kernel's sum of squares (another order) moves the scale by an fp32 ulp."""
    from ao_amd import ops

    dev = _dev()
    g = torch.Generator().manual_seed(rows + dim)
    x = (torch.randn(rows, dim, generator=g) * 2).half().to(dev)
    w = (1 + 0.1 * torch.randn(dim, generator=g)).half().to(dev)
    xf = x.float()
    want = (xf * torch.rsqrt(torch.mean(xf * xf, dim=-1, keepdim=True) + 1e-5)).half() * w
    got = ops.rmsnorm(x, w, 1e-5)
    assert got.dtype is torch.float16 and got.shape == want.shape
    diff = (got != want).sum().item()
    assert diff <= 0.002 * got.numel() + 1 and rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 1e-3


@pytest.mark.parametrize("M", [1, 5, 16])
def test_fp6_fused_epilogues_match_the_module_chain(M):
    from ao_amd import ops

    dev = _dev()
    N, K = 256, 512
    g = torch.Generator().manual_seed(M)
    w = (torch.randn(N, K, generator=g) * 0.05).half().to(dev)
    data, scale = ops.fp6_quantize_pack(w, 3, 2)
    native = ops.fp6_repack(data, 6)
    x = torch.randn(M, K, generator=g).half().to(dev)
    other = torch.randn(M, N, generator=g).half().to(dev)
    y = ops.fp6_linear_native(3, 2, x, native, scale)
    assert torch.equal(ops.fp6_linear_native_fused(3, 2, x, native, scale, other, False), other + y)
    got = ops.fp6_linear_native_fused(3, 2, x, native, scale, other, True).float().cpu().numpy()
    want = (torch.nn.functional.silu(other) * y).float().cpu().numpy()
    assert np.count_nonzero(got != want) <= 0.002 * got.size + 1 and rel_l2(got, want) <= 1e-3
    with pytest.raises(Exception, match="at most 16"):
        ops.fp6_linear_native_fused(3, 2, torch.zeros(17, K, dtype=torch.float16, device=dev), native, scale,
                                    torch.zeros(17, N, dtype=torch.float16, device=dev), False)


@pytest.mark.parametrize("M,N,K,fmt", [(1, 256, 512, (3, 2)), (1, 4096, 4096, (3, 2)), (1, 1024, 14336, (3, 2)),
                                       (4, 512, 1024, (2, 3)), (16, 256, 1024, (3, 2)), (2, 256, 192, (2, 2)),
                                       (1, 14336, 4096, (3, 1))])
def test_fp6_staged_gemv_fusions_match_the_separate_kernels(M, N, K, fmt):
    """The LDS-staged fp6 GEMV (weights streamed through asm-issued loads with explicit waits): plain linear identical
    to the fp16 matmul on the dequantized weight within the kernel tolerance, fused RMSNorm against the fp16 RMSNorm
    kernel + linear, two-weight SwiGLU against linear -> gated linear (same roundings: equal but for a few elements
    where the norm's sum of squares rounds apart)."""
    from ao_amd import ops

    print(f"case fp6 staged M={M} N={N} K={K} fmt={fmt}", flush=True)
    dev = _dev()
    e, m = fmt
    g = torch.Generator().manual_seed(M + N + K)
    wg = (torch.randn(N, K, generator=g) * 0.05).half().to(dev)
    wu = (torch.randn(N, K, generator=g) * 0.05).half().to(dev)
    dg, sg = ops.fp6_quantize_pack(wg, e, m)
    du, su = ops.fp6_quantize_pack(wu, e, m)
    ng, nu = ops.fp6_repack(dg, 1 + e + m), ops.fp6_repack(du, 1 + e + m)
    x = torch.randn(M, K, generator=g).half().to(dev)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).half().to(dev)
    y = ops.fp6_linear_native(e, m, x, ng, sg)
    ref = x.float() @ ops.fp6_dequantize(dg, sg, e, m).float().t()
    assert rel_l2(y.float().cpu().numpy(), ref.cpu().numpy()) <= 1e-3
    xn = ops.rmsnorm(x, nw, 1e-5)
    want = ops.fp6_linear_native(e, m, xn, ng, sg).float().cpu().numpy()
    got = ops.fp6_rmsnorm_linear(e, m, x, nw, 1e-5, ng, sg).float().cpu().numpy()
    assert rel_l2(got, want) <= 2e-3 and np.count_nonzero(got != want) <= 0.02 * got.size + 1
    want2 = ops.fp6_linear_native_fused(e, m, x, nu, su, y, True)
    got2 = ops.fp6_swiglu(e, m, x, ng, sg, nu, su)
    g2, w2 = got2.float().cpu().numpy(), want2.float().cpu().numpy()
    assert rel_l2(g2, w2) <= 1e-3 and np.count_nonzero(g2 != w2) <= 0.002 * g2.size + 1
    want3 = ops.fp6_linear_native_fused(e, m, xn, nu, su, ops.fp6_linear_native(e, m, xn, ng, sg), True)
    got3 = ops.fp6_swiglu(e, m, x, ng, sg, nu, su, nw, 1e-5)
    g3, w3 = got3.float().cpu().numpy(), want3.float().cpu().numpy()
    assert rel_l2(g3, w3) <= 2e-3 and np.count_nonzero(g3 != w3) <= 0.02 * g3.size + 1


def test_fused_decode_step_on_the_llama3_8b_configuration():
    """The benchmark's own model (32 layers, dim 4096, 32 / 8 heads, FFN 14336, vocabulary 128256, int4wo-64 on every
    linear, random weights): one fused decode step against the module-by-module forward on the same cache state, then
    16 graph-replayed tokens against the eager fused loop."""
    from ao_amd._models.llama.generate import build_random_model, generate

    dev = _dev()
    print("case fused decode Llama-3-8B", flush=True)
    model = build_random_model("Llama-3-8B", dev, "int4wo-64")
    T = 24
    prompt = torch.randint(0, model.config.vocab_size, (T,), device=dev, dtype=torch.int)
    with torch.no_grad():
        model.setup_caches(1, 64)
        assert model.fused_decode_ready()
        model(prompt.view(1, -1), torch.arange(T, device=dev))
        tok = torch.tensor([[11]], device=dev, dtype=torch.int)
        p = torch.tensor([T], device=dev, dtype=torch.int)
        model.use_fused_decode = False
        ref = model(tok, p).float()
        model.use_fused_decode = True
        out = model(tok, p).float()
        # block by block on the same inputs: the hidden state the module path feeds block l goes through the fused
        # block l as well (same cache row) and through an fp32 restatement of the block on the dequantized weights.  The
        # two bf16 paths round at different places (norm folded into the linear, SwiGLU in the epilogue, K split of the
        # qkv projection), so they differ from each other by single bf16 steps on most elements; what is held is each
        # path's distance from the fp32 block: the fused one must not be further away than the module one by more than
        # a fifth (a block that is wrong by one percent is several times further away).
        from ao_amd import ops
        from ao_amd._models.llama.model import TransformerBlock

        inputs, outputs = [], []

        def record(module, args, output):
            inputs.append(args[0].detach().clone())
            outputs.append(output.detach().clone())

        hooks = [blk.register_forward_hook(record) for blk in model.layers]
        model.use_fused_decode = False
        model(tok, p)
        for hk in hooks:
            hk.remove()
        model.use_fused_decode = True
        cfg = model.config
        with torch.device(dev):
            ref_blk = TransformerBlock(cfg).float()
        mask = model.causal_mask[None, None, p]
        freqs = model.freqs_cis[p].float()
        worst_fused, worst_module = 0.0, 0.0
        for l, blk in enumerate(model.layers):
            got = model._fused_layer(blk, inputs[l].view(1, -1), p.to(torch.int32)).float().view(-1)
            # the same block in fp32 on the dequantized weights, its cache = the rows the prompt wrote
            for name in ("attention.wqkv", "attention.wo", "feed_forward.w1", "feed_forward.w2", "feed_forward.w3"):
                lay = blk.get_submodule(name).weight.layout_tensor
                ref_blk.get_submodule(name).weight.data = ops.int4wo_dequantize(lay.packed_weight, lay.scale_and_zero, lay.N, lay.K,
                                                                                 lay.group_size).float()
            ref_blk.attention_norm.weight.data = blk.attention_norm.weight.data.float()
            ref_blk.ffn_norm.weight.data = blk.ffn_norm.weight.data.float()
            kc = blk.attention.kv_cache
            ref_blk.attention.kv_cache = type(kc)(1, kc.k_cache.shape[2], cfg.n_local_heads, cfg.head_dim, torch.float32, dev)
            ref_blk.attention.kv_cache.k_cache.copy_(kc.k_cache)
            ref_blk.attention.kv_cache.v_cache.copy_(kc.v_cache)
            exact = ref_blk(inputs[l].float(), p, freqs, mask).view(-1)
            e_fused = float((got - exact).norm() / exact.norm())
            e_module = float((outputs[l].float().view(-1) - exact).norm() / exact.norm())
            worst_fused, worst_module = max(worst_fused, e_fused), max(worst_module, e_module)
            assert e_fused <= 2e-2 and e_fused <= 1.2 * e_module + 2e-4, (l, e_fused, e_module)
        print(f"  block outputs against the fp32 block: fused worst rel-L2 = {worst_fused:.3e}, module worst = {worst_module:.3e}", flush=True)
    assert out.shape == ref.shape == (1, 1, model.config.vocab_size)
    err = rel_l2(out.cpu().numpy(), ref.cpu().numpy())
    print(f"  fused vs module logits rel-L2 = {err:.3e}", flush=True)
    # end to end the per-block differences between the two bf16 paths add up like a random walk over the 32 layers
    assert err <= 1e-2 * model.config.n_layer ** 0.5, err
    a = generate(model, prompt, 16, use_graph=True, greedy=True)
    b = generate(model, prompt, 16, use_graph=False, greedy=True)
    assert torch.equal(a, b)
