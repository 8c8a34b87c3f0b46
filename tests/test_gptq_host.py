"""Host logic of the calibrated int4 quantizer and of the tinygemm weight importer (no GPU).

GPTQ (reference torchao/quantization/GPTQ.py:300-398) has no vectors in the reference (its test needs lm_eval and a
checkpoint), so the solver is pinned by what the mathematics fixes: an identity Hessian reduces it to plain
round-to-nearest, its blocked Cholesky recurrence must agree with textbook column-by-column OBQ (explicit inverse of
the remaining Hessian, float64, oracle.obq_quantize), and on correlated inputs its layer output error must be below
round-to-nearest's.  The tinygemm layout importer is checked against a lane-by-lane transcription of the published
packer kernel only (parity unpinned: no vectors of that format exist in the reference)."""
import numpy as np
import pytest
import torch

import oracle
from ao_amd.quantization.GPTQ import _LockStepCalibration, gptq_quantize_weight
from ao_amd.quantization.utils import _MultiInput, unpack_tinygemm_int4pack


# a plain min/max asymmetric 4-bit quantizer in float64, shared by the solver under test and the textbook oracle
def _np_qparams(w):
    w = np.asarray(w, np.float64)
    mn, mx = w.min(axis=1, keepdims=True), w.max(axis=1, keepdims=True)
    scale = np.maximum((mx - mn) / 15.0, 1e-9)
    return scale, mn


def _np_quant(w, qp):
    scale, mn = qp
    g = w.shape[1] // scale.shape[1]
    s, m = np.repeat(scale, g, axis=1), np.repeat(mn, g, axis=1)
    return np.clip(np.rint((np.asarray(w, np.float64) - m) / s), 0, 15)


def _np_dequant(q, qp):
    scale, mn = qp
    g = q.shape[1] // scale.shape[1]
    return q * np.repeat(scale, g, axis=1) + np.repeat(mn, g, axis=1)


def _torch_callbacks():
    to_t = lambda qp: tuple(torch.from_numpy(a) for a in qp)
    to_n = lambda qp: tuple(a.numpy() for a in qp)
    return dict(
        get_qparams_func=lambda w: to_t(_np_qparams(w.double().numpy())),
        quantize_func=lambda w, qp: torch.from_numpy(_np_quant(w.double().numpy(), to_n(qp))),
        dequantize_func=lambda q, qp: torch.from_numpy(_np_dequant(q.double().numpy(), to_n(qp))),
        combine_qparams_list_func=lambda lst: [torch.cat(x, dim=1) for x in zip(*lst)],
    )


def _problem(N, K, n_tokens, seed):
    rng = np.random.default_rng(seed)
    mix = rng.standard_normal((K, K)) * 0.3 + np.eye(K)
    X = rng.standard_normal((n_tokens, K)) @ mix  # correlated inputs
    W = rng.standard_normal((N, K)) * 0.05
    H = 2.0 / n_tokens * X.T @ X
    return X, W, H


def test_identity_hessian_is_round_to_nearest():
    _, W, _ = _problem(12, 64, 8, 0)
    cb = _torch_callbacks()
    Q, DQ, qp = gptq_quantize_weight(torch.eye(64), torch.from_numpy(W).float(), blocksize=16, percdamp=0.01,
                                     groupsize=32, **cb)
    Wf = torch.from_numpy(W).float().double().numpy()
    expect = np.concatenate([_np_dequant(_np_quant(Wf[:, g:g + 32], _np_qparams(Wf[:, g:g + 32])),
                                         _np_qparams(Wf[:, g:g + 32])) for g in (0, 32)], axis=1)
    np.testing.assert_array_equal(DQ.double().numpy(), expect.astype(np.float32).astype(np.float64))
    assert qp[0].shape == (12, 2) and Q.shape == (12, 64)
    np.testing.assert_array_equal(_np_dequant(Q.numpy(), tuple(a.numpy() for a in qp)).astype(np.float32), DQ.numpy())


@pytest.mark.parametrize("blocksize", [8, 32])
def test_blocked_cholesky_recurrence_matches_textbook_obq(blocksize):
    # groups start at block starts (blocksize divides groupsize), where both formulations take the qparams from
    # fully compensated weights
    _, W, H = _problem(16, 64, 256, 1)
    W32 = torch.from_numpy(W).float()
    cb = _torch_callbacks()
    _, DQ, _ = gptq_quantize_weight(torch.from_numpy(H).float(), W32, blocksize=blocksize, percdamp=0.01, groupsize=32,
                                    **cb)
    ref = oracle.obq_quantize(H.astype(np.float32).astype(np.float64), W32.double().numpy(), 32, _np_qparams,
                              lambda col, qp: _np_dequant(_np_quant(col[:, None], qp), qp)[:, 0], percdamp=0.01)
    got = DQ.double().numpy()
    # fp32 Cholesky against float64 inverses: a code may flip where a compensated weight sits on a rounding boundary
    # (and shift what follows in its row); all but a few rows must agree to float32 rounding
    rows_equal = np.all(np.abs(got - ref) <= 1e-5, axis=1)
    assert rows_equal.mean() >= 0.8, rows_equal
    err = lambda D: np.trace((W32.double().numpy() - D) @ H @ (W32.double().numpy() - D).T)
    assert abs(err(got) - err(ref)) <= 0.02 * err(ref)


def test_gptq_lowers_the_layer_output_error():
    X, W, H = _problem(32, 128, 512, 2)
    cb = _torch_callbacks()
    W32 = torch.from_numpy(W).float()
    _, DQ, _ = gptq_quantize_weight(torch.from_numpy(H).float(), W32, blocksize=32, percdamp=0.01, groupsize=32, **cb)
    Wd = W32.double().numpy()
    rtn = np.concatenate([_np_dequant(_np_quant(Wd[:, g:g + 32], _np_qparams(Wd[:, g:g + 32])),
                                      _np_qparams(Wd[:, g:g + 32])) for g in range(0, 128, 32)], axis=1)
    out_err = lambda D: np.linalg.norm(X @ (Wd - D).T)
    assert out_err(DQ.double().numpy()) < 0.8 * out_err(rtn)


def test_dead_inputs_are_zeroed():
    _, W, H = _problem(8, 32, 64, 3)
    H[:, 5] = 0
    H[5, :] = 0
    cb = _torch_callbacks()
    _, DQ, _ = gptq_quantize_weight(torch.from_numpy(H).float(), torch.from_numpy(W).float(), blocksize=16,
                                    percdamp=0.01, groupsize=32, **cb)
    assert torch.isfinite(DQ).all()
    # the dead column is quantized from 0, not from its weight
    scale, mn = _np_qparams(np.where(np.arange(32) == 5, 0.0, torch.from_numpy(W).float().double().numpy()))
    assert np.all(np.abs(DQ[:, 5].double().numpy()) <= scale[:, 0] + 1e-9)


class _Chain(torch.nn.Module):
    """Three linears with a model-owned buffer that is written and read back between the first two (the way a KV cache
    is written and read inside an attention block, between two linears); samples of different lengths."""

    def __init__(self):
        super().__init__()
        self.a = torch.nn.Linear(8, 8, bias=False)
        self.b = torch.nn.Linear(8, 8, bias=False)
        self.c = torch.nn.Linear(8, 4, bias=False)
        self.register_buffer("scratch", torch.zeros(16, 8))

    def forward(self, x, shift):
        h = torch.tanh(self.a(x))
        self.scratch[: h.shape[0]] = h
        h = self.scratch[: h.shape[0]].clone()
        return self.c(torch.tanh(self.b(h) + shift) + h)


def test_lock_step_calibration_feeds_each_linear_from_quantized_predecessors():
    torch.manual_seed(0)
    model = _Chain()
    xs = [torch.randn(t, 8) for t in (3, 5, 2, 7)]
    shift = torch.tensor(0.25)
    originals = {n: getattr(model, n).weight.detach().clone() for n in "abc"}
    seen = []

    def on_linear(module, H):
        seen.append((module, H.clone()))
        module.weight.data.mul_(0.5)  # stands for "quantize": later linears must see this change

    watched = {m: n for n, m in model.named_modules() if isinstance(m, torch.nn.Linear)}
    _LockStepCalibration(model, watched, on_linear).run([_MultiInput(xs), _MultiInput([shift])])
    assert [watched[m] for m, _ in seen] == ["a", "b", "c"]

    def hessian(inputs):
        H, n = torch.zeros(8, 8), 0
        for x in inputs:
            H *= n / (n + 1)
            n += 1
            x = x * (2.0 / n) ** 0.5
            H += x.t() @ x
        return H

    ha = [torch.tanh(x @ (0.5 * originals["a"]).t()) for x in xs]
    hb = [torch.tanh(h @ (0.5 * originals["b"]).t() + shift) + h for h in ha]
    torch.testing.assert_close(seen[0][1], hessian(xs))
    torch.testing.assert_close(seen[1][1], hessian(ha))
    torch.testing.assert_close(seen[2][1], hessian(hb))  # also shows no sample read another sample's scratch rows
    assert not any(h for h in model.a._forward_pre_hooks.values())


def test_lock_step_calibration_surfaces_a_failing_sample():
    model = _Chain()
    xs = [torch.randn(3, 8), torch.randn(3, 9)]  # the second sample does not fit the first linear
    watched = {m: n for n, m in model.named_modules() if isinstance(m, torch.nn.Linear)}
    with pytest.raises(RuntimeError):
        _LockStepCalibration(model, watched, lambda m, H: None).run([_MultiInput(xs), _MultiInput([torch.tensor(0.0)])])
    assert not model.a._forward_pre_hooks


@pytest.mark.parametrize("inner_k_tiles", [2, 4, 8])
def test_tinygemm_unpack_inverts_the_packer_transcription(inner_k_tiles):
    rng = np.random.default_rng(inner_k_tiles)
    codes = rng.integers(0, 16, size=(24, 256), dtype=np.int32)
    packed = oracle.tinygemm_int4pack(codes, inner_k_tiles)
    assert packed.shape == (3, 256 // (16 * inner_k_tiles), 32, inner_k_tiles // 2)
    got = unpack_tinygemm_int4pack(torch.from_numpy(packed.view(np.int32)), inner_k_tiles)
    assert got.dtype is torch.int32
    np.testing.assert_array_equal(got.numpy(), codes)


def test_tinygemm_word_is_four_k_pairs_under_the_half_word_mask():
    # the property the layout exists for: (word >> 4i) & 0x000F000F holds codes (k, k+1) of the lane's i-th pair, the
    # pairs being k0, k0+8 of the first k tile and of the second (mma.m16n8k16 B fragment, lane t: row t//4, k0 = 2*(t%4))
    codes = (np.arange(64)[None, :] * 7 + np.arange(8)[:, None] * 3) % 16
    packed = oracle.tinygemm_int4pack(codes.astype(np.int32), 2)
    for t in (0, 5, 31):
        word = int(packed[0, 1, t, 0])
        row, k0 = t // 4, 32 + 2 * (t % 4)
        for i, off in enumerate((0, 8, 16, 24)):
            pair = (word >> (4 * i)) & 0x000F000F
            assert pair & 0xF == codes[row, k0 + off] and pair >> 16 == codes[row, k0 + off + 1]


def _rocm_fixture():
    import os
    return np.load(os.path.join(os.path.dirname(__file__), "golden", "tinygemm_rocm_int4pack.npz"))


@pytest.mark.parametrize("inner_k_tiles", [2, 4, 8])
def test_rocm_tinygemm_layout_matches_the_words_pytorch_rocm_wrote(inner_k_tiles):
    # golden/tinygemm_rocm_int4pack.npz holds what aten._convert_weight_to_int4pack of PyTorch-ROCm wrote on gfx950
    # (tests/golden/make_tinygemm_rocm.py); the oracle's lane-by-lane restatement and the library's unpacker must
    # both agree with it
    fx = _rocm_fixture()
    codes, words = fx["codes"], fx[f"packed_ikt{inner_k_tiles}"]
    np.testing.assert_array_equal(oracle.tinygemm_int4pack_rocm(codes, inner_k_tiles).view(np.int32), words)
    got = unpack_tinygemm_int4pack(torch.from_numpy(words), inner_k_tiles, packed_by="rocm")
    np.testing.assert_array_equal(got.numpy(), codes)
    # and the CUDA layout is a different one: the unpacker of one must not read the other
    assert not np.array_equal(unpack_tinygemm_int4pack(torch.from_numpy(words), inner_k_tiles).numpy(), codes)


def test_pytorch_int4_matmul_rounds_once_where_dequantize_rounds_twice():
    # The fixture's aten._weight_int4pack_mm output is reproduced bit for bit by w = bf16((q-8)*s + z) (one rounding)
    # with fp32 accumulation; the reference's dequantize (torchao/quantization/quant_primitives.py:265-274), which the
    # linear of this library follows, rounds the product first, and lands within a few 1e-3 of it.
    fx = _rocm_fixture()
    bf = lambda name: torch.from_numpy(fx[name]).view(torch.bfloat16).double().numpy()
    rb = lambda a: torch.from_numpy(np.asarray(a, np.float32)).bfloat16().double().numpy()
    s, z = np.repeat(bf("scales_bits").T, 64, 1), np.repeat(bf("zeros_bits").T, 64, 1)
    q, x, y = fx["codes"].astype(np.float64) - 8.0, bf("x_bits"), bf("mm_bits")
    once = rb(x @ rb(q * s + z).T)
    twice = x @ rb(rb(q * s) + z).T
    np.testing.assert_array_equal(once, y)
    rel = np.linalg.norm(twice - y) / np.linalg.norm(twice)
    assert 1e-4 < rel < 5e-3
