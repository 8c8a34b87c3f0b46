"""The decode-attention entry point that allocates nothing (its workspace is an array inside the library's device image)
against the entry point that takes a caller-owned workspace: same kernels, so the outputs and the cache rows written must
be identical bit for bit.  Two calls in a row share the built-in array, the second with a smaller problem (fewer heads,
fewer context shares, a shorter cache), so stale triples of the first call lie beside the ones the second call reads.
This module is named to be collected after every other test module."""
import ctypes

import pytest
import torch


def _problem(dev, n_head, n_kv, S, pos, seed):
    g = torch.Generator().manual_seed(seed)
    hd = 128
    qkv = torch.randn(1, (n_head + 2 * n_kv) * hd, generator=g).bfloat16().to(dev)
    ang = torch.rand(S, hd // 2, generator=g) * 6.283
    freqs = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).bfloat16().to(dev)
    k = torch.randn(1, n_kv, S, hd, generator=g).bfloat16().to(dev)
    v = torch.randn(1, n_kv, S, hd, generator=g).bfloat16().to(dev)
    p = torch.tensor([pos], dtype=torch.int32, device=dev)
    return qkv, freqs, k, v, p


@pytest.mark.gpu
def test_static_workspace_matches_caller_workspace_on_two_calls_in_a_row(cabi):
    dev = torch.device("cuda:0")
    L = cabi.lib()
    st = torch.cuda.current_stream().cuda_stream
    for n_head, n_kv, S, pos, nsplit in [(32, 8, 8192, 8000, 16), (8, 2, 2048, 777, 4), (128, 8, 1024, 1023, 16), (4, 4, 256, 0, 2)]:
        print(f"case static workspace n_head={n_head} n_kv={n_kv} S={S} pos={pos} nsplit={nsplit}", flush=True)
        qkv, freqs, k, v, p = _problem(dev, n_head, n_kv, S, pos, seed=n_head + S)
        k1, v1, k2, v2 = k.clone(), v.clone(), k.clone(), v.clone()
        ws = torch.full((n_head * nsplit * 130,), float("nan"), device=dev)
        out1 = torch.empty(1, n_head * 128, dtype=torch.bfloat16, device=dev)
        out2 = torch.empty_like(out1)
        cabi.check(L.ao_amd_llama_decode_attention_split(qkv.data_ptr(), None, 0, freqs.data_ptr(), p.data_ptr(), k1.data_ptr(),
                                                         v1.data_ptr(), n_head, n_kv, 128, S, nsplit, ws.data_ptr(),
                                                         out1.data_ptr(), st))
        cabi.check(L.ao_amd_llama_decode_attention_split_static(qkv.data_ptr(), None, 0, freqs.data_ptr(), p.data_ptr(),
                                                                k2.data_ptr(), v2.data_ptr(), n_head, n_kv, 128, S, nsplit,
                                                                out2.data_ptr(), st))
        torch.cuda.synchronize()
        finite = bool(torch.isfinite(out1.float()).all())
        same = bool(torch.equal(out1.view(torch.int16), out2.view(torch.int16)))
        same_cache = bool(torch.equal(k1, k2)) and bool(torch.equal(v1, v2))
        assert finite and same and same_cache, (n_head, S, pos, nsplit, finite, same, same_cache)


def test_static_workspace_rejects_more_than_its_capacity(cabi):
    """2048 (head, context share) pairs fit; the check comes before anything touches a device, so it runs without one"""
    L = cabi.lib()
    dummy = ctypes.c_void_p(256)
    rc = L.ao_amd_llama_decode_attention_split_static(dummy, None, 0, dummy, dummy, dummy, dummy, 256, 8, 128, 4096, 16, dummy, None)
    assert rc != 0
    msg = L.ao_amd_last_error().decode()
    assert "4096" in msg and "2048" in msg and "ao_amd_llama_decode_attention_split" in msg, msg
