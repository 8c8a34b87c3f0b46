"""Batch-1 text generation loop and its metrics.

Follows torchao/_models/llama/generate.py: prefill (:53-56), decode_one_token (:58-62), decode_n_tokens
(:64-77), generate (:84-120) and the metric definition tokens/s = generated / wall time,
bandwidth = model_size * tokens/s with embeddings ignored (:220, :292-300).  Where the reference wraps
decode_one_token in torch.compile(mode="reduce-overhead") to get CUDA graphs (:225), this module
captures the decode step in a HIP graph directly (GraphedDecoder).
"""
import argparse
import time
from typing import Optional

import torch

from ...quantization import fp6_llm_weight_only, int4_weight_only, int8_weight_only, quantize
from ...utils import get_model_size_in_bytes
from .model import Transformer, prepare_inputs_for_model

__all__ = ["sample", "prefill", "decode_one_token", "decode_n_tokens", "generate", "GraphedDecoder",
           "random_init_", "build_random_model"]


def multinomial_sample_one_no_sync(probs_sort):
    q = torch.empty_like(probs_sort).exponential_(1)
    return torch.argmax(probs_sort / q, dim=-1, keepdim=True).to(dtype=torch.int)


def logits_to_probs(logits, temperature: float = 1.0, top_k: Optional[int] = None):
    logits = logits / max(temperature, 1e-5)
    if top_k is not None:
        v, _ = torch.topk(logits, min(top_k, logits.size(-1)))
        logits = torch.where(logits < v.select(-1, -1).unsqueeze(-1), -float("Inf"), logits)
    return torch.nn.functional.softmax(logits, dim=-1)


def sample(logits, temperature: float = 1.0, top_k: Optional[int] = None, greedy: bool = False):
    """Next token from the last position's logits.  greedy=True is argmax (no random numbers)."""
    if greedy:
        last = logits[0, -1]
        if last.is_cuda and last.dtype in (torch.bfloat16, torch.float16) and last.is_contiguous():
            from ... import ops

            return ops.argmax_bf16(last), None
        return torch.argmax(last, dim=-1, keepdim=True).to(dtype=torch.int), None
    probs = logits_to_probs(logits[0, -1], temperature, top_k)
    return multinomial_sample_one_no_sync(probs), probs


def prefill(model: Transformer, x: torch.Tensor, input_pos: torch.Tensor, **sampling_kwargs) -> torch.Tensor:
    return sample(model(x, input_pos), **sampling_kwargs)[0]


def decode_one_token(model: Transformer, x: torch.Tensor, input_pos: torch.Tensor, **sampling_kwargs):
    assert input_pos.shape[-1] == 1
    return sample(model(x, input_pos), **sampling_kwargs)


class GraphedDecoder:
    """decode_one_token captured once in a HIP graph and replayed per token.

    The graph owns static buffers for the current token and position; a replay reads them, writes the
    next token and advances the position in place, so a decode loop is nothing but replays.  Eager
    warm-up steps run on a side stream first, as graph capture requires."""

    def __init__(self, model: Transformer, device, **sampling_kwargs):
        self.model = model
        self.sampling_kwargs = sampling_kwargs
        self.token = torch.zeros(1, 1, dtype=torch.int, device=device)
        self.pos = torch.zeros(1, dtype=torch.int, device=device)
        self.next_token = torch.zeros(1, dtype=torch.int, device=device)
        self.graph = None
        # host mirror of the device-side position: a replay advances `pos` on the device, where the host cannot see it,
        # so the bound of the KV cache is enforced here (the attention kernel only degrades to NaN outputs past it)
        self.host_pos = 0

    def _step(self):
        if self.sampling_kwargs.get("greedy") and self.token.is_cuda:
            last = self.model(self.token, self.pos)[0, -1]
            if last.dtype in (torch.bfloat16, torch.float16) and last.is_contiguous():
                from ... import ops

                # argmax, next input token and position in one launch
                ops.decode_advance_(last, self.next_token, self.token, self.pos)
                return
            nxt = torch.argmax(last, dim=-1, keepdim=True).to(dtype=torch.int)
        else:
            nxt, _ = decode_one_token(self.model, self.token, self.pos, **self.sampling_kwargs)
        self.next_token.copy_(nxt.view(-1))
        self.token.copy_(nxt.view(1, 1))
        self.pos.add_(1)

    def capture(self, token: torch.Tensor, pos: int, warmup: int = 2):
        """Capture at position `pos`.  The warm-up and capture steps write KV-cache slots pos..pos+warmup,
        which later real steps overwrite; the static buffers are reset afterwards."""
        if pos >= self.model.max_seq_length:
            raise IndexError(f"capture at position {pos} is past the KV cache ({self.model.max_seq_length} positions)")
        warmup = max(0, min(warmup, self.model.max_seq_length - 1 - pos))  # warm-up steps stay inside the cache too
        self.token.copy_(token.view(1, 1))
        self.pos.fill_(pos)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(warmup):
                self._step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.token.copy_(token.view(1, 1))
        self.pos.fill_(pos)
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self._step()
        self.token.copy_(token.view(1, 1))
        self.pos.fill_(pos)
        self.host_pos = pos

    def step(self) -> torch.Tensor:
        """One decoded token (device tensor, valid until the next step)."""
        if self.host_pos >= self.model.max_seq_length:
            raise IndexError(f"decode step at position {self.host_pos} is past the KV cache "
                             f"({self.model.max_seq_length} positions); call setup_caches with a longer max_seq_length")
        self.graph.replay()
        self.host_pos += 1
        return self.next_token


def decode_n_tokens(model, cur_token, input_pos, num_new_tokens, callback=lambda _: _, graphed=None,
                    **sampling_kwargs):
    new_tokens, new_probs = [], []
    if graphed is not None:
        for _ in range(num_new_tokens):
            new_tokens.append(graphed.step().clone())
            callback(new_tokens[-1])
        return new_tokens, new_probs
    for _ in range(num_new_tokens):
        next_token, next_prob = decode_one_token(model, cur_token, input_pos, **sampling_kwargs)
        input_pos += 1
        new_tokens.append(next_token.clone())
        callback(new_tokens[-1])
        if next_prob is not None:
            new_probs.append(next_prob.clone())
        cur_token = next_token.view(1, -1)
    return new_tokens, new_probs


@torch.no_grad()
def generate(model: Transformer, prompt: torch.Tensor, max_new_tokens: int, *, interactive: bool = False,
             callback=lambda x: x, use_graph: bool = False, **sampling_kwargs) -> torch.Tensor:
    """prompt [T] int -> [T + max_new_tokens] int: one prefill pass, then token-by-token decode."""
    device = prompt.device
    T = prompt.numel()
    T_new = T + max_new_tokens
    seq = torch.empty(T_new, dtype=prompt.dtype, device=device)
    seq[:T] = prompt.view(-1)
    max_seq_length = min(T_new, model.config.block_size) if not interactive else 350
    if T_new > max_seq_length:
        raise ValueError(f"prompt ({T}) + max_new_tokens ({max_new_tokens}) = {T_new} positions do not fit the "
                         f"{max_seq_length}-position KV cache" + (" of interactive mode" if interactive else " (block_size)"))
    model.setup_caches(max_batch_size=1, max_seq_length=max_seq_length)
    x, input_pos = prepare_inputs_for_model(prompt, max_new_tokens)
    next_token = prefill(model, x, input_pos, **sampling_kwargs).clone()
    seq[T] = next_token
    graphed = None
    if use_graph and max_new_tokens > 1:
        graphed = GraphedDecoder(model, device, **sampling_kwargs)
        graphed.capture(next_token, T)
    input_pos = torch.tensor([T], device=device, dtype=torch.int)
    generated, _ = decode_n_tokens(model, next_token.view(1, -1), input_pos, max_new_tokens - 1, callback=callback,
                                   graphed=graphed, **sampling_kwargs)
    if generated:
        seq[T + 1:] = torch.cat(generated)
    return seq


def random_init_(model: torch.nn.Module, std: float = 0.02, seed: int = 1234) -> None:
    """All matrices ~N(0, std) from a seed (norm weights stay 1): the synthetic stand-in for a checkpoint."""
    gen = torch.Generator(device=next(model.parameters()).device).manual_seed(seed)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() >= 2:
                p.normal_(0.0, std, generator=gen)


def build_random_model(name: str, device, quantization: Optional[str] = None, seed: int = 1234) -> Transformer:
    """Random-init bf16 model on `device`, optionally quantized ("int4wo-<group>" or "int8wo", the names of the
    reference's generate.py:199-215; "fp6": FP6-LLM e3m2 weights on an fp16 model, the flow of
    torchao/prototype/quant_llm/README.md:9-20)."""
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(device):
            model = Transformer.from_name(name)
    finally:
        torch.set_default_dtype(prev)
    random_init_(model, seed=seed)
    model.eval()
    if quantization == "int8wo":
        quantize(model, int8_weight_only())
    elif quantization == "fp6":
        model = model.half()
        quantize(model, fp6_llm_weight_only())
    elif quantization:
        assert quantization.startswith("int4wo-"), f"unsupported quantization {quantization}"
        group = int(quantization.split("-")[-1])
        assert group in (32, 64, 128, 256), f"int4wo groupsize needs to be one of [32,64,128,256] but got {group}"
        quantize(model, int4_weight_only(group_size=group))
    return model


def main():
    ap = argparse.ArgumentParser(description="random-init Llama decode benchmark (tokens/s, model_size * tokens/s)")
    ap.add_argument("--model", default="Llama-3-8B")
    ap.add_argument("--quantization", default="int4wo-64")
    ap.add_argument("--prompt_len", type=int, default=128)
    ap.add_argument("--max_new_tokens", type=int, default=256)
    ap.add_argument("--num_samples", type=int, default=3)
    ap.add_argument("--no_graph", action="store_true")
    args = ap.parse_args()
    device = torch.device("cuda")
    model = build_random_model(args.model, device, args.quantization)
    model_size = get_model_size_in_bytes(model, ignore_embeddings=True) / 1e9
    g = torch.Generator(device=device).manual_seed(0)
    prompt = torch.randint(0, model.config.vocab_size, (args.prompt_len,), device=device, dtype=torch.int, generator=g)
    rates = []
    for i in range(args.num_samples):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        y = generate(model, prompt, args.max_new_tokens, use_graph=not args.no_graph, greedy=True)
        torch.cuda.synchronize()
        t = time.perf_counter() - t0
        rate = (y.numel() - args.prompt_len) / t
        rates.append(rate)
        print(f"Time for inference {i + 1}: {t:.02f} sec total, {rate:.02f} tokens/sec")
        print(f"Bandwidth achieved: {model_size * rate:.02f} GB/s")
    mean = sum(rates) / len(rates)
    print(f"Average tokens/sec: {mean:.2f}")
    print(f"Average Bandwidth: {model_size * mean:.02f} GB/s")
    print(f"Peak Memory Usage: {torch.cuda.max_memory_reserved() / 1e9:.02f} GB")
    print(f"Model Size: {model_size:.02f} GB")


if __name__ == "__main__":
    main()
