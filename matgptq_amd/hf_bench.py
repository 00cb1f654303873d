"""Tokens/s of the reference's transformers caller with this library's linears.

Counterpart of inference_lib/bench_transformers_e2e.py: a `LlamaForCausalLM` whose block linears are
`MatGPTQLinear` modules, decoded one token at a time over a `StaticCache` by
`torch.compile(decode_one_tokens, fullgraph=True, dynamic=True, mode="reduce-overhead")` and timed
like `time_prof` (:61-76: warm-ups, then the mean over runs of back-to-back calls with one
synchronisation per run).  Nothing is fetched: the model is built from a local `LlamaConfig`
(Llama-3-8B's shape by default) on the meta device, embeddings, norms and head get random values
on the GPU, and every linear gets seeded random master codes and scales, sliced to a per-layer
bitwidth drawn from `bit_choices`.

    python -m matgptq_amd.hf_bench [--layers 32] [--context 512] [--no_compile]
"""
from __future__ import annotations

import argparse
import json
import random
import time
from typing import Sequence

import torch

LINEARS = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
           "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")


def decode_one_tokens(model, cur_token, input_pos, cache_position, past_key_values):
    logits = model(cur_token, position_ids=input_pos, cache_position=cache_position,
                   past_key_values=past_key_values, return_dict=False, use_cache=True)[0]
    return torch.argmax(logits[:, -1], dim=-1)[:, None]


def time_prof(func, sync, benchmark_runs=8, number_of_runs=16, warmups=16):
    """Mean seconds per call of each run (bench_transformers_e2e.py:61-76)."""
    for _ in range(warmups):
        func()
    sync()
    times = []
    for _ in range(benchmark_runs):
        t1 = time.time()
        for _ in range(number_of_runs):
            func()
        sync()
        times.append((time.time() - t1) / number_of_runs)
    return times


def build_model(layers: int = 32, hidden: int = 4096, ffn: int = 14336, heads: int = 32, kv_heads: int = 8,
                vocab: int = 128256, bit_choices: Sequence[int] = (2, 3, 4, 6, 8), seed: int = 0,
                group_size: int = 128, dtype=torch.float16, device: str = "cuda"):
    """Random-weight Llama-shaped transformers model with every block linear a `MatGPTQLinear`."""
    from transformers import LlamaConfig, LlamaForCausalLM

    from matgptq_cuda.matgptq_linear import MatGPTQLinear

    from .ops import matryoshka_slice

    cfg = LlamaConfig(hidden_size=hidden, intermediate_size=ffn, num_hidden_layers=layers, num_attention_heads=heads,
                      num_key_value_heads=kv_heads, vocab_size=vocab, max_position_embeddings=8192, rms_norm_eps=1e-5,
                      rope_theta=500000.0, tie_word_embeddings=False, attention_bias=False, mlp_bias=False)
    with torch.device("meta"):
        model = LlamaForCausalLM(cfg)
    shapes = {name: tuple(model.get_submodule(f"model.layers.0.{name}").weight.shape) for name in LINEARS}
    # the block linears never get dense weights: they are replaced while still on the meta device
    gen = torch.Generator(device=device).manual_seed(seed)
    rnd = random.Random(seed)
    bits_of, weight_bytes, weights = {}, 0, 0
    for li in range(layers):
        for name in LINEARS:
            n, k = shapes[name]
            b = rnd.choice(tuple(bit_choices))
            master = torch.randint(0, 256, (n, k), dtype=torch.uint8, device=device, generator=gen)
            # weights of the size a trained layer has: |w| up to 128 * scale, about 1 / sqrt(k) overall
            scale = ((torch.randn(n, k // group_size, device=device, generator=gen).abs() * 0.01 + 1e-3)
                     * (1.0 / (k ** 0.5))).to(dtype)
            layer = MatGPTQLinear(matryoshka_slice(master, 8, b), scale, b, group_size)
            full = f"model.layers.{li}.{name}"
            parent, attr = full.rsplit(".", 1)
            setattr(model.get_submodule(parent), attr, layer)
            bits_of[full] = b
            weight_bytes += n * k * b // 8
            weights += n * k
            del master
    # what is still on the meta device (embeddings, norms, head) gets random values on the GPU; the
    # rotary embedding's buffers are rebuilt by a fresh module
    model.model.rotary_emb = type(model.model.rotary_emb)(cfg).to(device)
    for module in model.modules():
        for pname, p in list(module._parameters.items()):
            if p is None or not p.is_meta:
                continue
            if p.dim() == 1:
                value = torch.ones(p.shape, dtype=dtype, device=device)
            else:
                value = (torch.randn(p.shape, device=device, generator=gen) * 0.02).to(dtype)
            module._parameters[pname] = torch.nn.Parameter(value, requires_grad=False)
    assert not any(t.is_meta for t in list(model.parameters()) + list(model.buffers()))
    model.eval()
    return model, bits_of, weight_bytes, weights


def measure(layers: int = 32, context: int = 512, compile_forward: bool = True, seed: int = 0,
            bit_choices: Sequence[int] = (2, 3, 4, 6, 8), **shape) -> dict:
    from transformers import StaticCache

    t0 = time.perf_counter()
    model, bits_of, weight_bytes, weights = build_model(layers=layers, bit_choices=bit_choices, seed=seed, **shape)
    build_s = time.perf_counter() - t0
    dev = "cuda"
    vocab = model.config.vocab_size
    ids = torch.randint(0, vocab, (1, context), device=dev, generator=torch.Generator(device=dev).manual_seed(seed))
    runs, per_run, warm = 8, 16, 16
    budget = (runs * per_run + warm) * 2 + 8
    cache = StaticCache(config=model.config, max_batch_size=1, max_cache_len=context + budget, device=dev,
                        dtype=torch.float16)
    out = {"layers": layers, "context": context, "linears": len(bits_of),
           "mean_bits": round(weight_bytes * 8 / weights, 2), "build_s": round(build_s, 1)}
    with torch.no_grad():
        cache_position = torch.arange(context, dtype=torch.int64, device=dev)
        logits = model(ids, cache_position=cache_position, past_key_values=cache, return_dict=False, use_cache=True)[0]
        next_token = torch.argmax(logits[:, [-1]], dim=-1)
        torch._dynamo.config.capture_scalar_outputs = True
        variants = [("eager", decode_one_tokens)]
        if compile_forward:
            variants.append(("compiled", torch.compile(decode_one_tokens, fullgraph=True, dynamic=True,
                                                       mode="reduce-overhead")))
        cache_position = torch.tensor([context], device=dev)
        for tag, fn in variants:
            def one():
                nonlocal next_token
                next_token = fn(model, next_token.clone(), None, cache_position, cache)
                cache_position.add_(1)
            t0 = time.perf_counter()
            try:
                times = time_prof(one, torch.cuda.synchronize, runs, per_run, warm)
            except Exception as e:  # an absent inductor toolchain must not take the other figures along
                out[f"{tag}_error"] = f"{type(e).__name__}: {str(e)[:160]}"
                continue
            mean = sum(times) / len(times)
            out[f"tokens_per_s_{tag}"] = round(1.0 / mean, 1)
            out[f"ms_per_token_{tag}"] = round(mean * 1e3, 3)
            out[f"{tag}_wall_s_with_warmup"] = round(time.perf_counter() - t0, 1)
            out[f"sliced_weight_GBps_{tag}"] = round(weight_bytes / mean / 1e9, 1)
    return out


def main() -> None:
    ap = argparse.ArgumentParser(description="tokens/s of a random-weight Llama-3-8B-shaped transformers model "
                                             "whose linears are MatGPTQLinear modules")
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--context", type=int, default=512)
    ap.add_argument("--no_compile", action="store_true")
    ap.add_argument("--bits", type=int, nargs="+", default=[2, 3, 4, 6, 8])
    args = ap.parse_args()
    print(json.dumps(measure(args.layers, args.context, not args.no_compile, bit_choices=args.bits)))


if __name__ == "__main__":
    main()
