"""Callers of the bit-sliced linear: a Llama-shaped decoder whose linears are `MatGPTQLinear`
modules at per-layer bitwidths (Mix'n'Match), with a static key/value cache and a decode step
that can be captured into a HIP graph.

Counterpart of the reference's transformers path:
  replace_with_matgptq_linear   inference_lib/inference_demo_transformers.py:17-56 (same name and
                                arguments; works on any `torch.nn.Module` tree, so also on a
                                transformers model)
  DecodeSession.generate        inference_lib/inference_demo_transformers.py:134-176
  DecodeSession.tokens_per_s    inference_lib/bench_transformers_e2e.py:61-76,160-166

The reference wraps the step in `torch.compile(mode="reduce-overhead")` to get a device graph;
here the step is written with device-side position and token tensors and captured directly
(`torch.cuda.CUDAGraph` is a HIP graph on ROCm).  The linears are the product.  The operators
between them are plain torch operators for a prompt, and four small fused HIP kernels
(`_glue`: residual add + RMS norm, rotary embedding + cache write, attention over the cache,
SiLU gate) for decode steps of up to 16 rows in fp16, where some twenty separate torch kernels
per block took twice the time of the linears; the head is a dense torch linear.

    python -m matgptq_amd.decoder [--layers 32] [--context 512] [--new_tokens 64] [--bits 2 3 4 6 8]
"""
from __future__ import annotations

import argparse
import json
import os
import random
import time
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Union

import torch

from .checkpoint import load_quantised_layer, read_layer_bitwidths
from .ops import matryoshka_slice


def replace_with_matgptq_linear(model: torch.nn.Module, quantized_weights_path: Union[str, os.PathLike],
                                quantized_config_path: Optional[str] = None, master_bitwidth: int = 8,
                                slice_bitwidth: int = 8, group_size: int = 128) -> torch.nn.Module:
    """Replaces submodules of `model` by `MatGPTQLinear` modules built from the quantiser's
    per-layer directories `<quantized_weights_path>/<dotted.layer.name>/data.pt`.

    With `quantized_config_path` (lines `layer_name: bitwidth`, as written by the reference's
    search, evo_quant_search.py:660-672) exactly the listed layers are replaced, each at its own
    bitwidth; without it every layer directory is replaced at `slice_bitwidth`.  A stored
    `zero` tensor is used when present (the reference drops it and assumes 128), and a stored
    act-order `perm` is applied to the module's input features (the reference's kernel path
    ignores it; its fake-quantised path applies it, src/model_utils.py:185-195).
    """
    from matgptq_cuda.matgptq_linear import MatGPTQLinear

    def _replace(layer_name: str, bitwidth: int) -> None:
        data = load_quantised_layer(os.path.join(quantized_weights_path, layer_name))
        codes = matryoshka_slice(data["qweight"].cuda(), master_bitwidth, bitwidth)
        zero, perm = data.get("zero"), data.get("perm")
        layer = MatGPTQLinear(codes, data["scale"].cuda(), bitwidth, group_size,
                              zeros=zero.cuda() if zero is not None else None,
                              perm=perm.cuda() if perm is not None else None)
        *parent_path, attr = layer_name.split(".")
        parent = model.get_submodule(".".join(parent_path)) if parent_path else model
        setattr(parent, attr, layer)

    if quantized_config_path:
        for layer_name, bitwidth in read_layer_bitwidths(quantized_config_path).items():
            _replace(layer_name, bitwidth)
    else:
        for layer_name in sorted(os.listdir(quantized_weights_path)):
            if os.path.isdir(os.path.join(quantized_weights_path, layer_name)):
                _replace(layer_name, slice_bitwidth)
    return model


@dataclass
class DecoderConfig:
    """Shape of the decoder; the defaults are Llama-3-8B's."""
    hidden: int = 4096
    ffn: int = 14336
    layers: int = 32
    heads: int = 32
    kv_heads: int = 8
    vocab: int = 128256
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    group_size: int = 128

    @property
    def head_dim(self) -> int:
        return self.hidden // self.heads

    def linear_shapes(self) -> Dict[str, tuple]:
        """`name -> (N, K)` of the four linears of a block (q, k, v fused; gate, up fused)."""
        return {"qkv": ((self.heads + 2 * self.kv_heads) * self.head_dim, self.hidden),
                "o": (self.hidden, self.hidden),
                "gate_up": (2 * self.ffn, self.hidden),
                "down": (self.hidden, self.ffn)}


class Block(torch.nn.Module):
    """One decoder block.  The linears may be any module mapping `[M, K] -> [M, N]`."""

    def __init__(self, cfg: DecoderConfig, linears: Dict[str, torch.nn.Module], dtype, device):
        super().__init__()
        self.cfg = cfg
        self.qkv, self.o = linears["qkv"], linears["o"]
        self.gate_up, self.down = linears["gate_up"], linears["down"]
        self.fuse_prologues = True  # decode steps of up to four rows: norms and SiLU gate inside the linears
        self.input_norm = torch.nn.Parameter(torch.ones(cfg.hidden, dtype=dtype, device=device), requires_grad=False)
        self.post_norm = torch.nn.Parameter(torch.ones(cfg.hidden, dtype=dtype, device=device), requires_grad=False)

    def forward(self, h, cos, sin, pos, k_cache, v_cache, bias):
        """h [M, hidden]; cos/sin [M, head_dim]; pos int64 [M] (cache rows written);
        k_cache/v_cache [kv_heads, ctx, head_dim]; bias [rep * M, ctx] (0 = attend, -inf = not),
        rows ordered like the queries of one key/value head: query head major, batch row minor."""
        cfg = self.cfg
        m, d, rep = h.shape[0], cfg.head_dim, cfg.heads // cfg.kv_heads
        x = torch.nn.functional.rms_norm(h, (cfg.hidden,), self.input_norm, cfg.rms_eps)
        qkv = self.qkv(x).view(m, cfg.heads + 2 * cfg.kv_heads, d)
        qk = _rotate(qkv[:, :cfg.heads + cfg.kv_heads], cos, sin)  # queries and keys in one pass
        k_cache.index_copy_(1, pos, qk[:, cfg.heads:].transpose(0, 1))
        v_cache.index_copy_(1, pos, qkv[:, cfg.heads + cfg.kv_heads:].transpose(0, 1))
        # grouped-query attention: the `rep` query heads of a key/value head share one batched
        # product; the mask enters as the additive term of that product
        qg = qk[:, :cfg.heads].transpose(0, 1).reshape(cfg.kv_heads, rep * m, d)
        scores = torch.baddbmm(bias, qg, k_cache.transpose(1, 2), alpha=d ** -0.5)  # [kv, rep*m, ctx]
        probs = torch.softmax(scores, dim=-1)  # (accumulates in fp32 internally)
        attn = torch.bmm(probs, v_cache).view(cfg.heads, m, d).transpose(0, 1).reshape(m, cfg.hidden)
        h = h + self.o(attn)
        x = torch.nn.functional.rms_norm(h, (cfg.hidden,), self.post_norm, cfg.rms_eps)
        gu = self.gate_up(x)
        h = h + self.down(torch.nn.functional.silu(gu[:, :cfg.ffn]) * gu[:, cfg.ffn:])
        return h

    def forward_fused(self, h, delta, x, cos_table, sin_table, pos, k_cache, v_cache, attn_workspace):
        """The same block for a few rows with the operators between the linears fused: `h` [M, hidden]
        is updated in place with `delta` (the previous block's last linear output, or None) and this
        block's attention output; returns the output of `down`, which the next block (or the final
        norm) adds.  `x` [M, hidden] is scratch, `attn_workspace` the workspace of the split attention
        or None for the unsplit one.  Five launches for a single row (six with the split attention),
        eight or nine where the linears cannot take their prologues in the kernel."""
        from . import _glue
        from .ops import PRE_ADD_RMSNORM, PRE_SILU_MUL

        cfg = self.cfg
        m = h.shape[0]
        # Up to four rows the two norms and the SiLU gate ride in the linears behind them (five launches
        # per block instead of eight): the residual stream goes h -> x (= h + delta) in the qkv launch
        # and x -> h (= x + attention output) in the gate_up launch, so it is back in `h` at the end.
        in_kernel = self.prologues_apply(m)
        if in_kernel:
            qkv = self.qkv.forward_prologue(PRE_ADD_RMSNORM, h, delta, self.input_norm, x, cfg.rms_eps)
        else:
            _glue.add_rmsnorm(h, delta, self.input_norm, x, cfg.rms_eps)
            qkv = self.qkv(x)
        attn = torch.empty(m, cfg.hidden, dtype=h.dtype, device=h.device)
        # For a single row the rotary embedding and the cache write ride in the attention launch.
        # A long cache is split over workgroups (two launches; measured on MI355X with 32 / 8 heads,
        # one row: 10.9 against 12.6 us at 1024 rows, 28.9 against 60 us at 8192, 9.7 against 9.4 at 512).
        if m > 1:
            _glue.rope_cache(qkv, cos_table, sin_table, pos, k_cache, v_cache, cfg.heads, cfg.kv_heads)
        if attn_workspace is not None:
            _glue.attention_split(qkv, cos_table, sin_table, pos, k_cache, v_cache, attn, attn_workspace,
                                  cfg.heads, cfg.kv_heads, fuse_rotary=m == 1)
        elif m == 1:
            _glue.rope_attention(qkv, cos_table, sin_table, pos, k_cache, v_cache, attn, cfg.heads, cfg.kv_heads)
        else:
            _glue.attention(qkv, k_cache, v_cache, pos, attn, cfg.heads, cfg.kv_heads)
        if in_kernel:
            gate_up = self.gate_up.forward_prologue(PRE_ADD_RMSNORM, x, self.o(attn), self.post_norm, h, cfg.rms_eps)
            return self.down.forward_prologue(PRE_SILU_MUL, gate_up)
        _glue.add_rmsnorm(h, self.o(attn), self.post_norm, x, cfg.rms_eps)
        act = torch.empty(m, cfg.ffn, dtype=h.dtype, device=h.device)
        _glue.silu_mul(self.gate_up(x), act)
        return self.down(act)

    def prologues_apply(self, rows: int) -> bool:
        """Whether this block's qkv, gate_up and down linears take their prologues in the kernel."""
        from .ops import PRE_ADD_RMSNORM, PRE_SILU_MUL, prologue_applies

        if not self.fuse_prologues:
            return False
        cfg, dtype = self.cfg, self.input_norm.dtype
        def plain(lin):  # a pre-sliced layer without act-order permutation, as a module or behind the plugin
            params = getattr(lin, "layer", lin)
            return (hasattr(lin, "forward_prologue") and getattr(params, "matgptq_perm", None) is None
                    and getattr(params, "matgptq_planes", None) is None)

        return (all(plain(lin) for lin in (self.qkv, self.gate_up, self.down))
                and prologue_applies(PRE_ADD_RMSNORM, rows, cfg.hidden, cfg.group_size, dtype)
                and prologue_applies(PRE_SILU_MUL, rows, cfg.ffn, cfg.group_size, dtype))


def _rotate(t, cos, sin):
    """Rotary embedding, half-split convention: t [M, heads, d], cos/sin [M, d]."""
    half = t.shape[-1] // 2
    rot = torch.cat((-t[..., half:], t[..., :half]), dim=-1)
    return t * cos[:, None, :] + rot * sin[:, None, :]


class Decoder(torch.nn.Module):
    def __init__(self, cfg: DecoderConfig, blocks: Sequence[Block], embed: torch.Tensor, head: torch.Tensor,
                 max_context: int):
        super().__init__()
        self.cfg = cfg
        self.blocks = torch.nn.ModuleList(blocks)
        self.embed = torch.nn.Parameter(embed, requires_grad=False)     # [vocab, hidden]
        self.head = torch.nn.Parameter(head, requires_grad=False)       # [vocab, hidden], dense like the reference's lm_head
        self.final_norm = torch.nn.Parameter(torch.ones(cfg.hidden, dtype=embed.dtype, device=embed.device),
                                             requires_grad=False)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.float32) / cfg.head_dim))
        ang = torch.outer(torch.arange(max_context, dtype=torch.float32), inv)
        ang = torch.cat((ang, ang), dim=-1)
        self.register_buffer("cos", ang.cos().to(embed.dtype).to(embed.device), persistent=False)
        self.register_buffer("sin", ang.sin().to(embed.dtype).to(embed.device), persistent=False)
        self.register_buffer("arange", torch.arange(max_context, device=embed.device), persistent=False)
        self.max_context = max_context
        self.fused = True  # decode steps of a few rows use the fused operators between the linears
        # long caches: context split over workgroups (1, 2, 4 or 8 query heads per key/value head)
        self.split_attention = max_context > 768 and cfg.heads // cfg.kv_heads in (1, 2, 4, 8)
        self._attn_workspace = None

    def new_cache(self):
        cfg = self.cfg
        shape = (len(self.blocks), 2, cfg.kv_heads, self.max_context, cfg.head_dim)
        return torch.zeros(shape, dtype=self.embed.dtype, device=self.embed.device)

    def fused_applies(self, rows: int) -> bool:
        """The fused operators cover a few fp16 rows at head dimension 128 on a cache they can hold."""
        from . import _glue

        return (self.fused and rows <= 16 and self.embed.dtype == torch.float16 and self.cfg.head_dim == 128
                and self.max_context <= _glue.MAX_CONTEXT and self.cfg.hidden <= 8192)

    @torch.no_grad()
    def forward(self, tokens, pos, cache):
        """tokens int64 [M], pos int64 [M] (their positions) -> logits [M, vocab] (fp32)."""
        h = self.embed.index_select(0, tokens)
        if self.fused_applies(h.shape[0]):
            from . import _glue

            if self.split_attention and self._attn_workspace is None:
                # shared by all blocks: their launches follow one another
                self._attn_workspace = _glue.attention_workspace(16, self.cfg.heads, self.max_context, h.device)
            x = torch.empty_like(h)
            delta = None
            for i, block in enumerate(self.blocks):
                delta = block.forward_fused(h, delta, x, self.cos, self.sin, pos, cache[i, 0], cache[i, 1],
                                            self._attn_workspace if self.split_attention else None)
            _glue.add_rmsnorm(h, delta, self.final_norm, x, self.cfg.rms_eps)
            return torch.nn.functional.linear(x[-1:], self.head).float()
        cos, sin = self.cos.index_select(0, pos), self.sin.index_select(0, pos)
        rep = self.cfg.heads // self.cfg.kv_heads
        bias = torch.where(self.arange[None, :] <= pos[:, None], 0.0, float("-inf")).to(h.dtype).repeat(rep, 1)
        for i, block in enumerate(self.blocks):
            h = block(h, cos, sin, pos, cache[i, 0], cache[i, 1], bias)
        h = torch.nn.functional.rms_norm(h, (self.cfg.hidden,), self.final_norm, self.cfg.rms_eps)
        return torch.nn.functional.linear(h[-1:], self.head).float()


class PluginLinear(torch.nn.Module):
    """A linear driven the way vLLM drives a quantisation method (inference_lib/vllm_matgptq.py:
    89-201): `create_weights`, the loader's copies into `qweight` / `scales`, then
    `process_weights_after_loading`; `forward` is `apply`."""

    def __init__(self, quant_config, prefix: str, codes: torch.Tensor, scale: torch.Tensor,
                 zero: Optional[torch.Tensor]):
        super().__init__()
        import vllm_matgptq

        n, k = codes.shape
        self.layer = torch.nn.Module()
        self.method = vllm_matgptq.MatGPTQLinearMethod(quant_config, quant_config.bitwidth_for(prefix))
        self.method.create_weights(self.layer, k, [n], k, n, scale.dtype)
        self.layer.to(codes.device)
        self.layer.qweight.data.copy_(codes)
        self.layer.scales.data.copy_(scale)
        if zero is not None:
            self.layer.zeros = torch.nn.Parameter(zero.clone(), requires_grad=False)
        self.method.process_weights_after_loading(self.layer)
        self.bitwidth = self.method.bitwidth

    def forward(self, x):
        return self.method.apply(self.layer, x)

    def forward_prologue(self, kind, a, added=None, norm_weight=None, residual_out=None, eps=1e-5):
        return self.method.apply_prologue(self.layer, kind, a, added, norm_weight, residual_out, eps)


def random_mixnmatch_decoder(cfg: DecoderConfig, max_context: int, bit_choices: Sequence[int] = (2, 3, 4, 6, 8),
                             seed: int = 0, dtype=torch.float16, device="cuda", zero_points: bool = True,
                             keep_master: bool = False, via_plugin: bool = False):
    """A decoder with random master codes; every linear gets a bitwidth drawn from `bit_choices`
    (seeded).  Returns `(decoder, layer_bits, masters)`: `layer_bits` maps `blocks.<i>.<name>` to
    its bitwidth and `masters` (only with `keep_master`) to `(codes uint8 [N,K], scale, zero)`.
    With `via_plugin` the linears are built by the vLLM quantisation method, configured by a
    `layer_bitwidths` map as a packed checkpoint would, instead of as `MatGPTQLinear` modules.
    """
    from matgptq_cuda.matgptq_linear import MatGPTQLinear

    rnd = random.Random(seed)
    names = [f"blocks.{i}.{name}" for i in range(cfg.layers) for name in cfg.linear_shapes()]
    drawn = {name: rnd.choice(list(bit_choices)) for name in names}
    quant_config = None
    if via_plugin:
        import vllm_matgptq

        quant_config = vllm_matgptq.MatGPTQConfig.from_config({
            "group_size": cfg.group_size, "master_bitwidth": 8, "inference_bitwidth": 4,
            "quant_dtype": str(dtype).replace("torch.", ""), "modules_to_not_convert": ["head"],
            "layer_bitwidths": drawn})
    gen = torch.Generator(device=device).manual_seed(seed)
    layer_bits: Dict[str, int] = {}
    masters = {}
    blocks: List[Block] = []
    for i in range(cfg.layers):
        linears = {}
        for name, (n, k) in cfg.linear_shapes().items():
            bits = drawn[f"blocks.{i}.{name}"]
            codes = torch.randint(0, 256, (n, k), dtype=torch.uint8, device=device, generator=gen)
            groups = k // cfg.group_size
            # scale chosen so that a linear roughly preserves the norm of its input
            scale = ((torch.rand(n, groups, device=device, generator=gen) + 0.5) / (74.0 * k ** 0.5)).to(dtype)
            zero = torch.randint(112, 144, (n, groups), device=device, generator=gen).to(dtype) if zero_points else None
            if via_plugin:
                linears[name] = PluginLinear(quant_config, f"blocks.{i}.{name}", codes, scale, zero)
                assert linears[name].bitwidth == bits
            else:
                linears[name] = MatGPTQLinear(matryoshka_slice(codes, 8, bits), scale, bits, cfg.group_size, zeros=zero)
            layer_bits[f"blocks.{i}.{name}"] = bits
            if keep_master:
                masters[f"blocks.{i}.{name}"] = (codes, scale, zero)
        blocks.append(Block(cfg, linears, dtype, device))
    embed = (torch.randn(cfg.vocab, cfg.hidden, device=device, generator=gen)).to(dtype)
    head = (torch.randn(cfg.vocab, cfg.hidden, device=device, generator=gen) * cfg.hidden ** -0.5).to(dtype)
    return Decoder(cfg, blocks, embed, head, max_context), layer_bits, masters


class DecodeSession:
    """Greedy decoding with a static cache.  `prefill` runs the prompt in one pass (the M>16
    kernels), `step` decodes one token eagerly, `capture` records `step` into a graph whose
    replays read and advance device-side token and position tensors."""

    def __init__(self, decoder: Decoder):
        self.decoder = decoder
        dev = decoder.embed.device
        self.cache = decoder.new_cache()
        self.token = torch.zeros(1, dtype=torch.int64, device=dev)
        self.pos = torch.zeros(1, dtype=torch.int64, device=dev)
        self.logits = torch.zeros(1, decoder.cfg.vocab, dtype=torch.float32, device=dev)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.stream = torch.cuda.Stream(device=dev)

    def prefill(self, prompt: torch.Tensor) -> None:
        n = prompt.numel()
        if n + 1 > self.decoder.max_context:
            raise ValueError("prompt longer than the cache")
        pos = torch.arange(n, device=prompt.device)
        logits = self.decoder(prompt.to(torch.int64), pos, self.cache)
        self.logits.copy_(logits)
        self.token.copy_(logits.argmax(dim=-1))
        self.pos.fill_(n)

    def _step_body(self) -> None:
        from . import _glue

        logits = self.decoder(self.token, self.pos, self.cache)
        self.logits.copy_(logits)
        _glue.argmax(self.logits, self.token)  # (torch's own takes 38 us on 128256 logits, in one workgroup)
        self.pos.add_(1)

    def step(self) -> None:
        """One token, eagerly.  The caller keeps `pos` below the cache length."""
        self._step_body()

    def capture(self) -> None:
        """Records one step.  Token, position and cache are restored afterwards, so the capture
        (and its eager warm-up) does not advance the sequence."""
        saved = (self.token.clone(), self.pos.clone(), self.logits.clone())
        row = self.cache[:, :, :, int(self.pos.item())].clone()
        torch.cuda.synchronize()
        with torch.cuda.stream(self.stream):
            self._step_body()  # warm-up on the capture stream: library workspaces exist before capture
            self.stream.synchronize()
            self.token.copy_(saved[0]); self.pos.copy_(saved[1])
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=self.stream):
                self._step_body()
            self.stream.synchronize()
        self.token.copy_(saved[0]); self.pos.copy_(saved[1]); self.logits.copy_(saved[2])
        self.cache[:, :, :, int(saved[1].item())] = row
        torch.cuda.synchronize()
        self.graph = graph

    def replay(self) -> None:
        self.graph.replay()

    def generate(self, prompt: torch.Tensor, new_tokens: int, use_graph: bool = True) -> torch.Tensor:
        """Greedy continuation of `prompt`: returns the `new_tokens` generated ids."""
        if prompt.numel() + new_tokens > self.decoder.max_context:
            raise ValueError("prompt + new_tokens exceed the cache")
        self.prefill(prompt)
        if use_graph and self.graph is None:
            self.capture()
        out = [self.token.clone()]
        for _ in range(new_tokens - 1):
            self.replay() if use_graph else self.step()
            out.append(self.token.clone())
        torch.cuda.synchronize()
        return torch.cat(out)

    def tokens_per_s(self, steps: int, use_graph: bool, repeats: int = 3) -> float:
        """Best of `repeats` timings of `steps` consecutive tokens from the current position,
        which is restored after each timing: every repeat sees the same context and the
        session is left where it was."""
        if int(self.pos.item()) + steps > self.decoder.max_context:
            raise ValueError("not enough cache left for the timed steps")
        if use_graph and self.graph is None:
            self.capture()
        run = self.replay if use_graph else self.step
        saved = (self.token.clone(), self.pos.clone())
        best = float("inf")
        for _ in range(repeats):
            self.token.copy_(saved[0]); self.pos.copy_(saved[1])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                run()
            torch.cuda.synchronize()
            best = min(best, time.perf_counter() - t0)
        self.token.copy_(saved[0]); self.pos.copy_(saved[1])
        return steps / best


def measure(layers: int = 32, context: int = 512, new_tokens: int = 64, bit_choices: Sequence[int] = (2, 3, 4, 6, 8),
            seed: int = 0, dtype=torch.float16, via_plugin: bool = True) -> dict:
    """Builds the random-weight decoder, prefills `context` tokens, and times decoding."""
    cfg = DecoderConfig(layers=layers)
    decoder, layer_bits, _ = random_mixnmatch_decoder(cfg, context + new_tokens + 8, bit_choices, seed, dtype,
                                                      via_plugin=via_plugin)
    session = DecodeSession(decoder)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    prompt = torch.randint(0, cfg.vocab, (context,), device="cuda", generator=gen)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    session.prefill(prompt)
    torch.cuda.synchronize()
    first = time.perf_counter() - t0
    t0 = time.perf_counter()
    session.prefill(prompt)
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    eager = session.tokens_per_s(new_tokens, use_graph=False)
    graph = session.tokens_per_s(new_tokens, use_graph=True)
    shapes = cfg.linear_shapes()
    weight_bytes = sum(shapes[name.rsplit(".", 1)[1]][0] * shapes[name.rsplit(".", 1)[1]][1] * b // 8
                       for name, b in layer_bits.items())
    hist: Dict[str, int] = {}
    for b in layer_bits.values():
        hist[str(b)] = hist.get(str(b), 0) + 1
    return {"layers": layers, "context": context, "new_tokens": new_tokens, "dtype": str(dtype).replace("torch.", ""),
            "linears": "vllm_matgptq.MatGPTQLinearMethod" if via_plugin else "MatGPTQLinear",
            "bitwidth_histogram": dict(sorted(hist.items())),
            "mean_bits": round(weight_bytes * 8 / sum(shapes[n.rsplit(".", 1)[1]][0] * shapes[n.rsplit(".", 1)[1]][1]
                                                      for n in layer_bits), 2),
            "prefill_ms": round(prefill_s * 1e3, 2), "first_prefill_ms": round(first * 1e3, 2),
            "tokens_per_s_eager": round(eager, 1), "tokens_per_s_graph": round(graph, 1),
            "ms_per_token_graph": round(1e3 / graph, 3),
            "sliced_weight_GBps_graph": round(weight_bytes * graph / 1e9, 1)}


def main() -> None:
    ap = argparse.ArgumentParser(description="tokens/s of a random-weight Llama-3-8B-shaped Mix'n'Match decoder")
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--context", type=int, default=512)
    ap.add_argument("--new_tokens", type=int, default=64)
    ap.add_argument("--bits", type=int, nargs="+", default=[2, 3, 4, 6, 8])
    ap.add_argument("--bf16", action="store_true")
    ap.add_argument("--modules", action="store_true", help="build the linears as MatGPTQLinear modules "
                    "instead of through the vLLM quantisation method")
    args = ap.parse_args()
    print(json.dumps(measure(args.layers, args.context, args.new_tokens, args.bits,
                             dtype=torch.bfloat16 if args.bf16 else torch.float16, via_plugin=not args.modules)))


if __name__ == "__main__":
    main()
