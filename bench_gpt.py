#!/usr/bin/env python3
"""End-to-end GPT training step with Fastmax causal attention in every layer (the caller side of
the attention path: reference model.py:464-603 calls fastmax_custom on contiguous (B,H,T,hs)
q, k, v with RoPE applied and transposes the result back).

    python bench_gpt.py [--steps K] [--warmup W] [--p 2] [--layers 12] [--batch 8] [--seq 2048]

A step = forward + loss + backward + AdamW update, bf16 autocast, random-init weights (std 0.02,
as reference model.py:267-274), token ids uniform over the vocabulary from a seed.  Prints one JSON
line with tokens/s and the share of the step spent in attention forward + backward (HIP events
around the attention module and around its backward, summed over layers).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import torch  # noqa: E402
import torch.nn as nn  # noqa: E402
import torch.nn.functional as F  # noqa: E402


def rope_cache(seq: int, hs: int, device, base: float = 10000.0):
    theta = 1.0 / (base ** (torch.arange(0, hs, 2, device=device).float() / hs))
    idx = torch.outer(torch.arange(seq, device=device).float(), theta).repeat(1, 2)
    return torch.cos(idx), torch.sin(idx)


def apply_rope(x, cos, sin):
    hs = x.size(-1)
    x1, x2 = x[..., : hs // 2], x[..., hs // 2:]
    rotated = torch.cat((-x2, x1), dim=-1)
    return (x * cos + rotated * sin).to(x.dtype)


class Block(nn.Module):
    def __init__(self, d_model, n_head, d_mlp, attn, p, layout):
        super().__init__()
        self.n_head, self.hs, self.p, self.layout = n_head, d_model // n_head, p, layout
        self.ln1 = nn.LayerNorm(d_model)
        self.qkv = nn.Linear(d_model, 3 * d_model)
        self.proj = nn.Linear(d_model, d_model)
        self.ln2 = nn.LayerNorm(d_model)
        self.fc = nn.Linear(d_model, d_mlp)
        self.out = nn.Linear(d_mlp, d_model)
        self.attn = attn

    def forward(self, x, cos, sin):
        B, T, C = x.shape
        qkv = self.qkv(self.ln1(x))
        if self.layout == "packed":
            # no layout copies at all: RoPE in place in the projection (packed per head as [q, k, v], the
            # reference's group-major layout with one query per group, model.py:474-497), q, k, v read as
            # strided views of it, the output written token-major, and in backward dq, dk, dv written
            # straight into the projection's gradient
            y = self.attn(qkv, cos, sin, self.n_head, 1, self.hs, self.hs, True, True, 1.0, 1.0, 1.0, 0.5, 1.0, self.p)
            x = x + self.proj(y)
            return x + self.out(F.gelu(self.fc(self.ln2(x))))
        if self.layout == "split":
            # one HBM pass: split of the projection (packed per head as [q, k, v], the reference's
            # group-major layout with one query per group, model.py:474-497), RoPE on q and k,
            # contiguous (B, H, T, hs) outputs
            from fastmax_amd import qkv_rope_split
            q, k, v = qkv_rope_split(qkv, cos, sin, self.n_head, 1, self.hs)
        else:
            q, k, v = qkv.view(B, T, self.n_head, 3, self.hs).permute(3, 0, 2, 1, 4)
            q, k = apply_rope(q, cos, sin).contiguous(), apply_rope(k, cos, sin).contiguous()
            v = v.contiguous()
        # same call as reference model.py:575: mask, no dropout, normalize, lim 1, a = (1, 1, 0.5)
        y = self.attn(q, k, v, None, True, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, self.p)
        x = x + self.proj(y.transpose(1, 2).reshape(B, T, C))
        return x + self.out(F.gelu(self.fc(self.ln2(x))))


class MiniGPT(nn.Module):
    def __init__(self, vocab, d_model, n_layer, n_head, d_mlp, seq, attn, p, layout):
        super().__init__()
        self.wte = nn.Embedding(vocab, d_model)
        self.blocks = nn.ModuleList(Block(d_model, n_head, d_mlp, attn, p, layout) for _ in range(n_layer))
        self.ln_f = nn.LayerNorm(d_model)
        self.lm_head = nn.Linear(d_model, vocab, bias=False)
        self.seq, self.hs = seq, d_model // n_head
        self.apply(self._init)

    @staticmethod
    def _init(m):
        if isinstance(m, (nn.Linear, nn.Embedding)):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)
            if isinstance(m, nn.Linear) and m.bias is not None:
                nn.init.zeros_(m.bias)

    def forward(self, idx):
        cos, sin = rope_cache(idx.size(1), self.hs, idx.device)
        x = self.wte(idx)
        for b in self.blocks:
            x = b(x, cos, sin)
        return self.lm_head(self.ln_f(x))


class PackedAttention(nn.Module):
    """The attention of a block on its packed projection (layout "packed")."""

    def forward(self, *args):
        from fastmax_amd import qkv_attention
        return qkv_attention(*args)


class TimedAttention(nn.Module):
    """Wraps the attention module with HIP events around its forward and its backward."""

    def __init__(self, inner):
        super().__init__()
        self.inner = inner
        self.events = []
        self.register_full_backward_pre_hook(self._bwd_start)
        self.register_full_backward_hook(self._bwd_end)

    def _mark(self):
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        return e

    def _bwd_start(self, module, grad_output):
        self._b0 = self._mark()

    def _bwd_end(self, module, grad_input, grad_output):
        self.events.append((self._b0, self._mark()))

    def forward(self, *args):
        e0 = self._mark()
        y = self.inner(*args)
        self.events.append((e0, self._mark()))
        return y

    def total_ms(self):
        torch.cuda.synchronize()
        t = sum(a.elapsed_time(b) for a, b in self.events)
        self.events.clear()
        return t


def run(steps: int = 5, warmup: int = 2, p: int = 2, layers: int = 12, batch: int = 8, seq: int = 2048,
        pytorch_attention: bool = False, split_rope: bool = False, unfused_rope: bool = False) -> dict:
    """Times the training step and returns the result record (main() prints it as one JSON line)."""
    from fastmax_amd import FASTMultiHeadAttention

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    layout = "pytorch" if unfused_rope else ("split" if (split_rope or pytorch_attention) else "packed")
    if layout == "packed":
        attn = TimedAttention(PackedAttention())
    else:
        attn = TimedAttention(FASTMultiHeadAttention(use_custom_gradient=not pytorch_attention))
    model = MiniGPT(50304, 768, layers, 12, 3072, seq, attn, p, layout).to(dev)
    opt = torch.optim.AdamW(model.parameters(), lr=3e-4, weight_decay=0.1)
    gen = torch.Generator(device=dev).manual_seed(0)
    idx = torch.randint(0, 50304, (batch, seq + 1), device=dev, generator=gen)
    x, y = idx[:, :-1].contiguous(), idx[:, 1:].contiguous()

    def step():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits = model(x)
        loss = F.cross_entropy(logits.float().view(-1, logits.size(-1)), y.view(-1))
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()
        return loss.detach()

    losses = []
    for _ in range(warmup):
        losses.append(float(step()))
    attn.total_ms()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        losses.append(float(step()))
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    attn_ms = attn.total_ms() / steps
    return {
        "metric": "GPT training step with Fastmax causal attention in every layer",
        "value": batch * seq / (ms * 1e-3), "unit": "tokens/s", "ms_per_step": ms,
        "attention_fwd_bwd_ms_per_step": attn_ms, "attention_share_of_step": attn_ms / ms,
        "dtype": "bf16 autocast (attention: bf16 in/out, bf16 matrix instructions, fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"{layers} layers, d_model 768, 12 heads x 64, MLP 3072 GELU, RoPE, vocab 50304, "
                               f"seq {seq}, batch {batch}, p={p}, AdamW",
                   "attention": "pytorch function" if pytorch_attention else "hip kernels",
                   "qkv split + rope": {"pytorch": "pytorch ops", "split": "fused hip kernel, contiguous q/k/v",
                                        "packed": "rotated q, k to a packed tensor, attention on strided views of it and of the projection, "
                                                  "token-major output (includes the rope pass in the attention time)"}[layout]},
        "loss_first_last": [losses[0], losses[-1]], "steps": steps, "warmup": warmup,
        "finite": all(math.isfinite(v) for v in losses),
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--p", type=int, default=2, help="polynomial order (the reference model hard-codes 1)")
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--seq", type=int, default=2048)
    ap.add_argument("--pytorch-attention", action="store_true", help="use_custom_gradient=False path")
    ap.add_argument("--split-rope", action="store_true",
                    help="split the projection into contiguous (B, H, T, hs) q, k, v with RoPE in one fused kernel and "
                         "transpose the attention output back (two extra passes over q, k, v, o per direction) "
                         "instead of running the attention on strided views of the packed projection")
    ap.add_argument("--unfused-rope", action="store_true",
                    help="split the projection, apply RoPE and make q, k, v contiguous with PyTorch ops "
                         "(the reference's chain, model.py:474-497, 812-825, 572-574) instead of the fused kernel")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("bench_gpt.py: no GPU visible", file=sys.stderr)
        return 3
    res = run(args.steps, args.warmup, args.p, args.layers, args.batch, args.seq, args.pytorch_attention,
              args.split_rope, args.unfused_rope)
    print(json.dumps(res))
    return 0 if res["finite"] else 1


if __name__ == "__main__":
    sys.exit(main())
