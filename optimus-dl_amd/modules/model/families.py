"""Llama / Qwen3 / GPT-2 shaped models (``transformer.{wte,h,ln_f}`` + ``lm_head``
as in optimus_dl/modules/model/{llama2,qwen3,gpt2}.py), random-initialised with
the reference's standard deviations (gpt2.py:167-180: 0.02, and 0.02/sqrt(2*n_layer)
for the residual projections ``c_proj`` / ``wo``)."""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn as nn

from .blocks import GPT2Block, LlamaBlock, Qwen3Block, RMSNorm


@dataclass
class LlamaConfig:
    vocab_size: int = 32000
    n_layer: int = 2
    n_head: int = 8
    n_kv_head: int | None = None
    n_embd: int = 512
    intermediate_size: int | None = None
    block_size: int = 2048
    rmsnorm_eps: float = 1e-5
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False


@dataclass
class Qwen3Config(LlamaConfig):
    head_dim: int | None = None
    rmsnorm_eps: float = 1e-6
    rope_theta: float = 1e6
    tie_word_embeddings: bool = True


@dataclass
class GPT2Config:
    vocab_size: int = 50304
    n_layer: int = 2
    n_head: int = 12
    n_embd: int = 768
    block_size: int = 1024
    bias: bool = True
    tie_word_embeddings: bool = True


def _init_weights(model: nn.Module, n_layer: int) -> None:
    for m in model.modules():
        if isinstance(m, nn.Linear):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)
            if m.bias is not None:
                nn.init.zeros_(m.bias)
        elif isinstance(m, nn.Embedding):
            nn.init.normal_(m.weight, mean=0.0, std=0.02)
    for name, p in model.named_parameters():
        if name.endswith("c_proj.weight") or name.endswith("wo.weight"):
            nn.init.normal_(p, mean=0.0, std=0.02 / math.sqrt(2 * n_layer))


class _DecoderLM(nn.Module):
    def _finish(self, cfg) -> None:
        self.lm_head = nn.Linear(cfg.n_embd, cfg.vocab_size, bias=False)
        if cfg.tie_word_embeddings:
            self.transformer.wte.weight = self.lm_head.weight
        _init_weights(self, cfg.n_layer)

    def embed(self, input_ids: torch.Tensor) -> torch.Tensor:
        return self.transformer.wte(input_ids)

    def forward(self, input_ids: torch.Tensor, **kwargs) -> dict:
        x = self.embed(input_ids)
        for block in self.transformer.h:
            x = block(x)
        return {"logits": self.lm_head(self.transformer.ln_f(x))}


class Llama(_DecoderLM):
    def __init__(self, config: LlamaConfig):
        super().__init__()
        self.config = config
        self.transformer = nn.ModuleDict({
            "wte": nn.Embedding(config.vocab_size, config.n_embd),
            "h": nn.ModuleList([LlamaBlock(config.n_embd, config.n_head, config.n_kv_head, config.intermediate_size,
                                           eps=config.rmsnorm_eps, rope_theta=config.rope_theta)
                                for _ in range(config.n_layer)]),
            "ln_f": RMSNorm(config.n_embd, config.rmsnorm_eps),
        })
        self._finish(config)


class Qwen3(_DecoderLM):
    def __init__(self, config: Qwen3Config):
        super().__init__()
        self.config = config
        self.transformer = nn.ModuleDict({
            "wte": nn.Embedding(config.vocab_size, config.n_embd),
            "h": nn.ModuleList([Qwen3Block(config.n_embd, config.n_head, config.n_kv_head, config.intermediate_size,
                                           head_dim=config.head_dim, eps=config.rmsnorm_eps,
                                           rope_theta=config.rope_theta) for _ in range(config.n_layer)]),
            "ln_f": RMSNorm(config.n_embd, config.rmsnorm_eps),
        })
        self._finish(config)


class GPT2(_DecoderLM):
    def __init__(self, config: GPT2Config):
        super().__init__()
        self.config = config
        self.transformer = nn.ModuleDict({
            "wte": nn.Embedding(config.vocab_size, config.n_embd),
            "wpe": nn.Embedding(config.block_size, config.n_embd),
            "h": nn.ModuleList([GPT2Block(config.n_embd, config.n_head, config.bias) for _ in range(config.n_layer)]),
            "ln_f": nn.LayerNorm(config.n_embd, bias=config.bias),
        })
        self._finish(config)

    def embed(self, input_ids: torch.Tensor) -> torch.Tensor:
        pos = torch.arange(input_ids.shape[1], device=input_ids.device)
        return self.transformer.wte(input_ids) + self.transformer.wpe(pos)
