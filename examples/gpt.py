"""Char-level GPT: the model graph of dlgrad's examples/gpt.py:33-129 on this package's Tensor.

RMSNorm (not LayerNorm), ReLU MLP, no biases, no dropout, untied lm_head, learned
positional embedding -- what that file builds, not what its config comment suggests.
Differences that do not change values: the causal mask (seven small kernels,
examples/gpt.py:52-53) is built once per (T, device) instead of once per block per step,
and every parameter is created on the model's device.
"""
from __future__ import annotations

import numpy as np

from dlgrad_amd import Tensor, nn


class GPTConfig:
    def __init__(self, vocab_size: int = 65, block_size: int = 128, n_layer: int = 6, n_head: int = 4,
                 n_embd: int = 128, batch_size: int = 16, learning_rate: float = 1e-4, device: str = "hip") -> None:
        self.vocab_size, self.block_size, self.n_layer = vocab_size, block_size, n_layer
        self.n_head, self.n_embd, self.batch_size = n_head, n_embd, batch_size
        self.learning_rate, self.device = learning_rate, device


_mask_cache: dict = {}


def causal_mask(T: int, device) -> Tensor:
    """1.0 where attention is NOT allowed: tril(ones) == 0 (examples/gpt.py:52-53)."""
    key = (T, str(device))
    if key not in _mask_cache:
        _mask_cache[key] = Tensor.tril(Tensor.ones((T, T), device=device), k=0.0) == Tensor(0.0)
    return _mask_cache[key]


class CausalSelfAttention:
    def __init__(self, c: GPTConfig) -> None:
        assert c.n_embd % c.n_head == 0
        self.n_head, self.head_dim = c.n_head, c.n_embd // c.n_head
        self.scale = self.head_dim ** -0.5
        self.q_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)
        self.k_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)
        self.v_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)
        self.c_proj = nn.Linear(c.n_embd, c.n_embd, bias=False, device=c.device)

    def __call__(self, x: Tensor) -> Tensor:
        B, T, C = x.shape
        split = (B, T, self.n_head, self.head_dim)
        q = self.q_proj(x).reshape(split).transpose(1, 2)            # (B, h, T, d)
        k = self.k_proj(x).reshape(split).transpose(1, 2)
        v = self.v_proj(x).reshape(split).transpose(1, 2)
        att = (q @ k.transpose(2, 3)) * self.scale                   # (B, h, T, T)
        att = att.masked_fill(causal_mask(T, x.device), float("-inf"))
        att = att.softmax(dim=3)
        y = (att @ v).transpose(1, 2).reshape((B, T, C))
        return self.c_proj(y)


class MLP:
    def __init__(self, c: GPTConfig) -> None:
        self.c_fc = nn.Linear(c.n_embd, 4 * c.n_embd, bias=False, device=c.device)
        self.c_proj = nn.Linear(4 * c.n_embd, c.n_embd, bias=False, device=c.device)

    def __call__(self, x: Tensor) -> Tensor:
        return self.c_proj(self.c_fc(x).relu())


class Block:
    def __init__(self, c: GPTConfig) -> None:
        self.ln1 = nn.RMSNorm(c.n_embd, device=c.device)
        self.attn = CausalSelfAttention(c)
        self.ln2 = nn.RMSNorm(c.n_embd, device=c.device)
        self.mlp = MLP(c)

    def __call__(self, x: Tensor) -> Tensor:
        x = x + self.attn(self.ln1(x))
        return x + self.mlp(self.ln2(x))


class GPT:
    def __init__(self, c: GPTConfig) -> None:
        self.config = c
        self.wte = nn.Embedding(c.vocab_size, c.n_embd, device=c.device)
        self.wpe = nn.Embedding(c.block_size, c.n_embd, device=c.device)
        self.blocks = [Block(c) for _ in range(c.n_layer)]
        self.ln_f = nn.RMSNorm(c.n_embd, device=c.device)
        self.lm_head = nn.Linear(c.n_embd, c.vocab_size, bias=False, device=c.device)

    def __call__(self, idx: Tensor, targets: Tensor | None = None):
        """idx, targets: (B, T) token ids stored as fp32.  Returns (logits, loss)."""
        B, T = idx.shape
        pos = Tensor.arange((T,), device=idx.device)            # 0..T-1 made on the device (no upload per step)
        x = self.wte(idx) + self.wpe(pos)
        for block in self.blocks:
            x = block(x)
        logits = self.lm_head(self.ln_f(x))
        if targets is None:
            return logits, None
        V = self.config.vocab_size
        loss = logits.reshape((B * T, V)).cross_entropy_loss(targets.reshape((B * T, 1)))
        return logits, loss

    def generate_greedy(self, first_token: int, max_new_tokens: int) -> list[int]:
        """Greedy decode with full-context recompute per token, context cropped to
        block_size (the loop of examples/gpt.py:231-279 with argmax in place of sampling)."""
        c = self.config
        ids = [int(first_token)]
        for _ in range(max_new_tokens):
            ctx = ids[-c.block_size:]
            T = len(ctx)
            logits, _ = self(Tensor(np.asarray(ctx, dtype=np.float32).reshape(1, T), device=c.device))
            last = logits.reshape((T, c.vocab_size))[T - 1:T]                       # (1, V) view
            ids.append(int(last.argmax(1).numpy()[0, 0]))
        return ids


def init_weights_(model: GPT, seed: int, std: float = 0.02) -> None:
    """Overwrites every parameter with seeded numpy values: N(0, std) for matrices and
    embeddings, ones for the RMSNorm gains -- the same values on any device."""
    rng = np.random.default_rng(seed)
    dev = model.config.device
    for name, p in nn.utils.get_state_dict(model).items():
        if ".ln" in f".{name}" and name.endswith("weight"):
            w = np.ones(p.shape, dtype=np.float32)
        else:
            w = (rng.standard_normal(p.shape) * std).astype(np.float32)
        p.data = Tensor(w, device=dev).data
