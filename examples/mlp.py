"""MNIST-shaped MLP 784 -> 64 -> 10 with ReLU: the graph of dlgrad's examples/mnist_mlp.py:12-45
and test/test_forward_backward.py:16-101."""
from __future__ import annotations

import math

import numpy as np

from dlgrad_amd import Tensor, nn


class MLP:
    def __init__(self, device: str = "hip", n_in: int = 784, n_hidden: int = 64, n_out: int = 10) -> None:
        self.device = device
        self.fc1 = nn.Linear(n_in, n_hidden, device=device)
        self.fc2 = nn.Linear(n_hidden, n_out, device=device)

    def __call__(self, x: Tensor) -> Tensor:
        return self.fc2(self.fc1(x).relu())


def init_weights_(model: MLP, seed: int) -> None:
    """Seeded Kaiming-uniform U(-1/sqrt(fan_in), 1/sqrt(fan_in)) (nn/__init__.py:10-12)."""
    rng = np.random.default_rng(seed)
    for layer in (model.fc1, model.fc2):
        bound = 1 / math.sqrt(layer.weight.shape[1])
        for p in (layer.weight, layer.bias):
            w = rng.uniform(-bound, bound, p.shape).astype(np.float32)
            p.data = Tensor(w, device=model.device).data


def synthetic_batch(seed: int, batch: int = 128, n_in: int = 784, n_out: int = 10):
    rng = np.random.default_rng(seed)
    return rng.random((batch, n_in), dtype=np.float32), rng.integers(0, n_out, (batch, 1)).astype(np.float32)
