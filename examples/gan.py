"""The two MNIST-shaped MLPs of dlgrad's examples/mnist_gan.py:29-58 and its two training steps (:70-96): a
generator 128 -> 256 -> 512 -> 1024 -> 784 (leaky ReLU 0.2, tanh) and a discriminator 784 -> 1024 -> 512 -> 256 -> 1
(leaky ReLU 0.2, logits), trained against each other with the logits form of the binary cross-entropy and Adam
(lr 5e-4, betas (0.5, 0.999)).  Only what the graph needs: no image grid, no progress bar, no data download."""
from __future__ import annotations

import math

import numpy as np

from dlgrad_amd import Tensor, nn


class LinearGen:
    def __init__(self, device: str = "hip") -> None:
        self.net = [nn.Linear(128, 256, device=device), lambda t: t.leaky_relu(0.2),
                    nn.Linear(256, 512, device=device), lambda t: t.leaky_relu(0.2),
                    nn.Linear(512, 1024, device=device), lambda t: t.leaky_relu(0.2),
                    nn.Linear(1024, 784, device=device), Tensor.tanh]

    def __call__(self, x: Tensor) -> Tensor:              # (BS, 128) -> (BS, 784)
        return x.sequential(self.net)


class LinearDisc:
    def __init__(self, device: str = "hip") -> None:
        self.net = [nn.Linear(784, 1024, device=device), lambda t: t.leaky_relu(0.2),
                    nn.Linear(1024, 512, device=device), lambda t: t.leaky_relu(0.2),
                    nn.Linear(512, 256, device=device), lambda t: t.leaky_relu(0.2),
                    nn.Linear(256, 1, device=device)]

    def __call__(self, x: Tensor) -> Tensor:              # (BS, 784) -> (BS, 1) logits
        return x.sequential(self.net)


def init_weights_(model, seed: int, device: str) -> None:
    """Seeded U(-1/sqrt(fan_in), 1/sqrt(fan_in)) for every Linear of the model (nn/__init__.py:10-12)."""
    rng = np.random.default_rng(seed)
    for layer in model.net:
        if isinstance(layer, nn.Linear):
            bound = 1 / math.sqrt(layer.weight.shape[1])
            for p in (layer.weight, layer.bias):
                p.data = Tensor(rng.uniform(-bound, bound, p.shape).astype(np.float32), device=device).data


def make_targets(bs: int, value: float, device: str) -> Tensor:
    return Tensor.full((bs, 1), value, device=device)


def train_discriminator(discriminator, optimizer, data_real: Tensor, data_fake: Tensor) -> Tensor:
    """mnist_gan.py:70-84: real -> 1, fake -> 0, the mean of the two losses."""
    bs, device = data_real.shape[0], data_real.device
    optimizer.zero_grad()
    loss_real = discriminator(data_real).bcewithlogitsloss(make_targets(bs, 1.0, device))
    loss_fake = discriminator(data_fake).bcewithlogitsloss(make_targets(bs, 0.0, device))
    d_loss = (loss_real + loss_fake) / 2.0
    d_loss.backward()
    optimizer.step()
    return d_loss


def train_generator(discriminator, optimizer, data_fake: Tensor) -> Tensor:
    """mnist_gan.py:86-96: the non-saturating form, D(G(z)) pushed towards "real"."""
    optimizer.zero_grad()
    g_loss = discriminator(data_fake).bcewithlogitsloss(make_targets(data_fake.shape[0], 1.0, data_fake.device))
    g_loss.backward()
    optimizer.step()
    return g_loss
