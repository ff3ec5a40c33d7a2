"""Small models and deterministic data for the glue tests."""
from __future__ import annotations

import torch

import gen


def cnn(seed: int = 0) -> torch.nn.Module:
    """The 2-conv + 2-FC CNN of the end-to-end step (1x28x28 inputs, 10 classes)."""
    torch.manual_seed(seed)
    return torch.nn.Sequential(
        torch.nn.Conv2d(1, 8, 3, padding=1), torch.nn.ReLU(), torch.nn.MaxPool2d(2),
        torch.nn.Conv2d(8, 16, 3, padding=1), torch.nn.ReLU(), torch.nn.MaxPool2d(2),
        torch.nn.Flatten(), torch.nn.Linear(16 * 7 * 7, 64), torch.nn.ReLU(), torch.nn.Linear(64, 10))


def images(seed: int, batch: int = 64) -> torch.Tensor:
    return (gen.uniform_pm1(seed, batch, 1, 28, 28) + 1) * 0.5  # uniform [0,1)


def train_steps(model, loss_fn, opt, x, y, steps: int):
    """A few optimisation steps; returns (final logits, losses)."""
    losses = []
    for _ in range(steps):
        opt.zero_grad()
        out = model(x)
        loss = loss_fn(out, y)
        loss.backward()
        opt.step()
        losses.append(loss.detach().cpu().clone())
    with torch.no_grad():
        logits = model(x)
    return logits, losses
