"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.

Law: matrices ~ N(0, 0.02), norm weights ~ 1 + N(0, 0.02), biases ~ N(0, 0.02), drawn
in float32 from one seeded generator in the order of the configuration's tensor plan,
then stored in ``dtype``.  (The reference's ``Weights::random`` draws
``U(-1,1)/sqrt(d)`` and no biases, ``crates/mach-model/src/weights.rs:230-245,
336-374``; biases are drawn here so that the q/k/v bias path is exercised.)
"""
from __future__ import annotations

import json
import os
from typing import Dict, Iterator, Tuple

import torch

from ..config import config_from_dict
from .safetensors_io import write_safetensors

STD = 0.02


def _draw(shape, law: str, gen: torch.Generator, device) -> torch.Tensor:
    """One tensor of a law.  Beside the three above: 'filter' ~ N(0, 0.3) (a short convolution, a narrow projection
    inside a recurrence); 'mixing' = identity + N(0, 0.1) (a square matrix that mixes heads); 'blend' ~ U(0.3, 0.7) (a
    weight between two tensors); 'a_log' = ln(1 .. n) along the last axis (the decays of a scan); 'step_bias': the
    inverse softplus of step sizes drawn log-uniformly from 0.001 to 0.1."""
    if law in ("matrix", "bias", "norm"):
        t = torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * STD
        return t + 1.0 if law == "norm" else t
    if law == "filter":
        return torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * 0.3
    if law == "mixing":
        return torch.eye(shape[0], shape[1], device=device) + torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * 0.1
    if law == "blend":
        return 0.3 + 0.4 * torch.rand(shape, generator=gen, dtype=torch.float32, device=device)
    if law == "a_log":
        return torch.log(torch.arange(1, shape[-1] + 1, dtype=torch.float32, device=device)).expand(shape).clone()
    if law == "step_bias":
        import math
        u = torch.rand(shape, generator=gen, dtype=torch.float32, device=device)
        dt = torch.exp(u * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
        return dt + torch.log(-torch.expm1(-dt))
    raise ValueError(f"unknown law {law!r}")


def random_tensors(config, seed: int, dtype: torch.dtype = torch.float32,
                   device: str = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    for name, shape, law in config.random_tensor_plan():
        yield name, _draw(shape, law, gen, device).to(dtype)


def random_tensor_dict(config, seed: int, dtype=torch.float32, device="cpu") -> Dict[str, torch.Tensor]:
    return dict(random_tensors(config, seed, dtype, device))


def write_random_model(config, seed: int, out_dir: str, dtype: torch.dtype = torch.float32) -> str:
    """``config`` is a typed configuration or a config.json dict.  Returns ``out_dir``."""
    if isinstance(config, dict):
        config = config_from_dict(config)
    os.makedirs(out_dir, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = {torch.float32: "float32", torch.bfloat16: "bfloat16", torch.float16: "float16"}[dtype]
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=1)
    it = random_tensors(config, seed, dtype)
    plan = [(n, s, dtype) for n, s, _ in config.random_tensor_plan()]

    def produce(name):
        got, t = next(it)
        assert got == name
        return t

    write_safetensors(os.path.join(out_dir, "model.safetensors"), plan, produce)
    return out_dir
