"""Seeded random weights, and writing a model folder from a configuration."""
from __future__ import annotations

import hashlib
import json
import os

import torch

from ..parts.base import WeightSpec
from .safetensors_io import save_file

MATRIX_STD = 0.02
NORM_STD = 0.1
VECTOR_STD = 0.5
#: laws whose tensors are kept as drawn (float32, or int32 for a table of indices) whatever the matrices are stored in
FLOAT32_INITS = ("norm", "norm_offset", "vector", "unit_interval", "decay_log", "depth_coef", "index_table")


def tensor_seed(seed: int, name: str) -> int:
    """A seed per tensor, so values do not depend on the order of creation."""
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(spec: WeightSpec, seed: int, name: str, device="cpu") -> torch.Tensor:
    """float32 values: matrices and embeddings N(0, 0.02), norm weights
    1 + N(0, 0.1) (``norm_offset``: stored around zero, N(0, 0.1)), small vectors that
    enter scores or logits (``vector``) N(0, 0.5)."""
    g = torch.Generator(device=device)
    g.manual_seed(tensor_seed(seed, name))
    if any(n is None for n in spec.shape):
        raise ValueError(f"random weights for '{name}': its shape {spec.shape} leaves a size open; "
                         "give the part that size as an argument")
    if spec.init == "index_table":
        # int32: every row the first numbers of a random order of 0 .. bound - 1
        rows, per = spec.shape
        if not 0 < per <= spec.bound:
            raise ValueError(f"random weights for '{name}': rows of {per} different numbers below {spec.bound}")
        order = torch.rand(rows, spec.bound, generator=g, dtype=torch.float32, device=device).argsort(1)
        return order[:, :per].to(torch.int32).contiguous()
    if spec.init in ("unit_interval", "decay_log"):
        x = torch.rand(spec.shape, generator=g, dtype=torch.float32, device=device)
        return x if spec.init == "unit_interval" else 3.5 * x - 3.0
    x = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
    if spec.init == "depth_coef":
        x = 0.2 * x
        x.view(-1)[-1] += 1.0
        return x
    if spec.init == "norm":
        return 1.0 + NORM_STD * x
    if spec.init == "norm_offset":
        return NORM_STD * x
    if spec.init == "vector":
        return VECTOR_STD * x
    return MATRIX_STD * x


def write_random_model(model_dir: str, config, seed: int, dtype: str = "bfloat16") -> str:
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (a typed
    configuration or a config.json dict) with weights drawn from ``seed``.
    Matrices are stored in ``dtype``; norm weights always in float32."""
    from ..models.registry import build_model_skeleton, config_from_dict
    if isinstance(config, dict):
        config = config_from_dict(config)
    store = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    expected = build_model_skeleton(config).expected_tensors()
    tensors = {}
    for name, spec in expected.items():
        if spec.optional:
            continue        # (a tensor a file may leave out is left out)
        t = random_tensor(spec, seed, name)
        tensors[name] = t if spec.init in FLOAT32_INITS else t.to(store)
    os.makedirs(model_dir, exist_ok=True)
    d = config.to_dict()
    d["torch_dtype"] = dtype
    with open(os.path.join(model_dir, "config.json"), "w") as f:
        json.dump(d, f, indent=2)
    save_file(tensors, os.path.join(model_dir, "model.safetensors"),
              metadata={"format": "pt", "seed": seed})
    return model_dir
