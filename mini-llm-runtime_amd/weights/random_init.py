"""Random-weights mode: write a model folder (config.json, model.safetensors) from a
configuration and a seed.  Matrices are N(0, 0.02), norm weights 1 + N(0, 0.1); every tensor
has a generator of its own, seeded from (seed, tensor name), so the values of one tensor do
not depend on which other tensors exist."""
from __future__ import annotations

import hashlib
import json
import os

import torch

from .safetensors_io import write_safetensors


def _generator(seed, name):
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


def random_tensors(expected, seed, dtype=torch.bfloat16, matrix_std=0.02, norm_std=0.1):
    """expected: {name: WeightSpec}.  Optional tensors are left out.  Every tensor has a generator of its own,
    so they are drawn side by side in threads (the values do not depend on how many)."""
    from concurrent.futures import ThreadPoolExecutor

    def draw(item):
        name, spec = item
        g = _generator(seed, name)
        if any(e is None for e in spec.shape):
            raise ValueError(f"tensor {name}: a size that only a file gives; the configuration must name it for random weights")
        if spec.init is not None:
            kind, a, b = spec.init
            if kind == "normal":
                t = a + b * torch.randn(spec.shape, generator=g, dtype=torch.float32)
            elif kind == "uniform":
                t = a + (b - a) * torch.rand(spec.shape, generator=g, dtype=torch.float32)
            else:
                raise ValueError(f"tensor {name}: unknown initialisation {kind!r}")
        elif spec.keep_float32:
            t = 1.0 + norm_std * torch.randn(spec.shape, generator=g, dtype=torch.float32)
        else:
            t = matrix_std * torch.randn(spec.shape, generator=g, dtype=torch.float32)
        return name, t.to(dtype)
    todo = [(name, spec) for name, spec in expected.items() if not spec.optional]
    workers = max(1, min(16, os.cpu_count() or 1, len(todo)))
    if workers == 1 or sum(_numel(spec.shape) for _, spec in todo) < (1 << 22):
        return dict(draw(item) for item in todo)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        return dict(pool.map(draw, todo))              # (in the order of `expected`)


def random_tensors_on_device(expected, seed, dtype, device, matrix_std=0.02, norm_std=0.1):
    """The same kinds of tensors drawn on the device itself (other values than `random_tensors` gives for the
    seed): a model of many gigabytes without the trip through a file.  32-bit vectors stay float32, the rest gets
    `dtype`, as the loader would place them."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    out = {}
    for name, spec in expected.items():
        if spec.optional:
            continue
        if any(e is None for e in spec.shape):
            raise ValueError(f"tensor {name}: a size that only a file gives; the configuration must name it for random weights")
        kind = torch.float32 if spec.keep_float32 else dtype
        if spec.init is not None and spec.init[0] == "uniform":
            t = torch.rand(spec.shape, generator=g, device=device, dtype=torch.float32)
            t = t.mul_(spec.init[2] - spec.init[1]).add_(spec.init[1])
        else:
            mean, std = (spec.init[1], spec.init[2]) if spec.init is not None else (1.0, norm_std) if spec.keep_float32 \
                else (0.0, matrix_std)
            t = torch.randn(spec.shape, generator=g, device=device, dtype=kind).mul_(std).add_(mean)
        out[name] = t.to(kind)
    return out


def _numel(shape):
    count = 1
    for extent in shape:
        count *= int(extent or 0)
    return count


def write_random_model(folder, config, seed, dtype=torch.bfloat16, matrix_std=0.02, norm_std=0.1):
    """`config` is an architecture's configuration object (e.g. Qwen3Config)."""
    from ..parts.model import expected_tensors

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config.to_dict(), f, indent=1)
    expected = expected_tensors(config)
    tensors = random_tensors(expected, seed, dtype, matrix_std, norm_std)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      {"format": "pt", "seed": seed})
    return folder
