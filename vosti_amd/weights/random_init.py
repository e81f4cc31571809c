"""Random weights from a configuration and a seed.

Every element is a function of (seed, tensor name, element index) only: the
generator is counter-based, so a tensor can be drawn in any order, in pieces,
on the host (numpy, here) or on the GPU (fill_random_kernel) with the same
bits.  Matrices and the embedding are approximately normal with standard
deviation 0.02 (a sum of four 16-bit uniforms, scaled); norm weights are
uniform in [0.9, 1.1).
"""
from __future__ import annotations

import hashlib
import json
import math
from pathlib import Path

import numpy as np
import torch

_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_GOLD = np.uint64(0x9E3779B97F4A7C15)


def tensor_seed(seed: int, name: str) -> int:
    h = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    return int.from_bytes(h, "little")


def _mix64(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def _init_params(init: tuple) -> tuple[int, float, float]:
    """(kind, p0, p1) as the kernel takes them, both as float32 values."""
    if init[0] == "normal":
        return 0, float(np.float32(init[1] * math.sqrt(3.0) / 65536.0)), 0.0
    if init[0] == "uniform":
        return 1, float(np.float32(init[1])), float(np.float32(init[2] - init[1]))
    raise ValueError(f"unknown init {init!r}")


def random_tensor_cpu(seed: int, name: str, shape: tuple[int, ...], init: tuple) -> torch.Tensor:
    """float32 values of tensor ``name`` (before any rounding to a storage type)."""
    n = int(np.prod(shape)) if shape else 1
    kind, p0, p1 = _init_params(init)
    s = np.uint64(tensor_seed(seed, name))
    out = np.empty(n, dtype=np.float32)
    step = 1 << 22
    with np.errstate(over="ignore"):
        for a in range(0, n, step):
            idx = np.arange(a, min(n, a + step), dtype=np.uint64)
            z = _mix64(s ^ (idx * _GOLD))
            if kind == 0:
                m = np.uint64(0xFFFF)
                tot = ((z & m) + ((z >> np.uint64(16)) & m) + ((z >> np.uint64(32)) & m) + (z >> np.uint64(48))).astype(np.int64)
                out[a:a + len(idx)] = (tot - 131070).astype(np.float32) * np.float32(p0)
            else:
                u = (z >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
                out[a:a + len(idx)] = np.float32(p0) + u * np.float32(p1)
    return torch.from_numpy(out).reshape(shape)


def expected_tensor_specs(config) -> dict[str, tuple[tuple[int, ...], tuple]]:
    """Tensor name -> (shape, init) for a configuration; needs no GPU."""
    from ..models.decoder import DecoderModel
    model = DecoderModel(config.model_spec(), None)
    return {name: (e.spec.shape, e.spec.init) for name, e in model.expected_tensors().items()}


def write_random_model(config, seed: int, out_dir: str | Path, dtype: torch.dtype = torch.bfloat16) -> Path:
    """Writes config.json and model.safetensors for ``config`` with weights drawn from ``seed``."""
    from safetensors.torch import save_file
    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    tensors = {}
    for name, (shape, init) in expected_tensor_specs(config).items():
        tensors[name] = random_tensor_cpu(seed, name, shape, init).to(dtype).contiguous()
    cfg = config.to_dict()
    cfg["torch_dtype"] = str(dtype).replace("torch.", "")
    (out / "config.json").write_text(json.dumps(cfg, indent=2) + "\n")
    save_file(tensors, str(out / "model.safetensors"), metadata={"format": "pt", "seed": str(seed)})
    return out


def random_weights_on_gpu(model, seed: int) -> None:
    """Fills a model with the same values ``write_random_model`` would store in its compute type, on the GPU."""
    k = model.kernels
    tensors = {}
    for name, e in model.expected_tensors().items():
        ps = e.spec
        t = torch.empty(ps.shape, dtype=k.dtype, device="cuda")
        kind, p0, p1 = _init_params(ps.init)
        k.fill_random(t, tensor_seed(seed, name), kind, p0, p1)
        tensors[name] = t
    model.load_tensors(tensors)
