"""Weights from safetensors files, by tensor name.

File mechanics follow the reference's helper
(python/vosti_kernels/checkpoint.py:15-78): ``model.safetensors.index.json``
with its ``weight_map`` if present, else a single ``model.safetensors``; shard
paths must stay inside the model folder; the key set must equal what the model
expects and every shape must match.  All problems are gathered into one error.

Floating tensors are converted to the compute type (bfloat16 or float32);
a parameter marked ``keep_f32`` that the file stores in 32-bit stays so;
integer tensors become int32.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Mapping

import torch
from safetensors import safe_open

_ST_DTYPES = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
              "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
              "BOOL": torch.bool}


class WeightError(RuntimeError):
    pass


class Checkpoint:
    """Name -> (file, shape, dtype) of every tensor in a model folder."""

    def __init__(self, model_dir: str | Path):
        self.dir = Path(model_dir).resolve()
        index = self.dir / "model.safetensors.index.json"
        single = self.dir / "model.safetensors"
        if index.is_file():
            weight_map = json.loads(index.read_text()).get("weight_map")
            if not isinstance(weight_map, dict) or not weight_map:
                raise WeightError(f"{index} has no 'weight_map'")
            files = sorted(set(weight_map.values()))
        elif single.is_file():
            files = [single.name]
        else:
            raise WeightError(f"{self.dir} holds neither model.safetensors nor model.safetensors.index.json")
        self.entries: dict[str, tuple[Path, tuple[int, ...], str]] = {}
        for f in files:
            path = (self.dir / f).resolve()
            if self.dir not in path.parents:
                raise WeightError(f"shard {f!r} lies outside the model folder")
            if not path.is_file():
                raise WeightError(f"shard {path} is missing")
            with safe_open(str(path), framework="pt", device="cpu") as sf:
                for name in sf.keys():
                    sl = sf.get_slice(name)
                    self.entries[name] = (path, tuple(sl.get_shape()), sl.get_dtype())

    def read(self, names) -> Mapping[str, torch.Tensor]:
        by_file: dict[Path, list[str]] = {}
        for n in names:
            by_file.setdefault(self.entries[n][0], []).append(n)
        out = {}
        for path, ns in by_file.items():
            with safe_open(str(path), framework="pt", device="cpu") as sf:
                for n in ns:
                    out[n] = sf.get_tensor(n)
        return out


def open_checkpoint(model_dir) -> Checkpoint:
    return Checkpoint(model_dir)


def check_against(model, ckpt: Checkpoint) -> None:
    """Raises one WeightError listing missing, unexpected and misshapen tensors."""
    expected = model.expected_tensors()
    ignorable = set(model.spec.ignored_names)
    missing = sorted(n for n in expected if n not in ckpt.entries)
    unexpected = sorted(n for n in ckpt.entries if n not in expected and n not in ignorable)
    wrong = []
    for n, e in expected.items():
        ps = e.spec
        if n in ckpt.entries:
            _, shape, dt = ckpt.entries[n]
            if tuple(shape) != tuple(ps.shape):
                wrong.append(f"{n}: file has {list(shape)}, model needs {list(ps.shape)}")
            elif dt not in _ST_DTYPES:
                wrong.append(f"{n}: unsupported stored type {dt}")
    if missing or unexpected or wrong:
        lines = [f"weights in {ckpt.dir} do not fit the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape or type ({len(wrong)}): " + "; ".join(sorted(wrong)))
        raise WeightError("\n".join(lines))


def convert(t: torch.Tensor, compute_dtype: torch.dtype, keep_f32: bool) -> torch.Tensor:
    if t.dtype.is_floating_point:
        if keep_f32 and t.dtype == torch.float32:
            return t
        return t.to(compute_dtype)
    return t.to(torch.int32)


def load_weights(model, model_dir, device: str = "cuda") -> None:
    """Check the folder against the model, then load tensor by tensor onto the GPU."""
    ckpt = Checkpoint(model_dir)
    check_against(model, ckpt)
    expected = model.expected_tensors()
    dtype = model.kernels.dtype
    tensors = {}
    # One tensor at a time: the whole checkpoint never sits in host memory.
    for name, e in expected.items():
        t = ckpt.read([name])[name]
        tensors[name] = convert(t, dtype, e.spec.keep_f32).contiguous().to(device)
    model.load_tensors(tensors)
