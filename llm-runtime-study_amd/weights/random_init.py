"""Random weights from a configuration and a seed.

`write_model_dir` writes a complete model folder (config.json, model.safetensors) that loads
like any checkpoint.  Tensors are drawn one by one, in sorted name order, from one CPU
generator, so a folder is a function of (configuration, seed, init) alone.

init = "normal": matrices and embedding N(0, 0.02), norm weights 1 + N(0, 0.02), biases
N(0, 0.02).  init = "scaled": matrices N(0, 1/fan_in), embedding N(0, 1), norm weights
1 + N(0, 0.1), biases N(0, 0.1), which keeps every part's contribution at order one so that
tests see faults that tiny weights would hide.

`device_weights` makes tensors on the device directly (same distributions, other numbers: every
tensor has a generator of its own, seeded by the seed and the tensor's place in the sorted names) for
benchmark-sized models, where a file would only cost time.  Each tensor is drawn when it is asked for,
so a model that takes its tensors part by part never holds two copies of its weights.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch

from ..config import spec_for
from ..models import DecoderModel
from ..parts import LazyTensors, TensorSpec
from .safetensors_io import write_safetensors

TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _draw(spec: TensorSpec, init: str, generator, device="cpu") -> torch.Tensor:
    if spec.dtype == "int32":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    noise = torch.randn(spec.shape, generator=generator, device=device, dtype=torch.float32)
    if init == "normal":
        return 1.0 + 0.02 * noise if spec.role == "norm" else 0.02 * noise
    if init == "scaled":
        if spec.role == "norm":
            return 1.0 + 0.1 * noise
        if spec.role == "bias":
            return 0.1 * noise
        if spec.role == "embedding":
            return noise
        return noise / float(spec.shape[-1]) ** 0.5
    raise ValueError(f"unknown init {init!r}; expected 'normal' or 'scaled'")


def random_tensors(expected: dict[str, TensorSpec], seed: int, dtype: torch.dtype, init: str = "normal") -> dict[str, torch.Tensor]:
    generator = torch.Generator().manual_seed(seed)
    return {name: _draw(expected[name], init, generator).to(torch.int32 if expected[name].dtype == "int32" else dtype)
            for name in sorted(expected) if not expected[name].optional}


def write_model_dir(config, seed: int, model_dir, init: str = "normal") -> Path:
    """Write config.json and model.safetensors for `config` (a typed configuration)."""
    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    spec = spec_for(config)
    expected = DecoderModel(spec).tensors()
    tensors = random_tensors(expected, seed, TORCH_DTYPES[spec.checkpoint_dtype], init)
    (model_dir / "config.json").write_text(json.dumps(config.to_json_dict(), indent=2) + "\n")
    write_safetensors(model_dir / "model.safetensors", tensors, {"seed": seed, "init": init})
    return model_dir


def device_weights(model: DecoderModel, seed: int, dtype: torch.dtype, device, init: str = "normal") -> LazyTensors:
    expected = model.tensors()
    names = [name for name in sorted(expected) if not expected[name].optional]
    place = {name: index for index, name in enumerate(names)}

    def draw(name: str) -> torch.Tensor:
        generator = torch.Generator(device=device).manual_seed((seed << 20) + place[name])
        return _draw(expected[name], init, generator, device).to(torch.int32 if expected[name].dtype == "int32" else dtype)

    return LazyTensors(names, draw)


def main(argv=None) -> int:
    """`python -m llm_runtime_study_amd.weights.random_init --config config.json --seed 0 --out DIR`"""
    import argparse

    from ..config import config_from_dict

    parser = argparse.ArgumentParser(description="Write a model folder with random weights for a config.json.")
    parser.add_argument("--config", type=Path, required=True, help="a config.json (or a folder holding one)")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--out", type=Path, required=True)
    parser.add_argument("--init", choices=("normal", "scaled"), default="normal")
    args = parser.parse_args(argv)
    path = args.config / "config.json" if args.config.is_dir() else args.config
    config = config_from_dict(json.loads(path.read_text()))
    write_model_dir(config, args.seed, args.out, args.init)
    print(f"wrote {args.out}/config.json and model.safetensors")
    return 0


if __name__ == "__main__":
    import sys

    sys.exit(main())
