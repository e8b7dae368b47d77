"""Weights by tensor name: safetensors reader, random-weights source, folder writer.

The reader follows the reference's ``load_state_dict``
(src/cloud_engine/weights.py:81-121): every ``*.safetensors`` of the folder in
sorted order, duplicate names refused, names and shapes checked against the
table the model's parts declare.  Where the reference raises at the first kind
of fault, this raises one :class:`WeightError` that lists missing tensors,
unexpected tensors and wrong shapes together.  A tied model that also ships
``lm_head.weight`` is accepted only when that tensor equals the embedding (the
reference drops it unchecked, src/cloud_engine/weights.py:31-33,103-104).

Floating tensors run in the engine's dtype (bfloat16 or float32); a tensor the
part marks ``keeps_float32`` stays in 32-bit if the file stores it so; integer
tables become int32.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Any, Mapping

import torch

from .tensors import TensorSpec

INIT_STD = 0.02
_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class WeightError(Exception):
    """Checkpoint and model disagree; the message lists every disagreement."""

    def __init__(self, missing: list[str], unexpected: list[str], wrong_shape: list[str],
                 other: list[str] | None = None) -> None:
        self.missing = missing
        self.unexpected = unexpected
        self.wrong_shape = wrong_shape
        self.other = other or []
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        for line in self.other:
            lines.append("  " + line)
        super().__init__("\n".join(lines))


def torch_dtype(name: str) -> torch.dtype:
    return _TORCH_DTYPES[name]


def _target_dtype(spec: TensorSpec, stored: torch.dtype, dtype: torch.dtype) -> torch.dtype:
    if spec.kind == "int":
        return torch.int32
    if spec.keeps_float32 and stored == torch.float32:
        return torch.float32
    return dtype


class SafetensorsSource:
    """Tensors of a model folder, checked against ``expected`` before any is used."""

    def __init__(self, model_dir: str | Path) -> None:
        self.model_dir = Path(model_dir)
        self.paths = sorted(self.model_dir.glob("*.safetensors"))
        if not self.paths:
            raise FileNotFoundError(f"no *.safetensors found in {self.model_dir}")

    def _index(self) -> dict[str, tuple[Path, tuple[int, ...]]]:
        import safetensors

        index: dict[str, tuple[Path, tuple[int, ...]]] = {}
        for path in self.paths:
            with safetensors.safe_open(str(path), framework="pt", device="cpu") as handle:
                for key in handle.keys():
                    if key in index:
                        raise ValueError(
                            f"duplicate tensor {key!r} in {path.name} and {index[key][0].name}"
                        )
                    index[key] = (path, tuple(handle.get_slice(key).get_shape()))
        return index

    def load(self, expected: Mapping[str, TensorSpec], dtype: str, device: str | torch.device,
             tied_optional: Mapping[str, str] | None = None) -> dict[str, torch.Tensor]:
        """``tied_optional`` maps a tensor name that may be present although the
        model does not use it (a tied head) to the tensor it must equal."""
        import safetensors

        tied_optional = dict(tied_optional or {})
        index = self._index()
        missing = sorted(set(expected) - set(index))
        unexpected = sorted(set(index) - set(expected) - set(tied_optional))
        wrong = [
            f"{name}: expected {tuple(spec.shape)}, got {index[name][1]}"
            for name, spec in expected.items()
            if name in index and tuple(index[name][1]) != tuple(spec.shape)
        ]
        if missing or unexpected or wrong:
            raise WeightError(missing, unexpected, wrong)

        target = torch_dtype(dtype)
        present_twins = {twin for name, twin in tied_optional.items() if name in index}
        by_path: dict[Path, list[str]] = {}
        for name in list(expected) + [n for n in tied_optional if n in index]:
            by_path.setdefault(index[name][0], []).append(name)
        out: dict[str, torch.Tensor] = {}
        stored: dict[str, torch.Tensor] = {}  # raw copies needed for the tied-head check only
        for path, names in by_path.items():
            with safetensors.safe_open(str(path), framework="pt", device="cpu") as handle:
                for name in names:
                    tensor = handle.get_tensor(name)
                    if name in expected:
                        spec = expected[name]
                        out[name] = tensor.to(_target_dtype(spec, tensor.dtype, target)).to(device)
                    if name in tied_optional or name in present_twins:
                        stored[name] = tensor
        problems = [
            f"{name} is present in a tied model but differs from {twin}"
            for name, twin in tied_optional.items()
            if name in stored
            and (twin not in stored or stored[twin].shape != stored[name].shape
                 or not torch.equal(stored[twin], stored[name]))
        ]
        if problems:
            raise WeightError([], [], [], problems)
        return out


class RandomSource:
    """Seeded random weights: every tensor N(0, 0.02), norm weights 1 + N(0, 0.02).

    Tensors are drawn in float32 in the order of ``expected`` from one generator
    per tensor (seeded by the run's seed and the tensor's index), then cast, so a
    seed names the same model on every device.  ``draw_device="cuda"`` draws on
    the GPU instead: faster for benchmark-sized models, different numbers.
    """

    def __init__(self, seed: int, std: float = INIT_STD, draw_device: str = "cpu") -> None:
        self.seed = int(seed)
        self.std = float(std)
        self.draw_device = draw_device

    def draw(self, index: int, spec: TensorSpec) -> torch.Tensor:
        generator = torch.Generator(device=self.draw_device)
        generator.manual_seed((self.seed * 1_000_003 + index * 7919 + 12345) % (2**63 - 1))
        if spec.kind == "int":
            return torch.zeros(spec.shape, dtype=torch.int32, device=self.draw_device)
        values = torch.randn(spec.shape, generator=generator, dtype=torch.float32,
                             device=self.draw_device) * self.std
        if spec.init == "norm":
            values += 1.0
        elif spec.init != "normal":
            raise ValueError(f"unknown init {spec.init!r}")
        return values

    def load(self, expected: Mapping[str, TensorSpec], dtype: str, device: str | torch.device,
             tied_optional: Mapping[str, str] | None = None) -> dict[str, torch.Tensor]:
        target = torch_dtype(dtype)
        out = {}
        for index, (name, spec) in enumerate(expected.items()):
            tensor = self.draw(index, spec)
            out[name] = tensor.to(_target_dtype(spec, torch.bfloat16, target)).to(device)
        return out


def write_model_folder(model_dir: str | Path, config: Any, seed: int,
                       store_dtype: str = "bfloat16", std: float = INIT_STD) -> Path:
    """Random-weights mode: write ``config.json`` and ``model.safetensors`` for
    ``config`` (a typed configuration of a registered architecture)."""
    import safetensors.torch

    from ..parts.model import expected_tensors

    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    expected = expected_tensors(config.model_spec())
    tensors = RandomSource(seed, std).load(expected, store_dtype, "cpu")
    with open(model_dir / "config.json", "w", encoding="utf-8") as handle:
        raw = config.to_hf_config()
        raw["torch_dtype"] = store_dtype
        json.dump(raw, handle, indent=2)
    safetensors.torch.save_file({k: v.contiguous() for k, v in tensors.items()},
                                str(model_dir / "model.safetensors"))
    return model_dir


def write_tensors(model_dir: str | Path, raw_config: dict[str, Any],
                  tensors: Mapping[str, torch.Tensor]) -> Path:
    """Write given tensors and a raw ``config.json`` (used to craft test folders)."""
    import safetensors.torch

    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    with open(model_dir / "config.json", "w", encoding="utf-8") as handle:
        json.dump(raw_config, handle, indent=2)
    safetensors.torch.save_file({k: v.contiguous() for k, v in tensors.items()},
                                str(model_dir / "model.safetensors"))
    return model_dir
