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

    def open(self, expected: Mapping[str, TensorSpec], dtype: str, device: str | torch.device,
             tied_optional: Mapping[str, str] | None = None) -> "TensorsOnDemand":
        """Check names and shapes of the whole folder against ``expected`` (one
        :class:`WeightError` for all faults), then hand out tensors as they are asked
        for.  ``tied_optional`` maps a tensor name that may be present although the
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
        handles: dict[Path, Any] = {}

        def stored(name: str) -> torch.Tensor:
            path = index[name][0]
            if path not in handles:
                handles[path] = safetensors.safe_open(str(path), framework="pt", device="cpu")
            return handles[path].get_tensor(name)

        problems = []
        for name, twin in tied_optional.items():
            if name in index and (twin not in index or index[twin][1] != index[name][1]
                                  or not torch.equal(stored(twin), stored(name))):
                problems.append(f"{name} is present in a tied model but differs from {twin}")
        if problems:
            raise WeightError([], [], [], problems)

        def make(name: str) -> torch.Tensor:
            tensor = stored(name)
            return tensor.to(_target_dtype(expected[name], tensor.dtype, target)).to(device)

        return TensorsOnDemand(expected, make)

    def load(self, expected: Mapping[str, TensorSpec], dtype: str, device: str | torch.device,
             tied_optional: Mapping[str, str] | None = None) -> dict[str, torch.Tensor]:
        """All tensors of :meth:`open` at once, as a dictionary."""
        return dict(self.open(expected, dtype, device, tied_optional).items())


class TensorsOnDemand(Mapping):
    """Name → tensor on the target device, made when it is asked for and not kept.

    A model binds its tensors one after the other and keeps its own forms of some
    (q/k/v as one matrix, gate and up as one); with every tensor made at its turn the
    checkpoint's tensors and the model's never lie side by side in device memory in
    full, so a model may take more than half of it."""

    def __init__(self, names, make) -> None:
        self._names = tuple(names)
        self._known = frozenset(self._names)
        self._make = make

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self._known:
            raise KeyError(name)
        return self._make(name)

    def __iter__(self):
        return iter(self._names)

    def __len__(self) -> int:
        return len(self._names)


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

    def open(self, expected: Mapping[str, TensorSpec], dtype: str, device: str | torch.device,
             tied_optional: Mapping[str, str] | None = None) -> TensorsOnDemand:
        """Tensors drawn as they are asked for (each from its own seed, so the order of asking does not matter)."""
        target = torch_dtype(dtype)
        place = {name: index for index, name in enumerate(expected)}

        def make(name: str) -> torch.Tensor:
            spec = expected[name]
            return self.draw(place[name], spec).to(_target_dtype(spec, torch.bfloat16, target)).to(device)

        return TensorsOnDemand(expected, make)

    def load(self, expected: Mapping[str, TensorSpec], dtype: str, device: str | torch.device,
             tied_optional: Mapping[str, str] | None = None) -> dict[str, torch.Tensor]:
        """All tensors of :meth:`open` at once, as a dictionary."""
        return dict(self.open(expected, dtype, device, tied_optional).items())


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
