"""Reads a model's tensors from safetensors by name.

The reference opens ``model.safetensors`` or the shards named by
``model.safetensors.index.json`` and takes the tensors its name map asks for
(tokasaurus/model/safetensors_utils.py:29-97); a missing name surfaces there as
a bare ``KeyError`` (tokasaurus/model/llama.py:938) and shapes are not checked.
Here everything wrong with a checkpoint is reported in one error: tensors that
are missing, tensors nobody asked for, and tensors of the wrong shape.

Storage types: floating tensors of 16 bits are taken as they are and widened
exactly when the engine runs in 32-bit; integer tables become int32; a tensor
stored in 32-bit is handed on in 32-bit (a part that needs the engine dtype for
its kernels, such as a matrix product, narrows it itself when it places it).
"""

from __future__ import annotations

import json
import logging
from pathlib import Path

import torch
from safetensors import safe_open

from tokasaurus_amd.parts.base import INT_TABLE, TensorSpec

SINGLE_FILE = "model.safetensors"
INDEX_FILE = "model.safetensors.index.json"


log = logging.getLogger("tokasaurus_amd")


class WeightError(ValueError):
    """A checkpoint that does not hold what the model needs."""

    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_type=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.wrong_type = sorted(wrong_type)
        lines = [f"checkpoint in {folder} does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(
                f"  wrong shapes ({len(self.wrong_shape)}): "
                + ", ".join(f"{n}: has {list(h)}, wanted {list(w)}" for n, h, w in self.wrong_shape)
            )
        if self.wrong_type:
            lines.append(
                f"  wrong types ({len(self.wrong_type)}): "
                + ", ".join(f"{n}: {t}" for n, t in self.wrong_type)
            )
        super().__init__("\n".join(lines))


def _files_by_tensor(folder: Path) -> dict[str, Path]:
    """tensor name -> file that holds it (safetensors_utils.py:34-68)."""
    single, index = folder / SINGLE_FILE, folder / INDEX_FILE
    if single.is_file():
        with safe_open(str(single), framework="pt") as f:
            return {name: single for name in f.keys()}
    if index.is_file():
        weight_map = json.loads(index.read_text())["weight_map"]
        return {name: folder / fname for name, fname in weight_map.items()}
    raise FileNotFoundError(f"no {SINGLE_FILE} or {INDEX_FILE} in {folder}")


def read_tensors(
    folder: str | Path,
    specs: list[TensorSpec],
    allow_unexpected: tuple[str, ...] = (),
) -> dict[str, torch.Tensor]:
    """Host tensors for every spec, or one WeightError naming all faults.

    ``allow_unexpected`` lists names that may be present without being used (a
    checkpoint that ties its head may still carry ``lm_head.weight``)."""
    folder = Path(folder)
    where = _files_by_tensor(folder)
    wanted = {s.name: s for s in specs}
    missing = [n for n in wanted if n not in where]
    unexpected = [n for n in where if n not in wanted and n not in allow_unexpected]
    ignored = [n for n in where if n not in wanted and n in allow_unexpected]
    if ignored:
        # the reference reads such a tensor's storage from the tensor it is tied to (llama.py:842-845)
        log.warning("checkpoint in %s carries %s, which this model does not read: ignored", folder, ", ".join(sorted(ignored)))
    wrong_shape, wrong_type = [], []
    out: dict[str, torch.Tensor] = {}
    by_file: dict[Path, list[str]] = {}
    for name in wanted:
        if name in where:
            by_file.setdefault(where[name], []).append(name)
    for path, names in by_file.items():
        if not path.is_file():
            missing.extend(names)
            continue
        with safe_open(str(path), framework="pt") as f:
            present = set(f.keys())
            for name in names:
                if name not in present:
                    missing.append(name)
                    continue
                shape = tuple(f.get_slice(name).get_shape())
                if shape != tuple(wanted[name].shape):
                    wrong_shape.append((name, shape, tuple(wanted[name].shape)))
                    continue
                t = f.get_tensor(name)
                if wanted[name].kind == INT_TABLE:
                    if t.is_floating_point():
                        wrong_type.append((name, f"integer table stored as {t.dtype}"))
                        continue
                    t = t.to(torch.int32)
                elif not t.is_floating_point():
                    wrong_type.append((name, f"float tensor stored as {t.dtype}"))
                    continue
                elif t.dtype == torch.float64:
                    t = t.to(torch.float32)
                out[name] = t
    if missing or unexpected or wrong_shape or wrong_type:
        raise WeightError(folder, missing, unexpected, wrong_shape, wrong_type)
    return out
