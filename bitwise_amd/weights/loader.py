"""Weights by tensor name: checking a checkpoint against a model's tensor specs, and
seeded random weights written as a model folder.

Dtype policy (the reference's converter, tools/convert.py:85-92, keeps BF16 and F32
bytes and widens F16 to F32): bfloat16 stays bfloat16, a tensor stored in 32-bit stays
32-bit, float16 is widened to float32, integer tables become int32.  Names are the
checkpoint's own (src/model.cpp:136-171); nothing is renamed.
"""

from __future__ import annotations

import json
import warnings
from pathlib import Path
from typing import Dict, Iterator, Mapping, Sequence, Tuple

import torch

from ..parts.base import TensorSpec
from . import safetensors_io


class WeightError(ValueError):
    """One error for everything wrong with a checkpoint: missing, unexpected, misshapen."""


class UnusedTensorWarning(UserWarning):
    """A checkpoint tensor that the architecture knows of and this configuration does not read."""


def check_and_convert(specs: Mapping[str, TensorSpec], found: Mapping[str, torch.Tensor],
                      source: str = "checkpoint", ignored_suffixes: Sequence[str] = (),
                      unused: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """``ignored_suffixes`` and ``unused`` come from the architecture (``ModelSpec``): tensors it
    knows to carry nothing (passed over in silence) or nothing this configuration reads (passed
    over with an ``UnusedTensorWarning``).  Any other tensor the model has no use for is an error."""
    missing = [n for n in specs if n not in found]
    ignored = tuple(ignored_suffixes)
    extra = [n for n in found if n not in specs and not (ignored and n.endswith(ignored))]
    unexpected = [n for n in extra if n not in unused]
    tolerated = [n for n in extra if n in unused]
    wrong = []
    out: Dict[str, torch.Tensor] = {}
    for name, spec in specs.items():
        if name not in found:
            continue
        t = found[name]
        if tuple(t.shape) != tuple(spec.shape):
            wrong.append(f"{name}: stored {tuple(t.shape)}, the configuration needs {tuple(spec.shape)}")
            continue
        if spec.kind == "int":
            if t.dtype not in (torch.int32, torch.int64):
                wrong.append(f"{name}: stored as {t.dtype}, an integer table is needed")
                continue
            out[name] = t.to(torch.int32)
        elif t.dtype == torch.bfloat16 or t.dtype == torch.float32:
            out[name] = t
        elif t.dtype == torch.float16:
            out[name] = t.to(torch.float32)
        else:
            wrong.append(f"{name}: unsupported dtype {t.dtype}")
    if missing or unexpected or wrong:
        lines = [f"{source} does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape or dtype ({len(wrong)}):")
            lines.extend("    " + w for w in wrong)
        raise WeightError("\n".join(lines))
    if tolerated:
        warnings.warn(f"{source}: tensors stored and not used by this configuration: " + ", ".join(tolerated),
                      UnusedTensorWarning, stacklevel=2)
    return out


def load_folder(folder: str | Path, specs: Mapping[str, TensorSpec], ignored_suffixes: Sequence[str] = (),
                unused: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")       # read-only memory maps viewed as tensors
        found = safetensors_io.read_folder(folder)
    return check_and_convert(specs, found, str(folder), ignored_suffixes, unused)


def random_tensors(specs: Mapping[str, TensorSpec], seed: int, sigma: float = 0.02,
                   dtype: torch.dtype = torch.bfloat16) -> Iterator[Tuple[str, torch.Tensor]]:
    """Seeded random weights, one tensor after the other in the order of ``specs``.

    All draws come from one ``torch.Generator`` (CPU, ``manual_seed(seed)``) as float32
    standard normals in tensor order: linear and embedding weights are ``sigma * z``,
    norm weights ``1 + 0.1 * z``, integer tables uniform in [0, 2**15).  Values are then
    rounded to ``dtype`` (round to nearest even for bfloat16).
    """
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    for name, spec in specs.items():
        if spec.kind == "int":
            yield name, torch.randint(0, 2 ** 15, spec.shape, generator=g, dtype=torch.int32)
            continue
        z = torch.randn(spec.shape, generator=g, dtype=torch.float32)
        if spec.kind == "norm":
            z = 1.0 + 0.1 * z
        else:
            z = sigma * z
        yield name, z.to(dtype)


def write_model_folder(folder: str | Path, config: Mapping[str, object], specs: Mapping[str, TensorSpec],
                       seed: int, sigma: float = 0.02, dtype: torch.dtype = torch.bfloat16) -> Path:
    """Random-weights mode: ``folder/config.json`` and ``folder/model.safetensors``."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(dict(config), indent=1))
    safetensors_io.write_file(folder / "model.safetensors", random_tensors(specs, seed, sigma, dtype))
    return folder
