"""The user-facing model: a folder with config.json and safetensors (or seeded random
weights) turned into an assembled model on the GPU.  Names follow the reference's Python
module (python/bindings.cpp:24-52): ``Model.load``, ``.config``, ``.weight_bytes``,
``.logits(tokens)``; ``Model.random`` is the counterpart of Model::random
(src/model.cpp:176-218) with the weight distributions of this build's test configurations.
"""

from __future__ import annotations

import json
import tempfile
from pathlib import Path
from typing import Any, Dict, Mapping, Optional, Sequence

import numpy as np
import torch

from . import registry
from .models.assembled import AssembledModel
from .parts.base import TensorSpec
from .runtime import Runtime
from .weights import loader


def model_spec(config: Mapping[str, Any]):
    """The ``ModelSpec`` its architecture makes of a configuration (a config.json dictionary)."""
    arch = registry.architecture_of(config)
    return arch.spec_from_config(arch.config_from_dict(config))


def describe(config: Mapping[str, Any]) -> Dict[str, TensorSpec]:
    """Names and shapes of the checkpoint tensors a configuration needs (no GPU involved)."""
    return AssembledModel(model_spec(config), Runtime("float32", device=None)).tensor_specs()


def write_random_model(folder: str | Path, config: Mapping[str, Any], seed: int, sigma: float = 0.02,
                       dtype: str = "bfloat16") -> Path:
    """Random-weights mode: writes ``config.json`` and ``model.safetensors`` into ``folder``.
    Linear and embedding weights are N(0, sigma), norm weights 1 + N(0, 0.1), drawn in the
    model's tensor order from one generator seeded with ``seed``."""
    arch = registry.architecture_of(config)
    typed = arch.config_from_dict(config)
    torch_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}[dtype]
    return loader.write_model_folder(folder, typed.to_dict(), describe(config), seed, sigma, torch_dtype)


class Model:
    def __init__(self, config: Any, assembled: AssembledModel):
        self.config = config
        self.assembled = assembled

    # ------------------------------------------------------------------ construction
    @classmethod
    def load(cls, path: str | Path, dtype: str = "bfloat16", device: str = "cuda:0") -> "Model":
        """``path``: a folder with config.json and *.safetensors; the model class is chosen by
        ``architectures[0]``.  dtype "bfloat16" or "float32" picks the precision mode."""
        raw = registry.read_config(path)
        arch = registry.architecture_of(raw)
        typed = arch.config_from_dict(raw)
        rt = Runtime(dtype, device)
        spec = arch.spec_from_config(typed)
        assembled = AssembledModel(spec, rt)
        tensors = loader.load_folder(path, assembled.tensor_specs(), spec.ignored_tensor_suffixes, spec.unused_tensors)
        assembled.bind_tensors(tensors)
        return cls(typed, assembled)

    @classmethod
    def random(cls, config: Mapping[str, Any], seed: int, dtype: str = "bfloat16", sigma: float = 0.02,
               device: str = "cuda:0", weight_dtype: str = "bfloat16", on_device: bool = False) -> "Model":
        """Seeded random weights for a configuration (a config.json dictionary).

        By default the weights go through a model folder in a temporary directory, so that
        the same bytes can be loaded by anything else.  ``on_device`` draws them on the GPU
        instead (for large benchmark shapes; other bits than the folder route)."""
        if not on_device:
            with tempfile.TemporaryDirectory(prefix="bitwise_amd_") as tmp:
                write_random_model(tmp, config, seed, sigma, weight_dtype)
                return cls.load(tmp, dtype, device)
        arch = registry.architecture_of(config)
        typed = arch.config_from_dict(config)
        rt = Runtime(dtype, device)
        assembled = AssembledModel(arch.spec_from_config(typed), rt)
        gen = torch.Generator(device=rt.device)
        gen.manual_seed(int(seed))
        wd = {"bfloat16": torch.bfloat16, "float32": torch.float32}[weight_dtype]
        tensors = {}
        for name, ts in assembled.tensor_specs().items():
            if ts.kind == "int":
                tensors[name] = torch.randint(0, 2 ** 15, ts.shape, generator=gen, dtype=torch.int32, device=rt.device)
                continue
            z = torch.randn(ts.shape, generator=gen, dtype=torch.float32, device=rt.device)
            tensors[name] = ((1.0 + 0.1 * z) if ts.kind == "norm" else (sigma * z)).to(wd)
        assembled.bind_tensors(tensors)
        return cls(typed, assembled)

    # ------------------------------------------------------------------ facts
    @property
    def dtype(self) -> str:
        return self.assembled.rt.mode

    @property
    def weight_bytes(self) -> int:
        return self.assembled.weight_bytes()

    # ------------------------------------------------------------------ numerics entry
    def logits(self, tokens: Sequence[int], chunk: Optional[int] = None, block_size: int = 16) -> np.ndarray:
        """Logits [n, vocab] at every position of one sequence, run as a prompt through a
        fresh cache of its own (python/bindings.cpp:35-52); ``chunk`` cuts the prompt into
        steps.  It shares nothing with engines that run the same model."""
        from .engine.runner import ModelRunner
        from .engine.batch import Segment
        from .engine.storage import CacheStorage

        asm = self.assembled
        n = len(tokens)
        if n > asm.spec.max_positions:
            raise ValueError(f"{n} tokens exceed the model's {asm.spec.max_positions} positions")
        if n == 0:
            return np.empty((0, asm.spec.vocab_size), np.float32)
        step = max(1, min(chunk or 256, 256, n))
        pages = (n + block_size - 1) // block_size
        storage = CacheStorage(asm, pages, 1, block_size)
        runner = ModelRunner(asm, storage, max_model_len=n, max_rows=step, use_graphs=False)
        tables = [list(range(pages)) for _ in asm.group_specs]
        out = np.empty((n, asm.spec.vocab_size), np.float32)
        for start in range(0, n, step):
            part = list(tokens[start:start + step])
            lg = runner.step([Segment(part, start, tables, 0, list(range(len(part))))])
            out[start:start + len(part)] = lg.cpu().numpy()
        return out
