"""bitwise_amd: a small, whole inference engine for the Llama decoder on one MI355X.

The interface follows the reference's Python module (python/bitwise/__init__.py:3-10,
README.md:182-191):

    import bitwise_amd as bw
    model = bw.Model.load("model_folder")                    # config.json + safetensors
    cfg = bw.EngineConfig(); cfg.max_batched_tokens = 256
    engine = bw.Engine(model, None, cfg)
    rid = engine.add_request(prompt_token_ids, bw.SamplingParams(temperature=0.7, seed=1, max_new_tokens=64))
    while not engine.idle():
        engine.step()
    print(engine.result(rid).tokens, hex(engine.result(rid).logits_fingerprint))
"""

from .config.engine import EngineConfig, SamplingParams  # noqa: F401
from .config.llama import ConfigError, LlamaConfig  # noqa: F401
from .engine.engine import Engine, EngineStats, RequestResult, StepEvent  # noqa: F401
from .model import Model, describe, write_random_model  # noqa: F401
from .registry import ARCHITECTURES, register_architecture  # noqa: F401
from .weights.loader import WeightError  # noqa: F401


def generate(model: "Model", prompts, params=None, config: "EngineConfig | None" = None):
    """Run prompts (lists of token ids) to completion; returns one RequestResult per prompt."""
    cfg = config or EngineConfig(dtype=model.dtype)
    engine = Engine(model, None, cfg)
    if params is None or isinstance(params, SamplingParams):
        params = [params or SamplingParams()] * len(prompts)
    ids = [engine.add_request(p, sp) for p, sp in zip(prompts, params)]
    while not engine.idle():
        engine.step()
    return [engine.result(i) for i in ids]
