"""Engine-side option structs, with the reference's field names and meanings.

SamplingParams: src/engine.h:26-31.  EngineConfig: src/engine.h:38-50, less the fields of
speculative decoding, static batching and kernel-mode comparison, plus the choices the
reference fixes at compile time (block_size, src/block_manager.h:20) or does not have
(dtype, max_model_len).
"""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 0.0   # <= 0 means greedy (src/engine.cpp:469)
    seed: int = 0              # key of the counter-based generator
    max_new_tokens: int = 32
    ignore_eos: bool = False


class Fault:
    """Bugs the simulator must catch, switched on by ``EngineConfig.fault`` (src/engine.h:52-62: each a slip of one
    line that an implementation could plausibly make; 3 belongs to speculative decoding, which is not here)."""
    NONE = 0
    PREFIX_COVERS_LAST_TOKEN = 1     # a prefix hit may take the page that holds the request's last known token
    RNG_KEYED_BY_STEP = 2            # a draw is keyed by the engine's step instead of the request's position
    REGISTER_UNFINISHED_PAGE = 4     # a page enters the prefix cache while a portion of its prompt is still to come
    CANCEL_KEEPS_PAGES = 5           # a cancelled request's pages are not given back
    NAMES = {1: "prefix hit covers the last token", 2: "randomness keyed by the engine's step",
             4: "page registered before it is full", 5: "cancel keeps the pages"}


@dataclass
class EngineConfig:
    num_blocks: int = 512            # pages in every cache group's pool
    max_batched_tokens: int = 256    # token budget of one step
    max_num_seqs: int = 32           # running requests at a time
    prefix_caching: bool = True
    fingerprint_logits: bool = True
    block_size: int = 16             # tokens in a page
    dtype: str = "bfloat16"          # "bfloat16" (serving precision) or "float32" (true 32-bit)
    max_model_len: int = 0           # 0: the model's max_position_embeddings
    use_graphs: bool = True          # replay pure-decode steps from captured HIP graphs
    run_ahead: bool = True           # launch the next pure-decode step before the last one's tokens are read back
    decode_phases: bool = False      # captured decode steps of up to 16 rows run their products as phases of a few
                                     # launches that wait for each other inside the kernel (ops.chain): the same
                                     # bits; on MI355X some 5 % slower than a launch each, so off
    portion_align: int = 64          # a prompt portion that ends before its prompt does ends at a multiple of this many
                                     # tokens where the budget allows (whole pages and whole 64-key partitions: the
                                     # kernels' rows of 16 then never straddle a page); 1: cut exactly at the budget
    fault: int = 0                   # a test-only bug (``Fault``) for the simulator to catch; 0: none

    def validate(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {self.dtype!r}")
        if self.block_size < 1 or self.block_size & (self.block_size - 1):
            raise ValueError(f"block_size must be a power of two, got {self.block_size}")   # (which ones a model takes: its mixers say)
        if self.num_blocks < 1 or self.max_batched_tokens < 1 or self.max_num_seqs < 1:
            raise ValueError("num_blocks, max_batched_tokens and max_num_seqs must be positive")
        if self.portion_align < 1:
            raise ValueError(f"portion_align must be at least 1, got {self.portion_align}")
        if self.fault and self.fault not in Fault.NAMES:
            raise ValueError(f"fault must be 0 or one of {sorted(Fault.NAMES)}, got {self.fault}")
