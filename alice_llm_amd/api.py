"""The Python entry point: load a model folder (or build random weights from a configuration),
make an engine over a cache, step it, generate from it.

The reference's surface this corresponds to is Llama3Model::{from_gguf, forward, generate, reset}
(llama3.rs:12886, 13496, 16042, 13488) and the sampling functions (src/sampling.rs:10-123).
"""
from __future__ import annotations

import os
from typing import List, Optional, Sequence, Union

import torch

from .config import config_from_dict, load_config
from .engine.model import CausalLM
from .engine.step import Engine
from .cache import PAGE_SIZE
from .engine.generate import MAX_STEP_TOKENS, GenerationResult, Generator
from .hip import ops
from .parts import Precision
from .weights.loader import init_random, load_weights


class Model:
    def __init__(self, config, lm: CausalLM):
        self.config = config
        self.lm = lm
        self.precision = lm.precision
        self.device = lm.device
        self._kept_engine: Optional[Engine] = None

    # ------------------------------------------------------------------ construction
    @classmethod
    def load(cls, folder: str, dtype=None, device: Union[str, torch.device, None] = None, strict: bool = True,
             keep_stored_dtype: bool = False) -> "Model":
        """A folder with config.json and model.safetensors; the model class is chosen by config.json.
        strict=False: tensors in the folder that the model does not declare are warned about, not an error.
        keep_stored_dtype: on the bfloat16 path, matrices that the folder stores in 32-bit stay 32-bit (and run
        on the plain kernel) instead of being rounded to bfloat16 once at load."""
        config = load_config(folder)
        device = torch.device(device) if device is not None else ops.require_gpu()
        precision = Precision.of(dtype or getattr(config, "torch_dtype", "bfloat16"), keep_stored_dtype)
        lm = CausalLM(config.plan(), precision, device)
        load_weights(lm, folder, strict)
        return cls(config, lm)

    @classmethod
    def random(cls, config, seed: int = 0, dtype=None, device=None, stored_dtype: Optional[torch.dtype] = None,
               fast: bool = False, keep_stored_dtype: bool = False) -> "Model":
        """Random weights straight onto the device: the same tensors write_random_model(config, seed) writes
        (with fast=True they are drawn on the GPU instead: same distribution, other values)."""
        if isinstance(config, dict):
            config = config_from_dict(config)
        device = torch.device(device) if device is not None else ops.require_gpu()
        precision = Precision.of(dtype or getattr(config, "torch_dtype", "bfloat16"), keep_stored_dtype)
        lm = CausalLM(config.plan(), precision, device)
        if stored_dtype is None:
            stored_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[getattr(config, "torch_dtype", "bfloat16")]
        init_random(lm, seed, stored_dtype, on_device=fast)
        return cls(config, lm)

    # ------------------------------------------------------------------ use
    def engine(self, max_tokens: Optional[int] = None, max_seqs: Optional[int] = None,
               use_graphs: Optional[bool] = None, *, seq_lens: Optional[Sequence[int]] = None, **kw) -> Engine:
        """A cache and the step function over it.  The cache is sized for max_tokens (each live sequence's count
        rounded up to whole pages) or for sequences of the lengths `seq_lens` held together.  use_graphs: record
        decode steps into HIP graphs (default: whenever every part of the model allows it)."""
        return Engine(self.lm, max_tokens=max_tokens, seq_lens=seq_lens, max_seqs=max_seqs, use_graphs=use_graphs, **kw)

    new_cache = engine

    def step(self, engine: Engine, slots: Sequence[int], new_tokens: Sequence[Sequence[int]], want="last") -> torch.Tensor:
        """One step of `engine` (made by this model's engine()): new_tokens[i] for the sequence in slots[i]; float32
        logits at the wanted places.  The same as engine.step; the reference's Llama3Model::forward (llama3.rs:13496)."""
        if engine.model is not self.lm:
            raise ValueError("this engine belongs to another model")
        return engine.step(slots, new_tokens, want)

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: Union[int, Sequence[int]] = 256,
                 temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, seed: int = 0,
                 stop_token_ids: Optional[Sequence[int]] = None, max_batch: Optional[int] = None,
                 max_tokens: Optional[int] = None, engine: Optional[Engine] = None,
                 observer=None, max_step_tokens: Optional[int] = MAX_STEP_TOKENS) -> List[GenerationResult]:
        """Generate for every prompt (token ids); as many batches one after another as needed.  A request whose
        prompt and cap together outgrow the model's positions ends at the last position with finish_reason
        "length".  observer, max_step_tokens: see Generator.

        Without `engine` the model keeps the engine it made for the last call (cache, captured steps) and uses it
        again whenever the new call fits into it: as many sequences at once and as many tokens; otherwise it
        makes a larger one.  `release_engine()` gives its memory back."""
        if prompts and isinstance(prompts[0], int):
            prompts = [prompts]
        caps = [max_new_tokens] * len(prompts) if isinstance(max_new_tokens, int) else list(max_new_tokens)
        if engine is None:
            batch = max_batch or len(prompts)
            most = self.lm.plan.max_positions
            longest = sorted((min(len(p) + max(c - 1, 0), most) for p, c in zip(prompts, caps)), reverse=True)[:batch]
            engine = self._engine_for(max_tokens, longest, batch)
        if stop_token_ids is None:
            stop_token_ids = self.lm.plan.stop_token_ids
        gen = Generator(engine, temperature=temperature, top_k=top_k, top_p=top_p, seed=seed,
                        stop_token_ids=stop_token_ids, max_batch=max_batch, observer=observer,
                        max_step_tokens=max_step_tokens)
        return gen.run(prompts, caps)

    def _engine_for(self, max_tokens: Optional[int], seq_lens: Sequence[int], max_seqs: int) -> Engine:
        """The engine kept from an earlier generate() if this call fits into it, else a new one (which is kept)."""
        page = PAGE_SIZE
        need = max_tokens or sum(-(-int(n) // page) * page for n in seq_lens)
        kept = self._kept_engine
        if (kept is not None and kept.cache.page_size == page and kept.cache.max_tokens >= need
                and kept.cache.slots.n_slots >= max_seqs and kept.cache.slots.n_free() == kept.cache.slots.n_slots):
            return kept
        self._kept_engine = None                                  # free the old cache before the new one is made
        del kept
        self._kept_engine = self.engine(max_tokens=need, max_seqs=max_seqs)
        return self._kept_engine

    def release_engine(self) -> None:
        """Drop the engine that generate() keeps between calls (its cache and captured steps)."""
        self._kept_engine = None


def sample(logits: torch.Tensor, temperature: float = 0.0, top_k: int = 0, top_p: float = 1.0, u=None) -> torch.Tensor:
    """One token id per row of float32 logits [rows, vocab] (or one row [vocab]) on the GPU, as int32 [rows]:
    temperature, then top-k, then top-p, then softmax, then the inverse CDF at u[row] in [0, 1)
    (src/sampling.rs:10-123; the order of examples/generate_gpu.rs:125-128).  A temperature below 1e-6 is greedy,
    the lowest index among equal maxima, and needs no u."""
    from .sampling import GREEDY_BELOW
    if logits.dim() == 1:
        logits = logits[None]
    logits = logits.contiguous()
    if temperature < GREEDY_BELOW:
        return ops.argmax(logits)
    if u is None:
        raise ValueError("sampling at a temperature needs u: one uniform number in [0, 1) per row")
    u = torch.as_tensor(u, dtype=torch.float32).reshape(-1).to(logits.device)
    if u.numel() != logits.shape[0] or bool(((u < 0) | (u >= 1)).any()):
        raise ValueError("u must hold one number in [0, 1) per row of logits")
    if top_k < 0 or not top_p > 0:
        raise ValueError("top_k must not be negative and top_p must be positive")
    return ops.sample(logits, u, float(temperature), int(top_k), float(top_p))


def load(path_or_config, dtype=None, random_seed: Optional[int] = None, device=None, strict: bool = True,
         keep_stored_dtype: bool = False) -> Model:
    """load("folder") reads a model folder; load(config_dict_or_object, random_seed=0) makes random weights.
    keep_stored_dtype: see Model.load."""
    if isinstance(path_or_config, (str, os.PathLike)):
        return Model.load(os.fspath(path_or_config), dtype, device, strict, keep_stored_dtype)
    return Model.random(path_or_config, random_seed or 0, dtype, device, keep_stored_dtype=keep_stored_dtype)
