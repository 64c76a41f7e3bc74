"""Loading a model's tensors by name, and the random-weights mode.

Every tensor the model declares is looked up by its full name; its shape and dtype are checked
against the declaration; all problems of a folder (missing and unexpected tensors, wrong shapes,
dtypes without a kernel) are gathered into one error.  Tensors reach the parts as stored: bfloat16
as bfloat16, float32 as float32, integer tables as int32.  What a part then keeps is its own matter: norm
weights stay as stored on every path; the bfloat16 path rounds a matrix stored in float32 to bfloat16 once,
when it is put into the layout its kernels read, unless the run keeps stored dtypes (Precision.keep_stored).
The reference
derives shapes from its configuration and trusts them (llama3.rs:18226-18240) and reports a
missing tensor by returning None (llama3.rs:12887-12906); its newer loaders name the tensor
(llama3.rs:1137-1175), which is the behaviour kept here.
"""
from __future__ import annotations

import json
import os
import warnings
from typing import Callable, Dict, Iterable, Iterator, List, Optional, Tuple

import torch

from ..config import config_from_dict, load_config
from ..parts import ParamSpec, Precision
from .safetensors_io import TensorSource, WeightFileError, write_safetensors


class WeightError(ValueError):
    """The tensors of a model folder do not match what the model declares."""

    def __init__(self, where: str, missing: List[str], unexpected: List[str], wrong: List[str]):
        self.missing, self.unexpected, self.wrong = missing, unexpected, wrong
        lines = [f"{where}: the tensors do not match the model"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape or dtype ({len(wrong)}): " + "; ".join(wrong))
        super().__init__("\n".join(lines))


_FLOAT_OK = (torch.float32, torch.bfloat16)
_INT_OK = (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8)


class UnexpectedTensorsWarning(UserWarning):
    """A model folder holds tensors that the model does not declare; they were left unread (strict=False)."""


def check_tensors(where: str, specs: Dict[str, ParamSpec], found: Dict[str, Tuple[torch.dtype, Tuple[int, ...]]],
                  strict: bool = True) -> List[str]:
    """Raises one WeightError that lists every problem.  Tensors that the model does not declare are a problem
    when `strict`; otherwise they are returned (and listed in the error only if there is another problem)."""
    missing = [n for n in specs if n not in found]
    unexpected = sorted(n for n in found if n not in specs)
    wrong = []
    for n, spec in specs.items():
        if n not in found:
            continue
        dt, shape = found[n]
        if tuple(shape) != tuple(spec.shape):
            wrong.append(f"{n}: expected shape {list(spec.shape)}, found {list(shape)}")
        elif spec.integer and dt not in _INT_OK:
            wrong.append(f"{n}: expected an integer table, found {dt}")
        elif not spec.integer and dt not in _FLOAT_OK:
            wrong.append(f"{n}: dtype {dt} has no kernel (float32 and bfloat16 only)")
    if missing or wrong or (unexpected and strict):
        raise WeightError(where, missing, unexpected, wrong)
    return unexpected


def _place(model, name: str, spec: ParamSpec, t: torch.Tensor) -> None:
    if spec.integer:
        t = t.to(torch.int32)
    model.assign(name, t.to(model.device, non_blocking=False))


def load_weights(model, folder: str, strict: bool = True) -> List[str]:
    """Fill the model from a folder.  strict: tensors that the model does not declare are an error (listed with
    the missing and the misshapen ones); otherwise they stay unread, are named in one UnexpectedTensorsWarning
    and returned."""
    src = TensorSource(folder)
    try:
        specs = model.param_specs()
        unexpected = check_tensors(folder, specs, {k: src.info(k) for k in src.keys()}, strict)
        if unexpected:
            warnings.warn(f"{folder}: {len(unexpected)} tensors that the model does not declare were left unread: "
                          + ", ".join(unexpected), UnexpectedTensorsWarning, stacklevel=2)
        for name, spec in specs.items():
            _place(model, name, spec, src.tensor(name))
        model.finalize()
        return unexpected
    finally:
        src.close()


# --------------------------------------------------------------------------- random weights

def random_tensors(specs: Dict[str, ParamSpec], seed: int, dtype: torch.dtype, device="cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    """Tensors in the order of `specs` from one generator seeded with `seed`: N(0, init_std) drawn in
    float32 (on the host unless a device is given, whose generator draws other values), then cast to
    `dtype`; integer tables are zeros."""
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    for name, spec in specs.items():
        if spec.integer:
            yield name, torch.zeros(spec.shape, dtype=torch.int32, device=device)
        else:
            t = torch.empty(spec.shape, dtype=torch.float32, device=device)
            t.normal_(0.0, spec.init_std, generator=gen)
            yield name, t.to(dtype)


def init_random(model, seed: int, dtype: Optional[torch.dtype] = None, on_device: bool = False) -> None:
    """Fill the model with the tensors that `write_random_model` would write for the same seed
    (on_device: drawn by the GPU's generator instead, for large models where only the distribution matters)."""
    dtype = dtype or torch.bfloat16
    specs = model.param_specs()
    for name, t in random_tensors(specs, seed, dtype, model.device if on_device else "cpu"):
        _place(model, name, specs[name], t)
    model.finalize()


def write_random_model(folder: str, config, seed: int, dtype: Optional[torch.dtype] = None) -> None:
    """Write config.json and model.safetensors for a configuration (an object with to_dict/plan, or a
    parsed config.json) and a seed.  The stored dtype is the configuration's torch_dtype unless given."""
    from ..engine.model import CausalLM
    if isinstance(config, dict):
        raw = dict(config)
        config = config_from_dict(raw)
    else:
        raw = config.to_dict()
    if dtype is None:
        dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[raw.get("torch_dtype", "bfloat16")]
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    specs = _specs_without_device(config)
    it = random_tensors(specs, seed, dtype)

    def produce(name: str) -> torch.Tensor:
        n, t = next(it)
        assert n == name
        return t

    write_safetensors(os.path.join(folder, "model.safetensors"),
                      [(n, torch.int32 if s.integer else dtype, s.shape) for n, s in specs.items()], produce,
                      metadata={"format": "pt", "seed": str(seed)})


def _specs_without_device(config) -> Dict[str, ParamSpec]:
    """The model's declared tensors, from a skeleton built on the CPU (no kernels run, no GPU needed)."""
    from ..engine.model import CausalLM
    return CausalLM(config.plan(), Precision.of("float32"), "cpu").param_specs()
