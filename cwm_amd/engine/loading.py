"""From a model folder (or a configuration and a seed) to a model with its weights
on the device."""

from __future__ import annotations

from typing import Any, Mapping, Tuple, Union

import torch

from ..config.registry import load_config, parse_config
from ..models.model import Model
from ..parts.base import Runtime
from ..weights.loader import load_tensors
from ..weights.random_init import random_tensor

_DTYPES = {
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
    "float32": torch.float32,
    "fp32": torch.float32,
}


def parse_dtype(dtype: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"the engine runs in bfloat16 or float32, not {dtype}")
        return dtype
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be one of {', '.join(_DTYPES)}, found {dtype!r}") from None


def load_model(
    folder: str, dtype: Union[str, torch.dtype], device: Union[str, torch.device], keep_float32: bool = False
) -> Tuple[Model, Any]:
    """The model that `folder/config.json` names, with the folder's tensors.  In bfloat16 mode
    matrices stored in 32 bits are cast to bfloat16 unless `keep_float32`."""
    device = torch.device(device)
    act_dtype = parse_dtype(dtype)
    arch, config = load_config(folder)
    model = Model(arch.build_plan(config))
    tensors = load_tensors(folder, model.tensor_specs(), act_dtype, device, keep_float32)
    model.bind(tensors, Runtime(device=device, act_dtype=act_dtype))
    return model, config


def random_model(
    config: Mapping[str, Any],
    seed: int,
    dtype: Union[str, torch.dtype],
    device: Union[str, torch.device],
    std: float = 0.02,
    norm_init: str = "ones",
) -> Tuple[Model, Any]:
    """A model with random weights drawn on the device, without a folder in between
    (for shapes whose weights would not pass through host memory quickly)."""
    device = torch.device(device)
    act_dtype = parse_dtype(dtype)
    arch, typed = parse_config(config)
    model = Model(arch.build_plan(typed))
    tensors = {
        name: random_tensor(name, spec, seed, std, norm_init, act_dtype, device)
        for name, spec in model.tensor_specs().items()
    }
    model.bind(tensors, Runtime(device=device, act_dtype=act_dtype))
    return model, typed
