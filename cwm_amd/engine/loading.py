"""From a model folder (or a configuration and a seed) to a model with its weights
on the device."""

from __future__ import annotations

import os
from typing import Any, Mapping, Optional, Tuple, Union

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


# share of the device's memory that the weights may take with their streaming copies
STREAM_COPY_SHARE = 0.5


def wants_stream_copies(model: Model, act_dtype: torch.dtype, device: torch.device, choice: Optional[bool] = None) -> bool:
    """Whether the model's matrices also keep the copy laid out for the weight-streaming product (see
    `Runtime.stream_copies`).  `choice` decides if given, else CWM_AMD_STREAM_COPIES (0 or 1) in the
    environment; else they are kept where the matrices, twice, take at most half of the device's memory (the
    rest is the cache's): a 32B model on 288 GB keeps them, a 70B model does not."""
    if act_dtype != torch.bfloat16 or device.type != "cuda":
        return False
    if choice is None and os.environ.get("CWM_AMD_STREAM_COPIES", "") != "":
        choice = os.environ["CWM_AMD_STREAM_COPIES"] not in ("0", "false", "no")
    if choice is not None:
        return choice
    matrix_bytes = 0
    for spec in model.tensor_specs().values():
        if len(spec.shape) == 2 and spec.kind == "float":
            matrix_bytes += 2 * spec.shape[0] * spec.shape[1]
    total = torch.cuda.get_device_properties(device).total_memory
    return 2 * matrix_bytes <= STREAM_COPY_SHARE * total


def load_model(
    folder: str, dtype: Union[str, torch.dtype], device: Union[str, torch.device], keep_float32: bool = False,
    stream_copies: Optional[bool] = None,
) -> Tuple[Model, Any]:
    """The model that `folder/config.json` names, with the folder's tensors.  In bfloat16 mode
    matrices stored in 32 bits are cast to bfloat16 unless `keep_float32`.  `stream_copies`: see
    `wants_stream_copies` (None: by the memory there is)."""
    device = torch.device(device)
    act_dtype = parse_dtype(dtype)
    arch, config = load_config(folder)
    model = Model(arch.build_plan(config))
    tensors = load_tensors(folder, model.tensor_specs(), act_dtype, device, keep_float32)
    model.bind(tensors, Runtime(device=device, act_dtype=act_dtype, stream_copies=wants_stream_copies(model, act_dtype, device, stream_copies)))
    return model, config


def random_model(
    config: Mapping[str, Any],
    seed: int,
    dtype: Union[str, torch.dtype],
    device: Union[str, torch.device],
    std: float = 0.02,
    norm_init: str = "ones",
    stream_copies: Optional[bool] = None,
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
    model.bind(tensors, Runtime(device=device, act_dtype=act_dtype, stream_copies=wants_stream_copies(model, act_dtype, device, stream_copies)))
    return model, typed
