"""Reads a model folder's safetensors by tensor name.

The reference loads a PyTorch distributed checkpoint non-strictly, so missing and
unexpected tensors pass silently (cwm/checkpoint/stateful_utils.py:32-38;
cwm/fastgen/utils/loading.py:57-60), and casts every parameter to bfloat16
(cwm/model/parallelize_transformer.py:50-59).  This loader is strict: one error
lists every missing tensor, every unexpected one and every wrong shape.

Storage types after loading:
  activation type bfloat16: tensors stored in 16 bits become bfloat16; a tensor stored
    in 32 (or 64) bits becomes bfloat16 too if its spec has precision "activation"
    (the matrices: the reference casts every parameter,
    cwm/model/parallelize_transformer.py:50-59, and the bfloat16 kernels need them so)
    and stays float32 if its spec says "stored" (norm weights) or the caller asks to
    keep 32-bit tensors as they are; integer tables become int32;
  activation type float32: every floating tensor becomes float32.
"""

from __future__ import annotations

import glob
import os
from typing import Dict, List, Mapping

import torch

from ..parts.base import TensorSpec


class WeightError(ValueError):
    """The tensors of a model folder do not fit the model."""


_FLOAT_16 = {"BF16", "F16"}
_FLOAT_WIDE = {"F32", "F64"}
_INTS = {"I8", "U8", "I16", "U16", "I32", "U32", "I64", "U64", "BOOL"}


def weight_files(folder: str) -> List[str]:
    files = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
    if not files:
        raise WeightError(f"{folder} holds no .safetensors file")
    return files


def target_dtype(
    stored: str, kind: str, act_dtype: torch.dtype, name: str, precision: str = "activation", keep_float32: bool = False
) -> torch.dtype:
    """Type a tensor is kept in, from how it is stored and what its spec asks."""
    if kind == "int":
        if stored not in _INTS:
            raise WeightError(f"{name}: an integer table is stored as {stored}")
        return torch.int32
    if stored in _FLOAT_WIDE:
        if act_dtype == torch.bfloat16 and precision == "activation" and not keep_float32:
            return torch.bfloat16
        return torch.float32
    if stored in _FLOAT_16:
        return torch.float32 if act_dtype == torch.float32 else torch.bfloat16
    raise WeightError(f"{name}: stored type {stored} is not supported (bfloat16, float16, float32, float64)")


def load_tensors(
    folder: str,
    specs: Mapping[str, TensorSpec],
    act_dtype: torch.dtype,
    device: torch.device,
    keep_float32: bool = False,
) -> Dict[str, torch.Tensor]:
    """All tensors that `specs` names, checked and moved to `device`.  `keep_float32`: in
    bfloat16 mode, tensors stored in 32 bits all stay float32 (their products then run on the
    float32 kernel)."""
    from safetensors import safe_open

    where: Dict[str, str] = {}
    shapes: Dict[str, tuple] = {}
    stored: Dict[str, str] = {}
    duplicates: List[str] = []
    for path in weight_files(folder):
        with safe_open(path, framework="pt", device="cpu") as fh:
            for name in fh.keys():
                if name in where:
                    duplicates.append(name)
                    continue
                where[name] = path
                sl = fh.get_slice(name)
                shapes[name] = tuple(sl.get_shape())
                stored[name] = str(sl.get_dtype())

    missing = sorted(set(specs) - set(where))
    unexpected = sorted(set(where) - set(specs))
    wrong = [
        f"{name}: expected {tuple(specs[name].shape)}, found {shapes[name]}"
        for name in sorted(set(specs) & set(where))
        if tuple(specs[name].shape) != shapes[name]
    ]
    if missing or unexpected or wrong or duplicates:
        lines = [f"the tensors in {folder} do not fit the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape ({len(wrong)}): " + "; ".join(wrong))
        if duplicates:
            lines.append(f"  stored in more than one file ({len(duplicates)}): " + ", ".join(sorted(duplicates)))
        raise WeightError("\n".join(lines))

    out: Dict[str, torch.Tensor] = {}
    by_file: Dict[str, List[str]] = {}
    for name, path in where.items():
        by_file.setdefault(path, []).append(name)
    for path, names in by_file.items():
        with safe_open(path, framework="pt", device="cpu") as fh:
            for name in names:
                dtype = target_dtype(stored[name], specs[name].kind, act_dtype, name, specs[name].precision, keep_float32)
                out[name] = fh.get_tensor(name).to(device=device, dtype=dtype).contiguous()
    return out
