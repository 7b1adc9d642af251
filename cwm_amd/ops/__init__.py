"""Python entry points of the hand-written gfx950 kernels.

Every function checks shapes, types and devices on the host, then launches on
torch's current HIP stream through the C entry points of `cwm_amd/csrc`.  There is
no CPU path and no library substitute: tensors that are not on a HIP device, or a
missing kernel library, raise an error.

The only library routine on the model's path is the bfloat16 matrix product for
more rows than the hand-written kernels take (`torch.mm`, i.e. hipBLASLt), where
the reference also calls a library
(cwm/fastgen/forward.py:593-606).
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np
import torch

from . import build as _build
from .attention_plan import WIDE_TILES
from .build import KernelBuildError

F32, BF16 = 0, 1


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments."""


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 and bfloat16 tensors, not {dtype}")


def _need_gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError(
                "cwm_amd kernels run on a HIP device only; got a tensor on "
                f"{t.device}. There is no CPU path."
            )


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream() -> ctypes.c_void_p:
    """The current HIP stream of the current device (the raw handle; building a torch
    Stream object for every launch costs several microseconds)."""
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _check(lib: ctypes.CDLL, status: int) -> None:
    if status != 0:
        raise KernelError(lib.cwm_error_message().decode("utf-8", "replace"))


def _rows_contiguous(t: torch.Tensor, what: str) -> None:
    if t.dim() < 1 or t.stride(-1) != 1:
        raise KernelError(f"{what}: innermost dimension must be contiguous, strides are {t.stride()}")


def _i32(t: torch.Tensor, what: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what} must be a contiguous int32 tensor, found {t.dtype} with strides {t.stride()}")


# --------------------------------------------------------------------------- #
def embedding(tokens: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 [T, D]: `scale` times the rows of `table` ([V, D], float32 or bfloat16) for int32 `tokens` [T]."""
    _need_gpu(tokens, table)
    _i32(tokens, "tokens")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous [V, D] tensor")
    lib = _build.load("rowwise")
    out = torch.empty((tokens.numel(), table.shape[1]), dtype=torch.float32, device=table.device)
    _check(
        lib,
        lib.cwm_embedding(
            _ptr(out), _ptr(table), _code(table.dtype), _ptr(tokens),
            ctypes.c_int(tokens.numel()), ctypes.c_int(table.shape[1]), ctypes.c_int(table.shape[0]), ctypes.c_float(scale), _stream(),
        ),
    )
    return out


def add_rmsnorm(
    h: torch.Tensor,
    delta: Optional[torch.Tensor],
    weight: torch.Tensor,
    eps: float,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """`h` (float32 [T, D]) += `delta` in place, then RMSNorm(h) * weight.

    `delta` is [T, D], or float32 partial sums [P, T, D] (a matrix product whose K
    was split) that are added in order.  With `rows` (int32 [R]) only those rows are
    normalised and `h` is not changed (the sum with `delta` is still what is
    normalised).
    """
    _need_gpu(h, delta, weight, rows)
    if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
        raise KernelError("the residual stream must be a contiguous float32 [T, D] tensor")
    n_tokens, dim = h.shape
    n_partials = 1
    if delta is not None:
        if delta.dim() == 3:
            if delta.dtype != torch.float32:
                raise KernelError("partial sums must be float32")
            n_partials = delta.shape[0]
        if tuple(delta.shape[-2:]) != tuple(h.shape) or not delta.is_contiguous():
            raise KernelError(f"delta {tuple(delta.shape)} does not match the residual stream {tuple(h.shape)}")
    if weight.shape != (dim,) or not weight.is_contiguous():
        raise KernelError(f"norm weight has shape {tuple(weight.shape)}, expected ({dim},)")
    if rows is not None:
        _i32(rows, "rows")
    n_out = n_tokens if rows is None else rows.numel()
    out = torch.empty((n_out, dim), dtype=out_dtype, device=h.device)
    lib = _build.load("rowwise")
    _check(
        lib,
        lib.cwm_add_rmsnorm(
            _ptr(h), _ptr(delta), ctypes.c_int(_code(delta.dtype) if delta is not None else F32),
            ctypes.c_int(n_partials), ctypes.c_long(n_tokens * dim), _ptr(weight), ctypes.c_int(_code(weight.dtype)), _ptr(out), ctypes.c_int(_code(out_dtype)),
            _ptr(rows), ctypes.c_int(n_out), ctypes.c_int(dim), ctypes.c_float(eps), _stream(),
        ),
    )
    return out


def silu_mul(gate_up: torch.Tensor, out_dtype: Optional[torch.dtype] = None, grouped: bool = False) -> torch.Tensor:
    """[T, 2F] -> [T, F]: silu(gate) * up, computed in float32; gate is the first half
    of a row and up the second, or, with `grouped`, they alternate in groups of 8
    columns (the order in which a product with row-interleaved gate/up weights
    delivers them).  Float32 partial sums [P, T, 2F] of a product with a split K are
    taken too: they are added in order, rounded to `out_dtype` as the product would
    have stored them, and then treated alike."""
    _need_gpu(gate_up)
    if grouped and (gate_up.shape[-1] // 2) % 8 != 0:
        raise KernelError("gate and up in groups of 8 need a width that is a multiple of 8")
    lib = _build.load("rowwise")
    if gate_up.dim() == 3:
        if gate_up.dtype != torch.float32 or gate_up.shape[2] % 2 != 0 or not gate_up.is_contiguous():
            raise KernelError("partial sums for silu_mul must be a contiguous float32 [P, T, 2F] tensor")
        n_part, n_tokens, two_f = gate_up.shape
        if (two_f // 2) % 4 != 0:
            return silu_mul(sum_partials(gate_up, out_dtype or torch.float32), grouped=grouped)
        out = torch.empty((n_tokens, two_f // 2), dtype=out_dtype or torch.float32, device=gate_up.device)
        _check(
            lib,
            lib.cwm_silu_mul_partials(
                _ptr(out), ctypes.c_int(_code(out.dtype)), _ptr(gate_up), ctypes.c_int(n_part),
                ctypes.c_int(n_tokens), ctypes.c_int(two_f // 2), ctypes.c_int(int(grouped)), _stream(),
            ),
        )
        return out
    if gate_up.dim() != 2 or gate_up.shape[1] % 2 != 0 or not gate_up.is_contiguous():
        raise KernelError("silu_mul takes a contiguous [T, 2F] tensor")
    n_tokens, two_f = gate_up.shape
    out = torch.empty((n_tokens, two_f // 2), dtype=gate_up.dtype, device=gate_up.device)
    _check(
        lib,
        lib.cwm_silu_mul(
            _ptr(out), _ptr(gate_up), ctypes.c_int(_code(gate_up.dtype)),
            ctypes.c_int(n_tokens), ctypes.c_int(two_f // 2), ctypes.c_int(int(grouped)), _stream(),
        ),
    )
    return out


def gate_up_silu(
    x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], grouped: bool, streamed: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) for the joined weight [2F, D] of a gated feed-forward
    (cwm/fastgen/forward.py:776-781): rows Wg then Wu, or, with `grouped`, alternating
    in groups of 8.  A grouped weight lets a decode batch in bfloat16 finish the
    activation in the product's epilogue; every other case runs the product and the
    activation kernel, with the same roundings."""
    n = weight.shape[0]
    fused = (
        grouped and n % 16 == 0
        and x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
        and x.shape[0] <= STREAM_EPILOGUE_ROWS and _stream_takes(x, weight)
        and x.shape[1] <= stream_unsplit_k(x.shape[0])  # K fits one group of wavefronts: no split
    )
    tiled = x.is_cuda and x.dim() == 2 and _prefers_tile(x, weight, bias, streamed)
    if fused and not tiled:
        return gemm_bf16_stream(x, weight, bias, torch.bfloat16, glu=True, streamed=streamed)
    if tiled and grouped and x.shape[0] <= TILE_ROWS:
        return gemm_bf16_tile(x, weight, None, torch.bfloat16, glu=True)
    return silu_mul(linear(x, weight, bias, partials_ok=True, streamed=streamed), out_dtype=x.dtype, grouped=grouped)


# --------------------------------------------------------------------------- #
def gemm_f32(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """x [M, K] @ weight[N, K]^T (+ bias) with float32 multiply-add (no matrix cores)."""
    _need_gpu(x, weight, bias)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm: x {tuple(x.shape)} and weight {tuple(weight.shape)} do not fit")
    _rows_contiguous(x, "gemm x")
    _rows_contiguous(weight, "gemm weight")
    m, k = x.shape
    n = weight.shape[0]
    if bias is not None and (bias.shape != (n,) or not bias.is_contiguous()):
        raise KernelError(f"gemm: bias {tuple(bias.shape)} does not fit {n} outputs")
    out_dtype = out_dtype or x.dtype
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    lib = _build.load("gemm_f32")
    _check(
        lib,
        lib.cwm_gemm_f32(
            _ptr(x), ctypes.c_int(_code(x.dtype)), ctypes.c_long(x.stride(0) if m > 1 else k),
            _ptr(weight), ctypes.c_int(_code(weight.dtype)), ctypes.c_long(weight.stride(0) if n > 1 else k),
            _ptr(out), ctypes.c_int(_code(out_dtype)), ctypes.c_long(n),
            _ptr(bias), ctypes.c_int(_code(bias.dtype) if bias is not None else F32),
            ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k), _stream(),
        ),
    )
    return out


F32_STREAM_MAX_ROWS = 16
_f32_stream_block_steps: Optional[int] = None


def _f32_stream_takes(x: torch.Tensor, weight: torch.Tensor) -> bool:
    return (
        x.dtype == torch.float32 and weight.dtype == torch.float32
        and x.dim() == 2 and weight.dim() == 2 and x.shape[0] <= F32_STREAM_MAX_ROWS
        and x.shape[1] % 4 == 0 and x.stride(-1) == 1 and weight.stride(-1) == 1
        and (x.shape[0] <= 1 or x.stride(0) % 4 == 0) and (weight.shape[0] <= 1 or weight.stride(0) % 4 == 0)
        and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
    )


def gemm_f32_stream(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
    partials_ok: bool = False,
) -> torch.Tensor:
    """float32 x [M <= 16, K] @ float32 weight[N, K]^T with float32 multiply-add, the weight
    streamed once by persistent blocks (the decode-step product of the 32-bit path).  Returns
    [M, N]; with `partials_ok` it may return float32 partial sums [P, M, N] of a split K."""
    global _f32_stream_block_steps
    _need_gpu(x, weight, bias)
    if not _f32_stream_takes(x, weight) or x.shape[1] != weight.shape[1]:
        raise KernelError(
            f"the float32 streaming product takes float32 x [M <= {F32_STREAM_MAX_ROWS}, K] and weight [N, K] with K a multiple "
            f"of 4 and 16-byte aligned rows; got {tuple(x.shape)} {x.dtype} and {tuple(weight.shape)} {weight.dtype}"
        )
    m, k = x.shape
    n = weight.shape[0]
    if bias is not None and (bias.shape != (n,) or not bias.is_contiguous()):
        raise KernelError(f"gemm: bias {tuple(bias.shape)} does not fit {n} outputs")
    out_dtype = out_dtype or torch.float32
    lib = _build.load("gemm_f32_stream")
    if _f32_stream_block_steps is None:
        _f32_stream_block_steps = int(lib.cwm_gemm_f32_stream_steps_per_block())
    steps = (k + 15) // 16
    n_tiles = (n + 15) // 16
    cus = _compute_units(x.device)
    k_split = -(-steps // _f32_stream_block_steps)  # K longer than one block's registers is split
    if partials_ok:
        while n_tiles * k_split < 2 * cus and k_split < 8 and steps >= 2 * k_split * 16:
            k_split *= 2  # too few tiles to fill the chip
    blocks = max(k_split, min(cus, n_tiles * k_split) // k_split * k_split)
    if k_split == 1:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    else:
        out = torch.empty((k_split, m, n), dtype=torch.float32, device=x.device)
    _check(
        lib,
        lib.cwm_gemm_f32_stream(
            _ptr(x), ctypes.c_long(x.stride(0) if m > 1 else k), _ptr(weight), ctypes.c_long(weight.stride(0) if n > 1 else k),
            _ptr(out), ctypes.c_int(_code(out.dtype)), ctypes.c_long(n), ctypes.c_long(m * n),
            _ptr(bias), ctypes.c_int(_code(bias.dtype) if bias is not None else F32),
            ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k), ctypes.c_int(k_split), ctypes.c_int(blocks), _stream(),
        ),
    )
    if k_split > 1 and not partials_ok:
        return sum_partials(out, out_dtype)
    return out


def linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
    partials_ok: bool = False,
    streamed: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """y = x W^T (+ b).  cwm/fastgen/forward.py:593-606.

    float32 activations or float32 weights: the float32 kernels (exact products; up to 16
    rows of float32 on the weight-streaming one, whose sums differ from the other's by rounding).
    bfloat16 activations and weights: matrix cores with float32 accumulation, the
    library product for many rows.  With `partials_ok` the result may be float32
    partial sums [P, M, N] that the caller adds (see `add_rmsnorm`).  `streamed`: the weight's
    streaming copy (`stream_layout`), which the products of few rows read instead where there is one.
    """
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32 or weight.dtype == torch.float32:
        if x.is_cuda and _f32_stream_takes(x, weight):
            return gemm_f32_stream(x, weight, bias, out_dtype, partials_ok)
        return gemm_f32(x, weight, bias, out_dtype)
    return gemm_bf16(x, weight, bias, out_dtype, partials_ok, streamed)


STREAM_MAX_ROWS = 64
_cu_count: dict = {}


_stream_shapes: dict = {}  # rows -> (wavefronts of a block, steps of K a wavefront holds)


def _compute_units(device: torch.device) -> int:
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _cu_count:
        _cu_count[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _cu_count[idx]


def _stream_block_shape(m: int) -> Tuple[int, int]:
    """(wavefronts of a block, steps of 32 along K that one wavefront keeps of x in registers) of the streaming
    product for `m` rows, asked of the library: the kernel's register budget is stated there and nowhere else."""
    shape = _stream_shapes.get(m)
    if shape is None:
        lib = _build.load("gemm_bf16_stream")
        shape = _stream_shapes[m] = (lib.cwm_gemm_bf16_stream_waves(ctypes.c_int(m)), lib.cwm_gemm_bf16_stream_steps_per_wave(ctypes.c_int(m)))
    return shape


def stream_unsplit_k(m: int) -> int:
    """The longest K that one group of wavefronts of the streaming product holds for `m` rows, so that K is not
    split over blocks: the fused epilogues (rotation + cache write, gated activation) need that."""
    waves, regs = _stream_block_shape(m)
    return 32 * waves * regs


def stream_layout(weight: torch.Tensor) -> torch.Tensor:
    """The streaming copy of a bfloat16 matrix W [N, K]: [tiles of 16 rows, steps of 32 columns, 64, 8], lane
    16 j + r of a step holding W[16 tile + r][32 step + 8 j ..+8] (one operand of the matrix instruction), zeros
    past N and K.  The streaming product reads it 1 KB a wavefront's load, every cache line once."""
    _need_gpu(weight)
    if weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.stride(1) != 1:
        raise KernelError("a streaming copy is made of a bfloat16 matrix with contiguous rows")
    n, k = weight.shape
    out = torch.empty((-(-n // 16), -(-k // 32), 64, 8), dtype=torch.bfloat16, device=weight.device)
    lib = _build.load("gemm_bf16_stream")
    _check(lib, lib.cwm_gemm_bf16_stream_copy(_ptr(weight), ctypes.c_long(weight.stride(0)), _ptr(out), ctypes.c_int(n), ctypes.c_int(k), _stream()))
    return out


def gemm_bf16_stream(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
    partials_ok: bool = False,
    rope: Optional[tuple] = None,
    glu: bool = False,
    streamed: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """bfloat16 x [M <= 64, K] @ weight[N, K]^T with persistent blocks that keep x in
    registers and stream the weight once.  `streamed` is the matrix's streaming copy
    (`stream_layout(weight)`); with it the kernel reads that copy, in whole cache lines and past the
    caches, instead of `weight`.  Returns [M, N]; with `partials_ok` it may
    return float32 partial sums [P, M, N] of a split K for the caller to add (the
    residual-add + RMSNorm kernel takes them).  `rope`
    (positions, seq_of_token, inv_freq, cache, block_table, n_q_heads, n_kv_heads,
    head_dim) makes the epilogue rotate the q and k columns and write k and v into the
    paged cache (see `qkv_rope_write`).  `glu`: the weight's rows are gate and up rows in
    alternating groups of 8 and the result is silu(gate) * up, [M, N / 2] (see
    `gate_up_silu`)."""
    _need_gpu(x, weight, bias)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise KernelError("the streaming product takes bfloat16 operands")
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm: x {tuple(x.shape)} and weight {tuple(weight.shape)} do not fit")
    m, k = x.shape[0], weight.shape[1]
    n = weight.shape[0]
    if m > STREAM_MAX_ROWS:
        raise KernelError(f"the streaming product takes at most {STREAM_MAX_ROWS} rows, not {m}")
    if bias is not None and (bias.shape != (n,) or not bias.is_contiguous()):
        raise KernelError(f"gemm: bias {tuple(bias.shape)} does not fit {n} outputs")
    out_dtype = out_dtype or torch.bfloat16
    lib = _build.load("gemm_bf16_stream")
    waves, regs = _stream_block_shape(m)
    steps = (k + 31) // 32
    n_tiles = (n + 15) // 16
    cus = _compute_units(x.device)
    k_split = -(-steps // (waves * regs))  # K longer than one group of wavefronts' registers is split
    if (rope is not None or glu) and (k_split != 1 or m > 16):
        raise KernelError("the fused epilogues need at most 16 rows and a K that one group of wavefronts holds")
    if glu:
        partials_ok = False
    if partials_ok:
        while n_tiles * k_split < 2 * cus and k_split < 8 and steps >= 2 * k_split * waves:
            k_split *= 2  # too few tiles to fill the chip
    blocks = max(k_split, min(cus, n_tiles * k_split) // k_split * k_split)
    if k_split == 1:
        out = torch.empty((m, n // 2 if glu else n), dtype=out_dtype, device=x.device)
    else:
        out = torch.empty((k_split, m, n), dtype=torch.float32, device=x.device)
    if streamed is not None:
        if streamed.shape != (n_tiles, steps, 64, 8) or streamed.dtype != torch.bfloat16 or not streamed.is_contiguous() or streamed.device != x.device:
            raise KernelError(f"the streaming copy of a [{n}, {k}] matrix is bfloat16 [{n_tiles}, {steps}, 64, 8], not {tuple(streamed.shape)}")
        w_ptr, w_stride = _ptr(streamed), ctypes.c_long(steps * 512)
    else:
        w_ptr, w_stride = _ptr(weight), ctypes.c_long(weight.stride(0) if n > 1 else k)
    _check(
        lib,
        lib.cwm_gemm_bf16_stream(
            _ptr(x), ctypes.c_long(x.stride(0) if m > 1 else x.shape[1]), w_ptr, w_stride,
            _ptr(out), ctypes.c_int(_code(out.dtype)), ctypes.c_long(out.shape[-1]), ctypes.c_long(m * n),
            _ptr(bias), ctypes.c_int(_code(bias.dtype) if bias is not None else F32),
            ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k), ctypes.c_int(k_split), ctypes.c_int(blocks),
            *_rope_args(rope), ctypes.c_int(int(glu)), ctypes.c_int(int(streamed is not None)), _stream(),
        ),
    )
    if k_split > 1 and not partials_ok:
        return sum_partials(out, out_dtype)
    return out


_NO_ROPE_ARGS = [ctypes.c_void_p(0)] * 5 + [ctypes.c_int(0)] * 6


def _rope_args(rope: Optional[tuple]) -> list:
    if rope is None:
        return _NO_ROPE_ARGS
    positions, seq_of_token, inv_freq, cache, block_table, n_q, n_kv, hd = rope
    return [
        _ptr(positions), _ptr(seq_of_token), _ptr(inv_freq), _ptr(cache), _ptr(block_table),
        ctypes.c_int(block_table.shape[1]), ctypes.c_int(cache.shape[3] // hd), ctypes.c_int(cache.shape[0]),
        ctypes.c_int(n_q), ctypes.c_int(n_kv), ctypes.c_int(hd),
    ]


def qkv_rope_write(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    positions: torch.Tensor,
    inv_freq: Optional[torch.Tensor],
    cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_of_token: torch.Tensor,
    streamed: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """The joined q/k/v projection of x [T, D] (weight [(Hq + 2 Hkv) * hd, D]), the
    rotation of its q and k columns by each token's position, and the write of the
    rotated keys and of the values into the paged cache
    (cwm/fastgen/forward.py:593-632).  Returns [T, (Hq + 2 Hkv) * hd] with q rotated.
    Decode batches in bfloat16 do all three in the streaming product's epilogue; any
    other case runs the product and then the rotation + cache-write kernel, with the
    same arithmetic."""
    n_out = (n_q_heads + 2 * n_kv_heads) * head_dim
    if weight.shape[0] != n_out:
        raise KernelError(f"q/k/v weight has {weight.shape[0]} rows, expected {n_out}")
    fused = (
        x.is_cuda
        and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16
        and x.shape[0] <= STREAM_EPILOGUE_ROWS
        and head_dim <= 256
        and _stream_takes(x, weight)
        and x.shape[1] <= stream_unsplit_k(x.shape[0])  # K fits one group of wavefronts: no split
        and not _prefers_tile(x, weight, bias, streamed)
    )
    if fused:
        _i32(positions, "positions")
        _i32(seq_of_token, "seq_of_token")
        _i32(block_table, "block_table")
        if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2 or not inv_freq.is_contiguous()):
            raise KernelError(f"the rotary table must be float32 [{head_dim // 2}]")
        if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[2] != n_kv_heads or cache.shape[3] % head_dim != 0 or not cache.is_contiguous():
            raise KernelError(f"cache {tuple(cache.shape)} does not fit {n_kv_heads} heads of size {head_dim}")
        if positions.numel() != x.shape[0] or seq_of_token.numel() != x.shape[0] or block_table.dim() != 2:
            raise KernelError("positions and seq_of_token must be [T], block_table [B, W]")
        return gemm_bf16_stream(
            x, weight, bias, torch.bfloat16,
            rope=(positions, seq_of_token, inv_freq, cache, block_table, n_q_heads, n_kv_heads, head_dim), streamed=streamed,
        )
    qkv = linear(x, weight, bias, partials_ok=True, streamed=streamed)
    if qkv.dim() == 3:
        # partial sums of a split K: added by the rotation kernel where it can, else by a kernel of their own
        if x.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16 and head_dim % 8 == 0 and head_dim <= 256:
            return rope_kv_write_partials(qkv, n_q_heads, n_kv_heads, head_dim, positions, inv_freq, cache, block_table, seq_of_token)
        qkv = sum_partials(qkv, x.dtype)
    q_out, kv_out = n_q_heads * head_dim, n_kv_heads * head_dim
    q = qkv[:, :q_out].unflatten(1, (n_q_heads, head_dim))
    k = qkv[:, q_out : q_out + kv_out].unflatten(1, (n_kv_heads, head_dim))
    v = qkv[:, q_out + kv_out :].unflatten(1, (n_kv_heads, head_dim))
    rope_kv_write(q, k, v, positions, inv_freq, cache, block_table, seq_of_token)
    return qkv


def rope_kv_write_partials(
    partials: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    head_dim: int,
    positions: torch.Tensor,
    inv_freq: Optional[torch.Tensor],
    cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_of_token: torch.Tensor,
) -> torch.Tensor:
    """`rope_kv_write` from the float32 partial sums [P, T, (Hq + 2 Hkv) * hd] of the joined q/k/v
    projection: they are added in order and rounded to bfloat16 (the bits `sum_partials` gives), q
    and k are rotated, k and v written to the paged bfloat16 cache.  Returns [T, (Hq + 2 Hkv) * hd]."""
    _need_gpu(partials, positions, inv_freq, cache, block_table, seq_of_token)
    width = (n_q_heads + 2 * n_kv_heads) * head_dim
    if partials.dim() != 3 or partials.dtype != torch.float32 or partials.shape[2] != width or not partials.is_contiguous():
        raise KernelError(f"partial sums must be a contiguous float32 [P, T, {width}] tensor")
    n_part, n_tokens, _ = partials.shape
    if head_dim % 8 != 0 or cache.dtype != torch.bfloat16:
        raise KernelError("the rotation from partial sums takes head sizes of a multiple of 8 and a bfloat16 cache")
    _i32(positions, "positions")
    _i32(seq_of_token, "seq_of_token")
    _i32(block_table, "block_table")
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2 or not inv_freq.is_contiguous()):
        raise KernelError(f"the rotary table must be float32 [{head_dim // 2}]")
    if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[2] != n_kv_heads or cache.shape[3] % head_dim != 0 or not cache.is_contiguous():
        raise KernelError(f"cache {tuple(cache.shape)} does not fit {n_kv_heads} heads of size {head_dim}")
    if positions.numel() != n_tokens or seq_of_token.numel() != n_tokens or block_table.dim() != 2:
        raise KernelError("positions and seq_of_token must be [T], block_table [B, W]")
    out = torch.empty((n_tokens, width), dtype=torch.bfloat16, device=partials.device)
    lib = _build.load("rope_kv")
    _check(
        lib,
        lib.cwm_rope_kv_write_partials(
            _ptr(out), ctypes.c_long(width), _ptr(partials), ctypes.c_int(n_part), ctypes.c_long(n_tokens * width),
            _ptr(positions), _ptr(seq_of_token), _ptr(inv_freq), _ptr(cache), _ptr(block_table),
            ctypes.c_int(block_table.shape[1]), ctypes.c_int(cache.shape[3] // head_dim), ctypes.c_int(cache.shape[0]),
            ctypes.c_int(n_tokens), ctypes.c_int(n_q_heads), ctypes.c_int(n_kv_heads), ctypes.c_int(head_dim), _stream(),
        ),
    )
    return out


def sum_partials(partials: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[P, M, N] float32 -> [M, N]: the partial sums added in order."""
    _need_gpu(partials)
    if partials.dim() != 3 or partials.dtype != torch.float32 or not partials.is_contiguous():
        raise KernelError("partial sums must be a contiguous float32 [P, M, N] tensor")
    p, m, n = partials.shape
    out = torch.empty((m, n), dtype=out_dtype, device=partials.device)
    lib = _build.load("rowwise")
    _check(lib, lib.cwm_sum_partials(_ptr(out), ctypes.c_int(_code(out_dtype)), _ptr(partials), ctypes.c_int(p), ctypes.c_long(m * n), _stream()))
    return out


TILE_MAX_ROWS = 512
_tile_slabs: dict = {}  # (rows, columns, K, blocks) -> slabs of partial results


def _tile_takes(x: torch.Tensor, weight: torch.Tensor) -> bool:
    k, n = x.shape[1], weight.shape[0]
    return (
        x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
        and k % 64 == 0 and n % 16 == 0 and 0 < x.shape[0] <= TILE_MAX_ROWS
        and x.stride(-1) == 1 and weight.stride(-1) == 1
        and (x.shape[0] <= 1 or x.stride(0) % 8 == 0) and (n <= 1 or weight.stride(0) % 8 == 0)
        and max(x.stride(0), weight.stride(0)) < (1 << 22)
        and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
    )


def gemm_bf16_tile(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
    partials_ok: bool = False,
    glu: bool = False,
    units: Optional[int] = None,
) -> torch.Tensor:
    """bfloat16 x [M <= 512, K] @ weight[N, K]^T with float32 sums: persistent blocks whose tiles
    of 64, 128 or 256 rows reach LDS by direct loads and that share the work by steps of K.  Returns
    [M, N]; with `partials_ok` it may return float32 partial sums [P, M, N] for the caller to add.
    `glu`: the weight's rows are gate and up rows in alternating groups of 8 and the result is
    silu(gate) * up, [M, N / 2] (in the kernel where a block owns whole tiles, else after it).
    `units` (tests) stands in for the number of compute units."""
    _need_gpu(x, weight, bias)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1] or not _tile_takes(x, weight):
        raise KernelError(
            f"the tiled product takes bfloat16 x [0 < M <= {TILE_MAX_ROWS}, K] and weight [N, K] with K a multiple of 64, N of "
            f"16 and 16-byte aligned rows; got {tuple(x.shape)} {x.dtype} and {tuple(weight.shape)} {weight.dtype}"
        )
    m, k = x.shape
    n = weight.shape[0]
    if bias is not None and (bias.shape != (n,) or not bias.is_contiguous()):
        raise KernelError(f"gemm: bias {tuple(bias.shape)} does not fit {n} outputs")
    out_dtype = out_dtype or torch.bfloat16
    lib = _build.load("gemm_bf16_tile")
    units = units or _compute_units(x.device)
    slabs = _tile_slabs.get((m, n, k, units))
    if slabs is None:
        slabs = _tile_slabs[(m, n, k, units)] = int(lib.cwm_gemm_bf16_tile_slabs(m, n, k, units))
        if slabs < 1:
            raise KernelError(f"the tiled product has no cut for M={m} N={n} K={k}")
    fused_glu = glu and slabs == 1 and bias is None
    if fused_glu:
        out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    elif slabs == 1:
        out = torch.empty((m, n), dtype=torch.float32 if bias is not None else (torch.bfloat16 if glu else out_dtype), device=x.device)
    else:
        out = torch.empty((slabs, m, n), dtype=torch.float32, device=x.device)
    _check(
        lib,
        lib.cwm_gemm_bf16_tile(
            _ptr(x), ctypes.c_long(x.stride(0) if m > 1 else k), _ptr(weight), ctypes.c_long(weight.stride(0) if n > 1 else k),
            _ptr(out), ctypes.c_int(_code(out.dtype)), ctypes.c_long(out.shape[-1]), ctypes.c_long(m * n),
            ctypes.c_int(m), ctypes.c_int(n), ctypes.c_int(k), ctypes.c_int(units), ctypes.c_int(slabs), ctypes.c_int(int(fused_glu)),
            _stream(),
        ),
    )
    if fused_glu:
        return out
    if bias is not None:  # not in the kernel; no model of this architecture has one on a product of this size
        if out.dim() == 3:
            out[0] += bias.float()
        else:
            out = out + bias.float()
    if glu:
        return silu_mul(out if out.dim() == 3 else out.to(torch.bfloat16), out_dtype=torch.bfloat16, grouped=True)
    if out.dim() == 3 and not partials_ok:
        return sum_partials(out, out_dtype)
    return out if out.dim() == 3 or out.dtype == out_dtype else out.to(out_dtype)


# rows up to which the streaming product (x in registers, every epilogue in the kernel) is preferred; its epilogues take
# up to 16, but from 9 on the tiled product is as fast or faster where it takes the sizes (a decode step of the 32B shape at
# batch 16: 15.3 against 15.6 ms)
STREAM_FUSED_ROWS = 8
STREAM_EPILOGUE_ROWS = 16
TILE_ROWS = 128  # rows up to which the tiled product is the fastest whatever the shape
TILE_TALL_ROWS = 256  # rows of its tallest block: up to there it reads W once
TILE_COLUMNS = 128  # columns of a tall block's tile


# entries of a matrix from which on reading it is what a product of few rows costs (below, a launch more or less counts as much)
TILE_FEW_ROWS_ENTRIES = 1 << 24


def _prefers_tile(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], streamed: Optional[torch.Tensor] = None) -> bool:
    """Whether this product goes to the tiled kernel (which has no bias of its own): from 9 rows on; and for
    fewer rows where the matrix is large and has no streaming copy, since the tiled kernel reads the row-major
    matrix in whole cache lines past the caches, which the streaming kernel can only do with that copy (a
    layer's four products of the 32B shape at 8 rows: 159 us tiled, 187 us streamed from the row-major
    matrices, 159 us streamed from the copies; at 1 row 163, 178 and 154 us)."""
    if bias is not None:
        return False
    if x.shape[0] <= STREAM_FUSED_ROWS and (streamed is not None or weight.numel() < TILE_FEW_ROWS_ENTRIES):
        return False
    return _tile_wins(x, weight)


def _tile_wins(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether the tiled product takes this product and is the fastest for it.  Above 128 rows its blocks of
    256 rows are bound by LDS and matrix cores, and the library is faster wherever its own tiles fill the
    chip.  Measured on the matrices of the 8B, 32B and 70B shapes at 160 and 256 rows: the tiled product,
    which shares K between blocks, is ahead where its tiles are at most half as many as the compute units
    (up to 16,384 columns: 41 against 67 us for the 32B shape's q/k/v product at 256 rows, 89 against 234 us
    for its feed-forward's second product).  With two blocks of rows (up to 512) it was ahead on that second
    product alone (144 against 195 us at 384 rows), which the float32 partial sums that the next kernel then
    reads cost again in a decode step, so more than 256 rows go to the library."""
    m = x.shape[0]
    if m > TILE_TALL_ROWS or not _tile_takes(x, weight):
        return False
    if m <= TILE_ROWS:
        return True
    return 2 * -(-weight.shape[0] // TILE_COLUMNS) <= _compute_units(x.device)


def _stream_takes(x: torch.Tensor, weight: torch.Tensor) -> bool:
    k = x.shape[1]
    return (
        k % 8 == 0
        and x.stride(-1) == 1 and weight.stride(-1) == 1
        and (x.shape[0] <= 1 or x.stride(0) % 8 == 0)
        and (weight.shape[0] <= 1 or weight.stride(0) % 8 == 0)
        and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
    )


def gemm_bf16(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
    partials_ok: bool = False,
    streamed: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """bfloat16 x [M, K] @ bfloat16 weight[N, K]^T, float32 accumulation.

    Up to 8 rows: the hand-written persistent weight-streaming kernel, x in registers.
    Up to 128 rows (256 for a result of at most 16,384 columns): the hand-written tiled kernel, x and W
    through LDS (it needs K % 64 == 0 and N % 16 == 0; other sizes of up to 64 rows stream).
    More rows: the library product (hipBLASLt through torch), as the reference calls a
    library here, with a bfloat16 or a float32 result.  Row lengths that are no multiple
    of 8 go to the float32 kernel, which takes any size.
    """
    _need_gpu(x, weight, bias)
    out_dtype = out_dtype or torch.bfloat16
    m = x.shape[0]
    if not _stream_takes(x, weight):
        return gemm_f32(x, weight, bias, out_dtype)
    if _prefers_tile(x, weight, bias, streamed):
        return gemm_bf16_tile(x, weight, None, out_dtype, partials_ok)
    if m <= STREAM_MAX_ROWS:
        return gemm_bf16_stream(x, weight, bias, out_dtype, partials_ok, streamed=streamed)
    if out_dtype == torch.float32:
        y = torch.mm(x, weight.t(), out_dtype=torch.float32)  # bfloat16 operands, float32 sums written as they are
        return y if bias is None else y + bias.float()
    if bias is not None:
        return torch.addmm(bias.to(x.dtype), x, weight.t())  # the bias rides in the library's epilogue
    # one call whatever the shape: nothing is timed or tuned inside a step, so the same step gives the same bits
    # in every process.  (Calls on column ranges of a wide output were measured: at most 3% faster at 2,048 rows.)
    return torch.mm(x, weight.t())


# --------------------------------------------------------------------------- #
def rope_kv_write(
    q: torch.Tensor,
    k: Optional[torch.Tensor],
    v: Optional[torch.Tensor],
    positions: torch.Tensor,
    inv_freq: Optional[torch.Tensor],
    cache: Optional[torch.Tensor] = None,
    block_table: Optional[torch.Tensor] = None,
    seq_of_token: Optional[torch.Tensor] = None,
) -> None:
    """Rotate `q` [T, Hq, hd] and `k` [T, Hkv, hd] in place by positions * inv_freq
    (adjacent pairs) and write the rotated keys and `v` into the paged `cache`
    ([pages, 2, Hkv, page * hd]; keys [slot][dim], values [slot / 8][dim][slot % 8])
    at the rows the block table gives.  `q`, `k`, `v`
    may be views into one wider tensor (token stride free, heads contiguous)."""
    _need_gpu(q, k, v, positions, inv_freq, cache, block_table, seq_of_token)
    if q.dim() != 3 or q.stride(2) != 1 or q.stride(1) != q.shape[2]:
        raise KernelError("q must be [T, Hq, hd] with contiguous heads")
    n_tokens, n_q, hd = q.shape
    n_kv = 0
    for name, t in (("k", k), ("v", v)):
        if t is not None:
            if t.dim() != 3 or t.shape[0] != n_tokens or t.shape[2] != hd or t.stride(2) != 1 or t.stride(1) != hd:
                raise KernelError(f"{name} must be [T, Hkv, hd] with contiguous heads")
            if t.dtype != q.dtype:
                raise KernelError("q, k and v must have one type")
            n_kv = t.shape[1]
    _i32(positions, "positions")
    if positions.numel() != n_tokens:
        raise KernelError("one position per token is needed")
    if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != hd // 2 or not inv_freq.is_contiguous()):
        raise KernelError(f"the rotary table must be float32 [{hd // 2}]")
    page_size = num_pages = width = 0
    if cache is not None:
        if k is None or v is None or block_table is None or seq_of_token is None:
            raise KernelError("a cache write needs k, v, a block table and the sequence of each token")
        if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[2] != n_kv or cache.shape[3] % hd != 0 or not cache.is_contiguous():
            raise KernelError(f"cache {tuple(cache.shape)} does not fit {n_kv} heads of size {hd}")
        if cache.dtype != q.dtype:
            raise KernelError("the cache and q, k, v must have one type")
        _i32(block_table, "block_table")
        _i32(seq_of_token, "seq_of_token")
        if block_table.dim() != 2 or seq_of_token.numel() != n_tokens:
            raise KernelError("block_table must be [B, W] and seq_of_token [T]")
        num_pages, page_size, width = cache.shape[0], cache.shape[3] // hd, block_table.shape[1]
    lib = _build.load("rope_kv")
    _check(
        lib,
        lib.cwm_rope_kv_write(
            _ptr(q), ctypes.c_long(q.stride(0)),
            _ptr(k), ctypes.c_long(k.stride(0) if k is not None else 0),
            _ptr(v), ctypes.c_long(v.stride(0) if v is not None else 0),
            ctypes.c_int(_code(q.dtype)), _ptr(positions), _ptr(seq_of_token), _ptr(inv_freq),
            _ptr(cache), _ptr(block_table), ctypes.c_int(width), ctypes.c_int(page_size), ctypes.c_int(num_pages),
            ctypes.c_int(n_tokens), ctypes.c_int(n_q), ctypes.c_int(n_kv if k is not None else 0), ctypes.c_int(hd),
            _stream(),
        ),
    )


def paged_attention_simple(
    q: torch.Tensor,
    cache: torch.Tensor,
    block_table: torch.Tensor,
    positions: torch.Tensor,
    seq_of_token: torch.Tensor,
    window: Optional[int],
    scale: float,
    max_keys: Optional[int] = None,
) -> torch.Tensor:
    """Causal attention of `q` [T, Hq, hd] over the paged cache by the plain kernel:
    float32 arithmetic, a key/value head's query heads sharing its keys and values, long
    key ranges cut into segments that a second kernel joins.  `window`: keys read per
    query, own included (None: all).  `max_keys`: the most keys any token reads (default:
    from the largest position, which costs a copy to the host).  Returns [T, Hq * hd]."""
    _need_gpu(q, cache, block_table, positions, seq_of_token)
    if q.dim() != 3 or q.stride(2) != 1 or q.stride(1) != q.shape[2]:
        raise KernelError("q must be [T, Hq, hd] with contiguous heads")
    n_tokens, n_q, hd = q.shape
    if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[3] % hd != 0 or not cache.is_contiguous():
        raise KernelError(f"cache {tuple(cache.shape)} does not fit heads of size {hd}")
    if cache.dtype != q.dtype:
        raise KernelError("the cache and q must have one type")
    n_kv = cache.shape[2]
    _i32(block_table, "block_table")
    _i32(positions, "positions")
    _i32(seq_of_token, "seq_of_token")
    if positions.numel() != n_tokens or seq_of_token.numel() != n_tokens or block_table.dim() != 2:
        raise KernelError("positions and seq_of_token must be [T], block_table [B, W]")
    if window is not None and window < 1:
        raise KernelError("a window holds at least the query's own key")
    out = torch.empty((n_tokens, n_q * hd), dtype=q.dtype, device=q.device)
    lib = _build.load("attention_simple")
    if max_keys is None:
        max_keys = int(positions.max()) + 1 if n_tokens else 1
    if window is not None:
        max_keys = min(max_keys, window)
    max_keys = max(1, max_keys)
    partial = None
    if max_keys > lib.cwm_attention_simple_segment_keys():
        partial = torch.empty(n_tokens * n_q * lib.cwm_attention_simple_max_segments() * (hd + 2), dtype=torch.float32, device=q.device)
    _check(
        lib,
        lib.cwm_attention_simple(
            _ptr(q), ctypes.c_long(q.stride(0)), _ptr(out), ctypes.c_long(n_q * hd), _ptr(cache),
            ctypes.c_int(_code(q.dtype)), _ptr(block_table), ctypes.c_int(block_table.shape[1]),
            _ptr(positions), _ptr(seq_of_token), ctypes.c_int(n_tokens), ctypes.c_int(n_q), ctypes.c_int(n_kv),
            ctypes.c_int(hd), ctypes.c_int(cache.shape[3] // hd), ctypes.c_int(cache.shape[0]),
            ctypes.c_int(-1 if window is None else window - 1), ctypes.c_float(scale),
            ctypes.c_int(max_keys), _ptr(partial), _stream(),
        ),
    )
    return out


@dataclass
class _UploadedPlan:
    """A step's attention work lists on the device, and what the launch needs to know of them."""

    work: torch.Tensor  # items of one row tile
    wide: torch.Tensor  # items of WIDE_TILES row tiles
    merge: torch.Tensor
    n_work: int
    n_wide: int
    n_merge: int
    n_merge_mid: int  # merge items of at most 32 partials, after those with more
    n_merge_wide: int  # merge items of cut wide items, last in the list
    n_partials: int
    work_keys: int  # keys of an average item of one row tile
    wide_shape: Tuple[int, float]  # key tiles of the longest wide item, and the mean


class StaticPlans:
    """The attention work lists of a step that is captured once and replayed: every list has a home of a
    fixed size at a fixed address, which `refresh` fills for each new step (unused places hold null items),
    so that the captured launches stay valid while the sequences grow.  The first, uncaptured run of the step
    finds out which lists the model's layers ask for and makes their homes."""

    def __init__(self, device: torch.device, max_keys: int) -> None:
        self.device = device
        self.max_keys = max_keys  # the most keys a sequence may hold while the capture is in use
        self.homes: dict = {}  # (group, key/value heads, window) -> (capacity, device vector, uploaded plan)

    def _padded(self, batch, group: int, n_kv: int, window: Optional[int], capacity):
        from .attention_plan import build_plan, capacity_until, pad_plan

        wide_cut_below = -(-2 * _compute_units(self.device) // n_kv)
        if capacity is None:
            plan, capacity = capacity_until(batch.q_lens, batch.kv_lens, group, window, wide_cut_below, self.max_keys)
        else:
            plan = build_plan(batch.q_lens, batch.kv_lens, group, window, wide_cut_below)
        flat = pad_plan(plan, capacity)
        return plan, capacity, flat

    def plan(self, batch, group: int, n_kv: int, window: Optional[int]) -> "_UploadedPlan":
        key = (group, n_kv, window)
        home = self.homes.get(key)
        if home is None:
            plan, capacity, flat = self._padded(batch, group, n_kv, window, None)
            if flat is None:
                raise KernelError("this step's attention work has items that a captured step does not take")
            dev = torch.from_numpy(flat).pin_memory().to(self.device, non_blocking=True)
            a = capacity.work * 6
            uploaded = _UploadedPlan(
                work=dev[:a], wide=dev[a:a], merge=dev[a:], n_work=capacity.work, n_wide=0, n_merge=capacity.merge,
                n_merge_mid=capacity.merge_mid, n_merge_wide=0, n_partials=capacity.work,
                work_keys=int((plan.work[:, 3] - plan.work[:, 2]).mean()) if plan.work.shape[0] else 0, wide_shape=(0, 0.0),
            )
            home = self.homes[key] = (capacity, dev, uploaded)
        return home[2]

    def refresh(self, batch) -> bool:
        """Fill every home with the lists of `batch`; False if one of them has outgrown its home."""
        for (group, n_kv, window), (capacity, dev, _) in self.homes.items():
            _, _, flat = self._padded(batch, group, n_kv, window, capacity)
            if flat is None:
                return False
            dev.copy_(torch.from_numpy(flat).pin_memory(), non_blocking=True)
        return True


def _attention_plan(batch, group: int, n_kv: int, window: Optional[int], device: torch.device) -> _UploadedPlan:
    """The step's work list for this (group size, key/value heads, window), uploaded once per step."""
    from .attention_plan import build_plan

    static = getattr(batch, "static", None)
    if static is not None:
        return static.plan(batch, group, n_kv, window)
    key = ("attention_plan", group, n_kv, window)
    cached = batch.scratch.get(key)
    if cached is None:
        # a sequence whose blocks of 128 rows, over all key/value heads, would not give every compute unit two
        wide_cut_below = -(-2 * _compute_units(device) // n_kv) if device.type == "cuda" else 0
        plan = build_plan(batch.q_lens, batch.kv_lens, group, window, wide_cut_below)
        flat = np.concatenate([plan.work.reshape(-1), plan.work_wide.reshape(-1), plan.merge.reshape(-1)]).astype(np.int32)
        host = torch.from_numpy(flat)
        if device.type == "cuda":
            host = host.pin_memory()
        dev = host.to(device, non_blocking=True)
        n_work, n_wide, n_merge = plan.work.shape[0], plan.work_wide.shape[0], plan.merge.shape[0]
        a, b = n_work * 6, (n_work + n_wide) * 6
        wide_tiles = (plan.work_wide[:, 3] - (plan.work_wide[:, 2] & ~31) + 31) // 32 if n_wide else None  # key tiles of each wide item
        cached = _UploadedPlan(
            work=dev[:a], wide=dev[a:b], merge=dev[b:], n_work=n_work, n_wide=n_wide, n_merge=n_merge,
            n_merge_mid=plan.n_merge_mid, n_merge_wide=plan.n_merge_wide, n_partials=plan.n_partials,
            work_keys=int((plan.work[:, 3] - plan.work[:, 2]).mean()) if n_work else 0,
            wide_shape=(int(wide_tiles.max()), float(wide_tiles.mean())) if n_wide else (0, 0.0),
        )
        batch.scratch[key] = cached
    return cached


# a block's time for one tile of keys when three blocks share a compute unit, over that with two
_THREE_BLOCKS_TILE_TIME = 1.38


def _three_blocks_a_unit(n_blocks: int, shape: Tuple[int, float], device: torch.device) -> int:
    """Whether the blocks that share keys and values through LDS finish sooner three to a
    compute unit (the build with three buffers) than two (four buffers): `shape` is the
    longest block and the mean, in key tiles.  Two finish a launch of few, uneven blocks
    sooner (the longest block sets the time, and runs faster with one neighbour); three hide
    more latency when there are rounds of blocks.  Estimate of either: the longer of the
    longest block and the mean times the number of rounds, times a tile's time."""
    if n_blocks == 0:
        return 0
    units = _compute_units(device)
    longest, mean = shape
    two = max(longest, mean * -(-n_blocks // (2 * units)))
    three = _THREE_BLOCKS_TILE_TIME * max(longest, mean * -(-n_blocks // (3 * units)))
    return int(three < two)


def mfma_attention_takes(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    """Sizes the matrix-core attention kernel covers; everything else runs on the
    plain kernel."""
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and page_size % 8 == 0


def paged_attention_mfma(
    q: torch.Tensor,
    cache: torch.Tensor,
    block_table: torch.Tensor,
    batch,
    window: Optional[int],
    scale: float,
) -> torch.Tensor:
    """Matrix-core attention (bfloat16): prompt portions and decoded tokens in one
    launch, long key ranges of short sequences split and merged."""
    _need_gpu(q, cache, block_table)
    if q.dtype != torch.bfloat16 or cache.dtype != torch.bfloat16:
        raise KernelError("the matrix-core attention kernel takes bfloat16 only")
    if q.dim() != 3 or q.stride(2) != 1 or q.stride(1) != q.shape[2]:
        raise KernelError("q must be [T, Hq, hd] with contiguous heads")
    n_tokens, n_q, hd = q.shape
    if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[3] % hd != 0 or not cache.is_contiguous():
        raise KernelError(f"cache {tuple(cache.shape)} does not fit heads of size {hd}")
    n_kv = cache.shape[2]
    page_size = cache.shape[3] // hd
    if not mfma_attention_takes(q.dtype, hd, page_size):
        raise KernelError(f"the matrix-core attention kernel does not take head_dim {hd} with pages of {page_size}")
    if n_q % n_kv != 0:
        raise KernelError(f"{n_q} query heads do not divide into {n_kv} key/value heads")
    if q.stride(0) % 8 != 0 or q.data_ptr() % 16 != 0:
        raise KernelError("q rows must be 16-byte aligned")
    _i32(block_table, "block_table")
    if block_table.dim() != 2 or block_table.shape[0] != batch.n_seqs or n_tokens != batch.n_tokens:
        raise KernelError("block_table must be [B, W] for the batch's sequences, q [T, ...] for its tokens")
    if window is not None and window < 1:
        raise KernelError("a window holds at least the query's own key")
    plan = _attention_plan(batch, n_q // n_kv, n_kv, window, q.device)
    out = torch.empty((n_tokens, n_q * hd), dtype=q.dtype, device=q.device)
    partial = None
    if plan.n_partials:
        partial = torch.empty(plan.n_partials * n_kv * 16 * (hd + 4), dtype=torch.float32, device=q.device)
    lib = _build.load("attention_mfma", {"HEAD_DIM": hd})
    _check(
        lib,
        lib.cwm_attention_mfma(
            _ptr(q), ctypes.c_long(q.stride(0)), _ptr(out), ctypes.c_long(n_q * hd), _ptr(cache),
            _ptr(block_table), ctypes.c_int(block_table.shape[1]), _ptr(batch.cu_q), _ptr(batch.kv_len),
            _ptr(plan.work), ctypes.c_int(plan.n_work), ctypes.c_int(plan.work_keys),
            _ptr(plan.wide), ctypes.c_int(plan.n_wide), ctypes.c_int(WIDE_TILES),
            ctypes.c_int(_three_blocks_a_unit(plan.n_wide * n_kv, plan.wide_shape, q.device)),
            _ptr(plan.merge), ctypes.c_int(plan.n_merge), ctypes.c_int(plan.n_merge_mid), ctypes.c_int(plan.n_merge_wide), _ptr(partial),
            ctypes.c_int(n_q), ctypes.c_int(n_kv), ctypes.c_int(hd), ctypes.c_int(page_size),
            ctypes.c_int(cache.shape[0]), ctypes.c_int(-1 if window is None else window - 1),
            ctypes.c_float(scale), _stream(),
        ),
    )
    return out


def paged_attention(
    q: torch.Tensor,
    cache: torch.Tensor,
    block_table: torch.Tensor,
    batch,
    window: Optional[int],
    scale: float,
) -> torch.Tensor:
    """Attention of the step's tokens over the cache.  `batch` is the step's
    `StepBatch` (positions, sequence of each token and the per-sequence lengths).
    bfloat16 with head sizes in steps of 16 and pages in steps of 8 runs on the
    matrix cores; float32, and other sizes, on the plain kernel."""
    hd = q.shape[2]
    if q.is_cuda and mfma_attention_takes(q.dtype, hd, cache.shape[3] // hd):
        return paged_attention_mfma(q, cache, block_table, batch, window, scale)
    static = getattr(batch, "static", None)
    max_keys = batch.max_kv_len if static is None else static.max_keys
    return paged_attention_simple(q, cache, block_table, batch.positions, batch.seq_of_token, window, scale, max_keys=max_keys)


# --------------------------------------------------------------------------- #
def sample_packed(
    logits: torch.Tensor,
    temperature: torch.Tensor,
    top_p: torch.Tensor,
    uniform: torch.Tensor,
) -> torch.Tensor:
    """Per row of float32 `logits` [R, V]: greedy where temperature <= 0, else a draw
    from softmax(logits / T) cut to the nucleus `top_p`, using the row's uniform
    number.  Returns one int32 tensor [3, R], so that everything reaches the host in one
    copy: the tokens, then the bits of the float32 log-probabilities log softmax(logits)
    at the token and of the token under the sampling distribution (`unpack_sampled`)."""
    _need_gpu(logits, temperature, top_p, uniform)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("logits must be float32 [R, V] with contiguous rows")
    n_rows, vocab = logits.shape
    for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
        if t.dtype != torch.float32 or t.numel() != n_rows or not t.is_contiguous():
            raise KernelError(f"{name} must be float32 [{n_rows}]")
    dev = logits.device
    out = torch.empty((3, n_rows), dtype=torch.int32, device=dev)
    workspace = torch.empty((max(n_rows, 1), vocab), dtype=torch.float32, device=dev)
    lib = _build.load("sampling")
    _check(
        lib,
        lib.cwm_sample(
            _ptr(logits), ctypes.c_long(logits.stride(0) if n_rows > 1 else vocab), ctypes.c_int(n_rows),
            ctypes.c_int(vocab), _ptr(temperature), _ptr(top_p), _ptr(uniform), _ptr(workspace),
            _ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _stream(),
        ),
    )
    return out


def unpack_sampled(packed: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(tokens int32, logprobs float32, sample_logprobs float32) as views of what `sample_packed` returned
    ([3, R], on any device)."""
    return packed[0], packed[1].view(torch.float32), packed[2].view(torch.float32)


def sample(
    logits: torch.Tensor,
    temperature: torch.Tensor,
    top_p: torch.Tensor,
    uniform: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """`sample_packed` as three tensors: (tokens int32, logprobs, sample_logprobs)."""
    return unpack_sampled(sample_packed(logits, temperature, top_p, uniform))


def token_logprobs(logits: torch.Tensor, rows: torch.Tensor, targets: torch.Tensor) -> torch.Tensor:
    """log softmax(logits[rows[i]])[targets[i]] (float32 [n]) for int32 `rows`, `targets`."""
    _need_gpu(logits, rows, targets)
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("logits must be float32 [R, V] with contiguous rows")
    _i32(rows, "rows")
    _i32(targets, "targets")
    if rows.numel() != targets.numel():
        raise KernelError("one target per row is needed")
    out = torch.empty(rows.numel(), dtype=torch.float32, device=logits.device)
    lib = _build.load("sampling")
    _check(
        lib,
        lib.cwm_token_logprob(
            _ptr(logits), ctypes.c_long(logits.stride(0) if logits.shape[0] > 1 else logits.shape[1]),
            ctypes.c_int(logits.shape[0]), ctypes.c_int(logits.shape[1]), _ptr(rows), _ptr(targets),
            ctypes.c_int(rows.numel()), _ptr(out), _stream(),
        ),
    )
    return out


__all__ = [
    "KernelError",
    "KernelBuildError",
    "embedding",
    "add_rmsnorm",
    "silu_mul",
    "gemm_f32",
    "gemm_f32_stream",
    "gemm_bf16",
    "gemm_bf16_stream",
    "sum_partials",
    "linear",
    "rope_kv_write",
    "qkv_rope_write",
    "paged_attention_simple",
    "paged_attention_mfma",
    "mfma_attention_takes",
    "paged_attention",
    "sample",
    "sample_packed",
    "unpack_sampled",
    "token_logprobs",
]


# --------------------------------------------------------------------------- #
# what the GPU at hand reaches (for the measurement program; nothing on the model's path)
def measure_read_rate(buffer: torch.Tensor, window_bytes: int, launches: int, blocks: int) -> float:
    """GB/s at which a kernel that only reads gets through `window_bytes` of `buffer` (uint8, on the device):
    `launches` launches back to back, each on the next window of the buffer (so that, with a buffer several times
    the last-level cache, no launch finds its bytes cached), timed by events around all of them."""
    _need_gpu(buffer)
    if buffer.dtype != torch.uint8 or not buffer.is_contiguous() or window_bytes % 16 != 0 or not 0 < window_bytes <= buffer.numel():
        raise KernelError("measure_read_rate takes a contiguous uint8 buffer and a window that is a multiple of 16 bytes within it")
    lib = _build.load("ceilings")
    windows = max(1, buffer.numel() // window_bytes)
    base = buffer.data_ptr()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = _stream()
    for timed in (False, True):
        if timed:
            start.record()
        for i in range(launches if timed else 2):
            offset = (i % windows) * window_bytes
            _check(lib, lib.cwm_ceiling_read(ctypes.c_void_p(base + offset), ctypes.c_long(window_bytes), ctypes.c_int(blocks), ctypes.c_void_p(0), stream))
        if timed:
            end.record()
        torch.cuda.synchronize(buffer.device)
    return window_bytes * launches / (start.elapsed_time(end) * 1e-3) / 1e9


def measure_mfma_rate(device: torch.device, blocks: int, rounds: int, launches: int = 3, shape: int = 16, seed: float = 1.0) -> float:
    """PFLOP/s of the bfloat16 matrix instruction (`shape` 16: 16x16x32, 32: 32x32x16; float32 sums) issued from
    registers by `blocks` blocks of four wavefronts, `rounds` rounds of eight independent instructions each, on
    operands of `seed` times small varied numbers (0: all zeros, which costs the least power)."""
    lib = _build.load("ceilings")
    lib.cwm_ceiling_mfma_flops.restype = ctypes.c_double
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.device(device):
        stream = _stream()
        for timed in (False, True):
            if timed:
                start.record()
            for _ in range(launches if timed else 1):
                _check(lib, lib.cwm_ceiling_mfma(ctypes.c_int(blocks), ctypes.c_int(rounds), ctypes.c_int(shape), ctypes.c_float(seed), ctypes.c_void_p(0), stream))
            if timed:
                end.record()
            torch.cuda.synchronize(device)
    flops = lib.cwm_ceiling_mfma_flops(ctypes.c_int(blocks), ctypes.c_int(rounds)) * launches
    return flops / (start.elapsed_time(end) * 1e-3) / 1e15
