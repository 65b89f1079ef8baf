"""Block-FP8 checkpoint dequantization on the GPU: the `fp8_block` method of the reference's
checkpoint-dequantizer registry (paddleformers/quantization/checkpoint_dequant.py:191-292, 353-392),
same class and function names, same configuration steps and error behaviour, with `dequantize`
running libpf8's `pf8_block_dequant` instead of a table gather + repeat_interleave + multiply.

Raw e4m3 bytes arrive as uint8/int8 tensors (safetensors keeps unsupported 8-bit formats as raw
storage) or as torch.float8_e4m3fn; scales as UE8M0 exponent bytes or fp32/bf16/fp16.  Blocking is
supported on the last two axes of the weight (every block-FP8 checkpoint layout in the reference:
[out, in] matrices with `block_shape: [128, 128]`, transformers/deepseek_v4/modeling.py:400-417).
The MXFP4 method of the same registry is not part of this package.
"""
from __future__ import annotations

import ctypes as C
import math

import torch

from . import _lib

_VALUE_FORMATS = frozenset({"e4m3", "fp8_e4m3", "float8_e4m3"})
_UE8M0_NAMES = frozenset({"ue8m0", "e8m0", "float8_e8m0"})
_FLOAT_NAMES = frozenset({"float", "fp16", "fp32", "bf16", "float16", "float32", "bfloat16"})


class FP8BlockCheckpointDequantizer:
    method = "fp8_block"
    value_formats = _VALUE_FORMATS
    scale_formats = _UE8M0_NAMES | _FLOAT_NAMES

    def __init__(self, value_format=None, scale_format=None, block_axes=None, block_shape=None):
        self.value_format = value_format
        self.scale_format = scale_format
        self.block_axes = block_axes
        self.block_shape = block_shape

    # -- configuration (checkpoint_dequant.py:210-236): every step returns a new object ----------
    def configure_formats(self, value_format, scale_format):
        value_format, scale_format = value_format.strip().lower(), scale_format.strip().lower()
        if value_format not in self.value_formats:
            raise ValueError(f"Unsupported {self.method} value_format {value_format!r}.")
        if scale_format not in self.scale_formats:
            raise ValueError(f"Unsupported {self.method} scale_format {scale_format!r}.")
        return type(self)(value_format, scale_format, self.block_axes, self.block_shape)

    def configure_geometry(self, block_axes, block_shape):
        bad = (not block_axes or len(block_axes) != len(block_shape) or len(set(block_axes)) != len(block_axes)
               or any(a < 0 for a in block_axes) or any(b <= 0 for b in block_shape))
        if bad:
            raise ValueError(f"Invalid block geometry for {self.method}.")
        return type(self)(self.value_format, self.scale_format, tuple(block_axes), tuple(block_shape))

    def _geometry(self, rank):
        if self.block_axes is None or self.block_shape is None:
            raise ValueError(f"{self.method} requires block geometry.")
        axes = tuple(a + rank if a < 0 else a for a in self.block_axes)
        if any(a >= rank for a in axes):
            raise ValueError(f"Invalid block_axes {self.block_axes} for a rank-{rank} tensor.")
        return axes, self.block_shape

    # -- shape contracts (checkpoint_dequant.py:238-265): fp8 storage is one byte per element -----
    def logical_shape(self, physical_shape):
        return tuple(physical_shape)

    def physical_qweight_shape(self, logical_shape):
        return tuple(logical_shape)

    def physical_qweight_slice(self, global_offset, local_shape):
        return tuple(global_offset), tuple(local_shape)

    def logical_shard_is_aligned(self, global_shape, local_shape, global_offset):
        axes, block_shape = self._geometry(len(global_shape))
        for axis, size in zip(axes, block_shape):
            start, end = global_offset[axis], global_offset[axis] + local_shape[axis]
            if start % size != 0 and start != 0:
                return False
            if end % size != 0 and end != global_shape[axis]:
                return False
        return True

    # -- the GPU path ----------------------------------------------------------------------------
    def dequantize(self, components, output_dtype):
        missing = {"qweight", "scale"} - set(components)
        if missing:
            raise KeyError(f"Missing checkpoint quantization components: {sorted(missing)}.")
        q, scale = components["qweight"], components["scale"]
        if q.dtype not in (torch.uint8, torch.int8, torch.float8_e4m3fn):
            raise TypeError(f"qweight must use raw uint8/int8 storage, got {q.dtype}. "
                            "The safetensors reader must preserve unsupported 8-bit formats as raw bytes.")
        if output_dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("output_dtype must be torch.bfloat16 or torch.float32")
        fmt = (self.scale_format or "").strip().lower()
        if fmt in _UE8M0_NAMES:
            if scale.dtype not in (torch.uint8, torch.int8):
                raise TypeError(f"scale must use raw uint8/int8 storage, got {scale.dtype}.")
            code = 1
        elif fmt in _FLOAT_NAMES:
            code = {torch.float32: 0, torch.bfloat16: 2, torch.float16: 3}.get(scale.dtype)
            if code is None:
                raise TypeError(f"scale must be float32, bfloat16 or float16 for scale_format {fmt!r}, got {scale.dtype}.")
        else:
            raise ValueError(f"Unsupported scale_format {fmt!r}.")
        if not q.is_cuda or not scale.is_cuda:
            raise RuntimeError("checkpoint dequantization runs on the GPU only: move qweight and scale to the device (no CPU path)")
        shape = tuple(q.shape)
        rank = len(shape)
        axes, block_shape = self._geometry(rank)
        if scale.dim() != rank:
            raise ValueError(f"Scale rank must match logical weight rank: scale={tuple(scale.shape)}, logical={shape}.")
        axis_to_block = dict(zip(axes, block_shape))
        expected = tuple(math.ceil(d / axis_to_block[a]) if a in axis_to_block else d for a, d in enumerate(shape))
        if tuple(scale.shape) != expected:
            raise ValueError(f"Invalid scale grid shape: expected {expected}, got {tuple(scale.shape)} for logical shape {shape}.")
        if any(a < rank - 2 for a in axes):
            raise ValueError("fp8_block on the GPU supports blocking on the last two axes only")
        R = shape[-2] if rank >= 2 else 1
        Cc = shape[-1]
        B = 1
        for d in shape[:-2]:
            B *= d
        br = axis_to_block.get(rank - 2, 1) if rank >= 2 else 1
        bc = axis_to_block.get(rank - 1, 1)
        q, scale = q.contiguous(), scale.contiguous()
        out = torch.empty(shape, dtype=output_dtype, device=q.device)
        _lib.call("pf8_block_dequant", C.c_void_p(q.data_ptr()), C.c_void_p(scale.data_ptr()), code, B, R, Cc, br, bc,
                  C.c_void_p(out.data_ptr()), int(output_dtype == torch.float32), C.c_void_p(torch.cuda.current_stream().cuda_stream))
        return out


# -- registry (checkpoint_dequant.py:353-392): unconfigured prototypes by normalised method name ----
_CHECKPOINT_DEQUANTIZERS = {}


def _normalize_method(method):
    if not isinstance(method, str):
        raise TypeError(f"Checkpoint quantization method must be a string, got {type(method).__name__}.")
    normalized = method.strip().lower()
    if not normalized:
        raise ValueError("Checkpoint quantization method must not be empty.")
    return normalized


def register_checkpoint_dequantizer(method, dequantizer):
    method = _normalize_method(method)
    if method in _CHECKPOINT_DEQUANTIZERS:
        raise ValueError(f"Checkpoint dequantizer {method!r} is already registered.")
    if not callable(getattr(dequantizer, "dequantize", None)):
        raise TypeError("Checkpoint dequantizer must provide a callable dequantize() method.")
    _CHECKPOINT_DEQUANTIZERS[method] = dequantizer


def get_checkpoint_dequantizer(method):
    method = _normalize_method(method)
    if method not in _CHECKPOINT_DEQUANTIZERS:
        raise ValueError(f"Unsupported checkpoint quantization method {method!r}; registered methods: {sorted(_CHECKPOINT_DEQUANTIZERS)}.")
    return _CHECKPOINT_DEQUANTIZERS[method]


register_checkpoint_dequantizer("fp8_block", FP8BlockCheckpointDequantizer())
