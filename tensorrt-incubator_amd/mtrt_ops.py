"""Front door for the quantization markers the reference recognises, dispatching to libmtrt_hip.so.

The reference reaches its quantize / dequantize kernels through named markers:
  * `stablehlo.custom_call @tensorrt.quantize / @tensorrt.dequantize / @tensorrt.dynamic_quantize` with a
    `mode` string and an optional `axis`, emitted by the JAX primitives
    (mlir-tensorrt/integrations/PJRT/python/mlir_tensorrt_jax/mtrt_ops/quantize.py:117-143,
     dequantize.py, dynamic_quantize.py:150-200);
  * `stablehlo.composite "tensorrt.{pt,pc,block}_{q,dq}"` with attributes {scale, axis}, produced by
    mlir-tensorrt/compiler/lib/Dialect/StablehloExt/Transforms/StablehloRaiseQDQ.cpp:98-110.
This module is the run-time side of those markers: the same entry names (`mtrt_quantize`,
`mtrt_dequantize`, `mtrt_dynamic_quantize`), the same argument meaning, the same shape rules with the
same assertion messages as the primitives' abstract evaluation (quantize.py:44-103,
dynamic_quantize.py:41-84), and `custom_call` / `composite` dispatchers keyed by the marker names.
Device tensors are torch tensors (memory and stream only); scales are host constants, as in the
reference.  Without the library or a gfx950 device the calls raise.
"""
import numpy as np

from . import (BF16, F16, F32, F4_PACKED, F8E4M3FN, I4_PACKED, I8, SCALE_COL, SCALE_ROW, SCALE_UNIFORM, check,
               float_dtype_of, lib, nvfp4_quantize)

# output / input code types by the names the JAX dtypes carry
_CODE = {"int8": I8, "float8_e4m3fn": F8E4M3FN, "int4": I4_PACKED, "float4_e2m1fn": F4_PACKED}
_SUPPORTED_BLOCK_QUANT_OUTPUT_DTYPES = ["float8_e4m3fn", "int4", "float4_e2m1fn"]   # quantize.py:26-32


def _torch():
    import torch
    return torch


def _dtype_name(d):
    """'int8', 'float8_e4m3fn', 'int4', 'float4_e2m1fn', 'float32', ... from a string, numpy or torch dtype."""
    if isinstance(d, str):
        return d
    name = getattr(d, "__name__", None) or str(d)
    return name.replace("torch.", "").replace("<class '", "").replace("'>", "").split(".")[-1]


class QuantizedArray:
    """Quantized codes with their logical shape and type.  int8 and float8 codes are one byte per element;
    int4 and float4 are packed two per byte over the flattened array (element 2i in the low nibble)."""

    def __init__(self, codes, dtype, shape):
        self.codes, self.dtype, self.shape = codes, dtype, tuple(shape)

    def torch(self):
        torch = _torch()
        if self.dtype == "int8":
            return self.codes.view(torch.int8).reshape(self.shape)
        if self.dtype == "float8_e4m3fn":
            return self.codes.view(torch.float8_e4m3fn).reshape(self.shape)
        raise TypeError("%s has no torch element type; use .codes" % self.dtype)


def _as_quantized(x, dtype_hint=None):
    torch = _torch()
    if isinstance(x, QuantizedArray):
        return x
    if x.dtype == torch.int8:
        return QuantizedArray(x.contiguous().view(torch.uint8).reshape(-1), "int8", x.shape)
    if x.dtype == torch.float8_e4m3fn:
        return QuantizedArray(x.contiguous().view(torch.uint8).reshape(-1), "float8_e4m3fn", x.shape)
    raise AssertionError(f"Unsupported input dtype for dequantization: {x.dtype}")


def _check_mode(shape, scale_shape, mode, axis, kind, out_name):
    """Shape rules of the primitives' abstract evaluation (quantize.py:55-97), same messages.
    Returns the C ABI's scale addressing (kind, d0, d1, nb)."""
    rank = len(shape)
    numel = int(np.prod(shape)) if rank else 1
    if mode == f"tensorrt.pt_{kind}":
        assert axis is None, f"axis is only valid for tensorrt.pc_{kind} mode"
        assert scale_shape == (), f"tensorrt.pt_{kind} (per-tensor) mode expects scalar scale, got shape {scale_shape}"
        d1 = shape[-1] if rank else 1
        return SCALE_UNIFORM, numel // d1 if d1 else 0, d1, 1
    if mode == f"tensorrt.pc_{kind}":
        assert axis is not None, f"tensorrt.pc_{kind} mode requires axis"
        assert axis >= 0 and axis < rank, (
            f"tensorrt.pc_{kind} mode requires axis to be in range [0, {rank}), " f"got {axis}")
        assert len(scale_shape) == 1, (
            f"tensorrt.pc_{kind} (per-channel) mode expects 1-D scale tensor, got shape {scale_shape}")
        assert scale_shape[0] == shape[axis], (
            f"tensorrt.pc_{kind} (per-channel) mode expects scale size {shape[axis]} "
            f"(matching axis {axis}), got {scale_shape[0]}")
        c = shape[axis]
        inner = int(np.prod(shape[axis + 1:])) if axis + 1 < rank else 1
        if inner == 1:
            return SCALE_COL, numel // c if c else 0, c, max(numel // c, 1) if c else 1
        return SCALE_ROW, numel // inner, inner, c
    if mode == f"tensorrt.block_{kind}":
        assert axis is None, f"axis is only valid for tensorrt.pc_{kind} mode"
        assert len(scale_shape) == rank, (
            f"tensorrt.block_{kind} mode expects scale with same rank as input ({rank}), "
            f"got rank {len(scale_shape)}")
        diff_dims = [i for i in range(rank) if shape[i] != scale_shape[i]]
        assert len(diff_dims) == 1, (
            f"tensorrt.block_{kind} mode expects exactly one blocking dimension, "
            f"but found {len(diff_dims)} blocking dimensions")
        blocking_dim = diff_dims[0]
        assert blocking_dim in [rank - 1, rank - 2], (
            f"tensorrt.block_{kind} mode requires blocking dimension to be last or second-to-last, "
            f"got dimension {blocking_dim} in shape of rank {rank}")
        assert out_name in _SUPPORTED_BLOCK_QUANT_OUTPUT_DTYPES, (
            f"tensorrt.block_{kind} mode supports output_dtype to be one of {_SUPPORTED_BLOCK_QUANT_OUTPUT_DTYPES}, "
            f"got {out_name}")
        assert scale_shape[blocking_dim] > 0 and shape[blocking_dim] % scale_shape[blocking_dim] == 0, (
            f"tensorrt.block_{kind} mode expects the scale extent to divide the blocked extent, "
            f"got {shape[blocking_dim]} and {scale_shape[blocking_dim]}")
        block = shape[blocking_dim] // scale_shape[blocking_dim]
        if blocking_dim == rank - 1:        # blocks along the last axis: rows of one block each, scale[row]
            return SCALE_ROW, numel // block, block, max(numel // block, 1)
        # blocks of `block` rows along the second-to-last axis; leading axes fold into the rows
        return SCALE_COL, numel // shape[-1], shape[-1], block
    raise ValueError(f"Unknown {'quantization' if kind == 'q' else 'dequantization'} mode: {mode}")


def _scale_dev(scale, device):
    torch = _torch()
    s = np.asarray(scale.detach().cpu().numpy() if hasattr(scale, "detach") else scale, dtype=np.float32)
    return torch.from_numpy(s.reshape(-1).copy()).to(device), tuple(s.shape)


def _stream():
    return _torch().cuda.current_stream().cuda_stream


def mtrt_quantize(input, scale, *, mode, axis=None, output_dtype="int8"):
    """`tensorrt.quantize` marker: clamp(round_half_even(input / scale)) in `output_dtype`
    (int8, float8_e4m3fn, int4 or float4_e2m1fn); mode in tensorrt.{pt,pc,block}_q."""
    torch = _torch()
    out_name = _dtype_name(output_dtype)
    assert input.dtype in [torch.float16, torch.bfloat16, torch.float32], (
        f"Unsupported input dtype for quantization: {input.dtype}")
    s_dev, s_shape = _scale_dev(scale, input.device)
    kind, d0, d1, nb = _check_mode(tuple(input.shape), s_shape, mode, axis, "q", out_name)
    assert out_name in _CODE, f"Unsupported output dtype for quantization: {out_name}"
    x = input.contiguous()
    n = x.numel()
    packed = out_name in ("int4", "float4_e2m1fn")
    codes = torch.empty((n + 1) // 2 if packed else n, dtype=torch.uint8, device=x.device)
    if n:
        check(lib().mtrt_hip_quantize(_stream(), x.data_ptr(), float_dtype_of(x), codes.data_ptr(), _CODE[out_name],
                                      s_dev.data_ptr(), kind, d0, d1, nb, 0))
    return QuantizedArray(codes, out_name, input.shape)


def mtrt_dequantize(input, scale, *, mode, axis=None, output_dtype="float32"):
    """`tensorrt.dequantize` marker: input * scale in `output_dtype`; mode in tensorrt.{pt,pc,block}_dq.
    `scale` may be a device tensor (the block scales a dynamic quantization produced)."""
    torch = _torch()
    qa = _as_quantized(input)
    out_t = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}.get(_dtype_name(output_dtype))
    assert out_t is not None, f"Unsupported output dtype for dequantization: {output_dtype}"
    if hasattr(scale, "is_cuda") and scale.is_cuda:
        s_dev, s_shape = scale.to(torch.float32).contiguous().reshape(-1), tuple(scale.shape)
    else:
        s_dev, s_shape = _scale_dev(scale, qa.codes.device)
    kind, d0, d1, nb = _check_mode(qa.shape, s_shape, mode, axis, "dq", qa.dtype)
    y = torch.empty(qa.shape, dtype=out_t, device=qa.codes.device)
    if y.numel():
        check(lib().mtrt_hip_dequantize(_stream(), qa.codes.data_ptr(), _CODE[qa.dtype], y.data_ptr(), float_dtype_of(y),
                                        s_dev.data_ptr(), kind, d0, d1, nb))
    return y


def mtrt_dynamic_quantize(input, double_quant_scale, *, axis, block_size=16, output_dtype="float4_e2m1fn",
                          scale_dtype="float8_e4m3fn"):
    """`tensorrt.dynamic_quantize` marker (NVFP4): returns (float4 codes, float8 block scales); the block scale
    is quantized against `double_quant_scale`, the per-tensor second-level scale (tensor amax / 2688)."""
    torch = _torch()
    rank = input.dim()
    assert axis is not None, "axis is required for dynamic quantization"
    assert axis in [rank - 1, rank - 2], (
        f"axis must be the last dimension or the second to last dimension, " f"got {axis}")
    assert block_size == 16, "currently only blocks of 16 elements are supported"
    dqs = np.asarray(double_quant_scale, dtype=np.float32)
    assert dqs.shape == (), f"`double_quant_scale` is expected to be scalar, got shape {dqs.shape}"
    assert input.shape[axis] % block_size == 0, (
        f"Input shape[{axis}]={input.shape[axis]} must be divisible by block_size={block_size}")
    assert _dtype_name(output_dtype) == "float4_e2m1fn", (
        f"dynamic quantization supports output_dtype to be one of ['float4_e2m1fn'], got {output_dtype}")
    assert _dtype_name(scale_dtype) == "float8_e4m3fn", (
        f"dynamic quantization supports scale_dtype to be one of ['float8_e4m3fn'], got {scale_dtype}")
    assert input.dtype in [torch.float16, torch.bfloat16, torch.float32], (
        f"Unsupported input dtype for dynamic quantization: {input.dtype}")
    amax = torch.tensor(float(np.float32(dqs) * np.float32(2688.0)), dtype=torch.float32, device=input.device)
    q, s = nvfp4_quantize(input.contiguous(), amax, axis=axis - rank)
    return QuantizedArray(q, "float4_e2m1fn", input.shape), QuantizedArray(s.reshape(-1), "float8_e4m3fn", s.shape)


def custom_call(call_target_name, operands, mode=None, axis=None, **attrs):
    """`stablehlo.custom_call @<call_target_name>` with the attribute names the JAX lowerings attach."""
    if call_target_name == "tensorrt.quantize":
        return mtrt_quantize(operands[0], operands[1], mode=mode, axis=axis, output_dtype=attrs.get("output_dtype", "int8"))
    if call_target_name == "tensorrt.dequantize":
        return mtrt_dequantize(operands[0], operands[1], mode=mode, axis=axis,
                               output_dtype=attrs.get("output_dtype", "float32"))
    if call_target_name == "tensorrt.dynamic_quantize":
        return mtrt_dynamic_quantize(operands[0], operands[1], axis=axis, block_size=attrs.get("block_size", 16))
    raise ValueError(f"Unknown custom call target: {call_target_name}")


def composite(name, operand, scale, axis=-1, **attrs):
    """`stablehlo.composite "<name>"` with attributes {scale, axis} (StablehloRaiseQDQ.cpp:98-110): axis is -1 for
    the per-tensor and block forms, the channel axis for tensorrt.pc_q / pc_dq."""
    if not name.startswith("tensorrt.") or name.split(".")[1] not in ("pt_q", "pc_q", "block_q", "pt_dq", "pc_dq", "block_dq"):
        raise ValueError(f"Unknown composite: {name}")
    ax = axis if name.split(".")[1].startswith("pc_") else None
    if name.endswith("_dq"):
        return mtrt_dequantize(operand, scale, mode=name, axis=ax, output_dtype=attrs.get("output_dtype", "float32"))
    return mtrt_quantize(operand, scale, mode=name, axis=ax, output_dtype=attrs.get("output_dtype", "int8"))
