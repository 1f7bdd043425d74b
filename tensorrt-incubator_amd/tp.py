"""Host-side mirror of the Tripy quantization surface over libmtrt_hip.so.

What is mirrored (names, argument meaning, validation order and error text):

  quantize(input, scale, dtype, dim=None)    tripy/nvtripy/frontend/ops/quantize.py:32-119
  dequantize(input, scale, dtype, dim=None)  tripy/nvtripy/frontend/ops/dequantize.py:32-114
  check_qdq_args                             tripy/nvtripy/frontend/ops/utils.py:179-256
  cast (the float8 / int4 routes)            tripy/nvtripy/frontend/ops/cast.py:67-84
  Linear (fake-quant forward)                tripy/nvtripy/frontend/module/linear.py:112-151
  layernorm / LayerNorm                      tripy/nvtripy/frontend/module/layernorm.py:36-156
  softmax(input, dim=None)                   tripy/nvtripy/frontend/ops/softmax.py:30-82
  scale from calibration amax                tripy/examples/nanogpt/weight_loader.py:67-68

Tripy builds a trace and hands `tensorrt.quantize` / `tensorrt.dequantize` to TensorRT
(tripy/nvtripy/trace/ops/quantize.py:27-46).  Here every call runs at once: the wrapper
maps (input shape, scale shape, dim) to the scale addressing of the C ABI and launches
the gfx950 cluster on the current stream.  torch owns the device memory; nothing else of
it is used on the quantization path.  Without the library or a gfx950 device the calls
raise: there is no other path.

Storage of the quantized types: int8 as int8; float8 as the e4m3fn byte; int4 one code per
byte in the low nibble (the executor's buffer form,
mlir-tensorrt/executor/lib/Runtime/Backend/Common/DataTypes.cpp:494-519).
"""
import numbers

import numpy as np

from . import (BF16, F16, F32, F8E4M3FN, I4, I8, SCALE_COL, SCALE_ROW, SCALE_UNIFORM, check, lib)


class TripyException(Exception):
    """tripy/nvtripy/common/exception.py:26-31"""


def raise_error(summary, details=None):
    """Summary first, then the details joined, as tripy/nvtripy/common/exception.py:123-170 prints them
    (source-code excerpts of the reference's message are left out)."""
    raise TripyException(summary + "".join("\n    " + str(d) if i == 0 else str(d) for i, d in enumerate(details or [])))


class dtype:
    def __init__(self, name, code, itemsize, np_dtype=None):
        self.name, self.code, self.itemsize, self.np_dtype = name, code, itemsize, np_dtype

    def __repr__(self):
        return self.name

    __str__ = __repr__


float32 = dtype("float32", F32, 4, np.float32)
float16 = dtype("float16", F16, 2, np.float16)
bfloat16 = dtype("bfloat16", BF16, 2)
int8 = dtype("int8", I8, 1, np.int8)
int4 = dtype("int4", I4, 1)
float8 = dtype("float8", F8E4M3FN, 1)
int32 = dtype("int32", None, 4, np.int32)

# tripy/nvtripy/frontend/ops/utils.py:183-184
QUANTIZABLE_DTYPES = (float32, float16, bfloat16)
QUANTIZED_DTYPES = (int8, int4, float8)


def is_quantized_dtype(d):
    return d in QUANTIZED_DTYPES


def _torch():
    import torch
    return torch


def _torch_dtype(d):
    torch = _torch()
    return {float32: torch.float32, float16: torch.float16, bfloat16: torch.bfloat16, int8: torch.int8,
            int4: torch.int8, float8: torch.uint8, int32: torch.int32}[d]


def _from_torch_dtype(td):
    torch = _torch()
    table = {torch.float32: float32, torch.float16: float16, torch.bfloat16: bfloat16, torch.int8: int8,
             torch.int32: int32, torch.int64: int32, torch.float64: float32}
    if td not in table:
        raise_error("Unsupported data type.", ["Got: %s" % td])
    return table[td]


class Tensor:
    """A value with a Tripy dtype.  `is_cpu_constant` is what the reference reads off the trace:
    the tensor was made from host data and has not gone through an operation
    (`isinstance(scale.trace_tensor.producer, Constant) and producer.device.kind == "cpu"`,
    utils.py:246)."""

    def __init__(self, data, dtype=None, _produced=False, _tp_dtype=None):
        torch = _torch()
        if isinstance(data, Tensor):
            self._t, self.dtype, self.is_cpu_constant = data._t, data.dtype, data.is_cpu_constant
            return
        if _produced:
            self._t, self.dtype, self.is_cpu_constant = data, _tp_dtype, False
            return
        if isinstance(data, np.ndarray):
            t = torch.from_numpy(data if data.flags.c_contiguous else data.copy(order="C"))
        elif isinstance(data, torch.Tensor):
            t = data
        else:
            t = torch.tensor(data)
        want = dtype if dtype is not None else _from_torch_dtype(t.dtype)
        if want in (int4, float8):
            raise_error("Tensors of a quantized type are made with cast or quantize.", ["Got dtype=%s" % want])
        t = t.to(_torch_dtype(want))
        self.is_cpu_constant = not t.is_cuda
        self._t, self.dtype = t, want

    @property
    def shape(self):
        return tuple(self._t.shape)

    @property
    def rank(self):
        return self._t.dim()

    def device_data(self):
        """The values in device memory (uploaded once)."""
        if not self._t.is_cuda:
            self._t = self._t.cuda()
        return self._t

    def torch(self):
        """A torch view of the stored values (codes for int4 / float8)."""
        return self._t

    def __repr__(self):
        return "tensor(shape=%s, dtype=%s)" % (self.shape, self.dtype)


def _produced(t, d):
    return Tensor(t, _produced=True, _tp_dtype=d)


def ones(shape, dtype=float32):
    """An operation result, hence not a constant (tripy/tests/frontend/ops/test_quantize.py:76-84 relies on it).
    Values are made on the host and uploaded on first use by a kernel."""
    return _produced(_torch().ones(tuple(shape), dtype=_torch_dtype(dtype)), dtype)


def zeros(shape, dtype=float32):
    return _produced(_torch().zeros(tuple(shape), dtype=_torch_dtype(dtype)), dtype)


def allclose(input, other, rtol=1e-5, atol=1e-8):
    """|input - other| <= atol + rtol * |other| everywhere (tripy/nvtripy/frontend/ops/allclose.py)."""
    torch = _torch()
    a, b = input.device_data().float(), other.device_data().float()
    return bool(torch.all(torch.abs(a - b) <= atol + rtol * torch.abs(b)))


def iota(shape, dim=0, dtype=float32):
    torch = _torch()
    shape = tuple(shape)
    idx = torch.arange(shape[dim], dtype=torch.float32)
    view = [1] * len(shape)
    view[dim] = shape[dim]
    return _produced(idx.reshape(view).expand(shape).contiguous().to(_torch_dtype(dtype)), dtype)


def _convert_scale(scale, want):
    """`convert_to_tensors={"scale"}` of the reference's interface decorator: numbers and sequences
    become constants in the dtype the input requirements ask for (wrappers.py:364-370)."""
    if isinstance(scale, Tensor):
        return scale
    if isinstance(scale, (numbers.Number, list, tuple)):
        return Tensor(np.asarray(scale, dtype=np.float64).astype(np.float32), dtype=want if want in QUANTIZABLE_DTYPES else float32)
    return Tensor(scale)


def _invalid_inputs(func, expected):
    raise_error("Invalid inputs for function: '%s'." % func, ["Expected: ", expected])


def check_qdq_args(input, scale, dtype, dim, is_quantize):
    """tripy/nvtripy/frontend/ops/utils.py:191-256, same order, same text."""
    valid_input_dtypes = QUANTIZABLE_DTYPES if is_quantize else QUANTIZED_DTYPES
    valid_target_dtypes = QUANTIZED_DTYPES if is_quantize else QUANTIZABLE_DTYPES
    op_str = "quantize op" if is_quantize else "dequantize op"

    if input.dtype not in valid_input_dtypes:
        raise_error(f"Input does not have a valid dtype in {op_str}.",
                    [f"input.dtype must be one of {valid_input_dtypes}, ", f"Got dtype={input.dtype}"])
    if dtype not in valid_target_dtypes:
        raise_error(f"Unsupported data type in {op_str}.",
                    [f"Supported data types are: {valid_target_dtypes}. ", f"Got dtype={dtype}"])

    quantizable_dtype, quantized_dtype = (input.dtype, dtype) if is_quantize else (dtype, input.dtype)
    if scale.dtype != quantizable_dtype:
        raise_error(f"Scale dtype does not match expected dtype in {op_str}.",
                    [f"scale should have dtype={quantizable_dtype}, got {scale.dtype}"])

    if dim is not None:
        if scale.rank != 1:
            raise_error(f"If dim is given, scale must be a 1-D tensor in per-channel {op_str}.",
                        [f"scale has rank={scale.rank}."])
    elif scale.rank == 2:
        if input.rank != 2:
            raise_error(f"Input must be a 2-D tensor in block-wise {op_str}.", [f"input has rank={input.rank}."])
        if quantized_dtype != int4:
            raise_error(f"Unsupported data type in block-wise {op_str}.",
                        [f"Only `tp.int4` is supported, got {quantized_dtype}"])
    elif scale.rank != 0:
        raise_error(f"Scale must be a scalar tensor in per-tensor {op_str}.", [f"scale has rank={scale.rank}."])

    if not scale.is_cpu_constant:
        raise_error("`scale` argument must be a constant in CPU memory.",
                    ["Hint: Use `scale = tp.copy(scale, tp.device('cpu'))` to copy the scale to CPU memory. "])


def _scale_addressing(shape, scale, dim, op_str):
    """(scale kind, d0, d1, nb) of the C ABI for the three modes of the op
    (mlir-tensorrt/tensorrt/include/mlir-tensorrt-dialect/TensorRT/IR/TensorRTOps.td:3133-3194;
    shape rules of mlir-tensorrt/tensorrt/lib/TensorRT/IR/Verification.cpp:1182-1265)."""
    numel = int(np.prod(shape)) if len(shape) else 1
    if dim is not None:
        rank = len(shape)
        if not -rank <= dim < rank:
            raise_error(f"Dimension argument is out of bounds in {op_str}.", [f"dim={dim}, input rank={rank}"])
        dim %= rank
        c = shape[dim]
        if scale.shape[0] != c:
            raise_error(f"Scale size must match the size of the quantization axis in per-channel {op_str}.",
                        [f"scale has {scale.shape[0]} elements, input.shape[{dim}]={c}"])
        inner = int(np.prod(shape[dim + 1:])) if dim + 1 < rank else 1
        if inner == 1:
            return SCALE_COL, numel // c if c else 0, c, max(numel // c, 1) if c else 1
        return SCALE_ROW, numel // inner, inner, c
    if scale.rank == 2:
        d0, d1 = shape
        s0, s1 = scale.shape
        if s1 != d1 or s0 == 0 or d0 % s0 != 0:
            raise_error(f"Scale shape does not divide the input in block-wise {op_str}.",
                        [f"input.shape={list(shape)}, scale.shape={list(scale.shape)}"])
        return SCALE_COL, d0, d1, d0 // s0
    d1 = shape[-1] if len(shape) else 1
    return SCALE_UNIFORM, numel // d1 if d1 else 0, d1, 1


def _scale_on_device(scale):
    """The device ABI takes f32 scales; f16 / bf16 constants widen exactly."""
    cached = getattr(scale, "_f32_dev", None)
    if cached is None:
        cached = scale.torch().to(_torch().float32).contiguous().cuda().reshape(-1)
        scale._f32_dev = cached
    return cached


def _stream():
    return _torch().cuda.current_stream().cuda_stream


def quantize(input, scale, dtype, dim=None):
    """tp.quantize: clamp(round_half_even(input / scale)) in `dtype` (int8, int4 or float8)."""
    if not isinstance(input, Tensor):
        input = Tensor(input)
    scale = _convert_scale(scale, input.dtype)
    # the interface decorator's input requirements are checked first (quantize.py:33-39)
    if input.dtype not in QUANTIZABLE_DTYPES or scale.dtype != input.dtype or dtype not in QUANTIZED_DTYPES:
        _invalid_inputs("quantize", "input.dtype to be one of [float32, float16, bfloat16], scale.dtype == input.dtype "
                                    "and dtype to be one of [int4, int8, float8]")
    check_qdq_args(input, scale, dtype, dim, True)
    kind, d0, d1, nb = _scale_addressing(input.shape, scale, dim, "quantize op")
    torch = _torch()
    x = input.device_data().contiguous()
    q = torch.empty(input.shape, dtype=_torch_dtype(dtype), device=x.device)
    if x.numel():
        check(lib().mtrt_hip_quantize(_stream(), x.data_ptr(), input.dtype.code, q.data_ptr(), dtype.code,
                                      _scale_on_device(scale).data_ptr(), kind, d0, d1, nb, 0))
    return _produced(q, dtype)


def dequantize(input, scale, dtype, dim=None):
    """tp.dequantize: input * scale in `dtype` (float32, float16 or bfloat16)."""
    if not isinstance(input, Tensor):
        input = Tensor(input)
    scale = _convert_scale(scale, dtype)
    if input.dtype not in QUANTIZED_DTYPES or dtype not in QUANTIZABLE_DTYPES or scale.dtype != dtype:
        _invalid_inputs("dequantize", "input.dtype to be one of [int4, int8, float8], dtype to be one of "
                                      "[float32, float16, bfloat16] and scale.dtype == dtype")
    check_qdq_args(input, scale, dtype, dim, False)
    kind, d0, d1, nb = _scale_addressing(input.shape, scale, dim, "dequantize op")
    torch = _torch()
    q = input.device_data().contiguous()
    y = torch.empty(input.shape, dtype=_torch_dtype(dtype), device=q.device)
    if q.numel():
        check(lib().mtrt_hip_dequantize(_stream(), q.data_ptr(), input.dtype.code, y.data_ptr(), dtype.code,
                                        _scale_on_device(scale).data_ptr(), kind, d0, d1, nb))
    return _produced(y, dtype)


def cast(input, dtype):
    """tripy/nvtripy/frontend/ops/cast.py:67-84: quantized types other than int8 convert through
    quantize / dequantize with scale 1."""
    if not isinstance(input, Tensor):
        input = Tensor(input)
    if input.dtype == dtype:
        return input
    if is_quantized_dtype(input.dtype) and input.dtype != int8:
        input = dequantize(input, 1.0, float32)
        if dtype == float32:
            return input
    if is_quantized_dtype(dtype) and dtype != int8:
        if input.dtype != float32:
            input = _produced(input.device_data().to(_torch().float32), float32)
        return quantize(input, 1.0, dtype)
    return _produced(input.device_data().to(_torch_dtype(dtype)), dtype)


def scale_from_amax(input, dtype):
    """`scale = amax / maxbound` of the calibration flow (weight_loader.py:67-68; maxbound 127, 448 or 7),
    computed on the device in one launch; returns (amax, scale) as 0-d f32 device tensors."""
    from . import amax
    qmax = {int8: 127.0, float8: 448.0, int4: 7.0}[dtype]
    return amax(input.device_data().contiguous(), qmax)


class Linear:
    """tp.Linear (linear.py:30-151): out = x @ W^T + b, with the fake-quant pair on the input and on the
    weight when `quant_dtype` is set.  weight: [out_features, in_features]; x: [*, in_features].

    Every product runs on a hand-written kernel of this library; which one follows from the parameters:

      * int8 in a float16 module, an input scale, weight scale per tensor or per output channel (dim 0): the product
        of the two dequantized operands equals (q_x . q_W^T) * s_x * s_w[n] exactly in real arithmetic, so it runs on
        the integer matrix cores (W8A8 cluster: int32 accumulation, f16 result).  The cluster writes f16, so a
        float32 or bfloat16 module keeps the literal form below: its results are not rounded to f16 on the way and
        values beyond 65504 stay finite.
      * int4 weight-only in a float16 module, weight scale per tensor or per output channel, in_features a
        multiple of 64: the W4A16 cluster dequantizes the packed codes on the way into the matrix cores.
        (The rank-2 scale of this API groups OUTPUT features, [out/B, in] as weight_loader.py:102-115 builds it;
        the W4A16 cluster's blocks run along the reduction axis, so that form takes the next route.)
      * everything else (float8 codes, scales along the input features, int4 blocks, other dtypes, no
        quantization): the literal fake-quant form, DQ(Q(x)) @ DQ(Q(W))^T on the dense Linear kernel.

    Weights are program constants: they are quantized, re-laid out and (for the last route) dequantized ONCE,
    when first needed after `weight` / `weight_scale` were assigned; the forward pass only touches x."""

    def __init__(self, in_features, out_features, bias=True, dtype=float32, quant_dtype=None, weight_quant_dim=None):
        torch = _torch()
        self.dtype = dtype
        self.weight = _produced(torch.zeros((out_features, in_features), dtype=_torch_dtype(dtype)), dtype)
        self.bias = _produced(torch.zeros((out_features,), dtype=_torch_dtype(dtype)), dtype) if bias else None
        self.quant_dtype = quant_dtype
        self.weight_quant_dim = weight_quant_dim
        self.weight_scale = None
        self.input_scale = None
        self._plan_key = None
        self._plan_owners = None
        self._plan = None

    def invalidate(self):
        """Forget the prepared weight side.  Call after changing a parameter's device memory in a way torch does not
        see (a kernel of this library writing into it, a raw pointer): assignments of new Tensors and torch's own
        in-place updates are noticed without it."""
        self._plan_key = self._plan_owners = self._plan = None

    def __call__(self, x):
        return self.forward(x)

    def load_state_dict(self, state_dict):
        """Assigns `weight`, `bias`, `weight_scale`, `input_scale` from a name -> Tensor mapping and prepares the
        weight side (quantize, re-layout) right away, as a loader does once per model."""
        for name in ("weight", "bias", "weight_scale", "input_scale"):
            if name in state_dict:
                v = state_dict[name]
                setattr(self, name, v if isinstance(v, Tensor) else Tensor(v))
        self._prepared()

    def route(self):
        """'w8a8', 'w4a16' or 'dense': the kernel family the next forward pass uses."""
        return self._prepared()["route"]

    # -- weight side, once ---------------------------------------------------------------------------
    def _prepared(self):
        torch = _torch()
        # The plan belongs to these very parameter objects (held here, so that none of them can be freed and its
        # identity handed to another object) at these versions of their storage.
        owners = (self.weight, self.weight_scale, self.input_scale)
        key = (tuple(t._t._version if isinstance(t, Tensor) else t for t in owners), self.quant_dtype, self.weight_quant_dim)
        if (self._plan is not None and self._plan_key == key and
                all(a is b for a, b in zip(self._plan_owners, owners))):
            return self._plan
        from . import gemm_w4a16_prepack, gemm_w8a8_prepack_fragments
        N, K = self.weight.shape
        plan = {"route": "dense"}
        if self.quant_dtype is None:
            plan["weight"] = self.weight.device_data().contiguous()
        else:
            has_x_scale = isinstance(self.input_scale, Tensor)
            if has_x_scale and self.weight_quant_dim == 1:
                raise_error("Unsupported quantization parameters for Linear module.",
                            ["weight_quant_dim cannot be 1 when input_scale is provided. ",
                             f"input_scale={self.input_scale}, weight_quant_dim={self.weight_quant_dim}"])
            q_weight = quantize(self.weight, self.weight_scale, self.quant_dtype, self.weight_quant_dim)
            w_scale = _convert_scale(self.weight_scale, self.dtype)
            per_out = w_scale.rank == 0 or (w_scale.rank == 1 and self.weight_quant_dim == 0)
            if self.quant_dtype == int8 and has_x_scale and per_out and self.dtype == float16:
                plan["route"] = "w8a8"
                codes = q_weight.device_data().contiguous()          # [N, K], K contiguous
                plan["s_w"] = _scale_on_device(w_scale).reshape(-1).expand(N).contiguous()
                if K % 128 == 0:
                    plan["w_frag"] = gemm_w8a8_prepack_fragments(codes, is_nk=True)
                else:
                    plan["w_nk"] = codes
            elif (self.quant_dtype == int4 and not has_x_scale and per_out and self.dtype == float16 and K % 64 == 0):
                plan["route"] = "w4a16"
                # the cluster takes [K, N] codes packed two per byte and f16 scales [K / block, N]: one block = all of K
                kn = q_weight.device_data().to(torch.uint8).bitwise_and(0xF).transpose(0, 1).contiguous().reshape(-1)
                packed = (kn[0::2] | (kn[1::2] << 4)).contiguous()
                plan["w_prepacked"] = gemm_w4a16_prepack(packed, K, N)
                plan["scale_kn"] = _scale_on_device(w_scale).reshape(-1).expand(N).to(torch.float16).reshape(1, N).contiguous()
            else:
                plan["weight"] = dequantize(q_weight, self.weight_scale, self.dtype, self.weight_quant_dim).device_data().contiguous()
        self._plan_key, self._plan_owners, self._plan = key, owners, plan
        return plan

    # -- forward ---------------------------------------------------------------------------------------
    def forward(self, x):
        from . import gemm_w4a16, gemm_w8a8, gemm_w8a8_fragments, linear_dense
        torch = _torch()
        if not isinstance(x, Tensor):
            x = Tensor(x)
        plan = self._prepared()
        N, K = self.weight.shape
        lead = x.shape[:-1]
        bias = None if self.bias is None else self.bias.device_data().contiguous()
        if plan["route"] == "w8a8":
            q_x = quantize(x, self.input_scale, int8).device_data().reshape(-1, K)
            M = q_x.shape[0]
            s_x = _scale_on_device(_convert_scale(self.input_scale, self.dtype)).reshape(-1).expand(M).contiguous()
            if "w_frag" in plan:
                y = gemm_w8a8_fragments(q_x, plan["w_frag"], s_x, plan["s_w"], N)
            else:
                y = gemm_w8a8(q_x, plan["w_nk"], s_x, plan["s_w"])
            out = y.to(_torch_dtype(self.dtype))
            if bias is not None:
                out = out + bias.unsqueeze(0)
        elif plan["route"] == "w4a16":
            a = x.device_data().reshape(-1, K).contiguous()
            out = gemm_w4a16(a, plan["scale_kn"], K, N, K, w_prepacked=plan["w_prepacked"])
            if bias is not None:
                out = out + bias.unsqueeze(0)
        else:
            if self.quant_dtype is not None and isinstance(self.input_scale, Tensor):
                x = dequantize(quantize(x, self.input_scale, self.quant_dtype), self.input_scale, self.dtype)
            a = x.device_data().reshape(-1, K).contiguous()
            out = linear_dense(a, plan["weight"], bias)
        return _produced(out.reshape(lead + (N,)), self.dtype)


# ---- fused reduce clusters -----------------------------------------------------------------------
def _check_float_input(func, input):
    if input.dtype not in (float32, float16, bfloat16):
        _invalid_inputs(func, "input.dtype to be one of [float32, float16, bfloat16] (but it was '%s')" % input.dtype)


def layernorm(input, weight, bias, eps):
    """tripy/nvtripy/frontend/module/layernorm.py:36-77: normalises over the last D = weight.rank
    dimensions, y = (x - mean) * rsqrt(var + eps) * weight + bias, in the input's dtype.  One launch of the
    LayerNorm cluster over [prod(leading dims), prod(normalized_shape)]."""
    from . import layernorm as _layernorm_rows
    for t in (input, weight, bias):
        if not isinstance(t, Tensor):
            raise_error("layernorm expects tensors.", ["Got %s" % type(t).__name__])
    _check_float_input("layernorm", input)
    if weight.dtype != input.dtype:
        _invalid_inputs("layernorm", "weight.dtype to be the same as input.dtype (but it was '%s' while input.dtype was '%s')"
                        % (weight.dtype, input.dtype))
    if bias.dtype != input.dtype:
        _invalid_inputs("layernorm", "bias.dtype to be the same as input.dtype (but it was '%s' while input.dtype was '%s')"
                        % (bias.dtype, input.dtype))
    normalized_shape = weight.shape
    D = len(normalized_shape)
    if input.rank < 2:
        raise_error(f"Input must have a rank of at least 2, but got input of rank: {input.rank}",
                    ["Input is expected to have shape (N, *) where N is the batch size, and * represents any number "
                     "of channel dimension + spatial dimensions"])
    # what the network builder reports when weight, seen as (1,) * (rank - D) + normalized_shape, does not
    # broadcast against the input (tripy/tests/frontend/module/test_layernorm.py:24-32)
    lead = input.rank - D
    if lead < 0:
        raise_error("The normalization scale has a higher rank than the input.", [f"scale rank={D}, input rank={input.rank}"])
    for i, extent in enumerate(normalized_shape):
        if extent != input.shape[lead + i]:
            raise_error(f"The normalization scale is not broadcast-compatible with the input at dimension {lead + i}",
                        [f"input has shape {input.shape}, normalized_shape is {tuple(normalized_shape)}"])
    if bias.shape != normalized_shape:
        raise_error("The normalization bias must have the shape of the scale.", [f"bias has shape {bias.shape}"])
    d = 1
    for extent in normalized_shape:
        d *= extent
    x = input.device_data().contiguous()
    y = _layernorm_rows(x.reshape(-1, d), weight.device_data().contiguous().reshape(d),
                        bias.device_data().contiguous().reshape(d), eps)
    return _produced(y.reshape(input.shape), input.dtype)


class DefaultParameter:
    """A parameter that has to be replaced with real weights before the module runs
    (tripy/nvtripy/frontend/module/parameter.py:27-34)."""

    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), dtype


class LayerNorm:
    """tripy/nvtripy/frontend/module/layernorm.py:80-156."""

    def __init__(self, normalized_shape, dtype=float32, eps=1e-5):
        if isinstance(normalized_shape, int):
            normalized_shape = (normalized_shape,)
        self.dtype = dtype
        self.normalized_shape = tuple(normalized_shape)
        self.weight = DefaultParameter(self.normalized_shape, dtype)
        self.bias = DefaultParameter(self.normalized_shape, dtype)
        self.eps = eps

    def initialize_dummy_parameters(self):
        """Fills parameters that are still placeholders (tripy/nvtripy/frontend/module/module.py, same name)."""
        if isinstance(self.weight, DefaultParameter):
            self.weight = ones(self.normalized_shape, self.dtype)
        if isinstance(self.bias, DefaultParameter):
            self.bias = zeros(self.normalized_shape, self.dtype)

    def __call__(self, x):
        return self.forward(x)

    def forward(self, x):
        for name in ("weight", "bias"):
            if isinstance(getattr(self, name), DefaultParameter):
                raise_error(f"Parameter '{name}' of LayerNorm has not been set.",
                            ["Assign real weights or call initialize_dummy_parameters() first."])
        if not isinstance(x, Tensor):
            x = Tensor(x)
        return layernorm(x, self.weight, self.bias, self.eps)


def softmax(input, dim=None):
    """tripy/nvtripy/frontend/ops/softmax.py:30-82: over `dim`, or over the flattened input when dim is None.
    The cluster works on rows; another dimension is brought last for the launch and put back."""
    from . import softmax as _softmax_rows
    if not isinstance(input, Tensor):
        input = Tensor(input)
    _check_float_input("softmax", input)
    # shapes first (softmax.py:62-76): flatten when dim is None, then at least two dimensions, then process_dim
    flatten = dim is None
    seen_shape = (int(np.prod(input.shape, dtype=np.int64)),) if flatten else input.shape
    if flatten:
        dim = 0
    if len(seen_shape) < 2:                            # the softmax layer needs two dimensions
        seen_shape = tuple(seen_shape) + (1,)
    rank = len(seen_shape)
    new_dim = dim + rank if dim < 0 else dim           # tripy/nvtripy/frontend/ops/utils.py:120-138
    if new_dim < 0 or new_dim >= rank:
        raise_error("Dimension argument is out of bounds.",
                    [f"Note: provided dimension was: {dim}, while the tensor has a rank of: {rank}.\n"
                     f"Dimension should be in the half-open interval: [{-rank}, {rank})."])
    x = input.device_data().reshape(seen_shape)
    if new_dim == rank - 1:
        y = _softmax_rows(x.contiguous())
    else:
        y = _softmax_rows(x.movedim(new_dim, -1).contiguous()).movedim(-1, new_dim).contiguous()
    return _produced(y.reshape(input.shape), input.dtype)
