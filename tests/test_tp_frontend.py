"""Validation behaviour of the Tripy-compatible quantize / dequantize / Linear mirror; CPU only.

The cases and the expected message fragments are those of the reference's own front-end tests:
  tripy/tests/frontend/ops/test_quantize.py:24-85
  tripy/tests/frontend/ops/test_dequantize.py:24-84
  tripy/tests/integration/test_linear.py:88-100 (Linear parameter rejection)
  tripy/tests/frontend/module/test_layernorm.py:22-45 (LayerNorm shape and rank rejection)
No kernel is launched: every case fails validation before any device work.
"""
import importlib
import re

import numpy as np
import pytest


@pytest.fixture(scope="module")
def tp(pkg):
    return importlib.import_module(pkg.__name__ + ".tp")


def raises(tp, match):
    return pytest.raises(tp.TripyException, match=re.escape(match))


class TestQuantize:
    def test_invalid_input_dtype(self, tp):
        a = tp.Tensor([1, 2])
        with raises(tp, "Invalid inputs for function: 'quantize'."):
            tp.quantize(a, 1, tp.int8)

    def test_unsupported_quant_dtype(self, tp):
        a = tp.Tensor([1.0, 2.0])
        with raises(tp, "Invalid inputs for function: 'quantize'."):
            tp.quantize(a, 1, tp.float16)

    def test_scale_dtype_mismatch(self, tp):
        a = tp.Tensor(np.ones((2,), dtype=np.float16))
        with raises(tp, "Invalid inputs for function: 'quantize'."):
            tp.quantize(a, tp.Tensor(np.float32(1.0)), tp.int8)

    def test_invalid_scale_per_channel(self, tp):
        a = tp.ones((4, 4))
        with raises(tp, "If dim is given, scale must be a 1-D tensor in per-channel quantize op"):
            tp.quantize(a, 0.5, tp.int8, dim=0)

    def test_invalid_input_blockwise(self, tp):
        a = tp.ones((4,))
        scale = tp.Tensor(np.ones((2, 4), dtype=np.float32))
        with raises(tp, "Input must be a 2-D tensor in block-wise quantize op"):
            tp.quantize(a, scale, tp.int4)

    def test_unsupported_blockwise_dtype(self, tp):
        a = tp.ones((4, 4))
        scale = tp.Tensor(np.ones((2, 4), dtype=np.float32))
        with raises(tp, "Unsupported data type in block-wise quantize op"):
            tp.quantize(a, scale, tp.int8)

    def test_invalid_scale_per_tensor(self, tp):
        a = tp.ones((4, 4))
        scale = tp.Tensor([0.5] * 4)
        with raises(tp, "Scale must be a scalar tensor in per-tensor quantize op"):
            tp.quantize(a, scale, tp.int8)

    def test_non_constant_scale(self, tp):
        a = tp.ones((4, 4))
        scale = tp.ones((4,))
        with raises(tp, "`scale` argument must be a constant"):
            tp.quantize(a, scale, tp.int8, dim=0)

    def test_per_channel_scale_size(self, tp):
        # tensorrt.quantize verifier: scale size must equal input.shape[axis]
        # (mlir-tensorrt/tensorrt/lib/TensorRT/IR/Verification.cpp:1182-1265)
        a = tp.ones((4, 3))
        with raises(tp, "Scale size must match the size of the quantization axis"):
            tp.quantize(a, [1.0, 1.0, 1.0], tp.int8, dim=0)

    def test_block_scale_shape(self, tp):
        a = tp.ones((6, 4))
        with raises(tp, "Scale shape does not divide the input in block-wise quantize op"):
            tp.quantize(a, tp.Tensor(np.ones((4, 4), dtype=np.float32)), tp.int4)


class TestDequantize:
    def test_invalid_input_dtype(self, tp):
        a = tp.Tensor([1.0, 2.0])
        with raises(tp, "Invalid inputs for function: 'dequantize'."):
            tp.dequantize(a, 0.9, tp.float32)

    def test_invalid_dequant_dtype(self, tp):
        a = tp.ones([2], dtype=tp.int8)
        with raises(tp, "Invalid inputs for function: 'dequantize'."):
            tp.dequantize(a, 1, tp.int32)

    def test_invalid_scale_per_channel(self, tp):
        a = tp.ones([2], dtype=tp.int8)
        with raises(tp, "If dim is given, scale must be a 1-D tensor in per-channel dequantize op"):
            tp.dequantize(a, 0.5, tp.float32, dim=0)

    def test_invalid_input_blockwise(self, tp):
        a = tp.Tensor(np.ones((4,), dtype=np.int8))
        scale = tp.Tensor(np.ones((2, 4), dtype=np.float32))
        with raises(tp, "Input must be a 2-D tensor in block-wise dequantize op"):
            tp.dequantize(a, scale, tp.float32)

    def test_unsupported_blockwise_dtype(self, tp):
        a = tp.Tensor(np.ones((4, 4), dtype=np.int8))
        scale = tp.Tensor(np.ones((2, 4), dtype=np.float32))
        with raises(tp, "Unsupported data type in block-wise dequantize op"):
            tp.dequantize(a, scale, tp.float32)

    def test_invalid_scale_per_tensor(self, tp):
        a = tp.Tensor(np.ones((4, 4), dtype=np.int8))
        scale = tp.Tensor([0.5] * 4)
        with raises(tp, "Scale must be a scalar tensor in per-tensor dequantize op"):
            tp.dequantize(a, scale, tp.float32)

    def test_non_constant_scale(self, tp):
        a = tp.ones((4, 4), dtype=tp.int8)
        scale = tp.ones((4,))
        with raises(tp, "`scale` argument must be a constant"):
            tp.dequantize(a, scale, tp.float32, dim=0)


class TestQuantLinear:
    def test_input_scale_with_weight_quant_dim_1(self, tp):
        lin = tp.Linear(4, 2, quant_dtype=tp.int8, weight_quant_dim=1)
        lin.weight_scale = tp.Tensor([1.0] * 4)
        lin.input_scale = tp.Tensor(1.0)
        with raises(tp, "Unsupported quantization parameters for Linear module."):
            lin(tp.ones((3, 4)))


def test_scale_addressing_modes(tp):
    """The three modes map onto the C ABI's scale addressing as documented in include/mtrt_hip.h."""
    from_shape = tp._scale_addressing
    pkg = importlib.import_module(tp.__name__.rsplit(".", 1)[0])
    s1 = tp.Tensor(np.ones((5,), dtype=np.float32))
    # per-channel on the last axis: scale[col]
    assert from_shape((3, 4, 5), s1, 2, "quantize op") == (pkg.SCALE_COL, 12, 5, 12)
    assert from_shape((3, 4, 5), s1, -1, "quantize op") == (pkg.SCALE_COL, 12, 5, 12)
    # per-channel on a middle axis: rows of `inner` elements, scale[row % C]
    s4 = tp.Tensor(np.ones((4,), dtype=np.float32))
    assert from_shape((3, 4, 5), s4, 1, "quantize op") == (pkg.SCALE_ROW, 12, 5, 4)
    s3 = tp.Tensor(np.ones((3,), dtype=np.float32))
    assert from_shape((3, 4, 5), s3, 0, "quantize op") == (pkg.SCALE_ROW, 3, 20, 3)
    # blocks of D0/S0 rows along axis 0
    sb = tp.Tensor(np.ones((32, 64), dtype=np.float32))
    assert from_shape((4096, 64), sb, None, "quantize op") == (pkg.SCALE_COL, 4096, 64, 128)
    # per-tensor
    s0 = tp.Tensor(np.float32(1.0))
    assert from_shape((7, 9), s0, None, "quantize op") == (pkg.SCALE_UNIFORM, 7, 9, 1)
    assert from_shape((), s0, None, "quantize op")[0] == pkg.SCALE_UNIFORM


class TestLayerNormAndSoftmax:
    def test_layernorm_improper_dimensions(self, tp):
        ln = tp.LayerNorm(normalized_shape=[2, 2])
        ln.initialize_dummy_parameters()
        with raises(tp, "The normalization scale is not broadcast-compatible with the input at dimension 1"):
            ln(tp.ones((5, 5, 5)))

    def test_layernorm_improper_rank(self, tp):
        ln = tp.LayerNorm(normalized_shape=[2])
        ln.initialize_dummy_parameters()
        x = tp.ones((2,))
        with raises(tp, f"Input must have a rank of at least 2, but got input of rank: {x.rank}"):
            ln(x)

    def test_layernorm_parameters_and_dtypes(self, tp):
        ln = tp.LayerNorm(3)
        assert ln.normalized_shape == (3,) and ln.eps == 1e-5 and ln.dtype == tp.float32
        assert isinstance(ln.weight, tp.DefaultParameter) and ln.weight.shape == (3,)
        with raises(tp, "Parameter 'weight' of LayerNorm has not been set."):
            ln(tp.ones((2, 3)))
        ln.initialize_dummy_parameters()
        with raises(tp, "Invalid inputs for function: 'layernorm'."):
            ln(tp.ones((2, 3), dtype=tp.float16))             # weight dtype differs from the input's
        with raises(tp, "Invalid inputs for function: 'layernorm'."):
            tp.layernorm(tp.Tensor([[1, 2, 3]]), ln.weight, ln.bias, 1e-5)   # int32 input

    def test_softmax_rejections(self, tp):
        with raises(tp, "Invalid inputs for function: 'softmax'."):
            tp.softmax(tp.Tensor([[1, 2]]), dim=0)
        with raises(tp, "Dimension argument is out of bounds."):
            tp.softmax(tp.ones((2, 2)), dim=2)
        with raises(tp, "Dimension argument is out of bounds."):
            tp.softmax(tp.ones((2,)), dim=-3)              # a rank-1 input is seen as (2, 1): [-2, 2) is valid
