"""The marker front door (mtrt_quantize / mtrt_dequantize / mtrt_dynamic_quantize, custom_call, composite).

CPU part: the shape rules and assertion messages of the JAX primitives' abstract evaluation
(mlir-tensorrt/integrations/PJRT/python/mlir_tensorrt_jax/mtrt_ops/quantize.py:44-103,
dynamic_quantize.py:41-84); every case fails before any device work.
GPU part: the literal known answers of the reference's custom-primitive tests
(mlir-tensorrt/integrations/PJRT/test/JAX/CustomPrimitives/test_quantize.py:60-83, test_dequantize.py:62-101,
test_dynamic_quantize.py), kept as data in tests/golden/jax_custom_primitives.json."""
import importlib
import json
import os

import numpy as np
import pytest

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "jax_custom_primitives.json")))


@pytest.fixture(scope="module")
def ops(pkg):
    return importlib.import_module(pkg.__name__ + ".mtrt_ops")


def test_quantize_shape_rules(ops):
    import torch
    x = torch.zeros((2, 4))
    with pytest.raises(AssertionError, match="expects scalar scale"):
        ops.mtrt_quantize(x, np.ones(2), mode="tensorrt.pt_q")
    with pytest.raises(AssertionError, match="axis is only valid for tensorrt.pc_q mode"):
        ops.mtrt_quantize(x, np.array(1.0), mode="tensorrt.pt_q", axis=0)
    with pytest.raises(AssertionError, match="tensorrt.pc_q mode requires axis"):
        ops.mtrt_quantize(x, np.ones(2), mode="tensorrt.pc_q")
    with pytest.raises(AssertionError, match=r"requires axis to be in range \[0, 2\)"):
        ops.mtrt_quantize(x, np.ones(2), mode="tensorrt.pc_q", axis=2)
    with pytest.raises(AssertionError, match="expects 1-D scale tensor"):
        ops.mtrt_quantize(x, np.ones((2, 1)), mode="tensorrt.pc_q", axis=0)
    with pytest.raises(AssertionError, match=r"expects scale size 2 \(matching axis 0\), got 4"):
        ops.mtrt_quantize(x, np.ones(4), mode="tensorrt.pc_q", axis=0)
    with pytest.raises(AssertionError, match="expects scale with same rank as input"):
        ops.mtrt_quantize(x, np.ones(4), mode="tensorrt.block_q", output_dtype="int4")
    with pytest.raises(AssertionError, match="exactly one blocking dimension, but found 2"):
        ops.mtrt_quantize(x, np.ones((1, 2)), mode="tensorrt.block_q", output_dtype="int4")
    with pytest.raises(AssertionError, match="blocking dimension to be last or second-to-last"):
        ops.mtrt_quantize(torch.zeros((4, 2, 4)), np.ones((2, 2, 4)), mode="tensorrt.block_q", output_dtype="int4")
    with pytest.raises(AssertionError, match="tensorrt.block_q mode supports output_dtype to be one of"):
        ops.mtrt_quantize(x, np.ones((1, 4)), mode="tensorrt.block_q", output_dtype="int8")
    with pytest.raises(ValueError, match="Unknown quantization mode"):
        ops.mtrt_quantize(x, np.array(1.0), mode="tensorrt.q")
    with pytest.raises(AssertionError, match="Unsupported input dtype for quantization"):
        ops.mtrt_quantize(torch.zeros((2, 4), dtype=torch.int32), np.array(1.0), mode="tensorrt.pt_q")


def test_dynamic_quantize_rules(ops):
    import torch
    x = torch.zeros((2, 32))
    with pytest.raises(AssertionError, match="axis must be the last dimension or the second to last dimension"):
        ops.mtrt_dynamic_quantize(torch.zeros((2, 2, 32)), 1.0, axis=0)
    with pytest.raises(AssertionError, match="only blocks of 16 elements"):
        ops.mtrt_dynamic_quantize(x, 1.0, axis=1, block_size=32)
    with pytest.raises(AssertionError, match="expected to be scalar"):
        ops.mtrt_dynamic_quantize(x, np.ones(2), axis=1)
    with pytest.raises(AssertionError, match=r"Input shape\[1\]=24 must be divisible by block_size=16"):
        ops.mtrt_dynamic_quantize(torch.zeros((2, 24)), 1.0, axis=1)
    with pytest.raises(AssertionError, match="Unsupported input dtype for dynamic quantization"):
        ops.mtrt_dynamic_quantize(torch.zeros((2, 32), dtype=torch.int8), 1.0, axis=1)
    with pytest.raises(ValueError, match="Unknown custom call target"):
        ops.custom_call("tensorrt.softmax", [x, 1.0])
    with pytest.raises(ValueError, match="Unknown composite"):
        ops.composite("tensorrt.pt_x", x, 1.0)


@pytest.mark.gpu
def test_quantize_known_answers(ops):
    import torch
    g = GOLD["quantize_pt"]
    x = torch.tensor(g["x"], dtype=torch.float32, device="cuda")
    q = ops.mtrt_quantize(x, np.array(g["scale"]), mode="tensorrt.pt_q", output_dtype="int8")
    assert np.array_equal(q.torch().cpu().numpy(), np.array(g["expected"], dtype=np.int8))
    g = GOLD["quantize_pc"]
    x = torch.tensor(g["x"], dtype=torch.float32, device="cuda")
    q = ops.custom_call("tensorrt.quantize", [x, np.array(g["scale"])], mode="tensorrt.pc_q", axis=g["axis"])
    assert np.array_equal(q.torch().cpu().numpy(), np.array(g["expected"], dtype=np.int8))
    q = ops.composite("tensorrt.pc_q", x, np.array(g["scale"]), axis=g["axis"])
    assert np.array_equal(q.torch().cpu().numpy(), np.array(g["expected"], dtype=np.int8))
    g = GOLD["quantize_block"]
    x = torch.tensor(g["x"], dtype=torch.float32, device="cuda")
    q = ops.mtrt_quantize(x, np.array(g["scale"]), mode="tensorrt.block_q", output_dtype="float8_e4m3fn")
    got = q.torch().float().cpu().numpy()
    # the reference builds `expected` as a float8_e4m3fn array: the literal is rounded to that type (50 -> 48, 70 -> 72)
    expected = torch.tensor(g["expected"], dtype=torch.float32).to(torch.float8_e4m3fn).float().numpy()
    np.testing.assert_allclose(got, expected, rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_dequantize_known_answers(ops):
    import torch
    g = GOLD["dequantize_pt"]
    x = torch.tensor(g["x"], dtype=torch.int8, device="cuda")
    y = ops.mtrt_dequantize(x, np.array(g["scale"]), mode="tensorrt.pt_dq", output_dtype=np.float32)
    np.testing.assert_allclose(y.cpu().numpy(), np.array(g["expected"], dtype=np.float32), atol=1e-5, rtol=1e-7)
    g = GOLD["dequantize_pc"]
    y = ops.mtrt_dequantize(x, np.array(g["scale"]), mode="tensorrt.pc_dq", axis=g["axis"], output_dtype=np.float32)
    np.testing.assert_allclose(y.cpu().numpy(), np.array(g["expected"], dtype=np.float32), atol=1e-5, rtol=1e-7)
    g = GOLD["dequantize_block"]
    x8 = torch.tensor(g["x"], dtype=torch.float32).to(torch.float8_e4m3fn).cuda()
    y = ops.composite("tensorrt.block_dq", x8, np.array(g["scale"]))
    np.testing.assert_allclose(y.cpu().numpy(), np.array(g["expected"], dtype=np.float32), atol=1e-5, rtol=1e-7)


@pytest.mark.gpu
def test_dynamic_quantize_known_answer(ops):
    """NVFP4 with double_quant_scale 1: the quantize -> dequantize-scales -> block-dequantize chain of the
    reference's test, expected values as its literal array."""
    import torch
    g = GOLD["dynamic_quantize_pt"]
    x = torch.tensor(g["x"], dtype=torch.float32, device="cuda")
    dqs = np.array(g["double_quant_scale"])
    fp4_out, fp8_scale = ops.mtrt_dynamic_quantize(x, dqs, axis=g["axis"])
    assert fp4_out.dtype == "float4_e2m1fn" and fp8_scale.shape == (2, 2)
    scales = ops.mtrt_dequantize(fp8_scale, dqs, mode="tensorrt.pt_dq", output_dtype=np.float32)
    out = ops.mtrt_dequantize(fp4_out, scales, mode="tensorrt.block_dq", output_dtype=np.float32)
    np.testing.assert_allclose(out.cpu().numpy(), np.array(g["expected"], dtype=np.float32), rtol=1e-6, atol=0)


@pytest.mark.gpu
def test_dynamic_quantize_along_the_second_to_last_axis(ops, orc):
    """axis = rank - 2: the same chain as the reference's test on the transposed input gives the transposed result."""
    import torch
    g = GOLD["dynamic_quantize_pt"]
    x = torch.tensor(g["x"], dtype=torch.float32).t().contiguous().cuda()           # [32, 2]: blocks down the rows
    x4 = torch.cat([x, x, x, x], dim=1).contiguous()                                   # [32, 8]: whole vectors
    dqs = np.array(1.0)
    fp4_out, fp8_scale = ops.mtrt_dynamic_quantize(x4, dqs, axis=0)
    assert fp8_scale.shape == (2, 8)
    scales = ops.mtrt_dequantize(fp8_scale, dqs, mode="tensorrt.pt_dq", output_dtype=np.float32)
    out = ops.mtrt_dequantize(fp4_out, scales, mode="tensorrt.block_dq", output_dtype=np.float32)
    expected = np.array(g["expected"], dtype=np.float32).T
    np.testing.assert_allclose(out.cpu().numpy(), np.concatenate([expected] * 4, axis=1), rtol=1e-6, atol=0)


@pytest.mark.gpu
def test_block_modes_on_both_axes_against_oracle(ops, orc):
    """block_q / block_dq with int4 and float4 codes, blocks along the last and the second-to-last axis,
    with a leading batch axis; bit-exact against the oracle addressed per element."""
    import torch
    from helpers import rng
    r = rng(91)
    for out_name, o_q in (("int4", orc.I4_PACKED), ("float4_e2m1fn", orc.F4_PACKED), ("float8_e4m3fn", orc.F8E4M3FN)):
        for shape, sshape in (((3, 64, 48), (3, 2, 48)), ((3, 8, 128), (3, 8, 4))):
            x = (r.standard_normal(shape) * 2).astype(np.float32)
            s = r.uniform(0.3, 1.2, sshape).astype(np.float32)
            reps = [shape[i] // sshape[i] for i in range(3)]
            full = np.repeat(np.repeat(s, reps[1], axis=1), reps[2], axis=2)
            n = x.size
            q_ref = orc.quantize(x.ravel(), orc.F32, o_q, full.ravel(), orc.SCALE_ROW, n, 1, n) if o_q == orc.F8E4M3FN else None
            if q_ref is None:
                # packed nibbles: element pairs share a byte, so quantize the flat array in one row with per-column scales
                q_ref = orc.quantize(x.ravel(), orc.F32, o_q, full.ravel(), orc.SCALE_COL, 1, n, 1)
            q = ops.mtrt_quantize(torch.from_numpy(x).cuda(), s, mode="tensorrt.block_q", output_dtype=out_name)
            assert np.array_equal(q.codes.cpu().numpy(), q_ref.view(np.uint8)), (out_name, shape)
            y = ops.mtrt_dequantize(q, s, mode="tensorrt.block_dq", output_dtype="float32")
            y_ref = (orc.dequantize(q_ref, o_q, orc.F32, full.ravel(), orc.SCALE_COL, 1, n, 1))
            assert np.array_equal(y.cpu().numpy().ravel().view(np.uint32), y_ref.view(np.uint32)), (out_name, shape)
