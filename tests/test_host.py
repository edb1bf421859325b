"""Host-side mirror of the reference interface: enums, configs, containers, frontends'
argument handling (no GPU needed)."""

import numpy as np
import pytest
import torch
import torch.nn as nn

import fouroversix_amd as fos
from fouroversix_amd.quantize import from_blocked, to_blocked
from fouroversix_amd.utils import ScaleType


def test_enum_tables():
    assert fos.DataType.nvfp4.block_size == 16 and fos.DataType.mxfp4.block_size == 32
    assert fos.DataType.bfloat16.torch_dtype == torch.bfloat16 and fos.DataType.nvfp4.torch_dtype is None
    assert fos.DataType.nvfp4.supported_scale_rules == set(fos.ScaleRule)
    assert fos.DataType.if4.supported_scale_rules == {fos.ScaleRule.mse, fos.ScaleRule.mae, fos.ScaleRule.abs_max}
    assert fos.DataType.nvint4.supported_scale_rules == {fos.ScaleRule.static_6}
    assert [r.cuda_id for r in (fos.ScaleRule.static_6, fos.ScaleRule.static_4, fos.ScaleRule.mae,
                                fos.ScaleRule.mse, fos.ScaleRule.abs_max)] == [0, 1, 2, 3, 4]
    vt = fos.DataType.nvfp4.quantized_value_type
    assert vt.get_maximum_value(fos.ScaleRule.static_4) == 4 and vt.get_maximum_value(fos.ScaleRule.mse) == 6
    assert vt.packing_factor == 2
    assert ScaleType.nv.get_maximum_value(fos.ScaleRule.mse) == 256
    assert ScaleType.nv.get_maximum_value(fos.ScaleRule.static_6) == 448
    assert ScaleType.nv_if.get_maximum_value(fos.ScaleRule.mse) == 448
    assert fos.RoundStyle.stochastic_unbiased.adjustment_factor == 16 / 17
    assert fos.RoundStyle.stochastic.is_stochastic and not fos.RoundStyle.nearest.is_stochastic


def test_config_defaults_and_coercion():
    c = fos.QuantizationConfig()
    assert (c.dtype, c.scale_rule, c.round_style, c.block_scale_2d) == (
        fos.DataType.nvfp4, fos.ScaleRule.mse, fos.RoundStyle.nearest, False)
    c = fos.QuantizationConfig(dtype="if4", scale_rule="mae", round_style="stochastic", backend="pytorch")
    assert c.dtype is fos.DataType.if4 and c.scale_rule is fos.ScaleRule.mae
    assert c.round_style is fos.RoundStyle.stochastic and c.backend is fos.QuantizeBackend.pytorch
    m = fos.ModelQuantizationConfig(weight_scale_2d=True, activation_scale_rule="static_6",
                                    module_config_overrides={"a": {"scale_rule": "static_4"}})
    assert m.get_weight_config().block_scale_2d and m.get_weight_config().scale_rule is fos.ScaleRule.mse
    assert m.get_activation_config().scale_rule is fos.ScaleRule.static_6
    assert m.get_module_config("a").weight_scale_rule is fos.ScaleRule.static_4
    assert m.get_module_config("b") is m
    assert m.get_weight_config(scale_rule="static_6").scale_rule is fos.ScaleRule.static_6
    assert m.modules_to_not_convert == ["lm_head"]


def test_quantize_rejects_unsupported():
    x = torch.zeros(128, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="No backend found"):
        fos.quantize(x)  # CPU tensor
    with pytest.raises(ValueError, match="No backend found"):
        fos.quantize(torch.zeros(2, 128, 64, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="No backend found"):
        fos.quantize(x, fos.QuantizationConfig(dtype="if4", scale_rule="static_6"))
    with pytest.raises(ValueError, match="Backend .* does not support"):
        fos.quantize(x, fos.QuantizationConfig(backend="cuda", dtype="mxfp4", scale_rule="static_6"))


def test_quantized_tensor_padding_rules():
    v = torch.zeros(100, 40, dtype=torch.uint8)
    sf = torch.full((100, 5), 0x38, dtype=torch.uint8).view(torch.float8_e4m3fn)
    q = fos.QuantizedTensor(v, sf, torch.ones(()), "nvfp4", torch.Size((100, 80)), "mse", "nearest")
    assert q.padded_shape == (128, 128) and q.values.shape == (128, 64)
    assert q.scale_factors.shape == (128 * 8,) and q.scale_factors_are_in_blackwell_layout
    rows = from_blocked(q.scale_factors, (128, 8)).view(torch.uint8)
    assert (rows[:100, :5] == 0x38).all() and rows[100:].sum() == 0 and rows[:, 5:].sum() == 0
    q = fos.QuantizedTensor(torch.zeros(128, 32, dtype=torch.uint8), torch.zeros(512, dtype=torch.uint8),
                            torch.ones(()), fos.DataType.if4, (128, 64), fos.ScaleRule.mse, fos.RoundStyle.nearest,
                            scale_factors_are_in_blackwell_layout=False)
    assert q.padded_shape == (128, 64)
    with pytest.raises(ValueError, match="scale factors"):
        fos.QuantizedTensor(torch.zeros(128, 32, dtype=torch.uint8), torch.zeros(100, dtype=torch.uint8),
                            torch.ones(()), "nvfp4", (128, 64), "mse", "nearest")
    q = fos.QuantizedTensor(v, sf, torch.ones(()), "nvfp4", (100, 80), "mse", "nearest", (128, 128))
    assert q.values is v  # an explicit padded shape means "trust the buffers"


def test_layout_helpers_round_trip():
    a = torch.arange(256 * 8, dtype=torch.int32).to(torch.uint8).reshape(256, 8)
    ref = a.view(2, 128, 2, 4).transpose(1, 2).reshape(-1, 4, 32, 4).transpose(1, 2).reshape(-1, 32, 16).flatten()
    assert torch.equal(to_blocked(a), ref)
    assert torch.equal(from_blocked(ref, (256, 8)), a)
    f8 = a.view(torch.float8_e4m3fn)
    assert torch.equal(from_blocked(to_blocked(f8), (256, 8)).view(torch.uint8), a)


def test_matmul_inner_dimension_mismatch():
    def qt(r, c):
        return fos.QuantizedTensor(torch.zeros(r, c // 2, dtype=torch.uint8), torch.zeros(r * c // 16, dtype=torch.uint8),
                                   torch.ones(()), "nvfp4", (r, c), "mse", "nearest")

    with pytest.raises(ValueError, match="same inner"):
        fos.quantized_matmul(qt(128, 64), qt(128, 128))
    with pytest.raises(ValueError, match="No backend found"):
        fos.quantized_matmul(qt(128, 64), qt(128, 64))  # CPU tensors


def test_quantize_model_replaces_linears():
    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.q = nn.Linear(64, 64, bias=False, dtype=torch.bfloat16)
            self.mlp = nn.Sequential(nn.Linear(64, 128, dtype=torch.bfloat16), nn.GELU(), nn.Linear(128, 64, dtype=torch.bfloat16))
            self.lm_head = nn.Linear(64, 100, dtype=torch.bfloat16)

    m = Block()
    fos.quantize_model(m, fos.ModelQuantizationConfig(weight_scale_2d=True))
    assert isinstance(m.q, fos.FourOverSixLinear) and isinstance(m.mlp[0], fos.FourOverSixLinear)
    assert type(m.lm_head) is nn.Linear and isinstance(m.mlp[1], nn.GELU)
    assert m.q.quantized_weight_values.shape == (64, 32)
    assert m.q.quantized_weight_scale_factors.dtype == torch.float8_e4m3fn
    assert m.q.quantized_weight_metadata.shape == (6,) and m.q.config.weight_scale_2d
    sd = m.state_dict()
    assert "q.quantized_weight_values" in sd and "mlp.0.quantized_weight_amax" in sd
    m2 = Block()
    fos.quantize_model(m2)  # config is optional here
    assert isinstance(m2.q, fos.FourOverSixLinear)


def test_registry_rules():
    from fouroversix_amd.model import QuantizedModule

    with pytest.raises(ValueError, match="already registered"):
        QuantizedModule.register(nn.Linear)

    class MyLinear(nn.Linear):
        pass

    with pytest.raises(TypeError, match="subclass"):
        QuantizedModule.register(MyLinear)
    assert QuantizedModule.is_quantized_module_type(fos.FourOverSixLinear)
    assert QuantizedModule.get_cls(nn.Linear) is fos.FourOverSixLinear


def test_quantize_of_meta_tensors_returns_padded_shapes():
    """Meta-device inputs (model construction before the weights exist) yield zero-filled meta
    tensors of the padded sizes, as the reference's PyTorch backend does
    (src/fouroversix/quantize/pytorch/backend.py:57-97): no kernel, no GPU."""
    x = torch.empty(100, 80, dtype=torch.bfloat16, device="meta")
    q = fos.quantize(x)
    assert q.values.device.type == "meta" and tuple(q.values.shape) == (128, 64) and q.values.dtype == torch.uint8
    assert q.scale_factors.numel() == 128 * 128 // 16 and q.scale_factors.dtype == torch.float8_e4m3fn
    assert tuple(q.amax.shape) in ((1,), ()) and q.original_shape == (100, 80) and tuple(q.padded_shape) == (128, 128)
    assert q.scale_factors_are_in_blackwell_layout
    q = fos.quantize(x, fos.QuantizationConfig(dtype="mxfp4", scale_rule="static_6", transpose=True))
    assert q.original_shape == (80, 100) and q.scale_factors.numel() == 128 * 128 // 32
    q = fos.quantize(x, fos.QuantizationConfig(dtype="if4"))
    assert not q.scale_factors_are_in_blackwell_layout
    y = fos.quantize(x, fos.QuantizationConfig(pseudo_quantize=True))
    assert y.device.type == "meta" and y.shape == x.shape and y.dtype == x.dtype


def test_reference_import_name_and_rht_matrix(oracle):
    """`import fouroversix` serves code written against the reference package (same public names,
    sub-packages included), and get_rht_matrix is the matrix the reference's transform applies
    (src/fouroversix/quantize/utils.py:68-85): diag(signs) H16 / 4, orthogonal."""
    import fouroversix
    import fouroversix_amd
    from fouroversix import QuantizationConfig, dequantize, quantize, quantize_model, quantized_matmul  # noqa: F401
    from fouroversix.model import FourOverSixLinear, ModuleQuantizationConfig  # noqa: F401
    from fouroversix.quantize import QuantizedTensor, from_blocked, get_rht_matrix  # noqa: F401
    from fouroversix.utils import DataType, ScaleRule  # noqa: F401

    assert fouroversix.quantize is fouroversix_amd.quantize and QuantizationConfig is fouroversix_amd.QuantizationConfig
    assert set(fouroversix.__all__) == set(fouroversix_amd.__all__)
    m = get_rht_matrix(device="cpu")
    assert m.dtype == torch.bfloat16 and m.shape == (16, 16)
    assert np.array_equal(m.float().numpy(), oracle.rht_matrix())
    assert torch.equal(m.float() @ m.float().T, torch.eye(16))
    plain = get_rht_matrix(with_random_sign_mask=False, device="cpu")
    assert torch.equal(plain[0].float(), torch.full((16,), 0.25)) and torch.equal(plain.float(), plain.float().T)
