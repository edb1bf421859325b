"""``FourOverSixLinear``: ``nn.Linear`` whose forward quantizes the activations on the fly
and multiplies them with a (pre-)quantized weight on the FP4 GEMM
(reference ``src/fouroversix/model/modules/linear.py:43-94, 291-453``), and whose backward
(``keep_master_weights=True``) computes both gradients on the FP4 GEMM as well
(``linear.py:96-288``, without the Quartet-II variant): dgrad from the stochastically
rounded gradient and the weight quantized along its other dimension, wgrad from the
transposed, random-Hadamard-rotated gradient and activations.

The quantized weight lives in four buffers with the reference's names and shapes --
``quantized_weight_values`` u8 [out, in/2], ``quantized_weight_scale_factors`` E4M3 flat,
``quantized_weight_amax`` f32[1], ``quantized_weight_metadata`` int32[6] = (rows, cols,
padded rows, padded cols, 1, tiled-layout flag) -- so checkpoints interchange.
"""

from __future__ import annotations

from typing import Any

import torch
import torch.nn as nn

from fouroversix_amd.matmul import quantized_matmul
from fouroversix_amd.quantize import QuantizedTensor, dequantize, quantize
from fouroversix_amd.quantize.frontend import attach_known_amax, known_amax
from fouroversix_amd.utils import DataType

from .config import ModuleQuantizationConfig
from .quantize import QuantizedModule


def fp4_linear(
    config: ModuleQuantizationConfig,
    input: torch.Tensor,
    weight: QuantizedTensor | torch.Tensor,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """``input @ weight.T + bias`` with both operands in the configured 4-bit formats."""
    if config.disable_fprop_quantization:
        out = torch.matmul(input, weight.T)
    else:
        if isinstance(weight, torch.Tensor):
            weight = quantize(weight.data if isinstance(weight, nn.Parameter) else weight, config.get_weight_config())
        flat = input.reshape(-1, input.shape[-1])
        if config.pseudo_quantize:
            out = torch.matmul(quantize(flat, config.get_activation_config()), weight.T)
            out = out.reshape(*input.shape[:-1], weight.shape[0])
        else:
            # (a maximum recorded on `input` by the layer that produced it survives the flattening:
            # a view shares the version counter)
            amax_in = known_amax(input)
            if amax_in is not None and flat is not input:
                attach_known_amax(flat, amax_in)
            # (the bias goes into the GEMM's epilogue with the two roundings of `out + bias`; the recorded
            # maximum is then that of the sum)
            out2d = quantized_matmul(
                flat,
                weight,
                backend=config.matmul_backend,
                input_config=config.get_activation_config(),
                out_dtype=config.output_dtype,
                emit_amax=config.emit_output_amax,
                bias=bias,
            )
            out = out2d.reshape(*input.shape[:-1], weight.original_shape[0])
            amax_out = known_amax(out2d)
            if amax_out is not None and out is not out2d:
                attach_known_amax(out, amax_out)
            return out
    if bias is not None:
        out = out + bias
    return out


class FourOverSixLinearFunction(torch.autograd.Function):
    """Differentiable FP4 linear layer (reference ``linear.py:40-288``)."""

    @staticmethod
    def forward(ctx, config: ModuleQuantizationConfig, input: torch.Tensor, weight, bias=None) -> torch.Tensor:
        if isinstance(weight, nn.Parameter):
            ctx.config = config
            ctx.save_for_backward(input, weight, bias)
        return fp4_linear(config, input, weight, bias)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        input, weight, bias = ctx.saved_tensors
        cfg: ModuleQuantizationConfig = ctx.config
        if cfg.quartet_ii_dtype is not None:
            msg = "the Quartet-II backward is not implemented"
            raise NotImplementedError(msg)
        out_dtype = cfg.output_dtype.torch_dtype
        g = grad_output.reshape(-1, grad_output.shape[-1])  # [tokens, out]
        x = input.reshape(-1, input.shape[-1])              # [tokens, in]
        w = weight.data

        # dgrad = g @ W: W is quantized along its other dimension (blocks along `out`)
        grad_input = None
        if ctx.needs_input_grad[1]:
            g_cfg = cfg.get_gradient_config()
            w_cfg = cfg.get_weight_config(transpose=True)
            if cfg.disable_dgrad_quantization == "quantize_grad_only":
                gq = dequantize(quantize(g, g_cfg), torch.float32)
                grad_input = torch.matmul(gq, w.float()).to(out_dtype)
            elif cfg.disable_dgrad_quantization:
                grad_input = torch.matmul(g, w)
            elif cfg.pseudo_quantize:
                grad_input = torch.matmul(quantize(g, g_cfg), quantize(w, w_cfg).T)
            else:
                grad_input = quantized_matmul(g, w, backend=cfg.matmul_backend, input_config=g_cfg, other_config=w_cfg,
                                              out_dtype=cfg.output_dtype)
            grad_input = grad_input.reshape(*grad_output.shape[:-1], weight.shape[1])

        # wgrad = g^T @ x: both operands transposed and rotated by the random Hadamard
        # transform along the token dimension (the rotation cancels in the product)
        grad_weight = None
        if ctx.needs_input_grad[2]:
            extra = {"dtype": DataType.nvint4} if cfg.wgrad_nvint4 else {}
            g_cfg = cfg.get_gradient_config(rht=True, transpose=True, **extra)
            x_cfg = cfg.get_activation_config(rht=True, transpose=True, **extra)
            if cfg.disable_wgrad_quantization:
                grad_weight = torch.matmul(g.T, x)
            elif cfg.pseudo_quantize:
                grad_weight = torch.matmul(quantize(g, g_cfg), quantize(x, x_cfg).T)
            else:
                grad_weight = quantized_matmul(g, x, backend=cfg.matmul_backend, input_config=g_cfg, other_config=x_cfg,
                                               out_dtype=cfg.output_dtype)

        grad_bias = g.sum(0) if bias is not None and ctx.needs_input_grad[3] else None
        return None, grad_input, grad_weight, grad_bias


@QuantizedModule.register(nn.Linear)
class FourOverSixLinear(nn.Linear):
    """Drop-in ``nn.Linear`` replacement with 4-bit weights and activations."""

    def __init__(self, module: nn.Linear, config: ModuleQuantizationConfig) -> None:
        super().__init__(
            module.in_features,
            module.out_features,
            module.bias is not None,
            module.weight.device,
            module.weight.dtype,
        )
        self.weight = module.weight
        self.bias = module.bias
        self.config = config

        if not config.keep_master_weights:
            wdt = config.weight_dtype
            pack = wdt.quantized_value_type.packing_factor
            # (on the weight's device, so that a checkpoint of quantized buffers loads in place)
            dev = module.weight.device
            self.register_buffer(
                "quantized_weight_values",
                torch.zeros(self.out_features, self.in_features // pack, dtype=torch.uint8, device=dev),
            )
            self.register_buffer(
                "quantized_weight_scale_factors",
                torch.zeros(self.out_features * self.in_features // wdt.block_size, dtype=wdt.scale_type.torch_dtype, device=dev),
            )
            self.register_buffer("quantized_weight_amax", torch.zeros(1, dtype=torch.float32, device=dev))
            self.register_buffer("quantized_weight_metadata", torch.zeros(6, dtype=torch.int32, device=dev))

    @property
    def parameters_to_quantize(self) -> tuple[str, ...]:
        return ("weight",)

    def get_element_size(self, parameter_name: str) -> float:
        """Bytes per element: 0.5 for the packed values, (8 + 1) / 16 for a quantized weight."""
        sizes = {"quantized_weight_values": 0.5, "weight": 9 / 16}
        if parameter_name in sizes:
            return sizes[parameter_name]
        return getattr(self, parameter_name).element_size()

    def get_quantized_parameters(self, parameter_name: str, parameter: torch.Tensor) -> dict[str, Any]:
        """Quantize ``parameter`` (the weight) and return the four buffers as a dict."""
        if parameter_name != "weight":
            msg = f"Unsupported high-precision parameter: {parameter_name}"
            raise ValueError(msg)
        q = quantize(parameter, self.config.get_weight_config())
        return {
            "quantized_weight_values": q.values,
            "quantized_weight_scale_factors": q.scale_factors,
            "quantized_weight_amax": q.amax,
            "quantized_weight_metadata": torch.tensor(
                [*q.original_shape, *q.padded_shape, 1, int(q.scale_factors_are_in_blackwell_layout)],
            ),
        }

    def quantize_weight_(self) -> "FourOverSixLinear":
        """Fill the quantized buffers from ``self.weight`` and drop the high-precision
        weight (what the reference leaves to its checkpoint-loading integrations)."""
        if self.config.keep_master_weights:
            return self
        params = self.get_quantized_parameters("weight", self.weight.data)
        dev = self.weight.device
        for name, value in params.items():
            setattr(self, name, value.reshape(getattr(self, name).shape if name == "quantized_weight_amax" else value.shape).to(dev))
        self.quantized_weight_metadata = self.quantized_weight_metadata.to(torch.int32)
        self.weight = None
        if hasattr(self, "_quantized_weight"):
            del self._quantized_weight
        return self

    def quantized_weight(self) -> QuantizedTensor | nn.Parameter:
        if self.config.keep_master_weights:
            return self.weight
        if not hasattr(self, "_quantized_weight"):
            meta = self.quantized_weight_metadata.tolist()
            self._quantized_weight = QuantizedTensor(
                self.quantized_weight_values,
                self.quantized_weight_scale_factors,
                self.quantized_weight_amax,
                self.config.weight_dtype,
                tuple(meta[:2]),
                self.config.weight_scale_rule,
                self.config.weight_round_style,
                tuple(meta[2:4]),
                scale_factors_are_in_blackwell_layout=meta[5] == 1,
            )
        return self._quantized_weight

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return FourOverSixLinearFunction.apply(self.config, input, self.quantized_weight(), self.bias)
