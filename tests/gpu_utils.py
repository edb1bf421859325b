"""Helpers shared by the GPU parity tests."""

import numpy as np
import torch

import fouroversix_amd as fos


def make_input(kind, shape, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    if kind == "zeros":
        x = torch.zeros(*shape)
    elif kind == "ones":
        x = torch.ones(*shape)
    elif kind == "rand01":
        x = torch.randint(0, 2, shape, generator=g).float()
    elif kind == "randn":
        x = torch.randn(*shape, generator=g)
    elif kind == "weight":
        x = 0.02 * torch.randn(*shape, generator=g)
    elif kind == "outlier":
        x = torch.randn(*shape, generator=g)
        n_out = max(1, shape[1] // 100)
        idx = torch.randperm(shape[1], generator=g)[:n_out]
        z = torch.randn(4, shape[0], n_out, generator=g)
        x[:, idx] = 50 * z[0] / torch.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3)
    elif kind == "tiny_blocks":
        x = torch.randn(*shape, generator=g)
        per_block = 10.0 ** (-torch.rand(shape[1] // 16, generator=g) * 6)
        per_block[0] = 1.0
        x = x * per_block.repeat_interleave(16)
    else:
        raise ValueError(kind)
    return x.bfloat16()


def u8(t):
    return t.detach().contiguous().view(torch.uint8).cpu().numpy()


def bits16(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def assert_same_quantization(q, ref, what=""):
    """HIP QuantizedTensor vs OracleQuantized: bit-exact codes, scales, amax."""
    assert tuple(q.padded_shape) == tuple(ref.padded_shape), what
    assert q.scale_factors_are_in_blackwell_layout == ref.blocked, what
    assert float(q.amax) == float(ref.amax), f"{what}: amax {float(q.amax)} vs {float(ref.amax)}"
    v, s = u8(q.values), u8(q.scale_factors).reshape(-1)
    ns = int((s != ref.scale_factors).sum())
    nv = int((v != ref.values).sum())
    assert ns == 0 and nv == 0, f"{what}: {ns}/{s.size} scale bytes and {nv}/{v.size} code bytes differ"


def hip_quantize(x_cpu, **cfg):
    return fos.quantize(x_cpu.cuda(), fos.QuantizationConfig(**cfg))
