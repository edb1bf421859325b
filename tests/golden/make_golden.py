"""Write golden vectors for the quantize / dequantize / matmul path by running the
REFERENCE implementation (its PyTorch CPU backend) on seeded inputs.

Run in the build container only (the reference tree is not available anywhere else):

    python tests/golden/make_golden.py [--time]

The reference package is not pip-installed, so the script puts its ``src`` directory on
``sys.path`` and answers the one ``importlib.metadata.version("fouroversix")`` lookup it
makes at import time.  Outputs are data only (inputs + expected bytes) in
``tests/golden/*.npz``; large cases store SHA-256 digests instead of arrays.

What these vectors pin that nothing else can: the mse/mae block decisions on real data
(they depend on torch.sum's fp32 summation order), the zero-padding of shapes that are
not multiples of (128, 64), and the PyTorch matmul backend's bf16 outputs.
"""

from __future__ import annotations

import argparse
import hashlib
import importlib.metadata as md
import os
import sys
import time

import numpy as np
import torch

REFERENCE_SRC = "/root/reference/src"
HERE = os.path.dirname(os.path.abspath(__file__))


def import_reference():
    real_version = md.version
    md.version = lambda name: "1.1.0" if name == "fouroversix" else real_version(name)
    sys.path.insert(0, REFERENCE_SRC)
    import fouroversix  # noqa: PLC0415

    md.version = real_version
    return fouroversix


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def u8(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint8).numpy().copy()


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def make_input(kind: str, shape: tuple[int, int], seed: int) -> torch.Tensor:
    g = torch.Generator("cpu").manual_seed(seed)
    if kind == "randn":
        x = torch.randn(*shape, generator=g)
    elif kind == "weight":
        x = 0.02 * torch.randn(*shape, generator=g)
    elif kind == "rand01":
        x = torch.randint(0, 2, shape, generator=g).float()
    elif kind == "outlier":
        # rows N(0,1); 1 % of the channels replaced by 50 * Student-t(nu=3)
        x = torch.randn(*shape, generator=g)
        n_out = max(1, shape[1] // 100)
        idx = torch.randperm(shape[1], generator=g)[:n_out]
        z = torch.randn(4, shape[0], n_out, generator=g)
        t3 = z[0] / torch.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3)
        x[:, idx] = 50 * t3
    elif kind == "tiny_blocks":
        # blocks whose maximum is far below the tensor maximum: sub-normal E4M3 scales
        x = torch.randn(*shape, generator=g)
        per_block = 10.0 ** (-torch.rand(shape[1] // 16, generator=g) * 6)
        per_block[0] = 1.0
        x = x * per_block.repeat_interleave(16)
    else:
        raise ValueError(kind)
    return x.bfloat16()


QUANT_INPUTS = [
    ("randn_256x128", "randn", (256, 128), 11),
    ("outlier_128x256", "outlier", (128, 256), 12),
    ("weight_128x128", "weight", (128, 128), 13),
    ("rand01_128x64", "rand01", (128, 64), 14),
    ("ragged_100x80", "randn", (100, 80), 15),
    ("ragged_16x64", "randn", (16, 64), 16),
    ("tiny_blocks_128x128", "tiny_blocks", (128, 128), 17),
]

QUANT_CONFIGS = [
    ("nvfp4", rule, two_d)
    for rule in ("mse", "mae", "abs_max", "static_6", "static_4")
    for two_d in (False, True)
] + [("if4", rule, two_d) for rule in ("mse", "mae", "abs_max") for two_d in (False, True)]


def write_transform_vectors() -> None:
    """transpose / random-Hadamard options of the reference quantizer
    (quantize/pytorch/reference.py:567-571).  Its backend wrapper builds the Hadamard
    matrix on "cuda" (quantize/utils.py:68-85 default), which this container lacks, so the
    reference function is called directly with the CPU matrix; shapes are multiples of
    (128, 64) in both orientations, for which the wrapper adds no padding."""
    from fouroversix.quantize.pytorch.reference import quantize as ref_quantize  # noqa: PLC0415
    from fouroversix.quantize.utils import get_rht_matrix  # noqa: PLC0415
    from fouroversix.utils import DataType, RoundStyle, ScaleRule  # noqa: PLC0415

    had = get_rht_matrix(device="cpu")
    out: dict[str, np.ndarray] = {"had": bits(had)}
    for name, kind, shape, seed in [
        ("randn_256x128", "randn", (256, 128), 31),
        ("outlier_128x256", "outlier", (128, 256), 32),
        ("tiny_blocks_128x128", "tiny_blocks", (128, 128), 33),
    ]:
        x = make_input(kind, shape, seed)
        out[f"{name}.x"] = bits(x)
        for transpose in (False, True):
            for rht in (False, True):
                if not transpose and not rht:
                    continue
                for rule, two_d in (("mse", False), ("static_6", False), ("mse", True)):
                    v, sf, amax = ref_quantize(
                        x.clone(), had=had if rht else None, fp4_format=DataType.nvfp4,
                        round_style=RoundStyle.nearest, scale_rule=ScaleRule(rule), block_scale_2d=two_d,
                        transpose=transpose, use_blackwell_scale_layout=True,
                    )
                    key = f"{name}.t{int(transpose)}.h{int(rht)}.{rule}.{'2d' if two_d else '1d'}"
                    out[key + ".values"] = u8(v)
                    out[key + ".sf"] = u8(sf)
                    out[key + ".amax"] = np.array([float(amax)], dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "transform.npz"), **out)
    print("wrote transform", len(out))


def write_fp16_transform_vectors() -> None:
    """The same options on fp16 tensors (values with 11 significant bits): the reference casts the
    Hadamard matrix to the input's type and multiplies in that type
    (quantize/pytorch/reference.py:570-571), then quantizes the fp16 result."""
    from fouroversix.quantize.pytorch.reference import quantize as ref_quantize  # noqa: PLC0415
    from fouroversix.quantize.utils import get_rht_matrix  # noqa: PLC0415
    from fouroversix.utils import DataType, RoundStyle, ScaleRule  # noqa: PLC0415

    had = get_rht_matrix(device="cpu")
    out: dict[str, np.ndarray] = {}
    for name, shape, seed, scale in [("randn_256x128", (256, 128), 61, 1.0), ("wide_128x256", (128, 256), 62, 40.0)]:
        g = torch.Generator("cpu").manual_seed(seed)
        x = (torch.randn(*shape, generator=g) * scale).half()
        out[f"{name}.x"] = x.contiguous().view(torch.int16).numpy().view(np.uint16)
        for transpose in (False, True):
            for rht in (False, True):
                if not transpose and not rht:
                    continue
                for rule, two_d in (("mse", False), ("static_6", True)):
                    v, sf, amax = ref_quantize(
                        x.clone(), had=had if rht else None, fp4_format=DataType.nvfp4,
                        round_style=RoundStyle.nearest, scale_rule=ScaleRule(rule), block_scale_2d=two_d,
                        transpose=transpose, use_blackwell_scale_layout=True,
                    )
                    key = f"{name}.t{int(transpose)}.h{int(rht)}.{rule}.{'2d' if two_d else '1d'}"
                    out[key + ".values"] = u8(v)
                    out[key + ".sf"] = u8(sf)
                    out[key + ".amax"] = np.array([float(amax)], dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "transform_fp16.npz"), **out)
    print("wrote transform_fp16", len(out))


def write_ragged_transpose_vectors(quantize, QuantizationConfig) -> None:  # noqa: N803
    """`transpose=True` on shapes that are not multiples of (128, 64), through the reference's
    PyTorch backend wrapper (quantize/pytorch/backend.py:57-79): it sizes the zero padding from
    the transposed shape but applies it to the tensor before transposing.  Shapes whose padded,
    transposed extent is not block-aligned make the reference raise; that is recorded too
    (`<name>.raised` = 1, no outputs)."""
    out: dict[str, np.ndarray] = {}
    for name, shape, seed in [("16x80", (16, 80), 41), ("80x144", (80, 144), 42), ("48x112", (48, 112), 43),
                              ("100x80", (100, 80), 44), ("16x64", (16, 64), 45), ("200x72", (200, 72), 46)]:
        x = make_input("randn", shape, seed)
        out[f"{name}.x"] = bits(x)
        for rule, two_d in (("mse", False), ("static_6", True)):
            key = f"{name}.{rule}.{'2d' if two_d else '1d'}"
            try:
                q = quantize(x.clone(), QuantizationConfig(backend="pytorch", scale_rule=rule, block_scale_2d=two_d, transpose=True))
                out[key + ".values"] = u8(q.values)
                out[key + ".sf"] = u8(q.scale_factors)
                out[key + ".amax"] = np.array([float(q.amax)], dtype=np.float32)
                out[key + ".padded"] = np.array(q.padded_shape)
                out[key + ".shape"] = np.array(q.original_shape)
                out[key + ".raised"] = np.array([0])
                print(key, "ok", tuple(q.values.shape), q.original_shape, q.padded_shape)
            except Exception as e:  # noqa: BLE001
                out[key + ".raised"] = np.array([1])
                print(key, "raised", type(e).__name__, str(e)[:100])
    np.savez_compressed(os.path.join(HERE, "ragged_transpose.npz"), **out)
    print("wrote ragged_transpose", len(out))


def write_mxfp4_vectors(quantize, dequantize, quantized_matmul, QuantizationConfig) -> None:  # noqa: N803
    """MXFP4 (E2M1 codes, E8M0 scale per 1x32 block; quantize/pytorch/reference.py:149-181)
    through the reference's PyTorch backend: quantize, dequantize and matmul."""
    out: dict[str, np.ndarray] = {}
    for name, kind, shape, seed in [
        ("randn_256x256", "randn", (256, 256), 41),
        ("outlier_128x384", "outlier", (128, 384), 42),
        ("tiny_blocks_128x128", "tiny_blocks", (128, 128), 43),
        ("ragged_100x80", "randn", (100, 80), 44),
        ("weight_16x128", "weight", (16, 128), 45),
    ]:
        x = make_input(kind, shape, seed)
        if kind == "randn":
            x[1, :32] = 0  # an all-zero block
            x[2, 5] = -0.0
        out[f"{name}.x"] = bits(x)
        for rule in ("static_6", "static_4"):
            q = quantize(x.clone(), QuantizationConfig(backend="pytorch", dtype="mxfp4", scale_rule=rule))
            key = f"{name}.{rule}"
            out[key + ".values"] = u8(q.values)
            out[key + ".sf"] = u8(q.scale_factors)
            out[key + ".amax"] = np.array([float(q.amax)], dtype=np.float32)
            out[key + ".padded"] = np.array(q.padded_shape)
            out[key + ".deq_bf16"] = bits(dequantize(q))
            out[key + ".deq_f32"] = dequantize(q, torch.float32).numpy().copy()
    for tag, (m, n, k), rule, seed in [("256x128x256", (256, 128, 256), "static_6", 46),
                                       ("100x72x160", (100, 72, 160), "static_4", 47)]:
        g = torch.Generator("cpu").manual_seed(seed)
        a = torch.randn(m, k, generator=g).bfloat16()
        b = torch.randn(n, k, generator=g).bfloat16()
        cfg = QuantizationConfig(backend="pytorch", dtype="mxfp4", scale_rule=rule)
        o = quantized_matmul(quantize(a, cfg), quantize(b, cfg), backend="pytorch")
        out[f"mm.{tag}.a"] = bits(a)
        out[f"mm.{tag}.b"] = bits(b)
        out[f"mm.{tag}.out"] = bits(o)
        out[f"mm.{tag}.rule"] = np.array(rule)
    np.savez_compressed(os.path.join(HERE, "mxfp4.npz"), **out)
    print("wrote mxfp4", len(out))


def write_f32_intermediate_vectors(quantize, dequantize, QuantizationConfig) -> None:  # noqa: N803
    """dequantize(..., intermediate_dtype=torch.float32) -- value and block scale multiplied in
    fp32 instead of fp16 (quantize/backend.py:89-160), which the reference's own pseudo-quantize
    test relies on -- for the formats where that changes the result: IF4 (integer blocks carry
    the factor 6/7) and MXFP4 (scales outside fp16's range), NVFP4 for completeness."""
    out: dict[str, np.ndarray] = {}
    for name, kind, shape, seed in [("randn_256x128", "randn", (256, 128), 51), ("tiny_blocks_128x128", "tiny_blocks", (128, 128), 52),
                                    ("ragged_100x80", "randn", (100, 80), 53), ("outlier_128x384", "outlier", (128, 384), 54)]:
        x = make_input(kind, shape, seed)
        for dtype, rule in (("if4", "mse"), ("if4", "abs_max"), ("mxfp4", "static_6"), ("nvfp4", "mse")):
            if kind == "tiny_blocks" and dtype == "mxfp4":
                x = (x.float() * 2.0**-30).bfloat16()  # block scales below fp16's range
            q = quantize(x.clone(), QuantizationConfig(backend="pytorch", dtype=dtype, scale_rule=rule))
            key = f"{name}.{dtype}.{rule}"
            out[key + ".values"] = u8(q.values)
            out[key + ".sf"] = u8(q.scale_factors)
            out[key + ".amax"] = np.array([float(q.amax)], dtype=np.float32)
            out[key + ".shape"] = np.array(shape)
            out[key + ".padded"] = np.array(q.padded_shape)
            out[key + ".blocked"] = np.array([int(q.scale_factors_are_in_blackwell_layout)])
            out[key + ".deq_bf16"] = bits(dequantize(q, torch.bfloat16, intermediate_dtype=torch.float32))
            out[key + ".deq_f32"] = dequantize(q, torch.float32, intermediate_dtype=torch.float32).numpy().copy()
    np.savez_compressed(os.path.join(HERE, "dequantize_f32_intermediate.npz"), **out)
    print("wrote dequantize_f32_intermediate", len(out))


def write_input_dtype_vectors(quantize, QuantizationConfig) -> None:  # noqa: N803
    """fp32 and fp16 inputs: the reference converts whatever it is given with `.float()`
    (quantize/pytorch/reference.py:577,593,596), so an input with more significant bits than
    bf16 reaches the block arithmetic unrounded."""
    out: dict[str, np.ndarray] = {}
    for name, kind, shape, seed in [("randn_128x128", "randn", (128, 128), 61), ("ragged_100x80", "randn", (100, 80), 62),
                                    ("outlier_128x256", "outlier", (128, 256), 63)]:
        g = torch.Generator("cpu").manual_seed(seed)
        base = torch.randn(*shape, generator=g)
        if kind == "outlier":
            base[:, 7] *= 50.0
        for tname, x in (("f32", base), ("f16", base.half())):
            out[f"{name}.{tname}.x"] = x.numpy().copy() if tname == "f32" else x.numpy().view(np.uint16).copy()
            for dtype, rule, two_d in (("nvfp4", "mse", False), ("nvfp4", "static_6", False), ("nvfp4", "mse", True),
                                       ("nvfp4", "abs_max", False), ("if4", "mse", False)):
                if two_d and shape[0] % 16:
                    continue
                q = quantize(x.clone(), QuantizationConfig(backend="pytorch", dtype=dtype, scale_rule=rule, block_scale_2d=two_d))
                key = f"{name}.{tname}.{dtype}.{rule}.{'2d' if two_d else '1d'}"
                out[key + ".values"] = u8(q.values)
                out[key + ".sf"] = u8(q.scale_factors)
                out[key + ".amax"] = np.array([float(q.amax)], dtype=np.float32)
    np.savez_compressed(os.path.join(HERE, "input_dtypes.npz"), **out)
    print("wrote input_dtypes", len(out))


def write_mxfp4_input_dtype_vectors(quantize, QuantizationConfig) -> None:  # noqa: N803
    """MXFP4 on fp32 and fp16 inputs: quantize_to_mxfp4 converts its input with `.float()`
    (quantize/pytorch/reference.py:149-181) like the other formats."""
    out: dict[str, np.ndarray] = {}
    for name, shape, seed in [("randn_128x256", (128, 256), 71), ("ragged_100x80", (100, 80), 72), ("wide_64x1024", (64, 1024), 73)]:
        g = torch.Generator("cpu").manual_seed(seed)
        base = torch.randn(*shape, generator=g) * 3.0
        base[1, :32] = 0
        base[2, 5] = -0.0
        base[3, :8] *= 1e-4
        for tname, x in (("f32", base), ("f16", base.half())):
            out[f"{name}.{tname}.x"] = x.numpy().copy() if tname == "f32" else x.numpy().view(np.uint16).copy()
            for rule in ("static_6", "static_4"):
                q = quantize(x.clone(), QuantizationConfig(backend="pytorch", dtype="mxfp4", scale_rule=rule))
                key = f"{name}.{tname}.{rule}"
                out[key + ".values"] = u8(q.values)
                out[key + ".sf"] = u8(q.scale_factors)
                out[key + ".padded"] = np.array(q.padded_shape)
    np.savez_compressed(os.path.join(HERE, "mxfp4_input_dtypes.npz"), **out)
    print("wrote mxfp4_input_dtypes", len(out))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--only-input-dtypes", action="store_true", help="write only input_dtypes.npz")
    ap.add_argument("--only-dequant32", action="store_true", help="write only dequantize_f32_intermediate.npz")
    ap.add_argument("--time", action="store_true", help="also time the reference CPU path")
    ap.add_argument("--only-transform", action="store_true", help="write only transform.npz")
    ap.add_argument("--only-mxfp4", action="store_true", help="write only mxfp4.npz")
    ap.add_argument("--only-ragged-transpose", action="store_true", help="write only ragged_transpose.npz")
    ap.add_argument("--only-transform-fp16", action="store_true", help="write only transform_fp16.npz")
    ap.add_argument("--only-mxfp4-dtypes", action="store_true", help="write only mxfp4_input_dtypes.npz")
    args = ap.parse_args()

    fos = import_reference()
    from fouroversix import QuantizationConfig, dequantize, quantize, quantized_matmul  # noqa: PLC0415

    torch.set_num_threads(os.cpu_count() or 1)
    write_mxfp4_input_dtype_vectors(quantize, QuantizationConfig)
    if args.only_mxfp4_dtypes:
        return
    write_fp16_transform_vectors()
    if args.only_transform_fp16:
        return
    write_ragged_transpose_vectors(quantize, QuantizationConfig)
    if args.only_ragged_transpose:
        return
    write_input_dtype_vectors(quantize, QuantizationConfig)
    if args.only_input_dtypes:
        return
    write_f32_intermediate_vectors(quantize, dequantize, QuantizationConfig)
    if args.only_dequant32:
        return
    if not args.only_mxfp4:
        write_transform_vectors()
    if not args.only_transform:
        write_mxfp4_vectors(quantize, dequantize, quantized_matmul, QuantizationConfig)
    if args.only_transform or args.only_mxfp4:
        return

    # ---- quantize + dequantize ------------------------------------------------------
    for name, kind, shape, seed in QUANT_INPUTS:
        x = make_input(kind, shape, seed)
        out: dict[str, np.ndarray] = {"x": bits(x), "shape": np.array(shape)}
        for dtype, rule, two_d in QUANT_CONFIGS:
            cfg = QuantizationConfig(backend="pytorch", dtype=dtype, scale_rule=rule, block_scale_2d=two_d)
            q = quantize(x.clone(), cfg)
            key = f"{dtype}.{rule}.{'2d' if two_d else '1d'}"
            out[key + ".values"] = u8(q.values)
            out[key + ".sf"] = u8(q.scale_factors)
            out[key + ".amax"] = np.array([float(q.amax)], dtype=np.float32)
            out[key + ".padded"] = np.array(q.padded_shape)
            out[key + ".blocked"] = np.array([int(q.scale_factors_are_in_blackwell_layout)])
            if name in ("randn_256x128", "ragged_100x80", "tiny_blocks_128x128") and not two_d:
                out[key + ".deq_bf16"] = bits(dequantize(q))
                out[key + ".deq_f32_sha"] = np.array(sha(dequantize(q, torch.float32).numpy()))
        np.savez_compressed(os.path.join(HERE, f"quantize_{name}.npz"), **out)
        print("wrote", name, len(out))

    # ---- the CPU-runnable headline case: 1024x1024 randn seed 0, static_6 ------------
    g = torch.Generator("cpu").manual_seed(0)
    x = torch.randn(1024, 1024, generator=g).bfloat16()
    big = {"x_sha": np.array(sha(bits(x)))}
    for rule in ("static_6", "mse"):
        q = quantize(x, QuantizationConfig(backend="pytorch", scale_rule=rule))
        big[f"{rule}.values_sha"] = np.array(sha(u8(q.values)))
        big[f"{rule}.sf_sha"] = np.array(sha(u8(q.scale_factors)))
        big[f"{rule}.amax"] = np.array([float(q.amax)], dtype=np.float32)
        big[f"{rule}.values_head"] = u8(q.values)[:4].copy()
        big[f"{rule}.sf_head"] = u8(q.scale_factors)[:512].copy()
    np.savez_compressed(os.path.join(HERE, "quantize_config1_1024x1024.npz"), **big)
    print("wrote config1")

    # ---- matmul (PyTorch backend: dequantize -> fp32 matmul -> bf16) -----------------
    mm: dict[str, np.ndarray] = {}
    for tag, (m, n, k), rule, seed in [
        ("mse_256x256x256", (256, 256, 256), "mse", 21),
        ("static6_128x256x512", (128, 256, 512), "static_6", 22),
        ("static4_128x128x128", (128, 128, 128), "static_4", 23),
        ("ragged_100x72x80", (100, 72, 80), "mse", 24),
    ]:
        g = torch.Generator("cpu").manual_seed(seed)
        a = torch.randn(m, k, generator=g).bfloat16()
        b = torch.randn(n, k, generator=g).bfloat16()
        cfg = QuantizationConfig(backend="pytorch", scale_rule=rule)
        qa, qb = quantize(a, cfg), quantize(b, cfg)
        o = quantized_matmul(qa, qb, backend="pytorch")
        mm[tag + ".a"] = bits(a)
        mm[tag + ".b"] = bits(b)
        mm[tag + ".out"] = bits(o)
        mm[tag + ".rule"] = np.array(rule)
    np.savez_compressed(os.path.join(HERE, "matmul.npz"), **mm)
    print("wrote matmul")

    if args.time:
        from torch.utils.benchmark import Timer  # noqa: PLC0415

        g = torch.Generator("cpu").manual_seed(0)
        x1 = torch.randn(1024, 1024, generator=g).bfloat16()
        cfg1 = QuantizationConfig(backend="pytorch", scale_rule="static_6")
        t1 = Timer("quantize(x, cfg)", globals={"quantize": quantize, "x": x1, "cfg": cfg1}).timeit(5).mean
        g = torch.Generator("cpu").manual_seed(1)
        x2 = torch.randn(8192, 4096, generator=g).bfloat16()
        cfg2 = QuantizationConfig(backend="pytorch", scale_rule="mse")
        t0 = time.time()
        quantize(x2, cfg2)
        t2 = time.time() - t0
        print(f"reference CPU path, {torch.get_num_threads()} threads: "
              f"1024x1024 static_6 {t1 * 1e3:.1f} ms ({1024 * 1024 * 2.5625 / t1 / 1e9:.3f} GB/s); "
              f"8192x4096 mse {t2:.2f} s ({8192 * 4096 * 2.5625 / t2 / 1e9:.3f} GB/s)")
    del fos


if __name__ == "__main__":
    main()
