"""Parity of the gfx950 quantize / dequantize kernels with the CPU oracle and with the
vectors written by the reference.  Round-to-nearest must be bit-exact (codes, scale
bytes, amax); stochastic rounding is bit-exact against the oracle for the same Philox
key and statistically pinned to the reference's known answers."""

import glob
import os

import numpy as np
import pytest
import torch

import fouroversix_amd as fos
from gpu_utils import assert_same_quantization, bits16, hip_quantize, make_input, u8

pytestmark = pytest.mark.gpu

NVFP4_RULES = ["mse", "mae", "abs_max", "static_6", "static_4"]
IF4_RULES = ["mse", "mae", "abs_max"]
CONFIGS = [("nvfp4", r) for r in NVFP4_RULES] + [("if4", r) for r in IF4_RULES]
QUANT_FILES = sorted(f for f in glob.glob(os.path.join(os.path.dirname(__file__), "golden", "quantize_*.npz"))
                     if "config1" not in f)


@pytest.mark.parametrize("two_d", [False, True], ids=["1d", "2d"])
@pytest.mark.parametrize(("dtype", "rule"), CONFIGS)
@pytest.mark.parametrize(("kind", "shape"), [
    ("zeros", (1024, 512)), ("ones", (1024, 512)), ("rand01", (1024, 512)),
    ("randn", (1024, 1024)), ("randn", (1024, 512)), ("randn", (512, 1024)),
])
def test_matches_oracle_on_reference_test_inputs(oracle, kind, shape, dtype, rule, two_d):
    """The reference's own test grid (tests/test_quantize.py:23-314): zeros / ones / 0-1 /
    randn at three shapes, every rule, 1-D and 2-D scaling."""
    # ten seeds per case, as the reference runs its grid (tests/test_quantize.py:19-20,151-153);
    # zeros and ones do not depend on the seed
    for seed in range(10):
        x = make_input(kind, shape, seed)
        q = hip_quantize(x, dtype=dtype, scale_rule=rule, block_scale_2d=two_d)
        ref = oracle.quantize(x, dtype=dtype, scale_rule=rule, block_scale_2d=two_d)
        assert_same_quantization(q, ref, f"{kind}{shape} {dtype}/{rule}/2d={two_d} seed {seed}")
        if kind in ("zeros", "ones"):
            break


@pytest.mark.parametrize("path", QUANT_FILES, ids=[os.path.basename(p)[9:-4] for p in QUANT_FILES])
def test_matches_reference_vectors(path):
    """Vectors written by the reference's PyTorch backend, incl. ragged shapes (zero
    padding to 128 x 64 multiples) and sub-normal block scales."""
    d = np.load(path)
    x = torch.from_numpy(d["x"].view(np.int16).copy()).view(torch.bfloat16)
    for k in sorted({k.rsplit(".", 1)[0] for k in d.files if k.endswith(".values")}):
        dt, rule, dim = k.split(".")
        q = hip_quantize(x, dtype=dt, scale_rule=rule, block_scale_2d=(dim == "2d"))
        assert tuple(q.padded_shape) == tuple(d[k + ".padded"]), k
        assert float(q.amax) == float(d[k + ".amax"][0]), k
        assert np.array_equal(u8(q.values), d[k + ".values"]), k
        assert np.array_equal(u8(q.scale_factors).reshape(-1), d[k + ".sf"].reshape(-1)), k
        if k + ".deq_bf16" in d.files:
            want = d[k + ".deq_bf16"]
            assert np.array_equal(bits16(fos.dequantize(q)), want), k
            # the fused quantize -> dequantize kernel against the reference's own dequantized bits
            r = fos.quantize(x.cuda(), fos.QuantizationConfig(dtype=dt, scale_rule=rule, block_scale_2d=(dim == "2d"),
                                                              pseudo_quantize=True))
            assert r.shape == x.shape and np.array_equal(bits16(r), want[: x.shape[0], : x.shape[1]]), k + " (pseudo)"


def test_fp32_and_fp16_inputs_match_reference_vectors(golden_dir):
    """Inputs with more significant bits than bf16, which the reference converts with `.float()`:
    bytes written by its PyTorch backend for fp32 and fp16 tensors (ragged and outlier shapes too)."""
    d = np.load(os.path.join(golden_dir, "input_dtypes.npz"))
    keys = sorted({k.rsplit(".", 1)[0] for k in d.files if k.endswith(".values")})
    assert len(keys) >= 24
    for k in keys:
        name, tname, dt, rule, dim = k.split(".")
        raw = d[f"{name}.{tname}.x"]
        x = torch.from_numpy(raw.copy()) if tname == "f32" else torch.from_numpy(raw.view(np.int16).copy()).view(torch.float16)
        q = hip_quantize(x, dtype=dt, scale_rule=rule, block_scale_2d=(dim == "2d"))
        assert tuple(q.original_shape) == tuple(x.shape), k
        assert float(q.amax) == float(d[k + ".amax"][0]), k
        assert np.array_equal(u8(q.values), d[k + ".values"]), k
        assert np.array_equal(u8(q.scale_factors).reshape(-1), d[k + ".sf"].reshape(-1)), k


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.float16], ids=["f32", "f16"])
@pytest.mark.parametrize(("cfg"), [
    dict(scale_rule="mse"), dict(scale_rule="mae", block_scale_2d=True), dict(scale_rule="abs_max"),
    dict(scale_rule="static_4", block_scale_2d=True), dict(dtype="if4", scale_rule="mse"), dict(dtype="if4", scale_rule="mae", block_scale_2d=True),
    dict(scale_rule="mse", round_style="stochastic"), dict(scale_rule="static_6", round_style="stochastic_unbiased"),
    dict(dtype="if4", scale_rule="abs_max", round_style="stochastic"),
], ids=str)
def test_fp32_and_fp16_inputs_match_oracle(oracle, in_dtype, cfg):
    """Every rule / format / rounding style on fp32 and fp16 data (element-wise kernel, and the streaming one for
    aligned fp16 NVFP4 inputs with 1x16 blocks and round to nearest), aligned and ragged shapes, strided rows; bf16 values handed over in the wider type give the bf16 kernels' bytes."""
    g = torch.Generator("cpu").manual_seed(17)
    kwargs = {"seed": 7, "offset": 1} if "round_style" in cfg else {}
    okw = dict(seed=7, offset=1) if "round_style" in cfg else {}
    for shape in ((256, 320), (100, 80), (16, 4096)):
        x = (torch.randn(*shape, generator=g) * 3.0).to(in_dtype)
        q = hip_quantize(x, kwargs=kwargs, **cfg)
        assert_same_quantization(q, oracle.quantize(x, **okw, **cfg), f"{in_dtype} {shape} {cfg}")
    wide = (torch.randn(64, 512, generator=g)).to(in_dtype).cuda()
    view = wide[:, 64:320]  # row stride 512 elements, offset start
    q = fos.quantize(view, fos.QuantizationConfig(kwargs=kwargs, **cfg))
    assert_same_quantization(q, oracle.quantize(view.cpu().contiguous(), **okw, **cfg), f"strided {in_dtype} {cfg}")
    xb = torch.randn(128, 256, generator=g).bfloat16()
    if in_dtype == torch.float32:
        same = hip_quantize(xb.float(), kwargs=kwargs, **cfg)
        base = hip_quantize(xb, kwargs=kwargs, **cfg)
        assert torch.equal(same.values, base.values) and torch.equal(same.scale_factors.view(torch.uint8), base.scale_factors.view(torch.uint8))
        assert float(same.amax) == float(base.amax)


@pytest.mark.parametrize("rule", NVFP4_RULES)
def test_fp16_inputs_on_the_streaming_kernel(oracle, rule):
    """Aligned fp16 inputs with 1x16 blocks and round to nearest run on the streaming kernel (fp16 instantiation):
    bit-exact with the oracle at full size, on ragged shapes, on fp16's own corner values (sub-normals, the
    largest finite values, 11-bit significands next to block maxima), with a caller's maximum of 24
    significant bits (undecided blocks take the operation-by-operation form), and on strided rows."""
    g = torch.Generator("cpu").manual_seed(23)
    cfg = dict(scale_rule=rule)
    big = (torch.randn(2048, 4096, generator=g) * 2.0).half()
    big[5, 7] = 900.0  # an outlier: most block scales become small
    assert_same_quantization(hip_quantize(big, **cfg), oracle.quantize(big, **cfg), f"fp16 2048x4096 {rule}")
    flat = (torch.rand(8192, 2048, generator=g) * 4.0).half()  # >= 16 MiB, cols % 2048 == 0: window-order scan
    assert_same_quantization(hip_quantize(flat, **cfg), oracle.quantize(flat, **cfg), f"fp16 8192x2048 {rule}")
    for shape in ((130, 272), (100, 80), (16, 4096), (257, 1024)):
        x = (torch.randn(*shape, generator=g) * 3.0).half()
        assert_same_quantization(hip_quantize(x, **cfg), oracle.quantize(x, **cfg), f"fp16 {shape} {rule}")
    # corner values: sub-normals (down to 2^-24), 65504, values one fp16 ulp apart, exact grid values
    c = torch.zeros(256, 256, dtype=torch.float16)
    c[0, :16] = torch.tensor([6e-8, 1.2e-7, -6e-8, 5.96e-8] * 4, dtype=torch.float16)
    c[1, :16] = torch.tensor([65504.0, -65504.0, 32752.0, 1.0] * 4, dtype=torch.float16)
    c[2, :16] = torch.tensor([1.0, 1.0009765625, 0.99951171875, 1.5] * 4, dtype=torch.float16)
    c[3:, :] = (torch.randn(253, 256, generator=g) * 1e-3).half()
    for scale in (1.0, 2.0 ** -10):
        x = (c.float() * scale).half()
        assert_same_quantization(hip_quantize(x, **cfg), oracle.quantize(x, **cfg), f"fp16 corners x{scale} {rule}")
    x = (torch.randn(512, 1024, generator=g)).half()
    given = float(np.float32(float(x.abs().max()) * 1.2345678))
    q = fos.quantize(x.cuda(), fos.QuantizationConfig(kwargs={"amax": torch.tensor(given, device="cuda")}, **cfg))
    assert_same_quantization(q, oracle.quantize(x, amax=given, **cfg), f"fp16 amax given {rule}")
    wide = torch.randn(256, 1024, generator=g).half().cuda()
    view = wide[:, 256:768]
    assert_same_quantization(fos.quantize(view, fos.QuantizationConfig(**cfg)), oracle.quantize(view.cpu().contiguous(), **cfg),
                             f"fp16 strided {rule}")


def test_fp32_and_fp16_inputs_other_paths(oracle):
    """pseudo-quantize composes quantize -> dequantize in the input's type; amax can be supplied; formats and
    options without a kernel for these types say so."""
    g = torch.Generator("cpu").manual_seed(3)
    x = torch.randn(128, 128, generator=g)
    for t in (torch.float32, torch.float16):
        xt = x.to(t).cuda()
        out = fos.quantize(xt, fos.QuantizationConfig(pseudo_quantize=True))
        assert out.dtype == t and out.shape == xt.shape
        q = fos.quantize(xt)
        assert torch.equal(out, fos.dequantize(q, dtype=t))
        q2 = fos.quantize(xt, fos.QuantizationConfig(kwargs={"amax": q.amax}))
        assert torch.equal(q2.values, q.values)
        assert fos.quantize(xt, fos.QuantizationConfig(dtype="mxfp4", scale_rule="static_6")).original_shape == (128, 128)
        for option in (dict(rht=True), dict(transpose=True)):
            assert fos.quantize(xt, fos.QuantizationConfig(**option)).original_shape == (128, 128)
    with pytest.raises(ValueError, match="bfloat16, float16 or float32"):
        fos.quantize(x.double().cuda())


@pytest.mark.parametrize(("transpose", "rht"), [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("shape", [(256, 512), (100, 80), (130, 8)])
def test_fp32_inputs_with_transpose_and_rht(oracle, shape, transpose, rht):
    """fp32 tensors under the `transpose` / `rht` options (reference src/fouroversix/quantize/pytorch/reference.py:567-571:
    `x.float()` times the fp32 Hadamard matrix, a library matmul whose summation order is not fixed).  Parity
    with the reference is therefore to tolerance: the transformed tensor lies within 2^-21 |x| |H| of the exact
    product (four fp32 roundings of partial sums; a plain transposition is exact), and the quantization of that
    tensor is the oracle's, bit for bit."""
    from fouroversix_amd.quantize import ops

    g = torch.Generator("cpu").manual_seed(21)
    x = torch.randn(*shape, generator=g) * torch.exp(torch.randn(shape[0], 1, generator=g))
    y, amax = ops.transform(x.cuda(), transpose, rht)
    y = y.cpu().numpy()
    exact = oracle.transform(x.numpy(), transpose=transpose, rht=rht, x_type=2)
    assert y.shape == exact.shape
    if rht:
        xt = x.numpy().T if transpose else x.numpy()
        xt = np.pad(xt, ((0, 0), (0, -xt.shape[1] % 16)))
        bound = np.repeat(np.abs(xt).astype(np.float64).reshape(-1, 16).sum(axis=1) * 0.25, 16).reshape(exact.shape) * 2.0**-21
        assert (np.abs(y.astype(np.float64) - exact.astype(np.float64)) <= bound + 1e-45).all()
    else:
        assert np.array_equal(y, exact)
    assert float(amax) == float(np.abs(y).max())
    for cfg in (dict(scale_rule="mse"), dict(scale_rule="static_6", block_scale_2d=shape[0] % 16 == 0 and shape[1] % 16 == 0)):
        q = fos.quantize(x.cuda(), fos.QuantizationConfig(transpose=transpose, rht=rht, **cfg))
        ref = oracle.quantize(torch.from_numpy(y), **cfg)
        assert q.original_shape == ((shape[1], shape[0]) if transpose else shape)
        assert float(q.amax) == float(ref.amax)
        assert np.array_equal(u8(q.values), ref.values) and np.array_equal(u8(q.scale_factors).reshape(-1), ref.scale_factors)


WEIGHT_CASES = [(shape, "weight", cfg)
                for shape in ((4096, 4096), (14336, 4096), (4096, 14336))
                for cfg in (dict(scale_rule="mse", block_scale_2d=True), dict(scale_rule="static_6", block_scale_2d=True),
                            dict(dtype="if4", scale_rule="mse", block_scale_2d=True))]


@pytest.mark.parametrize(("shape", "kind", "cfg"), [
    ((8192, 4096), "outlier", dict(scale_rule="mse")),            # activation-style
    ((8192, 8192), "randn", dict(scale_rule="mse")),              # headline size
    ((8192, 8192), "randn", dict(scale_rule="static_6")),
    *WEIGHT_CASES,                                                # Llama-3-8B weight shapes x {4/6-MSE, static_6, IF4}, 16 x 16 blocks
    ((16384, 4096), "randn", dict(scale_rule="mse")),             # the decoder stack's activations
    ((16384, 14336), "randn", dict(scale_rule="mse")),            # ... the down projection's
    ((2048, 4096), "weight", dict(dtype="if4", scale_rule="mse")),
    # the other two adaptive rules through their certified shortcuts: 4 M blocks each, the closest calls among
    # them a few 1e-7 apart, plus the stochastic style on top
    ((8192, 8192), "randn", dict(scale_rule="mae")),
    ((8192, 8192), "randn", dict(scale_rule="abs_max")),
    ((8192, 4096), "outlier", dict(scale_rule="mae")),
    ((8192, 8192), "randn", dict(scale_rule="mae", block_scale_2d=True)),
    ((4096, 14336), "weight", dict(scale_rule="mae", block_scale_2d=True)),
    ((8192, 8192), "randn", dict(scale_rule="abs_max", block_scale_2d=True)),
    ((14336, 4096), "weight", dict(scale_rule="abs_max", block_scale_2d=True)),
    ((8192, 4096), "outlier", dict(scale_rule="abs_max")),
    ((4096, 4096), "weight", dict(scale_rule="mae", round_style="stochastic", seed=5)),
    ((4096, 4096), "weight", dict(scale_rule="abs_max", round_style="stochastic", seed=6)),
], ids=str)
def test_full_size_workloads_bit_exact(oracle, shape, kind, cfg):
    x = make_input(kind, shape, 1)
    cfg = dict(cfg)
    seed = cfg.pop("seed", None)
    q = hip_quantize(x, **cfg, **({} if seed is None else {"kwargs": {"seed": seed}}))
    ref = oracle.quantize(x, **cfg, **({} if seed is None else {"seed": seed}))
    assert_same_quantization(q, ref, f"{shape} {cfg}")
    # size-independent properties: block holding the tensor maximum gets the top scale,
    # 2-D tiles carry 16 equal scale bytes
    if cfg.get("dtype", "nvfp4") == "nvfp4" and cfg["scale_rule"] in ("static_6", "mse") and seed is None:
        rows = oracle.from_blocked(u8(q.scale_factors).reshape(-1), shape[0], shape[1] // 16)
        # static_6: the block with the tensor maximum scales to 448 (0x7E); 4/6: to 256
        # (0x78) or, if it picked "4", up to 384 (0x7C)
        lo, hi = {"static_6": (0x7E, 0x7E), "mse": (0x78, 0x7C)}[cfg["scale_rule"]]
        assert lo <= int(rows.max()) <= hi
        if cfg.get("block_scale_2d"):
            t = rows.reshape(shape[0] // 16, 16, -1)
            assert (t == t[:, :1]).all()


@pytest.mark.parametrize("tile_map", range(1, 9))
def test_tile_orders_give_the_same_bytes(monkeypatch, oracle, tile_map):
    """FOS_QUANT_MAP only changes which workgroup quantizes which tile (row-major, one band per XCD,
    column-major, the 16x16 kernel's column windows apart or side by side) and FOS_QUANT_GRID how many
    workgroups share the tiles: the output does not depend on either, also for widths that leave an
    incomplete run of windows and for ragged shapes."""
    monkeypatch.setenv("FOS_QUANT_MAP", str(tile_map))
    monkeypatch.setenv("FOS_QUANT_GRID", "24")
    for shape in ((1024, 4096 + 1536), (384, 8192), (200, 1200)):
        x = make_input("randn", shape, 17)
        for cfg in (dict(scale_rule="mse"), dict(scale_rule="mse", block_scale_2d=True), dict(scale_rule="static_6", block_scale_2d=True),
                    dict(dtype="if4", scale_rule="mse", block_scale_2d=True)):
            assert_same_quantization(hip_quantize(x, **cfg), oracle.quantize(x, **cfg), f"{shape} {cfg} map {tile_map}")


@pytest.mark.parametrize("shape", [(100, 80), (16, 64), (1, 16), (130, 8), (257, 1000), (128, 72)])
def test_ragged_shapes_are_zero_padded(oracle, shape):
    x = make_input("randn", shape, 3)
    for cfg in (dict(scale_rule="mse"), dict(scale_rule="static_6", block_scale_2d=True), dict(dtype="if4", scale_rule="mae"),
                dict(dtype="if4", scale_rule="mse"), dict(dtype="if4", scale_rule="mse", block_scale_2d=True)):
        assert_same_quantization(hip_quantize(x, **cfg), oracle.quantize(x, **cfg), f"{shape} {cfg}")


@pytest.mark.parametrize("scale", [2.0**-110, 2.0**-118, 2.0**105])
@pytest.mark.parametrize("two_d", [False, True], ids=["1d", "2d"])
def test_extreme_ranges_take_the_operation_by_operation_path(oracle, scale, two_d):
    """Tensors whose maximum leaves [2^-100, 2^100] (fp32 intermediates of the scale math
    go sub-normal or overflow) must still match the oracle bit for bit."""
    x = (make_input("randn", (256, 128), 12).float() * scale).bfloat16()
    for rule in ("mse", "static_6", "abs_max"):
        q = hip_quantize(x, scale_rule=rule, block_scale_2d=two_d)
        ref = oracle.quantize(x, scale_rule=rule, block_scale_2d=two_d)
        assert_same_quantization(q, ref, f"scale {scale} {rule}")
    q = hip_quantize(x, dtype="if4", scale_rule="mse", block_scale_2d=two_d)
    assert_same_quantization(q, oracle.quantize(x, dtype="if4", scale_rule="mse", block_scale_2d=two_d), f"scale {scale} if4")


_FAR_CONFIGS = [dict(scale_rule="mse"), dict(scale_rule="mse", block_scale_2d=True), dict(scale_rule="mae"),
                dict(scale_rule="mae", block_scale_2d=True), dict(scale_rule="abs_max", block_scale_2d=True),
                dict(scale_rule="mse", round_style="stochastic"), dict(scale_rule="mse", round_style="stochastic", block_scale_2d=True),
                dict(dtype="if4", scale_rule="mse"), dict(dtype="if4", scale_rule="mse", block_scale_2d=True)]


@pytest.mark.parametrize("cfg", _FAR_CONFIGS, ids=lambda c: "-".join(str(v) for v in c.values()))
@pytest.mark.parametrize("exponent", [-98, -90, -72, -66, -61, -59, -50, -41, -39, -30, 30, 39, 41, 59, 61, 90, 99])
def test_tensor_maxima_far_from_one(oracle, exponent, cfg):
    """The certified shortcuts model the reference's error sums with relative rounding errors, which holds
    only while the reference's own fp32 squares and sums neither underflow nor overflow: a tensor of
    values around 2^-70 has every squared error flushed to zero there, so every block ties and takes the
    first candidate.  The kernels decide from their shortcuts for tensor maxima in [2^-40, 2^40] (with
    the weights taken relative to the maximum's power of two) and evaluate exactly beyond.  Every
    shortcut against the oracle, bit for bit, on both sides of the limits."""
    x = (make_input("randn", (512, 1024), 14).float() * 2.0**exponent).bfloat16()
    kw = {"kwargs": {"seed": 3}} if "round_style" in cfg else {}
    okw = {"seed": 3} if "round_style" in cfg else {}
    assert_same_quantization(hip_quantize(x, **cfg, **kw), oracle.quantize(x, **cfg, **okw), f"2^{exponent} {cfg}")
    if cfg.get("dtype", "nvfp4") == "nvfp4" and "round_style" not in cfg:
        r = fos.quantize(x.cuda(), fos.QuantizationConfig(pseudo_quantize=True, **cfg))
        q = hip_quantize(x, **cfg)
        assert torch.equal(r.view(torch.int16), fos.dequantize(q, dtype=torch.bfloat16).view(torch.int16))


@pytest.mark.parametrize("two_d", [False, True], ids=["1d", "2d"])
def test_if4_mse_fast_path_inputs(oracle, two_d):
    """IF4 with the MSE rule decides most blocks from sums in the scaled domain; inputs that
    make the two candidates tie or nearly tie (constant blocks, 0/1 data, outlier channels,
    blocks with tiny scales) must fall through to the exact evaluation and still match."""
    for kind, shape, seed in (("ones", (128, 256), 0), ("rand01", (256, 256), 1), ("outlier", (256, 1024), 2),
                              ("tiny_blocks", (256, 512), 3), ("weight", (512, 512), 4), ("randn", (1024, 1024), 5)):
        x = make_input(kind, shape, seed)
        q = hip_quantize(x, dtype="if4", scale_rule="mse", block_scale_2d=two_d)
        assert_same_quantization(q, oracle.quantize(x, dtype="if4", scale_rule="mse", block_scale_2d=two_d), kind)
    x = make_input("randn", (256, 256), 6)
    given = float(np.float32(float(x.abs().max()) * 1.2345678))
    q = fos.quantize(x.cuda(), fos.QuantizationConfig(dtype="if4", block_scale_2d=two_d, kwargs={"amax": torch.tensor(given, device="cuda")}))
    assert_same_quantization(q, oracle.quantize(x, dtype="if4", block_scale_2d=two_d, amax=given), "24-bit maximum")


def _near_tie_cases(golden_dir):
    d = np.load(os.path.join(golden_dir, "near_ties.npz"))
    return d, sorted(k[:-2] for k in d.files if k.endswith(".x"))


def test_near_ties_take_the_exact_decision(oracle, golden_dir):
    """Blocks and tiles whose two candidate errors differ by a few units in the last place (found
    by a CPU search, tests/golden/make_near_ties.py): the kernels' certified shortcuts must hand
    every one of them to the exact evaluation.  4/6 under the MSE, MAE and abs-max rules and IF4,
    1-D and 2-D, tensor maximum from the data and a caller-supplied 24-bit maximum, round to nearest
    and the stochastic style (whose candidates are the stochastically rounded ones of the stored
    seed); round to nearest also under the fused pseudo-quantize epilogue."""
    d, cases = _near_tie_cases(golden_dir)
    rules = set()
    for case in cases:
        parts = case.split(".")
        dtype, two_d, rule, style, given = parts[0], parts[1] == "2d", parts[2], parts[3], len(parts) == 5
        rules.add((dtype, two_d, rule, style))
        x = torch.from_numpy(d[case + ".x"].view(np.int16).copy()).view(torch.bfloat16)
        amax, seed = float(d[case + ".amax"][0]), int(d[case + ".seed"][0])
        kwargs = {"amax": torch.tensor(amax, device="cuda")} if given else {}
        if style != "nearest":
            kwargs["seed"] = seed
        q = fos.quantize(x.cuda(), fos.QuantizationConfig(dtype=dtype, scale_rule=rule, round_style=style, block_scale_2d=two_d, kwargs=kwargs))
        ref = oracle.quantize(x, dtype=dtype, scale_rule=rule, round_style=style, block_scale_2d=two_d, seed=seed, amax=amax if given else None)
        assert_same_quantization(q, ref, case)
        if dtype == "nvfp4" and style == "nearest":
            r = fos.quantize(x.cuda(), fos.QuantizationConfig(scale_rule=rule, block_scale_2d=two_d, pseudo_quantize=True, kwargs=kwargs))
            assert torch.equal(r.view(torch.int16), fos.dequantize(q, dtype=torch.bfloat16).view(torch.int16)), case
    # every instantiation that decides from a shortcut has a case
    for need in (("nvfp4", False, "mse", "nearest"), ("nvfp4", True, "mse", "nearest"), ("nvfp4", False, "mae", "nearest"),
                 ("nvfp4", True, "mae", "nearest"), ("nvfp4", True, "abs_max", "nearest"), ("if4", False, "mse", "nearest"),
                 ("if4", True, "mse", "nearest"), ("nvfp4", False, "mse", "stochastic"), ("nvfp4", False, "mae", "stochastic"),
                 ("nvfp4", True, "mse", "stochastic")):
        assert need in rules, need


def test_near_ties_on_fp16_inputs(oracle, golden_dir):
    """The same near-tie blocks handed over as fp16 tensors (every bf16 value of the fixture, at most 8
    in magnitude, is an fp16 value too): the fp16 instantiation of the 1 x 16 streaming kernel decides
    them as the oracle does on the fp16 input."""
    d, cases = _near_tie_cases(golden_dir)
    for case in cases:
        parts = case.split(".")
        if parts[0] != "nvfp4" or parts[1] != "1d" or parts[3] != "nearest" or len(parts) == 5:
            continue
        x = torch.from_numpy(d[case + ".x"].view(np.int16).copy()).view(torch.bfloat16).half()
        q = fos.quantize(x.cuda(), fos.QuantizationConfig(scale_rule=parts[2]))
        assert_same_quantization(q, oracle.quantize(x, scale_rule=parts[2]), case + " as fp16")


def test_negative_zero_inputs(oracle):
    """-0.0 encodes as +0 (the reference multiplies by sign(x)); a small negative value
    that rounds to zero keeps its sign bit."""
    x = make_input("randn", (256, 256), 13)
    x[::3, ::5] = -0.0
    x[1::7, 3::11] = -1e-4
    for cfg in (dict(scale_rule="mse"), dict(scale_rule="static_6"), dict(scale_rule="mse", block_scale_2d=True),
                dict(dtype="if4", scale_rule="mse")):
        assert_same_quantization(hip_quantize(x, **cfg), oracle.quantize(x, **cfg), str(cfg))
    x[:, :] = -0.0
    q = hip_quantize(x, scale_rule="mse")
    assert int(u8(q.values).max()) == 0 and int(u8(q.scale_factors).max()) == 0


def test_strided_and_unaligned_inputs(oracle):
    base = make_input("randn", (256, 384), 4).cuda()
    view = base[:, 64:320]                      # ld 384, cols 256, 16-byte aligned
    ref = oracle.quantize(view.cpu().contiguous(), scale_rule="mse")
    assert_same_quantization(fos.quantize(view), ref, "strided")
    flat = make_input("randn", (1, 256 * 130 + 1), 5).cuda().reshape(-1)
    odd = flat[1:].reshape(256, 130)[:, :128]   # 2-byte aligned only, ld 130
    ref = oracle.quantize(odd.cpu().contiguous(), scale_rule="mse")
    assert_same_quantization(fos.quantize(odd), ref, "unaligned")
    ref = oracle.quantize(base.T.contiguous().cpu(), scale_rule="static_6")
    assert_same_quantization(fos.quantize(base.T, fos.QuantizationConfig(scale_rule="static_6")), ref, "transposed view")


def test_caller_supplied_amax(oracle):
    x = make_input("randn", (256, 256), 6)
    ref = oracle.quantize(x, scale_rule="mse")
    amax = torch.tensor(float(ref.amax), device="cuda")
    q = fos.quantize(x.cuda(), fos.QuantizationConfig(kwargs={"amax": amax}))
    assert_same_quantization(q, ref, "amax given")
    # a maximum that is not a bf16 value (24 significant bits, larger than max|x|), on inputs
    # whose blocks tie or nearly tie: the undecided blocks must take the generic evaluation
    for kind, shape in (("randn", (1024, 1024)), ("rand01", (256, 256)), ("outlier", (256, 1024))):
        x = make_input(kind, shape, 7)
        given = float(np.float32(float(x.abs().max()) * 1.2345678))
        for cfg in (dict(scale_rule="mse"), dict(scale_rule="mse", block_scale_2d=True), dict(scale_rule="static_6"),
                    dict(scale_rule="mse", round_style="stochastic", kwargs={"seed": 3})):
            ocfg = {k: v for k, v in cfg.items() if k != "kwargs"}
            ref = oracle.quantize(x, amax=given, seed=cfg.get("kwargs", {}).get("seed", 0), **ocfg)
            kw = dict(cfg.get("kwargs", {}), amax=torch.tensor(given, device="cuda"))
            q = fos.quantize(x.cuda(), fos.QuantizationConfig(**{**ocfg, "kwargs": kw}))
            assert_same_quantization(q, ref, f"{kind} {cfg}")


@pytest.mark.parametrize(("rows", "cols", "ld"), [
    (2051, 4096, 4096),     # window order (cols % 2048 == 0, >= 16 MiB), rows not a multiple of anything
    (4096, 2048, 2048 + 64),  # the same scan over a strided view
    (1024, 8192, 8192),     # exactly one step of the window-order scan
    (1023, 8192, 8192),     # just below it: the flat scan
    (3000, 6144, 6144),
    (777, 14336, 14336),
])
def test_tensor_maximum_scan_covers_every_element(rows, cols, ld):
    """pass 1 reads every element exactly where the tensor says it is: a single non-zero element, moved
    through corners, row ends and random places, is the maximum each time (and a larger value in the
    gap of a strided view is not)."""
    from fouroversix_amd import _native as nat

    L = nat.lib()
    dev = torch.device("cuda", 0)
    base = torch.zeros(rows, ld, dtype=torch.bfloat16, device=dev)
    if ld > cols:
        base[:, cols:] = 1000.0
    amax = torch.zeros(1, dtype=torch.float32, device=dev)
    ws_bytes = L.fos_quantize_workspace_bytes(rows, cols)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = nat.current_stream(dev)
    rng = np.random.default_rng(rows * 31 + cols)
    spots = [(0, 0), (0, cols - 1), (rows - 1, 0), (rows - 1, cols - 1), (rows - 1, cols - 257), (rows // 2, 255), (rows // 2, 256),
             (1, 2047), (rows - 2, 2048 % cols)]
    spots += [(int(rng.integers(rows)), int(rng.integers(cols))) for _ in range(40)]
    for k, (r, c) in enumerate(spots):
        value = -(2.0 + k) if k % 2 else 2.0 + k
        base[r, c] = value
        nat.check(L.fos_amax(base.data_ptr(), nat.T_BF16, rows, cols, ld, amax.data_ptr(), ws.data_ptr(), ws_bytes, stream), "amax")
        assert float(amax.item()) == abs(value), (rows, cols, ld, r, c)
        base[r, c] = 0.0
    # and the quantizer behind it sees the same maximum
    base[rows - 1, cols - 1] = 3.0
    q = fos.quantize(base[:, :cols], fos.QuantizationConfig(scale_rule="static_6"))
    assert float(q.amax) == 3.0


def test_two_pass_quantize_replays_in_a_hip_graph():
    """A 32 MiB input (tensor-maximum scan in window order + streaming pass 2, non-temporal code stores)
    captured in a HIP graph: every replay, with eager work and synchronisations in between, equals the
    eager result on the input's new contents."""
    cfg = fos.QuantizationConfig(scale_rule="mse")
    static_x = make_input("randn", (4096, 4096), 90).cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fos.quantize(static_x, cfg)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_q = fos.quantize(static_x, cfg)
    for i in range(4):
        xi = make_input("randn", (4096, 4096), 91 + i).cuda() * float(i + 1)
        static_x.copy_(xi)
        graph.replay()
        torch.cuda.synchronize()
        eager = fos.quantize(xi, cfg)
        torch.cuda.synchronize()
        assert torch.equal(static_q.values, eager.values), f"replay {i}"
        assert torch.equal(static_q.scale_factors.view(torch.uint8), eager.scale_factors.view(torch.uint8)), f"replay {i}"
        assert float(static_q.amax) == float(eager.amax), f"replay {i}"


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_configurations_match_the_oracle(oracle, seed):
    """120 configurations per seed drawn over shape (whole and ragged workgroup tiles, single rows), format, rule,
    rounding style, block shape, input type, input kind and tensor scale: codes, scales and maximum are the
    oracle's, and a fused round trip equals dequantize(quantize(x)) bit for bit."""
    import random

    rng = random.Random(seed)
    for it in range(120):
        rows = rng.choice([1, 16, 37, 100, 128, 130, 256, 384, 512, 777])
        cols = rng.choice([16, 48, 80, 256, 272, 512, 528, 1024, 1040, 2048])
        fmt = rng.choice(["nvfp4", "nvfp4", "nvfp4", "if4"])
        rule = rng.choice(["mse", "mae", "abs_max"] + ([] if fmt == "if4" else ["static_6", "static_4"]))
        kw = dict(dtype=fmt, scale_rule=rule, round_style=rng.choice(["nearest", "stochastic", "stochastic", "stochastic_unbiased"]),
                  block_scale_2d=rng.random() < 0.5)
        kind = rng.choice(["randn", "outlier", "tiny_blocks", "weight", "rand01"])
        if kind == "tiny_blocks" and cols % 16:
            kind = "randn"
        scale = rng.choice([1.0, 1.0, 2.0**-20, 2.0**30, 2.0**-50, 3e4])
        dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        x = make_input(kind, (rows, cols), 1000 * seed + it).float() * scale
        x = (x.clamp(-6e4, 6e4) if dtype == torch.float16 else x).to(dtype)
        key = dict(seed=rng.randrange(2**40), offset=rng.randrange(100))
        what = f"case {it}: {rows}x{cols} {kw} {kind} x {scale} {dtype} {key}"
        q = fos.quantize(x.cuda(), fos.QuantizationConfig(**kw, kwargs=key))
        assert_same_quantization(q, oracle.quantize(x, **key, **kw), what)
        if rng.random() < 0.3:
            p = fos.quantize(x.cuda(), fos.QuantizationConfig(**kw, pseudo_quantize=True, kwargs=key))
            bits = torch.int32 if dtype == torch.float32 else torch.int16
            assert torch.equal(p.view(bits), fos.dequantize(q, dtype=dtype).view(bits)), what


@pytest.mark.parametrize(("shape", "cfg"), [
    ((256, 512), dict(scale_rule="mse")), ((256, 512), dict(scale_rule="mse", block_scale_2d=True)),
    ((100, 80), dict(scale_rule="mae", block_scale_2d=True)), ((128, 256), dict(scale_rule="static_6", round_style="stochastic_unbiased")),
    ((128, 256), dict(dtype="if4", scale_rule="mse")), ((128, 264), dict(scale_rule="abs_max", round_style="stochastic_unbiased")),
])
def test_dither_key_read_from_device_memory(shape, cfg):
    """kwargs['key'] (int64[2] on the device: seed, offset) gives the bytes of the same two integers passed as
    launch arguments, on every kernel that rounds stochastically (streaming 1x16 and 16x16, element-wise)."""
    kw = {"round_style": "stochastic", **cfg}
    x = make_input("randn", shape, 60).cuda()
    key = torch.tensor([2**40 + 99, 3], dtype=torch.int64, device="cuda")
    for src in (x, x.float()):
        q = fos.quantize(src, fos.QuantizationConfig(**kw, kwargs={"key": key}))
        ref = fos.quantize(src, fos.QuantizationConfig(**kw, kwargs={"seed": 2**40 + 99, "offset": 3}))
        assert torch.equal(q.values, ref.values) and torch.equal(q.scale_factors.view(torch.uint8), ref.scale_factors.view(torch.uint8))
    p = fos.quantize(x, fos.QuantizationConfig(**kw, pseudo_quantize=True, kwargs={"key": key}))
    ref = fos.quantize(x, fos.QuantizationConfig(**kw, kwargs={"seed": 2**40 + 99, "offset": 3}))
    assert torch.equal(p, fos.dequantize(ref, dtype=x.dtype))
    with pytest.raises(RuntimeError, match="key"):
        fos.quantize(x, fos.QuantizationConfig(**kw, kwargs={"key": key.int()}))


def test_captured_stochastic_rounding_advances_its_key():
    """A stochastic quantize recorded into a HIP graph together with an increment of its key's offset rounds
    with fresh bits on every replay: replay i equals the eager call with offset i (a launch argument would
    freeze the bits drawn at capture)."""
    cfg = dict(scale_rule="mse", round_style="stochastic")
    x = make_input("randn", (512, 1024), 61).cuda()
    key = torch.tensor([7, 0], dtype=torch.int64, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fos.quantize(x, fos.QuantizationConfig(**cfg, kwargs={"key": key}))
            key[1:].add_(1)
    torch.cuda.current_stream().wait_stream(side)
    key.copy_(torch.tensor([7, 0], dtype=torch.int64))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_q = fos.quantize(x, fos.QuantizationConfig(**cfg, kwargs={"key": key}))
        key[1:].add_(1)
    seen = []
    for i in range(4):
        graph.replay()
        torch.cuda.synchronize()
        eager = fos.quantize(x, fos.QuantizationConfig(**cfg, kwargs={"seed": 7, "offset": i}))
        torch.cuda.synchronize()
        assert torch.equal(static_q.values, eager.values), f"replay {i}"
        assert torch.equal(static_q.scale_factors.view(torch.uint8), eager.scale_factors.view(torch.uint8)), f"replay {i}"
        seen.append(static_q.values.clone())
    assert not torch.equal(seen[0], seen[1])
    assert int(key[1]) == 4


@pytest.mark.parametrize("shape", [(16, 4096), (4, 4096), (16, 1024), (1, 8192), (16, 4064)])
def test_decode_sized_quantize_eager_and_captured(oracle, shape):
    """Decode-sized inputs take one launch (every workgroup scans the tensor for its maximum) up to
    32 KiB, and up to 128 KiB when the call is not being captured; above, two launches.  Eager
    and captured calls of the same input -- which differ in form between those limits -- give the
    same bytes, those of the oracle, on every replay."""
    cfg = fos.QuantizationConfig(scale_rule="mse")
    static_x = make_input("randn", shape, 70).cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fos.quantize(static_x, cfg)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_q = fos.quantize(static_x, cfg)
    for i in range(3):
        xi = make_input("randn", shape, 71 + i) * float(2 * i + 1)
        static_x.copy_(xi.cuda())
        graph.replay()
        torch.cuda.synchronize()
        eager = fos.quantize(xi.cuda(), cfg)
        ref = oracle.quantize(xi, scale_rule="mse")
        for q in (static_q, eager):
            assert np.array_equal(u8(q.values), ref.values), f"replay {i}"
            assert np.array_equal(u8(q.scale_factors), ref.scale_factors), f"replay {i}"
            assert float(q.amax) == float(ref.amax), f"replay {i}"


@pytest.mark.parametrize("cfg", [dict(scale_rule="mse"), dict(scale_rule="static_6", block_scale_2d=True), dict(dtype="mxfp4", scale_rule="static_6")],
                         ids=["nvfp4-mse-1d", "nvfp4-static6-2d", "mxfp4"])
def test_tensors_beyond_four_gib(cfg):
    """A 49152 x 49152 input (4.5 GiB, 2^31.2 elements): byte offsets and element counts beyond 32 bits.  Its
    quantization equals that of its four row bands quantized on their own with the tensor's maximum."""
    rows = cols = 49152
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.empty(rows, cols, dtype=torch.bfloat16, device="cuda")
    for r in range(0, rows, 8192):
        x[r : r + 8192] = torch.randn(8192, cols, generator=g, device="cuda").bfloat16()
    x[rows - 1, cols - 1] = 40.0  # the maximum sits in the last element
    q = fos.quantize(x, fos.QuantizationConfig(**cfg))
    mx = cfg.get("dtype") == "mxfp4"
    if not mx:
        assert float(q.amax) == 40.0
    block = 32 if mx else 16
    sf = q.scale_factors.view(torch.uint8).reshape(-1)
    band = rows // 4
    for i in range(4):
        kw = {} if mx else {"kwargs": {"amax": q.amax.reshape(1)}}
        qb = fos.quantize(x[i * band : (i + 1) * band], fos.QuantizationConfig(**cfg, **kw))
        assert torch.equal(qb.values, q.values[i * band : (i + 1) * band]), (cfg, i)
        n = band * cols // block  # the tiled layout keeps 128-row bands contiguous
        assert torch.equal(qb.scale_factors.view(torch.uint8).reshape(-1), sf[i * n : (i + 1) * n]), (cfg, i)
        del qb
    del x, q
    torch.cuda.empty_cache()


def test_concurrent_streams_do_not_share_the_workspace(oracle):
    """Two streams quantize different tensors at the same time (the two-launch path, which
    hands partial maxima from pass 1 to pass 2 through a per-stream workspace)."""
    xs = [make_input("randn", (1024, 2048), 50 + i) * (1.0 + 3.0 * i) for i in range(2)]
    refs = [oracle.quantize(x, scale_rule="mse") for x in xs]
    dev = [x.cuda() for x in xs]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    outs = [[], []]
    for _ in range(8):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                outs[i].append(fos.quantize(dev[i]))
    torch.cuda.synchronize()
    for i in range(2):
        for q in outs[i]:
            assert_same_quantization(q, refs[i], f"stream {i}")


def test_reference_op_schema(oracle):
    """torch.ops.fouroversix.quantize with the reference's positional schema."""
    x = make_input("randn", (256, 128), 7)
    from fouroversix_amd.quantize import ops

    values, sf, amax = ops.quantize(x.cuda(), True, True, False, False, False, fos.ScaleRule.mse.cuda_id, -1)
    ref = oracle.quantize(x, scale_rule="mse")
    assert values.shape == (256, 64) and sf.shape == (256 * 8,) and amax.shape == (1,)
    assert np.array_equal(u8(values), ref.values) and np.array_equal(u8(sf), ref.scale_factors)
    with pytest.raises(RuntimeError, match="selection_rule"):
        ops.quantize(x.cuda(), True, True, False, False, False, 9, -1)
    with pytest.raises(RuntimeError):
        ops.quantize(x.cuda().float(), True, True, False, False, False, 0, -1)
    # fp16 is the other input type of the reference's op (csrc/quantize/fp4_quant.cu:134-136)
    h = make_input("randn", (256, 128), 7).half()
    values, sf, amax = ops.quantize(h.cuda(), True, True, False, True, False, fos.ScaleRule.mae.cuda_id, -1)
    ref = oracle.quantize(h, scale_rule="mae", block_scale_2d=True)
    assert np.array_equal(u8(values), ref.values) and np.array_equal(u8(sf), ref.scale_factors) and float(amax) == float(ref.amax)


@pytest.mark.parametrize(("dtype", "rule", "two_d"), [
    ("nvfp4", "static_6", False), ("nvfp4", "mse", False), ("nvfp4", "mse", True), ("if4", "mse", False),
    ("nvfp4", "abs_max", False), ("nvfp4", "mae", False), ("nvfp4", "static_4", True), ("nvfp4", "mae", True),
    ("if4", "abs_max", True),
])
@pytest.mark.parametrize("style", ["stochastic", "stochastic_unbiased"])
def test_stochastic_rounding_bit_exact_with_oracle_key(oracle, dtype, rule, two_d, style):
    """Same Philox key => same dither => identical bytes; different seeds differ."""
    x = make_input("randn", (512, 256), 8)
    kw = dict(dtype=dtype, scale_rule=rule, block_scale_2d=two_d, round_style=style)
    q = hip_quantize(x, kwargs={"seed": 99, "offset": 3}, **kw)
    ref = oracle.quantize(x, seed=99, offset=3, **kw)
    assert_same_quantization(q, ref, str(kw))
    q2 = hip_quantize(x, kwargs={"seed": 100, "offset": 3}, **kw)
    assert (u8(q2.values) != u8(q.values)).mean() > 0.05


@pytest.mark.parametrize("rule", ["static_6", "static_4", "mse", "mae", "abs_max"])
@pytest.mark.parametrize("style", ["stochastic", "stochastic_unbiased"])
def test_stochastic_rounding_on_tiles_bit_exact(oracle, rule, style):
    """16x16 tiles with a stochastic style on the streaming kernel: whole and ragged workgroup tiles, data whose
    tiles tie or come close (outlier channels, blocks spanning six decades), every rule; the dither is keyed per
    row of a tile, so a tile sent through the operation-by-operation path must draw the same bits."""
    for kind, shape, seed in (("randn", (256, 1024), 31), ("outlier", (384, 528), 32), ("tiny_blocks", (128, 512), 33),
                              ("weight", (1024, 2048), 34)):
        x = make_input(kind, shape, seed)
        kw = dict(scale_rule=rule, block_scale_2d=True, round_style=style)
        q = hip_quantize(x, kwargs={"seed": 1234 + seed, "offset": 2}, **kw)
        assert_same_quantization(q, oracle.quantize(x, seed=1234 + seed, offset=2, **kw), f"{kind} {shape} {kw}")


@pytest.mark.parametrize("style", ["stochastic", "stochastic_unbiased"])
def test_stochastic_rounding_edge_cases_bit_exact(oracle, style):
    """The stochastic styles on the inputs that steer the kernels off their main path:
    ragged shapes (zero padding, partial tiles), tensors outside [2^-100, 2^100] and blocks
    with sub-normal scales (operation-by-operation form), negative zeros, an input that is
    only 2-byte aligned (generic kernel), outlier channels (exact ties between the candidates)."""
    def check(x, what, **cfg):
        kw = dict(round_style=style, **cfg)
        q = hip_quantize(x, kwargs={"seed": 5, "offset": 1}, **kw)
        assert_same_quantization(q, oracle.quantize(x.cpu().contiguous(), seed=5, offset=1, **kw), f"{what} {kw}")

    for shape in ((100, 80), (1, 16), (257, 1000), (130, 272)):
        x = make_input("randn", shape, 21)
        check(x, f"ragged {shape}", scale_rule="mse")
        check(x, f"ragged {shape}", scale_rule="static_6", block_scale_2d=True)
        check(x, f"ragged {shape}", scale_rule="mse", block_scale_2d=True)
    for scale in (2.0**-110, 2.0**105):
        x = (make_input("randn", (256, 128), 12).float() * scale).bfloat16()
        for two_d in (False, True):
            check(x, f"scale {scale}", scale_rule="mse", block_scale_2d=two_d)
            check(x, f"scale {scale}", scale_rule="static_6", block_scale_2d=two_d)
    x = make_input("tiny_blocks", (256, 512), 22)
    check(x, "tiny blocks", scale_rule="mse")
    check(x, "tiny blocks", scale_rule="static_4")
    x = make_input("randn", (256, 256), 13)
    x[::3, ::5] = -0.0
    x[1::7, 3::11] = -1e-4
    check(x, "negative zeros", scale_rule="mse")
    check(x, "negative zeros", scale_rule="static_6")
    flat = make_input("randn", (1, 256 * 130 + 1), 5).cuda().reshape(-1)
    odd = flat[1:].reshape(256, 130)[:, :128]   # 2-byte aligned only, ld 130
    check(odd, "unaligned", scale_rule="mse")
    x = make_input("outlier", (256, 1024), 23)
    check(x, "outlier", scale_rule="mse")
    check(x, "outlier", scale_rule="mse", block_scale_2d=True)


def test_stochastic_rounding_known_answers():
    """The reference's SR known answers (tests/test_quantize.py:360-372) on randn 1024^2:
    torch.dist(dequantize(quantize(x)), x) within 5 % of 137 / 122 (158 / 139 unbiased)."""
    x = make_input("randn", (1024, 1024), 0).cuda()
    for rule, style, expect in (("static_6", "stochastic", 137), ("mse", "stochastic", 122),
                                ("static_6", "stochastic_unbiased", 158), ("mse", "stochastic_unbiased", 139)):
        q = fos.quantize(x, fos.QuantizationConfig(scale_rule=rule, round_style=style))
        dist = float(torch.dist(fos.dequantize(q).float(), x.float()))
        assert abs(dist - expect) / expect < 0.05, (rule, style, dist)
    # IF4 + MSE: 110 / 122 (tests/test_quantize.py:321)
    for style, expect in (("stochastic", 110), ("stochastic_unbiased", 122)):
        q = fos.quantize(x, fos.QuantizationConfig(dtype="if4", scale_rule="mse", round_style=style))
        dist = float(torch.dist(fos.dequantize(q).float(), x.float()))
        assert abs(dist - expect) / expect < 0.05, ("if4", style, dist)
    cfg = fos.QuantizationConfig(scale_rule="static_6", round_style="stochastic")
    mean_err = torch.stack([(fos.dequantize(fos.quantize(x, cfg), torch.float32) - x.float()) for _ in range(4)]).mean()
    assert abs(float(mean_err)) < 1e-3


@pytest.mark.parametrize("rule", ["mse", "static_6"])
def test_activation_style_stochastic_seeds(oracle, rule):
    """The activation-style input at its full size (8192 x 4096, 1 % outlier channels): 4/6-MSE and
    static_6 with stochastic rounding over seeds 0..9 are bit-exact for the shared key, their error
    stays within 5 % of the oracle's, and the rounding is unbiased (mean error ~ 0)."""
    x = make_input("outlier", (8192, 4096), 1)
    xf = x.float().numpy()
    dev = x.cuda()
    for seed in range(10):
        q = fos.quantize(dev, fos.QuantizationConfig(scale_rule=rule, round_style="stochastic", kwargs={"seed": seed}))
        ref = oracle.quantize(x, scale_rule=rule, round_style="stochastic", seed=seed)
        assert_same_quantization(q, ref, f"{rule} seed {seed}")
    deq = fos.dequantize(q, torch.float32).cpu().numpy()
    rdeq = oracle.dequantize(ref.values, ref.scale_rows, ref.amax, scale_rule=rule, round_style="stochastic")
    assert np.array_equal(deq, rdeq)
    assert abs(np.linalg.norm(deq - xf) / np.linalg.norm(rdeq - xf) - 1) < 0.05
    nearest = fos.dequantize(fos.quantize(dev, fos.QuantizationConfig(scale_rule=rule)), torch.float32).cpu().numpy()
    assert abs(float((deq - xf).mean())) < 5e-3 and np.linalg.norm(deq - xf) > np.linalg.norm(nearest - xf)


@pytest.mark.parametrize(("dtype", "rule"), [("nvfp4", "mse"), ("nvfp4", "static_4"), ("if4", "mse")])
@pytest.mark.parametrize("out", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize(("kind", "shape"), [("tiny_blocks", (200, 144)),
                                             ("randn", (300, 1024)),  # whole wavefronts per row: fp32 output as whole lines
                                             ("randn", (3, 2560))])
def test_dequantize_bit_exact(oracle, dtype, rule, out, kind, shape):
    x = make_input(kind, shape, 9)
    q = hip_quantize(x, dtype=dtype, scale_rule=rule)
    ref = oracle.quantize(x, dtype=dtype, scale_rule=rule)
    expect = torch.from_numpy(oracle.dequantize(ref.values, ref.scale_rows, ref.amax, dtype=dtype, scale_rule=rule,
                                                original_shape=shape).copy()).to(out)
    got = fos.dequantize(q, out).cpu()
    assert got.shape == shape and got.dtype == out
    assert torch.equal(got.view(torch.int16 if out != torch.float32 else torch.int32),
                       expect.view(torch.int16 if out != torch.float32 else torch.int32))


def test_dequantize_with_f32_intermediate_matches_reference_vectors(golden_dir):
    """dequantize(..., intermediate_dtype=torch.float32) on codes and scales written by the
    reference (IF4 with integer blocks, MXFP4 with scales below fp16's range, NVFP4), against
    the reference's own outputs, bit for bit."""
    from fouroversix_amd.utils import DataType, RoundStyle, ScaleRule

    z = np.load(os.path.join(golden_dir, "dequantize_f32_intermediate.npz"))
    keys = sorted({k.rsplit(".", 1)[0] for k in z.files})
    assert len(keys) == 16
    for key in keys:
        _, dtype, rule = key.split(".")
        sf = torch.from_numpy(z[key + ".sf"].reshape(-1).copy()).cuda()
        sf = sf.view(torch.float8_e8m0fnu if dtype == "mxfp4" else torch.float8_e4m3fn)
        q = fos.QuantizedTensor(
            torch.from_numpy(z[key + ".values"].copy()).cuda(), sf,
            torch.tensor(float(z[key + ".amax"][0]), device="cuda"), DataType(dtype), tuple(int(v) for v in z[key + ".shape"]),
            ScaleRule(rule), RoundStyle.nearest, tuple(int(v) for v in z[key + ".padded"]),
            scale_factors_are_in_blackwell_layout=bool(z[key + ".blocked"][0]),
        )
        got32 = fos.dequantize(q, torch.float32, intermediate_dtype=torch.float32).cpu().numpy()
        assert np.array_equal(got32.view(np.uint32), z[key + ".deq_f32"].view(np.uint32)), key
        got16 = fos.dequantize(q, torch.bfloat16, intermediate_dtype=torch.float32)
        assert np.array_equal(bits16(got16), z[key + ".deq_bf16"]), key


@pytest.mark.parametrize("two_d", [False, True])
@pytest.mark.parametrize("rule", ["mse", "mae", "abs_max", "static_6", "static_4"])
@pytest.mark.parametrize(
    ("kind", "shape", "scale"),
    [
        ("randn", (512, 1024), 1.0),
        ("outlier", (256, 512), 1.0),
        ("tiny_blocks", (200, 144), 1.0),   # ragged rows, cols % 64 != 0, sub-normal block scales
        ("rand01", (128, 256), 1.0),
        ("zeros", (128, 64), 1.0),
        ("randn", (130, 272), 2.0 ** -110),  # outside the fast range: IEEE division path
        ("randn", (128, 256), 2.0 ** 105),
    ],
)
def test_pseudo_quantize_is_the_round_trip(kind, shape, scale, rule, two_d):
    """quantize(pseudo_quantize=True), one fused kernel, is bit-identical to
    dequantize(quantize(x), dtype=x.dtype) (reference tests/test_quantize.py:391-458;
    QuantizeBackendBase.pseudo_quantize, quantize/backend.py:213-234), signs of zeros
    included."""
    x = (make_input(kind, shape, 10).float() * scale).bfloat16()
    x[0, :16] = -x[0, :16].abs()
    x[1, 3] = -0.0
    x = x.cuda()
    assert fos.quantize.__module__ and fos.quantize  # public entry
    from fouroversix_amd.quantize import ops

    assert ops.pseudo_quantize_is_fused(x, 0, fos.QuantizationConfig(scale_rule=rule).scale_rule.cuda_id, 0, two_d)
    r = fos.quantize(x, fos.QuantizationConfig(scale_rule=rule, block_scale_2d=two_d, pseudo_quantize=True))
    e = fos.dequantize(fos.quantize(x, fos.QuantizationConfig(scale_rule=rule, block_scale_2d=two_d)), dtype=x.dtype)
    assert isinstance(r, torch.Tensor) and r.dtype == torch.bfloat16 and r.shape == x.shape
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))


def test_pseudo_quantize_unfused_cases_and_amax():
    """Configurations without a fused kernel take the two-step path (same result type);
    a caller-supplied amax is honoured by the fused kernel."""
    from fouroversix_amd.quantize import ops

    x = make_input("randn", (256, 200), 3).cuda()  # cols % 16 != 0
    assert not ops.pseudo_quantize_is_fused(x, 0, 3, 0, False)
    r = fos.quantize(x, fos.QuantizationConfig(pseudo_quantize=True))
    e = fos.dequantize(fos.quantize(x), dtype=x.dtype)
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))
    x = make_input("randn", (256, 256), 4).cuda()
    cfg = dict(scale_rule="mse", round_style="stochastic", kwargs={"seed": 5})
    r = fos.quantize(x, fos.QuantizationConfig(pseudo_quantize=True, **cfg))
    e = fos.dequantize(fos.quantize(x, fos.QuantizationConfig(**cfg)), dtype=x.dtype)
    assert torch.equal(r, e)
    r = fos.quantize(x, fos.QuantizationConfig(dtype="if4", pseudo_quantize=True))
    assert torch.equal(r, fos.dequantize(fos.quantize(x, fos.QuantizationConfig(dtype="if4")), dtype=x.dtype))
    amax = torch.tensor(8.0, device="cuda")
    r = fos.quantize(x, fos.QuantizationConfig(pseudo_quantize=True, kwargs={"amax": amax}))
    e = fos.dequantize(fos.quantize(x, fos.QuantizationConfig(kwargs={"amax": amax})), dtype=x.dtype)
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))


_FUSED_ROUND_TRIPS = (
    [("nvfp4", r, "nearest", torch.float16) for r in ("static_6", "static_4", "mse", "mae", "abs_max")]
    + [("nvfp4", r, "stochastic", torch.bfloat16) for r in ("static_6", "static_4", "mse", "mae", "abs_max")]
    + [("nvfp4", r, "stochastic_unbiased", torch.bfloat16) for r in ("static_6", "mse")]
    + [("if4", "mse", "nearest", torch.bfloat16)]
)


@pytest.mark.parametrize(("fmt", "rule", "style", "dtype"), _FUSED_ROUND_TRIPS)
@pytest.mark.parametrize(("shape", "scale"), [((256, 512), 1.0), ((200, 208), 1.0), ((128, 256), 2.0**-30), ((384, 1024), 3.0e4)])
def test_fused_round_trip_of_the_other_formats_and_styles(fmt, rule, style, dtype, shape, scale):
    """The fused kernels for fp16 inputs, the stochastic styles and IF4 (1x16 blocks) return, bit for bit, what
    dequantize(quantize(x), dtype=x.dtype) returns under the same dither key (the reference's fused kernel
    covers every format and style: src/fouroversix/kernels/triton/ops.py:212-374)."""
    from fouroversix_amd.quantize import ops

    jitter = 1 + 2.0**-9 * torch.randn(shape, generator=torch.Generator("cpu").manual_seed(22))  # (fills fp16's mantissa)
    x = (make_input("outlier", shape, 21).float() * jitter * scale).to(dtype)
    x[0, :16] = -x[0, :16].abs()
    x[1, 3] = -0.0
    x[2] = 0
    x = x.cuda()
    kw = dict(dtype=fmt, scale_rule=rule, round_style=style, kwargs={"seed": 77, "offset": 3})
    cfg = fos.QuantizationConfig(**kw)
    assert ops.pseudo_quantize_is_fused(x, 0 if fmt == "nvfp4" else 1, cfg.scale_rule.cuda_id, cfg.round_style.native_id, False)
    r = fos.quantize(x, fos.QuantizationConfig(pseudo_quantize=True, **kw))
    e = fos.dequantize(fos.quantize(x, cfg), dtype=x.dtype)
    assert r.dtype == dtype and r.shape == x.shape
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))


@pytest.mark.parametrize("rule", ["static_6", "static_4", "mse", "mae", "abs_max"])
@pytest.mark.parametrize("style", ["stochastic", "stochastic_unbiased"])
@pytest.mark.parametrize(("shape", "scale"), [((256, 512), 1.0), ((200, 208), 1.0), ((128, 1024), 2.0**-30), ((2048, 2048), 1.0)])
def test_fused_round_trip_of_the_stochastic_styles_on_tiles(rule, style, shape, scale):
    """... and with 16x16 tiles (the unbiased style's MAE and abs-max rules take the two-step path)."""
    from fouroversix_amd.quantize import ops

    x = (make_input("outlier", shape, 23).float() * scale).bfloat16()
    x[0, :16] = -x[0, :16].abs()
    x[1, 3] = -0.0
    x[16:32] = 0
    x = x.cuda()
    kw = dict(scale_rule=rule, round_style=style, block_scale_2d=True, kwargs={"seed": 78, "offset": 1})
    cfg = fos.QuantizationConfig(**kw)
    fused = ops.pseudo_quantize_is_fused(x, 0, cfg.scale_rule.cuda_id, cfg.round_style.native_id, True)
    assert fused == (style == "stochastic" or rule in ("static_6", "static_4", "mse"))
    r = fos.quantize(x, fos.QuantizationConfig(pseudo_quantize=True, **kw))
    e = fos.dequantize(fos.quantize(x, cfg), dtype=x.dtype)
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))


@pytest.mark.parametrize(("fmt", "rule", "style", "dtype"), [_FUSED_ROUND_TRIPS[2], _FUSED_ROUND_TRIPS[7], _FUSED_ROUND_TRIPS[-1]])
def test_fused_round_trip_of_the_other_formats_and_styles_full_size(fmt, rule, style, dtype):
    x = make_input("randn", (8192, 8192), 5).to(dtype).cuda()
    kw = dict(dtype=fmt, scale_rule=rule, round_style=style, kwargs={"seed": 9})
    r = fos.quantize(x, fos.QuantizationConfig(pseudo_quantize=True, **kw))
    e = fos.dequantize(fos.quantize(x, fos.QuantizationConfig(**kw)), dtype=x.dtype)
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))


def test_pseudo_quantize_full_size():
    """North-star shape: the fused kernel against the two-step path, and idempotence (a
    dequantised tensor re-quantises to itself with the same tensor maximum)."""
    x = make_input("randn", (8192, 8192), 1).cuda()
    cfg = fos.QuantizationConfig(scale_rule="mse", pseudo_quantize=True)
    r = fos.quantize(x, cfg)
    e = fos.dequantize(fos.quantize(x, fos.QuantizationConfig(scale_rule="mse")), dtype=x.dtype)
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))
    # 16x16 tiles: a few hundred of the 262144 take the undecided-tile path under the fused epilogue
    r = fos.quantize(x, fos.QuantizationConfig(scale_rule="mse", block_scale_2d=True, pseudo_quantize=True))
    e = fos.dequantize(fos.quantize(x, fos.QuantizationConfig(scale_rule="mse", block_scale_2d=True)), dtype=x.dtype)
    assert torch.equal(r.view(torch.int16), e.view(torch.int16))
    del e
    s6 = fos.QuantizationConfig(scale_rule="static_6", pseudo_quantize=True)
    once = fos.quantize(x, s6)
    # by value: a -0.0 (a negative input that rounded to zero) re-quantizes to +0.0
    assert torch.equal(fos.quantize(once, s6), once)


# ---- transpose / random Hadamard transform ------------------------------------------------

def test_transform_options_match_reference_vectors(golden_dir):
    """config.transpose / config.rht against the vectors the reference function wrote
    (quantize/pytorch/reference.py:567-571): codes, scales and amax, bit for bit."""
    d = np.load(os.path.join(golden_dir, "transform.npz"))
    n = 0
    for key in d.files:
        if not key.endswith(".values"):
            continue
        base = key[: -len(".values")]
        name, t, hh, rule, dim = base.split(".")
        x = torch.from_numpy(d[f"{name}.x"].view(np.int16).copy()).view(torch.bfloat16).cuda()
        q = fos.quantize(x, fos.QuantizationConfig(scale_rule=rule, block_scale_2d=(dim == "2d"),
                                                   transpose=(t == "t1"), rht=(hh == "h1")))
        assert tuple(q.original_shape) == (tuple(x.shape)[::-1] if t == "t1" else tuple(x.shape))
        assert np.array_equal(u8(q.values), d[base + ".values"]), base
        assert np.array_equal(u8(q.scale_factors).reshape(-1), d[base + ".sf"].reshape(-1)), base
        assert float(q.amax) == float(d[base + ".amax"][0]), base
        n += 1
    assert n == 27


@pytest.mark.parametrize(("transpose", "rht"), [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize(("kind", "shape"), [("randn", (1024, 2048)), ("outlier", (272, 144)), ("tiny_blocks", (48, 400)),
                                             ("zeros", (64, 64))])
def test_transform_matches_oracle(oracle, kind, shape, transpose, rht):
    """fos_transform (through ops.transform) and the quantization that follows it, against
    the oracle's restatement, on shapes that are not multiples of (128, 64) or of the
    64 x 64 transposition tile."""
    from fouroversix_amd.quantize import ops

    x = make_input(kind, shape, 21)
    y, amax = ops.transform(x.cuda(), transpose, rht)
    ref_y = oracle.transform(bits16(x), transpose=transpose, rht=rht)
    assert np.array_equal(bits16(y), ref_y)
    assert float(amax) == float(np.abs(oracle.bf16_bits_to_f32(ref_y)).max())
    for rule, two_d in (("mse", False), ("static_6", True)):
        q = hip_quantize(x, scale_rule=rule, block_scale_2d=two_d, transpose=transpose, rht=rht)
        ref = oracle.quantize(x, scale_rule=rule, block_scale_2d=two_d, transpose=transpose, rht=rht)
        assert_same_quantization(q, ref, f"{kind} t={transpose} h={rht} {rule}")


def test_transform_properties_full_size():
    """8192 x 8192: the RHT matrix is orthonormal up to bf16 rounding (energy preserved to
    1e-3), transposing twice is the identity, and unsupported shapes are refused."""
    from fouroversix_amd.quantize import ops

    x = make_input("randn", (8192, 8192), 2).cuda()
    y, amax = ops.transform(x, False, True)
    assert abs(float(y.float().pow(2).sum() / x.float().pow(2).sum()) - 1.0) < 1e-3
    assert float(amax) == float(y.abs().max())
    t, amax_t = ops.transform(x, True, False)
    assert torch.equal(t, x.T) and float(amax_t) == float(x.abs().max())
    tt, _ = ops.transform(t, True, False)
    assert torch.equal(tt, x)
    th, _ = ops.transform(x, True, True)
    assert torch.equal(th, ops.transform(t, False, True)[0])


@pytest.mark.parametrize("name", ["16x80", "48x112", "200x72"])
@pytest.mark.parametrize("rule,two_d", [("mse", False), ("static_6", True)])
def test_ragged_transpose_matches_the_reference(golden_dir, name, rule, two_d):
    """Shapes the reference's own backend gets through with transpose=True although neither side
    is a multiple of its block sizes (vectors written by tests/golden/make_golden.py
    --only-ragged-transpose): same codes, scales, amax and shapes."""
    g = np.load(os.path.join(golden_dir, "ragged_transpose.npz"))
    key = f"{name}.{rule}.{'2d' if two_d else '1d'}"
    assert int(g[f"{key}.raised"][0]) == 0
    x = torch.from_numpy(g[f"{name}.x"].view(np.int16)).view(torch.bfloat16).cuda()
    q = fos.quantize(x, fos.QuantizationConfig(scale_rule=rule, block_scale_2d=two_d, transpose=True))
    assert tuple(q.original_shape) == tuple(int(v) for v in g[f"{key}.shape"])
    assert tuple(q.padded_shape) == tuple(int(v) for v in g[f"{key}.padded"])
    assert float(q.amax) == float(g[f"{key}.amax"][0])
    assert np.array_equal(u8(q.values), g[f"{key}.values"])
    assert np.array_equal(u8(q.scale_factors).reshape(-1), g[f"{key}.sf"].reshape(-1))


@pytest.mark.parametrize("shape", [(16, 64), (80, 144), (100, 80), (37, 50), (130, 200), (1000, 72)])
@pytest.mark.parametrize("transpose,rht", [(True, False), (False, True), (True, True)])
def test_ragged_transform_matches_oracle(oracle, shape, transpose, rht):
    """Shapes that are not multiples of 16 (several of which the reference's backend refuses when
    transposing): the result is that of quantizing the transposed, zero-completed tensor."""
    x = make_input("randn", shape, 11)
    for rule, two_d in (("mse", False), ("static_6", True)):
        q = hip_quantize(x, scale_rule=rule, block_scale_2d=two_d, transpose=transpose, rht=rht)
        ref = oracle.quantize(bits16(x), scale_rule=rule, block_scale_2d=two_d, transpose=transpose, rht=rht)
        assert tuple(q.original_shape) == ((shape[1], shape[0]) if transpose else shape)
        assert_same_quantization(q, ref, f"{shape} {rule} transpose={transpose} rht={rht}")


def test_fp16_transform_matches_reference_vectors_and_oracle(oracle, golden_dir):
    """transpose / rht on fp16 tensors: the reference's vectors, then larger and ragged shapes
    against the oracle."""
    d = np.load(os.path.join(golden_dir, "transform_fp16.npz"))
    n = 0
    for key in d.files:
        if not key.endswith(".values"):
            continue
        base = key[: -len(".values")]
        name, t, hh, rule, dim = base.split(".")
        x = torch.from_numpy(d[f"{name}.x"].view(np.float16).copy()).cuda()
        q = fos.quantize(x, fos.QuantizationConfig(scale_rule=rule, block_scale_2d=(dim == "2d"), transpose=(t == "t1"), rht=(hh == "h1")))
        assert np.array_equal(u8(q.values), d[base + ".values"]), base
        assert np.array_equal(u8(q.scale_factors).reshape(-1), d[base + ".sf"].reshape(-1)), base
        assert float(q.amax) == float(d[base + ".amax"][0]), base
        n += 1
    assert n == 12
    g = torch.Generator("cpu").manual_seed(9)
    for shape in ((1024, 2048), (100, 200), (37, 50)):
        x = (torch.randn(*shape, generator=g) * 3).half()
        for transpose, rht in ((True, False), (False, True), (True, True)):
            q = hip_quantize(x, transpose=transpose, rht=rht)
            ref = oracle.quantize(x, transpose=transpose, rht=rht)
            assert_same_quantization(q, ref, f"fp16 {shape} transpose={transpose} rht={rht}")


@pytest.mark.parametrize(("shape", "dtype"), [((512, 1024), torch.bfloat16), ((100, 200), torch.bfloat16), ((256, 384), torch.float16),
                                              ((130, 272), torch.float32)])
@pytest.mark.parametrize(("transpose", "rht"), [(True, False), (False, True), (True, True)])
def test_transform_and_quantize_in_one_call_equals_the_two_calls(shape, dtype, transpose, rht):
    """fos_transform_quantize (the frontend's path for the transpose / rht options) leaves out the kernel that
    reduces the transform's partial maxima; its bytes are those of transform, then quantize with that maximum."""
    from fouroversix_amd import _native as nat
    from fouroversix_amd.quantize import ops

    x = (make_input("outlier", shape, 41).float() * 1.37).to(dtype).cuda()
    for fmt, rule, style, two_d in ((0, 3, 0, False), (0, 0, 1, False), (1, 3, 0, False)) + (((0, 3, 0, True),) if shape[0] % 16 == 0 else ()):
        y, amax = ops.transform(x, transpose, rht)
        layout = nat.SF_LINEAR if fmt == 1 else nat.SF_TILED
        want = ops.quantize_ex(y, fmt, rule, style, two_d, 5, 2, layout, amax)
        got = ops.transform_quantize(x, transpose, rht, fmt, rule, style, two_d, 5, 2, layout)
        for g, w, name in zip(got, want, ("values", "scales", "amax")):
            assert torch.equal(g.view(torch.uint8), w.view(torch.uint8)), f"{name} fmt {fmt} rule {rule} style {style} 2d {two_d}"


def test_transform_reads_unaligned_rows():
    """x whose rows start at odd element offsets takes the element-wise loads."""
    from fouroversix_amd.quantize import ops

    base = make_input("randn", (256, 264), 5).cuda()
    x = base[:, 3:259]
    t, amax = ops.transform(x, True, False)
    assert torch.equal(t, x.T) and float(amax) == float(x.abs().max())
    h, _ = ops.transform(x, False, True)
    assert torch.equal(h, ops.transform(x.contiguous(), False, True)[0])
