"""Pins of the CPU oracle (oracle/fos_oracle.c) that do not need a GPU.

Each test checks the oracle against something it was not derived from: vectors written by
the reference itself, torch library routines, the reference's second statement of a
rule, or a closed form.
"""

import glob
import hashlib
import os

import numpy as np
import pytest
import torch

QUANT_FILES = sorted(
    f for f in glob.glob(os.path.join(os.path.dirname(__file__), "golden", "quantize_*.npz")) if "config1" not in f
)


def _keys(d):
    return sorted({k.rsplit(".", 1)[0] for k in d.files if k.endswith(".values")})


@pytest.mark.parametrize("path", QUANT_FILES, ids=[os.path.basename(p)[9:-4] for p in QUANT_FILES])
def test_quantize_matches_reference_vectors(oracle, path):
    """Bit-exact codes, scales (in the stored layout) and amax for every format / rule /
    1-D / 2-D combination, incl. ragged shapes and sub-normal block scales."""
    d = np.load(path)
    for k in _keys(d):
        dt, rule, dim = k.split(".")
        q = oracle.quantize(d["x"], dtype=dt, scale_rule=rule, block_scale_2d=(dim == "2d"))
        assert q.padded_shape == tuple(d[k + ".padded"]), k
        assert q.blocked == bool(d[k + ".blocked"][0]), k
        assert q.amax == d[k + ".amax"][0], k
        assert np.array_equal(q.values, d[k + ".values"]), k
        assert np.array_equal(q.scale_factors, d[k + ".sf"].reshape(-1)), k


def _typed_input(d, name, tname):
    x = d[f"{name}.{tname}.x"]
    return x if tname == "f32" else x.view(np.float16)


def test_quantize_of_fp32_and_fp16_inputs_matches_reference_vectors(oracle, golden_dir):
    """The reference converts any input with `.float()`: inputs with more significant bits than
    bf16 (fp32 randn, fp16 randn, ragged and outlier shapes) against its PyTorch backend's bytes."""
    d = np.load(os.path.join(golden_dir, "input_dtypes.npz"))
    keys = _keys(d)
    assert len(keys) >= 24
    for k in keys:
        name, tname, dt, rule, dim = k.split(".")
        q = oracle.quantize(_typed_input(d, name, tname), dtype=dt, scale_rule=rule, block_scale_2d=(dim == "2d"))
        assert q.amax == d[k + ".amax"][0], k
        assert np.array_equal(q.values, d[k + ".values"]), k
        assert np.array_equal(q.scale_factors, d[k + ".sf"].reshape(-1)), k


def test_quantize_input_type_does_not_matter_for_bf16_values(oracle):
    """bf16 values handed over as fp32 (and fp16 values as fp32) give the same bytes."""
    g = torch.Generator("cpu").manual_seed(71)
    x = torch.randn(128, 192, generator=g)
    for narrow in (x.bfloat16(), x.half()):
        for kw in (dict(scale_rule="mse"), dict(scale_rule="mae", block_scale_2d=True), dict(dtype="if4", scale_rule="mse"),
                   dict(scale_rule="static_6", round_style="stochastic", seed=5)):
            a, b = oracle.quantize(narrow, **kw), oracle.quantize(narrow.float(), **kw)
            assert a.amax == b.amax and np.array_equal(a.values, b.values) and np.array_equal(a.scale_factors, b.scale_factors), kw


def test_quantize_config1_digest(oracle, golden_dir):
    """1024x1024 randn seed 0, static_6 and mse: SHA-256 of codes and scales."""
    d = np.load(os.path.join(golden_dir, "quantize_config1_1024x1024.npz"))
    g = torch.Generator("cpu").manual_seed(0)
    x = torch.randn(1024, 1024, generator=g).bfloat16()
    xb = oracle.bf16_bits(x)
    if hashlib.sha256(xb.tobytes()).hexdigest() != str(d["x_sha"]):
        pytest.skip("torch.randn stream differs from the one the vectors were made with")
    for rule in ("static_6", "mse"):
        q = oracle.quantize(xb, scale_rule=rule)
        assert q.amax == d[f"{rule}.amax"][0]
        assert hashlib.sha256(q.values.tobytes()).hexdigest() == str(d[f"{rule}.values_sha"])
        assert hashlib.sha256(q.scale_factors.tobytes()).hexdigest() == str(d[f"{rule}.sf_sha"])


def test_transform_options_match_reference_vectors(oracle, golden_dir):
    """transpose / random-Hadamard options (reference quantize/pytorch/reference.py:567-571):
    vectors written by the reference function on CPU, all three combinations, 1-D and 2-D;
    the RHT matrix itself is pinned against the reference's bf16 matrix."""
    d = np.load(os.path.join(golden_dir, "transform.npz"))
    assert np.array_equal(oracle.f32_to_bf16_bits(oracle.rht_matrix()), d["had"])
    # symmetric up to the sign vector, orthonormal: H H^T = I
    h = oracle.rht_matrix()
    assert np.array_equal(h @ h.T, np.eye(16, dtype=np.float32))
    n = 0
    for key in d.files:
        if not key.endswith(".values"):
            continue
        name, t, hh, rule, dim = key[: -len(".values")].split(".")
        x = d[f"{name}.x"]
        q = oracle.quantize(x, scale_rule=rule, block_scale_2d=(dim == "2d"), transpose=(t == "t1"), rht=(hh == "h1"))
        base = key[: -len(".values")]
        assert np.array_equal(q.values, d[base + ".values"]), base
        assert np.array_equal(q.scale_factors, d[base + ".sf"].reshape(-1)), base
        assert q.amax == d[base + ".amax"][0], base
        n += 1
    assert n == 27


def test_fp16_transform_matches_reference_vectors(oracle, golden_dir):
    """transpose / random-Hadamard on fp16 tensors: the reference multiplies by the matrix cast to
    fp16 (quantize/pytorch/reference.py:570-571); vectors written by the reference function on CPU."""
    d = np.load(os.path.join(golden_dir, "transform_fp16.npz"))
    n = 0
    for key in d.files:
        if not key.endswith(".values"):
            continue
        base = key[: -len(".values")]
        name, t, hh, rule, dim = base.split(".")
        x = d[f"{name}.x"].view(np.float16)
        q = oracle.quantize(x, scale_rule=rule, block_scale_2d=(dim == "2d"), transpose=(t == "t1"), rht=(hh == "h1"))
        assert np.array_equal(q.values, d[base + ".values"]), base
        assert np.array_equal(q.scale_factors, d[base + ".sf"].reshape(-1)), base
        assert q.amax == d[base + ".amax"][0], base
        n += 1
    assert n == 12


def test_ragged_transpose_matches_reference_vectors(oracle, golden_dir):
    """transpose=True on shapes outside the block multiples: where the reference's backend gets
    through (its padding is sized from the transposed shape but applied before the transpose,
    src/fouroversix/quantize/pytorch/backend.py:57-79, which fits only some shapes) the result
    is that of transposing first and completing with zeros; the fixture also records the
    shapes on which it raised."""
    d = np.load(os.path.join(golden_dir, "ragged_transpose.npz"))
    ok = raised = 0
    for key in d.files:
        if not key.endswith(".raised"):
            continue
        base = key[: -len(".raised")]
        name, rule, dim = base.split(".")
        if int(d[key][0]):
            raised += 1
            continue
        q = oracle.quantize(d[f"{name}.x"], scale_rule=rule, block_scale_2d=(dim == "2d"), transpose=True)
        assert np.array_equal(q.values, d[base + ".values"]), base
        assert np.array_equal(q.scale_factors, d[base + ".sf"].reshape(-1)), base
        assert q.amax == d[base + ".amax"][0], base
        assert tuple(q.padded_shape) == tuple(d[base + ".padded"]) and tuple(q.original_shape) == tuple(d[base + ".shape"])
        ok += 1
    assert (ok, raised) == (6, 6)


def test_dequantize_matches_reference_vectors(oracle, golden_dir):
    for name in ("randn_256x128", "ragged_100x80", "tiny_blocks_128x128"):
        d = np.load(os.path.join(golden_dir, f"quantize_{name}.npz"))
        for k in sorted({k.rsplit(".", 1)[0] for k in d.files if k.endswith(".deq_bf16")}):
            dt, rule, _ = k.split(".")
            pad = tuple(d[k + ".padded"])
            sf = d[k + ".sf"].reshape(-1)
            rows = oracle.from_blocked(sf, pad[0], pad[1] // 16) if d[k + ".blocked"][0] else sf.reshape(pad[0], pad[1] // 16)
            out = oracle.dequantize(d[k + ".values"], rows, d[k + ".amax"][0], dtype=dt, scale_rule=rule,
                                    original_shape=tuple(d["shape"]))
            assert hashlib.sha256(np.ascontiguousarray(out).tobytes()).hexdigest() == str(d[k + ".deq_f32_sha"]), k
            bf = torch.from_numpy(out.copy()).bfloat16().view(torch.int16).numpy().view(np.uint16)
            assert np.array_equal(bf, d[k + ".deq_bf16"]), k


def test_matmul_within_reference_budget(oracle, golden_dir):
    """The reference allows <= 1e-3 of the bf16 outputs to differ between its own matmul
    backends (tests/test_matmul.py:15,81-88); the oracle is held to the same budget
    against the PyTorch backend's outputs, in both the dequantize-matmul form and the
    native alpha-in-epilogue form."""
    mm = np.load(os.path.join(golden_dir, "matmul.npz"))
    for tag in sorted({k.rsplit(".", 1)[0] for k in mm.files}):
        rule = str(mm[tag + ".rule"])
        qa = oracle.quantize(mm[tag + ".a"], scale_rule=rule)
        qb = oracle.quantize(mm[tag + ".b"], scale_rule=rule)
        ref = mm[tag + ".out"]
        o16, _ = oracle.quantized_matmul(qa, qb)
        assert (o16 != ref).mean() <= 1e-3, tag
        g16, _ = oracle.gemm_nvfp4(qa.values, qa.scale_rows, qb.values, qb.scale_rows, oracle.gemm_alpha(qa, qb))
        assert (g16[: ref.shape[0], : ref.shape[1]] != ref).mean() <= 1e-3, tag
        rel = np.abs(oracle.bf16_bits_to_f32(o16) - oracle.bf16_bits_to_f32(ref)).max() / np.abs(
            oracle.bf16_bits_to_f32(ref)).max()
        assert rel <= 1e-2


def test_e4m3_cast_equals_torch(oracle):
    """torch's own float32 -> float8_e4m3fn cast is the reference semantics
    (reference.py:225): every bf16-representable value plus dense samples around every
    rounding boundary."""
    L = oracle.lib()
    vals = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    grid = torch.tensor([L.fos_oracle_e4m3_to_f32(b) for b in range(0x7F)], dtype=torch.float64)
    mids = (grid[:-1] + grid[1:]) / 2
    near = torch.cat([mids * (1 + e) for e in (-1e-6, -6e-8, 0.0, 6e-8, 1e-6)]).float()
    extra = torch.tensor([0.0, 2.0**-10, 2.0**-10 * 1.0000001, 463.9, 464.0, 464.1, 479.9])
    allv = torch.cat([vals, near, extra])
    allv = allv[allv < 480]  # beyond that torch yields NaN patterns; the scale path cannot get there
    expect = allv.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([L.fos_oracle_e4m3_from_f32(float(v)) for v in allv.tolist()], dtype=np.uint8)
    assert np.array_equal(got, expect)
    # decode against torch's widening cast
    back = torch.arange(0, 0x7F, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(back, grid.float().numpy())


def test_e2m1_rounding_equals_threshold_table(oracle):
    """The reference states round-to-nearest a second time as thresholds
    (kernels/triton/fp4.py:21-41): <=.25 0, <.75 .5, <=1.25 1, <1.75 1.5, <=2.5 2,
    <3.5 3, <=5 4, else 6.  Brute force over every non-negative bf16 below 7."""
    L = oracle.lib()
    vals = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    vals = vals[vals < 7.0].tolist()

    def table(a):
        if a <= 0.25: return 0.0
        if a < 0.75: return 0.5
        if a <= 1.25: return 1.0
        if a < 1.75: return 1.5
        if a <= 2.5: return 2.0
        if a < 3.5: return 3.0
        if a <= 5.0: return 4.0
        return 6.0

    for a in vals:
        assert L.fos_oracle_e2m1_rtn(a) == table(a), a
        assert L.fos_oracle_e2m1_rtn(-a) == -table(a), a
    # the unclamped top regime: [7, 9) -> 8 (reference.py:38)
    assert L.fos_oracle_e2m1_rtn(7.0) == 8.0 and L.fos_oracle_e2m1_rtn(8.9) == 8.0
    # codes <-> values (kernels/triton/fp4.py:78-102)
    mags = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for c in range(16):
        assert L.fos_oracle_e2m1_decode(c) == (-1.0 if c & 8 else 1.0) * mags[c & 7]


def test_sum_order_equals_torch_sum(oracle):
    """The mse/mae decisions hinge on torch.sum(dim=-1)'s fp32 summation order over 16 and
    256 elements; the oracle's order must reproduce torch.sum on this host bit for bit."""
    L = oracle.lib()
    g = torch.Generator("cpu").manual_seed(5)
    for n, fn in ((16, L.fos_oracle_sum16), (256, L.fos_oracle_sum256)):
        v = (torch.randn(20000, n, generator=g) ** 2) * torch.logspace(-3, 3, 20000).unsqueeze(1)
        expect = v.sum(dim=-1).numpy()
        arr = np.ascontiguousarray(v.numpy())
        got = np.array([fn(arr[i].ctypes.data) for i in range(arr.shape[0])], dtype=np.float32)
        assert np.array_equal(got, expect), f"sum over {n} differs from torch.sum on this host"


def test_closed_forms(oracle):
    """Inputs of the reference's own tests (tests/test_quantize.py:155-164) whose outputs
    follow from the definition."""
    z = np.zeros((128, 64), dtype=np.uint16)
    for rule in ("static_6", "mse"):
        q = oracle.quantize(z, scale_rule=rule)
        assert q.amax == 0 and not q.values.any() and not q.scale_factors.any()
    ones = np.full((128, 64), 0x3F80, dtype=np.uint16)
    q = oracle.quantize(ones, scale_rule="static_6")
    assert q.amax == 1 and (q.values == 0x77).all() and (q.scale_factors == 0x7E).all()
    q = oracle.quantize(ones, scale_rule="static_4")
    assert (q.values == 0x66).all() and (q.scale_factors == 0x7E).all()
    q = oracle.quantize(ones, scale_rule="mse")  # both candidates exact, tie goes to "6"
    assert (q.values == 0x77).all() and (q.scale_factors == 0x78).all()
    # 2-D scaling: 16 equal scale bytes down every tile column, and W / W.T commute
    g = torch.Generator("cpu").manual_seed(3)
    w = (0.02 * torch.randn(128, 128, generator=g)).bfloat16()
    q = oracle.quantize(w, scale_rule="static_6", block_scale_2d=True)
    assert (q.scale_rows.reshape(8, 16, 8) == q.scale_rows.reshape(8, 16, 8)[:, :1]).all()
    qt = oracle.quantize(w.T.contiguous(), scale_rule="static_6", block_scale_2d=True)
    a = oracle.dequantize(q.values, q.scale_rows, q.amax, scale_rule="static_6")
    b = oracle.dequantize(qt.values, qt.scale_rows, qt.amax, scale_rule="static_6")
    assert np.array_equal(a, b.T)


def test_tiled_layout_round_trip_and_formula(oracle):
    """Offset formula (quantize/utils.py:88-96 restated in fp4_quant_kernel.h:447-454)
    against the reshape/transpose statement, via torch on a ragged-tile shape."""
    rows, cols = 256, 12
    a = np.arange(rows * cols, dtype=np.uint32).astype(np.uint8).reshape(rows, cols)
    t = torch.from_numpy(a)
    expect = (
        t.view(rows // 128, 128, cols // 4, 4).transpose(1, 2).reshape(-1, 4, 32, 4).transpose(1, 2).reshape(-1, 32, 16).flatten()
    ).numpy()
    got = oracle.to_blocked(a)
    assert np.array_equal(got, expect)
    assert np.array_equal(oracle.from_blocked(got, rows, cols), a)


def test_stochastic_rounding_known_answers(oracle):
    """The reference's SR known answers (tests/test_quantize.py:360-372): L2 distance of
    dequantize(quantize(randn 1024^2)) to the input within 5 % of 137 (static_6) / 122
    (mse), 158 / 139 for the unbiased variant; and the dither is unbiased in range."""
    g = torch.Generator("cpu").manual_seed(0)
    x = torch.randn(1024, 1024, generator=g).bfloat16()
    xf = x.float().numpy()
    for rule, style, expect in (("static_6", "stochastic", 137), ("mse", "stochastic", 122),
                                ("static_6", "stochastic_unbiased", 158), ("mse", "stochastic_unbiased", 139)):
        q = oracle.quantize(x, scale_rule=rule, round_style=style, seed=1234)
        deq = oracle.dequantize(q.values, q.scale_rows, q.amax, scale_rule=rule, round_style=style)
        deq = torch.from_numpy(deq).bfloat16().float().numpy()
        dist = float(np.sqrt(((deq - xf) ** 2).sum()))
        assert abs(dist - expect) / expect < 0.05, (rule, style, dist)
    q = oracle.quantize(x, scale_rule="static_6", round_style="stochastic", seed=7)
    deq = oracle.dequantize(q.values, q.scale_rows, q.amax, scale_rule="static_6", round_style="stochastic")
    assert abs(float((deq - xf).mean())) < 2e-3


def test_mxfp4_fp32_and_fp16_inputs_match_reference_vectors(oracle, golden_dir):
    """MXFP4 on inputs with more significant bits than bf16 (the reference converts with `.float()`)."""
    import torch

    d = np.load(os.path.join(golden_dir, "mxfp4_input_dtypes.npz"))
    keys = sorted(k[: -len(".values")] for k in d.files if k.endswith(".values"))
    assert len(keys) == 12
    for base in keys:
        name, tname, rule = base.split(".")
        raw = d[f"{name}.{tname}.x"]
        x = torch.from_numpy(raw.copy()) if tname == "f32" else torch.from_numpy(raw.view(np.int16).copy()).view(torch.float16)
        q = oracle.quantize_mxfp4(x, scale_rule=rule)
        assert tuple(q.padded_shape) == tuple(d[base + ".padded"]), base
        assert np.array_equal(q.values, d[base + ".values"]), base
        assert np.array_equal(q.scale_factors, d[base + ".sf"].reshape(-1)), base


def test_mxfp4_matches_reference_vectors(oracle, golden_dir):
    """MXFP4 quantize / dequantize / matmul restatement against vectors written by the
    reference's PyTorch backend (quantize/pytorch/reference.py:149-181, quantize/backend.py:89-160):
    codes, E8M0 scales in the 128x4-tile layout, amax == 1, padded shapes (cols to 128),
    dequantized values bit for bit; matmul within the reference's own budget."""
    d = np.load(os.path.join(golden_dir, "mxfp4.npz"))
    n = 0
    for key in d.files:
        if not key.endswith(".values"):
            continue
        base = key[: -len(".values")]
        name, rule = base.split(".")
        q = oracle.quantize_mxfp4(d[f"{name}.x"], scale_rule=rule)
        assert tuple(q.padded_shape) == tuple(d[base + ".padded"]), base
        assert np.array_equal(q.values, d[base + ".values"]), base
        assert np.array_equal(q.scale_factors, d[base + ".sf"].reshape(-1)), base
        assert q.amax == d[base + ".amax"][0] == 1.0
        deq = oracle.dequantize_mxfp4(q.values, q.scale_rows, q.original_shape)
        assert np.array_equal(deq, d[base + ".deq_f32"]), base
        assert np.array_equal(oracle.f32_to_bf16_bits(deq), d[base + ".deq_bf16"]), base
        n += 1
    assert n == 10
    for tag in ("256x128x256", "100x72x160"):
        rule = str(d[f"mm.{tag}.rule"])
        qa = oracle.quantize_mxfp4(d[f"mm.{tag}.a"], scale_rule=rule)
        qb = oracle.quantize_mxfp4(d[f"mm.{tag}.b"], scale_rule=rule)
        o16, _ = oracle.gemm_mxfp4(qa.values, qa.scale_rows, qb.values, qb.scale_rows)
        m, nn = qa.original_shape[0], qb.original_shape[0]
        ref = d[f"mm.{tag}.out"]
        got = o16[:m, :nn]
        assert float((got != ref).mean()) <= 1e-3


def test_dequantize_with_f32_intermediate_matches_reference_vectors(oracle, golden_dir):
    """dequantize(..., intermediate_dtype=float32) of the reference on IF4 (integer blocks carry
    6/7), MXFP4 (scales below fp16's range) and NVFP4 codes written by the reference itself."""
    z = np.load(os.path.join(golden_dir, "dequantize_f32_intermediate.npz"))
    keys = sorted({k.rsplit(".", 1)[0] for k in z.files})
    assert len(keys) == 16
    differs = 0
    for key in keys:
        _, dtype, rule = key.split(".")
        values, sf, shape, padded = z[key + ".values"], z[key + ".sf"], z[key + ".shape"], z[key + ".padded"]
        if dtype == "mxfp4":
            rows = oracle.from_blocked(sf, int(padded[0]), int(padded[1]) // 32)
            got = oracle.dequantize_mxfp4(values, rows, tuple(shape), f32_intermediate=True)
            other = oracle.dequantize_mxfp4(values, rows, tuple(shape))
        else:
            rows = oracle.from_blocked(sf, int(padded[0]), int(padded[1]) // 16) if int(z[key + ".blocked"][0]) else sf.reshape(int(padded[0]), -1)
            kw = dict(dtype=dtype, scale_rule=rule, original_shape=tuple(shape))
            got = oracle.dequantize(values, rows, float(z[key + ".amax"][0]), f32_intermediate=True, **kw)
            other = oracle.dequantize(values, rows, float(z[key + ".amax"][0]), **kw)
        assert np.array_equal(got.view(np.uint32), z[key + ".deq_f32"].view(np.uint32)), key
        assert np.array_equal(oracle.f32_to_bf16_bits(got), z[key + ".deq_bf16"]), key
        differs += int(not np.array_equal(got.view(np.uint32), other.view(np.uint32)))
    assert differs >= 4  # the option matters on the IF4 / out-of-range MXFP4 cases


def test_philox4x32_10_known_answers(oracle):
    """The three published Random123 known-answer vectors for Philox4x32 with 10 rounds
    (counter, key -> output): zeros, all ones, and the digits of pi."""
    L = oracle.lib()
    cases = (
        ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
        ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
        ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
         (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
    )
    for ctr, key, want in cases:
        c = np.array(ctr, dtype=np.uint32)
        k = np.array(key, dtype=np.uint32)
        out = np.zeros(4, dtype=np.uint32)
        L.fos_oracle_philox4x32_10(c.ctypes.data, k.ctypes.data, out.ctypes.data)
        assert tuple(int(v) for v in out) == want


def test_if4_stochastic_rounding_known_answers(oracle):
    """IF4 + MSE under the stochastic styles (the INT4 dither and the IF4 stochastic branch):
    the reference's known answers 110 / 122 (unbiased) +- 5 % on randn 1024^2
    (tests/test_quantize.py:321,360-372)."""
    g = torch.Generator("cpu").manual_seed(0)
    x = torch.randn(1024, 1024, generator=g).bfloat16()
    xf = x.float().numpy()
    for style, expect in (("stochastic", 110), ("stochastic_unbiased", 122)):
        for seed in (1234, 99):
            q = oracle.quantize(x, dtype="if4", scale_rule="mse", round_style=style, seed=seed)
            deq = oracle.dequantize(q.values, q.scale_rows, q.amax, dtype="if4", scale_rule="mse", round_style=style)
            deq = torch.from_numpy(deq).bfloat16().float().numpy()
            dist = float(np.sqrt(((deq - xf) ** 2).sum()))
            assert abs(dist - expect) / expect < 0.05, (style, seed, dist)
        # both kinds of block occur, so the integer branch's dither is exercised
        frac_int = float((q.scale_factors >= 128).mean())
        assert 0.05 < frac_int < 0.95


def _mac_tree_sum(lanes):
    stage = [np.float32(v) for v in lanes]
    while len(stage) > 1:
        nxt = [np.float32(stage[i] + stage[i + 1]) for i in range(0, len(stage) - 1, 2)]
        if len(stage) % 2:
            nxt.append(stage[-1])
        stage = nxt
    return stage[0]


@pytest.mark.parametrize("fmt", ["nvfp4", "if4"])
def test_decode_and_scale_against_mac_known_answers(oracle, golden_dir, fmt):
    """The reference's MAC test benches hold three dot products of K = 160 each for NVFP4 and
    IF4 operands with their expected fp32 bit patterns (if4_mac/tb/nvfp4_mac_golden_ref.svh:1119-1121,
    if4_mac/tb/if4_mac_golden_ref.svh; arithmetic of if4_mac/scripts/gen_golden_ref.py:164-209:
    fp16 product of the two decoded values times the fp32 product of the two decoded scales,
    one fp32 accumulator per lane, pairwise tree at the end).  Here the operands go through
    the oracle's dequantize (code decode, E4M3 decode, IF4 integer blocks with bit 7 of the
    scale byte) and the products are accumulated as the MAC does.  NVFP4 is bit-exact: value
    x scale is exact in both formulations.  An IF4 integer block carries 6/7 in the decoded
    value here and in the scale product there, so that file agrees to fp32 rounding only.
    The MAC reads the scale byte 0x7F as 448 (gen_golden_ref.py:76-79), the float8_e4m3fn
    cast never produces that byte: it is mapped to 0x7E before decoding."""
    d = np.load(os.path.join(golden_dir, "if4_mac.npz"))
    first, a, w = d[f"{fmt}.first"], d[f"{fmt}.a"], d[f"{fmt}.w"]
    a_sf, w_sf = d[f"{fmt}.a_sf"].copy(), d[f"{fmt}.w_sf"].copy()
    for sf in (a_sf, w_sf):
        sf[(sf & 0x7F) == 0x7F] -= 1
    n = first.size

    def dequant(codes, sf):
        # one 1x16 block per cycle: rows = cycles, 16 columns (packed low nibble first)
        packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
        div = 6.0 * 448.0
        return oracle.dequantize(packed, sf.reshape(n, 1), div, dtype=fmt, scale_rule="static_6", f32_intermediate=True)

    da, dw = dequant(a, a_sf), dequant(w, w_sf)
    # amax == divisor, so the tensor scale is exactly 1 (the products below 2^12 * 2688 are exact)
    got = []
    acc = np.zeros(16, dtype=np.float32)
    for i in range(n):
        if first[i] and i:
            got.append(_mac_tree_sum(acc))
            acc = np.zeros(16, dtype=np.float32)
        prod = (da[i].astype(np.float64) * dw[i].astype(np.float64)).astype(np.float32)
        acc = (acc + prod).astype(np.float32)
    got = np.array(got, dtype=np.float32)
    want = d[f"{fmt}.expected"].view(np.float32)
    assert got.size == 3
    if fmt == "nvfp4":
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (got, want)
    else:
        assert np.allclose(got, want, rtol=2e-6, atol=0.0), (got, want)
        assert int((d["if4.a_sf"] >= 128).sum()) > 5  # integer blocks are present


def test_near_tie_fixture_holds_near_ties(oracle, golden_dir):
    """tests/golden/near_ties.npz (written by make_near_ties.py): every stored block's two
    selection errors differ, by at most 2e-4 relative, and a good share of them by at most
    2e-6 -- the inputs on which an approximate decision would go wrong.  One case per rule,
    block shape, rounding style and origin of the tensor maximum that a kernel decides from a
    certified shortcut."""
    d = np.load(os.path.join(golden_dir, "near_ties.npz"))
    cases = sorted(k[:-2] for k in d.files if k.endswith(".x"))
    assert len(cases) == 18
    for case in cases:
        parts = case.split(".")
        dtype, two_d, rule, style, given = parts[0], parts[1] == "2d", parts[2], parts[3], len(parts) == 5
        x, amax, seed = d[case + ".x"], float(d[case + ".amax"][0]), int(d[case + ".seed"][0])
        e = oracle.selection_errors(x, dtype=dtype, scale_rule=rule, block_scale_2d=two_d, amax=amax if given else None,
                                    round_style=style, seed=seed)
        unit = 16 if two_d else 1
        ea, eb = e[::unit, :, 0].astype(np.float64).ravel()[1:], e[::unit, :, 1].astype(np.float64).ravel()[1:]
        live = np.maximum(ea, eb) > 0
        assert live.sum() >= 20, case
        rel = np.abs(ea - eb)[live] / np.maximum(ea, eb)[live]
        assert (rel > 0).all() and (rel <= 2e-4).all(), case
        # (abs-max errors are single residuals on a coarse grid: under a bf16 maximum they differ by a few units in
        # the last place or by much more, under a 24-bit maximum the closest pairs found lie 1e-4 apart)
        if rule != "abs_max":
            assert (rel <= 2e-6).sum() >= 4 and (rel <= 2e-6).mean() > 0.1, case
        if not given:
            assert float(oracle.bf16_bits_to_f32(x).max()) == amax == 8.0
