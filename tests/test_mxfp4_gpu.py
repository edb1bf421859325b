"""MXFP4 (E2M1 codes, E8M0 scale per 1x32 block) on the GPU: quantize, dequantize and the
GEMM on the scaled FP4 matrix instruction, against the reference's vectors and the oracle's
numpy restatement.  Quantize / dequantize are bit-exact; the GEMM is held to the budget the
reference gives its own backends (tests/test_matmul.py:15,81-88)."""

import os

import numpy as np
import pytest
import torch

import fouroversix_amd as fos
from gpu_utils import bits16, make_input, u8

pytestmark = pytest.mark.gpu

MISMATCH_BUDGET = 1e-3
MAX_REL = 1e-2


def mx_config(rule="static_6", **kw):
    return fos.QuantizationConfig(dtype="mxfp4", scale_rule=rule, **kw)


def from_bits(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_mxfp4_matches_reference_vectors(golden_dir):
    d = np.load(os.path.join(golden_dir, "mxfp4.npz"))
    n = 0
    for key in d.files:
        if not key.endswith(".values"):
            continue
        base = key[: -len(".values")]
        name, rule = base.split(".")
        x = from_bits(d[f"{name}.x"]).cuda()
        q = fos.quantize(x, mx_config(rule))
        assert tuple(q.padded_shape) == tuple(d[base + ".padded"]), base
        assert q.scale_factors.dtype == torch.float8_e8m0fnu and q.scale_factors_are_in_blackwell_layout
        assert np.array_equal(u8(q.values), d[base + ".values"]), base
        assert np.array_equal(u8(q.scale_factors).reshape(-1), d[base + ".sf"].reshape(-1)), base
        assert float(q.amax) == 1.0
        assert np.array_equal(bits16(fos.dequantize(q)), d[base + ".deq_bf16"]), base
        assert np.array_equal(fos.dequantize(q, torch.float32).cpu().numpy(), d[base + ".deq_f32"]), base
        n += 1
    assert n == 10
    for tag in ("256x128x256", "100x72x160"):
        rule = str(d[f"mm.{tag}.rule"])
        a, b = from_bits(d[f"mm.{tag}.a"]).cuda(), from_bits(d[f"mm.{tag}.b"]).cuda()
        out = fos.quantized_matmul(a, b, input_config=mx_config(rule), other_config=mx_config(rule))
        ref = d[f"mm.{tag}.out"]
        assert out.shape == ref.shape
        assert float((bits16(out) != ref).mean()) <= MISMATCH_BUDGET, tag


@pytest.mark.parametrize("rule", ["static_6", "static_4"])
@pytest.mark.parametrize(("kind", "shape", "scale"), [
    ("randn", (1024, 2048), 1.0), ("outlier", (300, 200), 1.0), ("tiny_blocks", (130, 528), 1.0),
    ("zeros", (128, 128), 1.0), ("randn", (64, 96), 2.0 ** -120), ("randn", (256, 640), 2.0 ** 100),
])
def test_mxfp4_quantize_dequantize_match_oracle(oracle, kind, shape, scale, rule):
    """Shapes that are not multiples of (128, 128) or of the 128 x 512 workgroup tile,
    unaligned row pitch, sub-normal and huge magnitudes (fp16 intermediate under/overflow in
    dequantize follows the reference)."""
    x = (make_input(kind, shape, 5).float() * scale).bfloat16()
    x[0, :3] = -x[0, :3].abs()
    x[1, 1] = -0.0
    ref = oracle.quantize_mxfp4(x, scale_rule=rule)
    for xin in (x.cuda(), torch.nn.functional.pad(x, (0, 3)).cuda()[:, : shape[1]]):  # second: ld % 8 != 0
        q = fos.quantize(xin, mx_config(rule))
        assert tuple(q.padded_shape) == tuple(ref.padded_shape)
        assert np.array_equal(u8(q.values), ref.values)
        assert np.array_equal(u8(q.scale_factors).reshape(-1), ref.scale_factors)
    rdeq = oracle.dequantize_mxfp4(ref.values, ref.scale_rows, ref.original_shape)
    got = fos.dequantize(q, torch.float32).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), rdeq.view(np.uint32))
    assert np.array_equal(bits16(fos.dequantize(q)), oracle.f32_to_bf16_bits(rdeq))
    assert np.array_equal(fos.dequantize(q, torch.float16).cpu().numpy().view(np.uint16), rdeq.astype(np.float16).view(np.uint16))


def test_mxfp4_streaming_kernel_full_size_and_layouts(oracle, monkeypatch):
    """Aligned inputs run on the streaming kernel: bit-exact with the oracle at 8192 x 4096 and on a strided
    view, identical to the tile kernel, and its row-major scale output (C ABI) is the tiled one re-ordered."""
    from fouroversix_amd import _native as nat

    x = make_input("outlier", (8192, 4096), 77)
    ref = oracle.quantize_mxfp4(x, scale_rule="static_6")
    q = fos.quantize(x.cuda(), mx_config())
    assert np.array_equal(u8(q.values), ref.values) and np.array_equal(u8(q.scale_factors).reshape(-1), ref.scale_factors)
    monkeypatch.setenv("FOS_MX_QUANT", "1")  # the tile kernel
    q_tile = fos.quantize(x.cuda(), mx_config())
    monkeypatch.delenv("FOS_MX_QUANT")
    assert torch.equal(q_tile.values, q.values) and torch.equal(q_tile.scale_factors.view(torch.uint8), q.scale_factors.view(torch.uint8))
    wide = make_input("randn", (384, 2048), 78).cuda()
    view = wide[:, 512:1536]
    rv = oracle.quantize_mxfp4(view.cpu().contiguous(), scale_rule="static_4")
    qv = fos.quantize(view, mx_config("static_4"))
    assert np.array_equal(u8(qv.values), rv.values) and np.array_equal(u8(qv.scale_factors).reshape(-1), rv.scale_factors)
    # row-major scales through the C ABI (ragged rows, half a 256-column tile at the end)
    L = nat.lib()
    rows, cols = 200, 640
    xs = make_input("randn", (rows, cols), 79).cuda()
    rows_p, cols_p = 256, 640
    outs = {}
    for layout in (nat.SF_TILED, nat.SF_LINEAR):
        codes = torch.zeros(rows_p, cols_p // 2, dtype=torch.uint8, device="cuda")
        sf = torch.zeros(rows_p * cols_p // 32, dtype=torch.uint8, device="cuda")
        amax = torch.zeros(1, dtype=torch.float32, device="cuda")
        ws = torch.empty(L.fos_quantize_workspace_bytes(rows, cols), dtype=torch.uint8, device="cuda")
        nat.check(L.fos_quantize(xs.data_ptr(), nat.T_BF16, rows, cols, cols, 2, 0, 0, 0, 0, 0, layout, codes.data_ptr(), sf.data_ptr(),
                                 amax.data_ptr(), 0, ws.data_ptr(), ws.numel(), nat.current_stream(xs.device)), "quantize")
        torch.cuda.synchronize()
        outs[layout] = (codes.cpu().numpy(), sf.cpu().numpy())
    assert np.array_equal(outs[nat.SF_TILED][0], outs[nat.SF_LINEAR][0])
    assert np.array_equal(oracle.from_blocked(outs[nat.SF_TILED][1], rows_p, cols_p // 32).reshape(-1), outs[nat.SF_LINEAR][1])


def test_mxfp4_fp32_and_fp16_inputs(oracle, golden_dir):
    """fp32 and fp16 inputs (the reference converts with `.float()`): the reference's vectors, and the oracle
    on aligned (streaming kernel for fp16), ragged and strided inputs."""
    d = np.load(os.path.join(golden_dir, "mxfp4_input_dtypes.npz"))
    keys = sorted(k[: -len(".values")] for k in d.files if k.endswith(".values"))
    assert len(keys) == 12
    for base in keys:
        name, tname, rule = base.split(".")
        raw = d[f"{name}.{tname}.x"]
        x = torch.from_numpy(raw.copy()) if tname == "f32" else torch.from_numpy(raw.view(np.int16).copy()).view(torch.float16)
        q = fos.quantize(x.cuda(), mx_config(rule))
        assert tuple(q.padded_shape) == tuple(d[base + ".padded"]), base
        assert np.array_equal(u8(q.values), d[base + ".values"]), base
        assert np.array_equal(u8(q.scale_factors).reshape(-1), d[base + ".sf"].reshape(-1)), base
        assert float(q.amax) == 1.0
    g = torch.Generator("cpu").manual_seed(9)
    for dt in (torch.float16, torch.float32):
        for shape in ((1024, 2048), (130, 528), (300, 200), (64, 96)):
            x = (torch.randn(*shape, generator=g) * 2.5).to(dt)
            x[0, :4] = torch.tensor([6e-8, -6e-8, 65504.0, -0.0]).to(dt)
            ref = oracle.quantize_mxfp4(x, scale_rule="static_6")
            for xin in (x.cuda(), torch.nn.functional.pad(x, (0, 3)).cuda()[:, : shape[1]]):  # second: odd row pitch
                q = fos.quantize(xin, mx_config())
                assert np.array_equal(u8(q.values), ref.values), (dt, shape)
                assert np.array_equal(u8(q.scale_factors).reshape(-1), ref.scale_factors), (dt, shape)


def test_mxfp4_unsupported_configurations():
    x = make_input("randn", (128, 128), 1).cuda()
    for bad in (dict(scale_rule="mse"), dict(scale_rule="static_6", block_scale_2d=True),
                dict(scale_rule="static_6", round_style="stochastic")):
        with pytest.raises(ValueError, match="No backend found"):
            fos.quantize(x, fos.QuantizationConfig(dtype="mxfp4", **bad))


@pytest.mark.parametrize(("m", "n", "k"), [(128, 128, 128), (256, 384, 640), (512, 256, 1152), (100, 72, 80),
                                           (4096, 4096, 1024), (8192, 8192, 8192)])
@pytest.mark.parametrize("out_dtype", ["bfloat16", "float16"])
def test_mxfp4_gemm(oracle, m, n, k, out_dtype):
    """Both tile shapes, odd numbers of 128-wide K steps, ragged shapes through the frontend;
    192 sampled rows of each operand are multiplied by the oracle in fp64."""
    if out_dtype == "float16" and m > 1024:
        pytest.skip("fp16 output covered by the smaller shapes")
    a, b = make_input("randn", (m, k), 5), make_input("randn", (n, k), 6)
    qa, qb = fos.quantize(a.cuda(), mx_config()), fos.quantize(b.cuda(), mx_config("static_4"))
    out = fos.quantized_matmul(qa, qb, out_dtype=out_dtype)
    assert out.shape == (m, n) and out.dtype == getattr(torch, out_dtype)
    g = torch.Generator("cpu").manual_seed(7)
    rows = torch.randperm(m, generator=g)[: min(m, 192)].sort().values
    cols = torch.randperm(n, generator=g)[: min(n, 192)].sort().values
    va, vb = u8(qa.values), u8(qb.values)
    kp = va.shape[1] * 2
    sa = oracle.from_blocked(u8(qa.scale_factors).reshape(-1), va.shape[0], kp // 32)
    sb = oracle.from_blocked(u8(qb.scale_factors).reshape(-1), vb.shape[0], kp // 32)
    _, ref32 = oracle.gemm_mxfp4(va[rows.numpy()], sa[rows.numpy()], vb[cols.numpy()], sb[cols.numpy()])
    got = out[rows.cuda()][:, cols.cuda()].float().cpu().numpy()
    expect = torch.from_numpy(ref32).to(getattr(torch, out_dtype)).float().numpy()
    frac = float((got != expect).mean())
    rel = float(np.abs(got - expect).max() / max(np.abs(expect).max(), 1e-30))
    assert frac <= MISMATCH_BUDGET and rel <= MAX_REL, f"{frac:.2e} of outputs differ, max rel {rel:.2e}"


@pytest.mark.parametrize("k", [128, 256, 384, 1152, 4224])
def test_mxfp4_gemm_kernels_agree_bitwise(monkeypatch, k):
    """The big-tile kernel that loads operands straight into LDS (four stages), the
    register-staged big-tile kernel and the small-tile kernel contract K in the same order
    with the same matrix instruction: whole outputs are bit-identical.  K covers fewer steps
    than stages, a partial last round of stages, and many rounds."""
    m = n = 4096
    qa = fos.quantize(make_input("randn", (m, k), 21).cuda(), mx_config())
    qb = fos.quantize(make_input("outlier", (n, k), 22).cuda(), mx_config("static_4"))
    outs = []
    for tile in (None, "256", "128"):
        if tile is None:
            monkeypatch.delenv("FOS_MX_TILE", raising=False)
        else:
            monkeypatch.setenv("FOS_MX_TILE", tile)
        outs.append(fos.quantized_matmul(qa, qb))
        torch.cuda.synchronize()
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
