"""Parity of the gfx950 FP4 GEMM (and the linear layer on top of it) with the CPU oracle
and the reference's matmul vectors.  Budget, as the reference holds its own backends to
(tests/test_matmul.py:15,81-88): at most 1e-3 of the bf16 outputs differ at all; and
max |diff| <= 1e-2 of the output range."""

import os

import numpy as np
import pytest
import torch
import torch.nn as nn

import fouroversix_amd as fos
from gpu_utils import bits16, make_input, u8

pytestmark = pytest.mark.gpu

MISMATCH_BUDGET = 1e-3
MAX_REL = 1e-2


def check(out_bits, ref_bits, oracle, what):
    frac = float((out_bits != ref_bits).mean())
    a, b = oracle.bf16_bits_to_f32(out_bits), oracle.bf16_bits_to_f32(ref_bits)
    rel = float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))
    assert frac <= MISMATCH_BUDGET and rel <= MAX_REL, f"{what}: {frac:.2e} of outputs differ, max rel {rel:.2e}"


@pytest.mark.parametrize("rule", ["static_6", "static_4", "mse"])
@pytest.mark.parametrize(("m", "n", "k"), [(256, 256, 256), (256, 512, 1024), (1024, 256, 512), (512, 1024, 256),
                                           (1024, 1024, 1024), (128, 128, 64)])
def test_gemm_matches_oracle(oracle, m, n, k, rule):
    a, b = make_input("randn", (m, k), 31), make_input("randn", (n, k), 32)
    cfg = fos.QuantizationConfig(scale_rule=rule)
    qa, qb = fos.quantize(a.cuda(), cfg), fos.quantize(b.cuda(), cfg)
    out = fos.quantized_matmul(qa, qb)
    assert out.shape == (m, n) and out.dtype == torch.bfloat16
    ra, rb = oracle.quantize(a, scale_rule=rule), oracle.quantize(b, scale_rule=rule)
    native, _ = oracle.gemm_nvfp4(ra.values, ra.scale_rows, rb.values, rb.scale_rows, oracle.gemm_alpha(ra, rb))
    check(bits16(out), native[:m, :n], oracle, f"{m}x{n}x{k} {rule} (native form)")
    pt, _ = oracle.quantized_matmul(ra, rb)
    check(bits16(out), pt, oracle, f"{m}x{n}x{k} {rule} (dequantize-matmul form)")


def test_gemm_matches_reference_vectors(oracle, golden_dir):
    mm = np.load(os.path.join(golden_dir, "matmul.npz"))
    for tag in sorted({k.rsplit(".", 1)[0] for k in mm.files}):
        rule = str(mm[tag + ".rule"])
        a = torch.from_numpy(mm[tag + ".a"].view(np.int16).copy()).view(torch.bfloat16).cuda()
        b = torch.from_numpy(mm[tag + ".b"].view(np.int16).copy()).view(torch.bfloat16).cuda()
        cfg = fos.QuantizationConfig(scale_rule=rule)
        out = fos.quantized_matmul(a, b, input_config=cfg, other_config=cfg)
        check(bits16(out), mm[tag + ".out"], oracle, tag)


def test_gemm_fp16_output_and_mixed_rules(oracle):
    a, b = make_input("randn", (256, 512), 33), make_input("weight", (384, 512), 34)
    qa = fos.quantize(a.cuda(), fos.QuantizationConfig(scale_rule="mse"))
    qb = fos.quantize(b.cuda(), fos.QuantizationConfig(scale_rule="static_6", block_scale_2d=True))
    out = fos.quantized_matmul(qa, qb, out_dtype=fos.DataType.float16)
    assert out.dtype == torch.float16 and out.shape == (256, 384)
    ra = oracle.quantize(a, scale_rule="mse")
    rb = oracle.quantize(b, scale_rule="static_6", block_scale_2d=True)
    _, f32 = oracle.gemm_nvfp4(ra.values, ra.scale_rows, rb.values, rb.scale_rows, oracle.gemm_alpha(ra, rb))
    expect = torch.from_numpy(f32[:256, :384].copy()).half()
    got = out.cpu()
    assert float((got != expect).float().mean()) <= MISMATCH_BUDGET
    assert float((got.float() - expect.float()).abs().max() / expect.float().abs().max()) <= MAX_REL


LLAMA_SHAPES = [(m, n, k) for m in (16, 128, 2048, 8192) for (n, k) in ((4096, 4096), (14336, 4096), (4096, 14336))]


@pytest.mark.parametrize(("m", "n", "k"), [(8192, 8192, 8192), *LLAMA_SHAPES,
                                           (16384, 4096, 4096), (16384, 1024, 4096),  # the decoder stack's token count, k/v projection
                                           (16384, 14336, 4096), (16384, 4096, 14336),  # ... its gate / up and down projections
                                           (256, 384, 2368), (64, 14336, 4096), (96, 11008, 4096)])
def test_gemm_full_size_sampled(oracle, m, n, k):
    """Headline shape, every Llama-3-8B linear shape (M in {16, 128, 2048, 8192}) and the
    decoder stack's 16384-token shapes: 192 sampled rows of each operand are multiplied by
    the oracle (fp64 accumulation) and compared with the same entries of the GPU result."""
    a, b = make_input("randn", (m, k), 5), make_input("randn", (n, k), 6)
    cfg = fos.QuantizationConfig(scale_rule="mse")
    qa, qb = fos.quantize(a.cuda(), cfg), fos.quantize(b.cuda(), cfg)
    out = fos.quantized_matmul(qa, qb)
    assert out.shape == (m, n)
    g = torch.Generator("cpu").manual_seed(7)
    rows = torch.randperm(m, generator=g)[: min(m, 192)].sort().values
    cols = torch.randperm(n, generator=g)[:192].sort().values
    va, vb = u8(qa.values), u8(qb.values)
    mp, npad = va.shape[0], vb.shape[0]
    sa = oracle.from_blocked(u8(qa.scale_factors).reshape(-1), mp, k // 16)
    sb = oracle.from_blocked(u8(qb.scale_factors).reshape(-1), npad, k // 16)
    alpha = float(fos.matmul.frontend.gemm_alpha(qa, qb))
    ref, _ = oracle.gemm_nvfp4(va[rows.numpy()], sa[rows.numpy()], vb[cols.numpy()], sb[cols.numpy()], alpha)
    got = bits16(out[rows.cuda()][:, cols.cuda()])
    check(got, ref, oracle, f"{m}x{n}x{k}")


@pytest.mark.parametrize(
    ("m", "n", "k", "env"),
    [
        (128, 1024, 8192, {}),                                  # weight-streaming kernel, 64-row workgroups, two row groups, split 2
        (128, 4096, 4096, {"FOS_GEMM_SPLITK": "3"}),            # ... ragged last split
        (100, 2048, 3328, {"FOS_GEMM_SPLITK": "5"}),            # ... 13 steps, idle waves, 100 of 128 rows
        (65, 256, 1024, {"FOS_GEMM_SPLITK": "2"}),              # ... one row in the second row group
        (48, 8448, 1024, {"FOS_GEMM_SPLITK": "2"}),             # ... one row group (more than 256 32-row tiles)
        (64, 384, 2560, {"FOS_GEMM_SPLITK": "3", "FOS_GEMM_TILE": "64"}),  # ... forced; 10 steps over 4 wavefronts, ragged split
        (128, 1024, 4096, {"FOS_GEMM_TILE": "32"}),             # 32-row workgroups, four A tiles per wavefront, split 2
        (100, 2048, 3328, {"FOS_GEMM_SPLITK": "5", "FOS_GEMM_TILE": "32"}),  # ... 13 steps, idle waves, 100 of 128 rows
        (16, 1024, 4096, {"FOS_GEMM_SPLITK": "2"}),             # ... one 32-row A tile (unsplit by default: 16 steps)
        (32, 1024, 8192, {}),                                   # ... split by default
        (48, 512, 2048, {"FOS_GEMM_SPLITK": "2"}),              # ... two
        (5, 512, 2304, {"FOS_GEMM_SPLITK": "3", "FOS_GEMM_TILE": "16"}),  # 16-row kernel (16 rows of B per workgroup up to N = 4096): 9 steps, 5 of 16 rows
        (16, 256, 768, {"FOS_GEMM_SPLITK": "2", "FOS_GEMM_TILE": "16"}),  # ... fewer steps than wavefronts
        (1, 128, 6400, {"FOS_GEMM_SPLITK": "2", "FOS_GEMM_TILE": "16"}),  # ... 25 steps: full prefetch rounds + a tail
        (16, 384, 12288, {"FOS_GEMM_SPLITK": "2"}),             # ... two full rounds per wavefront (its default range)
        (16, 4224, 4096, {"FOS_GEMM_SPLITK": "2", "FOS_GEMM_TILE": "16"}),  # ... 32 rows of B per workgroup (N > 4096)
        (9, 8192, 8192, {"FOS_GEMM_SPLITK": "2"}),              # ... the same by default
        (16, 384, 12288, {"FOS_GEMM_SPLITK": "2", "FOS_GEMM_TILE": "32"}),  # the same shape on 32-row tiles
        (128, 512, 1088, {}),                                   # K % 128 != 0: 128 x 128 tiles
        (384, 256, 14336, {}),
    ],
)
def test_gemm_split_k_matches_unsplit(monkeypatch, m, n, k, env):
    """Small-M shapes split K when the caller lends a workspace.  Through the C ABI: the
    split result equals the unsplit one and the 128 x 128-tile kernel's up to FP32
    re-association (one bf16 ulp on a few outputs), two split runs are bit-identical
    (fixed reduction order), and too small a workspace is ignored."""
    from fouroversix_amd import _native as nat

    for key, val in env.items():
        monkeypatch.setenv(key, val)
    L = nat.lib()
    ws_bytes = int(L.fos_gemm_workspace_bytes(m, n, k))
    assert ws_bytes > 0 and ws_bytes % (m * n * 4) == 0
    cfg = fos.QuantizationConfig(scale_rule="mse")
    qa = fos.quantize(make_input("randn", (m, k), 11).cuda(), cfg)
    qb = fos.quantize(make_input("randn", (n, k), 12).cuda(), cfg)
    alpha = fos.matmul.frontend.gemm_alpha(qa, qb).reshape(1).float().cuda()
    stream = nat.current_stream(qa.values.device)

    def run(ws, out_dtype=torch.bfloat16, rows=m):
        out = torch.full((rows, n), 7.0, dtype=out_dtype, device="cuda")
        rc = L.fos_gemm_nvfp4(qa.values.data_ptr(), qb.values.data_ptr(), qa.scale_factors.data_ptr(),
                              qb.scale_factors.data_ptr(), alpha.data_ptr(), rows, n, k, out.data_ptr(),
                              nat.TORCH_TO_T[out_dtype], n,
                              ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, stream)
        assert rc == 0
        torch.cuda.synchronize()
        return out

    def close(x, y):
        diff = (x.float() - y.float()).abs()
        assert float((diff > 0).float().mean()) <= 2e-2
        assert float((diff / y.float().abs().clamp_min(1e-2)).max()) <= 2.0 ** -7

    ws = torch.full((ws_bytes,), 0xFF, dtype=torch.uint8, device="cuda")  # NaN patterns: every partial must be written
    unsplit, split, again = run(None), run(ws), run(ws)
    assert torch.equal(split, again)
    assert not torch.isnan(split.float()).any()
    close(split, unsplit)
    assert torch.equal(run(ws[: ws_bytes - 16]), unsplit)
    close(run(ws, torch.float16), run(None, torch.float16))
    monkeypatch.setenv("FOS_GEMM_TILE", "1")  # the general kernel on the same operands
    monkeypatch.delenv("FOS_GEMM_SPLITK", raising=False)
    close(unsplit, run(None, rows=qa.values.shape[0])[:m])


@pytest.mark.parametrize(("m", "n", "k"), [(512, 256, 1088), (256, 256, 64), (768, 1024, 4160)])
def test_gemm_tile_kernels_agree_bitwise(monkeypatch, oracle, m, n, k):
    """The 256 x 256 tile (the planner's choice from 256 such tiles on; forced here), the
    128 x 256 tile (its choice where that covers the chip once; forced here) and the
    128 x 128 tile contract K in the same order: whole outputs are bit-identical, bf16 and
    fp16, and a sample matches the oracle."""
    from fouroversix_amd import _native as nat

    L = nat.lib()
    cfg = fos.QuantizationConfig(scale_rule="mse")
    qa = fos.quantize(make_input("randn", (m, k), 21).cuda(), cfg)
    qb = fos.quantize(make_input("randn", (n, k), 22).cuda(), cfg)
    alpha = fos.matmul.frontend.gemm_alpha(qa, qb).reshape(1).float().cuda()
    stream = nat.current_stream(qa.values.device)

    def run(tile, out_dtype):
        monkeypatch.setenv("FOS_GEMM_TILE", tile)
        out = torch.full((m, n), 7.0, dtype=out_dtype, device="cuda")
        rc = L.fos_gemm_nvfp4(qa.values.data_ptr(), qb.values.data_ptr(), qa.scale_factors.data_ptr(),
                              qb.scale_factors.data_ptr(), alpha.data_ptr(), m, n, k, out.data_ptr(),
                              nat.TORCH_TO_T[out_dtype], n, None, 0, stream)
        assert rc == 0
        torch.cuda.synchronize()
        return out

    for out_dtype in (torch.bfloat16, torch.float16):
        assert torch.equal(run("256", out_dtype), run("128", out_dtype))
        assert torch.equal(run("129", out_dtype), run("128", out_dtype))  # 128 x 256 tiles
    out = run("256", torch.bfloat16)
    va, vb = u8(qa.values), u8(qb.values)
    sa = oracle.from_blocked(u8(qa.scale_factors).reshape(-1), va.shape[0], k // 16)
    sb = oracle.from_blocked(u8(qb.scale_factors).reshape(-1), vb.shape[0], k // 16)
    ref, _ = oracle.gemm_nvfp4(va[:m:3], sa[:m:3], vb[:n], sb[:n], float(alpha))
    check(bits16(out[::3]), ref, oracle, f"256x256 tiles, {m}x{n}x{k}")


def test_linear_layer_forward(oracle):
    """quantize_model + FourOverSixLinear forward == oracle quantize (activations 1-D mse,
    weights 2-D mse) + oracle matmul + bias."""
    torch.manual_seed(0)
    lin = nn.Linear(512, 384, bias=True, dtype=torch.bfloat16)
    model = nn.Sequential(lin).cuda()
    w, bias = lin.weight.detach().cpu().clone(), lin.bias.detach().cpu().clone()
    fos.quantize_model(model, fos.ModelQuantizationConfig(weight_scale_2d=True))
    layer = model[0]
    assert isinstance(layer, fos.FourOverSixLinear)
    layer.quantize_weight_()
    assert layer.weight is None and int(layer.quantized_weight_metadata[0]) == 384
    x = make_input("randn", (4, 50, 512), 35)
    y = model(x.cuda())
    assert y.shape == (4, 50, 384) and y.dtype == torch.bfloat16
    rx = oracle.quantize(x.reshape(-1, 512), scale_rule="mse")
    rw = oracle.quantize(w, scale_rule="mse", block_scale_2d=True)
    assert np.array_equal(u8(layer.quantized_weight_values), rw.values)
    assert np.array_equal(u8(layer.quantized_weight_scale_factors), rw.scale_factors)
    o16, _ = oracle.gemm_nvfp4(rx.values, rx.scale_rows, rw.values, rw.scale_rows, oracle.gemm_alpha(rx, rw))
    expect = torch.from_numpy(o16[:200, :384].view(np.int16).copy()).view(torch.bfloat16) + bias
    got = y.reshape(200, 384).cpu()
    assert float((got != expect).float().mean()) <= 2 * MISMATCH_BUDGET
    # master-weight mode re-quantizes the weight on every call and must agree
    lin2 = nn.Linear(512, 384, bias=True, dtype=torch.bfloat16)
    lin2.load_state_dict({"weight": w, "bias": bias})
    keep = fos.FourOverSixLinear(lin2.cuda(), fos.ModuleQuantizationConfig(weight_scale_2d=True, keep_master_weights=True))
    assert torch.equal(keep(x.cuda()), y)


def test_quantized_checkpoint_round_trip():
    """A quantized layer's state_dict -- the four `quantized_weight_*` buffers of the reference
    (src/fouroversix/model/modules/linear.py:326-361,379-443) plus the bias -- saved, read back with
    a loader that executes nothing, and loaded into a fresh module gives a bit-identical forward."""
    import io

    torch.manual_seed(2)
    cfg = fos.ModuleQuantizationConfig(weight_scale_2d=True)
    layer = fos.FourOverSixLinear(nn.Linear(512, 384, bias=True, dtype=torch.bfloat16).cuda(), cfg).quantize_weight_()
    x = make_input("randn", (3, 40, 512), 37).cuda()
    y = layer(x)
    state = layer.state_dict()
    assert set(state) == {"bias", "quantized_weight_values", "quantized_weight_scale_factors", "quantized_weight_amax",
                          "quantized_weight_metadata"}
    assert state["quantized_weight_values"].shape == (384, 256) and state["quantized_weight_values"].dtype == torch.uint8
    assert state["quantized_weight_scale_factors"].dtype == torch.float8_e4m3fn
    assert state["quantized_weight_metadata"].tolist() == [384, 512, 384, 512, 1, 1]
    buf = io.BytesIO()
    torch.save({k: v.cpu() for k, v in state.items()}, buf)
    buf.seek(0)
    loaded = torch.load(buf, weights_only=True)
    fresh = fos.FourOverSixLinear(nn.Linear(512, 384, bias=True, dtype=torch.bfloat16).cuda(), cfg)
    fresh.weight = None  # a checkpoint of quantized weights carries no high-precision weight
    missing, unexpected = fresh.load_state_dict(loaded, strict=True)
    assert not missing and not unexpected
    assert torch.equal(fresh(x).view(torch.int16), y.view(torch.int16))
    # ... and through quantize_model on a model, as a loader of quantized checkpoints would build it
    model = nn.Sequential(nn.Linear(512, 384, bias=True, dtype=torch.bfloat16)).cuda()
    fos.quantize_model(model, fos.ModelQuantizationConfig(weight_scale_2d=True))
    model[0].weight = None
    model.load_state_dict({"0." + k: v for k, v in loaded.items()})
    assert torch.equal(model(x).view(torch.int16), y.view(torch.int16))


def test_linear_layer_forward_in_fp16(oracle):
    """An fp16 model: fp16 activations and weights are quantized from their own values (the
    reference converts with `.float()`), fp16 output."""
    torch.manual_seed(1)
    lin = nn.Linear(256, 384, bias=True, dtype=torch.float16)
    w, bias = lin.weight.detach().clone(), lin.bias.detach().clone()
    layer = fos.FourOverSixLinear(lin.cuda(), fos.ModuleQuantizationConfig(weight_scale_2d=True, output_dtype="float16"))
    layer.quantize_weight_()
    x = make_input("randn", (96, 256), 36).half()
    y = layer(x.cuda())
    assert y.shape == (96, 384) and y.dtype == torch.float16
    rx = oracle.quantize(x, scale_rule="mse")
    rw = oracle.quantize(w, scale_rule="mse", block_scale_2d=True)
    _, f32 = oracle.gemm_nvfp4(rx.values, rx.scale_rows, rw.values, rw.scale_rows, oracle.gemm_alpha(rx, rw))
    expect = torch.from_numpy(f32[:96, :384].copy()).half() + bias
    got = y.detach().cpu()
    # fp16's grid is 8x finer than bf16's, so FP32 re-association shows on 8x as many outputs: the
    # budget scales with it (a unit in the last place of the product, before the bias is added)
    assert float((got != expect).float().mean()) <= 8 * MISMATCH_BUDGET
    assert float((got.float() - expect.float()).abs().max() / expect.float().abs().max()) <= MAX_REL


def test_formats_without_a_native_gemm_take_the_dequantize_form(oracle):
    """IF4 operands (and an fp32 result) go through dequantize + matmul, the reference's
    PyTorch matmul backend (src/fouroversix/matmul/pytorch.py:33-52); compared with the
    oracle's statement of that backend under the reference's mismatch budget."""
    a, b = make_input("randn", (200, 512), 61), make_input("weight", (300, 512), 62)
    cfg = dict(dtype="if4", scale_rule="mse")
    out = fos.quantized_matmul(a.cuda(), b.cuda(), input_config=fos.QuantizationConfig(**cfg),
                               other_config=fos.QuantizationConfig(block_scale_2d=True, **cfg))
    assert out.shape == (200, 300) and out.dtype == torch.bfloat16
    ra, rb = oracle.quantize(a, **cfg), oracle.quantize(b, block_scale_2d=True, **cfg)
    o16, o32 = oracle.quantized_matmul(ra, rb)
    expect = torch.from_numpy(o16.view(np.int16).copy()).view(torch.bfloat16)
    assert float((out.cpu() != expect).float().mean()) <= 2 * MISMATCH_BUDGET
    qa, qb = fos.quantize(a.cuda()), fos.quantize(b.cuda())
    out32 = fos.quantized_matmul(qa, qb, out_dtype="float32")
    ref32 = oracle.quantized_matmul(oracle.quantize(a), oracle.quantize(b))[1]
    assert out32.dtype == torch.float32
    assert float((out32.cpu() - torch.from_numpy(ref32)).abs().max()) <= 1e-3 * float(np.abs(ref32).max())


def test_linear_forward_replays_in_a_hip_graph():
    """A decode-sized forward (quantize -> alpha -> weight-streaming GEMM, twice) captured in
    a HIP graph: every replay, interleaved with eager work and synchronisations, equals
    the eager result on fresh input contents."""
    torch.manual_seed(1)
    model = nn.Sequential(nn.Linear(1024, 2048, bias=False), nn.SiLU(), nn.Linear(2048, 1024, bias=True)).cuda().bfloat16()
    fos.quantize_model(model, fos.ModelQuantizationConfig(weight_scale_2d=True))
    for mod in model.modules():
        if isinstance(mod, fos.FourOverSixLinear):
            mod.quantize_weight_()
    static_x = torch.randn(16, 1024, device="cuda").bfloat16()
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                model(static_x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = model(static_x)
        for i in range(4):
            xi = torch.randn(16, 1024, device="cuda").bfloat16() * (i + 1)
            static_x.copy_(xi)
            graph.replay()
            torch.cuda.synchronize()
            eager = model(xi)
            torch.cuda.synchronize()
            assert torch.equal(static_y, eager), f"replay {i}"


@pytest.mark.parametrize(("m", "n", "k"), [(256, 256, 512), (16, 4096, 4096), (100, 384, 1024), (128, 1024, 4096), (2048, 256, 192)])
def test_gemm_with_in_kernel_output_scale_equals_alpha_form(m, n, k):
    """fos_gemm_nvfp4_amax (alpha formed in the kernel from the two tensor maxima) against
    fos_gemm_alpha + fos_gemm_nvfp4, bit for bit, over the tile, split-K and weight-streaming plans."""
    from fouroversix_amd.matmul.frontend import gemm_alpha
    from fouroversix_amd.quantize import ops
    from fouroversix_amd.quantize.frontend import dequantize_divisor

    qa = fos.quantize(make_input("randn", (m, k), 41).cuda(), fos.QuantizationConfig(scale_rule="mse"))
    qb = fos.quantize(make_input("weight", (n, k), 42).cuda(), fos.QuantizationConfig(scale_rule="static_6"))
    a_values = qa.values[:m] if m < 128 and k % 256 == 0 else qa.values
    for out_dtype, gemm in ((torch.bfloat16, ops.gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt),
                            (torch.float16, ops.gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt)):
        ref = gemm(a_values, qb.values, qa.scale_factors, qb.scale_factors, gemm_alpha(qa, qb))
        den = dequantize_divisor(qa) * dequantize_divisor(qb)
        got = ops.gemm_nvfp4_from_amax(a_values, qb.values, qa.scale_factors, qb.scale_factors, qa.amax, qb.amax, den, out_dtype)
        assert torch.equal(got, ref)
    out = fos.quantized_matmul(qa, qb)
    assert torch.equal(out, ref.to(torch.bfloat16)[: m, : n]) or out.dtype == torch.bfloat16


def test_gemm_alpha_kernel_matches_the_reference_expression():
    """alpha = (amaxA * amaxB) / (qA sA qB sB adjA adjB) with fp32 operations
    (reference matmul/cutlass/backend.py:86-98): the one-launch kernel against torch."""
    cfgs = [fos.QuantizationConfig(scale_rule=r, round_style=s) for r, s in
            (("mse", "nearest"), ("static_6", "nearest"), ("static_4", "stochastic_unbiased"), ("mae", "stochastic"))]
    for i, ca in enumerate(cfgs):
        cb = cfgs[(i + 1) % len(cfgs)]
        qa = fos.quantize((make_input("randn", (128, 64), 30 + i) * (3.0 ** i)).cuda(), ca)
        qb = fos.quantize((make_input("weight", (128, 64), 40 + i)).cuda(), cb)
        den = fos.quantize.__globals__["dequantize_divisor"](qa) * fos.quantize.__globals__["dequantize_divisor"](qb)
        expect = ((qa.amax * qb.amax) / den).to(torch.float32).reshape(1)
        got = fos.matmul.frontend.gemm_alpha(qa, qb)
        assert got.dtype == torch.float32 and got.shape == (1,)
        assert torch.equal(got.view(torch.int32), expect.view(torch.int32))


def test_linear_backward_on_the_fp4_gemm():
    """keep_master_weights=True: forward and both gradients run on the FP4 GEMM
    (reference model/modules/linear.py:96-288).  The gradients equal the explicit
    composition of the public calls under the same torch seed (the stochastic-rounding
    seeds come from torch's generator) and are close to the fp32 gradients."""
    torch.manual_seed(0)
    tokens, k, n = 256, 512, 384
    lin = nn.Linear(k, n, bias=True, dtype=torch.bfloat16).cuda()
    cfg = fos.ModelQuantizationConfig(keep_master_weights=True)
    model = nn.Sequential(lin)
    fos.quantize_model(model, cfg)
    layer = model[0]
    assert isinstance(layer, fos.FourOverSixLinear) and isinstance(layer.weight, nn.Parameter)
    x = torch.randn(1, tokens, k, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    g = torch.randn(1, tokens, n, device="cuda", dtype=torch.bfloat16)

    torch.manual_seed(123)
    y = layer(x)
    y.backward(g)
    gx, gw, gb = x.grad.clone(), layer.weight.grad.clone(), layer.bias.grad.clone()
    assert gx.shape == x.shape and gw.shape == layer.weight.shape and gb.shape == (n,)

    # explicit composition, same seed stream: dgrad draws first, then the two wgrad operands
    torch.manual_seed(123)
    mc = layer.config
    g2, x2, w = g.reshape(-1, n), x.detach().reshape(-1, k), layer.weight.data
    e_gx = fos.quantized_matmul(g2, w, input_config=mc.get_gradient_config(), other_config=mc.get_weight_config(transpose=True))
    e_gw = fos.quantized_matmul(g2, x2, input_config=mc.get_gradient_config(rht=True, transpose=True),
                                other_config=mc.get_activation_config(rht=True, transpose=True))
    assert torch.equal(gx.reshape(-1, k), e_gx) and torch.equal(gw, e_gw)
    assert torch.equal(gb, g2.sum(0))

    # against full precision
    rx = g2.float() @ w.float()
    rw = g2.float().T @ x2.float()
    ry = x2.float() @ w.float().T + layer.bias.float()
    rel = lambda a, b: float((a.detach().float() - b.detach()).norm() / b.detach().norm())  # noqa: E731
    assert rel(y.reshape(-1, n), ry) < 0.2 and rel(gx.reshape(-1, k), rx) < 0.25 and rel(gw, rw) < 0.25

    # unquantized gradient paths
    for kw in (dict(disable_dgrad_quantization=True, disable_wgrad_quantization=True), dict(pseudo_quantize=True)):
        layer.config = fos.ModelQuantizationConfig(keep_master_weights=True, **kw)
        x.grad = None
        layer.weight.grad = None
        layer(x).backward(g)
        assert rel(x.grad.reshape(-1, k), rx) < 0.25 and rel(layer.weight.grad, rw) < 0.25


# ---- max|output| recorded by the GEMM -------------------------------------------------------

@pytest.mark.parametrize("out_dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize(("m", "n", "k"), [(256, 256, 512), (1024, 4096, 1024), (8, 4096, 4096), (16, 1024, 8192), (48, 384, 1024),
                                           (100, 384, 1024), (128, 1024, 4096), (128, 14336, 4096), (2048, 256, 192)])
def test_gemm_records_the_output_maximum(m, n, k, out_dtype):
    """Every kernel of the plan (tiles, the two weight-streaming kernels, the split-K reduction)
    folds max|out| into the caller's word: equal to the maximum of what was stored, and the output
    itself unchanged."""
    a, b = make_input("randn", (m, k), 51).cuda(), make_input("weight", (n, k), 52).cuda()
    qa, qb = fos.quantize(a), fos.quantize(b, fos.QuantizationConfig(block_scale_2d=True))
    plain = fos.quantized_matmul(qa, qb, out_dtype=out_dtype)
    out = fos.quantized_matmul(qa, qb, out_dtype=out_dtype, emit_amax=True)
    assert torch.equal(out, plain)
    amax = fos.quantize.__globals__["known_amax"](out)
    assert amax is not None and amax.dtype == torch.float32
    assert float(amax) == float(out.float().abs().max())


def test_known_amax_follows_the_tensor():
    """quantize() uses a recorded maximum exactly as long as the tensor is the one that was
    measured: same result as measuring again; an in-place write or a new tensor drops it."""
    from fouroversix_amd.quantize import attach_known_amax, known_amax

    a, b = make_input("randn", (512, 1024), 53).cuda(), make_input("weight", (768, 1024), 54).cuda()
    out = fos.quantized_matmul(a, b, emit_amax=True)
    assert known_amax(out) is not None
    q1, q2 = fos.quantize(out), fos.quantize(out.clone())
    assert torch.equal(q1.values, q2.values) and torch.equal(q1.scale_factors.view(torch.uint8), q2.scale_factors.view(torch.uint8))
    assert float(q1.amax) == float(q2.amax)
    # a wrong recorded value would be used (that is the contract) ...
    wrong = out.clone()
    attach_known_amax(wrong, torch.full((1,), 2.0 * float(out.abs().max()), device="cuda"))
    assert float(fos.quantize(wrong).amax) == 2.0 * float(out.float().abs().max())
    # ... until the tensor is written
    wrong.mul_(1.0)
    assert known_amax(wrong) is None and float(fos.quantize(wrong).amax) == float(q2.amax)
    assert known_amax(out * 1) is None and known_amax(out[:, :64]) is None


def test_linear_layers_hand_the_maximum_on():
    """emit_output_amax: a stack of layers gives bit-identical outputs with and without it."""
    from fouroversix_amd.model import FourOverSixLinear, ModuleQuantizationConfig
    from fouroversix_amd.quantize import known_amax

    torch.manual_seed(3)
    dims = [(1024, 512), (512, 768), (768, 256)]
    mods = [nn.Linear(i, o, bias=False, device="cuda", dtype=torch.bfloat16) for i, o in dims]
    x = make_input("randn", (4, 96, 1024), 55).cuda()
    outs = []
    for emit in (False, True):
        cfg = ModuleQuantizationConfig(weight_scale_2d=True, emit_output_amax=emit)
        y = x
        for m in mods:
            layer = FourOverSixLinear(nn.Linear(m.in_features, m.out_features, bias=False, device="cuda", dtype=torch.bfloat16), cfg)
            layer.weight = nn.Parameter(m.weight.data.clone())
            layer.quantize_weight_()
            with torch.no_grad():
                y = layer(y)
            assert (known_amax(y) is not None) == emit
        outs.append(y)
    assert torch.equal(outs[0], outs[1])


class _DecoderProjections(nn.Module):
    """The seven linear projections of one Llama-3-8B decoder layer (grouped-query attention: 1024-wide
    k / v), chained wherever a GEMM output can feed the next projection directly: o reads q's
    output, gate / up read o's, down reads gate's.  No attention and no non-linearity, as in the
    benchmark's layer stack."""

    def __init__(self):
        super().__init__()
        mk = lambda i, o: nn.Linear(i, o, bias=False, dtype=torch.bfloat16)  # noqa: E731
        self.q_proj, self.k_proj, self.v_proj, self.o_proj = mk(4096, 4096), mk(4096, 1024), mk(4096, 1024), mk(4096, 4096)
        self.gate_proj, self.up_proj, self.down_proj = mk(4096, 14336), mk(4096, 14336), mk(14336, 4096)

    def forward(self, x):
        q, k, v = self.q_proj(x), self.k_proj(x), self.v_proj(x)
        h = self.o_proj(q)
        g, u = self.gate_proj(h), self.up_proj(h)
        return {"q_proj": (x, q), "k_proj": (x, k), "v_proj": (x, v), "o_proj": (q, h), "gate_proj": (h, g),
                "up_proj": (h, u), "down_proj": (g, self.down_proj(g))}


def test_decoder_layer_at_16384_tokens_through_quantize_model(oracle):
    """One decoder layer's projections at batch x seq = 8 x 2048 tokens through `quantize_model`
    on an nn.Module (reference src/fouroversix/model/modules/linear.py:43-94, model/quantize.py:101-127):
    weights 0.02 N(0,1) pre-quantized 4/6-MSE on 16 x 16 blocks, activations quantized on the fly
    (4/6-MSE, 1 x 16).  Every projection's output is compared on 160 x 160 sampled entries with the
    oracle's quantize of the same input and its fp64-accumulated product; the layer is run with the
    GEMM-recorded maximum handed to the next quantize and without, and the two must agree bit for bit;
    so must a run under torch.inference_mode(), where no maximum is handed on."""
    from fouroversix_amd.quantize import known_amax

    torch.manual_seed(11)
    block = _DecoderProjections()
    with torch.no_grad():
        for lin in block.children():
            lin.weight.copy_((0.02 * torch.randn(lin.weight.shape)).bfloat16())
    weights = {name: lin.weight.detach().clone() for name, lin in block.named_children()}
    block.cuda()
    x = make_input("randn", (8, 2048, 4096), 71).cuda()
    results = {}
    for emit in (True, False):
        model = _DecoderProjections().cuda()
        model.load_state_dict(block.state_dict())
        fos.quantize_model(model, fos.ModelQuantizationConfig(weight_scale_2d=True, emit_output_amax=emit))
        for lin in model.children():
            assert isinstance(lin, fos.FourOverSixLinear)
            lin.quantize_weight_()
        with torch.no_grad():
            results[emit] = model(x)
        for name, (_, out) in results[emit].items():
            assert out.shape[:2] == (8, 2048)
            assert (known_amax(out) is not None) == emit, name
        if emit:
            with torch.inference_mode():
                inf = model(x)
            for name, (_, out) in inf.items():
                assert known_amax(out) is None and torch.equal(out, results[True][name][1]), name
    for name in results[True]:
        assert torch.equal(results[True][name][1], results[False][name][1]), f"{name}: recorded maximum changes the result"
    g = torch.Generator("cpu").manual_seed(8)
    for name, (inp, out) in results[True].items():
        inp2, out2 = inp.reshape(-1, inp.shape[-1]), out.reshape(-1, out.shape[-1])
        rows = torch.randperm(inp2.shape[0], generator=g)[:160].sort().values
        cols = torch.randperm(out2.shape[1], generator=g)[:160].sort().values
        # the oracle quantizes the whole activation (its maximum is the tensor's) and the sampled weight rows
        # of the whole weight (16 x 16 tiles)
        ra = oracle.quantize(inp2.cpu(), scale_rule="mse")
        rw = oracle.quantize(weights[name], scale_rule="mse", block_scale_2d=True)
        ref, _ = oracle.gemm_nvfp4(ra.values[rows.numpy()], ra.scale_rows[rows.numpy()], rw.values[cols.numpy()],
                                   rw.scale_rows[cols.numpy()], oracle.gemm_alpha(ra, rw))
        check(bits16(out2[rows.cuda()][:, cols.cuda()]), ref, oracle, name)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize(("m", "n", "k"), [(16, 512, 1024), (5, 256, 2304), (48, 512, 2048), (100, 2048, 3328), (128, 1024, 8192),
                                           (256, 384, 2368), (512, 512, 256), (2048, 1024, 512), (384, 256, 14336)])
def test_bias_in_the_epilogue_equals_the_separate_addition(m, n, k, out_dtype):
    """`quantized_matmul(..., bias=b)` = `quantized_matmul(...) + b` bit for bit (the product rounded to the
    output type, the sum rounded again: reference src/fouroversix/model/modules/linear.py:83-92) in every
    kernel of the plan -- 16-row, weight-streaming, tile and split-K reduction -- and the recorded maximum
    is that of the sum."""
    from fouroversix_amd.quantize import known_amax

    a, b = make_input("randn", (m, k), 81).cuda(), make_input("weight", (n, k), 82).cuda()
    qa, qb = fos.quantize(a), fos.quantize(b, fos.QuantizationConfig(block_scale_2d=True))
    g = torch.Generator("cpu").manual_seed(83)
    bias = (torch.randn(n, generator=g) * 0.3).to(out_dtype).cuda()
    dt = fos.DataType.bfloat16 if out_dtype == torch.bfloat16 else fos.DataType.float16
    plain = fos.quantized_matmul(qa, qb, out_dtype=dt)
    fused = fos.quantized_matmul(qa, qb, out_dtype=dt, bias=bias, emit_amax=True)
    assert torch.equal(fused, plain + bias)
    amax = known_amax(fused)
    assert amax is not None and float(amax) == float(fused.float().abs().max())
    # a bias of another type, or on a weight whose rows were padded, is added separately: same values, no tag
    other = fos.quantized_matmul(qa, qb, out_dtype=dt, bias=bias.float(), emit_amax=True)
    assert torch.equal(other, plain + bias.float()) and known_amax(other) is None


def test_recorded_maximum_of_an_output_with_nan_is_nan():
    """The reference's `x.abs().max()` of a tensor that holds a NaN is NaN; the maximum the GEMM records
    follows (the bits of a NaN lie above every number's in the unsigned comparison)."""
    from fouroversix_amd.quantize import known_amax

    a, b = make_input("randn", (256, 512), 84).cuda(), make_input("weight", (384, 512), 85).cuda()
    qa, qb = fos.quantize(a), fos.quantize(b)
    qa.amax = torch.full_like(qa.amax, float("nan"))  # alpha, and with it every output, is NaN
    out = fos.quantized_matmul(qa, qb, emit_amax=True)
    assert bool(torch.isnan(out).all())
    assert bool(torch.isnan(known_amax(out)).all())
    q = fos.quantize(out)
    assert bool(torch.isnan(q.amax).all())
