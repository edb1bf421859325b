"""Benchmark of the quantize + FP4-GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one synthetic batch already resident in HBM:
``quantize`` of an 8192 x 8192 bf16 tensor to NVFP4 with 4/6-MSE selection, round to
nearest, 1x16 blocks (tensor-max pass + quantize pass).  Inputs rotate over four buffers
(512 MiB) so that a step never finds its input in the 256 MB Infinity Cache left over from
the previous step.  ``value`` is algorithmic GB/s (2.5625 B per element: bf16 in, packed
nibbles + E4M3 scales out) of the whole step.  The same line carries the FP4 GEMM at
8192^3 (TFLOP/s, ``gemm``), the roofline of the dominant kernel of each, and the CPU
oracle timed on the host cores on a bounded sample.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
BYTES_PER_ELEM = 2.0 + 0.5 + 1.0 / 16.0


def make_activation(rows, cols, seed, outliers=False):
    import torch

    g = torch.Generator("cpu").manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    if outliers:
        n_out = max(1, cols // 100)
        idx = torch.randperm(cols, generator=g)[:n_out]
        z = torch.randn(4, rows, n_out, generator=g)
        x[:, idx] = 50 * z[0] / torch.sqrt((z[1] ** 2 + z[2] ** 2 + z[3] ** 2) / 3)
    return x.bfloat16()


def profiled_traffic(rows, cols):
    """HBM bytes per launch of the pass-2 kernel at this shape, as the committed rocprofv3 summary holds them
    (FETCH_SIZE and WRITE_SIZE, scaled by a copy kernel of known size): (bytes, source) or (None, None).
    The summary, not this script, is the evidence; a kernel change that moves the figure shows up there."""
    import re

    path = os.path.join(ROOT, "profiles", "quantize_nvfp4_mse_8192x8192.md")
    if (rows, cols) != (8192, 8192) or not os.path.exists(path):
        return None, None
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", open(path).read(), re.M)
    return (float(m.group(1)), "profiles/quantize_nvfp4_mse_8192x8192.md") if m else (None, None)


def event_ms(fn, steps):
    """Average milliseconds of ``fn`` per call, from HIP events on the current stream."""
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / steps


def linear_stack(dev, steps, warmup, layers=32, tokens=8 * 2048, hidden=4096, kv=1024, ffn=14336):
    """Per layer: on-the-fly activation quantize (4/6-MSE, 1x16) + FP4 GEMM for q/k/v/o and
    gate/up/down against random weights (N(0, 1 / in_features), which keeps the activations of this
    normalisation-free chain at unit scale) pre-quantized 4/6-MSE with 16x16 blocks.  No attention, no
    nonlinearity: the output of q feeds o, the output of o feeds gate / up, the output of gate
    feeds down.  The headline figure is an nn.Module of nn.Linear layers converted with
    ``quantize_model`` (every projection quantizes its own input, as the reference's linear layer
    does; a GEMM output that goes straight into the next projection brings its maximum along);
    beside it the same chain with ``emit_output_amax=False`` and as hand-written calls of
    ``quantized_matmul`` on the same weights."""
    import torch
    import torch.nn as nn

    import fouroversix_amd as fos

    acfg = fos.QuantizationConfig(scale_rule="mse")
    shapes = [("q", hidden, hidden), ("k", kv, hidden), ("v", kv, hidden), ("o", hidden, hidden),
              ("gate", ffn, hidden), ("up", ffn, hidden), ("down", hidden, ffn)]

    class Projections(nn.Module):
        def __init__(self):
            super().__init__()
            for name, n, k in shapes:
                setattr(self, name, nn.Linear(k, n, bias=False, device=dev, dtype=torch.bfloat16))

        def forward(self, x):
            q = self.q(x)
            self.k(x)
            self.v(x)
            h = self.o(q)
            gate = self.gate(h)
            self.up(h)
            return self.down(gate)

    g = torch.Generator(device=dev).manual_seed(7)
    model = nn.Sequential(*[Projections() for _ in range(layers)])
    with torch.no_grad():
        for lin in model.modules():
            if isinstance(lin, nn.Linear):
                # N(0, 1 / in_features): the chain has no normalisation layers, and with a fixed 0.02 its activations
                # would grow fivefold per layer, out of the range activations live in
                std = lin.in_features ** -0.5
                lin.weight.copy_((std * torch.randn(lin.weight.shape, generator=g, device=dev)).bfloat16())
    model_cfg = fos.ModelQuantizationConfig(weight_scale_2d=True, modules_to_not_convert=[])
    fos.quantize_model(model, model_cfg)
    for lin in model.modules():
        if isinstance(lin, fos.FourOverSixLinear):
            lin.quantize_weight_()
    torch.cuda.empty_cache()
    weights = [{name: getattr(layer, name).quantized_weight() for name, _, _ in shapes} for layer in model]
    x0 = torch.randn(tokens, hidden, generator=g, device=dev).bfloat16()

    def step_module():
        with torch.no_grad():
            return model(x0)

    def step_module_no_amax():
        model_cfg.emit_output_amax = False
        try:
            with torch.no_grad():
                return model(x0)
        finally:
            model_cfg.emit_output_amax = True

    def step():
        x = x0
        for layer in weights:
            q = fos.quantized_matmul(x, layer["q"], input_config=acfg)
            fos.quantized_matmul(x, layer["k"], input_config=acfg)
            fos.quantized_matmul(x, layer["v"], input_config=acfg)
            h = fos.quantized_matmul(q, layer["o"], input_config=acfg)
            gate = fos.quantized_matmul(h, layer["gate"], input_config=acfg)
            fos.quantized_matmul(h, layer["up"], input_config=acfg)
            x = fos.quantized_matmul(gate, layer["down"], input_config=acfg)
        return x

    def step_shared():
        # variant: projections that read the same tensor share one quantization of it
        x = x0
        for layer in weights:
            qx = fos.quantize(x, acfg)
            q = fos.quantized_matmul(qx, layer["q"])
            fos.quantized_matmul(qx, layer["k"])
            fos.quantized_matmul(qx, layer["v"])
            qh = fos.quantize(fos.quantized_matmul(q, layer["o"], input_config=acfg), acfg)
            gate = fos.quantized_matmul(qh, layer["gate"])
            fos.quantized_matmul(qh, layer["up"])
            x = fos.quantized_matmul(gate, layer["down"], input_config=acfg)
        return x

    def step_amax():
        # variant of step_shared: every GEMM records max|output|, so only x0 is reduced by a pass of its own
        x = x0
        for layer in weights:
            qx = fos.quantize(x, acfg)
            q = fos.quantized_matmul(qx, layer["q"], emit_amax=True)
            fos.quantized_matmul(qx, layer["k"])
            fos.quantized_matmul(qx, layer["v"])
            qh = fos.quantize(fos.quantized_matmul(q, layer["o"], input_config=acfg, emit_amax=True), acfg)
            gate = fos.quantized_matmul(qh, layer["gate"], emit_amax=True)
            fos.quantized_matmul(qh, layer["up"])
            x = fos.quantized_matmul(gate, layer["down"], input_config=acfg, emit_amax=True)
        return x

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    assert model_cfg.emit_output_amax, "the module path hands the GEMM-recorded maximum on by default"
    sec = timed(step_module)
    sec_module_no_amax = timed(step_module_no_amax)
    sec_raw = timed(step)
    sec_shared = timed(step_shared)
    sec_amax = timed(step_amax)
    flops = 2.0 * tokens * sum(n * k for _, n, k in shapes) * layers

    def fig(s):
        return {"ms_per_step": round(s * 1e3, 3), "tokens_per_s": round(tokens / s, 1)}

    return {
        "workload": f"{layers} layers x (q,k,v,o,gate,up,down) quantize+GEMM, {tokens} tokens, hidden {hidden}, "
                    f"kv {kv}, ffn {ffn}; nn.Module converted with quantize_model (default config + weight_scale_2d)",
        "ms_per_step": round(sec * 1e3, 3),
        "tokens_per_s": round(tokens / sec, 1),
        "TFLOP/s": round(flops / sec / 1e12, 1),
        "module_without_recorded_amax": fig(sec_module_no_amax),
        "raw_calls": fig(sec_raw),
        "shared_activation_quantize": fig(sec_shared),
        "shared_and_gemm_recorded_amax": fig(sec_amax),
    }


def c_abi_gemm(qa, qb, m: int, dev):
    """A closure that calls fos_gemm_nvfp4 on two quantized operands (first m rows of A)."""
    import torch

    import fouroversix_amd as fos
    from fouroversix_amd import _native as nat

    lib = nat.lib()
    n, k = qb.values.shape[0], qa.values.shape[1] * 2
    alpha = fos.matmul.frontend.gemm_alpha(qa, qb).reshape(1).float().to(dev)
    ws_bytes = int(lib.fos_gemm_workspace_bytes(m, n, k))
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    args = (qa.values.data_ptr(), qb.values.data_ptr(), qa.scale_factors.data_ptr(), qb.scale_factors.data_ptr(),
            alpha.data_ptr(), m, n, k, out.data_ptr(), nat.T_BF16, n, ws.data_ptr() if ws_bytes else None, ws_bytes,
            nat.current_stream(dev))
    keep = (alpha, ws, out)

    def call(_keep=keep):
        rc = lib.fos_gemm_nvfp4(*args)
        if rc != 0:
            raise RuntimeError(f"fos_gemm_nvfp4 returned {rc}")

    return call


def extras(dev, steps: int) -> dict:
    """Timings of the rows built around the headline path (whole calls through the public
    API, microseconds): small-M GEMMs, fused pseudo-quantize, dequantize, the transpose /
    random-Hadamard options, stochastic rounding and MXFP4."""
    import torch

    import fouroversix_amd as fos

    def us(fn):
        fn()  # warm-up
        return round(event_ms(fn, steps) * 1e3, 1)

    out = {}
    xs = [make_activation(8192, 8192, 200 + i).to(dev) for i in range(2)]
    n = [0]

    def nxt():
        n[0] += 1
        return xs[n[0] % 2]

    q = fos.quantize(xs[0], fos.QuantizationConfig(scale_rule="mse"))
    out["dequantize_8192x8192_us"] = us(lambda: fos.dequantize(q))
    del q
    for name, kw in (("pseudo_quantize_mse", dict(scale_rule="mse", pseudo_quantize=True)),
                     ("quantize_mse_2d", dict(scale_rule="mse", block_scale_2d=True)),
                     ("quantize_mse_rht", dict(scale_rule="mse", rht=True)),
                     ("quantize_mse_transpose_rht", dict(scale_rule="mse", rht=True, transpose=True)),
                     ("quantize_mse_stochastic", dict(scale_rule="mse", round_style="stochastic", kwargs={"seed": 1})),
                     ("quantize_mse_2d_stochastic", dict(scale_rule="mse", round_style="stochastic", block_scale_2d=True, kwargs={"seed": 1})),
                     ("pseudo_quantize_mse_stochastic", dict(scale_rule="mse", round_style="stochastic", pseudo_quantize=True, kwargs={"seed": 1})),
                     ("quantize_if4_mse", dict(dtype="if4", scale_rule="mse")),
                     ("pseudo_quantize_if4_mse", dict(dtype="if4", scale_rule="mse", pseudo_quantize=True)),
                     ("quantize_mxfp4_static_6", dict(dtype="mxfp4", scale_rule="static_6"))):
        cfg = fos.QuantizationConfig(**kw)
        out[f"{name}_8192x8192_us"] = us(lambda: fos.quantize(nxt(), cfg))
    xh = xs[0].half()
    cfg = fos.QuantizationConfig(scale_rule="mse", pseudo_quantize=True)
    out["pseudo_quantize_mse_fp16_8192x8192_us"] = us(lambda: fos.quantize(xh, cfg))
    del xs, xh
    mse = fos.QuantizationConfig(scale_rule="mse")
    for m, nn, k in ((16, 4096, 4096), (16, 14336, 4096), (16, 4096, 14336), (128, 4096, 4096), (128, 14336, 4096),
                     (128, 4096, 14336), (2048, 14336, 4096), (2048, 4096, 4096), (2048, 4096, 14336)):
        qa = fos.quantize(make_activation(m, k, 7).to(dev), mse)
        qb = fos.quantize(make_activation(nn, k, 8).to(dev), mse)
        out[f"gemm_nvfp4_{m}x{nn}x{k}_us"] = us(lambda: fos.quantized_matmul(qa, qb))
        if m <= 128:
            # the same GEMM through the C entry point alone (output and workspace allocated once):
            # at these sizes the Python frontend costs more than the kernels
            out[f"gemm_nvfp4_{m}x{nn}x{k}_c_abi_us"] = us(c_abi_gemm(qa, qb, m, dev))
    mx = fos.QuantizationConfig(dtype="mxfp4", scale_rule="static_6")
    qa = fos.quantize(make_activation(8192, 8192, 5).to(dev), mx)
    qb = fos.quantize(make_activation(8192, 8192, 6).to(dev), mx)
    fos.quantized_matmul(qa, qb)
    t = event_ms(lambda: fos.quantized_matmul(qa, qb), steps)
    out["gemm_mxfp4_8192x8192x8192"] = {"ms": round(t, 4), "TFLOP/s": round(2.0 * 8192 ** 3 / (t * 1e-3) / 1e12, 1),
                                        "frac_of_fp4_peak": round(2.0 * 8192 ** 3 / (t * 1e-3) / 1e12 / 10100.0, 4)}
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--rows", type=int, default=8192)
    ap.add_argument("--cols", type=int, default=8192)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-oracle baseline leg")
    ap.add_argument("--no-gemm", action="store_true")
    ap.add_argument("--no-activation", action="store_true", help="skip the 8192 x 4096 outlier-channel input (profiling runs)")
    ap.add_argument("--no-stack", action="store_true", help="skip the 32-layer quantized-linear stack")
    ap.add_argument("--no-extras", action="store_true", help="skip the timings of the surrounding operations")
    ap.add_argument("--settle-ms", type=float, default=40.0,
                    help="untimed whole steps run for this long before the timed legs (0 for counter-collection runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch

    import fouroversix_amd as fos
    from fouroversix_amd import _native as nat

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    L = nat.lib()
    rows, cols, K, W = args.rows, args.cols, args.steps, args.warmup
    elems = rows * cols
    algo_bytes = elems * BYTES_PER_ELEM

    # ---- inputs ------------------------------------------------------------------------
    n_buf = 4
    xs = [make_activation(rows, cols, 100 + i).to(dev) for i in range(n_buf)]
    # counter calibration for profiling runs: a plain elementwise kernel of known size
    # (reads and writes rows*cols*2 bytes) appears once in every rocprofv3 trace of this script
    calib = xs[0].view(torch.int16) + 1
    del calib
    cfg = fos.QuantizationConfig(scale_rule="mse")

    # ---- quantize: the whole step through the public API (the headline figure) --------
    def timed_steps():
        for i in range(W):
            fos.quantize(xs[i % n_buf], cfg)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            q = fos.quantize(xs[i % n_buf], cfg)
        torch.cuda.synchronize()
        del q
        return (time.perf_counter() - t0) * 1e3 / K

    # An idle MI355X runs its first ~25 ms of load below its sustained rate, whatever the load is: from
    # idle, whole steps take 57-61 us for ~100 steps and reach their steady 51-52 us after ~450.  W warm-up
    # steps and K timed ones straight from idle measure that ramp (reported as `cold_start`); the headline
    # figure is the same W + K steps after `--settle-ms` of the same steps, untimed.
    cold_ms = timed_steps()
    settle_steps = 0
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        for i in range(50):
            fos.quantize(xs[i % n_buf], cfg)
        torch.cuda.synchronize()
        settle_steps += 50
    step_ms = timed_steps()
    value = algo_bytes / (step_ms * 1e-3) / 1e9

    # ---- quantize: per-kernel durations from HIP events, straight through the C ABI --
    rows_p, cols_p = L.fos_padded_rows(rows), L.fos_padded_cols(cols)
    # (one set of outputs per input: a launch that overwrites what the previous one has just left dirty in
    # the 32 MiB of L2 never sends those lines to memory, which reads 2-3 us better than any real use)
    codes_sets = [torch.empty(rows_p, cols_p // 2, dtype=torch.uint8, device=dev) for _ in range(n_buf)]
    sf_sets = [torch.empty(rows_p * cols_p // 16, dtype=torch.uint8, device=dev) for _ in range(n_buf)]
    codes, sf = codes_sets[0], sf_sets[0]
    amax = torch.zeros(1, dtype=torch.float32, device=dev)
    ws_bytes = L.fos_quantize_workspace_bytes(rows, cols)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = nat.current_stream(dev)
    counter = [0]

    # Pass 2's average launch duration inside the step, from HIP events on the launch stream: K back-to-back
    # steps through the C ABI (one call = pass 1 + pass 2 of one input, inputs rotating, as in the
    # timed region above) minus K back-to-back launches of pass 1 alone (the same call with FOS_QUANT_PASSES=1).
    # An event between the two kernels of a step would add the idle time of its own packet, 4 us, to the figure.
    # Inside a step pass 2 reads what pass 1 has just pulled through the memory-side cache; the kernel trace of
    # this same command (profiles/) shows steps without gaps and gives the same two durations.
    amaxes = torch.zeros(n_buf, dtype=torch.float32, device=dev)

    def run_step(rotate_outputs=False):
        i = counter[0] % n_buf
        counter[0] += 1
        o = i if rotate_outputs else 0
        nat.check(L.fos_quantize(xs[i].data_ptr(), 0, rows, cols, cols, 0, 3, 0, 0, 0, 0, 1, codes_sets[o].data_ptr(),
                                 sf_sets[o].data_ptr(), amaxes[i:].data_ptr(), 0, ws.data_ptr(), ws_bytes, stream), "quantize")

    def run_amax():
        i = counter[0] % n_buf
        counter[0] += 1
        nat.check(L.fos_amax(xs[i].data_ptr(), 0, rows, cols, cols, amaxes[i:].data_ptr(), ws.data_ptr(), ws_bytes, stream), "amax")

    def run_quant_only():
        i = counter[0] % n_buf
        counter[0] += 1
        nat.check(L.fos_quantize(xs[i].data_ptr(), 0, rows, cols, cols, 0, 3, 0, 0, 0, 0, 1, codes_sets[i].data_ptr(),
                                 sf_sets[i].data_ptr(), amaxes[i:].data_ptr(), 1, ws.data_ptr(), ws_bytes, stream), "quantize")

    def pass1_only(on):
        if on:
            os.environ["FOS_QUANT_PASSES"] = "1"
        else:
            os.environ.pop("FOS_QUANT_PASSES", None)
        L.fos_tuning_reload()

    # (outputs: a set per input.  In the timed region above a call's result is freed once the next call has returned,
    # so the allocator alternates between two sets; with ONE set, which a launch partly finds dirty in L2 and never
    # sends to memory, a step reads ~1 us shorter: timed beside it.  The five loops are
    # measured in turn, five times over, and each reports the median of its averages: whichever loop runs first
    # after a pause reads 1-2 us longer per step.)
    # pass 2 alone, back to back (every buffer's maximum computed beforehand): each launch then starts while its
    # predecessor's 36 MiB of stores drain and finds nothing of its input cached -- no caller runs it that way;
    # kept as the conservative figure.  fos_amax: pass 1 and its one-workgroup reduction kernel.
    loops = {"step": lambda: run_step(True), "step_one_output_set": run_step, "pass1": run_step, "amax": run_amax,
             "alone": run_quant_only}
    samples = {name: [] for name in loops}
    for _ in range(n_buf):
        run_amax()
    try:
        for _ in range(5):
            for name, fn in loops.items():
                pass1_only(name == "pass1")
                for _ in range(W):
                    fn()
                samples[name].append(event_ms(fn, K))
    finally:
        pass1_only(False)
    med = {name: sorted(v)[len(v) // 2] for name, v in samples.items()}
    step_c_abi_ms, step_one_set_ms, pass1_ms = med["step"], med["step_one_output_set"], med["pass1"]
    amax_ms, quant_alone_ms = med["amax"], med["alone"]
    quant_ms = step_c_abi_ms - pass1_ms
    counter[0] = 0
    same_buffer_ms = event_ms(lambda: (
        nat.check(L.fos_quantize(xs[0].data_ptr(), 0, rows, cols, cols, 0, 3, 0, 0, 0, 0, 1, codes.data_ptr(), sf.data_ptr(),
                                 amax.data_ptr(), 0, ws.data_ptr(), ws_bytes, stream), "quantize")), K)
    q_achieved = algo_bytes / (quant_ms * 1e-3) / 1e9
    traffic, traffic_source = profiled_traffic(rows, cols)
    roofline = {
        "kernel": "fos::quantize_nvfp4_rows_kernel<3, true, false, false, false, false> (pass 2: scale, 4/6 select, pack)",
        "bound": "hbm",
        "achieved": round(q_achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(q_achieved / HBM_PEAK_GBS, 4),
        "traffic": traffic,
        "traffic_source": traffic_source,
        "kernel_ms": round(quant_ms, 5),
        "kernel_ms_is": "pass 2 inside the step: K steps (pass 1 + pass 2) minus K launches of pass 1, HIP events, C ABI",
        "step_c_abi_ms": round(step_c_abi_ms, 5),
        "pass1_ms": round(pass1_ms, 5),
        "pass1_GBs": round(elems * 2 / (pass1_ms * 1e-3) / 1e9, 1),
        "kernel_with_one_output_set_ms": round(step_one_set_ms - pass1_ms, 5),
        "kernel_alone_back_to_back_ms": round(quant_alone_ms, 5),
        "kernel_alone_back_to_back_frac": round(algo_bytes / (quant_alone_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "fos_amax_ms": round(amax_ms, 5),
        "whole_step_frac": round(value / HBM_PEAK_GBS, 4),
        "same_buffer_step_ms": round(same_buffer_ms, 5),
    }

    # ---- activation-style input with outlier channels (8192 x 4096) -----------------
    act_ms = None
    if not args.no_activation:
        xo = [make_activation(8192, 4096, 1 + i, outliers=True).to(dev) for i in range(6)]
        for i in range(W):
            fos.quantize(xo[i % 6], cfg)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            fos.quantize(xo[i % 6], cfg)
        torch.cuda.synchronize()
        act_ms = (time.perf_counter() - t0) * 1e3 / K
        del xo

    # ---- FP4 GEMM 8192^3 on pre-quantized operands ------------------------------------
    gemm = None
    if not args.no_gemm:
        m = n = k = 8192
        qa = fos.quantize(make_activation(m, k, 5).to(dev), cfg)
        qb = fos.quantize(make_activation(n, k, 6).to(dev), cfg)
        for _ in range(max(2, W // 2)):
            fos.quantized_matmul(qa, qb)
        # every call between its own pair of events: the sustained rate (the mean, which the roofline
        # fraction uses) lies below the first calls' because the clocks come down under this load
        gk = max(20, K // 2)
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(gk + 1)]
        evs[0].record()
        for i in range(gk):
            fos.quantized_matmul(qa, qb)
            evs[i + 1].record()
        torch.cuda.synchronize()
        per_call = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(gk))
        gemm_ms = sum(per_call) / gk
        tflops = 2.0 * m * n * k / (gemm_ms * 1e-3) / 1e12
        gemm = {
            "workload": "NVFP4 x NVFP4 -> bf16, M=N=K=8192, FP32 accumulate, alpha on device",
            "calls": gk,
            "ms": round(gemm_ms, 4),
            "ms_median": round(per_call[gk // 2], 4),
            "ms_min": round(per_call[0], 4),
            "value": round(tflops, 1),
            "unit": "TFLOP/s",
            "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None,
                         "frac_median": round(2.0 * m * n * k / (per_call[gk // 2] * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
                         "frac_best_call": round(2.0 * m * n * k / (per_call[0] * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4)},
        }

    # ---- 32-layer quantized-linear stack (Llama-3-8B projection shapes, 8 x 2048 tokens) --
    stack = None
    if not args.no_stack and not args.no_gemm:
        stack = linear_stack(dev, steps=3, warmup=1)

    extra = None
    if not args.no_extras:
        del xs[1:]
        torch.cuda.empty_cache()
        extra = extras(dev, steps=max(5, K // 5))

    # ---- CPU baseline: the C oracle on the host cores, bounded sample -----------------
    cpu = None
    if not args.no_cpu:
        import oracle

        oracle.build()
        threads = min(oracle.default_threads(), 16)
        sample_rows = 1024
        sample = xs[0][:sample_rows].cpu()
        oracle.quantize(sample[:128], scale_rule="mse", threads=threads)
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 10 and reps < 50):
            oracle.quantize(sample, scale_rule="mse", threads=threads)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        cpu = {
            "value": round(sample_rows * cols * BYTES_PER_ELEM / cpu_s / 1e9, 4),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"{sample_rows} x {cols} rows of the same tensor, {reps} repetitions, C oracle with OpenMP",
        }

    line = {
        "metric": "quantize GB/s (% HBM peak) + FP4 GEMM TFLOP/s (% roofline), 1 MI355X",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(step_ms, 5),
        "untimed_steps_before_timing": W + K + settle_steps + W,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"quantize {rows}x{cols} bf16 N(0,1) -> NVFP4, 4/6-MSE, round-to-nearest, 1x16 blocks, "
                        "E4M3 scales in the 128x4-tile layout (tensor-max pass + quantize pass), "
                        "4 rotating input buffers",
            "algorithmic_bytes_per_element": BYTES_PER_ELEM,
            "activation_8192x4096_outliers_ms": None if act_ms is None else round(act_ms, 5),
            "activation_8192x4096_outliers_GBs": None if act_ms is None else round(8192 * 4096 * BYTES_PER_ELEM / (act_ms * 1e-3) / 1e9, 1),
        },
        "cold_start": {
            "ms_per_step": round(cold_ms, 5),
            "value": round(algo_bytes / (cold_ms * 1e-3) / 1e9, 1),
            "note": "the same W + K steps on the idle GPU, before the untimed settling steps",
            "settle_ms": args.settle_ms,
            "settle_steps": settle_steps,
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
        "gemm": gemm,
        "linear_stack": stack,
        "extras": extra,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
