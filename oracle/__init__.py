"""CPU oracle for the quantize / FP4-matmul path -- TEST INFRASTRUCTURE ONLY.

Thin ctypes/numpy wrapper around ``fos_oracle.c`` (a scalar C restatement of the
reference's PyTorch path; its header lists the reference file:line of every function).
Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this
package; the product package never does.

The host-side glue here restates ``PyTorchQuantizeBackend.quantize``
(reference ``src/fouroversix/quantize/pytorch/backend.py:39-121``): zero-pad to a
multiple of (128, 64), quantize, put NVFP4 scales into the 128x4-tile layout and leave
IF4 scales row-major.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "fos_oracle.c")
_LIB = os.path.join(_HERE, "libfos_oracle.so")

DTYPE_IDS = {"nvfp4": 0, "if4": 1}
RULE_IDS = {"static_6": 0, "static_4": 1, "mae": 2, "mse": 3, "abs_max": 4}
ROUND_IDS = {"nearest": 0, "stochastic": 1, "stochastic_unbiased": 2}

_lib = None


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (strict IEEE: no contraction, no fast-math)."""
    if force or not os.path.exists(_LIB) or os.path.getmtime(_LIB) < os.path.getmtime(_SRC):
        cmd = [
            "gcc", "-O2", "-std=c11", "-fPIC", "-shared", "-fopenmp",
            "-ffp-contract=off", "-fno-fast-math", "-o", _LIB, _SRC, "-lm",
        ]
        subprocess.run(cmd, check=True)
    return _LIB


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        L = ctypes.CDLL(_LIB)
        c = ctypes
        vp, i64, u64, f32, i32 = c.c_void_p, c.c_int64, c.c_uint64, c.c_float, c.c_int
        L.fos_oracle_e4m3_from_f32.argtypes = [f32]
        L.fos_oracle_e4m3_from_f32.restype = c.c_uint8
        L.fos_oracle_e4m3_to_f32.argtypes = [c.c_uint8]
        L.fos_oracle_e4m3_to_f32.restype = f32
        L.fos_oracle_e2m1_rtn.argtypes = [f32]
        L.fos_oracle_e2m1_rtn.restype = f32
        L.fos_oracle_e2m1_sr_code.argtypes = [f32, c.c_uint32]
        L.fos_oracle_e2m1_sr_code.restype = c.c_uint8
        L.fos_oracle_e2m1_decode.argtypes = [c.c_uint8]
        L.fos_oracle_e2m1_decode.restype = f32
        L.fos_oracle_sum16.argtypes = [vp]
        L.fos_oracle_sum16.restype = f32
        L.fos_oracle_sum256.argtypes = [vp]
        L.fos_oracle_sum256.restype = f32
        L.fos_oracle_philox4x32_10.argtypes = [vp, vp, vp]
        L.fos_oracle_philox4x32_10.restype = None
        L.fos_oracle_quantize.argtypes = [vp, i64, i64, i32, i32, i32, i32, u64, u64, vp, vp, vp, i32]
        L.fos_oracle_quantize.restype = i32
        L.fos_oracle_quantize_with_amax.argtypes = [vp, i64, i64, i32, i32, i32, i32, u64, u64, vp, vp, vp, vp, i32]
        L.fos_oracle_quantize_with_amax.restype = i32
        L.fos_oracle_quantize_typed.argtypes = [vp, i32, i64, i64, i32, i32, i32, i32, u64, u64, vp, vp, vp, vp, i32]
        L.fos_oracle_quantize_typed.restype = i32
        L.fos_oracle_quantize_errors.argtypes = [vp, i32, i64, i64, i32, i32, i32, i32, u64, u64, vp, vp, vp, vp, i32, vp]
        L.fos_oracle_quantize_errors.restype = i32
        L.fos_oracle_blocked_offset.argtypes = [i64, i64, i64]
        L.fos_oracle_blocked_offset.restype = i64
        L.fos_oracle_to_blocked.argtypes = [vp, i64, i64, vp]
        L.fos_oracle_to_blocked.restype = None
        L.fos_oracle_from_blocked.argtypes = [vp, i64, i64, vp]
        L.fos_oracle_from_blocked.restype = None
        L.fos_oracle_dequantize.argtypes = [vp, vp, f32, i32, c.c_double, i64, i64, vp, i32]
        L.fos_oracle_dequantize.restype = i32
        L.fos_oracle_dequantize_ex.argtypes = [vp, vp, f32, i32, c.c_double, i64, i64, vp, i32, i32]
        L.fos_oracle_dequantize_ex.restype = i32
        L.fos_oracle_matmul_nt.argtypes = [vp, vp, i64, i64, i64, vp, vp, i32]
        L.fos_oracle_matmul_nt.restype = None
        L.fos_oracle_gemm_nvfp4.argtypes = [vp, vp, vp, vp, f32, i64, i64, i64, vp, vp, i32]
        L.fos_oracle_gemm_nvfp4.restype = None
        _lib = L
    return _lib


def _ptr(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def default_threads() -> int:
    return max(1, len(os.sched_getaffinity(0)))


def bf16_bits(x) -> np.ndarray:
    """torch bf16 tensor (CPU) or uint16 ndarray -> contiguous uint16 ndarray."""
    if isinstance(x, np.ndarray):
        assert x.dtype == np.uint16
        return np.ascontiguousarray(x)
    import torch

    assert x.dtype == torch.bfloat16
    return x.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def qmax_smax(dtype: str, rule: str) -> tuple[float, float]:
    """(largest element magnitude, largest block scale) used by the format + rule."""
    qmax = 4.0 if rule == "static_4" else 6.0
    smax = 448.0 if (dtype == "if4" or rule in ("static_6", "static_4")) else 256.0
    return qmax, smax


def adjustment(round_style: str) -> float:
    return 16 / 17 if round_style == "stochastic_unbiased" else 1.0


@dataclass
class OracleQuantized:
    values: np.ndarray          # u8 [Mp, Np/2]
    scale_factors: np.ndarray   # u8 flat: 128x4 tiles (nvfp4) or row-major (if4)
    scale_rows: np.ndarray      # u8 [Mp, Np/16] row-major, always
    amax: np.float32
    dtype: str
    scale_rule: str
    round_style: str
    original_shape: tuple[int, int]
    padded_shape: tuple[int, int]
    blocked: bool


def pad_bits(xb: np.ndarray) -> np.ndarray:
    m, n = xb.shape
    mp, np_ = -(-m // 128) * 128, -(-n // 64) * 64
    if (mp, np_) == (m, n):
        return xb
    out = np.zeros((mp, np_), dtype=xb.dtype)
    out[:m, :n] = xb
    return out


def input_bits(x) -> tuple[np.ndarray, int]:
    """(array, input type id) of a quantize input: bf16 (torch tensor or uint16 bit patterns) -> uint16, 0;
    fp16 (torch or numpy) -> uint16 bit patterns, 1; fp32 -> float32, 2."""
    if isinstance(x, np.ndarray):
        if x.dtype == np.float32:
            return np.ascontiguousarray(x), 2
        if x.dtype == np.float16:
            return np.ascontiguousarray(x).view(np.uint16), 1
        return bf16_bits(x), 0
    import torch

    if x.dtype == torch.float32:
        return x.detach().cpu().contiguous().numpy(), 2
    if x.dtype == torch.float16:
        return x.detach().cpu().contiguous().numpy().view(np.uint16), 1
    return bf16_bits(x), 0


# Hard-coded sign vector and Sylvester-ordered 16-point Hadamard matrix of the reference's
# random Hadamard transform (src/fouroversix/quantize/utils.py:19-85): RHT = diag(signs) @ H / 4.
RHT_SIGNS = np.array([1, 1, 1, -1, 1, -1, -1, -1, -1, -1, -1, 1, -1, 1, -1, -1], dtype=np.float32)


def rht_matrix() -> np.ndarray:
    idx = np.arange(16)
    had = np.array([[(-1.0) ** bin(i & j).count("1") for j in idx] for i in idx], dtype=np.float32)
    return (RHT_SIGNS[:, None] * had * np.float32(0.25)).astype(np.float32)


def f32_to_bf16_bits(f: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(f, dtype=np.float32).view(np.uint32)
    return ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


def transform(xb: np.ndarray, *, transpose=False, rht=False, x_type=0) -> np.ndarray:
    """Bit patterns (bf16, or fp16 when ``x_type`` is 1) of the tensor the reference quantizes when
    ``transpose`` / ``rht`` are set (src/fouroversix/quantize/pytorch/reference.py:567-571): ``x.T``,
    then every group of 16 consecutive elements of a row times the RHT matrix cast to the input's
    type, as a matmul of that type, i.e. exact products, fp32 accumulation (here in the order
    i = 0..15), one rounding to the input's type.  A ragged width is first completed with zeros
    (the reference pads to its block multiples before the transform,
    src/fouroversix/quantize/pytorch/backend.py:57-79), so with ``rht`` the result is a multiple
    of 16 wide."""
    if x_type == 2:
        # fp32 input: the reference's product is a library fp32 matmul (summation order not fixed); the target
        # stated here is the exact product, formed in fp64 and rounded once to fp32
        xf = np.asarray(xb, dtype=np.float32)
        if transpose:
            xf = np.ascontiguousarray(xf.T)
        if rht:
            if xf.shape[1] % 16:
                xf = np.pad(xf, ((0, 0), (0, 16 - xf.shape[1] % 16)))
            xf = (xf.astype(np.float64).reshape(-1, 16) @ rht_matrix().astype(np.float64)).astype(np.float32).reshape(xf.shape)
        return xf
    xb = np.asarray(xb, dtype=np.uint16)
    if transpose:
        xb = np.ascontiguousarray(xb.T)
    if rht:
        if xb.shape[1] % 16:
            xb = np.pad(xb, ((0, 0), (0, 16 - xb.shape[1] % 16)))
        g = (xb.view(np.float16).astype(np.float32) if x_type == 1 else bf16_bits_to_f32(xb)).reshape(-1, 16)
        h = rht_matrix()
        acc = np.zeros_like(g)
        for i in range(16):
            acc = acc + g[:, i:i + 1] * h[i][None, :]
        out = acc.astype(np.float16).view(np.uint16) if x_type == 1 else f32_to_bf16_bits(acc)
        xb = out.reshape(xb.shape)
    return xb


def quantize(x, *, dtype="nvfp4", scale_rule="mse", round_style="nearest",
             block_scale_2d=False, seed=0, offset=0, threads=None,
             transpose=False, rht=False, amax=None) -> OracleQuantized:
    xb, x_type = input_bits(x)
    assert xb.ndim == 2
    if transpose or rht:
        xb = transform(xb, transpose=transpose, rht=rht, x_type=x_type)
    orig = tuple(int(v) for v in xb.shape)
    xp = np.ascontiguousarray(pad_bits(xb))
    mp, np_ = xp.shape
    codes = np.zeros((mp, np_ // 2), dtype=np.uint8)
    sf = np.zeros((mp, np_ // 16), dtype=np.uint8)
    amax_in = None if amax is None else np.array([amax], dtype=np.float32)
    amax = np.zeros(1, dtype=np.float32)
    rc = lib().fos_oracle_quantize_typed(
        _ptr(xp), x_type, mp, np_, DTYPE_IDS[dtype], RULE_IDS[scale_rule], ROUND_IDS[round_style],
        int(block_scale_2d), seed, offset, _ptr(codes), _ptr(sf), _ptr(amax),
        None if amax_in is None else _ptr(amax_in), threads or default_threads(),
    )
    if rc != 0:
        raise ValueError(f"oracle: unsupported combination {dtype}/{scale_rule}")
    blocked = dtype == "nvfp4"
    flat = to_blocked(sf) if blocked else sf.reshape(-1).copy()
    return OracleQuantized(codes, flat, sf, amax[0], dtype, scale_rule, round_style,
                           orig, (mp, np_), blocked)


def selection_errors(x, *, dtype="nvfp4", scale_rule="mse", block_scale_2d=False, amax=None, threads=None,
                     round_style="nearest", seed=0, offset=0) -> np.ndarray:
    """f32 [M, N/16, 2]: the two errors the adaptive rule compared for every 1x16 block of an
    unpadded-or-padded bf16 input, first the "6" / E2M1 candidate, second the "4" / INT4 one; the
    second wins when strictly smaller.  With a stochastic ``round_style`` the candidates are the
    stochastically rounded ones of (seed, offset), and the width must already be a multiple of 64
    (the dither is keyed by the block's index in the padded tensor)."""
    xb, x_type = input_bits(x)
    xp = np.ascontiguousarray(xb)
    m, n = xp.shape
    codes = np.zeros((m, n // 2), dtype=np.uint8)
    sf = np.zeros((m, n // 16), dtype=np.uint8)
    errors = np.zeros((m, n // 16, 2), dtype=np.float32)
    amax_in = None if amax is None else np.array([amax], dtype=np.float32)
    amax_out = np.zeros(1, dtype=np.float32)
    rc = lib().fos_oracle_quantize_errors(
        _ptr(xp), x_type, m, n, DTYPE_IDS[dtype], RULE_IDS[scale_rule], ROUND_IDS[round_style], int(block_scale_2d),
        seed, offset, _ptr(codes), _ptr(sf), _ptr(amax_out), None if amax_in is None else _ptr(amax_in),
        threads or default_threads(), _ptr(errors))
    assert rc == 0
    return errors


def to_blocked(sf_rows: np.ndarray) -> np.ndarray:
    sf_rows = np.ascontiguousarray(sf_rows)
    out = np.zeros(sf_rows.size, dtype=np.uint8)
    lib().fos_oracle_to_blocked(_ptr(sf_rows), sf_rows.shape[0], sf_rows.shape[1], _ptr(out))
    return out


def from_blocked(flat: np.ndarray, rows: int, cols: int) -> np.ndarray:
    flat = np.ascontiguousarray(flat)
    out = np.zeros((rows, cols), dtype=np.uint8)
    lib().fos_oracle_from_blocked(_ptr(flat), rows, cols, _ptr(out))
    return out


def dequantize(values: np.ndarray, scale_rows: np.ndarray, amax, *, dtype="nvfp4",
               scale_rule="mse", round_style="nearest", original_shape=None,
               threads=None, f32_intermediate=False) -> np.ndarray:
    """f32 [M, N] = the reference's ``dequantize(..., dtype=float32)``; value and block scale
    meet in fp16 (its default intermediate dtype) or, with ``f32_intermediate``, in fp32."""
    values = np.ascontiguousarray(values)
    scale_rows = np.ascontiguousarray(scale_rows)
    mp, half = values.shape
    qmax, smax = qmax_smax(dtype, scale_rule)
    div = qmax * smax * adjustment(round_style)
    out = np.zeros((mp, half * 2), dtype=np.float32)
    rc = lib().fos_oracle_dequantize_ex(_ptr(values), _ptr(scale_rows), float(amax), DTYPE_IDS[dtype],
                                        div, mp, half * 2, _ptr(out), threads or default_threads(), int(f32_intermediate))
    assert rc == 0
    if original_shape is not None:
        out = out[: original_shape[0], : original_shape[1]]
    return out


def matmul_nt(a: np.ndarray, b: np.ndarray, threads=None) -> tuple[np.ndarray, np.ndarray]:
    """(bf16 bits, f32) of a @ b.T accumulated in double."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    n = b.shape[0]
    o16 = np.zeros((m, n), dtype=np.uint16)
    o32 = np.zeros((m, n), dtype=np.float32)
    lib().fos_oracle_matmul_nt(_ptr(a), _ptr(b), m, n, k, _ptr(o16), _ptr(o32), threads or default_threads())
    return o16, o32


def quantized_matmul(qa: OracleQuantized, qb: OracleQuantized, threads=None):
    """PyTorch-backend form: dequantize both to f32, multiply, round to bf16, crop."""
    a = dequantize(qa.values, qa.scale_rows, qa.amax, dtype=qa.dtype, scale_rule=qa.scale_rule,
                   round_style=qa.round_style, threads=threads)
    b = dequantize(qb.values, qb.scale_rows, qb.amax, dtype=qb.dtype, scale_rule=qb.scale_rule,
                   round_style=qb.round_style, threads=threads)
    o16, o32 = matmul_nt(a, b, threads)
    m, n = qa.original_shape[0], qb.original_shape[0]
    return o16[:m, :n], o32[:m, :n]


def gemm_alpha(qa: OracleQuantized, qb: OracleQuantized) -> np.float32:
    """alpha of the native GEMM form (reference matmul/cutlass/backend.py:86-98), with the
    arithmetic torch uses for ``tensor / python_scalar`` on a GPU (where that backend
    runs): the product times the reciprocal, taken in double and rounded to fp32."""
    qa_max, sa_max = qmax_smax(qa.dtype, qa.scale_rule)
    qb_max, sb_max = qmax_smax(qb.dtype, qb.scale_rule)
    den = qa_max * sa_max * qb_max * sb_max * adjustment(qa.round_style) * adjustment(qb.round_style)
    return np.float32(np.float32(np.float32(qa.amax) * np.float32(qb.amax)) * np.float32(1.0 / den))


def gemm_nvfp4(values_a, sf_rows_a, values_b, sf_rows_b, alpha, threads=None):
    """Native-GEMM form: bf16(alpha * sum_k (vA sA)(vB sB)) on padded operands."""
    m, n, k = values_a.shape[0], values_b.shape[0], values_a.shape[1] * 2
    o16 = np.zeros((m, n), dtype=np.uint16)
    o32 = np.zeros((m, n), dtype=np.float32)
    # (named, so that the copies made for strided arguments live until the call returns)
    va, vb = np.ascontiguousarray(values_a), np.ascontiguousarray(values_b)
    sa, sb = np.ascontiguousarray(sf_rows_a), np.ascontiguousarray(sf_rows_b)
    lib().fos_oracle_gemm_nvfp4(_ptr(va), _ptr(vb), _ptr(sa), _ptr(sb),
                                float(alpha), m, n, k, _ptr(o16), _ptr(o32), threads or default_threads())
    return o16, o32


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


# ---- MXFP4: E2M1 codes, one E8M0 scale per 1x32 block --------------------------------------
# numpy restatement of quantize_to_mxfp4 + fake_quantize_to_e2m1 + the code packing
# (src/fouroversix/quantize/pytorch/reference.py:30-51, 82-132, 149-181) and of the mx branch
# of dequantize (src/fouroversix/quantize/backend.py:89-160).  Pinned by tests/golden/mxfp4.npz.

E2M1_VALUES = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6], dtype=np.float32)


def pad_bits_mx(xb: np.ndarray) -> np.ndarray:
    """Zero-pad to rows % 128 == 0, cols % 128 == 0 (4 blocks of 32;
    src/fouroversix/quantize/pytorch/backend.py:57-79)."""
    m, n = xb.shape
    out = np.zeros((-(-m // 128) * 128, -(-n // 128) * 128), dtype=np.uint16)
    out[:m, :n] = xb
    return out


def quantize_mxfp4(x, *, scale_rule="static_6") -> OracleQuantized:
    """``x``: bf16 tensor / uint16 bit array, or an fp16 / fp32 torch tensor (the reference converts
    whatever it is given with ``.float()``; pinned by tests/golden/mxfp4_input_dtypes.npz)."""
    assert scale_rule in ("static_6", "static_4")
    if not isinstance(x, np.ndarray) and str(x.dtype) in ("torch.float16", "torch.float32"):
        xf = x.detach().cpu().float().contiguous().numpy()
        orig = tuple(int(v) for v in xf.shape)
        xp32 = np.zeros((-(-orig[0] // 128) * 128, -(-orig[1] // 128) * 128), dtype=np.float32)
        xp32[: orig[0], : orig[1]] = xf
        mp, np_ = xp32.shape
        blocks = xp32.reshape(-1, 32)
    else:
        xb = bf16_bits(x)
        orig = tuple(int(v) for v in xb.shape)
        xp = pad_bits_mx(xb)
        mp, np_ = xp.shape
        blocks = bf16_bits_to_f32(xp).reshape(-1, 32)
    qmax = np.float32(6.0 if scale_rule == "static_6" else 4.0)
    s_hp = (np.abs(blocks).max(axis=1) / qmax).astype(np.float32)
    u = s_hp.view(np.uint32)
    e = ((u >> np.uint32(23)) & np.uint32(0xFF)).astype(np.uint8)
    e = np.where((u & np.uint32(0x7FFFFF)) == 0, e, e + np.uint8(1)).astype(np.uint8)  # round up to a power of two
    s = (e.astype(np.uint32) << np.uint32(23)).view(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        xs = np.where((e != 0)[:, None], blocks / s[:, None], np.float32(0)).astype(np.float32)
    a = np.abs(xs)
    r = np.where(a < 2, np.rint(a + a) * np.float32(0.5), np.where(a < 4, np.rint(a), np.float32(2) * np.rint(a * np.float32(0.5))))
    fq = (r * np.sign(xs)).astype(np.float32)  # sign(+-0) = 0; a negative value rounding to zero gives -0.0
    mag = np.searchsorted(E2M1_VALUES, np.abs(fq)).astype(np.uint8)
    code = (mag | (np.signbit(fq).astype(np.uint8) << 3)).reshape(mp, np_)
    values = (code[:, 0::2] | (code[:, 1::2] << 4)).astype(np.uint8)
    sf_rows = e.reshape(mp, np_ // 32)
    return OracleQuantized(values, to_blocked(sf_rows), sf_rows, np.float32(1.0), "mxfp4", scale_rule, "nearest",
                           orig, (mp, np_), True)


def dequantize_mxfp4(values: np.ndarray, scale_rows: np.ndarray, original_shape=None, f32_intermediate=False) -> np.ndarray:
    """f32 [M, N]: fp16(value) * fp16(2^(e - 127)), the product rounded to fp16 (the reference's
    intermediate dtype; scales outside fp16's range become 0 or inf there), widened; with
    ``f32_intermediate`` the product is formed in fp32 (exact short of overflow)."""
    code = np.empty((values.shape[0], values.shape[1] * 2), dtype=np.uint8)
    code[:, 0::2] = values & 0xF
    code[:, 1::2] = values >> 4
    inter = np.float32 if f32_intermediate else np.float16
    v16 = (E2M1_VALUES[code & 7] * np.where(code & 8, np.float32(-1), np.float32(1))).astype(inter)
    with np.errstate(over="ignore", invalid="ignore"):  # 0 * inf = NaN, as in the reference's fp16 product
        s16 = np.ldexp(np.float64(1.0), scale_rows.astype(np.int32) - 127).astype(inter)
        out = (v16 * np.repeat(s16, 32, axis=1)).astype(np.float32)
    if original_shape is not None:
        out = out[: original_shape[0], : original_shape[1]]
    return out


def gemm_mxfp4(values_a, sf_rows_a, values_b, sf_rows_b):
    """bf16 bits and f32 of sum_k (a 2^ea)(b 2^eb) on padded operands, accumulated in double
    (alpha = 1: src/fouroversix/matmul/cutlass/backend.py:79-85)."""
    def expand(values, sf_rows):
        code = np.empty((values.shape[0], values.shape[1] * 2), dtype=np.uint8)
        code[:, 0::2] = values & 0xF
        code[:, 1::2] = values >> 4
        v = E2M1_VALUES[code & 7].astype(np.float64) * np.where(code & 8, -1.0, 1.0)
        return v * np.repeat(np.ldexp(1.0, sf_rows.astype(np.int32) - 127), 32, axis=1)

    o32 = (expand(values_a, sf_rows_a) @ expand(values_b, sf_rows_b).T).astype(np.float32)
    return f32_to_bf16_bits(o32), o32
