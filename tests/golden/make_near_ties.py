"""Search for blocks whose two candidates' selection errors nearly tie, and write them to
``near_ties.npz`` (inputs only; the expected bytes come from the oracle when the test runs).

    python tests/golden/make_near_ties.py

The adaptive rules compare two error sums per block (4/6: "6" against "4"; IF4: E2M1 against
INT4).  The kernels decide most blocks from cheaper sums with a certified tolerance and fall
back to the exact evaluation inside it, so the inputs that matter are blocks whose errors
differ by a few units in the last place without being equal.  Random data almost never
holds one; this script draws blocks (1 x 16) and tiles (16 x 16) from several distributions
under a fixed tensor maximum, keeps those with 0 < |eA - eB| <= tol * max(eA, eB) according to
the oracle, and stores them per case:

    <case>.x      uint16 [rows, cols] bf16 bits (row 0 holds the planted tensor maximum)
    <case>.amax   float32 [1] the tensor maximum the search ran under (for the cases with a
                  caller-supplied maximum it is not a bf16 value and exceeds max|x|)
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

TOL = 2e-6        # relative distance of the two errors that counts as a near tie
TOL_WIDE = 2e-4   # a second band: inside the kernels' tolerance, far from the last place
COLS = 1024


def draw(rng, rows, cols, peak):
    kind = rng.integers(0, 4)
    if kind == 0:
        x = rng.standard_normal((rows, cols))
    elif kind == 1:
        x = rng.standard_normal((rows, cols)) * np.exp(rng.standard_normal((rows, cols // 16)) * 1.5).repeat(16, axis=1)
    elif kind == 2:
        x = rng.standard_t(3, (rows, cols))
    else:
        x = rng.uniform(-1, 1, (rows, cols)) * rng.uniform(0.01, 4.0, (rows, cols // 16)).repeat(16, axis=1)
    x = np.clip(x, -peak, peak).astype(np.float32)
    bits = oracle.f32_to_bf16_bits(x).reshape(rows, cols)
    return bits


def search(dtype, two_d, given_amax, want, wide, seed):
    rng = np.random.default_rng(seed)
    peak = 8.0
    amax = np.float32(given_amax) if given_amax else np.float32(peak)
    peak_bits = oracle.f32_to_bf16_bits(np.array([peak], np.float32))[0]
    found, found_wide = [], []
    rows = 4096
    unit = 16 if two_d else 1
    n_seen = 0
    while len(found) < want or len(found_wide) < wide:
        bits = draw(rng, rows, COLS, peak)
        if not given_amax:
            bits[0, 0] = peak_bits
        e = oracle.selection_errors(bits, dtype=dtype, scale_rule="mse", block_scale_2d=two_d, amax=float(amax) if given_amax else None)
        ea, eb = e[::unit, :, 0].astype(np.float64), e[::unit, :, 1].astype(np.float64)
        rel = np.abs(ea - eb) / np.maximum(np.maximum(ea, eb), 1e-300)
        close = (ea != eb) & (rel <= TOL)
        wide_band = (ea != eb) & (rel > TOL) & (rel <= TOL_WIDE)
        for mask, out, cap in ((close, found, want), (wide_band, found_wide, wide)):
            for r, c in zip(*np.nonzero(mask)):
                if len(out) < cap and not (r == 0 and c == 0):
                    out.append(bits[r * unit:(r + 1) * unit, c * 16:(c + 1) * 16].copy())
        n_seen += ea.size
        if n_seen > 4e8:
            break
    print(f"{dtype} 2d={two_d} amax={amax}: {len(found)} near ties, {len(found_wide)} in the wide band, {n_seen} blocks seen")
    blocks = found + found_wide
    # assemble: row band 0 carries the planted maximum, the found blocks follow
    per_row = COLS // 16
    n_rows = -(-(len(blocks) + 1) // per_row)
    x = np.zeros((n_rows * unit, COLS), dtype=np.uint16)
    if not given_amax:
        x[0, 0] = peak_bits
    for i, b in enumerate(blocks, start=1):
        r, c = divmod(i, per_row)
        x[r * unit:(r + 1) * unit, c * 16:(c + 1) * 16] = b
    return x, np.array([amax], np.float32)


def main():
    out = {}
    given = float(np.float32(8.0 * 1.2345678))
    cases = [
        ("nvfp4.1d", "nvfp4", False, 0.0, 192, 192),
        ("nvfp4.2d", "nvfp4", True, 0.0, 24, 64),
        ("if4.1d", "if4", False, 0.0, 192, 192),
        ("if4.2d", "if4", True, 0.0, 24, 64),
        ("nvfp4.1d.given", "nvfp4", False, given, 96, 96),
        ("nvfp4.2d.given", "nvfp4", True, given, 12, 32),
        ("if4.1d.given", "if4", False, given, 96, 96),
    ]
    for i, (name, dtype, two_d, amax, want, wide) in enumerate(cases):
        x, a = search(dtype, two_d, amax, want, wide, 1000 + i)
        out[name + ".x"], out[name + ".amax"] = x, a
    np.savez_compressed(os.path.join(HERE, "near_ties.npz"), **out)


if __name__ == "__main__":
    main()
