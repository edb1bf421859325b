"""Search for blocks whose two candidates' selection errors nearly tie, and write them to
``near_ties.npz`` (inputs only; the expected bytes come from the oracle when the test runs).

    python tests/golden/make_near_ties.py

The adaptive rules compare two errors per block (4/6: "6" against "4"; IF4: E2M1 against
INT4).  The kernels decide most blocks from cheaper reductions with a certified tolerance and
fall back to the exact evaluation inside it, so the inputs that matter are blocks whose errors
differ by a few units in the last place without being equal.  Random data almost never
holds one; this script draws blocks (1 x 16) and tiles (16 x 16) from several distributions
under a fixed tensor maximum, keeps those with 0 < |eA - eB| <= tol * max(eA, eB) according to
the oracle, and stores them per case.  A case is named

    <format>.<1d|2d>.<rule>.<nearest|stochastic>[.given]

(``given``: the tensor maximum is handed in by the caller, is not a bf16 value and exceeds
max|x|) and holds

    <case>.x      uint16 [rows, cols] bf16 bits (block (0, 0) holds the planted tensor maximum)
    <case>.amax   float32 [1] the tensor maximum the search ran under
    <case>.seed   int64 [1]   seed of the stochastic style (0 for round to nearest)

Round to nearest: a block's result depends on its elements and the tensor maximum only, so
the blocks found are packed densely.  Stochastic styles: the dither is keyed by the block's
position, so the search draws whole tensors of the fixture's shape and keeps a found block at
the position where it was found (zeros elsewhere).
"""

import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

TOL = 2e-6        # relative distance of the two errors that counts as a near tie
TOL_WIDE = 2e-4   # a second band: inside the kernels' tolerance, far from the last place
COLS = 1024
PEAK = 8.0
BUDGET_S = 240.0  # per case


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


def bands(bits, unit, **kw):
    """(near-tie mask, wide-band mask) over the blocks / tiles of one drawn tensor."""
    e = oracle.selection_errors(bits, **kw)
    ea, eb = e[::unit, :, 0].astype(np.float64), e[::unit, :, 1].astype(np.float64)
    rel = np.abs(ea - eb) / np.maximum(np.maximum(ea, eb), 1e-300)
    return (ea != eb) & (rel <= TOL), (ea != eb) & (rel > TOL) & (rel <= TOL_WIDE), ea.size


def search(dtype, rule, two_d, given_amax, want, wide, seed):
    """Round to nearest: found blocks are packed densely behind the planted maximum."""
    rng = np.random.default_rng(seed)
    amax = np.float32(given_amax) if given_amax else np.float32(PEAK)
    peak_bits = oracle.f32_to_bf16_bits(np.array([PEAK], np.float32))[0]
    found, found_wide = [], []
    rows = 4096
    unit = 16 if two_d else 1
    n_seen, t0 = 0, time.time()
    while len(found) < want or len(found_wide) < wide:
        bits = draw(rng, rows, COLS, PEAK)
        if not given_amax:
            bits[0, 0] = peak_bits
        close, wide_band, n = bands(bits, unit, dtype=dtype, scale_rule=rule, block_scale_2d=two_d,
                                    amax=float(amax) if given_amax else None)
        for mask, out, cap in ((close, found, want), (wide_band, found_wide, wide)):
            for r, c in zip(*np.nonzero(mask)):
                if len(out) < cap and not (r == 0 and c == 0):
                    out.append(bits[r * unit:(r + 1) * unit, c * 16:(c + 1) * 16].copy())
        n_seen += n
        if n_seen > 4e8 or time.time() - t0 > BUDGET_S:
            break
    print(f"{dtype} {rule} 2d={two_d} amax={amax}: {len(found)} near ties, {len(found_wide)} in the wide band, "
          f"{n_seen} blocks seen", flush=True)
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


def search_in_place(dtype, rule, two_d, given_amax, want, wide, seed, sr_seed):
    """Stochastic style: a found block stays where the search saw it (the dither of a block is
    keyed by its position in the padded tensor and by ``sr_seed``)."""
    rng = np.random.default_rng(seed)
    amax = np.float32(given_amax) if given_amax else np.float32(PEAK)
    peak_bits = oracle.f32_to_bf16_bits(np.array([PEAK], np.float32))[0]
    unit = 16 if two_d else 1
    rows = 128 * unit if two_d else 256
    x = np.zeros((rows, COLS), dtype=np.uint16)
    if not given_amax:
        x[0, 0] = peak_bits
    taken = np.zeros((rows // unit, COLS // 16), dtype=bool)
    taken[0, 0] = True
    n_close = n_wide = n_seen = 0
    t0 = time.time()
    while n_close < want or n_wide < wide:
        bits = draw(rng, rows, COLS, PEAK)
        if not given_amax:
            bits[0, 0] = peak_bits
        close, wide_band, n = bands(bits, unit, dtype=dtype, scale_rule=rule, block_scale_2d=two_d,
                                    amax=float(amax) if given_amax else None, round_style="stochastic", seed=sr_seed)
        for mask, is_close in ((close, True), (wide_band, False)):
            for r, c in zip(*np.nonzero(mask & ~taken)):
                if (n_close < want) if is_close else (n_wide < wide):
                    x[r * unit:(r + 1) * unit, c * 16:(c + 1) * 16] = bits[r * unit:(r + 1) * unit, c * 16:(c + 1) * 16]
                    taken[r, c] = True
                    if is_close:
                        n_close += 1
                    else:
                        n_wide += 1
        n_seen += n
        if time.time() - t0 > BUDGET_S:
            break
    print(f"{dtype} {rule} 2d={two_d} amax={amax} stochastic: {n_close} near ties, {n_wide} in the wide band, "
          f"{n_seen} blocks seen", flush=True)
    # the result must be what the search saw: same errors at the kept positions
    close, wide_band, _ = bands(x, unit, dtype=dtype, scale_rule=rule, block_scale_2d=two_d,
                                amax=float(amax) if given_amax else None, round_style="stochastic", seed=sr_seed)
    assert int(close.sum()) >= n_close and int(wide_band.sum()) >= n_wide
    return x, np.array([amax], np.float32)


def main():
    out = {}
    given = float(np.float32(PEAK * 1.2345678))
    # (format, rule, 2-D, caller's maximum, near ties wanted, wide-band blocks wanted)
    nearest = [
        ("nvfp4", "mse", False, 0.0, 192, 192),
        ("nvfp4", "mse", True, 0.0, 24, 64),
        ("if4", "mse", False, 0.0, 192, 192),
        ("if4", "mse", True, 0.0, 24, 64),
        ("nvfp4", "mse", False, given, 96, 96),
        ("nvfp4", "mse", True, given, 12, 32),
        ("if4", "mse", False, given, 96, 96),
        ("nvfp4", "mae", False, 0.0, 192, 192),
        ("nvfp4", "mae", True, 0.0, 24, 64),
        ("nvfp4", "mae", False, given, 96, 96),
        ("nvfp4", "mae", True, given, 12, 32),
        ("nvfp4", "abs_max", False, 0.0, 96, 96),
        ("nvfp4", "abs_max", True, 0.0, 24, 64),
        ("nvfp4", "abs_max", True, given, 12, 32),
    ]
    for i, (dtype, rule, two_d, amax, want, wide) in enumerate(nearest):
        x, a = search(dtype, rule, two_d, amax, want, wide, 1000 + i)
        name = f"{dtype}.{'2d' if two_d else '1d'}.{rule}.nearest" + (".given" if amax else "")
        out[name + ".x"], out[name + ".amax"], out[name + ".seed"] = x, a, np.array([0], np.int64)
    stochastic = [
        ("nvfp4", "mse", False, 0.0, 96, 96, 11),
        ("nvfp4", "mae", False, 0.0, 96, 96, 12),
        ("nvfp4", "mse", True, 0.0, 8, 32, 13),
        ("nvfp4", "mse", False, given, 48, 48, 14),
    ]
    for i, (dtype, rule, two_d, amax, want, wide, sr_seed) in enumerate(stochastic):
        x, a = search_in_place(dtype, rule, two_d, amax, want, wide, 2000 + i, sr_seed)
        name = f"{dtype}.{'2d' if two_d else '1d'}.{rule}.stochastic" + (".given" if amax else "")
        out[name + ".x"], out[name + ".amax"], out[name + ".seed"] = x, a, np.array([sr_seed], np.int64)
    np.savez_compressed(os.path.join(HERE, "near_ties.npz"), **out)


if __name__ == "__main__":
    main()
