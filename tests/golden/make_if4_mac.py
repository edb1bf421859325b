"""Transcribe the dot-product known answers of the reference's MAC test benches into
``if4_mac.npz`` (data only: codes, scale bytes, expected fp32 bit patterns).

    python tests/golden/make_if4_mac.py [/root/reference]

Source: ``if4_mac/tb/nvfp4_mac_golden_ref.svh`` and ``if4_mac/tb/if4_mac_golden_ref.svh``
(31 cycles of 16 lanes each: three dot products of K = 160 and a closing all-zero cycle;
``expected_acc[0..2]`` at the end of each file).  Runs in the build container only.
"""

import os
import re
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def parse(path):
    text = open(path).read()
    n = 1 + max(int(m) for m in re.findall(r"first_vec\[(\d+)\]", text))
    first = np.zeros(n, np.uint8)
    a_sf = np.zeros(n, np.uint8)
    w_sf = np.zeros(n, np.uint8)
    a = np.zeros((n, 16), np.uint8)
    w = np.zeros((n, 16), np.uint8)
    for i, v in re.findall(r"first_vec\[(\d+)\] = 1'b([01]);", text):
        first[int(i)] = int(v)
    for name, arr in (("a_sf_vec", a_sf), ("w_sf_vec", w_sf)):
        for i, v in re.findall(name + r"\[(\d+)\] = 8'h([0-9A-F]{2});", text):
            arr[int(i)] = int(v, 16)
    for name, arr in (("a_vec", a), ("w_vec", w)):
        for i, lane, v in re.findall(name + r"\[(\d+)\]\[(\d+)\] = 4'h([0-9A-F]);", text):
            arr[int(i), int(lane)] = int(v, 16)
    expected = np.array([int(v, 16) for _, v in sorted(re.findall(r"expected_acc\[(\d+)\] = 32'h([0-9A-F]{8});", text))],
                        dtype=np.uint32)
    assert n == 31 and expected.size == 3
    return {"first": first, "a_sf": a_sf, "w_sf": w_sf, "a": a, "w": w, "expected": expected}


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    out = {}
    for tag, name in (("nvfp4", "nvfp4_mac_golden_ref.svh"), ("if4", "if4_mac_golden_ref.svh")):
        for k, v in parse(os.path.join(ref, "if4_mac", "tb", name)).items():
            out[f"{tag}.{k}"] = v
    np.savez_compressed(os.path.join(HERE, "if4_mac.npz"), **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
