"""fos_quantize_static (the entry point that allocates nothing) against fos_quantize, both
through the C ABI: same bytes on two calls in a row, the second on a smaller input."""

import numpy as np
import pytest
import torch

from fouroversix_amd import _native as nat

pytestmark = pytest.mark.gpu

MSE, STATIC_6 = 3, 0


def _call(entry, x, rule, block2d, layout, workspace=None):
    rows, cols = x.shape
    L = nat.lib()
    rows_p, cols_p = L.fos_padded_rows(rows), L.fos_padded_cols(cols)
    # poisoned outputs: every byte must be written by the call
    codes = torch.full((rows_p, cols_p // 2), 0xAB, dtype=torch.uint8, device=x.device)
    sf = torch.full((rows_p * cols_p // 16,), 0xCD, dtype=torch.uint8, device=x.device)
    amax = torch.full((1,), -1.0, dtype=torch.float32, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    head = (x.data_ptr(), nat.T_BF16, rows, cols, x.stride(0), 0, rule, 0, block2d, 0, 0, layout,
            codes.data_ptr(), sf.data_ptr(), amax.data_ptr(), 0)
    if entry == "static":
        rc = L.fos_quantize_static(*head, stream)
    else:
        rc = L.fos_quantize(*head, workspace.data_ptr(), workspace.numel(), stream)
    assert rc == 0, L.fos_error_string(rc)
    torch.cuda.synchronize()
    return codes.cpu().numpy(), sf.cpu().numpy(), float(amax)


def test_static_entry_point_matches_fos_quantize_on_two_calls_in_a_row():
    dev = torch.device("cuda:0")
    L = nat.lib()
    workspace = torch.empty(L.fos_quantize_workspace_bytes(4096, 4096), dtype=torch.uint8, device=dev)
    g = torch.Generator("cpu").manual_seed(11)
    big = torch.randn(4096, 4096, generator=g).bfloat16().to(dev)        # 256 pass-1 partials
    small = (0.01 * torch.randn(384, 1024, generator=g)).bfloat16().to(dev)  # fewer partials, smaller maximum
    tiny = torch.randn(100, 80, generator=g).bfloat16().to(dev)          # ragged, element-wise kernels
    for x, rule, block2d, layout in ((big, MSE, 0, nat.SF_TILED), (small, MSE, 0, nat.SF_TILED),
                                     (big, STATIC_6, 1, nat.SF_TILED), (tiny, MSE, 1, nat.SF_LINEAR)):
        got = _call("static", x, rule, block2d, layout)
        want = _call("plain", x, rule, block2d, layout, workspace)
        assert got[2] == want[2] == float(x.abs().max())
        assert np.array_equal(got[0], want[0]), "codes differ"
        assert np.array_equal(got[1], want[1]), "scales differ"


def test_static_entry_point_leaves_device_memory_alone_and_replays_in_a_graph():
    """What the entry point is for: the free device memory is the same before and after a call (nothing is
    allocated once the first call has looked the scratch array up), and a call recorded into a HIP graph
    -- where an allocation would fail -- gives fos_quantize's bytes on every replay, on new contents."""
    dev = torch.device("cuda:0")
    L = nat.lib()
    g = torch.Generator("cpu").manual_seed(12)
    x = torch.randn(1024, 2048, generator=g).bfloat16().to(dev)  # 4 MiB: two launches (tensor maximum, then codes)
    rows, cols = x.shape
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev)
    sf = torch.empty(rows * cols // 16, dtype=torch.uint8, device=dev)
    amax = torch.empty(1, dtype=torch.float32, device=dev)
    workspace = torch.empty(L.fos_quantize_workspace_bytes(rows, cols), dtype=torch.uint8, device=dev)

    def static_call(stream):
        rc = L.fos_quantize_static(x.data_ptr(), nat.T_BF16, rows, cols, cols, 0, MSE, 0, 0, 0, 0, nat.SF_TILED,
                                   codes.data_ptr(), sf.data_ptr(), amax.data_ptr(), 0, stream)
        assert rc == 0, L.fos_error_string(rc)

    static_call(torch.cuda.current_stream(dev).cuda_stream)  # (looks the scratch array up)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    static_call(torch.cuda.current_stream(dev).cuda_stream)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call(torch.cuda.current_stream(dev).cuda_stream)
    for i in range(2):
        xi = (float(i + 2) * torch.randn(rows, cols, generator=g)).bfloat16().to(dev)
        x.copy_(xi)
        codes.fill_(0xAB)
        sf.fill_(0xCD)
        graph.replay()
        torch.cuda.synchronize()
        want = _call("plain", xi, MSE, 0, nat.SF_TILED, workspace)
        assert float(amax) == want[2] == float(xi.abs().max())
        assert np.array_equal(codes.cpu().numpy(), want[0]), f"replay {i}: codes differ"
        assert np.array_equal(sf.cpu().numpy(), want[1]), f"replay {i}: scales differ"


def test_static_entry_point_argument_checks():
    L = nat.lib()
    dev = torch.device("cuda:0")
    x = torch.zeros(128, 64, dtype=torch.bfloat16, device=dev)
    out = torch.empty(128 * 64, dtype=torch.uint8, device=dev)
    a = torch.empty(1, dtype=torch.float32, device=dev)
    args = [x.data_ptr(), 0, 128, 64, 64, 0, MSE, 0, 0, 0, 0, 1, out.data_ptr(), out.data_ptr(), a.data_ptr(), 0, None]
    bad = list(args); bad[2] = 0
    assert L.fos_quantize_static(*bad) == -1
    bad = list(args); bad[0] = None
    assert L.fos_quantize_static(*bad) == -4
    bad = list(args); bad[5] = 9
    assert L.fos_quantize_static(*bad) == -3
    assert L.fos_quantize_static(*args) == 0
    torch.cuda.synchronize()
    assert float(a) == 0.0
