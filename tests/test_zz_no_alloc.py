"""df11_decode_static_workspace (the entry point for callers that cannot allocate):
its output equals df11_decode's, on two calls in a row that share the library's
static workspace, the second with a smaller stream."""
import ctypes

import numpy as np
import pytest
import torch

from dfloat11_amd import _native
from dfloat11_amd import decode as D
from tests.df11_cases import compress_product, make_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _upload(c):
    g = {k: torch.from_numpy(np.ascontiguousarray(c[k]).view(np.uint8).reshape(-1)).to(DEV)
         for k in ("luts", "encoded_exponent", "sign_mantissa", "gaps", "output_positions")}
    g["luts"] = g["luts"].view(-1, 256)
    return g


def _decode_with_caller_workspace(g, n):
    ws, max_sub = D.prepare(g["luts"], g["encoded_exponent"], g["output_positions"], g["gaps"], n)
    out = torch.full((n,), float("nan"), dtype=torch.bfloat16, device=DEV)
    D.decode(g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"], g["gaps"], out, ws, max_sub)
    torch.cuda.synchronize()
    return out, max_sub


def _decode_static(lib, g, n, out, hint):
    return lib.df11_decode_static_workspace(
        g["luts"].data_ptr(), g["encoded_exponent"].data_ptr(), g["sign_mantissa"].data_ptr(),
        g["output_positions"].data_ptr(), g["gaps"].data_ptr(), out.data_ptr(), g["luts"].shape[0],
        g["encoded_exponent"].numel(), n, hint, torch.cuda.current_stream().cuda_stream)


def test_static_workspace_decode_matches_df11_decode():
    lib = _native.hip_lib()
    # a large stream first, then a smaller one with another code: the second call finds the
    # first call's tables and positions in the shared array
    cases = [("normal", 3_000_001, 11), ("fib", 70_001, 13), ("zeros", 1_200_000, 17), ("uniform256", 9, 19)]
    streams = []
    for kind, n, seed in cases:
        w = make_case(kind, n, seed)
        g = _upload(compress_product(w))
        want, max_sub = _decode_with_caller_workspace(g, n)
        assert np.array_equal(want.view(torch.int16).cpu().numpy().view(np.uint16), w)
        streams.append((kind, n, w, g, want, max_sub))
    outs = [torch.full((n,), float("nan"), dtype=torch.bfloat16, device=DEV) for _, n, *_ in streams]
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    allocated_before = torch.cuda.memory_allocated()
    # back to back on one stream, no synchronisation in between: stream order alone
    # separates one call's use of the shared array from the next call's
    for (kind, n, w, g, want, max_sub), out, hint in zip(streams, outs, (0, 0, -1, 0)):
        print(f"case static workspace kind={kind} n={n} hint={hint}", flush=True)
        assert _decode_static(lib, g, n, out, hint) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == allocated_before
    assert torch.cuda.mem_get_info()[0] == free_before          # nothing was allocated on the device
    for (kind, n, w, g, want, max_sub), out in zip(streams, outs):
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), kind
    # with the exact bound that df11_prepare reports
    for (kind, n, w, g, want, max_sub), out in zip(streams, outs):
        out.fill_(1.0)
        assert _decode_static(lib, g, n, out, max_sub) == 0
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), kind


def test_static_workspace_rejects_streams_beyond_its_capacity():
    lib = _native.hip_lib()
    one = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    p = one.data_ptr()
    too_many = 533385216 + 1        # DF11_STATIC_MAX_STREAM_BYTES + 1: only sizes are looked at before the refusal
    rc = lib.df11_decode_static_workspace(p, p, p, p, p, p, 2, too_many, 10, 0, None)
    assert rc == -4
    assert lib.df11_error_string(rc) == b"buffer too small or fixed capacity exceeded"
    assert lib.df11_decode_static_workspace(p, p, p, p, p, p, 2, 0, 0, 0, None) == 0     # empty stream
    assert lib.df11_decode_static_workspace(None, p, p, p, p, p, 2, 8, 1, 0, None) == -1


def test_static_workspace_decode_in_a_captured_graph():
    """The callers this entry point is for include code under graph capture: captured,
    every replay rebuilds the tables in the library's array and reproduces the eager
    result, also after an eager call for another stream has overwritten that array."""
    lib = _native.hip_lib()
    w = make_case("laplace", 900_001, 23)
    other = make_case("fib", 50_000, 29)
    g, g_other = _upload(compress_product(w)), _upload(compress_product(other))
    out = torch.zeros(w.size, dtype=torch.bfloat16, device=DEV)
    out_other = torch.zeros(other.size, dtype=torch.bfloat16, device=DEV)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        assert _decode_static(lib, g, w.size, out, 0) == 0      # first use outside the capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert _decode_static(lib, g, w.size, out, 0) == 0
    for replay in range(3):
        print(f"case static workspace graph replay {replay}", flush=True)
        out.fill_(1.0)
        assert _decode_static(lib, g_other, other.size, out_other, 0) == 0   # eager, same shared array
        torch.cuda.synchronize()
        assert np.array_equal(out_other.view(torch.int16).cpu().numpy().view(np.uint16), other)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), w)
