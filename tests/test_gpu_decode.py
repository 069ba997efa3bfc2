"""Parity of the HIP decode path (through the C-ABI) with the CPU oracle, on a real MI355X."""
import ctypes
import os
import subprocess

import numpy as np
import pytest
import torch

from dfloat11_amd import decode as D
from tests.df11_cases import (locked_make, KINDS, compress_product, make_case, max_rows_case, random_code_case,
                              short_positions_case)

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def to_gpu(c, pad_front=0):
    """Upload the five stream tensors.  pad_front > 0 shifts every buffer by that many
    bytes from its allocation start to exercise the unaligned paths."""
    def up(a):
        a = np.ascontiguousarray(a)
        t = torch.empty(a.nbytes + pad_front, dtype=torch.uint8, device=DEV)
        t[pad_front:].copy_(torch.from_numpy(a.view(np.uint8).reshape(-1)))
        return t[pad_front:]
    g = {k: up(c[k]) for k in ("luts", "encoded_exponent", "sign_mantissa", "gaps")}
    g["luts"] = g["luts"].view(-1, 256)
    g["output_positions"] = torch.from_numpy(np.ascontiguousarray(c["output_positions"]).view(np.uint8)).to(DEV)
    return g


def gpu_decode(c, max_elems=None, pad_front=0, out=None, plan=None):
    g = to_gpu(c, pad_front)
    n = c["sign_mantissa"].size
    ws, max_sub = D.prepare(g["luts"].contiguous(), g["encoded_exponent"], g["output_positions"],
                            g["gaps"], n)
    if out is None:
        out = torch.full((n,), float("nan"), dtype=torch.bfloat16, device=DEV)
    if max_elems is None:
        max_elems = max_sub
    D.decode(g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"], g["gaps"],
             out, ws, max_elems, plan=plan)
    torch.cuda.synchronize()
    return out.view(torch.int16).cpu().numpy().view(np.uint16)[:n]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("n", [1, 2, 511, 4097, 300_000])
def test_gpu_matches_oracle(oracle, kind, n):
    print(f"case kind={kind} n={n}", flush=True)
    w = make_case(kind, n, 61)
    c = compress_product(w)
    ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                          c["output_positions"], c["gaps"])
    got = gpu_decode(c)
    assert np.array_equal(got, ref)
    assert np.array_equal(got, w)


@pytest.mark.parametrize("plan", [0, 1, 2, 3], ids=["wide", "deep", "deepest", "portable"])
def test_gpu_every_launch_plan_matches_oracle(oracle, plan):
    """The plans differ in resident workgroups and in how many groups of sign|mantissa
    bytes are requested early (`portable` is `wide` with LDS addressed through its symbol,
    the compilation kept for a toolchain on which the constant LDS base of the others does
    not hold); the automatic choice sends small streams to one of them only.  Through df11_decode_with_plan each plan decodes every kind, ragged sizes,
    unaligned buffers and the worst-case staging to the oracle's bits."""
    for kind in KINDS:
        for n in (1, 511, 4097, 70_001, 300_000):
            print(f"case plan={plan} kind={kind} n={n}", flush=True)
            w = make_case(kind, n, 211 + plan)
            c = compress_product(w)
            ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                                  c["output_positions"], c["gaps"])
            assert np.array_equal(gpu_decode(c, plan=plan), ref), (kind, n)
            assert np.array_equal(ref, w)
    w = make_case("laplace", 120_000, 79)
    c = compress_product(w)
    for pad in (1, 4, 7):
        assert np.array_equal(gpu_decode(c, pad_front=pad, plan=plan), w), pad
    buf = torch.zeros(w.size + 16, dtype=torch.bfloat16, device=DEV)
    for shift in (1, 3, 8):
        buf.zero_()
        assert np.array_equal(gpu_decode(c, out=buf[shift:shift + w.size], plan=plan), w)
        whole = buf.view(torch.int16).cpu().numpy()
        assert not whole[:shift].any() and not whole[shift + w.size:].any()
    for kind in ("normal", "zeros", "fib"):
        w = make_case(kind, 200_000, 67)
        assert np.array_equal(gpu_decode(compress_product(w), max_elems=0, plan=plan), w), kind


def test_gpu_random_codes_and_fillings(oracle):
    """Random prefix codes (deep, incomplete, symbols >= 240) with the unowned LUT
    slots filled three ways, and tiny tensors over large alphabets: GPU == original
    words wherever the reference kernel's restatement can decode the LUTs."""
    ran = 0
    for seed in range(2000, 2120):
        made = random_code_case(seed)
        if made is None:
            continue
        w, cases = made
        for policy, c in cases.items():
            try:
                ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                                      c["output_positions"], c["gaps"])
            except RuntimeError:
                continue
            print(f"case random code seed={seed} filling={policy} n={w.size}", flush=True)
            assert np.array_equal(ref, w)
            assert np.array_equal(gpu_decode(c), w), (seed, policy)
            ran += 1
    assert ran > 100
    rng = np.random.default_rng(5)
    for n in (15, 32, 43, 64, 200):
        print(f"case few elements, many symbols n={n}", flush=True)
        syms = np.concatenate([rng.permutation(np.arange(240, 256))[:8], rng.permutation(240)[:190]])
        e = rng.choice(syms, n).astype(np.uint16)
        sm = rng.integers(0, 256, n).astype(np.uint16)
        w = (((sm & 0x80) << 8) | (e << 7) | (sm & 0x7F)).astype(np.uint16)
        assert np.array_equal(gpu_decode(compress_product(w)), w)


@pytest.mark.parametrize("n", [1, 700, 40_000, 2_000_000])
def test_gpu_every_lut_row(oracle, n):
    """A code that fills the layout's 16 sub-tables on all four levels (luts of 18 rows,
    codes of 1 to 32 bits, long codes common) x three fillings of the unowned slots."""
    w, cases = max_rows_case(300 + n, n)
    for policy, c in cases.items():
        print(f"case every LUT row n={n} filling={policy}", flush=True)
        ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                              c["output_positions"], c["gaps"])
        assert np.array_equal(ref, w)
        assert np.array_equal(gpu_decode(c), ref), policy
    # all 17 decode rows together with the staging of the worst case (4096 elements per
    # 512 bytes of bitstream): the largest LDS allocation a launch can ask for
    assert np.array_equal(gpu_decode(cases["product"], max_elems=0), w)


@pytest.mark.parametrize("kind", ["normal", "zeros", "fib"])
def test_gpu_worst_case_staging(kind):
    print(f"case worst-case staging kind={kind}", flush=True)
    w = make_case(kind, 200_000, 67)
    c = compress_product(w)
    assert np.array_equal(gpu_decode(c, max_elems=0), w)


def test_gpu_workspace_matches_host_build():
    """Header, tables and sub-block positions: device build == host build of the same code."""
    print("case workspace", flush=True)
    emul_dir = os.path.join(os.path.dirname(os.path.abspath(__file__)), "emul")
    lib_path = os.path.join(emul_dir, "libdf11_emul.so")
    if not os.path.exists(lib_path):
        locked_make(emul_dir, "libdf11_emul.so")
    L = ctypes.CDLL(lib_path)
    vp = ctypes.c_void_p
    L.df11_emul_prepare.argtypes = [vp, vp, vp, vp, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, vp]
    for kind, n in (("normal", 400_000), ("fib", 400_000), ("uniform256", 100_000), ("high", 9_000),
                    ("zeros", 300_000), ("single", 5)):
        c = compress_product(make_case(kind, n, 71))
        luts = np.ascontiguousarray(c["luts"])
        host = np.zeros(D.workspace_bytes(c["encoded_exponent"].size), np.uint8)
        p = lambda a: a.ctypes.data_as(vp)
        host_max = L.df11_emul_prepare(p(luts), p(c["encoded_exponent"]), p(c["output_positions"]),
                                       p(c["gaps"]), luts.shape[0], c["encoded_exponent"].size, n, p(host))
        g = to_gpu(c)
        dev, dev_max = D.prepare(g["luts"], g["encoded_exponent"], g["output_positions"], g["gaps"], n)
        torch.cuda.synchronize()
        assert dev_max == host_max, kind
        n_blocks = -(-c["encoded_exponent"].size // 4096)
        got = dev.cpu().numpy()
        # header, the two tables and the fused rows that exist (rows past them are never written)
        tables = 64 + 2048 * 8 + 2048 + 512 * (luts.shape[0] - 1)
        assert np.array_equal(got[:tables], host[:tables]), kind
        first = 64 + 2048 * 8 + 2048 + 512 * 17                  # sub-block positions; the rest is padding
        assert np.array_equal(got[first:first + 4 * (8 * n_blocks + 1)], host[first:first + 4 * (8 * n_blocks + 1)]), kind


@pytest.mark.parametrize("pad", [1, 2, 4, 7])
def test_gpu_unaligned_inputs(pad):
    print(f"case unaligned pad={pad}", flush=True)
    w = make_case("normal", 120_000, 73)
    c = compress_product(w)
    assert np.array_equal(gpu_decode(c, pad_front=pad), w)


def test_gpu_unaligned_output():
    print("case unaligned output", flush=True)
    w = make_case("laplace", 120_000, 79)
    c = compress_product(w)
    buf = torch.zeros(w.size + 16, dtype=torch.bfloat16, device=DEV)
    for shift in (1, 3, 8):
        buf.zero_()
        got = gpu_decode(c, out=buf[shift:shift + w.size])
        assert np.array_equal(got, w)
        whole = buf.view(torch.int16).cpu().numpy()
        assert not whole[:shift].any() and not whole[shift + w.size:].any()


def test_gpu_reads_reference_encoder_streams(oracle):
    """Streams laid out by the oracle's restatement of the reference encoder."""
    print("case reference-encoder stream", flush=True)
    w = make_case("outliers", 250_000, 83)
    c = oracle.compress(w)
    n_blocks = -(-c["encoded_exponent"].size // 4096)
    pos = np.full(n_blocks + 1, w.size, np.uint32)
    pos[: c["output_positions"].size] = c["output_positions"]
    c = dict(c, output_positions=pos)
    assert np.array_equal(gpu_decode(c), w)


def test_gpu_reads_positions_one_entry_short(oracle):
    """The reference encoder leaves output_positions one entry short when the last code
    crosses a block boundary and ends on a byte boundary (dfloat11_utils.py:146-162):
    n_blocks entries, the last being the element count.  The array goes to the device
    exactly as the reference would have saved it, unpadded."""
    print("case positions one short", flush=True)
    from oracle.df11_oracle import EOF
    table = {1: (8, 0b10000000), 2: (16, 0b0000000000000001), EOF: (16, 0)}
    data = np.array([1] * 4095 + [2], np.uint8)
    enc, gaps, pos = oracle.c_encode(data, table)
    luts = np.zeros((3, 256), np.uint8)
    luts[0, :] = 1
    luts[0, 0] = 255
    luts[1, :] = 2
    luts[2, 1], luts[2, 2] = 8, 16
    sm = (np.arange(data.size) % 251).astype(np.uint8)
    assert pos.size == 2 and -(-enc.size // 4096) == 2 and int(pos[-1]) == data.size
    c = dict(luts=luts, encoded_exponent=enc, sign_mantissa=sm, output_positions=pos, gaps=gaps)
    g = to_gpu(c)
    assert g["output_positions"].numel() == 4 * 2          # n_blocks entries, not n_blocks + 1
    D.validate_stream(g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"], g["gaps"])
    want = oracle.merge_bf16(data, sm)
    assert np.array_equal(gpu_decode(c), want)
    # multi-block streams with realistic code lengths whose positions are one short
    for seed, n_full in ((1, 1), (2, 3), (3, 9)):
        print(f"case positions one short, {n_full + 1} blocks", flush=True)
        w, c = short_positions_case(oracle, seed, n_full)
        ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
        assert np.array_equal(ref, w)
        got = gpu_decode(c)
        assert np.array_equal(got, w)


def test_gpu_does_not_write_outside_output():
    print("case guard bands", flush=True)
    w = make_case("normal", 77_777, 89)
    c = compress_product(w)
    guard = 4096
    buf = torch.full((w.size + 2 * guard,), 1.0, dtype=torch.bfloat16, device=DEV)
    got = gpu_decode(c, out=buf[guard:guard + w.size])
    assert np.array_equal(got, w)
    whole = buf.view(torch.int16).cpu().numpy()
    assert (whole[:guard] == 0x3F80).all() and (whole[guard + w.size:] == 0x3F80).all()


def test_gpu_side_stream_and_repeat():
    print("case side stream", flush=True)
    w1 = make_case("normal", 500_000, 97)
    w2 = make_case("laplace", 300_000, 101)
    c1, c2 = compress_product(w1), compress_product(w2)
    g1, g2 = to_gpu(c1), to_gpu(c2)
    (t1, m1), (t2, m2) = (D.prepare(g["luts"], g["encoded_exponent"], g["output_positions"], g["gaps"], w.size)
                          for g, w in ((g1, w1), (g2, w2)))
    out = torch.empty(max(w1.size, w2.size), dtype=torch.bfloat16, device=DEV)
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        for _ in range(3):   # same output buffer reused, stream order is the only guard
            D.decode(g1["luts"], g1["encoded_exponent"], g1["sign_mantissa"], g1["output_positions"],
                     g1["gaps"], out, t1, m1)
            a = out[: w1.size].clone()
            D.decode(g2["luts"], g2["encoded_exponent"], g2["sign_mantissa"], g2["output_positions"],
                     g2["gaps"], out, t2, m2)
            b = out[: w2.size].clone()
    s.synchronize()
    assert np.array_equal(a.view(torch.int16).cpu().numpy().view(np.uint16), w1)
    assert np.array_equal(b.view(torch.int16).cpu().numpy().view(np.uint16), w2)


def test_gpu_host_threads_decode_at_once():
    """The library keeps no launch state between calls: host threads that prepare and decode
    streams of their own at the same time, each on a stream of its own, all get their words."""
    import threading
    print("case host threads", flush=True)
    specs = [("normal", 400_003, 5), ("zeros", 250_000, 6), ("uniform256", 120_001, 7), ("sparse", 300_000, 8)]
    cases = [(make_case(kind, n, seed), kind) for kind, n, seed in specs]
    packed = [(w, to_gpu(compress_product(w))) for w, _ in cases]
    torch.cuda.synchronize()
    results, errors = [None] * len(packed), []

    def work(i):
        try:
            torch.cuda.set_device(0)
            w, g = packed[i]
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                good = True
                for _ in range(8):
                    ws, max_sub = D.prepare(g["luts"].contiguous(), g["encoded_exponent"], g["output_positions"],
                                            g["gaps"], w.size)
                    out = torch.full((w.size,), float("nan"), dtype=torch.bfloat16, device=DEV)
                    D.decode(g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"],
                             g["gaps"], out, ws, max_sub)
                    s.synchronize()
                    good = good and np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), w)
            results[i] = good
        except Exception as e:   # reported by the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(packed))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(100)
    assert not errors, errors
    assert results == [True] * len(packed), results


def test_gpu_decode_in_a_captured_graph():
    """df11_decode allocates nothing and never synchronises, so it can be captured into
    a HIP graph; every replay (with eager work and synchronisation between replays)
    reproduces the eager result."""
    print("case graph capture", flush=True)
    w = make_case("outliers", 400_000, 131)
    c = compress_product(w)
    g = to_gpu(c)
    ws, max_sub = D.prepare(g["luts"], g["encoded_exponent"], g["output_positions"], g["gaps"], w.size)
    out = torch.zeros(w.size, dtype=torch.bfloat16, device=DEV)
    args = (g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"], g["gaps"], out, ws, max_sub)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        D.decode(*args)                      # warm-up outside the capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        D.decode(*args)
    for _ in range(4):
        out.fill_(1.0)                       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), w)


def test_gpu_row_decode_in_a_captured_graph():
    """df11_decode_rows reads the row numbers from device memory when it runs, so a graph
    that captured one launch decodes whatever rows the caller has written into that buffer
    by the time of each replay (also more rows than workgroups, where every wavefront takes
    ids of its own)."""
    print("case graph capture rows", flush=True)
    n_rows, row_elements = 6000, 160
    w = make_case("normal", n_rows * row_elements, 133)
    c = compress_product(w)
    g = to_gpu(c)
    ws, max_sub = D.prepare(g["luts"], g["encoded_exponent"], g["output_positions"], g["gaps"], w.size)
    sentinel = 0x7F81                        # a NaN pattern no stream of these kinds holds
    out = torch.full((w.size,), sentinel, dtype=torch.int16, device=DEV).view(torch.bfloat16)
    ids = torch.zeros(3000, dtype=torch.int64, device=DEV)
    bound = D.bind(g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"], g["gaps"],
                   out, ws, max_sub)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        D.launch_rows(bound, torch.device(DEV), ids, row_elements)   # warm-up outside the capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        D.launch_rows(bound, torch.device(DEV), ids, row_elements)
    rng = np.random.default_rng(5)
    matrix = w.reshape(n_rows, row_elements)
    for replay in range(4):
        chosen = rng.integers(0, n_rows, ids.numel())
        if replay == 3:
            chosen[:] = chosen[0]            # one row, asked for 3000 times
        out.view(torch.int16).fill_(sentinel)                        # eager work between the replays
        ids.copy_(torch.from_numpy(chosen))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.view(torch.int16).cpu().numpy().view(np.uint16).reshape(n_rows, row_elements)
        assert np.array_equal(got[chosen], matrix[chosen]), replay
        written = got != sentinel
        assert np.array_equal(got[written], matrix[written]), replay
        if replay == 3:
            assert written.sum() < 3 * 4096 + row_elements, replay    # the row and its sub-blocks' neighbours only


def test_gpu_full_size_linear_round_trip():
    """4096x4096 N(0, 0.02): encode -> decode is the identity (size-independent property)."""
    print("case 4096x4096", flush=True)
    g = torch.Generator(device="cpu").manual_seed(0)
    w = (torch.randn(4096, 4096, generator=g) * 0.02).to(torch.bfloat16)
    wu = w.view(torch.int16).numpy().view(np.uint16).reshape(-1)
    c = compress_product(wu)
    assert c["sign_mantissa"].size == 16_777_216
    got = gpu_decode(c)
    assert np.array_equal(got, wu)


def test_gpu_llama_block_round_trip():
    """Llama-3-8B-shaped decoder block compressed as one stream: 218 103 808 elements."""
    print("case llama block", flush=True)
    shapes = [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]
    parts = []
    for i, (r, cdim) in enumerate(shapes):
        g = torch.Generator(device=DEV).manual_seed(1000 + i)
        parts.append((torch.randn(r * cdim, generator=g, device=DEV) * 0.02).to(torch.bfloat16))
    w = torch.cat(parts)
    assert w.numel() == 218_103_808
    wu = w.view(torch.int16).cpu().numpy().view(np.uint16)
    c = compress_product(wu)
    g = to_gpu(c)
    ws, max_sub = D.prepare(g["luts"], g["encoded_exponent"], g["output_positions"], g["gaps"], w.numel())
    out = torch.empty_like(w)
    D.decode(g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"], g["gaps"],
             out, ws, max_sub)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), w.view(torch.int16))


@pytest.mark.parametrize("rows,cols", [(151936, 4096), (4096, 14336)])
@pytest.mark.parametrize("kind", ["laplace", "outliers", "uniform256", "zeros", "sparse70", "alphabet100"])
def test_gpu_embedding_sized_adversarial_round_trip(kind, rows, cols):
    """151936 x 4096 (622 329 856 elements, the largest tensor of the Qwen3-8B shape) and
    4096 x 14336 with an adversarial exponent mix (the last two: chunks of thirty and more
    codes, and of nine to eleven table lookups): encode -> decode is the identity."""
    print(f"case {rows}x{cols} {kind}", flush=True)
    import bench_extra
    w = bench_extra.make_mix(torch, kind, rows * cols, torch.device(DEV), seed=23)
    from dfloat11_amd import dfloat11_utils as U
    w_cpu = w.cpu()
    _, counter = U.get_codec(w_cpu)
    codec, _, table = U.get_32bit_codec(counter)
    luts = U.get_luts(table)
    enc, sm, pos, gaps, _ = U.encode_weights([w_cpu], codec)
    del w_cpu
    d = [t.to(DEV) for t in (luts, enc, sm, pos.view(torch.uint8), gaps)]
    ws, max_sub = D.prepare(d[0], d[1], d[3], d[4], w.numel())
    out = torch.empty_like(w)
    D.decode(d[0], d[1], d[2], d[3], d[4], out, ws, max_sub)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), w.view(torch.int16))


def test_gpu_more_than_2_31_elements():
    """2^31 + 12345 elements in one stream: the reference's kernel indexes with a 32-bit
    int and stops short of 2^31; here element indices are unsigned 32-bit and byte
    offsets 64-bit."""
    print("case above 2^31 elements", flush=True)
    import bench_extra
    from dfloat11_amd import dfloat11_utils as U
    n = (1 << 31) + 12345
    w = bench_extra.make_mix(torch, "zeros", n, torch.device(DEV), seed=29)
    w[-5:] = torch.tensor([1.5, -2.0, 0.007, 3e-5, -0.0], dtype=torch.bfloat16, device=DEV)
    w[n // 2] = 1234.0
    w_cpu = w.cpu()
    _, counter = U.get_codec(w_cpu)
    codec, _, table = U.get_32bit_codec(counter)
    luts = U.get_luts(table)
    enc, sm, pos, gaps, _ = U.encode_weights([w_cpu], codec)
    del w_cpu
    assert int(pos.view(torch.int32)[-1].item()) & 0xFFFFFFFF == n
    d = [t.to(DEV) for t in (luts, enc, sm, pos.view(torch.uint8), gaps)]
    D.validate_stream(d[0], d[1], d[2], d[3], d[4])
    ws, max_sub = D.prepare(d[0], d[1], d[3], d[4], n)
    out = torch.empty_like(w)
    D.decode(d[0], d[1], d[2], d[3], d[4], out, ws, max_sub)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), w.view(torch.int16))


@pytest.mark.parametrize("n", [1, 4097, 3_000_001])
def test_gpu_plain_c_caller_round_trip(n):
    """The C program of tests/abi: host codec + GPU decode through the C-ABI alone."""
    print(f"case plain C caller n={n}", flush=True)
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi", "abi_roundtrip")
    if not os.path.exists(exe):
        locked_make(os.path.dirname(exe))
    res = subprocess.run([exe, str(n)], capture_output=True, text=True, timeout=100)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "mismatches 0" in res.stdout


@pytest.mark.parametrize("kind,n_rows,row_elements", [("normal", 3000, 512), ("normal", 200, 4096), ("zeros", 4000, 256),
                                                     ("uniform256", 1500, 320), ("fib", 5000, 64),
                                                     ("laplace", 7, 100_003), ("outliers", 100_000, 3)])
def test_gpu_rows_match_full_decode(oracle, kind, n_rows, row_elements):
    """df11_decode_rows writes the requested rows exactly as df11_decode (and the oracle)
    does, writes nothing but correct values anywhere else, and leaves elements that are far
    from every requested row alone.  Row numbers repeat, come unsorted, include the first
    and the last row and numbers outside the matrix; they are fewer and more than the
    workgroups of a launch (the kernel hands them out differently)."""
    n = n_rows * row_elements
    print(f"case rows kind={kind} rows={n_rows} row_elements={row_elements}", flush=True)
    w = make_case(kind, n, 91)
    c = compress_product(w)
    ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
    assert np.array_equal(ref, w)
    g = to_gpu(c)
    ws, max_sub = D.prepare(g["luts"].contiguous(), g["encoded_exponent"], g["output_positions"], g["gaps"], n)
    rng = np.random.default_rng(17)
    for n_ids in (1, 5, 64, 2000):           # the last: more ids than workgroups, a wavefront per id
        ids = rng.integers(0, n_rows, n_ids)
        ids[0] = n_rows - 1
        if n_ids > 2:
            ids[1], ids[2] = 0, ids[0]
        asked = np.concatenate([ids, [-1, n_rows, n_rows + 5, 2 ** 40]]) if n_ids > 1 else ids
        rng.shuffle(asked)
        sentinel = 0xEEEE
        out = torch.full((n,), sentinel - 65536, dtype=torch.int16, device=DEV).view(torch.bfloat16)
        D.decode_rows(g["luts"], g["encoded_exponent"], g["sign_mantissa"], g["output_positions"], g["gaps"],
                      out, ws, max_sub, torch.from_numpy(asked.astype(np.int64)).to(DEV), row_elements)
        torch.cuda.synchronize()
        got = out.view(torch.int16).cpu().numpy().view(np.uint16)
        wanted = np.zeros(n, bool)
        for i in ids:
            wanted[i * row_elements:(i + 1) * row_elements] = True
        assert np.array_equal(got[wanted], w[wanted]), (kind, n_ids)
        written = got != sentinel
        assert np.array_equal(got[written], w[written]), (kind, n_ids)       # whatever else was written is right too
        # a sub-block holds at most 4096 elements: nothing further than that from a requested row is touched
        near = np.zeros(n + 1, np.int64)
        for i in ids:
            near[max(0, i * row_elements - 4096)] += 1
            near[min(n, (i + 1) * row_elements + 4096)] -= 1
        far = np.cumsum(near[:-1]) == 0
        assert not (written & far & (w != sentinel)).any(), (kind, n_ids)


@pytest.mark.parametrize("kind", ["normal", "laplace", "outliers"])
def test_gpu_stream_of_one_round_of_four_workgroups_per_cu(oracle, kind):
    """Streams of 10 M to 12.9 M weight-like elements run the compilation of the wide plan
    that keeps four workgroups per CU resident; the library says so without a GPU, and the
    decode equals the oracle's and the original words."""
    from dfloat11_amd import _native
    n = 11_000_003
    print(f"case wide/full kind={kind} n={n}", flush=True)
    w = make_case(kind, n, 23)
    c = compress_product(w)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    name = _native.hip_lib().df11_launch_plan_name(c["encoded_exponent"].size, n, cus).decode()
    if cus == 256:
        assert name == "wide/full", name
    ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
    assert np.array_equal(ref, w)
    assert np.array_equal(gpu_decode(c), ref)
    assert np.array_equal(gpu_decode(c, max_elems=0, pad_front=4), ref)
