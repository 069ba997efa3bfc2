"""Pins the CPU oracle itself.  The reference holds no golden vectors for this
path, so each oracle function is checked against hand-worked cases derived
from the reference source by hand, closed forms, brute force and invariants."""
import heapq

import numpy as np
import pytest

from oracle.df11_oracle import EOF


# ---------------------------------------------------------------- split / merge
def test_split_merge_exhaustive(oracle):
    w = np.arange(65536, dtype=np.uint16)
    e, s = oracle.split_bf16(w)
    # closed form straight from the BF16 layout: sign(1) exponent(8) mantissa(7)
    assert np.array_equal(e, ((w >> 7) & 0xFF).astype(np.uint8))
    assert np.array_equal(s, (((w >> 15) << 7) | (w & 0x7F)).astype(np.uint8))
    ce, cs = oracle.c_split(w)
    assert np.array_equal(ce, e) and np.array_equal(cs, s)
    assert np.array_equal(oracle.merge_bf16(e, s), w)
    assert np.array_equal(oracle.c_merge(e, s), w)


def test_split_known_values(oracle):
    # 1.0 = 0x3F80, -2.0 = 0xC000, +inf = 0x7F80, smallest subnormal = 0x0001
    w = np.array([0x3F80, 0xC000, 0x7F80, 0x0001], dtype=np.uint16)
    e, s = oracle.split_bf16(w)
    assert e.tolist() == [127, 128, 255, 0]
    assert s.tolist() == [0x00, 0x80, 0x00, 0x01]


# ---------------------------------------------------------------- Huffman
def _textbook_cost(freqs):
    """Sum of merged weights == sum(f * len) for any optimal prefix code."""
    h = list(freqs)
    heapq.heapify(h)
    cost = 0
    while len(h) > 1:
        m = heapq.heappop(h) + heapq.heappop(h)
        cost += m
        heapq.heappush(h, m)
    return cost


def _assert_prefix_free(table):
    codes = sorted(format(v, "b").rjust(l, "0") for (l, v) in table.values())
    for a, b in zip(codes, codes[1:]):
        assert not b.startswith(a), (a, b)


@pytest.mark.parametrize("seed", range(6))
def test_huffman_optimal_and_complete(oracle, seed):
    rng = np.random.default_rng(seed)
    n_sym = int(rng.integers(1, 60))
    syms = rng.choice(256, n_sym, replace=False)
    freqs = {int(s): int(f) for s, f in zip(syms, rng.integers(1, 10 ** int(rng.integers(1, 7)), n_sym))}
    table = oracle.huffman_from_frequencies(freqs)
    assert set(table) == set(freqs) | {EOF}
    _assert_prefix_free(table)
    kraft = sum(2.0 ** -l for (l, _) in table.values())
    assert kraft == 1.0
    cost = sum(freqs[k] * l for k, (l, _) in table.items() if k is not EOF) + table[EOF][0]
    assert cost == _textbook_cost(list(freqs.values()) + [1])


def test_huffman_hand_worked(oracle):
    # weights 10, 3 and the implicit end-of-stream leaf of weight 1:
    # first merge: EOF(1) gets bit 0, symbol 7 (3) gets bit 1 -> node of weight 4
    # second merge: that node (4) gets bit 0, symbol 5 (10) gets bit 1.
    table = oracle.huffman_from_frequencies({5: 10, 7: 3})
    assert table[EOF] == (2, 0b00)
    assert table[7] == (2, 0b01)
    assert table[5] == (1, 0b1)
    assert list(table) == [EOF, 7, 5]          # left-to-right leaf order


def test_single_symbol_gets_one_bit(oracle):
    table = oracle.huffman_from_frequencies({42: 1000})
    assert table[42][0] == 1 and table[EOF][0] == 1


def test_32bit_limit(oracle):
    # Fibonacci weights make a maximally skewed tree: 40 symbols -> 40-bit codes.
    fib = [1, 1]
    while len(fib) < 40:
        fib.append(fib[-1] + fib[-2])
    counter = {i: f for i, f in enumerate(fib)}
    assert max(l for l, _ in oracle.huffman_from_frequencies(counter).values()) > 32
    _, table = oracle.get_32bit_codec(counter)
    assert max(l for l, _ in table.values()) <= 32
    _assert_prefix_free(table)
    assert sum(2.0 ** -l for (l, _) in table.values()) == 1.0


# ---------------------------------------------------------------- LUTs
CHAIN = {  # unary-style chain reaching a second LUT level; EOF shares the deepest node
    10: (1, 0b1), 20: (2, 0b01), 30: (3, 0b001), 40: (4, 0b0001), 50: (5, 0b00001),
    60: (6, 0b000001), 70: (7, 0b0000001), 80: (8, 0b00000001),
    90: (9, 0b000000001), EOF: (9, 0b000000000),
}


def test_luts_hand_worked_one_level(oracle):
    table = {5: (1, 0b0), 7: (2, 0b10), EOF: (2, 0b11)}
    luts = oracle.get_luts(table)
    assert luts.shape == (2, 256)
    # '0xxxxxxx' -> 5 ; '10xxxxxx' -> 7 ; '11xxxxxx' (EOF) inherits 7 by forward fill
    assert luts[0].tolist() == [5] * 128 + [7] * 128
    lens = [0] * 256
    lens[5], lens[7] = 1, 2
    assert luts[1].tolist() == lens


def test_luts_hand_worked_two_levels(oracle):
    luts = oracle.get_luts(CHAIN)
    assert luts.shape == (3, 256)
    root = [255, 80] + [70] * 2 + [60] * 4 + [50] * 8 + [40] * 16 + [30] * 32 + [20] * 64 + [10] * 128
    assert luts[0].tolist() == root            # index 0 -> pointer to row 1 (256 - 1)
    # row 1: '1xxxxxxx' -> 90; '0xxxxxxx' is EOF's slot and inherits the last
    # value written to the previous row (10) through the leaked fill variable.
    assert luts[1].tolist() == [10] * 128 + [90] * 128
    assert luts[2, 90] == 9 and luts[2, 80] == 8 and luts[2, 10] == 1 and luts[2, 0] == 0


def _walk(luts, window):
    """decode.cu:105-113 on a 64-bit window, in Python."""
    d = int(luts[0, window >> 56])
    for level in (1, 2, 3):
        if d < 240:
            break
        d = int(luts[256 - d, (window >> (56 - 8 * level)) & 0xFF])
    return d


@pytest.mark.parametrize("seed", range(5))
def test_luts_brute_force(oracle, seed):
    rng = np.random.default_rng(100 + seed)
    if seed == 0:   # deep tree: geometric weights push codes past 24 bits
        freqs = {int(s): 3 ** i for i, s in enumerate(rng.choice(240, 30, replace=False))}
    else:
        n_sym = int(rng.integers(2, 200))
        freqs = {int(s): int(f) for s, f in
                 zip(rng.choice(240, n_sym, replace=False), rng.integers(1, 1 << 20, n_sym))}
    _, table = oracle.get_32bit_codec(freqs)
    luts = oracle.get_luts(table)
    n_rows = luts.shape[0] - 1
    assert n_rows - 1 <= 16
    for sym, (l, v) in table.items():
        if sym is EOF:
            continue
        assert luts[-1, sym] == l
        for pad in (0, (1 << (64 - l)) - 1, int(rng.integers(0, 1 << 62)) & ((1 << (64 - l)) - 1)):
            assert _walk(luts, (v << (64 - l)) | pad) == sym
    if seed == 0:
        assert max(l for l, _ in table.values()) > 24     # all four levels in use


# ---------------------------------------------------------------- bit packer
def test_encode_hand_packed(oracle):
    # 10,20,10,90 -> 1 01 1 000000001 = 1011 0000 | 00001 + EOF 000000000 -> 0000 1000
    data = [10, 20, 10, 90]
    for enc_fn in (oracle.encode, oracle.c_encode):
        enc, gaps, pos = enc_fn(np.array(data, np.uint8), CHAIN)
        assert enc.tolist() == [0xB0, 0x08]
        assert pos.tolist() == [0, 4]
        assert gaps.tolist() == [0] * 320


def test_encode_gap_hand_packed(oracle):
    # seven 8-bit codes (56 bits), one 9-bit code ends at bit 65: the first code
    # starting in the second 8-byte chunk starts at bit offset 1.
    data = [80] * 7 + [90] + [10] * 3
    for enc_fn in (oracle.encode, oracle.c_encode):
        enc, gaps, pos = enc_fn(np.array(data, np.uint8), CHAIN)
        assert enc[:8].tolist() == [1] * 7 + [0]
        # bit 64 = last bit of the 9-bit code (1), bits 65..67 = three 1-bit codes,
        # then EOF (nine zeros) fills the byte: 1111 0000
        assert enc[8:].tolist() == [0xF0]
        # 5-bit fields: 00000 00001 -> bit 9 set -> byte 1 = 0100 0000
        assert gaps[:3].tolist() == [0x00, 0x40, 0x00]
        assert not gaps[3:].any() and gaps.size == 320
        assert pos.tolist() == [0, 11]


def test_encode_block_positions(oracle):
    n = 4096 + 10                        # 8-bit codes: one element per byte
    data = np.full(n, 80, np.uint8)
    enc, gaps, pos = oracle.c_encode(data, CHAIN)
    assert enc.size == n and pos.tolist() == [0, 4096, n]
    assert gaps.size == 640 and not gaps.any()


def test_encode_positions_one_short_quirk(oracle):
    # last code starts in block 0, crosses into block 1 and ends byte aligned:
    # the reference emits no entry for block 1 (dfloat11_utils.py:146-162).
    table = {1: (8, 0b10000000), 2: (16, 0b0000000000000001), EOF: (16, 0)}
    data = np.array([1] * 4095 + [2], np.uint8)
    for enc_fn in (oracle.encode, oracle.c_encode):
        enc, gaps, pos = enc_fn(data, table)
        assert enc.size == 4097
        assert pos.tolist() == [0, 4096]
        assert gaps.size == 640


@pytest.mark.parametrize("seed", range(4))
def test_encode_c_matches_python(oracle, seed):
    rng = np.random.default_rng(200 + seed)
    p = rng.dirichlet(np.ones(20) * 0.3)
    syms = rng.choice(240, 20, replace=False)
    data = rng.choice(syms, size=int(rng.integers(3000, 30000)), p=p).astype(np.uint8)
    _, table = oracle.get_32bit_codec(oracle.get_counter(data))
    a = oracle.encode(data, table)
    b = oracle.c_encode(data, table)
    for x, y in zip(a, b):
        assert x.dtype == y.dtype and np.array_equal(x, y)


def _code_starts(data, table):
    lens = np.array([table[int(s)][0] for s in data], dtype=np.int64)
    return np.concatenate(([0], np.cumsum(lens)))[:-1], int(lens.sum())


@pytest.mark.parametrize("seed", range(3))
def test_gaps_and_positions_definitions(oracle, seed):
    rng = np.random.default_rng(300 + seed)
    syms = rng.choice(240, 12, replace=False)
    data = rng.choice(syms, size=60000, p=rng.dirichlet(np.ones(12))).astype(np.uint8)
    _, table = oracle.get_32bit_codec(oracle.get_counter(data))
    enc, gaps, pos = oracle.c_encode(data, table)
    starts, total_bits = _code_starts(data, table)
    assert enc.size == -(-total_bits // 8)
    n_blocks = -(-enc.size // 4096)
    gap_vals = np.packbits(np.unpackbits(gaps).reshape(-1, 5), axis=1, bitorder="big")[:, 0] >> 3
    assert gap_vals.size == 512 * n_blocks
    chunk_of = starts // 64
    first_in_chunk = np.searchsorted(chunk_of, np.arange(chunk_of.max() + 1))
    assert np.array_equal(gap_vals[: chunk_of.max() + 1], (starts[first_in_chunk] % 64))
    assert gap_vals.max() <= 31
    block_of = starts // 32768
    first_in_block = np.searchsorted(block_of, np.arange(block_of.max() + 1))
    assert pos[:-1].tolist() == first_in_block.tolist() and pos[-1] == data.size


# ---------------------------------------------------------------- decoder
@pytest.mark.parametrize("seed", range(4))
def test_decode_identity_and_sequential(oracle, seed):
    rng = np.random.default_rng(400 + seed)
    n = int(rng.integers(1, 200000))
    w = (rng.standard_normal(n) * 0.02).astype(np.float32).view(np.uint32) >> 16
    w = w.astype(np.uint16)
    c = oracle.compress(w)
    out = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                          c["output_positions"], c["gaps"])
    assert np.array_equal(out, w)
    seq = oracle.c_decode_sequential(c["table"], c["encoded_exponent"], c["sign_mantissa"])
    assert np.array_equal(seq, w)


def test_decode_hand_packed(oracle):
    # stream from test_encode_gap_hand_packed, sign/mantissa chosen by hand
    data = np.array([80] * 7 + [90] + [10] * 3, np.uint8)
    sm = np.arange(11, dtype=np.uint8) * 23
    luts = oracle.get_luts(CHAIN)
    enc, gaps, pos = oracle.c_encode(data, CHAIN)
    out = oracle.c_decode(luts, enc, sm, pos, gaps)
    expect = [((int(s) & 0x80) << 8) | (int(e) << 7) | (int(s) & 0x7F) for e, s in zip(data, sm)]
    assert out.tolist() == expect


def test_decode_survives_short_positions(oracle):
    table = {1: (8, 0b10000000), 2: (16, 0b0000000000000001), EOF: (16, 0)}
    data = np.array([1] * 4095 + [2], np.uint8)
    enc, gaps, pos = oracle.c_encode(data, table)
    # LUTs by hand: root '10000000' -> 1, '00000000' -> row 1; row 1 '00000001' -> 2
    luts = np.zeros((3, 256), np.uint8)
    luts[0, :] = 1
    luts[0, 0] = 255
    luts[1, :] = 2
    luts[2, 1], luts[2, 2] = 8, 16
    sm = np.zeros(data.size, np.uint8)
    out = oracle.c_decode(luts, enc, sm, pos, gaps)
    assert np.array_equal(out, oracle.merge_bf16(data, sm))


def test_decode_block_range(oracle):
    rng = np.random.default_rng(7)
    w = ((rng.standard_normal(100000) * 0.02).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    c = oracle.compress(w)
    n_blocks = -(-c["encoded_exponent"].size // 4096)
    assert n_blocks >= 3
    out = np.zeros(w.size, np.uint16)
    for b in range(n_blocks):
        oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                        c["output_positions"], c["gaps"], block_range=(b, b + 1), out=out)
    assert np.array_equal(out, w)


def test_config_1_full_size_linear_through_the_cpu_path(oracle):
    """BASELINE configuration 1 at its stated size: a 4096x4096 BF16 weight, N(0, 0.02)
    from seed 0, compressed by the product encoder (8 bytes per thread, 512 threads per
    block) and decoded by the CPU restatement of the reference kernel: bit-exact."""
    import torch
    from dfloat11_amd import dfloat11_utils as U
    g = torch.Generator(device="cpu").manual_seed(0)
    w = (torch.randn(4096, 4096, generator=g) * 0.02).to(torch.bfloat16).flatten()
    codec, _ = U.get_codec(w)
    luts = U.get_luts(codec.get_code_table())
    enc, sm, pos, gaps, split = U.encode_weights([w], codec, 8, 512)
    assert sm.numel() == 16_777_216 and split.numel() == 0
    n_blocks = -(-enc.numel() // 4096)
    assert 1300 < n_blocks < 1360 and pos.numel() == n_blocks + 1 and gaps.numel() == 320 * n_blocks
    ratio = (enc.numel() + sm.numel() + gaps.numel() + 4 * pos.numel()) / (2 * sm.numel())
    assert 0.66 < ratio < 0.69
    got = oracle.c_decode(luts.numpy(), enc.numpy(), sm.numpy(), pos.numpy(), gaps.numpy())
    assert np.array_equal(got, w.view(torch.int16).numpy().view(np.uint16))
