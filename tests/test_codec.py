"""Product host codec (libdf11_codec.so) against the oracle's restatement of the reference codec."""
import numpy as np
import pytest

from dfloat11_amd import dfloat11_utils as U
from oracle.df11_oracle import EOF
from tests.df11_cases import locked_make, KINDS, compress_product, make_case


def _oracle_table(codec):
    """The product's code as an oracle-style table, in code-word order."""
    t = codec.get_code_table()
    return {(EOF if not isinstance(k, int) else k): v for k, v in t.items()}


def test_split_exhaustive(oracle):
    w = np.arange(65536, dtype=np.uint16)
    import torch
    e, s = U.split_bf16(torch.from_numpy(w.view(np.int16)).view(torch.bfloat16))
    oe, os_ = oracle.split_bf16(w)
    assert np.array_equal(e, oe) and np.array_equal(s, os_)


@pytest.mark.parametrize("kind", ["normal", "laplace", "outliers", "zeros", "single"])
def test_code_is_optimal_like_the_reference(oracle, kind):
    """No layout limit bites on these mixes, so the product code must cost exactly
    what the reference's Huffman code costs.  Cost counts the end-of-stream leaf
    (weight 1) too: only the total is independent of tie-breaks."""
    w = make_case(kind, 200_000, 11)
    c = compress_product(w)
    counter = oracle.get_counter(oracle.split_bf16(w)[0])
    assert dict(counter) == c["counter"]
    _, ref_table = oracle.get_32bit_codec(counter)
    ref_bits = sum(counter[k] * l for k, (l, _) in ref_table.items() if k is not EOF)
    got_bits = sum(counter[k] * int(c["codec"].code_len[k]) for k in counter)
    assert got_bits + c["codec"].eof_len == ref_bits + ref_table[EOF][0]
    assert c["encoded_exponent"].size == -(-got_bits // 8)
    assert abs(got_bits - ref_bits) <= 32


@pytest.mark.parametrize("kind", KINDS)
def test_code_properties(kind):
    w = make_case(kind, 100_000, 5)
    c = compress_product(w)
    codec = c["codec"]
    lens = codec.code_len.astype(int)
    present = sorted(c["counter"])
    assert all(lens[s] > 0 for s in present)
    assert lens.max() <= 32 and codec.eof_len <= 32
    codes = sorted(format(int(codec.code_val[s]), "b").rjust(lens[s], "0") for s in present)
    codes.append(format(codec.eof_val, "b").rjust(codec.eof_len, "0"))
    codes.sort()
    for a, b in zip(codes, codes[1:]):
        assert not b.startswith(a)
    kraft = sum(2.0 ** -len(x) for x in codes)
    assert kraft <= 1.0
    # symbols the reference decoder would misread as pointers sit on the fourth level only
    assert all(lens[s] >= 25 for s in present if s >= 240)
    assert c["luts"].shape[0] - 2 <= 16


def _assert_luts_equal_up_to_eof_fill(ref, got, table):
    """Rows, pointers, symbol entries and lengths must be identical.  The only
    licence: the slots of the end-of-stream code, which no valid stream ever
    decodes.  The reference fills them with whatever entry came before, even a
    pointer (which its kernel would then chase); the product always fills them
    with a real symbol so that padding bits can never stall a decoder."""
    assert got.shape == ref.shape
    assert np.array_equal(got[-1], ref[-1])
    diff = np.argwhere(ref != got)
    if diff.size == 0:
        return
    l, v = table[EOF]
    rem = l - 8 * ((l - 1) // 8)
    lo = (v & ((1 << rem) - 1)) << (8 - rem)
    rows = set(diff[:, 0].tolist())
    assert len(rows) == 1
    assert sorted(diff[:, 1].tolist()) == list(range(lo, lo + (1 << (8 - rem))))
    assert all(ref[r, i] >= 240 for r, i in diff)          # an inherited pointer
    assert all(got[-1, got[r, i]] > 0 for r, i in diff)     # a real symbol instead


@pytest.mark.parametrize("kind", ["normal", "outliers", "fib", "zeros"])
def test_luts_match_reference_layout(oracle, kind):
    """Same code table in, same LUT bytes out as the reference's get_luts."""
    w = make_case(kind, 150_000, 3)
    c = compress_product(w)
    table = _oracle_table(c["codec"])
    _assert_luts_equal_up_to_eof_fill(oracle.get_luts(table), c["luts"], table)


@pytest.mark.parametrize("seed", range(6))
def test_luts_match_reference_on_reference_tables(oracle, seed):
    """...and for the reference's own (dahuffman-ordered) tables."""
    rng = np.random.default_rng(seed)
    n_sym = int(rng.integers(2, 120))
    freqs = {int(s): int(f) for s, f in zip(rng.choice(240, n_sym, replace=False),
                                            rng.integers(1, 1 << 18, n_sym))}
    _, table = oracle.get_32bit_codec(freqs)
    ref = oracle.get_luts(table)
    got = U.get_luts({k: v for k, v in table.items() if k is not EOF}).numpy()
    _assert_luts_equal_up_to_eof_fill(ref, got, table)


@pytest.mark.parametrize("kind", ["normal", "laplace", "fib", "zeros", "single"])
@pytest.mark.parametrize("n", [1, 7, 4099, 123_457])
def test_bitstream_matches_reference_packer(oracle, kind, n):
    """Same table in, same encoded bytes / gaps / positions out as the reference's
    encode() -- except that the product always writes n_blocks + 1 positions."""
    w = make_case(kind, n, 17)
    c = compress_product(w)
    table = _oracle_table(c["codec"])
    enc, gaps, pos = oracle.c_encode(c["exponent"], table)
    assert np.array_equal(enc, c["encoded_exponent"])
    assert np.array_equal(gaps, c["gaps"])
    n_blocks = -(-enc.size // 4096)
    assert c["output_positions"].size == n_blocks + 1
    assert np.array_equal(pos, c["output_positions"][: pos.size])
    assert (c["output_positions"][pos.size:] == n).all()


def test_positions_quirk_is_not_inherited(oracle):
    """Last code crosses a block boundary and ends byte-aligned: the reference
    is one entry short; the product emits the entry."""
    table = {1: (8, 0b10000000), 2: (16, 0b0000000000000001), EOF: (16, 0)}
    data = np.array([1] * 4095 + [2], np.uint8)
    codec = U.DF11Codec.from_table({1: table[1], 2: table[2], U._EOF: table[EOF]})
    enc, gaps, pos = U.encode(data, codec)
    renc, rgaps, rpos = oracle.c_encode(data, table)
    assert np.array_equal(enc, renc) and np.array_equal(gaps, rgaps)
    assert rpos.tolist() == [0, 4096] and pos.tolist() == [0, 4096, 4096]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("n", [1, 513, 70_001])
def test_reference_decoder_reads_product_streams(oracle, kind, n):
    """The oracle's restatement of the reference kernel decodes what the product
    encoder wrote, bit for bit -- including the mixes the reference's own
    encoder cannot lay out (exponents >= 240)."""
    w = make_case(kind, n, 23)
    c = compress_product(w)
    out = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                          c["output_positions"], c["gaps"])
    assert np.array_equal(out, w)
    seq = oracle.c_decode_sequential(_oracle_table(c["codec"]), c["encoded_exponent"], c["sign_mantissa"])
    assert np.array_equal(seq, w)


@pytest.mark.parametrize("hist", [{250: 5, 243: 1000}, {250: 5}, {241: 1, 247: 1, 255: 9},
                                  {s: 1 + s % 7 for s in range(240, 256)}, {250: 5, 241: 7, 100: 3}])
def test_reference_decoder_reads_streams_of_high_exponents_only(oracle, hist):
    """With no exponent below 240 there is no symbol that may fill the unowned
    slots of the first three LUT levels (the reference kernel reads 240..255 there
    as pointers, decode.cu:105-116): its trailing threads, which decode the padding
    and the zeros past the stream, must still stay inside the rows that exist."""
    codec = U.DF11Codec.from_frequencies(hist)
    luts = U.get_luts(codec.get_code_table()).numpy()
    n_rows = luts.shape[0] - 1
    rng = np.random.default_rng(1)
    e = np.concatenate([np.array(list(hist), np.uint8), rng.choice(np.array(list(hist), np.uint8), 700)])
    enc, gaps, pos = U.encode(e, codec)
    sm = rng.integers(0, 256, e.size).astype(np.uint8)
    w = (((sm.astype(np.uint16) & 0x80) << 8) | (e.astype(np.uint16) << 7) | (sm & 0x7F)).astype(np.uint16)
    assert np.array_equal(oracle.c_decode(luts, enc, sm, pos, gaps), w)
    # Rows are ordered by (level, prefix).  On levels 0..2 a value >= 240 must be a
    # pointer to a row that exists, anything else a symbol that has a code.
    lens, vals = codec.code_len.astype(int), codec.code_val.astype(int)
    prefixes = sorted({(lv, vals[s] >> (lens[s] - 8 * lv)) for s in hist for lv in range((lens[s] - 1) // 8 + 1)})
    assert len(prefixes) == n_rows
    for r, (level, _) in enumerate(prefixes):
        for v in luts[r]:
            if level < 3 and v >= 240:
                assert 0 < 256 - int(v) < n_rows, (r, int(v))
            else:
                assert luts[-1][v] > 0, (r, int(v))


@pytest.mark.parametrize("seed", range(6))
def test_random_histograms_build_valid_codes_the_reference_decoder_reads(oracle, seed):
    """Counts over 50 orders of magnitude, few and many symbols, with and without
    exponents >= 240: prefix-free, Kraft <= 1, <= 32 bits, high exponents on the
    fourth level, <= 16 sub-tables, and a round trip through the oracle."""
    for case in range(60):
        rng = np.random.default_rng(seed * 1000 + case)
        k = int(rng.choice([1, 2, 3, 5, 17, 40, 100, 200, 240, 256]))
        pool = int(rng.integers(0, 3))
        if pool == 0:
            syms = rng.permutation(256)[:k]
        elif pool == 1:
            syms = rng.permutation(240)[:min(k, 240)]
        else:
            hi = rng.permutation(np.arange(240, 256))[:min(k, 16)]
            syms = np.concatenate([hi, rng.permutation(240)[:max(0, k - hi.size)]])
        fam = int(rng.integers(0, 4))
        if fam == 0:
            cnt = np.floor(2.0 ** rng.uniform(0, 50, syms.size))
        elif fam == 1:
            cnt = np.floor(1.618 ** np.arange(syms.size) % 2 ** 52) + 1
        elif fam == 2:
            cnt = np.ones(syms.size)
        else:
            cnt = np.floor(2.0 ** (np.arange(syms.size) % 45))
        hist = {int(s): int(c) for s, c in zip(syms, cnt)}
        codec = U.DF11Codec.from_frequencies(hist)
        luts = U.get_luts(codec.get_code_table()).numpy()
        lens = codec.code_len.astype(int)
        words = sorted([format(int(codec.code_val[s]), "b").rjust(lens[s], "0") for s in hist]
                       + [format(codec.eof_val, "b").rjust(codec.eof_len, "0")])
        assert all(not b.startswith(a) for a, b in zip(words, words[1:])), (seed, case)
        assert sum(2.0 ** -len(x) for x in words) <= 1.0
        assert lens.max() <= 32 and 0 < codec.eof_len <= 32
        assert all(lens[s] >= 25 for s in hist if s >= 240)
        assert luts.shape[0] - 2 <= 16
        e = np.concatenate([np.array(list(hist), np.uint8), rng.choice(np.array(list(hist), np.uint8), 500)])
        rng.shuffle(e)
        enc, gaps, pos = U.encode(e, codec)
        sm = rng.integers(0, 256, e.size).astype(np.uint8)
        w = (((sm.astype(np.uint16) & 0x80) << 8) | (e.astype(np.uint16) << 7) | (sm & 0x7F)).astype(np.uint16)
        assert np.array_equal(oracle.c_decode(luts, enc, sm, pos, gaps), w), (seed, case)


def test_luts_for_a_first_byte_that_only_32_bit_codes_share(oracle):
    """Codes 0, 1{30 zeros}0 and 1{30 zeros}1: the root row's pointer at 0x80 is
    owned by 32-bit codes alone (their prefix test shifts by the full word width)."""
    code_len = np.zeros(256, np.uint8)
    code_val = np.zeros(256, np.uint32)
    code_len[7], code_val[7] = 1, 0
    code_len[9], code_val[9] = 32, 0x80000000
    code_len[11], code_val[11] = 32, 0x80000001
    codec = U.DF11Codec(code_len, code_val, 31, 0x40000001)
    luts = U.get_luts(codec.get_code_table()).numpy()
    assert luts.shape[0] == 5 and luts[0, 0x80] == 255 and luts[0, 0x7F] == 7
    e = np.array([7, 9, 7, 7, 11, 11, 9, 7] * 40, np.uint8)
    enc, gaps, pos = U.encode(e, codec)
    sm = np.arange(e.size, dtype=np.uint8)
    w = (((sm.astype(np.uint16) & 0x80) << 8) | (e.astype(np.uint16) << 7) | (sm & 0x7F)).astype(np.uint16)
    assert np.array_equal(oracle.c_decode(luts, enc, sm, pos, gaps), w)


def test_fibonacci_reaches_32_bits():
    w = make_case("fib", 400_000, 1)
    c = compress_product(w)
    assert int(c["codec"].code_len.max()) > 24      # fourth LUT level in use
    assert int(c["codec"].code_len.max()) <= 32


def test_too_many_subtables_falls_back():
    """One dominant exponent and 239 equally rare ones would need ~120 sub-tables
    under plain Huffman; the builder must shorten the code until 16 suffice."""
    hist = {0: 1 << 30}
    hist.update({s: 1000 + s for s in range(1, 240)})
    codec = U.DF11Codec.from_frequencies(hist)
    luts = U.get_luts(codec.get_code_table())
    assert luts.shape[0] - 2 <= 16
    assert int(codec.code_len.max()) <= 32


def test_encode_rejects_symbol_without_code():
    codec = U.DF11Codec.from_frequencies({5: 10, 6: 3})
    with pytest.raises(ValueError):
        U.encode(np.array([5, 6, 7], np.uint8), codec)


def test_codec_under_sanitizers():
    """tests/emul/df11_codec_san: the host codec built with AddressSanitizer and
    UndefinedBehaviorSanitizer, random cases plus a Fibonacci histogram with 32-bit
    codes, each decoded back by the oracle's C restatement."""
    import os
    import subprocess
    d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "emul")
    locked_make(d, "df11_codec_san")
    res = subprocess.run([os.path.join(d, "df11_codec_san"), "60"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, (res.stdout + res.stderr)[-3000:]
    assert "0 failures" in res.stdout and "32 bits" in res.stdout
