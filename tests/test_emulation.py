"""Runs the decode kernel's shared host/device logic (dfloat11_amd/csrc/df11_core.h)
on the CPU, thread by thread, against the oracle -- with exact-size buffers and,
for a subset, under AddressSanitizer.  This is where indexing mistakes are meant
to surface before anything is launched on a GPU."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from tests.df11_cases import (locked_make, KINDS, compress_product, make_case, max_elems_per_block, max_rows_case,
                              random_code_case)

EMUL_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "emul")


@pytest.fixture(scope="module")
def emul():
    locked_make(EMUL_DIR)
    L = ctypes.CDLL(os.path.join(EMUL_DIR, "libdf11_emul.so"))
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.df11_emul_decode.argtypes = [vp, vp, vp, vp, vp, vp, i32, i64, i64, i32, i32, i32, i32, i32]
    L.df11_emul_decode.restype = i32
    L.df11_emul_decode_rows.argtypes = [vp, vp, vp, vp, vp, vp, i32, i64, i64, i32, vp, i64, i64]
    L.df11_emul_decode_rows.restype = i32
    return L


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


SLOTS = {"usual": 0, "few": 1, "short": 2}


def run_emul(L, c, max_elems=0, grid=3, codes_misalign=0, out_misalign=0, two_pass=False, slots="usual"):
    """slots: which compilation's register slots to emulate (10, 7 or 14 lookups inside a chunk)."""
    n = c["sign_mantissa"].size
    out = np.zeros(n, np.uint16)
    luts = np.ascontiguousarray(c["luts"])
    rc = L.df11_emul_decode(_p(luts), _p(c["encoded_exponent"]), _p(c["sign_mantissa"]),
                            _p(c["output_positions"]), _p(c["gaps"]), _p(out), luts.shape[0],
                            c["encoded_exponent"].size, n, max_elems, grid, codes_misalign, out_misalign,
                            (1 if two_pass else 0) | (SLOTS[slots] << 8))
    assert rc == 0
    return out


def run_asan(c, max_elems=0, grid=2, codes_misalign=0, out_misalign=0, tmp_path=None, two_pass=False,
             ok_codes=(0,), rows=False, slots="usual"):
    """rows: df11_decode_rows for rows 6, 0, 3 of the output as a seven-row matrix (and numbers
    outside it) into a buffer of 0xEEEE, instead of the whole stream."""
    n = c["sign_mantissa"].size
    n_bytes = c["encoded_exponent"].size
    n_blocks = -(-n_bytes // 4096)
    luts = np.ascontiguousarray(c["luts"])
    inp, outp = str(tmp_path / "case.bin"), str(tmp_path / "out.bin")
    with open(inp, "wb") as f:
        f.write(np.array([luts.shape[0], n_bytes, n, n_blocks, max_elems, grid, codes_misalign,
                          out_misalign, (1 if two_pass else 0) | (4 if rows else 0) | (SLOTS[slots] << 8)],
                         np.int64).tobytes())
        f.write(luts.tobytes())
        f.write(c["encoded_exponent"].tobytes())
        f.write(c["sign_mantissa"].tobytes())
        f.write(np.ascontiguousarray(c["output_positions"][:n_blocks]).tobytes())
        f.write(c["gaps"].tobytes())
    res = subprocess.run([os.path.join(EMUL_DIR, "df11_emul_asan"), inp, outp],
                         capture_output=True, text=True)
    assert res.returncode in ok_codes and "AddressSanitizer" not in res.stderr, res.stderr[-3000:]
    return np.fromfile(outp, dtype=np.uint16) if res.returncode == 0 else None


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("n", [1, 2, 511, 4097, 60_000])
def test_emulated_kernel_matches_oracle(emul, oracle, kind, n):
    w = make_case(kind, n, 31)
    c = compress_product(w)
    ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                          c["output_positions"], c["gaps"])
    assert np.array_equal(ref, w)
    got = run_emul(emul, c, max_elems=max_elems_per_block(c["output_positions"]))
    assert np.array_equal(got, ref)
    # worst-case staging selected by max_elems <= 0; the two-pass fall-back route on every input
    assert np.array_equal(run_emul(emul, c, max_elems=0, grid=1, two_pass=True), ref)
    # the compilations with other numbers of register slots
    for slots in ("few", "short"):
        assert np.array_equal(run_emul(emul, c, max_elems=0, grid=2, slots=slots), ref), slots


@pytest.mark.parametrize("kind", ["normal", "zeros", "fib", "uniform256"])
def test_emulated_kernel_multi_block(emul, oracle, kind):
    w = make_case(kind, 700_000, 37)
    c = compress_product(w)
    assert c["encoded_exponent"].size > 3 * 4096
    got = run_emul(emul, c, max_elems=max_elems_per_block(c["output_positions"]), grid=5)
    assert np.array_equal(got, w)


@pytest.mark.parametrize("codes_misalign,out_misalign", [(1, 0), (0, 1), (3, 5), (4, 4)])
def test_emulated_kernel_unaligned_pointers(emul, codes_misalign, out_misalign):
    w = make_case("normal", 50_000, 41)
    c = compress_product(w)
    got = run_emul(emul, c, max_elems=max_elems_per_block(c["output_positions"]),
                   codes_misalign=codes_misalign, out_misalign=out_misalign)
    assert np.array_equal(got, w)


def test_emulated_kernel_reads_reference_streams(emul, oracle):
    """Streams written by the oracle's restatement of the reference encoder
    (dahuffman-ordered table, reference LUT fill, positions possibly one short)."""
    w = make_case("outliers", 90_000, 43)
    c = oracle.compress(w)
    n_blocks = -(-c["encoded_exponent"].size // 4096)
    pos = np.full(n_blocks + 1, w.size, np.uint32)
    pos[: c["output_positions"].size] = c["output_positions"]
    c2 = dict(c, output_positions=pos)
    assert np.array_equal(run_emul(emul, c2, max_elems=max_elems_per_block(pos)), w)


def test_emulated_kernel_short_positions_quirk(emul, oracle):
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
    # the kernel reads one position per block: entry 1 is the reference's sentinel
    c = dict(luts=luts, encoded_exponent=enc, sign_mantissa=sm, output_positions=pos, gaps=gaps)
    assert pos.size == 2 and -(-enc.size // 4096) == 2
    assert np.array_equal(run_emul(emul, c), oracle.merge_bf16(data, sm))


@pytest.mark.parametrize("seed,n_full", [(1, 1), (2, 3), (3, 9)])
def test_emulated_kernel_short_positions_multi_block(emul, oracle, seed, n_full):
    """Realistic code lengths, several blocks, positions one entry short."""
    from tests.df11_cases import short_positions_case
    w, c = short_positions_case(oracle, seed, n_full)
    ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
    assert np.array_equal(ref, w)
    assert np.array_equal(run_emul(emul, c), w)


def test_emulated_kernel_small_staging_is_clamped_not_overrun(emul, tmp_path):
    """A caller that understates max_elems_per_block loses elements but never
    writes outside the staging area (checked under AddressSanitizer)."""
    w = make_case("zeros", 100_000, 47)
    c = compress_product(w)
    got = run_asan(c, max_elems=1000, tmp_path=tmp_path)
    assert got.size == w.size          # ran to completion without a sanitizer report


@pytest.mark.parametrize("kind,n,cm,om", [("normal", 40_000, 0, 0), ("zeros", 70_000, 0, 0),
                                          ("fib", 330_000, 0, 0), ("uniform256", 9_000, 2, 3),
                                          ("high", 5_000, 0, 1), ("single", 1, 0, 0),
                                          ("laplace", 4096 * 3, 7, 0)])
def test_emulated_kernel_under_asan(emul, tmp_path, kind, n, cm, om):
    w = make_case(kind, n, 53)
    c = compress_product(w)
    for two_pass in (False, True):
        got = run_asan(c, max_elems=max_elems_per_block(c["output_positions"]), codes_misalign=cm,
                       out_misalign=om, tmp_path=tmp_path, two_pass=two_pass)
        assert np.array_equal(got, w)
    for slots in ("few", "short"):
        got = run_asan(c, max_elems=max_elems_per_block(c["output_positions"]), codes_misalign=cm,
                       out_misalign=om, tmp_path=tmp_path, slots=slots)
        assert np.array_equal(got, w), slots
    got = run_asan(c, max_elems=max_elems_per_block(c["output_positions"]), tmp_path=tmp_path, rows=True)
    row = max(1, n // 7)
    for i in (6, 0, 3):
        if (i + 1) * row <= n:
            assert np.array_equal(got[i * row:(i + 1) * row], w[i * row:(i + 1) * row]), i
    written = got != 0xEEEE
    assert np.array_equal(got[written], w[written])


def test_emulated_kernel_malformed_streams_stay_in_bounds(emul, tmp_path):
    """Random bytes in place of the bitstream, the gaps, the LUTs, the code
    lengths or the block positions, flipped bytes, and an element count smaller
    than the stream holds: the decode logic must terminate without reading or
    writing outside its buffers (AddressSanitizer build).  The output is
    unspecified; the two decode routes may disagree (exit status 3)."""
    for case in range(40):
        rng = np.random.default_rng(4000 + case)
        kind = str(rng.choice(["normal", "fib", "uniform256", "zeros", "outliers"]))
        base = compress_product(make_case(kind, int(rng.integers(1, 40_000)), case))
        c = {k: np.array(v, copy=True) for k, v in base.items() if isinstance(v, np.ndarray)}
        what = case % 7
        if what == 0:
            c["encoded_exponent"] = rng.integers(0, 256, c["encoded_exponent"].size).astype(np.uint8)
        elif what == 1:
            c["gaps"] = rng.integers(0, 256, c["gaps"].size).astype(np.uint8)
        elif what == 2:
            c["luts"] = rng.integers(0, 256, c["luts"].shape).astype(np.uint8)
        elif what == 3:
            c["output_positions"] = rng.integers(0, 2 ** 32, c["output_positions"].size,
                                                 dtype=np.uint64).astype(np.uint32)
        elif what == 4:
            c["luts"][-1] = rng.integers(0, 40, 256).astype(np.uint8)
        elif what == 5:
            for k in ("encoded_exponent", "gaps"):
                idx = rng.integers(0, c[k].size, max(1, c[k].size // 50))
                c[k][idx] ^= rng.integers(1, 256, idx.size).astype(np.uint8)
        else:
            c["sign_mantissa"] = c["sign_mantissa"][: max(1, c["sign_mantissa"].size // 3)]
        run_asan(c, max_elems=int(rng.choice([0, 1, 7, 100])), grid=int(rng.integers(1, 4)), tmp_path=tmp_path,
                 two_pass=bool(case & 8), ok_codes=(0, 3))


# ---------------------------------------------------------------- derived tables
def _host_tables(luts):
    L = ctypes.CDLL(os.path.join(EMUL_DIR, "libdf11_emul.so"))
    luts = np.ascontiguousarray(luts)
    blob = np.zeros(2048 * 8 + 2048 + 17 * 512, np.uint8)      # dec | cntt | fused rows
    L.df11_emul_tables(_p(luts), luts.shape[0], _p(blob))
    dec = blob[: 2048 * 8].view(np.uint32).reshape(2048, 2)
    return dec, blob[2048 * 8: 2048 * 8 + 2048]


def _host_fused_rows(luts):
    L = ctypes.CDLL(os.path.join(EMUL_DIR, "libdf11_emul.so"))
    luts = np.ascontiguousarray(luts)
    blob = np.zeros(2048 * 8 + 2048 + 17 * 512, np.uint8)
    L.df11_emul_tables(_p(luts), luts.shape[0], _p(blob))
    return blob[2048 * 8 + 2048:].view(np.uint16).reshape(17, 256)[: luts.shape[0] - 1]


def _check_fused_rows(luts, codec=None):
    """The 16-bit rows the hierarchical lookup reads, from their definition: the LUT
    byte, the recorded length of that byte taken as a symbol (1 where 0), and the flag
    'names a row that exists'.  An 11-bit pattern that settles no code carries the place
    where its lookup starts (a row and the code byte that indexes it): walking on from
    there with the bits of any code word that begins with the pattern must give that
    code word's symbol and length, exactly as the walk from the root does."""
    luts = np.asarray(luts)
    n_rows = luts.shape[0] - 1
    d = luts[:n_rows].astype(np.uint32)
    length = np.maximum(luts[-1].astype(np.uint32)[d], 1)
    flag = (d >= 240) & (256 - d < n_rows)
    want = (d | (length << 8) | (flag.astype(np.uint32) << 15)).astype(np.uint16)
    assert np.array_equal(_host_fused_rows(luts), want)
    dec, _ = _host_tables(luts)
    unresolved = np.nonzero(dec[:, 1] >> 31)[0]
    assert ((dec[:, 1] >> 31 == 1) | ((dec[:, 1] >> 8) - 1 < 4)).all()      # marked, or one to four codes
    rows, shifts = dec[unresolved, 0] // 512, dec[unresolved, 1] & 0x7FFFFFFF
    assert (dec[unresolved, 0] % 512 == 0).all()
    assert (rows < n_rows).all() and np.isin(shifts, (24, 16, 8, 0)).all()
    levels = (24 - shifts) // 8
    if codec is None:
        return
    start = {int(i): (int(r), int(lv)) for i, r, lv in zip(unresolved, rows, levels)}
    checked = 0
    for s in range(256):
        n = int(codec.code_len[s])
        if n <= 11:
            continue
        word = int(codec.code_val[s])
        for pad in (0, (1 << (32 - n)) - 1, 0x5A5A5A5A & ((1 << (32 - n)) - 1)):
            top = (word << (32 - n)) | pad
            idx = top >> 21
            assert idx in start, (s, n)          # a pattern that begins a longer code settles nothing
            row, level = start[idx]
            while True:
                e = int(luts[row, (top >> (24 - 8 * level)) & 0xFF])
                if level < 3 and e >= 240 and 256 - e < n_rows:
                    row, level = 256 - e, level + 1
                    continue
                break
            assert e == s and int(luts[-1, e]) == n, (s, n, start[idx])
            checked += 1
    return checked


def _first_code(bits, codes):
    """('sym', s, len) if a code word is a prefix of `bits`; ('open',) if `bits` is
    a proper prefix of some symbol's code word (too short to tell); ('void',) if it
    runs into the end-of-stream code or into code space no symbol uses."""
    for s, word in codes.items():
        if s != "eof" and bits.startswith(word):
            return ("sym", s, len(word))
    if any(s != "eof" and word.startswith(bits) for s, word in codes.items()):
        # could still become a symbol -- unless only the end-of-stream code continues it
        return ("open",)
    return ("void",)


def _check_tables_against_code(codec, luts):
    """Every entry of the multi-symbol tables against the code table itself: for
    each 11-bit pattern the first (up to four) code words that END inside it,
    and for each shorter pattern the number of code words that START inside it.
    Paths that run into the end-of-stream code or into unused code space are
    exempt from there on: no valid stream contains them before its padding."""
    codes = {int(s): format(int(codec.code_val[s]), "b").rjust(int(codec.code_len[s]), "0")
             for s in range(256) if codec.code_len[s]}
    codes["eof"] = format(codec.eof_val, "b").rjust(codec.eof_len, "0")
    dec, cntt = _host_tables(luts)
    checked = 0
    for idx in range(2048):
        bits = format(idx, "011b")
        syms, pos, void = [], 0, False
        while len(syms) < 4:
            r = _first_code(bits[pos:], codes)
            if r[0] != "sym":
                void = r[0] == "void"
                break
            syms.append(r[1])
            pos += r[2]
        word, meta = int(dec[idx, 0]), int(dec[idx, 1])
        if meta >> 31:                                    # settles no code: the words say where the lookup starts
            meta = 0
        k, nbits = meta >> 8, meta & 0xFF
        got = [(word >> (8 * i)) & 0xFF for i in range(k)]
        assert got[: len(syms)] == syms, (idx, got, syms)
        if not void:
            checked += 1
            assert k == len(syms) and nbits == (pos if syms else 0), (idx, meta, syms, pos)
    assert checked > 0
    for r in range(1, 11):
        for v in range(1 << r):
            bits = format(v, "b").rjust(r, "0")
            pos, starts, void = 0, 0, False
            while pos < r:
                res = _first_code(bits[pos:], codes)
                if res[0] == "void":
                    void = True
                    break
                starts += 1
                if res[0] == "open":
                    break
                pos += res[2]
            if not void:
                assert int(cntt[(1 << r) | v]) == starts, (r, bits, int(cntt[(1 << r) | v]), starts)


@pytest.mark.parametrize("kind,n,seed", [("normal", 300_000, 1), ("outliers", 4097, 61),
                                         ("outliers", 200_000, 2), ("fib", 330_000, 3),
                                         ("uniform256", 50_000, 4), ("zeros", 10_000, 5),
                                         ("high", 3_000, 6), ("single", 100, 7)])
def test_derived_tables_brute_force(emul, kind, n, seed):
    c = compress_product(make_case(kind, n, seed))
    _check_tables_against_code(c["codec"], c["luts"])
    _check_fused_rows(c["luts"], c["codec"])


@pytest.mark.parametrize("seed", [900, 905, 911, 922, 1059, 1065, 1165, 1195])
def test_derived_tables_brute_force_random_codes(emul, seed):
    """Incomplete prefix codes with the unowned LUT slots filled three ways: the
    tables must not depend on what those slots hold.  (A short code carried into
    the slots next to a pointer once made an 11-bit prefix of a 26-bit code look
    like that short code.)"""
    made = random_code_case(seed, max_n=50)
    if made is None:
        pytest.skip("drawn code does not fit the DF11 layout")
    _, cases = made
    for policy, c in cases.items():
        _check_tables_against_code(c["codec"], c["luts"])
        _check_fused_rows(c["luts"], c["codec"])


@pytest.mark.parametrize("chunk", range(8))
def test_emulated_kernel_random_codes_and_fillings(emul, oracle, chunk):
    """Random prefix codes (deep, incomplete, symbols >= 240) x three fillings of
    the unowned LUT slots: kernel == original words, both decode routes.  Where
    the reference kernel itself could not decode the LUTs (it would spin on a
    zero-length filling in the stream's padding) only termination is required."""
    ran = 0
    for seed in range(1000 + 40 * chunk, 1040 + 40 * chunk):
        made = random_code_case(seed)
        if made is None:
            continue
        w, cases = made
        for policy, c in cases.items():
            try:
                ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                                      c["output_positions"], c["gaps"])
            except RuntimeError:
                run_emul(emul, c)
                continue
            assert np.array_equal(ref, w), (seed, policy)
            for two_pass in (False, True):
                assert np.array_equal(run_emul(emul, c, two_pass=two_pass), w), (seed, policy, two_pass)
            for slots in ("few", "short"):
                assert np.array_equal(run_emul(emul, c, slots=slots), w), (seed, policy, slots)
            ran += 1
    assert ran > 20


@pytest.mark.parametrize("n", [1, 700, 40_000])
def test_emulated_kernel_every_lut_row(emul, oracle, n):
    """A code that fills the layout's 16 sub-tables on all four levels (luts of 18 rows,
    codes of 1 to 32 bits) x three fillings of the unowned slots: derived tables from
    their definition, and kernel == oracle == original words on both decode routes."""
    w, cases = max_rows_case(300 + n, n)
    for policy, c in cases.items():
        _check_tables_against_code(c["codec"], c["luts"])
        assert _check_fused_rows(c["luts"], c["codec"]) > 0
        ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"],
                              c["output_positions"], c["gaps"])
        assert np.array_equal(ref, w), policy
        for two_pass in (False, True):
            assert np.array_equal(run_emul(emul, c, two_pass=two_pass), w), (policy, two_pass)
        for slots in ("few", "short"):
            assert np.array_equal(run_emul(emul, c, slots=slots), w), (policy, slots)


@pytest.mark.parametrize("slots", ["usual", "few", "short"])
def test_emulated_kernel_chunks_of_many_lookups(emul, slots):
    """Streams whose chunks need more lookups than weight-like ones: sparse weights (one- to
    three-bit codes next to long ones, up to sixteen lookups of four codes) and alphabets of
    48 to 240 equally likely exponents (six- to eight-bit codes, one per lookup, up to eleven).
    Whatever the compilation's register slots hold or not, the output is the original words
    (the emulation also compares the register route's counts with the counting pass)."""
    rng = np.random.default_rng(11)
    n = 120_000
    sm = rng.integers(0, 256, n).astype(np.uint16)

    def words(e):
        return (((sm & 0x80) << 8) | (e.astype(np.uint16) << 7) | (sm & 0x7F)).astype(np.uint16)

    for p_zero in (1.0, 0.97, 0.9, 0.7, 0.5):
        e = np.where(rng.random(n) < p_zero, 0, np.clip(rng.normal(121, 2.5, n), 90, 135).astype(np.int64))
        w = words(e)
        assert np.array_equal(run_emul(emul, compress_product(w), grid=2, slots=slots), w), p_zero
    for alphabet in (48, 64, 100, 128, 200, 240):
        w = words(rng.integers(0, alphabet, n))
        assert np.array_equal(run_emul(emul, compress_product(w), grid=2, slots=slots), w), alphabet


def test_emulated_kernel_few_elements_many_symbols(emul, oracle):
    """A handful of elements over a large alphabet that includes exponents >= 240:
    short codes next to 26-bit ones in a stream of a few bytes."""
    rng = np.random.default_rng(5)
    for n in (15, 32, 43, 64, 200):
        syms = np.concatenate([rng.permutation(np.arange(240, 256))[:8], rng.permutation(240)[:190]])
        e = rng.choice(syms, n).astype(np.uint16)
        sm = rng.integers(0, 256, n).astype(np.uint16)
        w = (((sm & 0x80) << 8) | (e << 7) | (sm & 0x7F)).astype(np.uint16)
        c = compress_product(w)
        ref = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
        assert np.array_equal(ref, w)
        for two_pass in (False, True):
            assert np.array_equal(run_emul(emul, c, two_pass=two_pass), w), (n, two_pass)


@pytest.mark.parametrize("seed", range(60, 72))
def test_emulated_kernel_long_codes_many_seeds(emul, seed):
    """Sparse outliers give 12..14-bit codes next to 2-bit ones: the slow path and
    the table boundaries in every position."""
    w = make_case("outliers", 4097 + 37 * seed, seed)
    c = compress_product(w)
    assert np.array_equal(run_emul(emul, c, max_elems=max_elems_per_block(c["output_positions"]), grid=2), w)


@pytest.mark.parametrize("kind,n_rows,row_elements", [("normal", 700, 512), ("zeros", 900, 256), ("uniform256", 300, 320),
                                                     ("fib", 2000, 64), ("laplace", 5, 30_011), ("outliers", 40_000, 3),
                                                     ("single", 1, 1)])
def test_emulated_row_decode(emul, kind, n_rows, row_elements):
    """The steps of df11_decode_rows on the host: the search for the sub-block that holds a
    row's first element lands on it (the emulation checks that), the requested rows come
    out as the original words, whatever else is written is right as well, and elements far
    from every requested row keep what the buffer held."""
    n = n_rows * row_elements
    w = make_case(kind, n, 77)
    c = compress_product(w)
    luts = np.ascontiguousarray(c["luts"])
    rng = np.random.default_rng(3)
    for n_ids in (1, 4, 40):
        ids = rng.integers(0, n_rows, n_ids)
        ids[0] = n_rows - 1
        if n_ids > 2:
            ids[1], ids[2] = 0, ids[0]
        asked = np.concatenate([ids, [-1, n_rows, 2 ** 40]]).astype(np.int64)
        rng.shuffle(asked)
        sentinel = 0xEEEE
        out = np.full(n, sentinel, np.uint16)
        rc = emul.df11_emul_decode_rows(_p(luts), _p(c["encoded_exponent"]), _p(c["sign_mantissa"]),
                                        _p(c["output_positions"]), _p(c["gaps"]), _p(out), luts.shape[0],
                                        c["encoded_exponent"].size, n, 0, _p(asked), asked.size, row_elements)
        assert rc == 0, (kind, n_ids, rc)
        wanted = np.zeros(n, bool)
        for i in ids:
            wanted[i * row_elements:(i + 1) * row_elements] = True
        assert np.array_equal(out[wanted], w[wanted]), (kind, n_ids)
        written = out != sentinel
        assert np.array_equal(out[written], w[written]), (kind, n_ids)
        near = np.zeros(n + 1, np.int64)
        for i in ids:
            near[max(0, i * row_elements - 4096)] += 1
            near[min(n, (i + 1) * row_elements + 4096)] -= 1
        far = np.cumsum(near[:-1]) == 0
        assert not (written & far & (w != sentinel)).any(), (kind, n_ids)
