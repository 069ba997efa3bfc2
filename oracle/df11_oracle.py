"""TEST INFRASTRUCTURE ONLY -- CPU oracle for the DFloat11 weight-decompression path.

Nothing that ships may import this module.  It restates, in numpy / plain
Python, the reference's offline codec (dfloat11/dfloat11_utils.py) and binds
the C restatement of the reference decode kernel (oracle/df11_oracle.c).

Third-party arithmetic: the reference builds its prefix code with
``dahuffman==0.4.2`` (setup.py:20; call sites dfloat11_utils.py:32,38,57).  That
package is not in the reference tree and is not installed, so
``huffman_from_frequencies`` restates its published algorithm
(``HuffmanCodec.from_frequencies``: a heap of ``(weight, [(symbol, (nbits,
value))...])`` tuples, the two lightest popped, the first prefixed with bit 0 and
the second with bit 1, ties decided by Python tuple/list comparison, the
end-of-stream pseudo-symbol ordered below every symbol).

Pinning status:
  * huffman_from_frequencies : PARITY UNPINNED for the exact code words and
    tie-breaks (no dahuffman here to compare against, no golden table in the
    reference).  Pinned for what decoding depends on: prefix-freeness, Kraft
    sum == 1 including the end-of-stream leaf, and total cost equal to an
    independent textbook Huffman cost (cost is tie-invariant).
  * get_32bit_codec          : PARITY UNPINNED for which symbols the heuristic
    flattens (depends on dahuffman ties and numpy's argpartition); pinned for
    the property it exists for (max length <= 32).
  * get_luts                 : pinned by brute force (every symbol, every
    padding of trailing bits, walks back to itself through the reference's
    4-level lookup) and by hand-worked tables.
  * encode                   : pinned by hand-packed streams, by agreement of
    this pure-Python restatement with the C restatement, and by invariants
    (sequential decode recovers the data; gaps/positions definitions).
"""
from __future__ import annotations

import ctypes
import heapq
import os
import subprocess
from collections import OrderedDict

import numpy as np

BYTES_PER_THREAD = 8      # dfloat11.py:45
THREADS_PER_BLOCK = 512   # dfloat11.py:46
BLOCK_BYTES = BYTES_PER_THREAD * THREADS_PER_BLOCK

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdf11_oracle.so")


# --------------------------------------------------------------------------
# dahuffman 0.4.2 restatement
# --------------------------------------------------------------------------
class _EndOfStream:
    """Pseudo-symbol appended by dahuffman; compares below every other symbol."""

    def __repr__(self):
        return "_EOF"

    def __lt__(self, other):
        return True

    def __gt__(self, other):
        return False

    def __eq__(self, other):
        return other.__class__ == self.__class__

    def __hash__(self):
        return hash(self.__class__)


EOF = _EndOfStream()


def huffman_from_frequencies(frequencies):
    """symbol -> (nbits, value), in the insertion order dahuffman's table has
    (left-to-right leaf order of the tree).  Always contains EOF."""
    heap = [(f, [(s, (0, 0))]) for s, f in frequencies.items()]
    if EOF not in frequencies:
        heap.append((1, [(EOF, (0, 0))]))
    heapq.heapify(heap)
    while len(heap) > 1:
        a = heapq.heappop(heap)
        b = heapq.heappop(heap)
        merged = (
            a[0] + b[0],
            [(s, (n + 1, v)) for (s, (n, v)) in a[1]]
            + [(s, (n + 1, (1 << n) + v)) for (s, (n, v)) in b[1]],
        )
        heapq.heappush(heap, merged)
    return OrderedDict(heapq.heappop(heap)[1])


# --------------------------------------------------------------------------
# dfloat11_utils.py restatement
# --------------------------------------------------------------------------
def split_bf16(w_u16):
    """dfloat11_utils.py:175-178 on a uint16/int16 view of BF16 data."""
    w = np.asarray(w_u16).view(np.int16).astype(np.int32)
    exponent = ((w >> 7) & 0xFF).astype(np.uint8)
    sign_mantissa = (((w >> 8) & 0x80) | (w & 0x7F)).astype(np.uint8)
    return exponent, sign_mantissa


def merge_bf16(exponent, sign_mantissa):
    """decode.cu:207-210."""
    e = np.asarray(exponent, dtype=np.uint16)
    s = np.asarray(sign_mantissa, dtype=np.uint16)
    hi = (s & 128) | (e >> 1)
    lo = ((e << 7) | (s & 127)) & 0xFF
    return ((hi << 8) | lo).astype(np.uint16)


def get_counter(exponent):
    """dfloat11_utils.py:24-30: exponent histogram as {value: count}, ascending value."""
    vals, freqs = np.unique(np.asarray(exponent), return_counts=True)
    return OrderedDict((int(v), int(f)) for v, f in zip(vals, freqs))


def _max_len(table):
    return max(l for (l, _) in table.values())


def get_32bit_codec(counter):
    """dfloat11_utils.py:37-65: while the longest code exceeds 32 bits, set the k
    rarest symbols' counts to 1 and rebuild, k = 2, 3, ..."""
    table = huffman_from_frequencies(counter)
    compressed_counter = counter
    min_k = 2
    freq = np.array(list(counter.values()))
    keys = np.array(list(counter.keys()))
    while _max_len(table) > 32:
        min_indices = np.argpartition(freq, min_k)[:min_k]
        min_k += 1
        compressed_counter = OrderedDict(counter)
        for k in keys[min_indices]:
            compressed_counter[int(k)] = 1
        table = huffman_from_frequencies(compressed_counter)
    return compressed_counter, table


def get_luts(table):
    """dfloat11_utils.py:68-115.  Rows 0..n-2: decode LUTs (row 0 the root), last
    row: code length per symbol.  A code of L bits lives at level (L-1)//8 in
    the LUT named by its first 8*level bits."""
    int_items = [(k, l, v) for k, (l, v) in table.items() if isinstance(k, int)]

    def prefix_of(l, v, level):
        return (level, v >> (l - 8 * level))

    prefixes = [(0, 0)]
    for _, l, v in int_items:
        p = prefix_of(l, v, (l - 1) // 8)
        if p not in prefixes:
            prefixes.append(p)
    prefixes.sort(key=lambda p: p[0])     # stable, by prefix length

    luts = np.zeros((len(prefixes), 256), dtype=np.uint8)
    carried = None                        # `curr_val` leaks across rows in the reference
    for pi, (pl, pv) in enumerate(prefixes):
        entries = {}
        for k, l, v in int_items:
            if l >= 8 * pl and (v >> (l - 8 * pl)) == pv:
                if l == 8 * pl:
                    raise ValueError("a code equals a LUT prefix: table is not prefix-free")
                if (l - 1) // 8 == pl:
                    rem = l - 8 * pl
                    key = (v & ((1 << rem) - 1)) << (8 - rem)
                    value = k
                else:
                    key = (v >> (l - 8 * pl - 8)) & 0xFF
                    value = 256 - prefixes.index(prefix_of(l, v, pl + 1))
                if key in entries and entries[key] != value:
                    raise ValueError(f"Key {key} already exists in {entries}")
                entries[key] = value
        for i in range(256):
            if i in entries:
                carried = entries[i]
            if carried is None:
                raise ValueError("root LUT has no entry at index 0")
            luts[pi, i] = carried
    lens = np.zeros((1, 256), dtype=np.uint8)
    for k, l, _ in int_items:
        lens[0, k] = l
    return np.concatenate((luts, lens), axis=0)


def encode(data, table, bytes_per_thread=BYTES_PER_THREAD, threads_per_block=THREADS_PER_BLOCK):
    """dfloat11_utils.py:118-170, pure Python (small inputs only)."""
    chunk_bits = 8 * bytes_per_thread
    block_bits = chunk_bits * threads_per_block
    encoded, gaps, output_positions = [], [], []
    buffer = size = total_size = element_count = 0

    def note_start():
        if total_size // chunk_bits + 1 > len(gaps):
            gaps.append(total_size % chunk_bits)
        if total_size // block_bits + 1 > len(output_positions):
            output_positions.append(element_count)

    for s in data:
        note_start()
        b, v = table[int(s)]
        buffer = (buffer << b) + v
        size += b
        total_size += b
        element_count += 1
        while size >= 8:
            byte = buffer >> (size - 8)
            encoded.append(byte)
            buffer -= byte << (size - 8)
            size -= 8
    if size > 0:
        note_start()
        b, v = table[EOF]
        buffer = (buffer << b) + v
        size += b
        encoded.append(buffer >> (size - 8) if size >= 8 else buffer << (8 - size))
    output_positions.append(len(data))

    blocks_per_grid = -(-len(encoded) // (threads_per_block * bytes_per_thread))
    gaps = gaps + [0] * (threads_per_block * blocks_per_grid - len(gaps))
    bits = np.zeros(len(gaps) * 5, dtype=np.uint8)
    for i, g in enumerate(gaps):
        for k in range(5):
            bits[5 * i + k] = (g >> (4 - k)) & 1
    return (np.array(encoded, dtype=np.uint8), np.packbits(bits),
            np.array(output_positions, dtype=np.uint32))


def table_arrays(table):
    """(code_len u8[256], code_val u32[256], eof_len, eof_val) for the C entry points."""
    code_len = np.zeros(256, dtype=np.uint8)
    code_val = np.zeros(256, dtype=np.uint32)
    for k, (l, v) in table.items():
        if isinstance(k, int):
            code_len[k] = l
            code_val[k] = v
    eof_len, eof_val = table[EOF] if EOF in table else (0, 0)
    return code_len, code_val, int(eof_len), int(eof_val)


# --------------------------------------------------------------------------
# C restatement bindings
# --------------------------------------------------------------------------
_lib = None


def build_lib():
    subprocess.run(["make", "-s", "-C", _HERE, "libdf11_oracle.so"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build_lib()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.df11o_split.argtypes = [vp, i64, vp, vp]
        L.df11o_split.restype = None
        L.df11o_merge.argtypes = [vp, vp, i64, vp]
        L.df11o_merge.restype = None
        L.df11o_decode_blocks.argtypes = [vp, vp, vp, vp, vp, vp, i32, i64, i64, i64, i64, i64, i64]
        L.df11o_decode_blocks.restype = i32
        L.df11o_decode_sequential.argtypes = [vp, vp, vp, i64, vp, i64, vp]
        L.df11o_decode_sequential.restype = i32
        L.df11o_encode.argtypes = [vp, i64, vp, vp, i32, ctypes.c_uint32,
                                   vp, i64, vp, vp, i64, vp, vp, i64, vp]
        L.df11o_encode.restype = i32
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def c_split(w_u16):
    w = np.ascontiguousarray(w_u16).view(np.uint16)
    e = np.empty(w.size, np.uint8)
    s = np.empty(w.size, np.uint8)
    lib().df11o_split(_p(w), w.size, _p(e), _p(s))
    return e, s


def c_merge(exponent, sign_mantissa):
    e = np.ascontiguousarray(exponent, dtype=np.uint8)
    s = np.ascontiguousarray(sign_mantissa, dtype=np.uint8)
    w = np.empty(e.size, np.uint16)
    lib().df11o_merge(_p(e), _p(s), e.size, _p(w))
    return w


def c_encode(data, table):
    """C restatement of encode(): returns (encoded, gaps, output_positions)."""
    data = np.ascontiguousarray(data, dtype=np.uint8)
    code_len, code_val, eof_len, eof_val = table_arrays(table)
    cap_bytes = data.size * 4 + 16
    cap_blocks = cap_bytes // BLOCK_BYTES + 2
    enc = np.empty(cap_bytes, np.uint8)
    gaps = np.empty(cap_blocks * 320, np.uint8)
    pos = np.empty(cap_blocks + 2, np.uint32)
    nb, ng, npos = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    rc = lib().df11o_encode(_p(data), data.size, _p(code_len), _p(code_val), eof_len, eof_val,
                            _p(enc), cap_bytes, ctypes.byref(nb), _p(gaps), gaps.size,
                            ctypes.byref(ng), _p(pos), pos.size, ctypes.byref(npos))
    if rc != 0:
        raise RuntimeError(f"df11o_encode failed: {rc}")
    return enc[:nb.value].copy(), gaps[:ng.value].copy(), pos[:npos.value].copy()


def c_decode(luts, encoded, sign_mantissa, output_positions, gaps, n_elements=None,
             block_range=None, out=None, stage_elems=0):
    """C restatement of one launch of the reference decode kernel.  Returns the
    BF16 words as uint16.  Raises on the conditions the reference cannot survive."""
    luts = np.ascontiguousarray(luts, dtype=np.uint8)
    encoded = np.ascontiguousarray(encoded, dtype=np.uint8)
    sign_mantissa = np.ascontiguousarray(sign_mantissa, dtype=np.uint8)
    output_positions = np.ascontiguousarray(output_positions).view(np.uint32)
    gaps = np.ascontiguousarray(gaps, dtype=np.uint8)
    n_bytes = encoded.size
    n_elements = sign_mantissa.size if n_elements is None else n_elements
    n_blocks = -(-n_bytes // BLOCK_BYTES)
    if gaps.size < n_blocks * 320:
        raise ValueError("gaps shorter than 320 bytes per block")
    b0, b1 = (0, n_blocks) if block_range is None else block_range
    if out is None:
        out = np.zeros(n_elements, np.uint16)
    rc = lib().df11o_decode_blocks(_p(luts), _p(encoded), _p(sign_mantissa), _p(output_positions),
                                   _p(gaps), _p(out), luts.shape[0], n_bytes, n_elements,
                                   output_positions.size, b0, b1, stage_elems)
    if rc != 0:
        raise RuntimeError(f"df11o_decode_blocks failed: {rc}")
    return out


def c_decode_sequential(table, encoded, sign_mantissa):
    code_len, code_val, _, _ = table_arrays(table)
    encoded = np.ascontiguousarray(encoded, dtype=np.uint8)
    sign_mantissa = np.ascontiguousarray(sign_mantissa, dtype=np.uint8)
    out = np.zeros(sign_mantissa.size, np.uint16)
    rc = lib().df11o_decode_sequential(_p(code_len), _p(code_val), _p(encoded), encoded.size,
                                       _p(sign_mantissa), sign_mantissa.size, _p(out))
    if rc != 0:
        raise RuntimeError(f"df11o_decode_sequential failed: {rc}")
    return out


def compress(w_u16, use_c=True):
    """Whole reference pipeline on one flat BF16 tensor (uint16 view):
    histogram -> <=32-bit Huffman table -> LUTs -> bit packing."""
    exponent, sign_mantissa = split_bf16(w_u16)
    counter = get_counter(exponent)
    _, table = get_32bit_codec(counter)
    luts = get_luts(table)
    enc, gaps, pos = (c_encode if use_c else encode)(exponent, table)
    return dict(luts=luts, encoded_exponent=enc, sign_mantissa=sign_mantissa,
                output_positions=pos, gaps=gaps, table=table)
