"""Offline DF11 codec with the reference's function names and argument meaning
(reference: dfloat11/dfloat11_utils.py), backed by the native host library.

Differences from the reference, none of which change what a DF11 decoder reads:
  * the prefix code is built natively (Huffman, then optimal length-limited
    codes when the 32-bit or LUT-layout limits require it) with canonical code
    words, instead of dahuffman's heap order; the file carries its own LUTs;
  * symbols >= 240 (|w| >= 2^113, Inf, NaN) are given 25..32-bit codes so the
    LUT layout can hold them, and at most 16 sub-tables are ever produced;
  * output_positions always has one entry per bitstream block plus the final
    element count.
"""
import ctypes

import numpy as np
import torch

from . import _native

BYTES_PER_THREAD = 8
THREADS_PER_BLOCK = 512


class _EndOfStream:
    """Key of the end-of-stream pseudo-symbol in code tables."""

    def __repr__(self):
        return "_EOF"


_EOF = _EndOfStream()


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


class DF11Codec:
    """A prefix code over exponent bytes: code_len[s] bits, value code_val[s]."""

    def __init__(self, code_len, code_val, eof_len, eof_val):
        self.code_len = np.ascontiguousarray(code_len, dtype=np.uint8)
        self.code_val = np.ascontiguousarray(code_val, dtype=np.uint32)
        self.eof_len = int(eof_len)
        self.eof_val = int(eof_val)

    @classmethod
    def from_frequencies(cls, counter):
        hist = np.zeros(256, dtype=np.uint64)
        for k, f in counter.items():
            if not 0 <= int(k) < 256 or int(f) < 0:
                raise ValueError(f"bad histogram entry {k}: {f}")
            hist[int(k)] = int(f)
        code_len = np.zeros(256, dtype=np.uint8)
        code_val = np.zeros(256, dtype=np.uint32)
        eof_len, eof_val = ctypes.c_int32(), ctypes.c_uint32()
        rc = _native.codec_lib().df11_build_code(_ptr(hist), _ptr(code_len), _ptr(code_val),
                                                 ctypes.byref(eof_len), ctypes.byref(eof_val))
        if rc != 0:
            raise ValueError(f"df11_build_code failed with code {rc}")
        return cls(code_len, code_val, eof_len.value, eof_val.value)

    @classmethod
    def from_table(cls, table):
        code_len = np.zeros(256, dtype=np.uint8)
        code_val = np.zeros(256, dtype=np.uint32)
        eof_len = eof_val = 0
        for k, (l, v) in table.items():
            if isinstance(k, (int, np.integer)):
                code_len[int(k)] = l
                code_val[int(k)] = v
            else:
                eof_len, eof_val = l, v
        return cls(code_len, code_val, eof_len, eof_val)

    def get_code_table(self):
        """symbol -> (bits, value), in code-word order, end-of-stream included."""
        items = [(int(s), (int(self.code_len[s]), int(self.code_val[s])))
                 for s in range(256) if self.code_len[s]]
        if self.eof_len:
            items.append((_EOF, (self.eof_len, self.eof_val)))
        items.sort(key=lambda kv: kv[1][1] << (32 - kv[1][0]))
        return dict(items)

    def print_code_table(self):
        print("Bits Code Value Symbol")
        for sym, (l, v) in self.get_code_table().items():
            print(f"{l:4d} {format(v, 'b').rjust(l, '0')} {v} {sym!r}")


def _as_int16_numpy(weight):
    if isinstance(weight, torch.Tensor):
        if weight.dtype != torch.bfloat16:
            raise TypeError(f"expected a bfloat16 tensor, got {weight.dtype}")
        return weight.detach().cpu().contiguous().view(torch.int16).numpy().reshape(-1)
    return np.ascontiguousarray(weight).view(np.int16).reshape(-1)


def get_codec(weight):
    """Exponent histogram and a code for it (dfloat11_utils.py:24-34).
    Returns (codec, counter) with counter = {exponent value: count}."""
    w = _as_int16_numpy(weight)
    hist = np.zeros(256, dtype=np.uint64)
    rc = _native.codec_lib().df11_histogram(_ptr(w), w.size, _ptr(hist), 0)
    if rc != 0:
        raise RuntimeError(f"df11_histogram failed with code {rc}")
    counter = {int(s): int(hist[s]) for s in range(256) if hist[s]}
    return DF11Codec.from_frequencies(counter), counter


def get_32bit_codec(counter):
    """Code with every length <= 32 (dfloat11_utils.py:37-65).
    Returns (codec, counter, table)."""
    codec = DF11Codec.from_frequencies(counter)
    return codec, counter, codec.get_code_table()


def get_luts(table):
    """Hierarchical 256-entry LUTs plus the code-length row (dfloat11_utils.py:68-115)."""
    codec = DF11Codec.from_table(table)
    luts = np.zeros((18, 256), dtype=np.uint8)
    n_luts = ctypes.c_int32()
    rc = _native.codec_lib().df11_build_luts(_ptr(codec.code_len), _ptr(codec.code_val), _ptr(luts),
                                             luts.shape[0], ctypes.byref(n_luts))
    if rc != 0:
        raise ValueError(f"code table cannot be laid out as DF11 LUTs (code {rc})")
    return torch.from_numpy(luts[:n_luts.value].copy())


def encode(data, codec, bytes_per_thread=BYTES_PER_THREAD, threads_per_block=THREADS_PER_BLOCK):
    """Bit-pack exponent bytes (dfloat11_utils.py:118-170).
    Returns (encoded u8, gaps u8, output_positions u32) as numpy arrays."""
    if bytes_per_thread != BYTES_PER_THREAD or threads_per_block != THREADS_PER_BLOCK:
        raise NotImplementedError("only bytes_per_thread=8, threads_per_block=512 are supported")
    data = np.ascontiguousarray(data, dtype=np.uint8).reshape(-1)
    L = _native.codec_lib()
    n_bytes, n_blocks = ctypes.c_int64(), ctypes.c_int64()
    rc = L.df11_encode_size(_ptr(data), data.size, _ptr(codec.code_len), ctypes.byref(n_bytes),
                            ctypes.byref(n_blocks), 0)
    if rc != 0:
        raise ValueError(f"df11_encode_size failed with code {rc} (symbol without a code?)")
    encoded = np.empty(n_bytes.value, dtype=np.uint8)
    gaps = np.empty(n_blocks.value * 320, dtype=np.uint8)
    positions = np.empty(n_blocks.value + 1, dtype=np.uint32)
    rc = L.df11_encode(_ptr(data), data.size, _ptr(codec.code_len), _ptr(codec.code_val),
                       codec.eof_len, codec.eof_val, _ptr(encoded), n_bytes.value, _ptr(gaps),
                       _ptr(positions), n_blocks.value, 0)
    if rc != 0:
        raise RuntimeError(f"df11_encode failed with code {rc}")
    return encoded, gaps, positions


def split_bf16(weight):
    """(exponent u8, sign_mantissa u8) of a flat BF16 tensor (dfloat11_utils.py:175-178)."""
    w = _as_int16_numpy(weight)
    exponent = np.empty(w.size, dtype=np.uint8)
    sign_mantissa = np.empty(w.size, dtype=np.uint8)
    rc = _native.codec_lib().df11_split(_ptr(w), w.size, _ptr(exponent), _ptr(sign_mantissa), 0)
    if rc != 0:
        raise RuntimeError(f"df11_split failed with code {rc}")
    return exponent, sign_mantissa


def encode_weights(weights, codec, bytes_per_thread=BYTES_PER_THREAD, threads_per_block=THREADS_PER_BLOCK):
    """Concatenate flat BF16 weights and compress them (dfloat11_utils.py:173-187).
    Returns (encoded, sign_mantissa, output_positions, gaps, split_positions) as tensors."""
    split_positions = torch.cumsum(torch.LongTensor([w.numel() for w in weights]), dim=0)[:-1]
    combined = torch.cat([w.reshape(-1) for w in weights])
    exponent, sign_mantissa = split_bf16(combined)
    encoded, gaps, positions = encode(exponent, codec, bytes_per_thread, threads_per_block)
    return (torch.from_numpy(encoded), torch.from_numpy(sign_mantissa), torch.from_numpy(positions),
            torch.from_numpy(gaps), split_positions)
