"""Seeded BF16 test tensors (as uint16 words) and the product compression pipeline."""
import numpy as np
import torch

from dfloat11_amd import dfloat11_utils as U

KINDS = ("normal", "laplace", "outliers", "uniform256", "zeros", "fib", "single", "high")


def _bf16(x):
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def make_case(kind, n, seed):
    rng = np.random.default_rng(seed)
    if kind == "normal":
        return _bf16(rng.standard_normal(n) * 0.02)
    if kind == "laplace":
        return _bf16(rng.laplace(0.0, 0.01, n))
    if kind == "outliers":        # N(0, 0.02) with 0.1 % outliers of magnitude in [1, 64]
        x = rng.standard_normal(n) * 0.02
        k = max(1, n // 1000)
        idx = rng.choice(n, k, replace=False)
        x[idx] = rng.uniform(1, 64, k) * rng.choice([-1.0, 1.0], k)
        return _bf16(x)
    if kind == "uniform256":      # every 16-bit pattern equally likely: all 256 exponents
        return rng.integers(0, 1 << 16, n, dtype=np.uint16)
    if kind == "zeros":           # zeros with sparse subnormals: one-bit codes
        w = np.zeros(n, dtype=np.uint16)
        k = max(1, n // 500)
        w[rng.choice(n, k, replace=False)] = rng.integers(1, 128, k).astype(np.uint16)
        return w
    if kind == "fib":             # exact Fibonacci exponent counts: a maximally deep code tree
        fib = [1, 2]                  # (25 symbols / 25+ bits from ~320k elements, the 32-bit
        while sum(fib) + fib[-1] + fib[-2] <= n and len(fib) < 60:   # limit from ~9.3M elements)
            fib.append(fib[-1] + fib[-2])
        exps = rng.permutation(240)[: len(fib)]
        e = np.full(n, exps[-1], dtype=np.uint16)
        rep = np.repeat(exps, fib)[:n]
        e[: rep.size] = rep
        rng.shuffle(e)
        sm = rng.integers(0, 256, n).astype(np.uint16)
        return (((sm & 0x80) << 8) | (e << 7) | (sm & 0x7F)).astype(np.uint16)
    if kind == "single":
        sm = rng.integers(0, 256, n).astype(np.uint16)
        return (((sm & 0x80) << 8) | (np.uint16(121) << 7) | (sm & 0x7F)).astype(np.uint16)
    if kind == "high":            # only exponents >= 240 (huge values, Inf, NaN)
        e = rng.integers(240, 256, n).astype(np.uint16)
        sm = rng.integers(0, 256, n).astype(np.uint16)
        return (((sm & 0x80) << 8) | (e << 7) | (sm & 0x7F)).astype(np.uint16)
    raise ValueError(kind)


def compress_product(w_u16):
    """Product pipeline on a flat BF16 tensor given as uint16 words."""
    w = torch.from_numpy(np.ascontiguousarray(w_u16).view(np.int16)).view(torch.bfloat16)
    codec, counter = U.get_codec(w)
    table = codec.get_code_table()
    luts = U.get_luts(table).numpy()
    exponent, sign_mantissa = U.split_bf16(w)
    enc, gaps, pos = U.encode(exponent, codec)
    return dict(luts=luts, encoded_exponent=enc, sign_mantissa=sign_mantissa,
                output_positions=pos, gaps=gaps, codec=codec, counter=counter, table=table,
                exponent=exponent)


def max_elems_per_block(pos):
    pos = np.asarray(pos).astype(np.int64)
    return int((pos[1:] - pos[:-1]).max()) if pos.size > 1 else 0
