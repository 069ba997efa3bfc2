"""Seeded BF16 test tensors (as uint16 words) and the product compression pipeline."""
import os

import numpy as np
import torch

from dfloat11_amd import dfloat11_utils as U

KINDS = ("normal", "laplace", "outliers", "uniform256", "zeros", "fib", "single", "high", "sparse", "alphabet100")


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
    if kind == "sparse":          # pruned weights: 70 % exact zeros among N(0, 0.02): one-bit codes next to
        x = rng.standard_normal(n) * 0.02                     # four- to ten-bit ones, 30 and more per chunk
        x[rng.random(n) < 0.7] = 0.0
        return _bf16(x)
    if kind == "alphabet100":     # 100 equally likely exponents: six- and seven-bit codes, one per table
        e = rng.integers(20, 120, n).astype(np.uint16)        # lookup, nine to eleven lookups per chunk
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


def random_prefix_code(rng):
    """A random, possibly incomplete prefix code in the DF11 layout, or None when
    the drawn tree does not fit it (more than 16 sub-tables).  Leaves of a random
    binary tree of depth <= 32; some leaves stay unused, one is the end-of-stream
    code, symbols >= 240 only sit on leaves of 25 bits and more."""
    leaves = [(1, 0), (1, 1)]
    target = int(rng.choice([2, 3, 4, 6, 10, 20, 40, 80]))
    deep_bias = rng.random()
    while len(leaves) < target:
        if rng.random() < deep_bias:
            i = int(np.argmax([l for l, _ in leaves]))
        else:
            i = int(rng.integers(len(leaves)))
        l, v = leaves[i]
        if l >= 32:
            if all(l2 >= 32 for l2, _ in leaves):
                break
            continue
        leaves[i] = (l + 1, v << 1)
        leaves.append((l + 1, (v << 1) | 1))
    rng.shuffle(leaves)
    n_unused = int(rng.integers(0, max(1, len(leaves) // 2)))
    used = leaves[: max(2, len(leaves) - n_unused)]
    eof, used = used[0], used[1:]
    code_len = np.zeros(256, np.uint8)
    code_val = np.zeros(256, np.uint32)
    low = list(rng.permutation(240))
    high = list(rng.permutation(np.arange(240, 256)))
    for l, v in used:
        s = high.pop() if (l >= 25 and high and rng.random() < 0.5) else low.pop()
        code_len[s], code_val[s] = l, v
    codec = U.DF11Codec(code_len, code_val, eof[0], eof[1])
    try:
        luts = U.get_luts(codec.get_code_table()).numpy()
    except ValueError:
        return None
    return codec, luts


def refill_unowned_slots(luts, codec, policy, rng):
    """The same LUT rows with every slot that no code word and no pointer owns
    rewritten: 'forward' = rows start at zero and a slot repeats its predecessor,
    pointers included (the reference builder's forward fill,
    dfloat11_utils.py:103-106); 'random' = any symbol that has a code or any
    pointer to an existing row."""
    code_len, code_val = codec.code_len, codec.code_val
    n_rows = luts.shape[0] - 1
    syms = [s for s in range(256) if code_len[s]]
    prefixes = sorted({(lv, int(code_val[s]) >> (int(code_len[s]) - 8 * lv)) for s in syms
                       for lv in range((int(code_len[s]) - 1) // 8 + 1)})
    assert len(prefixes) == n_rows
    out = luts.copy()
    for pi, (lv, pv) in enumerate(prefixes):
        owned = np.zeros(256, bool)
        for s in syms:
            l, v = int(code_len[s]), int(code_val[s])
            if l <= 8 * lv or (v >> (l - 8 * lv)) != pv:
                continue
            if (l - 1) // 8 == lv:
                rem = l - 8 * lv
                key = (v & ((1 << rem) - 1)) << (8 - rem)
                owned[key:key + (1 << (8 - rem))] = True
            else:
                owned[(v >> (l - 8 * lv - 8)) & 0xFF] = True
        row = out[pi]
        if policy == "forward":
            prev = 0
            for j in range(256):
                if owned[j]:
                    prev = row[j]
                else:
                    row[j] = prev
        elif policy == "random":
            choices = np.array(syms + [256 - r for r in range(1, n_rows)], dtype=np.uint8)
            fill = rng.choice(choices, 256)
            row[~owned] = fill[~owned]
        else:
            raise ValueError(policy)
    return out


def random_code_case(seed, max_n=20_000):
    """(w, streams per fill policy) for a random prefix code, or None."""
    rng = np.random.default_rng(seed)
    made = random_prefix_code(rng)
    if made is None:
        return None
    codec, luts = made
    syms = np.array([s for s in range(256) if codec.code_len[s]], dtype=np.uint8)
    n = int(np.exp(rng.uniform(0, np.log(max_n))))
    p = rng.random(syms.size) ** 3 + 1e-6
    e = rng.choice(syms, n, p=p / p.sum())
    enc, gaps, pos = U.encode(e, codec)
    sm = rng.integers(0, 256, n).astype(np.uint8)
    w = (((sm.astype(np.uint16) & 0x80) << 8) | (e.astype(np.uint16) << 7) | (sm & 0x7F)).astype(np.uint16)
    cases = {}
    for policy in ("product", "forward", "random"):
        l = luts if policy == "product" else refill_unowned_slots(luts, codec, policy, rng)
        cases[policy] = dict(luts=l, encoded_exponent=enc, sign_mantissa=sm, output_positions=pos, gaps=gaps,
                             codec=codec)
    return w, cases


def max_rows_case(seed, n):
    """(w, streams per fill policy) for a hand-made code that needs every LUT row the
    layout has: the root, thirteen second-level rows (first bytes 0xF0..0xFC, 9-bit
    codes), and a chain below first byte 0xFD through a second-, a third- and a
    fourth-level row (17-, 25- and 32-bit codes, the longest for exponents >= 240):
    16 sub-tables, luts of 18 rows.  Exponents are drawn so that long codes are common."""
    rng = np.random.default_rng(seed)
    codes = [(1, 0b0), (2, 0b10), (3, 0b110), (4, 0b1110), (8, 0xFE), (8, 0xFF)]
    for first in range(0xF0, 0xFD):
        codes += [(9, first << 1), (9, (first << 1) | 1)]
    codes += [(9, 0xFD << 1)]                                   # 0xFD 0
    codes += [(17, (0xFDFF << 1))]                              # 0xFD 0xFF 0
    long_codes = [(25, 0xFDFFFF << 1), (32, 0xFDFFFFFE), (30, (0xFDFFFF << 6) | 0b100000)]
    eof = (32, 0xFDFFFFFF)
    code_len = np.zeros(256, np.uint8)
    code_val = np.zeros(256, np.uint32)
    low = list(rng.permutation(240))
    high = list(rng.permutation(np.arange(240, 256)))
    for l, v in codes:
        s = low.pop()
        code_len[s], code_val[s] = l, v
    for l, v in long_codes:
        s = high.pop()
        code_len[s], code_val[s] = l, v
    codec = U.DF11Codec(code_len, code_val, eof[0], eof[1])
    luts = U.get_luts(codec.get_code_table()).numpy()
    assert luts.shape[0] == 18, luts.shape
    syms = np.array([s for s in range(256) if code_len[s]], dtype=np.uint8)
    p = 1.0 / np.sqrt(code_len[syms].astype(np.float64))        # long codes nearly as likely as short ones
    e = rng.choice(syms, n, p=p / p.sum())
    enc, gaps, pos = U.encode(e, codec)
    sm = rng.integers(0, 256, n).astype(np.uint8)
    w = (((sm.astype(np.uint16) & 0x80) << 8) | (e.astype(np.uint16) << 7) | (sm & 0x7F)).astype(np.uint16)
    cases = {}
    for policy in ("product", "forward", "random"):
        l = luts if policy == "product" else refill_unowned_slots(luts, codec, policy, rng)
        cases[policy] = dict(luts=l, encoded_exponent=enc, sign_mantissa=sm, output_positions=pos, gaps=gaps,
                             codec=codec)
    return w, cases


def short_positions_case(oracle, seed, n_full_blocks):
    """A stream laid out by the oracle's restatement of the reference encoder whose
    output_positions comes out one entry short: the last code starts in block
    n_full_blocks - 1, crosses into the next block and ends on a byte boundary, so the
    end-of-stream branch that would note the new block is skipped
    (dfloat11_utils.py:146-162).  The code table is built from a longer run of the same
    data, then the run is cut and its last exponent chosen so that the quirk occurs.
    Returns (w, stream dict) with n_full_blocks + 1 bitstream blocks and as many positions."""
    rng = np.random.default_rng(seed)
    n = 60_000 * n_full_blocks
    p = 0.93 ** np.arange(120)
    e = (rng.choice(120, n, p=p / p.sum()) + 60).astype(np.uint8)
    _, table = oracle.get_32bit_codec(oracle.get_counter(e))
    luts = oracle.get_luts(table)
    lens = luts[-1].astype(np.int64)
    by_len = {int(lens[s]): s for s in range(256) if lens[s]}
    cum = np.cumsum(lens[e])
    boundary = 32768 * n_full_blocks
    i = int(np.searchsorted(cum, boundary))
    while True:
        d = boundary - (int(cum[i - 1]) if i else 0)   # bits left in the block before element i
        if d >= 1 and (d + 8) in by_len:
            break
        i -= 1
    e = e[: i + 1].copy()
    e[i] = by_len[d + 8]                               # ends 8 bits into the next block
    sm = rng.integers(0, 256, e.size).astype(np.uint8)
    enc, gaps, pos = oracle.c_encode(e, table)
    n_blocks = -(-enc.size // 4096)
    assert n_blocks == n_full_blocks + 1 and pos.size == n_blocks and int(pos[-1]) == e.size
    w = oracle.merge_bf16(e, sm)
    return w, dict(luts=luts, encoded_exponent=enc, sign_mantissa=sm, output_positions=pos, gaps=gaps)


def locked_make(directory, *targets):
    """`make` in `directory`, one process at a time: test workers that run in parallel
    would otherwise build the same out-of-date target at once and load half-written files."""
    import fcntl
    import subprocess
    with open(os.path.join(directory, ".make.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        subprocess.run(["make", "-s", "-C", directory, *targets], check=True)
