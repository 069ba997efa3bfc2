"""Writes the DF11 regression vectors in this folder.

The reference holds no golden vectors for its decode path and cannot run here
(its kernel is NVIDIA PTX and its encoder needs a package that is not
installed), so these vectors do not come from the reference.  They are written
by the CPU oracle of this repository, which restates the reference's encoder
(dfloat11/dfloat11_utils.py:24-187) and kernel (dfloat11/decode.cu:35-252) and
is itself pinned by tests/test_oracle.py.  They freeze the stream layout: a
change that alters what the oracle, the product encoder's decoder contract or
the HIP kernel make of these bytes shows up as a failing test.

Each case is one .npz (numpy arrays only, loadable with allow_pickle=False):
  weights            u16[n]   BF16 bit patterns that were compressed
  luts               u8[k,256]
  encoded_exponent   u8[n_bytes]
  sign_mantissa      u8[n]
  output_positions   u32[n_blocks + 1]
  gaps               u8[320 * n_blocks]
The expected decode of every case is `weights`.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import df11_oracle as O            # noqa: E402
from tests.df11_cases import make_case         # noqa: E402

CASES = [("normal", 40000, 11), ("outliers", 6000, 12), ("laplace", 14001, 13), ("fib", 5000, 14)]


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    for kind, n, seed in CASES:
        w = make_case(kind, n, seed)
        c = O.compress(w)
        out = O.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
        assert np.array_equal(out, w), kind
        np.savez_compressed(os.path.join(here, f"{kind}_{n}.npz"), weights=w, luts=c["luts"],
                            encoded_exponent=c["encoded_exponent"], sign_mantissa=c["sign_mantissa"],
                            output_positions=c["output_positions"].astype(np.uint32), gaps=c["gaps"])
        print(kind, n, "bytes", c["encoded_exponent"].size, "blocks", c["output_positions"].size - 1)


if __name__ == "__main__":
    main()
