"""The committed DF11 vectors of tests/golden (written by tests/golden/make_fixtures.py
from the CPU oracle; the reference itself holds no vectors for this path)."""
import glob
import os

import numpy as np
import pytest

from tests.df11_cases import compress_product
from tests.test_emulation import emul, run_emul   # noqa: F401  (fixture)

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz")))


def load(path):
    with np.load(path, allow_pickle=False) as z:
        return {k: np.ascontiguousarray(z[k]) for k in z.files}


def test_fixtures_present():
    assert len(GOLDEN) >= 4


@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_oracle_decodes_golden(oracle, path):
    c = load(path)
    out = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
    assert np.array_equal(out, c["weights"])
    # the layout invariants of the format
    n_blocks = -(-c["encoded_exponent"].size // 4096)
    assert c["gaps"].size == 320 * n_blocks and c["output_positions"].size == n_blocks + 1
    assert int(c["output_positions"][-1]) == c["weights"].size and c["luts"].shape[1] == 256


@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_oracle_encoder_still_writes_golden(oracle, path):
    """Byte-for-byte: the oracle's restatement of the reference encoder has not drifted."""
    c = load(path)
    again = oracle.compress(c["weights"])
    for key in ("luts", "encoded_exponent", "sign_mantissa", "gaps"):
        assert np.array_equal(again[key], c[key]), key
    assert np.array_equal(again["output_positions"].astype(np.uint32), c["output_positions"])


@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_kernel_logic_decodes_golden(emul, path):   # noqa: F811
    c = load(path)
    assert np.array_equal(run_emul(emul, c), c["weights"])
    assert np.array_equal(run_emul(emul, c, two_pass=True), c["weights"])


@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_product_encoder_round_trips_golden_weights(oracle, path):
    w = load(path)["weights"]
    c = compress_product(w)
    out = oracle.c_decode(c["luts"], c["encoded_exponent"], c["sign_mantissa"], c["output_positions"], c["gaps"])
    assert np.array_equal(out, w)


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=os.path.basename)
def test_gpu_decodes_golden(path):
    print(f"case golden {os.path.basename(path)}", flush=True)
    from tests.test_gpu_decode import gpu_decode
    c = load(path)
    assert np.array_equal(gpu_decode(c), c["weights"])
