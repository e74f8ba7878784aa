"""Exhaustive product closure on the CPU, in the design of the reference's own sweep
(lut/test.cc:41-107): every pair of operands built from all 2^14 (sign, exponent, 5-bit mantissa)
patterns, 2^28 products per multiplier, at mantissa width 5.

Three implementations must agree bit for bit (NaNs as a class) on all of them:
  * the reference's compiled functional models (oracle/_ref, built from the reference's own
    lut/FPmultMBM_fast14.inl and lut/Mitchell_14.inl where they lie),
  * the oracle's restatement of those models,
  * the oracle's LUT product (table lookup + exponent / special-case logic), which is what the
    GPU kernels are checked against.
Unlike lut/test.cc:88, operands with a zero exponent field are NOT excluded."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from oracle import cpu
from tests.util import lut_bytes, same_bits_or_both_nan

BITS = 14            # sign + exponent + 5 mantissa bits
SHIFT = 32 - BITS
BLOCK = 1 << 10      # first-operand patterns per task: 2^10 x 2^14 = 2^24 products


def _block(i0):
    i = (np.arange(i0, i0 + BLOCK, dtype=np.uint32) << SHIFT)
    j = (np.arange(1 << BITS, dtype=np.uint32) << SHIFT)
    a = np.repeat(i, 1 << BITS).view(np.float32)
    b = np.tile(j, BLOCK).view(np.float32)
    return a, b


@pytest.mark.parametrize("kind", ["MBM", "MIT"])
def test_all_top_bit_patterns_width5_three_implementations_agree(kind):
    if not cpu.ref_available():
        pytest.skip("oracle/_ref not built (no reference tree at build time)")
    lut32 = cpu.expand_u8(lut_bytes(kind, 5), 5)

    def task(i0):
        a, b = _block(i0)
        model = cpu.model_array(kind, 5, a, b)
        ref = cpu.ref_model_array(kind, 5, a, b)
        lut = cpu.lut_mul_array(lut32, 5, a, b)
        return (int((~same_bits_or_both_nan(model, ref)).sum()), int((~same_bits_or_both_nan(lut, model)).sum()), a.size)

    with ThreadPoolExecutor(max_workers=min(8, cpu.max_threads())) as pool:
        res = list(pool.map(task, range(0, 1 << BITS, BLOCK)))
    assert sum(r[2] for r in res) == 1 << 28
    assert sum(r[0] for r in res) == 0, "oracle model differs from the reference's compiled model"
    assert sum(r[1] for r in res) == 0, "oracle LUT product differs from the functional model"
