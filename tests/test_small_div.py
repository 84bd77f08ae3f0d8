"""The device code divides small numbers by runtime divisors as floor((e + 0.5) * (1 / d)) in float32 (dbk::small_div,
csrc/dbk_common.h): exact for dividends below 2^20 whatever the divisor, with the reciprocal one unit in the last place
off in either direction (the hardware's reciprocal instruction is allowed that much). Checked here by brute force."""
import numpy as np


def test_quotient_by_reciprocal_is_exact_below_2_pow_20():
    e = np.arange(1 << 20, dtype=np.float32)
    exact = np.arange(1 << 20, dtype=np.int64)
    divisors = list(range(1, 200)) + [255, 256, 257, 511, 640, 1000, 1023, 1024, 4095, 4096, 10240, 40960, 65535, 65536, 99991, (1 << 20) - 1]
    for d in divisors:
        inv0 = np.float32(1.0) / np.float32(d)
        for inv in (inv0, np.nextafter(inv0, np.float32(0)), np.nextafter(inv0, np.float32(2))):
            q = ((e + np.float32(0.5)) * inv).astype(np.int64)
            assert np.array_equal(q, exact // d), "divisor %d, reciprocal %r" % (d, inv)
