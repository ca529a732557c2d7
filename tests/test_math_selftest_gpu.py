"""The library's cheap correctly-rounded division / square root must return the compiler's IEEE
bits: exhaustively for sqrt and x / 0.1f over [2^-96, 2^96] and 0, on ~4e9 hashed and structured pairs for n / d."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu


def test_exact_math_matches_ieee_on_the_gpu():
    from customnetworklayers_amd._lib import last_error, lib

    out = (ctypes.c_ulonglong * 4)()
    rc = lib.inpaint_selftest_math(out, 4096)
    assert rc == 0, last_error()
    print("mismatches: sqrt %d, x/0.1 %d, n/d %d, shared-reciprocal n/d %d" % tuple(out), flush=True)
    assert list(out) == [0, 0, 0, 0]


def test_tgv_rsqrt_and_divisions_match_ieee_on_the_gpu():
    from customnetworklayers_amd._lib import last_error, lib

    out = (ctypes.c_ulonglong * 4)()
    rc = lib.inpaint_selftest_rsqrt(out, 4096)
    assert rc == 0, last_error()
    print("mismatches: 1/sqrt %d, x/0.2 %d, 1/m %d, w/h2 %d" % tuple(out), flush=True)
    assert list(out) == [0, 0, 0, 0]
