"""The library's cheap correctly-rounded division / reciprocal / square root must return the compiler's IEEE
bits: exhaustively for sqrt and x / 0.1f over [2^-96, 2^96] and 0, for 1 / x over [2^-40, 2^40), for n / d over all
2^46 pairs of mantissas, and on ~4e9 hashed and structured pairs with exponents far apart."""
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


@pytest.mark.parametrize("first", range(0, 64, 8))
def test_division_is_correctly_rounded_on_every_pair_of_mantissas(first):
    # the division corrects its quotient once where the compiler's expansion corrects twice; that one correction is
    # enough is a fact about this GPU's reciprocal instruction, checked here on all 2^23 x 2^23 mantissa pairs (eight
    # slices of 2^17 denominators per case, about 5 s each)
    from customnetworklayers_amd._lib import last_error, lib

    out = (ctypes.c_ulonglong * 2)()
    rc = lib.inpaint_selftest_division_pairs(first, 8, out)
    assert rc == 0, last_error()
    pairs = 8 * (1 << 17) * (1 << 23)
    print("slices %d..%d: %d mismatches in %.2e pairs (uncorrected product: %d)" % (first, first + 7, out[0], pairs, out[1]), flush=True)
    assert out[0] == 0
    assert out[1] > pairs // 10  # the comparison does see last-bit errors


def test_stream_bandwidth_diagnostics_report_plausible_rates():
    # the copy and the mixed read / write streams that bench.py quotes beside the published HBM peak: well above what a
    # mistake in the byte count or the timing would leave (1 TB/s), below the peak; bad plane counts are refused
    import torch

    from customnetworklayers_amd._lib import last_error, lib

    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = ctypes.c_double(0)
    assert lib.inpaint_copy_bandwidth(1 << 30, 5, ctypes.byref(g), st) == 0, last_error()
    copy = g.value
    rates = {}
    for nr, nw in ((1, 0), (2, 1), (4, 2)):
        assert lib.inpaint_stream_bandwidth(1 << 29, nr, nw, 5, ctypes.byref(g), st) == 0, last_error()  # far beyond the last-level cache
        rates[(nr, nw)] = g.value
    print("copy %.0f GB/s, streams %s" % (copy, {k: round(v) for k, v in rates.items()}), flush=True)
    for v in [copy] + list(rates.values()):
        assert 1000.0 < v < 8000.0  # (the published peak)
    assert lib.inpaint_stream_bandwidth(1 << 27, 5, 1, 5, ctypes.byref(g), st) != 0
    assert lib.inpaint_stream_bandwidth(1 << 27, 1, 3, 5, ctypes.byref(g), st) != 0
