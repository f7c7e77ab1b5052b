"""Oracle codecs: bf16, fp8 e4m3 and the fp16 query staging.

Pinned against the reference's own header code where oracle/_ref was built
(dev/tests/engine/Q8PageFormatReference.hpp:66-80, Fp8PageFormatReference.hpp:27-69),
against numpy's IEEE half, and against what the formats fix by definition.
"""
import numpy as np
import pytest

from oracle import kvoracle as ko

L = ko.lib()
needs_ref = pytest.mark.skipif(ko.ref() is None, reason="oracle/_ref not built")


def interesting_floats(n=20000, seed=3):
    rng = np.random.default_rng(seed)
    parts = [rng.standard_normal(n).astype(np.float32),
             (rng.standard_normal(n) * 200).astype(np.float32),
             np.exp(rng.uniform(-40, 12, n)).astype(np.float32) * rng.choice([-1, 1], n).astype(np.float32),
             rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32),
             np.array([0.0, -0.0, 1.0, -3.5, 1e-20, 65504.0, 448.0, 464.0, 480.0, 479.99, 512.0,
                       np.inf, -np.inf, 2.0 ** -6, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10,
                       2.0 ** -14, 2.0 ** -24, 2.0 ** -25, 65519.9, 65520.0], dtype=np.float32)]
    return np.concatenate(parts)


def test_bf16_round_trip_known_answers():
    # dev/tests/engine/q8_paged_kv_test.cc:77-90
    for v in (0.0, -0.0, 1.0, -3.5, 1.0e-20, 65504.0):
        rt = L.ko_bf16_to_float(L.ko_float_to_bf16(v))
        if v == 0.0:
            assert rt == v and np.signbit(np.float32(rt)) == np.signbit(np.float32(v))
        else:
            assert abs(rt - v) <= abs(v) / 128.0
    assert np.isinf(L.ko_bf16_to_float(L.ko_float_to_bf16(float("inf"))))
    assert np.isnan(L.ko_bf16_to_float(L.ko_float_to_bf16(float("nan"))))
    # every bf16 pattern widens and narrows back to itself (NaNs stay NaNs)
    for bits in range(0, 1 << 16):
        f = L.ko_bf16_to_float(bits)
        back = L.ko_float_to_bf16(f)
        assert back == bits or (np.isnan(f) and (back & 0x7F80) == 0x7F80 and back & 0x7F)
    # round to nearest even at the midpoint: 1 + 2^-8 is halfway between two bf16
    assert L.ko_float_to_bf16(np.float32(1.0 + 2.0 ** -8)) == 0x3F80
    assert L.ko_float_to_bf16(np.float32(1.0 + 3 * 2.0 ** -8)) == 0x3F82


def test_numpy_bf16_helper_matches_oracle():
    x = interesting_floats()
    got = ko.f32_to_bf16(x)
    want = np.array([L.ko_float_to_bf16(float(v)) if not np.isnan(v) else 0 for v in x], dtype=np.uint16)
    ok = ~np.isnan(x)
    assert np.array_equal(got[ok], want[ok])
    assert np.array_equal(ko.bf16_to_f32(got[ok]).view(np.uint32), (got[ok].astype(np.uint32) << 16))


@needs_ref
def test_bf16_matches_reference():
    R = ko.ref()
    for v in interesting_floats(6000):
        a, b = L.ko_float_to_bf16(float(v)), R.ref_float_to_bf16(float(v))
        assert a == b, (v, a, b)


def test_fp8_decode_definition_and_round_trip():
    for code in range(256):
        f = L.ko_fp8e4m3_to_float(code)
        e, m, s = (code >> 3) & 15, code & 7, -1.0 if code & 0x80 else 1.0
        if e == 15 and m == 7:
            assert np.isnan(f)
            continue
        want = s * (m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7))
        assert f == want
        enc = L.ko_float_to_fp8e4m3(f)
        assert enc == code or (f == 0 and enc & 0x7F == 0)
    assert L.ko_fp8e4m3_to_float(0x7E) == 448.0


def test_fp8_encode_rounds_to_nearest_even_and_saturates():
    values = sorted({abs(L.ko_fp8e4m3_to_float(c)) for c in range(0x7F)})
    for lo, hi in zip(values, values[1:]):
        mid = (lo + hi) / 2
        clo, chi = L.ko_float_to_fp8e4m3(lo), L.ko_float_to_fp8e4m3(hi)
        cm = L.ko_float_to_fp8e4m3(mid)
        assert cm in (clo, chi) and (cm & 1) == 0  # ties to even mantissa
        assert L.ko_float_to_fp8e4m3(np.nextafter(np.float32(mid), np.float32(0))) == clo
        assert L.ko_float_to_fp8e4m3(np.nextafter(np.float32(mid), np.float32(1e9))) == chi
        assert L.ko_float_to_fp8e4m3(-mid) == cm | 0x80
    for v in (464.0, 479.0, 480.0, 500.0, 512.0, 1e9, float("inf")):
        assert L.ko_float_to_fp8e4m3(v) in (0x7E, 0x7F)
        assert L.ko_float_to_fp8e4m3(v) == (0x7F if np.isinf(v) else 0x7E)
    assert L.ko_float_to_fp8e4m3(463.9) == 0x7E  # below the 448/480 midpoint


@needs_ref
def test_fp8_matches_reference():
    R = ko.ref()
    for c in range(256):
        a, b = L.ko_fp8e4m3_to_float(c), R.ref_fp8_to_float(c)
        assert (np.isnan(a) and np.isnan(b)) or a == b
    for v in interesting_floats(6000):
        if np.isnan(v):
            continue
        assert L.ko_float_to_fp8e4m3(float(v)) == R.ref_float_to_fp8(float(v)), v


def test_f16_rounding_matches_ieee_half():
    x = interesting_floats()
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).astype(np.float32)
    got = np.array([L.ko_round_to_f16(float(v)) for v in x], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@needs_ref
def test_f16_rounding_matches_reference_query_stage():
    R = ko.ref()
    for v in interesting_floats(4000):
        if np.isnan(v):
            continue
        a, b = np.float32(L.ko_round_to_f16(float(v))), np.float32(R.ref_query_stage(float(v)))
        assert a.view(np.uint32) == b.view(np.uint32), v
