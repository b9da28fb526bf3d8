"""Pins the oracle's own fp16 <-> fp32 converters (reference: core/mlas/inc/mlas_float16.h:46-86)."""
import numpy as np


def test_widen_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = oracle.C.f16_to_f32(h.view(np.float16))
    want = h.view(np.float16).astype(np.float32)  # numpy's independent conversion
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_narrow_roundtrip_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = h.view(np.float16).astype(np.float32)
    back = oracle.C.f32_to_f16(f).view(np.uint16)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], h[~nan])
    assert np.all(back[nan] & 0x7fff == 0x7e00)  # NaN -> quiet NaN, as the reference does


def test_narrow_rne_against_numpy(oracle):
    rng = np.random.default_rng(7)
    # every midpoint between adjacent halves, and its two fp32 neighbours: the ties and near-ties
    h = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)  # exact: 12 significant bits
    cases = [mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), -mid]
    cases.append(rng.standard_normal(200000).astype(np.float32) * np.float32(100))
    cases.append((rng.standard_normal(100000) * 1e-6).astype(np.float32))   # subnormal halves
    cases.append(np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0**-24, 2.0**-25,
                           np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-26], np.float32))
    f = np.concatenate(cases)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = oracle.C.f32_to_f16(f).view(np.uint16)
    assert np.array_equal(got, want)
