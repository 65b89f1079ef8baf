"""Pins the oracle's scalar codecs (CPU only): e4m3 decode/encode, bf16 rounding, expf, silu.

Each check is chosen so that a plausible mistake (wrong bias, wrong tie rule, dropped subnormal
handling, wrong sign of zero) fails it; none of them re-types the oracle's own formula."""
import math

import numpy as np
import pytest
import torch

from oracle import pf8_oracle as O


def test_e4m3_decode_reference_kats():
    """The reference's own known answers (tests/coverage_test/quantization/
    test_coverage_hf_checkpoint_dequant.py:210-219): 0x00,0x01,0x38,0x7E,0xFE,0x7F."""
    got = [O.e4m3_decode(c) for c in (0x00, 0x01, 0x38, 0x7E, 0xFE)]
    assert got == [0.0, 2.0**-9, 1.0, 448.0, -448.0]
    assert math.isnan(O.e4m3_decode(0x7F)) and math.isnan(O.e4m3_decode(0xFF))


def test_e4m3_decode_matches_closed_form_and_torch():
    tab = O.e4m3_table()
    c_dec = np.array([O.e4m3_decode(c) for c in range(256)], dtype=np.float64)
    lib = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    fin = ~np.isnan(tab)
    assert np.array_equal(c_dec[fin], tab[fin]) and np.isnan(c_dec[~fin]).all()
    assert np.array_equal(lib[fin], tab[fin]) and np.isnan(lib[~fin]).all()
    # negative zero keeps its sign
    assert math.copysign(1.0, O.e4m3_decode(0x80)) == -1.0


def _brute_force_encode(v):
    """Nearest-even search over the 254 finite codes, independent of the oracle's bit tricks."""
    tab = O.e4m3_table()
    codes = np.array([c for c in range(128) if not np.isnan(tab[c])])
    vals = tab[codes]
    a = np.abs(v.astype(np.float64))
    out = np.empty(v.shape, np.uint8)
    idx = np.searchsorted(vals, a)          # first grid value >= a
    idx = np.clip(idx, 1, len(vals) - 1)
    lo, hi = vals[idx - 1], vals[idx]
    pick_hi = (a - lo > hi - a) | ((a - lo == hi - a) & (codes[idx] % 2 == 0))
    mag = np.where(pick_hi, codes[idx], codes[idx - 1])
    mag = np.where(a <= vals[0], codes[0], mag)
    mag = np.where(a >= vals[-1], codes[-1], mag)
    out[:] = mag.astype(np.uint8) | (np.signbit(v).astype(np.uint8) << 7)
    return out


def _sweep_values():
    h = np.arange(65536, dtype=np.uint16)
    f = O.bf16_bits_to_f32(h)
    vals = [f]
    with np.errstate(all="ignore"):
        for sc in (0.37, 3.3e-3, 17.0, 448.0, 1 / 448.0, 1.7e-5):
            vals.append((f / np.float32(sc)).astype(np.float32))
    tab = O.e4m3_table()
    grid = np.sort(tab[np.isfinite(tab)]).astype(np.float32)
    mids = ((grid[1:].astype(np.float64) + grid[:-1]) / 2).astype(np.float32)
    for base in (grid, mids):
        vals += [base, np.nextafter(base, np.float32(np.inf)), np.nextafter(base, np.float32(-np.inf))]
    rng = np.random.default_rng(0)
    vals.append((rng.standard_normal(1 << 18) * 100).astype(np.float32))
    v = np.concatenate(vals).astype(np.float32)
    return v[np.isfinite(v)]


def test_e4m3_encode_brute_force_and_torch():
    v = _sweep_values()
    v = v[np.abs(v) <= 448.0]
    enc = O.e4m3_encode_array(v)
    assert np.array_equal(enc, _brute_force_encode(v))
    lib = torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(enc, lib)


def test_e4m3_encode_invariants_and_edges():
    # round trip of every finite code
    for c in range(256):
        if (c & 0x7F) == 0x7F:
            continue
        assert O.e4m3_encode(O.e4m3_decode(c)) == c, hex(c)
    # monotone and sign-symmetric
    v = np.sort(_sweep_values())
    v = v[np.abs(v) <= 448.0]
    dec = O.e4m3_table()[O.e4m3_encode_array(v)]
    assert np.all(np.diff(dec) >= 0)
    assert np.array_equal(O.e4m3_encode_array(-v) ^ 0x80, O.e4m3_encode_array(v))
    # documented edge cases: ties to even, smallest subnormal tie to zero, sign of -tiny
    assert O.e4m3_encode(2.0**-10) == 0x00 and O.e4m3_encode(1.5 * 2.0**-9) == 0x02
    assert O.e4m3_encode(-(2.0**-11)) == 0x80
    assert O.e4m3_decode(O.e4m3_encode(17.0)) == 16.0 and O.e4m3_decode(O.e4m3_encode(19.0)) == 20.0
    assert O.e4m3_encode(448.0) == 0x7E and O.e4m3_encode(463.9) == 0x7E
    # finite overflow saturates (documented deviation from the non-saturating OCP cast), NaN stays NaN
    assert O.e4m3_encode(1e9) == 0x7E and O.e4m3_encode(-1e9) == 0xFE
    assert (O.e4m3_encode(float("nan")) & 0x7F) == 0x7F


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    # force a good share of exact ties
    bits[::7] = (bits[::7] & 0xFFFF0000) | 0x8000
    f = bits.view(np.float32)
    f = f[np.isfinite(f)]
    lib = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16_array(f), lib)
    assert np.array_equal(O.f32_to_bf16_bits(f), lib)
    assert np.array_equal(O.bf16_bits_to_f32(lib), torch.from_numpy(lib.view(np.int16)).view(torch.bfloat16).float().numpy())


def test_expf_within_two_to_the_minus_17_of_libm():
    """The oracle's expf is a short fixed sequence (one rounded product, a degree-4 polynomial): relative error below
    2^-17, which is 500 times finer than the bf16 rounding its results go through."""
    x = np.concatenate([np.linspace(-86.6, 87.3, 200001), np.linspace(-1, 1, 100001)]).astype(np.float32)
    got = O.expf_array(x).astype(np.float64)
    exact = np.exp(x.astype(np.float64))
    assert np.max(np.abs(got / exact - 1.0)) <= 2.0**-17
    assert O.expf(0.0) == 1.0 and O.expf(np.log(2.0)) == 2.0
    # powers of two come out exactly wherever x * log2(e) rounds to the integer
    assert O.expf(float(np.float32(3 * np.log(2.0)))) == 8.0
    # outside the clamp (2^-125 .. 2^126) the value is the clamp's (documented)
    assert O.expf(-200.0) == O.expf(-87.0) == 2.0**-125 and O.expf(200.0) == O.expf(88.5) == 2.0**126


def test_silu_within_one_bf16_ulp_of_float64_and_special_values():
    h = np.arange(65536, dtype=np.uint16)
    g = O.bf16_bits_to_f32(h)
    g = g[np.isfinite(g) & (np.abs(g) <= 80)]
    got = O.silu_array(g).astype(np.float64)
    g64 = g.astype(np.float64)
    exact = g64 / (1 + np.exp(-g64))
    # far inside one bf16 ulp (2^-8 relative): 2^-17 everywhere, 2^-18 where activations live
    rel = np.abs(got - exact) / np.maximum(np.abs(exact), 1e-300)
    assert np.max(rel[exact != 0]) <= 2.0**-17
    assert np.max(rel[(exact != 0) & (np.abs(g) <= 16)]) <= 2.0**-18
    # rounded to bf16, as every use of it is, the result is the correctly rounded one or its neighbour
    got_b, exact_b = O.f32_to_bf16_bits(got.astype(np.float32)).astype(np.int64), O.f32_to_bf16_bits(exact.astype(np.float32)).astype(np.int64)
    assert np.max(np.abs(got_b - exact_b)) <= 1 and np.mean(got_b != exact_b) < 2e-3
    assert O.silu(0.0) == 0.0 and O.silu(30.0) == 30.0
    assert np.signbit(O.silu(-0.0)) and O.silu(-0.0) == 0.0
    assert abs(O.silu(1.0) - 0.7310585786300049) < 1e-6
    assert abs(O.silu(-1.0) + 0.2689414213699951) < 1e-6


def test_scale_rule():
    assert O.scale_from_amax(448.0) == 1.0 and O.scale_from_amax(0.0) == 1.0
    assert O.scale_from_amax(1.0) == np.float32(1.0) / np.float32(448.0)
    # pow2: smallest power of two >= amax/448, exact powers stay
    for amax in (1.0, 3.7, 448.0, 449.0, 1e-3, 7e4):
        s = O.scale_from_amax(amax, True)
        m, _ = math.frexp(s)
        assert m == 0.5 and s >= np.float32(amax) / np.float32(448.0) > s / 2
    assert O.scale_from_amax(448.0 * 4, True) == 4.0


def test_reciprocal_and_residual_division_gives_the_divides_codes_for_every_bf16_pair():
    """The device quantizers replace the per-element IEEE divide x / s by y = 1/s once per tile and
    q0 = x*y, r = fma(-q0, s, x), q = fma(r, y, q0).  Inputs are bf16 and s = amax/448 of a bf16 amax, so the
    claim "same e4m3 code as the divide" is checked on ALL pairs (amax, x <= amax), about 5.2e8 of them, for
    both scale rules.  The fp32 quotients may differ only far below the e4m3 grid."""
    pairs, bad_code, bad_q = O.check_reciprocal_division(pow2=False)
    assert pairs > 500_000_000 and bad_code == 0, (pairs, bad_code, bad_q)
    pairs, bad_code, bad_q = O.check_reciprocal_division(pow2=True)
    assert pairs > 500_000_000 and bad_code == 0 and bad_q == 0, (pairs, bad_code, bad_q)
