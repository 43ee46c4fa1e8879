"""Pins for the oracle's scalar steps and generators (CPU only).

Each check compares the C oracle with an independent formulation: numpy's
float16 conversions, exact arithmetic in float64 followed by one rounding, a
brute-force nearest-value search, or libstdc++ itself built by g++.
"""
import os
import subprocess

import numpy as np
import pytest

import orc


def _all_halves():
    return np.arange(65536, dtype=np.uint32).astype(np.uint16)


def test_f16_to_f32_exhaustive():
    h = _all_halves()
    got = np.array([orc.lib().orc_f16_to_f32(int(x)) for x in h], np.float32)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.all(np.isnan(got[nan]))


def test_f32_to_f16_rne_dense():
    rng = np.random.default_rng(7)
    # every half value, the midpoints between neighbours, and random floats
    h = _all_halves().view(np.float16).astype(np.float32)
    h = h[np.isfinite(h)]
    mids = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    rnd = rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 200000).astype(np.float32)
    edge = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 1e9, -1e9,
                     2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26,
                     np.inf, -np.inf, 0.1], np.float32)
    xs = np.concatenate([h, mids, np.nextafter(mids, np.float32(np.inf)),
                         np.nextafter(mids, np.float32(-np.inf)), rnd, edge])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([orc.lib().orc_f32_to_f16(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, want)
    assert orc.lib().orc_f32_to_f16(0.1) == 0x2E66
    assert orc.lib().orc_f32_to_f16(float("nan")) & 0x7C00 == 0x7C00


def test_dequant_one_vs_exact_product():
    # RNE_half(s * (q - z)) with the product formed exactly in float64.
    h = _all_halves()
    s = h.view(np.float16).astype(np.float64)
    fin = np.isfinite(s)
    L = orc.lib()
    for d in range(-15, 16):
        with np.errstate(over="ignore"):
            want = (s[fin] * d).astype(np.float16).view(np.uint16)
        q, z = (d, 0) if d >= 0 else (0, -d)
        got = np.array([L.orc_dequant_one(int(x), q, z) for x in h[fin][::7]], np.uint16)
        assert np.array_equal(got, want[::7]), d
    # zero-point form used by symmetric weights
    assert L.orc_dequant_one(0x3C00, 15, 8) == np.float16(7.0).view(np.uint16)
    assert L.orc_dequant_one(0x3C00, 0, 8) == np.float16(-8.0).view(np.uint16)
    assert L.orc_dequant_one(0x0000, 3, 8) == 0x8000  # 0 * -5 = -0


def test_dequant_one_mx_all_codes():
    tab = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    L = orc.lib()
    for se in range(255):  # byte 255 is the NaN scale, never emitted
        for q in range(16):
            v = tab[q & 7] * (-1.0 if q & 8 else 1.0) * 2.0 ** (se - 127)
            with np.errstate(over="ignore", under="ignore"):
                want = np.array([v], np.float64).astype(np.float16).view(np.uint16)[0]
            if (q & 7) == 0:
                want = 0x8000 if q & 8 else 0
            assert L.orc_dequant_one_mx(se, q) == want, (se, q)


def test_decode_f8_table():
    L = orc.lib()
    for b in range(256):
        e, m = (b >> 3) & 15, b & 7
        mag = m / 8.0 * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert L.orc_decode_f8_e4m3(b) == (-mag if b & 0x80 else mag)
    assert L.orc_decode_f8_e4m3(0x7E) == 448.0
    assert L.orc_decode_f8_e4m3(0x7F) == 480.0  # documented, never emitted


def test_e4m3_encode_is_nearest_even():
    L = orc.lib()
    vals = np.array([L.orc_decode_f8_e4m3(b) for b in range(0x7F)])  # 0..448
    rng = np.random.default_rng(3)
    xs = np.concatenate([
        vals, (vals[:-1] + vals[1:]) / 2,
        np.nextafter(((vals[:-1] + vals[1:]) / 2).astype(np.float32), np.float32(np.inf)),
        np.nextafter(((vals[:-1] + vals[1:]) / 2).astype(np.float32), np.float32(0)),
        rng.uniform(0, 460, 20000), 10.0 ** rng.uniform(-6, 3, 20000),
        [448.0, 449.0, 464.0, 1000.0, 1e30, 2.0 ** -10, 2.0 ** -11],
    ]).astype(np.float32)
    for x in xs:
        ax = min(float(x), 448.0)
        d = np.abs(vals - ax)
        best = np.flatnonzero(d == d.min())
        want = int(best[0]) if len(best) == 1 else int([b for b in best if b % 2 == 0][0])
        assert L.orc_f32_to_e4m3_satfinite(float(x)) == want, x
        assert L.orc_f32_to_e4m3_satfinite(-float(x)) == (want | 0x80), x
    assert L.orc_f32_to_e4m3_satfinite(1.0 * 448) == 0x7E


def test_mt19937_64_standard_check_value():
    # [rand.predef]: the 10000th draw of a default-seeded mt19937_64
    assert int(orc.mt_stream(5489, 10000)[-1]) == 9981545732273789042


_CXX = r"""
#include <cstdint>
#include <cstdio>
#include <random>
int main() {
  std::mt19937_64 a(0x44A1); std::normal_distribution<double> d(0.0, 1.0);
  for (int i = 0; i < 1001; ++i) std::printf("%a\n", d(a));
  std::mt19937_64 b(0x0B1E); std::uniform_real_distribution<double> u(-1.0, 1.0);
  for (int i = 0; i < 100; ++i) std::printf("%a\n", u(b));
  std::mt19937_64 c(0x1A9A); std::exponential_distribution<double> e(1.0);
  std::uniform_int_distribution<int> s(0, 1);
  for (int i = 0; i < 100; ++i) { double v = s(c) ? e(c) : -e(c); std::printf("%a\n", v); }
  std::mt19937_64 g(0x07A1); std::uniform_int_distribution<int> pick(0, 512 * 4096 - 1);
  for (int i = 0; i < 100; ++i) std::printf("%d\n", pick(g));
  return 0;
}
"""


def test_generators_match_libstdcxx(tmp_path):
    src = tmp_path / "g.cpp"
    src.write_text(_CXX)
    exe = tmp_path / "g"
    subprocess.check_call(["g++", "-O1", "-std=c++17", str(src), "-o", str(exe)])
    lines = subprocess.check_output([str(exe)]).decode().split()
    n = [float.fromhex(x) for x in lines[:1001]]
    assert np.array_equal(orc.normal_weights(1001, 0x44A1), np.array(n))
    u = [float.fromhex(x) for x in lines[1001:1101]]
    assert np.array_equal(orc.uniform_weights(100, 0x0B1E), np.array(u))
    l = [float.fromhex(x) for x in lines[1101:1201]]
    assert np.array_equal(orc.laplace_weights(100, 0x1A9A), np.array(l))
    p = [int(x) for x in lines[1201:1301]]
    assert np.array_equal(orc.uniform_int_stream(0x07A1, 512 * 4096, 100), np.array(p, np.uint64))
    # activations are the same stream rounded float -> half
    a = orc.normal_activations(1001, 0x44A1)
    with np.errstate(over="ignore"):
        assert np.array_equal(a, np.array(n).astype(np.float32).astype(np.float16).view(np.uint16))
