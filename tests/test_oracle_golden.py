"""The oracle against the numbers the reference records for its own host path.

tests/golden/reference_known_answers.json holds rel-L2 figures printed in the
reference's ERROR_ANALYSIS.md and recorded in its data/*.json bench files; they
depend on the exact generator stream, quantizer rounding rules, dequant
arithmetic and FP64 GEMM, so a dropped term or a wrong tie-break moves them.
"""
import json
import os

import numpy as np
import pytest

import orc

with open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")) as f:
    GOLD = json.load(f)


def _same_printed(value, recorded, digits):
    """`recorded` is `value` at `digits` significant digits.  Machine-printed
    figures (4-5 digits) must match the printf rounding exactly; the 3-digit
    figures were shortened by hand from a longer print, so they get 0.6 of a
    unit in the last place."""
    if digits >= 4:
        return float(f"{value:.{digits - 1}e}") == pytest.approx(recorded, rel=1e-12)
    import math
    unit = 10.0 ** (math.floor(math.log10(abs(recorded))) - (digits - 1))
    return abs(value - recorded) <= 0.6 * unit


@pytest.fixture(scope="module")
def ea_weights():
    ea = GOLD["error_analysis"]
    return orc.normal_weights(ea["N"] * ea["K"], ea["seed"])


def test_error_analysis_group_size_table(ea_weights):
    ea, ea5 = GOLD["error_analysis"], GOLD["error_analysis_5digit"]
    N, K = ea["N"], ea["K"]
    for gs in (8, 16, 32, 64, 128):
        for sym in (True, False):
            p = orc.quantize(ea_weights, N, K, gs, sym)
            wd = orc.dequant_all(p)
            r = orc.rel_l2_f16_vs_f64(ea_weights, wd)
            key = "w4_sym_rel_l2" if sym else "w4_asym_rel_l2"
            if str(gs) in ea[key]:
                assert _same_printed(r, ea[key][str(gs)], 3), (gs, sym, r)
            assert _same_printed(r, ea5[key][str(gs)], 5), (gs, sym, r)
            if sym:
                m = orc.max_abs_f16_vs_f64(ea_weights, wd)
                assert _same_printed(m, ea["w4_sym_max_abs"][str(gs)], 3), (gs, m)


def test_error_analysis_mxfp4(ea_weights):
    ea, ea5 = GOLD["error_analysis"], GOLD["error_analysis_5digit"]
    p = orc.quantize_mx(ea_weights, ea["N"], ea["K"])
    wd = orc.dequant_all_mx(p)
    r = orc.rel_l2_f16_vs_f64(ea_weights, wd)
    assert _same_printed(r, ea["mxfp4_rel_l2"], 3)
    assert _same_printed(r, ea5["mxfp4_rel_l2"], 5)
    assert _same_printed(orc.max_abs_f16_vs_f64(ea_weights, wd), ea["mxfp4_max_abs"], 3)


def test_error_analysis_outliers_and_shapes(ea_weights):
    ea, ea5 = GOLD["error_analysis"], GOLD["error_analysis_5digit"]
    N, K = ea["N"], ea["K"]
    wo = ea_weights.copy()
    for i in orc.uniform_int_stream(ea["outlier_seed"], N * K, N * K // 1000):
        wo[int(i)] *= 20.0
    for gs in (16, 128):
        r = orc.rel_l2_f16_vs_f64(wo, orc.dequant_all(orc.quantize(wo, N, K, gs, True)))
        assert _same_printed(r, ea["outlier_rel_l2"][str(gs)], 3)
        assert _same_printed(r, ea5["outlier_rel_l2"][str(gs)], 5)
    lap = orc.laplace_weights(N * K, ea["laplace_seed"])
    r = orc.rel_l2_f16_vs_f64(lap, orc.dequant_all(orc.quantize(lap, N, K, 128, True)))
    assert _same_printed(r, ea["laplace_rel_l2"], 3) and _same_printed(r, ea5["laplace_rel_l2"], 5)
    uni = orc.uniform_weights(N * K, ea["uniform_seed"])
    r = orc.rel_l2_f16_vs_f64(uni, orc.dequant_all(orc.quantize(uni, N, K, 128, True)))
    assert _same_printed(r, ea["uniform_rel_l2"], 3) and _same_printed(r, ea5["uniform_rel_l2"], 5)


@pytest.mark.parametrize("Ke", [256, 1024, 4096])
def test_error_analysis_gemm_level(Ke):
    """Pins gemm_oracle together with the quantizers: GEMM over quantized W vs
    GEMM over FP16-rounded W, both FP64-accumulated (error_analysis.cpp:150-194)."""
    g = GOLD["error_analysis"]["gemm_level"][str(Ke)]
    M, Ne = 4, 512
    we = orc.normal_weights(Ne * Ke, 0xE110 + Ke)
    x = orc.normal_activations(M * Ke, 0xE220 + Ke)
    w16 = we.astype(np.float32).astype(np.float16).view(np.uint16)
    c16 = orc.gemm_oracle(x, M, Ke, w16, Ne)
    xd = x.view(np.float16).astype(np.float64).reshape(M, Ke)
    csrc = xd @ we.reshape(Ne, Ke).T
    fp16_only = orc.rel_l2(c16, csrc)
    assert _same_printed(fp16_only, g["fp16_vs_fp64"], 3)
    for name, wq in (
        ("w4s32", orc.dequant_all(orc.quantize(we, Ne, Ke, 32, True))),
        ("w4s128", orc.dequant_all(orc.quantize(we, Ne, Ke, 128, True))),
        ("mxfp4", orc.dequant_all_mx(orc.quantize_mx(we, Ne, Ke))),
    ):
        r = orc.rel_l2(orc.gemm_oracle(x, M, Ke, wq, Ne), c16)
        assert _same_printed(r, g[name], 3), (Ke, name, r)
        if Ke == 4096:
            assert _same_printed(r, GOLD["error_analysis_5digit"]["gemm_level_4096"][name], 5)


@pytest.mark.parametrize("case", GOLD["mx_bench"]["cases"], ids=lambda c: f"case{c['i']}")
def test_mx_bench_recorded_format_error(case):
    mb = GOLD["mx_bench"]
    N, K = case["N"], case["K"]
    w = orc.normal_weights(N * K, mb["seed"] + case["i"] * mb["stride"])
    r_mx = orc.rel_l2_f16_vs_f64(w, orc.dequant_all_mx(orc.quantize_mx(w, N, K)))
    r_w4 = orc.rel_l2_f16_vs_f64(w, orc.dequant_all(orc.quantize(w, N, K, 128, True)))
    assert _same_printed(r_mx, case["mxfp4"], 4)
    assert _same_printed(r_w4, case["w4_gs128_sym"], 4)


@pytest.mark.parametrize("case", GOLD["kv_bench"]["cases"], ids=lambda c: f"case{c['i']}")
def test_kv_bench_recorded_cache_error(case):
    """quantize_cache / quantize_cache_f8 + their dequant on the bench's seeded
    caches reproduce the recorded 5-digit figures (K and V pooled)."""
    kb = GOLD["kv_bench"]
    H, S, D, gs = case["H"], case["S"], 128, 128
    seed = kb["seed"] + case["i"] * kb["stride"]
    k = orc.normal_weights(H * S * D, seed)
    v = orc.normal_weights(H * S * D, seed + 1)
    src = np.concatenate([k, v])
    c4 = orc.quantize_cache(k, v, H, S, D, gs, True)
    d4 = np.concatenate([orc.dequant_cache(c4, False).ravel(), orc.dequant_cache(c4, True).ravel()])
    assert _same_printed(orc.rel_l2_f16_vs_f64(src, d4), case["w4"], 5)
    c8 = orc.quantize_cache_f8(k, v, H, S, D, gs)
    d8 = np.concatenate([orc.dequant_cache_f8(c8, False).ravel(), orc.dequant_cache_f8(c8, True).ravel()])
    assert _same_printed(orc.rel_l2_f16_vs_f64(src, d8), case["f8"], 5)
