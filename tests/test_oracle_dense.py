"""Pins of the CPU oracle's dense functions (Q1 quant, G1 accumulate, G3 epilogue, bf16) by checks
that do not retype its formula: the committed golden vectors (made by a numpy brute force, see
tests/golden/make_fixtures.py), float64 identities, int64 products, torch's own bf16 rounding,
and crafted inputs on which a plausible mistake gives a different answer."""
import os

import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import synth

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "dense_small.npz"))
NCASES = 5


def gold(i):
    M, N, K, w8 = [int(v) for v in GOLD[f"c{i}_meta"]]
    return {k: GOLD[f"c{i}_{k}"] for k in ("X", "W", "ws", "q", "a_scale", "S", "C")}, M, N, K, bool(w8)


@pytest.mark.parametrize("i", range(NCASES))
def test_oracle_matches_golden_vectors(i):
    g, M, N, K, w8 = gold(i)
    r = ref.linear(g["X"], g["W"], g["ws"], w8)
    np.testing.assert_array_equal(r["q"], g["q"])
    np.testing.assert_array_equal(r["a_scale"].view(np.uint32), g["a_scale"].view(np.uint32))
    np.testing.assert_array_equal(r["S"], g["S"])
    np.testing.assert_array_equal(r["C"], g["C"])
    np.testing.assert_array_equal(ref.gemm_ref(g["q"], g["W"], w8), g["S"])


def test_bf16_rne_equals_torch_on_every_upper_pattern():
    # every bf16 exponent/mantissa pattern with lower halves that hit below / at / above the tie
    hi = np.arange(65536, dtype=np.uint32) << 16
    for low in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        x = (hi | low).view(np.float32)
        ok = np.isfinite(x)
        want = torch.from_numpy(x[ok].copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        got = synth.f32_to_bf16_bits(x[ok])
        np.testing.assert_array_equal(got, want)
    xs = (hi[::97] | 0x8000).view(np.float32)
    xs = xs[np.isfinite(xs)]
    want = torch.from_numpy(xs.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(ref.bf16_rne(xs), want)


def test_quant_invariants_and_special_rows():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((7, 512)).astype(np.float32) * 3
    x[2] = 0.0                      # all-zero row
    x[3, 17] = 1e4                  # one outlier
    x[4] = 2.5                      # constant row: every code 127
    xb = synth.f32_to_bf16_bits(x)
    xf = synth.bf16_bits_to_f32(xb)
    q, sc = ref.quant_bf16(xb)
    assert np.abs(q.astype(np.int32)).max() <= 127
    for m in range(7):
        amax = np.abs(xf[m]).max()
        if amax == 0:
            assert sc[m] == np.float32(1e-30) and not q[m].any()
            continue
        assert sc[m] == np.float32(amax) / np.float32(127)
        assert abs(int(q[m, np.argmax(np.abs(xf[m]))])) == 127          # the absmax element lands on +-127
        # |q*sc - x| <= sc/2 (plus rounding slack): the codes are the nearest integers
        err = np.abs(q[m].astype(np.float64) * float(sc[m]) - xf[m].astype(np.float64))
        assert err.max() <= (0.5 + 127 * 2.0 ** -22) * float(sc[m])  # f32 rounding of the quotient
    assert (q[4] == 127).all()


def test_quant_rounds_half_to_even_not_half_away():
    # sc = 1 exactly (amax 127): x = k + 0.5 must go to the even neighbour
    x = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 126.5], np.float32)
    q, sc = ref.quant_row_f32(x)
    assert sc == np.float32(1.0)
    np.testing.assert_array_equal(q, np.array([127, 0, 2, 2, 0, -2, -2, 4, 126], np.int8))


def test_quant_divides_instead_of_multiplying_by_reciprocal():
    # rows where x * (1/sc) rounds differently from x / sc would expose a reciprocal shortcut
    rng = np.random.default_rng(11)
    found = 0
    for _ in range(200):
        x = synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(rng.standard_normal(1024).astype(np.float32) * 7))
        amax = np.abs(x).max()
        sc = np.maximum(np.float32(amax) / np.float32(127), np.float32(1e-30))
        by_div = np.rint(np.clip((x / sc).astype(np.float32), -127, 127)).astype(np.int8)
        by_rcp = np.rint(np.clip((x * (np.float32(1) / sc)).astype(np.float32), -127, 127)).astype(np.int8)
        q, s = ref.quant_row_f32(x)
        np.testing.assert_array_equal(q, by_div)
        found += int((by_div != by_rcp).any())
    assert found > 0, "the crafted set never separates divide from reciprocal-multiply"


def test_gemm_scalar_law_equals_int64_product_and_fast_body_twin():
    rng = np.random.default_rng(3)
    for (M, N, K, w8) in [(3, 32, 128, False), (5, 48, 256, True), (17, 16, 640, False), (1, 64, 1152, True)]:
        A = rng.integers(-127, 128, (M, K), dtype=np.int8)
        if w8:
            W = rng.integers(-127, 128, (N, K), dtype=np.int8)
            want = A.astype(np.int64) @ W.astype(np.int64).T
        else:
            codes = rng.integers(-8, 8, (N, K), dtype=np.int8)
            W = synth.pack_w4(codes)
            want = A.astype(np.int64) @ codes.astype(np.int64).T
        np.testing.assert_array_equal(ref.gemm_ref(A, W, w8), want)
        for isa in (0, 1, 2):
            for threads in (1, 3):
                S, used = ref.gemm_fast(A, W, w8, threads=threads, isa=isa)
                np.testing.assert_array_equal(S, want)
        # tile halves == whole (the partition is not numerics)
        S = np.zeros((M, N), np.int32)
        ref.gemm_fast(A, W, w8, tile_lo=0, tile_hi=N // 32, S=S)
        ref.gemm_fast(A, W, w8, tile_lo=N // 32, tile_hi=N // 16, S=S)
        np.testing.assert_array_equal(S, want)


def test_gemm_extremes_stay_inside_int32():
    K = 17408
    A = np.full((1, K), 127, np.int8)
    W = synth.pack_w4(np.full((16, K), -8, np.int8))
    S, _ = ref.gemm_fast(A, W, False)
    assert (S == -127 * 8 * K).all() and abs(int(S[0, 0]) * 16) < 2 ** 31
    W8 = np.full((16, K), -127, np.int8)
    S, _ = ref.gemm_fast(A, W8, True)
    assert (S == -127 * 127 * K).all()


def _epi64(acc, a_s, wsu):
    t = np.float32(np.float64(np.float32(acc)) * np.float64(a_s))
    return int(synth.f32_to_bf16_bits(np.array([np.float32(np.float64(t) * np.float64(wsu))]))[0])


def test_epilogue_is_two_separately_rounded_f32_products_in_that_order():
    rng = np.random.default_rng(9)
    L = ref.lib()
    n = 2_000_000
    acc = rng.integers(-2 ** 28, 2 ** 28, n).astype(np.int32)
    a_s = (np.abs(rng.normal(size=n)) * 0.05 + 1e-3).astype(np.float32)
    wsu = (np.abs(rng.normal(size=n)) * 0.02 + 1e-4).astype(np.float32)
    f = acc.astype(np.float32).astype(np.float64)
    t = (f * a_s.astype(np.float64)).astype(np.float32)
    want = synth.f32_to_bf16_bits((t.astype(np.float64) * wsu.astype(np.float64)).astype(np.float32))
    inner = (a_s.astype(np.float64) * wsu.astype(np.float64)).astype(np.float32)
    other = synth.f32_to_bf16_bits((f * inner.astype(np.float64)).astype(np.float32))   # acc * (as * ws)
    fused = synth.f32_to_bf16_bits((f * a_s.astype(np.float64) * wsu.astype(np.float64)).astype(np.float32))  # one rounding
    pick = np.flatnonzero((other != want) | (fused != want))
    # negative controls: the sample holds inputs on which each plausible mistake changes the bf16
    assert (other != want).any() and (fused != want).any()
    pick = np.concatenate([pick[:300], np.arange(2000)])
    for i in pick:
        assert L.w4a8_epilogue(int(acc[i]), float(a_s[i]), float(wsu[i]), 1) == int(want[i])
        # W4: ws * 0.0625 is exact, so epi(acc, as, 16 * wsu) with w8 = 0 is the same value
        assert L.w4a8_epilogue(int(acc[i]), float(a_s[i]), float(np.float32(wsu[i] * 16)), 0) == int(want[i])


def test_w4_accumulator_conventions_give_the_same_bytes():
    # epi(16*S, ws/16) == epi(S, ws): the x16 of the nibble unpack is exact in f32
    rng = np.random.default_rng(2)
    L = ref.lib()
    for _ in range(3000):
        S = int(rng.integers(-17_700_000, 17_700_000))
        a_s = np.float32(abs(rng.normal()) * 0.05 + 1e-3)
        w_s = np.float32(abs(rng.normal()) * 0.02 + 1e-4)
        assert L.w4a8_epilogue(16 * S, float(a_s), float(w_s), 0) == int(_epi64(S, a_s, w_s))


def test_int32_to_f32_conversion_rounds_to_nearest_even_above_2_24():
    L = ref.lib()
    for acc in (2 ** 24 + 1, 2 ** 24 + 3, 2 ** 27 + 8, -(2 ** 25 + 2), 283_000_001):
        want = int(_epi64(acc, np.float32(1.0), np.float32(1.0)))
        assert L.w4a8_epilogue(acc, 1.0, 1.0, 1) == want
