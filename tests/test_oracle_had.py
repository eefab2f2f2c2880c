"""Pins of the oracle's Hadamard-basis producers (crates/saber-kernels/hip/macaq_had.h,
hip/mxfp4_hadi8.hip): the 32-point transform against the Sylvester matrix, its staged float32
butterfly restated in numpy, invariants, and the producers built on it."""
import numpy as np
import pytest
from scipy.linalg import hadamard

from oracle import ref
from saber_engine_amd import synth

INV = np.uint32(0x3E3504F3).view(np.float32)


def np_butterfly(u):
    """The staged f32 butterfly over element bits 0..4, numpy float32, no help from the oracle."""
    v = u.astype(np.float32).copy()
    for s in (1, 2, 4, 8, 16):
        idx = np.arange(32)
        lo, hi = idx[(idx & s) == 0], idx[(idx & s) == 0] | s
        a, b = v[..., lo] + v[..., hi], v[..., lo] - v[..., hi]
        v[..., lo], v[..., hi] = a, b
    return v * INV


def test_had32_is_the_sylvester_matrix_on_exact_inputs():
    rng = np.random.default_rng(0)
    v = rng.integers(-64, 65, size=(7, 96)).astype(np.float32)      # small integers: every add is exact
    t = rng.choice([-1.0, 1.0], size=96).astype(np.float32)
    got = ref.had32_rows(v, t)
    H = hadamard(32).astype(np.float64)
    for b in range(3):
        want = (v[:, 32 * b:32 * b + 32] * t[32 * b:32 * b + 32]).astype(np.float64) @ H.T
        np.testing.assert_array_equal(got[:, 32 * b:32 * b + 32], (want.astype(np.float32) * INV))
    assert INV == np.float32(1 / np.sqrt(32))


def test_had32_equals_the_staged_float32_butterfly_bit_for_bit():
    rng = np.random.default_rng(1)
    v = (rng.standard_normal((64, 160)) * 3).astype(np.float32)
    t = (rng.standard_normal(160)).astype(np.float32)
    got = ref.had32_rows(v, t)
    want = np_butterfly((v * t).reshape(64, 5, 32)).reshape(64, 160)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    # a different stage order gives other bits somewhere (the order is part of the law)
    w2 = (v * t).reshape(64, 5, 32).astype(np.float32).copy()
    for s in (16, 8, 4, 2, 1):
        idx = np.arange(32)
        lo, hi = idx[(idx & s) == 0], idx[(idx & s) == 0] | s
        a, b = w2[..., lo] + w2[..., hi], w2[..., lo] - w2[..., hi]
        w2[..., lo], w2[..., hi] = a, b
    assert (np.float32(w2 * INV).reshape(64, 160).view(np.uint32) != got.view(np.uint32)).any()


def test_had32_is_orthogonal_and_an_involution():
    rng = np.random.default_rng(2)
    v = rng.standard_normal((16, 64)).astype(np.float32)
    one = np.ones(64, np.float32)
    x = ref.had32_rows(v, one)
    np.testing.assert_allclose((x.astype(np.float64) ** 2).sum(1), (v.astype(np.float64) ** 2).sum(1), rtol=1e-5)
    np.testing.assert_allclose(ref.had32_rows(x, one), v, atol=2e-6)
    # a single spike spreads to +-1/sqrt(32) with the row of the Sylvester matrix as signs
    e = np.zeros((1, 32), np.float32)
    e[0, 5] = 1
    np.testing.assert_array_equal(ref.had32_rows(e, one[:32])[0], hadamard(32)[5].astype(np.float32) * INV)


def test_quant_had_is_the_int8_law_on_the_transformed_row():
    rng = np.random.default_rng(3)
    X = synth.activations(rng, 5, 256)
    t = rng.choice([-1.0, 1.0], size=256).astype(np.float32)
    q, s = ref.quant_had(X, t)
    x = ref.had32_rows(synth.bf16_bits_to_f32(X), t)
    for m in range(5):
        qq, ss = ref.quant_row_f32(x[m])
        np.testing.assert_array_equal(q[m], qq)
        assert s[m] == ss
    # what the transform is for: one outlier a row is spread over its 32-block, the scale shrinks
    Xo = synth.bf16_bits_to_f32(X).copy()
    Xo[:, 17] = 64.0
    Xo = synth.f32_to_bf16_bits(Xo)
    _, s_had = ref.quant_had(Xo, t)
    _, s_plain = ref.quant_bf16(Xo)
    assert (s_had < 0.5 * s_plain).all()


def test_silu_mul_quant_had_composes_the_pinned_pieces():
    rng = np.random.default_rng(4)
    gu = synth.f32_to_bf16_bits(rng.standard_normal((3, 2 * 128)).astype(np.float32) * 2)
    t = rng.choice([-1.0, 1.0], size=128).astype(np.float32)
    q, s = ref.silu_mul_quant_had(gu, t)
    _, _, p = ref.silu_mul_quant(gu)                      # the un-transformed producer's bf16 values
    x = ref.had32_rows(synth.bf16_bits_to_f32(p), t)
    for m in range(3):
        qq, ss = ref.quant_row_f32(x[m])
        np.testing.assert_array_equal(q[m], qq)
        assert s[m] == ss


@pytest.mark.parametrize("threads", [256, 512])
def test_add_rms_quant_had_against_float64(threads):
    rng = np.random.default_rng(5)
    K, eps = 1024, 1e-6
    y = synth.f32_to_bf16_bits(rng.standard_normal((4, K)).astype(np.float32))
    r = synth.f32_to_bf16_bits(rng.standard_normal((4, K)).astype(np.float32))
    w = synth.f32_to_bf16_bits((rng.standard_normal(K) * 0.1).astype(np.float32))
    t = rng.choice([-1.0, 1.0], size=K).astype(np.float32)
    q, s, ro = ref.add_rms_quant_had(y, r, w, t, eps, threads)
    v = synth.bf16_bits_to_f32(y).astype(np.float64) + synth.bf16_bits_to_f32(r).astype(np.float64)
    np.testing.assert_array_equal(ro, synth.f32_to_bf16_bits(v.astype(np.float32)))     # the sum of two bf16 is exact in f32
    inv = 1 / np.sqrt((v ** 2).mean(1, keepdims=True) + eps)
    pre = v * inv * (synth.bf16_bits_to_f32(w).astype(np.float64) + 1)
    x64 = (pre * t).reshape(4, K // 32, 32) @ hadamard(32).T.astype(np.float64) / np.sqrt(32)
    x64 = x64.reshape(4, K)
    # the float64 model differs by bf16 roundings of `pre` (2^-9 relative) spread by the transform
    np.testing.assert_allclose(s, np.abs(x64).max(1) / 127, rtol=2e-2)
    deq = q.astype(np.float64) * s[:, None]
    assert np.abs(deq - x64).max() < 0.6 * s.max() + 0.02 * np.abs(x64).max()
    # the sum tree is part of the law: the two workgroup sizes may differ in the last bit of the scale,
    # never by more
    q2, s2, _ = ref.add_rms_quant_had(y, r, w, t, eps, 768 - threads)
    np.testing.assert_allclose(s, s2, rtol=1e-6)


def _bf16(x):
    return synth.bf16_bits_to_f32(synth.f32_to_bf16_bits(np.asarray(x, np.float32)))


def test_sigmoid_and_silu_tables_against_float64():
    bits = np.arange(65536, dtype=np.uint16)
    g = synth.bf16_bits_to_f32(bits).astype(np.float64)
    ok = np.isfinite(g)
    sig = synth.bf16_bits_to_f32(ref.sigmoid_bf16_table()).astype(np.float64)
    with np.errstate(over="ignore"):
        want = 1 / (1 + np.exp(-g[ok]))
    assert np.abs(sig[ok] - want).max() <= 2.0 ** -9            # one bf16 rounding of a value in [0, 1]
    assert (np.diff(sig[:0x7F80]) >= 0).all()                   # monotone over the non-negative inputs
    assert sig[0] == 0.5 and sig[0x7F80] == 1.0 and sig[0xFF80] == 0.0
    silu = ref.silu_f32_table().astype(np.float64)
    with np.errstate(over="ignore", invalid="ignore"):
        want = g[ok] / (1 + np.exp(-g[ok]))
    fin = np.isfinite(want) & (g[ok] > -88)                     # below, expf(-z) overflows f32 and the law gives -0
    err = np.abs(silu[ok][fin] - want[fin])
    assert (err <= np.maximum(np.abs(want[fin]) * 2.0 ** -22, 1e-44)).all()   # f32 roundings of exp, add, divide
    assert (silu[ok][g[ok] < -89] == 0).all()


def test_attn_gate_quant_had_composes_the_pinned_pieces():
    rng = np.random.default_rng(6)
    M, H, hd = 3, 4, 64
    n = H * hd
    core = synth.f32_to_bf16_bits(rng.standard_normal((M, n)).astype(np.float32))
    block = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * n + 32)) * 3).astype(np.float32))   # a padded row stride
    t = rng.choice([-1.0, 1.0], size=n).astype(np.float32)
    q, s = ref.attn_gate_quant_had(core, block, t, hd)
    gate = block[:, :2 * n].reshape(M, H, 2, hd)[:, :, 1, :].reshape(M, n)      # head h: [q(hd) | gate(hd)]
    sig = synth.bf16_bits_to_f32(ref.sigmoid_bf16_table()[gate])
    p = _bf16(synth.bf16_bits_to_f32(core) * sig)
    x = ref.had32_rows(p, t)
    for m in range(M):
        qq, ss = ref.quant_row_f32(x[m])
        np.testing.assert_array_equal(q[m], qq)
        assert s[m] == ss
    # taking the q half of the block instead gives another result
    wrong = synth.bf16_bits_to_f32(ref.sigmoid_bf16_table()[block[:, :2 * n].reshape(M, H, 2, hd)[:, :, 0, :].reshape(M, n)])
    assert (ref.quant_row_f32(ref.had32_rows(_bf16(synth.bf16_bits_to_f32(core) * wrong), t)[0])[0] != q[0]).any()


def test_gdn_norm_quant_had_against_a_numpy_float32_restatement():
    rng = np.random.default_rng(7)
    M, H, eps = 4, 3, 1e-6
    N = H * 128
    xb = synth.f32_to_bf16_bits((rng.standard_normal((M, N)) * 2).astype(np.float32))
    zb = synth.f32_to_bf16_bits((rng.standard_normal((M, N)) * 2).astype(np.float32))
    wb = synth.f32_to_bf16_bits((1 + rng.standard_normal(128) * 0.1).astype(np.float32))
    t = rng.choice([-1.0, 1.0], size=N).astype(np.float32)
    q, s = ref.gdn_norm_quant_had(xb, zb, wb, t, eps)
    x = synth.bf16_bits_to_f32(xb).reshape(M, H, 16, 8)
    f64 = np.float64

    def fma(a, b, c):       # products of two f32 are exact in f64; the one f64 rounding before the f32
        return (a.astype(f64) * b.astype(f64) + c.astype(f64)).astype(np.float32)    # one is harmless here
    ssq = x[..., 1] * x[..., 1]
    ssq = fma(x[..., 0], x[..., 0], ssq)
    for j in range(2, 8):
        ssq = fma(x[..., j], x[..., j], ssq)
    lanes = np.arange(16)
    for o in (8, 4, 2, 1):
        ssq = ssq + ssq[..., lanes ^ o]
    assert (ssq == ssq[..., :1]).all()                                # every lane holds the same bits
    inv = np.float32(1) / np.sqrt(ssq[..., 0] * np.float32(1 / 128) + np.float32(eps))       # [M, H]
    sg = ref.silu_f32_table()[zb].reshape(M, H, 128)
    w = synth.bf16_bits_to_f32(wb)
    pre = _bf16(((x.reshape(M, H, 128) * inv[..., None]) * w) * sg).reshape(M, N)
    xt = ref.had32_rows(pre, t)
    for m in range(M):
        qq, ss = ref.quant_row_f32(xt[m])
        np.testing.assert_array_equal(q[m], qq)
        assert s[m] == ss
    # and the mathematics: per-head RMS norm times the weight times silu(z), in float64
    x64, z64 = x.reshape(M, H, 128).astype(f64), synth.bf16_bits_to_f32(zb).reshape(M, H, 128).astype(f64)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + eps) * w * (z64 / (1 + np.exp(-z64)))
    np.testing.assert_allclose(pre.reshape(M, H, 128), want, rtol=2.0 ** -7, atol=1e-6)
    # a table handed in replaces the host's libm
    q2, s2 = ref.gdn_norm_quant_had(xb, zb, wb, t, eps, silu_tab=np.zeros(65536, np.float32))
    assert not q2.any() and (s2 == np.float32(1e-30)).all()
