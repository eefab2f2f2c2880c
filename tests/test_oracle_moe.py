"""Pins of the CPU oracle's routed-expert functions (router, expert-major sort, SiLU*up requant,
weighted combine) by independent checks: float64 references with stated bounds, a numpy float32
restatement of the IEEE-only exp, brute-force sorts, and crafted ties."""
import numpy as np
import pytest

from oracle import ref
from saber_engine_amd import synth


def f32(u):
    return np.array([u], np.uint32).view(np.float32)[0]


def exp_nonpos_np(x):
    """Vectorised numpy-float32 restatement of the IEEE-only exp (every op rounds to f32)."""
    x = np.asarray(x, np.float32)
    n = np.rint(x * f32(0x3FB8AA3B)).astype(np.float32)
    r = (x - (n * f32(0x3F317200)).astype(np.float32)).astype(np.float32)
    r = (r - (n * f32(0x35BFBE8E)).astype(np.float32)).astype(np.float32)
    p = np.full_like(x, f32(0x39500D01))
    for c in (0x3AB60B61, 0x3C088889, 0x3D2AAAAB, 0x3E2AAAAB, 0x3F000000):
        p = ((p * r).astype(np.float32) + f32(c)).astype(np.float32)
    p = ((p * r).astype(np.float32) + np.float32(1)).astype(np.float32)
    p = ((p * r).astype(np.float32) + np.float32(1)).astype(np.float32)
    out = np.ldexp(p, n.astype(np.int32)).astype(np.float32)
    return np.where(x > -80, out, np.float32(0)).astype(np.float32)


def test_exp_nonpos_is_exp_within_two_ulp_and_matches_the_f32_restatement():
    L = ref.lib()
    xs = np.concatenate([np.linspace(-79.9, 0, 4001), [-80.0, -81.0, -1e9, -0.0, -1e-7]]).astype(np.float32)
    got = np.array([L.w4a8_exp_nonpos(float(x)) for x in xs], np.float32)
    np.testing.assert_array_equal(got.view(np.uint32), exp_nonpos_np(xs).view(np.uint32))
    live = xs > -80
    true = np.exp(xs[live].astype(np.float64))
    assert np.max(np.abs(got[live] - true) / true) < 3e-7
    assert (got[~live] == 0).all() and got[xs == 0][0] == 1.0


def route_np(logits_bits, topk):
    """Independent router: f32 softmax with the grouped summation tree, brute-force top-k."""
    x = synth.bf16_bits_to_f32(logits_bits)
    T, E = x.shape
    ids = np.zeros((T, topk), np.int32)
    w = np.zeros((T, topk), np.float32)
    for t in range(T):
        p = exp_nonpos_np((x[t] - x[t].max()).astype(np.float32))
        g = np.zeros(E // 16, np.float32)
        for l in range(E // 16):
            s = np.float32(0)
            for j in range(16):
                s = np.float32(s + p[l * 16 + j])
            g[l] = s
        o = E // 32
        while o:
            g = np.array([np.float32(g[l] + g[l ^ o]) for l in range(len(g))], np.float32)
            o //= 2
        q = (p * (np.float32(1) / g[0])).astype(np.float32)
        order = sorted(range(E), key=lambda e: (-q[e], e))[:topk]   # ties: the lower id first
        sel = np.float32(0)
        for e in order:
            sel = np.float32(sel + q[e])
        ids[t] = order
        w[t] = (q[order] * (np.float32(1) / (sel if sel > 0 else np.float32(1)))).astype(np.float32)
    return ids, w


@pytest.mark.parametrize("E,topk", [(128, 8), (512, 10), (16, 2)])
def test_router_matches_independent_restatement(E, topk):
    rng = np.random.default_rng(E)
    lg = synth.f32_to_bf16_bits(rng.standard_normal((24, E)).astype(np.float32))
    ids, w = ref.route(lg, topk)
    ids2, w2 = route_np(lg, topk)
    np.testing.assert_array_equal(ids, ids2)
    np.testing.assert_array_equal(w.view(np.uint32), w2.view(np.uint32))
    assert np.allclose(w.sum(1), 1, atol=1e-6) and (np.diff(w, axis=1) <= 0).all()
    for t in range(24):
        assert len(set(ids[t])) == topk
    # against float64 softmax: the same experts (bf16 logits make near-ties rare) and close weights
    x = synth.bf16_bits_to_f32(lg).astype(np.float64)
    p = np.exp(x - x.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    top = np.take_along_axis(p, ids.astype(np.int64), 1)
    assert np.allclose(w, top / top.sum(1, keepdims=True), rtol=1e-5)


def test_router_tie_rule_lower_expert_id_wins():
    lg = np.zeros((2, 128), np.float32)
    lg[0, [5, 9, 77]] = 2.0          # three equal maxima, then a flat field of equals
    lg[1, :] = -1.0                  # everything equal
    ids, w = ref.route(synth.f32_to_bf16_bits(lg), 8)
    assert ids[0].tolist() == [5, 9, 77, 0, 1, 2, 3, 4]
    assert ids[1].tolist() == list(range(8))
    assert np.allclose(w[1], 1 / 8)


def test_router_refuses_widths_without_a_summation_tree():
    with pytest.raises(ValueError):
        ref.route(np.zeros((1, 48), np.uint16), 2)


@pytest.mark.parametrize("T,E,topk,tb", [(16, 128, 8, 1), (300, 128, 8, 4), (7, 16, 2, 1), (64, 128, 8, 16)])
def test_sort_layout_against_a_stable_sort(T, E, topk, tb):
    rng = np.random.default_rng(T)
    ids = np.stack([rng.choice(E, topk, replace=False) for _ in range(T)]).astype(np.int32)
    lay = ref.sort_layout(ids, E, tb)
    flat = ids.ravel()
    cnt = np.bincount(flat, minlength=E)
    np.testing.assert_array_equal(lay["expert_cnt"], cnt)
    off = np.concatenate([[0], np.cumsum((cnt + 15) // 16 * 16)])
    assert lay["rows"] == off[-1] <= lay["rows_cap"] and lay["tiles"] <= lay["tiles_cap"]
    order = np.argsort(flat, kind="stable")          # expert-major, route (token) order inside
    want_tok = np.full(lay["rows"], -1, np.int32)
    pos = np.zeros(T * topk, np.int32)
    fill = np.zeros(E, np.int64)
    for r in order:
        e = flat[r]
        pos[r] = off[e] + fill[e]
        want_tok[pos[r]] = r // topk
        fill[e] += 1
    np.testing.assert_array_equal(lay["row_tok"], want_tok)
    np.testing.assert_array_equal(lay["route_pos"].ravel(), pos)
    # tiles: one expert each, whole coverage of the live rows, at most 16*tb rows
    covered = []
    for e, r0, rows in zip(lay["tile_expert"], lay["tile_row0"], lay["tile_rows"]):
        assert 0 < rows <= 16 * tb and off[e] <= r0 and r0 + rows <= off[e] + cnt[e] and (r0 - off[e]) % (16 * tb) == 0
        covered += list(range(r0, r0 + rows))
    assert sorted(covered) == sorted(np.flatnonzero(want_tok >= 0).tolist())


def test_geometry_caps_hold_at_the_worst_routing():
    L = ref.lib()
    assert L.w4a8_rows_cap(16, 8, 128) == 2048 and L.w4a8_tiles_cap(16, 8, 128, 1) == 137
    assert L.w4a8_rows_cap(4096, 8, 128) == 34688 and L.w4a8_tiles_cap(4096, 8, 128, 16) == 257
    # every route on its own expert block: the cap is reached, not exceeded
    ids = np.arange(16 * 8, dtype=np.int32).reshape(16, 8) % 128
    lay = ref.sort_layout(ids, 128, 1)
    assert lay["rows"] == 2048 and lay["tiles"] == 128


def test_silu_table_against_float64():
    tab = ref.silu_bf16_table()
    x = synth.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16)).astype(np.float64)
    fin = np.isfinite(x)
    with np.errstate(over="ignore"):
        true = x[fin] / (1 + np.exp(-x[fin]))
    got = synth.bf16_bits_to_f32(tab[fin]).astype(np.float64)
    # one bf16 rounding of a value computed to ~1 ulp of f32: within 2^-8 relative, or below the
    # range where expf(-x) overflows f32 and the law returns -0 (|true| < 1e-36)
    err = np.abs(got - true)
    assert (err <= np.maximum(np.abs(true) * 2.0 ** -8, 1e-36)).all()
    assert tab[0] == 0 and synth.bf16_bits_to_f32(tab[0x3F80:0x3F81])[0] == synth.bf16_bits_to_f32(
        synth.f32_to_bf16_bits(np.array([1 / (1 + np.exp(-1.0))], np.float32)))[0]
    # far negative inputs: -x * e^x underflows to -0 or a tiny negative, never NaN
    assert np.isfinite(synth.bf16_bits_to_f32(tab[fin])).all()


def test_silu_mul_quant_row_composes_table_product_and_quant():
    rng = np.random.default_rng(8)
    I = 256
    gu = synth.f32_to_bf16_bits((rng.standard_normal((5, 2 * I)) * 2).astype(np.float32))
    q, s, p = ref.silu_mul_quant(gu)
    tab = ref.silu_bf16_table()
    t = synth.bf16_bits_to_f32(tab[gu[:, :I]])
    want_p = synth.f32_to_bf16_bits((t.astype(np.float64) * synth.bf16_bits_to_f32(gu[:, I:]).astype(np.float64)).astype(np.float32))
    np.testing.assert_array_equal(p, want_p)
    q2, s2 = ref.quant_bf16(want_p)
    np.testing.assert_array_equal(q, q2)
    np.testing.assert_array_equal(s, s2)


def test_combine_is_an_ordered_f32_sum_with_one_rounding():
    rng = np.random.default_rng(6)
    T, topk, H, rows = 9, 8, 64, 200
    Y = synth.f32_to_bf16_bits(rng.standard_normal((rows, H)).astype(np.float32))
    w = rng.random((T, topk)).astype(np.float32)
    pos = rng.integers(0, rows, (T, topk)).astype(np.int32)
    pos[2, 3] = -1                    # a non-local route contributes nothing
    out = ref.combine(Y, w, pos, H)
    yf = synth.bf16_bits_to_f32(Y)
    acc = np.zeros((T, H), np.float32)
    for k in range(topk):
        live = pos[:, k] >= 0
        pr = (w[:, k, None].astype(np.float64) * yf[np.maximum(pos[:, k], 0)].astype(np.float64)).astype(np.float32)
        acc = np.where(live[:, None], (acc + pr).astype(np.float32), acc)
    np.testing.assert_array_equal(out, synth.f32_to_bf16_bits(acc))
    # order matters at f32: the reversed order differs somewhere, so the check above sees the order
    acc_r = np.zeros((T, H), np.float32)
    for k in reversed(range(topk)):
        live = pos[:, k] >= 0
        pr = (w[:, k, None].astype(np.float64) * yf[np.maximum(pos[:, k], 0)].astype(np.float64)).astype(np.float32)
        acc_r = np.where(live[:, None], (acc_r + pr).astype(np.float32), acc_r)
    assert (acc_r != acc).any()


def test_sigmoid_is_the_logistic_within_rounding_and_matches_the_f32_restatement():
    """The shared expert's gate (hip/moe_route.hip:59-63). Pinned by a numpy-f32 restatement built on the
    pinned exp (bit-equal), by float64 (a few ulp), and by what the function must satisfy whatever the
    exp's last bit: s(0) = 1/2, s(g) + s(-g) = 1 within an ulp, monotone, saturating ends."""
    gs = np.concatenate([np.linspace(-30, 30, 2401), [0.0, -0.0, 1e-8, -1e-8, 90.0, -90.0, 1e30, -1e30]]).astype(np.float32)
    got = ref.sigmoid(gs)
    e = exp_nonpos_np(-np.abs(gs))
    d = (np.float32(1) + e).astype(np.float32)
    want = np.where(gs >= 0, (np.float32(1) / d).astype(np.float32), (e / d).astype(np.float32)).astype(np.float32)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    true = 1.0 / (1.0 + np.exp(-gs.astype(np.float64)))
    live = np.abs(gs) < 60
    assert np.max(np.abs(got[live] - true[live]) / true[live]) < 4e-7
    assert got[gs == 0][0] == 0.5 and got[-2] == 1.0 and got[-1] == 0.0
    half = np.linspace(0, 30, 1201).astype(np.float32)
    assert np.max(np.abs(ref.sigmoid(half) + ref.sigmoid(-half) - 1.0)) <= 1.2e-7
    line = ref.sigmoid(np.linspace(-30, 30, 2401).astype(np.float32))
    assert (np.diff(line) >= 0).all()


def test_combine_shared_adds_the_gated_shared_row_last():
    rng = np.random.default_rng(16)
    T, topk, H, rows = 7, 8, 64, 150
    sh0 = 128
    Y = synth.f32_to_bf16_bits(rng.standard_normal((rows, H)).astype(np.float32))
    w = rng.random((T, topk)).astype(np.float32)
    pos = rng.integers(0, sh0, (T, topk)).astype(np.int32)
    pos[4, 0] = -1
    sgate = synth.f32_to_bf16_bits((3 * rng.standard_normal(T)).astype(np.float32))
    out = ref.combine_shared(Y, w, pos, sgate, sh0, H)
    yf = synth.bf16_bits_to_f32(Y)
    acc = np.zeros((T, H), np.float32)
    for k in range(topk):
        live = pos[:, k] >= 0
        pr = (w[:, k, None].astype(np.float64) * yf[np.maximum(pos[:, k], 0)].astype(np.float64)).astype(np.float32)
        acc = np.where(live[:, None], (acc + pr).astype(np.float32), acc)
    sg = ref.sigmoid(synth.bf16_bits_to_f32(sgate))
    pr = (sg[:, None].astype(np.float64) * yf[sh0:sh0 + T].astype(np.float64)).astype(np.float32)
    np.testing.assert_array_equal(out, synth.f32_to_bf16_bits((acc + pr).astype(np.float32)))
    # without shared rows it is the plain combine; and the shared term is really there
    np.testing.assert_array_equal(ref.combine_shared(Y, w, pos, sgate, -1, H), ref.combine(Y, w, pos, H))
    assert (out != ref.combine(Y, w, pos, H)).any()


def test_moe_layer_equals_per_route_composition():
    c = synth.moe_case(T=6, E=16, topk=2, H=256, I=128, seed=3)
    ids, w = ref.route(c["logits"], 2)
    lay = ref.sort_layout(ids, 16, 1)
    r = ref.moe_layer(c["X"], w, lay, c["Wgu"], c["wsgu"], c["Wdn"], c["wsdn"], 128, taps=True)
    for t in range(6):
        for k in range(2):
            e, p = ids[t, k], lay["route_pos"][t, k]
            a = ref.linear(c["X"][t:t + 1], c["Wgu"][e], c["wsgu"][e], False)
            np.testing.assert_array_equal(r["gu"][p], a["C"][0])
            q2, s2, _ = ref.silu_mul_quant(a["C"])
            S = ref.gemm_ref(q2, c["Wdn"][e], False)
            np.testing.assert_array_equal(r["Y"][p], ref.epilogue(S, s2, c["wsdn"][e], False)[0])
    np.testing.assert_array_equal(r["out"], ref.combine(r["Y"], w, lay["route_pos"], 256))
