"""Seeded random-shape parity sweeps of the hot path against the CPU oracle, through the C ABI: the dense linear
with whatever kernel the launch law picks for the shape, the routed layer, and the row producers. Bit-exact,
like the fixed cases elsewhere; the shapes, magnitudes and special values are drawn so that the corners between
the hand-picked cases get visited (ragged rows and columns, every regime of M, rows whose magnitudes spread over
many orders, infinities, NaN, zeros and denormals in the producers' inputs)."""
import os
import re

import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import DenseRun, assert_dense_matches, dev_bf16_bits, dev_f32, dev_u8, host_u16, say
from tests.test_gpu_chain import SLOTS, Mlp
from tests.test_gpu_moe import check_layer, run_layer
from tests.test_gpu_pair import halves
from tests.test_gpu_pfq import CELLS as PFQ_CELLS, run_pfq

pytestmark = pytest.mark.gpu

ROWS = [1, 2, 3, 4, 5, 8, 15, 16, 17, 31, 33, 48, 49, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 511, 513,
        700, 1000, 1025, 1500, 2048, 2100, 3000]


def test_dense_linear_random_shapes(ctx):
    rng = np.random.default_rng(20240)
    for n in range(160):
        M, w8 = int(rng.choice(ROWS)), bool(rng.integers(0, 2))
        N, K = int(rng.integers(1, 321)) * 16, int(rng.integers(1, 41)) * 128
        if rng.random() < 0.2:
            N = int(rng.choice([5120, 7168, 4352]))
        if rng.random() < 0.2:
            K = int(rng.choice([5120, 17408, 1536, 4096]))
        while M * N * K > 6e9:
            N = max(16, (N // 2) // 16 * 16)
        say(f"sweep dense {n}: M={M} N={N} K={K} w8={w8}")
        case = synth.dense_case(M, N, K, w8=w8, seed=int(rng.integers(0, 1 << 30)))
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        run = DenseRun(ctx, case, want_acc=(M <= 64))
        assert_dense_matches(run, r, w8)
        if iu8.fused_holds(M, K):      # the fused decode linear on the same operands
            c = torch.zeros((M, N), dtype=torch.int16, device="cuda")
            ctx.linear_fused(iu8.W8 if w8 else iu8.W4, run.dev["x"].data_ptr(), run.dev["wf"].data_ptr(), run.dev["ws"].data_ptr(),
                             c.data_ptr(), M, N, K)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(host_u16(c), r["C"])


def test_named_cells_random_shapes(ctx):
    """Every dense cell by its name -- the tile cells at any row count, the streaming cells with K shared over one to
    three workgroups, the `_ks` tile cells, the fused-quant cells -- on random ragged shapes: what the host's
    rule lets through gives the oracle's bytes (and leaves the arrival counters at zero), the rest is refused."""
    rng = np.random.default_rng(20243)
    text = open(os.path.join(iu8.PKG, "csrc", "kernels", "iu8_variants.def")).read()
    names = [n for n in re.findall(r"^IU8_(?:DEC|PF)_VARIANT\((\w+),", text, flags=re.M) if not n.endswith("_acc")]
    split = ["macaq_iu8_pf_w4_t128x128_ks", "macaq_iu8_pf_w8_t128x128_ks", "macaq_iu8_pf_w4_t256x160_ks", "macaq_iu8_pf_w8_t256x160_ks",
             "macaq_iu8_pf_w4_t64x128_s_ks"]
    ran = 0
    for n in range(320):
        kind, ks = str(rng.choice(["pf", "pf", "dec", "ks", "pfq"])), 1
        if kind == "dec":
            name, M, ks = str(rng.choice([x for x in names if "_dec_" in x])), int(rng.integers(1, 65)), int(rng.integers(1, 4))
        elif kind == "ks":
            name, M, ks = str(rng.choice(split)), int(rng.choice([33, 64, 65, 100, 128, 200, 256, 300, 513])), int(rng.integers(1, 5))
        elif kind == "pfq":
            w8 = bool(rng.integers(0, 2))
            name, M = f"macaq_iu8_pfq_{'w8' if w8 else 'w4'}_{rng.choice(PFQ_CELLS[w8])}", int(rng.choice([65, 100, 128, 129, 200, 256, 300, 513, 1000]))
        else:
            name = str(rng.choice([x for x in names if "_pf_" in x]))
            M = int(rng.choice([1, 17, 64, 65, 100, 128, 129, 200, 256, 257, 300, 511, 513, 700, 1025, 2100]))
        w8 = "_w8_" in name
        N, K = int(rng.integers(1, 161)) * 16, int(rng.integers(1, 25)) * 128
        while M * N * K > 3e9:
            N = max(16, (N // 2) // 16 * 16)
        say(f"sweep named {n}: {name} ks={ks} M={M} N={N} K={K}")
        case = synth.dense_case(M, N, K, w8=w8, seed=int(rng.integers(0, 1 << 30)))
        try:
            iu8.describe(name, M, N, K, ks)
        except iu8.IU8Error:
            continue                     # the host's rule: more rows than the cell holds, more shares than K steps
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        if kind == "pfq":
            s, c = run_pfq(ctx, case, name)
            np.testing.assert_array_equal(s.view(np.uint32), r["a_scale"].view(np.uint32))
            np.testing.assert_array_equal(c, r["C"])
        else:
            run = DenseRun(ctx, case, kernel=name, ks=ks, want_acc=False)
            np.testing.assert_array_equal(run.C, r["C"])
            if run.counter is not None:
                assert not run.counter.cpu().numpy().any()
        ran += 1
    assert ran >= 200


def test_one_row_form_random_shapes(ctx):
    """The one-row fused form by name on rows of any length it holds (128 to 20,480), ragged N, any grid the
    host's rule lets through: c and the optional code output equal the oracle's."""
    rng = np.random.default_rng(20248)
    for n in range(60):
        w8 = bool(rng.integers(0, 2))
        tag = "w8" if w8 else "w4"
        N, K = int(rng.integers(1, 200)) * 16, int(rng.integers(1, 161)) * 128
        nblk = (N + 31) // 32
        grid = int(rng.integers(max(1, (nblk + 7) // 8), min(nblk, 256) + 1))
        say(f"sweep one-row {n}: {tag} N={N} K={K} grid={grid}")
        case = synth.dense_case(1, N, K, w8=w8, seed=int(rng.integers(0, 1 << 30)))
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
        d = iu8.describe_raw(f"macaq_iu8_decq_{tag}_r1", (grid, 1, 1), 1024, m=1, n=N, k=K)
        c = torch.full((1, N), 0x7FC0, dtype=torch.int16, device="cuda")
        q = torch.full((iu8.a_bytes(1, K),), 0x55, dtype=torch.uint8, device="cuda")
        s = torch.zeros(1, dtype=torch.float32, device="cuda")
        ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr(), q=q.data_ptr(), scale=s.data_ptr()))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), 1, K), r["q"])
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), r["a_scale"].view(np.uint32))


def test_staged_tile_form_random_shapes(ctx):
    """The persistent GEMV that stages the rows' 16-row tile once a workgroup, by name: 1 to 16 rows of any K it holds
    (128 to 5,120 at 9 to 16 rows, up to 32,768 at one or two), ragged N, any grid the host's rule lets through: c equals the oracle's."""
    rng = np.random.default_rng(20249)
    for n in range(60):
        w8 = bool(rng.integers(0, 2))
        tag = "w8" if w8 else "w4"
        M, N = int(rng.integers(1, 17)), int(rng.integers(1, 300)) * 16
        K = int(rng.integers(1, min(32768, 80 * 1024 // (1 << (M - 1).bit_length())) // 128 + 1)) * 128      # the live rows' codes fit 80 KiB (and the producer's 32,768)
        while M * N * K > 2e9:
            N = max(16, (N // 2) // 16 * 16)
        nblk = (N + 31) // 32
        grid = int(rng.integers(max(1, (nblk + 7) // 8), min(nblk, 256) + 1))
        say(f"sweep staged tile {n}: {tag} M={M} N={N} K={K} grid={grid}")
        case = synth.dense_case(M, N, K, w8=w8, seed=int(rng.integers(0, 1 << 30)))
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
        q = torch.full((iu8.a_bytes(M, K),), 0x55, dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        ctx.quant(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
        d = iu8.describe(f"macaq_iu8_dec_{tag}_tm1_s80" + ("r" if K > 5120 or n % 2 else ""), M, N, K)
        d.grid[0] = grid
        c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
        ctx.launch(d, {"a": q.data_ptr(), "w": wf.data_ptr(), "as": s.data_ptr(), "ws": ws.data_ptr(), "c": c.data_ptr()})
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])


def test_pair_chain_static_gemm_and_back_half_random_shapes(ctx):
    """The decode pair, the decode MLP chain (two launches in a row on one state block), the GEMM on the
    library's static workspace (twice in a row) and the routed layer's back half as two and as three launches."""
    rng = np.random.default_rng(20244)
    for n in range(150):
        kind = str(rng.choice(["pair", "chain", "static", "back", "back"]))
        if kind == "pair":
            M, K = int(rng.integers(1, 49)), int(rng.integers(1, 41)) * 128
            n0, n1 = int(rng.integers(1, 200)) * 16, int(rng.integers(1, 40)) * 16
            say(f"sweep {n}: pair M={M} K={K} N={n0}+{n1}")
            X, (W0, ws0), (W1, ws1) = halves(rng, M, K, n0, n1)
            xd = dev_bf16_bits(X)
            q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
            s = torch.zeros(M, dtype=torch.float32, device="cuda")
            ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
            w0, w1, s0, s1 = dev_u8(iu8.repack_w4(W0)), dev_u8(iu8.repack_w4(W1)), dev_f32(ws0), dev_f32(ws1)
            c0 = torch.full((M, n0), 0x7FC0, dtype=torch.int16, device="cuda")
            c1 = torch.full((M, n1), 0x7FC0, dtype=torch.int16, device="cuda")
            ctx.gemm_pair(q.data_ptr(), s.data_ptr(), w0.data_ptr(), s0.data_ptr(), c0.data_ptr(), n0,
                          w1.data_ptr(), s1.data_ptr(), c1.data_ptr(), n1, M, K)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(host_u16(c0), ref.linear(X, W0, ws0, False, threads=8)["C"])
            np.testing.assert_array_equal(host_u16(c1), ref.linear(X, W1, ws1, False, threads=8)["C"])
        elif kind == "chain":
            M = int(rng.integers(1, 5))
            cap = 20480 // (1 << (M - 1).bit_length()) // 128        # the fused form's staged rows: pow2(M) * width <= 20 KiB
            H, I = int(rng.integers(1, cap + 1)) * 128, int(rng.integers(1, cap + 1)) * 128
            say(f"sweep {n}: chain M={M} H={H} I={I}")
            assert iu8.mlp_chain_holds(M, H, I)
            mlp = Mlp(M, H, I, seed=int(rng.integers(0, 1 << 30)))
            gu, p, c = mlp.oracle()
            for _ in range(2):
                mlp.chain(ctx)
                assert not mlp.state[SLOTS:].any().item()
                np.testing.assert_array_equal(host_u16(mlp.gu), gu)
                np.testing.assert_array_equal(host_u16(mlp.p), p)
                np.testing.assert_array_equal(host_u16(mlp.c), c)
        elif kind == "static":
            M, w8 = int(rng.choice([1, 3, 16, 17, 40, 64, 65, 100, 128, 200, 300])), bool(rng.integers(0, 2))
            N, K = int(rng.integers(1, 200)) * 16, int(rng.integers(1, 137)) * 128
            while M * N * K > 3e9:
                N = max(16, (N // 2) // 16 * 16)
            say(f"sweep {n}: static-workspace GEMM M={M} N={N} K={K} w8={w8}")
            case = synth.dense_case(M, N, K, w8=w8, seed=int(rng.integers(0, 1 << 30)))
            r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
            x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
            q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
            s = torch.zeros(M, dtype=torch.float32, device="cuda")
            c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
            ctx.quant(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
            for _ in range(2):
                ctx.gemm_static(iu8.W8 if w8 else iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), ws.data_ptr(), c.data_ptr(), M, N, K)
                torch.cuda.synchronize()
                np.testing.assert_array_equal(host_u16(c), r["C"])
        else:
            T, H = int(rng.choice([1, 3, 8, 16, 33, 64, 100, 112, 113, 200, 300])), int(rng.choice([256, 512, 1024]))
            I, fused = int(rng.choice([128, 256, 640, 1536])), bool(rng.integers(0, 2))
            say(f"sweep {n}: routed back half T={T} H={H} I={I} two launches={fused}")
            assert iu8.moe_back_holds(1, I)
            case = synth.moe_case(T=T, E=128, topk=8, H=H, I=I, seed=int(rng.integers(0, 1 << 30)), experts=4)
            layer = run_layer(ctx, case, tile_blocks=1, fused_back=fused)
            check_layer(layer, case)
            del layer


def test_routed_layer_random_shapes(ctx):
    rng = np.random.default_rng(20241)
    tokens = [1, 2, 5, 13, 16, 17, 31, 48, 64, 90, 111, 112, 113, 128, 129, 200, 256, 300, 480, 512, 700, 1000, 1500, 2047, 2048, 2500]
    for n in range(60):
        T, H, I = int(rng.choice(tokens)), int(rng.choice([256, 512, 640, 1024])), int(rng.choice([128, 256, 384, 512, 1536]))
        tb = rng.choice([None, None, 1, 8, 16])
        tb = None if tb is None or (T > 600 and tb == 1) else int(tb)
        skew = rng.random() < 0.3
        say(f"sweep routed layer {n}: T={T} H={H} I={I} tile_blocks={tb} skew={skew}")
        case = synth.moe_case(T=T, E=128, topk=8, H=H, I=I, seed=int(rng.integers(0, 1 << 30)), experts=4)
        if skew:      # a few hot experts: long tile runs beside many nearly empty tiles
            lg = synth.bf16_bits_to_f32(case["logits"])
            lg[:, rng.integers(0, 128, size=3)] += np.float32(rng.uniform(1.0, 5.0))
            case["logits"] = synth.f32_to_bf16_bits(lg)
        layer = run_layer(ctx, case, tile_blocks=tb)
        check_layer(layer, case)
        del layer


def test_row_producers_random_shapes(ctx):
    rng = np.random.default_rng(20242)
    tab = torch.zeros(65536, dtype=torch.float32, device="cuda")
    ctx.launch(iu8.describe_raw("mxfp4_hadi8_silu_f32_table", (256, 1, 1), 256, plugin="mxfp4_hadi8"), dict(out=tab.data_ptr()))
    silu_lut = torch.zeros(65536, dtype=torch.int16, device="cuda")
    sig_lut = torch.zeros(65536, dtype=torch.int16, device="cuda")
    ctx.silu_table(silu_lut.data_ptr())
    ctx.sigmoid_table(sig_lut.data_ptr())
    torch.cuda.synchronize()
    silu_tab = tab.cpu().numpy()      # the GDN norm's f32 gate is the card's own expf: its table goes to the oracle

    def outs(M, K):
        return (torch.full((iu8.a_bytes(M, K),), 0x55, dtype=torch.uint8, device="cuda"), torch.zeros(M, dtype=torch.float32, device="cuda"))

    def bits(shape, scale):
        x = (rng.standard_normal(shape) * scale).astype(np.float32)
        if rng.random() < 0.3:        # rows of very different magnitudes
            x *= np.exp(rng.uniform(-12, 6, size=(shape[0], 1))).astype(np.float32)
        b = synth.f32_to_bf16_bits(x)
        if rng.random() < 0.3:        # a few special patterns
            b.reshape(-1)[rng.integers(0, b.size, size=6)] = [0x7F80, 0xFF80, 0x7FC0, 0x0000, 0x8000, 0x0001]
        return b

    def check(q, s, M, K, wq, wsc):
        torch.cuda.synchronize()
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), wq)

    ops = ["quant", "quant_rm", "quant_had", "silu_had", "silu_had_lut", "add_rms", "add_rms", "gdn", "attn", "attn_lut"]
    for n in range(240):
        M, K = int(rng.choice([1, 2, 3, 7, 8, 9, 15, 16, 17, 33, 100, 128, 130, 500, 1024, 1030, 2048])), int(rng.integers(1, 321)) * 64
        if rng.random() < 0.25:
            K = int(rng.choice([5120, 17408, 1536, 4096, 6144, 20480]))
        while M * K > 6e6:
            M = max(1, M // 2)
        op = str(rng.choice(ops))
        say(f"sweep producer {n}: {op} M={M} K={K}")
        t = (rng.choice([-1.0, 1.0], size=K) * rng.uniform(0.5, 2.0, size=K)).astype(np.float32)
        td = dev_f32(t)
        q, s = outs(M, K)
        if op in ("quant", "quant_rm"):
            X = bits((M, K), 2.0)
            xd = dev_bf16_bits(X)
            wq, wsc = ref.quant_bf16(X)
            if op == "quant":
                ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
                check(q, s, M, K, wq, wsc)
            else:
                qr = torch.zeros(M * K, dtype=torch.uint8, device="cuda")
                ctx.quant_rowmajor(xd.data_ptr(), qr.data_ptr(), s.data_ptr(), M, K)
                torch.cuda.synchronize()
                np.testing.assert_array_equal(qr.cpu().numpy().view(np.int8).reshape(M, K), wq)
                np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
        elif op == "quant_had":
            X = bits((M, K), 2.0)
            xd = dev_bf16_bits(X)
            ctx.quant_had(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K, td.data_ptr())
            check(q, s, M, K, *ref.quant_had(X, t))
        elif op in ("silu_had", "silu_had_lut"):
            gu = bits((M, 2 * K), 2.0)
            gd = dev_bf16_bits(gu)
            if op == "silu_had":
                ctx.silu_mul_quant_had(gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K, td.data_ptr())
            else:
                ctx.silu_mul_quant_had_lut(gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K, td.data_ptr(), silu_lut.data_ptr())
            check(q, s, M, K, *ref.silu_mul_quant_had(gu, t))
        elif op == "add_rms":
            y, r = bits((M, K), 1.0), bits((M, K), 4.0)
            w = synth.f32_to_bf16_bits((rng.standard_normal(K) * 0.1).astype(np.float32))
            ro = torch.zeros((M, K), dtype=torch.int16, device="cuda")
            yd, rd, wd = dev_bf16_bits(y), dev_bf16_bits(r), dev_bf16_bits(w)
            ctx.add_rms_quant_had(yd.data_ptr(), rd.data_ptr(), wd.data_ptr(), q.data_ptr(), s.data_ptr(), ro.data_ptr(), M, K, 1e-6, td.data_ptr())
            wq, wsc, wro = ref.add_rms_quant_had(y, r, w, t, 1e-6, 256 if K <= 10240 else 512)
            check(q, s, M, K, wq, wsc)
            np.testing.assert_array_equal(host_u16(ro), wro)
        elif op == "gdn":
            N, pad = max(128, min(K, 10240) // 128 * 128), int(rng.choice([0, 8, 64]))
            q, s = outs(M, N)
            x, z = bits((M, N), 2.0), bits((M, N + pad), 3.0)
            w = synth.f32_to_bf16_bits((1 + rng.standard_normal(128) * 0.1).astype(np.float32))
            t2 = np.resize(t, N).astype(np.float32)
            td2, xd, zd, wd = dev_f32(t2), dev_bf16_bits(x), dev_bf16_bits(z), dev_bf16_bits(w)
            ctx.gdn_norm_quant_had(xd.data_ptr(), zd.data_ptr(), N + pad, wd.data_ptr(), q.data_ptr(), s.data_ptr(), M, N, 1e-6, td2.data_ptr())
            check(q, s, M, N, *ref.gdn_norm_quant_had(x, z[:, :N], w, t2, 1e-6, silu_tab=silu_tab))
        else:
            hd = int(rng.choice([64, 128, 256]))
            n_ = max(1, min(K, 6144) // hd) * hd
            if n_ % 64:
                continue
            q, s = outs(M, n_)
            t2 = np.resize(t, n_).astype(np.float32)
            core, blk = bits((M, n_), 1.0), bits((M, 2 * n_), 3.0)
            td2, cd, gd = dev_f32(t2), dev_bf16_bits(core), dev_bf16_bits(blk)
            if op == "attn":
                ctx.attn_gate_quant_had(cd.data_ptr(), gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, n_, hd, 2 * n_, td2.data_ptr())
            else:
                ctx.attn_gate_quant_had_lut(cd.data_ptr(), gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, n_, hd, 2 * n_, td2.data_ptr(),
                                            sig_lut.data_ptr())
            check(q, s, M, n_, *ref.attn_gate_quant_had(core, blk, t2, hd))
