"""GPU parity of the Hadamard-basis int8 producers (code objects `mxfp4_hadi8`, `attn_glue_hadi8`), through the C ABI,
against the CPU oracle: codes, scales and the residual output, bit for bit."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import dev_bf16_bits, dev_f32, host_u16, say

pytestmark = pytest.mark.gpu


def outs(M, K):
    return (torch.full((iu8.a_bytes(M, K),), 0x55, dtype=torch.uint8, device="cuda"),
            torch.zeros(M, dtype=torch.float32, device="cuda"))


@pytest.mark.parametrize("M,K", [(1, 64), (5, 5120), (16, 17408), (130, 1536), (33, 10240), (3, 10304)])
def test_quant_had(ctx, M, K):
    say(f"quant_had M={M} K={K}")
    rng = np.random.default_rng(M + K)
    X = synth.activations(rng, M, K)
    t = (rng.choice([-1.0, 1.0], size=K) * rng.uniform(0.5, 2.0, size=K)).astype(np.float32)
    q, s = outs(M, K)
    xd, td = dev_bf16_bits(X), dev_f32(t)          # named: the buffers must outlive the launch
    ctx.quant_had(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K, td.data_ptr())
    torch.cuda.synchronize()
    wq, wsc = ref.quant_had(X, t)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), wq)


@pytest.mark.parametrize("M,N", [(2, 128), (40, 1536), (16, 17408)])
def test_silu_mul_quant_had(ctx, M, N):
    say(f"silu_mul_quant_had M={M} N={N}")
    rng = np.random.default_rng(M + N)
    gu = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * N)) * 2).astype(np.float32))
    t = rng.choice([-1.0, 1.0], size=N).astype(np.float32)
    q, s = outs(M, N)
    gd, td = dev_bf16_bits(gu), dev_f32(t)
    ctx.silu_mul_quant_had(gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, N, td.data_ptr())
    torch.cuda.synchronize()
    wq, wsc = ref.silu_mul_quant_had(gu, t)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, N), wq)


@pytest.mark.parametrize("M,N", [(2, 2048), (130, 6144), (33, 10240), (70, 10304), (523, 17408), (19, 20480), (77, 64), (40, 1536)])
def test_silu_mul_quant_had_table_form(ctx, M, N):
    """For rows of SABER_IU8_SILU_LUT_MIN_WIDTH elements and more the launch reads the bf16 silu from the middle
    of the caller's table (both thread counts a row, one to five groups a thread, full and ragged; gates
    outside the table's range -- infinities, NaN, zeros, denormals, huge values -- take the computed branch);
    narrower rows are the computed form. The oracle's bytes either way."""
    say(f"silu_mul_quant_had_lut M={M} N={N}")
    rng = np.random.default_rng(M + N)
    gu = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * N)) * 2).astype(np.float32))
    gu[M // 2, :8] = [0x7F80, 0xFF80, 0x7FC0, 0x0000, 0x8000, 0x7F7F, 0xFF7F, 0x0001]   # gate: inf, -inf, NaN, zeros, extremes
    gu[0, 8:16] = [0x36FF, 0x3700, 0xB6FF, 0xB700, 0x46FF, 0x4700, 0xC6FF, 0xC700]     # both sides of the table's two edges
    t = (rng.choice([-1.0, 1.0], size=N) * rng.uniform(0.5, 2.0, size=N)).astype(np.float32)
    q, s = outs(M, N)
    lut = torch.zeros(65536, dtype=torch.int16, device="cuda")
    ctx.silu_table(lut.data_ptr())
    gd, td = dev_bf16_bits(gu), dev_f32(t)
    ctx.silu_mul_quant_had_lut(gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, N, td.data_ptr(), lut.data_ptr())
    torch.cuda.synchronize()
    wq, wsc = ref.silu_mul_quant_had(gu, t)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, N), wq)
    # ... and the computed form's bytes, whichever of the two the row count picked
    q2, s2 = outs(M, N)
    ctx.silu_mul_quant_had(gd.data_ptr(), q2.data_ptr(), s2.data_ptr(), M, N, td.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(q, q2) and torch.equal(s.view(torch.int32), s2.view(torch.int32))


@pytest.mark.parametrize("M,K", [(3, 256), (20, 5120), (9, 17408)])
def test_add_rms_quant_had(ctx, M, K):
    say(f"add_rms_quant_had M={M} K={K}")
    rng = np.random.default_rng(M + K)
    y = synth.f32_to_bf16_bits(rng.standard_normal((M, K)).astype(np.float32))
    r = synth.f32_to_bf16_bits((rng.standard_normal((M, K)) * 4).astype(np.float32))
    w = synth.f32_to_bf16_bits((rng.standard_normal(K) * 0.1).astype(np.float32))
    t = rng.choice([-1.0, 1.0], size=K).astype(np.float32)
    q, s = outs(M, K)
    ro = torch.zeros((M, K), dtype=torch.int16, device="cuda")
    yd, rd, wd, td = dev_bf16_bits(y), dev_bf16_bits(r), dev_bf16_bits(w), dev_f32(t)
    ctx.add_rms_quant_had(yd.data_ptr(), rd.data_ptr(), wd.data_ptr(), q.data_ptr(), s.data_ptr(), ro.data_ptr(), M, K, 1e-6,
                          td.data_ptr())
    torch.cuda.synchronize()
    wq, wsc, wro = ref.add_rms_quant_had(y, r, w, t, 1e-6, 256 if K <= 10240 else 512)
    np.testing.assert_array_equal(host_u16(ro), wro)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), wq)


@pytest.mark.parametrize("M,K", [(1024, 20480), (700, 5120), (200, 8192), (256, 4160)])
def test_add_rms_quant_had_rows_of_many_magnitudes(ctx, M, K):
    """Many rows whose sums of squares spread over fifteen orders of magnitude: the square root under `inv` must
    be the correctly rounded one on every row (an ulp of `inv` flips a bf16 value of the row once in some
    hundred thousand elements, and with it a code or two of that 32-block)."""
    say(f"add_rms_quant_had, row magnitudes, M={M} K={K}")
    rng = np.random.default_rng(K + M)
    y = synth.f32_to_bf16_bits((rng.standard_normal((M, K)) * np.exp(rng.uniform(-12, 6, size=(M, 1)))).astype(np.float32))
    r = synth.f32_to_bf16_bits((rng.standard_normal((M, K)) * 4 * np.exp(rng.uniform(-12, 6, size=(M, 1)))).astype(np.float32))
    w = synth.f32_to_bf16_bits((rng.standard_normal(K) * 0.1).astype(np.float32))
    t = (rng.choice([-1.0, 1.0], size=K) * rng.uniform(0.5, 2.0, size=K)).astype(np.float32)
    q, s = outs(M, K)
    ro = torch.zeros((M, K), dtype=torch.int16, device="cuda")
    yd, rd, wd, td = dev_bf16_bits(y), dev_bf16_bits(r), dev_bf16_bits(w), dev_f32(t)
    ctx.add_rms_quant_had(yd.data_ptr(), rd.data_ptr(), wd.data_ptr(), q.data_ptr(), s.data_ptr(), ro.data_ptr(), M, K, 1e-6,
                          td.data_ptr())
    torch.cuda.synchronize()
    wq, wsc, wro = ref.add_rms_quant_had(y, r, w, t, 1e-6, 256 if K <= 10240 else 512)
    np.testing.assert_array_equal(host_u16(ro), wro)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), wq)


def tap(ctx, kernel, plugin, dtype):
    """A checker's tap kernel: one value for each of the 65,536 bf16 inputs."""
    out = torch.zeros(65536, dtype=dtype, device="cuda")
    ctx.launch(iu8.describe_raw(kernel, (256, 1, 1), 256, plugin=plugin), dict(out=out.data_ptr()))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_device_sigmoid_equals_host_formula_on_all_65536_inputs(ctx):
    say("sigmoid table, all bf16 inputs")
    got = tap(ctx, "attn_glue_hadi8_sigmoid_bf16_table", "attn_glue_hadi8", torch.int16).view(np.uint16)
    want = ref.sigmoid_bf16_table()
    fin = np.isfinite(synth.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16)))
    bad = np.flatnonzero(fin & (got != want))
    assert bad.size == 0, [(hex(i), hex(got[i]), hex(want[i])) for i in bad[:8]]


def device_silu_f32_table(ctx):
    return tap(ctx, "mxfp4_hadi8_silu_f32_table", "mxfp4_hadi8", torch.float32)


def test_device_silu_f32_is_within_an_ulp_of_the_host_formula(ctx):
    """The f32 gate of gdn_norm carries the device's expf: held against the host's libm value to
    2 units in the last place over every finite bf16 input (and reported: how many differ)."""
    say("silu f32 table, all bf16 inputs")
    got, want = device_silu_f32_table(ctx), ref.silu_f32_table()
    x = synth.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16))
    fin = np.isfinite(x) & np.isfinite(want)
    gi, wi = got.view(np.int32).astype(np.int64), want.view(np.int32).astype(np.int64)
    d = np.abs(gi - wi)[fin]
    say(f"silu f32: {int((d != 0).sum())} of {int(fin.sum())} inputs differ from libm, max {int(d.max())} ulp")
    assert d.max() <= 2


@pytest.mark.parametrize("M,H,zs_pad", [(1, 1, 0), (7, 48, 64), (130, 16, 0), (3, 80, 8)])
def test_gdn_norm_quant_had(ctx, M, H, zs_pad):
    N = H * 128
    say(f"gdn_norm_quant_had M={M} N={N} z stride {N + zs_pad}")
    rng = np.random.default_rng(M + N)
    x = synth.f32_to_bf16_bits((rng.standard_normal((M, N)) * 2).astype(np.float32))
    zfull = synth.f32_to_bf16_bits((rng.standard_normal((M, N + zs_pad)) * 3).astype(np.float32))
    w = synth.f32_to_bf16_bits((1 + rng.standard_normal(128) * 0.1).astype(np.float32))
    t = rng.choice([-1.0, 1.0], size=N).astype(np.float32)
    q, s = outs(M, N)
    xd, zd, wd, td = dev_bf16_bits(x), dev_bf16_bits(zfull), dev_bf16_bits(w), dev_f32(t)
    ctx.gdn_norm_quant_had(xd.data_ptr(), zd.data_ptr(), N + zs_pad, wd.data_ptr(), q.data_ptr(), s.data_ptr(), M, N, 1e-6,
                           td.data_ptr())
    torch.cuda.synchronize()
    # the gate's f32 values are the card's own (its expf), tabled by the tap kernel
    wq, wsc = ref.gdn_norm_quant_had(x, zfull[:, :N], w, t, 1e-6, silu_tab=device_silu_f32_table(ctx))
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, N), wq)


@pytest.mark.parametrize("M,H,hd,pad", [(1033, 24, 256, 0), (1024, 16, 128, 96), (1100, 48, 128, 0), (1030, 8, 128, 0), (40, 40, 128, 0)])
def test_attn_gate_quant_had_table_form(ctx, M, H, hd, pad):
    """The gate read from the middle of the product's own table (saber_iu8_sigmoid_table), gates outside it
    computed; narrow rows and few rows take the computed kernel. The computed form's bytes and the oracle's."""
    n = H * hd
    say(f"attn_gate_quant_had_lut M={M} n={n} hd={hd} gate stride {2 * n + pad}")
    rng = np.random.default_rng(M + n + hd + 1)
    core = synth.f32_to_bf16_bits(rng.standard_normal((M, n)).astype(np.float32))
    block = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * n + pad)) * 3).astype(np.float32))
    block[M // 2, hd:hd + 12] = [0x7F80, 0xFF80, 0x7FC0, 0x0000, 0x8000, 0x7F7F, 0xFF7F, 0x0001, 0x36FF, 0x3700, 0xC6FF, 0xC700]
    t = rng.choice([-1.0, 1.0], size=n).astype(np.float32)
    lut = torch.zeros(65536, dtype=torch.int16, device="cuda")
    ctx.sigmoid_table(lut.data_ptr())
    cd, gd, td = dev_bf16_bits(core), dev_bf16_bits(block), dev_f32(t)
    q, s = outs(M, n)
    ctx.attn_gate_quant_had_lut(cd.data_ptr(), gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, n, hd, 2 * n + pad, td.data_ptr(),
                                lut.data_ptr())
    q2, s2 = outs(M, n)
    ctx.attn_gate_quant_had(cd.data_ptr(), gd.data_ptr(), q2.data_ptr(), s2.data_ptr(), M, n, hd, 2 * n + pad, td.data_ptr())
    torch.cuda.synchronize()
    assert torch.equal(q, q2) and torch.equal(s.view(torch.int32), s2.view(torch.int32))
    wq, wsc = ref.attn_gate_quant_had(core, block, t, hd)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, n), wq)


@pytest.mark.parametrize("M,H,hd,pad", [(1, 1, 64, 0), (9, 24, 256, 0), (140, 16, 128, 96), (2, 48, 128, 0)])
def test_attn_gate_quant_had(ctx, M, H, hd, pad):
    n = H * hd
    say(f"attn_gate_quant_had M={M} n={n} hd={hd} gate stride {2 * n + pad}")
    rng = np.random.default_rng(M + n + hd)
    core = synth.f32_to_bf16_bits(rng.standard_normal((M, n)).astype(np.float32))
    block = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * n + pad)) * 3).astype(np.float32))
    t = rng.choice([-1.0, 1.0], size=n).astype(np.float32)
    q, s = outs(M, n)
    cd, gd, td = dev_bf16_bits(core), dev_bf16_bits(block), dev_f32(t)
    ctx.attn_gate_quant_had(cd.data_ptr(), gd.data_ptr(), q.data_ptr(), s.data_ptr(), M, n, hd, 2 * n + pad, td.data_ptr())
    torch.cuda.synchronize()
    wq, wsc = ref.attn_gate_quant_had(core, block, t, hd)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, n), wq)


@pytest.mark.parametrize("M,H", [(5, 40), (16, 136), (3, 80), (9, 48), (300, 32)])
def test_every_form_of_the_producers_by_name(ctx, M, H):
    """Each producer in each of its workgroup sizes, launched by kernel name (the reference's `_t256` / `_t512`
    symbols are what its host launches at any row count; the `_t1024` forms are what this library's law picks for
    few long rows): the oracle's bytes from every one."""
    W = H * 128
    say(f"had producers by name M={M} W={W}")
    rng = np.random.default_rng(M * 7 + W)
    t = (rng.choice([-1.0, 1.0], size=W) * rng.uniform(0.5, 2.0, size=W)).astype(np.float32)
    td = dev_f32(t)
    sizes = [T for T in (256, 512, 1024) if W <= 40 * T]

    def check(name, plugin, T, bufs, want, scalars, eps=None):
        q, s = outs(M, W)
        d = iu8.describe_raw(name, (M, 1, 1), T, plugin=plugin, **scalars)
        if eps is not None:
            d.arg("eps").kind, d.arg("eps").fval = iu8.ARG_F32, eps
        ctx.launch(d, dict(bufs, q=q.data_ptr(), scale=s.data_ptr(), had_t=td.data_ptr()))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), want[1].view(np.uint32), err_msg=name)
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, W), want[0], err_msg=name)

    X = synth.activations(rng, M, W)
    xd = dev_bf16_bits(X)
    want = ref.quant_had(X, t)
    for T in sizes:
        check(f"quant_hadi8_t{T}" + ("" if T == 1024 else "_tiled1"), "mxfp4_hadi8", T, dict(x=xd.data_ptr()), want, dict(k=W))
    gu = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * W)) * 2).astype(np.float32))
    gu[M // 2, :4] = [0x7F80, 0x7FC0, 0x0000, 0xC700]
    gd = dev_bf16_bits(gu)
    lut = torch.zeros(65536, dtype=torch.int16, device="cuda")
    ctx.silu_table(lut.data_ptr())
    want = ref.silu_mul_quant_had(gu, t)
    for T in sizes:
        check(f"silu_mul_quant_hadi8_t{T}" + ("" if T == 1024 else "_tiled1"), "mxfp4_hadi8", T, dict(gu=gd.data_ptr()), want, dict(n=W))
        check(f"silu_mul_quant_hadi8_lut_t{T}", "mxfp4_hadi8", T, dict(gu=gd.data_ptr(), lut=lut.data_ptr()), want, dict(n=W))
    # add_rms: its sum of squares is a tree over 256 threads (rows up to 10,240) or 512 (above); the 16-wave form for
    # rows up to 8,192 hands the 256-thread form's chains through LDS, so it is held to that form's oracle
    res = synth.f32_to_bf16_bits((rng.standard_normal((M, W)) * 4).astype(np.float32))
    wn = synth.f32_to_bf16_bits((rng.standard_normal(W) * 0.1).astype(np.float32))
    rd, wnd = dev_bf16_bits(res), dev_bf16_bits(wn)
    for name, T in [("add_rms_quant_hadi8_t256_tiled1", 256)] * (W <= 10240) + [("add_rms_quant_hadi8_t512_tiled1", 512)] * (W > 10240) + \
                   [("add_rms_quant_hadi8_t1024", 1024)] * (W <= 8192):
        wq, wsc, wro = ref.add_rms_quant_had(X, res, wn, t, 1e-6, 256 if W <= 10240 else 512)
        ro = torch.zeros((M, W), dtype=torch.int16, device="cuda")
        check(name, "mxfp4_hadi8", T, dict(y=xd.data_ptr(), res=rd.data_ptr(), w=wnd.data_ptr(), res_out=ro.data_ptr()), (wq, wsc), dict(k=W), eps=1e-6)
        np.testing.assert_array_equal(host_u16(ro), wro, err_msg=name)
    if W <= 10240:
        z = synth.f32_to_bf16_bits((rng.standard_normal((M, W + 8)) * 3).astype(np.float32))
        w = synth.f32_to_bf16_bits((1 + rng.standard_normal(128) * 0.1).astype(np.float32))
        zd, wd = dev_bf16_bits(z), dev_bf16_bits(w)
        want = ref.gdn_norm_quant_had(X, z[:, :W], w, t, 1e-6, silu_tab=device_silu_f32_table(ctx))
        for name, T in (("gdn_norm_quant_hadi8_t256_tiled1", 256), ("gdn_norm_quant_hadi8_t1024", 1024)):
            check(name, "mxfp4_hadi8", T, dict(x=xd.data_ptr(), z=zd.data_ptr(), w=wd.data_ptr()), want, dict(n=W, zs=W + 8), eps=1e-6)
    if W <= 6144:
        block = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * W + 16)) * 3).astype(np.float32))
        bd = dev_bf16_bits(block)
        sig = torch.zeros(65536, dtype=torch.int16, device="cuda")
        ctx.sigmoid_table(sig.data_ptr())
        want = ref.attn_gate_quant_had(X, block, t, 128)
        for name, T, tab in (("attn_gate_quant_hadi8_t256_tiled1", 256, False), ("attn_gate_quant_hadi8_t1024", 1024, False),
                             ("attn_gate_quant_hadi8_lut_t256", 256, True), ("attn_gate_quant_hadi8_lut_t1024", 1024, True)):
            bufs = dict(core=xd.data_ptr(), gate=bd.data_ptr())
            if tab:
                bufs["lut"] = sig.data_ptr()
            check(name, "attn_glue_hadi8", T, bufs, want, dict(n=W, hd=128, gs=2 * W + 16))


def test_had_producers_feed_the_gemm(ctx):
    """The transformed codes are ordinary A operands: producer + GEMM equals the oracle's GEMM on them."""
    say("quant_had -> gemm")
    M, N, K = 4, 256, 1024
    case = synth.dense_case(M, N, K, seed=9)
    t = np.random.default_rng(9).choice([-1.0, 1.0], size=K).astype(np.float32)
    q, s = outs(M, K)
    xd, td, wsd = dev_bf16_bits(case["X"]), dev_f32(t), dev_f32(case["ws"])
    ctx.quant_had(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K, td.data_ptr())
    wf = torch.from_numpy(iu8.repack_w4(case["W"])).cuda()
    c = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), M, N, K)
    torch.cuda.synchronize()
    wq, wsc = ref.quant_had(case["X"], t)
    S, _ = ref.gemm_fast(wq, case["W"], False, threads=4)
    np.testing.assert_array_equal(host_u16(c), ref.epilogue(S, wsc, case["ws"], False))


def test_had_refusals(ctx):
    q, s = outs(1, 64)
    for (m, k) in [(0, 64), (1, 96), (1, 20544)]:       # nothing to do, not whole fragments, too wide
        with pytest.raises(iu8.IU8Error) as e:
            ctx.quant_had(q.data_ptr(), q.data_ptr(), s.data_ptr(), m, k, s.data_ptr())
        assert e.value.code == iu8.E_RULE
    p = q.data_ptr()
    for args in [(p, p, 128, p, p, s.data_ptr(), 1, 192, 1e-6, p),          # not whole heads
                 (p, p, 64, p, p, s.data_ptr(), 1, 128, 1e-6, p),           # z stride under the row
                 (p, p, 10368, p, p, s.data_ptr(), 1, 10368, 1e-6, p)]:     # too wide
        with pytest.raises(iu8.IU8Error) as e:
            ctx.gdn_norm_quant_had(*args)
        assert e.value.code == iu8.E_RULE
    for args in [(p, p, p, s.data_ptr(), 1, 6208, 64, 12416, p),            # past the t256 form
                 (p, p, p, s.data_ptr(), 1, 256, 96, 512, p),               # heads do not divide the row
                 (p, p, p, s.data_ptr(), 1, 256, 64, 256, p)]:              # stride under the [q | gate] block
        with pytest.raises(iu8.IU8Error) as e:
            ctx.attn_gate_quant_had(*args)
        assert e.value.code == iu8.E_RULE
