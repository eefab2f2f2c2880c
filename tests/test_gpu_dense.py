"""GPU parity of the dense W4A8-iu8 linear: quant codes, int32 accumulators and bf16 outputs of the
HIP path, called through the C ABI, against the CPU oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import DenseRun, assert_dense_matches, dev_bf16_bits, dev_f32, dev_u8, host_u16, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("w8", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 64, 256), (1, 5120, 5120), (4, 96, 512), (8, 7168, 5120), (16, 48, 1024),
                                   (16, 5120, 17408), (17, 64, 384), (40, 128, 640), (64, 256, 1280)])
def test_decode_band(ctx, M, N, K, w8):
    say(f"decode M={M} N={N} K={K} w8={w8}")
    case = synth.dense_case(M, N, K, w8=w8, seed=M * 7 + N + K)
    r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
    run = DenseRun(ctx, case, want_acc=(M <= 16))
    assert_dense_matches(run, r, w8)


@pytest.mark.parametrize("w8", [False, True])
@pytest.mark.parametrize("M,N,K", [(65, 64, 256), (128, 256, 512), (256, 512, 1024), (300, 304, 640), (512, 5120, 5120)])
def test_prefill_tile(ctx, M, N, K, w8):
    say(f"prefill M={M} N={N} K={K} w8={w8}")
    case = synth.dense_case(M, N, K, w8=w8, seed=M + N + K)
    r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
    run = DenseRun(ctx, case)
    assert_dense_matches(run, r, w8)


@pytest.mark.parametrize("M,N,K", [(1, 256, 1024), (1, 5120, 17408), (2, 176, 5120), (3, 304, 2560), (4, 7168, 5120)])
def test_fused_quant_decode_linear_gives_the_bytes_of_the_two_launch_path(ctx, M, N, K):
    """One launch (quantisation fused into the GEMV's activation staging) against the oracle: the
    bf16 output, and the optional code / scale outputs, are those of producer + GEMM."""
    for w8 in (False, True):
        say(f"fused decode linear M={M} N={N} K={K} w8={w8}")
        case = synth.dense_case(M, N, K, w8=w8, seed=41 + M)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        wk = iu8.W8 if w8 else iu8.W4
        assert iu8.fused_holds(M, K)
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
        c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
        q = torch.full((iu8.a_bytes(M, K),), 0x55, dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        ctx.linear_fused(wk, x.data_ptr(), wf.data_ptr(), ws.data_ptr(), c.data_ptr(), M, N, K, q=q.data_ptr(), scale=s.data_ptr())
        c2 = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
        ctx.linear_fused(wk, x.data_ptr(), wf.data_ptr(), ws.data_ptr(), c2.data_ptr(), M, N, K)     # no optional outputs
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])
        np.testing.assert_array_equal(host_u16(c2), r["C"])
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), r["q"])
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), r["a_scale"].view(np.uint32))


@pytest.mark.parametrize("M,N,K,grid", [(2, 16400, 640, None),     # 513 blocks: 171 workgroups x 3; k-waves of 1, 1, 1, 1, 1, 0, 0, 0 steps
                                          (3, 688, 384, 3),         # up to 8 blocks a workgroup; five k-waves with no step
                                          (1, 1040, 128, 5),        # one K step: seven idle k-waves
                                          (4, 2080, 5120, 17),      # the ring crossing block ends in its steady state
                                          (2, 2080, 1024, 60),      # a thin last round: 5 of 60 workgroups take a second block
                                          (1, 1104, 640, 16),       # an odd number of 16-column tiles: the last block holds one
                                          (4, 34816, 1024, None)])  # the widest layer shape: 1,088 blocks, 218 workgroups x 5
def test_fused_linear_walks_column_blocks(ctx, M, N, K, grid):
    """The fused form is persistent: a workgroup streams several column blocks against rows it
    quantised once, its load ring running across the block ends."""
    for w8 in (False, True):
        say(f"fused decode linear, blocks walked: M={M} N={N} K={K} grid={grid} w8={w8}")
        case = synth.dense_case(M, N, K, w8=w8, seed=77 + M)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        wk = iu8.W8 if w8 else iu8.W4
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
        c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
        d = iu8.resolve_fused(wk, M, N, K)
        if grid is None:
            nblk = (N + 31) // 32              # one workgroup a CU, equal shares of the blocks
            assert d.grid[0] <= 256 < nblk <= d.grid[0] * -(-nblk // 256) < nblk + -(-nblk // 256) and d.block[0] == 1024
        else:
            d.grid[0] = grid
        for name in ("q", "scale"):
            d.arg(name).kind = iu8.ARG_NULL_BUFFER
        ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr()))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])
    d.grid[0] = 1                                  # more than 8 blocks a workgroup: refused on the host
    if (N + 31) // 32 > 8:
        with pytest.raises(iu8.IU8Error) as e:
            ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr()))
        assert e.value.code == iu8.E_RULE


@pytest.mark.parametrize("M,N,K,grid", [(2, 5120, 17408, None),    # what the law launches it for: down at 2 rows
                                          (3, 352, 17408, None),
                                          (16, 480, 5120, None),     # the most rows; K a multiple of 512: a wave's pieces lie in one row
                                          (16, 7168, 5120, None),
                                          (9, 208, 4992, 2),         # K = 39 steps, not a multiple of 512: rows change inside a wave
                                          (5, 1104, 640, 5),         # several blocks a workgroup, an odd tile count, k-waves with no step
                                          (4, 96, 17408, None),      # 4 rows of the widest K
                                          (1, 64, 128, None)])       # one step
def test_fused_decode_linear_80_kib_form(ctx, M, N, K, grid):
    """macaq_iu8_decq_{w4,w8}_tm1_a80: up to 16 rows staged in 80 KiB, the bytes of producer + GEMV.
    The law launches it for two rows of a long K; the other shapes reach it by name."""
    for w8 in (False, True):
        say(f"fused decode linear, 80 KiB form: M={M} N={N} K={K} grid={grid} w8={w8}")
        case = synth.dense_case(M, N, K, w8=w8, seed=31 + M)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        wk, tag = (iu8.W8, "w8") if w8 else (iu8.W4, "w4")
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
        c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
        q = torch.full((iu8.a_bytes(M, K),), 0x55, dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        if iu8.fused_holds(M, K) and grid is None and not iu8.fused_small_holds(M, K):
            d = iu8.resolve_fused(wk, M, N, K)
            assert d.kernel.decode() == f"macaq_iu8_decq_{tag}_tm1_a80" and d.block[0] == 1024
        else:
            nblk = (N + 31) // 32
            d = iu8.describe_raw(f"macaq_iu8_decq_{tag}_tm1_a80", (grid or min(nblk, 256), 1, 1), 1024, m=M, n=N, k=K)
        ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr(), q=q.data_ptr(), scale=s.data_ptr()))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), r["q"])
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), r["a_scale"].view(np.uint32))
    # what the kernel does not hold is refused at launch, by name
    d = iu8.describe_raw("macaq_iu8_decq_w4_tm1_a80", (1, 1, 1), 1024, m=17, n=64, k=128)
    with pytest.raises(iu8.IU8Error) as e:
        ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr(), q=q.data_ptr(), scale=s.data_ptr()))
    assert e.value.code == iu8.E_RULE


@pytest.mark.parametrize("N,K,grid", [(5120, 17408, None),    # the benchmark's GEMV: 17 steps a k-wave, five chunks, the last of one step
                                        (96, 20480, None),      # the longest row the form holds: 20 steps a k-wave
                                        (7168, 5120, None),     # 5 steps a k-wave: one chunk ahead, then one step
                                        (1040, 128, 5),         # one K step: seven k-waves without a step, several blocks a workgroup
                                        (1104, 640, 16),        # five k-waves with one step; an odd number of 16-column tiles
                                        (2080, 1536, 9),        # 12 steps: k-waves of 2 and 1; up to 8 blocks a workgroup
                                        (34816, 5120, None),    # 1,088 blocks: 218 workgroups x 5, later blocks on codes in place
                                        (272, 4224, 3),         # 33 steps: one k-wave with 5, the others 4
                                        (64, 16512, 2)])        # 129 steps: one k-wave with 17
def test_fused_decode_linear_one_row_form(ctx, N, K, grid):
    """macaq_iu8_decq_{w4,w8}_r1: the row's codes made just in time, a chunk of 4 steps ahead of the MFMAs,
    by the waves that multiply them; the bytes of producer + GEMV, optional outputs included."""
    for w8 in (False, True):
        say(f"fused decode linear, one-row form: N={N} K={K} grid={grid} w8={w8}")
        case = synth.dense_case(1, N, K, w8=w8, seed=N + K)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        wk, tag = (iu8.W8, "w8") if w8 else (iu8.W4, "w4")
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
        d = iu8.resolve_fused(wk, 1, N, K)
        assert d.kernel.decode() == (f"macaq_iu8_decq_{tag}_r1" if K >= 8192 else f"macaq_iu8_decq_{tag}_tm1") and d.block[0] == 1024
        d = iu8.describe_raw(f"macaq_iu8_decq_{tag}_r1", (grid or d.grid[0], 1, 1), 1024, m=1, n=N, k=K)   # short rows reach it by name
        c = torch.full((1, N), 0x7FC0, dtype=torch.int16, device="cuda")
        q = torch.full((iu8.a_bytes(1, K),), 0x55, dtype=torch.uint8, device="cuda")
        s = torch.zeros(1, dtype=torch.float32, device="cuda")
        ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr(), q=q.data_ptr(), scale=s.data_ptr()))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), 1, K), r["q"])
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), r["a_scale"].view(np.uint32))
        # ... and the same bytes as the several-row form at one row
        d2 = iu8.describe_raw(f"macaq_iu8_decq_{tag}_tm1", (d.grid[0], 1, 1), 1024, m=1, n=N, k=K)
        c2 = torch.full((1, N), 0x7FC0, dtype=torch.int16, device="cuda")
        for a in ("q", "scale"):
            d2.arg(a).kind = iu8.ARG_NULL_BUFFER
        ctx.launch(d2, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c2.data_ptr()))
        torch.cuda.synchronize()
        assert torch.equal(c, c2)
    d = iu8.describe_raw("macaq_iu8_decq_w4_r1", (1, 1, 1), 1024, m=2, n=64, k=128)   # more than one row: refused by name
    with pytest.raises(iu8.IU8Error) as e:
        ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr(), q=q.data_ptr(), scale=s.data_ptr()))
    assert e.value.code == iu8.E_RULE


def test_one_row_form_on_ties_nan_and_infinity(ctx):
    """The one-row form on rows of crafted ties (the reciprocal path must hand them to the divide) and on rows
    with NaNs and infinities (the packed maximum's NaN branch, an infinite scale): codes, scale and output
    against the oracle's."""
    say("one-row form: ties, nan, inf")
    K, N = 2048, 64
    rows = []
    for amax in (127.0, 254.0, 63.5, 1.984375):
        sc = np.float32(amax) / np.float32(127.0)
        ks = np.arange(K, dtype=np.float32) % 126
        xr = (ks + np.float32(0.5)) * sc * np.where(np.arange(K) % 2 == 0, 1, -1).astype(np.float32)
        xr[0] = amax
        b0 = synth.f32_to_bf16_bits(xr).astype(np.uint16)
        rows.append(b0)
        for step in (1, -1):                      # the neighbouring bf16 values of every tie
            b = (b0.astype(np.int32) + step).astype(np.uint16)
            b[0] = b0[0]
            rows.append(b)
    rng = np.random.default_rng(5)
    base = synth.f32_to_bf16_bits((rng.standard_normal((6, K)) * 3).astype(np.float32))
    base[0, 17] = 0x7FC0                      # a lone NaN
    base[1, K - 1] = 0x7F80                   # an infinity in the last piece
    base[2, 0], base[2, 1] = 0x7FC0, 0xFF80   # both in one pair
    base[3, :] = 0x7FC0                       # nothing but NaNs: the maximum stays 0
    base[4, np.arange(0, K, 129)] = 0xFFC1    # negative NaNs with a payload in many pieces
    base[5, :] = 0                            # an all-zero row: scale 1e-30, codes 0
    rows += list(base)
    W, wsc = synth.weights(np.random.default_rng(3), N, K, False)
    wf, wsd = dev_u8(iu8.repack_w4(W)), dev_f32(wsc)
    for i, row in enumerate(rows):
        X = np.ascontiguousarray(row.reshape(1, K))
        want_q, want_s = ref.quant_bf16(X)
        xs = dev_bf16_bits(X)
        q = torch.zeros(iu8.a_bytes(1, K), dtype=torch.uint8, device="cuda")
        s = torch.zeros(1, dtype=torch.float32, device="cuda")
        c = torch.zeros((1, N), dtype=torch.int16, device="cuda")
        d = iu8.describe_raw("macaq_iu8_decq_w4_r1", (2, 1, 1), 1024, m=1, n=N, k=K)
        ctx.launch(d, dict(x=xs.data_ptr(), w=wf.data_ptr(), ws=wsd.data_ptr(), c=c.data_ptr(), q=q.data_ptr(), scale=s.data_ptr()))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), want_s.view(np.uint32), err_msg=f"row {i}")
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), 1, K), want_q, err_msg=f"row {i}")
        if i < len(rows) - 6 or i == len(rows) - 1:    # finite rows: the output too (NaN payloads of c are not pinned)
            r = ref.linear(X, W, wsc, False, threads=4)
            np.testing.assert_array_equal(host_u16(c), r["C"], err_msg=f"row {i}")


@pytest.mark.parametrize("w8", [False, True])
@pytest.mark.parametrize("M,N,K", [(12, 256, 1024),     # the streaming body (decode band)
                                   (200, 320, 1024)])    # the tile body (MFMA cells)
def test_rows_with_nan_and_infinity_through_the_gemm_epilogue(ctx, M, N, K, w8):
    """Activation rows with NaNs and infinities through producer + GEMM on both body families. A row with a
    NaN among finite values has a finite scale (the maximum passes the NaN over) and a finite output: bit-exact.
    A row with an infinity has an infinite scale: its outputs are infinities where the accumulator is not zero
    (bit-exact) and NaNs where it is (0 * inf); of a NaN in c only its being one is pinned -- the sign and payload
    come from the multiplier that made it (the card's on one side, the host's on the other), which no contract
    of the reference fixes (crates/saber-kernels/hip/macaq_iu8.hip:20-24)."""
    say(f"nan/inf rows through the epilogue M={M} N={N} K={K} w8={w8}")
    case = synth.dense_case(M, N, K, w8=w8, seed=M + K)
    X = case["X"]
    X[1, 17] = 0x7FC0                         # a lone NaN
    X[2, K - 1] = 0x7F80                      # +inf
    X[3, 5], X[3, 6] = 0xFF80, 0x7FC0         # -inf beside a NaN
    X[4, :] = 0x7FC0                          # nothing but NaNs
    X[5, 0], X[5, 1] = 0x7F80, 0xFF80         # both infinities: codes -127 and -127, the rest 0
    r = ref.linear(X, case["W"], case["ws"], w8, threads=8)
    run = DenseRun(ctx, case, want_acc=True)
    np.testing.assert_array_equal(run.q, r["q"])
    np.testing.assert_array_equal(run.a_scale.view(np.uint32), r["a_scale"].view(np.uint32))
    np.testing.assert_array_equal(run.acc, r["S"] if w8 else r["S"] * 16)
    want, got = r["C"], run.C
    nan_w, nan_g = (want & 0x7FFF) > 0x7F80, (got & 0x7FFF) > 0x7F80
    np.testing.assert_array_equal(nan_g, nan_w)                       # NaN exactly where the law makes one
    np.testing.assert_array_equal(got[~nan_w], want[~nan_w])          # everything else bit for bit, infinities included
    assert nan_w[[2, 3, 5]].any() or (r["S"][[2, 3, 5]] != 0).all()   # the infinite rows were exercised either way
    assert not nan_w[[0, 1, 4] + list(range(6, M))].any()             # rows with a finite scale never give a NaN


def test_fused_form_refuses_what_it_does_not_hold(ctx):
    assert not iu8.fused_holds(5, 1024) and not iu8.fused_holds(4, 20608) and not iu8.fused_holds(2, 41088)
    assert iu8.fused_holds(1, 17408) and iu8.fused_holds(4, 5120) and iu8.fused_holds(2, 10240)
    assert iu8.fused_holds(2, 17408) and iu8.fused_holds(2, 16384) and not iu8.fused_small_holds(2, 17408)   # the 80 KiB form: two rows of a long K
    assert not iu8.fused_holds(4, 17408) and not iu8.fused_holds(4, 5248) and not iu8.fused_holds(3, 8192)   # slower than producer + GEMV: two launches
    assert not iu8.fused_holds(3, 17408) and not iu8.fused_holds(2, 12288)
    with pytest.raises(iu8.IU8Error) as e:
        iu8.resolve_fused(iu8.W4, 5, 256, 1024)
    assert e.value.code == iu8.E_RULE
    with pytest.raises(iu8.IU8Error):
        iu8.resolve_fused(iu8.W4, 1, 250, 1024)


def test_quant_ties_and_near_ties_round_like_the_ieee_divide(ctx):
    """Rows built so that x / scale lands on half-integers (exact ties, half to even) and one bf16
    step beside them: the producer's reciprocal fast path must hand these to the divide."""
    say("quant ties")
    K = 1024
    rows = []
    for amax in (127.0, 254.0, 63.5, 1.984375, 3.96875e-3, 508.0):
        sc = np.float32(amax) / np.float32(127.0)
        ks = np.arange(K, dtype=np.float32) % 126          # below the row maximum, which x[0] sets
        x = (ks + np.float32(0.5)) * sc * np.where(np.arange(K) % 2 == 0, 1, -1).astype(np.float32)
        x[0] = amax
        rows.append(x)
        b = synth.f32_to_bf16_bits(x).astype(np.uint16)
        for step in (1, -1):                      # the neighbouring bf16 values of every tie
            rows.append(synth.bf16_bits_to_f32((b.astype(np.int32) + step).astype(np.uint16)))
            rows[-1][0] = amax
    X = synth.f32_to_bf16_bits(np.stack(rows).astype(np.float32))
    M = X.shape[0]
    want_q, want_s = ref.quant_bf16(X)
    x = dev_bf16_bits(X)
    q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    ctx.quant(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), want_q)
    # ... and through the fused decode linear, which quantises in its prologue
    W, ws = synth.weights(np.random.default_rng(3), 64, K, False)
    wf, wsd = dev_u8(iu8.repack_w4(W)), dev_f32(ws)
    for r0 in range(0, M - M % 4, 4):
        xs = dev_bf16_bits(X[r0:r0 + 4])
        q4 = torch.zeros(iu8.a_bytes(4, K), dtype=torch.uint8, device="cuda")
        s4 = torch.zeros(4, dtype=torch.float32, device="cuda")
        c = torch.zeros((4, 64), dtype=torch.int16, device="cuda")
        ctx.linear_fused(iu8.W4, xs.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), 4, 64, K, q=q4.data_ptr(), scale=s4.data_ptr())
        torch.cuda.synchronize()
        np.testing.assert_array_equal(iu8.unpack_a(q4.cpu().numpy(), 4, K), want_q[r0:r0 + 4])


@pytest.mark.parametrize("K", [1024, 5120, 17408, 24576])
def test_quant_rows_with_nan_and_infinity(ctx, K):
    """Rows that hold NaNs and infinities, on every register-width form of the producer (one, two, five
    and eight groups a thread): the row maximum passes a NaN over, a NaN's code is -127, an infinite
    maximum makes the scale infinite (finite elements 0, the infinities themselves -127)."""
    say(f"quant nan/inf K={K}")
    rng = np.random.default_rng(K)
    M = 12
    X = synth.f32_to_bf16_bits((rng.standard_normal((M, K)) * 3).astype(np.float32))
    nan, pinf, ninf = 0x7FC0, 0x7F80, 0xFF80
    X[1, 17] = nan                                  # a lone NaN
    X[2, K - 1] = pinf                              # an infinity in the row's last group
    X[3, 0], X[3, 1] = nan, ninf                    # both in one pair
    X[4, :] = nan                                   # nothing but NaNs: the maximum stays 0
    X[5, 4096 % K] = 0xFFC1                         # a negative NaN with a payload
    X[6, K // 2], X[6, K // 2 + 9] = 0x7F81, 0x7F7F  # a signalling pattern beside the largest finite value
    X[7, np.arange(0, K, 257)] = nan                # a NaN in many threads' groups
    want_q, want_s = ref.quant_bf16(X)
    x = dev_bf16_bits(X)
    for rm in (False, True):
        q = torch.zeros(M * K if rm else iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        (ctx.quant_rowmajor if rm else ctx.quant)(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
        got = q.cpu().numpy().view(np.int8).reshape(M, K) if rm else iu8.unpack_a(q.cpu().numpy(), M, K)
        np.testing.assert_array_equal(got, want_q)


def _row_forms(base, width):
    """Every form of a row producer that holds rows of `width`, by kernel name and block size."""
    slots = -(-width // 4096)
    forms = [(base + "_t256" + sfx, 256) for need, sfx in ((1, "_g1"), (2, "_g2"), (5, "_g5"), (8, "")) if slots <= need]
    return forms + [(base + "_t1024", 1024)]


@pytest.mark.parametrize("M,K", [(1, 17408), (3, 5120), (12, 4160), (16, 32768), (5, 64), (33, 16384), (2, 20480)])
def test_row_producers_every_form_that_holds_the_row(ctx, M, K):
    """The quantiser and the SiLU * up + requant producer, launched by name in each of their register
    forms (256 threads with 1, 2, 5 or 8 groups a thread; 1024 threads with 2): the same codes and
    scales as the oracle from all of them, on rows with a NaN and an infinity among them."""
    say(f"row producers, every form: M={M} K={K}")
    rng = np.random.default_rng(M * 131 + K)
    X = synth.f32_to_bf16_bits((rng.standard_normal((M, K)) * 2).astype(np.float32))
    GU = synth.f32_to_bf16_bits((rng.standard_normal((M, 2 * K)) * 3).astype(np.float32))
    X[M - 1, K - 1] = 0x7FC0
    if M > 1:
        X[0, K // 2], GU[0, K + K // 3] = 0x7F80, 0xFF80
    want_q, want_s = ref.quant_bf16(X)
    want_q2, want_s2, _ = ref.silu_mul_quant(GU)
    x, gu = dev_bf16_bits(X), dev_bf16_bits(GU)
    law_q, law_a = iu8.resolve_quant(M, K), iu8.resolve_silu_mul_quant(M, K)
    assert (law_q.kernel.decode(), law_q.block[0]) in _row_forms("macaq_i8_quant", K)
    assert (law_a.kernel.decode(), law_a.block[0]) in _row_forms("macaq_i8_silu_mul_quant", K)
    for base, src, key, resolve, wq, wsc in (("macaq_i8_quant", x, "x", iu8.resolve_quant, want_q, want_s),
                                            ("macaq_i8_silu_mul_quant", gu, "gu", iu8.resolve_silu_mul_quant, want_q2, want_s2)):
        for name, block in _row_forms(base, K):
            d = resolve(M, K)
            d.kernel, d.block[0] = name.encode(), block
            q = torch.full((iu8.a_bytes(M, K),), 0x55, dtype=torch.uint8, device="cuda")
            s = torch.zeros(M, dtype=torch.float32, device="cuda")
            ctx.launch(d, {key: src.data_ptr(), "q": q.data_ptr(), "scale": s.data_ptr()})
            torch.cuda.synchronize()
            np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), wsc.view(np.uint32), err_msg=name)
            np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, K), wq, err_msg=name)


@pytest.mark.parametrize("w8", [False, True])
@pytest.mark.parametrize("M,N,K,grid", [(16, 5120, 5120, 0), (9, 96, 5120, 0), (13, 34816, 5120, 0), (11, 7184, 640, 0), (5, 4112, 128, 0),
                                        (1, 256, 5120, 0), (16, 2048, 3072, 8), (12, 2064, 384, 9),
                                        (4, 5120, 17408, 0), (2, 272, 32768, 0), (8, 1040, 10240, 5), (3, 2064, 20480, 0), (1, 96, 17408, 0)])
def test_sixteen_row_tile_staged_once_a_workgroup(ctx, M, N, K, grid, w8):
    """The persistent GEMV that copies the rows' 16-row tile into LDS once a workgroup (`_s80`), by name: full and
    ragged row counts, a last column block of 16 columns, one K step (seven idle k-waves), five column blocks a
    workgroup at the benchmark layer's gate+up, grids that give a workgroup 8 blocks or an uneven share, and fewer
    live rows of a longer K (the copy then takes the live rows' pieces of the tile: 1, 2, 4 or 8 of every 16).
    The tile's rows past M hold whatever the producer's buffer held (0x55 here): they reach no output."""
    tag = "w8" if w8 else "w4"
    # the whole-tile kernel holds K <= 5120 at any row count; the rows kernel (`_s80r`) whatever fits 80 KiB, taken
    # here for the longer K and, for every other case below it, so that both kernels see short and long loops
    name = f"macaq_iu8_dec_{tag}_tm1_s80" + ("r" if K > 5120 or (M + N // 16) % 2 else "")
    say(f"staged 16-row tile {name} M={M} N={N} K={K} grid={grid}")
    case = synth.dense_case(M, N, K, w8=w8, seed=M * 11 + N + K)
    r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=16)
    run = DenseRun(ctx, case, kernel=name, want_acc=False)
    assert run.desc.block[0] == 1024 and run.desc.grid[0] * 8 >= -(-N // 32)
    np.testing.assert_array_equal(run.C, r["C"])
    if grid:
        d = iu8.describe(name, M, N, K)
        d.grid[0] = grid
        assert grid * 8 >= -(-N // 32)
        c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
        bufs = {"a": run.dev["q"].data_ptr(), "w": run.dev["wf"].data_ptr(), "as": run.dev["a_scale"].data_ptr(),
                "ws": run.dev["ws"].data_ptr(), "c": c.data_ptr()}
        ctx.launch(d, bufs)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])
        # descriptors edited past what the kernel holds are refused at launch: more than 8 blocks a workgroup, a K
        # whose tile passes 80 KiB, more than 16 rows
        mr = 1 << (M - 1).bit_length()
        for field, value in (("grid", max(1, (-(-N // 32) - 1) // 8)), ("k", 80 * 1024 // (mr if name.endswith("r") else 16) + 128), ("m", 17)):
            bad = iu8.describe(name, M, N, K)
            if field == "grid":
                if value * 8 >= -(-N // 32):
                    continue
                bad.grid[0] = value
            else:
                bad.arg(field).ival = value
            with pytest.raises(iu8.IU8Error) as e:
                ctx.launch(bad, bufs)
            assert e.value.code == iu8.E_RULE, field
