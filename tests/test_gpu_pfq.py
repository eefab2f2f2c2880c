"""GPU parity of the tile GEMM with the per-token quantisation fused into its A-tile load
(macaq_iu8_pfq_*: bf16 rows + row scales in, codes made on the way into the A stage) against the
oracle and against the two-launch path (producer + GEMM), through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import dev_bf16_bits, dev_f32, dev_u8, host_u16, say

pytestmark = pytest.mark.gpu

CELLS = {False: ("t128x128", "t128x128_o2", "t256x160"), True: ("t128x128", "t256x160")}


def run_pfq(ctx, case, kernel=None):
    M, N, K, w8 = case["M"], case["N"], case["K"], case["w8"]
    wk = iu8.W8 if w8 else iu8.W4
    x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
    s = torch.full((M,), -1.0, dtype=torch.float32, device="cuda")
    ctx.rowscale(x.data_ptr(), s.data_ptr(), M, K)
    c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
    if kernel is None:
        ctx.linear_prefill_fused(wk, x.data_ptr(), s.data_ptr(), wf.data_ptr(), ws.data_ptr(), c.data_ptr(), M, N, K)
    else:
        d = iu8.describe(kernel, M, N, K)
        bufs = dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr())
        bufs["as"] = s.data_ptr()
        ctx.launch(d, bufs)
    torch.cuda.synchronize()
    return s.cpu().numpy(), host_u16(c)


@pytest.mark.parametrize("shape", [(65, 16, 128), (129, 304, 384), (200, 272, 640), (300, 1040, 2048), (4160, 1088, 256)])
def test_every_fused_quant_cell_gives_the_oracle_bytes(ctx, shape):
    """One and two K steps (fewer than the LDS stages), ragged rows and columns, more tiles than
    persistent workgroups (the register pieces and the weights' stream crossing tile ends)."""
    M, N, K = shape
    for w8 in (False, True):
        case = synth.dense_case(M, N, K, w8=w8, seed=61 + M)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        for cell in CELLS[w8]:
            name = f"macaq_iu8_pfq_{'w8' if w8 else 'w4'}_{cell}"
            say(f"fused-quant tile GEMM {shape} {name}")
            s, c = run_pfq(ctx, case, name)
            np.testing.assert_array_equal(s.view(np.uint32), r["a_scale"].view(np.uint32))
            np.testing.assert_array_equal(c, r["C"])


@pytest.mark.parametrize("M,N,K", [(256, 5120, 5120), (2048, 7168, 5120), (512, 5120, 17408)])
def test_fused_quant_linear_equals_producer_plus_gemm(ctx, M, N, K):
    """The operator entry (the law's cell) at layer shapes: the bytes of saber_iu8_quant + saber_iu8_gemm,
    which an oracle slice pins."""
    say(f"fused-quant linear M={M} N={N} K={K}")
    case = synth.dense_case(M, N, K, seed=M)
    s, c = run_pfq(ctx, case)
    x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_w4(case["W"])), dev_f32(case["ws"])
    q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    s2 = torch.zeros(M, dtype=torch.float32, device="cuda")
    c2 = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    ctx.quant(x.data_ptr(), q.data_ptr(), s2.data_ptr(), M, K)
    ctx.gemm(iu8.W4, q.data_ptr(), s2.data_ptr(), wf.data_ptr(), ws.data_ptr(), c2.data_ptr(), M, N, K)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(s.view(np.uint32), s2.cpu().numpy().view(np.uint32))
    np.testing.assert_array_equal(c, host_u16(c2))
    qh, sh = ref.quant_bf16(case["X"])
    S, _ = ref.gemm_fast(qh, case["W"][-256:], False, threads=16)
    np.testing.assert_array_equal(c[:, -256:], ref.epilogue(S, sh, case["ws"][-256:], False))


def test_fused_quant_rounds_ties_like_the_producer(ctx):
    """Rows whose x / scale sits on half-integers: the GEMM's own conversion must send them to the divide."""
    say("fused-quant tile GEMM, crafted ties")
    K, N = 1024, 128
    rows = []
    for amax in (127.0, 254.0, 63.5, 1.984375):
        sc = np.float32(amax) / np.float32(127.0)
        ks = np.arange(K, dtype=np.float32) % 126
        x = (ks + np.float32(0.5)) * sc * np.where(np.arange(K) % 2 == 0, 1, -1).astype(np.float32)
        x[0] = amax
        rows.append(x)
    X = synth.f32_to_bf16_bits(np.tile(np.stack(rows).astype(np.float32), (20, 1)))
    M = X.shape[0]
    W, ws = synth.weights(np.random.default_rng(9), N, K, False)
    case = dict(M=M, N=N, K=K, w8=False, X=X, W=W, ws=ws)
    r = ref.linear(X, W, ws, False, threads=8)
    for cell in CELLS[False]:
        s, c = run_pfq(ctx, case, f"macaq_iu8_pfq_w4_{cell}")
        np.testing.assert_array_equal(c, r["C"])
