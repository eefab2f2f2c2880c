"""GPU parity of the Hadamard-basis int8 producers (code object `mxfp4_hadi8`), through the C ABI,
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
