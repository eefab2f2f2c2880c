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


def test_fused_form_refuses_what_it_does_not_hold(ctx):
    assert not iu8.fused_holds(5, 1024) and not iu8.fused_holds(2, 17408) and not iu8.fused_holds(4, 5248)
    assert iu8.fused_holds(1, 17408) and iu8.fused_holds(4, 5120) and iu8.fused_holds(2, 10240)
    with pytest.raises(iu8.IU8Error) as e:
        iu8.resolve_fused(iu8.W4, 5, 256, 1024)
    assert e.value.code == iu8.E_RULE
    with pytest.raises(iu8.IU8Error):
        iu8.resolve_fused(iu8.W4, 1, 250, 1024)
