"""GPU parity of the dense W4A8-iu8 linear: quant codes, int32 accumulators and bf16 outputs of the
HIP path, called through the C ABI, against the CPU oracle on the same seeded inputs."""
import numpy as np
import pytest

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import DenseRun, assert_dense_matches, say

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
