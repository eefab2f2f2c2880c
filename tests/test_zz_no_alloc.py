"""The GEMM entry point that allocates nothing (saber_iu8_gemm_static: the split-K workspaces in the
library's static device array) against saber_iu8_gemm with caller-owned workspaces, through the C ABI:
same bytes, on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import dev_bf16_bits, dev_f32, dev_u8, host_u16, say

pytestmark = pytest.mark.gpu


def run_both(ctx, M, N, K, seed):
    case = synth.dense_case(M, N, K, seed=seed)
    x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_w4(case["W"])), dev_f32(case["ws"])
    q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    ctx.quant(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
    pb, cb = iu8.gemm_workspace(iu8.W4, M, N, K)
    partial = torch.full((max(pb, 4) // 4,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
    counter = torch.zeros(max(cb, 4) // 4, dtype=torch.int32, device="cuda")
    want = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
    ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), ws.data_ptr(), want.data_ptr(), M, N, K,
             partial.data_ptr() if pb else None, counter.data_ptr() if cb else None)
    got = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    ctx.gemm_static(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), ws.data_ptr(), got.data_ptr(), M, N, K)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return case, pb, host_u16(got), host_u16(want), (q, s)


def test_static_workspace_gemm_equals_the_caller_workspace_gemm_twice_in_a_row(ctx):
    assert iu8.lib().saber_iu8_static_workspace_bytes() == 8 * 1024 * 1024 + 64 * 1024
    # the band where the launch law splits K (K >= 16384, 49..128 rows, at most 80 tiles): first the
    # largest such launch of the 27B-class layer, then a smaller one on the same static array
    for (M, N, K) in ((128, 5120, 17408), (64, 384, 16384)):
        say(f"static-workspace GEMM {M}x{N}x{K}")
        case, pb, got, want, keep = run_both(ctx, M, N, K, seed=M)
        assert pb > 0, "the case must be one the law splits"
        np.testing.assert_array_equal(got, want)
        qh, sh = ref.quant_bf16(case["X"])
        cols = min(N, 256)
        S, _ = ref.gemm_fast(qh, case["W"][-cols:], False, threads=16)
        np.testing.assert_array_equal(got[:, -cols:], ref.epilogue(S, sh, case["ws"][-cols:], False))
    # a launch the law does not split needs no workspace and runs through the same entry point
    say("static-workspace GEMM, unsplit shapes")
    for (M, N, K) in ((1, 5120, 5120), (300, 304, 640)):
        case, pb, got, want, keep = run_both(ctx, M, N, K, seed=7)
        assert pb == 0
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got, ref.linear(case["X"], case["W"], case["ws"], False, threads=8)["C"])


def test_static_workspace_holds_every_launch_the_law_splits(ctx):
    # no shape the law splits today passes 8 MiB of partials (its band ends at 128 rows of at most
    # 80 tiles); the refusal is checked on the size arithmetic the entry point applies
    pb, cb = iu8.gemm_workspace(iu8.W4, 128, 5120, 17408)
    assert 0 < pb <= 8 * 1024 * 1024 and 0 < cb <= 64 * 1024
