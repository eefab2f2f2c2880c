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
    # the device's own count of free memory (hipMemGetInfo), which a hipMalloc inside the library would move;
    # torch's allocator statistics only see torch's own allocations
    free_before = torch.cuda.mem_get_info()[0]
    ctx.gemm_static(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), ws.data_ptr(), got.data_ptr(), M, N, K)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    return case, pb, host_u16(got), host_u16(want), (q, s, x, wf, ws)


def test_static_workspace_gemm_equals_the_caller_workspace_gemm_twice_in_a_row(ctx):
    assert iu8.lib().saber_iu8_static_workspace_bytes() == 8 * 1024 * 1024 + 64 * 1024
    # the band where the launch law splits K (K >= 16384, 33..128 rows, at most 80 tiles): first the
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


def test_static_workspace_gemm_under_graph_capture_on_two_inputs(ctx):
    """The entry point inside a captured graph: an allocation or a synchronisation in it would fail the capture.
    One graph holds two split launches in a row on the same static array (different inputs, the second smaller),
    and is replayed three times with eager work between the replays; every replay gives the oracle's bytes and
    leaves the arrival counters at zero for the next."""
    say("static-workspace GEMM under graph capture")
    shapes = ((128, 5120, 17408), (64, 384, 16384))
    runs = []
    for i, (M, N, K) in enumerate(shapes):
        case = synth.dense_case(M, N, K, seed=100 + i)
        r = ref.linear(case["X"], case["W"], case["ws"], False, threads=16)
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_w4(case["W"])), dev_f32(case["ws"])
        q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        ctx.quant(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
        assert iu8.gemm_workspace(iu8.W4, M, N, K)[0] > 0, "the case must be one the law splits"
        runs.append(dict(M=M, N=N, K=K, want=r["C"], q=q, s=s, wf=wf, ws=ws, c=torch.zeros((M, N), dtype=torch.int16, device="cuda")))
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    free_before = torch.cuda.mem_get_info()[0]
    with torch.cuda.graph(g, stream=stream):
        for r in runs:
            ctx.gemm_static(iu8.W4, r["q"].data_ptr(), r["s"].data_ptr(), r["wf"].data_ptr(), r["ws"].data_ptr(), r["c"].data_ptr(),
                            r["M"], r["N"], r["K"], stream.cuda_stream)
    for rep in range(3):
        for r in runs:
            r["c"].fill_(0x7FC0)                       # poison; eager work between the replays
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            g.replay()
        torch.cuda.synchronize()
        for r in runs:
            np.testing.assert_array_equal(host_u16(r["c"]), r["want"], err_msg=f"replay {rep}, {r['M']}x{r['N']}x{r['K']}")
    assert torch.cuda.mem_get_info()[0] >= free_before - (8 << 20)   # the graph's own bookkeeping, nothing of the order of a workspace
    # the recovery helper: counters refilled with zeros by a kernel on the stream, and the array still works
    ctx.static_workspace_reset(stream.cuda_stream)
    with torch.cuda.stream(stream):
        g.replay()
    torch.cuda.synchronize()
    for r in runs:
        np.testing.assert_array_equal(host_u16(r["c"]), r["want"])
