"""GPU parity of the decode pair (code object `macaq_iu8f`): two W4 GEMMs on one activation operand
in one dispatch give the bytes of the oracle and of two separate launches."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import dev_bf16_bits, dev_f32, dev_u8, host_u16, say

pytestmark = pytest.mark.gpu


def halves(rng, M, K, n0, n1):
    X = synth.activations(rng, M, K)
    W0, ws0 = synth.weights(rng, n0, K, False)
    W1, ws1 = synth.weights(rng, n1, K, False)
    return X, (W0, ws0), (W1, ws1)


# GDN's in_proj_qkvz + in_proj_ba at hidden 5120 (the reference's pair), ragged column blocks, each
# row tiling (tm1 staged and streamed, tm2..tm4), a long K
@pytest.mark.parametrize("M,K,n0,n1", [(1, 5120, 12288, 96), (4, 5120, 1040, 48), (16, 5120, 272, 528), (8, 17408, 320, 64),
                                       (20, 1024, 144, 32), (40, 640, 80, 304), (48, 512, 64, 64)])
def test_pair_matches_the_oracle_and_two_launches(ctx, M, K, n0, n1):
    say(f"pair M={M} K={K} N={n0}+{n1}")
    rng = np.random.default_rng(M * 7 + n0)
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
    e0, e1 = torch.zeros_like(c0), torch.zeros_like(c1)
    ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), w0.data_ptr(), s0.data_ptr(), e0.data_ptr(), M, n0, K)
    ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), w1.data_ptr(), s1.data_ptr(), e1.data_ptr(), M, n1, K)
    torch.cuda.synchronize()
    assert torch.equal(c0, e0) and torch.equal(c1, e1)
    r0 = ref.linear(X, W0, ws0, False, threads=8)
    r1 = ref.linear(X, W1, ws1, False, threads=8)
    np.testing.assert_array_equal(host_u16(c0), r0["C"])
    np.testing.assert_array_equal(host_u16(c1), r1["C"])


def test_pair_of_named_cells_past_the_streaming_band(ctx):
    """From 49 rows the launch law hands a linear to the tile GEMM, which does not pair (refused by name);
    the four-tile streaming cell still pairs when it is named."""
    say("pair of named tm4 cells, M=64")
    M, K, n0, n1 = 64, 512, 80, 48
    rng = np.random.default_rng(64)
    X, (W0, ws0), (W1, ws1) = halves(rng, M, K, n0, n1)
    xd = dev_bf16_bits(X)
    q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
    w0, w1, s0, s1 = dev_u8(iu8.repack_w4(W0)), dev_u8(iu8.repack_w4(W1)), dev_f32(ws0), dev_f32(ws1)
    c0 = torch.full((M, n0), 0x7FC0, dtype=torch.int16, device="cuda")
    c1 = torch.full((M, n1), 0x7FC0, dtype=torch.int16, device="cuda")
    with pytest.raises(iu8.IU8Error) as e:
        ctx.gemm_pair(q.data_ptr(), s.data_ptr(), w0.data_ptr(), s0.data_ptr(), c0.data_ptr(), n0,
                      w1.data_ptr(), s1.data_ptr(), c1.data_ptr(), n1, M, K)
    assert e.value.code == iu8.E_RULE
    d = iu8.pair(iu8.describe("macaq_iu8_dec_w4_tm4", M, n0, K), iu8.describe("macaq_iu8_dec_w4_tm4", M, n1, K))
    assert d.kernel == b"macaq_iu8f_pairb_w4_tm4"
    bufs = dict(a=q.data_ptr(), w=w0.data_ptr(), ws=s0.data_ptr(), c=c0.data_ptr(), w_b=w1.data_ptr(), ws_b=s1.data_ptr(),
                c_b=c1.data_ptr())
    bufs["as"] = s.data_ptr()
    ctx.launch(d, bufs)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(host_u16(c0), ref.linear(X, W0, ws0, False)["C"])
    np.testing.assert_array_equal(host_u16(c1), ref.linear(X, W1, ws1, False)["C"])


def test_pair_with_explicitly_split_halves(ctx):
    """Each half keeps its own split count, partial slab and self-resetting counters."""
    say("pair, halves split 2 and 3")
    M, K, n0, n1 = 3, 2048, 208, 96
    rng = np.random.default_rng(5)
    X, (W0, ws0), (W1, ws1) = halves(rng, M, K, n0, n1)
    xd = dev_bf16_bits(X)
    q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
    w0, w1, s0, s1 = dev_u8(iu8.repack_w4(W0)), dev_u8(iu8.repack_w4(W1)), dev_f32(ws0), dev_f32(ws1)
    d = iu8.pair(iu8.describe("macaq_iu8_dec_w4_tm1", M, n0, K, ks=2), iu8.describe("macaq_iu8_dec_w4_tm1", M, n1, K, ks=3))
    ws_bufs = {}
    for i in range(d.n_workspaces):
        w = d.workspaces[i]
        fill = 0 if w.zero_once else 0x5A5A5A5A              # Scratch is undefined at entry, Persistent zeroed once
        ws_bufs[w.name.decode()] = torch.full((w.bytes // 4,), fill, dtype=torch.int32, device="cuda")
    assert set(ws_bufs) == {"decode_partial", "decode_counter", "decode_partial_b", "decode_counter_b"}
    r0, r1 = ref.linear(X, W0, ws0, False), ref.linear(X, W1, ws1, False)
    for rep in range(2):                                      # twice on the same counters
        c0 = torch.full((M, n0), 0x7FC0, dtype=torch.int16, device="cuda")
        c1 = torch.full((M, n1), 0x7FC0, dtype=torch.int16, device="cuda")
        bufs = dict(a=q.data_ptr(), w=w0.data_ptr(), ws=s0.data_ptr(), c=c0.data_ptr(), w_b=w1.data_ptr(), ws_b=s1.data_ptr(),
                    c_b=c1.data_ptr(), **{k: v.data_ptr() for k, v in ws_bufs.items()})
        bufs["as"] = s.data_ptr()
        ctx.launch(d, bufs)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c0), r0["C"])
        np.testing.assert_array_equal(host_u16(c1), r1["C"])
        assert not ws_bufs["decode_counter"].cpu().numpy().any() and not ws_bufs["decode_counter_b"].cpu().numpy().any()


@pytest.mark.parametrize("M,K,n0,n1", [(1, 5120, 12288, 96), (16, 1024, 272, 528), (40, 640, 80, 304)])
def test_both_block_orders_give_the_same_bytes(ctx, M, K, n0, n1):
    """`pair` (problem 0's workgroups first) and `pairb` (the second problem's first, the law's pick as
    in the reference, crates/saber-kernels/src/macaq_iu8.rs:549-553): one kernarg list, the oracle's bytes."""
    rng = np.random.default_rng(M + n1)
    X, (W0, ws0), (W1, ws1) = halves(rng, M, K, n0, n1)
    xd = dev_bf16_bits(X)
    q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
    w0, w1, s0, s1 = dev_u8(iu8.repack_w4(W0)), dev_u8(iu8.repack_w4(W1)), dev_f32(ws0), dev_f32(ws1)
    r0, r1 = ref.linear(X, W0, ws0, False, threads=8), ref.linear(X, W1, ws1, False, threads=8)
    a, b = iu8.resolve(iu8.W4, M, n0, K), iu8.resolve(iu8.W4, M, n1, K)
    for second_first in (False, True):
        d = iu8.pair_ordered(a, b, second_first)
        say(f"pair order {d.kernel.decode()} M={M} K={K} N={n0}+{n1}")
        assert (b"_pairb_" in d.kernel) == second_first
        c0 = torch.full((M, n0), 0x7FC0, dtype=torch.int16, device="cuda")
        c1 = torch.full((M, n1), 0x7FC0, dtype=torch.int16, device="cuda")
        bufs = dict(a=q.data_ptr(), w=w0.data_ptr(), ws=s0.data_ptr(), c=c0.data_ptr(), w_b=w1.data_ptr(), ws_b=s1.data_ptr(),
                    c_b=c1.data_ptr())
        bufs["as"] = s.data_ptr()
        ctx.launch(d, bufs)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c0), r0["C"])
        np.testing.assert_array_equal(host_u16(c1), r1["C"])
