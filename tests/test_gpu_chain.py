"""GPU parity of the dense decode MLP as one persistent launch (macaq_iu8f_mlp_w4_tm1): gate+up
linear -> SiLU * up + requantisation -> down linear. Bit-exact against the oracle's three steps and
against the library's own three launches; the launch's working rows are checked too; the bounded
wait of its meetings is exercised from the host with a one-poll limit (every workgroup still exits
normally)."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import dev_bf16_bits, dev_f32, dev_u8, host_u16, say

pytestmark = pytest.mark.gpu
STATUS = iu8.MLP_CHAIN_STATUS_OFFSET // 4               # the status word; in front of it arrival and passed words, behind it `go`
SLOTS = 8 * 1024 // 4                                    # the first 8 KiB: the workgroups' maxima, rewritten every launch


class Mlp:
    def __init__(self, M, H, I, seed):
        rng = np.random.default_rng(seed)
        self.M, self.H, self.I = M, H, I
        self.Wgu, self.wsgu = synth.weights(rng, 2 * I, H, False)
        self.Wdn, self.wsdn = synth.weights(rng, H, I, False)
        self.X = synth.activations(rng, M, H)
        self.x = dev_bf16_bits(self.X)
        self.wgu, self.wsg = dev_u8(iu8.repack_w4(self.Wgu)), dev_f32(self.wsgu)
        self.wdn, self.wsd = dev_u8(iu8.repack_w4(self.Wdn)), dev_f32(self.wsdn)
        self.gu = torch.full((M, 2 * I), 0x7FC0, dtype=torch.int16, device="cuda")
        self.p = torch.full((M, I), 0x7FC0, dtype=torch.int16, device="cuda")
        self.state = torch.zeros(iu8.MLP_CHAIN_STATE_BYTES // 4, dtype=torch.int32, device="cuda")
        self.c = torch.full((M, H), 0x7FC0, dtype=torch.int16, device="cuda")

    def oracle(self):
        gu = ref.linear(self.X, self.Wgu, self.wsgu, False, threads=16)["C"]
        _, _, p = ref.silu_mul_quant(gu)
        c = ref.linear(p, self.Wdn, self.wsdn, False, threads=16)["C"]
        return gu, p, c

    def chain(self, ctx, spin=0, tap=True):
        ctx.mlp_chain(self.x.data_ptr(), self.wgu.data_ptr(), self.wsg.data_ptr(), self.wdn.data_ptr(), self.wsd.data_ptr(),
                      self.gu.data_ptr() if tap else None, self.p.data_ptr(), self.state.data_ptr(), self.c.data_ptr(),
                      self.M, self.H, self.I, spin=spin)
        torch.cuda.synchronize()

    def three_launches(self, ctx):
        M, H, I = self.M, self.H, self.I
        gu = torch.full((M, 2 * I), 0x7FC0, dtype=torch.int16, device="cuda")
        q = torch.zeros(iu8.a_bytes(M, I), dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        c = torch.full((M, H), 0x7FC0, dtype=torch.int16, device="cuda")
        ctx.linear_fused(iu8.W4, self.x.data_ptr(), self.wgu.data_ptr(), self.wsg.data_ptr(), gu.data_ptr(), M, 2 * I, H)
        ctx.launch(iu8.resolve_silu_mul_quant(M, I), dict(gu=gu.data_ptr(), q=q.data_ptr(), scale=s.data_ptr()))
        ctx.gemm_static(iu8.W4, q.data_ptr(), s.data_ptr(), self.wdn.data_ptr(), self.wsd.data_ptr(), c.data_ptr(), M, H, I)
        torch.cuda.synchronize()
        return host_u16(gu), host_u16(c)


# rows, hidden, intermediate: the benchmark layer at one row (5120 / 17408); the most rows the form
# holds at a narrower layer; two rows at the widest they fit; three rows (staged as four) with K
# steps that do not divide among the k-waves (11 and 23); fewer column blocks than workgroups
# ... and the 80 KiB form of the second linear: 2 and 4 rows of the benchmark layer, 3 rows of a ragged width
SHAPES = [(1, 5120, 17408), (4, 5120, 5120), (2, 2048, 10240), (3, 1408, 2944), (1, 384, 384),
          (2, 5120, 17408), (4, 5120, 17408), (3, 640, 12672)]


@pytest.mark.parametrize("M,H,I", SHAPES)
def test_chain_matches_the_oracle_and_the_three_launches(ctx, M, H, I):
    say(f"mlp chain M={M} H={H} I={I}")
    d = iu8.resolve_mlp_chain(M, H, I)
    assert d.kernel == (b"macaq_iu8f_mlp_w4_tm1" if iu8.fused_small_holds(M, I) else b"macaq_iu8f_mlp_w4_tm1_a80") and d.block[0] == 1024
    assert d.grid[0] <= 256 and d.grid[0] * 8 >= max(I // 16, H // 32)      # one workgroup a CU, at most 8 blocks each
    assert {w.name: w.bytes for w in d.workspaces[:d.n_workspaces]} == {b"p": M * I * 2, b"state": iu8.MLP_CHAIN_STATE_BYTES}
    mlp = Mlp(M, H, I, seed=M + I)
    want_gu, want_p, want_c = mlp.oracle()
    for rep in range(3):                                # launches in a row on one state block: no clearing between
        mlp.c.fill_(0x7FC0)
        mlp.chain(ctx)
        assert not mlp.state[SLOTS:].any().item(), "a completed launch leaves its meeting words and the status at zero"
        np.testing.assert_array_equal(host_u16(mlp.gu), want_gu)
        np.testing.assert_array_equal(host_u16(mlp.p), want_p)
        np.testing.assert_array_equal(host_u16(mlp.c), want_c)
    mlp.gu.fill_(0x7FC0), mlp.c.fill_(0x7FC0)            # without the [gate | up] tap: nothing stored there
    mlp.chain(ctx, tap=False)
    assert (mlp.gu == 0x7FC0).all().item()
    np.testing.assert_array_equal(host_u16(mlp.c), want_c)
    gu3, c3 = mlp.three_launches(ctx)
    np.testing.assert_array_equal(gu3, want_gu)
    np.testing.assert_array_equal(c3, want_c)


def test_chain_meeting_gives_up_after_its_poll_limit_and_says_so(ctx):
    """One poll a meeting: the first workgroup to look finds the others not yet arrived, raises the
    status word and leaves, and every other workgroup leaves at its next meeting. The launch ends by
    itself; after the host clears `state` the same buffers give the right bytes."""
    M, H, I = 1, 1024, 2048
    say(f"mlp chain poll limit M={M} H={H} I={I}")
    mlp = Mlp(M, H, I, seed=5)
    mlp.c.zero_()
    mlp.chain(ctx, spin=1)
    assert mlp.state[STATUS].item() != 0, "a wait that ran out of polls raises the status word"
    assert (mlp.c == 0x7FC0).all().item(), "a launch that gave up fills its output with bf16 NaNs"
    # a later launch on the state block as it was left (a graph replay that nobody checked): it cannot
    # complete either, and its output says so instead of carrying stale rows
    mlp.c.zero_()
    mlp.chain(ctx)
    assert mlp.state[STATUS].item() != 0 and (mlp.c == 0x7FC0).all().item()
    mlp.state.zero_()
    mlp.chain(ctx)
    assert not mlp.state[SLOTS:].any().item()
    np.testing.assert_array_equal(host_u16(mlp.c), mlp.oracle()[2])


def test_one_state_block_serves_launches_of_different_shapes_and_inputs(ctx):
    """One state block handed from launch to launch: a larger grid then a smaller one, larger magnitudes then
    smaller ones (the maxima slots of workgroups the second launch does not have keep the first launch's
    values and must not reach its scales), then back; every launch against the oracle."""
    say("mlp chain: one state block, different shapes and inputs")
    state = torch.zeros(iu8.MLP_CHAIN_STATE_BYTES // 4, dtype=torch.int32, device="cuda")
    big, small = Mlp(1, 5120, 17408, seed=21), Mlp(2, 1024, 2048, seed=22)
    big.X = synth.f32_to_bf16_bits(synth.bf16_bits_to_f32(big.X) * np.float32(64.0))     # large rows first
    big.x = dev_bf16_bits(big.X)
    assert iu8.resolve_mlp_chain(1, 5120, 17408).grid[0] > iu8.resolve_mlp_chain(2, 1024, 2048).grid[0]
    want = {id(m): m.oracle() for m in (big, small)}
    for mlp in (big, small, big, small, small):
        mlp.state = state
        mlp.c.fill_(0x7FC0)
        mlp.chain(ctx)
        assert not state[SLOTS:].any().item()
        np.testing.assert_array_equal(host_u16(mlp.p), want[id(mlp)][1])
        np.testing.assert_array_equal(host_u16(mlp.c), want[id(mlp)][2])


def test_chain_refuses_what_the_form_does_not_hold(ctx):
    for m, h, i, word in ((5, 1024, 2048, "fused form"), (4, 5120, 20608, "fused form"), (4, 5248, 5120, "fused form"), (1, 5120, 17400, "multiple"),
                          (0, 1024, 2048, "nothing")):
        with pytest.raises(iu8.IU8Error) as e:
            iu8.resolve_mlp_chain(m, h, i)
        assert e.value.code == iu8.E_RULE and word in str(e.value)
    # a grid the kernel's bounds or the device's residency do not allow is refused at launch
    d = iu8.resolve_mlp_chain(1, 1024, 2048)
    x = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    bufs = {k: x.data_ptr() for k in ("x", "w", "ws", "w_b", "ws_b", "gu", "p", "state", "c")}
    assert x.numel() >= iu8.MLP_CHAIN_STATE_BYTES
    before = ctx.counters().launches
    d.grid[0] = 4096
    with pytest.raises(iu8.IU8Error) as e:
        ctx.launch(d, bufs)
    assert e.value.code == iu8.E_RULE and "at most 512 workgroups" in str(e.value)
    d.grid[0] = 300                                     # fits the state block, but one 16-wave workgroup a CU: 256 at once
    with pytest.raises(iu8.IU8Error) as e:
        ctx.launch(d, bufs)
    assert e.value.code == iu8.E_RULE and "resident" in str(e.value)
    d.grid[0] = 8                                       # 128 column blocks of gate+up: more than 8 x 8
    with pytest.raises(iu8.IU8Error) as e:
        ctx.launch(d, bufs)
    assert e.value.code == iu8.E_RULE and "column blocks" in str(e.value)
    assert ctx.counters().launches == before


@pytest.mark.parametrize("M,H,I,grid", [(16, 5120, 17408, 0), (8, 5120, 17408, 0), (5, 1408, 2944, 0), (13, 640, 12672, 100), (1, 384, 384, 0),
                                         (3, 17408, 256, 0), (16, 2048, 4096, 32)])
def test_gate_up_linear_with_the_activation_in_its_epilogue(ctx, M, H, I, grid):
    """saber_iu8_gate_up_act: quantised rows in, p = bf16(bf16(silu(gate)) * up) out, the [gate | up] tap beside it --
    the oracle's linear and its SiLU * up, and the plain quantiser on p gives silu_mul_quant's codes and scales. Full and
    ragged row counts, the benchmark layer, K steps that do not divide among the k-waves, few live rows of a long K,
    a grid that gives workgroups an uneven share."""
    say(f"gate+up with activation M={M} H={H} I={I} grid={grid}")
    mlp = Mlp(M, H, I, seed=3 * M + I)
    want_gu = ref.linear(mlp.X, mlp.Wgu, mlp.wsgu, False, threads=16)["C"]
    want_q, want_s, want_p = ref.silu_mul_quant(want_gu)
    assert iu8.gate_up_act_holds(M, H, I)
    q0 = torch.full((iu8.a_bytes(M, H),), 0x55, dtype=torch.uint8, device="cuda")
    s0 = torch.zeros(M, dtype=torch.float32, device="cuda")
    ctx.quant(mlp.x.data_ptr(), q0.data_ptr(), s0.data_ptr(), M, H)
    for tap in (True, False):
        gu = torch.full((M, 2 * I), 0x7FC0, dtype=torch.int16, device="cuda")
        p = torch.full((M, I), 0x7FC0, dtype=torch.int16, device="cuda")
        if grid:
            d = iu8.resolve_gate_up_act(M, H, I)
            assert grid * 8 >= I // 16
            d.grid[0] = grid
            if not tap:
                d.arg("gu").kind = iu8.ARG_NULL_BUFFER
            bufs = {"a": q0.data_ptr(), "w": mlp.wgu.data_ptr(), "as": s0.data_ptr(), "ws": mlp.wsg.data_ptr(), "p": p.data_ptr()}
            if tap:
                bufs["gu"] = gu.data_ptr()
            ctx.launch(d, bufs)
        else:
            ctx.gate_up_act(q0.data_ptr(), s0.data_ptr(), mlp.wgu.data_ptr(), mlp.wsg.data_ptr(), gu.data_ptr() if tap else None, p.data_ptr(), M, H, I)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(p), want_p)
        if tap:
            np.testing.assert_array_equal(host_u16(gu), want_gu)
        else:
            assert (host_u16(gu) == 0x7FC0).all()
    q = torch.full((iu8.a_bytes(M, I),), 0x55, dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    ctx.quant(p.data_ptr(), q.data_ptr(), s.data_ptr(), M, I)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, I), want_q)
    if I % 64 == 0:   # ... and in the Hadamard basis: the transform + quantiser on p is silu_mul_quant_had on [gate | up]
        t = (np.random.default_rng(I).choice([-1.0, 1.0], size=I) * np.random.default_rng(I + 1).uniform(0.5, 2.0, size=I)).astype(np.float32)
        td = dev_f32(t)
        qh = torch.full((iu8.a_bytes(M, I),), 0x55, dtype=torch.uint8, device="cuda")
        sh = torch.zeros(M, dtype=torch.float32, device="cuda")
        ctx.quant_had(p.data_ptr(), qh.data_ptr(), sh.data_ptr(), M, I, td.data_ptr())
        torch.cuda.synchronize()
        hq, hs = ref.silu_mul_quant_had(want_gu, t)
        np.testing.assert_array_equal(sh.cpu().numpy().view(np.uint32), hs.view(np.uint32))
        np.testing.assert_array_equal(iu8.unpack_a(qh.cpu().numpy(), M, I), hq)
    for bad in (lambda: iu8.resolve_gate_up_act(17, H, I), lambda: iu8.resolve_gate_up_act(16, 5248, I), lambda: iu8.resolve_gate_up_act(M, H, I + 8)):
        with pytest.raises(iu8.IU8Error) as e:
            bad()
        assert e.value.code == iu8.E_RULE
