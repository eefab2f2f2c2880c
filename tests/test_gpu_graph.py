"""Capture legality and re-entrancy (launch conventions of crates/saber-exec/src/launch.rs:590-660: no
allocation, no synchronisation, one launch an op, kernels re-entrant across graph replays): a launch
train of every kind of launch this library makes -- fused decode linear, producer + GEMV, the decode
pair, the decode MLP chain, a tile GEMM whose law splits K (arrival counters), the quarter-tile 256x256 cell, a routed layer
-- is captured into one HIP graph and replayed several times with other work in between; every
replay's bytes equal the eager run's."""
import numpy as np
import pytest
import torch

from saber_engine_amd import iu8, synth
from saber_engine_amd.moe import MoeLayerIU8
from tests.gpu_util import dev_bf16_bits, dev_f32, dev_u8, host_u16, say

pytestmark = pytest.mark.gpu


def test_launch_train_replays_bit_identically(ctx):
    say("graph capture of a mixed launch train, three replays")
    rng = np.random.default_rng(11)
    stream = torch.cuda.Stream()
    sh = stream.cuda_stream
    keep, outs, train = [], [], []

    def linear(M, N, K, fused=False):
        W, ws = synth.weights(rng, N, K, False)
        x = dev_bf16_bits(synth.activations(rng, M, K))
        wf, wsd = dev_u8(iu8.repack_w4(W)), dev_f32(ws)
        c = torch.zeros((M, N), dtype=torch.int16, device="cuda")
        keep.extend([x, wf, wsd])
        outs.append(c)
        if fused:
            train.append(lambda: ctx.linear_fused(iu8.W4, x.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), M, N, K, stream=sh))
            return
        q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        pb, cb = iu8.gemm_workspace(iu8.W4, M, N, K)
        part = torch.full((max(pb // 4, 1),), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
        cnt = torch.zeros(max(cb // 4, 1), dtype=torch.int32, device="cuda")
        keep.extend([q, s, part, cnt])
        train.append(lambda: ctx.quant(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K, stream=sh))
        train.append(lambda: ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), M, N, K,
                                      part.data_ptr() if pb else None, cnt.data_ptr() if cb else None, stream=sh))

    linear(1, 512, 1024, fused=True)          # fused decode linear
    linear(8, 640, 1024)                      # producer + streaming GEMV
    linear(64, 384, 16384)                    # the law splits K: partials and arrival counters
    assert iu8.resolve(iu8.W4, 64, 384, 16384).ks == 4
    linear(300, 528, 640)                     # tile GEMM
    # the decode pair on shared activations
    M, K, n0, n1 = 4, 1024, 768, 96
    W0, s0 = synth.weights(rng, n0, K, False)
    W1, s1 = synth.weights(rng, n1, K, False)
    xp = dev_bf16_bits(synth.activations(rng, M, K))
    qp = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    sp = torch.zeros(M, dtype=torch.float32, device="cuda")
    w0, w1, sd0, sd1 = dev_u8(iu8.repack_w4(W0)), dev_u8(iu8.repack_w4(W1)), dev_f32(s0), dev_f32(s1)
    c0 = torch.zeros((M, n0), dtype=torch.int16, device="cuda")
    c1 = torch.zeros((M, n1), dtype=torch.int16, device="cuda")
    outs.extend([c0, c1])
    train.append(lambda: ctx.quant(xp.data_ptr(), qp.data_ptr(), sp.data_ptr(), M, K, stream=sh))
    train.append(lambda: ctx.gemm_pair(qp.data_ptr(), sp.data_ptr(), w0.data_ptr(), sd0.data_ptr(), c0.data_ptr(), n0,
                                       w1.data_ptr(), sd1.data_ptr(), c1.data_ptr(), n1, M, K, stream=sh))
    # the decode MLP as one persistent launch: its workgroups meet through a state block that the
    # kernel itself leaves at zero, so a replay needs nothing cleared between launches
    Mc, Hc, Ic = 2, 1024, 2560
    Wg, sg = synth.weights(rng, 2 * Ic, Hc, False)
    Wd, sdn = synth.weights(rng, Hc, Ic, False)
    xc = dev_bf16_bits(synth.activations(rng, Mc, Hc))
    wg, wd, sgd, sdd = dev_u8(iu8.repack_w4(Wg)), dev_u8(iu8.repack_w4(Wd)), dev_f32(sg), dev_f32(sdn)
    pc = torch.zeros((Mc, Ic), dtype=torch.int16, device="cuda")
    cc = torch.zeros((Mc, Hc), dtype=torch.int16, device="cuda")
    state = torch.zeros(iu8.MLP_CHAIN_STATE_BYTES // 4, dtype=torch.int32, device="cuda")
    keep.extend([xc, wg, wd, sgd, sdd, pc, state])
    outs.append(cc)
    train.append(lambda: ctx.mlp_chain(xc.data_ptr(), wg.data_ptr(), sgd.data_ptr(), wd.data_ptr(), sdd.data_ptr(), None,
                                       pc.data_ptr(), state.data_ptr(), cc.data_ptr(), Mc, Hc, Ic, stream=sh))
    # a routed layer (router's arrival counter, tile tables rebuilt every replay)
    case = synth.moe_case(T=150, E=128, topk=8, H=512, I=256, seed=3, experts=4)
    layer = MoeLayerIU8(ctx, 150, 128, 8, 512, 256)
    E = 128
    layer.set_weights(torch.from_numpy(np.stack([iu8.repack_w4(case["Wgu"][e]) for e in range(E)])).cuda(), torch.from_numpy(case["wsgu"]).cuda(),
                      torch.from_numpy(np.stack([iu8.repack_w4(case["Wdn"][e]) for e in range(E)])).cuda(), torch.from_numpy(case["wsdn"]).cuda())
    xm, lg = dev_bf16_bits(case["X"]), dev_bf16_bits(case["logits"])
    outs.append(layer.out)
    train.append(lambda: layer.forward(xm, lg, sh))

    def run_train():
        for fn in train:
            fn()

    with torch.cuda.stream(stream):
        run_train()
    torch.cuda.synchronize()
    want = [host_u16(o).copy() for o in outs]
    assert all(w.any() for w in want)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        run_train()
    scratch = torch.zeros(1 << 20, dtype=torch.float32, device="cuda")
    for replay in range(3):
        for o in outs:
            o.fill_(0x7FC0)                    # poison what the replay must rewrite
        scratch.add_(1.0)                      # other eager work and a synchronisation between the replays
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            g.replay()
        torch.cuda.synchronize()
        for i, (o, w) in enumerate(zip(outs, want)):
            np.testing.assert_array_equal(host_u16(o), w, err_msg=f"replay {replay}, output {i}")
