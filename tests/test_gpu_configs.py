"""GPU parity at the benchmark configurations' own shapes and edge cases: golden vectors, the mixed
W4/W8 launch sequence, every kernel variant of a regime giving the same bytes, the explicit grid
split with its workspaces, and size-independent properties at the full sizes."""
import os
import re

import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from tests.gpu_util import DenseRun, assert_dense_matches, dev_bf16_bits, dev_f32, dev_u8, host_u16, say

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "dense_small.npz"))


@pytest.mark.parametrize("i", range(5))
def test_golden_vectors(ctx, i):
    M, N, K, w8 = [int(v) for v in GOLD[f"c{i}_meta"]]
    say(f"golden vector {i}: M={M} N={N} K={K} w8={w8}")
    case = dict(M=M, N=N, K=K, w8=bool(w8), X=GOLD[f"c{i}_X"], W=GOLD[f"c{i}_W"], ws=GOLD[f"c{i}_ws"])
    run = DenseRun(ctx, case, want_acc=True)
    want = dict(q=GOLD[f"c{i}_q"], a_scale=GOLD[f"c{i}_a_scale"], S=GOLD[f"c{i}_S"], C=GOLD[f"c{i}_C"])
    assert_dense_matches(run, want, bool(w8))


def test_config0_single_gemv(ctx):
    say("config 0: M=1 K=5120 N=5120 seed 0")
    case = synth.dense_case(1, 5120, 5120, seed=0)
    r = ref.linear(case["X"], case["W"], case["ws"], False, threads=8)
    assert_dense_matches(DenseRun(ctx, case), r, False)


@pytest.mark.parametrize("M", [1, 4, 8, 16])
def test_config1_decode_layer_set(ctx, M):
    for name, n, k in synth.LAYER_LINEARS:
        say(f"config 1: {name} M={M} N={n} K={k}")
        case = synth.dense_case(M, n, k, seed=M)
        r = ref.linear(case["X"], case["W"], case["ws"], False, threads=16)
        assert_dense_matches(DenseRun(ctx, case), r, False)


@pytest.mark.parametrize("M", [1, 2, 4])
def test_config1_decode_layer_set_as_the_fused_launches_the_benchmark_times(ctx, M):
    """The hot path as bench.py launches it: one fused quant + GEMV launch a linear where the law fuses
    (macaq_iu8_decq_w4_r1 at one long row, macaq_iu8_decq_w4_tm1, the 80 KiB form for down at two rows), producer + GEMV
    where it does not (down at four rows), on the four full layer shapes, against the oracle."""
    for name, n, k in synth.LAYER_LINEARS:
        say(f"config 1, as the benchmark launches it: {name} M={M} N={n} K={k}")
        case = synth.dense_case(M, n, k, seed=M)
        r = ref.linear(case["X"], case["W"], case["ws"], False, threads=16)
        if not iu8.fused_holds(M, k):
            assert (M, k) in ((4, 17408), (3, 17408))
            assert_dense_matches(DenseRun(ctx, case, want_acc=False), r, False)
            continue
        x, wf, ws = dev_bf16_bits(case["X"]), dev_u8(iu8.repack_w4(case["W"])), dev_f32(case["ws"])
        c = torch.full((M, n), 0x7FC0, dtype=torch.int16, device="cuda")
        d = iu8.resolve_fused(iu8.W4, M, n, k)
        # one long row (down): the just-in-time form; down at 2 rows: the 80 KiB form
        assert d.kernel == (b"macaq_iu8_decq_w4_r1" if M == 1 and k >= 8192 else b"macaq_iu8_decq_w4_tm1" if iu8.fused_small_holds(M, k) else b"macaq_iu8_decq_w4_tm1_a80")
        for a in ("q", "scale"):                # as the benchmark launches it: no optional outputs
            d.arg(a).kind = iu8.ARG_NULL_BUFFER
        ctx.launch(d, dict(x=x.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr()))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host_u16(c), r["C"])


# the iu8 linears of the reference's own 27B graph at TP = 1 (crates/saber-kernels/src/macaq_iu8.rs:931-947:
# GDN in_proj_qkvz / in_proj_ba, gated attention qkv, out_proj / o_proj, MLP gate_up / down) -- the benchmark's
# "27B-class" set shares only the last two with it
SERVED_27B = [("gdn_qkvz", 16384, 5120), ("gdn_ba", 96, 5120), ("attn_qkv", 14336, 5120), ("o_proj", 5120, 6144),
              ("gate_up", 34816, 5120), ("down", 5120, 17408)]


@pytest.mark.parametrize("M", [1, 3, 16, 40, 300])
def test_linear_shapes_of_the_served_27b_graph(ctx, M):
    """Decode (fused where the law fuses, else producer + GEMM), the streamed band and a ragged prefill row count on
    the served model's shapes, N = 96 (six column tiles: a workgroup with a dead tile) included."""
    for name, n, k in SERVED_27B:
        w8 = name in ("o_proj", "down") and M in (3, 40)     # the graph promotes some output-side projections to int8 rows
        say(f"served 27B shape: {name} M={M} N={n} K={k} w8={w8}")
        case = synth.dense_case(M, n, k, w8=w8, seed=100 + M)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=16)
        run = DenseRun(ctx, case, want_acc=False)
        assert_dense_matches(run, r, w8)
        if iu8.fused_holds(M, k):
            c = torch.full((M, n), 0x7FC0, dtype=torch.int16, device="cuda")
            ctx.linear_fused(iu8.W8 if w8 else iu8.W4, run.dev["x"].data_ptr(), run.dev["wf"].data_ptr(), run.dev["ws"].data_ptr(),
                             c.data_ptr(), M, n, k)
            torch.cuda.synchronize()
            np.testing.assert_array_equal(host_u16(c), r["C"])


def test_launch_refuses_a_block_the_kernel_is_not_written_for(ctx):
    """A descriptor under another launch law (the reference's 256-thread blocks under its own names,
    crates/saber-kernels/src/macaq_iu8.rs:429-489) is refused by name before anything is launched."""
    x = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    for kernel, m in (("macaq_iu8_pf_w4_tn4_lbk64", 256), ("macaq_iu8_dec_w4_tm1", 1)):
        d = iu8.describe(kernel, m, 128, 256)
        d.block[0] = 256                         # the reference's block
        bufs = dict(a=x.data_ptr(), w=x.data_ptr(), ws=x.data_ptr(), c=x.data_ptr())
        bufs["as"] = x.data_ptr()
        before = ctx.counters().launches
        with pytest.raises(iu8.IU8Error) as e:
            ctx.launch(d, bufs)
        assert e.value.code == iu8.E_RULE and "threads" in str(e.value)
        assert ctx.counters().launches == before


def all_variants(prefix):
    text = open(os.path.join(iu8.PKG, "csrc", "kernels", "iu8_variants.def")).read()
    names = re.findall(r"^IU8_(?:DEC|PF)_VARIANT\((\w+),", text, flags=re.M)
    return [n for n in names if n.startswith(prefix) and not n.endswith("_acc")]


@pytest.mark.parametrize("tag,w8", [("w4", False), ("w8", True)])
def test_every_decode_variant_gives_the_same_bytes(ctx, tag, w8):
    case = synth.dense_case(5, 176, 1664, w8=w8, seed=21)     # 11 n-tiles (ragged blocks), 13 K steps
    r = ref.linear(case["X"], case["W"], case["ws"], w8)
    names = all_variants(f"macaq_iu8_dec_{tag}_tm")
    assert len(names) >= 4
    for name in names:
        for ks in (1, 2, 3):
            say(f"variant {name} ks={ks}")
            run = DenseRun(ctx, case, kernel=name, ks=ks, want_acc=False)
            np.testing.assert_array_equal(run.C, r["C"])
            if ks > 1:
                assert not run.counter.cpu().numpy().any(), "the arrival counters must be left at zero"


@pytest.mark.parametrize("tag,w8", [("w4", False), ("w8", True)])
def test_every_prefill_variant_gives_the_same_bytes(ctx, tag, w8):
    case = synth.dense_case(200, 272, 640, w8=w8, seed=22)
    r = ref.linear(case["X"], case["W"], case["ws"], w8)
    for name in all_variants(f"macaq_iu8_pf_{tag}_"):
        say(f"variant {name}")
        run = DenseRun(ctx, case, kernel=name, want_acc=False)
        np.testing.assert_array_equal(run.C, r["C"])


def test_prefill_several_tiles_a_workgroup_on_every_tile(ctx):
    """More tiles than workgroups for every cell, the largest included, and seven K steps a tile: more
    than the deepest cell's load stream runs ahead, so every cell hands a tile's epilogue scales over
    through LDS a tile ahead (with fewer steps a cell fetches them in the epilogue: the edge shapes below
    take that path, on two to five steps)."""
    M, N, K = 8320, 4352, 896
    for tag, w8 in (("w4", False), ("w8", True)):
        case = synth.dense_case(M, N, K, w8=w8, seed=5)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        for name in all_variants(f"macaq_iu8_pf_{tag}_"):
            say(f"prefill, several tiles a workgroup {(M, N, K)} {name}")
            run = DenseRun(ctx, case, kernel=name, want_acc=False)
            np.testing.assert_array_equal(run.C, r["C"])


@pytest.mark.parametrize("shape", [(65, 16, 128), (97, 48, 256), (129, 304, 384), (4160, 1088, 256), (4160, 1088, 384), (4160, 1088, 512)])
def test_prefill_edges_on_every_tile(ctx, shape):
    """One K step, two K steps (fewer than the LDS stages), ragged rows and columns, a tile count
    above the persistent grid (several tiles a workgroup, the load stream running across tiles)."""
    M, N, K = shape
    for tag, w8 in (("w4", False), ("w8", True)):
        case = synth.dense_case(M, N, K, w8=w8, seed=31 + M)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        for name in all_variants(f"macaq_iu8_pf_{tag}_"):
            say(f"prefill edge {shape} {name}")
            run = DenseRun(ctx, case, kernel=name, want_acc=False)
            np.testing.assert_array_equal(run.C, r["C"])
        run = DenseRun(ctx, case, want_acc=True)            # the launch law's cell and the int32 tap
        assert_dense_matches(run, r, w8)


SPLIT_CELLS = {"w4": ("t128x128", "t256x160", "t64x128_s"), "w8": ("t128x128", "t256x160")}


@pytest.mark.parametrize("shape,splits", [((200, 272, 640), (1, 2, 3, 5)), ((129, 304, 384), (2, 3)), ((300, 1040, 2048), (4, 8)),
                                          ((520, 528, 1280), (2, 5))])
def test_tile_gemm_with_k_split_over_workgroups(ctx, shape, splits):
    """The `_ks` forms: shares of the K steps on gridDim.z, partials handed over through memory, the
    last share to arrive sums and stores. Same bytes as the oracle for every cell and share count,
    ragged edges, more tiles than workgroups a share, counters left at zero and re-usable."""
    M, N, K = shape
    for tag, w8 in (("w4", False), ("w8", True)):
        case = synth.dense_case(M, N, K, w8=w8, seed=51 + M)
        r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
        for cell in SPLIT_CELLS[tag]:
            for ks in splits:
                name = f"macaq_iu8_pf_{tag}_{cell}_ks"
                say(f"split tile GEMM {shape} {name} ks={ks}")
                run = DenseRun(ctx, case, kernel=name, ks=ks, want_acc=False)
                assert run.desc.grid[2] == ks
                np.testing.assert_array_equal(run.C, r["C"])
                if ks > 1:
                    assert not run.counter.cpu().numpy().any(), "the arrival counters must be left at zero"
                    d = run.dev
                    d["c"].fill_(0)
                    bufs = dict(a=d["q"].data_ptr(), w=d["wf"].data_ptr(), ws=d["ws"].data_ptr(), c=d["c"].data_ptr(),
                                decode_partial=run.partial.data_ptr(), decode_counter=run.counter.data_ptr())
                    bufs["as"] = d["a_scale"].data_ptr()
                    ctx.launch(run.desc, bufs)
                    torch.cuda.synchronize()
                    np.testing.assert_array_equal(host_u16(d["c"]), r["C"])
    with pytest.raises(iu8.IU8Error):
        iu8.describe("macaq_iu8_pf_w4_t128x128_ks", 200, 272, 640, ks=4)          # 5 steps in 4 shares: the last is empty
    with pytest.raises(iu8.IU8Error):
        iu8.describe("macaq_iu8_pf_w4_t128x128", 200, 272, 640, ks=2)             # the plain cell does not split


@pytest.mark.parametrize("shape,ks", [((64, 384, 16384), 4), ((100, 640, 17408), 4), ((128, 5120, 17408), 3),
                                      ((129, 5120, 17408), 2), ((192, 3072, 16384), 3), ((77, 8192, 16384), 2)])
def test_launch_law_splits_deep_narrow_tile_gemm(ctx, shape, ks):
    """Where the law shares K over workgroups (K >= 16384, up to 192 rows, at most 128 tiles of the 64x128 cell) the
    descriptor lists the workspaces and the launch through it gives the oracle's bytes."""
    M, N, K = shape
    say(f"law-split tile GEMM {shape}")
    case = synth.dense_case(M, N, K, seed=77 + M)
    run = DenseRun(ctx, case, want_acc=False)
    assert run.desc.kernel.decode() == "macaq_iu8_pf_w4_t64x128_s_ks" and run.desc.ks == ks
    cols = min(N, 512)
    qh, sh = ref.quant_bf16(case["X"])
    S, _ = ref.gemm_fast(qh, case["W"][:cols], False, threads=16)
    np.testing.assert_array_equal(run.C[:, :cols], ref.epilogue(S, sh, case["ws"][:cols], False))
    S, _ = ref.gemm_fast(qh, case["W"][-cols:], False, threads=16)
    np.testing.assert_array_equal(run.C[:, -cols:], ref.epilogue(S, sh, case["ws"][-cols:], False))
    assert not run.counter.cpu().numpy().any()


@pytest.mark.parametrize("grid", [8, 10, 11])
@pytest.mark.parametrize("tag,w8", [("w4", False), ("w8", True)])
def test_last_round_of_the_256x256_cell_runs_as_quarter_tiles(ctx, grid, tag, w8):
    """12 tiles of the 256 x 256 cell (ragged both ways) on 8, 10 or 11 persistent workgroups: one full
    round, then the 4 / 2 / 1 remaining tiles as quarter tiles on the 128 x 128 cell; same bytes as the oracle."""
    M, N, K = 700, 1008, 640
    say(f"256x256 cell, last round as quarter tiles: grid {grid} {tag}")
    case = synth.dense_case(M, N, K, w8=w8, seed=grid)
    r = ref.linear(case["X"], case["W"], case["ws"], w8, threads=8)
    q, s = ref.quant_bf16(case["X"])
    qd = dev_u8(iu8.repack_a(q))
    sd, wf, wsd = dev_f32(s), dev_u8(iu8.repack_weights(case["W"], w8)), dev_f32(case["ws"])
    c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
    d = iu8.describe_raw(f"macaq_iu8_pf_{tag}_tn4_lbk64", (grid, 1, 1), 512, plugin="macaq_iu8", m=M, n=N, k=K)
    bufs = dict(a=qd.data_ptr(), w=wf.data_ptr(), ws=wsd.data_ptr(), c=c.data_ptr())
    bufs["as"] = sd.data_ptr()
    ctx.launch(d, bufs)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(host_u16(c), r["C"])


def test_split_counter_is_reusable_across_launches(ctx):
    say("explicit split, two launches on one counter")
    case = synth.dense_case(3, 256, 2048, seed=23)
    r = ref.linear(case["X"], case["W"], case["ws"], False)
    run = DenseRun(ctx, case, kernel="macaq_iu8_dec_w4_tm1", ks=4, want_acc=False)
    np.testing.assert_array_equal(run.C, r["C"])
    d = run.dev
    d["c"].fill_(0)
    bufs = dict(a=d["q"].data_ptr(), w=d["wf"].data_ptr(), ws=d["ws"].data_ptr(), c=d["c"].data_ptr(),
                decode_partial=run.partial.data_ptr(), decode_counter=run.counter.data_ptr())
    bufs["as"] = d["a_scale"].data_ptr()
    ctx.launch(run.desc, bufs)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(host_u16(d["c"]), r["C"])


def test_config3_mixed_w4_w8_sequence(ctx):
    """19 int8-row linears among 64, one launch sequence on shared per-token activations, M=16 and
    (on an N slice of the oracle) M=2048; int32 accumulators bit-exact per linear."""
    seq = synth.mixed_sequence()
    assert sum(1 for s in seq if s[3]) == 19
    shapes = sorted({(n, k, w8) for _, n, k, w8 in seq})
    for M in (16, 2048):
        rng = np.random.default_rng(M)
        acts = {k: synth.activations(rng, M, k) for k in (5120, 17408)}
        quant = {k: ref.quant_bf16(x) for k, x in acts.items()}
        dev = {}
        for k, x in acts.items():
            xd = dev_bf16_bits(x)
            q = torch.zeros(iu8.a_bytes(M, k), dtype=torch.uint8, device="cuda")
            s = torch.zeros(M, dtype=torch.float32, device="cuda")
            ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, k)
            dev[k] = (q, s)
        for (n, k, w8) in shapes:
            say(f"config 3: M={M} N={n} K={k} w8={w8}")
            W, ws = synth.weights(rng, n, k, w8)
            wk = iu8.W8 if w8 else iu8.W4
            wf, wsd = dev_u8(iu8.repack_weights(W, w8)), dev_f32(ws)
            c = torch.zeros((M, n), dtype=torch.int16, device="cuda")
            q, s = dev[k]
            ctx.gemm(wk, q.data_ptr(), s.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), M, n, k)
            acc = torch.zeros((M, n), dtype=torch.int32, device="cuda")
            ctx.gemm_acc(wk, q.data_ptr(), wf.data_ptr(), acc.data_ptr(), M, n, k)
            torch.cuda.synchronize()
            qh, sh = quant[k]
            cols = n if M == 16 else 512                      # the oracle checks an N slice at M=2048
            Wc = W[:cols]
            S, _ = ref.gemm_fast(qh, Wc, w8, threads=16)
            np.testing.assert_array_equal(acc.cpu().numpy()[:, :cols], S if w8 else S * 16)
            np.testing.assert_array_equal(host_u16(c)[:, :cols], ref.epilogue(S, sh, ws[:cols], w8))
            # the whole int32 accumulator through a size-independent property: column sums are the
            # product of the activations' column-summed codes with the weights (exact in int64)
            colsum = qh.astype(np.int64).sum(0)
            wfull = W.astype(np.int64) if w8 else synth.unpack_w4(W).astype(np.int64)
            want = wfull @ colsum * (1 if w8 else 16)
            np.testing.assert_array_equal(acc.cpu().numpy().astype(np.int64).sum(0), want)
            del wf, wsd, c, acc


@pytest.mark.parametrize("M", [256, 2048, 8192])
def test_config2_prefill_full_shapes_by_properties(ctx, M):
    """Full prefill shapes: an oracle slice bit for bit, and the whole accumulator by linearity
    (sum over rows of A.W^T == (sum over rows of A).W^T, exact in integers)."""
    rng = np.random.default_rng(M)
    for name, n, k in synth.LAYER_LINEARS:
        if M == 8192 and name == "gate_up":
            continue                                       # its int32 tap would be 1.1 GB: the test below, by column quarters
        say(f"config 2: {name} M={M} N={n} K={k}")
        W, ws = synth.weights(rng, n, k, False)
        X = synth.activations(rng, M, k)
        xd, wf, wsd = dev_bf16_bits(X), dev_u8(iu8.repack_w4(W)), dev_f32(ws)
        q = torch.zeros(iu8.a_bytes(M, k), dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        c = torch.zeros((M, n), dtype=torch.int16, device="cuda")
        acc = torch.zeros((M, n), dtype=torch.int32, device="cuda")
        ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, k)
        ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), M, n, k)
        ctx.gemm_acc(iu8.W4, q.data_ptr(), wf.data_ptr(), acc.data_ptr(), M, n, k)
        torch.cuda.synchronize()
        qh, sh = ref.quant_bf16(X)
        np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, k), qh)
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), sh.view(np.uint32))
        rows = np.unique(np.concatenate([np.arange(0, M, max(1, M // 37)), [M - 1]]))
        cols = 256
        S, _ = ref.gemm_fast(qh[rows], W[-cols:], False, threads=16)
        np.testing.assert_array_equal(acc.cpu().numpy()[rows][:, -cols:], S * 16)
        np.testing.assert_array_equal(host_u16(c)[rows][:, -cols:], ref.epilogue(S, sh[rows], ws[-cols:], False))
        want = synth.unpack_w4(W).astype(np.int64) @ qh.astype(np.int64).sum(0) * 16
        np.testing.assert_array_equal(acc.sum(0, dtype=torch.int64).cpu().numpy(), want)
        # bf16 outputs of the whole matrix from the device's own accumulators (the epilogue is elementwise)
        t = (acc.to(torch.float32) * s[:, None]) * (wsd * 0.0625)[None, :]
        assert torch.equal(t.to(torch.bfloat16).view(torch.int16), c)
        del xd, wf, wsd, q, s, c, acc, t
        torch.cuda.empty_cache()


def test_config2_gate_up_at_8192_rows_full_width(ctx):
    """gate+up 34816 x 5120 at M = 8192, the largest cell of configs[2], at its full width: the bf16
    output of ONE launch over all 34,816 columns; the int32 tap on column quarters (the rows of W are
    16-row fragments, so a quarter of the columns is a contiguous quarter of the weight bytes), every
    quarter by linearity and by the device-side epilogue identity, an oracle slice bit for bit."""
    M, n, k = 8192, 34816, 5120
    say(f"config 2: gate_up M={M} N={n} K={k}, full width")
    rng = np.random.default_rng(8192)
    W, ws = synth.weights(rng, n, k, False)
    X = synth.activations(rng, M, k)
    xd, wf, wsd = dev_bf16_bits(X), dev_u8(iu8.repack_w4(W)), dev_f32(ws)
    q = torch.zeros(iu8.a_bytes(M, k), dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    c = torch.zeros((M, n), dtype=torch.int16, device="cuda")
    ctx.quant(xd.data_ptr(), q.data_ptr(), s.data_ptr(), M, k)
    ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), M, n, k)
    torch.cuda.synchronize()
    qh, sh = ref.quant_bf16(X)
    np.testing.assert_array_equal(iu8.unpack_a(q.cpu().numpy(), M, k), qh)
    colsum = qh.astype(np.int64).sum(0)
    rows = np.unique(np.concatenate([np.arange(0, M, 331), [M - 1]]))
    nq = n // 4
    acc = torch.zeros((M, nq), dtype=torch.int32, device="cuda")
    for part in range(4):
        say(f"config 2: gate_up M={M}, int32 tap on columns {part * nq}..{(part + 1) * nq}")
        c0 = part * nq
        ctx.gemm_acc(iu8.W4, q.data_ptr(), wf.data_ptr() + c0 * k // 2, acc.data_ptr(), M, nq, k)
        torch.cuda.synchronize()
        want = synth.unpack_w4(W[c0:c0 + nq]).astype(np.int64) @ colsum * 16
        np.testing.assert_array_equal(acc.sum(0, dtype=torch.int64).cpu().numpy(), want)
        t = (acc.to(torch.float32) * s[:, None]) * (wsd[c0:c0 + nq] * 0.0625)[None, :]
        assert torch.equal(t.to(torch.bfloat16).view(torch.int16), c[:, c0:c0 + nq])
        S, _ = ref.gemm_fast(qh[rows], W[c0 + nq - 128:c0 + nq], False, threads=16)
        np.testing.assert_array_equal(acc.cpu().numpy()[rows][:, -128:], S * 16)
        np.testing.assert_array_equal(host_u16(c)[rows][:, c0 + nq - 128:c0 + nq], ref.epilogue(S, sh[rows], ws[c0 + nq - 128:c0 + nq], False))
        del t


def test_split_k_hand_over_repeats_on_full_size_shapes(ctx):
    """A bounded soak of the cross-workgroup hand-over of the split forms (partials straight through
    memory, a relaxed device-scope arrival counter, no fences) at the sizes the launch law and the
    explicit splits run at: every repeat must give the first launch's bytes, which are the oracle's on
    a column slice; the counters stay zero. Stops at its first mismatch."""
    for kernel, (M, N, K), ks, reps in (("macaq_iu8_pf_w4_t64x128_s_ks", (128, 5120, 17408), 3, 40),
                                        ("macaq_iu8_pf_w4_t64x128_s_ks", (64, 5120, 17408), 4, 40),
                                        ("macaq_iu8_dec_w4_tm1", (1, 5120, 17408), 4, 60),
                                        ("macaq_iu8_dec_w4_tm1_a0", (16, 7168, 5120), 2, 60),
                                        ("macaq_iu8_dec_w4_tm2", (32, 5120, 5120), 3, 40)):
        say(f"split hand-over soak {kernel} {M}x{N}x{K} ks={ks} x{reps}")
        case = synth.dense_case(M, N, K, seed=ks * 100 + M)
        run = DenseRun(ctx, case, kernel=kernel, ks=ks, want_acc=False)
        qh, sh = ref.quant_bf16(case["X"])
        S, _ = ref.gemm_fast(qh, case["W"][:512], False, threads=16)
        np.testing.assert_array_equal(run.C[:, :512], ref.epilogue(S, sh, case["ws"][:512], False))
        d = run.dev
        first = d["c"].clone()
        bufs = dict(a=d["q"].data_ptr(), w=d["wf"].data_ptr(), ws=d["ws"].data_ptr(), c=d["c"].data_ptr(),
                    decode_partial=run.partial.data_ptr(), decode_counter=run.counter.data_ptr())
        bufs["as"] = d["a_scale"].data_ptr()
        for rep in range(reps):
            d["c"].fill_(0x7FC0)
            run.partial.fill_(0x5A5A5A5A + rep)           # scratch: undefined at entry
            ctx.launch(run.desc, bufs)
            torch.cuda.synchronize()
            assert torch.equal(d["c"], first), f"repeat {rep} of {kernel} differs"
            assert not run.counter.any().item(), "the arrival counters must be left at zero"


def test_config4_moe_prefill_shape(ctx):
    """T=4096 routed tokens, 128 experts, top-8, H=4096, I=1536 (4 distinct expert weight sets)."""
    from saber_engine_amd.moe import MoeLayerIU8
    from tests.test_gpu_moe import check_layer, run_layer

    say("config 4: T=4096 E=128 top-8 H=4096 I=1536")
    case = synth.moe_case(T=4096, E=128, topk=8, H=4096, I=1536, seed=0, experts=4)
    layer = run_layer(ctx, case)
    assert layer.tb == 16 and layer.gather == 2
    check_layer(layer, case, taps=False)
