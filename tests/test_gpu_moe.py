"""GPU parity of the routed-expert layer (router, sort, grouped gate+up, SiLU*up requant, grouped
down, combine), called through the C ABI, against the CPU oracle on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from saber_engine_amd.moe import MoeLayerIU8
from tests.gpu_util import dev_bf16_bits, host_u16, say

pytestmark = pytest.mark.gpu


def test_device_silu_equals_host_formula_on_all_65536_inputs(ctx):
    say("silu table, all bf16 inputs")
    out = torch.zeros(65536, dtype=torch.int16, device="cuda")
    ctx.silu_table(out.data_ptr())
    torch.cuda.synchronize()
    got, want = host_u16(out), ref.silu_bf16_table()
    x = synth.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16))
    fin = np.isfinite(x)
    bad = np.flatnonzero(fin & (got != want))
    assert bad.size == 0, [(hex(i), hex(got[i]), hex(want[i])) for i in bad[:8]]


def run_layer(ctx, case, tile_blocks=None, fused_back=None):
    T, E, k, H, I = case["T"], case["E"], case["topk"], case["H"], case["I"]
    layer = MoeLayerIU8(ctx, T, E, k, H, I, tile_blocks=tile_blocks, fused_back=fused_back)
    wgu = torch.from_numpy(np.stack([iu8.repack_w4(case["Wgu"][e]) for e in range(E)])).cuda()
    wdn = torch.from_numpy(np.stack([iu8.repack_w4(case["Wdn"][e]) for e in range(E)])).cuda()
    layer.set_weights(wgu, torch.from_numpy(case["wsgu"]).cuda(), wdn, torch.from_numpy(case["wsdn"]).cuda())
    # poison what the kernels must overwrite
    for t in (layer.gu, layer.y, layer.out) + ((layer.p,) if layer.fused_back else ()):
        t.fill_(0x7FC0)
    x, lg = dev_bf16_bits(case["X"]), dev_bf16_bits(case["logits"])
    layer.forward(x, lg)
    layer.forward(x, lg)            # twice: the arrival counter must have been left at zero
    torch.cuda.synchronize()
    return layer


def check_layer(layer, case, taps=True):
    T, E, k, H, I = case["T"], case["E"], case["topk"], case["H"], case["I"]
    ids, w = ref.route(case["logits"], k)
    lay = ref.sort_layout(ids, E, layer.tb)
    b = {n: t.cpu().numpy() for n, t in layer.buf.items()}
    np.testing.assert_array_equal(b["topk_ids"].reshape(T, k), ids)
    np.testing.assert_array_equal(b["topk_w"].reshape(T, k).view(np.uint32), w.view(np.uint32))
    assert int(b["meta"][0]) == lay["tiles"] and int(b["meta"][1]) == lay["rows"] and int(b["meta"][3]) == T * k
    assert int(b["arrive"][0]) == 0
    np.testing.assert_array_equal(b["expert_cnt"], lay["expert_cnt"])
    np.testing.assert_array_equal(b["route_pos"].reshape(T, k), lay["route_pos"])
    np.testing.assert_array_equal(b["row_tok"][:lay["rows"]], lay["row_tok"])
    nt = lay["tiles"]
    np.testing.assert_array_equal(b["tile_expert"][:nt], lay["tile_expert"])
    np.testing.assert_array_equal(b["tile_row0"][:nt], lay["tile_row0"])
    np.testing.assert_array_equal(b["tile_rows"][:nt], lay["tile_rows"])
    r = ref.moe_layer(case["X"], w, lay, case["Wgu"], case["wsgu"], case["Wdn"], case["wsdn"], I, threads=8, taps=taps)
    live = lay["row_tok"] >= 0
    rows = lay["rows"]
    if taps and layer.fused_back:   # the activation sits in gate+up's epilogue: p is the tap
        np.testing.assert_array_equal(host_u16(layer.p)[:rows][live], ref.silu_mul_quant(r["gu"][live])[2])
    elif taps:
        np.testing.assert_array_equal(host_u16(layer.gu)[:rows][live], r["gu"][live])
        q2 = iu8.unpack_a(layer.q2.cpu().numpy(), rows, I)
        np.testing.assert_array_equal(q2[live], r["q2"][live])
        np.testing.assert_array_equal(layer.s2.cpu().numpy()[:rows][live].view(np.uint32), r["s2"][live].view(np.uint32))
    np.testing.assert_array_equal(host_u16(layer.y)[:rows][live], r["Y"][live])
    np.testing.assert_array_equal(host_u16(layer.out), r["out"])


@pytest.mark.parametrize("T,tb", [(1, None), (16, None), (16, 8), (100, None), (100, 1), (300, None), (300, 1), (40, 16), (300, 16), (700, 16)])
def test_moe_layer_small_experts(ctx, T, tb):
    say(f"moe layer T={T} tile_blocks={tb} E=128 top-8 H=512 I=256")
    case = synth.moe_case(T=T, E=128, topk=8, H=512, I=256, seed=T, experts=8)
    layer = run_layer(ctx, case, tile_blocks=tb)
    check_layer(layer, case)


@pytest.mark.parametrize("I", [256, 1536, 2048, 2560, 4096])
def test_silu_mul_requant_table_form(ctx, I):
    """SiLU * up + requant over many expert-major rows, the form that reads the bf16 silu from the table in
    LDS: rows of 256 to 4,096 elements (one to four 16-element groups a lane), pad rows skipped, against
    the oracle's row routine (codes, scales)."""
    T, E, k = 520, 128, 8
    say(f"silu * up requant, table form: I={I}")
    rng = np.random.default_rng(I)
    layer = MoeLayerIU8(ctx, T, E, k, 128, I, tile_blocks=8)
    assert layer.rows_cap >= 4096
    lg = dev_bf16_bits(synth.f32_to_bf16_bits(rng.standard_normal(size=(T, E), dtype=np.float32)))
    ctx.moe_route(lg.data_ptr(), T, E, k, layer.tb, layer.tables)
    gu = synth.f32_to_bf16_bits((rng.standard_normal(size=(layer.rows_cap, 2 * I)) * rng.choice([0.1, 1.0, 6.0], size=(layer.rows_cap, 1))).astype(np.float32))
    layer.gu.copy_(dev_bf16_bits(gu))
    layer.q2.fill_(0x55)
    layer.s2.fill_(-1.0)
    ctx.moe_silu_mul_quant(layer.gu.data_ptr(), layer.q2.data_ptr(), layer.s2.data_ptr(), I, layer.rows_cap, layer.tables)
    torch.cuda.synchronize()
    rows = int(layer.buf["meta"][1].item())
    live = layer.buf["row_tok"][:rows].cpu().numpy() >= 0
    assert live.sum() == T * k and (~live).sum() > 0
    want_q, want_s, _ = ref.silu_mul_quant(gu[:rows][live])
    np.testing.assert_array_equal(iu8.unpack_a(layer.q2.cpu().numpy(), rows, I)[live], want_q)
    s2 = layer.s2.cpu().numpy()
    np.testing.assert_array_equal(s2[:rows][live].view(np.uint32), want_s.view(np.uint32))
    assert (s2[:rows][~live] == -1.0).all() and (s2[rows:] == -1.0).all()      # pad rows and the rows past the live ones are left alone


@pytest.mark.parametrize("T,H,I", [(1, 512, 256), (16, 4096, 1536), (37, 512, 1536), (100, 640, 384), (112, 1024, 256), (300, 512, 256)])
def test_moe_back_half_in_two_launches(ctx, T, H, I):
    """Few tokens (16-row tiles): gate+up with SiLU * up in its epilogue, then down with p's per-token
    quantisation in front of its K loop. Same bytes as the three launches (grouped gate+up, SiLU * up
    requant, grouped down) and as the oracle; gate+up with one and with two tiles of p a wave (by routes
    an expert), tiles of 1 to 16 rows, the widest intermediate the form holds. Other tile sizes are refused."""
    say(f"moe back half in two launches T={T} H={H} I={I}")
    case = synth.moe_case(T=T, E=128, topk=8, H=H, I=I, seed=T + I, experts=8)
    fused = run_layer(ctx, case, tile_blocks=1, fused_back=True)
    three = run_layer(ctx, case, tile_blocks=1, fused_back=False)
    assert fused.fused_back and not three.fused_back and iu8.moe_back_holds(1, I)
    rows = int(fused.buf["meta"][1].item())
    live = fused.buf["row_tok"][:rows] >= 0
    assert torch.equal(fused.y[:rows][live], three.y[:rows][live])
    assert torch.equal(fused.out, three.out)
    check_layer(fused, case)
    assert not iu8.moe_back_holds(8, I) and not iu8.moe_back_holds(1, 1664) and not iu8.moe_back_holds(1, 200)
    with pytest.raises(iu8.IU8Error) as e:
        ctx.moe_gate_up_act(fused.q1.data_ptr(), fused.s1.data_ptr(), fused.xptr_gu.data_ptr(), fused.p.data_ptr(), I, H,
                            T, 128, 8, 8, fused.tables)
    assert e.value.code == iu8.E_RULE
    with pytest.raises(iu8.IU8Error) as e:
        ctx.moe_down_rows(fused.p.data_ptr(), fused.xptr_dn.data_ptr(), fused.y.data_ptr(), H, 1664, T, 128, 8, 1, fused.tables)
    assert e.value.code == iu8.E_RULE


@pytest.mark.parametrize("T,tb", [(1, None), (16, None), (37, None), (100, 8), (300, None), (300, 1), (520, 16)])
def test_moe_layer_with_a_shared_expert(ctx, T, tb):
    """The layer with a shared expert (crates/saber-kernels/hip/moe_route.hip:244-272, 299-321): the router
    appends every token as a row of expert index 128 behind the routed rows (meta[2] = its first row, tiles
    of `tile_blocks` blocks, pad rows marked), both grouped GEMMs and the SiLU*up requant run those rows
    on the shared expert's weights, and the combine adds sigmoid(sgate[t]) times the token's shared row.
    Expected: the oracle's routed layer, the shared expert as a dense MLP of the oracle's linears over all
    tokens, and the oracle's combine with the gate term."""
    E, k, H, I = 128, 8, 512, 256
    say(f"moe layer with a shared expert T={T} tile_blocks={tb}")
    case = synth.moe_case(T=T, E=E, topk=k, H=H, I=I, seed=100 + T, experts=6)
    rng = np.random.default_rng(T)
    Wgu_s, wsgu_s = synth.weights(rng, 2 * I, H, False)
    Wdn_s, wsdn_s = synth.weights(rng, H, I, False)
    sgate = synth.f32_to_bf16_bits((2.5 * rng.standard_normal(T)).astype(np.float32))
    layer = MoeLayerIU8(ctx, T, E, k, H, I, tile_blocks=tb, shared=True)
    wgu = torch.from_numpy(np.stack([iu8.repack_w4(case["Wgu"][e]) for e in range(E)] + [iu8.repack_w4(Wgu_s)])).cuda()
    wdn = torch.from_numpy(np.stack([iu8.repack_w4(case["Wdn"][e]) for e in range(E)] + [iu8.repack_w4(Wdn_s)])).cuda()
    layer.set_weights(wgu, torch.from_numpy(np.concatenate([case["wsgu"], wsgu_s[None]])).cuda(), wdn,
                      torch.from_numpy(np.concatenate([case["wsdn"], wsdn_s[None]])).cuda())
    layer.sgate.copy_(dev_bf16_bits(sgate))
    for t in (layer.gu, layer.y, layer.out):
        t.fill_(0x7FC0)
    x, lg = dev_bf16_bits(case["X"]), dev_bf16_bits(case["logits"])
    layer.forward(x, lg)
    layer.forward(x, lg)
    torch.cuda.synchronize()
    # ---- the tables: the routed part as without a shared expert, then the shared rows and tiles
    ids, w = ref.route(case["logits"], k)
    lay = ref.sort_layout(ids, E, layer.tb)
    b = {n: t.cpu().numpy() for n, t in layer.buf.items()}
    rows, nt, G = lay["rows"], lay["tiles"], layer.tb
    sh_blocks = (T + 15) // 16
    sh_tiles = -(-sh_blocks // G)
    assert b["meta"][:6].tolist() == [nt + sh_tiles, rows + sh_blocks * 16, rows, T * k, int((lay["expert_cnt"] > 0).sum()), rows]
    assert layer.rows_cap >= rows + sh_blocks * 16 and layer.tiles_cap >= nt + sh_tiles and int(b["arrive"][0]) == 0
    np.testing.assert_array_equal(b["row_tok"][:rows], lay["row_tok"])
    np.testing.assert_array_equal(b["row_tok"][rows:rows + sh_blocks * 16], np.where(np.arange(sh_blocks * 16) < T, np.arange(sh_blocks * 16), -1))
    np.testing.assert_array_equal(b["tile_expert"][:nt + sh_tiles], np.concatenate([lay["tile_expert"], np.full(sh_tiles, E)]))
    np.testing.assert_array_equal(b["tile_row0"][nt:nt + sh_tiles], rows + 16 * G * np.arange(sh_tiles))
    np.testing.assert_array_equal(b["tile_rows"][nt:nt + sh_tiles], np.minimum(16 * G, T - 16 * G * np.arange(sh_tiles)))
    np.testing.assert_array_equal(b["route_pos"].reshape(T, k), lay["route_pos"])
    # ---- the arithmetic
    r = ref.moe_layer(case["X"], w, lay, case["Wgu"], case["wsgu"], case["Wdn"], case["wsdn"], I, threads=8)
    live = lay["row_tok"] >= 0
    np.testing.assert_array_equal(host_u16(layer.y)[:rows][live], r["Y"][live])
    gu_s = ref.linear(case["X"], Wgu_s, wsgu_s, False, threads=8)["C"]
    _, _, p_s = ref.silu_mul_quant(gu_s)
    y_s = ref.linear(p_s, Wdn_s, wsdn_s, False, threads=8)["C"]
    if layer.fused_back:
        np.testing.assert_array_equal(host_u16(layer.p)[rows:rows + T], p_s)
    else:
        np.testing.assert_array_equal(host_u16(layer.gu)[rows:rows + T], gu_s)
    np.testing.assert_array_equal(host_u16(layer.y)[rows:rows + T], y_s)
    Y = np.concatenate([r["Y"], y_s])
    want = ref.combine_shared(Y, w, lay["route_pos"], sgate, rows, H)
    np.testing.assert_array_equal(host_u16(layer.out), want)
    assert (want != r["out"]).any()                      # the gate term is in the output


def test_moe_layer_streamed_rows_cell(ctx):
    """K past the short-K form and more routes than the LDS staging is sized for: the streaming cell
    that reads the rows beside the weights (gate+up), the short-K cell (down)."""
    say("moe layer T=100 tile_blocks=1 E=128 top-8 H=2560 I=256")
    case = synth.moe_case(T=100, E=128, topk=8, H=2560, I=256, seed=21, experts=4)
    layer = run_layer(ctx, case)
    assert layer.tb == 1
    check_layer(layer, case)


@pytest.mark.parametrize("T,I,hot,boost", [(512, 2560, 0, 0.0), (2048, 4352, 8, 6.0), (1024, 256, 4, 1.5)])
def test_moe_layer_two_cell_walk(ctx, T, I, hot, boost):
    """The 128-row tile cell runs tiles of up to 64 rows on a second, smaller cell between two parts of
    its heavy items, and resolves a workgroup's items eight heavy and eight light rounds at a time: ten
    rounds of light items (512 tokens over 128 experts, 20 column blocks), seventeen of heavy ones
    (2,048 tokens on 8 experts, 34 column blocks), and a skewed routing with both kinds in one launch."""
    say(f"moe layer T={T} tile_blocks=8 E=128 top-8 H=256 I={I} hot experts={hot} (+{boost})")
    case = synth.moe_case(T=T, E=128, topk=8, H=256, I=I, seed=T + 3, experts=2)
    if hot:
        lg = synth.bf16_bits_to_f32(case["logits"])
        if boost > 3:
            lg = lg * np.float32(0.25) - np.float32(3.0)
        lg[:, :hot] += np.float32(boost)
        case["logits"] = synth.f32_to_bf16_bits(lg)
    layer = run_layer(ctx, case, tile_blocks=8)
    tr = layer.buf["tile_rows"][:int(layer.buf["meta"][0].item())].cpu().numpy()
    light, heavy, gx = int((tr <= 64).sum()), int((tr > 64).sum()), (2 * I + 255) // 256
    if hot == 0:
        assert light * gx > 8 * 256
    elif boost > 3:
        assert heavy * gx > 8 * 256
    else:
        assert light >= 32 and heavy >= 8
    check_layer(layer, case)


@pytest.mark.parametrize("T,H", [(1, 128), (16, 4096), (37, 640), (19, 8192), (112, 16384), (300, 512), (2101, 1024)])
def test_route_and_quant_in_one_launch(ctx, T, H):
    """The merged launch writes what the router and the int8 producer write on their own: tables,
    codes (A fragment order for the streaming cell's 16-row tiles, row-major for the tile cells) and
    scales, byte for byte; twice in a row (the arrival counter). Rows of 256, 512 and 1,024 threads,
    a last quantising workgroup with fewer rows than it holds."""
    say(f"moe route + quant in one launch: T={T} H={H}")
    E, k = 128, 8
    rng = np.random.default_rng(T * 31 + H)
    X = synth.activations(rng, T, H)
    if T > 2:
        X[1] = 0                                            # an all-zero row: scale 1e-30, codes 0
    logits = synth.f32_to_bf16_bits(rng.standard_normal(size=(T, E), dtype=np.float32))
    x, lg = dev_bf16_bits(X), dev_bf16_bits(logits)
    a, b = MoeLayerIU8(ctx, T, E, k, H, 256), MoeLayerIU8(ctx, T, E, k, H, 256)
    qa = torch.full((iu8.a_bytes(T, H),), 0x55, dtype=torch.uint8, device="cuda")
    sa = torch.zeros(T, dtype=torch.float32, device="cuda")
    for _ in range(2):
        ctx.moe_route_quant(lg.data_ptr(), x.data_ptr(), qa.data_ptr(), sa.data_ptr(), T, E, k, H, a.tb, a.tables)
    ctx.moe_route(lg.data_ptr(), T, E, k, b.tb, b.tables)
    torch.cuda.synchronize()
    want_q, want_s = ref.quant_bf16(X)
    np.testing.assert_array_equal(sa.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    if a.tb == 1:
        np.testing.assert_array_equal(iu8.unpack_a(qa.cpu().numpy(), T, H), want_q)
    else:
        np.testing.assert_array_equal(qa.cpu().numpy()[:T * H].view(np.int8).reshape(T, H), want_q)
    nt, rows = int(a.buf["meta"][0].item()), int(a.buf["meta"][1].item())
    for name in ("topk_ids", "topk_w", "route_pos", "expert_cnt", "meta", "arrive"):
        assert torch.equal(a.buf[name], b.buf[name]), name
    for name in ("tile_expert", "tile_row0", "tile_rows"):
        assert torch.equal(a.buf[name][:nt], b.buf[name][:nt]), name
    for name in ("row_tok", "row_route"):
        assert torch.equal(a.buf[name][:rows], b.buf[name][:rows]), name
    ids, _ = ref.route(logits, k)
    np.testing.assert_array_equal(a.buf["topk_ids"].cpu().numpy().reshape(T, k), ids)
    with pytest.raises(iu8.IU8Error) as e:
        ctx.moe_route_quant(lg.data_ptr(), x.data_ptr(), qa.data_ptr(), sa.data_ptr(), T, E, k, 16512, a.tb, a.tables)
    assert e.value.code == iu8.E_RULE


@pytest.mark.parametrize("T,tb", [(129, 8), (700, 8), (3000, 16)])
def test_one_launch_router_under_the_reference_name(ctx, T, tb):
    """Above 128 tokens the C ABI routes in two launches; the one-launch kernel under the reference's name
    (its last workgroup to arrive lays out the tables alone) stays in the plugin for a host that launches
    that name: same tables, arrival counter left at zero, twice in a row."""
    say(f"one-launch router by name: T={T} tile_blocks={tb}")
    E, k = 128, 8
    rng = np.random.default_rng(T)
    lg = dev_bf16_bits(synth.f32_to_bf16_bits(rng.standard_normal(size=(T, E), dtype=np.float32)))
    two, one = MoeLayerIU8(ctx, T, E, k, 128, 128, tile_blocks=tb), MoeLayerIU8(ctx, T, E, k, 128, 128, tile_blocks=tb)
    ctx.moe_route(lg.data_ptr(), T, E, k, tb, two.tables)
    d = iu8.describe_raw("moe_iu8_route_topk8_sort_e128", ((T + 127) // 128, 1, 1), 1024, plugin="moe_iu8",
                         t=T, e_lo=0, e_loc=E, tile_blocks=tb, with_shared=0)
    bufs = dict(logits=lg.data_ptr(), **{n_: one.buf[n_].data_ptr() for n_ in (
        "topk_ids", "topk_w", "route_pos", "row_tok", "row_route", "tile_expert", "tile_row0", "tile_rows", "expert_cnt",
        "meta", "blk_cnt", "rank", "arrive")})
    for _ in range(2):
        ctx.launch(d, bufs)
    torch.cuda.synchronize()
    nt, rows = int(two.buf["meta"][0].item()), int(two.buf["meta"][1].item())
    assert int(one.buf["arrive"][0].item()) == 0 and int(two.buf["arrive"][0].item()) == 0
    for name in ("topk_ids", "topk_w", "route_pos", "expert_cnt", "meta"):
        assert torch.equal(one.buf[name], two.buf[name]), name
    for name in ("tile_expert", "tile_row0", "tile_rows"):
        assert torch.equal(one.buf[name][:nt], two.buf[name][:nt]), name
    for name in ("row_tok", "row_route"):
        assert torch.equal(one.buf[name][:rows], two.buf[name][:rows]), name
    ids, _ = ref.route(synth.f32_to_bf16_bits(np.random.default_rng(T).standard_normal(size=(T, E), dtype=np.float32)), k)
    np.testing.assert_array_equal(two.buf["topk_ids"].cpu().numpy().reshape(T, k), ids)


def test_grouped_tile_kernels_on_a_tiny_grid(ctx):
    """The tile kernels are persistent: on 3 workgroups instead of one a CU every workgroup walks more
    items than its item table holds (the 256-row kernel then resolves items as it goes, the 128-row
    one runs several passes over its table) and writes the same bytes."""
    T, E, k, H, I = 300, 128, 8, 512, 256
    case = synth.moe_case(T=T, E=E, topk=k, H=H, I=I, seed=9, experts=4)
    for tb, kern in ((16, "moe_iu8_grouped_w4_pf16_g2"), (8, "moe_iu8_grouped_w4_pf_g2")):
        say(f"grouped gate+up on 3 workgroups: {kern}")
        layer = run_layer(ctx, case, tile_blocks=tb)
        want = layer.gu.clone()
        nt, rows = int(layer.buf["meta"][0].item()), int(layer.buf["meta"][1].item())
        assert nt * ((2 * I + 255) // 256) > 3 * 64
        d = iu8.describe_raw(kern, (3, 1, 1), 512, plugin="moe_iu8", n=2 * I, k=H, pmax=0)
        for name in ("p", "cnt"):
            d.arg(name).kind = iu8.ARG_NULL_BUFFER
        layer.gu.fill_(0x7FC0)
        bufs = dict(a=layer.q1.data_ptr(), xptr=layer.xptr_gu.data_ptr(), c=layer.gu.data_ptr(),
                    **{n_: layer.buf[n_].data_ptr() for n_ in ("tile_expert", "tile_row0", "tile_rows", "row_tok", "meta")})
        bufs["as"] = layer.s1.data_ptr()
        ctx.launch(d, bufs)
        torch.cuda.synchronize()
        live = layer.buf["row_tok"][:rows] >= 0
        assert torch.equal(layer.gu[:rows][live], want[:rows][live])


def test_moe_router_ties_and_skew(ctx):
    say("moe router: ties and one hot expert")
    case = synth.moe_case(T=40, E=128, topk=8, H=512, I=256, seed=5, experts=4)
    lg = np.zeros((40, 128), np.float32)
    lg[:, 7] = 3.0                  # every token routes to expert 7 first, then ties: lower ids win
    lg[5:, 100] = 3.0
    case["logits"] = synth.f32_to_bf16_bits(lg)
    layer = run_layer(ctx, case)
    check_layer(layer, case)


@pytest.mark.parametrize("T", [129, 1000, 4096, 5001])
def test_moe_router_many_workgroups(ctx, T):
    """The router alone at token counts that take several workgroups (128 tokens each): ids, weights
    and the whole sort / tile table against the oracle, twice on the same tables."""
    say(f"moe router T={T}")
    E, k = 128, 8
    rng = np.random.default_rng(T)
    logits = synth.f32_to_bf16_bits(rng.standard_normal((T, E)).astype(np.float32))
    layer = MoeLayerIU8(ctx, T, E, k, 512, 256)
    lg = dev_bf16_bits(logits)
    for _ in range(2):
        ctx.moe_route(lg.data_ptr(), T, E, k, layer.tb, layer.tables)
    torch.cuda.synchronize()
    ids, w = ref.route(logits, k)
    lay = ref.sort_layout(ids, E, layer.tb)
    b = {n: t.cpu().numpy() for n, t in layer.buf.items()}
    np.testing.assert_array_equal(b["topk_ids"].reshape(T, k), ids)
    np.testing.assert_array_equal(b["topk_w"].reshape(T, k).view(np.uint32), w.view(np.uint32))
    assert int(b["meta"][0]) == lay["tiles"] and int(b["meta"][1]) == lay["rows"] and int(b["meta"][3]) == T * k
    assert int(b["arrive"][0]) == 0
    np.testing.assert_array_equal(b["expert_cnt"], lay["expert_cnt"])
    np.testing.assert_array_equal(b["route_pos"].reshape(T, k), lay["route_pos"])
    np.testing.assert_array_equal(b["row_tok"][:lay["rows"]], lay["row_tok"])
    nt = lay["tiles"]
    np.testing.assert_array_equal(b["tile_expert"][:nt], lay["tile_expert"])
    np.testing.assert_array_equal(b["tile_row0"][:nt], lay["tile_row0"])
    np.testing.assert_array_equal(b["tile_rows"][:nt], lay["tile_rows"])


def test_moe_layer_config4_decode_shape(ctx):
    say("moe layer config 4: T=16 E=128 top-8 H=4096 I=1536")
    case = synth.moe_case(T=16, E=128, topk=8, H=4096, I=1536, seed=0, experts=6)
    layer = run_layer(ctx, case)
    check_layer(layer, case, taps=True)


def test_quant_rowmajor_matches_the_oracle_codes(ctx):
    say("row-major per-token quantisation")
    rng = np.random.default_rng(3)
    for M, K in ((5, 512), (33, 4096), (7, 5120)):
        X = synth.activations(rng, M, K)
        q = torch.full((M * K,), 0x55, dtype=torch.uint8, device="cuda")
        s = torch.zeros(M, dtype=torch.float32, device="cuda")
        ctx.quant_rowmajor(dev_bf16_bits(X).data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
        torch.cuda.synchronize()
        qh, sh = ref.quant_bf16(X)
        np.testing.assert_array_equal(q.cpu().numpy().view(np.int8).reshape(M, K), qh)
        np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), sh.view(np.uint32))


def test_moe_layer_config4_prefill_shape(ctx):
    """T=4096 at the full expert shape: the tables against the oracle, every route of a sample of
    tokens (those that land in an expert's nearly empty last tile among them) through both GEMMs
    and the combine against the oracle, and the whole output against the same layer run on 128-row
    tiles over rows gathered by the quantiser -- other cells, other operand orders, same bytes."""
    T, E, k, H, I = 4096, 128, 8, 4096, 1536
    say(f"moe layer config 4: T={T} E=128 top-8 H=4096 I=1536")
    case = synth.moe_case(T=T, E=E, topk=k, H=H, I=I, seed=1, experts=3)
    ne = 3
    fgu = torch.from_numpy(np.stack([iu8.repack_w4(case["Wgu"][e]) for e in range(ne)])).cuda()
    fdn = torch.from_numpy(np.stack([iu8.repack_w4(case["Wdn"][e]) for e in range(ne)])).cuda()
    idx = torch.arange(E, device="cuda") % ne
    wgu, wdn = fgu[idx].contiguous(), fdn[idx].contiguous()
    wsgu, wsdn = torch.from_numpy(case["wsgu"]).cuda(), torch.from_numpy(case["wsdn"]).cuda()
    x, lg = dev_bf16_bits(case["X"]), dev_bf16_bits(case["logits"])
    layer = MoeLayerIU8(ctx, T, E, k, H, I)
    assert layer.tb == 16 and layer.gather == 2
    layer.set_weights(wgu, wsgu, wdn, wsdn)
    layer.gu.fill_(0x7FC0)
    layer.y.fill_(0x7FC0)
    layer.forward(x, lg)
    layer.forward(x, lg)
    torch.cuda.synchronize()
    ids, w = ref.route(case["logits"], k)
    lay = ref.sort_layout(ids, E, layer.tb)
    b = {n: t.cpu().numpy() for n, t in layer.buf.items()}
    np.testing.assert_array_equal(b["topk_ids"].reshape(T, k), ids)
    np.testing.assert_array_equal(b["route_pos"].reshape(T, k), lay["route_pos"])
    np.testing.assert_array_equal(b["row_tok"][:lay["rows"]], lay["row_tok"])
    nt = lay["tiles"]
    assert int(b["meta"][0]) == nt
    np.testing.assert_array_equal(b["tile_rows"][:nt], lay["tile_rows"])
    # sample: the token of the last route of every expert whose last tile holds at most 32 rows, and a few others
    cnt = lay["expert_cnt"]
    off = np.concatenate([[0], np.cumsum((cnt + 15) // 16 * 16)])
    tail = [int(lay["row_tok"][off[e] + cnt[e] - 1]) for e in range(E) if 0 < cnt[e] % 256 <= 32][:10]
    assert tail, "the draw has no expert with a nearly empty last tile"
    toks = sorted(set(tail + [0, 1, 2047, 4095] + list(np.random.default_rng(0).integers(0, T, 6))))
    gu_d, y_d, out_d = host_u16(layer.gu), host_u16(layer.y), host_u16(layer.out)
    for t in toks:
        rows = []
        for j in range(k):
            e, p = int(ids[t, j]), int(lay["route_pos"][t, j])
            r1 = ref.linear(case["X"][t:t + 1], case["Wgu"][e], case["wsgu"][e], False)
            np.testing.assert_array_equal(gu_d[p], r1["C"][0], err_msg=f"gate+up token {t} route {j}")
            q2, s2, _ = ref.silu_mul_quant(r1["C"])
            S, _ = ref.gemm_fast(q2, case["Wdn"][e], False)
            yrow = ref.epilogue(S, s2, case["wsdn"][e], False)
            np.testing.assert_array_equal(y_d[p], yrow[0], err_msg=f"down token {t} route {j}")
            rows.append(yrow[0])
        want = ref.combine(np.stack(rows), w[t:t + 1], np.arange(k, dtype=np.int32)[None], H)
        np.testing.assert_array_equal(out_d[t], want[0], err_msg=f"combine token {t}")
    # the same layer through the 128-row cells on rows the quantiser gathered
    tb = 8
    other = MoeLayerIU8(ctx, T, E, k, H, I, tile_blocks=tb)
    other.set_weights(wgu, wsgu, wdn, wsdn)
    q1 = torch.zeros(iu8.a_bytes(other.rows_cap, H), dtype=torch.uint8, device="cuda")
    s1 = torch.zeros(other.rows_cap, dtype=torch.float32, device="cuda")
    ctx.moe_route(lg.data_ptr(), T, E, k, tb, other.tables)
    ctx.moe_quant_rows(x.data_ptr(), q1.data_ptr(), s1.data_ptr(), H, other.rows_cap, other.tables)
    ctx.moe_grouped(q1.data_ptr(), s1.data_ptr(), other.xptr_gu.data_ptr(), other.gu.data_ptr(), 2 * I, H, 0, T, E, k, tb, other.tables)
    ctx.moe_silu_mul_quant(other.gu.data_ptr(), other.q2.data_ptr(), other.s2.data_ptr(), I, other.rows_cap, other.tables)
    ctx.moe_grouped(other.q2.data_ptr(), other.s2.data_ptr(), other.xptr_dn.data_ptr(), other.y.data_ptr(), H, I, 0, T, E, k, tb, other.tables)
    ctx.moe_combine(other.y.data_ptr(), other.tables, other.out.data_ptr(), T, k, H)
    torch.cuda.synchronize()
    live = lay["row_tok"] >= 0
    np.testing.assert_array_equal(host_u16(other.y)[:lay["rows"]][live], y_d[:lay["rows"]][live])
    np.testing.assert_array_equal(host_u16(other.out), out_d)
