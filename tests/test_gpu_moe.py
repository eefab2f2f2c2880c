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


def run_layer(ctx, case, tile_blocks=None):
    T, E, k, H, I = case["T"], case["E"], case["topk"], case["H"], case["I"]
    layer = MoeLayerIU8(ctx, T, E, k, H, I, tile_blocks=tile_blocks)
    wgu = torch.from_numpy(np.stack([iu8.repack_w4(case["Wgu"][e]) for e in range(E)])).cuda()
    wdn = torch.from_numpy(np.stack([iu8.repack_w4(case["Wdn"][e]) for e in range(E)])).cuda()
    layer.set_weights(wgu, torch.from_numpy(case["wsgu"]).cuda(), wdn, torch.from_numpy(case["wsdn"]).cuda())
    # poison what the kernels must overwrite
    layer.gu.fill_(0x7FC0)
    layer.y.fill_(0x7FC0)
    layer.out.fill_(0x7FC0)
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
    if taps:
        np.testing.assert_array_equal(host_u16(layer.gu)[:rows][live], r["gu"][live])
        q2 = iu8.unpack_a(layer.q2.cpu().numpy(), rows, I)
        np.testing.assert_array_equal(q2[live], r["q2"][live])
        np.testing.assert_array_equal(layer.s2.cpu().numpy()[:rows][live].view(np.uint32), r["s2"][live].view(np.uint32))
    np.testing.assert_array_equal(host_u16(layer.y)[:rows][live], r["Y"][live])
    np.testing.assert_array_equal(host_u16(layer.out), r["out"])


@pytest.mark.parametrize("T,tb", [(1, None), (16, None), (16, 8), (100, None), (300, None)])
def test_moe_layer_small_experts(ctx, T, tb):
    say(f"moe layer T={T} tile_blocks={tb} E=128 top-8 H=512 I=256")
    case = synth.moe_case(T=T, E=128, topk=8, H=512, I=256, seed=T, experts=8)
    layer = run_layer(ctx, case, tile_blocks=tb)
    check_layer(layer, case)


def test_moe_router_ties_and_skew(ctx):
    say("moe router: ties and one hot expert")
    case = synth.moe_case(T=40, E=128, topk=8, H=512, I=256, seed=5, experts=4)
    lg = np.zeros((40, 128), np.float32)
    lg[:, 7] = 3.0                  # every token routes to expert 7 first, then ties: lower ids win
    lg[5:, 100] = 3.0
    case["logits"] = synth.f32_to_bf16_bits(lg)
    layer = run_layer(ctx, case)
    check_layer(layer, case)


def test_moe_layer_config4_decode_shape(ctx):
    say("moe layer config 4: T=16 E=128 top-8 H=4096 I=1536")
    case = synth.moe_case(T=16, E=128, topk=8, H=4096, I=1536, seed=0, experts=6)
    layer = run_layer(ctx, case)
    check_layer(layer, case, taps=True)
