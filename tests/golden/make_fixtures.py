"""Writes the small golden vectors of tests/golden/ (run from the repo root:
`python tests/golden/make_fixtures.py`).

The reference holds no input/output vector for the iu8 arithmetic (its GPU gate replays captures
that are not in its tree), so these vectors are produced HERE by an independent brute-force
restatement of the written contract in numpy -- float32 IEEE divide / np.rint for the codes, an
int64 matrix product for the accumulators, float64 products rounded once to float32 for the two
epilogue multiplies (exact: a product of two float32 fits float64), the bit trick for bf16 -- and
NOT by the C oracle. The oracle and the HIP path are both checked against them.

kernarg_gfx1201.json holds data read off the reference's committed manifests
(prebuilt/gfx1201/macaq_iu8.manifest.toml and those of the pair and the int8 producers): the explicit
kernarg offsets/sizes the host packs; kernarg_gfx1201_moe.json the same for the routed layer's
kernels (prebuilt/gfx1201/moe_route.manifest.toml, moe_grouped.manifest.toml), each with the gfx950
kernels that keep its list.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from saber_engine_amd import synth  # noqa: E402  (seeded operand generator only)


def bf16_rne_np(x):
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def brute_linear(Xbits, W, ws, w8):
    x = synth.bf16_bits_to_f32(Xbits)
    amax = np.max(np.abs(x), axis=1)
    sc = np.maximum((amax / np.float32(127.0)).astype(np.float32), np.float32(1e-30))
    y = (x / sc[:, None]).astype(np.float32)
    q = np.rint(np.clip(y, -127.0, 127.0)).astype(np.int8)
    w = W.astype(np.int64) if w8 else synth.unpack_w4(W).astype(np.int64)
    S = q.astype(np.int64) @ w.T
    assert np.abs(S).max() < 2 ** 27
    acc = S if w8 else S * 16
    wsu = ws if w8 else (ws.astype(np.float64) * 0.0625).astype(np.float32)
    t = (acc.astype(np.float32).astype(np.float64) * sc[:, None].astype(np.float64)).astype(np.float32)
    yv = (t.astype(np.float64) * wsu[None, :].astype(np.float64)).astype(np.float32)
    return q, sc, S.astype(np.int32), bf16_rne_np(yv)


def main():
    cases = [(1, 64, 256, False, 0), (16, 48, 128, False, 1), (5, 32, 256, True, 2), (64, 64, 256, False, 3),
             (33, 16, 128, True, 4)]
    out = {}
    for i, (M, N, K, w8, seed) in enumerate(cases):
        c = synth.dense_case(M, N, K, w8=w8, seed=seed)
        if i == 1:
            c["X"][3, :] = 0  # an all-zero token row: scale 1e-30, codes 0
        q, sc, S, C = brute_linear(c["X"], c["W"], c["ws"], w8)
        for k, v in dict(X=c["X"], W=c["W"], ws=c["ws"], q=q, a_scale=sc, S=S, C=C).items():
            out[f"c{i}_{k}"] = v
        out[f"c{i}_meta"] = np.array([M, N, K, int(w8)], np.int32)
    np.savez_compressed(os.path.join(HERE, "dense_small.npz"), **out)

    write_kernarg_table()


# The reference's committed manifests hold the explicit kernarg offsets/sizes its host packs; the
# symbols this build also ships are kept (every macaq_iu8 kernel, the decode pair, the int8 twins).
KERNARG_SOURCES = {
    "macaq_iu8": None,
    "macaq_iu8f": ("macaq_iu8f_pair_w4_tm", "macaq_iu8f_pairb_w4_tm"),
    "mxfp4_hadi8": ("add_rms_quant_hadi8_", "silu_mul_quant_hadi8_", "gdn_norm_quant_hadi8_"),
    "attn_glue_hadi8": ("attn_gate_quant_hadi8_",),
}


# The routed layer: the reference's kernels carry other names (its router is 512 experts / top-10, its
# grouped GEMM MXFP4 x e4m3) but the argument lists are the launch contract this build keeps; each
# reference kernel is listed with the gfx950 kernels that take the same list.
MOE_KERNARG_SOURCES = {
    "moe_route": {
        "moe_route_topk10_sort_e512": ["moe_iu8_route_topk8_sort_e128"],
        "moe_combine_bf16": ["moe_iu8_combine_bf16"],
    },
    "moe_grouped": {
        "moe_grouped_w4a8_bk128_ks1_tm1_g0": ["moe_iu8_grouped_w4_dec_g0", "moe_iu8_grouped_w4_deca_g0", "moe_iu8_grouped_w4_deck_g0"],
        "moe_grouped_w4a8_bk128_ks1_tm1_g1": ["moe_iu8_grouped_w4_dec_g1", "moe_iu8_grouped_w4_deca_g1", "moe_iu8_grouped_w4_deck_g1"],
        "moe_grouped_w4a8_pf_tm8_g0": ["moe_iu8_grouped_w4_pf_g0"],
        "moe_grouped_w4a8_pf_tm8_g1": ["moe_iu8_grouped_w4_pf_g1", "moe_iu8_grouped_w4_pf_g2"],
        "moe_grouped_w4a8_pf_tm16_g0": ["moe_iu8_grouped_w4_pf16_g0"],
        "moe_grouped_w4a8_pf_tm16_g1": ["moe_iu8_grouped_w4_pf16_g1", "moe_iu8_grouped_w4_pf16_g2"],
        "moe_silu_mul_quant_t256": ["macaq_i8_silu_mul_quant_t256", "macaq_i8_silu_mul_quant_t256_g1", "macaq_i8_silu_mul_quant_w64"],
    },
}


def _manifest_args(ref_dir, plugin):
    import re

    text = open(os.path.join(ref_dir, plugin + ".manifest.toml")).read()
    out = {}
    for blk in text.split("[[kernel]]")[1:]:
        name = re.search(r'name = "(\w+)"', blk).group(1)
        args = re.findall(r'offset = (\d+)\nsize = (\d+)\nvalue_kind = "(\w+)"\nname = "(\w+)"', blk)
        out[name] = [dict(name=a[3], offset=int(a[0]), size=int(a[1]), value_kind=a[2]) for a in args]
    return out


def write_moe_kernarg_table(ref_dir="/root/reference/prebuilt/gfx1201"):
    if not os.path.isdir(ref_dir):
        return
    table = {}
    for plugin, names in MOE_KERNARG_SOURCES.items():
        args = _manifest_args(ref_dir, plugin)
        for ref_name, ours in names.items():
            table[ref_name] = dict(args=args[ref_name], gfx950=ours)
    json.dump(table, open(os.path.join(HERE, "kernarg_gfx1201_moe.json"), "w"), indent=1, sort_keys=True)


def write_kernarg_table(ref_dir="/root/reference/prebuilt/gfx1201"):
    import re

    if not os.path.isdir(ref_dir):
        return
    write_moe_kernarg_table(ref_dir)
    table = {}
    for plugin, prefixes in KERNARG_SOURCES.items():
        text = open(os.path.join(ref_dir, plugin + ".manifest.toml")).read()
        for blk in text.split("[[kernel]]")[1:]:
            name = re.search(r'name = "(\w+)"', blk).group(1)
            if prefixes is not None and not name.startswith(prefixes):
                continue
            args = re.findall(r'offset = (\d+)\nsize = (\d+)\nvalue_kind = "(\w+)"\nname = "(\w+)"', blk)
            table[name] = [dict(name=a[3], offset=int(a[0]), size=int(a[1]), value_kind=a[2]) for a in args]
    json.dump(table, open(os.path.join(HERE, "kernarg_gfx1201.json"), "w"), indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
