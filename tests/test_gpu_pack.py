"""A linear read from a tier pack runs on the GPU path: pack bytes (the reference's layout 17 / 19
records) -> offline repack -> quant + GEMM through the C ABI, against the oracle."""
import numpy as np
import pytest
import torch

from oracle import ref
from saber_engine_amd import iu8, synth
from saber_engine_amd.pack import Pack
from tests import pack_writer as pw
from tests.gpu_util import dev_bf16_bits, dev_f32, dev_u8, host_u16, say
from tests.test_pack_reader import gfx12_w4

pytestmark = pytest.mark.gpu


def test_linear_from_a_pack_equals_the_oracle(ctx, tmp_path):
    say("pack -> repack -> quant + gemm")
    M, N, K = 3, 64, 512
    case = synth.dense_case(M, N, K, seed=5)
    codes = synth.unpack_w4(case["W"])
    recs = [dict(name="L7.down.wi4", dtype="U8", shape=[N // 16, K * 8], layout_id=17, shard_kind=2, data=gfx12_w4(codes).tobytes()),
            dict(name="L7.down.wi4s", dtype="F32", shape=[N], layout_id=19, data=case["ws"].astype(np.float32).tobytes())]
    p = tmp_path / "rank0.pack"
    p.write_bytes(pw.build(recs))
    with Pack(p) as pk:
        wk, n, k, w, ws = pk.load_linear("L7.down")
    assert (wk, n, k) == (iu8.W4, N, K)
    x, wf, wsd = dev_bf16_bits(case["X"]), dev_u8(w), dev_f32(ws)
    q = torch.zeros(iu8.a_bytes(M, K), dtype=torch.uint8, device="cuda")
    s = torch.zeros(M, dtype=torch.float32, device="cuda")
    c = torch.zeros((M, N), dtype=torch.int16, device="cuda")
    ctx.quant(x.data_ptr(), q.data_ptr(), s.data_ptr(), M, K)
    ctx.gemm(iu8.W4, q.data_ptr(), s.data_ptr(), wf.data_ptr(), wsd.data_ptr(), c.data_ptr(), M, N, K)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(host_u16(c), ref.linear(case["X"], case["W"], case["ws"], False)["C"])
