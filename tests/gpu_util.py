"""Helpers of the GPU parity tests: move seeded operands to the device, run the hot path through
the C ABI, bring results back as numpy bit patterns."""
import sys

import numpy as np
import torch

from saber_engine_amd import iu8


def say(msg):
    """Name the case before the GPU step, flushed, so a dead box still tells which one it was."""
    print("[gpu-case]", msg, flush=True)
    sys.stdout.flush()


def dev_u8(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)).cuda()


def dev_f32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def dev_bf16_bits(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda()


def host_u16(t):
    return t.cpu().numpy().view(np.uint16)


class DenseRun:
    """quant -> GEMM of one dense case; keeps every intermediate for the checks."""

    def __init__(self, ctx, case, kernel=None, ks=None, want_acc=True):
        M, N, K, w8 = case["M"], case["N"], case["K"], case["w8"]
        wk = iu8.W8 if w8 else iu8.W4
        x = dev_bf16_bits(case["X"])
        wf = dev_u8(iu8.repack_weights(case["W"], w8))
        ws = dev_f32(case["ws"])
        q = torch.full((iu8.a_bytes(M, K),), 0x55, dtype=torch.uint8, device="cuda")
        a_scale = torch.zeros(M, dtype=torch.float32, device="cuda")
        c = torch.full((M, N), 0x7FC0, dtype=torch.int16, device="cuda")
        ctx.quant(x.data_ptr(), q.data_ptr(), a_scale.data_ptr(), M, K)
        if kernel is None:
            desc = iu8.resolve(wk, M, N, K)
        else:
            desc = iu8.describe(kernel, M, N, K, ks or 1)
        bufs = dict(a=q.data_ptr(), w=wf.data_ptr(), ws=ws.data_ptr(), c=c.data_ptr())
        bufs["as"] = a_scale.data_ptr()
        self.partial = self.counter = None
        if desc.ks > 1:
            # Scratch: undefined at entry (poisoned here); Persistent: zeroed once
            self.partial = torch.full((desc.workspace("decode_partial").bytes // 4,), 0x5A5A5A5A, dtype=torch.int32, device="cuda")
            self.counter = torch.zeros(desc.workspace("decode_counter").bytes // 4, dtype=torch.int32, device="cuda")
            bufs["decode_partial"] = self.partial.data_ptr()
            bufs["decode_counter"] = self.counter.data_ptr()
        ctx.launch(desc, bufs)
        self.acc = None
        if want_acc:
            acc = torch.full((M, N), 0x7BADBAD, dtype=torch.int32, device="cuda")
            ctx.gemm_acc(wk, q.data_ptr(), wf.data_ptr(), acc.data_ptr(), M, N, K)
            self.acc = acc
        torch.cuda.synchronize()
        self.desc = desc
        self.q = iu8.unpack_a(q.cpu().numpy(), M, K)
        self.a_scale = a_scale.cpu().numpy()
        self.C = host_u16(c)
        if want_acc:
            self.acc = self.acc.cpu().numpy()
        self._keep = (x, wf, ws, q, a_scale, c, bufs)
        self.dev = dict(x=x, wf=wf, ws=ws, q=q, a_scale=a_scale, c=c)


def assert_dense_matches(run, ref, w8):
    """Bit-exact: int8 codes, f32 scales, int32 accumulators (16*S for W4), bf16 outputs."""
    np.testing.assert_array_equal(run.q, ref["q"])
    np.testing.assert_array_equal(run.a_scale.view(np.uint32), ref["a_scale"].view(np.uint32))
    if run.acc is not None:
        np.testing.assert_array_equal(run.acc, ref["S"] if w8 else ref["S"] * 16)
    np.testing.assert_array_equal(run.C, ref["C"])
