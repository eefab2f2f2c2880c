"""The routed-expert layer as a launch train over the C ABI: route+sort with the per-token quant ->
grouped gate+up (token rows gathered) -> SiLU*up requant -> grouped down -> weighted combine; with few
tokens (16-row tiles) the activation rides in gate+up's epilogue and the requant in front of down's K loop.  The train and
its buffers follow the reference's MoE block (crates/saber-kernels/src/moe.rs:9-28, 142-171); the
arithmetic of every GEMM is the iu8 contract.  torch is used for device memory only.
"""
import numpy as np
import torch

from . import iu8


class MoeLayerIU8:
    def __init__(self, ctx, tokens, experts=128, topk=8, hidden=4096, inter=1536, tile_blocks=None, device="cuda", shared=False,
                 fused_back=None):
        """shared: the layer has a shared expert (crates/saber-kernels/src/moe.rs:688-711): every token also
        runs through expert index `experts`, whose weights are the last entry given to set_weights, and
        the combine adds sigmoid(sgate[t]) times that row."""
        self.ctx, self.T, self.E, self.topk, self.H, self.I = ctx, tokens, experts, topk, hidden, inter
        self.shared = bool(shared)
        self.tb = tile_blocks or iu8.moe_tile_blocks(tokens, topk, experts)
        self.rows_cap = iu8.moe_rows_cap(tokens, topk, experts, self.shared)
        self.tiles_cap = iu8.moe_tiles_cap(tokens, topk, experts, self.tb, self.shared)
        i32 = dict(dtype=torch.int32, device=device)
        R = tokens * topk
        self.buf = dict(
            topk_ids=torch.zeros(R, **i32), topk_w=torch.zeros(R, dtype=torch.float32, device=device),
            route_pos=torch.zeros(R, **i32), row_tok=torch.full((self.rows_cap,), -1, **i32),
            row_route=torch.zeros(self.rows_cap, **i32), tile_expert=torch.zeros(self.tiles_cap, **i32),
            tile_row0=torch.zeros(self.tiles_cap, **i32), tile_rows=torch.zeros(self.tiles_cap, **i32),
            expert_cnt=torch.zeros(experts, **i32), meta=torch.zeros(8, **i32),
            blk_cnt=torch.zeros(((tokens + 31) // 32) * experts, **i32), rank=torch.zeros(R, **i32),
            arrive=torch.zeros(1, **i32))          # persistent: zeroed once, left zero by the kernel
        # the bf16 silu of every bf16 input as the device computes it, for the table form of SiLU*up
        self.buf["silu_lut"] = torch.zeros(65536, dtype=torch.int16, device=device)
        ctx.silu_table(self.buf["silu_lut"].data_ptr())
        torch.cuda.synchronize()
        # the shared expert's gate logits, bf16 [T]: bound into the tables only when the layer has one
        self.sgate = torch.zeros(tokens, dtype=torch.int16, device=device) if self.shared else None
        ptr = {n: self.buf[n].data_ptr() for n in self.buf}
        ptr["sgate"] = self.sgate.data_ptr() if self.shared else None
        self.tables = iu8.MoeTables(*[ptr[n] for n in iu8.MOE_TABLE_FIELDS])
        u8 = dict(dtype=torch.uint8, device=device)
        # tokens are quantised once and the grouped gate+up GEMM gathers their rows: the streaming cell
        # (16-row tiles) from the A edge, the MFMA cells from row-major codes (whole 64-byte runs a row)
        self.gather = 1 if self.tb == 1 else 2
        self.q1 = torch.zeros(max(iu8.a_bytes(tokens, hidden), tokens * hidden), **u8)
        self.s1 = torch.zeros(tokens, dtype=torch.float32, device=device)
        # few tokens: the back half as two launches, p = silu(gate) * up straight out of the first GEMM
        self.fused_back = iu8.moe_back_pays(tokens, topk, experts, self.tb, inter) if fused_back is None else bool(fused_back)
        self.p = torch.zeros((self.rows_cap, inter), dtype=torch.int16, device=device) if self.fused_back else None
        self.gu = torch.zeros((self.rows_cap, 2 * inter), dtype=torch.int16, device=device)
        self.q2 = torch.zeros(iu8.a_bytes(self.rows_cap, inter), **u8)
        self.s2 = torch.zeros(self.rows_cap, dtype=torch.float32, device=device)
        self.y = torch.zeros((self.rows_cap, hidden), dtype=torch.int16, device=device)
        self.out = torch.zeros((tokens, hidden), dtype=torch.int16, device=device)
        self.xptr_gu = self.xptr_dn = None

    def set_weights(self, wgu_frag, wsgu, wdn_frag, wsdn):
        """Per-expert gfx950 W4 fragments [E, 2I*H/2] / [E, H*I/2] (uint8) and scales [E,2I] / [E,H] (f32) on device;
        E + 1 of each with a shared expert (the shared expert's last)."""
        self._w = (wgu_frag, wsgu, wdn_frag, wsdn)
        E = self.E + (1 if self.shared else 0)
        assert wgu_frag.shape[0] >= E and wdn_frag.shape[0] >= E
        gu = [[wgu_frag[e].data_ptr(), wsgu[e].data_ptr()] for e in range(E)]
        dn = [[wdn_frag[e].data_ptr(), wsdn[e].data_ptr()] for e in range(E)]
        self.xptr_gu = torch.tensor(np.array(gu, np.int64).ravel(), device=wgu_frag.device)
        self.xptr_dn = torch.tensor(np.array(dn, np.int64).ravel(), device=wgu_frag.device)

    def forward(self, x, logits, stream=0):
        """x bf16 bits [T,H] (int16 tensor), logits bf16 bits [T,E]; with a shared expert its gate logits
        (bf16 bits [T]) are read from self.sgate, which the caller fills; every launch on `stream`."""
        c, T, E, k, H, I = self.ctx, self.T, self.E, self.topk, self.H, self.I
        if H <= 16384:   # the router and the tokens' quantisation, which do not depend on each other, in one launch
            c.moe_route_quant(logits.data_ptr(), x.data_ptr(), self.q1.data_ptr(), self.s1.data_ptr(), T, E, k, H, self.tb,
                              self.tables, stream)
        else:
            c.moe_route(logits.data_ptr(), T, E, k, self.tb, self.tables, stream)
            if self.gather == 1:
                c.quant(x.data_ptr(), self.q1.data_ptr(), self.s1.data_ptr(), T, H, stream)
            else:
                c.quant_rowmajor(x.data_ptr(), self.q1.data_ptr(), self.s1.data_ptr(), T, H, stream)
        if self.fused_back:
            c.moe_gate_up_act(self.q1.data_ptr(), self.s1.data_ptr(), self.xptr_gu.data_ptr(), self.p.data_ptr(), I, H,
                              T, E, k, self.tb, self.tables, stream)
            c.moe_down_rows(self.p.data_ptr(), self.xptr_dn.data_ptr(), self.y.data_ptr(), H, I, T, E, k, self.tb,
                            self.tables, stream)
        else:
            c.moe_grouped(self.q1.data_ptr(), self.s1.data_ptr(), self.xptr_gu.data_ptr(), self.gu.data_ptr(), 2 * I, H,
                          self.gather, T, E, k, self.tb, self.tables, stream)
            c.moe_silu_mul_quant(self.gu.data_ptr(), self.q2.data_ptr(), self.s2.data_ptr(), I, self.rows_cap, self.tables, stream)
            c.moe_grouped(self.q2.data_ptr(), self.s2.data_ptr(), self.xptr_dn.data_ptr(), self.y.data_ptr(), H, I, False,
                          T, E, k, self.tb, self.tables, stream)
        c.moe_combine(self.y.data_ptr(), self.tables, self.out.data_ptr(), T, k, H, stream)
        return self.out
