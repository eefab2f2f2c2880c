"""A reference point for the tile GEMM, never part of the product path: what the vendor library's plain
int8 x int8 -> int32 GEMM (torch._int_mm) sustains on this card on the benchmark's four linear shapes at a given
row count. Operands are distributed like the workload's once unpacked (activation codes ~ N(0, 2.1), weights 16 * w
with w uniform in [-8, 7]); one warm weight matrix a shape, the better of the two B orders, no scaling, int32 output.

    python -m saber_engine_amd.library_ref [rows]      # prints one JSON object

`bench.py` runs this as a child process, so that nothing the library does can take the benchmark line with it.
"""
import json
import sys

SHAPES = (("qkv", 7168, 5120), ("o", 5120, 5120), ("gate_up", 34816, 5120), ("down", 5120, 17408))


def measure(rows=2048):
    import torch
    dev = "cuda"
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    out, ops_all, us_all = {}, 0.0, 0.0
    for name, n, k in SHAPES:
        a = torch.round(torch.randn((rows, k), device=dev, generator=g) * 2.1).clamp(-127, 127).to(torch.int8)
        w = torch.randint(-8, 8, (n, k), device=dev, generator=g, dtype=torch.int8) * 16
        ops = 2.0 * rows * n * k
        best = None
        for b in (w.t(), w.t().contiguous()):
            for _ in range(max(30, int(0.1 / (ops / 2.5e15)))):   # 0.1 s of the shape: the card's clock settles under it
                c = torch._int_mm(a, b)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                c = torch._int_mm(a, b)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 20
            best = us if best is None else min(best, us)
        out[name] = dict(us=round(best, 2), tops=round(ops / best / 1e6, 1))
        ops_all += ops
        us_all += best
        del a, w, b, c
    out["value"] = round(ops_all / us_all / 1e6, 1)
    out["rows"] = rows
    return out


if __name__ == "__main__":
    print(json.dumps(measure(int(sys.argv[1]) if len(sys.argv) > 1 else 2048)))
