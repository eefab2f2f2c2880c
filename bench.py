#!/usr/bin/env python3
"""Benchmark of the W4A8-iu8 decoder-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--m 1] [--no-prefill] [--no-cpu]

A step is one pass of the hot path over one batch: the four W4A8 linears of one 27B-class decoder
layer (QKV 7168x5120, O 5120x5120, gate+up 34816x5120, down 5120x17408), each as
per-token int8 quantisation + int4 x int8 GEMM + scale epilogue to bf16, at M tokens (default 1).
Successive steps walk over LAYERS distinct copies of the weights (> 3x the 256 MB Infinity Cache),
so every weight byte comes from HBM ("cold"); all inputs are resident in HBM before the timed
region. The K timed steps are one HIP-graph replay bracketed by synchronisation.

Prints ONE JSON line. `value` is algorithmic GB/s of the whole step (quant + GEMM launches);
`roofline` is the dominant kernel (the decode GEMM) timed alone with HIP events on its stream;
`prefill_m2048` carries the second half of the metric (int8 TOPS at M=2048, MFMA roofline);
`cpu_baseline` is the CPU oracle's vectorised body on the host cores, on a bounded sample.
"""
import argparse
import math
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0     # MI355X published dense int8 MFMA peak
LAYERS = 6                  # distinct weight copies walked by successive steps (6 x 165 MB)
# HBM-side bytes of one launch of the dominant kernel, mean over the four layer shapes. A counter
# figure cannot be read inside this process: it comes from two rocprofv3 --pmc runs of this very
# command (FETCH_SIZE, then WRITE_SIZE), each counter scaled by what it reads for the 256 MiB copy
# probe, and is kept in the profile summary named below. Keyed by (kernel, M); None = not measured.
TRAFFIC_SOURCE = "profiles/macaq_iu8_decq_w4__layer_set_m1.txt"
TRAFFIC = {("macaq_iu8_decq_w4_r1 + macaq_iu8_decq_w4_tm1", 1): 41749312.0, ("macaq_iu8_dec_w4_tm1", 1): 41995646.0}


def alg_bytes(m, n, k, w8=False):
    """Algorithmic bytes of one linear: weights + row scales + bf16 activations in + bf16 out."""
    return (n * k if w8 else n * k // 2) + 4 * n + 2 * m * k + 2 * m * n


SETTLE_MS = 30.0   # of the step's own graph, replayed untimed in front of the timed replay


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=120)
    ap.add_argument("--warmup", type=int, default=600)   # 24 ms of the step: the card's clock settles over tens of ms
    ap.add_argument("--m", type=int, default=1, help="tokens per step (decode band, 1..16)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-moe", action="store_true")
    ap.add_argument("--no-producers", action="store_true", help="skip the Hadamard-basis producers' section")
    ap.add_argument("--no-library", action="store_true", help="skip the vendor library's int8 GEMM reference figure (a child process)")
    ap.add_argument("--no-other-m", action="store_true", help="prefill at M = 2048 only (a profiler run that wants one M a kernel)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--probe-copy", action="store_true",
                    help="also launch the 256 MiB copy probe (scale factor of the HBM byte counters under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU (no sharding, no collectives); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from saber_engine_amd import iu8, synth

    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    ctx = iu8.Context()
    M, K_steps, W_steps = args.m, args.steps, args.warmup
    linears = synth.LAYER_LINEARS

    # ---- operands: one seeded layer (W -> ws -> A per linear), replicated to LAYERS distinct buffers
    rng = np.random.default_rng(0)
    host = {}
    for name, n, k in linears:
        Wc, ws = synth.weights(rng, n, k, False)
        X = synth.activations(rng, max(M, 1), k)
        host[name] = dict(W=Wc, ws=ws, X=X)
    dev_w = {name: [] for name, _, _ in linears}
    dev_ws, dev_x, dev_q, dev_as, dev_c = {}, {}, {}, {}, {}
    for name, n, k in linears:
        frag = torch.from_numpy(iu8.repack_w4(host[name]["W"])).to(dev)
        dev_w[name] = [frag] + [frag.clone() for _ in range(LAYERS - 1)]
        dev_ws[name] = torch.from_numpy(host[name]["ws"]).to(dev)
        dev_x[name] = torch.from_numpy(host[name]["X"].view(np.int16)).to(dev)
        dev_q[name] = torch.zeros(iu8.a_bytes(M, k), dtype=torch.uint8, device=dev)
        dev_as[name] = torch.zeros(M, dtype=torch.float32, device=dev)
        dev_c[name] = torch.zeros((M, n), dtype=torch.int16, device=dev)
    descs = {name: iu8.resolve(iu8.W4, M, n, k) for name, n, k in linears}
    # one launch a linear (quantisation fused into the GEMV's activation staging) where every shape allows
    fused = all(iu8.fused_holds(M, k) for _, _, k in linears)
    fdescs = {name: iu8.resolve_fused(iu8.W4, M, n, k) for name, n, k in linears} if fused else {}
    qdescs = {name: iu8.resolve_quant(M, k) for name, n, k in linears}
    pbytes = max([d.workspace("decode_partial").bytes for d in descs.values() if d.ks > 1] + [4])
    cbytes = max([d.workspace("decode_counter").bytes for d in descs.values() if d.ks > 1] + [4])
    partial = torch.zeros(pbytes // 4, dtype=torch.int32, device=dev)
    counter = torch.zeros(cbytes // 4, dtype=torch.int32, device=dev)

    stream = torch.cuda.Stream()
    sh = stream.cuda_stream
    if args.probe_copy:
        nbytes = 256 << 20
        src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        pd = iu8.describe_raw("iu8_probe_copy", (4096, 1, 1), 256, n=nbytes // 16)
        for _ in range(3):
            ctx.launch(pd, dict(src=src.data_ptr(), dst=dst.data_ptr()), sh)
        stream.synchronize()
        del src, dst

    def launch_quant(name):
        ctx.launch(qdescs[name], dict(x=dev_x[name].data_ptr(), q=dev_q[name].data_ptr(), scale=dev_as[name].data_ptr()), sh)

    def launch_gemm(name, layer):
        b = dict(a=dev_q[name].data_ptr(), w=dev_w[name][layer].data_ptr(), ws=dev_ws[name].data_ptr(), c=dev_c[name].data_ptr(),
                 decode_partial=partial.data_ptr(), decode_counter=counter.data_ptr())
        b["as"] = dev_as[name].data_ptr()
        ctx.launch(descs[name], b, sh)

    def launch_fused(name, layer):
        # the optional code / scale outputs stay unbound: the step needs the bf16 output only
        d = fdescs[name]
        for i in range(d.n_args):
            if d.args[i].name in (b"q", b"scale"):
                d.args[i].kind = iu8.ARG_NULL_BUFFER
        ctx.launch(d, dict(x=dev_x[name].data_ptr(), w=dev_w[name][layer].data_ptr(), ws=dev_ws[name].data_ptr(),
                           c=dev_c[name].data_ptr()), sh)

    def step(i, mode="hot"):
        """hot: the path as a caller runs it (fused launch where the shapes allow, else producer +
        GEMM); two: always producer + GEMM; gemm: the GEMM launches alone."""
        for name, _, _ in linears:
            if mode == "hot" and fused:
                launch_fused(name, i % LAYERS)
                continue
            if mode != "gemm":
                launch_quant(name)
            launch_gemm(name, i % LAYERS)

    def capture(nsteps, mode="hot"):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(nsteps):
                step(i, mode)
        return g

    with torch.cuda.stream(stream):
        for i in range(W_steps):
            step(i)
    stream.synchronize()
    g_all = capture(K_steps)
    g_two = capture(K_steps, "two")
    g_gemm = capture(K_steps, "hot" if fused else "gemm")
    with torch.cuda.stream(stream):
        g_all.replay()
        g_two.replay()
        g_gemm.replay()
    torch.cuda.synchronize()

    # ---- settle phase (untimed, beside the W warm-up steps the caller asked for): the card's clock takes tens of
    # milliseconds under a kernel to reach the rate it then keeps, and it settles upwards; a handful of
    # warm-up steps is a fraction of a millisecond. The same graph of K steps is replayed until SETTLE_MS of it
    # have run; the count is reported as config.settle_steps. Nothing of the timed region moves here.
    ev_a, ev_b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        ev_a.record(stream)
        g_all.replay()
        ev_b.record(stream)
    torch.cuda.synchronize()
    settle_replays = max(1, int(math.ceil(SETTLE_MS / max(ev_a.elapsed_time(ev_b), 1e-3))))
    with torch.cuda.stream(stream):
        for _ in range(settle_replays):
            g_all.replay()
        # the last settling replays go out the way the timed one does -- a replay, then a synchronisation -- so that
        # the host's side of that pair (its caches, the wake-up from a short wait instead of a 30 ms one) is settled too
        for _ in range(4):
            torch.cuda.synchronize()
            g_all.replay()

    # ---- the timed region: exactly K steps, one graph replay, bracketed by synchronisation; the host clock gives
    # ms_per_step and `value`, HIP events on the replay's stream give the same K steps without the host's
    # launch and wake-up latency (ms_per_step_events)
    with torch.cuda.stream(stream):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        g_all.replay()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ms_per_step = (t1 - t0) * 1e3 / K_steps
        # the same replay once more between two events (their records stay out of the host-timed region)
        ev_a.record(stream)
        g_all.replay()
        ev_b.record(stream)
        torch.cuda.synchronize()
    ms_per_step_events = ev_a.elapsed_time(ev_b) / K_steps
    step_bytes = sum(alg_bytes(M, n, k) for _, n, k in linears)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- the same K steps as producer + GEMM launches (what the fused launch replaces)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    with torch.cuda.stream(stream):
        g_two.replay()
    torch.cuda.synchronize()
    two_ms = (time.perf_counter() - t2) * 1e3 / K_steps

    # ---- the same K steps on ONE weight copy (165 MB at M = 1: resident in the 256 MB Infinity Cache after the
    # first step): the warm figure, reported beside the cold one and labelled, never as `value`
    g_warm = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g_warm, stream=stream):
        for _ in range(K_steps):
            step(0)
    with torch.cuda.stream(stream):
        g_warm.replay()
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    with torch.cuda.stream(stream):
        g_warm.replay()
    torch.cuda.synchronize()
    warm_ms = (time.perf_counter() - t3) * 1e3 / K_steps

    # ---- the dominant kernel alone (the decode GEMV, 4 launches a step), HIP events on its stream
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        for _ in range(max(1, settle_replays // 2)):
            g_gemm.replay()
        ev0.record(stream)
        g_gemm.replay()
        ev1.record(stream)
    torch.cuda.synchronize()
    gemm_us = ev0.elapsed_time(ev1) * 1e3 / (K_steps * len(linears))
    if fused:   # reads the bf16 rows itself
        gemm_bytes = sum(alg_bytes(M, n, k) for _, n, k in linears) / len(linears)
        kname = " + ".join(sorted({d.kernel.decode() for d in fdescs.values()}))   # the step's launches: one symbol or two
    else:       # reads the int8 codes and the row scales
        gemm_bytes = sum(alg_bytes(M, n, k) - 2 * M * k + M * k + 4 * M for _, n, k in linears) / len(linears)
        kname = " + ".join(sorted({d.kernel.decode() for d in descs.values()}))
    achieved = gemm_bytes / (gemm_us * 1e-6) / 1e9
    roofline = dict(bound="hbm", kernel=kname, achieved=round(achieved, 1), peak=HBM_PEAK_GBPS,
                    unit="GB/s", frac=round(achieved / HBM_PEAK_GBPS, 4), traffic=TRAFFIC.get((kname, M)),
                    traffic_source="not of this run: FETCH_SIZE + WRITE_SIZE per launch from rocprofv3 --pmc runs of this command, "
                                   "scaled by the copy probe, " + TRAFFIC_SOURCE,
                    avg_launch_us=round(gemm_us, 3), bytes_per_launch=gemm_bytes,
                    note="mean over the four layer shapes, cold weights (rotating %d copies), graph replay" % LAYERS)

    # ---- the measured HBM ceiling beside the nominal one: the streaming-read probe over 1 GiB (four times the
    # 256 MB Infinity Cache, so every launch reads from memory), best of three grids, HIP events on its stream
    def probe_read_us(ptr, nbytes, grid, reps):
        pd = iu8.describe_raw("iu8_probe_read", (grid, 1, 1), 256, n=nbytes // 16)
        pb = dict(src=ptr, out=probe_out.data_ptr())
        with torch.cuda.stream(stream):
            ctx.launch(pd, pb, sh)
            p0, p1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            p0.record(stream)
            for _ in range(reps):
                ctx.launch(pd, pb, sh)
            p1.record(stream)
        torch.cuda.synchronize()
        return p0.elapsed_time(p1) * 1e3 / reps

    probe_out = torch.zeros(16, dtype=torch.int32, device=dev)
    big = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    big.random_(0, 255)
    hbm_probe = max((1 << 30) / probe_read_us(big.data_ptr(), 1 << 30, g, 8) / 1e3 for g in (1024, 2048, 4096))
    del big
    roofline["hbm_probe_gbps"] = round(hbm_probe, 1)
    roofline["frac_of_probe"] = round(achieved / hbm_probe, 4)

    # ---- every linear of the step by itself: the fused launch alone (graph of K launches walking the weight
    # copies), and the read probe on the same weight bytes, cold the same way. down = the 5120 x 17408 GEMV.
    # (the side figures from here on do not depend on --steps: graphs of at least 120 launches, replayed a few
    # times before the timed replay, so a short driver run reads the same per-linear numbers as a long one)
    SIDE_STEPS = max(K_steps, 120)
    per_linear = {}
    for name, n, k in linears:
        gl = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gl, stream=stream):
            for i in range(SIDE_STEPS):
                if fused:
                    launch_fused(name, i % LAYERS)
                else:
                    launch_gemm(name, i % LAYERS)
        with torch.cuda.stream(stream):
            for _ in range(4):
                gl.replay()
            l0, l1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            l0.record(stream)
            gl.replay()
            l1.record(stream)
        torch.cuda.synchronize()
        us = l0.elapsed_time(l1) * 1e3 / SIDE_STEPS
        nb = alg_bytes(M, n, k) if fused else alg_bytes(M, n, k) - M * k + 4 * M
        wbytes = n * k // 2
        pus = min(sum(probe_read_us(dev_w[name][layer].data_ptr(), wbytes, g, 1) for layer in range(LAYERS)) / LAYERS for g in (512, 1024, 2048))
        per_linear[name] = dict(n=n, k=k, kernel=(fdescs if fused else descs)[name].kernel.decode(), us=round(us, 2), bytes=nb,
                                gbps=round(nb / us / 1e3, 1), hbm_frac=round(nb / us / 1e3 / HBM_PEAK_GBPS, 4),
                                frac_of_probe=round(nb / us / 1e3 / hbm_probe, 4), read_probe_us=round(pus, 2))
        del gl

    # ---- the MLP of the step (gate+up -> SiLU * up + requantisation -> down) as ONE persistent launch
    # (macaq_iu8f_mlp_w4_tm1) beside the three launches it replaces (fused linear, silu-mul-quant
    # producer, GEMV), both as graphs walking the weight copies. More work than the step's two linears
    # (the activation between them), so it is reported here and not part of `value`.
    mlp = None
    (_, n_gu, hid), (_, _, inter) = [l for l in linears if l[0] == "gate_up"][0], [l for l in linears if l[0] == "down"][0]
    if fused and n_gu == 2 * inter and iu8.mlp_chain_holds(M, hid, inter):
        p_rows = torch.zeros((M, inter), dtype=torch.int16, device=dev)
        state = torch.zeros(iu8.MLP_CHAIN_STATE_BYTES // 4, dtype=torch.int32, device=dev)
        q_dn = torch.zeros(iu8.a_bytes(M, inter), dtype=torch.uint8, device=dev)
        s_dn = torch.zeros(M, dtype=torch.float32, device=dev)
        d_silu, d_dn = iu8.resolve_silu_mul_quant(M, inter), descs["down"]

        def chain(layer):
            ctx.mlp_chain(dev_x["gate_up"].data_ptr(), dev_w["gate_up"][layer].data_ptr(), dev_ws["gate_up"].data_ptr(),
                          dev_w["down"][layer].data_ptr(), dev_ws["down"].data_ptr(), None, p_rows.data_ptr(), state.data_ptr(),
                          dev_c["down"].data_ptr(), M, hid, inter, stream=sh)

        def three(layer):
            launch_fused("gate_up", layer)
            ctx.launch(d_silu, dict(gu=dev_c["gate_up"].data_ptr(), q=q_dn.data_ptr(), scale=s_dn.data_ptr()), sh)
            b = dict(a=q_dn.data_ptr(), w=dev_w["down"][layer].data_ptr(), ws=dev_ws["down"].data_ptr(), c=dev_c["down"].data_ptr(),
                     decode_partial=partial.data_ptr(), decode_counter=counter.data_ptr())
            b["as"] = s_dn.data_ptr()
            ctx.launch(d_dn, b, sh)

        times, bits = {}, {}
        for tag, fn in (("three_launches", three), ("chain", chain)):
            gl = torch.cuda.CUDAGraph()
            with torch.cuda.stream(stream):
                fn(0)
            stream.synchronize()
            with torch.cuda.graph(gl, stream=stream):
                for i in range(SIDE_STEPS):
                    fn(i % LAYERS)
            with torch.cuda.stream(stream):
                for _ in range(4):
                    gl.replay()
                l0, l1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                l0.record(stream)
                gl.replay()
                l1.record(stream)
            torch.cuda.synchronize()
            times[tag] = l0.elapsed_time(l1) * 1e3 / SIDE_STEPS
            bits[tag] = dev_c["down"].clone()
            del gl
        wb = (n_gu * hid + hid * inter) // 2
        mlp = dict(kernel="macaq_iu8f_mlp_w4_tm1", weight_bytes=wb, us_chain=round(times["chain"], 2),
                   us_three_launches=round(times["three_launches"], 2),
                   us_two_linears_alone=round(per_linear["gate_up"]["us"] + per_linear["down"]["us"], 2),
                   chain_pays_by_law=iu8.mlp_chain_pays(M, hid, inter),
                   gbps_chain=round(wb / times["chain"] / 1e3, 1), same_bytes=bool(torch.equal(bits["chain"], bits["three_launches"])),
                   state_status=int(state[iu8.MLP_CHAIN_STATUS_OFFSET // 4].item()))
        launch_fused("down", (K_steps - 1) % LAYERS)   # dev_c["down"] back to the step's own output for the spot check below
        stream.synchronize()

    # ---- parity spot check against the CPU oracle, and the CPU baseline beside it
    out = dict(metric="W4A8 GEMM GB/s (%HBM) at M=1; int8 TOPS (%MFMA peak) at M=2048", value=round(value, 1), unit="GB/s",
               n_gpus=1, steps=K_steps, warmup=W_steps, ms_per_step=round(ms_per_step, 5),
               ms_per_step_events=round(ms_per_step_events, 5), higher_is_better=True,
               scaling="weak", vs_baseline=None, dtype="int8", data="synthetic (seed 0)",
               config=dict(workload="configs[1]: decode-batch W4A8 linear set of one 27B-class layer (QKV, O, gate+up, down), "
                                    "hidden 5120, TP=1", arithmetic="int4 weights x int8 activations -> int32 accumulators -> bf16 outputs", m=M, layers_rotated=LAYERS, cold=True,
                           launches_per_step=(1 if fused else 2) * len(linears), fused_quant=fused,
                           settle_steps=settle_replays * K_steps, settle_ms=SETTLE_MS,
                           gbps_by_events=round(step_bytes / (ms_per_step_events * 1e-3) / 1e9, 1),
                           hbm_frac=round(value / HBM_PEAK_GBPS, 4),
                           two_launch_gbps=round(step_bytes / (two_ms * 1e-3) / 1e9, 1),
                           warm_cache_gbps=round(step_bytes / (warm_ms * 1e-3) / 1e9, 1),
                           hbm_frac_of_probe=round(value / hbm_probe, 4)),
               roofline=roofline)
    out["decode_m%d" % M] = dict(per_linear=per_linear, mlp_chain=mlp, note="one launch a linear, cold weights, graph replay; read_probe_us = a plain "
                                 "streaming read of the same weight bytes, cold the same way; down is the 5120x17408 GEMV")

    if not args.no_cpu:
        from oracle import ref

        threads = min(os.cpu_count() or 1, 16)
        ok = True
        t_cpu, n_cpu = 0.0, 0
        while t_cpu < args.cpu_seconds:
            for name, n, k in linears:
                c0 = time.perf_counter()
                r = ref.linear(host[name]["X"][:M], host[name]["W"], host[name]["ws"], False, threads=threads, pin=1)
                t_cpu += time.perf_counter() - c0
                if n_cpu == 0:
                    got = dev_c[name].cpu().numpy().view(np.uint16)
                    ok = ok and bool(np.array_equal(got, r["C"]))
            n_cpu += 1
        # ... and on one core (a quarter of the time budget again)
        t_one, n_one = 0.0, 0
        while t_one < args.cpu_seconds / 4:
            for name, n, k in linears:
                c0 = time.perf_counter()
                ref.linear(host[name]["X"][:M], host[name]["W"], host[name]["ws"], False, threads=1, pin=1)
                t_one += time.perf_counter() - c0
            n_one += 1
        isa = {0: "scalar", 1: "avx2", 2: "avx512-vnni"}[ref.lib().w4a8_isa()]
        try:    # the host's last-level cache against the step's 165 MB of weights, read again every step
            txt = open("/sys/devices/system/cpu/cpu0/cache/index3/size").read().strip()
            llc = int(txt[:-1]) * {"K": 1 << 10, "M": 1 << 20, "G": 1 << 30}[txt[-1]]
        except Exception:
            llc = None
        wbytes_step = sum(n * k // 2 for _, n, k in linears)
        out["cpu_baseline"] = dict(value=round(step_bytes * n_cpu / t_cpu / 1e9, 2), unit="GB/s", cores=threads, kind="port",
                                   sample="%d steps (quant + GEMM + epilogue of the same four linears, M=%d), %s body, "
                                          "threads pinned one per core, 16-column tiles" % (n_cpu, M, isa),
                                   single_core_gbps=round(step_bytes * n_one / t_one / 1e9, 2), single_core_steps=n_one,
                                   weight_bytes_per_step=wbytes_step, llc_bytes=llc,
                                   weights="unknown" if llc is None else ("DRAM-cold: the step's weights exceed the LLC and every step "
                                           "re-reads all of them" if wbytes_step > llc else "LLC-warm: the step's weights fit the LLC"))
        out["parity_vs_oracle"] = ok

    # ---- the other batch sizes of configs[1] (M = 4, 8, 16) through the same step: a linear is one fused
    # launch while its rows fit the fused form (M <= 4 and pow2(M) * K <= 20 KiB), else producer + GEMV;
    # graph replay, cold weights
    def decode_at(DM, nsteps=60):
        xs, qs, ss, cs = {}, {}, {}, {}
        for name, n, k in linears:
            xs[name] = torch.from_numpy(synth.activations(np.random.default_rng(2), DM, k).view(np.int16)).to(dev)
            qs[name] = torch.zeros(iu8.a_bytes(DM, k), dtype=torch.uint8, device=dev)
            ss[name] = torch.zeros(DM, dtype=torch.float32, device=dev)
            cs[name] = torch.zeros((DM, n), dtype=torch.int16, device=dev)
        nlaunch = sum(1 if iu8.fused_holds(DM, k) else 2 for _, _, k in linears)

        def one(i):
            for name, n, k in linears:
                w, wsd = dev_w[name][i % LAYERS].data_ptr(), dev_ws[name].data_ptr()
                if iu8.fused_holds(DM, k):
                    d = iu8.resolve_fused(iu8.W4, DM, n, k)
                    for j in range(d.n_args):
                        if d.args[j].name in (b"q", b"scale"):
                            d.args[j].kind = iu8.ARG_NULL_BUFFER
                    ctx.launch(d, dict(x=xs[name].data_ptr(), w=w, ws=wsd, c=cs[name].data_ptr()), sh)
                else:
                    ctx.launch(iu8.resolve_quant(DM, k), dict(x=xs[name].data_ptr(), q=qs[name].data_ptr(), scale=ss[name].data_ptr()), sh)
                    d = iu8.resolve(iu8.W4, DM, n, k)
                    assert d.ks == 1
                    b = dict(a=qs[name].data_ptr(), w=w, ws=wsd, c=cs[name].data_ptr())
                    b["as"] = ss[name].data_ptr()
                    ctx.launch(d, b, sh)

        def graph_us(fn, reps_settle=8):
            """nsteps calls of fn(i) as one graph: replayed to settle, then one replay timed by HIP events"""
            gg = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gg, stream=stream):
                for i in range(nsteps):
                    fn(i)
            d0, d1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            with torch.cuda.stream(stream):
                for _ in range(reps_settle):
                    gg.replay()
                d0.record(stream)
                gg.replay()
                d1.record(stream)
            torch.cuda.synchronize()
            del gg
            return d0.elapsed_time(d1) * 1e3 / nsteps

        with torch.cuda.stream(stream):
            for i in range(6):
                one(i)
        stream.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            for i in range(nsteps):
                one(i)
        with torch.cuda.stream(stream):
            for _ in range(8):
                g.replay()
        torch.cuda.synchronize()
        c0 = time.perf_counter()
        with torch.cuda.stream(stream):
            g.replay()
        torch.cuda.synchronize()
        us = (time.perf_counter() - c0) * 1e6 / nsteps
        nbytes = sum(alg_bytes(DM, n, k) for _, n, k in linears)
        # every linear of the step by itself: the producer launch and the GEMV apart (or the one fused launch)
        per = {}
        for name, n, k in linears:
            wsd = dev_ws[name].data_ptr()
            if iu8.fused_holds(DM, k):
                d = iu8.resolve_fused(iu8.W4, DM, n, k)
                for j in range(d.n_args):
                    if d.args[j].name in (b"q", b"scale"):
                        d.args[j].kind = iu8.ARG_NULL_BUFFER
                f_us = graph_us(lambda i: ctx.launch(d, dict(x=xs[name].data_ptr(), w=dev_w[name][i % LAYERS].data_ptr(), ws=wsd,
                                                             c=cs[name].data_ptr()), sh))
                per[name] = dict(kernel=d.kernel.decode(), us=round(f_us, 2), gbps=round(alg_bytes(DM, n, k) / f_us / 1e3, 1))
            else:
                qd, gd = iu8.resolve_quant(DM, k), iu8.resolve(iu8.W4, DM, n, k)
                q_us = graph_us(lambda i: ctx.launch(qd, dict(x=xs[name].data_ptr(), q=qs[name].data_ptr(), scale=ss[name].data_ptr()), sh))

                def gemv(i):
                    b = dict(a=qs[name].data_ptr(), w=dev_w[name][i % LAYERS].data_ptr(), ws=wsd, c=cs[name].data_ptr())
                    b["as"] = ss[name].data_ptr()
                    ctx.launch(gd, b, sh)

                g_us = graph_us(gemv)
                gb = alg_bytes(DM, n, k) - 2 * DM * k + DM * k + 4 * DM   # the GEMV reads codes and scales
                per[name] = dict(kernel=gd.kernel.decode(), gemv_us=round(g_us, 2), gemv_gbps=round(gb / g_us / 1e3, 1),
                                 producer=qd.kernel.decode(), producer_us=round(q_us, 2))
        del g
        res = dict(us_per_step=round(us, 2), gbps=round(nbytes / us / 1e3, 1), hbm_frac=round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                   launches_per_step=nlaunch, per_linear=per)
        # the step's MLP as one persistent launch beside its three launches, where the rows fit the chain's forms
        if iu8.mlp_chain_holds(DM, hid, inter):
            p_rows = torch.zeros((DM, inter), dtype=torch.int16, device=dev)
            state = torch.zeros(iu8.MLP_CHAIN_STATE_BYTES // 4, dtype=torch.int32, device=dev)
            q_dn = torch.zeros(iu8.a_bytes(DM, inter), dtype=torch.uint8, device=dev)
            s_dn = torch.zeros(DM, dtype=torch.float32, device=dev)
            d_gu, d_silu, d_dn = iu8.resolve_fused(iu8.W4, DM, n_gu, hid), iu8.resolve_silu_mul_quant(DM, inter), iu8.resolve(iu8.W4, DM, hid, inter)
            for j in range(d_gu.n_args):
                if d_gu.args[j].name in (b"q", b"scale"):
                    d_gu.args[j].kind = iu8.ARG_NULL_BUFFER

            def chain(i):
                ctx.mlp_chain(xs["gate_up"].data_ptr(), dev_w["gate_up"][i % LAYERS].data_ptr(), dev_ws["gate_up"].data_ptr(),
                              dev_w["down"][i % LAYERS].data_ptr(), dev_ws["down"].data_ptr(), None, p_rows.data_ptr(), state.data_ptr(),
                              cs["down"].data_ptr(), DM, hid, inter, stream=sh)

            def three(i):
                ctx.launch(d_gu, dict(x=xs["gate_up"].data_ptr(), w=dev_w["gate_up"][i % LAYERS].data_ptr(), ws=dev_ws["gate_up"].data_ptr(),
                                      c=cs["gate_up"].data_ptr()), sh)
                ctx.launch(d_silu, dict(gu=cs["gate_up"].data_ptr(), q=q_dn.data_ptr(), scale=s_dn.data_ptr()), sh)
                b = dict(a=q_dn.data_ptr(), w=dev_w["down"][i % LAYERS].data_ptr(), ws=dev_ws["down"].data_ptr(), c=cs["down"].data_ptr())
                b["as"] = s_dn.data_ptr()
                ctx.launch(d_dn, b, sh)

            with torch.cuda.stream(stream):
                three(0)
            stream.synchronize()
            want = cs["down"].clone()
            t3 = graph_us(three)
            with torch.cuda.stream(stream):
                chain(0)
            stream.synchronize()
            same = bool(torch.equal(want, cs["down"]))
            tc = graph_us(chain)
            res["mlp_chain"] = dict(kernel=iu8.resolve_mlp_chain(DM, hid, inter).kernel.decode(), us_chain=round(tc, 2), us_three_launches=round(t3, 2),
                                    chain_pays_by_law=iu8.mlp_chain_pays(DM, hid, inter), same_bytes=same, state_status=int(state[iu8.MLP_CHAIN_STATUS_OFFSET // 4].item()))
        elif iu8.gate_up_act_holds(DM, hid, inter):
            # the step's MLP at 5-16 rows: producer -> gate+up -> SiLU*up + requant -> down, against the same with the
            # activation in the gate+up linear's epilogue (producer -> gate+up with activation -> producer on p -> down)
            p_rows = torch.zeros((DM, inter), dtype=torch.int16, device=dev)
            q_dn = torch.zeros(iu8.a_bytes(DM, inter), dtype=torch.uint8, device=dev)
            s_dn = torch.zeros(DM, dtype=torch.float32, device=dev)
            d_q, d_gu, d_silu = iu8.resolve_quant(DM, hid), iu8.resolve(iu8.W4, DM, n_gu, hid), iu8.resolve_silu_mul_quant(DM, inter)
            d_qp, d_dn, d_act = iu8.resolve_quant(DM, inter), iu8.resolve(iu8.W4, DM, hid, inter), iu8.resolve_gate_up_act(DM, hid, inter)
            d_act.arg("gu").kind = iu8.ARG_NULL_BUFFER

            def down(i):
                b = dict(a=q_dn.data_ptr(), w=dev_w["down"][i % LAYERS].data_ptr(), ws=dev_ws["down"].data_ptr(), c=cs["down"].data_ptr())
                b["as"] = s_dn.data_ptr()
                ctx.launch(d_dn, b, sh)

            def four(i):
                ctx.launch(d_q, dict(x=xs["gate_up"].data_ptr(), q=qs["gate_up"].data_ptr(), scale=ss["gate_up"].data_ptr()), sh)
                b = dict(a=qs["gate_up"].data_ptr(), w=dev_w["gate_up"][i % LAYERS].data_ptr(), ws=dev_ws["gate_up"].data_ptr(), c=cs["gate_up"].data_ptr())
                b["as"] = ss["gate_up"].data_ptr()
                ctx.launch(d_gu, b, sh)
                ctx.launch(d_silu, dict(gu=cs["gate_up"].data_ptr(), q=q_dn.data_ptr(), scale=s_dn.data_ptr()), sh)
                down(i)

            def with_act(i):
                ctx.launch(d_q, dict(x=xs["gate_up"].data_ptr(), q=qs["gate_up"].data_ptr(), scale=ss["gate_up"].data_ptr()), sh)
                b = dict(a=qs["gate_up"].data_ptr(), w=dev_w["gate_up"][i % LAYERS].data_ptr(), ws=dev_ws["gate_up"].data_ptr(), p=p_rows.data_ptr())
                b["as"] = ss["gate_up"].data_ptr()
                ctx.launch(d_act, b, sh)
                ctx.launch(d_qp, dict(x=p_rows.data_ptr(), q=q_dn.data_ptr(), scale=s_dn.data_ptr()), sh)
                down(i)

            with torch.cuda.stream(stream):
                four(0)
            stream.synchronize()
            want = cs["down"].clone()
            t4 = graph_us(four)
            with torch.cuda.stream(stream):
                with_act(0)
            stream.synchronize()
            same = bool(torch.equal(want, cs["down"]))
            ta = graph_us(with_act)
            res["mlp"] = dict(kernel=d_act.kernel.decode(), us_four_launches=round(t4, 2), us_with_activation_in_gate_up=round(ta, 2), same_bytes=same)
        return res

    if M == 1 and not args.no_other_m:
        out["decode_other_m"] = {"m%d" % DM: decode_at(DM) for DM in (4, 8, 16)}

    # ---- the second half of the metric: int8 TOPS at M=2048 on the same four shapes. Activations are
    # the configuration's (bf16 N(0,1), 0.5 % of the channels x20), quantised by the producer kernel:
    # the operand values set the card's clock under MFMA load, so uniform random codes would misstate it.
    def prefill_at(PM, warm, reps, fused_too=False):
        pf = {}
        tot_ops, tot_us, tot_q_us = 0.0, 0.0, 0.0
        for name, n, k in linears:
            d = iu8.resolve(iu8.W4, PM, n, k)
            x = torch.from_numpy(synth.activations(np.random.default_rng(1), PM, k).view(np.int16)).to(dev)
            q = torch.zeros(iu8.a_bytes(PM, k), dtype=torch.uint8, device=dev)
            a_s = torch.zeros(PM, dtype=torch.float32, device=dev)
            c = torch.zeros((PM, n), dtype=torch.int16, device=dev)
            qd = iu8.resolve_quant(PM, k)
            qb = dict(x=x.data_ptr(), q=q.data_ptr(), scale=a_s.data_ptr())
            bs = []
            for layer in range(LAYERS):     # successive launches walk the weight copies: cold weights here too
                b = dict(a=q.data_ptr(), w=dev_w[name][layer].data_ptr(), ws=dev_ws[name].data_ptr(), c=c.data_ptr())
                b["as"] = a_s.data_ptr()
                bs.append(b)
            with torch.cuda.stream(stream):
                for _ in range(3):
                    ctx.launch(qd, qb, sh)
                for i in range(warm):  # 40-300 ms of this kernel: the card's clock takes tens of ms to settle where it stays under it
                    ctx.launch(d, bs[i % LAYERS], sh)
                e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
                e0.record(stream)
                for _ in range(reps):
                    ctx.launch(qd, qb, sh)
                e1.record(stream)
                for i in range(reps):
                    ctx.launch(d, bs[i % LAYERS], sh)
                e2.record(stream)
            torch.cuda.synchronize()
            q_us = e0.elapsed_time(e1) * 1e3 / reps
            us = e1.elapsed_time(e2) * 1e3 / reps
            ops = 2.0 * PM * n * k
            pf[name] = dict(kernel=d.kernel.decode(), grid=list(d.grid), us=round(us, 2), tops=round(ops / us / 1e6, 1),
                            quant_us=round(q_us, 2))
            if fused_too:
                # the north_star's form, measured beside it: row scales (a pass that stores no codes) + the tile GEMM
                # that quantises on the way into its A stage (macaq_iu8_pfq_*); same bytes, see tests/test_gpu_pfq.py
                fd = iu8.resolve_prefill_fused(iu8.W4, PM, n, k)
                fbs = []
                for layer in range(LAYERS):
                    fb = dict(x=x.data_ptr(), w=dev_w[name][layer].data_ptr(), ws=dev_ws[name].data_ptr(), c=c.data_ptr())
                    fb["as"] = a_s.data_ptr()
                    fbs.append(fb)
                with torch.cuda.stream(stream):
                    for i in range(max(reps, warm // 4)):
                        ctx.launch(fd, fbs[i % LAYERS], sh)
                    f0, f1, f2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
                    f0.record(stream)
                    for _ in range(reps):
                        ctx.rowscale(x.data_ptr(), a_s.data_ptr(), PM, k, sh)
                    f1.record(stream)
                    for i in range(reps):
                        ctx.launch(fd, fbs[i % LAYERS], sh)
                    f2.record(stream)
                torch.cuda.synchronize()
                pf[name]["fused_quant"] = dict(kernel=fd.kernel.decode(), rowscale_us=round(f0.elapsed_time(f1) * 1e3 / reps, 2),
                                               us=round(f1.elapsed_time(f2) * 1e3 / reps, 2))
            tot_ops += ops
            tot_us += us
            tot_q_us += q_us
            del x, q, a_s, c
        return pf, tot_ops, tot_us, tot_q_us

    if not args.no_prefill:
        pf, tot_ops, tot_us, tot_q_us = prefill_at(2048, 600, 60, fused_too=True)
        tops = tot_ops / tot_us / 1e6
        fq_us = sum(v["fused_quant"]["us"] + v["fused_quant"]["rowscale_us"] for v in pf.values())
        # what the matrix cores sustain on this card with such operands: the register-resident MFMA
        # loop of the probe object, fed zeros, codes like this workload's (small activations, 16*w
        # weights) and uniform random bytes. The card is power-bound under MFMA load, so the rate
        # depends on the operand values; the published peak is the denominator of `frac` regardless.
        probe = {}
        pblocks, piters = 512, 20000   # 9 ms a launch: four launches to settle the clock, four timed
        g = torch.Generator(device=dev)
        g.manual_seed(0)
        nbytes = pblocks * 256 * 128
        like = torch.empty(nbytes, dtype=torch.uint8, device=dev).view(pblocks * 256, 8, 16)
        like[:, :4] = torch.round(torch.randn((pblocks * 256, 4, 16), device=dev, generator=g) * 2.1).clamp(-127, 127).to(torch.int8).view(torch.uint8)
        like[:, 4:] = (torch.randint(0, 16, (pblocks * 256, 4, 16), device=dev, generator=g, dtype=torch.uint8) << 4)
        feeds = dict(zeros=torch.zeros(nbytes, dtype=torch.uint8, device=dev), workload_like=like.view(-1),
                     uniform=torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=dev, generator=g))
        pout = torch.zeros(16, dtype=torch.int32, device=dev)
        pd = iu8.describe_raw("iu8_probe_mfma32d", (pblocks, 1, 1), 256, n=piters)
        for tag, src in feeds.items():
            pb = dict(src=src.data_ptr(), out=pout.data_ptr())
            with torch.cuda.stream(stream):
                for _ in range(4):
                    ctx.launch(pd, pb, sh)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(4):
                    ctx.launch(pd, pb, sh)
                e1.record(stream)
            torch.cuda.synchronize()
            probe[tag] = round(4 * pblocks * 4 * piters * 16 * 65536.0 / (e0.elapsed_time(e1) * 1e3) / 1e6, 1)
        # a second reference point: the vendor library's plain int8 x int8 -> int32 GEMM (torch._int_mm) on the same
        # four shapes, operands distributed like this workload's already unpacked (no W4 unpack, no scaling, int32 out,
        # one warm weight matrix; the better of its two B orders) -- what a tuned library sustains on this card. It runs
        # as a child process (saber_engine_amd/library_ref.py): whatever the library does, this line is still printed.
        profiled = any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ) or "rocprof" in os.environ.get("LD_PRELOAD", "")
        try:
            import subprocess
            if args.no_library or profiled:   # no child process under a profiler's preloaded library
                raise RuntimeError("skipped (--no-library, or running under a profiler)")
            child = subprocess.run([sys.executable, "-m", "saber_engine_amd.library_ref", "2048"], cwd=ROOT, timeout=180,
                                   stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
            lib = json.loads(child.stdout.strip().splitlines()[-1]) if child.returncode == 0 else dict(error="exit %d" % child.returncode)
        except Exception as e:   # a side note, never the product path
            lib = dict(error=str(e)[:120])
        out["prefill_m2048"] = dict(value=round(tops, 1), unit="TOPS", library_int8_gemm=lib, with_quant=round(tot_ops / (tot_us + tot_q_us) / 1e6, 1),
                                    fused_quant=dict(tops=round(tot_ops / fq_us / 1e6, 1), vs_two_launch=round((tot_us + tot_q_us) / fq_us, 3),
                                                     note="row-scale pass + macaq_iu8_pfq_* (quantisation fused into the A-tile load), "
                                                          "per linear under per_linear.*.fused_quant; the launch law keeps producer + GEMM"),
                                    per_linear=pf, mfma_probe_tops=probe,
                                    frac_of_probe_workload_like=round(tops / probe["workload_like"], 4),
                                    roofline=dict(bound="mfma", achieved=round(tops / 1e3, 4), peak=INT8_PEAK_TOPS / 1e3,
                                                  unit="POP/s", frac=round(tops / INT8_PEAK_TOPS, 4), traffic=None,
                                                  note="GEMM launches alone over the four shapes (ops = 2*M*N*K); "
                                                       "with_quant adds the int8 producer launches"))
        # the other row counts of configs[2]: M = 256 sits near the ridge (both roofs reported: the weights'
        # GB/s beside the TOPS), M = 8192 is the matrix-bound end
        other = {}
        for PM, warm, reps in (() if args.no_other_m else ((256, 600, 60), (8192, 80, 12))):
            pfm, ops_m, us_m, q_us_m = prefill_at(PM, warm, reps)
            wbytes = sum(n * k // 2 for _, n, k in linears)
            other["m%d" % PM] = dict(tops=round(ops_m / us_m / 1e6, 1), with_quant=round(ops_m / (us_m + q_us_m) / 1e6, 1),
                                     weight_gbps=round(wbytes / us_m / 1e3, 1), mfma_frac=round(ops_m / us_m / 1e6 / INT8_PEAK_TOPS, 4),
                                     hbm_frac=round(wbytes / us_m / 1e3 / HBM_PEAK_GBPS, 4),
                                     per_linear={k_: dict(kernel=v["kernel"], us=v["us"], tops=v["tops"]) for k_, v in pfm.items()})
        out["prefill_other_m"] = other
    # ---- configs[3]: the 64-entry launch sequence with 19 int8-row linears among the int4 ones (output-side
    # projections), one HIP graph a sequence on shared per-token activations, every entry its own weights
    # (random codes generated on the device: parity of this sequence is the GPU tests' business)
    if not args.no_other_m:
        seq = synth.mixed_sequence()
        gen = torch.Generator(device=dev)
        gen.manual_seed(3)
        seq_w = []
        for _, n, k, w8 in seq:
            seq_w.append(torch.randint(0, 256, (n * k if w8 else n * k // 2,), dtype=torch.uint8, device=dev, generator=gen))
        mixed = {}
        for SM in (16, 2048):
            acts = {}
            for k in (5120, 17408):
                x = torch.from_numpy(synth.activations(np.random.default_rng(4), SM, k).view(np.int16)).to(dev)
                q = torch.zeros(iu8.a_bytes(SM, k), dtype=torch.uint8, device=dev)
                a_s = torch.zeros(SM, dtype=torch.float32, device=dev)
                ctx.quant(x.data_ptr(), q.data_ptr(), a_s.data_ptr(), SM, k, sh)
                acts[k] = (q, a_s)
            cbuf = {n: torch.zeros((SM, n), dtype=torch.int16, device=dev) for n in {e[1] for e in seq}}

            def run_seq():
                for (name, n, k, w8), w in zip(seq, seq_w):
                    d = iu8.resolve(iu8.W8 if w8 else iu8.W4, SM, n, k)
                    assert d.ks == 1
                    b = dict(a=acts[k][0].data_ptr(), w=w.data_ptr(), ws=dev_ws[name].data_ptr(), c=cbuf[n].data_ptr())
                    b["as"] = acts[k][1].data_ptr()
                    ctx.launch(d, b, sh)

            with torch.cuda.stream(stream):
                run_seq()
            stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                run_seq()
            reps = 60 if SM == 16 else 12
            with torch.cuda.stream(stream):
                for _ in range(reps // 2):   # sustained: tens of ms of the sequence before the timed replays
                    g.replay()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    g.replay()
                e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / reps
            wbytes = sum(n * k if w8 else n * k // 2 for _, n, k, w8 in seq)
            ops = sum(2.0 * SM * n * k for _, n, k, _ in seq)
            mixed["m%d" % SM] = dict(sequence_us=round(us, 1), launches=len(seq), w8_entries=sum(1 for e in seq if e[3]),
                                     weight_gbps=round(wbytes / us / 1e3, 1), tops=round(ops / us / 1e6, 1))
            del acts, cbuf, g
        out["mixed_w4_w8_sequence"] = mixed
        del seq_w

    # ---- the routed-expert layer of configs[4] (128 experts, top-8, hidden 4096, expert intermediate
    # 1536) as its launch train, T = 16 (weight streaming) and T = 4096 (MFMA); weights are random
    # nibbles generated on the device (parity of this path is the GPU tests' business)
    if not args.no_moe:
        from saber_engine_amd.moe import MoeLayerIU8

        E, topk, H, I = 128, 8, 4096, 1536
        g = torch.Generator(device=dev)
        g.manual_seed(0)
        wgu = torch.randint(0, 256, (E, 2 * I * H // 2), dtype=torch.uint8, device=dev, generator=g)
        wdn = torch.randint(0, 256, (E, H * I // 2), dtype=torch.uint8, device=dev, generator=g)
        wsgu = (torch.randn((E, 2 * I), device=dev, generator=g) * 0.02).abs() + 1e-4   # |N(0, 0.02)| + 1e-4
        wsdn = (torch.randn((E, H), device=dev, generator=g) * 0.02).abs() + 1e-4
        moe = {}
        for T in (16, 4096):
            layer = MoeLayerIU8(ctx, T, E, topk, H, I)
            layer.set_weights(wgu, wsgu, wdn, wsdn)
            x = torch.randn((T, H), device=dev, generator=g).to(torch.bfloat16).view(torch.int16)
            lg = torch.randn((T, E), device=dev, generator=g).to(torch.bfloat16).view(torch.int16)
            # a run long enough (0.2 s at T = 4096) to show the layer's own sustained rate, from an idle
            # card: straight after the dense prefill sections a short burst ran 15-20 % slower
            reps = 200
            torch.cuda.synchronize()
            time.sleep(1.0)
            with torch.cuda.stream(stream):
                for _ in range(20):
                    layer.forward(x, lg, sh)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    layer.forward(x, lg, sh)
                e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / reps
            live = int((layer.buf["expert_cnt"] > 0).sum().item())
            wbytes = live * (2 * I * H // 2 + H * I // 2 + 4 * (2 * I + H))
            ops = 2.0 * T * topk * (2 * I * H + H * I)
            moe["t%d" % T] = dict(layer_us=round(us, 1), launches=(4 if layer.fused_back else 5) + (1 if T > 128 and layer.tb != 1 else 0), tile_rows=16 * layer.tb, experts_touched=live,
                                  weight_gbps=round(wbytes / us / 1e3, 1), tops=round(ops / us / 1e6, 1),
                                  bound="hbm" if T == 16 else "mfma",
                                  frac=round((wbytes / us / 1e3) / HBM_PEAK_GBPS if T == 16 else (ops / us / 1e6) / INT8_PEAK_TOPS, 4))
            del layer, x, lg
        out["moe_e128_top8_h4096_i1536"] = moe
    # ---- the Hadamard-basis int8 producers that feed these GEMMs in the served model (memory-bound: a pass over
    # the bf16 rows in, the codes, scales and the new residual out), at decode and at prefill row counts
    if not args.no_producers:
        g = torch.Generator(device=dev)
        g.manual_seed(1)

        def bf16(*shape, scale=1.0):
            return (torch.randn(shape, device=dev, generator=g) * scale).to(torch.bfloat16).view(torch.int16)

        prod = {}
        for PM in (16, 2048):
            Kh, Ni, Ng, hd = 5120, 17408, 6144, 128
            t_k = (torch.randint(0, 2, (Ni,), device=dev, generator=g).float() * 2 - 1)
            q = torch.zeros(iu8.a_bytes(PM, Ni), dtype=torch.uint8, device=dev)
            sc = torch.zeros(PM, dtype=torch.float32, device=dev)
            xk, res, wk, ro = bf16(PM, Kh), bf16(PM, Kh, scale=4.0), bf16(Kh, scale=0.1), torch.zeros((PM, Kh), dtype=torch.int16, device=dev)
            gu = bf16(PM, 2 * Ni, scale=2.0)
            xg, zg, wg = bf16(PM, Ng, scale=2.0), bf16(PM, Ng, scale=3.0), bf16(hd)
            core, blk = bf16(PM, Kh), bf16(PM, 2 * Kh, scale=3.0)
            silu_lut = torch.zeros(65536, dtype=torch.int16, device=dev)
            ctx.silu_table(silu_lut.data_ptr(), sh)
            sig_lut = torch.zeros(65536, dtype=torch.int16, device=dev)
            ctx.sigmoid_table(sig_lut.data_ptr(), sh)
            cases = {
                "quant_had_k5120": (lambda: ctx.quant_had(xk.data_ptr(), q.data_ptr(), sc.data_ptr(), PM, Kh, t_k.data_ptr(), sh),
                                    PM * (3 * Kh + 4)),
                "add_rms_quant_had_k5120": (lambda: ctx.add_rms_quant_had(xk.data_ptr(), res.data_ptr(), wk.data_ptr(), q.data_ptr(), sc.data_ptr(),
                                                                          ro.data_ptr(), PM, Kh, 1e-6, t_k.data_ptr(), sh),
                                            PM * (7 * Kh + 4) + 2 * Kh),
                "silu_mul_quant_had_n17408": (lambda: ctx.silu_mul_quant_had(gu.data_ptr(), q.data_ptr(), sc.data_ptr(), PM, Ni, t_k.data_ptr(), sh),
                                              PM * (5 * Ni + 4)),
                "silu_mul_quant_had_lut_n17408": (lambda: ctx.silu_mul_quant_had_lut(gu.data_ptr(), q.data_ptr(), sc.data_ptr(), PM, Ni, t_k.data_ptr(),
                                                                                     silu_lut.data_ptr(), sh),
                                                  PM * (5 * Ni + 4)),
                "gdn_norm_quant_had_n6144": (lambda: ctx.gdn_norm_quant_had(xg.data_ptr(), zg.data_ptr(), Ng, wg.data_ptr(), q.data_ptr(), sc.data_ptr(),
                                                                            PM, Ng, 1e-6, t_k.data_ptr(), sh),
                                             PM * (5 * Ng + 4)),
                "attn_gate_quant_had_lut_n5120": (lambda: ctx.attn_gate_quant_had_lut(core.data_ptr(), blk.data_ptr(), q.data_ptr(), sc.data_ptr(), PM,
                                                                                      Kh, hd, 2 * Kh, t_k.data_ptr(), sig_lut.data_ptr(), sh),
                                                  PM * (5 * Kh + 4)),
                "attn_gate_quant_had_n5120": (lambda: ctx.attn_gate_quant_had(core.data_ptr(), blk.data_ptr(), q.data_ptr(), sc.data_ptr(), PM, Kh, hd,
                                                                              2 * Kh, t_k.data_ptr(), sh),
                                              PM * (5 * Kh + 4)),
            }
            row = {}
            for name, (fn, nbytes) in cases.items():
                reps = 100 if PM <= 16 else 40
                with torch.cuda.stream(stream):
                    for _ in range(4):
                        fn()
                stream.synchronize()
                gp = torch.cuda.CUDAGraph()      # a graph: eager launches of a few microseconds are bound by the host's launch rate
                with torch.cuda.graph(gp, stream=stream):
                    for _ in range(reps):
                        fn()
                with torch.cuda.stream(stream):
                    gp.replay()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(stream)
                    gp.replay()
                    e1.record(stream)
                torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 1e3 / reps
                del gp
                row[name] = dict(us=round(us, 2), bytes=int(nbytes), gbps=round(nbytes / us / 1e3, 1), hbm_frac=round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4))
            prod["m%d" % PM] = row
        prod["note"] = ("one launch a producer, back to back in a replayed graph (inputs of the decode rows stay in the caches: those lines are launch latency, "
                        "not bandwidth); bytes = bf16 rows in + codes + scales (+ the residual row out); *_lut = the same op with the caller's table of its gate at hand")
        out["hadamard_producers"] = prod
    print(json.dumps(out), flush=True)
    ctx.close()


if __name__ == "__main__":
    main()
