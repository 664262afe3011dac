#!/usr/bin/env python3
"""Benchmark of the bfAintBGemm hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sweep] [--no-cpu]
    python bench.py --scan [narrow]   (a map of kernel times over shapes and m, not the benchmark)

A step is one GEMM launch through the C ABI on synthetic, seeded inputs already resident in HBM.
The headline workload is the decode shape the metric is quoted on (bf16 A [1,4096] x int8 B
[4096,4096], per-channel bf16 scales); the prefill shape (M = 4096) is measured in the same run and
reported under "extra".  The metric definitions follow the reference driver's printout
(/root/reference/bfAintBGemm/bfAintBGemm.cc:186-195: flops = 2mnk, bytes = 2(mk+mn) + nk) with two
corrections stated in the output: decimal units, and the scale bytes are counted.

Timing: W untimed warm-up launches, then exactly K launches recorded into one HIP graph; the graph is
replayed five times, each replay between its own pair of events on the launch stream (and a host
clock, after/before a device synchronize), and the median replay is reported.  The graph keeps host launch overhead out of a microsecond-scale kernel's
measurement; the reference's own protocol is the same minus the graph (10 launches in one event pair,
bfAintBGemm.cc:171-186).  For the decode shape consecutive launches read DIFFERENT copies of B
(enough copies to exceed the 256 MB last-level cache), so the figure is an HBM figure; the
same-buffer ("hot") figure is reported beside it.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
LLC_BYTES = 256 << 20
REPLAYS = 5                   # timed replays of the K-launch graph; the median one is reported

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch,
# scaled by the same counters on a copy kernel of known size); see profiles/*.txt for the runs.
MEASURED_TRAFFIC_BYTES = {
    # fetch 8392.5 KiB x 1.997 + write 232.0 KiB (plain launches; profiles/bench_pmc_fetch_size.txt, bench_pmc_write_size.txt)
    "decode_m1_n4096_k4096_int8_perchannel": 17398385,
    # fetch 65698.5 KiB x 1.997 + write 32768.0 KiB (plain launches)
    "prefill_m4096_n4096_k4096_int8_perchannel": 167893415,
    # the same shapes through bfaintb_gemm_prepacked: fetch 8273.0 KiB x 1.997 + write 8.0 KiB; fetch 65712.0 KiB x 1.997 + write 32768.0 KiB
    "decode_m1_n4096_k4096_int8_perchannel_prepacked": 16924658,
    "prefill_m4096_n4096_k4096_int8_perchannel_prepacked": 167921020,
}


def algorithmic_bytes(m, n, k, bits, group):
    groups = k // group if group else 1
    return 2 * m * k + k * n * bits // 8 + 2 * groups * n + 2 * m * n


class Workload:
    def __init__(self, name, m, n, k, bits=8, group=0, seed=0, copies=None):
        import torch
        self.name, self.m, self.n, self.k, self.bits, self.group = name, m, n, k, bits, group
        rng = np.random.Generator(np.random.PCG64(seed))
        self.a_f32 = rng.standard_normal((m, k), dtype=np.float32)
        lo, hi = (-128, 128) if bits == 8 else (-8, 8)
        self.q = rng.integers(lo, hi, size=(k, n), dtype=np.int8)
        groups = k // group if group else 1
        self.s_f32 = rng.uniform(0.001, 0.01 if bits == 8 else 0.02, size=(groups, n)).astype(np.float32)
        if bits == 8:
            b_host = (self.q.astype(np.int16) + 128).astype(np.uint8)          # excess-128 (mem_transfer.hpp:30)
        else:
            u = (self.q.astype(np.int16) + 8).astype(np.uint8)
            b_host = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)         # excess-8, even column in the low nibble
        self.a = torch.from_numpy(self.a_f32).cuda().to(torch.bfloat16)
        self.s = torch.from_numpy(self.s_f32).cuda().to(torch.bfloat16)
        b0 = torch.from_numpy(b_host).cuda()
        if copies is None:
            copies = 1
        self.b = [b0] + [b0.clone() for _ in range(copies - 1)]
        self.c = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        self.bytes = algorithmic_bytes(m, n, k, bits, group)
        self.flops = 2 * m * n * k

    def workspace(self, af):
        import torch
        need = af.workspace_bytes(self.m, self.n, self.k, self.bits, self.group)
        if not need:
            return None
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        af.workspace_init(ws)
        return ws


def time_graph(af, w, steps, warmup, rotate, packed=False):
    """Returns (event_ms_per_step, wall_ms_per_step).  packed: every copy of B is reordered once (untimed, as a model
    loader would) and the launches go through bfaintb_gemm_prepacked."""
    import torch
    ws = w.workspace(af)
    nb = len(w.b) if rotate else 1
    if packed:
        need = af.prepacked_workspace_bytes(w.m, w.n, w.k, w.bits, w.group)
        pws = None
        if need:
            pws = torch.empty(need, dtype=torch.uint8, device="cuda")
            af.workspace_init(pws)
        pks = []
        for i in range(nb):
            pk = torch.empty(af.prepack_bytes(w.n, w.k, w.bits), dtype=torch.uint8, device="cuda")
            af.prepack(pk, w.b[i], w.n, w.k, weight_bits=w.bits)
            pks.append(pk)

    def launch(i):
        if packed:
            af.gemm_prepacked(w.c, w.a, pks[i % nb], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=pws)
        else:
            af.gemm(w.c, w.a, w.b[i % nb], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=ws)

    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(steps):
            launch(i)
    g.replay()  # untimed: first replay pays graph upload
    torch.cuda.synchronize()
    ev, wall = [], []
    for _ in range(REPLAYS):  # each replay is exactly `steps` launches inside one event pair; the median replay is reported
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ev.append(e0.elapsed_time(e1) / steps)
        wall.append((t1 - t0) * 1e3 / steps)
    mid = sorted(range(REPLAYS), key=lambda i: ev[i])[REPLAYS // 2]
    return ev[mid], wall[mid]


def time_fused_epilogue(af, w, steps, warmup):
    """(fused_ms, unfused_ms): C = A.W + bias + residual in one launch (bfaintb_gemm_fused), against the plain GEMM
    followed by torch's elementwise bias and residual additions on the bf16 output (two more passes over C)."""
    import torch
    ws = w.workspace(af)
    bias = torch.randn(w.n, device="cuda").to(torch.bfloat16)
    res = torch.randn((w.m, w.n), device="cuda").to(torch.bfloat16)

    def fused(i):
        af.gemm(w.c, w.a, w.b[i % len(w.b)], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=ws, bias=bias, residual=res)

    def unfused(i):
        af.gemm(w.c, w.a, w.b[i % len(w.b)], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=ws)
        w.c.add_(bias).add_(res)

    out = []
    for launch in (fused, unfused):
        for i in range(warmup):
            launch(i)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(steps):
                launch(i)
        g.replay()
        torch.cuda.synchronize()
        ev = []
        for _ in range(REPLAYS):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            ev.append(e0.elapsed_time(e1) / steps)
        out.append(sorted(ev)[REPLAYS // 2])
    return out[0], out[1]


def time_gated(af, w, steps, warmup, packed):
    """(fused_ms, unfused_ms) for silu(A.Wg) * (A.Wu) with interleaved (gate, up) columns in w: one launch with the
    SiLU-gate epilogue, against the plain GEMM followed by torch's silu and multiply on the strided halves."""
    import torch
    ws = w.workspace(af)
    nb = len(w.b)
    out = torch.zeros((w.m, w.n // 2), dtype=torch.bfloat16, device="cuda")
    if packed:
        pks = []
        for i in range(nb):
            pk = torch.empty(af.prepack_bytes(w.n, w.k, w.bits), dtype=torch.uint8, device="cuda")
            af.prepack(pk, w.b[i], w.n, w.k, weight_bits=w.bits)
            pks.append(pk)
        need = af.prepacked_workspace_bytes(w.m, w.n, w.k, w.bits, w.group)
        pws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        af.workspace_init(pws)

    def plain(i, c, act):
        if packed:
            af.gemm_prepacked(c, w.a, pks[i % nb], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=pws, activation=act)
        else:
            af.gemm(c, w.a, w.b[i % nb], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=ws, activation=act)

    def fused(i):
        plain(i, out, af.ACT_SILU_GATE)

    def unfused(i):
        plain(i, w.c, af.ACT_NONE)
        torch.mul(torch.nn.functional.silu(w.c[:, 0::2]), w.c[:, 1::2], out=out)

    res = []
    for launch in (fused, unfused):
        for i in range(warmup):
            launch(i)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for i in range(steps):
                launch(i)
        g.replay()
        torch.cuda.synchronize()
        ev = []
        for _ in range(REPLAYS):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize()
            ev.append(e0.elapsed_time(e1) / steps)
        res.append(sorted(ev)[REPLAYS // 2])
    return res[0], res[1]


def time_read_ceiling(af, w, steps, warmup):
    """The same rotation of B copies through a kernel that only fetches the bytes."""
    import torch
    nb = len(w.b)
    for i in range(warmup):
        af.probe_read(w.b[i % nb])
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(steps):
            af.probe_read(w.b[i % nb])
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def time_vendor_bf16_gemm(w, steps, warmup):
    """Context for the prefill figure: the vendor library's plain bf16 x bf16 GEMM (torch.matmul, i.e.
    hipBLASLt) on the same activations and the already dequantised weights, same graph protocol.  It does
    none of the dequantisation work; it shows what a tuned MFMA kernel sustains on this machine at this shape."""
    import torch
    wq = torch.from_numpy(w.q.astype(np.float32)).cuda()
    wb = (wq * w.s.float()[0][None, :]).to(torch.bfloat16)
    del wq
    out = torch.empty((w.m, w.n), dtype=torch.bfloat16, device="cuda")
    for _ in range(warmup):
        torch.matmul(w.a, wb, out=out)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(steps):
            torch.matmul(w.a, wb, out=out)
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def time_eager(af, w, steps, warmup):
    """The reference protocol: launches in a loop inside one event pair, no graph."""
    import torch
    ws = w.workspace(af)
    for i in range(warmup):
        af.gemm(w.c, w.a, w.b[0], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=ws)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for i in range(steps):
        af.gemm(w.c, w.a, w.b[0], w.s, w.m, w.n, w.k, weight_bits=w.bits, group_size=w.group, workspace=ws)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def roofline_entry(w, ms, bound, suffix=""):
    if bound == "hbm":
        achieved = w.bytes / (ms * 1e-3) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = w.flops / (ms * 1e-3) / 1e12
        peak, unit = MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"
    return {"bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit, "frac": round(achieved / peak, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(w.name + suffix), "kernel_us": round(ms * 1e3, 3),
            "algorithmic_bytes": w.bytes, "flops": w.flops}


SCAN_SHAPES = [(4096, 4096), (11008, 4096), (4096, 11008), (8192, 8192), (28672, 8192), (2048, 8192), (32000, 4096)]   # (n, k)
SCAN_SHAPES_NARROW = [(1024, 4096), (1024, 8192), (512, 4096), (2048, 4096), (1536, 8960), (256, 7168), (1024, 16384)]
SCAN_M = [1, 4, 8, 16, 24, 32, 48, 64, 128, 256, 512, 1024, 2048]


def scan(shapes=None):
    """Kernel time of bfaintb_gemm and bfaintb_gemm_prepacked, variant left to the library, over shapes x {8-bit per
    channel, 4-bit group 128} x SCAN_M.  Up to 32 rows of A the launches rotate over copies of B that exceed the last-level
    cache (the decode protocol of the headline figure); beyond, two copies.  Not a roofline statement: a map to read
    anomalies from (a time that falls as m grows, a weight order that loses to the other)."""
    import torch
    import awesome_fusion_amd as af
    af.lib()
    for (n, k) in (SCAN_SHAPES if shapes is None else shapes):
        for (bits, group) in ((8, 0), (4, 128)):
            row = {"n": n, "k": k, "weight_bits": bits, "group_size": group, "m": SCAN_M, "row_major_us": [], "prepacked_us": []}
            for m in SCAN_M:
                b_bytes = n * k * bits // 8
                copies = max(2, min(40, (640 << 20) // b_bytes)) if m <= 32 else 2
                w = Workload(f"scan_m{m}_n{n}_k{k}_b{bits}", m, n, k, bits, group, copies=copies)
                steps = 100 if m <= 64 else 20
                for packed in (False, True):
                    ev_ms, _ = time_graph(af, w, steps, 5, rotate=True, packed=packed)
                    row["prepacked_us" if packed else "row_major_us"].append(round(ev_ms * 1e3, 2))
                del w
                torch.cuda.empty_cache()
            print(json.dumps(row), flush=True)


def cpu_baseline(w, c_gpu_f32, budget_s=12.0):
    """host_ref.hpp's gemm_rrr timed on this machine's cores on the same inputs the GPU consumed:
    the reference's own compiled routine when the wrapper library is present, else the C port."""
    import ctypes as C
    from concurrent.futures import ThreadPoolExecutor
    import oracle
    import torch
    fp = C.POINTER(C.c_float)
    a = w.a.float().cpu().numpy()                       # the bf16 activations, widened
    s = w.s.float().cpu().numpy()[0].copy()             # the bf16 scales, widened (per-channel workloads)
    b = w.q.astype(np.float32)
    m, n, k = w.m, w.n, w.k
    if oracle.have_ref():
        fn, kind = oracle.ref().ref_gemm_rrr, "reference"
    else:
        fn, kind = oracle.lib.orc_gemm_rrr, "port"
    c = np.zeros((m, n), np.float32)

    def call(n0, nb):
        fn(C.cast(c.ctypes.data + 4 * n0, fp), a.ctypes.data_as(fp), C.cast(b.ctypes.data + 4 * n0, fp),
           C.cast(s.ctypes.data + 4 * n0, fp), m, nb, k, k, n, n)

    # 1 thread, the way the reference runs it
    reps, t0 = 0, time.perf_counter()
    while True:
        call(0, n)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s * 0.6 or reps >= 50:
            break
    t1 = el / reps
    c_single = c.copy()
    # all cores: columns split over threads, each output still one sequential-K fp32 sum
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    blk = max(16, (n // (cores * 4)) // 16 * 16)
    jobs = [(n0, min(blk, n - n0)) for n0 in range(0, n, blk)]
    with ThreadPoolExecutor(max_workers=cores) as ex:
        reps2, t0 = 0, time.perf_counter()
        while True:
            list(ex.map(lambda j: call(*j), jobs))
            reps2 += 1
            el = time.perf_counter() - t0
            if el > budget_s * 0.4 or reps2 >= 200:
                break
    tn = el / reps2
    assert np.array_equal(c.view(np.uint32), c_single.view(np.uint32)), "threaded CPU baseline changed the result"
    d = c_gpu_f32 - c
    nrms = float(np.sqrt((d.astype(np.float64) ** 2).sum() / (2.0 * (c.astype(np.float64) ** 2).sum())))
    unit_val = lambda t: w.bytes / t / 1e9
    return ({"value": round(unit_val(t1), 4), "unit": "GB/s", "cores": 1, "kind": kind,
             "sample": f"full {w.name} problem x{reps} repetitions ({el and t1 * reps:.1f} s), gemm_rrr on float inputs",
             "gflops": round(w.flops / t1 / 1e9, 3), "ms_per_step": round(t1 * 1e3, 3)},
            {"value": round(unit_val(tn), 4), "unit": "GB/s", "cores": cores, "kind": kind,
             "sample": f"full {w.name} problem x{reps2} repetitions, columns split over {cores} threads",
             "gflops": round(w.flops / tn / 1e9, 3), "ms_per_step": round(tn * 1e3, 3)},
            nrms)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--sweep", action="store_true", help="also time the secondary shapes (decode sweep, int4 group-128)")
    ap.add_argument("--scan", nargs="?", const="llm", default="", choices=["llm", "narrow"],
                    help="instead of the benchmark: what the library's own choice of kernel takes over a grid of "
                    "matrix shapes, code widths and m, row-major and pre-packed weights; one JSON line per matrix "
                    "(llm: projection and MLP shapes of 7B..70B models; narrow: 256..2048 columns, the key/value "
                    "projections of grouped-query attention)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="time only this workload family: decode | prefill | decode_cold | decode_packed_cold "
                    "(decode_cold: nothing but the headline's cold-B launches, for a kernel trace without the hot and eager variants; "
                    "decode_packed_cold: the same launches over pre-packed weights)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the GEMM would shard over the columns "
              "of B with no exchange between GPUs).  Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if args.scan:
        scan(SCAN_SHAPES_NARROW if args.scan == "narrow" else SCAN_SHAPES)
        return

    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    import awesome_fusion_amd as af
    af.lib()

    K, W = args.steps, args.warmup
    out_extra = {}

    # ---- headline: decode M=1, N=K=4096, int8 per-channel; cold B (rotating copies > last-level cache)
    res = None
    cold_only = args.only in ("decode_cold", "decode_packed_cold")
    if args.only in ("", "decode", "decode_cold", "decode_packed_cold"):
        copies = LLC_BYTES * 2 // (4096 * 4096) + 8  # 40 copies = 640 MiB
        w = Workload("decode_m1_n4096_k4096_int8_perchannel", 1, 4096, 4096, copies=copies)
        ev_ms, wall_ms = time_graph(af, w, K, W, rotate=True, packed=args.only == "decode_packed_cold")
        if args.only == "decode_packed_cold":
            w.name += "_prepacked"
        hot_ms, _ = (ev_ms, wall_ms) if cold_only else time_graph(af, w, K, W, rotate=False)
        eager_ms = ev_ms if cold_only else time_eager(af, w, K, W)
        read_ms = ev_ms if cold_only else time_read_ceiling(af, w, K, W)
        c_gpu = w.c.float().cpu().numpy()
        res = {
            "metric": "bfAintBGemm bf16 x int8 GEMM, N=K=4096, M=1: effective HBM bandwidth (algorithmic bytes / time per launch, B cold)",
            "value": round(w.bytes / (wall_ms * 1e-3) / 1e9, 3), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
            "ms_per_step": round(wall_ms, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16", "data": "synthetic",
            "config": {"workload": w.name, "m": 1, "n": 4096, "k": 4096, "weight_bits": 8, "group_size": 0,
                       "b_copies_rotated": copies, "split_k": af.split_k(1, 4096, 4096), "launch": "hip graph of K launches, median of 5 replays",
                       "units": "decimal; scale bytes counted"},
            "roofline": roofline_entry(w, ev_ms, "hbm"),
        }
        res["tflops"] = round(w.flops / (wall_ms * 1e-3) / 1e12, 4)
        b_bytes = w.b[0].numel()
        if not cold_only:
            res["roofline"]["fetch_only_kernel_us"] = round(read_ms * 1e3, 3)
            res["roofline"]["fetch_only_GBps"] = round(b_bytes / read_ms / 1e6, 1)
            res["roofline"]["frac_of_fetch_only"] = round(read_ms / ev_ms, 4)
            out_extra["decode_m1_hot_same_buffer"] = {"kernel_us": round(hot_ms * 1e3, 3), "GB/s": round(w.bytes / hot_ms / 1e6, 1),
                                                      "note": "B re-read from cache: not an HBM figure"}
            out_extra["decode_m1_eager_launch_loop"] = {"us_per_launch": round(eager_ms * 1e3, 3),
                                                        "note": "reference protocol (no graph): host launch rate included"}
            f_ms, u_ms = time_fused_epilogue(af, w, K, W)
            out_extra["decode_m1_bias_residual"] = {"fused_kernel_us": round(f_ms * 1e3, 3), "gemm_then_two_elementwise_us": round(u_ms * 1e3, 3),
                                                    "note": "C = A.W + bias + residual: one bfaintb_gemm_fused launch against bfaintb_gemm + torch add_ x2"}
            pk_ms, _ = time_graph(af, w, K, W, rotate=True, packed=True)
            out_extra["decode_m1_prepacked"] = {
                **roofline_entry(w, pk_ms, "hbm", "_prepacked"), "frac_of_fetch_only": round(read_ms / pk_ms, 4),
                "note": "same shape and cold-B rotation through bfaintb_gemm_prepacked (weights reordered once, offline): "
                        "no split-K, no workspace; not the drop-in row-major path, so not `value`"}
        if not args.no_cpu and not cold_only:
            one, allc, nrms = cpu_baseline(w, c_gpu)
            res["cpu_baseline"] = one
            out_extra["cpu_baseline_all_cores"] = allc
            out_extra["gpu_vs_cpu_nrms"] = round(nrms, 6)
        del w
        torch.cuda.empty_cache()

    # ---- prefill M=4096, N=K=4096
    if args.only in ("", "prefill"):
        w = Workload("prefill_m4096_n4096_k4096_int8_perchannel", 4096, 4096, 4096, copies=2)
        pk = max(20, min(K, 100))
        ev_ms, wall_ms = time_graph(af, w, pk, max(5, W // 4), rotate=True)
        entry = {"value": round(w.flops / (wall_ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "steps": pk,
                 "ms_per_step": round(wall_ms, 6), "GB/s": round(w.bytes / (wall_ms * 1e-3) / 1e9, 1),
                 "config": {"workload": w.name}, "roofline": roofline_entry(w, ev_ms, "mfma")}
        try:
            v_ms = time_vendor_bf16_gemm(w, pk, 5)
            entry["vendor_bf16_gemm_same_shape"] = {"TFLOP/s": round(w.flops / (v_ms * 1e-3) / 1e12, 2), "kernel_us": round(v_ms * 1e3, 3),
                                                    "note": "torch.matmul bf16 x bf16 on pre-dequantised weights (no dequantisation work): context, not a baseline"}
        except Exception as exc:  # context only
            entry["vendor_bf16_gemm_same_shape"] = {"error": str(exc)[:200]}
        f_ms, u_ms = time_fused_epilogue(af, w, pk, max(5, W // 4))
        entry["bias_residual"] = {"fused_kernel_us": round(f_ms * 1e3, 3), "gemm_then_two_elementwise_us": round(u_ms * 1e3, 3),
                                  "note": "C = A.W + bias + residual: one bfaintb_gemm_fused launch against bfaintb_gemm + torch add_ x2"}
        pk_ms, _ = time_graph(af, w, pk, max(5, W // 4), rotate=True, packed=True)
        entry["prepacked"] = {**roofline_entry(w, pk_ms, "mfma", "_prepacked"), "note": "bfaintb_gemm_prepacked, same shape"}
        out_extra["prefill_m4096"] = entry
        if res is None:
            res = {"metric": "bfAintBGemm bf16 x int8 GEMM, N=K=4096, M=4096: TFLOP/s", "value": entry["value"], "unit": "TFLOP/s",
                   "n_gpus": 1, "steps": pk, "warmup": W, "ms_per_step": entry["ms_per_step"], "higher_is_better": True,
                   "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                   "config": entry["config"], "roofline": entry["roofline"]}
        del w
        torch.cuda.empty_cache()

    if args.sweep:
        sweep = []
        for m in (1, 4, 8, 16, 32):
            w = Workload(f"decode_m{m}_n11008_k4096_int8_perchannel", m, 11008, 4096, copies=14)
            ev_ms, _ = time_graph(af, w, min(K, 200), W, rotate=True)
            sweep.append({"workload": w.name, **roofline_entry(w, ev_ms, "hbm")})
            if m <= 8:
                pk_ms, _ = time_graph(af, w, min(K, 200), W, rotate=True, packed=True)
                sweep.append({"workload": w.name + "_prepacked", **roofline_entry(w, pk_ms, "hbm")})
            del w
            torch.cuda.empty_cache()
        for m in (1, 16, 2048):
            w = Workload(f"m{m}_n28672_k8192_int4_group128", m, 28672, 8192, bits=4, group=128, copies=6 if m <= 32 else 1)
            ev_ms, _ = time_graph(af, w, min(K, 100) if m <= 32 else 10, min(W, 10), rotate=True)
            sweep.append({"workload": w.name, **roofline_entry(w, ev_ms, "hbm" if m <= 32 else "mfma")})
            if m == 1:
                pk_ms, _ = time_graph(af, w, min(K, 100), min(W, 10), rotate=True, packed=True)
                sweep.append({"workload": w.name + "_prepacked", **roofline_entry(w, pk_ms, "hbm")})
            del w
            torch.cuda.empty_cache()
        # between decode and prefill: what AUTO picks for a few hundred rows of A (row-blocked decode family, then 128x128 tiles)
        for m in (64, 256, 640, 1024):
            w = Workload(f"mid_m{m}_n4096_k4096_int8_perchannel", m, 4096, 4096, copies=4)
            ev_ms, _ = time_graph(af, w, min(K, 100), min(W, 10), rotate=True)
            v = af.variant(m, 4096, 4096)
            sweep.append({"workload": w.name, **roofline_entry(w, ev_ms, "mfma"),
                          "kernel": "row-blocked decode family" if v == af.DECODE else f"tiled, {af.prefill_tile(m, 4096)}x{af.prefill_tile(m, 4096)} tiles"})
            del w
            torch.cuda.empty_cache()
        # gated MLP, LLaMA-7B shape: 2 x 11008 interleaved (gate, up) columns over k = 4096
        for m in (1, 2048):
            w = Workload(f"gated_mlp_m{m}_n22016_k4096_int8_perchannel", m, 22016, 4096, copies=8 if m == 1 else 1)
            for packed in (False, True):
                f_ms, u_ms = time_gated(af, w, min(K, 100) if m == 1 else 10, min(W, 10), packed)
                sweep.append({"workload": w.name + ("_prepacked" if packed else ""), "fused_kernel_us": round(f_ms * 1e3, 3),
                              "gemm_then_silu_mul_us": round(u_ms * 1e3, 3),
                              "note": "silu(A.Wgate) * (A.Wup): one launch with the SiLU-gate epilogue against GEMM + torch silu, mul"})
            del w
            torch.cuda.empty_cache()
        out_extra["sweep"] = sweep

    res["extra"] = out_extra
    print(json.dumps(res))


if __name__ == "__main__":
    main()
