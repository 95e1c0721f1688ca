#!/usr/bin/env python3
"""bench.py --gpus 1 --steps K --warmup W  ->  one JSON line.

Workload (N=1): benchmark config 1 at M=1 — the 4-bit group-quantized decode GEMV
  x bf16 [1,4096] ~N(0,1);  W int4 [14336,4096] packed 2 per byte, group 32 along K, fp16 scale per group
  ~LogNormal(-5,0.5), zero-point 8;  y fp32 [1,14336].
A step is one GEMV launch through the C ABI (chadq_gemv_i4g32).  Weights are resident in HBM before the timed
region.  Steps rotate over 12 distinct copies of the weights (396 MB) so that the 256 MB last-level cache
cannot serve the stream; the same-buffer ("hot") rate is reported on the side.  Launches are replayed from HIP
graphs so that Python's per-call cost is not what is measured.

value = algorithmic bytes per launch / average launch duration (HIP events on the launch stream over the
timed K steps) = the same quantity as roofline.achieved.  Extras: M=4 and M=8, the int8 per-row GEMV
(config 0), the prefill dequant-GEMM (config 2, int4 and int8) in TFLOP/s, the mixture-of-experts FFN (config 3)
and the Gemma-2B-shaped decode step (config 4) in tokens/s.  cpu_baseline times this build's
numpy oracle (dequantise to fp32, then sgemv) on the host cores: the reference snapshot has no implementation
of this path, so there is no reference number to put beside it.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16
N_COPIES = 12
SEG = 48                     # launches per captured graph
DEC_STEPS = 1                 # decode steps per captured graph (config 4): several per graph save nothing in a queue of replays


def profile_figures():
    """(HBM bytes per launch of the headline kernel from hardware counters, the kernel's name) as the committed
    profile summaries state them: profiles/gemv_i4g32_m1_config1_hbm_traffic.txt carries a line
    `roofline.traffic = <bytes>` and a table row naming the kernel.  Whoever refreshes the counter runs edits those
    two lines and nothing here; (None, None) if the summary is missing."""
    import re

    path = os.path.join(ROOT, "profiles", "gemv_i4g32_m1_config1_hbm_traffic.txt")
    try:
        text = open(path).read()
    except OSError:
        return None, None
    t = re.search(r"^roofline\.traffic\s*=\s*([0-9,]+)", text, re.M)
    k = re.search(r"^roofline\.kernel\s*=\s*(\S+)", text, re.M)
    return (int(t.group(1).replace(",", "")) if t else None), (k.group(1) if k else None)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=960)
    ap.add_argument("--warmup", type=int, default=96)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the side measurements")
    ap.add_argument("--extras", default="gemv,int8,gemm,moe,decode",
                    help="comma list of the side measurements to run (gemv, int8, gemm, moe, decode; moe_ablation adds, "
                         "to moe, the tile-order call on the two measurement builds of the expert GEMM; gemm_ablation "
                         "adds, to gemm, config 2 on the build without dequantisation)")
    ap.add_argument("--short", action="store_true",
                    help="few launches per side measurement: for hardware-counter runs, which serialise every dispatch")
    ap.add_argument("--settle-ms", type=float, default=40.0,
                    help="run each measured workload for this long, untimed, right before its warm-up steps (0: not at all)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run three 256 MiB device copies before the timed region: a kernel of known traffic "
                         "that hardware-counter runs scale FETCH_SIZE / WRITE_SIZE by")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (no collectives are part of it)" % args.gpus,
              file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from chadslab_amd import QWeightInt4G32, QWeightInt8, _lib, ops

    _lib.load()  # fails loudly if libchadq.so is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = "cuda:0"
    torch.cuda.set_device(0)
    stream = torch.cuda.Stream()

    def bits(t):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)

    COVER = 24  # untimed launches queued in front of the start event (see run_direct)

    def settle(fn, per_call=1):
        """Runs the workload about to be measured for --settle-ms without a pause, untimed, in front of its warm-up
        steps.  A GPU coming out of idle goes through a transient of some ten milliseconds (fast at first, then slower
        than it will be, then steady), and the W warm-up steps of a 7 us kernel end inside it; the figures reported
        are those of the steady state a decode loop runs in.  The headline's figure without this phase is reported
        beside it.  fn(i) is called until the time is up; per_call = steps per call (a replayed graph)."""
        if args.settle_ms <= 0:
            return
        t_end = time.perf_counter() + args.settle_ms * 1e-3
        i = 0
        while time.perf_counter() < t_end:
            for _ in range(32):
                fn(i)
                i += per_call
            if i % (32 * 64 * per_call) == 0:
                torch.cuda.synchronize()  # bounds the backlog: the host may be faster than the GPU

    def run_direct(fn, steps, warmup, do_settle=True):
        """The steps as plain launches on the stream, one call of fn per step, back to back: `warmup` untimed steps, a
        synchronize, then COVER more untimed steps that are already queued when the start event is recorded - the timed
        steps are submitted while the GPU is still busy, so the cost of getting a first launch to an idle GPU is not
        spread over them, however few they are - then exactly `steps` timed steps between two events on the launch stream.
        Valid only while the host stays ahead of the GPU: returns None when its time per launch is not well below the
        GPU's time per step (the caller then measures the same steps replayed from a captured graph)."""
        with torch.cuda.stream(stream):
            if do_settle:
                settle(fn)
            for i in range(max(1, warmup)):
                fn(i)
            torch.cuda.synchronize()
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            for i in range(COVER):
                fn(i)
            a.record(stream)
            t0 = time.perf_counter()
            for i in range(steps):
                fn(COVER + i)
            t1 = time.perf_counter()
            b.record(stream)
            torch.cuda.synchronize()
        us, host = a.elapsed_time(b) * 1000.0 / steps, (t1 - t0) * 1e6 / steps
        return (us, host, 0) if host < 0.75 * us else None

    def run_steps(fn, steps, warmup, direct=False, do_settle=True):
        """fn(i) launches step i on the current stream.  Returns (us per step from HIP events, wall us per step,
        launches per replayed graph - 0 for plain stream launches).  direct: try run_direct first.  Graph form: the start
        event is recorded behind untimed replays (about 4 * COVER steps) that are already queued, for the reason given
        in run_direct."""
        if direct:
            res = run_direct(fn, steps, warmup, do_settle)
            if res is not None:
                return res
        seg = min(SEG, steps)
        with torch.cuda.stream(stream):
            graphs = {}
            for length in sorted({seg, steps % seg} - {0}):
                for i in range(length):
                    fn(i)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    for i in range(length):
                        fn(i)
                graphs[length] = g
            full, rem = divmod(steps, seg)
            if do_settle:
                settle(lambda i: graphs[seg].replay(), seg)
            for _ in range(max(1, warmup // seg)):
                graphs[seg].replay()
            torch.cuda.synchronize()
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            n_cover = (4 * COVER + seg - 1) // seg  # untimed replays that keep the GPU busy while the timed ones are submitted
            for _ in range(n_cover):
                graphs[seg].replay()
            a.record(stream)
            for _ in range(full):
                graphs[seg].replay()
            if rem:
                graphs[rem].replay()
            b.record(stream)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
        return a.elapsed_time(b) * 1000.0 / steps, (t1 - t0) * 1e6 / (steps + n_cover * seg), seg

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ------------------------------------------------------------------ config 1 (headline)
    N, K = 14336, 4096
    rng = np.random.Generator(np.random.PCG64(1001))
    u = rng.integers(0, 16, (N, K), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    del u
    scale = rng.lognormal(-5, 0.5, (N, K // 32)).astype(np.float16)
    x_np = {m: rng.standard_normal((m, K)).astype(np.float32) for m in (1, 4, 8)}
    base = QWeightInt4G32(torch.from_numpy(packed).to(dev), torch.from_numpy(scale).to(dev))
    copies = [base] + [QWeightInt4G32(base.packed.clone(), base.scale.clone()) for _ in range(N_COPIES - 1)]

    def gemv_bytes(m):
        return N * K // 2 + N * (K // 32) * 2 + m * K * 2 + m * N * 4

    def bound_step(fn, argv):
        """step(i) = fn(*argv[i % len(argv)]), return codes OR-ed into step.rc."""
        n = len(argv)

        def step(i):
            step.rc |= fn(*argv[i % n])

        step.rc = 0
        return step

    def gemv_step(x, weights, y, m):
        """step(i): one call of chadq_gemv_i4g32 on weight copy i % len(weights), arguments bound beforehand (a ctypes call
        costs the host about 3 us, well under the kernel's time).  Return codes are OR-ed into step.rc."""
        return bound_step(_lib.load().chadq_gemv_i4g32,
                          [(x.data_ptr(), w.packed.data_ptr(), w.scale.data_ptr(), y.data_ptr(), m, N, K, stream.cuda_stream)
                           for w in weights])

    want = set() if args.no_extras else {e for e in args.extras.split(",") if e}
    if args.short:
        args.settle_ms = 0.0  # hardware-counter runs serialise every dispatch: no phase that only spends launches
    n_side = (48, 24) if args.short else (480, 48)   # launches, warm-up of the GEMV side measurements
    n_gemm = (24, 24) if args.short else (240, 24)
    n_moe = 3 if args.short else 20
    n_dec = 4 if args.short else 64
    results = {}
    parity = {}
    host = {}  # host copies of the side measurements' inputs, for the CPU legs
    xs = {m: torch.from_numpy(x_np[m]).to(torch.bfloat16).to(dev) for m in (1, 4, 8)}
    ys = {m: torch.empty(m, N, dtype=torch.float32, device=dev) for m in (1, 4, 8)}

    def measure_gemv(m, do_settle=True, repeats=1):
        """repeats > 1: the whole measurement (warm-up steps, synchronize, exactly `steps` timed steps) is taken that
        many times in a row and the median is returned - a timed region of 20 steps lasts 140 us, and single ones
        scatter by 5 % and more."""
        steps = args.steps if m == 1 else min(args.steps, n_side[0])
        ops.qgemv(xs[m], copies[0], out=ys[m])  # once through the checked wrapper; the timed steps call the entry point itself
        step = gemv_step(xs[m], copies, ys[m], m)
        runs = []
        for r in range(repeats):
            runs.append(run_steps(step, steps, args.warmup, direct=True, do_settle=do_settle and r == 0))
        if step.rc:
            raise RuntimeError("chadq_gemv_i4g32 returned %d during the timed steps" % step.rc)
        us, wall, seg_used = sorted(runs)[len(runs) // 2]
        return us, wall, steps, seg_used

    # The headline measurement is taken twice: as the first thing this process runs on the GPU, with nothing but the W
    # warm-up steps in front of it, and again at the end of the GEMV measurements behind a settling phase (settle()
    # above).  The second figure is the one reported; the first is kept beside it in extras.
    first_m1 = measure_gemv(1, do_settle=False)
    from oracle import chadq_oracle as O  # the checker, used once outside the timed region

    parity["gemv_i4g32_m1_rel_l2_vs_f64"] = O.rel_l2(ys[1].cpu().numpy(), O.qgemm_int4g32_f64(bits(xs[1]), packed, scale))

    extras = {}
    if "gemv" in want:
        x1 = torch.from_numpy(x_np[1]).to(torch.bfloat16).to(dev)
        y1 = torch.empty(1, N, dtype=torch.float32, device=dev)
        us_hot = run_steps(gemv_step(x1, [base], y1, 1), *n_side, direct=True)[0]
        extras["gemv_i4g32"] = {}
        extras["gemv_i4g32"]["M1_same_buffer_every_step"] = {
            "us": round(us_hot, 3), "GBps": round(gemv_bytes(1) / us_hot * 1e-3, 1),
            "note": "weights served by the 256 MB last-level cache, not HBM; not a roofline figure"}
        # what this machine delivers for a cold read of the same number of bytes and no arithmetic (bench_probe.so,
        # built from bench_probe.hip): the practical ceiling next to which the GEMV's time should be read
        import ctypes

        probe_path = os.path.join(ROOT, "bench_probe.so")
        if os.path.exists(probe_path):
            plib = ctypes.CDLL(probe_path)
            plib.bench_probe_read.restype = ctypes.c_int
            plib.bench_probe_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
            nread = gemv_bytes(1) // 16384 * 16384
            flat = [torch.empty(nread, dtype=torch.uint8, device=dev).fill_(i + 1) for i in range(N_COPIES)]
            pout = torch.empty(nread // 16384, dtype=torch.int32, device=dev)

            pargs = [(f.data_ptr(), nread, pout.data_ptr(), stream.cuda_stream) for f in flat]

            def probe(i):
                if plib.bench_probe_read(*pargs[i % N_COPIES]):
                    raise RuntimeError("bench_probe_read failed")

            us_rd = run_steps(probe, *n_side, direct=True)[0]
            extras["gemv_i4g32"]["cold_read_same_bytes"] = {
                "us": round(us_rd, 3), "GBps": round(nread / us_rd * 1e-3, 1), "bytes": int(nread),
                "note": "loads only (bench_probe.hip), rotating buffers: the machine's ceiling for a read of this size"}
            del flat, pout
            # a dependent launch of a kernel that does nothing, replayed from a graph like everything else here
            plib.bench_probe_empty.restype = ctypes.c_int
            plib.bench_probe_empty.argtypes = [ctypes.c_void_p]

            def empty(i):
                if plib.bench_probe_empty(torch.cuda.current_stream().cuda_stream):
                    raise RuntimeError("bench_probe_empty failed")

            extras["launch_floor_us"] = {"us": round(run_steps(empty, *n_side)[0], 3),
                                         "note": "an empty kernel (bench_probe.hip) per step, dependent launches in a replayed graph"}
    if "gemv" in want:
        for m in (4, 8):
            results[m] = measure_gemv(m)
    M1_REPEATS = 1 if args.steps >= 500 else 5
    results[1] = measure_gemv(1, repeats=M1_REPEATS)  # the reported one (see above)
    us1, wall1, steps1, seg1 = results[1]
    achieved = gemv_bytes(1) / us1 * 1e-3  # GB/s
    if "gemv" in want:
        for m in (1, 4, 8):
            extras["gemv_i4g32"]["M%d" % m] = {"us": round(results[m][0], 3), "GBps": round(gemv_bytes(m) / results[m][0] * 1e-3, 1),
                                               "frac_hbm_peak": round(gemv_bytes(m) / results[m][0] * 1e-3 / HBM_PEAK_GBS, 4)}
    # the same steps replayed from captured graphs (the launch form of the other measurements), for comparison
    us_g, _, seg_g = run_steps(gemv_step(xs[1], copies, ys[1], 1), steps1, args.warmup, direct=False)
    extras["gemv_i4g32_M1_graph_replay"] = {
        "us": round(us_g, 3), "GBps": round(gemv_bytes(1) / us_g * 1e-3, 1),
        "note": "the headline's %d steps as replays of captured graphs of %d launches, settled like it: a replay costs "
                "about 8 us of its own, which a 20-step region shows and a 960-step region does not" % (steps1, seg_g)}
    extras["gemv_i4g32_M1_first_measurement_of_the_process"] = {
        "us": round(first_m1[0], 3), "GBps": round(gemv_bytes(1) / first_m1[0] * 1e-3, 1),
        "note": "the same %d steps after %d warm-up steps and no settling phase, on a GPU that was idle until then" % (first_m1[2], args.warmup)}
    del copies

    if "int8" in want:
        # config 0: int8 per-row GEMV
        N0, K0 = 16384, 2048
        r0 = np.random.Generator(np.random.PCG64(1000))
        host["cfg0"] = (r0.standard_normal((1, K0)).astype(np.float32), r0.integers(-127, 128, (N0, K0), dtype=np.int8),
                        r0.uniform(0.001, 0.02, N0).astype(np.float32))
        x0, w0, s0 = (torch.from_numpy(a).to(dev) for a in host["cfg0"])
        c0 = [QWeightInt8(w0.clone(), s0.clone()) for _ in range(N_COPIES)]
        y0 = torch.empty(1, N0, dtype=torch.float32, device=dev)
        ops.qgemv(x0, c0[0], out=y0)  # once through the checked wrapper

        def i8_step(xx, yy, m):
            return bound_step(_lib.load().chadq_gemv_i8row, [(xx.data_ptr(), c.w.data_ptr(), c.scale.data_ptr(), yy.data_ptr(), m, N0, K0,
                                                              stream.cuda_stream) for c in c0])

        st0 = i8_step(x0, y0, 1)
        us0 = run_steps(st0, *n_side, direct=True)[0]
        if st0.rc:
            raise RuntimeError("chadq_gemv_i8row returned %d during the timed steps" % st0.rc)
        b0 = N0 * K0 + N0 * 4 + K0 * 4 + N0 * 4
        extras["gemv_i8row_config0"] = {"us": round(us0, 3), "GBps": round(b0 / us0 * 1e-3, 1),
                                        "frac_hbm_peak": round(b0 / us0 * 1e-3 / HBM_PEAK_GBS, 4)}
        # labelled extras: the same matrix with 8 and 16 activation rows (one pass over the weights each)
        for m in (8, 16):
            xm = torch.from_numpy(r0.standard_normal((m, K0)).astype(np.float32)).to(dev)
            ym = torch.empty(m, N0, dtype=torch.float32, device=dev)
            usm = run_steps(i8_step(xm, ym, m), *n_side, direct=True)[0]
            bm = N0 * K0 + N0 * 4 + m * (K0 * 4 + N0 * 4)
            extras["gemv_i8row_config0"][f"M{m}_extra"] = {"us": round(usm, 3), "GBps": round(bm / usm * 1e-3, 1)}
        del c0, w0
    if "gemm" in want or "gemm_ablation" in want:
        # config 2: prefill dequant-GEMM, int4 group-32 and int8 per-row
        M2, N2, K2 = 512, 4096, 4096
        r2 = np.random.Generator(np.random.PCG64(1002))
        p2h, s2h = r2.integers(0, 256, (N2, K2 // 2), dtype=np.uint8), r2.lognormal(-5, 0.5, (N2, K2 // 32)).astype(np.float16)
        x2h = r2.standard_normal((M2, K2)).astype(np.float32)
        w8h, s8h = r2.integers(-127, 128, (N2, K2), dtype=np.int8), r2.uniform(0.001, 0.02, N2).astype(np.float32)
        host["cfg2"] = (x2h, p2h, s2h, w8h, s8h)
        p2, s2 = torch.from_numpy(p2h).to(dev), torch.from_numpy(s2h).to(dev)
        x2 = torch.from_numpy(x2h).to(torch.bfloat16).to(dev)
        y2 = torch.empty(M2, N2, dtype=torch.bfloat16, device=dev)
        q4 = QWeightInt4G32(p2, s2)
        q8 = QWeightInt8(torch.from_numpy(w8h).to(dev), torch.from_numpy(s8h).to(dev))
        flop = 2.0 * M2 * N2 * K2
        for name, qw in (("gemm_i4g32_config2", q4), ("gemm_i8row_config2", q8)):
            usg = run_steps(lambda i: ops.qgemm(x2, qw, out=y2), *n_gemm)[0]
            extras[name] = {"us": round(usg, 3), "TFLOPs": round(flop / usg * 1e-6, 1),
                            "frac_bf16_mfma_peak": round(flop / usg * 1e-6 / MFMA_BF16_PEAK_TFLOPS, 4)}

        if "gemm_ablation" in want:
            # the same two calls on the measurement build whose 128 x 64 kernel hands the packed words to the matrix
            # core without dequantising them: the floor under any variant of that kernel with cheaper (or no)
            # dequantisation, e.g. int8 weights on the int8 matrix core
            from chadslab_amd.build import ablation_path

            main_lib = _lib.load()
            if ablation_path("nodequant").exists():
                try:
                    _lib._lib = _lib.open_library(ablation_path("nodequant"))
                    for name, qw in (("gemm_i4g32_config2", q4), ("gemm_i8row_config2", q8)):
                        extras[name]["us_without_dequantisation"] = round(run_steps(lambda i: ops.qgemm(x2, qw, out=y2), *n_gemm)[0], 3)
                finally:
                    _lib._lib = main_lib
        # context: what the matrix cores sustain on non-zero operands with no memory traffic at all (bench_probe.hip)
        import ctypes

        probe_path = os.path.join(ROOT, "bench_probe.so")
        if os.path.exists(probe_path):
            plib2 = ctypes.CDLL(probe_path)
            plib2.bench_probe_mfma.restype = ctypes.c_int
            plib2.bench_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
            pbuf = torch.empty(512 * 256, dtype=torch.float32, device=dev)
            trips = 400
            sustained = {}
            for kind, kname in ((0, "fp16"), (1, "bf16")):
                def mf(i, kind=kind):
                    if plib2.bench_probe_mfma(kind, trips, pbuf.data_ptr(), torch.cuda.current_stream().cuda_stream):
                        raise RuntimeError("bench_probe_mfma failed")
                usm = run_steps(mf, 24, 8)[0]
                sustained[kname + "_TFLOPs"] = round(512 * 4 * trips * 24 * 32768.0 / usm * 1e-6, 1)
            sustained["note"] = ("v_mfma_f32_32x32x16 on non-zero operands held in registers, 2 waves per SIMD, no memory traffic: the "
                                 "matrix cores' practical ceiling on this machine (the clock follows the power drawn)")
            extras["mfma_sustained_registers_only"] = sustained
            del pbuf
        # context: the vendor library's plain bf16 GEMM (no dequantisation) on the same shape, through torch.matmul
        wb16 = torch.randn(N2, K2, device=dev).to(torch.bfloat16)
        yt = torch.empty(M2, N2, dtype=torch.bfloat16, device=dev)
        ust = run_steps(lambda i: torch.matmul(x2, wb16.t(), out=yt), *n_gemm)[0]
        extras["gemm_bf16_library_same_shape"] = {"us": round(ust, 3), "TFLOPs": round(flop / ust * 1e-6, 1),
                                                  "note": "torch.matmul on bf16 weights (hipBLASLt/rocBLAS): context, not this build's kernel"}
        # many rows (not a benchmark configuration: extra, labelled as such): the 256 x 256 tile kernel, and beside it the
        # vendor library's plain bf16 GEMM on the same shape and on random data, which is what the matrix cores of this
        # machine sustain once their power draw sets the clock (the same call on zeros runs half as long)
        M2b = 4096
        x2b = torch.randn(M2b, K2, device=dev).to(torch.bfloat16)
        y2b = torch.empty(M2b, N2, dtype=torch.bfloat16, device=dev)
        nbig = (max(8, n_gemm[0] // 8), 4)
        usb = run_steps(lambda i: ops.qgemm(x2b, q4, out=y2b), *nbig)[0]
        flopb = 2.0 * M2b * N2 * K2
        extras["gemm_i4g32_M4096_extra"] = {"us": round(usb, 2), "TFLOPs": round(flopb / usb * 1e-6, 1),
                                            "frac_bf16_mfma_peak": round(flopb / usb * 1e-6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                            "note": "M=4096, N=K=4096 (large-tile kernel): not a benchmark configuration"}
        ustb = run_steps(lambda i: torch.matmul(x2b, wb16.t(), out=y2b), *nbig)[0]
        extras["gemm_bf16_library_M4096_extra"] = {"us": round(ustb, 2), "TFLOPs": round(flopb / ustb * 1e-6, 1),
                                                   "frac_bf16_mfma_peak": round(flopb / ustb * 1e-6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                                   "note": "torch.matmul on bf16 weights, random data: context, not this build's kernel"}
        del wb16, yt
        del x2, y2, q4, q8, p2, s2, x2b, y2b
    if "moe" in want or "moe_ablation" in want:
        # config 3: mixture-of-experts FFN, 8 experts, top-2, 256 tokens, on config 3's own data: PCG64(1003), uniform
        # nibbles, fp16 group scales ~LogNormal(-5, 0.5), x and the router logits ~N(0,1)
        T3, H3, F3, E3 = 256, 4096, 14336, 8
        r3 = np.random.Generator(np.random.PCG64(1003))

        first3 = []  # expert 0's host arrays, for the CPU leg

        def mk(n, k):
            u3 = r3.integers(0, 16, (n, k), dtype=np.uint8)
            p3 = (u3[:, 0::2] | (u3[:, 1::2] << 4)).astype(np.uint8)
            s3 = r3.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
            if len(first3) < 6:
                first3.extend([p3, s3])
            return QWeightInt4G32(torch.from_numpy(p3).to(dev), torch.from_numpy(s3).to(dev))

        experts = [(mk(F3, H3), mk(F3, H3), mk(H3, F3)) for _ in range(E3)]
        z3h, x3h = r3.standard_normal((T3, E3)).astype(np.float32), r3.standard_normal((T3, H3)).astype(np.float32)
        host["cfg3"] = (x3h, z3h, tuple(first3))
        z3 = torch.from_numpy(z3h).to(dev)
        x3 = torch.from_numpy(x3h).to(torch.bfloat16).to(dev)
        torch.cuda.synchronize()  # the inputs were copied on the default stream

        def time_moe(ex):
            with torch.cuda.stream(stream):
                settle(lambda i: ops.moe_ffn(x3, z3, ex))
                for _ in range(3):
                    ops.moe_ffn(x3, z3, ex)
                a3, b3 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a3.record(stream)
                for _ in range(n_moe):
                    ops.moe_ffn(x3, z3, ex)
                b3.record(stream)
                torch.cuda.synchronize()
            return a3.elapsed_time(b3) * 1000.0 / n_moe

        hit = int(torch.unique(ops.moe_route(z3, 2, True)[0]).numel())
        flop3 = 2.0 * T3 * 2 * 3 * H3 * F3
        bytes3 = hit * 3 * (F3 * H3 // 2 + F3 * (H3 // 32) * 2)

        def moe_entry(us3, note):
            return {"us": round(us3, 1), "TFLOPs": round(flop3 / us3 * 1e-6, 1),
                    "frac_bf16_mfma_peak": round(flop3 / us3 * 1e-6 / MFMA_BF16_PEAK_TFLOPS, 4), "experts_hit": hit,
                    "expert_weight_GBps": round(bytes3 / us3 * 1e-3, 1),
                    "frac_hbm_peak": round(bytes3 / us3 * 1e-3 / HBM_PEAK_GBS, 4), "weights": note}

        extras["moe_ffn_i4g32_config3"] = moe_entry(time_moe(experts), "row-major containers")
        # the same experts repacked once into tile order (ops.to_tiles, a load-time step outside the timed region)
        with torch.cuda.stream(stream):
            tiled = []
            for tr in experts:  # one expert at a time: the row-major copy is dropped as soon as its tiles exist
                tiled.append(tuple(ops.to_tiles(m) for m in tr))
            torch.cuda.synchronize()
        del experts
        torch.cuda.empty_cache()
        extras["moe_ffn_i4g32_config3_tiled"] = moe_entry(time_moe(tiled), "tile order (chadq_repack_i4g32_tiles at load time)")
        if "moe_ablation" in want:
            # the same call on the measurement builds (chadslab_amd.build.build_ablations): the expert GEMM with its
            # arithmetic, or with its weight loads, compiled out - what each half of the loop takes on its own.  The
            # results of these builds are wrong by construction; only the clock is read.
            from chadslab_amd.build import ABLATIONS, ablation_path

            main_lib = _lib.load()
            abl = {"both": extras["moe_ffn_i4g32_config3_tiled"]["us"]}
            try:
                for name in ("stream", "arith"):
                    if not ablation_path(name).exists():
                        abl[name] = None
                        continue
                    _lib._lib = _lib.open_library(ablation_path(name))
                    abl[name] = round(time_moe(tiled), 1)
            finally:
                _lib._lib = main_lib
            extras["moe_ffn_i4g32_config3_tiled"]["ablation_us"] = abl
        del tiled, x3, z3
        torch.cuda.empty_cache()
    if "decode" in want:
        # config 4: decode step, 18 layers, d 2048, 8 query heads x 256, 1 KV head, FFN 16384, vocab 256000, batch 1,
        # KV cache pre-filled to 2048 positions; 64 graph-replayed greedy steps (context 2048..2111)
        from chadslab_amd.decoder import DecoderConfig, QuantDecoder, random_weights

        cfg4 = DecoderConfig(max_ctx=4096)
        w4 = random_weights(cfg4, 1004, dev)
        torch.cuda.synchronize()  # the weights were generated on the default stream
        with torch.cuda.stream(stream):
            dec = QuantDecoder(cfg4, w4, dev)
            for li in range(cfg4.n_layers):
                dec.kcache[li].normal_()
                dec.vcache[li].normal_()
            dec.token.fill_(5)
            dec.pos.fill_(2040)
            dec.capture(DEC_STEPS)
            settle(lambda i: dec.graph.replay())  # positions 2040 .. about 2110 (max_ctx 4096); then back to the start
            dec.pos.fill_(2040)
            for _ in range(8 // DEC_STEPS):
                dec.graph.replay()
            a4, b4 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a4.record(stream)
            for _ in range(n_dec // DEC_STEPS):
                dec.graph.replay()
            b4.record(stream)
            torch.cuda.synchronize()
        us4 = a4.elapsed_time(b4) * 1000.0 / n_dec
        wbytes = sum(q.packed.numel() + 2 * q.scale.numel() for L in w4["layers"] for q in (L["wqkv"], L["wo"], L["wgu"], L["wd"]))
        wbytes += w4["emb"].packed.numel() + 2 * w4["emb"].scale.numel()
        kvbytes = cfg4.n_layers * 2 * 2080 * cfg4.dh * 2
        extras["decode_step_config4"] = {"us_per_token": round(us4, 1), "tokens_per_s": round(1e6 / us4, 1),
                                         "bytes_per_token": wbytes + kvbytes, "GBps": round((wbytes + kvbytes) / us4 * 1e-3, 1),
                                         "frac_hbm_peak": round((wbytes + kvbytes) / us4 * 1e-3 / HBM_PEAK_GBS, 4),
                                         "context": "2048..2111",
                                         "launch": "one HIP graph per %d tokens (the token passes from step to step in device memory)" % DEC_STEPS}
        del dec
        # the same step ending in a draw from the 50 most likely tokens instead of the argmax (the uniform number stays
        # fixed during the replays: the draw's cost does not depend on it)
        with torch.cuda.stream(stream):
            dec = QuantDecoder(cfg4, w4, dev)
            for li in range(cfg4.n_layers):
                dec.kcache[li].normal_()
                dec.vcache[li].normal_()
            dec.token.fill_(5)
            dec.pos.fill_(2040)
            dec.set_sampling(50, 1.0, 1004)
            dec.capture(DEC_STEPS)
            settle(lambda i: dec.graph.replay())
            dec.pos.fill_(2040)
            for _ in range(8 // DEC_STEPS):
                dec.graph.replay()
            a4, b4 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a4.record(stream)
            for _ in range(n_dec // DEC_STEPS):
                dec.graph.replay()
            b4.record(stream)
            torch.cuda.synchronize()
        extras["decode_step_config4"]["us_per_token_sampling_top50"] = round(a4.elapsed_time(b4) * 1000.0 / n_dec, 1)
        if not args.no_cpu:  # two layers and the table go back to the host for the CPU leg

            def to_host(q):
                return q.packed.cpu().numpy(), q.scale.cpu().numpy()

            host["cfg4"] = {"layers": [{k: (to_host(v) if hasattr(v, "packed") else v.cpu().numpy()) for k, v in L.items()}
                                       for L in w4["layers"][:2]],
                            "lnf": w4["lnf"].cpu().numpy(), "emb": to_host(w4["emb"]), "cfg": cfg4}
        del dec, w4
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ CPU baseline (rank 0, N=1)
    # The reference snapshot holds no implementation of this path, so what is timed is this build's numpy oracle, written
    # the way a plain numpy runtime would be: (i) dequantise to fp32, then matmul - what a naive runtime pays per call -
    # and (ii) the matmul alone on weights dequantised beforehand - its best case.  Headline config in cpu_baseline,
    # the other configs under cpu_baseline.configs, each on a bounded sample.
    cpu = None
    if not args.no_cpu:
        from oracle import chadq_oracle as O

        try:
            from threadpoolctl import threadpool_info

            threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
        except Exception:
            threads = os.cpu_count() or 1

        def med(fn, reps, warm=1):
            for _ in range(warm):
                fn()
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            return float(np.median(ts))

        xb = O.f32_to_bf16(x_np[1])
        t0 = time.perf_counter()
        O.qgemv_int4g32(xb, packed, scale)
        first = time.perf_counter() - t0
        reps = int(min(40, max(3, 8.0 / max(first, 1e-3))))
        t_dq = med(lambda: O.qgemv_int4g32(xb, packed, scale), reps, 0)
        wd = O.dequant_int4g32(packed, scale)
        xf = O.bf16_to_f32(xb)
        t_pre = med(lambda: xf @ wd.T, 10)
        del wd
        per_cfg = {}
        if "cfg0" in host:
            x0h, w0h, s0h = host["cfg0"]
            b0h = w0h.size + 2 * s0h.size * 4 + x0h.size * 4
            t_a = med(lambda: O.qgemv_int8(x0h, w0h, s0h), 10)
            w0f = O.dequant_int8(w0h, s0h)
            t_b = med(lambda: x0h @ w0f.T, 10)
            del w0f
            per_cfg["config0_gemv_i8row"] = {"dequant_plus_matmul_ms": round(t_a * 1e3, 2), "predequantised_matmul_ms": round(t_b * 1e3, 3),
                                             "GBps": round(b0h / t_a * 1e-9, 3), "predequantised_GBps": round(b0h / t_b * 1e-9, 2),
                                             "sample": "full shape, median of 10"}
        if "cfg2" in host:
            x2h, p2h, s2h, w8h, s8h = host["cfg2"]
            x2b = O.f32_to_bf16(x2h)
            x2f = O.bf16_to_f32(x2b)
            fl = 2.0 * x2h.shape[0] * p2h.shape[0] * x2h.shape[1]
            t_a = med(lambda: O.qgemm_int4g32_bf16(x2b, p2h, s2h), 3)
            w2f = O.dequant_int4g32(p2h, s2h)
            t_b = med(lambda: x2f @ w2f.T, 5)
            del w2f
            t_c = med(lambda: O.qgemm_int8_bf16(x2b, w8h, s8h), 3)
            per_cfg["config2_gemm"] = {"int4_dequant_plus_matmul_ms": round(t_a * 1e3, 1), "int4_predequantised_matmul_ms": round(t_b * 1e3, 1),
                                       "int8_dequant_plus_matmul_ms": round(t_c * 1e3, 1), "int4_TFLOPs": round(fl / t_a * 1e-12, 3),
                                       "int4_predequantised_TFLOPs": round(fl / t_b * 1e-12, 3), "sample": "full shape, median of 3 / 5"}
        if "cfg3" in host:
            # one of the eight experts with the tokens routed to it; the call's time is taken as 8 x that
            x3h, z3h, (gp, gs, up_, us_, dp, ds) = host["cfg3"]
            idx3, _ = O.moe_route(z3h, 2, True)
            tok0 = np.nonzero((idx3 == 0).any(axis=1))[0]
            xe = O.f32_to_bf16(x3h[tok0])

            def expert_dq():
                g = O.qgemv_int4g32(xe, gp, gs)
                u_ = O.qgemv_int4g32(xe, up_, us_)
                return O.qgemv_int4g32(O.f32_to_bf16(O.silu(g) * u_), dp, ds)

            t_a = med(expert_dq, 1, 0)
            gf, uf, df = O.dequant_int4g32(gp, gs), O.dequant_int4g32(up_, us_), O.dequant_int4g32(dp, ds)
            xef = O.bf16_to_f32(xe)

            def expert_pre():
                h = O.bf16_to_f32(O.f32_to_bf16(O.silu(xef @ gf.T) * (xef @ uf.T)))
                return h @ df.T

            t_b = med(expert_pre, 3)
            del gf, uf, df
            per_cfg["config3_moe_ffn"] = {"dequant_plus_matmul_ms": round(8 * t_a * 1e3, 1), "predequantised_matmul_ms": round(8 * t_b * 1e3, 1),
                                          "sample": "expert 0 of 8 with its %d tokens, one call (three for the matmuls alone), scaled by 8" % tok0.size}
        if "cfg4" in host:
            # two of the 18 layers and the output table at context 2048; a token is taken as 9 x the layers + the table
            h4 = host["cfg4"]
            c4 = h4["cfg"]
            ctx = 2048
            kc = [np.zeros((ctx + 1, c4.dh), np.uint16) for _ in range(2)]
            vc = [np.zeros((ctx + 1, c4.dh), np.uint16) for _ in range(2)]
            xr = np.random.Generator(np.random.PCG64(1004)).standard_normal(c4.d).astype(np.float32)

            def two_layers():
                xx = xr
                for li in range(2):
                    xx = O.decode_layer(h4["layers"][li], xx, ctx, kc[li], vc[li], c4.hq, c4.dh, c4.eps, c4.rope_base)
                return xx

            t_l = med(two_layers, 1, 0)
            t_t = med(lambda: O.decode_logits(h4, xr, c4.eps), 1, 0)
            wf = [[O.dequant_int4g32(*L[k]) for k in ("wqkv", "wo", "wgu", "wd")] for L in h4["layers"]]
            tf = O.dequant_int4g32(*h4["emb"])
            vq, va, vh = xr, np.ones(c4.hq * c4.dh, np.float32), np.ones(c4.ffn, np.float32)
            t_lp = med(lambda: [(wl[0] @ vq, wl[1] @ va, wl[2] @ vq, wl[3] @ vh) for wl in wf], 3)
            t_tp = med(lambda: tf @ vq, 3)
            del wf, tf
            per_cfg["config4_decode_step"] = {"dequant_plus_matmul_tokens_per_s": round(1.0 / (9 * t_l + t_t), 4),
                                              "predequantised_matmul_tokens_per_s": round(1.0 / (9 * t_lp + t_tp), 2),
                                              "sample": "2 of 18 layers (x 9) + the 256000-row table, context 2048, one call; the matmul-only "
                                                        "figure leaves out attention and norms"}
        cpu = {
            "value": round(gemv_bytes(1) / t_dq * 1e-9, 4), "unit": "GB/s", "cores": int(threads), "kind": "port",
            "sample": "config 1 at M=1, full shape: numpy dequantise-to-fp32 + sgemv, median of %d calls after 1 warm-up "
                      "(%.1f ms per call); build-written numpy baseline, no reference implementation exists in the snapshot" % (reps, t_dq * 1e3),
            "predequantised_sgemv_GBps": round(gemv_bytes(1) / t_pre * 1e-9, 3),
            "host_cpus": os.cpu_count(), "blas_threads": int(threads), "oracle_dequant_workers": int(O.WORKERS),
            "configs": per_cfg,
        }

    traffic_bytes, kernel_name = profile_figures()
    out = {
        "metric": "int4 GEMV HBM GB/s (% peak) + dequant-GEMM TFLOP/s (% MFMA peak), 1 GPU",
        "value": round(achieved, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps1,
        "warmup": args.warmup,
        "ms_per_step": round(us1 * 1e-3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 x int4 -> fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": "config 1: int4 group-32 decode GEMV, M=1, W [14336,4096], x bf16, y fp32",
                   "M": 1, "N": N, "K": K, "weight_copies_rotated": N_COPIES, "launch": ("HIP graph replay, %d launches per graph" % seg1) if seg1 else
                   ("one chadq_gemv_i4g32 call per step on one stream, back to back (host %.1f us per call); %d untimed steps "
                    "queued in front of the start event" % (wall1, COVER)),
                   "algorithmic_bytes_per_launch": gemv_bytes(1),
                   "settle_ms": args.settle_ms, "repeats": M1_REPEATS,
                   "repeats_note": "the measurement (W warm-up steps, a synchronize, exactly K timed steps) taken this many times "
                                   "in a row, the median reported; 1 when K >= 500",
                   "settle": "the workload runs untimed for settle_ms right before its warm-up steps (steady clocks); "
                             "extras.gemv_i4g32_M1_first_measurement_of_the_process is the same measurement without it"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_bytes,
                     "traffic_source": "hardware counters of an earlier profiled run, read from the committed summary "
                                       "profiles/gemv_i4g32_m1_config1_hbm_traffic.txt (not measured by this run)",
                     "kernel": kernel_name, "host_us_per_step": round(wall1, 3)},
        "cpu_baseline": cpu,
        "parity": parity,
        "extras": extras,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
