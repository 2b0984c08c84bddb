#!/usr/bin/env python3
"""Benchmark of the MI355X quantized-matmul hot path (one GPU).

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Headline (``metric`` / ``value``): the Q4_0 4096x4096 decode GEMV of
BASELINE.json, as achieved HBM GB/s = algorithmic bytes of one GEMV
(weights + x + y = 9,469,952 B) / time of one step.  A step is one GEMV
launch through the C ABI; successive steps use successive distinct copies of
the weights out of a 604 MB ring, so every step streams its weights from HBM
rather than from the 256 MB memory-side cache.  All inputs are resident in HBM
before the timed region; timing is HIP events on the stream the kernels run on.

The same line carries ``roofline`` (dominant kernel against the 8 TB/s HBM
peak), ``cpu_baseline`` (the CPU restatement of the reference's path, timed on
this host's cores on a bounded sample) and ``others`` (the remaining BASELINE
configurations: Q6_K GEMV + argmax, RMSNorm + Q4_K N-column GEMV, Q4_K prefill
GEMM on MFMA, MoE layer at T=1 and T=64, plus a plain streaming-read probe).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0                # MI355X published HBM3E peak
MFMA_F16_PEAK_TFLOPS = 2500.0        # MI355X published dense fp16 / bf16 peak

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "q4_0_gemv_4096x4096_pmc_traffic.txt")


def measured_traffic_bytes():
    """HBM bytes per launch of the dominant kernel, read from the committed
    rocprofv3 --pmc summary (FETCH_SIZE and WRITE_SIZE per dispatch, each scaled
    by what the same counter reads for a plain copy of known size): the line
    ``traffic_bytes_per_launch = N`` of that file.  None when the file is absent
    or holds no such line."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.strip().startswith("traffic_bytes_per_launch"):
                    return int(line.split("=")[1].split()[0].replace(",", ""))
    except (OSError, ValueError, IndexError):
        pass
    return None


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=2000)
    p.add_argument("--warmup", type=int, default=200)
    p.add_argument("--skip-others", action="store_true", help="headline only")
    p.add_argument("--skip-cpu", action="store_true", help="no cpu_baseline leg")
    p.add_argument("--only", default="", help="comma-separated kernel families to run (for "
                   "profiling): q4_0, q6_k, q4_k, gemm, moe1, moe64, copy, floor (= sweep of the cold "
                   "9 MiB streaming read over workgroup counts; only when named)")
    p.add_argument("--select", action="append", default=[], metavar="OP:IN_DIM:ROWS:NCOL:FAMILY:ROWS_IN_FLIGHT:PERSISTENT",
                   help="install a forge schedule (lev_hip_forge_select) on the bench context before running, "
                        "to time a candidate other than the built-in choice; may be repeated")
    return p.parse_args()


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (got --gpus {args.gpus}); "
              "the path is built and measured on one GPU only; nothing here shards across GPUs.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from leviathan_amd import capi, ops          # raises if the HIP library is missing

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU path to measure.", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    # The context runs on a side stream so that steps can be recorded into a
    # program (HIP graph) and replayed: the host then costs nothing per step,
    # as in the reference, which records its decode programs once and replays
    # them (rust/crates/lev-vulkan/src/engine.rs:94-141).
    stream = torch.cuda.Stream(device=dev)
    torch.cuda.set_stream(stream)
    ctx = ops.Context(0, stream=stream)
    for spec in args.select:
        op, in_dim, nrows, ncol, fam, rif, pers = (int(v) for v in spec.split(":"))
        ctx.forge_select(in_dim, nrows, capi.Schedule(op, fam, rif, pers), ncol)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)

    eager_ms = {}
    thrash = torch.zeros(1 << 28, dtype=torch.int32, device=dev)      # 1 GiB, see flush_caches()
    flush_sink = torch.zeros(4, dtype=torch.int32, device=dev)

    PROGRAM_MIN_STEPS = 500

    def flush_caches():
        """A read-only pass over 1 GiB of other memory (about 0.17 ms): pushes whatever
        the previous steps touched out of the 256 MB memory-side cache and the L2s,
        and leaves no dirty lines behind (a flush that writes makes the steps that
        follow it pay for the write-back of its lines: +2 us per step over the first
        20 steps was measured that way)."""
        st = ctx.lib.lev_hip_stream_read_probe(ctx.ctx, thrash.data_ptr(), 1 << 30, flush_sink.data_ptr(), 512)
        if st:
            raise RuntimeError(ctx.lib.lev_hip_last_error(ctx.ctx).decode())

    def timed(fn, steps, warmup, tag=None):
        """ms per step over EXACTLY `steps` steps, read from HBM whatever `steps` is.

        `warmup` untimed eager steps come first.  Two timings follow, each between
        two HIP events on the launch stream with a device synchronisation on both
        sides, each behind a cache flush that is enqueued WITHOUT a synchronisation,
        so that the host enqueues the first event and the steps while the flush
        still runs and the timed region starts on the device the moment the flush
        ends (no host launch latency inside it):
          * host-launched: the steps are enqueued one by one behind the flush;
          * program: the steps are recorded once into a program (HIP graph),
            replayed once untimed, flushed, and replayed once timed.
        A program replay carries about 10 us of fixed start-up on the device, which
        is negligible over hundreds of steps but not over 20, so the step time
        reported is the program's from PROGRAM_MIN_STEPS steps on and the
        host-launched one below (unless the host did not keep ahead of the device:
        then the program's, and `timing_note` says so)."""
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        ef, e0, e1 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        ef.record(stream)
        t_host0 = time.perf_counter()
        for _ in range(4):                                     # about 0.7 ms of head start for the host
            flush_caches()
        e0.record(stream)
        for i in range(steps):
            fn(warmup + i)
        e1.record(stream)
        t_host = (time.perf_counter() - t_host0) * 1e3         # host ms to enqueue everything
        torch.cuda.synchronize()
        eager = e0.elapsed_time(e1) / steps
        # the host kept ahead if it had enqueued everything before the device was nearly through
        host_ahead = t_host < ef.elapsed_time(e0) + 0.9 * eager * steps
        ctx.program_begin()
        for i in range(steps):
            fn(warmup + i)
        prog = ctx.program_end()
        prog.run()
        torch.cuda.synchronize()
        flush_caches()
        e0.record(stream)
        prog.run()
        e1.record(stream)
        torch.cuda.synchronize()
        program = e0.elapsed_time(e1) / steps
        prog.destroy()
        use_program = steps >= PROGRAM_MIN_STEPS or not host_ahead
        if tag is not None:
            eager_ms[tag] = {"host_launched": eager, "program": program, "host_kept_ahead": host_ahead,
                             "used": "program" if use_program else "host_launched"}
            # spread, as the reference reports its timings (median of 11 samples,
            # rust/crates/lev-vulkan/src/lib.rs:683-704): the same region eleven more times, each behind
            # its own cache flush; `ms_per_step` stays the one region above
            samples = []
            es = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(11)]
            for a_ev, b_ev in es:
                for _ in range(4):
                    flush_caches()
                a_ev.record(stream)
                for i in range(steps):
                    fn(warmup + i)
                b_ev.record(stream)
            torch.cuda.synchronize()
            samples = sorted(a_ev.elapsed_time(b_ev) / steps for a_ev, b_ev in es)
            eager_ms[tag]["samples"] = {"n": len(samples), "steps_each": steps, "median_ms": samples[len(samples) // 2],
                                        "min_ms": samples[0], "max_ms": samples[-1], "launched": "host"}
        return program if use_program else eager

    def rand_bytes(n):
        return torch.randint(0, 256, (n,), dtype=torch.uint8, device=dev, generator=gen)

    def half_scales(n, sigma):
        s = (torch.randn(n, device=dev, generator=gen) * sigma).abs().to(torch.float16)
        return s.view(torch.uint8).reshape(n, 2)

    # ---- synthetic weights with the BASELINE distributions, built on the GPU ----
    def make_q4_0(nblocks, sigma=0.02):
        w = rand_bytes(nblocks * 18).reshape(nblocks, 18)
        w[:, 0:2] = half_scales(nblocks, sigma)
        return w.reshape(-1)

    def make_q6_k(nblocks, sigma=0.01):
        w = rand_bytes(nblocks * 210).reshape(nblocks, 210)
        sc = torch.randint(-32, 32, (nblocks, 16), dtype=torch.int8, device=dev, generator=gen)
        w[:, 192:208] = sc.view(torch.uint8)
        w[:, 208:210] = half_scales(nblocks, sigma)
        return w.reshape(-1)

    def make_q4_k(nblocks, sigma=0.01):
        w = rand_bytes(nblocks * 144).reshape(nblocks, 144)
        w[:, 0:2] = half_scales(nblocks, sigma)
        w[:, 2:4] = half_scales(nblocks, sigma)
        return w.reshape(-1)

    result = {}
    others = {}
    only = args.only
    only_set = {f for f in only.split(",") if f}

    def want(*families):
        return not only_set or any(f in only_set for f in families)

    # ------------------------------------------------------------------ Q4_0
    rows = cols = 4096
    q4_bytes_w = rows * cols // 32 * 18
    q4_alg_bytes = q4_bytes_w + cols * 4 + rows * 4            # 9,469,952
    if want("q4_0"):
        ncopy = 64                                             # 604 MB ring > 256 MB cache
        ring = make_q4_0(ncopy * rows * cols // 32)
        x = torch.randn(cols, device=dev, generator=gen)
        y = torch.empty(rows, device=dev)
        lib, c = ctx.lib, ctx.ctx
        wp, wn, xp, yp = ring.data_ptr(), ring.numel(), x.data_ptr(), y.data_ptr()

        def q4_step(i):
            st = lib.lev_hip_q4_0_gemv(c, wp, wn, (i % ncopy) * q4_bytes_w, xp, cols, yp, rows, cols, rows)
            if st:
                raise RuntimeError(lib.lev_hip_last_error(c).decode())

        ms = timed(q4_step, args.steps, args.warmup, tag="q4_0")
        gbs = q4_alg_bytes / (ms * 1e-3) / 1e9
        result.update(ms_per_step=ms, value=gbs)
        # correctness of what was just timed, against the CPU restatement
        check = {}
        if not args.skip_cpu:
            import oracle as O                                  # cpu_baseline leg only
            q4_step(0)
            torch.cuda.synchronize()
            w0 = ring[:q4_bytes_w].cpu().numpy()
            xh = x.cpu().numpy()
            ref64 = O.q4_0_matvec_f64(w0, rows, cols, xh)
            check["max_rel_err_vs_fp64"] = O.max_rel_err(y.cpu().numpy(), ref64)
            ncores = os.cpu_count() or 1
            threads = min(ncores, 64)

            def cpu_rate(nthreads, budget_s):
                n, t0 = 0, time.perf_counter()
                while True:
                    O.q4_0_matvec_ref(w0, rows, cols, xh, threads=nthreads)
                    n += 1
                    dt = time.perf_counter() - t0
                    if dt >= budget_s:
                        return n, q4_alg_bytes * n / dt / 1e9
            n1, gbs1 = cpu_rate(0, 6.0)
            nmt, gbsmt = cpu_rate(threads, 8.0)
            result["cpu_baseline"] = {
                "value": gbsmt, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": f"{nmt} Q4_0 4096x4096 GEMVs, rows split over {threads} threads "
                          f"(C restatement of Q4_0.matvecReference, gcc -O3, no FMA contraction, no fast-math)",
                "single_thread": {"value": gbs1, "unit": "GB/s", "cores": 1, "sample": f"{n1} GEMVs"},
            }
        result["check"] = check
        del ring

    def cpu_matvec_baseline(label, call, alg_bytes, what):
        """The reference's CPU GEMV of a configuration on this host's cores: single thread, then
        the rows split over the cores as Model::matvec does (lev-model/src/lib.rs:184-199); a
        bounded sample of about 3 s each, as GB/s of the configuration's algorithmic bytes."""
        ncores = os.cpu_count() or 1
        threads = min(ncores, 64)
        out = {}
        for nthreads, key, budget in ((0, "single_thread", 3.0), (threads, "row_parallel", 3.0)):
            n, t0 = 0, time.perf_counter()
            while True:
                call(nthreads)
                n += 1
                dt = time.perf_counter() - t0
                if dt >= budget:
                    break
            out[key] = {"value": alg_bytes * n / dt / 1e9, "unit": "GB/s", "cores": max(nthreads, 1),
                        "ms_per_gemv": dt / n * 1e3, "sample": f"{n} GEMVs"}
        out["kind"] = "port"
        out["what"] = what
        cpu_others[label] = out

    cpu_others = {}

    def run_other(name, fn, alg_bytes, steps, warmup, extra=None):
        ms = timed(fn, steps, warmup)
        entry = {"us_per_launch": ms * 1e3, "algorithmic_bytes": alg_bytes,
                 "achieved_GBps": alg_bytes / (ms * 1e-3) / 1e9,
                 "frac_of_hbm_peak": alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
        if extra:
            entry.update(extra(ms))
        others[name] = entry

    lib, c = ctx.lib, ctx.ctx

    def must(st):
        if st:
            raise RuntimeError(lib.lev_hip_last_error(c).decode())

    if not args.skip_others or only:
        # ---------------------------------------------------- streaming probe
        if want("copy"):
            buf = rand_bytes(1 << 30)
            sink = torch.zeros(4, dtype=torch.int32, device=dev)
            for nbytes, label in ((q4_bytes_w, "stream_read_9MiB_same_buffer"), (1 << 30, "stream_read_1GiB")):
                run_other(label, lambda i: must(lib.lev_hip_stream_read_probe(
                    c, buf.data_ptr(), nbytes, sink.data_ptr(), 2048 if nbytes < (1 << 28) else 512)), nbytes,
                    500 if nbytes < (1 << 28) else 50, 10)
            # the same 9 MiB read from a different part of the 1 GiB buffer every launch: what HBM
            # (not the memory-side cache) delivers to a launch of the headline kernel's size
            nrot = (1 << 30) // q4_bytes_w
            run_other("stream_read_9MiB_rotating", lambda i: must(lib.lev_hip_stream_read_probe(
                c, buf.data_ptr() + (i % nrot) * q4_bytes_w, q4_bytes_w, sink.data_ptr(), 2048)), q4_bytes_w, 600, 20)
            run_other("empty_kernel_launch", lambda i: must(lib.lev_hip_empty_launch(c)), 0, 1000, 100)
            # plain copy of known size: the calibration kernel for the
            # FETCH_SIZE / WRITE_SIZE counters (reads and writes 256 MiB each)
            src = buf[: 1 << 28].view(torch.int32)
            dst = torch.empty_like(src)
            run_other("copy_256MiB", lambda i: dst.copy_(src), 2 << 28, 20, 5)
            del buf, src, dst

        # ------------------------------------- floor of a cold read of the headline's bytes
        if "floor" in only_set:
            # One pass over 9 MiB that no cache holds (a different part of 1 GiB every launch),
            # by plain 128-bit loads and nothing else, for a range of grids: 256 threads a
            # workgroup, so 589,824 loads / (256 * workgroups) loads per thread, four in flight.
            buf = rand_bytes(1 << 30)
            sink = torch.zeros(4, dtype=torch.int32, device=dev)
            nrot = (1 << 30) // q4_bytes_w
            for wg in (128, 256, 512, 1024, 2048, 4096, 8192):
                run_other(f"stream_read_9MiB_rotating_wg{wg}", lambda i, wg=wg: must(lib.lev_hip_stream_read_probe(
                    c, buf.data_ptr() + (i % nrot) * q4_bytes_w, q4_bytes_w, sink.data_ptr(), wg)), q4_bytes_w,
                    600, 20, extra=lambda ms, wg=wg: {"workgroups": wg,
                                                      "loads_per_thread": q4_bytes_w / 16 / (256 * wg)})
            run_other("empty_kernel_launch", lambda i: must(lib.lev_hip_empty_launch(c)), 0, 1000, 100)
            del buf

        # ---------------------------------------------- Q4_0 large streaming
        if want("q4_0"):
            torch.cuda.empty_cache()   # every family starts from fresh allocations, as when it runs alone
            rows2 = 32768
            nb2 = rows2 * cols // 32
            ring2 = make_q4_0(8 * nb2)
            x = torch.randn(cols, device=dev, generator=gen)
            y2 = torch.empty(rows2, device=dev)
            run_other("q4_0_gemv_32768x4096", lambda i: must(lib.lev_hip_q4_0_gemv(
                c, ring2.data_ptr(), ring2.numel(), (i % 8) * nb2 * 18, x.data_ptr(), cols,
                y2.data_ptr(), rows2, cols, rows2)), nb2 * 18 + cols * 4 + rows2 * 4, 100, 20)
            del ring2

        # ------------------------------------------------------ Q6_K + argmax
        if want("q6_k"):
            torch.cuda.empty_cache()
            r6, nb6 = 32000, 32000 * 4096 // 256
            ring6 = make_q6_k(6 * nb6)
            x = torch.randn(cols, device=dev, generator=gen)
            y6 = torch.empty(r6, device=dev)
            idx = torch.empty(1, dtype=torch.int32, device=dev)
            mg = torch.empty(1, device=dev)
            run_other("q6_k_gemv_32000x4096_argmax", lambda i: must(lib.lev_hip_q6_k_gemv(
                c, ring6.data_ptr(), ring6.numel(), (i % 6) * nb6 * 210, x.data_ptr(), cols,
                y6.data_ptr(), r6, cols, r6, idx.data_ptr(), mg.data_ptr())),
                nb6 * 210 + cols * 4 + r6 * 4 + 8, 100, 20)
            run_other("q6_k_gemv_32000x4096_no_argmax", lambda i: must(lib.lev_hip_q6_k_gemv(
                c, ring6.data_ptr(), ring6.numel(), (i % 6) * nb6 * 210, x.data_ptr(), cols,
                y6.data_ptr(), r6, cols, r6, None, None)), nb6 * 210 + cols * 4 + r6 * 4, 100, 20)
            if not args.skip_cpu:
                import oracle as O                              # cpu_baseline leg only
                w6h = ring6[:nb6 * 210].cpu().numpy()
                x6h = x.cpu().numpy()
                cpu_matvec_baseline("q6_k_gemv_32000x4096", lambda nt: O.q6_k_matvec_f32(w6h, r6, cols, x6h, threads=nt),
                                    nb6 * 210 + cols * 4 + r6 * 4,
                                    "C restatement of matvec_q6k_f32 (lev-cpu/src/lib.rs:261-276: dequantise a superblock "
                                    "to f32, ascending f32 sum), gcc -O3, no FMA contraction, no fast-math")
                del w6h
            # the head on f32 activations, N columns per weight read
            for n in (2, 4, 8):
                xn = torch.randn(n, cols, device=dev, generator=gen)
                yn = torch.empty(n, r6, device=dev)
                run_other(f"q6_k_gemv_ncol_32000x4096_N{n}", lambda i: must(lib.lev_hip_q6_k_gemv_ncol(
                    c, ring6.data_ptr(), ring6.numel(), (i % 6) * nb6 * 210, xn.data_ptr(), xn.numel(), None, 0.0,
                    yn.data_ptr(), yn.numel(), cols, r6, n)), nb6 * 210 + n * (cols * 4 + r6 * 4), 100, 20)
            # the head on int8 activations, N columns per weight read (MTP verify)
            for n in (1, 4, 8, 16):
                xn = torch.randn(n, cols, device=dev, generator=gen)
                yn = torch.empty(n, r6, device=dev)
                xq = torch.empty(n, cols, dtype=torch.int8, device=dev)
                xs = torch.empty(n, cols // 32, 2, device=dev)
                must(lib.lev_hip_norm_quant_q8(c, xn.data_ptr(), xn.numel(), None, None, 0.0,
                                               xq.data_ptr(), xs.data_ptr(), None, cols, n))
                run_other(f"q6_k_gemv_q8_32000x4096_N{n}", lambda i: must(lib.lev_hip_q6_k_gemv_q8(
                    c, ring6.data_ptr(), ring6.numel(), (i % 6) * nb6 * 210, xq.data_ptr(), xs.data_ptr(),
                    xq.numel(), yn.data_ptr(), yn.numel(), cols, r6, n)),
                    nb6 * 210 + n * (cols + cols // 4 + r6 * 4), 50, 10)
            # the head as a prefill product: 512 tokens on the matrix cores
            tokens6 = 512
            xh6 = torch.randn(tokens6, cols, device=dev, generator=gen).to(torch.float16)
            yg6 = torch.empty(tokens6, r6, device=dev)
            flop6 = 2.0 * tokens6 * r6 * cols

            def gemm6_extra(ms):
                tf = flop6 / (ms * 1e-3) / 1e12
                return {"TFLOPs": tf, "mfma_frac_of_fp16_peak": tf / MFMA_F16_PEAK_TFLOPS,
                        "bound": "mfma"}
            run_other("q6_k_prefill_gemm_512x32000x4096", lambda i: must(lib.lev_hip_q6_k_gemm_prefill(
                c, ring6.data_ptr(), ring6.numel(), (i % 6) * nb6 * 210, xh6.data_ptr(), xh6.numel(),
                yg6.data_ptr(), yg6.numel(), cols, r6, tokens6)),
                nb6 * 210 + tokens6 * cols * 2 + tokens6 * r6 * 4, 100, 200, gemm6_extra)
            del ring6, xh6, yg6

        # ------------------------------------------- RMSNorm + Q4_K N columns
        if want("q4_k", "gemm"):
            torch.cuda.empty_cache()
            r4, nb4 = 12288, 12288 * 4096 // 256
            ncopy4 = 20
            ring4 = make_q4_k(ncopy4 * nb4)
        if want("q4_k"):
            gain = 1.0 + 0.1 * torch.randn(cols, device=dev, generator=gen)
            for n in (1, 2, 3, 4, 8):
                xn = torch.randn(n, cols, device=dev, generator=gen)
                yn = torch.empty(n, r4, device=dev)
                run_other(f"rmsnorm_q4_k_gemv_12288x4096_N{n}", lambda i: must(lib.lev_hip_q4_k_gemv_ncol(
                    c, ring4.data_ptr(), ring4.numel(), (i % ncopy4) * nb4 * 144, xn.data_ptr(),
                    xn.numel(), gain.data_ptr(), 1e-6, yn.data_ptr(), yn.numel(), cols, r4, n)),
                    nb4 * 144 + cols * 4 + n * (cols * 4 + r4 * 4), 200, 20)
            if not args.skip_cpu:
                import oracle as O                              # cpu_baseline leg only
                w4h = ring4[:nb4 * 144].cpu().numpy()
                x4h = torch.randn(cols, generator=torch.Generator().manual_seed(3)).numpy()
                g4h = gain.cpu().numpy()

                def c3_cpu(nt):
                    O.q4_k_matvec_f32(w4h, r4, cols, O.rmsnorm(x4h, g4h, 1e-6), threads=nt)
                cpu_matvec_baseline("rmsnorm_q4_k_gemv_12288x4096_N1", c3_cpu, nb4 * 144 + cols * 4 + cols * 4 + r4 * 4,
                                    "C restatement of rmsnorm (lev-model/src/lib.rs:110-114) + matvec_q4k_f32 "
                                    "(lev-cpu/src/lib.rs:158-175), one column, gcc -O3, no FMA contraction, no fast-math")
                del w4h
            # int8-activation path: RMSNorm+quantise, then the integer-dot GEMV
            # (timed together, as the reference's vk-q8 command times quantize + matvec)
            for n in (1, 2, 4, 8, 16):
                xn = torch.randn(n, cols, device=dev, generator=gen)
                yn = torch.empty(n, r4, device=dev)
                xq = torch.empty(n, cols, dtype=torch.int8, device=dev)
                xs = torch.empty(n, cols // 32, 2, device=dev)

                def q8_step(i, n=n, xn=xn, yn=yn, xq=xq, xs=xs):
                    must(lib.lev_hip_norm_quant_q8(c, xn.data_ptr(), xn.numel(), None, gain.data_ptr(),
                                                   1e-6, xq.data_ptr(), xs.data_ptr(), None, cols, n))
                    must(lib.lev_hip_q4_k_gemv_q8(c, ring4.data_ptr(), ring4.numel(),
                                                  (i % ncopy4) * nb4 * 144, xq.data_ptr(), xs.data_ptr(),
                                                  xq.numel(), yn.data_ptr(), yn.numel(), cols, r4, n))
                run_other(f"norm_quant_q8_q4_k_gemv_12288x4096_N{n}", q8_step,
                          nb4 * 144 + cols * 4 + n * (cols * 4 + cols + cols // 4 + r4 * 4), 200, 20)
                if n in (1, 8):
                    run_other(f"q4_k_gemv_q8_only_12288x4096_N{n}", lambda i: must(lib.lev_hip_q4_k_gemv_q8(
                        c, ring4.data_ptr(), ring4.numel(), (i % ncopy4) * nb4 * 144, xq.data_ptr(),
                        xs.data_ptr(), xq.numel(), yn.data_ptr(), yn.numel(), cols, r4, n)),
                        nb4 * 144 + n * (cols + cols // 4 + r4 * 4), 200, 20)

        # --------------------------------------------------- Q4_K prefill GEMM
        if want("gemm"):
            tokens = 512
            xh = torch.randn(tokens, cols, device=dev, generator=gen).to(torch.float16)
            yg = torch.empty(tokens, r4, device=dev)
            flop = 2.0 * tokens * r4 * cols

            def gemm_extra(ms):
                tf = flop / (ms * 1e-3) / 1e12
                return {"TFLOPs": tf, "mfma_frac_of_fp16_peak": tf / MFMA_F16_PEAK_TFLOPS,
                        "bound": "mfma"}
            run_other("q4_k_prefill_gemm_512x12288x4096", lambda i: must(lib.lev_hip_q4_k_gemm_prefill(
                c, ring4.data_ptr(), ring4.numel(), (i % ncopy4) * nb4 * 144, xh.data_ptr(), xh.numel(),
                yg.data_ptr(), yg.numel(), cols, r4, tokens)),
                nb4 * 144 + tokens * cols * 2 + tokens * r4 * 4, int(os.environ.get("LEV_BENCH_GEMM_STEPS", "500")), int(os.environ.get("LEV_BENCH_GEMM_WARMUP", "1500")), gemm_extra)
            # 1500 warm-up launches (about 0.1 s): this kernel is bound by the matrix
            # cores, whose clock takes tens of milliseconds of load to reach its
            # sustained level (launch 40 of a cold sequence runs 25 % slower than
            # launch 2000); prefill is a long sequence of such products.
        if want("q4_k", "gemm"):
            del ring4

        # ------------------------------------------------------------- MoE
        if want("moe1", "moe64"):
            # the blocks the earlier entries freed go back to the driver: the 1 GB of pools are then
            # fresh allocations, as when this entry runs alone, not pieces of torch's cache
            torch.cuda.empty_cache()
            hidden, inter, experts, top_k = 2048, 768, 128, 8
            gu = inter * (hidden // 32) * 18
            dn = hidden * (inter // 32) * 18
            expert_bytes = 2 * gu + dn                          # 2,654,208
            npool = 3                                           # three distinct 340 MB pools (1.02 GB)
            pools_t = [make_q4_0(experts * expert_bytes // 18) for _ in range(npool)]
            # router and tokens from a generator of their own: the routing (and with it the work per
            # expert) does not depend on which other families ran before
            gen_moe = torch.Generator(device=dev)
            gen_moe.manual_seed(0x6D6F65)
            wr = 0.02 * torch.randn(experts, hidden, device=dev, generator=gen_moe)
            # the router is read from a different copy every step as well (32 MB ring)
            nrouter = 32
            wr_ring = wr.unsqueeze(0).repeat(nrouter, 1, 1).contiguous()
            pools = [ops.Context.moe_pools(p, hidden, inter, experts, 0, experts * gu, 2 * experts * gu)
                     for p in pools_t]
            import ctypes as C
            for T in (1, 64):
                if not want(f"moe{T}"):
                    continue
                yt = torch.empty(T, hidden, device=dev)
                wts = torch.empty(T, top_k, device=dev)
                if T == 1:
                    # 16 single-token inputs that route to 16 DISJOINT sets of 8 experts (N(0,1)
                    # noise plus a component along the 8 router rows of the set), so that a
                    # cycle of 16 inputs x 3 pools touches each of the 384 (pool, expert) slices
                    # exactly once: between two uses of a slice 383 others (1.0 GB) are streamed.
                    ncyc = experts // top_k
                    perm = torch.randperm(experts, device=dev, generator=gen_moe).reshape(ncyc, top_k)
                    unit = wr / wr.norm(dim=1, keepdim=True)
                    xrows = torch.randn(ncyc, hidden, device=dev, generator=gen_moe) + 9.0 * unit[perm].sum(dim=1)
                    xrows = xrows.contiguous()
                    cycle = ncyc * npool
                    ids_all = torch.empty(cycle, top_k, dtype=torch.int32, device=dev)

                    def moe_step(i):
                        k = i % cycle
                        must(lib.lev_hip_moe_layer_q4_0(
                            c, C.byref(pools[k // ncyc]), wr_ring.data_ptr() + (i % nrouter) * experts * hidden * 4,
                            None, xrows.data_ptr() + (k % ncyc) * hidden * 4, yt.data_ptr(),
                            ids_all.data_ptr() + k * top_k * 4, wts.data_ptr(), top_k, 1))
                    for i in range(cycle):
                        moe_step(i)
                    ctx.sync()
                    # what was actually routed: every (pool, expert) slice at most once per cycle
                    routed = ids_all.cpu().numpy()
                    keys = [(k // ncyc, int(e)) for k in range(cycle) for e in routed[k]]
                    assert len(set(keys)) == len(keys) == cycle * top_k, "bench inputs do not route to disjoint experts"
                    assert sorted(routed[:ncyc].reshape(-1).tolist()) == list(range(experts))
                    between = (len(keys) - 1) * expert_bytes    # distinct slice bytes between two uses of a slice
                    assert between >= 512 << 20
                    distinct = top_k
                    alg = experts * hidden * 4 + distinct * expert_bytes + 2 * hidden * 4
                    extra_fields = {"distinct_bytes_between_reuse": between,
                                    "inputs": f"{ncyc} inputs routing to disjoint expert sets x {npool} pools, "
                                              f"router read from a ring of {nrouter} copies"}
                else:
                    xt = torch.randn(T, hidden, device=dev, generator=gen_moe)
                    ids = torch.empty(T, top_k, dtype=torch.int32, device=dev)

                    def moe_step(i):
                        must(lib.lev_hip_moe_layer_q4_0(
                            c, C.byref(pools[i % npool]), wr_ring.data_ptr() + (i % nrouter) * experts * hidden * 4,
                            None, xt.data_ptr(), yt.data_ptr(), ids.data_ptr(), wts.data_ptr(), top_k, T))
                    moe_step(0)
                    ctx.sync()
                    distinct = int(torch.unique(ids).numel())
                    alg = experts * hidden * 4 + distinct * expert_bytes + 2 * T * hidden * 4
                    # a pool is used again after the two other pools have been streamed
                    extra_fields = {"distinct_bytes_between_reuse": (npool - 1) * distinct * expert_bytes,
                                    # up to 5.5 pairs per expert on average the integer grouped kernels
                                    # run: four tokens a product, a second product for an expert's pairs
                                    # five to eight, another work item (and pass) beyond
                                    "max_pairs_per_expert": int(torch.bincount(ids.flatten().long()).max())}

                def moe_extra(ms, T=T, distinct=distinct, alg=alg, extra_fields=extra_fields):
                    out = {"us_per_token": ms * 1e3 / T, "tokens": T, "distinct_experts": distinct,
                           "ideal_us_at_hbm_peak": alg / HBM_PEAK_GBS / 1e3}
                    out.update(extra_fields)
                    return out
                run_other(f"moe_layer_q4_0_T{T}", moe_step, alg, 192 if T == 1 else 48, 24, moe_extra)

            # CPU form of the same layer at T=1 (the reference's per-slot expert loop,
            # Gemma4.swift:3856-3880, behind the F32 router matvec and the CPU top-k)
            if want("moe1") and not args.skip_cpu:
                import oracle as O                              # cpu_baseline leg only
                pool_h = pools_t[0].cpu().numpy()
                wr_h = wr.cpu().numpy()
                x_h = torch.randn(hidden, generator=torch.Generator().manual_seed(7)).numpy()
                g_h, u_h, d_h = pool_h[:experts * gu], pool_h[experts * gu:2 * experts * gu], pool_h[2 * experts * gu:]
                n, t0 = 0, time.perf_counter()
                while True:
                    sc = O.f32_matvec(wr_h, experts, hidden, x_h)
                    ids_h, w_h = O.router_topk(sc, top_k)
                    O.moe_experts_f32(g_h, u_h, d_h, hidden, inter, ids_h, w_h, x_h)
                    n += 1
                    dt = time.perf_counter() - t0
                    if dt >= 6.0:
                        break
                result["cpu_moe"] = {"value": dt / n * 1e6, "unit": "us/token", "cores": 1, "kind": "port",
                                     "sample": f"{n} single-token MoE layers (router matvec + top-8 + per-slot "
                                               "expert loop in f32), one thread"}

    if "value" not in result:                                  # --only run of another family
        print(json.dumps({"only": only, "others": others}))
        return

    achieved = result["value"]
    moe1 = others.get("moe_layer_q4_0_T1", {})
    if result.get("cpu_baseline") is not None and "cpu_moe" in result:
        result["cpu_baseline"]["moe_layer_T1"] = result["cpu_moe"]
    if result.get("cpu_baseline") is not None:
        result["cpu_baseline"].update(cpu_others)
    line = {
        "metric": "Q4 GEMV achieved HBM GB/s (% of 8 TB/s); MoE layer us/token at T=1",
        "value": achieved,
        "unit": "GB/s",
        "pct_of_hbm_peak": 100.0 * achieved / HBM_PEAK_GBS,
        "moe_us_per_token_T1": moe1.get("us_per_token"),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": result["ms_per_step"],
        "ms_per_step_host_launched": eager_ms.get("q4_0", {}).get("host_launched"),
        "ms_per_step_program": eager_ms.get("q4_0", {}).get("program"),
        "ms_per_step_samples": eager_ms.get("q4_0", {}).get("samples"),
        "timing": "HIP events on the launch stream around exactly `steps` steps, enqueued behind a read-only "
                  "1 GiB cache flush that is still running when they are enqueued (cold HBM, no host latency "
                  "inside the timed region); `ms_per_step` is the " + str(eager_ms.get("q4_0", {}).get("used")) +
                  " figure (program replay from 500 steps on, host-launched steps below: a replay has about "
                  "10 us of fixed start-up)",
        "timing_note": None if eager_ms.get("q4_0", {}).get("host_kept_ahead", True) else
                       "host did not keep ahead of the device while enqueueing; program replay reported",
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "Q4_0 decode GEMV y=W.x, W 4096x4096 GGUF Q4_0, x f32[4096], "
                               "one launch per step, 64 distinct weight copies in rotation (604 MB)",
                   "in_dim": cols, "out_rows": rows, "algorithmic_bytes_per_step": q4_alg_bytes},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic_bytes(),
                     "kernel": "q4_0_mfma_gemv<1,true>",
                     "note": "achieved = 9,469,952 B / mean launch-to-launch time of the timed "
                             "region (HIP events on the launch stream)"},
        "cpu_baseline": result.get("cpu_baseline"),
        "check": result.get("check"),
        "device": ctx.device_name(),
        "others": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
