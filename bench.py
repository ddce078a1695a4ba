#!/usr/bin/env python3
"""Benchmark of the fp16 GEMV + LSTM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  A step is one pass of the batch-1 fp16 GEMV sweep
(out,in) in {(4096,4096), (16384,4096), (4096,16384), (32000,1024)}, y = W.x + b, with every operand already
resident in HBM and the weights COLD: each shape rotates over enough distinct weight copies (>= 500 MB per shape,
about 2 GB per round) that the 256 MB Infinity Cache cannot hold what the next launch reads.  `value` is the
algorithmic bytes of a step (2NK + 2K + 2N + 2N per GEMV) divided by the measured time of a step, in GB/s.
The same line carries the LSTM figure of the metric (microseconds per layer-step of the 2-layer H=1024, T=200
sequence, persistent kernel), the MFMA utilisation of the input projection, a roofline object for the dominant
kernel and the CPU baseline (LibTorch CPU at::addmm, the op the reference's atenAddmm passes through to, on the
host cores of this box).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 matrix rate
SWEEP = [(4096, 4096), (16384, 4096), (4096, 16384), (32000, 1024)]
POOL_BYTES_PER_SHAPE = 512 << 20
# HBM bytes per launch of the dominant kernel, mean over its three shapes, from rocprofv3 --pmc runs of this script, one
# shape and one counter per run (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB per dispatch, factors from --calibration-copy);
# the per-shape figures and the commands are in profiles/gemv_sweep_pmc.md, and tests/test_profiles.py recomputes this
# number from that file.  A counter reading, not something this script can measure itself.
DOMINANT_KERNEL_TRAFFIC_BYTES = 101094400


def gemv_bytes(n, k, bias=True):
    return 2 * n * k + 2 * k + (2 * n if bias else 0) + 2 * n


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the LibTorch CPU timing")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="first run three out-of-place fp32 adds over 256 MiB (read 256 MiB, write 256 MiB each): "
                         "a kernel of known traffic that scales rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--sections", default="sweep,lstm,other",
                    help="comma list of what to run: sweep (the timed steps, always run), lstm (LSTM and input projection "
                         "figures), other (the other kernels of the path), decoder (the one-launch decoder step alone, "
                         "issued eagerly; not in the default set); counter runs use one of sweep, lstm, decoder at a time")
    ap.add_argument("--lstm-modes", default="",
                    help="comma list of LSTM plan modes to time in the lstm section (0 automatic, 4 per-XCD, 2 all-CU wavefront, "
                         "1 per-step launches); default: all four, under a counter run 1 only")
    ap.add_argument("--sweep-shapes", default="",
                    help="comma list of indices into the sweep's four shapes: a profiler run that has to tell apart shapes "
                         "which launch the same kernel on the same grid (4096x4096 and 4096x16384) runs one shape at a time; "
                         "`value` then covers those shapes only and says so in config.workload")
    ap.add_argument("--resident-kernels-under-counters", action="store_true",
                    help="under rocprofv3 --pmc, also run the kernels whose workgroups wait for one another (LSTM modes 0, 2, 4, "
                         "the decoder step); without this flag a counter run refuses them")
    args = ap.parse_args()
    sections = set(args.sections.split(","))
    t_start = time.perf_counter()

    def progress(msg):
        print(f"[bench {time.perf_counter() - t_start:7.1f}s] {msg}", file=sys.stderr, flush=True)
    # rocprofv3 --pmc (it exports ROCPROF_COUNTER_COLLECTION to the process it starts) lets one dispatch run at a time and
    # reads the counters around each.  A few counter runs that dispatched kernels whose workgroups wait for one another
    # (the persistent LSTM kernels, the decoder step, the MoE step, the sliced I_X_W reducers) or replayed HIP graphs went
    # silent for minutes, while counter runs of ordinary kernels never did.  A counter run therefore leaves the `other`
    # section out and REFUSES those kernels unless --resident-kernels-under-counters asks for them by name; with the flag
    # every wait is given a short poll limit on top of its one-second bound, so that a launch whose workgroups are not
    # run together completes by itself (slowly) instead of waiting.  Every phase prints a line with the time before
    # it starts: a run that goes silent names the phase it was in.
    counter_run = bool(os.environ.get("ROCPROF_COUNTER_COLLECTION"))
    if counter_run and "other" in sections:
        sections.discard("other")
        progress("counter run detected (ROCPROF_COUNTER_COLLECTION): section 'other' is left out")
    if counter_run and not args.resident_kernels_under_counters:
        asked = [m for m in args.lstm_modes.split(",") if m and m != "1"]
        if asked or "decoder" in sections:
            print("bench.py: this is a counter run (ROCPROF_COUNTER_COLLECTION is set) and it was asked for kernels whose "
                  "workgroups wait for one another (--lstm-modes other than 1, or --sections decoder); add "
                  "--resident-kernels-under-counters to run them under counter collection", file=sys.stderr)
            return 2
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU mode (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch
    import pimaicompiler_amd as P
    from pimaicompiler_amd import _lib as L

    if not torch.cuda.is_available():
        print("bench.py needs a gfx950 GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    P.initialize(0)
    lib = L.load()
    stream = torch.cuda.current_stream()
    sh = stream.cuda_stream

    if args.calibration_copy:
        src = torch.zeros(64 << 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    # ---- operands, resident in HBM ---------------------------------------------------------------------------
    # The sweep's inputs are the seeded ones of the configuration (seed 2001 + i for shape i: W = 0.02 randn, x = 2 rand - 1,
    # b = 0.01 randn, drawn on the CPU in that order, rounded to fp16).  Launches rotate over a pool of copies of the matrix
    # that is larger than the last-level cache, so that every launch reads its matrix from HBM; copy c is the same matrix
    # with its rows rotated by c (same values, its own addresses).
    from pimaicompiler_amd import workloads
    sweep = list(enumerate(SWEEP))
    if args.sweep_shapes:
        chosen = sorted({int(i) for i in args.sweep_shapes.split(",")})
        sweep = [(i, SWEEP[i]) for i in chosen]
        if sections & {"other", "decoder"}:
            print("bench.py: --sweep-shapes goes with --sections sweep or sweep,lstm (the other sections use the sweep's matrices)",
                  file=sys.stderr)
            return 2
    shapes = []
    for i, (n, k) in sweep:
        progress(f"sweep operands {n}x{k} (seed {2001 + i})")
        w_cpu, x_cpu, b_cpu = workloads.gemv_inputs(2001 + i, n, k)
        copies = max(2, math.ceil(POOL_BYTES_PER_SHAPE / (2 * n * k)))
        pool = torch.empty((copies, n, k), dtype=torch.float16, device=dev)
        pool[0] = w_cpu.to(dev)
        for c in range(1, copies):
            pool[c] = torch.roll(pool[0], c, 0)
        x = x_cpu.reshape(k).to(dev)
        b = b_cpu.to(dev)
        y = torch.empty(n, dtype=torch.float16, device=dev)
        # (device addresses taken once: indexing a tensor per launch would cost the host more than a short kernel runs)
        shapes.append(dict(n=n, k=k, copies=copies, pool=pool, x=x, b=b, y=y, it=0, w_ptrs=[pool[c].data_ptr() for c in range(copies)],
                           x_ptr=x.data_ptr(), b_ptr=b.data_ptr(), y_ptr=y.data_ptr()))
        del w_cpu
    torch.cuda.synchronize()

    def launch(s):
        w_ptr = s["w_ptrs"][s["it"] % s["copies"]]
        s["it"] += 1
        rc = lib.pimhip_execute_gemv(s["y_ptr"], s["x_ptr"], w_ptr, s["b_ptr"], s["k"], s["n"],
                                     0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, sh)
        if rc != 0:
            raise RuntimeError(lib.pimhip_last_error().decode())

    def step():
        for s in shapes:
            launch(s)

    progress("sweep: first launches and the check against float64")
    # ---- sanity: a few rows of every shape against float64 on the host (outside any timed region) ---------------
    for s in shapes:
        launch(s)
        torch.cuda.synchronize()
        w = s["pool"][(s["it"] - 1) % s["copies"]]
        rows = torch.arange(0, s["n"], max(1, s["n"] // 32), device=dev)[:32]
        want = w[rows].double().cpu() @ s["x"].double().cpu() + s["b"][rows].double().cpu()
        err = float((s["y"][rows].double().cpu() - want).abs().max())
        if not err <= 2e-3:
            raise RuntimeError(f"GEMV {s['n']}x{s['k']} differs from the float64 product by {err}")

    # ---- the timed region: exactly K steps -----------------------------------------------------------------------
    progress(f"sweep: {args.warmup} warm-up steps, {args.steps} timed steps")
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(args.steps):
        step()
    e1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = e0.elapsed_time(e1) / args.steps
    step_bytes = sum(gemv_bytes(n, k) for _, (n, k) in sweep)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- per-shape launch durations (HIP events on the launch stream, cold rotation, back to back) ---------------
    per_shape = []
    for s in shapes:
        progress(f"sweep: per-launch duration of {s['n']}x{s['k']} and of the read-only kernel on the same matrices")
        reps = max(50, args.steps)
        for _ in range(5):
            launch(s)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(reps):
            launch(s)
        e1.record(stream)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        bts = gemv_bytes(s["n"], s["k"])
        # the floor for these bytes: a kernel that only reads the same cold matrices with the same streaming loads
        wbytes = 2 * s["n"] * s["k"]

        def probe(s=s, wbytes=wbytes):
            w_ptr = s["w_ptrs"][s["it"] % s["copies"]]
            s["it"] += 1
            lib.pimhip_probe_stream_read(w_ptr, wbytes, sh)
        for _ in range(5):
            probe()
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(reps):
            probe()
        e1.record(stream)
        torch.cuda.synchronize()
        floor_us = e0.elapsed_time(e1) * 1e3 / reps
        per_shape.append(dict(out=s["n"], **{"in": s["k"]}, us=round(us, 3), gbs=round(bts / us / 1e3, 1),
                              frac_of_peak=round(bts / us / 1e3 / HBM_PEAK_GBS, 4), read_only_kernel_us=round(floor_us, 3),
                              frac_of_read_only_kernel=round(floor_us / us, 4)))
    # Dominant kernel: gemv_mv_f16_kernel<2,4,4,4>, which runs the three in >= 4096 shapes (90 % of a step's bytes).
    dom = [(p, gemv_bytes(p["out"], p["in"])) for p in per_shape if p["in"] >= 4096] or [(p, gemv_bytes(p["out"], p["in"])) for p in per_shape]
    dom_bytes = sum(b for _, b in dom) / len(dom)
    dom_us = sum(p["us"] for p, _ in dom) / len(dom)
    achieved = dom_bytes / dom_us / 1e3
    roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4), traffic=DOMINANT_KERNEL_TRAFFIC_BYTES if len(sweep) == len(SWEEP) else None,
                    kernel="gemv_mv_f16_kernel<2,4,4,4>", bytes_per_launch=int(dom_bytes), us_per_launch=round(dom_us, 3))

    progress("sweep timed")
    # ---- LSTM: RNNT-style 2 layers, I=240, H=1024, T=200 (400 layer-steps per call) ------------------------------
    params, x, h0, c0 = workloads.lstm_inputs(3001, 240, 1024, 2, False, 200)
    # mode 0 is what a caller gets (here: the two layers as a pipeline over the XCDs, one recurrence per XCD); modes 4, 2 and
    # 1 are forced beside it: the same pipeline, the two layers as a wavefront over all CUs, one launch per step
    lstm = {"automatic": None, "per_xcd_pipeline": None, "all_cu_wavefront": None, "per_step_launches": None}
    lstm_modes = ((0, "automatic"), (4, "per_xcd_pipeline"), (2, "all_cu_wavefront"), (1, "per_step_launches"))
    if args.lstm_modes:
        wanted = [int(m) for m in args.lstm_modes.split(",")]
        lstm_modes = tuple(mn for mn in lstm_modes if mn[0] in wanted)
    elif counter_run:
        # Only the per-step launches (no workgroup of theirs waits for another) unless the modes are asked for by name.
        lstm_modes = ((1, "per_step_launches"),)
        progress("counter run detected: only LSTM mode 1 (per-step launches) runs; the persistent kernels need --lstm-modes "
                 "and --resident-kernels-under-counters")
    lstm_fallbacks = {}
    for mode, name in lstm_modes if "lstm" in sections else ():
        progress(f"LSTM mode {name}: plan")
        plan = P.LstmPlan([p.to(dev) for p in params], True, 2, False, 200)
        plan.set_mode(mode)
        if counter_run:
            # A wait that gives up costs time, not the result (the launch completes the call by itself).  With a short poll
            # limit that happens after milliseconds; and mode 0 does not time its candidates under counters.
            plan.set_spin_limit(1 << 16)
            plan.set_measure(False)
        xd, hd, cd = x.reshape(200, 240).to(dev), h0.to(dev), c0.to(dev)
        progress(f"LSTM mode {name}: 5 warm-up calls")
        for _ in range(5):
            plan.forward(xd, hd, cd)
        torch.cuda.synchronize()
        plan.status()
        # per-step mode under counters: 400 launches per call, each of them bracketed by counter reads
        reps = 5 if (counter_run and mode == 1) else 30
        progress(f"LSTM mode {name}: {reps} timed calls")
        e0.record(stream)
        for _ in range(reps):
            plan.forward(xd, hd, cd)
        e1.record(stream)
        torch.cuda.synchronize()
        plan.status()
        lstm[name] = e0.elapsed_time(e1) * 1e3 / reps / 400
        events, exchanging = plan.fallbacks()
        lstm_fallbacks[name] = events
        if events:
            progress(f"LSTM mode {name}: {events} calls had a wait that gave up and completed by themselves")
    xp_us = xp_tflops = None
    xp_shapes = []
    if "lstm" in sections:
        progress("input projection shapes")
        # input projection of layer 1 (T=200, I=1024, 4H=4096): the MFMA kernel
        xp_x = torch.randn(200, 1024, device=dev).half()
        xp_w = (0.03 * torch.randn(4096, 1024, device=dev)).half()
        # timed through the C ABI on preallocated buffers, with the weight in fragment order as an LSTM plan keeps it
        # (the figure with the plain [4H, I] weight is reported beside it)
        xp_out = torch.empty(200, 4096, dtype=torch.float32, device=dev)
        xp_packed = P.pack_projection_weight(xp_w)
        xp_times = {}
        for name_, fn_ in (("packed", lambda: lib.pimhip_input_projection_packed(xp_out.data_ptr(), xp_x.data_ptr(), xp_packed.data_ptr(),
                                                                                None, 200, 1024, 4096, sh)),
                           ("plain", lambda: lib.pimhip_input_projection(xp_out.data_ptr(), xp_x.data_ptr(), xp_w.data_ptr(), None,
                                                                         200, 1024, 4096, sh))):
            for _ in range(5):
                fn_()
            torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(100):
                fn_()
            e1.record(stream)
            torch.cuda.synchronize()
            xp_times[name_] = e0.elapsed_time(e1) * 1e3 / 100
        xp_us = xp_times["packed"]
        xp_tflops = 2 * 200 * 1024 * 4096 / xp_us / 1e6
        # every projection shape of the LSTM configurations: (T, I) with 4H = 4096, weight in fragment order
        for T_, I_ in ((200, 240), (200, 1024), (50, 1024), (50, 2048)):
            x_ = torch.randn(T_, I_, device=dev).half()
            w_ = (0.03 * torch.randn(4096, I_, device=dev)).half()
            o_ = torch.empty(T_, 4096, dtype=torch.float32, device=dev)
            pk_ = P.pack_projection_weight(w_)

            def fn_(x_=x_, pk_=pk_, o_=o_, T_=T_, I_=I_):
                lib.pimhip_input_projection_packed(o_.data_ptr(), x_.data_ptr(), pk_.data_ptr(), None, T_, I_, 4096, sh)
            for _ in range(5):
                fn_()
            torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(100):
                fn_()
            e1.record(stream)
            torch.cuda.synchronize()
            us_ = e0.elapsed_time(e1) * 1e3 / 100
            tf_ = 2 * T_ * I_ * 4096 / us_ / 1e6
            # the floor beside it: one launch that only reads the (warm) weight, as the product does once per launch;
            # no kernel that has to read those bytes in a launch of its own can be faster, whatever it computes
            def ro_(pk_=pk_):
                lib.pimhip_probe_stream_read(pk_.data_ptr(), pk_.numel() * pk_.element_size(), sh)
            for _ in range(5):
                ro_()
            torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(100):
                ro_()
            e1.record(stream)
            torch.cuda.synchronize()
            ro_us = e0.elapsed_time(e1) * 1e3 / 100
            xp_shapes.append({"T": T_, "I": I_, "four_H": 4096, "us": round(us_, 2), "tflops": round(tf_, 2),
                              "mfma_utilisation": round(tf_ / MFMA_FP16_PEAK_TFLOPS, 5),
                              "read_only_kernel_over_the_weight_us": round(ro_us, 2),
                              "mfma_utilisation_if_it_took_only_that": round(2 * T_ * I_ * 4096 / ro_us / 1e6 / MFMA_FP16_PEAK_TFLOPS, 5)})
    progress("lstm and input projection timed")

    # ---- the other kernels of the path (reported beside the headline figures, not part of `value`) ---------------
    def timed_us(fn, reps, warm=5, settle_s=0.0):
        if settle_s:
            # A burst that saturates HBM leaves the GPU in a state (clocks) in which the next few hundred short launches
            # run up to 20 % slower (measured: 9.8 -> 11.6 us for the 4096 x 4096 I_X_W product right after 100 grouped
            # sweeps, back to 9.8 after half a second).  The side figures below each start from the same idle state.
            torch.cuda.synchronize()
            time.sleep(settle_s)
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(reps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    def graph_timed_us(fn, n):
        """Device-side time per call of fn(stream_handle): n calls captured into one HIP graph and replayed, so that the
        host's cost of issuing a launch from Python (about 5 us through ctypes) is outside the figure."""
        g_ = torch.cuda.CUDAGraph()
        side_ = torch.cuda.Stream()
        side_.wait_stream(stream)
        with torch.cuda.stream(side_):
            with torch.cuda.graph(g_, stream=side_):
                for _ in range(n):
                    fn(torch.cuda.current_stream().cuda_stream)
        stream.wait_stream(side_)
        torch.cuda.synchronize()
        return timed_us(g_.replay, 5, warm=3, settle_s=0.3) / n

    other = {}
    if "other" in sections:
        progress("other: GNMT stack")
        # GNMT-style stack: four at::lstm calls (L0 bidirectional I=1024, L1 I=2048, L2, L3 I=1024), T=50: 250 layer-steps
        gn = []
        seq = torch.randn(50, 1024, device=dev).half()
        for li, (in_w, bidir) in enumerate([(1024, True), (2048, False), (1024, False), (1024, False)]):
            prm, _, h0g, c0g = workloads.lstm_inputs(4001 + li, in_w, 1024, 1, bidir, 50)
            gn.append((P.LstmPlan([q.to(dev) for q in prm], True, 1, bidir, 50), h0g.to(dev), c0g.to(dev)))

        def gnmt_stack():
            cur = seq
            for plan_g, hg, cg in gn:
                cur, _, _ = plan_g.forward(cur, hg, cg)

        other["gnmt_lstm_stack_us_per_layer_step"] = round(timed_us(gnmt_stack, 30) / 250, 3)
        # the same stack after rewrite.fuse_lstm_stack: the three one-direction layers as ONE aten::lstm with num_layers = 3
        # (a pipeline over the XCDs in one launch), behind the bidirectional layer's call
        plan_123 = P.LstmPlan([q for pl, _, _ in gn[1:] for q in pl.params], True, 3, False, 50)
        h_123 = torch.cat([hg for _, hg, _ in gn[1:]], 0).contiguous()
        c_123 = torch.cat([cg for _, _, cg in gn[1:]], 0).contiguous()

        def gnmt_stack_two_calls():
            cur, _, _ = gn[0][0].forward(seq, gn[0][1], gn[0][2])
            plan_123.forward(cur, h_123, c_123)

        other["gnmt_lstm_stack_us_per_layer_step_layers_1_to_3_as_one_call"] = round(timed_us(gnmt_stack_two_calls, 30) / 250, 3)
        # the encoder as GNMT wires it, with residual sums around its two upper layers: one aten::lstm and one aten::add per
        # layer as the reference runs them, against the one call rewrite.fuse_lstm_stack makes of them
        def gnmt_upper_layers_op_by_op():
            cur = l0_out
            for li, (plan_g, hg, cg) in enumerate(gn[1:]):
                yl, _, _ = plan_g.forward(cur, hg, cg)
                cur = P.aten_add(yl, cur) if li >= 1 else yl

        l0_out = gn[0][0].forward(seq, gn[0][1], gn[0][2])[0]
        op_by_op_us = timed_us(gnmt_upper_layers_op_by_op, 30)
        plan_123.set_residual(1)
        other["gnmt_encoder_upper_layers_with_residual_sums"] = {
            "three_lstm_calls_and_two_adds_us": round(op_by_op_us, 2),
            "one_call_us": round(timed_us(lambda: plan_123.forward(l0_out, h_123, c_123), 30), 2), "steps": 50}
        plan_123.set_residual(None)
        # the same four calls (eight launches) replayed from a HIP graph
        other["gnmt_lstm_stack_us_per_layer_step_hip_graph"] = round(graph_timed_us(lambda _s: gnmt_stack(), 1) / 250, 3)
        progress("other: decoder cell and grouped sweep")
        # one decoder step (seq_len 1, I = H = 1024): the fused step kernel, W_ih and W_hh streamed once (16.8 MB)
        prm, _, h0d, c0d = workloads.lstm_inputs(4101, 1024, 1024, 1, False, 1)
        plan_d = P.LstmPlan([q.to(dev) for q in prm], True, 1, False, 1)
        xd1, h0d, c0d = torch.randn(1, 1024, device=dev).half(), h0d.to(dev).contiguous(), c0d.to(dev).contiguous()
        yd1, hnd, cnd = torch.empty(1024, dtype=torch.float16, device=dev), torch.empty_like(h0d), torch.empty_like(c0d)
        # (these small launches are timed through the C ABI on preallocated buffers: the operator layer's Python
        # bookkeeping costs more than the kernels)
        def decode_launch(s_h=sh):
            lib.pimhip_lstm_forward(plan_d._handle, xd1.data_ptr(), h0d.data_ptr(), c0d.data_ptr(), yd1.data_ptr(),
                                    hnd.data_ptr(), cnd.data_ptr(), 1, s_h)
        us = graph_timed_us(decode_launch, 32)
        # the floor beside it: a launch that only reads as many (warm) bytes as the step's two weight matrices
        probe_buf = torch.empty(2 * 4096 * 1024, dtype=torch.float16, device=dev).normal_()

        def decode_floor(s_h=sh):
            lib.pimhip_probe_stream_read(probe_buf.data_ptr(), probe_buf.numel() * 2, s_h)
        other["lstm_decode_step"] = {"us": round(us, 3), "gbs": round((2 * 4096 * 2048 + 8 * 4096) / us / 1e3, 1),
                                     "issued_from_python_us": round(timed_us(decode_launch, 200), 3),
                                     "read_only_kernel_us": round(graph_timed_us(decode_floor, 32), 3)}
        # the same sweep as ONE grouped launch (executeMultiStream's siblings in one grid), cold
        def grouped():
            ws = []
            for s_ in shapes:
                ws.append(s_["pool"][s_["it"] % s_["copies"]])
                s_["it"] += 1
            P.execute_gemv_group([s_["x"] for s_ in shapes], ws, [s_["b"] for s_ in shapes])
        us = timed_us(grouped, 100)
        other["gemv_sweep_grouped_launch"] = {"us": round(us, 2), "gbs": round(step_bytes / us / 1e3, 1)}
        progress("other: sweep in the I_X_W order")
        # the sweep in the other operand order (y = x . A, A [in, out] row-major: the un-swapped addmm / matmul route); the
        # same cold pools, read as [in, out]
        vm_times = []
        for s_ in shapes:
            xv = (2 * torch.rand(s_["k"], device=dev) - 1).half()

            def vm_launch(s_=s_, xv_ptr=xv.data_ptr()):
                w_ptr = s_["w_ptrs"][s_["it"] % s_["copies"]]
                s_["it"] += 1
                rc = lib.pimhip_execute_gemv(s_["y_ptr"], xv_ptr, w_ptr, s_["b_ptr"], s_["k"], s_["n"], 0,
                                             L.PIMHIP_ACT_NONE, L.PIMHIP_I_X_W, sh)
                if rc != 0:
                    raise RuntimeError(lib.pimhip_last_error().decode())
            us = timed_us(vm_launch, 50, settle_s=0.3)
            # a CONSTANT weight of this order is laid out transposed once at preload (executor.preload_constants), and the
            # same call then runs the W_X_I kernel: the sweep's own figure for the shape
            mv_us = next(p_["us"] for p_ in per_shape if p_["out"] == s_["n"] and p_["in"] == s_["k"])
            vm_times.append({"out": s_["n"], "in": s_["k"], "us": round(us, 2), "gbs": round(gemv_bytes(s_["n"], s_["k"]) / us / 1e3, 1),
                             "constant_weight_laid_out_at_preload_us": mv_us,
                             "gbs_constant_weight": round(gemv_bytes(s_["n"], s_["k"]) / mv_us / 1e3, 1)})
        other["gemv_vm_order"] = vm_times
        progress("other: 1024x1024 GEMV and the C++ operators")
        # the 1024 x 1024 GEMV of the reference's own unit-test size class (2 MB: launch-bound), cold rotation over 64 copies
        c1_pool = (0.02 * torch.randn(64, 1024, 1024, device=dev)).half()
        c1_x, c1_b, c1_y = torch.randn(1024, device=dev).half(), torch.randn(1024, device=dev).half(), torch.empty(1024, dtype=torch.float16, device=dev)
        c1_it = [0]

        def c1_launch(s_h=sh):
            c1_it[0] += 1
            lib.pimhip_execute_gemv(c1_y.data_ptr(), c1_x.data_ptr(), c1_pool[c1_it[0] % 64].data_ptr(), c1_b.data_ptr(), 1024, 1024, 0,
                                    L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, s_h)
        # launches this short are issued faster by the GPU than Python can enqueue them: the first figure is the
        # device's (64 launches replayed from a HIP graph), the second what a Python caller sees
        other["gemv_1024x1024_us"] = round(graph_timed_us(c1_launch, 64), 3)
        other["gemv_1024x1024_issued_from_python_us"] = round(timed_us(c1_launch, 200), 3)
        # The per-token calls of a decoding loop through the C++ operators with the reference's signatures: what one call
        # costs the host thread (shape logic, output allocation, launch; 300 calls in a row from C++, nothing synchronises
        # inside the loop) beside what its kernels take on the device (the same launches replayed from a HIP graph).
        try:
            from pimaicompiler_amd import _aten_ops_pimhip as cpp_ops
        except ImportError:
            cpp_ops = None
        if cpp_ops is not None:
            cpp_ops.initialize(0)
            c1_w, c1_w_t, c1_x2 = c1_pool[0], c1_pool[0].t(), c1_x.view(1, 1024)
            host = {}

            def host_us(op, tensors, prm=()):
                cpp_ops.opHostMicroseconds(op, list(tensors), list(prm), 30)
                torch.cuda.synchronize()
                e0.record(stream)
                us_h = cpp_ops.opHostMicroseconds(op, list(tensors), list(prm), 300)
                e1.record(stream)
                torch.cuda.synchronize()
                return round(us_h, 3), round(e0.elapsed_time(e1) * 1e3 / 300, 3)
            gemv_dev_us = other["gemv_1024x1024_us"]
            for name_, op_, ts_ in (("customAtenAddmm_1024x1024", "addmm", (c1_b, c1_x2, c1_w_t)),
                                    ("customAtenMatmul_1024x1024", "matmul", (c1_w, c1_x.view(1024, 1))),
                                    ("atenLinear_1024x1024", "linear", (c1_x2, c1_w, c1_b))):
                h_, s_ = host_us(op_, ts_)
                host[name_] = {"host_us_per_call": h_, "us_per_call_on_the_stream": s_, "kernel_us": gemv_dev_us}
            # what of that is the library call under the three operators (pimhip_execute_gemv, issued from the same C++ loop):
            # almost all of it, and almost all of that is the HIP runtime's kernel launch
            h_, s_ = host_us("c_abi_gemv", (c1_y, c1_x, c1_w, c1_b))
            host["pimhip_execute_gemv_1024x1024"] = {"host_us_per_call": h_, "us_per_call_on_the_stream": s_, "kernel_us": gemv_dev_us}
            # atenLstm1 at seq_len 1: one layer of H = I = 1024 (a GNMT decoder cell), and the RNNT prediction network's two
            # layers of H = I = 320; device time = the calls' launches on preallocated buffers, replayed from a graph
            for name_, (I_, H_, L_) in (("atenLstm1_seq_len_1_H1024", (1024, 1024, 1)), ("atenLstm1_seq_len_1_H320_two_layers", (320, 320, 2))):
                prm_, x_, h0_, c0_ = workloads.lstm_inputs(4201 + L_, I_, H_, L_, False, 1)
                prm_ = [q.to(dev) for q in prm_]
                x_, h0_, c0_ = x_.to(dev), h0_.to(dev).contiguous(), c0_.to(dev).contiguous()
                y_, hn_, cn_ = cpp_ops.atenLstm1(x_, [h0_, c0_], prm_, True, L_, 0.0, False, False, False)
                plan_ = P.LstmPlan(prm_, True, L_, False, 1)

                def lstm_launch(s_h=sh, plan_=plan_, x_=x_, h0_=h0_, c0_=c0_, y_=y_, hn_=hn_, cn_=cn_):
                    lib.pimhip_lstm_forward(plan_._handle, x_.data_ptr(), h0_.data_ptr(), c0_.data_ptr(), y_.data_ptr(),
                                            hn_.data_ptr(), cn_.data_ptr(), 1, s_h)
                dev_us = round(graph_timed_us(lstm_launch, 32), 3)
                h_, s_ = host_us("lstm1", (x_, h0_, c0_), prm_)
                hi_, si_ = host_us("lstm1_into", (x_, h0_, c0_, y_, hn_, cn_), prm_)
                host[name_] = {"host_us_per_call": h_, "us_per_call_on_the_stream": s_, "kernel_us": dev_us,
                               "into_caller_buffers_host_us_per_call": hi_, "into_caller_buffers_us_per_call_on_the_stream": si_}
            other["cpp_operators_per_token_calls"] = host
        progress("other: MoE step")
        # MoE FFN decode step (router 768 -> 8, then one expert 768 -> 3072 ReLU -> 768): three dependent launches on
        # resident (warm) weights, the expert fixed so that no host round trip for the argmax is inside the figure
        wr, w1, w2 = (0.02 * torch.randn(8, 768, device=dev)).half(), (0.02 * torch.randn(3072, 768, device=dev)).half(), \
            (0.02 * torch.randn(768, 3072, device=dev)).half()
        tok, logits = torch.randn(768, device=dev).half(), torch.empty(8, dtype=torch.float16, device=dev)
        hid, yo = torch.empty(3072, dtype=torch.float16, device=dev), torch.empty(768, dtype=torch.float16, device=dev)

        def moe_step(s_h=sh):
            lib.pimhip_execute_gemv(logits.data_ptr(), tok.data_ptr(), wr.data_ptr(), None, 768, 8, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, s_h)
            lib.pimhip_execute_gemv(hid.data_ptr(), tok.data_ptr(), w1.data_ptr(), None, 768, 3072, 0, L.PIMHIP_ACT_RELU, L.PIMHIP_W_X_I, s_h)
            lib.pimhip_execute_gemv(yo.data_ptr(), hid.data_ptr(), w2.data_ptr(), None, 3072, 768, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, s_h)
        other["moe_ffn_step_three_gemvs_us"] = round(graph_timed_us(moe_step, 32), 3)
        other["moe_ffn_step_issued_from_python_us"] = round(timed_us(moe_step, 200), 3)
        # the same block as ONE launch that also picks the expert (router, argmax on the GPU, W1[e], W2[e]; eight experts),
        # and as the reference's interpreter has to run it: the argmax read back on the host between the launches
        w1s = [w1] + [(0.02 * torch.randn(3072, 768, device=dev)).half() for _ in range(7)]
        w2s = [w2] + [(0.02 * torch.randn(768, 3072, device=dev)).half() for _ in range(7)]
        moe_plan = P.MoePlan((wr, None), w1s, w2s)
        y_one, e_one = torch.empty(768, dtype=torch.float16, device=dev), torch.empty(1, dtype=torch.int32, device=dev)
        moe_one = moe_plan.bind(tok, y_one, logits, e_one)
        moe_one()
        torch.cuda.synchronize()

        def moe_host_routed():
            lib.pimhip_execute_gemv(logits.data_ptr(), tok.data_ptr(), wr.data_ptr(), None, 768, 8, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, sh)
            e = int(torch.argmax(logits))
            lib.pimhip_execute_gemv(hid.data_ptr(), tok.data_ptr(), w1s[e].data_ptr(), None, 768, 3072, 0, L.PIMHIP_ACT_RELU, L.PIMHIP_W_X_I, sh)
            lib.pimhip_execute_gemv(yo.data_ptr(), hid.data_ptr(), w2s[e].data_ptr(), None, 3072, 768, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, sh)
        moe_host_routed()
        torch.cuda.synchronize()
        other["moe_ffn_step_one_launch"] = {
            "us": round(graph_timed_us(lambda s_: moe_one(s_), 32), 3),
            "issued_from_python_us": round(timed_us(moe_one, 200), 3),
            "three_gemvs_with_the_expert_chosen_on_the_host_us": round(timed_us(moe_host_routed, 100), 3),
            "max_abs_diff_to_the_three_gemvs": round(float((y_one.float() - yo.float()).abs().max()), 6),
            "expert": int(e_one.item())}
        moe_plan.status()
        progress("other: RNNT joint network, add, attention context")
        # RNNT joint network, one (t, u) step: relu(W1[512, 1344] . cat(f[1024], g[320]) + b1), then W2[29, 512] . + b2.  The
        # reference's RemoveCatForAddmm makes two dependent products of the first layer (three launches per step); one launch
        # that reads f and g where they lie leaves two.
        jw1, jb1 = (0.03 * torch.randn(512, 1344, device=dev)).half(), (0.05 * torch.randn(512, device=dev)).half()
        jw2, jb2 = (0.05 * torch.randn(29, 512, device=dev)).half(), (0.05 * torch.randn(29, device=dev)).half()
        jw1a, jw1b = jw1[:, :1024].contiguous(), jw1[:, 1024:].contiguous()
        jf, jg = torch.randn(1024, device=dev).half(), torch.randn(320, device=dev).half()
        jmid, jhid, jout = (torch.empty(n_, dtype=torch.float16, device=dev) for n_ in (512, 512, 29))

        def joint_three(s_h=sh):
            lib.pimhip_execute_gemv(jmid.data_ptr(), jf.data_ptr(), jw1a.data_ptr(), jb1.data_ptr(), 1024, 512, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, s_h)
            lib.pimhip_execute_gemv(jhid.data_ptr(), jg.data_ptr(), jw1b.data_ptr(), jmid.data_ptr(), 320, 512, 0, L.PIMHIP_ACT_RELU, L.PIMHIP_W_X_I, s_h)
            lib.pimhip_execute_gemv(jout.data_ptr(), jhid.data_ptr(), jw2.data_ptr(), jb2.data_ptr(), 512, 29, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, s_h)

        def joint_two(s_h=sh):
            lib.pimhip_execute_gemv_cat2(jhid.data_ptr(), jf.data_ptr(), 1024, jg.data_ptr(), 320, jw1.data_ptr(), jb1.data_ptr(), 512, 0,
                                         L.PIMHIP_ACT_RELU, s_h)
            lib.pimhip_execute_gemv(jout.data_ptr(), jhid.data_ptr(), jw2.data_ptr(), jb2.data_ptr(), 512, 29, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, s_h)
        joint_three()
        ref_out = jout.clone()
        joint_two()
        torch.cuda.synchronize()
        other["rnnt_joint_step"] = {"three_launches_us": round(graph_timed_us(joint_three, 32), 3),
                                    "two_launches_us": round(graph_timed_us(joint_two, 32), 3),
                                    "max_abs_diff": round(float((jout.float() - ref_out.float()).abs().max()), 6)}
        # A whole (t, u) step of the transducer's greedy loop: the prediction network (2 LSTM layers, H = I = 320, seq_len 1) and
        # the joint network, as ONE launch (pimhip_rnnt_step) and as the four launches it replaces (two cells, cat2 product,
        # 512 -> 29 product), all replayed from graphs; and the step after a blank, where only the joint network runs.
        rn_prm, rn_x, rn_h, rn_c = workloads.lstm_inputs(4301, 320, 320, 2, False, 1)
        rn_prm = [q.to(dev) for q in rn_prm]
        rn_x = rn_x.reshape(320).to(dev)
        rn_h, rn_c = (0.1 * torch.randn(2, 320, device=dev)).half(), (0.1 * torch.randn(2, 320, device=dev)).half()
        rn_hn, rn_cn = torch.empty_like(rn_h), torch.empty_like(rn_c)
        rn_logits = torch.empty(29, dtype=torch.float16, device=dev)
        rn_plan = P.RnntPlan(rn_prm, True, 2, (jw1, jb1, jw2, jb2))
        rn_full = rn_plan.bind(rn_x, rn_h, rn_c, jf, rn_hn, rn_cn, rn_logits)
        rn_blank = rn_plan.bind(None, rn_hn, None, jf, None, None, rn_logits, run_prediction=False)
        rn_lstm = P.LstmPlan(rn_prm, True, 2, False, 1)
        rn_y, rn_hn2, rn_cn2 = torch.empty(1, 320, dtype=torch.float16, device=dev), torch.empty_like(rn_h), torch.empty_like(rn_c)

        def rnnt_four(s_h=sh):
            lib.pimhip_lstm_forward(rn_lstm._handle, rn_x.data_ptr(), rn_h.data_ptr(), rn_c.data_ptr(), rn_y.data_ptr(), rn_hn2.data_ptr(),
                                    rn_cn2.data_ptr(), 1, s_h)
            lib.pimhip_execute_gemv_cat2(jhid.data_ptr(), jf.data_ptr(), 1024, rn_y.data_ptr(), 320, jw1.data_ptr(), jb1.data_ptr(), 512, 0,
                                         L.PIMHIP_ACT_RELU, s_h)
            lib.pimhip_execute_gemv(jout.data_ptr(), jhid.data_ptr(), jw2.data_ptr(), jb2.data_ptr(), 512, 29, 0, L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, s_h)
        rn_full()
        rnnt_four()
        torch.cuda.synchronize()
        rn_events = rn_plan.fallbacks()[0]
        other["rnnt_step_one_launch"] = {
            "us": round(graph_timed_us(lambda s_: rn_full(s_), 32), 3),
            "issued_from_python_us": round(timed_us(rn_full, 200), 3),
            "four_launches_us": round(graph_timed_us(rnnt_four, 32), 3),
            "four_launches_issued_from_python_us": round(timed_us(rnnt_four, 200), 3),
            "after_a_blank_us": round(graph_timed_us(lambda s_: rn_blank(s_), 32), 3),
            "after_a_blank_two_launches_us": other["rnnt_joint_step"]["two_launches_us"],
            "bytes": 2 * (2 * 4 * 320 * 640 + 512 * 1344 + 29 * 512),
            "max_abs_diff_of_states_to_the_four_launches": round(max(float((rn_hn.float() - rn_hn2.float()).abs().max()),
                                                                      float((rn_cn.float() - rn_cn2.float()).abs().max())), 6),
            "max_abs_diff_of_logits_to_the_four_launches": round(float((rn_logits.float() - jout.float()).abs().max()), 6),
            "waits_that_gave_up": rn_plan.fallbacks()[0] - rn_events}
        # The whole greedy loop over an utterance in one launch (pimhip_rnnt_greedy_decode), timed on its two kinds of step:
        # with the joint network's bias pushed towards the blank every frame passes with one step of the joint network alone;
        # pushed away from it every step emits a symbol and runs the prediction network (30 per frame).  Beside them the same
        # loop driven from the host: one pimhip_rnnt_step and one read of the argmax per iteration.
        progress("other: RNNT greedy decoding loop in one launch")
        gd_T, gd_blank = 400, 28
        gd_enc = torch.randn(gd_T, 1024, device=dev).half()
        gd_emb, gd_x0 = torch.randn(29, 320, device=dev).half(), torch.zeros(320, dtype=torch.float16, device=dev)
        greedy = {}
        for kind, push, frames in (("after_a_blank", 20.0, gd_T), ("with_a_symbol", -20.0, 40)):
            b2 = jb2.clone()
            b2[gd_blank] += push
            gd_plan = P.RnntPlan(rn_prm, True, 2, (jw1, jb1, jw2, b2))
            enc_k = gd_enc[:frames]
            _, gd_res, _, _ = gd_plan.greedy_decode(enc_k, gd_emb, gd_x0, gd_blank)
            torch.cuda.synchronize()
            steps_k = int(gd_res[2])
            us = timed_us(lambda: gd_plan.greedy_decode(enc_k, gd_emb, gd_x0, gd_blank), 10)
            # the host's loop over the first frames of the same utterance
            h_, c_ = torch.zeros(2, 320, dtype=torch.float16, device=dev), torch.zeros(2, 320, dtype=torch.float16, device=dev)
            hn_, cn_ = torch.empty_like(h_), torch.empty_like(c_)
            lg_ = torch.empty(29, dtype=torch.float16, device=dev)
            n_host = 200
            first = gd_plan.bind(gd_x0, h_, c_, enc_k[0], hn_, cn_, lg_)
            full_ = gd_plan.bind(gd_emb[3], h_, c_, enc_k[0], hn_, cn_, lg_)
            blank_ = gd_plan.bind(None, hn_, None, enc_k[1], None, None, lg_, run_prediction=False)
            first()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n_host):
                (blank_ if kind == "after_a_blank" else full_)()
                k_ = int(torch.argmax(lg_))          # the read that decides the next iteration
            host_us = (time.perf_counter() - t0) / n_host * 1e6
            greedy[kind] = {"steps": steps_k, "us_per_step": round(us / max(steps_k, 1), 3),
                            "driven_from_the_host_us_per_step": round(host_us, 2),
                            "one_workgroup_decoded_alone": int(gd_res[3]), "waits_that_gave_up": gd_plan.fallbacks()[0]}
        other["rnnt_greedy_decode_one_launch"] = greedy
        # residual add (fp16, c = a + b): 32 Mi elements (6 bytes each) and the decoder's 1024-element case
        big_a, big_b = torch.randn(32 << 20, device=dev).half().view(-1, 1024), torch.randn(32 << 20, device=dev).half().view(-1, 1024)
        big_c = torch.empty_like(big_a)
        us = timed_us(lambda: P.aten_add(big_a, big_b, out=big_c), 50)
        other["add_32Mi"] = {"us": round(us, 2), "gbs": round(6 * (32 << 20) / us / 1e3, 1)}
        sa, sb = big_a[:1].reshape(1, 1, 1024), big_b[:1].reshape(1, 1, 1024)
        def add_launch(s_h=sh):
            lib.pimhip_execute_add(sa.data_ptr(), sa.data_ptr(), sb.data_ptr(), 1, 1024, 0, s_h)
        other["add_1024_us"] = round(graph_timed_us(add_launch, 64), 3)
        other["add_1024_issued_from_python_us"] = round(timed_us(add_launch, 200), 3)
        del big_a, big_b, big_c
        # attention context: y[1, 1024] = p[1, 50] . enc[50, 1024], stored to three buffers
        pa, enc = torch.rand(1, 1, 50, device=dev).half(), torch.randn(1, 50, 1024, device=dev).half()
        dsts = [torch.empty(1024, dtype=torch.float16, device=dev) for _ in range(3)]
        import ctypes
        dst_arr = (ctypes.c_void_p * 3)(*[d_.data_ptr() for d_ in dsts])
        def bmm_launch(s_h=sh):
            lib.pimhip_execute_bmm(dst_arr, 3, pa.data_ptr(), enc.data_ptr(), 50, 1024, s_h)
        other["bmm_50x1024_three_destinations_us"] = round(graph_timed_us(bmm_launch, 64), 3)
        other["bmm_50x1024_issued_from_python_us"] = round(timed_us(bmm_launch, 200), 3)
        progress("other: decoder step (eight launches, one launch)")
        # a whole decoder step (4 LSTM layers at seq_len 1, attention context into three buffers, two residual adds,
        # the 1024 -> 32000 classifier): 8 launches, issued one by one and replayed from a HIP graph
        kq = 1.0 / 32.0
        dplans, dstate = [], []
        for in_w in (1024, 2048, 2048, 2048):
            prm_d = [((2 * torch.rand(sh_, device=dev) - 1) * kq).half() for sh_ in ((4096, in_w), (4096, 1024), (4096,), (4096,))]
            dplans.append(P.LstmPlan(prm_d, True, 1, False, 1))
            dstate.append((torch.zeros(1, 1024, dtype=torch.float16, device=dev), torch.zeros(1, 1024, dtype=torch.float16, device=dev)))
        d_x = torch.randn(1, 1024, device=dev).half()
        d_cat = [torch.zeros(1, 2048, dtype=torch.float16, device=dev) for _ in range(3)]
        d_y = [torch.zeros(1, 1024, dtype=torch.float16, device=dev) for _ in range(4)]
        d_hn = [torch.zeros(1, 1024, dtype=torch.float16, device=dev) for _ in range(4)]
        d_cn = [torch.zeros(1, 1024, dtype=torch.float16, device=dev) for _ in range(4)]
        d_res = [torch.zeros(1, 1024, dtype=torch.float16, device=dev) for _ in range(2)]
        d_logits = torch.zeros(32000, dtype=torch.float16, device=dev)
        d_ctx = [c_.view(-1)[1024:] for c_ in d_cat]
        d_y0 = d_cat[0].view(-1)[:1024].view(1, 1024)
        d_w = shapes[3]["pool"][0]

        d_y1, d_res0 = (c_.view(-1)[:1024].view(1, 1024) for c_ in d_cat[1:])   # heads of the next layers' inputs

        def decoder_step():
            # every result is stored where its consumer reads it (the heads of the concatenation buffers): no copies
            dplans[0].forward(d_x, *dstate[0], out=(d_y0, d_hn[0], d_cn[0]))
            P.aten_bmm(pa, enc, outs=d_ctx)
            dplans[1].forward(d_cat[0], *dstate[1], out=(d_y1, d_hn[1], d_cn[1]))
            dplans[2].forward(d_cat[1], *dstate[2], out=(d_y[2], d_hn[2], d_cn[2]))
            P.aten_add(d_y[2], d_y1, out=d_res0)
            dplans[3].forward(d_cat[2], *dstate[3], out=(d_y[3], d_hn[3], d_cn[3]))
            P.aten_add(d_y[3], d_res0, out=d_res[1])
            lib.pimhip_execute_gemv(d_logits.data_ptr(), d_res[1].data_ptr(), d_w.data_ptr(), None, 1024, 32000, 0,
                                    L.PIMHIP_ACT_NONE, L.PIMHIP_W_X_I, torch.cuda.current_stream().cuda_stream)
        eager_us = timed_us(decoder_step, 100, settle_s=0.3)
        # (replayed: sixteen steps per graph, as a decoding loop would record them; two graph launches are 15 us apart on
        # the device whatever they hold, which a graph of one step would add to every step)
        graph_us = graph_timed_us(lambda _s: decoder_step(), 16)
        other["decoder_step_8_launches"] = {"issued_one_by_one_us": round(eager_us, 2), "hip_graph_replay_us": round(graph_us, 2),
                                             "bytes": 4 * 4096 * 1024 * 2 + (4096 * 1024 + 3 * 4096 * 2048) * 2 + 32000 * 1024 * 2}
        # the same step as ONE launch (pimhip_decoder_step): same weights, state, attention weights and classifier; the
        # context columns of W_ih are multiplied with the encoder outputs once per sentence (set_encoder, timed beside it)
        fplan = P.DecoderPlan([q for pl_ in dplans for q in pl_.params], True, 4, first_takes_context=False, first_residual_layer=2,
                              classifier=(d_w, None))
        f_hn = [torch.zeros(1024, dtype=torch.float16, device=dev) for _ in range(4)]
        f_cn = [torch.zeros(1024, dtype=torch.float16, device=dev) for _ in range(4)]
        f_logits = torch.zeros(32000, dtype=torch.float16, device=dev)
        enc2d = enc.view(50, 1024)
        fstep = fplan.bind(d_x.view(-1), [h_.view(-1) for h_, _ in dstate], [c_.view(-1) for _, c_ in dstate], att=pa.view(-1), enc=enc2d,
                           hn=f_hn, cn=f_cn, logits=f_logits)
        fstep()
        decoder_step()
        torch.cuda.synchronize()
        fplan.status()
        fused_err = float((f_logits.float() - d_logits.float()).abs().max())
        if not fused_err <= 5e-3:
            raise RuntimeError(f"fused decoder step differs from the operator-by-operator step by {fused_err}")
        fused_eager_us = timed_us(fstep, 200, settle_s=0.3)
        fused_graph_us = graph_timed_us(lambda s_: fstep(s_), 16)
        fplan.status()

        def reproject():
            fplan.set_encoder(enc2d)
        # the floor beside it: one launch that only reads as many warm bytes as the step has weights
        dec_step_bytes = (2 * 4096 * 1024 + 3 * 2 * 4096 * 1024) * 2 + 3 * 4096 * 50 * 4 + 32000 * 1024 * 2
        probe_buf = torch.randn(dec_step_bytes // 4, device=dev)
        probe_us = timed_us(lambda: lib.pimhip_probe_stream_read(probe_buf.data_ptr(), dec_step_bytes // 16 * 16, sh), 100, settle_s=0.3)
        del probe_buf
        other["decoder_step_one_launch"] = {
            "issued_from_python_us": round(fused_eager_us, 2), "hip_graph_replay_us": round(fused_graph_us, 2),
            "read_only_kernel_us": round(probe_us, 2),
            "bytes": dec_step_bytes,
            "max_abs_diff_of_logits_to_the_8_launch_step": round(fused_err, 6),
            "set_encoder_once_per_sentence_us": round(timed_us(reproject, 20), 2),
            "waits_that_gave_up": fplan.fallbacks()[0]}
        progress("other: the reference's own GEMV kernel")
        # the reference's own HIP GEMV (custom_ops.h addmv_kernel_Axy, compiled from its tree) on the same cold weights
        from oracle import oracle  # the loader of the reference's own kernels, nothing else of the oracle
        ref = oracle.ref_lib()
        if ref is not None:
            ref_times = []
            for s_ in shapes:
                def ref_launch(s_=s_):
                    w = s_["pool"][s_["it"] % s_["copies"]]
                    s_["it"] += 1
                    ref.ref_addmv_Axy(sh, s_["b"].data_ptr(), w.data_ptr(), s_["x"].data_ptr(), s_["y"].data_ptr(), s_["n"], s_["k"], 0)
                us = timed_us(ref_launch, 30, settle_s=0.3)
                ref_times.append({"out": s_["n"], "in": s_["k"], "us": round(us, 2), "gbs": round(gemv_bytes(s_["n"], s_["k"]) / us / 1e3, 1)})
            other["reference_hip_gemv_kernel"] = ref_times

    progress("other kernels timed")
    # ---- the one-launch decoder step alone, issued eagerly: what a counter run of that kernel uses (no graph is recorded
    # or replayed here, so the section may run under rocprofv3 --pmc) ------------------------------------------------
    if "decoder" in sections:
        progress("decoder section: plan")
        kq = 1.0 / 32.0
        dprm = []
        for in_w in (1024, 2048, 2048, 2048):
            dprm += [((2 * torch.rand(sh_, device=dev) - 1) * kq).half() for sh_ in ((4096, in_w), (4096, 1024), (4096,), (4096,))]
        cls_w = shapes[3]["pool"][0]
        eplan = P.DecoderPlan(dprm, True, 4, first_takes_context=False, first_residual_layer=2, classifier=(cls_w, None))
        e_x = torch.randn(1024, device=dev).half()
        e_h = [torch.zeros(1024, dtype=torch.float16, device=dev) for _ in range(4)]
        e_c = [torch.zeros(1024, dtype=torch.float16, device=dev) for _ in range(4)]
        e_hn = [torch.zeros(1024, dtype=torch.float16, device=dev) for _ in range(4)]
        e_cn = [torch.zeros(1024, dtype=torch.float16, device=dev) for _ in range(4)]
        e_att = torch.softmax(torch.randn(50, device=dev), 0).half()
        e_enc = torch.randn(50, 1024, device=dev).half()
        e_logits = torch.zeros(32000, dtype=torch.float16, device=dev)
        estep = eplan.bind(e_x, e_h, e_c, att=e_att, enc=e_enc, hn=e_hn, cn=e_cn, logits=e_logits)
        if counter_run:
            eplan.set_spin_limit(1 << 16)  # a step whose workgroups are not run together reports that after milliseconds
        progress("decoder section: first step")
        estep()
        torch.cuda.synchronize()
        eplan.status()
        n_steps = 20 if counter_run else 200
        progress(f"decoder section: {n_steps} steps")
        other["decoder_step_one_launch_eager_section"] = {
            "issued_from_python_us": round(timed_us(estep, n_steps, settle_s=0.3), 2),
            "bytes": (2 * 4096 * 1024 + 3 * 2 * 4096 * 1024) * 2 + 3 * 4096 * 50 * 4 + 32000 * 1024 * 2}
        eplan.status()
        progress("decoder step timed")
    # ---- CPU baseline: LibTorch CPU at::addmm in fp16 on the same sweep, bounded sample ---------------------------
    cpu = None
    if not args.no_cpu_baseline:
        threads = torch.get_num_threads()
        t_total, b_total, detail = 0.0, 0, []
        for s in shapes:
            W = s["pool"][0].cpu()
            xc, bc = s["x"].cpu().reshape(1, -1), s["b"].cpu()
            Wt = W.t()
            for _ in range(2):
                torch.addmm(bc, xc, Wt)
            times = []
            t_cpu = time.perf_counter()
            while len(times) < 20 and (time.perf_counter() - t_cpu) < 4.0:
                t = time.perf_counter()
                torch.addmm(bc, xc, Wt)
                times.append(time.perf_counter() - t)
            med = sorted(times)[len(times) // 2]
            t_total += med
            b_total += gemv_bytes(s["n"], s["k"])
            detail.append(f"{s['n']}x{s['k']}: {med * 1e3:.2f} ms")

        def cpu_median_s(fn, n=7, limit_s=3.0):
            fn()
            ts, t_begin = [], time.perf_counter()
            while len(ts) < n and (time.perf_counter() - t_begin) < limit_s:
                t_ = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t_)
            return sorted(ts)[len(ts) // 2]
        # LibTorch CPU at::lstm on the LSTM configuration (fp16, as the reference's atenLstm1 calls it)
        pc = [q for q in params]
        other["cpu_libtorch_lstm_us_per_layer_step"] = round(
            cpu_median_s(lambda: torch.lstm(x, (h0, c0), pc, True, 2, 0.0, False, False, False), n=5, limit_s=5.0) / 400 * 1e6, 1)
        # context columns on the 4096 x 4096 shape: one thread (a per-core figure) and fp32 operands on all threads
        s0 = shapes[0]
        W0, x0, b0 = s0["pool"][0].cpu(), s0["x"].cpu().reshape(1, -1), s0["b"].cpu()
        bytes0 = gemv_bytes(s0["n"], s0["k"])
        W0f, x0f, b0f = W0.float(), x0.float(), b0.float()
        fp32_gbs = 2 * bytes0 / cpu_median_s(lambda: torch.addmm(b0f, x0f, W0f.t())) / 1e9
        torch.set_num_threads(1)
        try:
            one_thread_gbs = bytes0 / cpu_median_s(lambda: torch.addmm(b0, x0, W0.t())) / 1e9
        finally:
            torch.set_num_threads(threads)
        cpu = dict(value=round(b_total / t_total / 1e9, 2), unit="GB/s", cores=threads, kind="reference",
                   one_thread_fp16_4096x4096_gbs=round(one_thread_gbs, 2), fp32_operands_4096x4096_gbs=round(fp32_gbs, 2),
                   sample="LibTorch CPU at::addmm(b, x, W^T) in fp16, the op atenAddmm passes through to: median of <= 20 "
                          "runs (<= 4 s) per sweep shape after 2 warm-ups, same weight every run (cache-warm), one pass of the "
                          "same 4-GEMV sweep; " + "; ".join(detail))

    assert step_bytes == sum(gemv_bytes(n, k) for _, (n, k) in sweep) and abs(value * ms_per_step * 1e6 - step_bytes) <= 1e-3 * step_bytes
    workload = ("GEMV sweep, batch 1, fp16: (out,in) in {(4096,4096),(16384,4096),(4096,16384),(32000,1024)}, y = W.x + b, seeds "
                "2001-2004, cold weights (rotating copies, >= 500 MB per shape)")
    if len(sweep) != len(SWEEP):
        workload = "PART of the " + workload + ": only " + ", ".join(f"{n}x{k}" for _, (n, k) in sweep) + " (a profiler run of single shapes)"
    out = {
        "metric": "fp16 GEMV HBM GB/s (% of peak) at 1 GPU; LSTM us/layer-step at H=1024",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 storage, f32 accumulate",
        "data": "synthetic",
        "config": {"workload": workload, "bytes_per_step": step_bytes},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "gemv_per_shape": per_shape,
        "lstm_us_per_layer_step": None if lstm["automatic"] is None else round(lstm["automatic"], 3),
        "lstm_us_per_layer_step_by_mode": {k: (None if v is None else round(v, 3)) for k, v in lstm.items()},
        "lstm_calls_with_a_wait_that_gave_up_by_mode": lstm_fallbacks,
        "lstm_us_per_layer_step_per_step_launches": None if lstm["per_step_launches"] is None else round(lstm["per_step_launches"], 3),
        "lstm_config": "2 layers unidirectional, I=240, H=1024, T=200, batch 1 (400 layer-steps per call, input projection included)",
        "input_projection": None if xp_us is None else {
            "shape": "T=200, I=1024, 4H=4096", "us": round(xp_us, 2), "us_plain_weight_layout": round(xp_times["plain"], 2),
            "tflops": round(xp_tflops, 2),
            "mfma_utilisation": round(xp_tflops / MFMA_FP16_PEAK_TFLOPS, 5),
            "all_shapes": xp_shapes},
        "other_kernels": other,
        "wall_ms_timed_region": round(wall_ms, 2),
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
