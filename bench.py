"""Benchmark of the JIT-fused array-expression path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-configs] [--no-cpu]

A "step" is one fused softmax pass over one [4096, 1024] fp32 batch (BASELINE.json
configs[0], the shape the headline metric is quoted on). The batches rotate over
enough distinct input/output pairs that the working set exceeds the 256 MiB
Infinity Cache, so the inputs of a step come from HBM, where they were resident
before the timed region started. Steps are issued from a launch recording (the
expression is planned and hipRTC-compiled once, outside the timed region).

Prints ONE JSON line. `value` is algorithmic bytes (1 read + 1 write of the
matrix) per second over the K timed steps, timed with HIP events on the library
stream (host wall time is reported beside it); `roofline` is the same figure
priced against the 8 TB/s HBM peak; `configs`
carries the other four BASELINE.json configurations (GB/s, TFLOP/s or us);
`cpu_baseline` is the CPU checker (a port of the reference's sequential loops)
timed on one host core on a bounded sample of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_FP32_PEAK_TFLOPS = 157.3


def traffic_from_profile(kernel):
    """HBM bytes per launch of `kernel` from the committed counter summary, or None when that summary was made on
    another kernel (the name carries the hash of the generated code's structure and launch parameters)."""
    path = os.path.join(ROOT, "profiles", "softmax_c1_hbm_traffic_pmc.md")
    try:
        text = open(path).read()
    except OSError:
        return None, "profiles/softmax_c1_hbm_traffic_pmc.md is missing"
    got = dict(re.findall(r"^(measured_kernel|traffic_bytes_per_launch): (\S+)$", text, re.M))
    if got.get("measured_kernel") != kernel or "traffic_bytes_per_launch" not in got:
        return None, "profiles/softmax_c1_hbm_traffic_pmc.md covers %s, this run launched %s" % (got.get("measured_kernel"), kernel)
    return int(got["traffic_bytes_per_launch"]), "profiles/softmax_c1_hbm_traffic_pmc.md (measured on %s)" % kernel


def config_traffic():
    """kernel name -> HBM bytes per launch from the committed counter summary of the other configurations."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic_all_configs_pmc.md")
    try:
        text = open(path).read()
    except OSError:
        return {}
    return {k: int(v) for _, k, v in re.findall(r"^traffic: (\S+) (\S+) (\d+)$", text, re.M)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-configs", action="store_true", help="skip the other four configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--c1-only", action="store_true",
                    help="issue only the warm-up and the K timed softmax steps on the rotating pairs (what a kernel trace "
                         "of the headline should contain) and print a short JSON line")
    ap.add_argument("--graph", action="store_true", help="issue the timed softmax steps as HIP graph launches (one graph per group of steps)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="counter-collection helper: a few dispatches of every configuration's kernels (32 softmax steps on "
                         "rotating buffers first) and two plain copies of known size (64 MiB and 1000 MiB each way) that calibrate "
                         "the byte counters, nothing else; prints which kernel belongs to which configuration and no JSON "
                         "(with --no-configs: the softmax steps and the small copy only)")
    ap.add_argument("--copy-sweep", action="store_true",
                    help="streaming rates of the library's own kernels against size: a plain copy (op::identity) on one buffer "
                         "pair and on two alternating pairs, a read-only pass (op::sum) and a write-only pass (op::arange), "
                         "32 MiB to 1000 MiB; prints one JSON line and nothing else")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this path runs on ONE GPU (the reference has no multi-device support and this build "
                 "uses no collectives); run with --gpus 1")

    import numpy as np
    import dali_amd as D
    from dali_amd import op
    from dali_amd._native import hip, hip_check

    hip_check(hip.dali_hip_init(0), "dali_hip_init")

    def sync():
        hip_check(hip.dali_hip_sync(), "sync")

    class Events(object):
        def __init__(self):
            self.a, self.b = C.c_void_p(), C.c_void_p()
            hip_check(hip.dali_hip_event_create(C.byref(self.a)))
            hip_check(hip.dali_hip_event_create(C.byref(self.b)))

        def start(self):
            hip_check(hip.dali_hip_event_record(self.a))

        def stop_ms(self):
            hip_check(hip.dali_hip_event_record(self.b))
            ms = C.c_float()
            hip_check(hip.dali_hip_event_elapsed_ms(self.a, self.b, C.byref(ms)))
            return ms.value

    ev = Events()

    def time_recording(rec, reps, warm=3):
        """Average microseconds per replay of `rec`, HIP events on the library stream."""
        rec.replay(warm)
        sync()
        ev.start()
        rec.replay(reps)
        return ev.stop_ms() * 1e3 / reps

    if args.copy_sweep:
        # What bounds the read+write kernels: at which size a copy stops being helped by the 256 MiB Infinity Cache, and
        # what reads alone and writes alone reach beyond it.
        rows = []
        for mib in (32, 64, 128, 192, 256, 320, 384, 512, 768, 1000):
            n = mib * 262144
            srcs = [D.Array.from_numpy(np.random.RandomState(40 + i).randn(n).astype(np.float32)) for i in range(2)]
            reps = 40 if mib < 512 else 16
            row = {"MiB_each_way": mib}
            with D.Recording() as rec:
                kept = [op.identity(srcs[0]).eval()]
            row["copy_same_pair_frac_hbm"] = round(2.0 * n * 4 / time_recording(rec, reps) / 1e3 / HBM_PEAK_GBS, 4)
            with D.Recording() as rec:
                kept = [op.identity(x).eval() for x in srcs]
            row["copy_alternating_pairs_frac_hbm"] = round(2.0 * n * 4 / (time_recording(rec, reps // 2) / 2) / 1e3 / HBM_PEAK_GBS, 4)
            with D.Recording() as rec:
                kept = [op.sum(srcs[0]).eval()]
            row["read_only_frac_hbm"] = round(1.0 * n * 4 / time_recording(rec, reps) / 1e3 / HBM_PEAK_GBS, 4)
            with D.Recording() as rec:
                kept = [op.arange(n).eval()]
            row["write_only_frac_hbm"] = round(1.0 * n * 4 / time_recording(rec, reps) / 1e3 / HBM_PEAK_GBS, 4)
            rows.append(row)
            del srcs, kept, rec
        print(json.dumps({"copy_sweep": rows, "unit": "fraction of 8 TB/s by algorithmic bytes (copy: read + write)"}))
        return

    if args.pmc_probe:
        # Every dispatch below belongs to one configuration; "probe_kernel: <tag> <kernel names>" lines on stdout say which
        # generated kernel is which (their names carry a hash). The two copies calibrate the byte counters.
        def probe(tag, build, reps):
            with D.Recording() as rec:
                kept = build()
            names = D.last_kernel_names()
            rec.replay(reps - 1)
            sync()
            print("probe_kernel: %s %s launches_per_evaluation=%d evaluations=%d" % (tag, names or "-", rec.launches, reps), flush=True)
            return kept

        rng = np.random.RandomState(1)
        xs = [D.Array.from_numpy(rng.randn(4096, 1024).astype(np.float32)) for _ in range(16)]
        probe("c1_softmax_4096x1024", lambda: [op.softmax(x).eval() for x in xs], 2)  # 32 dispatches on 16 rotating pairs
        src = D.Array.from_numpy(rng.randn(16777216).astype(np.float32))
        probe("copy_64MiB_each_way", lambda: op.identity(src).eval(), 20)
        del xs, src
        if not args.no_configs:
            n = 67108864
            a, b, c, d = (D.Array.from_numpy(np.random.RandomState(s).uniform(-4, 4, n).astype(np.float32)) for s in (2, 3, 4, 5))
            probe("c2_chain_4x67108864", lambda: (op.sigmoid(a) * op.tanh(b) + c * d - 0.5 * op.square(a)).eval(), 6)
            del a, b, c, d
            m = D.Array.from_numpy(np.random.RandomState(6).randn(8192, 8192).astype(np.float32))
            for name, fn in (("sum_axis1", lambda: op.sum(m, [1])), ("max_axis1", lambda: op.max(m, [1])), ("sum_axis0", lambda: op.sum(m, [0])),
                             ("max_axis0", lambda: op.max(m, [0])), ("sum_all", lambda: op.sum(m)), ("max_all", lambda: op.max(m)),
                             ("argmax_axis1", lambda: op.argmax(m, 1))):
                probe("c3_" + name + "_8192x8192", lambda: fn().eval(), 6)
            del m
            rows, vocab = 8192, 32000
            x = D.Array.from_numpy((np.random.RandomState(7).randn(rows, vocab) * 2).astype(np.float32))
            t = D.Array.from_numpy(np.random.RandomState(8).randint(0, vocab, rows).astype(np.int32))
            probe("c4_cross_entropy_8192x32000", lambda: op.softmax_cross_entropy(x, t), 6)
            probe("copy_1000MiB_each_way", lambda: op.identity(x).eval(), 6)  # the plain copy of C4's size: 1,048,576,000 B each way
            del x, t
            B, I, H = 256, 1024, 1024
            X, Hp, Cp = (D.Array.from_numpy(np.random.RandomState(s).randn(B, k).astype(np.float32)) for s, k in ((9, I), (10, H), (11, H)))
            lim = np.sqrt(6.0 / (1024 + 4096))
            W, U = (D.Array.from_numpy(np.random.RandomState(s).uniform(-lim, lim, (1024, 4096)).astype(np.float32)) for s in (12, 13))
            bias = D.Array.zeros((4096,))
            probe("c5_gemm_pair_256x2048x4096", lambda: (op.dot(X, W) + op.dot(Hp, U)).eval(), 20)
            probe("c5_lstm_step_fused", lambda: op.lstm_step(X, Hp, Cp, W, U, bias), 20)
            del X, Hp, Cp, W, U, bias
            # the products of the backward pass of dot(h [256,1024], W [1024,32000]): many 128x128 tiles walked by one workgroup per
            # compute unit, and 64 tiles x 4 shares of a long inner extent
            bh, bg, bw = (D.Array.from_numpy((np.random.RandomState(s).randn(*shp) * 0.1).astype(np.float32))
                          for s, shp in ((60, (256, 1024)), (61, (256, 32000)), (62, (1024, 32000))))
            probe("dot_backward_weights_256x1024T_x_256x32000", lambda: op.dot(bh.transpose(), bg).eval(), 10)
            probe("dot_backward_inputs_256x32000_x_1024x32000T", lambda: op.dot(bg, bw.transpose()).eval(), 10)
        return

    # ------------------------------------------------------------ headline: C1
    R, Cn = 4096, 1024
    step_bytes = 2 * R * Cn * 4
    n_pairs = 16  # 16 x 32 MiB = 512 MiB of inputs + outputs in rotation
    rng = np.random.RandomState(1)
    inputs = [D.Array.from_numpy(rng.randn(R, Cn).astype(np.float32)) for _ in range(n_pairs)]
    # what lies outside the timed region: the first evaluation (planning + hipRTC compile, or the load of the code object
    # from the on-disk cache) and the host cost of an eager evaluation (build the expression, plan, launch) as opposed to a replay
    jit0 = [C.c_uint64() for _ in range(3)]
    hip.dali_hip_jit_stats(*[C.byref(v) for v in jit0])
    t_first = time.perf_counter()
    op.softmax(inputs[0]).eval()
    sync()
    t_first = time.perf_counter() - t_first
    jit1 = [C.c_uint64() for _ in range(3)]
    hip.dali_hip_jit_stats(*[C.byref(v) for v in jit1])
    t_eager = 0.0
    if not args.c1_only:  # (evaluations on one resident pair: kept out of a trace of the rotating steps)
        t_eager = time.perf_counter()
        for _ in range(200):
            op.softmax(inputs[0]).eval()
        t_eager = (time.perf_counter() - t_eager) / 200
        sync()
    outside = {"first_eval_ms": round(t_first * 1e3, 1), "first_eval_compiled": int(jit1[0].value - jit0[0].value),
               "first_eval_disk_hits": int(jit1[1].value - jit0[1].value), "eager_eval_host_us": round(t_eager * 1e6, 1)}
    with D.Recording() as cycle:
        for x in inputs:
            op.softmax(x).eval()
    softmax_kernel = D.last_kernel_names()
    assert cycle.launches == n_pairs

    def steps_recording(first, count):
        """`count` steps as one recording, on the pairs first, first + 1, ... of the rotation."""
        with D.Recording() as rec:
            for i in range(count):
                op.softmax(inputs[(first + i) % n_pairs]).eval()
        assert rec.launches == count
        return rec

    # The K timed steps go on from the pair after the last warm-up step, so no timed step finds its buffers in the
    # 256 MiB Infinity Cache (the 15 pairs touched in between are 480 MiB). They are issued by at most three calls
    # (the steps up to the start of the rotation, whole rotations, the rest): the host is not in the timed path.
    first = args.warmup % n_pairs
    lead_n = min(args.steps, (n_pairs - first) % n_pairs)
    cycles, tail_n = divmod(args.steps - lead_n, n_pairs)
    lead = steps_recording(first, lead_n) if lead_n else None
    tail = steps_recording(0, tail_n) if tail_n else None
    warm_cycles, warm_rest = divmod(args.warmup, n_pairs)
    warm_tail = steps_recording(0, warm_rest) if warm_rest else None
    preroll = steps_recording(first, n_pairs)

    if args.graph:
        for r in (cycle, lead, tail, preroll):
            if r:
                r.make_graph()
                r.replay(1)
    cycle.replay(warm_cycles)
    if warm_tail:
        warm_tail.replay(1)
    sync()
    t0 = time.perf_counter()
    # One more untimed rotation is queued in front of the start event and not waited for: while the device works
    # through it the host records the event and issues the timed steps, so the two events bracket the device's time
    # for exactly K launches and not the host's call latency (which at K = 20 would be a tenth of the region).
    preroll.replay(1)
    ev.start()
    if lead:
        lead.replay(1)
    if cycles:
        cycle.replay(cycles)
    if tail:
        tail.replay(1)
    ev_ms = ev.stop_ms()  # waits for the stop event: every timed step has finished
    sync()
    wall = time.perf_counter() - t0
    # one clock for the headline and for the roofline: HIP events on the library stream around the K launches
    kernel_us = ev_ms * 1e3 / args.steps
    gbs = step_bytes / (kernel_us * 1e-6) / 1e9
    wall_steps = args.steps + n_pairs  # the host clock also saw the untimed rotation in front

    traffic, traffic_note = traffic_from_profile(softmax_kernel)

    if args.c1_only:
        print(json.dumps({"kernel": softmax_kernel, "steps": args.steps, "warmup": args.warmup,
                          "avg_launch_us_hip_events": round(kernel_us, 3), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                          "host_wall_us_per_step": round(wall * 1e6 / wall_steps, 3)}))
        return

    # same kernel on one resident pair (served from the on-chip caches): reported, not the headline
    resident = steps_recording(0, 1)
    resident_us = time_recording(resident, 500, 20)

    result = {
        "metric": "fused softmax fp32 [4096,1024] achieved HBM GB/s",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(kernel_us * 1e-3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "clock": "value, ms_per_step and roofline: HIP events on the library stream around the K timed launches; "
                 "host_wall_ms_per_step: time.perf_counter around the same region plus the untimed rotation of %d steps queued "
                 "in front of the start event and the final synchronisation, per step issued" % n_pairs,
        "host_wall_ms_per_step": round(wall * 1e3 / wall_steps, 6),
        "config": {
            "workload": "C1 naive fused softmax exp(a-max)/sum over fp32 [4096,1024] ~ N(0,1), rotating over %d distinct "
                        "input/output pairs (512 MiB > 256 MiB Infinity Cache), one fused row kernel per step" % n_pairs,
            "algorithmic_bytes_per_step": step_bytes,
            "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
            "cache_resident_single_pair_us": round(resident_us, 3),
            "cache_resident_single_pair_gbs": round(step_bytes / resident_us / 1e3, 1),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": softmax_kernel,
            "achieved": round(gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "avg_launch_us": round(kernel_us, 3),
            # HBM bytes per launch from the committed counter runs (FETCH_SIZE + WRITE_SIZE, each scaled by the same
            # counter on a copy of known size), taken over only when they were made on this very kernel
            "traffic": traffic,
            "traffic_source": traffic_note,
        },
    }

    result["outside_timed_region"] = outside

    # ------------------------------------------------- the other four configs
    if not args.no_configs:
        configs = {}
        del inputs, cycle, lead, tail, warm_tail, resident, preroll
        measured = config_traffic()

        def with_traffic(row):
            """adds the kernel's name and, when the committed counter runs were made on this very kernel, its HBM bytes per launch"""
            name = D.last_kernel_names()
            row["kernel"] = name
            row["traffic"] = measured.get(name)
            return row

        # C2 elementwise chain, 4 x 67,108,864 fp32 in, 1 out
        n = 67108864
        a, b, c, d = (D.Array.from_numpy(np.random.RandomState(s).uniform(-4, 4, n).astype(np.float32)) for s in (2, 3, 4, 5))
        with D.Recording() as rec:
            (op.sigmoid(a) * op.tanh(b) + c * d - 0.5 * op.square(a)).eval()
        c2_row = with_traffic({})
        us = time_recording(rec, 30)
        configs["c2_chain_4x67108864"] = dict({"us": round(us, 2), "GB/s": round(5 * n * 4 / us / 1e3, 1),
                                               "frac_hbm": round(5 * n * 4 / us / 1e3 / HBM_PEAK_GBS, 4), "kernels": rec.launches}, **c2_row)
        del a, b, c, d, rec

        # C3 reductions over [8192, 8192]; two matrices alternate (268 MB each) to stay out of the cache
        mats = [D.Array.from_numpy(np.random.RandomState(6 + i).randn(8192, 8192).astype(np.float32)) for i in range(2)]
        nb = 8192 * 8192 * 4
        c3 = {}
        for name, fn in (("sum_axis1", lambda m: op.sum(m, [1])), ("max_axis1", lambda m: op.max(m, [1])),
                         ("sum_axis0", lambda m: op.sum(m, [0])), ("max_axis0", lambda m: op.max(m, [0])),
                         ("sum_all", lambda m: op.sum(m)), ("max_all", lambda m: op.max(m)),
                         ("argmax_axis1", lambda m: op.argmax(m, 1))):
            with D.Recording() as rec:
                for m in mats:
                    fn(m).eval()
            c3_row = with_traffic({})
            us = time_recording(rec, 20) / len(mats)
            c3[name] = dict({"us": round(us, 2), "GB/s": round(nb / us / 1e3, 1), "frac_hbm": round(nb / us / 1e3 / HBM_PEAK_GBS, 4),
                             "kernels": rec.launches // len(mats)}, **c3_row)
        configs["c3_reductions_8192x8192"] = c3
        del mats, rec

        # C4 softmax cross-entropy [8192, 32000]: loss + gradient
        rows, vocab = 8192, 32000
        x = D.Array.from_numpy((np.random.RandomState(7).randn(rows, vocab) * 2).astype(np.float32))
        t = D.Array.from_numpy(np.random.RandomState(8).randint(0, vocab, rows).astype(np.int32))
        with D.Recording() as rec:
            mean, rl, grad = op.softmax_cross_entropy(x, t)
        c4_row = with_traffic({})
        us = time_recording(rec, 10)
        ce_bytes = 2 * rows * vocab * 4
        configs["c4_cross_entropy_8192x32000"] = dict({"us": round(us, 2), "GB/s": round(ce_bytes / us / 1e3, 1),
                                                       "frac_hbm": round(ce_bytes / us / 1e3 / HBM_PEAK_GBS, 4),
                                                       "kernels": rec.launches, "passes_over_logits": 1,
                                                       "mean_loss": round(float(mean.numpy()), 5)}, **c4_row)
        del x, t, grad, rl, mean, rec

        # C5 LSTM step B=256, I=H=1024
        B, I, H = 256, 1024, 1024
        X, Hp, Cp = (D.Array.from_numpy(np.random.RandomState(s).randn(B, k).astype(np.float32)) for s, k in ((9, I), (10, H), (11, H)))
        lim = np.sqrt(6.0 / (1024 + 4096))
        W, U = (D.Array.from_numpy(np.random.RandomState(s).uniform(-lim, lim, (1024, 4096)).astype(np.float32)) for s in (12, 13))
        bias = D.Array.zeros((4096,))
        with D.Recording() as rec:
            op.lstm_step(X, Hp, Cp, W, U, bias)
        step_us = time_recording(rec, 200, 10)
        with D.Recording() as grec:
            (op.dot(X, W) + op.dot(Hp, U)).eval()
        gemm_us = time_recording(grec, 200, 10)
        flops = 2.0 * B * (I + H) * 4 * H
        configs["c5_lstm_step_256x1024x1024"] = {"step_us": round(step_us, 2), "launches": rec.launches,
                                                 "gemm_pair_us": round(gemm_us, 2),
                                                 "gemm_TFLOP/s": round(flops / gemm_us / 1e6, 2),
                                                 "gemm_frac_fp32_mfma": round(flops / gemm_us / 1e6 / MFMA_FP32_PEAK_TFLOPS, 4)}
        # the same step with an input size other than the hidden size (rows of x and of h differ in length)
        X5 = D.Array.from_numpy(np.random.RandomState(24).randn(B, 512).astype(np.float32))
        W5 = D.Array.from_numpy(np.random.RandomState(25).uniform(-lim, lim, (512, 4096)).astype(np.float32))
        with D.Recording() as rec5:
            op.lstm_step(X5, Hp, Cp, W5, U, bias)
        us5 = time_recording(rec5, 200, 10)
        configs["c5_lstm_step_256x1024x1024"]["step_input512_hidden1024"] = {"us": round(us5, 2), "launches": rec5.launches,
                                                                             "TFLOP/s": round(2.0 * B * (512 + H) * 4 * H / us5 / 1e6, 2)}
        del X5, W5, rec5
        # the same step along a sequence of 32: fused launches chained through one [T, B, H] buffer
        Xs = D.Array.from_numpy(np.random.RandomState(23).randn(32, B, H).astype(np.float32))
        with D.Recording() as srec:
            op.lstm_sequence(Xs, Hp, Cp, W, U, bias)
        seq_us = time_recording(srec, 10)
        configs["c5_lstm_step_256x1024x1024"]["sequence_of_32_us_per_step"] = round(seq_us / 32, 2)
        # small batches: the whole sequence as one product for the input half plus one persistent launch for the recurrent
        # half (U stays in the LDS, a grid barrier per step), beside the same sequence as one fused launch per step
        small = {}
        for Bs in (8, 32, 64):
            Xq = D.Array.from_numpy(np.random.RandomState(24).randn(32, Bs, H).astype(np.float32))
            hs0, cs0 = (D.Array.from_numpy(np.random.RandomState(s).randn(Bs, H).astype(np.float32)) for s in (25, 26))
            row = {}
            for name, flag in (("persistent", "2"), ("launch_per_step", "0")):  # "2": wherever the persistent kernels serve the size
                os.environ["DALI_HIP_LSTM_PERSISTENT"] = flag
                with D.Recording() as qrec:
                    op.lstm_sequence(Xq, hs0, cs0, W, U, bias)
                row[name + "_us_per_step"] = round(time_recording(qrec, 10) / 32, 2)
                row[name + "_launches"] = qrec.launches
            os.environ.pop("DALI_HIP_LSTM_PERSISTENT", None)
            row["front_end_takes"] = "persistent" if hip.dali_hip_lstm_recurrent_persistent_supported(Bs, H) == 2 else "launch_per_step"
            sflops = 2.0 * Bs * (I + H) * 4 * H
            row["mfma_fp32_bound_us"] = round(sflops / MFMA_FP32_PEAK_TFLOPS / 1e6, 2)
            row["weights_from_hbm_bound_us"] = round(2 * 1024 * 4096 * 4 / HBM_PEAK_GBS / 1e3, 2)  # what a launch per step re-reads
            small["B%d" % Bs] = row
            del Xq, hs0, cs0, qrec
        configs["c5_lstm_step_256x1024x1024"]["sequence_of_32_small_batches"] = small
        # sizes of the persistent kernel that keeps the weights in registers (other hidden sizes, more than 64 rows), again beside a
        # fused launch per step
        other = {}
        for Bs, Hs in ((96, 1024), (64, 640), (64, 1536), (32, 2048), (64, 2048)):
            Xq = D.Array.from_numpy(np.random.RandomState(24).randn(32, Bs, Hs).astype(np.float32))
            hs0, cs0 = (D.Array.from_numpy(np.random.RandomState(s).randn(Bs, Hs).astype(np.float32)) for s in (25, 26))
            limq = np.sqrt(6.0 / (5 * Hs))
            Wq, Uq = (D.Array.from_numpy(np.random.RandomState(s).uniform(-limq, limq, (Hs, 4 * Hs)).astype(np.float32)) for s in (12, 13))
            bq = D.Array.zeros((4 * Hs,))
            row = {}
            for name, flag in (("persistent", "2"), ("launch_per_step", "0")):  # "2": wherever the persistent kernels serve the size
                os.environ["DALI_HIP_LSTM_PERSISTENT"] = flag
                with D.Recording() as qrec:
                    op.lstm_sequence(Xq, hs0, cs0, Wq, Uq, bq)
                row[name + "_us_per_step"] = round(time_recording(qrec, 6) / 32, 2)
                row[name + "_launches"] = qrec.launches
            os.environ.pop("DALI_HIP_LSTM_PERSISTENT", None)
            row["front_end_takes"] = "persistent" if hip.dali_hip_lstm_recurrent_persistent_supported(Bs, Hs) == 2 else "launch_per_step"
            row["mfma_fp32_bound_us"] = round(2.0 * Bs * 2 * Hs * 4 * Hs / MFMA_FP32_PEAK_TFLOPS / 1e6, 2)
            other["B%d_H%d" % (Bs, Hs)] = row
            del Xq, hs0, cs0, Wq, Uq, bq, qrec
        configs["c5_lstm_step_256x1024x1024"]["sequence_of_32_other_sizes"] = other
        # the GRU (two dependent products per step): the recurrent half as one persistent launch beside the launch-per-step form
        gru = {}
        for Bs, Hs in ((8, 1024), (32, 1024), (8, 512)):
            Xq = D.Array.from_numpy(np.random.RandomState(24).randn(32, Bs, Hs).astype(np.float32))
            hq = D.Array.from_numpy(np.random.RandomState(25).randn(Bs, Hs).astype(np.float32))
            limq = np.sqrt(6.0 / (4 * Hs))
            Wq, Uq = (D.Array.from_numpy(np.random.RandomState(s).uniform(-limq, limq, (Hs, 3 * Hs)).astype(np.float32)) for s in (12, 13))
            bq = D.Array.zeros((3 * Hs,))
            row = {}
            for name, flag in (("persistent", "1"), ("launch_per_step", "0")):
                os.environ["DALI_HIP_GRU_PERSISTENT"] = flag
                with D.Recording() as qrec:
                    op.gru_sequence(Xq, hq, Wq, Uq, bq)
                row[name + "_us_per_step"] = round(time_recording(qrec, 6) / 32, 2)
                row[name + "_launches"] = qrec.launches
            os.environ.pop("DALI_HIP_GRU_PERSISTENT", None)
            row["weights_from_hbm_bound_us"] = round(2 * Hs * 3 * Hs * 4 / HBM_PEAK_GBS / 1e3, 2)  # what a launch per step re-reads
            gru["B%d_H%d" % (Bs, Hs)] = row
            del Xq, hq, Wq, Uq, bq, qrec
        configs["c5_lstm_step_256x1024x1024"]["gru_sequence_of_32"] = gru
        # one step at small batches (a decoder loop through the host): 16-row tiles with every compute unit on its own columns
        # of the weights, beside the 64-row tiles of the general kernel
        single = {}
        for Bs in (1, 8, 32, 64):
            xq, hq, cq = (D.Array.from_numpy(np.random.RandomState(s).randn(Bs, H).astype(np.float32)) for s in (29, 30, 31))
            row = {}
            # the path the front-end takes (the 16-row-tile kernel up to 16 rows, then the fused step with its inner extent cut into
            # one share per compute unit), and the fused step whatever the batch
            for name, flag in (("us", "1"), ("fused_step_us", "0")):
                os.environ["DALI_HIP_LSTM_SMALL"] = flag
                with D.Recording() as qrec:
                    op.lstm_step(xq, hq, cq, W, U, bias)
                row[name] = round(time_recording(qrec, 100, 10), 2)
                if flag == "1":
                    row["kernel"] = D.last_kernel_kinds()
            os.environ.pop("DALI_HIP_LSTM_SMALL", None)
            row["weights_from_hbm_bound_us"] = round(2 * 1024 * 4096 * 4 / HBM_PEAK_GBS / 1e3, 2)
            single["B%d" % Bs] = row
            del xq, hq, cq, qrec
        configs["c5_lstm_step_256x1024x1024"]["single_step_small_batches"] = single
        del X, Hp, Cp, W, U, bias, rec, grec, Xs, srec

        # the products of the backward pass of dot(h [256,1024], W [1024,32000]) (dali/tensor/op/dot.cpp:17-18): the weight gradient
        # h^T . g reads its left operand against its rows (inner extent 256), the input gradient g . W^T its right one (32000)
        bh, bg, bw = (D.Array.from_numpy((np.random.RandomState(s).randn(*shp) * 0.1).astype(np.float32))
                      for s, shp in ((60, (256, 1024)), (61, (256, 32000)), (62, (1024, 32000))))
        bwd = {}
        for tag, make in (("weights_256x1024T_x_256x32000", lambda: op.dot(bh.transpose(), bg)), ("inputs_256x32000_x_1024x32000T", lambda: op.dot(bg, bw.transpose()))):
            flops = 2.0 * 256 * 1024 * 32000
            with D.Recording() as brec:
                make().eval()
            bus = time_recording(brec, 20)
            bwd[tag] = {"us": round(bus, 2), "TFLOP/s": round(flops / bus / 1e6, 2), "frac_fp32_mfma": round(flops / bus / 1e6 / 157.3, 4), "launches": brec.launches}
            del brec
        configs["c5_lstm_step_256x1024x1024"]["dot_backward_products"] = bwd
        del bh, bg, bw
        sq = [D.Array.from_numpy(np.random.RandomState(s).randn(4096, 4096).astype(np.float32)) for s in (63, 64)]
        with D.Recording() as brec:
            op.dot(sq[0], sq[1]).eval()
        bus = time_recording(brec, 5)
        configs["c5_lstm_step_256x1024x1024"]["dot_4096x4096x4096"] = {"us": round(bus, 2), "TFLOP/s": round(2.0 * 4096 ** 3 / bus / 1e6, 2),
                                                                      "frac_fp32_mfma": round(2.0 * 4096 ** 3 / bus / 1e6 / 157.3, 4)}
        del sq, brec

        # the double-precision product (the reference's cublasDgemm branch)
        dA, dB = (D.Array.from_numpy(np.random.RandomState(s).randn(2048, 2048)) for s in (27, 28))
        with D.Recording() as drec:
            op.dot(dA, dB).eval()
        dus = time_recording(drec, 10)
        configs["c5_lstm_step_256x1024x1024"]["dot_fp64_2048x2048x2048"] = {"us": round(dus, 2), "TFLOP/s": round(2.0 * 2048 ** 3 / dus / 1e6, 2),
                                                                           "frac_fp64_mfma": round(2.0 * 2048 ** 3 / dus / 1e6 / 78.6, 4)}
        del dA, dB, drec

        # few rows against a wide weight matrix (the output projection of a decoder step): bound by streaming the weights once
        Wp = D.Array.from_numpy((np.random.RandomState(29).randn(1024, 32000) * 0.02).astype(np.float32))
        proj = {}
        for Bq in (8, 64):
            hq = D.Array.from_numpy(np.random.RandomState(30 + Bq).randn(Bq, 1024).astype(np.float32))
            with D.Recording() as prec:
                op.dot(hq, Wp).eval()
            pus = time_recording(prec, 20)
            proj["B%d" % Bq] = {"us": round(pus, 2), "weights_GB/s": round(1024 * 32000 * 4 / pus / 1e3, 1), "frac_hbm": round(1024 * 32000 * 4 / pus / 1e3 / HBM_PEAK_GBS, 4),
                                "TFLOP/s": round(2.0 * Bq * 1024 * 32000 / pus / 1e6, 2)}
            del hq, prec
        configs["c5_lstm_step_256x1024x1024"]["dot_few_rows_Bx1024x32000"] = proj

        # a whole decoder step around those pieces: embedding rows, two LSTM layers, the output projection, the loss and its gradient
        emb = D.Array.from_numpy((np.random.RandomState(40).randn(32000, 1024) * 0.1).astype(np.float32))
        lim_d = np.sqrt(6.0 / (1024 + 4096))
        Wd = [D.Array.from_numpy(np.random.RandomState(41 + i).uniform(-lim_d, lim_d, (1024, 4096)).astype(np.float32)) for i in range(4)]
        bd = [D.Array.zeros((4096,)) for _ in range(2)]
        step = {}
        for Bq in (8, 64):
            rs = np.random.RandomState(50 + Bq)
            ids, tgt = (D.Array.from_numpy(rs.randint(0, 32000, size=Bq).astype(np.int32)) for _ in range(2))
            hd = [D.Array.from_numpy(rs.randn(Bq, 1024).astype(np.float32)) for _ in range(2)]
            cd = [D.Array.from_numpy(rs.randn(Bq, 1024).astype(np.float32)) for _ in range(2)]
            with D.Recording() as srec:
                xq = op.gather(emb, ids)
                c1, h1 = op.lstm_step(xq, hd[0], cd[0], Wd[0], Wd[1], bd[0])
                c2, h2 = op.lstm_step(h1, hd[1], cd[1], Wd[2], Wd[3], bd[1])
                lossq = op.softmax_cross_entropy(op.dot(h2, Wp), tgt)
            sus = time_recording(srec, 20)
            weights_bytes = (4 * 1024 * 4096 + 1024 * 32000) * 4
            step["B%d" % Bq] = {"us": round(sus, 2), "launches": srec.launches, "weights_from_hbm_bound_us": round(weights_bytes / HBM_PEAK_GBS / 1e3, 2)}
            del ids, tgt, hd, cd, srec, xq, c1, h1, c2, h2, lossq
        configs["c5_lstm_step_256x1024x1024"]["decoder_step_2xLSTM1024_vocab32000"] = step
        del Wp, emb, Wd, bd

        # rows beyond the five configs: embedding-style gather and its scatter-add (table [32000, 1024], 8192 indices)
        V, Dm, Nidx = 32000, 1024, 8192
        table = D.Array.from_numpy(np.random.RandomState(14).randn(V, Dm).astype(np.float32))
        ids = D.Array.from_numpy(np.random.RandomState(15).randint(0, V, Nidx).astype(np.int32))
        upd = D.Array.from_numpy(np.random.RandomState(16).randn(Nidx, Dm).astype(np.float32))
        with D.Recording() as rec:
            op.gather(table, ids).eval()
        us = time_recording(rec, 50)
        gbytes = 2 * Nidx * Dm * 4
        nxt = {"gather_32000x1024_8192": {"us": round(us, 2), "GB/s": round(gbytes / us / 1e3, 1),
                                          "frac_hbm": round(gbytes / us / 1e3 / HBM_PEAK_GBS, 4), "kernels": rec.launches}}
        with D.Recording() as rec:
            g = table[ids]
            g += upd
        us = time_recording(rec, 50)
        uniq = int(np.unique(ids.numpy()).size)
        sbytes = Nidx * Dm * 4 + 2 * uniq * Dm * 4  # values once, every touched table row read and written once
        nxt["scatter_add_32000x1024_8192"] = {"us": round(us, 2), "GB/s": round(sbytes / us / 1e3, 1),
                                              "frac_hbm": round(sbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                                              "launches_incl_index_sort": rec.launches, "distinct_rows": uniq}
        # the same with 65536 indices: ordered first (stable radix sort), then one launch that walks runs of equal indices
        ids = D.Array.from_numpy(np.random.RandomState(15).randint(0, V, 65536).astype(np.int32))
        upd = D.Array.from_numpy(np.random.RandomState(16).randn(65536, Dm).astype(np.float32))
        with D.Recording() as rec:
            g = table[ids]
            g += upd
        us = time_recording(rec, 20)
        uniq = int(np.unique(ids.numpy()).size)
        sbytes = 65536 * Dm * 4 + 2 * uniq * Dm * 4
        nxt["scatter_add_32000x1024_65536"] = {"us": round(us, 2), "GB/s": round(sbytes / us / 1e3, 1), "frac_hbm": round(sbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                                               "launches_incl_index_sort": rec.launches, "distinct_rows": uniq}
        del table, ids, upd, g, rec
        # softmax away from the C1 shape: rows of a vocabulary that is no multiple of anything (one row = 201,028 bytes, every
        # row starts elsewhere within a cache line) and the middle axis of a 3-D array; bytes = one read + one write
        for tag, shp, axis in (("softmax_rows_2048x50257", (2048, 50257), -1), ("softmax_middle_axis_256x512x512", (256, 512, 512), 1),
                               ("softmax_middle_axis_64x1024x1024", (64, 1024, 1024), 1)):
            xs_ = D.Array.from_numpy(np.random.RandomState(18).randn(*shp).astype(np.float32))
            with D.Recording() as rec:
                op.softmax(xs_, axis).eval()
            us = time_recording(rec, 20)
            nb = 2.0 * 4 * float(np.prod(shp))
            nxt[tag] = {"us": round(us, 2), "GB/s": round(nb / us / 1e3, 1), "frac_hbm": round(nb / us / 1e3 / HBM_PEAK_GBS, 4), "launches": rec.launches,
                        "kernel": D.last_kernel_kinds()}
            del xs_, rec
        # few very long rows of a length that divides into nothing: the row kernel cuts them into pieces (bytes = one read)
        few = D.Array.from_numpy(np.random.RandomState(19).randn(7, 9999999).astype(np.float32))
        rows_few = {}
        for tag, build in (("sum_axis1", lambda: op.sum(few, [1])), ("argmax_axis1", lambda: op.argmax(few, 1))):
            with D.Recording() as rec:
                build().eval()
            us = time_recording(rec, 20)
            nb = 4.0 * 7 * 9999999
            rows_few[tag] = {"us": round(us, 2), "GB/s": round(nb / us / 1e3, 1), "frac_hbm": round(nb / us / 1e3 / HBM_PEAK_GBS, 4), "launches": rec.launches}
            del rec
        # maps over the same rows that need row statistics first (bytes = one read and one write)
        few_t = D.Array.from_numpy(np.random.RandomState(20).randint(0, 9999999, 7).astype(np.int32))
        for tag, build in (("softmax", lambda: op.softmax(few)), ("cross_entropy_gradient", lambda: op.softmax_cross_entropy(few, few_t)[2]),
                           ("minus_row_means", lambda: few - op.mean(few, [1], True))):
            with D.Recording() as rec:
                build().eval()
            us = time_recording(rec, 10)
            nb = 2 * 4.0 * 7 * 9999999
            rows_few[tag] = {"us": round(us, 2), "GB/s": round(nb / us / 1e3, 1), "frac_hbm": round(nb / us / 1e3 / HBM_PEAK_GBS, 4), "launches": rec.launches}
            del rec
        nxt["reductions_few_long_rows_7x9999999"] = rows_few
        del few, few_t
        # a tall narrow matrix whose row count has no divisor to go by: column sums, a bias added, columns standardised,
        # a cumsum along its rows of seven (bytes = one read, plus one write for the maps)
        tall = D.Array.from_numpy(np.random.RandomState(21).randn(9999999, 7).astype(np.float32))
        tall_b = D.Array.from_numpy(np.random.RandomState(22).randn(1, 7).astype(np.float32))
        rows_tall = {}
        for tag, passes, build in (("sum_axis0", 1, lambda: op.sum(tall, [0])), ("plus_bias", 2, lambda: tall + tall_b),
                                   ("minus_column_means", 2, lambda: tall - op.mean(tall, [0], True)), ("softmax_axis0", 2, lambda: op.softmax(tall, 0)),
                                   ("cumsum_axis1", 2, lambda: op.cumsum(tall))):
            with D.Recording() as rec:
                build().eval()
            us = time_recording(rec, 10)
            nb = passes * 4.0 * 7 * 9999999
            rows_tall[tag] = {"us": round(us, 2), "GB/s": round(nb / us / 1e3, 1), "frac_hbm": round(nb / us / 1e3 / HBM_PEAK_GBS, 4), "launches": rec.launches}
            del rec
        nxt["tall_narrow_9999999x7"] = rows_tall
        del tall, tall_b
        # a matrix times a column: the rows streamed once
        mv_a = D.Array.from_numpy(np.random.RandomState(20).randn(4096, 4096).astype(np.float32))
        mv_x = D.Array.from_numpy(np.random.RandomState(21).randn(4096, 1).astype(np.float32))
        with D.Recording() as rec:
            op.dot(mv_a, mv_x).eval()
        us = time_recording(rec, 50)
        nxt["dot_matrix_column_4096x4096"] = {"us": round(us, 2), "GB/s": round(4096 * 4096 * 4 / us / 1e3, 1), "frac_hbm": round(4096 * 4096 * 4 / us / 1e3 / HBM_PEAK_GBS, 4),
                                              "launches": rec.launches}
        del mv_a, mv_x, rec
        sm = D.Array.from_numpy(np.random.RandomState(17).uniform(0.5, 1.5, (8192, 8192)).astype(np.float32))
        with D.Recording() as rec:
            op.cumsum(sm).eval()
        us = time_recording(rec, 20)
        nxt["cumsum_8192x8192"] = {"us": round(us, 2), "GB/s": round(2 * 8192 * 8192 * 4 / us / 1e3, 1),
                                   "frac_hbm": round(2 * 8192 * 8192 * 4 / us / 1e3 / HBM_PEAK_GBS, 4), "kernels": rec.launches}
        del sm, rec
        # ordering along rows (the reference runs top_k on the CPU only): the 8 largest of 32000 scores in each of 1024 rows
        sc = D.Array.from_numpy(np.random.RandomState(20).randn(1024, 32000).astype(np.float32))
        with D.Recording() as rec:
            op.top_k(sc, 8).eval()
        us = time_recording(rec, 10)
        nxt["top_k_8_of_1024x32000"] = {"us": round(us, 2), "Mkeys/s": round(1024 * 32000 / us, 1), "launches": rec.launches}
        del sc, rec
        # sliding windows in the channels-last layout: a 3x3 convolution layer (64 -> 128 channels, 32 images of 56x56) as
        # im2col + one matrix product, its two gradients, and a 3x3 / stride 2 max pooling of 32 images of 112x112x64
        xi = D.Array.from_numpy(np.random.RandomState(18).randn(32, 56, 56, 64).astype(np.float32))
        wf = D.Array.from_numpy(np.random.RandomState(19).randn(128, 3, 3, 64).astype(np.float32))
        with D.Recording() as rec:
            op.im2col(xi, 3, 3, 1, 1, 1, 1, 1, 1, data_format="NHWC").eval()
        us = time_recording(rec, 20)
        ibytes = (32 * 56 * 56 * 64 + 576 * 32 * 56 * 56) * 4
        nxt["im2col_nhwc_32x56x56x64_3x3"] = {"us": round(us, 2), "GB/s": round(ibytes / us / 1e3, 1),
                                              "frac_hbm": round(ibytes / us / 1e3 / HBM_PEAK_GBS, 4), "kernels": rec.launches}
        with D.Recording() as rec:
            yc = op.conv2d(xi, wf, 1, 1, "same", "NHWC")
            yc.eval()
        us = time_recording(rec, 20)
        cflops = 2.0 * 128 * 576 * 32 * 56 * 56
        nxt["conv2d_nhwc_64to128_3x3_same"] = {"us": round(us, 2), "TFLOP/s": round(cflops / us / 1e6, 2), "launches": rec.launches,
                                               "frac_fp32_mfma": round(cflops / us / 1e6 / MFMA_FP32_PEAK_TFLOPS, 4)}
        dyc = D.Array.from_numpy(np.random.RandomState(20).randn(32, 54, 54, 128).astype(np.float32))
        vflops = 2.0 * 128 * 576 * 32 * 54 * 54
        with D.Recording() as rec:
            op.conv2d_backward_input(wf, dyc, 1, 1, (32, 56, 56, 64), "valid", "NHWC").eval()
        us = time_recording(rec, 20)
        nxt["conv2d_backward_input_nhwc_valid"] = {"us": round(us, 2), "TFLOP/s": round(vflops / us / 1e6, 2), "launches": rec.launches}
        with D.Recording() as rec:
            op.conv2d_backward_filters(xi, dyc, 1, 1, (128, 3, 3, 64), "valid", "NHWC").eval()
        us = time_recording(rec, 20)
        nxt["conv2d_backward_filters_nhwc_valid"] = {"us": round(us, 2), "TFLOP/s": round(vflops / us / 1e6, 2), "launches": rec.launches}
        del xi, wf, yc, dyc, rec
        xp = D.Array.from_numpy(np.random.RandomState(21).randn(32, 112, 112, 64).astype(np.float32))
        with D.Recording() as rec:
            yp = op.pool2d(xp, 3, 3, 2, 2, "max", "same", "NHWC")
            yp.eval()
        us = time_recording(rec, 20)
        pbytes = (32 * 112 * 112 * 64 + 32 * 56 * 56 * 64) * 4
        nxt["pool2d_max_nhwc_32x112x112x64_3x3_s2"] = {"us": round(us, 2), "GB/s": round(pbytes / us / 1e3, 1),
                                                       "frac_hbm": round(pbytes / us / 1e3 / HBM_PEAK_GBS, 4), "kernels": rec.launches}
        dyp = D.Array.from_numpy(np.random.RandomState(22).randn(32, 56, 56, 64).astype(np.float32))
        with D.Recording() as rec:
            op.pool2d_backward(yp, dyp, xp, 3, 3, 2, 2, "max", "same", "NHWC").eval()
        us = time_recording(rec, 20)
        nxt["pool2d_max_backward_nhwc"] = {"us": round(us, 2), "GB/s": round(2 * pbytes / us / 1e3, 1),
                                           "frac_hbm": round(2 * pbytes / us / 1e3 / HBM_PEAK_GBS, 4), "kernels": rec.launches}
        del xp, yp, dyp, rec
        configs["beyond_the_five_configs"] = nxt
        result["configs"] = configs

    # --------------------------------------------------------- CPU baseline
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import oracle as O
        xs = np.random.RandomState(1).randn(R, Cn).astype(np.float32)
        O.softmax(xs)  # warm
        reps, t_cpu = 0, 0.0
        t_start = time.perf_counter()
        while t_cpu < 10.0 and reps < 2000:
            O.softmax(xs)
            reps += 1
            t_cpu = time.perf_counter() - t_start
        result["cpu_baseline"] = {
            "value": round(step_bytes * reps / t_cpu / 1e9, 3),
            "unit": "GB/s",
            "cores": 1,
            "kind": "port",
            "sample": "%d passes of the same [4096,1024] softmax (%.1f s) through the CPU port of the reference's "
                      "generated loops (4 loop nests, sequential fp32 sums, libm expf), gcc -O3 no fast-math, "
                      "%d host cores visible" % (reps, t_cpu, os.cpu_count() or 0),
            "ms_per_step": round(t_cpu * 1e3 / reps, 3),
        }

    print(json.dumps(result))


if __name__ == "__main__":
    main()
