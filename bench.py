#!/usr/bin/env python3
"""FBW loss+grad benchmark on one MI355X.

One step = one call of i6fbw_run (C ABI of libi6fbw.so) on the headline workload
(CART-state full-sum, T=1000, B=32, F=12001, fp32) with all inputs, outputs and the
workspace resident in HBM; the call covers edge preparation, emission gather, alpha/beta
recursion, per-frame normalisation and the dense (T,B,F) posterior write.

Prints ONE JSON line.  `value` is the achieved algorithmic bandwidth of the whole call
(bytes = 4*T*B*F + 4*sum_b seq_len_b*E_b + 20*E + 4*T*B + 12*B, every datum once);
`ms_per_step` is ms per loss+grad call.  `roofline` prices the dominant kernel (the one that
writes the dense tensor: fbw_flat, or fbw_combine where the row writer runs) against 8 TB/s with
durations taken from HIP events on the stream it runs on; `cpu_baseline` times the fp32 CPU port
of the reference algorithm (oracle/fbw_oracle.c) on the host cores in the same run, with all
cores and with one; `config.per_config` holds, for each of the five benchmark configurations,
the time per call (median and minimum over single calls timed with HIP events), the roofline
fraction, sequence-frames per second and the worst loss / posterior error against the fp64 oracle.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
NAMES = ["tiny", "monophone", "cart", "ctc", "longform"]


class Problem:
    """One workload resident on the device, called through the C ABI."""

    def __init__(self, W, out_mode):
        import torch
        from i6_native_ops_amd import cabi
        self.W, self.out_mode, self.cabi, self.torch = W, out_mode, cabi, torch
        dev = torch.device("cuda:0")
        self.am = torch.from_numpy(W.am_scores).to(dev)
        self.edges = torch.from_numpy(W.edges).to(dev)
        self.weights = torch.from_numpy(W.weights).to(dev)
        self.start_end = torch.from_numpy(W.start_end_states).to(dev)
        self.seq_lens = torch.from_numpy(W.seq_lens).to(dev)
        self.out = torch.empty((W.T, W.B, W.F), dtype=torch.float32, device=dev)
        self.loss = torch.empty((W.T, W.B), dtype=torch.float32, device=dev)
        self.ws_bytes = cabi.workspace_size(W.T, W.B, W.F, W.E, W.n_states)
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device=dev)
        self.stream = torch.cuda.current_stream().cuda_stream

    def step(self):
        W = self.W
        self.cabi.run(self.am.data_ptr(), self.am.stride(0), self.am.stride(1), self.edges.data_ptr(), self.edges.stride(0),
                      self.weights.data_ptr(), self.start_end.data_ptr(), self.start_end.stride(0), self.seq_lens.data_ptr(),
                      W.T, W.B, W.F, W.E, W.n_states, self.out_mode, self.out.data_ptr(), self.loss.data_ptr(),
                      self.ws.data_ptr(), self.ws_bytes, self.stream)

    def check(self):
        code, seq = self.cabi.read_status(self.ws.data_ptr(), self.W.B, self.stream)
        if code != 0:
            raise self.cabi.FbwError(code, seq)

    def single_call_times(self, n, warmup):
        """ms of n single calls, each bracketed by HIP events on the stream the call is made on (the
        library joins its own streams into it before the call returns)"""
        torch = self.torch
        for _ in range(warmup):
            self.step()
        torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for a, b in ev:
            a.record()
            self.step()
            b.record()
        torch.cuda.synchronize()
        return sorted(a.elapsed_time(b) for a, b in ev)


def cpu_threads(W, fbw_oracle):
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    return max(1, min(W.B, cores, fbw_oracle.max_threads()))


def committed_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 --pmc summary of this workload (counters need the
    profiler, so they are not measured in this run), the name of that summary, and whether it was made from other kernel
    sources than the ones here (it records their digest)."""
    tpath = os.path.join(ROOT, "profiles", f"fbw_{workload}_hbm_traffic.txt")
    if not os.path.exists(tpath):
        return None, None, None
    import re
    text = open(tpath).read()
    m = re.search(kernel + r", scaled:.*= ([0-9.]+) MB per launch", text)
    if not m:
        return None, None, None
    from i6_native_ops_amd import build
    d = re.search(r"kernel sources sha256: ([0-9a-f]+)", text)
    stale = not (d and d.group(1) == build.sources_digest())
    return (int(float(m.group(1)) * 1e6),
            f"profiles/fbw_{workload}_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, committed)", stale)


def per_config_entry(name, headline=None):
    """Timing and parity of one benchmark configuration (the headline's device problem is reused)."""
    import numpy as np
    from i6_native_ops_amd.fbw.workloads import make_workload
    from oracle import fbw_oracle
    P = headline if headline is not None else Problem(make_workload(name), 1)
    W = P.W
    P.step()
    P.check()
    # the -log output, what the reference's own binding fbw_core.fbw returns (fbw_op.cu:366-377,392), first; the
    # posterior mode is timed last, so that its results are the ones checked below
    P.out_mode = 0
    neg_log = P.single_call_times(15, 3)
    P.out_mode = 1
    times = P.single_call_times(30, 5)
    med, mn = times[len(times) // 2], times[0]
    alg = W.algorithmic_bytes()
    # parity against the fp64 oracle at full size: relative error of the loss, absolute error of the posteriors
    want_out, want_loss = fbw_oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states,
                                                threads=cpu_threads(W, fbw_oracle))
    loss = P.loss.cpu().numpy()
    nz = want_loss != 0
    loss_err = float(np.max(np.abs(loss[nz] - want_loss[nz]) / np.abs(want_loss[nz]))) if nz.any() else 0.0
    post_err = 0.0
    out = P.out.cpu().numpy()
    for t0 in range(0, W.T, 64):          # in slices: exp of the whole oracle tensor at once doubles the host memory
        post_err = max(post_err, float(np.max(np.abs(out[t0:t0 + 64] - np.exp(-want_out[t0:t0 + 64].astype(np.float64))))))
    from i6_native_ops_amd import cabi
    writer = "fbw_flat" if cabi.last_dense_writer() == 1 else "fbw_combine"
    traffic, _, stale = committed_traffic(name, writer)
    return {"T": W.T, "B": W.B, "F": W.F, "E": W.E, "ms_median": round(med, 4), "ms_min": round(mn, 4),
            "dense_writer": writer, "dense_writer_traffic": traffic, "traffic_stale": stale,
            "neg_log_ms_median": round(neg_log[len(neg_log) // 2], 4),
            "algorithmic_bytes": alg, "gbps": round(alg / (med * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(alg / (med * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "seq_frames_per_s": round(W.seq_frames() / (med * 1e-3), 1),
            "loss_rel_err": float("%.3g" % loss_err), "posterior_abs_err": float("%.3g" % post_err)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cart", help="tiny | monophone | cart | ctc | longform")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-wrapper", action="store_true", help="skip the wrapper-level (fbw_loss + backward) timing")
    ap.add_argument("--no-best-path", action="store_true", help="skip the best-path (Viterbi) timing")
    ap.add_argument("--no-per-config", action="store_true",
                    help="skip the per-configuration table (timings and errors against the oracle for all five workloads)")
    ap.add_argument("--out-mode", type=int, default=1, help="0: -log posterior with +inf holes, 1: posterior")
    ap.add_argument("--no-other-mode", action="store_true",
                    help="skip the timing of the other output mode (a profile of the run then holds the kernels of one mode only)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain elementwise copy kernel over 1 GiB (3 times) so that a rocprofv3 --pmc run of "
                         "this command shows what FETCH_SIZE / WRITE_SIZE read for a known amount of traffic")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU only (sequences are independent; sharding the batch over "
              "GPUs needs no exchange and is not implemented). Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from i6_native_ops_amd import cabi
    from i6_native_ops_amd.fbw.workloads import make_workload

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    cabi.load()   # fails loudly if the HIP library is not built

    W = make_workload(args.workload)
    P = Problem(W, args.out_mode)
    dev = torch.device("cuda:0")
    am, edges, weights, start_end, seq_lens, ws, ws_bytes, stream = (P.am, P.edges, P.weights, P.start_end, P.seq_lens, P.ws,
                                                                      P.ws_bytes, P.stream)
    step = P.step

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)      # an elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    step()
    P.check()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # whole-call time: host clock around K back-to-back calls, device idle on both sides
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_call = elapsed / args.steps * 1e3

    # per-stage device time: HIP events recorded between the stages on the launch stream
    cabi.profile_enable(True)
    n_prof = min(args.steps, 200)
    for _ in range(n_prof):
        step()
    torch.cuda.synchronize()
    _, stage_ms = cabi.profile_read()
    cabi.profile_enable(False)
    flat = cabi.last_dense_writer() == 1

    alg_bytes = W.algorithmic_bytes()
    gbps = alg_bytes / (ms_per_call * 1e-3) / 1e9
    # Dominant kernel: the one that writes the dense tensor.  fbw_flat writes all T*B rows of F floats and
    # the loss of every frame, 4*T*B*F + 4*T*B bytes per launch; where the row writer runs, fbw_combine
    # writes the rows of the frames that carry probability mass, (4*F + 4) bytes each, sum_b seq_len_b
    # rows per launch (fbw_padfill writes the others and is timed separately).
    kernel = "fbw_flat" if flat else "fbw_combine"
    comb_bytes = 4 * W.T * W.B * W.F + 4 * W.T * W.B if flat else (4 * W.F + 4) * W.seq_frames()
    comb_ms = stage_ms[3]
    comb_gbps = comb_bytes / (comb_ms * 1e-3) / 1e9 if comb_ms > 0 else 0.0
    # HBM bytes per launch of that kernel: not measured in this run (counters need the profiler); the
    # figure comes from the committed rocprofv3 --pmc summary of this command and names it
    traffic, traffic_source, traffic_stale = committed_traffic(args.workload, kernel)

    result = {
        "metric": f"FBW loss+grad ms/call + achieved HBM GB/s at T={W.T},B={W.B},F={W.F} fp32",
        "value": round(gbps, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_call, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: T={W.T} B={W.B} F={W.F} E={W.E} states={W.n_states}, "
                               f"seed={1001 + NAMES.index(args.workload)}",
                   "out_mode": "posterior" if args.out_mode == 1 else "neg_log",
                   "algorithmic_bytes": alg_bytes,
                   "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
                   "seq_frames_per_s": round(W.seq_frames() / (ms_per_call * 1e-3), 1),
                   "stage_ms": {k: round(v, 4) for k, v in zip(cabi.STAGE_NAMES, stage_ms)}},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(comb_gbps, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(comb_gbps / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "traffic_source": traffic_source, "traffic_stale": traffic_stale,
                     "algorithmic_bytes_per_launch": comb_bytes, "kernel_ms_per_launch": round(comb_ms, 4)},
    }

    # the other output mode of the same call (informational): -log posteriors with +inf holes, as the reference's binding
    # fbw_core.fbw returns them (fbw_op.cu:366-377,392), when the timed mode is the posterior, and the other way round
    if not args.no_other_mode:
        other = Problem.__new__(Problem)
        other.__dict__.update(P.__dict__)
        other.out_mode = 0 if args.out_mode == 1 else 1
        ot = other.single_call_times(20, 5)
        result["config"]["neg_log_ms" if args.out_mode == 1 else "posterior_ms"] = round(ot[len(ot) // 2], 4)
        if args.out_mode == 1:
            step()      # the headline problem's buffers hold the posterior mode's results again (the per-config table checks them)
            torch.cuda.synchronize()

    # wrapper level (informational): fbw_loss(log_probs[B,T,F]).sum().backward() with the fused front end
    # and with the reference's literal neg/transpose/contiguous/exp chain around the same kernels
    if not args.no_wrapper:
        from i6_native_ops_amd.fbw import fbw_loss, fbw_loss_unfused
        fsa = (W.n_states, edges, weights, start_end)
        base = am.neg().transpose(0, 1).contiguous()
        wl = {}
        for name, fn in (("fused_ms", fbw_loss), ("unfused_ms", fbw_loss_unfused)):
            lp = base.clone().requires_grad_(True)
            for it in range(8):
                if it == 3:
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                lp.grad = None
                fn(lp, fsa, seq_lens).sum().backward()
            torch.cuda.synchronize()
            wl[name] = round((time.perf_counter() - t0) / 5 * 1e3, 4)
            del lp
        result["config"]["wrapper_level"] = wl
        del base

    # best path on the same automata (informational): i6fbw_viterbi maximises, so it gets -am and -weights
    if not args.no_best_path:
        vam = am.neg()
        vw = weights.neg()
        align = torch.empty((W.T, W.B), dtype=torch.int32, device=dev)
        scores = torch.empty((W.B,), dtype=torch.float32, device=dev)

        def vstep():
            cabi.viterbi(vam.data_ptr(), vam.stride(0), vam.stride(1), edges.data_ptr(), edges.stride(0), vw.data_ptr(),
                         start_end.data_ptr(), start_end.stride(0), seq_lens.data_ptr(), W.T, W.B, W.F, W.E, W.n_states,
                         align.data_ptr(), align.stride(0), align.stride(1), scores.data_ptr(), ws.data_ptr(), ws_bytes,
                         stream)
        for _ in range(5):
            vstep()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            vstep()
        torch.cuda.synchronize()
        bp = {"ms_per_call": round((time.perf_counter() - t0) / 20 * 1e3, 4)}
        if not args.no_cpu_baseline:
            from oracle import fbw_oracle
            t0 = time.perf_counter()
            fbw_oracle.viterbi_oracle(-W.am_scores, W.edges, -W.weights, W.start_end_states, W.seq_lens, W.n_states)
            bp["cpu_port_ms_per_call"] = round((time.perf_counter() - t0) * 1e3, 2)
            bp["cpu_port_cores"] = 1
        result["config"]["best_path"] = bp
        del vam, vw

    if not args.no_cpu_baseline:
        from oracle import fbw_oracle
        threads = cpu_threads(W, fbw_oracle)

        def cpu_ms(nthreads, budget_s):
            reps, t_cpu = 0, 0.0
            while reps < 3 or (t_cpu < budget_s and reps < 20):
                t0 = time.perf_counter()
                fbw_oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states,
                                      precision="f32", threads=nthreads)
                t_cpu += time.perf_counter() - t0
                reps += 1
            return t_cpu / reps * 1e3, reps
        ms_all, reps = cpu_ms(threads, 10.0)
        ms_one, reps_one = cpu_ms(1, 0.0)
        result["cpu_baseline"] = {
            "value": round(alg_bytes / (ms_all * 1e-3) / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "ms_per_call": round(ms_all, 2),
            "one_thread": {"value": round(alg_bytes / (ms_one * 1e-3) / 1e9, 3), "unit": "GB/s", "cores": 1,
                           "ms_per_call": round(ms_one, 2), "calls": reps_one},
            "sample": f"whole {args.workload} workload, {reps} calls of the fp32 CPU port of the reference algorithm "
                      f"(per-frame edge sweeps, normalise, scatter), OpenMP over sequences",
        }

    # all five configurations: time per call and parity against the fp64 oracle at full size
    if not args.no_per_config:
        per = {}
        for name in NAMES:
            reuse = P if (name == args.workload and args.out_mode == 1) else None
            if reuse is None and name == args.workload:
                continue
            per[name] = per_config_entry(name, reuse)
            if reuse is None:
                torch.cuda.empty_cache()
        result["config"]["per_config"] = per
    print(json.dumps(result))


if __name__ == "__main__":
    main()
