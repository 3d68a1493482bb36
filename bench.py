#!/usr/bin/env python3
"""FBW loss+grad benchmark on one MI355X.

One step = one call of i6fbw_run (C ABI of libi6fbw.so) on the headline workload
(CART-state full-sum, T=1000, B=32, F=12001, fp32) with all inputs, outputs and the
workspace resident in HBM; the call covers edge preparation, emission gather, alpha/beta
recursion, per-frame normalisation and the dense (T,B,F) posterior write.

Prints ONE JSON line.  `value` is the achieved algorithmic bandwidth of the whole call
(bytes = 4*T*B*F + 4*sum_b seq_len_b*E_b + 20*E + 4*T*B + 12*B, every datum once);
`ms_per_step` is ms per loss+grad call.  `roofline` prices the dominant kernel (the combine
kernel that writes the dense tensor) against 8 TB/s with durations taken from HIP events on
the stream it runs on; `cpu_baseline` times the fp32 CPU port of the reference algorithm
(oracle/fbw_oracle.c) on the host cores in the same run.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cart", help="tiny | monophone | cart | ctc | longform")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-wrapper", action="store_true", help="skip the wrapper-level (fbw_loss + backward) timing")
    ap.add_argument("--no-best-path", action="store_true", help="skip the best-path (Viterbi) timing")
    ap.add_argument("--out-mode", type=int, default=1, help="0: -log posterior with +inf holes, 1: posterior")
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
    dev = torch.device("cuda:0")
    am = torch.from_numpy(W.am_scores).to(dev)
    edges = torch.from_numpy(W.edges).to(dev)
    weights = torch.from_numpy(W.weights).to(dev)
    start_end = torch.from_numpy(W.start_end_states).to(dev)
    seq_lens = torch.from_numpy(W.seq_lens).to(dev)
    out = torch.empty((W.T, W.B, W.F), dtype=torch.float32, device=dev)
    loss = torch.empty((W.T, W.B), dtype=torch.float32, device=dev)
    ws_bytes = cabi.workspace_size(W.T, W.B, W.F, W.E, W.n_states)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def step():
        cabi.run(am.data_ptr(), am.stride(0), am.stride(1), edges.data_ptr(), edges.stride(0), weights.data_ptr(),
                 start_end.data_ptr(), start_end.stride(0), seq_lens.data_ptr(), W.T, W.B, W.F, W.E, W.n_states,
                 args.out_mode, out.data_ptr(), loss.data_ptr(), ws.data_ptr(), ws_bytes, stream)

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)      # an elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    step()
    code, seq = cabi.read_status(ws.data_ptr(), W.B, stream)
    if code != 0:
        raise cabi.FbwError(code, seq)
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

    alg_bytes = W.algorithmic_bytes()
    gbps = alg_bytes / (ms_per_call * 1e-3) / 1e9
    # dominant kernel: fbw_combine, which writes the F-wide posterior row and the loss of every frame
    # that carries probability mass: (4*F + 4) bytes per row, sum_b seq_len_b rows per call, spread
    # over the combine launches of one call (their durations are summed; fbw_padfill writes the
    # remaining rows and is timed separately)
    comb_bytes = (4 * W.F + 4) * W.seq_frames()
    comb_ms = stage_ms[3]
    comb_gbps = comb_bytes / (comb_ms * 1e-3) / 1e9 if comb_ms > 0 else 0.0
    # HBM bytes per call of the dominant kernel, from the committed rocprofv3 --pmc summary
    # (FETCH_SIZE and WRITE_SIZE, each scaled by what it reads for a copy kernel of known size)
    traffic = None
    tpath = os.path.join(ROOT, "profiles", f"fbw_{args.workload}_hbm_traffic.txt")
    if os.path.exists(tpath):
        import re
        m = re.search(r"fbw_combine, scaled:.*= ([0-9.]+) MB per launch", open(tpath).read())
        if m:
            traffic = int(float(m.group(1)) * 1e6)

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
                               f"seed={1001 + ['tiny', 'monophone', 'cart', 'ctc', 'longform'].index(args.workload)}",
                   "out_mode": "posterior" if args.out_mode == 1 else "neg_log",
                   "algorithmic_bytes": alg_bytes,
                   "frac_of_hbm_peak": round(gbps / HBM_PEAK_GBPS, 4),
                   "seq_frames_per_s": round(W.seq_frames() / (ms_per_call * 1e-3), 1),
                   "stage_ms": {k: round(v, 4) for k, v in zip(cabi.STAGE_NAMES, stage_ms)}},
        "roofline": {"bound": "hbm", "kernel": "fbw_combine", "achieved": round(comb_gbps, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(comb_gbps / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "algorithmic_bytes_per_call": comb_bytes, "kernel_ms_per_call": round(comb_ms, 4)},
    }

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
        cores = os.cpu_count() or 1
        try:
            cores = len(os.sched_getaffinity(0))
        except AttributeError:
            pass
        threads = max(1, min(W.B, cores, fbw_oracle.max_threads()))
        reps, t_cpu = 0, 0.0
        while reps < 3 or (t_cpu < 10.0 and reps < 20):
            t0 = time.perf_counter()
            fbw_oracle.fbw_oracle(W.am_scores, W.edges, W.weights, W.start_end_states, W.seq_lens, W.n_states,
                                  precision="f32", threads=threads)
            t_cpu += time.perf_counter() - t0
            reps += 1
        cpu_ms = t_cpu / reps * 1e3
        result["cpu_baseline"] = {
            "value": round(alg_bytes / (cpu_ms * 1e-3) / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "ms_per_call": round(cpu_ms, 2),
            "sample": f"whole {args.workload} workload, {reps} calls of the fp32 CPU port of the reference algorithm "
                      f"(per-frame edge sweeps, normalise, scatter), OpenMP over sequences",
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
