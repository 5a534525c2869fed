"""Throughput of the hot path on one MI355X.

A step = one pass over the metric's workloads, inputs resident in HBM:
  add      c = a + b          fp32, 2^28 elements             12 B/elem  3.221 GB
  sum_ax1  M.sum(axis=-1)     fp32, 16384 x 16384 (2^28)       4 B/elem  1.074 GB
  sum_ax0  M.sum(axis=0)      same matrix                      4 B/elem  1.074 GB
  argmax   x.argmax()         fp32, 2^28 elements -> int64     4 B/elem  1.074 GB
value = algorithmic bytes of the step / wall time of the step on the GPU (GB/s, 1 GB = 1e9 B).
All calls go through the dpnp-style Python surface, hence through the C ABI of libdpnp_amd.so.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def cpu_baseline(n_log2=26, repeats=5):
    """The C restatement of the reference's algorithms (oracle/oracle_c.c) on the host cores,
    on a bounded sample: the same add / sum / argmax over 2^n_log2 elements."""
    import numpy as np

    from oracle.oracle_c import OracleC

    oc = OracleC()
    n = 1 << n_log2
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, n).astype(np.float32)
    b = rng.uniform(-1, 1, n).astype(np.float32)
    out = np.empty_like(a)
    oc.add(a, b, out)
    oc.sum(a)
    oc.argmax(a)  # warm-up (page faults, thread pool)
    t0 = time.perf_counter()
    for _ in range(repeats):
        oc.add(a, b, out)
        oc.sum(a)
        oc.sum(b)
        oc.argmax(a)
    dt = time.perf_counter() - t0
    nbytes = repeats * n * (12 + 4 + 4 + 4)
    return {
        "value": nbytes / dt / 1e9, "unit": "GB/s", "cores": oc.threads, "kind": "port",
        "sample": f"{repeats} passes of add + 2 x sum + argmax over 2^{n_log2} fp32 elements "
                  "(C/OpenMP restatement of the reference's kernels, oracle/oracle_c.c)",
    }


PRIME_STEPS = 24


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--dump-steps", action="store_true", help="print every step's per-op times to stderr")
    ap.add_argument("--ops", default="add,sum_axis1,sum_axis0,argmax",
                    help="subset of add,sum_axis1,sum_axis0,argmax,copy to run (profiling runs); the metric is "
                         "the default set")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    import dpnp_amd as dpnp

    n = 1 << 28
    side = 1 << 14
    g = torch.Generator(device="cuda").manual_seed(0)

    def uniform(count):
        t = torch.rand(count, device="cuda", generator=g, dtype=torch.float32) * 2 - 1
        arr = dpnp.empty(count, dtype="f4")
        # hand the synthetic data over through a byte copy; no torch compute in the timed region
        arr.get_array()._buf[: count * 4].copy_(t.view(torch.uint8))
        return arr

    a, b = uniform(n), uniform(n)
    x = dpnp.empty(n, dtype="f4")
    x.get_array()._buf[: n * 4].copy_(torch.randn(n, device="cuda", generator=g).view(torch.uint8))
    c = dpnp.empty(n, dtype="f4")
    M = a.reshape(side, side)
    r1, r0 = dpnp.empty(side, dtype="f4"), dpnp.empty(side, dtype="f4")
    idx = dpnp.empty((), dtype="i8")
    all_ops = [
        ("add", lambda: dpnp.add(a, b, out=c), 12 * n),
        ("sum_axis1", lambda: dpnp.sum(M, axis=1, out=r1), 4 * n + 4 * side),
        ("sum_axis0", lambda: dpnp.sum(M, axis=0, out=r0), 4 * n + 4 * side),
        ("argmax", lambda: dpnp.argmax(x, out=idx), 4 * n + 8),
        # plain copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters
        ("copy", lambda: dpnp.copyto(c, a), 8 * n),
    ]
    wanted = [w for w in args.ops.split(",") if w]
    ops = [o for o in all_ops if o[0] in wanted]
    if not ops or len(ops) != len(wanted):
        print(f"--ops: unknown op in {wanted}", file=sys.stderr)
        sys.exit(2)
    step_bytes = sum(nb for _, _, nb in ops)

    host_us = []

    def step(events=None):
        for k, (_, fn, _) in enumerate(ops):
            if events is not None:
                events[k][0].record()
            if args.dump_steps:
                h0 = time.perf_counter()
            fn()
            if args.dump_steps:
                host_us.append((time.perf_counter() - h0) * 1e6)
            if events is not None:
                events[k][1].record()

    # Process start-up, not steady state: the first launch of each kernel loads its code object,
    # and the HIP runtime stalls the submitting thread once, for 30-40 ms, a few dozen launches
    # into a process (seen on the host clock around a launch, with the GPU idle).  Both are kept
    # out of the W + K steps whatever W is.
    for _ in range(PRIME_STEPS):
        step()
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev = [[[torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)] for _ in ops]
          for _ in range(args.steps)]
    t_begin, t_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    del host_us[:]
    wall0 = time.perf_counter()
    t_begin.record()
    for s in range(args.steps):
        step(ev[s])
    t_end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    gpu_ms = t_begin.elapsed_time(t_end)
    ms_per_step = max(gpu_ms, wall * 1e3) / args.steps
    per_op = {}
    for k, (name, _, nb) in enumerate(ops):
        ms = sum(ev[s][k][0].elapsed_time(ev[s][k][1]) for s in range(args.steps)) / args.steps
        per_op[name] = {"ms": round(ms, 5), "GB/s": round(nb / ms / 1e6, 1), "frac_of_peak": round(nb / ms / 1e6 / HBM_PEAK_GBS, 4),
                        "elements/s": round(n / ms * 1e3)}
    if args.dump_steps:
        for s in range(args.steps):
            print(s, " ".join("%s=%.4f(host %.0fus)" % (ops[k][0], ev[s][k][0].elapsed_time(ev[s][k][1]),
                                                         host_us[s * len(ops) + k]) for k in range(len(ops))),
                  file=sys.stderr)
    add_ms = per_op["add"]["ms"] if "add" in per_op else float("nan")
    out = {
        "metric": "achieved HBM GB/s for fp32 add, axis-sum, argmax at 2^28 elements",
        "value": round(step_bytes / ms_per_step / 1e6, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded uniform[-1,1) and normal(0,1), resident in HBM)",
        "config": {"workload": "fp32 add 2^28 + sum axis=-1 and axis=0 over 16384x16384 + argmax 2^28 (->int64)"
                   if args.ops == ap.get_default("ops") else "subset: " + args.ops,
                   "bytes_per_step": step_bytes, "frac_of_hbm_peak": round(step_bytes / ms_per_step / 1e6 / HBM_PEAK_GBS, 4)},
        "per_op": per_op,
        "roofline": {"bound": "hbm", "kernel": "ew_contig_kernel<add,f32> (c = a + b, 2^28 elements)",
                     "achieved": round(12 * n / add_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(12 * n / add_ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None},
    }
    traffic_file = os.path.join(ROOT, "profiles", "add_f32_2p28_traffic.json")
    if os.path.exists(traffic_file):  # HBM bytes per launch from the committed rocprofv3 --pmc summary
        out["roofline"]["traffic"] = json.load(open(traffic_file)).get("bytes_per_launch")
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
