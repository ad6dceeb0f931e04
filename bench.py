#!/usr/bin/env python3
"""Benchmark of the bidirectional linear-attention hot path on one MI355X.

Default workload (BASELINE.json configs[1] at the headline length): linear_attn
fused forward+backward, B=8, H=16, D=64, T=16384, fp16, eps=1e-6, scale=1/T,
q,k = elu(N(0,1))+1, v,dO ~ N(0,1) (synthetic, seeded).  One step is
`linear_attention(q, k, v).backward(dO)` (benchmarks/ops/benchmark_linear_attn.py:56).

Prints ONE JSON line:  value = algorithmic HBM bytes of a step / time per step
(GB/s), with `roofline` (dominant kernel, timed live with events on the launch
stream) and `cpu_baseline` (the torch restatement of the reference's naive
operator, on the host cores, on a bounded sample of the same workload).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--T 16384] [--sweep]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "flash-bidirectional-linear-attention_amd"), os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

# the per-kernel timings below launch single kernels through the library's phase mask, which the
# library only honours in a process that asked for it
os.environ.setdefault("FBLA_ALLOW_PHASE_MASK", "1")

import torch  # noqa: E402
import torch.nn.functional as F  # noqa: E402

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

CLOCK_RAMP_S = 0.1  # untimed work before the warm-up steps

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "linear_attn_fwd_bwd_B8H16T16384D64_fp16_hbm_traffic.md")
TRAFFIC_ROW = {"fwd_state": "state_kernel", "fwd_output": "rows_kernel NORM", "bwd_pass_a": "bwd_a_kernel",
               "bwd_pass_b": "rows_kernel x2"}


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` at the default workload, read from the counter summary
    under profiles/ (column "HBM MiB" of its table); None when the file or the row is missing."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                cells = [c.strip() for c in line.split("|")]
                if len(cells) > 6 and cells[1].startswith(TRAFFIC_ROW[kernel]):
                    return int(float(cells[5]) * 2 ** 20)
    except (OSError, ValueError, KeyError):
        pass
    return None


PHASES = {  # name -> (phase bit, tensors read+written once, entry point)
    "fwd_state": (1, 2, "fwd"),     # reads k, v
    "fwd_output": (4, 2, "fwd"),    # reads q, writes o
    "bwd_pass_a": (8, 3, "bwd"),    # reads q, dO, writes dq
    "bwd_pass_b": (32, 4, "bwd"),   # reads k, v, writes dk, dv
}


def make_inputs(B, H, T, D, dtype, device, seed=42):
    g = torch.Generator(device=device).manual_seed(seed)
    shape = (B, H, T, D)
    q = (F.elu(torch.randn(shape, generator=g, device=device)) + 1).to(dtype)
    k = (F.elu(torch.randn(shape, generator=g, device=device)) + 1).to(dtype)
    v = torch.randn(shape, generator=g, device=device).to(dtype)
    do = torch.randn(shape, generator=g, device=device).to(dtype)
    return q, k, v, do


def timed_loop(fn, n):
    """Average ms per call over n back-to-back calls, events on the current stream."""
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(n):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / n


def do_bench(fn, flush, quantiles=(0.5, 0.2, 0.8)):
    """Triton-free restatement of triton.testing.do_bench as used by
    benchmarks/ops/benchmark_linear_attn.py:45-58: warm call, 5-call estimate,
    ~25 ms warmup, ~100 ms of timed calls, cache-flush write before every call,
    one event pair per call, quantiles of the per-call times."""
    fn()
    torch.cuda.synchronize()
    est = timed_loop(lambda: (flush.zero_(), fn()), 5)
    n_warmup, n_repeat = max(1, int(25 / est)), max(1, int(100 / est))
    for _ in range(n_warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for i in range(n_repeat):
        flush.zero_()
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    times = torch.tensor([s.elapsed_time(e) for s, e in zip(starts, ends)], dtype=torch.float64)
    return [float(x) for x in torch.quantile(times, torch.tensor(quantiles, dtype=torch.float64))]


def _cpu_time(fn, reps):
    times = []
    for _ in range(reps + 1):  # the first run warms the allocator and the thread pool
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return sorted(times[1:])[len(times[1:]) // 2]


def _cpu_inputs(shape, dtype_round, seed=42):
    g = torch.Generator().manual_seed(seed)
    q = F.elu(torch.randn(shape, generator=g)) + 1
    k = F.elu(torch.randn(shape, generator=g)) + 1
    v = torch.randn(shape, generator=g)
    do = torch.randn(shape, generator=g)
    if dtype_round is not None:  # fp32 math on values already rounded to the GPU workload's type
        q, k, v, do = (t.to(dtype_round).float() for t in (q, k, v, do))
    return q, k, v, do


def cpu_baseline(T, D, H, sample_batches, reps=3):
    """Reference torch path (oracle.torch_ref, the restatement of the reference's naive operators,
    + autograd) on the host cores.  The headline entry is linear_attn fwd+bwd on `sample_batches`
    of the 8 batches of the workload; `configs` adds BASELINE config 1 (forward, fp32, 10 runs) and
    the other lengths of config 2, each on a bounded sample."""
    from oracle import torch_ref
    torch.set_num_threads(os.cpu_count() or 1)
    cores = torch.get_num_threads()

    def fwd_bwd_entry(Tn, batches, nreps):
        q, k, v, do = _cpu_inputs((batches, H, Tn, D), torch.float16)
        for t in (q, k, v):
            t.requires_grad_()

        def run():
            q.grad = k.grad = v.grad = None
            torch_ref.naive_linear_attn(q, k, v).backward(do)
        t = _cpu_time(run, nreps)
        nbytes = 11 * batches * H * Tn * D * 2
        return {"config": f"C2 linear_attn fwd+bwd T={Tn}", "value": round(nbytes / t / 1e9, 3), "unit": "GB/s",
                "ms": round(t * 1e3, 3), "reps": nreps,
                "sample": f"{batches} of 8 batches (B{batches},H{H},T{Tn},D{D}), fp32 math on the fp16-valued "
                          f"inputs; bytes counted as the fp16 workload's 11 tensor passes"}

    head = fwd_bwd_entry(T, sample_batches, reps)
    configs = []
    # BASELINE config 1: the reference's own CPU-runnable case, forward, fp32
    q, k, v, _ = _cpu_inputs((2, 4, 1024, 64), None)
    nb1 = 4 * q.numel() * 4
    with torch.no_grad():
        for name, fn in (("simple_la", lambda: torch_ref.naive_simple_la(q, k, v)),
                         ("linear_attn", lambda: torch_ref.naive_linear_attn(q, k, v))):
            t = _cpu_time(fn, 10)
            configs.append({"config": f"C1 {name} forward B2-H4-T1024-D64 fp32", "value": round(nb1 / t / 1e9, 3),
                            "unit": "GB/s", "ms": round(t * 1e3, 3), "reps": 10,
                            "sample": "the whole config; bytes = 4 fp32 tensor passes"})
    for Tn, batches, nreps in ((1024, 8, 5), (4096, 8, 3), (32768, 1, 2)):
        if Tn != T:
            configs.append(fwd_bwd_entry(Tn, batches, nreps))
    return {
        "value": head["value"], "unit": "GB/s", "cores": cores, "kind": "port",
        "sample": f"linear_attn fwd+bwd, {head['sample']}, median of {reps} runs; {head['ms']:.1f} ms per run",
        "ms": head["ms"], "configs": configs,
    }


def parity_spot_check(q, k, v, do, o, grads, heads=((0, 0), (7, 15))):
    from helpers import np64, parity_errors
    from oracle import closed_form as cf
    out = {}
    for b, h in heads:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = cf.dense_backward(np64(q[sl]), np64(k[sl]), np64(v[sl]), np64(do[sl]), 1.0 / q.shape[2])
        for name, t in (("o", o), ("dq", grads[0]), ("dk", grads[1]), ("dv", grads[2])):
            plain, excess, ok = parity_errors(t[sl], ref[name], q.dtype, ref.get(name + "_mag"))
            prev = out.get(name, (0.0, 0.0, True))
            out[name] = (max(prev[0], plain), max(prev[1], excess), prev[2] and ok)
    return {n: {"max_rel": round(p, 7), "excess": round(e, 7), "ok": ok} for n, (p, e, ok) in out.items()}


def kernel_times(q, k, v, do, n=20):
    """Average duration of each large kernel, launched alone through the phase mask."""
    from flash_bla import _hip
    lib = _hip.lib()
    T = q.shape[2]
    scale, eps = 1.0 / T, 1e-6
    o, s, km = _hip.la_fwd(q, k, v, None, None, scale, eps, _hip.NORMALIZE)
    res = {}
    for name, (bit, passes, entry) in PHASES.items():
        lib.fbla_set_phase_mask(bit)
        try:
            if entry == "fwd":
                fn = lambda: _hip.la_fwd(q, k, v, None, None, scale, eps, _hip.NORMALIZE)  # noqa: E731
            else:
                fn = lambda: _hip.la_bwd(q, k, v, None, None, do, s, km, scale, eps, _hip.NORMALIZE)  # noqa: E731
            for _ in range(3):
                fn()
            ms = timed_loop(fn, n)
        finally:
            lib.fbla_set_phase_mask(0)
        nbytes = passes * q.numel() * q.element_size()
        res[name] = {"ms": round(ms, 5), "alg_bytes": nbytes, "gbps": round(nbytes / ms / 1e6, 1),
                     "frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=200,
                    help="untimed steps first: a few milliseconds of work do not bring the GPU to its steady clocks")
    ap.add_argument("--T", type=int, default=16384)
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16", "fp32"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true",
                    help="skip the table over T in {1024,4096,16384,32768} (the `sweep` list of the JSON line)")
    ap.add_argument("--sweep", action="store_true", help="accepted for compatibility: the sweep is on by default")
    ap.add_argument("--tables-md", default=None, metavar="PATH",
                    help="with --tables: also write the tables as markdown to PATH")
    ap.add_argument("--probe", type=int, default=0, metavar="N",
                    help="counter-collection mode for rocprofv3 --pmc: run N steps of the workload, each "
                         "followed by a 256 MiB device copy of known traffic, then exit")
    ap.add_argument("--tables", action="store_true",
                    help="also print the reference's benchmark tables (torch formula, this library, SDPA) on stderr")
    ap.add_argument("--only", choices=["c3", "c5", "fm", "callers"], default=None,
                    help="profiling aid: time just BASELINE config 3 (packed variable-length, D=64 and "
                         "D=128), config 5 (piecewise attention), the feature map together with the "
                         "attention (fm) or the decoupled operator and the layer callers' head dims "
                         "(callers), table on stderr, no headline line")
    ap.add_argument("--configs", action="store_true",
                    help="also time the other operator families / BASELINE configs (table on stderr)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path needs no collective: heads "
              "are independent); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    from flash_bla.ops.linear_attn.fused import linear_attention
    dtype = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    B, H, D, T = 8, 16, 64, args.T
    dev = torch.device("cuda:0")
    if args.only:
        flush = torch.empty(256 << 20, dtype=torch.int8, device=dev)
        if args.only == "c3":
            varlen_config(dev, flush)
        elif args.only == "fm":
            feature_map_config(dev, flush)
        elif args.only == "callers":
            caller_configs(dev, flush)
        else:
            piecewise_config(dev, flush)
        return
    q, k, v, do = make_inputs(B, H, T, D, dtype, dev)
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    tensor_bytes = q.numel() * q.element_size()
    fwd_bytes, step_bytes = 4 * tensor_bytes, 11 * tensor_bytes

    def step():
        q.grad = k.grad = v.grad = None
        linear_attention(q, k, v).backward(do)

    def fwd_only():
        with torch.no_grad():
            return linear_attention(q, k, v)

    if args.probe:
        a = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        b = torch.empty_like(a)
        for _ in range(args.probe):
            step()
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"probe_steps": args.probe, "copy_bytes_each_way": a.numel()}))
        return

    # the GPU reaches its steady clocks only after tens of milliseconds of work: bring it there
    # first, whatever W is (untimed, like the W warm-up steps that follow)
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < CLOCK_RAMP_S:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    o = fwd_only()
    parity = parity_spot_check(q.detach(), k.detach(), v.detach(), do, o, (q.grad, k.grad, v.grad))

    flush = torch.empty(256 << 20, dtype=torch.int8, device=dev)
    for _ in range(args.warmup):
        fwd_only()
    # back-to-back, no cache-flush write in between; an auxiliary figure (the headline `value` times
    # exactly K steps): at least 200 calls, so that with a small K the first launches after the
    # synchronisation, which no queued work hides, do not weigh on it
    fwd_steps = max(args.steps, 200)
    fwd_loop_ms = timed_loop(fwd_only, fwd_steps)
    fwd_q = do_bench(fwd_only, flush)
    step_q = do_bench(step, flush)
    kern = kernel_times(q.detach(), k.detach(), v.detach(), do)
    dom = max(kern, key=lambda n: kern[n]["ms"])
    roofline = {
        "bound": "hbm", "kernel": dom, "achieved": kern[dom]["gbps"], "peak": HBM_PEAK_GBPS,
        "unit": "GB/s", "frac": kern[dom]["frac"],
        "traffic": measured_traffic(dom) if (T == 16384 and args.dtype == "fp16") else None,
        "traffic_source": os.path.relpath(TRAFFIC_PROFILE, ROOT),
        "alg_bytes_per_launch": kern[dom]["alg_bytes"], "avg_launch_ms": kern[dom]["ms"],
    }
    cpu = None if args.no_cpu else cpu_baseline(T, D, H, sample_batches=2)
    # context: what a plain device-to-device copy reaches on this box (read + write bytes)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    copy_ms = timed_loop(lambda: dst.copy_(src), 10)
    copy_gbps = round(2 * src.numel() / copy_ms / 1e6, 1)
    del src, dst

    line = {
        "metric": "linear_attn fwd+bwd ms and achieved HBM GB/s, B8-H16-D64 T=16384 fp16",
        "value": round(step_bytes / ms_per_step / 1e6, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "clock_ramp_s": CLOCK_RAMP_S,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": f"linear_attn fused fwd+bwd B{B}-H{H}-D{D} T={T} {args.dtype} eps=1e-6 scale=1/T",
                   "alg_bytes_per_step": step_bytes, "tensor_passes": 11},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "fwd_bwd": {"ms_p50_p20_p80_flushed": [round(x, 5) for x in step_q],
                    "gbps_p50": round(step_bytes / step_q[0] / 1e6, 1),
                    "frac_of_peak": round(step_bytes / step_q[0] / 1e6 / HBM_PEAK_GBPS, 4),
                    "frac_back_to_back": round(step_bytes / ms_per_step / 1e6 / HBM_PEAK_GBPS, 4)},
        "fwd": {"ms_back_to_back": round(fwd_loop_ms, 5), "calls_back_to_back": fwd_steps,
                "gbps_back_to_back": round(fwd_bytes / fwd_loop_ms / 1e6, 1),
                "frac_back_to_back": round(fwd_bytes / fwd_loop_ms / 1e6 / HBM_PEAK_GBPS, 4),
                "ms_p50_p20_p80_flushed": [round(x, 5) for x in fwd_q], "alg_bytes": fwd_bytes,
                "gbps_p50": round(fwd_bytes / fwd_q[0] / 1e6, 1),
                "frac_of_peak": round(fwd_bytes / fwd_q[0] / 1e6 / HBM_PEAK_GBPS, 4)},
        "kernels": kern,
        "device_copy_gbps": copy_gbps,
        "parity": parity,
    }
    if not args.no_sweep:
        del q, k, v, do, o
        line["sweep"] = sweep(dtype, dev, flush)
    if args.configs:
        other_configs(dev, flush)
        layer_config(dev, flush)
        piecewise_config(dev, flush)
    if args.tables:
        reference_tables(dev, flush, args.tables_md)
    print(json.dumps(line), flush=True)


def sweep(dtype, dev, flush):
    """Per-length rows (forward and forward+backward, flushed medians) of BASELINE config 2."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    rows = []
    for T in (1024, 4096, 16384, 32768):
        q, k, v, do = make_inputs(8, 16, T, 64, dtype, dev)
        q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
        nbytes = q.numel() * q.element_size()

        def step():
            q.grad = k.grad = v.grad = None
            linear_attention(q, k, v).backward(do)

        def fwd_only():
            with torch.no_grad():
                return linear_attention(q, k, v)

        f = do_bench(fwd_only, flush)
        s = do_bench(step, flush)
        rows.append({"T": T, "fwd_ms": round(f[0], 5), "fwd_gbps": round(4 * nbytes / f[0] / 1e6, 1),
                     "fwd_frac": round(4 * nbytes / f[0] / 1e6 / HBM_PEAK_GBPS, 4),
                     "fwd_bwd_ms": round(s[0], 5), "fwd_bwd_gbps": round(11 * nbytes / s[0] / 1e6, 1),
                     "fwd_bwd_frac": round(11 * nbytes / s[0] / 1e6 / HBM_PEAK_GBPS, 4)})
        if T <= 4096:
            # Short sequences: six short kernels per step, which a slow host issues more slowly than
            # the GPU runs them.  The same step through autograd recorded into one HIP graph
            # (flash_bla.utils.CapturedStep) is what such a caller would run.
            from flash_bla.utils import CapturedStep
            g = do_bench(CapturedStep(linear_attention, [q, k, v], do).replay, flush)
            rows[-1].update({"fwd_bwd_graph_ms": round(g[0], 5),
                             "fwd_bwd_graph_frac": round(11 * nbytes / g[0] / 1e6 / HBM_PEAK_GBPS, 4)})
        del q, k, v, do
    return rows


def _report(name, nbytes_fwd, nbytes_step, fwd_fn, step_fn, flush, extra=None):
    f = do_bench(fwd_fn, flush)
    s = do_bench(step_fn, flush) if step_fn else None
    row = {"config": name, "fwd_ms": round(f[0], 5), "fwd_gbps": round(nbytes_fwd / f[0] / 1e6, 1),
           "fwd_frac": round(nbytes_fwd / f[0] / 1e6 / HBM_PEAK_GBPS, 4)}
    if s:
        row.update({"fwd_bwd_ms": round(s[0], 5), "fwd_bwd_gbps": round(nbytes_step / s[0] / 1e6, 1),
                    "fwd_bwd_frac": round(nbytes_step / s[0] / 1e6 / HBM_PEAK_GBPS, 4)})
    if extra:
        row.update(extra)
    print(json.dumps(row), file=sys.stderr, flush=True)


def feature_map_config(dev, flush):
    """The blocks' feature map elu(x) + 1 together with linear_attn at the headline shape: applied by
    the kernels as they load q and k (forward; forward + backward with dq, dk from the kernels)
    against the map as launches of its own."""
    from flash_bla.ops.linear_attn.fused import linear_attention

    def leaves(*ts):
        return [t.requires_grad_() for t in ts]

    # the blocks' feature map with the attention (inference forward): applied by the kernels as they
    # load q and k, against one elementwise launch for q and k followed by the operator
    from flash_bla.ops.feature_map import elu_plus_one
    g = torch.Generator(device=dev).manual_seed(3)
    q, k, v = (torch.randn((8, 16, 16384, 64), generator=g, device=dev).half() for _ in range(3))
    nb = q.numel() * 2
    with torch.no_grad():
        t_load = do_bench(lambda: linear_attention(q, k, v, feature_map="elu+1"), flush)
        t_first = do_bench(lambda: linear_attention(*elu_plus_one(q, k), v), flush)
    # training step through the map: dq, dk with respect to the raw tensors from the backward kernels,
    # against the map differentiated by autograd (two more elementwise launches)
    from flash_bla.ops.linear_attn.fused import LinearAttnFunction
    do = torch.randn(q.shape, generator=g, device=dev).half()
    leaves(q, k, v)

    def step_kernels():
        linear_attention(q, k, v, feature_map="elu+1").backward(do)
        q.grad = k.grad = v.grad = None

    def step_autograd():
        LinearAttnFunction.apply(*elu_plus_one(q, k), v, 1.0 / q.shape[2], 1e-6).backward(do)
        q.grad = k.grad = v.grad = None

    t_step = do_bench(step_kernels, flush)
    t_step_auto = do_bench(step_autograd, flush)
    print(json.dumps({"config": "elu+1 feature map + linear_attn B8-H16-T16384-D64 fp16",
                      "fwd_mapped_on_load_ms": round(t_load[0], 5),
                      "fwd_mapped_on_load_gbps": round(4 * nb / t_load[0] / 1e6, 1),
                      "fwd_mapped_on_load_frac": round(4 * nb / t_load[0] / 1e6 / HBM_PEAK_GBPS, 4),
                      "fwd_mapped_first_ms": round(t_first[0], 5),
                      "fwd_bwd_gradients_from_kernels_ms": round(t_step[0], 5),
                      "fwd_bwd_map_by_autograd_ms": round(t_step_auto[0], 5)}), file=sys.stderr, flush=True)
    del q, k, v, do


def _fwd_and_step(op, args, do_):
    """(forward under no_grad, forward + backward with the gradients reset) of one operator call."""
    def step():
        for t in args:
            t.grad = None
        op(*args).backward(do_)

    def fwd():
        with torch.no_grad():
            return op(*args)
    return fwd, step


def other_configs(dev, flush):
    """Flushed-median timings of the remaining BASELINE configs and operator families."""
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    from flash_bla.ops.simple_la.fused import simple_la

    def leaves(*ts):
        return [t.requires_grad_() for t in ts]

    # config 1 shape on the GPU (the CPU-runnable reference case): fp32, tiny
    q, k, v, do = make_inputs(2, 4, 1024, 64, torch.float32, dev)
    leaves(q, k, v)
    nb = q.numel() * 4

    run = _fwd_and_step

    f, s = run(linear_attention, (q, k, v), do)
    _report("C1 linear_attn B2-H4-T1024-D64 fp32", 4 * nb, 11 * nb, f, s, flush)
    f, s = run(simple_la, (q, k, v), do)
    _report("C1 simple_la B2-H4-T1024-D64 fp32", 4 * nb, 11 * nb, f, s, flush)

    # simple_la / decoupled at the headline shape, and bf16 linear_attn
    for dtype, tag in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
        q, k, v, do = make_inputs(8, 16, 16384, 64, dtype, dev)
        leaves(q, k, v)
        nb = q.numel() * 2
        if dtype == torch.bfloat16:
            f, s = run(linear_attention, (q, k, v), do)
            _report(f"linear_attn B8-H16-T16384-D64 {tag}", 4 * nb, 11 * nb, f, s, flush)
        else:
            f, s = run(simple_la, (q, k, v), do)
            _report(f"simple_la B8-H16-T16384-D64 {tag}", 4 * nb, 11 * nb, f, s, flush)
    feature_map_config(dev, flush)
    caller_configs(dev, flush)
    varlen_config(dev, flush)


def caller_configs(dev, flush):
    """The decoupled operator at the shape of benchmark_decoupled_la.py and the head dims of the layer callers."""
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    run = _fwd_and_step

    def leaves(*ts):
        return [t.requires_grad_() for t in ts]

    q, k, v, do = make_inputs(2, 16, 16384, 64, torch.bfloat16, dev)
    qr, kr, _, _ = make_inputs(2, 16, 16384, 64, torch.bfloat16, dev, seed=7)
    leaves(q, k, qr, kr, v)
    nb = q.numel() * 2
    f, s = run(decoupled_la, (q, k, qr, kr, v), do)
    _report("decoupled_la B2-H16-T16384-D64 bf16 (benchmark_decoupled_la.py shape)", 6 * nb, 16 * nb, f, s, flush)
    del q, k, v, do, qr, kr

    # head dims of the layer callers: MLLA / RALA blocks (decoupled, D=32: mlla.py:88, rala.py:74),
    # PolaFormer (DK = 2d, DV = d/2: polaformer.py:75-90)
    def feats(B, H, T, D, seed):
        g = torch.Generator(device=dev).manual_seed(seed)
        return (F.elu(torch.randn((B, H, T, D), generator=g, device=dev)) + 1).half().requires_grad_()

    for name, B, H, T, DK, DV, dec in (("decoupled_la B64-H2-T3136-D32 fp16 (MLLA stage 1)", 64, 2, 3136, 32, 32, True),
                                       ("decoupled_la B8-H16-T4096-D32 fp16", 8, 16, 4096, 32, 32, True),
                                       ("linear_attn B8-H16-T4096-D32 fp16", 8, 16, 4096, 32, 32, False),
                                       ("linear_attn B8-H16-T4096-DK128-DV32 fp16 (PolaFormer)", 8, 16, 4096, 128, 32, False)):
        q, k = feats(B, H, T, DK, 1), feats(B, H, T, DK, 2)
        v = torch.randn(B, H, T, DV, device=dev).half().requires_grad_()
        do = torch.randn(B, H, T, DV, device=dev).half()
        nqk, nv = q.numel() * 2, v.numel() * 2
        if dec:
            qr, kr = feats(B, H, T, DK, 3), feats(B, H, T, DK, 4)
            f, s = run(decoupled_la, (q, k, qr, kr, v), do)
            _report(name, 4 * nqk + 2 * nv, 11 * nqk + 5 * nv, f, s, flush)
        else:
            f, s = run(linear_attention, (q, k, v), do)
            _report(name, 2 * nqk + 2 * nv, 6 * nqk + 5 * nv, f, s, flush)


def varlen_config(dev, flush):
    """BASELINE config 3: packed variable-length, 64 sequences U[256, 2048], H=16, bf16."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    g = torch.Generator().manual_seed(42)
    lengths = torch.randint(256, 2049, (64,), generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.int32), torch.cumsum(lengths, 0).to(torch.int32)]).to(dev)
    total, max_len = int(lengths.sum()), int(lengths.max())
    for D in (64, 128):
        gg = torch.Generator(device=dev).manual_seed(42)
        q = (F.elu(torch.randn(total, 16, D, generator=gg, device=dev)) + 1).bfloat16().requires_grad_()
        k = (F.elu(torch.randn(total, 16, D, generator=gg, device=dev)) + 1).bfloat16().requires_grad_()
        v = torch.randn(total, 16, D, generator=gg, device=dev).bfloat16().requires_grad_()
        do = torch.randn(total, 16, D, generator=gg, device=dev).bfloat16()
        nb = q.numel() * 2

        def step():
            q.grad = k.grad = v.grad = None
            varlen_linear_attention(q, k, v, cu, max_len).backward(do)

        def fwd():
            with torch.no_grad():
                return varlen_linear_attention(q, k, v, cu, max_len)
        _report(f"C3 varlen 64 seqs U[256,2048] H16 D{D} bf16", 4 * nb, 11 * nb, fwd, step, flush,
                {"total_tokens": total, "max_seqlen": max_len})


def layer_config(dev, flush):
    """BASELINE config 4: the LinFusion attention block, forward only, fp16, random-init weights:
    B2 with (L4096, C640, 10 heads x 64) and (L1024, C1280, 20 heads x 64).  Reports the whole
    layer with the HIP operator ('triton' mode name kept from the reference), the whole layer
    with the torch formula, and the operator alone."""
    from flash_bla.layers.linfusion import GeneralizedLinearAttention
    from flash_bla.ops.linear_attn.fused import linear_attention
    for L, C, heads in ((4096, 640, 10), (1024, 1280, 20)):
        torch.manual_seed(42)
        layer = GeneralizedLinearAttention(query_dim=C, heads=heads, dim_head=64).to(dev).half().eval()
        x = torch.randn(2, L, C, generator=torch.Generator().manual_seed(42)).half().to(dev)
        q = (F.elu(torch.randn(2, heads, L, 64, device=dev)) + 1).half()
        k = (F.elu(torch.randn(2, heads, L, 64, device=dev)) + 1).half()
        v = torch.randn(2, heads, L, 64, device=dev).half()
        with torch.no_grad():
            t_fast = do_bench(lambda: layer(x, mode="triton"), flush)
            t_torch = do_bench(lambda: layer(x, mode="torch"), flush)
            t_op = do_bench(lambda: linear_attention(q, k, v, eps=1e-4), flush)
            from flash_bla.utils import CapturedForward
            graphed = CapturedForward(layer, x, mode="triton")
            t_graph = do_bench(lambda: graphed(x), flush)
            graph_equal = bool(torch.equal(graphed(x), layer(x, mode="triton")))
            err = (layer(x, mode="triton").float() - layer(x, mode="torch").float()).abs().max().item()
            ref = layer(x, mode="torch").float().abs().max().item()
        nb = 4 * q.numel() * 2
        print(json.dumps({"config": f"C4 LinFusion layer fwd B2-L{L}-C{C}-{heads}x64 fp16",
                          "layer_ms": round(t_fast[0], 5), "layer_hip_graph_ms": round(t_graph[0], 5),
                          "hip_graph_equals_eager": graph_equal,
                          "layer_torch_mode_ms": round(t_torch[0], 5),
                          "op_ms": round(t_op[0], 5), "op_gbps": round(nb / t_op[0] / 1e6, 1),
                          "modes_max_abs_diff_over_max": round(err / ref, 6)}), file=sys.stderr, flush=True)


def reference_tables(dev, flush, md_path=None):
    """The tables of the reference's three benchmark scripts, columns named as there:
    benchmarks/ops/benchmark_linear_attn.py (providers torch_la / flash_bla / torch_sdpa, `_fwd` and
    `_bwd` = forward + backward, T in {1024, 4096, 16384, 32768}; the script runs B2-H16-D64 bf16,
    the README quotes B8 fp16: both), benchmark_decoupled_la.py:11-62 (B2-H16-D64 bf16) and
    benchmark_varlen_linear_attn.py:20-86 (8 equal sequences, H16-D64 bf16, the padded dense
    operator against the packed one, forward and forward + backward).  Flushed medians in ms;
    gradients are reset before every backward (the scripts let them accumulate in the leaves,
    which times one more elementwise pass per tensor)."""
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.linear_attn.naive import naive_decoupled_la, naive_linear_attn
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    rows = []

    def emit(row):
        rows.append(row)
        print(json.dumps(row), file=sys.stderr, flush=True)

    def time_providers(row, providers, leaves, do):
        def bwd_of(fn):
            def step():
                for t in leaves:
                    t.grad = None
                fn().backward(do)
            return step
        for name, fn in providers:
            with torch.no_grad():
                row[name + "_fwd"] = round(do_bench(fn, flush)[0], 4)
            row[name + "_bwd"] = round(do_bench(bwd_of(fn), flush)[0], 4)

    lengths = (1024, 4096, 16384, 32768)
    for B, dtype, tag in ((2, torch.bfloat16, "bf16"), (8, torch.float16, "fp16")):
        for T in lengths:
            q, k, v, do = make_inputs(B, 16, T, 64, dtype, dev)
            leaves = [t.requires_grad_() for t in (q, k, v)]
            row = {"table": f"linear_attn B{B}-H16-D64 {tag}", "T": T}
            time_providers(row, (("torch_la", lambda: naive_linear_attn(q, k, v)),
                                 ("flash_bla", lambda: linear_attention(q, k, v)),
                                 ("torch_sdpa", lambda: F.scaled_dot_product_attention(q, k, v))), leaves, do)
            emit(row)
            del q, k, v, do, leaves
    for T in lengths:
        q, k, v, do = make_inputs(2, 16, T, 64, torch.bfloat16, dev)
        qr, kr, _, _ = make_inputs(2, 16, T, 64, torch.bfloat16, dev, seed=7)
        leaves = [t.requires_grad_() for t in (q, k, qr, kr, v)]
        row = {"table": "decoupled_la B2-H16-D64 bf16", "T": T}
        time_providers(row, (("torch_la", lambda: naive_decoupled_la(q, k, qr, kr, v)),
                             ("flash_bla", lambda: decoupled_la(q, k, qr, kr, v)),
                             ("torch_sdpa", lambda: F.scaled_dot_product_attention(q, k, v))), leaves, do)
        emit(row)
        del q, k, v, do, qr, kr, leaves
    for max_len in (256, 1024, 4096):
        cu = (torch.arange(9, dtype=torch.int32) * max_len).to(dev)
        qd, kd, vd, dod = make_inputs(8, 16, max_len, 64, torch.bfloat16, dev)
        qp, kp, vp, dop = (t.transpose(1, 2).reshape(8 * max_len, 16, 64).contiguous() for t in (qd, kd, vd, dod))
        dense, packed = [t.requires_grad_() for t in (qd, kd, vd)], [t.requires_grad_() for t in (qp, kp, vp)]

        def fwdbwd(fn, leaves, do):
            def step():
                for t in leaves:
                    t.grad = None
                fn().backward(do)
            return step
        pad = lambda: linear_attention(qd, kd, vd)  # noqa: E731
        var = lambda: varlen_linear_attention(qp, kp, vp, cu, max_len)  # noqa: E731
        row = {"table": "varlen-equal-B8-H16-D64 bf16", "max_seqlen": max_len}
        with torch.no_grad():
            row["flash_padded_fwd"] = round(do_bench(pad, flush)[0], 4)
            row["varlen_fwd"] = round(do_bench(var, flush)[0], 4)
        row["flash_padded_fwdbwd"] = round(do_bench(fwdbwd(pad, dense, dod), flush)[0], 4)
        row["varlen_fwdbwd"] = round(do_bench(fwdbwd(var, packed, dop), flush)[0], 4)
        emit(row)
    if md_path:
        with open(md_path, "w") as f:
            f.write("Flushed medians in ms (`_bwd` columns = forward + backward, as in the reference's scripts).\n")
            table = None
            for row in rows:
                cols = [c for c in row if c != "table"]
                if row["table"] != table:
                    table = row["table"]
                    f.write(f"\n**{table}**\n\n| " + " | ".join(cols) + " |\n|" + "---|" * len(cols) + "\n")
                f.write("| " + " | ".join(str(row[c]) for c in cols) + " |\n")


def piecewise_config(dev, flush):
    """BASELINE config 5: PISA forward, B1-H24-T16384-D128 bf16, 64-token blocks, density 0.25."""
    from flash_bla.ops.piecewise_attn.kernel import (chunk_reduce_fp32, piecewise_sparse_attention,
                                                     select_blocks)
    g = torch.Generator(device=dev).manual_seed(42)
    shape = (1, 24, 16384, 128)
    q = torch.randn(shape, generator=g, device=dev).bfloat16()
    k = torch.randn(shape, generator=g, device=dev).bfloat16()
    v = torch.randn(shape, generator=g, device=dev).bfloat16()
    nb = q.numel() * 2
    scale = 128 ** -0.5
    qc, kc, vc, h, _ = chunk_reduce_fp32(q, k, v, 64)
    indices = select_blocks(qc, kc, scale, 0.25)
    flops_exact = 4.0 * 24 * 16384 * (indices.shape[-1] * 64) * 128
    t_all = do_bench(lambda: piecewise_sparse_attention(q, k, v, density=0.25), flush)
    t_red = do_bench(lambda: chunk_reduce_fp32(q, k, v, 64), flush)
    t_att = do_bench(lambda: piecewise_sparse_attention(q, k, v, indices=indices), flush)
    print(json.dumps({
        "config": "C5 piecewise fwd B1-H24-T16384-D128 bf16 block64 density0.25",
        "total_ms": round(t_all[0], 4), "chunk_reduce_ms": round(t_red[0], 4),
        "chunk_reduce_gbps": round(3 * nb / t_red[0] / 1e6, 1),
        "chunk_reduce_plus_attention_ms": round(t_att[0], 4),
        "exact_branch_tflops": round(flops_exact / ((t_att[0] - t_red[0]) * 1e-3) / 1e12, 1),
        "min_traffic_gbps": round(4 * nb / t_all[0] / 1e6, 1)}), file=sys.stderr, flush=True)


if __name__ == "__main__":
    main()
