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
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_FP32_PEAK_TFLOPS = 157.3  # dense bf16 / fp16 matrix peak

# Untimed work before the warm-up steps.  The GPU reaches its steady clocks after 0.15-0.2 s of continuous work: a
# timed region of 20 steps reads 0.522 ms per step after 0.1 s of work and 0.503 ms after 0.2 s or more, the value every
# later region of the same process reads.
CLOCK_RAMP_S = 0.25

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
                    help="the reference's benchmark tables (torch formula, this library, SDPA; `tables` of the "
                         "JSON line) are on by default; this adds the linear_attn table at the README's B8 fp16")
    ap.add_argument("--no-tables", action="store_true", help="skip the reference's benchmark tables")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the other BASELINE configs (the `configs` list of the JSON line)")
    ap.add_argument("--only", choices=["c3", "c5", "fm", "callers", "f32", "tables"], default=None,
                    help="profiling aid: time just BASELINE config 3 (packed variable-length, D=64 and "
                         "D=128), config 5 (piecewise attention), the feature map together with the "
                         "attention (fm), the decoupled operator, the layer callers' head dims and PolaFormer's "
                         "pairings (callers), fp32 inputs (f32), table on stderr, no headline line; tables: the "
                         "reference's benchmark tables as one JSON object")
    ap.add_argument("--configs", action="store_true",
                    help="add the other operator families (simple_la, bf16, the feature map, the layer callers' "
                         "head dims) to the `configs` list")
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
        elif args.only == "tables":
            print(json.dumps(reference_tables(dev, flush, args.tables_md, readme_table=args.tables)), flush=True)
        elif args.only == "fm":
            feature_map_config(dev, flush)
        elif args.only == "callers":
            caller_configs(dev, flush, head_dims=True)
        elif args.only == "f32":
            fp32_config(dev, flush)
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

    def clock_ramp():
        """The GPU reaches its steady clocks only after tens of milliseconds of work, and leaves them
        again while the host computes (the parity check below): untimed steps bring it there."""
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < CLOCK_RAMP_S:
            for _ in range(20):
                step()
            torch.cuda.synchronize()

    clock_ramp()
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
    clock_ramp()  # the GPU idled during the host-side parity check
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
    del q, k, v, do, o
    if not args.no_sweep:
        line["sweep"] = sweep(dtype, dev, flush)
    if not args.no_configs:
        # every other BASELINE config under the same clock: ms, algorithmic bytes (or FLOPs) per
        # second, fraction of the 8 TB/s (2.5 PFLOP/s) peak, parity of one head against the oracle
        rows = config1_on_gpu(dev, flush) + varlen_config(dev, flush) + layer_config(dev, flush)
        rows.append(piecewise_config(dev, flush))
        rows += caller_configs(dev, flush)
        if args.configs:
            rows += other_configs(dev, flush)
        line["configs"] = rows
    if not args.no_tables:
        line["tables"] = reference_tables(dev, flush, args.tables_md, readme_table=args.tables)
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


def _report(name, nbytes_fwd, nbytes_step, fwd_fn, step_fn, flush, extra=None, fp32_flops=None):
    """fp32_flops = (forward, forward + backward) FLOP: adds the fraction of the fp32 matrix peak."""
    f = do_bench(fwd_fn, flush)
    s = do_bench(step_fn, flush) if step_fn else None
    row = {"config": name, "fwd_ms": round(f[0], 5), "fwd_gbps": round(nbytes_fwd / f[0] / 1e6, 1),
           "fwd_frac": round(nbytes_fwd / f[0] / 1e6 / HBM_PEAK_GBPS, 4)}
    if s:
        row.update({"fwd_bwd_ms": round(s[0], 5), "fwd_bwd_gbps": round(nbytes_step / s[0] / 1e6, 1),
                    "fwd_bwd_frac": round(nbytes_step / s[0] / 1e6 / HBM_PEAK_GBPS, 4)})
    if fp32_flops:
        for key, flop, t in (("fwd", fp32_flops[0], f), ("fwd_bwd", fp32_flops[1], s)):
            if t:
                row[key + "_tflops"] = round(flop / (t[0] * 1e-3) / 1e12, 1)
                row[key + "_frac_of_fp32_mfma_peak"] = round(flop / (t[0] * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4)
    if extra:
        row.update(extra)
    print(json.dumps(row), file=sys.stderr, flush=True)
    return row


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
    row = {"config": "elu+1 feature map + linear_attn B8-H16-T16384-D64 fp16",
           "fwd_mapped_on_load_ms": round(t_load[0], 5),
           "fwd_mapped_on_load_gbps": round(4 * nb / t_load[0] / 1e6, 1),
           "fwd_mapped_on_load_frac": round(4 * nb / t_load[0] / 1e6 / HBM_PEAK_GBPS, 4),
           "fwd_mapped_first_ms": round(t_first[0], 5),
           "fwd_bwd_gradients_from_kernels_ms": round(t_step[0], 5),
           "fwd_bwd_map_by_autograd_ms": round(t_step_auto[0], 5)}
    print(json.dumps(row), file=sys.stderr, flush=True)
    del q, k, v, do
    return row


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


def _one_head_parity(tensors, refs, dtype):
    """{name: plain max-rel error} of GPU results against float64 oracle arrays, plus `ok` (both the
    plain and the rounding-removed gate of tests/helpers.py)."""
    from helpers import parity_errors
    out, ok = {}, True
    for name, (x, ref, floor) in zip(refs, tensors):
        plain, excess, good = parity_errors(x, ref, dtype, floor)
        out[name] = float(f"{plain:.2e}")
        out[name + "_excess"] = float(f"{excess:.2e}")
        ok = ok and good
    out["ok"] = ok
    return out


def config1_on_gpu(dev, flush):
    """BASELINE config 1 (the reference's CPU-runnable case: B2-H4-T1024-D64 fp32, simple_la and
    linear_attn) through the HIP path, every head against the float64 oracle."""
    from helpers import np64
    from oracle import closed_form as cf
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.simple_la.fused import simple_la
    q, k, v, do = make_inputs(2, 4, 1024, 64, torch.float32, dev)
    for t in (q, k, v):
        t.requires_grad_()
    nb = q.numel() * 4
    rows = []
    for name, op, scale, norm in (("linear_attn", linear_attention, 1.0 / 1024, True),
                                  ("simple_la", simple_la, 64 ** -0.5, False)):
        f, s = _fwd_and_step(op, (q, k, v), do)
        # (timing first: the GPU idles, and leaves its steady clocks, while the host evaluates the oracle)
        rows.append(_report(f"C1 {name} B2-H4-T1024-D64 fp32", 4 * nb, 11 * nb, f, s, flush))
        s()
        ref = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), scale, normalize=norm)
        rows[-1]["parity"] = _one_head_parity(
            [(f(), ref["o"], None), (q.grad, ref["dq"], ref.get("dq_mag")), (k.grad, ref["dk"], ref.get("dk_mag")),
             (v.grad, ref["dv"], None)], ("o", "dq", "dk", "dv"), torch.float32)
    return rows


def other_configs(dev, flush):
    """Flushed-median timings of the remaining operator families at the headline shape."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.simple_la.fused import simple_la
    run = _fwd_and_step
    rows = []
    # simple_la at the headline shape, and bf16 linear_attn
    for dtype, tag in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
        q, k, v, do = make_inputs(8, 16, 16384, 64, dtype, dev)
        for t in (q, k, v):
            t.requires_grad_()
        nb = q.numel() * 2
        if dtype == torch.bfloat16:
            f, s = run(linear_attention, (q, k, v), do)
            rows.append(_report(f"linear_attn B8-H16-T16384-D64 {tag}", 4 * nb, 11 * nb, f, s, flush))
        else:
            f, s = run(simple_la, (q, k, v), do)
            rows.append(_report(f"simple_la B8-H16-T16384-D64 {tag}", 4 * nb, 11 * nb, f, s, flush))
    rows.append(feature_map_config(dev, flush))
    rows += caller_configs(dev, flush, head_dims=True)
    rows += fp32_config(dev, flush)
    return rows


def caller_configs(dev, flush, head_dims=False):
    """The decoupled operator at the shape of benchmark_decoupled_la.py (one head against the float64
    oracle), and with `head_dims` the head dims of the layer callers."""
    from helpers import np64
    from oracle import closed_form as cf
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    run = _fwd_and_step
    rows = []

    def leaves(*ts):
        return [t.requires_grad_() for t in ts]

    T = 16384
    q, k, v, do = make_inputs(2, 16, T, 64, torch.bfloat16, dev)
    qr, kr, _, _ = make_inputs(2, 16, T, 64, torch.bfloat16, dev, seed=7)
    args = leaves(q, k, qr, kr, v)
    nb = q.numel() * 2
    f, s = run(decoupled_la, args, do)
    rows.append(_report("decoupled_la B2-H16-T16384-D64 bf16 (benchmark_decoupled_la.py shape)", 6 * nb, 16 * nb,
                        f, s, flush))
    s()
    sl = (slice(1, 2), slice(5, 6))
    ref = cf.dense_backward(np64(q[sl]), np64(k[sl]), np64(v[sl]), np64(do[sl]), 1.0 / T,
                            q_rope=np64(qr[sl]), k_rope=np64(kr[sl]))
    names = ("o", "dq", "dk", "dq_rope", "dk_rope", "dv")
    got = (f(), q.grad, k.grad, qr.grad, kr.grad, v.grad)
    rows[-1]["parity"] = _one_head_parity([(g[sl], ref[n], None) for g, n in zip(got, names)], names, torch.bfloat16)
    del q, k, v, do, qr, kr, args, got
    if not head_dims:
        return rows

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
            rows.append(_report(name, 4 * nqk + 2 * nv, 11 * nqk + 5 * nv, f, s, flush))
        else:
            f, s = run(linear_attention, (q, k, v), do)
            rows.append(_report(name, 2 * nqk + 2 * nv, 6 * nqk + 5 * nv, f, s, flush))
    rows.append(polaformer_config(dev, flush))
    return rows


def fp32_config(dev, flush):
    """fp32 inputs (the precision the reference's tests use, tests/ops/test_varlen_linear_attn.py:15-18) at
    B8-H16-T4096: heads of 64 and of 128 on the fp32 matrix instructions."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    rows = []
    for D in (64, 128):
        q, k, v, do = make_inputs(8, 16, 4096, D, torch.float32, dev)
        for t in (q, k, v):
            t.requires_grad_()
        nb = q.numel() * 4
        f, s = _fwd_and_step(linear_attention, (q, k, v), do)
        # the fp32 matrix instructions (157.3 TFLOP/s) bound these shapes next to HBM: forward 4 DK DV
        # FLOP per (token, head), backward about 10 more
        flop = q.numel() * D
        rows.append(_report(f"linear_attn B8-H16-T4096-D{D} fp32", 4 * nb, 11 * nb, f, s, flush,
                            fp32_flops=(4 * flop, 14 * flop)))
        del q, k, v, do
    return rows


def polaformer_config(dev, flush):
    """PolaFormer's attention core (layers/polaformer.py:89-90) at B8-H16-T4096, head dim 64 (DK = 128, two value
    halves of 32): the two operator calls that share k against the one-state-pass operator.  Bytes: the tensors
    the shared-state form has to move (forward q1, q2, k, v, o1, o2; backward q1, q2, k, v, dO, dq1, dq2, dk, dv)."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.linear_attn.paired import paired_linear_attention
    B, H, T, DK, DV = 8, 16, 4096, 128, 64
    g = torch.Generator(device=dev).manual_seed(5)
    feat = lambda: (F.elu(torch.randn(B, H, T, DK, generator=g, device=dev)) + 1).half().requires_grad_()  # noqa: E731
    q1, q2, k = feat(), feat(), feat()
    v = torch.randn(B, H, T, DV, generator=g, device=dev).half().requires_grad_()
    do1, do2 = (torch.randn(B, H, T, DV // 2, generator=g, device=dev).half() for _ in range(2))
    leaves = (q1, q2, k, v)

    def two_calls():
        v1, v2 = (t.contiguous() for t in v.chunk(2, dim=-1))
        return linear_attention(q1, k, v1), linear_attention(q2, k, v2)

    def shared():
        return paired_linear_attention(q1, q2, k, v)

    def step_of(fn):
        def step():
            for t in leaves:
                t.grad = None
            torch.autograd.backward(fn(), [do1, do2])
        return step
    nqk, nv = q1.numel() * 2, v.numel() * 2
    fwd_bytes, step_bytes = 3 * nqk + 2 * nv, 3 * nqk + 2 * nv + 4 * nqk + 3 * nv
    with torch.no_grad():
        f2, f1 = do_bench(two_calls, flush)[0], do_bench(shared, flush)[0]
        a, b = two_calls(), shared()
        same = max((x.float() - y.float()).abs().max().item() / y.float().abs().max().item() for x, y in zip(a, b))
    s2, s1 = do_bench(step_of(two_calls), flush)[0], do_bench(step_of(shared), flush)[0]
    row = {"config": "PolaFormer pairings B8-H16-T4096 DK128 DV2x32 fp16",
           "two_calls_fwd_ms": round(f2, 5), "two_calls_fwd_bwd_ms": round(s2, 5),
           "fwd_ms": round(f1, 5), "fwd_gbps": round(fwd_bytes / f1 / 1e6, 1),
           "fwd_frac": round(fwd_bytes / f1 / 1e6 / HBM_PEAK_GBPS, 4),
           "fwd_bwd_ms": round(s1, 5), "fwd_bwd_gbps": round(step_bytes / s1 / 1e6, 1),
           "fwd_bwd_frac": round(step_bytes / s1 / 1e6 / HBM_PEAK_GBPS, 4),
           "parity": {"shared_vs_two_calls_max_abs_over_max": float(f"{same:.2e}"), "ok": same <= 2e-3}}
    print(json.dumps(row), file=sys.stderr, flush=True)
    return row


def varlen_config(dev, flush):
    """BASELINE config 3: packed variable-length, 64 sequences U[256, 2048], H=16, bf16; sequence 17,
    heads 0-1 against the float64 oracle."""
    from helpers import np64
    from oracle import closed_form as cf
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    g = torch.Generator().manual_seed(42)
    lengths = torch.randint(256, 2049, (64,), generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.int32), torch.cumsum(lengths, 0).to(torch.int32)]).to(dev)
    total, max_len = int(lengths.sum()), int(lengths.max())
    bounds = cu.tolist()
    rows = []
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
        rows.append(_report(f"C3 varlen 64 seqs U[256,2048] H16 D{D} bf16", 4 * nb, 11 * nb, fwd, step, flush,
                            {"total_tokens": total, "max_seqlen": max_len}))
        step()
        b, e = bounds[17], bounds[18]
        head = lambda t: t[b:e, :2].transpose(0, 1)  # noqa: E731
        ref = cf.dense_backward(*(np64(head(t)) for t in (q, k, v, do)), 1.0 / (e - b))
        rows[-1]["parity"] = _one_head_parity(
            [(head(fwd()), ref["o"], None), (head(q.grad), ref["dq"], ref["dq_mag"]),
             (head(k.grad), ref["dk"], ref["dk_mag"]), (head(v.grad), ref["dv"], None)],
            ("o", "dq", "dk", "dv"), torch.bfloat16)
        del q, k, v, do
    return rows


def layer_config(dev, flush):
    """BASELINE config 4: the LinFusion attention block, forward only, fp16, random-init weights:
    B2 with (L4096, C640, 10 heads x 64) and (L1024, C1280, 20 heads x 64).  Reports the whole
    layer with the HIP operator ('triton' mode name kept from the reference), the whole layer
    with the torch formula, and the operator alone."""
    from flash_bla.layers.linfusion import GeneralizedLinearAttention
    from flash_bla.ops.linear_attn.fused import linear_attention
    rows = []
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
        rows.append({"config": f"C4 LinFusion layer fwd B2-L{L}-C{C}-{heads}x64 fp16",
                     "layer_ms": round(t_fast[0], 5), "layer_hip_graph_ms": round(t_graph[0], 5),
                     "hip_graph_equals_eager": graph_equal,
                     "layer_torch_mode_ms": round(t_torch[0], 5),
                     "op_ms": round(t_op[0], 5), "op_alg_bytes": nb, "op_gbps": round(nb / t_op[0] / 1e6, 1),
                     "op_frac": round(nb / t_op[0] / 1e6 / HBM_PEAK_GBPS, 4),
                     "parity": {"layer_vs_torch_mode_max_abs_over_max": round(err / ref, 6),
                                "ok": err / ref <= 2e-3}})
        print(json.dumps(rows[-1]), file=sys.stderr, flush=True)
    return rows


PROVIDERS6 = ["torch_la_fwd", "flash_bla_fwd", "torch_sdpa_fwd", "torch_la_bwd", "flash_bla_bwd", "torch_sdpa_bwd"]
# x axis, columns and plot names of the reference's three benchmark scripts
TABLE_SPECS = {
    "linear_attn": {"script": "benchmarks/ops/benchmark_linear_attn.py:11-29", "plot_name": "B2-H16-D64",
                    "dtype": "bf16", "x_name": "T", "x_vals": [1024, 4096, 16384, 32768], "line_vals": PROVIDERS6},
    "decoupled_la": {"script": "benchmarks/ops/benchmark_decoupled_la.py:11-29", "plot_name": "B2-H16-D64",
                     "dtype": "bf16", "x_name": "T", "x_vals": [1024, 4096, 16384, 32768], "line_vals": PROVIDERS6},
    "varlen_linear_attn": {"script": "benchmarks/ops/benchmark_varlen_linear_attn.py:18-44",
                           "plot_name": "varlen-equal-B8-H16-D64", "dtype": "bf16", "x_name": "max_seqlen",
                           "x_vals": [256, 1024, 4096],
                           "line_vals": ["flash_padded_fwd", "varlen_fwd", "flash_padded_fwdbwd", "varlen_fwdbwd"]},
}


def reference_tables(dev, flush, md_path=None, x_vals=None, readme_table=False):
    """The tables of the reference's three benchmark scripts, x axis and columns named as there:
    benchmarks/ops/benchmark_linear_attn.py (providers torch_la / flash_bla / torch_sdpa, `_fwd` and
    `_bwd` = forward + backward, T in {1024, 4096, 16384, 32768}, B2-H16-D64 bf16),
    benchmark_decoupled_la.py:11-62 (same axis and providers) and benchmark_varlen_linear_attn.py:20-86
    (8 equal sequences, H16-D64 bf16, the padded dense operator against the packed one, forward and
    forward + backward).  Flushed medians in ms; gradients are reset before every backward (the
    scripts let them accumulate in the leaves, which times one more elementwise pass per tensor).
    Returns {table: {script, plot_name, dtype, x_name, x_vals, line_vals, rows}} with one row of
    `line_vals` times per x value.  `x_vals` replaces every table's x axis (tests use tiny lengths);
    `readme_table` adds the linear_attn table at the README's B8 fp16."""
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.linear_attn.naive import naive_decoupled_la, naive_linear_attn
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    tables = {}

    def new_table(name, spec_name, **changes):
        spec = dict(TABLE_SPECS[spec_name], **changes)
        if x_vals is not None:
            spec["x_vals"] = list(x_vals)
        tables[name] = dict(spec, rows=[])
        return tables[name]

    def emit(table, name, x, row):
        table["rows"].append([row[c] for c in table["line_vals"]])
        print(json.dumps(dict({"table": name, table["x_name"]: x}, **row)), file=sys.stderr, flush=True)

    def fwd_bwd_of(fn, leaves, do):
        def step():
            for t in leaves:
                t.grad = None
            fn().backward(do)
        return step

    def time_providers(providers, leaves, do):
        row = {}
        for name, fn in providers:
            with torch.no_grad():
                row[name + "_fwd"] = round(do_bench(fn, flush)[0], 4)
            row[name + "_bwd"] = round(do_bench(fwd_bwd_of(fn, leaves, do), flush)[0], 4)
        return row

    variants = [("linear_attn", 2, torch.bfloat16, {})]
    if readme_table:
        variants.append(("linear_attn_readme_B8_fp16", 8, torch.float16, {"plot_name": "B8-H16-D64", "dtype": "fp16"}))
    for name, B, dtype, changes in variants:
        table = new_table(name, "linear_attn", **changes)
        for T in table["x_vals"]:
            q, k, v, do = make_inputs(B, 16, T, 64, dtype, dev)
            leaves = [t.requires_grad_() for t in (q, k, v)]
            emit(table, name, T, time_providers(
                (("torch_la", lambda: naive_linear_attn(q, k, v)),
                 ("flash_bla", lambda: linear_attention(q, k, v)),
                 ("torch_sdpa", lambda: F.scaled_dot_product_attention(q, k, v))), leaves, do))
            del q, k, v, do, leaves
    table = new_table("decoupled_la", "decoupled_la")
    for T in table["x_vals"]:
        q, k, v, do = make_inputs(2, 16, T, 64, torch.bfloat16, dev)
        qr, kr, _, _ = make_inputs(2, 16, T, 64, torch.bfloat16, dev, seed=7)
        leaves = [t.requires_grad_() for t in (q, k, qr, kr, v)]
        emit(table, "decoupled_la", T, time_providers(
            (("torch_la", lambda: naive_decoupled_la(q, k, qr, kr, v)),
             ("flash_bla", lambda: decoupled_la(q, k, qr, kr, v)),
             ("torch_sdpa", lambda: F.scaled_dot_product_attention(q, k, v))), leaves, do))
        del q, k, v, do, qr, kr, leaves
    table = new_table("varlen_linear_attn", "varlen_linear_attn")
    for max_len in table["x_vals"]:
        cu = (torch.arange(9, dtype=torch.int32) * max_len).to(dev)
        qd, kd, vd, dod = make_inputs(8, 16, max_len, 64, torch.bfloat16, dev)
        qp, kp, vp, dop = (t.transpose(1, 2).reshape(8 * max_len, 16, 64).contiguous() for t in (qd, kd, vd, dod))
        dense, packed = [t.requires_grad_() for t in (qd, kd, vd)], [t.requires_grad_() for t in (qp, kp, vp)]
        pad = lambda: linear_attention(qd, kd, vd)  # noqa: E731
        var = lambda: varlen_linear_attention(qp, kp, vp, cu, max_len)  # noqa: E731
        row = {}
        with torch.no_grad():
            row["flash_padded_fwd"] = round(do_bench(pad, flush)[0], 4)
            row["varlen_fwd"] = round(do_bench(var, flush)[0], 4)
        row["flash_padded_fwdbwd"] = round(do_bench(fwd_bwd_of(pad, dense, dod), flush)[0], 4)
        row["varlen_fwdbwd"] = round(do_bench(fwd_bwd_of(var, packed, dop), flush)[0], 4)
        emit(table, "varlen_linear_attn", max_len, row)
    if md_path:
        with open(md_path, "w") as f:
            f.write("Flushed medians in ms (`_bwd` columns = forward + backward, as in the reference's scripts).\n")
            for name, t in tables.items():
                cols = [t["x_name"]] + t["line_vals"]
                f.write(f"\n**{name}** ({t['script']}, plot {t['plot_name']}, {t['dtype']})\n\n| "
                        + " | ".join(cols) + " |\n|" + "---|" * len(cols) + "\n")
                for x, row in zip(t["x_vals"], t["rows"]):
                    f.write("| " + " | ".join(str(c) for c in [x] + row) + " |\n")
    return tables


def piecewise_config(dev, flush):
    """BASELINE config 5: PISA forward, B1-H24-T16384-D128 bf16, 64-token blocks, density 0.25; head 11
    against the dense float64 oracle evaluated with the kernel's own selection."""
    from helpers import np64
    from oracle import piecewise as pw
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
    o = piecewise_sparse_attention(q, k, v, density=0.25, indices=indices)
    hd = 11
    ref = pw.piecewise_forward(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], indices[0, hd].cpu().numpy(), 64)
    par = _one_head_parity([(o[0, hd], ref, None)], ("o",), torch.bfloat16)
    tflops = flops_exact / ((t_att[0] - t_red[0]) * 1e-3) / 1e12
    row = {"config": "C5 piecewise fwd B1-H24-T16384-D128 bf16 block64 density0.25",
           "total_ms": round(t_all[0], 4), "chunk_reduce_ms": round(t_red[0], 4),
           "chunk_reduce_gbps": round(3 * nb / t_red[0] / 1e6, 1),
           "chunk_reduce_plus_attention_ms": round(t_att[0], 4),
           "exact_branch_flops": flops_exact, "exact_branch_tflops": round(tflops, 1),
           "exact_branch_frac_of_mfma_peak": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
           "min_traffic_bytes": 4 * nb, "min_traffic_gbps": round(4 * nb / t_all[0] / 1e6, 1),
           "parity": par}
    print(json.dumps(row), file=sys.stderr, flush=True)
    return row


if __name__ == "__main__":
    main()
