#!/usr/bin/env python3
"""Benchmark of the Fastmax hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

One step = one forward + one backward of causal order-2 Fastmax on one batch of
synthetic input (the configuration the metric is quoted on: B=4, H=8, N=4096, D=Dv=64, bf16,
q, k, v, dO ~ N(0,1), tau = 8*sqrt(D), Taylor coefficients), inputs resident in
HBM, called through the C ABI (libfastmax_hip.so).  Prints ONE JSON line.

Besides the contract fields the line carries
  roofline:     the dominant kernel, measured live with HIP events on the launch
                stream (the same steps run through libfastmax_hip_bench.so, the product's
                sources built with per-kernel event brackets), priced with the ALGORITHMIC
                flop count 2*(D + D^2)*(Dv + 1) per (b, h, token) and unit of
                work (state build, readout, dQ, dK, dV each count one unit);
  cpu_baseline: the oracle's port of the reference's einops algorithm timed on
                this box's host cores on a bounded sample (a few (b, h) slices), and the
                reference's unfactorised closed form (compute_attn) beside it;
  step_ms:      median / p10 / p90 of the step, from HIP events on the launch stream;
  extra:        the other configurations of the path, a few steps each: fp32 on the same
                workload, and the long-context configuration (B=1, H=16, N=65536) in both orders.
Everything runs on one GPU; --gpus N > 1 is refused.  --workload long / --order 1 time the
long-context parity configuration (B=1, H=16, N=65536) for profiling; the metric is the default.
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

PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}      # MI355X dense matrix peaks (published)
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this file
# scaled by a copy of known size (the summaries under profiles/ give the commands); keyed by
# (N, order, dtype, --chunk, kernel).  A constant, not a live measurement: it belongs to the kernels as they
# were when the named summary was made.
TRAFFIC = {
    (4096, 2, "bf16", 0, "dkv"): {"bytes": int((42622.6 * 2 + 32768.1) * 1024), "source": "profiles/c2_bf16_hbm_traffic.md"},
    (4096, 2, "f32", 0, "dk"): {"bytes": int((324657.1 * 2 + 32768.9) * 1024), "source": "profiles/c2_fp32_kernel_trace.md"},
    (65536, 1, "bf16", 0, "dkv"): {"bytes": int((402949.3 * 2 + 393223.9) * 1024), "source": "profiles/long_order1_bf16_hbm_traffic.md"},
    (65536, 2, "bf16", 0, "build"): {"bytes": int((130128.6 * 2 + 544747.5) * 1024), "source": "profiles/long_order2_bf16_hbm_traffic.md"},
    (65536, 2, "bf16", 0, "dkv"): {"bytes": int((609337.0 * 2 + 262146.4) * 1024), "source": "profiles/long_order2_bf16_hbm_traffic.md"},
}

WORKLOAD = dict(name="configs[1]: causal order-2 fwd+bwd", B=4, H=8, N=4096, D=64, p=2, mask=True, scale=1.0)
# not a bench line of its own: the long-context parity configuration, selectable for profiling (--workload long)
LONG_WORKLOAD = dict(name="configs[2]: causal long-context fwd+bwd", B=1, H=16, N=65536, D=64, p=2, mask=True, scale=0.5)

# Units of algorithmic work (each 2*M_p*(Dv+1) flop per (b, h, token)) carried by one launch of
# each kernel; 7 units per forward+backward in both cases (fwd 4, bwd 10 of the 14*M_p*(Dv+1)).
# With moment states: two state walks (forward, backward) of one unit each, the readouts one
# each, and dQ also carries the unit of the prefix rebuild it is spared by reading the forward's.
# Without (a sequence short enough for one segment) each kernel carries its walk as well.
UNITS_STATE = {"build": 1, "fwd": 1, "dq": 2, "dk": 1, "dv": 1, "dkv": 2}
UNITS_DENSE = {"fwd": 2, "dq": 2, "dk": 2, "dv": 1, "dkv": 3}
# 32x32x16 MFMA instructions per 32x32 score tile in the dense loops of each kernel
MFMA_PER_TILE = {"fwd": 8, "dv": 8, "dq": 12, "dk": 12, "dkv": 16}


def alg_flops_unit(bh: int, n: int, d: int, p: int) -> float:
    m = d + (d * d if p == 2 else 0)
    return 2.0 * m * (d + 1) * bh * n


def sclk_under(run, sync, seconds: float = 0.4):
    """Shader clock while `run` is called in a loop for `seconds`: the driver's pp_dpm_sclk file sampled every 10 ms
    from a second thread, median of the samples of the second half (MHz), or None where the file cannot be read."""
    import glob
    import threading
    files = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
    if not files:
        return None
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                with open(files[0]) as fh:
                    for line in fh:
                        if "*" in line:
                            samples.append(float(line.split(":")[1].lower().split("mhz")[0]))
            except (OSError, ValueError, IndexError):
                return
            time.sleep(0.01)

    th = threading.Thread(target=sampler, daemon=True)
    th.start()
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end:
        for _ in range(8):
            run()
        sync()
    stop.set()
    th.join()
    half = sorted(samples[len(samples) // 2:])
    return half[len(half) // 2] if len(half) >= 3 else None


NOMINAL_SCLK_MHZ = 2400.0     # the engine clock the published matrix peaks are quoted at


def cpu_model_name() -> str:
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_closed_form(n: int, d: int, p: int, tokens_per_step: int, heads_total: int, slices: int = 2):
    """The reference's unfactorised form (compute_attn, fastattention_einops.py:337-381: the N x N weights of one
    (b, h) slice at a time) with torch autograd for the gradients, fp32, on the host cores."""
    import torch
    from oracle import fastmax_oracle as O
    gen = torch.Generator().manual_seed(2)
    tau = 8.0 * math.sqrt(d)
    slices = max(1, min(slices, heads_total))
    dt = 0.0
    for _ in range(slices):
        q, k, v, go = (torch.randn(1, n, d, generator=gen) for _ in range(4))
        t0 = time.perf_counter()
        O.closed_form_forward_backward(q, k, v, go, mask=True, tau=tau, p=p, dtype=torch.float32)
        dt += time.perf_counter() - t0
    t_step = dt * heads_total / slices
    return {"value": tokens_per_step / t_step, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"closed form (N x N weights) + autograd, {slices} of {heads_total} (b,h) slices at N={n}, fp32, "
                      f"scaled x{heads_total / slices:g}; {dt:.1f} s measured"}


def cpu_baseline(n: int, d: int, p: int, tokens_per_step: int, heads_total: int, max_n: int, slices: int = 4):
    """Port of the reference's einops factorised path (oracle), fp32, a few (b, h) slices one after another."""
    import torch
    from oracle import fastmax_oracle as O
    threads = torch.get_num_threads()          # follows OMP_NUM_THREADS (the box's CPU share)
    n_run = min(n, max_n)
    gen = torch.Generator().manual_seed(1)
    slices = max(1, min(slices, heads_total))
    tau = 8.0 * math.sqrt(d)
    dt = 0.0
    for _ in range(slices):
        q, k, v, go = (torch.randn(1, 1, n_run, d, generator=gen) for _ in range(4))
        t0 = time.perf_counter()
        o, g = O.factorised_forward(q, k, v, mask=True, tau=tau, p=p)
        dq, dk, dv = O.factorised_backward(q, k, v, o, g, go, mask=True, tau=tau, p=p)
        dt += time.perf_counter() - t0
        del o, g, dq, dk, dv
    # linear-time algorithm: scale the slices to the full sequence and to all heads
    t_step = dt * (n / n_run) * heads_total / slices
    sample = f"{slices} of {heads_total} (b,h) slices, N={n_run}" + \
             ("" if n_run == n else f" (scaled linearly to N={n})") + \
             f", fp32, fwd+bwd, scaled x{heads_total / slices:g}; {dt:.1f} s measured"
    return {"value": tokens_per_step / t_step, "unit": "tokens/s", "cores": threads, "kind": "port", "sample": sample,
            "cpu_model": cpu_model_name()}


def model_step(args, dev):
    """One optimiser step of the model counterparts (the callers of the operator), synthetic data."""
    import torch
    from reproducing_fastmax_results_amd.transformer.model import gpt_for_c5, vit_for_c4
    torch.manual_seed(0)
    if args.model_step == "vit":
        model = vit_for_c4().to(dev)
        x = torch.rand(256, 1, 28, 28, device=dev)
        y = torch.randint(0, 10, (256,), device=dev)
        tokens, dtype, name = 256 * 50, "f32", "ViT 4 layers d_model=128 4 heads of 32, 256 images 28x28 in 4x4 patches + class token"

        def loss_of():
            return torch.nn.functional.cross_entropy(model(x), y)
    else:
        model = gpt_for_c5().to(dev).to(torch.bfloat16)
        x = torch.randint(0, 50257, (16, 1024), device=dev)
        y = torch.randint(0, 50257, (16, 1024), device=dev)
        tokens, dtype, name = 16 * 1024, "bf16", "decoder-only LM 6 layers d_model=512 8 heads of 64, 16 x 1024 tokens, vocabulary 50257"

        def loss_of():
            return torch.nn.functional.cross_entropy(model(x).float().view(-1, 50257), y.view(-1))
    opt = torch.optim.AdamW(model.parameters(), lr=1e-4)

    def step():
        opt.zero_grad(set_to_none=True)
        loss = loss_of()
        loss.backward()
        opt.step()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    return {"metric": f"{args.model_step} training step tokens/s", "value": tokens / dt, "unit": "tokens/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": 1e3 * dt, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
            "config": {"workload": name, "optimizer": "AdamW", "attention": "Fastmax order 2, normalised q and k"},
            "final_loss": float(loss.detach())}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    ap.add_argument("--chunk", type=int, default=0, help="segment length of the causal moment scan (0 = library default)")
    ap.add_argument("--independent-backward", action="store_true",
                    help="backward rebuilds the key-side copies and states instead of taking them from the forward")
    ap.add_argument("--model-step", choices=["vit", "gpt"], default=None,
                    help="instead of the operator benchmark, time one training step (forward, backward, AdamW) of "
                         "the minimal ViT (fp32, 256 images of 28x28) or decoder-only LM (bf16, 16 x 1024 tokens)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the short runs of the other configurations")
    ap.add_argument("--decode-only", action="store_true",
                    help="only the incremental-decoding line (for profiling its kernel)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device copy, the yardstick for the HBM traffic counters")
    ap.add_argument("--workload", choices=["headline", "long"], default="headline",
                    help="headline: the configuration the metric is quoted on (default); long: B=1, H=16, N=65536 "
                         "(inputs scaled by 0.5), for profiling the moment-state kernels")
    ap.add_argument("--order", type=int, choices=[1, 2], default=2, help="order of the polynomial (the metric is order 2)")
    ap.add_argument("--graph", action="store_true", help="time replays of the step captured as one HIP graph")
    ap.add_argument("--cpu-max-n", type=int, default=2048, help="longest slice the CPU baseline materialises")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (every (b,h) slice is independent, so the path "
              "would shard over batch*heads without communication); run with --gpus 1", file=sys.stderr)
        return 2

    import torch
    from reproducing_fastmax_results_amd._capi import get_bench_lib, get_lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    lib = get_lib()
    dev = torch.device("cuda:0")
    if args.model_step:
        print(json.dumps(model_step(args, dev)))
        return 0
    if args.decode_only:
        print(json.dumps(decode_line(lib, dev)))
        return 0
    W = dict(WORKLOAD if args.workload == "headline" else LONG_WORKLOAD, p=args.order)
    out = operator_line(lib, dev, W, args.dtype, args, args.steps, args.warmup, full=True)
    if args.workload == "headline" and args.order == 2 and args.dtype == "bf16" and not args.no_extra:
        # the other configurations of the path, a few steps each (same measurement, shorter)
        extra = {}
        for key, w, dt in (("c2_fp32", dict(WORKLOAD), "f32"),
                           ("c3_order1_bf16", dict(LONG_WORKLOAD, p=1), "bf16"),
                           ("c3_order2_bf16", dict(LONG_WORKLOAD, p=2), "bf16")):
            plain = argparse.Namespace(**dict(vars(args), chunk=0, graph=False, independent_backward=False))
            r = operator_line(lib, dev, w, dt, plain, steps=30, warmup=10, full=False)
            extra[key] = {"workload": r["config"]["workload"], "dtype": dt, "ms_per_step": r["ms_per_step"],
                          "step_ms": r["step_ms"], "tokens_per_s": r["value"], "forward_only_ms": r["forward_only"]["ms"],
                          "roofline": r["roofline"], "hbm_bound_helpers": r["hbm_bound_helpers"]}
        extra["decode_state_order2_bf16"] = decode_line(lib, dev)
        extra["c1_fp32_forward"] = c1_line(lib, dev, not args.no_cpu_baseline)
        # the two model counterparts (the operator's callers): one optimiser step each, a few steps
        ms_args = argparse.Namespace(**dict(vars(args), steps=5, warmup=3))
        extra["model_steps"] = {}
        for name in ("vit", "gpt"):
            ms_args.model_step = name
            r = model_step(ms_args, dev)
            extra["model_steps"][name] = {"ms_per_step": r["ms_per_step"], "tokens_per_s": r["value"], "dtype": r["dtype"],
                                          "workload": r["config"]["workload"]}
            torch.cuda.empty_cache()
        if not args.no_cpu_baseline:
            extra["cpu_baselines_long"] = cpu_long_baselines()
        out["extra"] = extra
    print(json.dumps(out))
    return 0


def c1_line(lib, dev, with_cpu):
    """The small unmasked case (the one the reference can run on a CPU): order-2 forward, unmasked, fp32, B=1, H=2, N=256, D=Dv=32: the GPU call event-timed and the
    oracle's port of the reference's factorised path on the host cores, measured directly."""
    import torch
    from oracle import fastmax_oracle as O
    gen = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 2, 256, 32, generator=gen) for _ in range(3))
    tau = 8.0 * math.sqrt(32)
    qd, kd, vd = (t.view(2, 256, 32).to(dev) for t in (q, k, v))
    kw = dict(mask=False, inv_tau=1.0 / tau, p=2)
    for _ in range(3):
        lib.forward(qd, kd, vd, **kw)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        lib.forward(qd, kd, vd, **kw)
    e1.record()
    e1.synchronize()
    gpu_us = 1e3 * e0.elapsed_time(e1) / 20
    out = {"workload": "configs[0]: order-2 forward, unmasked, fp32, B=1 H=2 N=256 D=Dv=32", "gpu_us_per_call": gpu_us,
           "gpu_tokens_per_s": 256 / (gpu_us * 1e-6),
           "note": "a call of 512 (b,h,token) rows: launch-bound on the GPU (two launches, host side of the Python front included)"}
    if with_cpu:
        O.factorised_forward(q, k, v, mask=False, tau=tau, p=2)
        t0 = time.perf_counter()
        reps = 20
        for _ in range(reps):
            O.factorised_forward(q, k, v, mask=False, tau=tau, p=2)
        dt = (time.perf_counter() - t0) / reps
        out["cpu_baseline"] = {"value": 256 / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"the whole configuration, measured directly, {reps} calls, {1e3 * dt:.2f} ms per call"}
    return out


def cpu_long_baselines():
    """The oracle's port of the reference's factorised path on the long-context shape (B=1, H=16, N=65536, D=64), fp32,
    fwd+bwd, on a bounded sample: one head, a slice of the sequence, scaled linearly in N (the algorithm is linear in
    N) and by the 16 heads.  Order 1 would fit whole (1.07 GB per intermediate and head); order 2 would not (68.7 GB per
    intermediate and head): both are flagged as extrapolated."""
    import torch
    from oracle import fastmax_oracle as O
    tau = 8.0 * math.sqrt(64)
    gen = torch.Generator().manual_seed(2)
    out = {}
    for p, n_run in ((1, 32768), (2, 1024)):
        q, k, v, go = (0.5 * torch.randn(1, 1, n_run, 64, generator=gen) for _ in range(4))
        t0 = time.perf_counter()
        o, g = O.factorised_forward(q, k, v, mask=True, tau=tau, p=p)
        grads = O.factorised_backward(q, k, v, o, g, go, mask=True, tau=tau, p=p)
        dt = time.perf_counter() - t0
        del o, g, grads
        t_step = dt * 16 * (65536 / n_run)
        out[f"order{p}"] = {"value": 65536 / t_step, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                            "extrapolated": n_run != 65536,
                            "sample": f"1 of 16 heads at N={n_run}" + ("" if n_run == 65536 else " (scaled linearly to N=65536)") +
                                      f", scaled x16, fp32, fwd+bwd; {dt:.1f} s measured"}
    return out


def decode_line(lib, dev, bh=16, d=64, prompt=4096, steps=200):
    """Incremental decoding on the persistent moment state (the long shape's heads, order 2): a prompt is absorbed,
    then one token per call; a step reads and writes the state once, so it is priced against HBM."""
    import torch
    gen = torch.Generator().manual_seed(5)
    q, k, v = ((torch.randn(bh, prompt + steps, d, generator=gen)).to(torch.bfloat16).to(dev) for _ in range(3))
    kw = dict(inv_tau=1.0 / (8.0 * math.sqrt(d)), p=2)
    state = lib.decode_state(k, **kw)
    # the prompt's keys and values summed into the state (one launch; bf16 at D = 64: matrix instructions), timed as
    # five calls in a row between two events, then once more into the cleared state the steps below continue from
    import ctypes as C
    kp, vp = k[:, :prompt], v[:, :prompt]
    pdesc = lib.make_desc(kp, kp, vp, mask=True, a0=1.0, a1=1.0, a2=0.5, **kw)
    s0 = torch.cuda.current_stream().cuda_stream
    ea, eb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    lib.check(lib.lib.fastmax_decode_absorb(C.byref(pdesc), kp.data_ptr(), vp.data_ptr(), state.data_ptr(), s0), "fastmax_decode_absorb")
    torch.cuda.synchronize()
    ea.record()
    for _ in range(5):
        lib.lib.fastmax_decode_absorb(C.byref(pdesc), kp.data_ptr(), vp.data_ptr(), state.data_ptr(), s0)
    eb.record()
    eb.synchronize()
    absorb_ms = ea.elapsed_time(eb) / 5
    state.zero_()
    lib.decode_absorb(kp, vp, state, **kw)
    # the C entry point itself, on buffers made once (the Python front allocates o, g and the scratch per call)
    from reproducing_fastmax_results_amd._capi import _strides, _gstrides
    q1, k1, v1 = q[:, :1], k[:, :1], v[:, :1]
    desc = lib.make_desc(q1, k1, v1, mask=True, a0=1.0, a1=1.0, a2=0.5, **kw)
    o = torch.empty(bh, 1, d, dtype=q.dtype, device=dev)
    g = torch.empty(bh, 1, dtype=torch.float32, device=dev)
    desc.so, desc.sg = _strides(o), _gstrides(g)
    scratch = torch.empty(max(lib.lib.fastmax_decode_scratch_bytes(C.byref(desc)) // 4, 1), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    row = q.stride(1) * q.element_size()

    def one(t):
        nonlocal stream
        st = lib.lib.fastmax_decode_step(C.byref(desc), q.data_ptr() + t * row, k.data_ptr() + t * row, v.data_ptr() + t * row,
                                         state.data_ptr(), o.data_ptr(), g.data_ptr(), scratch.data_ptr(), stream)
        lib.check(st, "fastmax_decode_step")

    for t in range(prompt, prompt + 10):
        one(t)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = steps - 10
    e0.record()
    for t in range(prompt + 10, prompt + steps):
        one(t)
    e1.record()
    e1.synchronize()
    us_eager = 1e3 * e0.elapsed_time(e1) / n
    # the same steps captured as one HIP graph and replayed: what the device needs per token when the host side of
    # the launches (the Python call and the runtime's enqueue, about as long as the kernel itself) is out of the way
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        stream = side.cuda_stream
        one(prompt)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = torch.cuda.current_stream().cuda_stream
        for t in range(prompt + 10, prompt + steps):
            one(t)
    stream = torch.cuda.current_stream().cuda_stream
    graph.replay()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(3):
        graph.replay()
    e1.record()
    e1.synchronize()
    us = 1e3 * e0.elapsed_time(e1) / (3 * n)
    state_bytes = state.numel() * 4
    return {"workload": f"one token per call on the moment state, B*H={bh}, D={d}, after a {prompt}-token prompt",
            "us_per_token": us, "tokens_per_s": 1e6 / us, "us_per_token_eager_python_calls": us_eager, "state_bytes": state_bytes,
            "prompt_absorb_ms": absorb_ms, "prompt_tokens_per_s": bh * prompt / (absorb_ms * 1e-3),
            "roofline": {"bound": "hbm", "achieved": 2 * state_bytes / (us * 1e-6) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": 2 * state_bytes / (us * 1e-6) / 1e9 / PEAK_HBM_GBS,
                         "what": "state read and written once per step, one launch per token; timed as replays of a HIP "
                                 "graph of the steps (eager calls from Python are bound by the host side of the launch)"}}


def percentiles(xs):
    xs = sorted(xs)

    def at(f):
        return xs[min(len(xs) - 1, max(0, int(round(f * (len(xs) - 1)))))]
    return {"median": at(0.5), "p10": at(0.1), "p90": at(0.9), "n": len(xs)}


def operator_line(lib, dev, W, dtype, args, steps, warmup, full):
    """Times one workload: K steps by the wall clock between synchronisations (the contract's figure), the same
    K steps again between HIP events on the launch stream (median / p10 / p90), the forward alone, and every
    kernel by events inside the library.  Every buffer (outputs, workspaces) is allocated once, before."""
    import torch
    B, H, N, D, p = W["B"], W["H"], W["N"], W["D"], W["p"]
    bh = B * H
    tdtype = torch.bfloat16 if dtype == "bf16" else torch.float32
    gen = torch.Generator(device="cpu").manual_seed(1)
    q, k, v = ((W["scale"] * torch.randn(B, H, N, D, generator=gen)).to(tdtype).to(dev).view(bh, N, D) for _ in range(3))
    go = torch.randn(B, H, N, D, generator=gen).to(tdtype).to(dev).view(bh, N, D)
    tau = 8.0 * math.sqrt(D)
    kw = dict(mask=True, inv_tau=1.0 / tau, a0=1.0, a1=1.0, a2=0.5, p=p, chunk=args.chunk)
    from reproducing_fastmax_results_amd._capi import FLAG_SAVE_FOR_BACKWARD
    indep = args.independent_backward
    desc = lib.make_desc(q, k, v, flags=0 if indep else FLAG_SAVE_FOR_BACKWARD, **kw)
    fwd_b, bwd_b = lib.workspace_bytes(desc)
    fwd_plain_b, _ = lib.workspace_bytes(lib.make_desc(q, k, v, **kw))
    o, g = torch.empty_like(q), torch.empty(bh, N, dtype=torch.float32, device=dev)
    grads = tuple(torch.empty_like(q) for _ in range(3))
    ws_f, ws_b = (torch.empty(nb, dtype=torch.uint8, device=dev) for nb in (fwd_b, bwd_b))
    ws_p = torch.empty(fwd_plain_b, dtype=torch.uint8, device=dev)

    # The step as the autograd wrapper runs it: the forward keeps its workspace (key-side copies, prefix states, what
    # bf16 rounding took from o) and the backward of the same step reads it.  The descriptors are filled once and the
    # two C entry points are called directly, so the timed loop holds the library's launches and little else.
    import ctypes as C
    from reproducing_fastmax_results_amd._capi import _gstrides, _strides

    def make_step(L, live_stream=False):
        # live_stream: the stream is looked up at every call (under HIP graph capture torch's current stream is the
        # capturing one, not the one this closure was made on)
        df = L.make_desc(q, k, v, flags=0 if indep else FLAG_SAVE_FOR_BACKWARD, **kw)
        df.so, df.sg = _strides(o), _gstrides(g)
        db = L.make_desc(q, k, v, flags=0 if indep else FLAG_SAVE_FOR_BACKWARD, **kw)
        db.so, db.sg, db.sdo = _strides(o), _gstrides(g), _strides(go)
        db.sdq, db.sdk, db.sdv = (_strides(t) for t in grads)
        stream = torch.cuda.current_stream().cuda_stream
        pf, pb = C.byref(df), C.byref(db)
        ptr = [t.data_ptr() for t in (q, k, v, o, g, go) + grads + (ws_f, ws_b)]
        nf, nb = ws_f.numel(), ws_b.numel()
        fwd, bwd, bwds = L.lib.fastmax_forward, L.lib.fastmax_backward, L.lib.fastmax_backward_saved

        def step():
            nonlocal stream
            if live_stream:
                stream = torch.cuda.current_stream().cuda_stream
            st = fwd(pf, ptr[0], ptr[1], ptr[2], ptr[3], ptr[4], ptr[9], nf, stream)
            if indep:
                st |= bwd(pb, ptr[0], ptr[1], ptr[2], ptr[3], ptr[4], ptr[5], ptr[6], ptr[7], ptr[8], ptr[10], nb, stream)
            else:
                st |= bwds(pb, ptr[0], ptr[1], ptr[2], ptr[3], ptr[4], ptr[5], ptr[6], ptr[7], ptr[8], ptr[9], nf, ptr[10], nb, stream)
            if st:
                raise RuntimeError(f"fastmax step failed with status {st}")
        return step

    step = make_step(lib, live_stream=args.graph)
    from reproducing_fastmax_results_amd._capi import get_bench_lib
    blib = get_bench_lib()
    box = None
    if full:
        # what this box sustains, beside the published peaks the fractions below are priced against (measured first: the
        # device is then at its working clocks when the W warm-up steps of the timed loop begin): a
        # register-only loop of 32x32x16 _Float16 matrix products, and a 1 GiB device-to-device copy
        # (read + write counted)
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            dst.copy_(src)
        e1.record()
        e1.synchronize()
        box = {"mfma_f16_loop_TFLOPs": blib.mfma_rate(dev),
               # the same products fed from LDS with the dense kernels' instruction mix: what a
               # kernel of this structure can reach (one / two own tiles per wavefront)
               "mfma_f16_lds_fed_mix_TFLOPs": blib.mix_rate(dev, 1),
               "mfma_f16_lds_fed_mix_two_tiles_TFLOPs": blib.mix_rate(dev, 2),
               "hbm_copy_GBps": 5 * 2 * float(1 << 30) / (e0.elapsed_time(e1) * 1e-3) / 1e9,
               "published": {"mfma_bf16_TFLOPs": PEAK_TFLOPS["bf16"], "mfma_f32_TFLOPs": PEAK_TFLOPS["f32"],
                             "hbm_GBps": PEAK_HBM_GBS}}
        del src, dst
    run = step
    if args.graph:
        # the whole step as one HIP graph: the library allocates nothing and never synchronises, so
        # a caller can capture it; replays skip the host side of the launches
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        run = graph.replay
    def timed_window():
        """W untimed steps, then exactly K steps between two synchronisations, by the wall clock"""
        for _ in range(warmup):
            run()
        torch.cuda.synchronize()
        t_a = time.perf_counter()
        for _ in range(steps):
            run()
        torch.cuda.synchronize()
        return time.perf_counter() - t_a

    # On this hardware the steps between about 2 and 12 ms after a cold start of this kernel sequence run 5 - 15 %
    # slower than the ones before and after them (the device settling its clocks: the first four steps take 0.384 ms,
    # steps 5 - 28 up to 0.455, every later one 0.381), which is exactly a window of W = 5 and K = 20.  So the window
    # is measured twice: once from the cold start (reported as `first_window`), then the steps again between HIP events
    # (their distribution, `step_ms`), then the window whose figure is the line's `value`: the rate a loop of many
    # steps runs at.
    first_elapsed = timed_window()
    # the same steps between HIP events on the launch stream (torch's current stream is the stream the library
    # launches on): the distribution of one step
    nev = max(steps, 30)
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(nev + 1)]
    evs[0].record()
    for i in range(nev):
        run()
        evs[i + 1].record()
    torch.cuda.synchronize()
    step_ms = percentiles([evs[i].elapsed_time(evs[i + 1]) for i in range(nev)])
    elapsed = timed_window()
    ms_per_step = 1e3 * elapsed / steps
    tokens = B * N
    value = tokens * steps / elapsed
    sclk = sclk_under(run, torch.cuda.synchronize)

    # forward alone (the inference call: no workspace kept for a backward)
    for _ in range(3):
        lib.forward(q, k, v, out=o, g=g, ws=ws_p, **kw)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        lib.forward(q, k, v, out=o, g=g, ws=ws_p, **kw)
    torch.cuda.synchronize()
    fwd_ms = 1e3 * (time.perf_counter() - t0) / steps

    # per-kernel durations, HIP events on the launch stream: the same step through the bench build of the library
    # (same kernels, every launch bracketed by events; the product library carries no such hooks)
    bstep = make_step(blib)
    nprof = max(3, min(10, steps))
    for _ in range(max(20, warmup)):         # the bench build is a code object of its own: its first launches run slower
        bstep()
    torch.cuda.synchronize()
    blib.profile_begin()
    for _ in range(nprof):
        bstep()
    recs = blib.profile_end()
    per_kernel = {}
    for name, ms in recs:
        tot, cnt = per_kernel.get(name, (0.0, 0))
        per_kernel[name] = (tot + ms, cnt + 1)
    units = UNITS_STATE if "build" in per_kernel else UNITS_DENSE
    # tensors (bh * N * D elements each) a kernel of an order-1 step has to read and write once
    k_tensors = {"fwd": 4, "dq": 5, "dk": 5, "dv": 4, "dkv": 8, "build": 2}
    heavy = {nme: v for nme, v in per_kernel.items() if nme in (k_tensors if p == 1 else units)}
    dominant = max(heavy, key=lambda nme: heavy[nme][0] / heavy[nme][1])
    avg_ms = per_kernel[dominant][0] / per_kernel[dominant][1]
    unit = alg_flops_unit(bh, N, D, p)
    achieved = units.get(dominant, 0) * unit / (avg_ms * 1e-3) / 1e12
    peak = PEAK_TFLOPS[dtype]
    # `achieved` / `frac`: ALGORITHMIC flop of the moment formulation per launch of the dominant kernel (the
    # definition the metric fixes, whatever form the kernel computes in); `executed`: what its matrix
    # instructions actually execute (set below when the kernel runs dense causal tiles only)
    roofline = {"bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                "frac": achieved / peak, "traffic": None, "avg_ms": avg_ms,
                "algorithmic_flop_per_launch": units.get(dominant, 0) * unit,
                "whole_step": {"achieved": 7 * unit / (ms_per_step * 1e-3) / 1e12,
                               "frac": 7 * unit / (ms_per_step * 1e-3) / 1e12 / peak},
                "kernels_ms_per_step": {nme: tot / nprof for nme, (tot, cnt) in sorted(per_kernel.items())}}
    if p == 1:
        # order 1 is bandwidth bound (M_1 = D features: 130 flop per byte of q, k, v, o): price it against HBM.
        # Algorithmic bytes: the forward reads q, k, v and writes o; the backward reads q, k, v, o, dO and
        # writes dq, dk, dv; per kernel, the tensors it must read and write once.
        esz_io = 2 if dtype == "bf16" else 4
        tensor_b = bh * N * D * esz_io
        dom_b = k_tensors[dominant] * tensor_b
        roofline = {"bound": "hbm", "kernel": dominant, "achieved": dom_b / (avg_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                    "unit": "GB/s", "frac": dom_b / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None, "avg_ms": avg_ms,
                    "whole_step": {"achieved": 12 * tensor_b / (ms_per_step * 1e-3) / 1e9,
                                   "frac": 12 * tensor_b / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBS},
                    "kernels_ms_per_step": roofline["kernels_ms_per_step"]}
    if "build" not in per_kernel and dtype == "bf16" and p == 2:
        # what the matrix cores actually execute when one segment covers the sequence: causal 32x32 tiles only
        nt = (N + 31) // 32
        tiles = bh * nt * (nt + 1) // 2
        per_tile = 2.0 * 32 * 32 * 16
        executed = sum(MFMA_PER_TILE[nme] for nme in per_kernel if nme in MFMA_PER_TILE) * tiles * per_tile
        dom_exec = MFMA_PER_TILE[dominant] * tiles * per_tile
        roofline["executed"] = {"flop_per_launch": dom_exec, "achieved": dom_exec / (avg_ms * 1e-3) / 1e12,
                                "frac": dom_exec / (avg_ms * 1e-3) / 1e12 / peak}
        roofline["executed_mfma"] = {"flop_per_step": executed,
                                     "achieved": executed / (ms_per_step * 1e-3) / 1e12,
                                     "frac": executed / (ms_per_step * 1e-3) / 1e12 / peak}
    if sclk:
        # the published peak is quoted at the nominal engine clock; under these kernels the device holds a lower one
        # (power management), and the matrix rate it can deliver scales with it
        roofline["clock"] = {"sclk_MHz_under_this_step": sclk, "nominal_MHz": NOMINAL_SCLK_MHZ,
                             "what": "median of the driver's current shader clock, sampled every 10 ms while the step "
                                     "runs in a loop for 0.4 s"}
        if roofline["bound"] == "mfma":
            roofline["clock"]["peak_at_that_clock"] = peak * sclk / NOMINAL_SCLK_MHZ
            roofline["clock"]["frac_at_that_clock"] = roofline["frac"] * NOMINAL_SCLK_MHZ / sclk
    tkey = (W["N"], p, dtype, args.chunk, dominant)
    if tkey in TRAFFIC:
        roofline["traffic"] = TRAFFIC[tkey]["bytes"]
        roofline["traffic_source"] = TRAFFIC[tkey]["source"]

    out = {
        "metric": f"Fastmax fwd+bwd tokens/s, causal order-{p} N={N} D={D}",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": f"{W['name'].replace('order-2', f'order-{p}')} B={B} H={H} N={N} D=Dv={D} tau=8*sqrt(D) a=(1,1,0.5)",
                   "chunk": args.chunk or "auto", "launch": "hip graph replay" if args.graph else "eager",
                   "compute": "bf16 tensors, f16 MFMA operands, fp32 accumulate" if dtype == "bf16" else "fp32 tensors, fp32 MFMA"},
        "step_ms": step_ms,
        "first_window": {"ms_per_step": 1e3 * first_elapsed / steps, "tokens_per_s": tokens * steps / first_elapsed,
                         "what": "the same W + K steps run first, from a cold start of the kernel sequence"},
        "roofline": roofline,
        "forward_only": {"ms": fwd_ms, "tokens_per_s": tokens / (fwd_ms * 1e-3),
                         "algorithmic_TFLOPs": 2 * unit / (fwd_ms * 1e-3) / 1e12,
                         "frac_of_peak": 2 * unit / (fwd_ms * 1e-3) / 1e12 / peak},
    }
    # the bandwidth-bound helpers of the path on the same tensors: event-timed passes against the HBM peak
    esz = 2 if dtype == "bf16" else 4
    tensor = bh * N * D * esz
    helpers = {}
    for name, fn, nbytes in (
            # the statistics pass of the folded max-norm normalisation: q and k read once (the kernels scale as they load)
            ("normalize", lambda: blib.maxnorm_stats(q, k), 2 * tensor),) + (() if not full else (
            # the stand-alone passes (token-mean centring and other callers): forward one statistics read, one apply
            # read, one write; backward: x and dy twice, dx once
            ("normalize_pass", lambda: blib.normalize(q, centre=0, max_norm=True, scale=1.0), 3 * tensor),
            ("normalize_backward", lambda: blib.normalize_backward(q, go, centre=0, max_norm=True, scale=1.0), 5 * tensor))):
        fn()
        torch.cuda.synchronize()
        blib.profile_begin()
        for _ in range(5):
            fn()
        ms = sum(t for nme, t in blib.profile_end() if nme == "normalize") / 5
        helpers[name] = {"ms": ms, "bytes": nbytes, "achieved_GBps": nbytes / (ms * 1e-3) / 1e9,
                         "frac_of_8TBps": nbytes / (ms * 1e-3) / 8e12}
    if "transpose" in roofline["kernels_ms_per_step"]:
        t_ms = roofline["kernels_ms_per_step"]["transpose"]
        ncopies = 2 if (dtype == "bf16" and "build" not in per_kernel) else 4    # row-major (+ transposed) copies of k and v
        nbytes = 2 * tensor + ncopies * bh * N * D * esz
        helpers["transpose"] = {"ms": t_ms, "bytes": nbytes, "achieved_GBps": nbytes / (t_ms * 1e-3) / 1e9,
                                "frac_of_8TBps": nbytes / (t_ms * 1e-3) / 8e12}
    out["hbm_bound_helpers"] = helpers
    if not full:
        return out
    # the same step with q and k max-norm normalised on load and the gradients taken through the normalisation
    # (what the reference model's attention does, transformer/model.py:292-300), against the plain step
    qk, kk = lib.maxnorm_stats(q, k)
    nkw = dict(kw, norm=(qk, kk, 1.0, True), inv_tau=1.0)
    nf, nb = lib.workspace_bytes(lib.make_desc(q, k, v, flags=FLAG_SAVE_FOR_BACKWARD, **nkw))
    ws_nf, ws_nb = (torch.empty(x, dtype=torch.uint8, device=dev) for x in (nf, nb))

    def norm_step():
        lib.maxnorm_stats(q, k)
        lib.forward(q, k, v, save=True, out=o, g=g, ws=ws_nf, **nkw)
        return lib.backward(q, k, v, o, g, go, saved=ws_nf, out=grads, ws=ws_nb, **nkw)

    for _ in range(3):
        norm_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        norm_step()
    torch.cuda.synchronize()
    norm_ms = 1e3 * (time.perf_counter() - t0) / steps
    out["normalized_step"] = {"ms_per_step": norm_ms, "over_plain_step": norm_ms / ms_per_step,
                              "what": "max-norm normalisation of q and k folded into the loads, its Jacobian in the backward"}
    out["measured_on_this_box"] = box
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    if not args.no_cpu_baseline and args.workload == "headline" and p == 2:
        out["cpu_baseline"] = cpu_baseline(N, D, p, tokens, bh, args.cpu_max_n)
        out["cpu_baseline_closed_form"] = cpu_closed_form(N, D, p, tokens, bh)
    return out


if __name__ == "__main__":
    sys.exit(main())
