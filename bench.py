#!/usr/bin/env python3
"""Benchmark of the dynamic-k MoE-FFN forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload vit_b_50k] [--no-cpu-baseline] [--no-sweep]

One "step" is one pass of the whole layer (router MLP -> dynamic-k selection -> experts -> bias epilogue) over one
batch of synthetic tokens that already sit in HBM; the timed steps are replays of a HIP graph that holds up to 25
consecutive layer calls, as a model's captured forward pass holds its layers (the same steps launched eagerly from Python
are reported as ms_per_step_eager_launches, replays of a graph holding ONE call as ms_per_step_single_call_graph).  The default workload is the ViT-B-shape layer of the headline
metric: 256 x 197 = 50432 tokens, D = 768, 128 experts x 24 neurons, ReLU, bf16 storage with float32 accumulation,
module tau = 0.9 (the layer keeps expert e when norm_e >= (1 - tau) * max norm, the reference's convention).
The literal reading "norm_e >= 0.9 * max" of the same number is measured too and reported under "literal_rule".

Prints ONE JSON line.  Beyond the common fields it carries
  roofline      the dominant kernel (the experts kernel) against the MI355X bf16 MFMA peak: achieved = active-expert
                FLOPs (routed (token, expert) pairs x 4*D*Ed) / the kernel's mean duration, taken with HIP events on
                the launch stream inside this run
  sweep         the threshold number v in {0.5, 0.8, 0.9, 0.95, 0.99} under both readings (module tau: keep norm >=
                (1 - v) * max; literal: keep norm >= v * max) with mean / p99 experts per token
  dense_mlp_ms, measured_ceilings   the dense FFN of the same size on library GEMMs, and what this GPU sustains on
                a large library GEMM and a streaming copy
  cpu_baseline  the CPU restatement of the reference's PyTorch CPU path (router + gate + per-expert loop) timed on
                this machine's host cores over a bounded sample of the same layer shape
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3     # MI355X float32 matrix
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E

WORKLOADS = {
    # name: (batch, seq, D, E, Ed, W, activation)
    'vit_b_50k': (256, 197, 768, 128, 24, 128, 'relu'),
    'vit_b_1576': (8, 197, 768, 128, 24, 128, 'relu'),
    # skewed routing: router bypassed, norms = |randn| * w_e with w_e = rank_e^-1.2 (a few experts draw most tokens)
    'vit_b_skew': (256, 197, 768, 128, 24, 128, 'relu'),
    # the CPU baseline's own case (8 x 197 tokens, float32) on the GPU: float32 storage and float32 matrix arithmetic
    'vit_b_1576_f32': (8, 197, 768, 128, 24, 128, 'relu'),
    # float16 storage (the reference benches float32 and float16): same kernel families as bf16
    'vit_b_50k_f16': (256, 197, 768, 128, 24, 128, 'relu'),
    # one FFN layer of a GPT-2-medium-sized model (D = 1024, d_ff = 4096 as 128 experts x 32, GELU), 16 x 1024 tokens:
    # the D = 1024 sweep under module tau 0.9, expert-major kernels under the literal rule
    'gpt2_medium_layer': (16, 1024, 1024, 128, 32, 128, 'gelu'),
    # the expert split of the reference's own micro-benchmark (scripts/test_moe_implementations.py:109-126: 24 experts of
    # 128 neurons) behind a real router: the sweep under module tau 0.9, the expert-major kernel for big experts under
    # the literal rule (the Bernoulli sweep of that script is the default line's reference_shape sub-record)
    'vit_b_24x128': (256, 197, 768, 24, 128, 128, 'relu'),
}
TRAFFIC_TABLE = os.path.join(ROOT, 'profiles', 'traffic_per_launch.md')


def measured_traffic(workload):
    """HBM bytes per launch of the workload's dominant kernel(s), from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs: read from
    the table committed under profiles/ (one row per workload: bytes, the summary it comes from, the commit it was taken
    at).  Returns (bytes or None, source or None); nothing is assumed when the table or the row is missing."""
    try:
        with open(TRAFFIC_TABLE) as f:
            for row in f:
                cells = [c.strip().strip('`') for c in row.strip().strip('|').split('|')]
                if len(cells) >= 5 and cells[0] == workload:
                    return float(cells[2]) * 1e6, {'file': 'profiles/' + cells[3], 'kernels': cells[1], 'commit': cells[4]}
    except (OSError, ValueError):
        pass
    return None, None


# Gemma-2B-shape gated layer: (tokens, D, E, Ed, W, activation)
GATED_WORKLOADS = {
    'gemma_1': (1, 2048, 256, 64, 256, 'gelu_tanh'),
    'gemma_16': (16, 2048, 256, 64, 256, 'gelu_tanh'),
    'gemma_4096': (4096, 2048, 256, 64, 256, 'gelu_tanh'),
}


def make_params(D, E, Ed, W, seed, dtype, device):
    """Seeded weights with the reference's init (uniform +-1/sqrt(last dim); nn.Linear default for the router)."""
    g = torch.Generator().manual_seed(seed)

    def uni(*shape, fan):
        return ((torch.rand(*shape, generator=g) * 2 - 1) / fan ** 0.5).to(dtype).to(device)

    return dict(w1=uni(E, D, Ed, fan=Ed), b1=uni(E, Ed, fan=Ed), w2=uni(E, Ed, D, fan=D),
                last_bias=torch.zeros(D, dtype=dtype, device=device),
                router_w1=uni(W, D, fan=D), router_w2=uni(E, W, fan=W))


COLD_SETS = 4        # weight copies the small-batch workloads rotate over for their cold-operand figures
SPIN_UP_MS = 60.0   # see spin_up(); --spin-up-ms changes it, 0 switches it off


def spin_up(fn, ms=None):
    """Keeps the GPU under the load of fn for `ms` milliseconds before a timed region.  After ANY idle spell -- 50 ms are
    enough, and so is the pause around a graph capture -- this GPU runs the first ~20 launches of the dense sweep 15-20 %
    slower and reaches its steady rate only after ~40 ms of continuous load (measured per launch: 0.52, 0.457, 0.442,
    0.437, 0.433 ... ms as means over successive groups of 20).  A timed region of 20 steps behind 5 warm-up steps falls
    entirely inside that ramp.  The W warm-up steps the caller asked for still follow, then the K timed steps."""
    ms = SPIN_UP_MS if ms is None else ms
    if ms <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def time_events(fn, steps, warmup):
    """Mean milliseconds per call of fn, HIP events on torch's current stream (the stream fn launches on)."""
    spin_up(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


GRAPH_CALLS_MAX = 25   # calls of fn held by one captured graph at most (each call keeps its own output buffers alive)


def time_graph(fn, steps, warmup):
    """Mean milliseconds per call of fn when the calls are captured into a HIP graph and replayed (the C ABI calls neither
    allocate nor synchronise, so a whole layer captures).  The graph holds up to GRAPH_CALLS_MAX consecutive calls of fn,
    as the layers of a model follow each other in one captured forward pass: what is timed is `steps` calls, as whole
    replays of that graph plus single-call replays for the remainder, wall clock bracketed by synchronize.  (A replay of
    a graph that holds ONE call pays 8-9 us of replay-to-replay gap per call on this machine, which a model's graph pays
    once per forward pass; `ms_per_step_single_call_graph` in the output keeps that figure.)"""
    def capture(n_calls):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(n_calls):
                fn()
        return graph

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    per = max(1, min(steps, GRAPH_CALLS_MAX))
    single = capture(1)
    many = capture(per) if per > 1 else single
    torch.cuda.synchronize()
    spin_up(single.replay)
    for _ in range(warmup):
        single.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps // per):
        many.replay()
    for _ in range(steps % per):
        single.replay()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    # the same number of steps as single-call replays, for the record
    t0 = time.perf_counter()
    for _ in range(steps):
        single.replay()
    torch.cuda.synchronize()
    time_graph.last_single_call_ms = (time.perf_counter() - t0) * 1e3 / steps
    return ms


def time_quantiles(fn, iters, warmup):
    """Per-call durations of fn from one HIP event pair per call on the launch stream: median, 2.5 % and 97.5 %
    quantiles in milliseconds (the reference's own bench reports the same three, test_moe_implementations.py:171-175)."""
    spin_up(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in evs)
    return {'median_ms': t[len(t) // 2], 'q025_ms': t[int(0.025 * (len(t) - 1))], 'q975_ms': t[int(0.975 * (len(t) - 1))],
            'iters': iters}


def measured_ceilings(dev):
    """What this very GPU sustains on plain library work: a large bf16 GEMM (hipBLASLt through torch, in both layouts of
    the second operand; the faster one is the figure quoted) and a streaming copy.  Printed next to the published peaks; the roofline fractions stay relative to the published ones."""
    a = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
    b = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
    ms_nn = time_events(lambda: torch.matmul(a, b), 10, 3)
    ms_nt = time_events(lambda: torch.nn.functional.linear(a, b), 10, 3)   # the weight operand row-major in K: nn.Linear's layout
    gemm_nn, gemm_nt = 2 * 8192 ** 3 / ms_nn / 1e9, 2 * 8192 ** 3 / ms_nt / 1e9
    gemm = max(gemm_nn, gemm_nt)
    del a, b
    src = torch.zeros(64 << 20, dtype=torch.float32, device=dev)   # 256 MiB read + 256 MiB written per call
    dst = torch.empty_like(src)
    ms = time_events(lambda: dst.copy_(src), 10, 3)
    copy = 2 * src.numel() * 4 / ms / 1e6
    del src, dst
    return {'library_gemm_bf16_8192_tflops': gemm, 'library_gemm_bf16_8192_nn_tflops': gemm_nn,
            'library_gemm_bf16_8192_nt_tflops': gemm_nt, 'copy_gbps': copy}


def dense_mlp_ms(x, D, hidden, act, steps, warmup):
    """The dense FFN the MoE layer was split from (Linear(D, hidden) + activation + Linear(hidden, D), bf16, library
    GEMMs), timed on the same tokens; the reference times a compiled MLP alongside its kernels the same way
    (test_moe_implementations.py:128-131, 172-176)."""
    g = torch.Generator().manual_seed(7)
    fc1 = ((torch.rand(hidden, D, generator=g) * 2 - 1) / D ** 0.5).to(x.dtype).to(x.device)
    b1 = torch.zeros(hidden, dtype=x.dtype, device=x.device)
    fc2 = ((torch.rand(D, hidden, generator=g) * 2 - 1) / hidden ** 0.5).to(x.dtype).to(x.device)
    b2 = torch.zeros(D, dtype=x.dtype, device=x.device)
    fn_act = {'relu': torch.relu, 'gelu': torch.nn.functional.gelu}[act]
    return time_events(lambda: torch.nn.functional.linear(fn_act(torch.nn.functional.linear(x, fc1, b1)), fc2, b2), steps, warmup)


def run_regime(ops, x, p, packed, thr_scale, act, steps, warmup, D, E, Ed, W, path='auto', quantile_iters=0, norms_in=None):
    N = x.size(0)

    def layer():
        return ops.forward(x, p['router_w1'], p['router_w2'], thr_scale, p['w1'], p['b1'], p['w2'], None, p['last_bias'],
                           act, False, norms_in, False, False, path, packed)

    out, routing, _, _ = layer()
    torch.cuda.synchronize()
    per_token = routing.float().sum(-1)
    pairs = int(per_token.sum().item())
    mean_k = per_token.mean().item()
    p99_k = torch.quantile(per_token, 0.99).item()
    # whole layer, wall clock bracketed by synchronize
    spin_up(layer)
    for _ in range(warmup):
        layer()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        layer()
    torch.cuda.synchronize()
    ms_layer_eager = (time.perf_counter() - t0) * 1e3 / steps
    # the same step replayed from a HIP graph: removes the host's launch latency between the dependent kernels
    ms_layer = time_graph(layer, steps, warmup)
    ms_layer_single = time_graph.last_single_call_ms
    # dominant kernel alone (same routing), HIP events on the launch stream
    # the experts call the layer makes: under AUTO d2dmoe_forward takes the expert-major path for high thresholds
    experts_path = path if path != 'auto' else ('mfma_sparse' if thr_scale >= 0.75 and x.dtype in (torch.bfloat16, torch.float16) else 'auto')
    ms_experts = time_events(lambda: ops.experts(x, routing, p['w1'], p['b1'], p['w2'], None, p['last_bias'], act, False,
                                                 experts_path, packed), steps, warmup)
    quant = None
    if quantile_iters:
        quant = time_quantiles(lambda: ops.experts(x, routing, p['w1'], p['b1'], p['w2'], None, p['last_bias'], act, False,
                                                   experts_path, packed), quantile_iters, 20)
    ms_router = time_events(lambda: ops.router_select(x, p['router_w1'], p['router_w2'], thr_scale, packed, E, Ed),
                            steps, warmup)
    tokens_per_expert = routing.float().sum(0)
    active_flops = pairs * 4.0 * D * Ed
    router_flops = N * (2.0 * D * W + 2.0 * W * E)
    s = x.element_size()
    algo_bytes = N * D * s * 2 + N * E * s + (2 * E * D * Ed + E * Ed + D + W * D + E * W) * s
    return dict(ms_layer=ms_layer, ms_layer_eager=ms_layer_eager, ms_layer_single=ms_layer_single, ms_experts=ms_experts, ms_router=ms_router, pairs=pairs, mean_active=mean_k,
                p99_active=p99_k, active_tflops_layer=active_flops / ms_layer / 1e9,
                active_tflops_kernel=active_flops / ms_experts / 1e9,
                total_tflops_layer=(active_flops + router_flops) / ms_layer / 1e9,
                algo_bytes=algo_bytes, hbm_gbps_layer=algo_bytes / ms_layer / 1e6, tokens_per_s=N / ms_layer * 1e3,
                experts_quantiles=quant,
                expert_load_max_over_mean=(tokens_per_expert.max() / tokens_per_expert.mean().clamp_min(1e-9)).item())


def cold_regime(ops, x, p, packed, thr_scale, act, steps, warmup, D, E, Ed, path='auto'):
    """The layer with cold operands, as it runs inside a model: the step rotates over COLD_SETS sets of inputs, weights
    and packed buffers (> 256 MB in all from 16 384 tokens on, the size of the memory-side cache), so that a call finds
    none of its weights in a cache -- other layers' work has gone through them since.  The reference's timer clears the
    cache between repetitions too (triton do_bench, scripts/test_moe_implementations.py:171-175).  Returns the whole-layer
    time (replays of a graph holding whole rotations) and the experts kernel's (HIP events around a rotation)."""
    sets = [(x, p, packed)]
    for k in range(1, COLD_SETS):
        g = torch.Generator().manual_seed(100 + k)
        xk = torch.randn(x.shape, generator=g).to(x.dtype).to(x.device)
        pk = {name: v.clone() for name, v in p.items()}
        sets.append((xk, pk, ops.clone_packed(packed)))
    routings = []
    for xk, pk, pkd in sets:
        routings.append(ops.forward(xk, pk['router_w1'], pk['router_w2'], thr_scale, pk['w1'], pk['b1'], pk['w2'], None,
                                    pk['last_bias'], act, False, None, False, False, path, pkd)[1])
    experts_path = path if path != 'auto' else ('mfma_sparse' if thr_scale >= 0.75 and x.dtype in (torch.bfloat16, torch.float16) else 'auto')

    def rotation():
        for xk, pk, pkd in sets:
            ops.forward(xk, pk['router_w1'], pk['router_w2'], thr_scale, pk['w1'], pk['b1'], pk['w2'], None, pk['last_bias'],
                        act, False, None, False, False, path, pkd)

    def experts_rotation():
        for (xk, pk, pkd), r in zip(sets, routings):
            ops.experts(xk, r, pk['w1'], pk['b1'], pk['w2'], None, pk['last_bias'], act, False, experts_path, pkd)

    reps, wreps = max(steps // COLD_SETS, 3), max(warmup // COLD_SETS, 1)
    ms_layer = time_graph(rotation, reps, wreps) / COLD_SETS
    ms_experts = time_events(experts_rotation, reps, wreps) / COLD_SETS
    pairs = sum(r.float().sum().item() for r in routings) / COLD_SETS
    return {'operand_sets': COLD_SETS, 'ms_per_step': ms_layer, 'kernel_ms': ms_experts, 'mean_pairs': pairs}


def run_gated(args, ops, dev):
    print(json.dumps(gated_record(args, ops, dev, args.workload)))


def gated_record(args, ops, dev, workload):
    """Gemma-shape gated layer: whole-layer time and the HBM rate over the bytes that have to move (router weights,
    the weights of every expert some token routes to, token input/output)."""
    N, D, E, Ed, W, act = GATED_WORKLOADS[workload]
    traffic, traffic_src = measured_traffic(workload)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(0)

    def uni(*shape, fan):
        return ((torch.rand(*shape, generator=g) * 2 - 1) / fan ** 0.5).to(dtype).to(dev)

    wg, wd, wu = uni(E, D, Ed, fan=Ed), uni(E, Ed, D, fan=D), uni(E, D, Ed, fan=Ed)
    rw1, rw2 = uni(W, D, fan=D), uni(E, W, fan=W)
    x = torch.randn(N, D, generator=torch.Generator().manual_seed(1)).to(dtype).to(dev)
    shape = ops.make_shape(N, D, E, Ed, W, ops._dtype_code(x), act, gated=True)
    packed = ops.pack_weights(shape, wg, None, wd, wu, rw1, rw2)
    thr_scale = float(1.0 - args.tau)

    def layer():
        return ops.forward(x, rw1, rw2, thr_scale, wg, None, wd, wu, None, act, False, None, False, False, 'auto', packed)

    out, routing, _, _ = layer()
    torch.cuda.synchronize()
    union = int((routing.float().sum(0) > 0).sum().item())
    pairs = int(routing.float().sum().item())
    ms_layer_eager = time_events(layer, args.steps, args.warmup)
    # the step, as for the headline: replays of a HIP graph holding consecutive layer calls (eager launches are reported
    # beside it)
    ms_layer_graph = time_graph(layer, args.steps, args.warmup)
    ms_layer = ms_layer_graph
    ms_experts = time_events(lambda: ops.experts(x, routing, wg, None, wd, wu, None, act, False, 'auto', packed),
                             args.steps, args.warmup)
    s = x.element_size()
    algo_bytes = (W * D + E * W) * s + union * 3 * D * Ed * s + 2 * N * D * s + N * E * s
    cold = None
    if N <= 16:
        # Cold operands.  The step above runs on ONE set of weights, whose 201 MB the 256 MB memory-side cache keeps between
        # repetitions; the reference's timer clears the cache between repetitions (triton do_bench,
        # scripts/test_moe_implementations.py:171-175).  Here the step rotates over COLD_SETS copies of the weights (packed
        # buffer and router weights; > 2.4 GB in all, each copy's small-batch section 201 MB), so every call streams its
        # weights from HBM.  Timed over whole rotations: HIP events around eager launches, and replays of one graph that
        # holds one call per copy.
        sets = [(rw1, rw2, packed)] + [(rw1.clone(), rw2.clone(), ops.clone_packed(packed)) for _ in range(COLD_SETS - 1)]

        def layer_on(k):
            r1, r2, pk = sets[k]
            return ops.forward(x, r1, r2, thr_scale, wg, None, wd, wu, None, act, False, None, False, False, 'auto', pk)

        def rotation():
            for k in range(COLD_SETS):
                layer_on(k)

        def experts_rotation():
            for k in range(COLD_SETS):
                ops.experts(x, routing, wg, None, wd, wu, None, act, False, 'auto', sets[k][2])

        reps = max(args.steps // COLD_SETS, 3)
        cold_eager = time_events(rotation, reps, max(args.warmup // COLD_SETS, 1)) / COLD_SETS
        cold_graph = time_graph(rotation, reps, max(args.warmup // COLD_SETS, 1)) / COLD_SETS
        cold_layer = cold_graph
        cold_experts = time_events(experts_rotation, reps, max(args.warmup // COLD_SETS, 1)) / COLD_SETS
        kernel_bytes = union * 3 * D * Ed * s + 2 * N * D * s
        cold = {'weight_sets': COLD_SETS, 'ms_per_step': cold_layer, 'ms_per_step_eager_launches': cold_eager,
                'ms_per_step_graph_replay': cold_graph, 'layer_frac': algo_bytes / cold_layer / 1e6 / PEAK_HBM_GBPS,
                'kernel_ms': cold_experts, 'frac': kernel_bytes / cold_experts / 1e6 / PEAK_HBM_GBPS}
        del sets
    line = {
        'metric': f'MoE-FFN tokens/s + active TFLOP/s & HBM GB/s vs roofline, Gemma-2B-shape gated layer tau={args.tau}',
        'value': N / ms_layer * 1e3, 'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'spin_up_ms': SPIN_UP_MS,
        'ms_per_step': ms_layer, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16',
        'data': 'synthetic',
        'config': {'workload': f'{workload}: {N} tokens, D={D}, {E} gated experts x {Ed}, {act}, router {D}->{W}->{E}, '
                               f'module tau={args.tau}, whole layer', 'experts_routed_to': union,
                   'mean_active_experts': pairs / N, 'mfma_kernels': packed is not None},
        'ms_per_step_eager_launches': ms_layer_eager, 'ms_per_step_graph_replay': ms_layer_graph,
        'active_tflops': pairs * 6.0 * D * Ed / ms_layer / 1e9, 'hbm_gbps': algo_bytes / ms_layer / 1e6,
        'roofline': {'bound': 'hbm', 'kernel': 'experts (hidden + out kernels)',
                     'achieved': (union * 3 * D * Ed * s + 2 * N * D * s) / ms_experts / 1e6,
                     'peak': PEAK_HBM_GBPS, 'unit': 'GB/s',
                     'frac': (union * 3 * D * Ed * s + 2 * N * D * s) / ms_experts / 1e6 / PEAK_HBM_GBPS,
                     'traffic': traffic, 'traffic_source': traffic_src,
                     'kernel_ms': ms_experts, 'algorithmic_bytes_layer': algo_bytes,
                     'layer_frac': algo_bytes / ms_layer / 1e6 / PEAK_HBM_GBPS},
    }
    if cold is not None:
        # warm = the figures above (one weight set, resident in the memory-side cache between steps)
        line['roofline']['cold'] = cold
    if N > 16:
        # enough tokens per expert to be compute-bound: active-pair FLOPs against the MFMA peak; the tiled products
        # execute every (token, expert) pair, so the executed rate is reported as well
        active = pairs * 6.0 * D * Ed
        executed = N * E * 6.0 * D * Ed
        line['roofline'] = {'bound': 'mfma', 'kernel': 'experts (up + down products + finish)',
                            'achieved': active / ms_experts / 1e9, 'peak': PEAK_BF16_TFLOPS, 'unit': 'TFLOP/s',
                            'frac': active / ms_experts / 1e9 / PEAK_BF16_TFLOPS,
                            'traffic': traffic, 'traffic_source': traffic_src, 'kernel_ms': ms_experts,
                            'executed_tflops': executed / ms_experts / 1e9}
        # the literal reading of the same number (keep norm >= tau * max): a few experts per token, the layer is bound by
        # the weight stream again and takes the expert-major path
        lit_scale = float(args.tau)

        def layer_lit():
            return ops.forward(x, rw1, rw2, lit_scale, wg, None, wd, wu, None, act, False, None, False, False, 'auto', packed)

        _, r_lit, _, _ = layer_lit()
        torch.cuda.synchronize()
        ms_lit = time_graph(layer_lit, args.steps, args.warmup)
        union_lit = int((r_lit.float().sum(0) > 0).sum().item())
        pairs_lit = int(r_lit.float().sum().item())
        bytes_lit = (W * D + E * W) * s + union_lit * 3 * D * Ed * s + 2 * N * D * s + N * E * s
        line['literal_rule'] = {'rule': f'keep norm >= {args.tau}*max', 'ms_per_step': ms_lit, 'tokens_per_s': N / ms_lit * 1e3,
                                'mean_active_experts': pairs_lit / N, 'experts_routed_to': union_lit,
                                'roofline': {'bound': 'hbm', 'achieved': bytes_lit / ms_lit / 1e6, 'peak': PEAK_HBM_GBPS,
                                             'unit': 'GB/s', 'frac': bytes_lit / ms_lit / 1e6 / PEAK_HBM_GBPS,
                                             'algorithmic_bytes': bytes_lit}}
    return line


def gpt2_record(args, dev):
    """Whole-model workload: GPT-2-small (12 blocks, D = 768, 12 heads, vocab 50257) with every FFN replaced by a MoE layer
    of 128 experts x 24 neurons (GELU-erf, biases) and a 768 -> 128 -> 128 router; 16 x 1024 token ids; bf16; random
    weights.  Attention, LayerNorm, embeddings and the LM head are stock PyTorch; the MoE layers are this library."""
    from d2dmoe_amd import add_routers, gpt2, ops
    torch.manual_seed(0)
    cfg = gpt2.GPTConfig(block_size=1024, vocab_size=50257, n_layer=12, n_head=12, n_embd=768)
    dense = gpt2.GPT(cfg).eval().to(dev).to(torch.bfloat16)
    moe, names = gpt2.replace_with_moes(dense, num_experts=128, experts_class='hip_kernel')
    gpt2.split_original_parameters(dense, moe, names)
    add_routers(moe, dict(width=128, depth=2, bias=False, activation='relu', output_activation='abs'))
    moe = moe.to(dev).to(torch.bfloat16)
    layers = [gpt2.get_module_by_name(moe, n) for n in names]
    for layer in layers:
        layer.forward_mode, layer.tau = 'dynk_max', args.tau
        layer.experts.forward_mode = 'hip'
    B, T = 16, 1024
    idx = torch.randint(0, cfg.vocab_size, (B, T), generator=torch.Generator().manual_seed(1)).to(dev)
    captured = {}
    hooks = [layer.register_forward_hook(lambda m, inp, out, n=n: captured.__setitem__(n, (inp[0].detach(), out[1][n][0])))
             for n, layer in zip(names, layers)]
    moe(idx)
    for h in hooks:
        h.remove()
    torch.cuda.synchronize()
    ms_moe_model = time_events(lambda: moe(idx), args.steps, args.warmup)
    ms_dense_model = time_events(lambda: dense(idx), args.steps, args.warmup)
    per_layer = []
    for n, layer in zip(names, layers):
        x, routing = captured[n]
        ms = time_events(lambda: layer(x), args.steps, args.warmup)
        per_layer.append({'layer': n, 'ms': ms, 'mean_active_experts': routing.float().sum(-1).mean().item()})
    ms_moe_layers = sum(r['ms'] for r in per_layer)
    ms_dense_ffn = time_events(lambda: dense.transformer.h[0].mlp(captured[names[0]][0]), args.steps, args.warmup)
    # dominant kernel: the experts kernel of the first MoE layer on its real input and routing
    x0, r0 = captured[names[0]]
    ex = layers[0].experts
    x0 = x0.reshape(-1, 768).contiguous()
    r0 = r0.reshape(-1, 128).contiguous()
    packed = ex.packed_weights(layers[0].router.layers[0].weight, layers[0].router.layers[2].weight, 'relu', 'abs')
    lb = layers[0].last_bias.view(-1)
    ms_experts = time_events(lambda: ops.experts(x0, r0, ex.w1, ex.b1, ex.w2, None, lb, 'gelu', False, 'auto', packed),
                             args.steps, args.warmup)
    active = r0.float().sum().item() * 4.0 * 768 * 24
    N = B * T
    # the literal rule (keep norm >= tau * max) on the same model: module tau = 1 - tau
    for layer in layers:
        layer.tau = 1.0 - args.tau
    lit_k = {}
    hooks = [layer.register_forward_hook(lambda m, inp, out, n=n: lit_k.__setitem__(n, out[1][n][0].float().sum(-1).mean().item()))
             for n, layer in zip(names, layers)]
    moe(idx)
    for h in hooks:
        h.remove()
    torch.cuda.synchronize()
    ms_lit_model = time_events(lambda: moe(idx), args.steps, args.warmup)
    ms_lit_layers = sum(time_events(lambda: layer(captured[n][0]), args.steps, args.warmup) for n, layer in zip(names, layers))
    for layer in layers:
        layer.tau = args.tau
    line = {
        'metric': 'MoE-FFN tokens/s + active TFLOP/s & HBM GB/s vs roofline, ViT-B layer tau=0.9',
        'value': N / ms_moe_model * 1e3, 'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'spin_up_ms': SPIN_UP_MS,
        'ms_per_step': ms_moe_model, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16',
        'data': 'synthetic',
        'config': {'workload': f'gpt2_small: whole model forward, 12 blocks, {B}x{T}={N} token ids, MoE FFN 128 experts x 24 '
                               f'(gelu, biases), router 768->128->128, module tau={args.tau}; one step = one model forward'},
        'moe_layers_ms': ms_moe_layers, 'moe_share_of_model': ms_moe_layers / ms_moe_model,
        'dense_model_ms': ms_dense_model, 'dense_ffn_layer_ms': ms_dense_ffn, 'per_layer': per_layer,
        'literal_rule': {'rule': f'keep norm >= {args.tau}*max', 'model_ms': ms_lit_model, 'tokens_per_s': N / ms_lit_model * 1e3,
                         'moe_layers_ms': ms_lit_layers,
                         'mean_active_experts': sum(lit_k.values()) / max(len(lit_k), 1)},
        'roofline': {'bound': 'mfma', 'kernel': 'experts (first MoE layer, its real input and routing)',
                     'achieved': active / ms_experts / 1e9, 'peak': PEAK_BF16_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': active / ms_experts / 1e9 / PEAK_BF16_TFLOPS, 'traffic': None, 'kernel_ms': ms_experts},
    }
    return line


def run_gpt2(args, dev):
    print(json.dumps(gpt2_record(args, dev)))


def run_vit(args, dev):
    """Whole-model workload: ViT-B/16 (12 blocks, D = 768, 12 heads, 197 tokens per image) with every FFN replaced by a
    MoE layer of 128 experts x 24 neurons (GELU, biases) and a 768 -> 128 -> 128 router; 256 images = 50432 tokens per
    layer; bf16; random weights.  Attention, LayerNorm, patch embedding and head are stock PyTorch."""
    from d2dmoe_amd import add_routers, gpt2, vit
    torch.manual_seed(0)
    dense = vit.VisionTransformer().eval().to(dev).to(torch.bfloat16)
    moe, names = gpt2.replace_with_moes(dense, num_experts=128, experts_class='hip_kernel')
    gpt2.split_original_parameters(dense, moe, names)
    add_routers(moe, dict(width=128, depth=2, bias=False, activation='relu', output_activation='abs'))
    moe = moe.to(dev).to(torch.bfloat16)
    layers = [gpt2.get_module_by_name(moe, n) for n in names]
    B = 256
    x = torch.randn(B, 3, 224, 224, generator=torch.Generator().manual_seed(1)).to(dev).to(torch.bfloat16)
    N = B * 197

    def measure(tau):
        ks = {}
        for layer in layers:
            layer.forward_mode, layer.tau = 'dynk_max', tau
            layer.experts.forward_mode = 'hip'
        hooks = [layer.register_forward_hook(lambda m, inp, out, n=n: ks.__setitem__(n, out[1][n][0].float().sum(-1).mean().item()))
                 for n, layer in zip(names, layers)]
        moe(x)
        for h in hooks:
            h.remove()
        torch.cuda.synchronize()
        return time_events(lambda: moe(x), args.steps, args.warmup), sum(ks.values()) / len(ks)

    ms_moe, k_moe = measure(args.tau)
    ms_lit, k_lit = measure(1.0 - args.tau)
    ms_dense = time_events(lambda: dense(x), args.steps, args.warmup)
    xin = torch.randn(B, 197, 768, generator=torch.Generator().manual_seed(2)).to(dev).to(torch.bfloat16)
    ms_dense_ffn = time_events(lambda: dense.encoder.layers[0].mlp(xin), args.steps, args.warmup)
    line = {
        'metric': 'MoE-FFN tokens/s + active TFLOP/s & HBM GB/s vs roofline, ViT-B layer tau=0.9',
        'value': N / ms_moe * 1e3, 'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'spin_up_ms': SPIN_UP_MS,
        'ms_per_step': ms_moe, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16',
        'data': 'synthetic',
        'config': {'workload': f'vit_b_model: whole ViT-B/16 forward, 12 blocks, {B} images x 197 tokens = {N} tokens per layer, '
                               f'MoE FFN 128 experts x 24 (gelu, biases), router 768->128->128, module tau={args.tau}; '
                               f'one step = one model forward', 'mean_active_experts': k_moe},
        'images_per_s': B / ms_moe * 1e3, 'dense_model_ms': ms_dense, 'dense_ffn_layer_ms': ms_dense_ffn,
        'literal_rule': {'rule': f'keep norm >= {args.tau}*max', 'model_ms': ms_lit, 'images_per_s': B / ms_lit * 1e3,
                         'mean_active_experts': k_lit},
        'roofline': {'bound': 'mfma', 'kernel': 'see workload vit_b_50k (the same layer shape and token count)', 'achieved': None,
                     'peak': PEAK_BF16_TFLOPS, 'unit': 'TFLOP/s', 'frac': None, 'traffic': None},
    }
    print(json.dumps(line))


def run_norms(args, ops, dev):
    """Router-training targets: the L2 norm of every expert's output for every token (ViT-B layer, 256 x 197 tokens),
    by the HIP kernel and, beside it, by the reference's route on the same GPU (masked-mode stubs + vector_norm over
    the [E,N,D] outputs).  One step = one pass over the batch."""
    from d2dmoe_amd import HipKernelExperts
    torch.manual_seed(0)
    B, T, D, E, Ed = 256, 197, 768, 128, 24
    N = B * T
    ex = HipKernelExperts(D, E, 2, Ed, 'without_last', torch.nn.ReLU).to(dev).bfloat16()
    ex.b1.normal_(0.0, 0.1)
    x = torch.randn(N, D, generator=torch.Generator().manual_seed(1)).bfloat16().to(dev)

    def stubs():
        h = ex.intermediate_activation_extraction_stub(x.unsqueeze(0), ex.w1, ex.b1, ex.act)
        return torch.linalg.vector_norm(ex.output_activation_extraction_stub(h, ex.w2), ord=2, dim=-1)

    ms = time_events(lambda: ex.output_norms(x), args.steps, args.warmup)
    ms_stubs = time_events(stubs, 3, 1)
    executed = N * E * 2.0 * D * 32          # first product with experts padded to 32 neurons
    useful = N * E * 2.0 * D * Ed
    traffic, traffic_src = measured_traffic('vit_b_50k_norms')
    line = {
        'metric': 'MoE-FFN tokens/s + active TFLOP/s & HBM GB/s vs roofline, ViT-B layer tau=0.9',
        'value': N / ms * 1e3, 'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'spin_up_ms': SPIN_UP_MS,
        'ms_per_step': ms, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'bf16',
        'data': 'synthetic',
        'config': {'workload': f'vit_b_50k_norms: per-expert output norms (router-training targets), {B}x{T}={N} tokens, '
                               f'D={D}, {E} experts x {Ed}, relu; one step = norms [E,N] of one batch'},
        'reference_route_ms': ms_stubs,
        'roofline': {'bound': 'mfma', 'kernel': 'expert_norms_kernel', 'achieved': useful / ms / 1e9, 'peak': PEAK_BF16_TFLOPS,
                     'unit': 'TFLOP/s', 'frac': useful / ms / 1e9 / PEAK_BF16_TFLOPS, 'traffic': traffic, 'traffic_source': traffic_src,
                     'kernel_ms': ms, 'executed_tflops': executed / ms / 1e9},
    }
    print(json.dumps(line))


def cpu_baseline(D, E, Ed, W, act, tau, budget_s=16.0):
    """The oracle's restatement of the reference CPU path (router -> dynk_max gate -> per-expert loop), float32,
    8 x 197 tokens of the same layer shape, under both readings of the threshold number: the module's (keep norm >=
    (1 - tau) * max, the headline's) and the literal one (keep norm >= tau * max, i.e. module tau 1 - tau).  Each is
    repeated until its half of budget_s seconds has been spent."""
    from oracle import d2dmoe_oracle as O
    threads = os.cpu_count() or 1
    threads = min(threads, 16)   # the box's CPU share for one GPU
    torch.set_num_threads(threads)
    p = O.make_layer_params(D, E, Ed, W, seed=0)
    x = torch.randn(8, 197, D, generator=torch.Generator().manual_seed(1))

    def timed(module_tau, budget):
        with torch.no_grad():
            _, gating, _ = O.moe_layer_forward(x, p, module_tau, act, 'naive')
            times = []
            t_start = time.perf_counter()
            while (time.perf_counter() - t_start < budget and len(times) < 400) or len(times) < 3:
                t0 = time.perf_counter()
                O.moe_layer_forward(x, p, module_tau, act, 'naive')
                times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2], len(times), gating.float().sum(-1).mean().item()

    med, reps, k = timed(tau, budget_s / 2)
    med_lit, reps_lit, k_lit = timed(1.0 - tau, budget_s / 2)
    return dict(value=8 * 197 / med, unit='tokens/s', cores=threads, kind='port',
                sample=f'8x197=1576 tokens of the same layer (D={D}, {E}x{Ed} experts), float32, module tau={tau} '
                       f'({k:.1f} experts per token), {reps} repetitions, median {med * 1e3:.1f} ms per pass',
                literal_rule=dict(value=8 * 197 / med_lit, unit='tokens/s', rule=f'keep norm >= {tau}*max',
                                  sample=f'the same 1576 tokens, module tau={1.0 - tau:.2f} ({k_lit:.1f} experts per token), '
                                         f'{reps_lit} repetitions, median {med_lit * 1e3:.1f} ms per pass'))


def compact_gated(line):
    """The fields of a gated workload's line that matter inside another line."""
    keep = {'workload': line['config']['workload'], 'ms_per_step': line['ms_per_step'],
            'ms_per_step_eager_launches': line['ms_per_step_eager_launches'],
            'ms_per_step_graph_replay': line['ms_per_step_graph_replay'], 'tokens_per_s': line['value'],
            'mean_active_experts': line['config']['mean_active_experts'],
            'experts_routed_to': line['config']['experts_routed_to'], 'roofline': line['roofline']}
    if 'literal_rule' in line:
        keep['literal_rule'] = line['literal_rule']
    return keep


def skew_norms(N, E, dtype, dev):
    """Norms that bypass the router: |randn| * w_e with w_e = rank_e^-1.2 over a random ranking of the experts."""
    g = torch.Generator().manual_seed(2)
    ranks = torch.randperm(E, generator=g).float() + 1.0
    wts = ranks ** -1.2
    return (torch.randn(N, E, generator=g).abs() * (wts / wts.max())).to(dtype).to(dev)


def regime_roofline(r, N, peak, traffic_row=None):
    """The experts call of one regime against both ceilings: active-pair FLOPs over the MFMA peak and the layer's
    algorithmic bytes over the HBM peak; the bound named is the one the larger fraction belongs to.  traffic_row: the row
    of profiles/traffic_per_launch.md that holds the counter traffic of this regime's kernels, if there is one."""
    f_mfma = r['active_tflops_kernel'] / peak
    f_hbm = r['algo_bytes'] / r['ms_experts'] / 1e6 / PEAK_HBM_GBPS
    traffic, traffic_src = measured_traffic(traffic_row) if traffic_row else (None, None)
    if f_mfma >= f_hbm:
        return {'bound': 'mfma', 'achieved': r['active_tflops_kernel'], 'peak': peak, 'unit': 'TFLOP/s', 'frac': f_mfma,
                'traffic': traffic, 'traffic_source': traffic_src, 'kernel_ms': r['ms_experts']}
    return {'bound': 'hbm', 'achieved': r['algo_bytes'] / r['ms_experts'] / 1e6, 'peak': PEAK_HBM_GBPS, 'unit': 'GB/s',
            'frac': f_hbm, 'traffic': traffic, 'traffic_source': traffic_src, 'kernel_ms': r['ms_experts']}


def skew_record(args, ops, dev, steps, warmup):
    """vit_b_skew inside the default line: both readings of the threshold number on the skewed norms."""
    B, T, D, E, Ed, W, act = WORKLOADS['vit_b_skew']
    N = B * T
    p = make_params(D, E, Ed, W, seed=0, dtype=torch.bfloat16, device=dev)
    x = torch.randn(N, D, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
    packed = ops.pack_weights(ops.make_shape(N, D, E, Ed, W, ops._dtype_code(x), act), p['w1'], p['b1'], p['w2'], None,
                              p['router_w1'], p['router_w2'])
    norms_in = skew_norms(N, E, torch.bfloat16, dev)
    rec = {'workload': f'vit_b_skew: {N} tokens, D={D}, {E} experts x {Ed}, {act}, norms |randn| * rank^-1.2 in place of the router'}
    for key, thr in (('module_tau', 1.0 - args.tau), ('literal_rule', args.tau)):
        r = run_regime(ops, x, p, packed, float(thr), act, steps, warmup, D, E, Ed, W, norms_in=norms_in)
        rec[key] = {'keep_norm_ge_frac_of_max': round(thr, 4), 'ms_per_step': r['ms_layer'], 'tokens_per_s': r['tokens_per_s'],
                    'mean_active_experts': r['mean_active'], 'p99_active_experts': r['p99_active'],
                    'expert_load_max_over_mean': r['expert_load_max_over_mean'],
                    'roofline': regime_roofline(r, N, PEAK_BF16_TFLOPS, 'vit_b_skew' if key == 'module_tau' else 'vit_b_skew_literal')}
    return rec


def router_driven_record(args, ops, dev, name, steps, warmup):
    """One of the other ungated layer shapes inside the default line (router-driven, both readings of the threshold)."""
    B, T, D, E, Ed, W, act = WORKLOADS[name]
    N = B * T
    p = make_params(D, E, Ed, W, seed=0, dtype=torch.bfloat16, device=dev)
    x = torch.randn(N, D, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
    packed = ops.pack_weights(ops.make_shape(N, D, E, Ed, W, ops._dtype_code(x), act), p['w1'], p['b1'], p['w2'], None,
                              p['router_w1'], p['router_w2'])
    rec = {'workload': f'{name}: {B}x{T}={N} tokens, D={D}, {E} experts x {Ed}, {act}, router {D}->{W}->{E}, whole layer',
           'dense_mlp_ms': dense_mlp_ms(x, D, E * Ed, act, steps, warmup)}
    for key, thr in (('module_tau', 1.0 - args.tau), ('literal_rule', args.tau)):
        r = run_regime(ops, x, p, packed, float(thr), act, steps, warmup, D, E, Ed, W)
        rec[key] = {'keep_norm_ge_frac_of_max': round(thr, 4), 'ms_per_step': r['ms_layer'], 'tokens_per_s': r['tokens_per_s'],
                    'mean_active_experts': r['mean_active'], 'router_select_ms': r['ms_router'],
                    'roofline': regime_roofline(r, N, PEAK_BF16_TFLOPS, name if key == 'module_tau' else name + '_literal')}
    return rec


def reference_shape_record(ops, dev, steps, warmup):
    """The shape and sweep of the reference's own micro-benchmark (scripts/test_moe_implementations.py:109-142, 214-285):
    hidden 768, 24 experts x 128 neurons, ReLU, 256 x 197 tokens; the router's output is overridden by Bernoulli(k_frac)
    draws and the layer runs dynk_max with tau = 0.99, so a token keeps exactly the experts that drew 1 (every expert
    when a token drew none: all norms equal the maximum 0).  The draws enter through norms_in."""
    B, T, D, E, Ed, W, act = 256, 197, 768, 24, 128, 128, 'relu'
    N = B * T
    p = make_params(D, E, Ed, W, seed=0, dtype=torch.bfloat16, device=dev)
    x = torch.randn(N, D, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
    packed = ops.pack_weights(ops.make_shape(N, D, E, Ed, W, ops._dtype_code(x), act), p['w1'], p['b1'], p['w2'], None,
                              p['router_w1'], p['router_w2'])
    rows = []
    for k_frac in (1.0, 0.5, 0.3, 0.2, 0.1):
        g = torch.Generator().manual_seed(int(k_frac * 100))
        norms_in = (torch.rand(N, E, generator=g) < k_frac).to(torch.bfloat16).to(dev)
        r = run_regime(ops, x, p, packed, 0.01, act, steps, warmup, D, E, Ed, W, norms_in=norms_in)
        rows.append({'k_frac': k_frac, 'ms_per_step': r['ms_layer'], 'tokens_per_s': r['tokens_per_s'],
                     'mean_active_experts': r['mean_active'], 'roofline': regime_roofline(r, N, PEAK_BF16_TFLOPS)})
    dense_ms = dense_mlp_ms(x, D, E * Ed, act, steps, warmup)
    # float16 storage (the reference script times float32 and float16, :223-228): the same kernels on the other 16-bit type
    p16 = {k: v.to(torch.float16) for k, v in p.items()}
    x16 = x.to(torch.float16)
    packed16 = ops.pack_weights(ops.make_shape(N, D, E, Ed, W, ops._dtype_code(x16), act), p16['w1'], p16['b1'], p16['w2'],
                                None, p16['router_w1'], p16['router_w2'])
    rows16 = []
    for k_frac in (1.0, 0.1):
        g = torch.Generator().manual_seed(int(k_frac * 100))
        norms_in = (torch.rand(N, E, generator=g) < k_frac).to(torch.float16).to(dev)
        r = run_regime(ops, x16, p16, packed16, 0.01, act, steps, warmup, D, E, Ed, W, norms_in=norms_in)
        rows16.append({'k_frac': k_frac, 'ms_per_step': r['ms_layer'], 'tokens_per_s': r['tokens_per_s'],
                       'mean_active_experts': r['mean_active']})
    return {'workload': f'reference micro-benchmark shape: {B}x{T}={N} tokens, D={D}, {E} experts x {Ed}, {act}, bf16, '
                        f'Bernoulli(k_frac) router override, tau=0.99', 'dense_mlp_ms': dense_ms, 'rows': rows,
            'rows_float16': rows16}


def main():
    global SPIN_UP_MS
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--workload', default='vit_b_50k', choices=sorted(WORKLOADS) + sorted(GATED_WORKLOADS) + ['gpt2_small', 'vit_b_50k_norms', 'vit_b_model'])
    ap.add_argument('--tau', type=float, default=0.9, help='module tau (keep expert when norm >= (1 - tau) * max)')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-sweep', action='store_true', help='skip the threshold sweep (5 values x 2 readings)')
    ap.add_argument('--no-sub-records', action='store_true',
                    help='skip the other workloads the default line carries (gemma_1/16/4096, vit_b_skew, reference shape)')
    ap.add_argument('--path', default='auto', choices=['auto', 'mfma_dense', 'mfma_sparse', 'mfma_mid', 'generic'],
                    help='force the experts path of the ungated workloads (default: the library chooses)')
    ap.add_argument('--quantile-iters', type=int, default=200,
                    help='per-call timed launches of the experts kernel for median / 2.5 %% / 97.5 %% (0 = skip)')
    ap.add_argument('--spin-up-ms', type=float, default=SPIN_UP_MS,
                    help='milliseconds of untimed load ahead of every timed region, before its warm-up steps (0 = none)')
    ap.add_argument('--copy-probe', action='store_true',
                    help='also run a plain 512 MiB device copy (calibrates FETCH_SIZE / WRITE_SIZE counter units)')
    args = ap.parse_args()
    SPIN_UP_MS = args.spin_up_ms
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py: this path is single-GPU (tokens are independent; nothing is exchanged); run with --gpus 1',
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print('bench.py: no GPU visible', file=sys.stderr)
        sys.exit(1)
    from d2dmoe_amd import ops
    dev = torch.device('cuda:0')
    if args.copy_probe:
        # one elementwise kernel that reads 512 MiB and writes 512 MiB
        src = torch.zeros(128 << 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    if args.workload in GATED_WORKLOADS:
        with torch.no_grad():
            run_gated(args, ops, dev)
        return
    if args.workload == 'gpt2_small':
        with torch.no_grad():
            run_gpt2(args, dev)
        return
    if args.workload == 'vit_b_model':
        with torch.no_grad():
            run_vit(args, dev)
        return
    if args.workload == 'vit_b_50k_norms':
        with torch.no_grad():
            run_norms(args, ops, dev)
        return
    B, T, D, E, Ed, W, act = WORKLOADS[args.workload]
    N = B * T
    f32 = args.workload.endswith('_f32')
    f16 = args.workload.endswith('_f16')
    dtype = torch.float32 if f32 else (torch.float16 if f16 else torch.bfloat16)
    peak = PEAK_F32_TFLOPS if f32 else PEAK_BF16_TFLOPS
    p = make_params(D, E, Ed, W, seed=0, dtype=dtype, device=dev)
    x = torch.randn(N, D, generator=torch.Generator().manual_seed(1)).to(dtype).to(dev)
    shape = ops.make_shape(N, D, E, Ed, W, ops._dtype_code(x), act)
    packed = ops.pack_weights(shape, p['w1'], p['b1'], p['w2'], None, p['router_w1'], p['router_w2'])
    traffic, traffic_src = measured_traffic(args.workload)
    norms_in = skew_norms(N, E, dtype, dev) if args.workload == 'vit_b_skew' else None
    with torch.no_grad():
        main_r = run_regime(ops, x, p, packed, float(1.0 - args.tau), act, args.steps, args.warmup, D, E, Ed, W,
                            path=args.path, quantile_iters=args.quantile_iters, norms_in=norms_in)
        lit_r = run_regime(ops, x, p, packed, float(args.tau), act, args.steps, args.warmup, D, E, Ed, W, path=args.path,
                           norms_in=norms_in)
        sweep = []
        if not args.no_sweep:
            # the threshold number under both readings
            for v in (0.5, 0.8, 0.9, 0.95, 0.99):
                for rule, thr in (('module_tau', 1.0 - v), ('literal', v)):
                    r = run_regime(ops, x, p, packed, float(thr), act, max(args.steps // 5, 5), 3, D, E, Ed, W, path=args.path,
                                   norms_in=norms_in)
                    sweep.append({'v': v, 'rule': rule, 'keep_norm_ge_frac_of_max': round(thr, 4), 'ms_per_step': r['ms_layer'],
                                  'tokens_per_s': r['tokens_per_s'], 'mean_active_experts': r['mean_active'],
                                  'p99_active_experts': r['p99_active'], 'active_tflops': r['active_tflops_layer']})
        dense_ms = dense_mlp_ms(x, D, E * Ed, act, args.steps, args.warmup)
        ceil = measured_ceilings(dev)
        cold = None
        if norms_in is None and not f32:
            cold = cold_regime(ops, x, p, packed, float(1.0 - args.tau), act, args.steps, args.warmup, D, E, Ed, path=args.path)
    line = {
        'metric': 'MoE-FFN tokens/s + active TFLOP/s & HBM GB/s vs roofline, ViT-B layer tau=0.9',
        'value': main_r['tokens_per_s'], 'unit': 'tokens/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'spin_up_ms': SPIN_UP_MS,
        'ms_per_step': main_r['ms_layer'], 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32' if f32 else ('f16' if f16 else 'bf16'), 'data': 'synthetic',
        'config': {'workload': f'{args.workload}: {B}x{T}={N} tokens, D={D}, {E} experts x {Ed}, {act}, router {D}->{W}->{E}, '
                               f'module tau={args.tau} (keep norm >= {1 - args.tau:.2f}*max), whole layer',
                   'mean_active_experts': main_r['mean_active'], 'p99_active_experts': main_r['p99_active'],
                   'mfma_kernels': packed is not None, 'experts_path': args.path},
        'ms_per_step_eager_launches': main_r['ms_layer_eager'], 'ms_per_step_single_call_graph': main_r['ms_layer_single'],
        'graph_calls_per_replay': min(args.steps, GRAPH_CALLS_MAX),
        'active_tflops': main_r['active_tflops_layer'], 'hbm_gbps': main_r['hbm_gbps_layer'],
        'roofline': {'bound': 'mfma', 'kernel': 'experts', 'achieved': main_r['active_tflops_kernel'],
                     'peak': peak, 'unit': 'TFLOP/s', 'frac': main_r['active_tflops_kernel'] / peak,
                     'traffic': traffic, 'traffic_source': traffic_src, 'kernel_ms': main_r['ms_experts'],
                     'kernel_quantiles': main_r['experts_quantiles'], 'router_select_ms': main_r['ms_router'],
                     'frac_of_library_gemm': main_r['active_tflops_kernel'] / ceil['library_gemm_bf16_8192_tflops']},
        'measured_ceilings': ceil,
        'dense_mlp_ms': dense_ms,
        'expert_load_max_over_mean': main_r['expert_load_max_over_mean'],
        'literal_rule': {'rule': f'keep norm >= {args.tau}*max', 'tokens_per_s': lit_r['tokens_per_s'],
                         'ms_per_step': lit_r['ms_layer'], 'mean_active_experts': lit_r['mean_active'],
                         'p99_active_experts': lit_r['p99_active'], 'active_tflops': lit_r['active_tflops_layer'],
                         'roofline': {'bound': 'hbm', 'achieved': lit_r['hbm_gbps_layer'], 'peak': PEAK_HBM_GBPS,
                                      'unit': 'GB/s', 'frac': lit_r['hbm_gbps_layer'] / PEAK_HBM_GBPS,
                                      'algorithmic_bytes': lit_r['algo_bytes'], 'kernel_ms': lit_r['ms_experts']}},
        'sweep': sweep,
    }
    if cold is not None:
        # warm = the figures above (one set of operands, which the caches keep between steps)
        pairs_flops = cold['mean_pairs'] * 4.0 * D * Ed
        cold['tokens_per_s'] = N / cold['ms_per_step'] * 1e3
        cold['frac'] = pairs_flops / cold['kernel_ms'] / 1e9 / peak
        line['roofline']['cold'] = cold
    if args.workload == 'vit_b_50k' and args.path == 'auto' and not args.no_sub_records:
        # the other workloads this library is measured on, each with its own roofline, so that one run shows them all
        del x, p, packed
        sub_steps, sub_warmup = max(args.steps // 2, 10), max(args.warmup // 2, 3)
        sub = {}
        with torch.no_grad():
            saved = args.steps, args.warmup
            args.steps, args.warmup = sub_steps, sub_warmup
            for w in ('gemma_1', 'gemma_16', 'gemma_4096'):
                sub[w] = compact_gated(gated_record(args, ops, dev, w))
            args.steps, args.warmup = saved
            sub['vit_b_skew'] = skew_record(args, ops, dev, sub_steps, sub_warmup)
            sub['reference_shape'] = reference_shape_record(ops, dev, sub_steps, sub_warmup)
            for w in ('gpt2_medium_layer', 'vit_b_24x128'):
                sub[w] = router_driven_record(args, ops, dev, w, sub_steps, sub_warmup)
            # the GPT-2-small configuration in short: the whole GPT-2-small forward with MoE FFNs (few steps: a step is 7 ms)
            saved = args.steps, args.warmup
            args.steps, args.warmup = max(saved[0] // 5, 5), 2
            g = gpt2_record(args, dev)
            args.steps, args.warmup = saved
            sub['gpt2_small'] = {'workload': g['config']['workload'], 'model_ms': g['ms_per_step'], 'tokens_per_s': g['value'],
                                 'dense_model_ms': g['dense_model_ms'], 'moe_layers_ms': g['moe_layers_ms'],
                                 'dense_ffn_layer_ms': g['dense_ffn_layer_ms'],
                                 'mean_active_experts': sum(r['mean_active_experts'] for r in g['per_layer']) / len(g['per_layer']),
                                 'literal_rule': g['literal_rule'], 'roofline': g['roofline']}
        line['sub_records'] = sub
    if not args.no_cpu_baseline:
        line['cpu_baseline'] = cpu_baseline(D, E, Ed, W, act, args.tau)
    print(json.dumps(line))


if __name__ == '__main__':
    main()
