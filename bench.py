"""
Benchmark of the float8 linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one forward+backward pass of the OLMo-2-7B-shape SwiGLU feed-forward block
(d_model 4096, hidden 11008, tokens M = 16384 = batch 4 x seq 4096) with all three projections float8
tensorwise (e4m3 forward operands, e5m2 grad_output), synthetic seeded inputs resident in HBM.
Prints ONE JSON line: whole-step throughput in TFLOP/s (2*M*N*K per GEMM, 9 GEMMs per step), the
roofline of the dominant kernel (the fp8 GEMM, timed with HIP events on its launch stream during the
timed region) and the CPU baseline (the oracle's emulated float8 path on the host cores, on a bounded
sample of the same workload).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

D_MODEL, HIDDEN, TOKENS = 4096, 11008, 16384
FP8_MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense fp8 matrix peak
GEMMS_PER_STEP = 9
TRAFFIC_PROFILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "gemm_fp8_m16_kernel__mlp7b_traffic_pmc.txt")


def gemm_traffic_bytes_per_launch():
    """HBM-side bytes per GEMM launch (L2 fills + write-backs, mean over the GEMM work of a step), taken from the
    line `traffic_bytes_per_launch: N` of the FETCH_SIZE / WRITE_SIZE counter summary under profiles/ (a figure from
    rocprofv3 --pmc runs, not measured by this script); None when that file is missing."""
    try:
        for line in open(TRAFFIC_PROFILE):
            if line.startswith("traffic_bytes_per_launch:"):
                return float(line.split(":")[1].split()[0])
    except OSError:
        pass
    return None


def build_mlp(dev):
    from olmo_core_amd.float8 import AOFloat8LinearRecipe, Float8Config
    from olmo_core_amd.nn import FeedForward

    g = torch.Generator().manual_seed(1002)
    mlp = FeedForward(d_model=D_MODEL, hidden_size=HIDDEN, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        for p in mlp.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(torch.bfloat16))
    mlp = mlp.to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(mlp)
    x = torch.randn(TOKENS, D_MODEL, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
    go = (torch.randn(TOKENS, D_MODEL, generator=g) * 1e-3).to(torch.bfloat16).to(dev)
    return mlp, x, go


# ---- the other benchmark configurations (parity-test shapes; measured with --config N) ----


def build_config(n, dev, keep_float8_weights=False, routed=False, compile_model=False, recommended=False):
    """Returns (step_fn, flops_per_step, gemms_per_step, flops_per_gemm_launch or None, description).
    Configurations 2 and 4 only: `compile_model` runs the block through torch.compile (the mode the reference's training
    scripts run every block in); `recommended` converts with AOFloat8LinearConfig.recommended() (what those scripts
    set: power-of-two scales, float8 weights kept between weight updates) instead of the plain tensorwise recipe, and
    the timed steps are then micro-batches between two optimizer steps: no weight is quantised inside them.
    Configuration 5 only: `keep_float8_weights` keeps the experts' float8 weight copies from step to step (the
    steady state of gradient-accumulation micro-batches; by default every step quantises the weights again, as a
    step that follows an optimizer update must); `routed` times the whole routed layer (token gather fused into
    the quantisation, experts, weighted scatter back to token order) instead of the experts alone."""
    from olmo_core_amd.float8 import AOFloat8LinearRecipe, Float8Config
    from olmo_core_amd.float8.linear import float8_projections
    from olmo_core_amd.nn import DroplessMoEMLP, FeedForward, ParallelDroplessMLP

    def rand(shape, g, std=1.0):
        return (torch.randn(shape, generator=g) * std).to(torch.bfloat16)

    if n == 1:
        g = torch.Generator().manual_seed(0)
        x = rand((2048, 4096), g).to(dev)
        lin = torch.nn.Linear(4096, 11008, bias=False, dtype=torch.bfloat16)
        with torch.no_grad():
            lin.weight.copy_(rand((11008, 4096), g, 0.02))
        seq = torch.nn.Sequential(lin).to(dev)
        Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(seq)

        def fn():
            with torch.no_grad():
                seq(x)

        f = 2.0 * 2048 * 4096 * 11008
        return fn, f, 1, f, "config 1: one Float8Linear forward 2048x4096 -> 11008, tensorwise"
    if n in (2, 4):
        d, h, m, seed = (4096, 11008, 16384, 1002) if n == 2 else (5120, 27648, 8192, 1004)
        g = torch.Generator().manual_seed(seed)
        mlp = FeedForward(d_model=d, hidden_size=h, bias=False, dtype=torch.bfloat16)
        with torch.no_grad():
            for p in mlp.parameters():
                p.copy_(rand(p.shape, g, 0.02))
        mlp = mlp.to(dev)
        if recommended:
            from olmo_core_amd.float8 import AOFloat8LinearConfig

            Float8Config(ao=AOFloat8LinearConfig.recommended()).apply_float8_linear(mlp)
        else:
            Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(mlp)
        params = list(mlp.parameters())
        run = torch.compile(mlp) if compile_model else mlp
        x = torch.randn(m, d, generator=g)
        if n == 4:  # 0.1 % of the entries x100
            pos = torch.randperm(m * d, generator=g)[: m * d // 1000]
            x.view(-1)[pos] *= 100
        x = x.to(torch.bfloat16).to(dev).requires_grad_(True)
        go = rand((m, d), g, 1e-3).to(dev)
        f = 2.0 * m * d * h
        name = "OLMo-2-7B" if n == 2 else "OLMo-2-32B (0.1 % outliers x100)"
        desc = f"config {n}: {name} SwiGLU MLP fwd+bwd, tokens {m}, tensorwise"
        if recommended:
            desc += ", AOFloat8LinearConfig.recommended() (float8 weights kept between weight updates: micro-batch steady state)"
        if compile_model:
            desc += ", block under torch.compile"

        def fn_mlp():
            x.grad = None
            for p in params:
                p.grad = None
            run(x).backward(go)

        return fn_mlp, 9 * f, 9, f, desc
    if n == 3:
        g = torch.Generator().manual_seed(1003)
        m, d = 16384, 4096
        mods = torch.nn.ModuleList([torch.nn.Linear(d, d, bias=False, dtype=torch.bfloat16) for _ in range(4)])
        with torch.no_grad():
            for p in mods.parameters():
                p.copy_(rand(p.shape, g, 0.02))
        mods = mods.to(dev)
        Float8Config(ao_recipe=AOFloat8LinearRecipe.rowwise).apply_float8_linear(mods)
        # q, k and v are applied to one tensor, as in the attention block (float8_projections: one quantisation of
        # x, grad_x summed by the GEMM epilogues); the output projection has an input of its own
        x = rand((m, d), g).to(dev).requires_grad_(True)
        x_o = rand((m, d), g).to(dev).requires_grad_(True)
        go = rand((m, d), g, 1e-3).to(dev)

        def fn():
            x.grad = x_o.grad = None
            for lin in mods:
                lin.weight.grad = None
            ys = list(float8_projections(x, *mods[:3])) + [mods[3](x_o)]
            torch.autograd.backward(ys, [go] * 4)

        f = 2.0 * m * d * d
        return fn, 12 * f, 12, f, ("config 3: OLMo-3-7B q/k/v/o projections fwd+bwd, tokens 16384, rowwise recipe "
                                   "(q, k, v on one input, o on another)")
    if n == 5:
        g = torch.Generator().manual_seed(1005)
        E, d, h, T, top_k = 64, 2048, 1024, 16384, 8
        rank = torch.arange(1, E + 1, dtype=torch.float64)
        pmf = rank ** -1.1
        pmf = pmf / pmf.sum()
        logits = torch.randn(T, E, generator=g) + (1.75 * torch.log(pmf)).float()  # Zipf(s=1.1) bias: 7 of 64 experts get no token
        weights, experts = logits.float().softmax(-1).topk(top_k, dim=-1)
        idx = experts.reshape(-1)
        sizes = torch.bincount(idx, minlength=E)
        mlp = DroplessMoEMLP(d_model=d, hidden_size=h, num_experts=E, dtype=torch.bfloat16,
                             keep_float8_weights=keep_float8_weights)
        with torch.no_grad():
            for p in mlp.parameters():
                p.copy_(rand(p.shape, g, 0.02))
        mlp = mlp.to(dev)
        sizes_d = sizes.to(dev)
        f = float(T * top_k) * 18 * d * h
        desc = (f"config 5: dropless MoE experts fwd+bwd, 64 experts, {T * top_k} rows, group sizes min {int(sizes.min())} "
                f"max {int(sizes.max())} empty {int((sizes == 0).sum())}, grouped rowwise")
        if keep_float8_weights:
            desc += ", float8 expert weights kept across steps"
        if routed:
            layer = ParallelDroplessMLP(mlp=mlp, top_k=top_k)
            x = rand((T, d), g).to(dev).requires_grad_(True)
            go = rand((T, d), g, 1e-3).to(dev)
            w_d = weights.to(torch.bfloat16).to(dev).requires_grad_(True)
            experts_d = experts.to(dev)

            def fn_routed():
                x.grad = w_d.grad = None
                for p in mlp.parameters():
                    p.grad = None
                layer(x, w_d, experts_d, sizes_d).backward(go)

            return fn_routed, f, 9, None, desc + f"; whole routed layer from {T} tokens (sort, fused gather, experts, weighted scatter)"
        x = rand((T * top_k, d), g).to(dev).requires_grad_(True)
        go = rand((T * top_k, d), g, 1e-3).to(dev)

        def fn():
            x.grad = None
            for p in mlp.parameters():
                p.grad = None
            mlp(x, sizes_d).backward(go)

        return fn, f, 9, None, desc
    raise ValueError(n)


def measure_config(n, steps, warmup, **kw):
    """One line for configuration n: `warmup` untimed steps, `steps` timed ones between two device synchronisations."""
    dev = torch.device("cuda:0")
    fn, flops, _, _, desc = build_config(n, dev, **kw)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    del fn
    torch.cuda.empty_cache()
    return {"config": desc, "ms_per_step": round(ms, 4), "TFLOP/s": round(flops / ms / 1e9, 1),
            "pct_fp8_mfma_peak": round(100 * flops / ms / 1e9 / FP8_MFMA_PEAK_TFLOPS, 2), "steps": steps}


def run_other_config(n, steps, warmup, **kw):
    print(json.dumps(measure_config(n, steps, warmup, **kw)), flush=True)


def other_configs(steps=8, warmup=3):
    """The other benchmark configurations and the headline block's other modes, one line each (a failure is reported
    in its line and does not stop the rest)."""
    cases = (
        (1, {}), (3, {}), (4, {}), (5, {}), (5, {"keep_float8_weights": True}),
        (2, {"compile_model": True}), (2, {"recommended": True}),
    )
    lines = []
    for n, kw in cases:
        try:
            lines.append(measure_config(n, steps, warmup, **kw))
        except Exception as e:  # noqa: BLE001
            lines.append({"config": f"config {n} {kw}", "error": f"{type(e).__name__}: {e}"[:300]})
    return lines


def gemm_shapes(shapes, steps, warmup):
    """One line per shape: a single e4m3 x e4m3 GEMM with bf16 output and single scales, the kernel chosen by the
    library (few rows: the weight-streaming kernel; few tiles: split K; otherwise the tiled kernels)."""
    from olmo_core_amd.float8 import ops

    dev = torch.device("cuda:0")
    one = torch.ones(1, device=dev)
    g = torch.Generator().manual_seed(7)
    for (m, n, k) in shapes:
        a = torch.randn(m, k, generator=g).to(torch.float8_e4m3fn).to(dev)
        b = torch.randn(n, k, generator=g).to(torch.float8_e4m3fn).to(dev)
        for _ in range(warmup):
            ops.gemm_fp8(a, one, b, one)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(steps):
            ops.gemm_fp8(a, one, b, one)
        end.record()
        torch.cuda.synchronize()
        us = start.elapsed_time(end) / steps * 1e3
        print(json.dumps({"gemm": f"{m}x{n}x{k}", "us_per_call": round(us, 2), "TFLOP/s": round(2.0 * m * n * k / us / 1e6, 1),
                          "operand_GB/s": round((m * k + n * k + 2 * m * n) / us / 1e3, 1), "steps": steps}), flush=True)


HBM_PEAK_GBS = 8000.0


def cast_rates(iters: int = 10):
    """The HBM-bound half of the path, outside the timed region: the fused tensorwise cast (amax pass, then one pass
    that writes the row-major and the transposed fp8 copy) of the step's largest activation, h [tokens, hidden] bf16.
    Algorithmic bytes per element: 4 (2 read, 1 + 1 written); as the two passes stream it: 6 (the amax pass
    reads x once more)."""
    from olmo_core_amd.float8 import ops

    dev = torch.device("cuda:0")
    h = torch.randn(TOKENS, HIDDEN, device=dev, dtype=torch.bfloat16)
    n = h.numel()

    def run():
        slots = ops.amax_partials(h)
        ops.cast_tensorwise(h, torch.float8_e4m3fn, want_rowmajor=True, want_transposed=True, slots=slots)

    for _ in range(3):
        run()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        run()
    end.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(end) / iters * 1e3
    # as the step runs them: the producers leave the amax (of h) or the codes it follows from (of g1, g3), so each
    # tensor is read once
    slots = ops.amax_partials(h)
    us_h = _time_us(lambda: ops.cast_tensorwise(h, torch.float8_e4m3fn, want_rowmajor=True, want_transposed=True, slots=slots), iters)
    x1 = torch.randn(TOKENS, HIDDEN, device=dev, dtype=torch.bfloat16)
    gh = (torch.randn(TOKENS, HIDDEN, device=dev) * 1e-3).to(torch.bfloat16)
    gc, xc = ops.rowseg_max_codes(gh), ops.rowseg_max_codes(x1, h)
    us_g = _time_us(lambda: ops.swiglu_bwd_cast(x1, h, gh, torch.float8_e5m2, want_transposed=True, codes=(gc, xc)), iters)
    in_step = {
        "h (amax from the producing GEMM): tile_cast_kernel, 4 B/elem": {
            "us": round(us_h, 1), "GB/s_algorithmic": round(4.0 * n / us_h / 1e3, 1), "frac_hbm_peak_algorithmic": round(4.0 * n / us_h / 1e3 / HBM_PEAK_GBS, 4)},
        "g1, g3 (amax from row-segment codes): sparse amax + swiglu_bwd_cast_kernel, 10 B/elem": {
            "us": round(us_g, 1), "GB/s_algorithmic": round(10.0 * n / us_g / 1e3, 1), "frac_hbm_peak_algorithmic": round(10.0 * n / us_g / 1e3 / HBM_PEAK_GBS, 4)},
    }
    del x1, gh, gc, xc
    return {
        "as_run_in_the_step": in_step,
        "tensor": f"{TOKENS}x{HIDDEN} bf16 -> e4m3 row-major + transposed, tensorwise (amax pass + cast pass)",
        "us": round(us, 1),
        "GB/s_algorithmic_4B_per_elem": round(4.0 * n / us / 1e3, 1),
        "GB/s_streamed_6B_per_elem": round(6.0 * n / us / 1e3, 1),
        "frac_hbm_peak_algorithmic": round(4.0 * n / us / 1e3 / HBM_PEAK_GBS, 4),
        "frac_hbm_peak_streamed": round(6.0 * n / us / 1e3 / HBM_PEAK_GBS, 4),
    }


def _time_us(fn, iters=10, warmup=3):
    for _ in range(warmup):
        fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters * 1e3


def cast_table():
    """The HBM-bound kernels of the path one by one at the benchmark's shapes: one JSON line each with the time, the
    rate on the algorithmic bytes (what any implementation must move: inputs read once, outputs written once) and on
    the bytes the kernel streams (a second read of the input where a global amax separates two passes), and the
    fractions of the 8 TB/s HBM peak."""
    from olmo_core_amd import _C
    from olmo_core_amd.float8 import ops

    dev = torch.device("cuda:0")
    e4m3, e5m2 = torch.float8_e4m3fn, torch.float8_e5m2

    def line(kernel, shape, us, alg_bytes, streamed_bytes):
        print(json.dumps({
            "kernel": kernel, "shape": "x".join(map(str, shape)), "us": round(us, 1),
            "GB/s_algorithmic": round(alg_bytes / us / 1e3, 1), "frac_hbm_peak_algorithmic": round(alg_bytes / us / 1e3 / HBM_PEAK_GBS, 3),
            "GB/s_streamed": round(streamed_bytes / us / 1e3, 1), "frac_hbm_peak_streamed": round(streamed_bytes / us / 1e3 / HBM_PEAK_GBS, 3),
        }), flush=True)

    for shape in ((TOKENS, D_MODEL), (HIDDEN, D_MODEL), (TOKENS, HIDDEN)):
        n = shape[0] * shape[1]
        x = torch.randn(*shape, device=dev).to(torch.bfloat16)
        y = torch.empty_like(x)
        line("device copy (torch), for scale", shape, _time_us(lambda: y.copy_(x)), 4 * n, 4 * n)
        del y
        line("amax_partials_kernel", shape, _time_us(lambda: ops.amax_partials(x)), 2 * n, 2 * n)
        slots = ops.amax_partials(x)
        line("tile_cast_kernel (scale known): row-major + transposed", shape,
             _time_us(lambda: ops.cast_tensorwise(x, e4m3, want_transposed=True, slots=slots)), 4 * n, 4 * n)
        line("tile_cast_kernel (scale known): row-major only", shape,
             _time_us(lambda: ops.cast_tensorwise(x, e4m3, slots=slots)), 3 * n, 3 * n)
        line("tensorwise cast, fused amax + cast passes: row-major + transposed", shape,
             _time_us(lambda: ops.cast_tensorwise(x, e4m3, want_transposed=True)), 4 * n, 6 * n)
        line("rowwise_cast_kernel (single pass)", shape, _time_us(lambda: ops.cast_rowwise(x, e4m3, pow2=True)), 3 * n, 3 * n)
        line("colamax + per-column transposed cast", shape, _time_us(lambda: ops.cast_colwise_t(x, e4m3, pow2=True)), 3 * n, 5 * n)
        line("two-product cast (per-row copy + per-column transposed copy)", shape,
             _time_us(lambda: ops.cast_rows_and_colwise_t(x, e4m3, pow2=True)), 4 * n, 6 * n)
        del x, slots
    shape = (TOKENS, HIDDEN)
    n = shape[0] * shape[1]
    x1 = torch.randn(*shape, device=dev).to(torch.bfloat16)
    x3 = torch.randn(*shape, device=dev).to(torch.bfloat16)
    gh = (torch.randn(*shape, device=dev) * 1e-3).to(torch.bfloat16)
    line("swiglu_fwd_kernel (+ amax of h)", shape, _time_us(lambda: ops.swiglu_fwd(x1, x3)), 6 * n, 6 * n)
    s1 = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=dev)
    s3 = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    line("swiglu_bwd_kernel, amax-only pass", shape,
         _time_us(lambda: _C.lib().mi8_swiglu_bwd(x1.data_ptr(), x3.data_ptr(), gh.data_ptr(), None, None, n, s1.data_ptr(),
                                                  s3.data_ptr(), st)), 6 * n, 6 * n)
    line("swiglu backward to float8 (amax pass + swiglu_bwd_cast_kernel): g1, g3 row-major + transposed", shape,
         _time_us(lambda: ops.swiglu_bwd_cast(x1, x3, gh, e5m2, want_transposed=True)), 10 * n, 16 * n)
    # the route the feed-forward block takes: the producers of x1, x3 and gh leave row-segment codes, and the amax comes
    # from the few segments that can hold it
    gc, xc = ops.rowseg_max_codes(gh), ops.rowseg_max_codes(x1, x3)
    line("amax of g1, g3 from row-segment codes (three sparse launches)", shape,
         _time_us(lambda: ops.swiglu_bwd_amax_from_codes(x1, x3, gh, gc, xc)), 6 * n, 4 * (n // 64))
    line("swiglu backward to float8 (amax from codes + swiglu_bwd_cast_kernel): g1, g3 row-major + transposed", shape,
         _time_us(lambda: ops.swiglu_bwd_cast(x1, x3, gh, e5m2, want_transposed=True, codes=(gc, xc))), 10 * n, 10 * n)
    h = torch.randn(*shape, device=dev).to(torch.bfloat16)
    hs = ops.amax_partials(h)
    line("tensorwise cast of h with the amax from the GEMM that wrote it: row-major + transposed (= tile_cast_kernel)", shape,
         _time_us(lambda: ops.cast_tensorwise(h, e4m3, want_rowmajor=True, want_transposed=True, slots=hs)), 4 * n, 4 * n)
    del x1, x3, gh, h
    # grouped (configuration 5): 131072 routed rows of 2048, the benchmark's group sizes
    _, _, _, _, desc = build_config(5, dev)
    g = torch.Generator().manual_seed(1005)
    E, T, top_k, d = 64, 16384, 8, 2048
    rank = torch.arange(1, E + 1, dtype=torch.float64)
    pmf = rank ** -1.1
    pmf = pmf / pmf.sum()
    logits = torch.randn(T, E, generator=g) + (1.75 * torch.log(pmf)).float()
    experts = logits.float().softmax(-1).topk(top_k, dim=-1).indices
    sizes = torch.bincount(experts.reshape(-1), minlength=E).to(dev)
    indices = torch.sort(experts.reshape(-1).int(), stable=True)[1].int().to(dev)
    xs = torch.randn(T * top_k, d, device=dev).to(torch.bfloat16)
    n = xs.numel()
    line("grouped two-product cast (grouped_colamax + grouped_tile_cast), 64 ragged groups", (T * top_k, d),
         _time_us(lambda: ops.grouped_cast_rows_and_colwise_t(xs, sizes, e4m3, pow2=True)), 4 * n, 6 * n)
    del xs
    xt = torch.randn(T, d, device=dev).to(torch.bfloat16)
    line("token gather fused into the grouped two-product cast (top-8 of 16384 tokens)", (T * top_k, d),
         _time_us(lambda: ops.gather_cast_rows_and_colwise_t(xt, indices, top_k, sizes, e4m3, pow2=True)),
         2 * xt.numel() + 2 * n, 2 * xt.numel() + 2 * n)


def feed_probe():
    """What feeding operands costs a stream of MFMAs (mi8_probe_mfma_feed): shader cycles per 64-MFMA iteration, the
    clock the chip held, and the rate, for the pieces of a GEMM K step one at a time and together."""
    from olmo_core_amd import _C

    dev = torch.device("cuda:0")
    sink = torch.empty(256 * 256, dtype=torch.float32, device=dev)
    window = torch.zeros((2 << 20) + (128 << 10), dtype=torch.uint8, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    iters = 20000
    flop = 256 * 4 * iters * 2.0 * 128 ** 3
    cases = (
        (0, 0, 0, 0, "MFMAs only"),
        (0, 0, 0, 2, "MFMAs, two barriers"),
        (0, 0, 32, 0, "+ 32 LDS fragment reads (ds_read_b128)"),
        (0, 8, 0, 0, "+ 8 direct-to-LDS loads (global_load_lds_dwordx4)"),
        (0, 16, 0, 0, "+ 16 direct-to-LDS loads"),
        (0, 16, 0, 2, "+ 16 direct-to-LDS loads, two barriers"),
        (0, 16, 32, 0, "+ 16 direct-to-LDS loads + 32 LDS reads"),
        (0, 16, 32, 1, "+ 16 direct-to-LDS loads + 32 LDS reads, one barrier"),
        (0, 16, 32, 2, "+ 16 direct-to-LDS loads + 32 LDS reads, two barriers: the GEMM's K step"),
        (1, 16, 0, 0, "+ 16 loads to registers (global_load_dwordx4)"),
        (2, 16, 0, 0, "+ 16 LDS stores of resident registers (ds_write_b128)"),
        (3, 16, 0, 0, "+ 16 loads to registers and 16 LDS stores, interleaved"),
        (3, 16, 32, 2, "+ 16 loads to registers, 16 LDS stores, 32 LDS reads, two barriers"),
    )
    for rnd in (0, 1):
        for kind, loads, reads, barriers, name in cases:
            def run():
                _C.check_diag(_C.diag().mi8_probe_mfma_feed(kind, loads, reads, barriers, rnd, iters, window.data_ptr(), sink.data_ptr(),
                                                      clocks.data_ptr(), st))
            us = _time_us(run, iters=2, warmup=1)
            cyc, ticks = (int(v) for v in clocks.tolist())
            print(json.dumps({"probe": "64 MFMAs 16x16x128 per wave and iteration " + name, "operands": "random bytes" if rnd else "zeros",
                              "cycles_per_iteration": round(cyc / iters, 1), "clock_MHz": round(cyc / (ticks / 100.0), 0),
                              "TFLOP/s": round(flop / us / 1e6, 1)}), flush=True)


def store_probe():
    """What a compute unit's store path takes (mi8_probe_store_rate): cycles per 16-byte-per-lane store instruction and wave,
    and bytes per clock and compute unit, by lane pattern, waves per compute unit and number of compute units storing."""
    from olmo_core_amd import _C

    dev = torch.device("cuda:0")
    pitch = HIDDEN * 2
    window = torch.empty(16384 * pitch + 4096, dtype=torch.uint8, device=dev)
    cycles = torch.zeros(256 * 4, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    iters = 64
    for workgroups in (256, 8):
        for rows, waves in ((8, 4), (4, 4), (16, 4), (2, 4), (8, 2), (8, 1), (4, 1)):
            for _ in range(3):
                _C.check_diag(_C.diag().mi8_probe_store_rate(rows, waves, workgroups, iters, window.data_ptr(), pitch, cycles.data_ptr(), st))
            torch.cuda.synchronize()
            c = cycles.view(256, 4)[:workgroups, :waves].float()
            per = c.mean().item() / (iters * 8)
            print(json.dumps({"probe": f"global_store_dwordx4 stream, {rows} rows x {1024 // rows} B per instruction",
                              "compute_units_storing": workgroups, "waves_per_compute_unit": waves,
                              "cycles_per_store_and_wave": round(per, 1), "max": round(c.max().item() / (iters * 8), 1),
                              "bytes_per_clock_and_compute_unit": round(waves * 1024 / per, 1)}), flush=True)


def tile_timeline(shapes):
    """Where the cycles of a GEMM tile go (mi8_diag_gemm_tile_timeline: the library's persistent kernel built with time
    stamps): per shape and operand content, the mean shader-clock cycles of the K loop, of a K step, of the epilogue and
    of its passes over all tiles of all workgroups, the clock the chip held, and the duration of the stamped launch next
    to the product's own launch of the same GEMM."""
    from olmo_core_amd import _C
    from olmo_core_amd.float8 import ops

    E4M3 = torch.float8_e4m3fn
    dev = torch.device("cuda:0")
    one = torch.ones(1, device=dev)
    stamps = torch.zeros(256 * 256, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    for (m, n, k) in shapes:
        for kind in ("N(0,1)", "zeros"):
            if kind == "zeros":
                a = torch.zeros(m, k, device=dev).to(E4M3); b = torch.zeros(n, k, device=dev).to(E4M3)
            else:
                a = torch.randn(m, k, device=dev).to(E4M3); b = torch.randn(n, k, device=dev).to(E4M3)
            out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
            us_product = _time_us(lambda: ops.gemm_fp8(a, one, b, one, out=out), iters=5, warmup=4)
            ref = out.clone()

            def run():
                _C.check_diag(_C.diag().mi8_diag_gemm_tile_timeline(a.data_ptr(), one.data_ptr(), b.data_ptr(), one.data_ptr(), out.data_ptr(),
                                                              m, n, k, 0, 0, stamps.data_ptr(), st))
            us_stamped = _time_us(run, iters=5, warmup=2)
            assert torch.equal(out, ref), "the stamped kernel must produce the product kernel's bits"
            t = stamps.cpu().view(256, 256).to(torch.int64) & 0xFFFFFFFF
            ev = t[:, :13 * 16].view(256, 16, 13)
            used = ev[:, :, 0] != 0
            d = lambda i, j: ((ev[:, :, j] - ev[:, :, i]) & 0xFFFFFFFF)[used].double()
            ticks = ((t[:, 255] - t[:, 254]) & 0xFFFFFFFF)[used.any(1)].double()           # 100 MHz
            first = ev[:, 0, 0]
            last = torch.stack([ev[w, int(used[w].sum()) - 1, 12] if used[w].any() else first[w] for w in range(256)])
            span = ((last - first) & 0xFFFFFFFF)[used.any(1)].double()
            nk = k // 128
            passes = [round(d(3 + i, 4 + i).mean().item()) for i in range(7)]
            print(json.dumps({"gemm": f"{m}x{n}x{k}", "operands": kind, "us_product_kernel": round(us_product, 1),
                              "us_stamped_kernel_incl_two_synchronisations": round(us_stamped, 1),
                              "tiles_per_workgroup": [int(used.sum(1).min()), int(used.sum(1).max())],
                              "clock_MHz": round((span / (ticks / 100.0)).mean().item()),
                              "cycles": {"k_loop": round(d(0, 2).mean().item()), "per_k_step": round(d(0, 2).mean().item() / nk, 1),
                                         "first_three_k_steps": round(d(0, 1).mean().item()) if nk > 3 else None,
                                         "epilogue": round(d(2, 12).mean().item()), "epilogue_min_max": [int(d(2, 12).min().item()), int(d(2, 12).max().item())],
                                         "start_to_first_pass_staged": round(d(2, 3).mean().item()), "pass_to_pass": passes,
                                         "last_pass_staged_to_last_store_issued": round(d(10, 11).mean().item()),
                                         "refill_of_fragments": round(d(11, 12).mean().item())},
                              "epilogue_share_of_tile": round(d(2, 12).mean().item() / (d(0, 12).mean().item()), 4),
                              "mfma_floor_cycles_per_k_step": 2048}), flush=True)


def power_probe():
    """What the power limit leaves of the matrix peak: back-to-back MFMAs with nothing else running, and the
    benchmark's longest-K GEMM, each on all-zero and on random operands (under `rocprofv3 --pmc GRBM_GUI_ACTIVE` the
    kernel durations and active cycles give the clock in each case)."""
    from olmo_core_amd import _C
    from olmo_core_amd.float8 import ops

    dev = torch.device("cuda:0")
    sink = torch.empty(256 * 256, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    iters = 20000
    flop = 256 * 4 * iters * 2.0 * 128 ** 3
    for shape, name in ((1, "16x16x128"), (0, "32x32x64")):
        for rnd in (0, 1):
            us = _time_us(lambda: _C.check_diag(_C.diag().mi8_probe_mfma_loop(shape, rnd, iters, 256, sink.data_ptr(), st)), iters=3, warmup=1)
            print(json.dumps({"probe": f"bare v_mfma_f32_{name}_f8f6f4 loop, 256 workgroups x 4 waves",
                              "operands": "random bytes" if rnd else "zeros", "ms": round(us / 1e3, 2),
                              "TFLOP/s": round(flop / us / 1e6, 1), "frac_of_5.0_PFLOP/s": round(flop / us / 1e6 / FP8_MFMA_PEAK_TFLOPS, 3)}), flush=True)
    one = torch.ones(1, device=dev)
    for (m, n, k) in ((TOKENS, D_MODEL, HIDDEN), (TOKENS, HIDDEN, D_MODEL)):
        for rnd in (0, 1):
            if rnd:
                a = torch.randn(m, k, device=dev).to(torch.float8_e4m3fn)
                b = torch.randn(n, k, device=dev).to(torch.float8_e4m3fn)
            else:
                a = torch.zeros(m, k, device=dev, dtype=torch.float8_e4m3fn)
                b = torch.zeros(n, k, device=dev, dtype=torch.float8_e4m3fn)
            us = _time_us(lambda: ops.gemm_fp8(a, one, b, one), iters=20, warmup=5)
            print(json.dumps({"probe": f"gemm_fp8_m16_kernel {m}x{n}x{k}", "operands": "N(0,1) cast to e4m3" if rnd else "zeros",
                              "us": round(us, 1), "TFLOP/s": round(2.0 * m * n * k / us / 1e6, 1),
                              "frac_of_5.0_PFLOP/s": round(2.0 * m * n * k / us / 1e6 / FP8_MFMA_PEAK_TFLOPS, 3)}), flush=True)
            del a, b


def profile_summary(path):
    """Print the per-kernel table of a `rocprofv3 --kernel-trace --stats --output-format csv` run (its
    *_kernel_stats.csv) in the compact form kept under profiles/."""
    import csv
    import glob

    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "**", "*kernel_stats.csv"), recursive=True))
    if not files:
        print(f"no *kernel_stats.csv under {path}", file=sys.stderr)
        sys.exit(2)
    rows = list(csv.DictReader(open(files[0])))
    total = sum(float(r["TotalDurationNs"]) for r in rows)
    print(f"{'kernel':100s} {'calls':>6s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s} {'total_ms':>9s} {'pct':>6s}")
    for r in rows:
        t = float(r["TotalDurationNs"])
        if t < 0.001 * total:
            continue
        name = " ".join(r["Name"].split())
        name = name.replace("(anonymous namespace)::", "").replace("mi8::gemm::", "").replace("mi8::", "")
        print(f"{name[:100]:100s} {int(r['Calls']):6d} {float(r['AverageNs']) / 1e3:9.2f} {float(r['MinNs']) / 1e3:9.2f} "
              f"{float(r['MaxNs']) / 1e3:9.2f} {t / 1e6:9.3f} {100 * t / total:6.2f}")
    print(f"(kernels below 0.1 % of the {total / 1e6:.3f} ms of GPU time are left out)")


def traffic_probe():
    """Workload for the rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE, matrix-pipe counters): a plain 256 MiB device
    copy (the calibration: 268435456 bytes read and written per launch), then three steps of the benchmark's
    feed-forward block, nothing timed."""
    dev = torch.device("cuda:0")
    src = torch.randint(0, 255, (1 << 28,), dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst
    mlp, x, go = build_mlp(dev)
    for _ in range(3):
        step(mlp, x, go)
    torch.cuda.synchronize()
    print("traffic probe done", flush=True)


def counter_summary(path):
    """Per kernel and counter: dispatches, mean counter value and mean duration of a `rocprofv3 --pmc ... --kernel-trace
    --output-format csv` run (its *_counter_collection.csv)."""
    import csv
    import glob
    from collections import defaultdict

    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True))
    if not files:
        print(f"no *counter_collection.csv under {path}", file=sys.stderr)
        sys.exit(2)
    acc = defaultdict(lambda: [0, 0.0, 0.0])
    for r in csv.DictReader(open(files[0])):
        name = " ".join(r["Kernel_Name"].split())
        name = name.replace("(anonymous namespace)::", "").replace("mi8::gemm::", "").replace("mi8::", "")
        if len(name) > 90:
            name = name[:87] + "..."
        key = (name, int(r["Grid_Size"]), r["Counter_Name"])
        a = acc[key]
        a[0] += 1
        a[1] += float(r["Counter_Value"])
        a[2] += (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
    print(f"{'kernel':90s} {'grid':>9s} {'counter':28s} {'n':>4s} {'mean value':>16s} {'mean us':>9s}")
    for (name, grid, counter), (n, v, us) in sorted(acc.items(), key=lambda kv: -kv[1][2]):
        if us / n < 5.0:
            continue
        print(f"{name:90s} {grid:9d} {counter:28s} {n:4d} {v / n:16.1f} {us / n:9.1f}")
    print("(kernels shorter than 5 us are left out)")


def gemm_compare(shapes, reps=4):
    """Workload for counter runs that put this library's GEMM beside hipBLASLt's (through torch._scaled_mm) on the same
    operands: per shape, on all-zero and on N(0,1) operands, `reps` calls of each (the first of each is a warm-up).
    Under `rocprofv3 --kernel-trace [--pmc ...] --output-format csv`, --counter-cases prints one row per case from the
    dispatch order; without a profiler the calls are timed with events."""
    from olmo_core_amd.float8 import ops

    dev = torch.device("cuda:0")
    one = torch.ones(1, device=dev)
    e4m3 = torch.float8_e4m3fn
    for (m, n, k) in shapes:
        for rnd in (0, 1):
            if rnd:
                a = torch.randn(m, k, device=dev).to(e4m3)
                b = torch.randn(n, k, device=dev).to(e4m3)
            else:
                a = torch.zeros(m, k, device=dev, dtype=e4m3)
                b = torch.zeros(n, k, device=dev, dtype=e4m3)
            torch.cuda.synchronize()
            for name, fn in (("mi8_gemm_fp8", lambda: ops.gemm_fp8(a, one, b, one)),
                             ("hipBLASLt (torch._scaled_mm)", lambda: torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16))):
                us = _time_us(fn, iters=reps - 1, warmup=1)
                print(json.dumps({"case": f"{m}x{n}x{k} {'random' if rnd else 'zeros'} {name}", "calls": reps, "us": round(us, 1),
                                  "TFLOP/s": round(2.0 * m * n * k / us / 1e6, 1)}), flush=True)
            del a, b


def counter_cases(path, group=4):
    """The GEMM dispatches of a --gemm-compare run in dispatch order, `group` consecutive dispatches of one kernel per
    case (the first of each group is the warm-up and is left out): kernel, mean duration and mean of every counter."""
    import csv
    import glob
    from collections import OrderedDict

    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True))
    trace = None
    if not files:
        files = sorted(glob.glob(os.path.join(path, "**", "*kernel_trace.csv"), recursive=True))
        trace = True
    if not files:
        print(f"no *counter_collection.csv or *kernel_trace.csv under {path}", file=sys.stderr)
        sys.exit(2)
    disp = OrderedDict()
    for r in csv.DictReader(open(files[0])):
        name = " ".join(r["Kernel_Name"].split())
        if "gemm_fp8" not in name and "Cijk" not in name:
            continue
        d = disp.setdefault(int(r["Dispatch_Id"]), {"name": name, "us": (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3, "c": {}})
        if not trace:
            d["c"][r["Counter_Name"]] = d["c"].get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    rows = [disp[k] for k in sorted(disp)]
    counters = sorted({c for d in rows for c in d["c"]})
    print(f"{'#':>3s} {'kernel':44s} {'us':>8s} " + " ".join(f"{c[:22]:>22s}" for c in counters))
    i = case = 0
    while i < len(rows):
        j = i
        while j < len(rows) and j - i < group and rows[j]["name"] == rows[i]["name"]:
            j += 1
        use = rows[i + 1:j] if j - i > 1 else rows[i:j]
        name = rows[i]["name"].replace("(anonymous namespace)::", "").replace("mi8::gemm::", "").replace("void ", "")
        us = sum(d["us"] for d in use) / len(use)
        vals = " ".join(f"{sum(d['c'].get(c, 0.0) for d in use) / len(use):22.0f}" for c in counters)
        print(f"{case:3d} {name[:44]:44s} {us:8.1f} {vals}")
        case += 1
        i = j


def step(mlp, x, go):
    x.grad = None
    for p in mlp.parameters():
        p.grad = None
    y = mlp(x)
    y.backward(go)


def cpu_baseline(target_seconds: float = 15.0):
    """The oracle's emulated path (fp32 matmul on dequantised fp8 operands) on the host cores, MLP fwd+bwd at
    a reduced token count chosen to take about `target_seconds`."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from oracle import float8_oracle as O

    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or os.cpu_count() or 1
    cores = min(cores, os.cpu_count() or cores)
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(1002)
    w1 = (torch.randn(HIDDEN, D_MODEL, generator=g) * 0.02).bfloat16()
    w2 = (torch.randn(D_MODEL, HIDDEN, generator=g) * 0.02).bfloat16()
    w3 = (torch.randn(HIDDEN, D_MODEL, generator=g) * 0.02).bfloat16()
    spec = O.recipe("tensorwise")

    def run(m):
        x = torch.randn(m, D_MODEL, generator=g).bfloat16()
        go = (torch.randn(m, D_MODEL, generator=g) * 1e-3).bfloat16()
        t0 = time.perf_counter()
        O.mlp_fwd_bwd(x, w1, w2, w3, go, spec)
        return time.perf_counter() - t0

    probe_m = 1024
    run(256)  # warm the thread pool
    t_probe = run(probe_m)
    m = int(min(TOKENS, max(probe_m, probe_m * target_seconds / max(t_probe, 1e-3))))
    m = max(256, (m // 256) * 256)
    t = run(m) if m != probe_m else t_probe
    flops = GEMMS_PER_STEP * 2.0 * m * D_MODEL * HIDDEN
    return {
        "value": round(flops / t / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"oracle emulated float8 MLP fwd+bwd (fp32 torch-CPU matmul), {m} of {TOKENS} tokens, {t:.1f} s, same weights shape",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--config", type=int, default=2, help="benchmark configuration 1..5 (2 is the headline line)")
    ap.add_argument("--keep-float8-weights", action="store_true",
                    help="config 5: keep the experts' float8 weight copies across steps (micro-batch steady state)")
    ap.add_argument("--routed", action="store_true",
                    help="config 5: time the whole routed layer (fused gather, experts, weighted scatter)")
    ap.add_argument("--compile", action="store_true", help="configs 2, 4: run the block through torch.compile")
    ap.add_argument("--recommended", action="store_true",
                    help="configs 2, 4: convert with AOFloat8LinearConfig.recommended() (float8 weights kept between updates)")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the other configurations after the headline")
    ap.add_argument("--cast-table", action="store_true", help="time every HBM-bound kernel of the path at the benchmark's shapes")
    ap.add_argument("--power-probe", action="store_true", help="bare MFMA loops and the GEMM on zero / random operands")
    ap.add_argument("--feed-probe", action="store_true", help="an MFMA stream with the loads and LDS reads of a GEMM K step beside it")
    ap.add_argument("--store-probe", action="store_true", help="streams of 16-byte stores in the layout of a GEMM output tile: cycles per store, bytes per clock")
    ap.add_argument("--tile-timeline", type=str, default=None, metavar="M,N,K;...", help="shader-clock cycles of the K loop, the epilogue and its passes per tile of the persistent GEMM")
    ap.add_argument("--profile-summary", type=str, default=None, metavar="DIR_OR_CSV",
                    help="print the per-kernel table of a rocprofv3 --stats --output-format csv run (no GPU needed)")
    ap.add_argument("--counter-summary", type=str, default=None, metavar="DIR_OR_CSV",
                    help="print per-kernel means of a rocprofv3 --pmc --output-format csv run (no GPU needed)")
    ap.add_argument("--traffic-probe", action="store_true", help="workload for the rocprofv3 --pmc counter runs (a calibration copy, then three benchmark steps)")
    ap.add_argument("--gemm-compare", type=str, default=None, metavar="M,N,K[;M,N,K...]",
                    help="this library's GEMM and hipBLASLt's on the same zero / random operands (workload for counter runs)")
    ap.add_argument("--counter-cases", type=str, default=None, metavar="DIR_OR_CSV",
                    help="per-case table of a rocprofv3 run of --gemm-compare (no GPU needed)")
    ap.add_argument("--gemm", type=str, default=None, metavar="M,N,K[;M,N,K...]",
                    help="time single scaled GEMMs of these shapes (library's choice of kernel) instead of a step")
    ns = ap.parse_args()
    if ns.profile_summary:
        profile_summary(ns.profile_summary)
        return
    if ns.counter_summary:
        counter_summary(ns.counter_summary)
        return
    if ns.counter_cases:
        counter_cases(ns.counter_cases)
        return
    if ns.gpus != 1:
        print("bench.py: this build measures the float8 linear path on ONE GPU; --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the float8 path has no CPU implementation", file=sys.stderr)
        sys.exit(2)

    from olmo_core_amd.float8 import ops

    if ns.traffic_probe:
        traffic_probe()
        return
    if ns.cast_table:
        cast_table()
        return
    if ns.store_probe:
        store_probe()
        return
    if ns.tile_timeline:
        tile_timeline([tuple(int(v) for v in sh.split(",")) for sh in ns.tile_timeline.split(";")])
        return
    if ns.feed_probe:
        feed_probe()
        return
    if ns.power_probe:
        power_probe()
        return
    if ns.gemm_compare:
        gemm_compare([tuple(int(v) for v in part.split(",")) for part in ns.gemm_compare.split(";")])
        return
    if ns.gemm:
        gemm_shapes([tuple(int(v) for v in part.split(",")) for part in ns.gemm.split(";")], ns.steps, ns.warmup)
        return
    if ns.config != 2 or ns.compile or ns.recommended:
        run_other_config(ns.config, ns.steps, ns.warmup, keep_float8_weights=ns.keep_float8_weights, routed=ns.routed,
                         compile_model=ns.compile, recommended=ns.recommended)
        return

    dev = torch.device("cuda:0")
    mlp, x, go = build_mlp(dev)

    for _ in range(ns.warmup):
        step(mlp, x, go)
    torch.cuda.synchronize()

    # GEMM launches are bracketed by HIP events on their stream inside the timed region.  An event pair costs about
    # 10 us of command-processor time between two back-to-back GEMMs (1.3 % of the step when every launch carries
    # one), so the launches of every fourth timed step are sampled (all of them when fewer than 8 steps are timed).
    events = []
    every = 4 if ns.steps >= 8 else 1
    sampled_steps = 0
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(ns.steps):
        sample = i % every == 0
        ops.GEMM_EVENT_SINK = events if sample else None
        sampled_steps += sample
        step(mlp, x, go)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ops.GEMM_EVENT_SINK = None

    ms_per_step = elapsed / ns.steps * 1e3
    flops_per_step = GEMMS_PER_STEP * 2.0 * TOKENS * D_MODEL * HIDDEN
    tflops = flops_per_step / (ms_per_step * 1e-3) / 1e12

    # one event pair per GEMM launch; the fused launch of the two input projections counts as the two GEMMs it is
    gemm_ms = [s.elapsed_time(e) for s, e, _ in events]
    gemm_flops = sum(2.0 * m * n * k for _, _, (m, n, k) in events)
    flops_per_launch = 2.0 * TOKENS * D_MODEL * HIDDEN
    assert abs(gemm_flops - GEMMS_PER_STEP * sampled_steps * flops_per_launch) < 1e-6 * gemm_flops, (gemm_flops, sampled_steps)
    avg_gemm_s = sum(gemm_ms) / (GEMMS_PER_STEP * sampled_steps) * 1e-3  # per 2*M*N*K unit of work
    achieved = flops_per_launch / avg_gemm_s / 1e12

    result = {
        "metric": "Float8Linear fwd+bwd TFLOP/s at 7B MLP shape",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": ns.steps,
        "warmup": ns.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8 (e4m3/e5m2 operands, fp32 accumulate, bf16 out)",
        "data": "synthetic (seeded N(0,1) activations, N(0,0.02) weights, N(0,1e-3) grad_output)",
        "config": {
            "workload": "OLMo-2-7B SwiGLU MLP fwd+bwd, w1/w3 4096->11008, w2 11008->4096, tokens 16384, float8 tensorwise",
            "tokens": TOKENS,
            "d_model": D_MODEL,
            "hidden": HIDDEN,
            "recipe": "tensorwise",
        },
        "pct_fp8_mfma_peak": round(100.0 * tflops / FP8_MFMA_PEAK_TFLOPS, 2),
        "roofline": {
            "kernel": "gemm_fp8_m16_kernel (9 GEMMs of 2*16384*4096*11008 flop per step in 8 launches: the two input projections share one)",
            "bound": "mfma",
            "achieved": round(achieved, 2),
            "peak": FP8_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / FP8_MFMA_PEAK_TFLOPS, 4),
            "traffic": gemm_traffic_bytes_per_launch(),
            "traffic_source": "profiles/gemm_fp8_m16_kernel__mlp7b_traffic_pmc.txt (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; not measured in this run)",
            "avg_launch_us": round(avg_gemm_s * 1e6, 2),
            "gemm_share_of_step": round(sum(gemm_ms) / sampled_steps / ms_per_step, 4),
            "launches_timed": f"{len(gemm_ms)} launches of {sampled_steps} of the {ns.steps} timed steps",
        },
    }
    del mlp, x, go
    result["cast"] = cast_rates()
    # everything of the step that is not a GEMM launch: casts, amax passes, the SwiGLU backward pass
    n_x, n_w, n_h = TOKENS * D_MODEL, HIDDEN * D_MODEL, TOKENS * HIDDEN
    algorithmic = 4 * (2 * n_x + 3 * n_w + n_h) + 10 * n_h  # x, grad_y, three weights, h: 2 B read + 2 copies; g1, g3: 6 read + 4 written
    streamed = algorithmic + 2 * (2 * n_x + 3 * n_w)        # + the separate amax pass over x, grad_y and the weights
    non_gemm_ms = ms_per_step - sum(gemm_ms) / sampled_steps
    result["cast"]["step_totals"] = {
        "what": "all non-GEMM work of one step (casts of x, grad_y, W1, W2, W3, h; SwiGLU backward to float8 of g1, g3; amax passes): step time minus the event-timed GEMM launches",
        "ms": round(non_gemm_ms, 4),
        "algorithmic_GB": round(algorithmic / 1e9, 3),
        "streamed_GB": round(streamed / 1e9, 3),
        "GB/s_algorithmic": round(algorithmic / non_gemm_ms / 1e6, 1),
        "frac_hbm_peak_algorithmic": round(algorithmic / non_gemm_ms / 1e6 / HBM_PEAK_GBS, 4),
        "frac_hbm_peak_streamed": round(streamed / non_gemm_ms / 1e6 / HBM_PEAK_GBS, 4),
    }
    if not ns.no_other_configs:
        result["other_configs"] = other_configs()
    if not ns.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
