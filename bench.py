#!/usr/bin/env python3
"""Benchmark of the llama decoder-layer training step (fwd + loss + bwd) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--no-cpu-baseline] [--other-workloads C1,C3,C4,C5]

Prints ONE JSON line.  A step = one forward + cross-entropy loss + backward of the workload's layer
stack on one micro-batch of synthetic, HBM-resident inputs (random-init weights, seeded token ids);
weight gradients land in fp32 main-grad buffers.  `value` = tokens / second of whole steps (wall clock around exactly K
steps between two device synchronisations); `ms_per_step_median` is the median of the K per-step durations taken with
one event per step boundary on the compute stream in the same pass.
`roofline` describes the dominant kernel (the bf16 MFMA GEMM): its algorithmic FLOPs divided by its
launch durations, taken with events on the launch stream in a second pass of the same K steps (the
events serialise the queue, so the pass that `value` is computed from runs without them).
`cpu_baseline` = the fp32 CPU oracle (a port of the reference math) timed on this host's cores: one whole fwd+bwd step of
the workload where that is a few tens of seconds (C1, C2), else one decoder layer + LM head + loss extrapolated linearly.
`configs` lists the other workloads, measured after the headline figures are taken, each with ms/step, tokens/s, TFLOP/s and
the GEMM kernel's fraction of the MFMA peak.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "fwd+bwd tokens/sec + MFMA util %, 7B-shape llama layer bf16 seq4096, 1 GPU"
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA peak
# HBM-side bytes per GEMM launch (average over the launches of one step), from two rocprofv3 --pmc runs of this script
# (FETCH_SIZE, WRITE_SIZE) scaled by what the same counters read for the streaming kernels of known size in the same
# run (factor 2.0 for FETCH_SIZE, 1.0 for WRITE_SIZE); see profiles/c2_step_gemm_hbm_traffic.txt.
GEMM_HBM_BYTES_PER_LAUNCH = {"C2": 600.9e6}


def cpu_baseline(w, flops):
    """fp32 oracle on the host cores (the thread count the box gives this process: torch's default, i.e. OMP_NUM_THREADS).
    Workloads of up to 3e13 FLOPs per step run one whole fwd+bwd step; larger ones one decoder layer + final norm + LM head
    + loss, with t_step ~= L * t_layer + t_head.  Returns the dict that goes into the JSON line."""
    import torch
    from oracle import llama_oracle as O
    from easyllm_amd import workloads as W
    threads = torch.get_num_threads()
    note = "%d threads (os.cpu_count() = %s)" % (threads, os.cpu_count())
    b, s, h, V, L = w["batch"], w["seq"], w["hidden_size"], w["vocab_size"], w["num_layers"]
    cfg = dict(num_layers=L, hidden_size=h, num_attention_heads=w["num_attention_heads"],
               num_kv_attention_heads=w["num_kv_attention_heads"], head_dim=h // w["num_attention_heads"],
               intermediate_size=w["intermediate_size"], vocab_size=V)
    if flops <= 3e13 and "packed" not in w:
        Wt = {k: v.requires_grad_(True) for k, v in O.init_weights(cfg, seed=1).items()}
        inputs, (labels, loss_mask), _ = W.make_inputs(w)
        t0 = time.perf_counter()
        loss = O.cross_entropy_loss(O.model_forward(Wt, cfg, inputs[0]), labels, loss_mask)
        loss.backward()
        t_step = time.perf_counter() - t0
        return {"value": round(b * s / t_step, 2), "unit": "tokens/s", "cores": threads, "kind": "port",
                "sample": "fp32 CPU oracle, one whole fwd+bwd step of the same workload (%.1f s), %s" % (t_step, note)}
    cfg["num_layers"] = 1
    Wt = {k: v.requires_grad_(True) for k, v in O.init_weights(cfg, seed=1).items()}
    g = torch.Generator().manual_seed(2)
    x = torch.randn(s, b, h, generator=g).requires_grad_(True)
    labels = torch.randint(0, V, (b, s), generator=g)
    t0 = time.perf_counter()
    y = O.decoder_layer(x, Wt, "3.", cfg)
    y.backward(torch.ones_like(y))
    t_layer = time.perf_counter() - t0
    xh = torch.randn(b, s, h, generator=g).requires_grad_(True)
    t0 = time.perf_counter()
    logits = O.linear(O.rmsnorm(xh, Wt["5.weight"]), Wt["6.word_embeddings.weight"])
    loss = O.cross_entropy_loss(logits, labels, torch.ones(b, s))
    loss.backward()
    t_head = time.perf_counter() - t0
    t_step = L * t_layer + t_head
    return {"value": round(b * s / t_step, 2), "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": "fp32 CPU oracle, 1 of %d decoder layers (%.1f s) + final norm/LM head/loss (%.1f s) fwd+bwd at the "
                      "full shape; step time extrapolated as L*t_layer + t_head; %s" % (L, t_layer, t_head, note)}


class GemmTimer:
    """Per-launch timing of the GEMM kernel: while installed, every launch that goes through kernels.gemm or
    kernels.linear_dgrad_multi is bracketed by two events on the launch stream and (flops, start, end) is recorded."""

    def __init__(self, kernels):
        import torch
        self.kernels, self.torch, self.records = kernels, torch, []
        self._gemm, self._multi = kernels.gemm, kernels.linear_dgrad_multi

    def __enter__(self):
        torch = self.torch

        def gemm(A, B, M, N, K, *a, **kw):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            out = self._gemm(A, B, M, N, K, *a, **kw)
            end.record()
            self.records.append((2.0 * M * N * K, start, end))
            return out

        def multi(dy2ds, ws, *a, **kw):
            same = len({dy.stride(0) for dy in dy2ds}) == 1 and len({w.stride(0) for w in ws}) == 1 and len(ws) <= 3
            if not same:  # goes out as one kernels.gemm call per pair, each timed above
                return self._multi(dy2ds, ws, *a, **kw)
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            out = self._multi(dy2ds, ws, *a, **kw)
            end.record()
            self.records.append((2.0 * dy2ds[0].shape[0] * ws[0].shape[1] * sum(w.shape[0] for w in ws), start, end))
            return out

        self.kernels.gemm, self.kernels.linear_dgrad_multi = gemm, multi
        return self

    def __exit__(self, *exc):
        self.kernels.gemm, self.kernels.linear_dgrad_multi = self._gemm, self._multi
        return False


def measure(name, steps, warmup, mode, input_check):
    """Times `steps` fwd + loss + bwd steps of workload `name` (after `warmup` untimed ones) and, in a second pass, its GEMM
    launches.  Returns (figures, model): figures is a flat dict, the model is handed back for the optimizer timing."""
    import torch
    from easyllm_amd import functional, kernels, runner, workloads as W
    dev = torch.device("cuda:0")
    w = W.WORKLOADS[name]
    torch.manual_seed(w["seed"])
    model = runner.build_model({"type": "llama_custom", "kwargs": W.model_kwargs(w)})
    runner.attach_main_grads(model)
    functional.set_input_check(input_check)
    inputs, labels, doc_lens = W.make_inputs(w, device=dev)
    tokens_per_step = w["batch"] * w["seq"]
    flops = W.step_flops(w, doc_lens)

    def step():
        runner.zero_main_grads(model)
        return runner.forward_step(model, inputs, labels)

    def timed(fn, flush):
        """Exactly `steps` calls of fn between two device synchronisations: (last loss, wall seconds, per-step ms from
        one event per step boundary on the compute stream)."""
        events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        events[0].record()
        for i in range(steps):
            last = fn()
            events[i + 1].record()
        flush()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        return last, wall, [events[i].elapsed_time(events[i + 1]) for i in range(steps)]

    for _ in range(warmup):
        loss = step()
    loss, elapsed_eager, per_step = timed(step, functional.flush_input_checks)
    loss_value = float(loss.item())
    elapsed = elapsed_eager
    launch_mode = mode
    if mode == "graph":
        # the same kernels, captured once and replayed: no per-kernel host work, no launch gaps
        try:
            graphed = runner.GraphedStep(model, inputs, labels)
        except Exception as exc:  # capture refused by the runtime: report the eager figures and say so
            graphed = None
            launch_mode = "eager (graph capture failed: %s)" % (str(exc).splitlines()[0][:120] if str(exc) else type(exc).__name__)
            print("bench.py: %s" % launch_mode, file=sys.stderr)
        if graphed is not None:
            for _ in range(warmup):
                graphed()
            loss, elapsed, per_step = timed(graphed, graphed.flush)
            assert float(loss.item()) == loss_value, "graph replay and eager step disagree"
            del graphed
    per_step.sort()
    median_ms = per_step[len(per_step) // 2] if len(per_step) % 2 else 0.5 * (per_step[len(per_step) // 2 - 1] + per_step[len(per_step) // 2])

    # Second pass of the same K steps with every GEMM launch bracketed by two timing events on the launch stream.  The
    # events serialise the queue (about 20 us per launch), so they are kept out of the pass that `value` comes from.
    with GemmTimer(kernels) as timer:
        t1 = time.perf_counter()
        for _ in range(steps):
            step()
        functional.flush_input_checks()
        torch.cuda.synchronize()
        elapsed_instrumented = time.perf_counter() - t1
    timing = timer.records
    gemm_flops = sum(f for f, _, _ in timing)
    gemm_ms = sum(s.elapsed_time(e) for _, s, e in timing)
    ms_per_step = elapsed / steps * 1e3
    fig = dict(workload=w, name=name, tokens_per_step=tokens_per_step, flops=flops, loss=loss_value, launch=launch_mode,
               ms_per_step=ms_per_step, ms_per_step_median=median_ms, eager_ms_per_step=elapsed_eager / steps * 1e3,
               tok_s=tokens_per_step * steps / elapsed, tflops=flops * steps / elapsed / 1e12,
               recomputed_layers=model.recompute_count, gemm_launches=len(timing) // max(steps, 1),
               gemm_tflops=gemm_flops / (gemm_ms * 1e-3) / 1e12 if gemm_ms > 0 else 0.0,
               gemm_avg_launch_us=gemm_ms * 1e3 / max(len(timing), 1), gemm_share=gemm_ms / steps / ms_per_step,
               instrumented_ms_per_step=elapsed_instrumented / steps * 1e3)
    return fig, model


def gemm_vs_library(workload):
    """Every GEMM launch of one training step of `workload`, this library's kernel against the box's own GEMM library
    (torch.matmul / torch.mm -> hipBLASLt), timed alternately in one process on the same operands.  Prints a table and the
    step's total GEMM time under three choices: this kernel everywhere, the library everywhere, the faster of the two per
    launch -- the last is what a step could reach if every launch ran at the better of the two kernels."""
    import torch
    from easyllm_amd import kernels as K, workloads as W
    w = W.WORKLOADS[workload]
    dev = torch.device("cuda:0")
    T, h, f, V, L = w["batch"] * w["seq"], w["hidden_size"], w["intermediate_size"], w["vocab_size"], w["num_layers"]
    d = h // w["num_attention_heads"]
    nq, nk = w["num_attention_heads"] * d, w["num_kv_attention_heads"] * d

    def timeit(fn, n=30, warm=5):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n * 1e3

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, device=dev) * scale).bfloat16()

    def best(a, b):  # each timed twice, alternately; the better run of each
        ta, tb = timeit(a), timeit(b)
        return min(ta, timeit(a)), min(tb, timeit(b))

    rows = []

    def fwd(name, N, Kd, count):
        x, wt = rnd(T, Kd), rnd(N, Kd, scale=0.02)
        rows.append((name + " forward", 2.0 * T * N * Kd, count) + best(lambda: K.linear_fwd(x, wt), lambda: torch.matmul(x, wt.t())))

    def dgrad(name, outs, n_in, count):
        dys, ws = [rnd(T, o) for o in outs], [rnd(o, n_in, scale=0.02) for o in outs]
        dycat, wcat = torch.cat(dys, 1), torch.cat(ws, 0)
        rows.append((name + " input gradient", 2.0 * T * n_in * sum(outs), count) +
                    best(lambda: K.linear_dgrad_multi(dys, ws), lambda: torch.matmul(dycat, wcat)))

    def wgrad(name, N, Kd, count):
        dy, x = rnd(T, N), rnd(T, Kd)
        mg = torch.zeros(N, Kd, device=dev, dtype=torch.float32)
        try:
            torch.mm(dy.t(), x, out_dtype=torch.float32)
            lib, note = (lambda: torch.mm(dy.t(), x, out_dtype=torch.float32)), "fp32 result"
        except Exception:
            lib, note = (lambda: torch.matmul(dy.t(), x)), "library: bf16 result, no fp32-result call here"
        rows.append((name + " weight gradient (%s)" % note, 2.0 * T * N * Kd, count) +
                    best(lambda: K.linear_wgrad(dy, x, out=mg, accumulate=False), lib))

    if nq == nk == h:
        fwd("q/k/v/o", h, h, 4 * L)
        dgrad("q+k+v (one launch)", [h, h, h], h, L)
        dgrad("o", [h], h, L)
        wgrad("q/k/v/o", h, h, 4 * L)
    else:
        fwd("q/o", nq, h, 2 * L)
        fwd("k/v", nk, h, 2 * L)
        dgrad("q+k+v (one launch)", [nq, nk, nk], h, L)
        dgrad("o", [h], nq, L)
        wgrad("q/o", nq, h, 2 * L)
        wgrad("k/v", nk, h, 2 * L)
    fwd("gate/up", f, h, 2 * L)
    fwd("down", h, f, L)
    fwd("head", V, h, 1)
    dgrad("gate+up (one launch)", [f, f], h, L)
    dgrad("down", [h], f, L)
    dgrad("head", [V], h, 1)
    wgrad("gate/up", f, h, 2 * L)
    wgrad("down", h, f, L)
    wgrad("head", V, h, 1)
    print("GEMM launches of one %s step (M = %d tokens), this kernel against the library GEMM of the box" % (workload, T))
    print("%-66s %6s %10s %11s %8s %8s" % ("launch", "count", "this us", "library us", "this TF", "lib TF"))
    ta = tb = tm = fl = 0.0
    for name, flops, count, a, b in rows:
        print("%-66s %6d %10.1f %11.1f %8.0f %8.0f" % (name, count, a, b, flops / a / 1e6, flops / b / 1e6))
        ta, tb, tm, fl = ta + count * a, tb + count * b, tm + count * min(a, b), fl + count * flops
    for label, t in (("this kernel everywhere", ta), ("library everywhere", tb), ("faster of the two per launch", tm)):
        print("GEMM time per step, %-30s %8.3f ms  %6.0f TFLOP/s  %.3f of the bf16 MFMA peak" % (label + ":", t / 1e3, fl / t / 1e6, fl / t / 1e6 / PEAK_BF16_TFLOPS))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--mode", choices=("graph", "eager"), default="graph",
                    help="graph: the step is captured once into a HIP graph and replayed; eager: launched kernel by kernel")
    ap.add_argument("--no-optimizer-step", action="store_true", help="skip the separately timed AdamW + clipping step")
    ap.add_argument("--input-check", choices=("sync", "deferred"), default="deferred",
                    help="token-id range check of the embedding: blocking like the reference, or examined one call late")
    ap.add_argument("--other-workloads", default="C1,C3,C4,C5",
                    help="comma-separated workloads measured after the headline one (fewer steps each) and reported in the "
                         "`configs` array of the same JSON line; empty string to skip")
    ap.add_argument("--other-steps", type=int, default=6)
    ap.add_argument("--gemm-vs-library", action="store_true",
                    help="instead of the benchmark: time every GEMM launch of one step against the box's library GEMM and print a table")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share only (TP=1, one MI355X); --gpus %d is not supported. "
              "Run with --gpus 1." % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from easyllm_amd import workloads as W
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(torch.device("cuda:0"))
    if args.gemm_vs_library:
        gemm_vs_library(args.workload)
        return
    fig, model = measure(args.workload, args.steps, args.warmup, args.mode, args.input_check)
    w = fig["workload"]
    out = {
        "metric": METRIC, "value": round(fig["tok_s"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(fig["ms_per_step"], 3), "ms_per_step_median": round(fig["ms_per_step_median"], 3),
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "%s: %s" % (args.workload, w["desc"]), "tokens_per_step": fig["tokens_per_step"],
                   "fp32_main_grads": True, "recomputed_layers": fig["recomputed_layers"],
                   "input_id_check": args.input_check, "launch": fig["launch"],
                   "eager_ms_per_step": round(fig["eager_ms_per_step"], 3)},
        "tflops": round(fig["tflops"], 1), "mfma_frac_end_to_end": round(fig["tflops"] / PEAK_BF16_TFLOPS, 4),
        "loss": round(fig["loss"], 5),
        "roofline": {"kernel": "gemm_kernel (bf16 MFMA GEMM, %d launches/step)" % fig["gemm_launches"],
                     "bound": "mfma", "achieved": round(fig["gemm_tflops"], 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(fig["gemm_tflops"] / PEAK_BF16_TFLOPS, 4), "traffic": GEMM_HBM_BYTES_PER_LAUNCH.get(args.workload),
                     "avg_launch_us": round(fig["gemm_avg_launch_us"], 2),
                     "share_of_step_time": round(fig["gemm_share"], 4),
                     "measured_in": "second pass of the same %d steps with two timing events per GEMM launch (%.3f ms/step)"
                                    % (args.steps, fig["instrumented_ms_per_step"])},
    }
    if not args.no_optimizer_step:
        # AdamW + global-norm clipping over the same parameters, timed on its own (not part of `value`): per parameter
        # 4 B for the norm pass, 16 B read + 12 B written by the update, 2 B for the refreshed bf16 weight.
        from easyllm_amd import optimizer
        opt = optimizer.build_optimizer({"type": "FusedAdam", "kwargs": {"lr": 2e-5, "weight_decay": 0, "betas": [0.9, 0.95],
                                                                         "eps": 1e-8}}, model)
        nparams = sum(p.numel() for p in model.parameters())
        for _ in range(2):
            opt.step(clip_grad=1.0)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for _ in range(args.steps):
            opt.step(clip_grad=1.0)
        torch.cuda.synchronize()
        opt_ms = (time.perf_counter() - t2) / args.steps * 1e3
        out["optimizer_step"] = {"ms": round(opt_ms, 3), "params": nparams, "bound": "hbm",
                                 "achieved": round(34.0 * nparams / (opt_ms * 1e-3) / 1e9, 1), "peak": 8000.0, "unit": "GB/s",
                                 "frac": round(34.0 * nparams / (opt_ms * 1e-3) / 1e9 / 8000.0, 4)}
        del opt
    del model
    # The other workloads, each with the same procedure and fewer steps: throughput, TFLOP/s of algorithmic work (recompute
    # not counted) and the GEMM kernel's fraction of the MFMA peak.  The headline figures above are complete before these run.
    others = [n for n in args.other_workloads.split(",") if n and n != args.workload]
    if others:
        out["configs"] = []
    for n in others:
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        f, m = measure(n, args.other_steps, 2, args.mode, args.input_check)
        del m
        out["configs"].append({"workload": "%s: %s" % (n, f["workload"]["desc"]), "tokens_per_step": f["tokens_per_step"],
                               "steps": args.other_steps, "warmup": 2, "launch": f["launch"],
                               "ms_per_step": round(f["ms_per_step"], 3), "tokens_per_s": round(f["tok_s"], 1),
                               "tflops": round(f["tflops"], 1), "mfma_frac_end_to_end": round(f["tflops"] / PEAK_BF16_TFLOPS, 4),
                               "recomputed_layers": f["recomputed_layers"], "gemm_tflops": round(f["gemm_tflops"], 1),
                               "gemm_frac": round(f["gemm_tflops"] / PEAK_BF16_TFLOPS, 4),
                               "gemm_share_of_step_time": round(f["gemm_share"], 4), "loss": round(f["loss"], 5)})
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, fig["flops"])
    print(json.dumps(out))


if __name__ == "__main__":
    main()
