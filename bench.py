#!/usr/bin/env python3
"""Benchmark of the llama decoder-layer training step (fwd + loss + bwd) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--no-cpu-baseline]

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
GEMM_HBM_BYTES_PER_LAUNCH = {"C2": 609.6e6}


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
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share only (TP=1, one MI355X); --gpus %d is not supported. "
              "Run with --gpus 1." % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from easyllm_amd import functional, kernels, runner, workloads as W
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = W.WORKLOADS[args.workload]
    torch.manual_seed(w["seed"])
    model = runner.build_model({"type": "llama_custom", "kwargs": W.model_kwargs(w)})
    runner.attach_main_grads(model)
    functional.set_input_check(args.input_check)
    inputs, labels, doc_lens = W.make_inputs(w, device=dev)
    tokens_per_step = w["batch"] * w["seq"]
    flops = W.step_flops(w, doc_lens)

    def step():
        runner.zero_main_grads(model)
        return runner.forward_step(model, inputs, labels)

    def timed(fn, flush):
        """Exactly args.steps calls of fn between two device synchronisations: (last loss, wall seconds, per-step ms from
        one event per step boundary on the compute stream)."""
        events = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        events[0].record()
        for i in range(args.steps):
            last = fn()
            events[i + 1].record()
        flush()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        return last, wall, [events[i].elapsed_time(events[i + 1]) for i in range(args.steps)]

    for _ in range(args.warmup):
        loss = step()
    loss, elapsed_eager, per_step = timed(step, functional.flush_input_checks)
    loss_value = float(loss.item())
    elapsed = elapsed_eager
    launch_mode = args.mode
    if args.mode == "graph":
        # the same kernels, captured once and replayed: no per-kernel host work, no launch gaps
        try:
            graphed = runner.GraphedStep(model, inputs, labels)
        except Exception as exc:  # capture refused by the runtime: report the eager figures and say so
            graphed = None
            launch_mode = "eager (graph capture failed: %s)" % (str(exc).splitlines()[0][:120] if str(exc) else type(exc).__name__)
            print("bench.py: %s" % launch_mode, file=sys.stderr)
        if graphed is not None:
            for _ in range(args.warmup):
                graphed()
            loss, elapsed, per_step = timed(graphed, graphed.flush)
            assert float(loss.item()) == loss_value, "graph replay and eager step disagree"
            del graphed
    per_step.sort()
    median_ms = per_step[len(per_step) // 2] if len(per_step) % 2 else 0.5 * (per_step[len(per_step) // 2 - 1] + per_step[len(per_step) // 2])

    # Second pass of the same K steps with every GEMM launch bracketed by two timing events on the launch stream.  The
    # events serialise the queue (about 20 us per launch), so they are kept out of the pass that `value` comes from.
    kernels.GEMM_TIMING = []
    t1 = time.perf_counter()
    for _ in range(args.steps):
        step()
    functional.flush_input_checks()
    torch.cuda.synchronize()
    elapsed_instrumented = time.perf_counter() - t1
    timing, kernels.GEMM_TIMING = kernels.GEMM_TIMING, None

    ms_per_step = elapsed / args.steps * 1e3
    tok_s = tokens_per_step * args.steps / elapsed
    tflops = flops * args.steps / elapsed / 1e12
    gemm_flops = sum(f for f, _, _ in timing)
    gemm_ms = sum(s.elapsed_time(e) for _, s, e in timing)
    gemm_tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12 if gemm_ms > 0 else 0.0
    out = {
        "metric": METRIC, "value": round(tok_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3), "ms_per_step_median": round(median_ms, 3),
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "%s: %s" % (args.workload, w["desc"]), "tokens_per_step": tokens_per_step,
                   "fp32_main_grads": True, "recomputed_layers": model.recompute_count,
                   "input_id_check": args.input_check, "launch": launch_mode,
                   "eager_ms_per_step": round(elapsed_eager / args.steps * 1e3, 3)},
        "tflops": round(tflops, 1), "mfma_frac_end_to_end": round(tflops / PEAK_BF16_TFLOPS, 4), "loss": round(loss_value, 5),
        "roofline": {"kernel": "gemm_kernel (bf16 MFMA GEMM, %d launches/step)" % (len(timing) // max(args.steps, 1)),
                     "bound": "mfma", "achieved": round(gemm_tflops, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(gemm_tflops / PEAK_BF16_TFLOPS, 4), "traffic": GEMM_HBM_BYTES_PER_LAUNCH.get(args.workload),
                     "avg_launch_us": round(gemm_ms * 1e3 / max(len(timing), 1), 2),
                     "share_of_step_time": round(gemm_ms / args.steps / ms_per_step, 4),
                     "measured_in": "second pass of the same %d steps with two timing events per GEMM launch (%.3f ms/step)"
                                    % (args.steps, elapsed_instrumented / args.steps * 1e3)},
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
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w, flops)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
