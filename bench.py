#!/usr/bin/env python3
"""Headline benchmark: training tokens/s of the GPT-2-small-shape step (vocab 50304, d 768, 12 layers, 12 heads,
ctx 1024, batch 16; forward + backward + AdamW with gradient clipping) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--mode fast|backend|parity] [--no-cpu] [--no-extra] [--workload gpt2-small|gpt-350m]

`--mode fast` (default) is the hand-scheduled step (FusedTrainer) of the function an unchanged gpt.ts computes on a backend
with flashAttention (`--attention reference-flash`, gpt.ts:247-254: q, k, v re-read as [B H, T, D] slabs without a head
transpose; `--attention heads` = multi-head attention on the columns of the projection instead); `--mode backend` runs the generic tape-driven Trainer -- one
`Backend` call per op, host-side loss / norm / clip, exactly the call structure of the reference trainer -- on FastHipBackend
(bf16 storage, fused epilogues and grouped weight gradients behind the interface, steps replayed as recorded hipGraph
segments); `--mode parity` runs the same Trainer on the fp32 kernels.

The default workload is the one the metric is quoted on; `--workload gpt-350m` runs the 350M-shape step (d 1024, 24 layers,
16 heads, batch 8 with 4 accumulated micro-steps, whole step in one hipGraph) and reports it the same way.

After the headline measurement the default invocation also times, each in a child process of its own once the parent has
released its device memory, the path the reference's trainer would take -- `--mode backend` with the model's own attention
wiring and with multi-head attention (`heads`) --, the 350M-shape workload and the headline step with `heads`, and adds them
to the line as `backend_mode`, `workload_350m` and `fused_step_heads_attention` (`--no-extra` leaves them out).

Prints ONE JSON line.  `value` is tokens/s with parameters, optimizer state and the token batch already resident in
HBM; the scatter-add index of the token embedding's gradient (a sort of the batch's ids) is built inside the timed steps.  `roofline` is for the dominant kernel, the MFMA GEMM instantiation that does the most arithmetic in a step (which is
also the one with the largest summed duration; going by arithmetic keeps the choice the same from run to run):
2*M*N*K of its launches divided by their summed durations, each launch bracketed by HIP events on the library's
stream (`all_gemm` gives the same over every GEMM launch of the step).  `cpu_baseline` times the CPU oracle
(single-thread C restatement of the reference's cpu_ref loops) on a bounded sample of the same model.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

GPT2 = dict(vocabSize=50304, blockSize=1024, nLayer=12, nEmbd=768, nHead=12)
BATCH = 16
WORKLOADS = {        # name -> (model, micro-batch, accumulated micro-steps, token seed, description)
    "gpt2-small": (GPT2, BATCH, 1, 4, "GPT-2-small-shape train step: vocab 50304, d_model 768, 12 layers, 12 heads, ctx 1024, batch 16, "
                                      "untied lmHead (163.0M params), AdamW lr 3e-4 betas (0.9,0.95) wd 0.1, grad-clip 1.0"),
    "gpt-350m": (dict(vocabSize=50304, blockSize=1024, nLayer=24, nEmbd=1024, nHead=16), 8, 4, 5,
                 "350M-shape train step: vocab 50304, d_model 1024, 24 layers, 16 heads, ctx 1024, batch 8 x 4 accumulated micro-steps, "
                 "untied lmHead (406.2M params), AdamW lr 3e-4 betas (0.9,0.95) wd 0.1, grad-clip 1.0"),
}
PEAK = {"bf16": 2500.0, "f32": 157.3}          # MI355X dense MFMA, TFLOP/s
# Counter summaries of this benchmark (rocprofv3 --pmc passes; the files say how they were made and calibrated).  What the
# JSON line reports from counters -- HBM-side bytes per launch of the dominant kernel, time-weighted MFMA-busy fraction of the
# step -- is read from the table in the file of the workload, never typed in here.
COUNTER_TABLES = {"gpt2-small": "profiles/train_step_gpt2small_bf16_counters.md", "gpt-350m": "profiles/train_step_gpt350m_bf16_counters.md"}


def counter_table(workload: str):
    """Rows of the '| kernel | launches | us per step | clock GHz | MFMA busy | fetched MB | written MB | ...' table."""
    path = os.path.join(ROOT, COUNTER_TABLES.get(workload, ""))
    rows = {}
    if not os.path.isfile(path):
        return rows, None
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 7 and cells[0].startswith("k_"):
            try:
                rows[cells[0]] = {"launches": float(cells[1]), "us": float(cells[2]), "busy": float(cells[4]),
                                  "fetched_mb": float(cells[5]), "written_mb": float(cells[6])}
            except ValueError:
                pass
    return rows, COUNTER_TABLES[workload]


def step_flops(cfg, tokens, causal=False):
    """6*P_mm + 12*L*T*C per token: attention counted non-causal, the reference's convention (scripts/bench-ops.ts:652,673);
    `causal` counts the half of the score / value products a causal kernel has to do (6*L*T*C, the diagonal aside)."""
    C_, L, F, V, T = cfg["nEmbd"], cfg["nLayer"], 4 * cfg["nEmbd"], cfg["vocabSize"], cfg["blockSize"]
    p_mm = L * (3 * C_ * C_ + C_ * C_ + 2 * C_ * F) + V * C_
    return (6 * p_mm + (6 if causal else 12) * L * T * C_) * tokens


def cpu_baseline(model: dict, seq_tokens: int):
    """Oracle (port of the reference CPU path), one thread, on the SAME model with 1 sequence of `seq_tokens` tokens."""
    from oracle import ref_model as rm
    cfg = rm.ModelConfig(**model)
    tr = rm.Trainer(cfg, rm.TrainConfig(iters=50), seed=0)
    batch = rm.synthetic_batch(4, 1, seq_tokens, cfg.vocabSize)
    t0 = time.perf_counter()
    r = tr.step([batch])
    dt = time.perf_counter() - t0
    return {"value": seq_tokens / dt, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"same model ({sum(v.data.data.size for _, v in tr.entries) / 1e6:.1f}M params), 1 sequence x {seq_tokens} tokens, one full step "
                      f"(forward+backward+clip+AdamW) in {dt:.1f} s; loss {r.loss:.4f}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--mode", choices=["fast", "backend", "parity"], default="fast")
    ap.add_argument("--no-step-graphs", action="store_true", help="backend mode: issue every launch eagerly")
    ap.add_argument("--dw-groups", type=int, default=1, help="fast mode: weight-gradient GEMMs in this many runs on a second stream")
    ap.add_argument("--norm-over-arena", action="store_true", help="fast mode, for comparison: take the gradient norm by reading the whole gradient "
                    "arena again instead of summing the weight gradients' squares in the epilogue of the launch that stores them")
    ap.add_argument("--stream", choices=["f32", "bf16"], default="bf16", help="fast mode: storage type of the residual stream and its gradient")
    ap.add_argument("--attention", choices=["heads", "reference-flash", "unfused"], default="reference-flash",
                    help="which attention branch of the model runs (reference-flash = what the reference's flash branch computes, "
                         "gpt.ts:232-253; heads = multi-head attention; unfused = its CPU branch, backend / parity mode only)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="only the headline measurement: no backend-mode and no 350M-shape runs")
    ap.add_argument("--cpu-tokens", type=int, default=32)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="gpt2-small")
    ap.add_argument("--micro-per-pass", type=int, default=1,
                    help="fast mode, workloads with accumulated micro-steps: run this many micro-steps as one pass over their micro-batches "
                         "(FusedTrainer(micro_per_pass=...): the step's loss, gradient and update are the same numbers)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the step on ONE GPU; --gpus must be 1 (no multi-GPU path exists in this run)", file=sys.stderr)
        sys.exit(2)
    if args.mode == "backend" and not args.no_step_graphs:
        # a step plan takes a few steps to settle: one eager step, one recorded, and a first replay that rewrites the nodes
        # whose buffers were not yet at their steady addresses when the step was recorded
        args.warmup = max(args.warmup, 4)

    from alpha2_amd import FastHipBackend, HipBackend
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, zipfBatches

    B = FastHipBackend(0) if args.mode == "backend" else HipBackend(0)
    model, BATCH, accum, tok_seed, describe = WORKLOADS[args.workload]
    cfg = ModelConfig(**model, attention=args.attention)
    tc = TrainConfig(iters=50, batchSize=BATCH, gradAccumSteps=accum)
    tokens = BATCH * cfg.blockSize * accum
    # a ring of distinct resident batches: every step trains on the next `accum` of them, so the reported losses are a
    # training curve and not the memorisation of one batch
    ring = max(8, accum * 4)
    micro = zipfBatches(tok_seed, ring, BATCH, cfg.blockSize, cfg.vocabSize)        # one stream from the workload's seed
    if args.mode in ("parity", "backend"):
        from alpha2_amd.train import Trainer
        runner = Trainer(B, cfg, tc, seed=0)
        dtype = "f32" if args.mode == "parity" else "bf16"
        for x, y in micro:
            B._ptr(x), B._ptr(y)
        if args.mode == "backend" and not args.no_step_graphs:
            B.enableStepGraphs(True)

        cursor = [0]

        def one_step():
            # the generic trainer releases its batch after use; keep ours resident by handing it views
            pick = [micro[(cursor[0] + m) % ring] for m in range(accum)]
            cursor[0] += accum
            return runner.step([(B.reshape(x, x.shape), B.reshape(y, y.shape)) for x, y in pick])
    else:
        from alpha2_amd.fused import FusedTrainer
        runner = FusedTrainer(B, cfg, tc, BATCH, seed=0, accum=accum, dw_groups=args.dw_groups, stream=args.stream,
                              norm_in_epilogue=not args.norm_over_arena, index_in_step=True, micro_per_pass=args.micro_per_pass)
        dtype = "bf16"
        ids = [runner.add_batch(x, y) for x, y in micro]                   # resident in HBM before the timed region
        cursor = [0]

        def one_step():
            pick = [ids[(cursor[0] + m) % ring] for m in range(accum)]
            cursor[0] += accum
            # two 64 KB device-to-device copies, then the graph (which sorts the batch's ids for the embedding gradient itself)
            return runner.step(pick if accum > 1 else pick[0])

    losses = []
    for _ in range(args.warmup):
        losses.append(one_step())
    B.syncGpu()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        losses.append(one_step())
    B.syncGpu()
    dt = time.perf_counter() - t0
    ms = dt / args.steps * 1e3
    if hasattr(runner, "history"):
        hist = runner.history(0, args.warmup + args.steps)
        loss_first, loss_last = hist[0].loss, hist[-1].loss
    else:
        loss_first, loss_last = losses[0].loss, losses[-1].loss

    step_stats = None
    if args.mode == "backend":
        B.enableStepGraphs(False)
        step_stats = dict(B.stepStats(), fallbackNotes=B.stepFallbackNotes[-4:])
    # one instrumented step: every GEMM launch bracketed by HIP events on the library stream
    recs = runner.timed_step() if hasattr(runner, "timed_step") else _timed(B, one_step)
    gemm = [r for r in recs if r["kind"] == "gemm"]
    g_flops, g_ms = sum(r["flops"] for r in gemm), sum(r["ms"] for r in gemm)
    # the dominant kernel = the GEMM instantiation with the most arithmetic per step among launches that are one kernel
    # (a split-K launch is followed by its reduce kernel inside the same event bracket, so it is not a clean sample; the
    # grouped launch is kept: when the tiles of its last round are cut in two along k, the bracket also holds the ~25 us
    # kernel that joins the halves, which is counted against it)
    groups = {}
    for r in gemm:
        if r["nsplit"] == 1 or "grouped" in r["kernel"]:
            grp = groups.setdefault(r["kernel"], {"flops": 0.0, "ms": 0.0, "n": 0})
            grp["flops"] += r["flops"]; grp["ms"] += r["ms"]; grp["n"] += 1
    dom_name, dom = max(groups.items(), key=lambda kv: (kv[1]["flops"], kv[1]["ms"]))
    achieved = dom["flops"] / (dom["ms"] * 1e-3) / 1e12
    flops, flops_causal = step_flops(model, tokens), step_flops(model, tokens, causal=True)
    table, table_path = counter_table(args.workload) if args.mode == "fast" else ({}, None)
    trow = table.get(dom_name)
    traffic = (trow["fetched_mb"] + trow["written_mb"]) * 1e6 / trow["launches"] if trow else None
    # MFMA-busy fraction of the step by the SQ_VALU_MFMA_BUSY_CYCLES counter: kernels weighted by their time in the step
    busy = (sum(r["busy"] * r["us"] for r in table.values()) / sum(r["us"] for r in table.values())) if table else None
    out = {
        "metric": "train tokens/sec + MFMA util % on GPT-124M step, 1xMI355X", "value": tokens / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": f"synthetic (Zipf s=1.1 token ids, seed {tok_seed}; random-init N(0,0.02) weights, seed 0)",
        "config": {"workload": describe,
                   "tokens_per_step": tokens, "mode": args.mode, "loss_first_step": loss_first, "loss_last_step": loss_last,
                   "attention": args.attention, **({"micro_per_pass": args.micro_per_pass} if args.micro_per_pass != 1 else {})},
        # model flops per second against the dense bf16 MFMA peak: by the reference's (non-causal) attention count, and with
        # the causal half of the attention products only
        "step_tflops": flops / (ms * 1e-3) / 1e12, "mfu_vs_bf16_dense_peak": flops / (ms * 1e-3) / 1e12 / PEAK["bf16"],
        "step_tflops_causal": flops_causal / (ms * 1e-3) / 1e12, "mfu_causal": flops_causal / (ms * 1e-3) / 1e12 / PEAK["bf16"],
        # the "MFMA util %" of the metric: model flops / peak (= mfu_vs_bf16_dense_peak); beside it what the hardware counter
        # says, from the committed counter summary of this workload (not measured in this run)
        "mfma_util_pct": 100.0 * flops / (ms * 1e-3) / 1e12 / PEAK["bf16"],
        "mfma_busy_counter": {"frac_of_step_time": busy, "source": table_path},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK[dtype], "unit": "TFLOP/s", "frac": achieved / PEAK[dtype],
                     "traffic": traffic, "traffic_source": table_path if trow else None, "kernel": dom_name, "launches_per_step": dom["n"], "avg_launch_us": dom["ms"] / dom["n"] * 1e3,
                     "flops_per_launch": dom["flops"] / dom["n"], "ms_per_step": dom["ms"],
                     "all_gemm": {"launches_per_step": len(gemm), "ms_per_step": g_ms,
                                  "achieved": g_flops / (g_ms * 1e-3) / 1e12 if g_ms > 0 else 0.0}},
    }
    if step_stats is not None:
        out["config"]["step_plans"] = step_stats
    if args.mode == "fast" and args.dw_groups > 1:
        out["config"]["dw_groups"] = args.dw_groups
    if args.mode == "fast" and args.norm_over_arena:
        out["config"]["norm"] = "over the arena"
    if args.mode == "fast":
        out["config"]["residual_stream"] = args.stream
        out["index_us_outside_timed_region"] = 0.0      # the id sort of every batch is part of the captured step
    if args.mode == "fast":
        # the ceiling under the power limit, measured here and now: 10 launches of ~4 ms each way
        probe = mfma_probe(B)
        out["mfma_sustained"] = dict(probe, what="matrix pipes alone, operands in registers, 10 x ~4 ms (ah_probe_mfma_bf16)")
        out["roofline"]["frac_of_sustained"] = achieved / probe["toggling_operands_tflops"]
        out["mfu_vs_sustained"] = out["step_tflops"] / probe["toggling_operands_tflops"]
    if args.mode == "fast" and args.workload == "gpt2-small" and not args.no_extra:
        runner.close()
        del runner
        B.purgeBufferPools()
        out.update(extra_runs(args))
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(model, args.cpu_tokens)
    print(json.dumps(out))


def mfma_probe(B) -> dict:
    """What the matrix pipes alone sustain in this process on this box (ah_probe_mfma_bf16: independent 32x32x16 bf16 MFMAs
    on registers, no memory traffic): on all-zero operands the part runs at its published peak, on operands whose bits toggle
    at what its power limit leaves, which is the ceiling a GEMM on real data can be read against."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    lib, fl, out = B.lib, C.c_double(), {}
    for name, rnd in (("zero_operands_tflops", 0), ("toggling_operands_tflops", 1)):
        ffi.check(lib.ah_probe_mfma_bf16(1, 100, rnd, C.byref(fl)))
        ffi.check(lib.ah_sync())
        e0, e1 = B._event(), B._event()
        ffi.check(lib.ah_event_record(e0))
        for _ in range(10):
            ffi.check(lib.ah_probe_mfma_bf16(1, 30000, rnd, C.byref(fl)))
        ffi.check(lib.ah_event_record(e1))
        ms = C.c_float()
        ffi.check(lib.ah_event_elapsed_ms(e0, e1, C.byref(ms)))
        for e in (e0, e1):
            ffi.check(lib.ah_event_destroy(e))
        out[name] = fl.value * 10 / (ms.value * 1e-3) / 1e12
    return out


def extra_runs(args) -> dict:
    """The same steps through the reference's call structure (generic Trainer on FastHipBackend, step plans) with both
    attention wirings, and the 350M-shape workload: each a child process running this file, its JSON line parsed."""
    import subprocess

    def child(*flags):
        cmd = [sys.executable, os.path.abspath(__file__), "--steps", str(args.steps), "--warmup", str(args.warmup), "--no-cpu", "--no-extra", *flags]
        try:
            r = subprocess.run(cmd, capture_output=True, text=True, timeout=600, cwd=ROOT)
            line = [l for l in r.stdout.splitlines() if l.startswith("{")]
            if r.returncode != 0 or not line:
                return {"error": (r.stderr or r.stdout)[-300:]}
            return json.loads(line[-1])
        except Exception as e:                                   # a failed extra run must not cost the headline line
            return {"error": repr(e)[:300]}
    ref, heads, big = (child("--mode", "backend", "--attention", "reference-flash"), child("--mode", "backend", "--attention", "heads"),
                       child("--workload", "gpt-350m"))
    fused_heads, big_heads = child("--attention", "heads"), child("--workload", "gpt-350m", "--attention", "heads")
    big_pairs = child("--workload", "gpt-350m", "--micro-per-pass", "2")
    res = {"fused_step_heads_attention": {"ms_per_step": fused_heads.get("ms_per_step"),
                                          "what": "the headline step with multi-head attention on the columns of the projection instead of the reference's slabs"},
           "backend_mode": {"ms_per_step": heads.get("ms_per_step"), "ms_per_step_reference_flash": ref.get("ms_per_step"),
                            "step_plans": (heads.get("config") or {}).get("step_plans"),
                            "step_plans_reference_flash": (ref.get("config") or {}).get("step_plans"),
                            "what": "generic tape-driven Trainer, one Backend call per op, on FastHipBackend with step plans; same model, batches and steps"},
           "workload_350m": {"ms_per_step": big.get("ms_per_step"), "tokens_per_s": big.get("value"), "mfu": big.get("mfu_vs_bf16_dense_peak"),
                             "ms_per_step_heads_attention": big_heads.get("ms_per_step"),
                             # the same step with its four micro-steps run two to a pass (same loss, gradient and update:
                             # tests/test_gpu_fullsize.py): a pass then has 16384 rows for its products instead of 8192
                             "micro_steps_two_to_a_pass": {"ms_per_step": big_pairs.get("ms_per_step"), "tokens_per_s": big_pairs.get("value"),
                                                           "mfu": big_pairs.get("mfu_vs_bf16_dense_peak")},
                             "what": (big.get("config") or {}).get("workload")}}
    for k, v in (("backend_mode", heads), ("backend_mode", ref), ("workload_350m", big), ("workload_350m", big_heads), ("workload_350m", big_pairs),
                 ("fused_step_heads_attention", fused_heads)):
        if "error" in v:
            res[k].setdefault("errors", []).append(v["error"])
    return res


def _timed(B, one_step):
    B.syncGpu()
    B.startTiming()
    one_step()
    return B.stopTiming()


if __name__ == "__main__":
    main()
