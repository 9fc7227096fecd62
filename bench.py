#!/usr/bin/env python3
"""Batch-1 decode benchmark on one MI355X.

Workload (N=1): TinyLlama-1.1B-shaped Llama, random-init fp32 (weights N(0, 0.02), RMSNorm gains
1.0, seed 0), 22 layers, hidden 2048, 32 q / 4 kv heads, head_dim 64, SwiGLU 5632, vocab 32000;
prompt of 128 uniform-random token ids, then greedy decode.  A "step" is one decoded token: one
pass of the decode path (one HIP-graph replay) with weights and KV cache resident in HBM.

  python bench.py [--gpus 1] [--steps 128] [--warmup 8]

Prints ONE JSON line: decode tokens/s, the roofline of the dominant kernel (measured live with
HIP events on the library's stream) and the CPU baseline (the C restatement of Lumen's CPU
algorithms, OpenMP over the host cores, timed on a bounded sample of the same workload).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--mode", choices=["graph", "eager"], default="graph",
                    help="how decode steps are issued: a HIP graph replay per token (default) or kernel by kernel "
                         "(for rocprofv3 --kernel-trace, which cannot follow graph replays here)")
    ap.add_argument("--cpu-tokens", type=int, default=48)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the batch-1 decode path on ONE GPU; --gpus %d is not supported "
                 "(nothing here shards across GPUs)" % args.gpus)

    import numpy as np

    from lumen_amd import synth
    from lumen_amd.models import LlamaModel

    cfg = dict(synth.TINYLLAMA_1B)
    need = args.prompt + args.warmup + 2 * args.steps + 8
    if need > cfg["max_seq_len"]:
        sys.exit("bench.py: prompt + warmup + 2*steps = %d exceeds max_seq_len %d" % (need, cfg["max_seq_len"]))

    t0 = time.time()
    model = LlamaModel(cfg)
    model.set_decode_mode(args.mode)
    keep_host = not args.no_cpu_baseline
    params = {}
    for name, a in synth.iter_params(cfg, seed=0):
        model.set_param(name, a)
        if keep_host:
            params[name] = a
    prompt = synth.make_tokens(args.prompt, cfg["vocab_size"], seed=0)
    t_setup = time.time() - t0

    # prefill (untimed here; reported separately)
    ctx = model.ctx
    ctx.timer_start()
    last = model.forward(prompt, all_rows=False)
    prefill_ms = ctx.timer_stop()
    first = int(np.argmax(last))

    # warmup, then EXACTLY --steps decoded tokens between two events on the library's stream
    if args.warmup:
        w = model.decode_greedy(first, args.warmup)
        first = int(w[-1])
    len0 = model.kv_len
    ctx.synchronize()
    wall0 = time.perf_counter()
    ctx.timer_start()
    picks = model.decode_greedy(first, args.steps)
    ms = ctx.timer_stop()
    wall = time.perf_counter() - wall0
    ms_per_step = ms / args.steps
    tok_s = 1000.0 / ms_per_step
    mean_len = len0 + (args.steps + 1) / 2.0
    step_bytes = model.decode_bytes(int(round(mean_len)))

    # per-kernel event timing over a second pass of the same length (eager launches, same kernels)
    prof = model.decode_profile(int(picks[-1]), args.steps)
    H, I = cfg["hidden_size"], cfg["intermediate_size"]
    # dominant kernel: RMSNorm + gate|up GEMV + SwiGLU, W [2I, H] f32 read once per launch
    gu_ms, gu_n = prof["norm_gateup_gemv"]
    gu_bytes = 4.0 * (2.0 * I * H + H + I)
    gu_avg_ms = gu_ms / max(gu_n, 1)
    achieved = gu_bytes / (gu_avg_ms * 1e-3) / 1e9
    kernels = {}
    for name, (s_ms, n) in prof.items():
        if n:
            kernels[name] = {"avg_us": round(1e3 * s_ms / n, 3), "launches_per_step": n // args.steps}

    out = {
        "metric": "batch-1 decode tokens/s", "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "TinyLlama-1.1B-shaped Llama fp32 random-init seed 0, batch 1, prompt %d random ids, "
                               "greedy decode, static KV cache max_seq_len %d" % (args.prompt, cfg["max_seq_len"]),
                   "layers": cfg["num_hidden_layers"], "hidden": H, "heads": "32q/4kv", "head_dim": 64,
                   "intermediate": I, "vocab": cfg["vocab_size"], "kv_len_during_timing": [len0, len0 + args.steps]},
        "roofline": {"bound": "hbm", "kernel": "gemv_kernel<f32,R=2,RMSNORM,SWIGLU> (norm+gate|up GEMV, [11264,2048])",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "bytes_per_launch": gu_bytes, "avg_launch_us": round(gu_avg_ms * 1e3, 3)},
        "step_roofline": {"bytes_per_token": step_bytes, "achieved_GBps": round(step_bytes / (ms_per_step * 1e-3) / 1e9, 1),
                          "frac_of_8TBps": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                          "roofline_tokens_per_s": round(HBM_PEAK_GBS * 1e9 / step_bytes, 1)},
        "kernels": kernels,
        "prefill": {"tokens": args.prompt, "ms": round(prefill_ms, 3), "tokens_per_s": round(args.prompt / prefill_ms * 1e3, 1)},
        "decode_mode": args.mode, "wall_s_timed_region": round(wall, 4), "setup_s": round(t_setup, 1),
    }

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, params, prompt, args.cpu_tokens)
    print(json.dumps(out))


def cpu_baseline(cfg, params, prompt, n_tokens):
    """The C restatement of Lumen's CPU path (row-parallel M=1 GEMV, head-parallel online-softmax
    attention) on the host cores: prefill the same prompt, then time n_tokens greedy decode steps."""
    import numpy as np

    from oracle import lumen_oracle as lo

    ora = lo.Llama(cfg, params)
    rc, logits = ora.forward(prompt)
    assert rc == lo.LO_OK
    tok = lo.argmax(logits[-1])
    t0 = time.perf_counter()
    for _ in range(n_tokens):
        rc, lg = ora.forward(np.array([tok]))
        tok = lo.argmax(lg[0])
    dt = time.perf_counter() - t0
    return {"value": round(n_tokens / dt, 3), "unit": "tokens/s", "cores": lo.get_threads(), "kind": "port",
            "sample": "%d greedy decode tokens after the same %d-token prompt, same weights; C restatement of "
                      "Lumen's CPU algorithms (gcc -O3, OpenMP), Rust toolchain unavailable" % (n_tokens, len(prompt))}


if __name__ == "__main__":
    main()
