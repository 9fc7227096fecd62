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
MFMA_FP32_PEAK_TF = 157.3  # MI355X dense fp32 matrix peak, TFLOP/s
MFMA_BF16_PEAK_TF = 2500.0  # MI355X dense bf16 matrix peak, TFLOP/s
# the prompt-pass GEMM takes an f32 product as six bf16 matrix products (three bf16 parts per f32 value)
GEMM_BF16_PRODUCTS = 6


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--max-seq", type=int, default=2048,
                    help="rows of the static KV cache (2048: the headline configuration; 4096 with --prompt 3968 "
                         "--steps 32 is the long-context configuration)")
    ap.add_argument("--model", choices=["tinyllama-1.1b", "qwen3-0.6b", "llama2-7b-bf16"], default="tinyllama-1.1b",
                    help="shape of the random-init model: the headline configuration (default); the Qwen3-0.6B shape "
                         "(q/k norm, head_dim 128, tied embeddings: use --prompt 256 --steps 80 --max-seq 1024); the "
                         "Llama-2-7B shape with bf16 weights (--prompt 512 --steps 40 --max-seq 1024).  The bench line "
                         "the driver reads is the default one; the others carry no cpu_baseline")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the long-context, Qwen3-0.6B-shape and Llama-2-7B-shape decode records that the default "
                         "run appends (other_configs) after the headline measurement")
    ap.add_argument("--mode", choices=["graph", "eager"], default="graph",
                    help="how decode steps are issued: a HIP graph replay per token (default) or kernel by kernel "
                         "(for rocprofv3 --kernel-trace, which cannot follow graph replays here)")
    ap.add_argument("--cpu-tokens", type=int, default=48)
    ap.add_argument("--resident", action="store_true",
                    help="--workload gemv: every launch reads the SAME copy of W (what the caches hold counts: the "
                         "figure is no longer HBM bandwidth); default: >= 1.2 GB of copies in rotation")
    ap.add_argument("--workload", choices=["decode", "gemv", "gemm", "prefill", "copy"], default="decode",
                    help="decode: the headline batch-1 decode benchmark; gemv: the isolated M=1 GEMV shapes; "
                         "gemm: the prompt-pass GEMM shapes against the fp32 matrix-core peak; prefill: one long "
                         "prompt pass (3968 tokens, TinyLlama shape with a 4096-row cache); "
                         "copy: a plain 1 GiB copy kernel (calibrates the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the batch-1 decode path on ONE GPU; --gpus %d is not supported "
                 "(nothing here shards across GPUs)" % args.gpus)

    if args.workload == "gemv":
        return gemv_microbench(args)
    if args.workload == "copy":
        return copy_bench(args)
    if args.workload == "gemm":
        return gemm_microbench(args)
    if args.workload == "prefill":
        return prefill_bench(args)

    import numpy as np

    from lumen_amd import synth

    base = {"tinyllama-1.1b": synth.TINYLLAMA_1B, "qwen3-0.6b": synth.QWEN3_0P6B, "llama2-7b-bf16": synth.LLAMA2_7B}[args.model]
    cfg = dict(base, max_seq_len=args.max_seq)
    headline = args.model == "tinyllama-1.1b" and args.prompt == 128 and args.max_seq == 2048
    if not headline:
        args.no_cpu_baseline = True
        args.no_other_configs = True
    out, model, params, prompt = decode_bench(args.model, cfg, args.prompt, args.steps, args.warmup, args.mode,
                                              keep_host=not args.no_cpu_baseline, headline=headline)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, params, prompt, args.cpu_tokens, model)
    del model, params
    if not args.no_other_configs:
        # the other decode configurations of the benchmark, same library, same protocol, after the headline's timed
        # region: long context (cache 3976-4008 rows), the Qwen3-0.6B shape, the Llama-2-7B shape with bf16 weights
        out["other_configs"] = []
        for name, ocfg, n_prompt in (("tinyllama-1.1b", dict(synth.TINYLLAMA_1B_LONG), 3968),
                                     ("qwen3-0.6b", dict(synth.QWEN3_0P6B), 256),
                                     ("llama2-7b-bf16", dict(synth.LLAMA2_7B), 512)):
            steps = min(args.steps, (ocfg["max_seq_len"] - n_prompt - min(args.warmup, 8) - 8) // 2)
            o, m, _, _ = decode_bench(name, ocfg, n_prompt, steps, min(args.warmup, 8), args.mode, keep_host=False, headline=False)
            del m
            out["other_configs"].append({
                "workload": o["config"]["workload"], "dtype": o["dtype"], "steps": steps, "ms_per_step": o["ms_per_step"],
                "tokens_per_s": o["value"], "kv_len_during_timing": o["config"]["kv_len_during_timing"],
                "bytes_per_token": o["step_roofline"]["bytes_per_token"], "frac_of_8TBps": o["step_roofline"]["frac_of_8TBps"],
                "kernels": o["kernels"], "kernel_instances": o["kernel_instances"],
                "prefill_ms": o["prefill"]["ms"], "graph_picks_equal_eager_picks": o["self_check"]["graph_picks_equal_eager_picks"],
                "setup_s": o["setup_s"]})
    print(json.dumps(out))


MODEL_NAMES = {"tinyllama-1.1b": "TinyLlama-1.1B", "qwen3-0.6b": "Qwen3-0.6B", "llama2-7b-bf16": "Llama-2-7B"}


def decode_bench(model_name, cfg, n_prompt, steps, warmup, mode, keep_host, headline):
    """One decode measurement: build the random-init model, prompt pass, warm-up, EXACTLY `steps` greedy tokens
    between two events on the library's stream, then the per-kernel passes.  Returns (record, model, params, prompt)."""
    import numpy as np

    from lumen_amd import _lib, synth
    from lumen_amd.models import LlamaModel

    w_bf16 = cfg.get("weight_dtype") == "bf16"
    need = n_prompt + warmup + 2 * steps + 8
    if need > cfg["max_seq_len"]:
        sys.exit("bench.py: prompt + warmup + 2*steps = %d exceeds max_seq_len %d" % (need, cfg["max_seq_len"]))

    t0 = time.time()
    model = LlamaModel(cfg)
    model.set_decode_mode(mode)
    params = {}
    # bf16-stored weights: the values the reference would widen at load time
    to_bits = (lambda name, a: synth.bf16_round(a) if a.ndim == 2 and "embed" not in name else a) if w_bf16 else None
    for name, a in synth.iter_params_threaded(cfg, seed=0, workers=12, transform=to_bits):
        model.set_param(name, a)
        if keep_host:
            params[name] = a
    prompt = synth.make_tokens(n_prompt, cfg["vocab_size"], seed=0)
    t_setup = time.time() - t0

    # prefill (outside the timed decode region; reported separately).  The first pass sizes the
    # prompt buffers and the GEMM workspace; the second, from a reset cache, is the one timed.
    ctx = model.ctx
    short_ms = {}
    if headline:  # prompts of a few rows (a chat turn's new tokens): the weight-streaming prompt products
        for n_short in (4, 16, 32):
            if n_short >= n_prompt:
                continue
            best = None
            for _ in range(3):
                model.reset_kv_caches()
                ctx.timer_start()
                model.forward(prompt[:n_short], all_rows=False)
                t = ctx.timer_stop()
                best = t if best is None else min(best, t)
            short_ms[str(n_short)] = round(best, 3)
    prefill_all_ms = []
    for _ in range(3):  # the third pass is the steady one (the first two still see allocator / loader warm-up)
        model.reset_kv_caches()
        ctx.timer_start()
        last = model.forward(prompt, all_rows=False)
        prefill_all_ms.append(ctx.timer_stop())
    prefill_ms = prefill_all_ms[-1]
    first = int(np.argmax(last))

    # warmup, then EXACTLY --steps decoded tokens between two events on the library's stream
    if warmup:
        w = model.decode_greedy(first, warmup)
        first = int(w[-1])
    len0 = model.kv_len
    ctx.synchronize()
    wall0 = time.perf_counter()
    ctx.timer_start()
    picks = model.decode_greedy(first, steps)
    ms = ctx.timer_stop()
    wall = time.perf_counter() - wall0
    ms_per_step = ms / steps
    tok_s = 1000.0 / ms_per_step
    mean_len = len0 + (steps + 1) / 2.0
    step_bytes = model.decode_bytes(int(round(mean_len)))

    # The timed pass checks itself: the same steps again from the same cache state, launched kernel by kernel
    # instead of replayed from the graph, must pick the same tokens.  (That pass is also the plain eager timing.)
    model.set_kv_len(len0)
    model.set_decode_mode("eager")
    ctx.timer_start()
    picks_eager = model.decode_greedy(first, steps)
    eager_ms = ctx.timer_stop()
    model.set_decode_mode(mode)
    if not np.array_equal(picks, picks_eager):
        raise SystemExit("bench: the timed pass picked %s, eager launches of the same steps %s" % (picks.tolist(), picks_eager.tolist()))

    # Per-kernel durations, live: a further pass of the same length with every launch between two HIP
    # events on the library's stream (eager launches of the same kernels).  An event pair adds a fixed
    # cost to what it brackets; (bracketed total - plain eager total) / launches is that cost, and it is
    # taken off, so that the figures are kernel durations (they agree with the rocprofv3 trace).
    prof = model.decode_profile(int(picks[-1]), steps)
    n_launches = sum(n for _, n in prof.values())
    bracketed_ms = sum(s_ms for s_ms, _ in prof.values())
    event_overhead_ms = max(0.0, (bracketed_ms - eager_ms) / max(n_launches, 1))
    H, I = cfg["hidden_size"], cfg["intermediate_size"]
    # dominant kernel: RMSNorm + gate|up GEMV + SwiGLU, W [2I, H] read once per launch
    esz = 2.0 if w_bf16 else 4.0
    mlp_fused = prof["mlp_fused"][1] > 0  # narrow models: gate|up and down are one launch
    gu_ms, gu_n = prof["mlp_fused"] if mlp_fused else prof["norm_gateup_gemv"]
    gu_bytes = esz * 2.0 * I * H + 4.0 * (H + I) + (esz * H * I + 4.0 * 2 * H if mlp_fused else 0.0)
    gu_raw_ms = gu_ms / max(gu_n, 1)
    gu_avg_ms = gu_raw_ms - event_overhead_ms
    achieved = gu_bytes / (gu_avg_ms * 1e-3) / 1e9
    kernels = {}
    for name, (s_ms, n) in prof.items():
        if n:
            kernels[name] = {"avg_us": round(1e3 * (s_ms / n - event_overhead_ms), 3),
                             "launches_per_step": n // steps}

    # Kernel instances: the names the launchers recorded during that profile pass.  The dominant one must be what the
    # library's own dispatch reports for [2I, H] (lumen_gemv_kernel_name reads the decision launch_gemv takes), and
    # the committed counter figures are only quoted when they were taken on that same instance.
    names = {k: model.profile_kernel_name(k) for k in prof if prof[k][1]}
    gu_kernel = names["mlp_fused" if mlp_fused else "norm_gateup_gemv"]
    picked = _lib.gemv_kernel_name(ctx.num_cus, 2 * I, H, w_bf16, True, _lib.GEMV_EPI_SWIGLU)
    if not mlp_fused and gu_kernel != picked:
        raise SystemExit("bench: gate|up launched %r but the dispatch reports %r" % (gu_kernel, picked))
    # decode attention: K and V rows of every KV head, read once per launch (mean cache length of the timed
    # region); with short caches attention and o_proj are one launch, which also streams W_o [H, H]
    hq, hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    D = cfg.get("head_dim") or H // hq
    fused_attn = prof["attn_oproj_fused"][1] > 0
    at_ms, at_n = prof["attn_oproj_fused"] if fused_attn else prof["attn_decode"]
    at_avg_ms = at_ms / max(at_n, 1) - event_overhead_ms
    at_kernel = names["attn_oproj_fused" if fused_attn else "attn_decode"]
    at_bytes = 2.0 * hkv * mean_len * D * 4  # K and V rows
    at_what = "decode attention"
    if fused_attn:
        at_bytes += esz * H * hq * D  # + W_o
        at_what = "decode attention + o_proj"
        if prof["norm_qkv_gemv"][1] == 0:  # + W_qkv: the q|k|v product is part of the same launch
            at_bytes += esz * (hq + 2 * hkv) * D * H
            at_what = "RMSNorm + q|k|v + RoPE, decode attention, o_proj + residual"
    out = {
        "metric": "batch-1 decode tokens/s", "value": round(tok_s, 2), "unit": "tokens/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 weights, f32 accumulate" if w_bf16 else "f32", "data": "synthetic",
        "config": {"workload": "%s-shaped model %s random-init seed 0, batch 1, prompt %d random ids, "
                               "greedy decode, static KV cache max_seq_len %d"
                               % (MODEL_NAMES[model_name], "bf16 weights" if w_bf16 else "fp32", n_prompt, cfg["max_seq_len"]),
                   "layers": cfg["num_hidden_layers"], "hidden": H, "heads": "%dq/%dkv" % (hq, hkv), "head_dim": D,
                   "intermediate": I, "vocab": cfg["vocab_size"], "kv_len_during_timing": [len0, len0 + steps]},
        "roofline": {"bound": "hbm", "kernel": "%s (RMSNorm + gate|up GEMV [%d,%d] + SwiGLU%s)"
                               % (gu_kernel, 2 * I, H, ", down [%d,%d] + residual" % (H, I) if mlp_fused else ""),
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": measured_traffic(gu_kernel) if headline else None,
                     "bytes_per_launch": gu_bytes, "avg_launch_us": round(gu_avg_ms * 1e3, 3),
                     "avg_event_bracketed_us": round(gu_raw_ms * 1e3, 3),
                     "event_pair_overhead_us": round(event_overhead_ms * 1e3, 3)},
        "step_roofline": {"bytes_per_token": step_bytes, "achieved_GBps": round(step_bytes / (ms_per_step * 1e-3) / 1e9, 1),
                          "frac_of_8TBps": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                          "roofline_tokens_per_s": round(HBM_PEAK_GBS * 1e9 / step_bytes, 1)},
        "attention": {"kernel": "%s (%s)" % (at_kernel, at_what), "bytes_per_launch": at_bytes,
                      "avg_launch_us": round(at_avg_ms * 1e3, 3), "achieved_GBps": round(at_bytes / (at_avg_ms * 1e-3) / 1e9, 1),
                      "frac_of_8TBps": round(at_bytes / (at_avg_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)},
        "kernels": kernels, "kernel_instances": names,
        "prefill": dict(prefill_report(cfg, n_prompt, prefill_ms), passes_ms=[round(x, 3) for x in prefill_all_ms],
                        **({"short_prompts_ms": short_ms} if short_ms else {})),
        "decode_mode": mode, "eager_ms_per_step": round(eager_ms / steps, 5),
        "self_check": {"graph_picks_equal_eager_picks": True, "steps": steps},
        "wall_s_timed_region": round(wall, 4), "setup_s": round(t_setup, 1),
    }
    return out, model, params, prompt


def prefill_report(cfg, S, ms):
    """Prompt pass: tokens/s and the share of the fp32 matrix-core peak its GEMM flops amount to
    (all projections on S rows, lm_head on the last row only, causal attention counted once)."""
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    hq, hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    D = cfg.get("head_dim") or H // hq
    per_layer = hq * D * H + 2 * hkv * D * H + H * hq * D + 3 * H * I
    gemm_flops = 2.0 * S * L * per_layer + 2.0 * V * H
    attn_flops = 4.0 * L * hq * D * S * S / 2.0
    tf = (gemm_flops + attn_flops) / (ms * 1e-3) / 1e12
    issued = (GEMM_BF16_PRODUCTS * gemm_flops) / (ms * 1e-3) / 1e12  # bf16 matrix flops the GEMMs issue
    return {"tokens": S, "ms": round(ms, 3), "tokens_per_s": round(S / ms * 1e3, 1),
            "gemm_flops": gemm_flops, "attention_flops": attn_flops, "achieved_TFLOPs": round(tf, 2),
            "matrix_path": "GEMM: f32 values as 3 bf16 parts, 6 v_mfma_f32_32x32x16_bf16 products per f32 product; "
                           "attention: the same scheme",
            "mfma_fp32_peak_TFLOPs": MFMA_FP32_PEAK_TF, "vs_mfma_fp32_peak": round(tf / MFMA_FP32_PEAK_TF, 4),
            "gemm_bf16_TFLOPs_issued": round(issued, 1), "mfma_bf16_peak_TFLOPs": MFMA_BF16_PEAK_TF,
            "frac_of_mfma_bf16_peak": round(issued / MFMA_BF16_PEAK_TF, 4)}


def measured_traffic(kernel):
    """HBM bytes per launch of the dominant kernel from the committed rocprofv3 --pmc runs
    (FETCH_SIZE + WRITE_SIZE, calibrated on the copy kernel); counters cannot be read from here.
    None when those runs were taken on another kernel instance than the one launched now."""
    path = os.path.join(ROOT, "profiles", "decode_gateup_gemv_traffic.json")
    try:
        with open(path) as f:
            t = json.load(f)
        if t["kernel"] != kernel:
            return None
        return round(t["fetch_bytes_per_launch"] + t["write_bytes_per_launch"], 1)
    except (OSError, KeyError, ValueError):
        return None


def copy_bench(args):
    """out[i] = in[i] over 2^28 floats: 1 GiB read + 1 GiB written per launch."""
    import numpy as np

    from lumen_amd._lib import check, lib
    from lumen_amd.autograd import Tensor, default_ctx

    ctx = default_ctx()
    n = 1 << 28
    src, dst = Tensor.empty((n,), np.float32, ctx), Tensor.empty((n,), np.float32, ctx)
    check(lib.lumen_copy_f32(ctx.handle, dst.ptr, src.ptr, n))  # touch both
    iters = 10
    ctx.timer_start()
    for _ in range(iters):
        check(lib.lumen_copy_f32(ctx.handle, src.ptr, dst.ptr, n))
    ms = ctx.timer_stop() / iters
    print(json.dumps({"metric": "copy GB/s", "bytes_read": 4 * n, "bytes_written": 4 * n, "ms": round(ms, 4),
                      "GBps_read_plus_write": round(8 * n / ms / 1e6, 1)}))


GEMV_SHAPES = [(2048, 2048), (2048, 256), (2048, 5632), (5632, 2048), (2048, 32000), (4096, 11008), (11008, 4096)]


def gemv_microbench(args):
    """Isolated M=1 GEMV, fp32, logical (K, N) stored [N, K] like the reference's Linear weights.
    Each launch reads a different copy of W (>= 1.2 GB of copies in rotation) so the figure is HBM
    bandwidth, not L2 / memory-side-cache bandwidth; algorithmic bytes = 4 (K N + K + N)."""
    import ctypes as C

    import numpy as np

    from lumen_amd._lib import check, lib
    from lumen_amd.autograd import Tensor, default_ctx

    ctx = default_ctx()
    rows = []
    for K, N in GEMV_SHAPES:
        rng = np.random.default_rng(K * 100003 + N)
        W = (rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02))
        x = rng.standard_normal(K, dtype=np.float32)
        ncopies = 1 if args.resident else max(2, int(np.ceil(1.2e9 / W.nbytes)))
        slab = Tensor.empty((ncopies, N, K), np.float32, ctx)
        for c in range(ncopies):
            check(lib.lumen_upload(ctx.handle, slab.ptr + c * W.nbytes, W.ctypes.data, W.nbytes))
        xd, yd = Tensor.from_array_no_grad(x, ctx), Tensor.empty((N,), np.float32, ctx)
        ms = C.c_float()
        check(lib.lumen_gemv_bench(ctx.handle, slab.ptr, N * K, ncopies, 0, xd.ptr, yd.ptr, N, K, args.warmup or 8, C.byref(ms)))
        iters = max(args.steps, 200)
        check(lib.lumen_gemv_bench(ctx.handle, slab.ptr, N * K, ncopies, 0, xd.ptr, yd.ptr, N, K, iters, C.byref(ms)))
        ref = W.astype(np.float64) @ x.astype(np.float64)
        err = float(np.abs(yd.data() - ref).max() / np.abs(ref).max())
        us = ms.value * 1e3 / iters
        nbytes = 4.0 * (K * N + K + N)
        rows.append({"K": K, "N": N, "us": round(us, 3), "GBps": round(nbytes / us / 1e3, 1),
                     "frac_of_8TBps": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "max_rel_err": err,
                     "weight_copies": ncopies})
        del slab
    print(json.dumps({"metric": "M=1 GEMV HBM GB/s", "unit": "GB/s", "n_gpus": 1, "dtype": "f32", "data": "synthetic",
                      "layout": "[N,K] row-major (out,in)",
                      "weights": "one copy, cache-resident (not an HBM figure)" if args.resident else
                                 "copies in rotation (>= 1.2 GB): every launch reads from HBM",
                      "shapes": rows}))


GEMM_SHAPES = [(128, 2048, 2048), (128, 2560, 2048), (128, 11264, 2048), (128, 2048, 5632), (512, 2048, 2048),
               (512, 11264, 2048), (3968, 2048, 2048), (3968, 11264, 2048), (3968, 2048, 5632), (512, 4096, 4096)]


def gemm_microbench(args):
    """C[M,N] = A[M,K] W[N,K]^T at f32 accuracy on the matrix cores (the M > 1 branch of matmul, the prompt
    pass): M = prompt rows, (N, K) the projection shapes.  Useful flops 2 M N K; the kernel issues six bf16
    matrix products per f32 product, so its own bound is the bf16 peak / 6 = 417 TFLOP/s; the f32 matrix
    peak (157.3) is given for comparison."""
    import ctypes as C

    import numpy as np

    from lumen_amd._lib import check, lib
    from lumen_amd.autograd import Tensor, default_ctx

    ctx = default_ctx()
    rng = np.random.default_rng(0)
    rows = []
    for M, N, K in GEMM_SHAPES:
        A = rng.standard_normal((M, K), dtype=np.float32)
        W = rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.02)
        Ad, Wd = Tensor.from_array_no_grad(A, ctx), Tensor.from_array_no_grad(W, ctx)
        Cd = Tensor.empty((M, N), np.float32, ctx)
        ms = C.c_float()
        for iters in (3, 20):
            check(lib.lumen_timer_start(ctx.handle))
            for _ in range(iters):
                check(lib.lumen_gemm_f32(ctx.handle, Ad.ptr, Wd.ptr, Cd.ptr, M, N, K))
            check(lib.lumen_timer_stop(ctx.handle, C.byref(ms)))
        us = ms.value * 1e3 / 20
        ref = A[:32].astype(np.float64) @ W.T.astype(np.float64)
        err = float(np.abs(Cd.data()[:32] - ref).max() / np.abs(ref).max())
        tf = 2.0 * M * N * K / us / 1e6
        rows.append({"M": M, "N": N, "K": K, "us": round(us, 1), "TFLOPs": round(tf, 1),
                     "frac_of_mfma_bf16_peak": round(GEMM_BF16_PRODUCTS * tf / MFMA_BF16_PEAK_TF, 4),
                     "vs_mfma_fp32_peak": round(tf / MFMA_FP32_PEAK_TF, 4), "max_rel_err": err})
    print(json.dumps({"metric": "prompt-pass GEMM TFLOP/s at f32 accuracy", "unit": "TFLOP/s", "n_gpus": 1, "dtype": "f32",
                      "data": "synthetic", "mfma_bf16_peak_TFLOPs": MFMA_BF16_PEAK_TF,
                      "bf16_products_per_f32_product": GEMM_BF16_PRODUCTS, "mfma_fp32_peak_TFLOPs": MFMA_FP32_PEAK_TF,
                      "shapes": rows}))


def prefill_bench(args):
    """One long prompt pass: TinyLlama shape, 4096-row cache, 3968 random ids, last-row logits."""
    import numpy as np

    from lumen_amd import synth
    from lumen_amd.models import LlamaModel

    cfg = dict(synth.TINYLLAMA_1B_LONG)
    S = 3968 if args.prompt == 128 else args.prompt
    model = LlamaModel(cfg)
    for name, a in synth.iter_params(cfg, seed=0):
        model.set_param(name, a)
    ids = synth.make_tokens(S, cfg["vocab_size"], seed=0)
    # five passes in a row: the first sizes the workspaces and the GPU clock settles over the first three
    # (they run about 10 % slower); the figure is the mean of the last two
    passes = []
    for _ in range(5):
        model.reset_kv_caches()
        model.ctx.timer_start()
        model.forward(ids, all_rows=False)
        passes.append(model.ctx.timer_stop())
    ms = 0.5 * (passes[-1] + passes[-2])
    out = {"metric": "prompt tokens/s", "value": round(S / ms * 1e3, 1), "unit": "tokens/s", "n_gpus": 1,
           "dtype": "f32", "data": "synthetic", "warmup": 3, "steps": 2,
           "config": {"workload": "TinyLlama-1.1B-shaped Llama fp32 random-init seed 0, batch 1, one prompt pass of %d "
                                  "random ids into an empty cache of %d rows" % (S, cfg["max_seq_len"])}}
    out.update(prefill_report(cfg, S, ms))
    out["passes_ms"] = [round(x, 3) for x in passes]
    print(json.dumps(out))


def cpu_baseline(cfg, params, prompt, n_tokens, model):
    """The C restatement of Lumen's CPU path (row-parallel M=1 GEMV, head-parallel online-softmax
    attention) on the host cores: prefill the same prompt, then time n_tokens greedy decode steps.
    Its logits then check the GPU path of this very process: the same prompt and the same tokens through
    `model` (prompt pass, then one decode step per token), every row within 1e-4 or the run stops."""
    import numpy as np

    from oracle import lumen_oracle as lo

    ora = lo.Llama(cfg, params)
    rc, logits = ora.forward(prompt)
    assert rc == lo.LO_OK
    ref_rows = [logits[-1].copy()]
    tok = lo.argmax(logits[-1])
    toks = [tok]
    t0 = time.perf_counter()
    for _ in range(n_tokens):
        rc, lg = ora.forward(np.array([tok]))
        tok = lo.argmax(lg[0])
        ref_rows.append(lg[0].copy())
        toks.append(tok)
    dt = time.perf_counter() - t0
    model.reset_kv_caches()
    worst = 0.0
    for t, ref in enumerate(ref_rows):
        got = model.forward(prompt if t == 0 else np.array([toks[t - 1]]), all_rows=False)
        worst = max(worst, float(np.abs(got.astype(np.float64) - ref).max() / np.abs(ref).max()))
    if not worst <= 1e-4:
        raise SystemExit("bench: GPU logits differ from the CPU restatement's by %.3g (tolerance 1e-4)" % worst)
    return {"value": round(n_tokens / dt, 3), "unit": "tokens/s", "cores": lo.get_threads(), "kind": "port",
            "sample": "%d greedy decode tokens after the same %d-token prompt, same weights; C restatement of "
                      "Lumen's CPU algorithms (gcc -O3 -march=x86-64-v3 -ffp-contract=off, OpenMP), Rust toolchain "
                      "unavailable" % (n_tokens, len(prompt)),
            "gpu_logits_vs_cpu": {"rows": len(ref_rows), "max_rel_err": worst, "tolerance": 1e-4}}


if __name__ == "__main__":
    main()
