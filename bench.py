#!/usr/bin/env python3
"""Decode benchmark: batch-1 greedy decode of a synthetic Llama-3-8B-shaped Q4_K_S model on one
MI355X (the configuration the headline metric is quoted on).

    python bench.py [--gpus 1] [--steps 128] [--warmup 8] [--workload 8b-q4ks]

A step is one decode token (one pass of the per-token path).  The model (q4_K layers, q6_K output
projection, N(0, 0.02) weights, norms 1) is generated and quantized on the host cores, uploaded
once, then: a 32-token seeded prompt is fed (untimed), W warm-up tokens are decoded (untimed) and
exactly K tokens are decoded inside the timed region, with the weights and KV cache resident in
HBM.  One JSON line is printed on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E datasheet peak
# HBM traffic of the dominant kernel per launch, from rocprofv3 --pmc runs of this script (FETCH_SIZE x 2.000 KiB +
# WRITE_SIZE x 1.000 KiB per unit, the factors a plain read of known size gave in the same runs; the launches of the
# timed region):
#   (8b-q4ks, launch path 1): per matvec launch, 31.23 MB read + 0.04 MB written (profiles/pmc_fetch_write_bench_8b-q4ks.md)
#   launch path 3, per token launch (profiles/pmc_fetch_write_streaming_kernel_all_workloads.md):
#     8b-q4ks 4501.1 MB read + 30.3 MB written, 8b-q5km 5760.0 + 9.3, phi3-4k 5316.8 + 40.5 (per step: its launches run
#     eight), llama2c-f32 172.6 + 0.8,
#     8b-q4ks-prefill (its decode steps at positions 2048 and up) 5021.0 + 67.1
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {("8b-q4ks", 1): 31264000, ("8b-q4ks", 3): 4531362000, ("8b-q5km", 3): 5769380000,
                                     ("phi3-4k", 3): 5357300000, ("llama2c-f32", 3): 173480000,
                                     ("8b-q4ks-prefill", 3): 5088146000}

WORKLOADS = {
    # name: (plan, config kwargs, prompt length)
    "8b-q4ks": ("PLAN_Q4_K_S", dict(dim=4096, hidden_dim=14336, n_layers=32, n_heads=32, n_kv_heads=8,
                                    vocab_size=128256, seq_len=512, rope_freq_base=500000.0, rope_is_neox=False), 32),
    "8b-q5km": ("PLAN_Q5_K_M", dict(dim=4096, hidden_dim=14336, n_layers=32, n_heads=32, n_kv_heads=8,
                                    vocab_size=128256, seq_len=512, rope_freq_base=500000.0, rope_is_neox=False), 32),
    # the same shape with the tensor mix of a Q4_K_S file as llama.cpp is said to write it: attn_v and ffn_down of the
    # first four layers q5_K (typed pieces in the streaming kernel)
    "8b-q4ks-file": ("plan_q4_k_s_file", dict(dim=4096, hidden_dim=14336, n_layers=32, n_heads=32, n_kv_heads=8,
                                              vocab_size=128256, seq_len=512, rope_freq_base=500000.0, rope_is_neox=False), 32),
    # and with that of a Q4_K_M file: attn_v and ffn_down q6_K in about half of the layers
    "8b-q4km-file": ("plan_q4_k_m_file", dict(dim=4096, hidden_dim=14336, n_layers=32, n_heads=32, n_kv_heads=8,
                                              vocab_size=128256, seq_len=512, rope_freq_base=500000.0, rope_is_neox=False), 32),
    "llama2c-f32": ("PLAN_F32", dict(dim=512, hidden_dim=1376, n_layers=8, n_heads=8, n_kv_heads=8, vocab_size=32000,
                                     seq_len=1024, rope_freq_base=10000.0, rope_is_neox=False), 16),
    # Phi-3-mini shape, no GQA, neox RoPE, 4096-long cache pre-filled with 3840 seeded rows: attention-dominated
    "phi3-4k": ("PLAN_Q4_K", dict(dim=3072, hidden_dim=8192, n_layers=32, n_heads=32, n_kv_heads=32, vocab_size=32064,
                                  seq_len=4096, rope_freq_base=10000.0, rope_is_neox=True), 3841),
    # the headline model with a 4096-long cache: a 2048-token prompt goes through the batched prompt pass
    # (bf16 MFMA products), then tokens are decoded on top of it
    "8b-q4ks-prefill": ("PLAN_Q4_K_S", dict(dim=4096, hidden_dim=14336, n_layers=32, n_heads=32, n_kv_heads=8,
                                            vocab_size=128256, seq_len=4096, rope_freq_base=500000.0,
                                            rope_is_neox=False), 2048),
    # small shape for a quick functional run of this script
    "tiny-q4ks": ("PLAN_Q4_K_S", dict(dim=512, hidden_dim=1024, n_layers=4, n_heads=8, n_kv_heads=2, vocab_size=2048,
                                      seq_len=512, rope_freq_base=500000.0, rope_is_neox=False), 32),
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def w_elems(lm):
    """weights (elements) one position multiplies: every matrix of every layer + the classifier"""
    n = 0
    for lw in lm.weights.layers:
        for name in ("wq", "wk", "wv", "wo", "w1", "w2", "w3"):
            mtx = getattr(lw, name)
            n += int(np.prod(mtx.shape)) if not hasattr(mtx, "ne0") else mtx.ne0 * mtx.ne1
    o = lm.weights.output_weight
    n += int(np.prod(o.shape)) if not hasattr(o, "ne0") else o.ne0 * o.ne1
    return n


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default="8b-q4ks", choices=sorted(WORKLOADS))
    ap.add_argument("--repeats", type=int, default=3, help="timed regions; the median is reported")
    ap.add_argument("--path", type=int, default=0, help="0 auto, 1 kernel per phase, 2 persistent kernel, 3 streaming kernel")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--kv", default="fp32", choices=["fp32", "fp16"],
                    help="element type of the KV cache: fp32 as the reference's, or the fp16 option (launch paths 1 and 3)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on exactly one GPU (batch-1 decode of one sequence is not sharded here); "
            "--gpus %d is not supported" % args.gpus)
        sys.exit(2)

    pkg = entry.load_package()
    from llama2_jl_amd import _lib, synth
    plan_name, kw, n_prompt = WORKLOADS[args.workload]
    cfg = pkg.ModelConfig(**kw)
    K, W = args.steps, args.warmup
    if n_prompt - 1 + W + K > cfg.seq_len:
        log("steps + warmup + prompt exceed seq_len %d" % cfg.seq_len)
        sys.exit(2)

    ctx = pkg.default_context()
    info = ctx.device_info()
    log("device:", info)
    t0 = time.time()
    plan = getattr(synth, plan_name)
    if callable(plan):
        plan = plan(cfg.n_layers)
    # (norm weights all ones, as the benchmark configurations say)
    lm = synth.synthetic_model(cfg, plan, seed=20240607,
                               share_classifier=(plan_name == "PLAN_F32"), norm_spread=0.0)
    log("model generated + quantized on %d host threads in %.1f s" % (synth._threads(), time.time() - t0))
    t0 = time.time()
    dev = lm.device(path=args.path, kv_fp16=(args.kv == "fp16"))
    ctx.sync()
    log("uploaded in %.1f s; launch path %d (1 = kernel per phase, 2 = persistent kernel, 3 = streaming kernel)%s"
        % (time.time() - t0, dev.path, "; not 3 because: " + dev.path_reason if dev.path_reason else ""))

    w_bytes = synth.weight_bytes_per_token(lm)
    kv_dim = cfg.dim // cfg.n_heads * cfg.n_kv_heads
    # a prompt longer than 256 stands for a pre-filled cache: all but its last position are written
    # as seeded random K/V rows, and a single prompt token is fed at the next position
    use_prefill = args.workload.endswith("-prefill")
    n_pre = n_prompt - 1 if (n_prompt > 256 and not use_prefill) else 0
    prompt = synth.seeded_prompt(99, n_prompt - n_pre, cfg.vocab_size)
    if n_pre:
        rng = np.random.default_rng(7)
        for layer in range(cfg.n_layers):
            kv = rng.standard_normal((2, n_pre, kv_dim), dtype=np.float32)
            dev.kv_write(layer, 0, kv[0], kv[1])
        log("cache pre-filled with %d positions" % n_pre)

    # ---- batched prompt pass (only the -prefill workload): timed on its own, then decoding goes on
    # from the cache it wrote ------------------------------------------------------------------------
    prefill = None
    if use_prefill:
        pf_times = []
        for rep in range(max(2, args.repeats)):
            dev.reset()
            ctx.sync()
            t_start = time.perf_counter()
            _, nxt = dev.prefill(prompt, 0, want_logits=False)
            pf_times.append(time.perf_counter() - t_start)
            log("prompt pass %d: %d positions in %.1f ms" % (rep, n_prompt, pf_times[-1] * 1e3))
        pf_dt = float(np.min(pf_times[1:]))  # the first call also allocates its buffers
        hs = cfg.dim // cfg.n_heads
        gemm_flop = 2.0 * n_prompt * (w_elems(lm) - cfg.vocab_size * cfg.dim)
        attn_flop = 4.0 * cfg.n_layers * cfg.n_heads * hs * n_prompt * (n_prompt + 1) / 2.0
        prefill = {"positions": n_prompt, "ms": round(pf_dt * 1e3, 2), "tok_s": round(n_prompt / pf_dt, 1),
                   "TFLOP/s": round((gemm_flop + attn_flop) / pf_dt / 1e12, 1), "gemm_TFLOP": round(gemm_flop / 1e12, 2),
                   "attention_TFLOP": round(attn_flop / 1e12, 2), "peak_bf16_TFLOP/s": 2500.0,
                   "frac_of_mfma_peak": round((gemm_flop + attn_flop) / pf_dt / 2.5e15, 4),
                   # q|k|v, wo and w2 through hipBLASLt (the default where it can be opened; L2H_PF_LIBRARY=0: own kernels);
                   # w1|w3 + SwiGLU and the attention are this library's kernels either way
                   "plain_products": "hipBLASLt" if dev.prefill_library else "own kernels"}
        # the other forms of the same pass, one call each after a warm-up call: this library's product kernels for every
        # product, and the quantized blocks expanded inside the product kernel (no bf16 copy read)
        def other_form(library, copy):
            dev.set_prefill_library(library)
            dev.set_prefill_copy(copy)
            ts = []
            for _ in range(2):
                dev.reset()
                ctx.sync()
                t0 = time.perf_counter()
                dev.prefill(prompt, 0, want_logits=False)
                ts.append(time.perf_counter() - t0)
            return round(min(ts) * 1e3, 2)
        was_library = dev.prefill_library
        prefill["own_product_kernels_ms"] = other_form(False, True) if was_library else prefill["ms"]
        prefill["dequantized_in_the_product_kernel_ms"] = other_form(False, False)
        dev.set_prefill_library(True)
        dev.set_prefill_copy(True)
        dev.reset()
        _, nxt = dev.prefill(prompt, 0, want_logits=False)  # (the cache the decode steps continue from: the default form's)
        log("prompt pass:", json.dumps(prefill))
        prompt = np.array([nxt], np.int32)
        n_pre = n_prompt  # the cache now holds the whole prompt; decoding starts at the next position
        n_prompt = n_pre + 1

    # ---- timed region: K decode tokens after the prompt and W warm-up tokens --------------------
    times, ev_times, tokens = [], [], None
    for rep in range(args.repeats):
        if not n_pre:
            dev.reset()
        # prompt + warm-up tokens, untimed
        warm = dev.generate_greedy(prompt, W, pos0=n_pre) if W > 0 else np.zeros(0, np.int32)
        # next step: position pos0, fed with the last warm-up token (or the last prompt token)
        pos0 = n_prompt - 1 + W
        first = int(warm[-1]) if W > 0 else int(prompt[-1])
        ctx.sync()
        t_start = time.perf_counter()
        # (HIP events on the library's stream bracket the same K launches that the host clock wraps)
        ids, ev = dev.generate_greedy([first], K, pos0=pos0, timed=True)
        ctx.sync()
        dt = time.perf_counter() - t_start
        times.append(dt)
        ev_times.append(ev)
        if tokens is None:
            tokens = ids.tolist()
        elif tokens != ids.tolist():
            log("WARNING: repeat %d produced different tokens" % rep)
        log("repeat %d: %d tokens in %.2f ms -> %.1f tok/s" % (rep, K, dt * 1e3, K / dt))
    dt = float(np.median(times))
    tok_s = K / dt
    # positions read by the timed steps: pos0 .. pos0+K-1, each reads pos+1 cache rows
    kv_bytes = 2 * cfg.n_layers * kv_dim * (2 if args.kv == "fp16" else 4) * (pos0 + 1 + (K - 1) / 2.0)
    bytes_per_token = w_bytes + kv_bytes
    roofline_tok_s = HBM_PEAK_GBS * 1e9 / bytes_per_token

    # ---- dominant kernel -----------------------------------------------------------------------------
    # launch path 3: one launch per token does everything; its duration comes from HIP events around the K launches
    # of the timed region, on the library's stream; its algorithmic bytes are the token's
    ev_ms = ev_times[int(np.argsort(times)[len(times) // 2])]  # (of the repeat whose host time is the median)
    # the k-quant (or fp32) matvec of every phase, timed with HIP events on the library's stream, every layer's
    # tensor in turn so that nothing is cache-resident
    roles = [("qkv", _lib.WQ), ("wo", _lib.WO), ("w1w3", _lib.W1), ("w2", _lib.W2), ("output", _lib.OUTPUT)]
    per_kernel, tot_us, tot_b, n_launch = {}, 0.0, 0, 0
    dominant_type = lm.weights.layers[0].w1.type if hasattr(lm.weights.layers[0].w1, "type") else 0
    for name, role in roles:
        us, b = dev.profile_matvec(role, iters=10)
        per_kernel[name] = {"us": round(us, 2), "MB": round(b / 1e6, 2), "GB/s": round(b / us / 1e3, 1)}
        out_type = lm.weights.output_weight.type if hasattr(lm.weights.output_weight, "type") else 0
        if name != "output" or out_type == dominant_type:
            mult = cfg.n_layers if name != "output" else 1
            tot_us += us * mult
            tot_b += b * mult
            n_launch += mult
    log("per-launch matvec timings:", json.dumps(per_kernel))
    achieved = tot_b / tot_us / 1e3  # GB/s over the launches of the dominant kernel within one token
    kernel_name = "matvec_kq_kernel (k-quant x q8_K dequant-matvec)"
    bytes_per_launch, launches, avg_launch_us = int(tot_b / max(1, n_launch)), n_launch, tot_us / max(1, n_launch)
    if dev.path == 3:
        kernel_name = "flow_token_kernel (whole token: q4_K/q6_K x q8_K matvecs, attention, argmax)"
        # (a kernel launch runs dev.steps_per_launch steps of the token loop; bytes, traffic and time are per step)
        bytes_per_launch, launches, avg_launch_us = int(bytes_per_token), 1, ev_ms * 1e3 / K
        achieved = bytes_per_launch / avg_launch_us / 1e3
        log("streaming kernel: %.1f us per launch (HIP events), %.0f GB/s of algorithmic bytes" % (avg_launch_us, achieved))
    stream_us = pkg.lib().l2h_profile_stream_read
    import ctypes
    us = ctypes.c_float()
    ctx.check(stream_us(ctx.handle, 2 << 30, 5, ctypes.byref(us)))
    stream_gbs = (2 << 30) / us.value / 1e3
    log("plain streaming read of 2 GiB: %.0f GB/s" % stream_gbs)

    # ---- CPU baseline: the oracle in the reference's own arithmetic (float activations, fp32
    # sums), rows split over the host threads like Threads.@threads; a bounded number of tokens ---
    cpu = None
    if args.cpu_seconds > 0:
        orc = entry.load_oracle()
        cores = synth._threads()
        om = orc.model_from_language_model(lm, nthreads=cores)
        n_tok, t_cpu = 0, 0.0
        t_begin = time.perf_counter()
        while n_tok < 16 and (n_tok < 2 or t_cpu < args.cpu_seconds):
            om.forward(int(prompt[n_tok % len(prompt)]), n_tok, orc.REFERENCE)
            n_tok += 1
            t_cpu = time.perf_counter() - t_begin
        cpu = {"value": round(n_tok / t_cpu, 3), "unit": "tok/s", "cores": cores, "kind": "port",
               "sample": "%d decode steps (positions 0..%d) of the same model, C restatement of the Julia CPU path "
                         "(float activations, fp32 sums, rows split over %d threads); Julia itself is not installed"
                         % (n_tok, n_tok - 1, cores)}
        log("cpu baseline:", cpu)
        om.close()

    # HBM traffic of the dominant kernel per launch (FETCH_SIZE + WRITE_SIZE, scaled), measured with
    # rocprofv3 --pmc on this workload with its fp32 cache (null for a combination that no counter run covers)
    traffic = MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get((args.workload, dev.path)) if args.kv == "fp32" else None

    result = {
        "metric": "decode tok/s, Llama-3-8B-shape Q4_K_S, batch 1; % of HBM-BW roofline",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(dt * 1e3 / K, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot products (q4_K/q6_K x q8_K), fp64 accumulation, fp32 activations",
        "data": "synthetic",
        "config": {"workload": args.workload, "shape": kw, "plan": plan_name, "prompt_tokens": n_prompt,
                   "decode_positions": [pos0, pos0 + K - 1], "repeats": args.repeats, "launch_path": dev.path,
                   "kv_cache": args.kv,
                   "bytes_per_token": int(bytes_per_token), "weight_bytes_per_token": int(w_bytes),
                   "roofline_tok_s_at_8TBs": round(roofline_tok_s, 1),
                   "frac_of_roofline": round(tok_s / roofline_tok_s, 4),
                   "tokens_head": tokens[:8]},
        "roofline": {"bound": "hbm", "kernel": kernel_name,
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "bytes_per_launch": bytes_per_launch, "launches_per_token": launches,
                     "token_steps_per_kernel_launch": getattr(dev, "steps_per_launch", 1),
                     "avg_launch_us": round(avg_launch_us, 2), "per_phase_kernels": per_kernel,
                     "measured_stream_read_GBs": round(stream_gbs, 1)},
        "cpu_baseline": cpu,
    }
    if prefill:
        result["prefill"] = prefill
    print(json.dumps(result), flush=True)
    # release the device objects in order while the interpreter is still whole
    dev.close()
    ctx.sync()


if __name__ == "__main__":
    main()
