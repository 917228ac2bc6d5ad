"""Measurement of the engine on one MI355X: decode tokens/s at batch 8 (the headline), with
prefill tokens/s at 2,048 tokens and decode at batch 1 and 64 beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--shape 8b|14b|32b]

The model has the layer sizes of Qwen3-8B (the headline configuration) with random
weights drawn on the device; prompts are seeded uniform-random token ids of 1,024 tokens;
a "step" is one decode step of the whole engine (scheduler, step function, sampling).
It prints ONE JSON line.  More than one GPU is not supported: it says so and exits with 2.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN3_8B = dict(
    architectures=["Qwen3ForCausalLM"], num_hidden_layers=36, hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1000000.0,
    rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=40960,
)
# the layer sizes of Qwen3-14B and Qwen3-32B, for runs at further sizes: --shape
SHAPES = {
    "8b": ("Qwen3-8B-shaped", QWEN3_8B),
    "14b": ("Qwen3-14B-shaped", dict(QWEN3_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40,
                                     intermediate_size=17408)),
    "32b": ("Qwen3-32B-shaped", dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64,
                                     intermediate_size=25600)),
}
PROMPT_LEN = 1024
MAX_CONTEXT = 8192
PREFILL_TOKENS = 2048


def weight_bytes(cfg, layers, itemsize):
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    per_layer = (nq + 2 * nkv) * d * h + h * nq * d + 3 * i * h
    return (per_layer * layers + v * h) * itemsize, per_layer


def sync():
    import torch

    torch.cuda.synchronize()


def measure_decode(llm, batch, steps, warmup, rng, vocab, prompt_len=PROMPT_LEN):
    """Tokens/s of ``steps`` decode steps at ``batch`` after prefilling 1,024-token prompts."""
    from jax_vllm_amd import SamplingParams

    prompts = [rng.integers(0, vocab, size=prompt_len).tolist() for _ in range(batch)]
    # the first requests decode while the others' prompts run, about two prompts a step: nobody may finish meanwhile
    sp = SamplingParams(max_new_tokens=warmup + steps + max(128, batch))
    for p in prompts:
        llm.add_request(p, sp)
    while any(r.num_remaining > 1 or not r.output_ids for r in llm.scheduler.running) or llm.scheduler.waiting:
        llm.step()  # prefill, untimed
    for _ in range(warmup):
        llm.step()
    sync()
    ctx_start = sum(r.num_computed for r in llm.scheduler.running) / batch
    t0 = time.perf_counter()
    for _ in range(steps):
        ev = llm.step()
        assert len(ev) == batch
    sync()
    dt = time.perf_counter() - t0
    llm.abort_all()
    mean_ctx = ctx_start + (steps - 1) / 2.0
    return batch * steps / dt, dt / steps, mean_ctx


def measure_prefill(llm, rng, vocab, repeats=3):
    """Seconds of one 2,048-token prompt through the step function: the median of ``repeats`` runs
    after one that warms up."""
    from jax_vllm_amd.engine.entries import StepEntry

    core = llm.core
    times = []
    for i in range(repeats + 1):
        toks = rng.integers(0, vocab, size=PREFILL_TOKENS).tolist()
        rid = f"prefill{i}"
        core.start_request(rid)
        sync()
        t0 = time.perf_counter()
        core.run([StepEntry(rid, toks, [PREFILL_TOKENS - 1])])
        sync()
        dt = time.perf_counter() - t0
        core.finish_request(rid)
        if i > 0:  # the first run warms up
            times.append(dt)
    return sorted(times)[len(times) // 2]


KERNEL_GROUPS = (          # substring of a kernel's name -> what it is counted as
    ("gemm_skinny", "products_own"), ("gemm_tile64", "products_own"), ("gemm_rows", "products_own"),
    ("gemm_f32", "products_own"),
    ("Cijk", "products_library"), ("rocblas", "products_library"), ("hipblaslt", "products_library"),
    ("attn_", "attention"), ("paged_attention", "attention"),
    ("add_rmsnorm", "norm_residual"), ("add_parts", "norm_residual"), ("rmsnorm", "norm_residual"),
    ("qk_norm_rope", "rope_kv_write"), ("rope_table", "rope_kv_write"), ("v_pages_write", "rope_kv_write"),
    ("gated_mul", "activation"), ("embedding", "embedding"), ("sample_", "sampling"), ("add_bias", "bias"),
)


def kernel_shares(run) -> dict:
    """Share of the GPU's kernel time by kind of kernel while ``run()`` executes (torch's profiler over
    the HIP activity records; kernels of replayed graphs are seen too)."""
    import torch
    from torch.profiler import ProfilerActivity, profile

    sync()
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        run()
        sync()
    totals = {}
    for e in prof.key_averages():
        t = float(getattr(e, "self_device_time_total", 0.0))
        if t <= 0.0 or str(e.device_type).endswith("CPU"):
            continue
        group = next((g for key, g in KERNEL_GROUPS if key in e.key), "other")
        totals[group] = totals.get(group, 0.0) + t
    whole = sum(totals.values()) or 1.0
    return {g: round(t / whole, 4) for g, t in sorted(totals.items(), key=lambda kv: -kv[1])}


def calibrate(device="cuda") -> dict:
    """What a plain streaming read and a plain matrix-core loop reach on this box: GB/s of a kernel that
    only reads (8 buffers of 201 MB in turn, the size of one gate/up weight: nothing comes from a cache)
    and TFLOP/s of a kernel that only issues bf16 MFMA on registers."""
    import torch

    from jax_vllm_amd.ops import kernels as K

    sink = torch.zeros(4, dtype=torch.float32, device=device)
    nbytes = 2 * 12288 * 4096 * 2
    buffers = [torch.zeros(nbytes // 2, dtype=torch.bfloat16, device=device) for _ in range(8)]
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for b in buffers:
        K.calibrate_read(b, sink)
    sync()
    start.record()
    for _ in range(4):
        for b in buffers:
            K.calibrate_read(b, sink)
    end.record()
    sync()
    read_gbs = 32 * nbytes / (start.elapsed_time(end) * 1e-3) / 1e9
    blocks, turns = 256 * 8, 4096
    K.calibrate_mfma(sink, turns, blocks)
    sync()
    start.record()
    flops = sum(K.calibrate_mfma(sink, turns, blocks) for _ in range(4))
    end.record()
    sync()
    tflops = flops / (start.elapsed_time(end) * 1e-3) / 1e12
    del buffers
    return {"hbm_read_gbs": round(read_gbs, 1), "hbm_read_frac_of_peak": round(read_gbs / PEAK_HBM_GBS, 4),
            "mfma_bf16_tflops": round(tflops, 1), "mfma_frac_of_peak": round(tflops * 1e12 / PEAK_FLOPS["bf16"], 4)}


def measure_ttft(llm, rng, vocab, prompt_len=2048, shared=1024):
    """Time to the first token of a prompt, cold (nothing of it in the cache) and warm (its first
    ``shared`` tokens were another request's prompt prefix and are taken from the cache); the
    reference's harness measures this pair over HTTP (scripts/bench_vllm.py:728-789)."""
    from jax_vllm_amd import SamplingParams

    one = SamplingParams(max_new_tokens=1)
    llm.generate([rng.integers(0, vocab, size=prompt_len).tolist()], one)      # warms the kernels, shares nothing
    prefix = rng.integers(0, vocab, size=shared).tolist()
    out = {}
    for name in ("cold", "warm"):
        prompt = prefix + rng.integers(0, vocab, size=prompt_len - shared).tolist()
        hits = llm.stats.cache_hit_tokens
        sync()
        t0 = time.perf_counter()
        llm.generate([prompt], one)
        sync()
        out[f"{name}_ttft_ms"] = round((time.perf_counter() - t0) * 1e3, 3)
        out[f"{name}_cache_hit_tokens"] = llm.stats.cache_hit_tokens - hits
    out.update(prompt_len=prompt_len, shared_prefix=shared)
    return out


def measure_long_prompt(llm, rng, vocab, prompt_len):
    """One prompt of ``prompt_len`` tokens through the engine in portions of the token budget, from the
    request's arrival to its first token (a short prompt first, untimed, so that nothing is set up
    inside the timed part)."""
    from jax_vllm_amd import SamplingParams

    one = SamplingParams(max_new_tokens=1)
    llm.generate([rng.integers(0, vocab, size=llm.config.max_num_batched_tokens).tolist()], one)
    sync()
    prompt = rng.integers(0, vocab, size=prompt_len).tolist()
    t0 = time.perf_counter()
    llm.add_request(prompt, one)
    steps, last = 0, 0.0
    while llm.has_work():
        t1 = time.perf_counter()
        llm.step()
        sync()
        last, steps = time.perf_counter() - t1, steps + 1
    dt = time.perf_counter() - t0
    return {"prompt_tokens_per_s": round(prompt_len / dt, 1), "seconds": round(dt, 4), "prompt_len": prompt_len,
            "portions": steps, "last_portion_ms": round(last * 1e3, 3)}


def measure_mixed(llm, rng, vocab, running=32, joining=4, join_len=3000, shared=1024):
    """A continuous-batching mix: ``running`` requests decode at contexts
    uniform in [512, 4096] when ``joining`` prompts of ``join_len`` tokens arrive, two of which share
    their first ``shared`` tokens; timed from their arrival until all of them have their first token."""
    from jax_vllm_amd import SamplingParams

    keep = SamplingParams(max_new_tokens=256)   # far more than the steps this takes
    first = [llm.add_request(rng.integers(0, vocab, size=int(n)).tolist(), keep)
             for n in rng.integers(512, 4097, size=running)]
    while any(not llm.requests[r].output_ids for r in first):
        llm.step()
    for _ in range(8):                       # decode steps of the running requests alone (captured)
        llm.step()
    sync()
    prefix = rng.integers(0, vocab, size=shared).tolist()
    prompts = [rng.integers(0, vocab, size=join_len).tolist() for _ in range(joining)]
    for p in prompts[-2:]:
        p[:shared] = prefix
    before = (llm.stats.prefill_tokens, llm.stats.decode_tokens, llm.stats.cache_hit_tokens)
    t0 = time.perf_counter()
    new = [llm.add_request(p, SamplingParams(max_new_tokens=64)) for p in prompts]
    steps, longest, last = 0, 0.0, t0
    while any(not llm.requests[r].output_ids for r in new):
        llm.step()
        sync()
        now = time.perf_counter()
        longest, last, steps = max(longest, now - last), now, steps + 1
    dt = time.perf_counter() - t0
    pre, dec, hit = (a - b for a, b in zip((llm.stats.prefill_tokens, llm.stats.decode_tokens,
                                            llm.stats.cache_hit_tokens), before))
    return {"mixed_tokens_per_s": round((pre + dec) / dt, 1), "steps": steps, "ms_per_step": round(dt / steps * 1e3, 3),
            "longest_step_ms": round(longest * 1e3, 3), "prompt_tokens_computed": pre, "decoded_tokens": dec,
            "cache_hit_tokens": hit, "running": running, "joining": joining}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="8b",
                    help="layer sizes: 8b is the headline configuration, the others are for runs at further sizes")
    ap.add_argument("--layers", type=int, default=None,
                    help="run only the first layers of the shape's (both numbers are reported in config)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--skip-points", action="store_true", help="measure the headline batch only")
    ap.add_argument("--tune-library", action="store_true",
                    help="prewarm the engine with the matrix library timing its own kernels (steps of more than 64 rows)")
    ap.add_argument("--no-kernel-share", action="store_true", help="leave out the per-kernel time shares")
    ap.add_argument("--only", choices=["prefill", "decode", "mixed", "long-prompt", "ttft", "calibrate"], default=None,
                    help="run one phase alone and print its result (for profiling); mixed: 32 running decodes "
                         "joined by 4 prompts of 3,000 tokens in portions of 512 under a budget of 2,048; "
                         "long-prompt: one prompt of --prompt-len tokens (default 32,768) in portions of 2,048; "
                         "ttft: time to first token of a 2,048-token prompt, cold and with its first 1,024 tokens "
                         "in the cache; calibrate: the plain read and matrix-core rates of this box")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--prompt-len", type=int, default=None,
                    help="with --only decode: prompt length of the decoding requests (long-context runs, default "
                         "1,024); with --only long-prompt: the prompt's length")
    args = ap.parse_args()
    if args.prompt_len is None:
        args.prompt_len = 32768 if args.only == "long-prompt" else PROMPT_LEN
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {max(args.gpus, world)} is not supported")
        sys.exit(2)

    import numpy as np
    import torch

    from jax_vllm_amd import LLM

    model_name, shape = SHAPES[args.shape]
    cfg = dict(shape)
    layers = args.layers if args.layers is not None else shape["num_hidden_layers"]
    cfg["num_hidden_layers"] = layers
    vocab = cfg["vocab_size"]
    rng = np.random.default_rng(0)
    max_batch = args.batch if (args.skip_points or args.only) else max(64, args.batch)
    block = 16
    if args.only == "calibrate":
        print(json.dumps(calibrate()), flush=True)
        return
    if args.only == "ttft":
        llm = LLM(cfg, random_seed=0, dtype=args.dtype, block_size=block, max_num_seqs=4, max_model_len=4096,
                  num_blocks=1 + 4 * (4096 // block), max_num_batched_tokens=2048, enable_prefix_cache=True)
        res = measure_ttft(llm, rng, vocab)
        res.update(model=model_name, layers=layers)
        print(json.dumps(res), flush=True)
        return
    if args.only == "mixed":
        llm = LLM(cfg, random_seed=0, dtype=args.dtype, block_size=block, max_num_seqs=36, max_model_len=8192,
                  num_blocks=1 + 32 * (4608 // block) + 4 * (3200 // block), max_num_batched_tokens=2048,
                  max_chunk=512, enable_prefix_cache=True)
        res = measure_mixed(llm, rng, vocab)
        res.update(model=model_name, layers=layers)
        print(json.dumps(res), flush=True)
        return
    llm = LLM(cfg, random_seed=0, dtype=args.dtype, block_size=block, max_num_seqs=max_batch,
              max_model_len=max(MAX_CONTEXT, args.prompt_len + 2 * 1024),
              num_blocks=1 + max_batch * (-(-(args.prompt_len + 2 * 1024) // block)),
              max_num_batched_tokens=max(PREFILL_TOKENS, max_batch), enable_prefix_cache=False,
              tune_library=args.tune_library)
    if args.tune_library:
        llm.prewarm()
    itemsize = 2 if args.dtype == "bf16" else 4
    wbytes, per_layer_params = weight_bytes(cfg, layers, itemsize)
    kv_per_token = llm.core.kv_bytes_per_token

    if args.only == "long-prompt":
        res = measure_long_prompt(llm, rng, vocab, args.prompt_len)
        res.update(model=model_name, layers=layers)
        print(json.dumps(res), flush=True)
        return
    if args.only == "prefill":
        pre_s = measure_prefill(llm, rng, vocab)
        print(json.dumps({"prefill_ms": round(pre_s * 1e3, 3), "tokens": PREFILL_TOKENS, "layers": layers}), flush=True)
        return
    if args.only == "decode":
        tps, step_s, mean_ctx = measure_decode(llm, args.batch, args.steps, args.warmup, rng, vocab, args.prompt_len)
        print(json.dumps({"decode_tokens_per_s": round(tps, 1), "ms_per_step": round(step_s * 1e3, 4),
                          "batch": args.batch, "mean_context": round(mean_ctx, 1), "layers": layers}), flush=True)
        return

    # prefill of 2,048 tokens
    pre_s = measure_prefill(llm, rng, vocab)
    h, nq, d = cfg["hidden_size"], cfg["num_attention_heads"], cfg["head_dim"]
    t = PREFILL_TOKENS
    flops = 2.0 * t * per_layer_params * layers + 4.0 * nq * d * (t * (t + 1) / 2.0) * layers + 2.0 * vocab * h
    prefill = {"value": round(t / pre_s, 1), "tokens": t, "ms": round(pre_s * 1e3, 3),
               "frac": round(flops / pre_s / PEAK_FLOPS[args.dtype], 4)}

    # decode: headline batch, then the other points
    tps, step_s, mean_ctx = measure_decode(llm, args.batch, args.steps, args.warmup, rng, vocab)
    read_bytes = wbytes + args.batch * mean_ctx * kv_per_token
    achieved = read_bytes / step_s / 1e9
    points, detail = {}, {}
    if not args.skip_points:
        n = min(args.steps, 128)
        # batch 1 and 64 from 1,024-token prompts; batch 8 near the benchmark context of 8,192 tokens
        for name, b, plen, k in (("decode_b1", 1, PROMPT_LEN, n), ("decode_b64", 64, PROMPT_LEN, n),
                                 ("decode_b8_ctx8k", 8, 7900, min(n, 64))):
            p_tps, p_step, p_ctx = measure_decode(llm, b, k, min(args.warmup, 8), rng, vocab, plen)
            p_bytes = wbytes + b * p_ctx * kv_per_token
            points[name] = round(p_tps, 1)
            detail[name] = {"tok_s": round(p_tps, 1), "ms_per_step": round(p_step * 1e3, 4), "batch": b,
                            "mean_context": round(p_ctx, 1), "gb_read": round(p_bytes / 1e9, 3),
                            "frac": round(p_bytes / p_step / 1e9 / PEAK_HBM_GBS, 4)}
    # the line's headline is measured by now: what follows is told beside it, and says so instead of ending the run
    # if the box's profiler or the calibration kernels fail
    shares = None
    if not args.no_kernel_share:
        from jax_vllm_amd import SamplingParams
        from jax_vllm_amd.engine.entries import StepEntry

        try:
            for _ in range(args.batch):
                llm.add_request(rng.integers(0, vocab, size=PROMPT_LEN).tolist(), SamplingParams(max_new_tokens=64))
            while any(r.num_remaining > 1 or not r.output_ids for r in llm.scheduler.running) or llm.scheduler.waiting:
                llm.step()
            for _ in range(4):
                llm.step()
            shares = {"decode": kernel_shares(lambda: [llm.step() for _ in range(8)])}
            llm.abort_all()
            toks = rng.integers(0, vocab, size=PREFILL_TOKENS).tolist()
            llm.core.start_request("share")
            shares["prefill"] = kernel_shares(lambda: llm.core.run([StepEntry("share", toks, [PREFILL_TOKENS - 1])]))
            llm.core.finish_request("share")
        except Exception as e:      # noqa: BLE001
            shares = {"error": f"{type(e).__name__}: {e}"[:200]}
    try:
        calibration = calibrate()
    except Exception as e:          # noqa: BLE001
        calibration = {"error": f"{type(e).__name__}: {e}"[:200]}

    line = {
        "metric": "decode_tokens_per_s", "value": round(tps, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: seeded uniform-random token ids, random-init weights N(0,0.02), norms 1+N(0,0.02); "
                "prefill: median of 3 runs through the step function; decode: the whole engine",
        "config": {
            "model": model_name, "layers": layers, "layers_full": shape["num_hidden_layers"],
            "hidden": cfg["hidden_size"], "q_heads": nq, "kv_heads": cfg["num_key_value_heads"], "head_dim": d,
            "intermediate": cfg["intermediate_size"], "vocab": vocab, "global_batch": args.batch,
            "seq_len": PROMPT_LEN, "max_context": MAX_CONTEXT, "mean_decode_context": round(mean_ctx, 1),
            "page_size": block, "parallelism": "single-gpu", "rope_theta": cfg["rope_theta"],
            "hip_graphs": bool(llm.config.use_hip_graphs),
            "decode_ahead": bool(llm.config.decode_ahead),
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
        "points_detail": detail,
        "calibration": calibration,
        "kernel_share": shares,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
