"""Decode and prefill throughput of the Llama-3.2-1B shape on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The headline value is decoded tokens per second at batch 8 with every request near the
benchmark context (4,096 positions): W untimed decode steps, then exactly K timed ones through
the engine (schedule, forward from the paged cache, on-device greedy sampling, token fed
back), bracketed by device synchronisation.  On the same line: a 2,048-token prefill with its
fraction of the bf16 matrix peak, the decode step's achieved fraction of the HBM roofline
(bytes that must be read: every weight once plus the live requests' cache), and decode
throughput at batch 1 and 64 after 512-token prompts.  Weights are random (N(0, 0.02)),
prompts are uniform random token ids.

    python bench.py --serve --model llama-3.2-3b --max-batched-tokens 512

measures another workload instead (its own JSON line): R requests with prompts of uniform
random length under continuous batching with chunked prefill, N new tokens each with seeded
temperature sampling, timed from the first request's arrival to the last one's end."""
import argparse
import copy
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_GBPS = 8000.0            # MI355X HBM3E, published
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="llama-3.2-1b", help="preset name")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the preset")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points-context", type=int, default=512)
    ap.add_argument("--skip-points", action="store_true")
    ap.add_argument("--skip-prefill", action="store_true")
    ap.add_argument("--max-batched-tokens", type=int, default=8192,
                    help="token budget of the engine steps that prefill the decode runs")
    ap.add_argument("--serve", action="store_true",
                    help="time a batch of requests through Engine.generate instead")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--min-prompt", type=int, default=128)
    ap.add_argument("--max-prompt", type=int, default=2048)
    ap.add_argument("--new-tokens", type=int, default=256)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (single-GPU engine)")
        return 2

    import torch
    from rust_llm_inference_server_amd.config import EngineConfig, preset_dict
    from rust_llm_inference_server_amd.engine import Engine, ModelRunner, StepEntry, random_model
    from rust_llm_inference_server_amd.ops import lib
    from rust_llm_inference_server_amd.sampling import SamplingParams

    torch.cuda.set_device(0)
    lib.load()
    cfg = preset_dict(args.model)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    # room for the timed steps themselves when they are more than the context holds
    longest = max(args.context, args.prefill_tokens, 4096, args.steps + args.warmup + 128)
    if args.serve:
        longest = max(longest, args.max_prompt + args.new_tokens)
    cfg["max_position_embeddings"] = min(cfg["max_position_embeddings"], longest + 64)
    page = 16
    K, W = args.steps, args.warmup
    elem = 2 if args.dtype == "bfloat16" else 4
    t_load = time.time()
    model = random_model(cfg, seed=0, dtype=args.dtype, max_positions=cfg["max_position_embeddings"])
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t_load:.1f}s", file=sys.stderr, flush=True)
    L, H, I = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"]
    nh, nkv, d, V = (cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                     cfg["vocab_size"])
    layer_params = (nh + 2 * nkv) * d * H + H * nh * d + 3 * H * I + 2 * H
    weight_bytes = (L * layer_params + V * H + H + (0 if cfg["tie_word_embeddings"] else V * H)) * elem
    kv_bytes_per_token = 2 * L * nkv * d * elem
    g = torch.Generator().manual_seed(0)

    def prompts(n, length):
        return [torch.randint(0, V, (length,), generator=g).tolist() for _ in range(n)]

    def decode_run(batch, context, steps, warmup):
        """tokens/s and ms/step of `steps` decode steps of `batch` requests, none of which goes
        beyond `context`.  Prompts are prefilled in portions under the engine's token budget
        while earlier requests already decode, so every request is given room for the steps
        that the prefill of the others takes; the timed steps are pure decode steps."""
        budget = max(args.max_batched_tokens, batch)
        prefill_steps = -(-batch * context // budget) + 1
        new_tokens = steps + warmup + prefill_steps + 1
        context = max(context, new_tokens + 16)           # more steps than the context holds
        prompt_len = context - new_tokens
        pages = batch * (-(-context // page) + 1) + 8
        engine = Engine(model, EngineConfig(max_num_seqs=max(batch, 1), max_batched_tokens=budget,
                                            num_pages=pages, block_size=page,
                                            max_seq_len=context + 8, watermark_pages=0))
        sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True)
        for p in prompts(batch, prompt_len):
            engine.add_request(p, sp)
        while engine.stats().prefill_tokens < batch * prompt_len or engine.stats().waiting:
            engine.step()                                     # prefill, in portions
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        before = copy.copy(engine.stats())
        t0 = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        after = copy.copy(engine.stats())
        if (after.generated_tokens - before.generated_tokens != batch * steps
                or after.prefill_tokens != before.prefill_tokens
                or after.preemptions != before.preemptions):
            raise RuntimeError("the timed steps were not pure decode steps of the whole batch")
        mean_ctx = prompt_len + (before.generated_tokens + after.generated_tokens) / 2 / batch
        return batch * steps / dt, dt / steps * 1e3, mean_ctx

    if args.serve:
        # ---- continuous batching: R requests, chunked prefill under the token budget ---------
        lens = torch.randint(args.min_prompt, args.max_prompt + 1, (args.requests,), generator=g).tolist()
        reqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in lens]
        pages = sum(-(-(n + args.new_tokens) // page) + 1 for n in lens) + 64
        sp = SamplingParams(max_tokens=args.new_tokens, ignore_eos=True, temperature=0.8, seed=1)
        best = None
        for trial in range(2):                       # the first run also captures the graphs
            engine = Engine(model, EngineConfig(
                max_num_seqs=args.requests, max_batched_tokens=max(args.max_batched_tokens, args.requests),
                num_pages=pages, block_size=page, max_seq_len=args.max_prompt + args.new_tokens + 8))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            outs = engine.generate(reqs, sp)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
            stats = engine.stats()
            print(f"[bench] serve run {trial}: {dt:.3f}s, {stats.steps} steps, "
                  f"{stats.preemptions} preemptions", file=sys.stderr, flush=True)
        generated = sum(len(o.token_ids) for o in outs)
        print(json.dumps({
            "metric": f"served tok/s, {args.requests} requests ({args.model} shape)",
            "value": round(generated / best, 1), "unit": "generated tokens/s", "n_gpus": 1,
            "seconds": round(best, 4), "higher_is_better": True,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
            "config": {"model": args.model, "layers": L, "layers_full": full_layers,
                       "requests": args.requests, "min_prompt": args.min_prompt,
                       "max_prompt": args.max_prompt, "new_tokens": args.new_tokens,
                       "max_batched_tokens": args.max_batched_tokens, "page_size": page,
                       "prompt_tokens": sum(lens), "generated_tokens": generated,
                       "steps": stats.steps, "mean_ttft_ms": round(
                           sum(o.ttft for o in outs) / len(outs) * 1e3, 1)},
            "total_tokens_per_s": round((generated + sum(lens)) / best, 1),
        }))
        return 0

    # ---- prefill: one prompt of T tokens in one step, last-row logits ------------------
    T = args.prefill_tokens
    runner = ModelRunner(model, num_pages=-(-T // page) + 1, page_size=page, max_num_seqs=1)
    prompt = prompts(1, T)[0]
    times = []
    for i in range(1 if args.skip_prefill else 4):
        runner.reserve(0, T)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry(0, prompt, [T - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.free(0)
    prefill_s = min(times[1:] or times)
    linear_flops = 2.0 * T * L * (layer_params - 2 * H)
    attn_flops = 4.0 * L * nh * d * T * (T + 1) / 2
    head_flops = 2.0 * V * H
    prefill_flops = linear_flops + attn_flops + head_flops
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(prefill_flops / prefill_s / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}
    del runner
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- headline: batch B near the benchmark context ------------------------------------
    value, ms_per_step, mean_ctx = decode_run(args.batch, args.context, K, W)
    step_bytes = weight_bytes + args.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_GBPS, 4)}
    print(f"[bench] decode b{args.batch}: {value:.0f} tok/s, {ms_per_step:.3f} ms/step",
          file=sys.stderr, flush=True)

    points = {}
    if not args.skip_points:
        for b in (1, 64):
            steps = min(K, 128)
            ctx = args.points_context + steps + W
            v, ms, _ = decode_run(b, ctx, steps, W)
            points[f"decode_b{b}"] = round(v, 1)
            print(f"[bench] decode b{b}: {v:.0f} tok/s, {ms:.3f} ms/step", file=sys.stderr, flush=True)

    print(json.dumps({
        "metric": f"decode tok/s at batch {args.batch} ({args.model} shape)", "value": round(value, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
        "config": {"model": args.model, "layers": L, "layers_full": full_layers, "hidden": H,
                   "heads": nh, "kv_heads": nkv, "head_dim": d, "intermediate": I, "vocab": V,
                   "global_batch": args.batch, "seq_len": args.context, "page_size": page,
                   "prefill_tokens": T, "points_context": args.points_context,
                   "parallelism": "single GPU"},
        "prefill": prefill, "roofline": roofline, "points": points,
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())
