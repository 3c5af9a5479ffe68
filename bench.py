"""Decode and prefill throughput of the Llama-3.2-1B shape on one MI355X, and the larger
workloads beside it.

    python bench.py --gpus 1 --steps K --warmup W

The headline value is decoded tokens per second at batch 8 with every request near the
benchmark context (4,096 positions): W untimed decode steps, then exactly K timed ones through
the engine (schedule, forward from the paged cache, on-device greedy sampling, token fed
back), bracketed by device synchronisation.  On the same line: a 2,048-token prefill (one
prompt in one step, the best of eight runs, the later of which replay the captured step) with its
fraction of the bf16 matrix peak, the decode step's achieved fraction of the HBM roofline
(bytes that must be read: every weight once plus the live requests' cache), and under
``points`` decode throughput at batch 1, 8, 32 and 64 over 256 new tokens after 512-token prompts,
whatever ``--steps`` says (each with its fraction of the HBM roofline, ``..._frac``, and the mean
context of its timed steps, ``..._ctx``) and, while the time budget lasts (``--extra-seconds``;
``--skip-extra`` leaves them out), three more workloads, each in a fresh model:

* ``serve_3b_...``: 64 requests with prompts of 128 to 2,048 tokens through the engine under
  continuous batching with a token budget of 512 (chunked prefill), 256 new tokens each, at the
  Llama-3.2-3B shape: generated tokens per second from the first arrival to the last end;
* ``long_8b_...``: 32 requests of 8,192 prompt tokens and 128 new tokens each at the
  Llama-3.1-8B shape: the same, plus tokens per second and HBM fraction of the steps that only
  decode (context about 8,256), and the prompt tokens per second of the steps before them;
* ``deep_8b_...``: the whole Llama-3.1-8B shape decoding at batch 4 with 32,768 positions each,
  and one prompt of 8,192 tokens in one step.

Each of them runs as a child process (the commands below): a failure there is reported on
stderr and leaves the headline as it is.
Weights are random (N(0, 0.02)), prompts are uniform random token ids.

    python bench.py --serve --model llama-3.2-3b --max-batched-tokens 512
    python bench.py --serve --model llama-3.1-8b --requests 32 --min-prompt 8192 \\
        --max-prompt 8192 --new-tokens 128 --max-batched-tokens 8192
    python bench.py --model llama-3.1-8b --batch 4 --context 32768 --prefill-tokens 8192 \
        --steps 32 --warmup 4 --skip-points

run one of those workloads alone and print its own JSON line."""
import argparse
import copy
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_GBPS = 8000.0            # MI355X HBM3E, published
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}
PAGE = 16


def say(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


class Shape:
    """Sizes of a preset and the bytes and flops that follow from them."""

    def __init__(self, cfg: dict, elem: int):
        self.cfg = cfg
        self.L, self.H, self.I = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"]
        self.nh, self.nkv, self.d = (cfg["num_attention_heads"], cfg["num_key_value_heads"],
                                     cfg["head_dim"])
        self.V = cfg["vocab_size"]
        self.layer_params = ((self.nh + 2 * self.nkv) * self.d * self.H + self.H * self.nh * self.d
                             + 3 * self.H * self.I + 2 * self.H)
        # What a decode step reads of the weights: the layers, the final norm and the output
        # head once (tied or not, it is one (V, H) matrix), and one row of the embedding table
        # per request; an untied model's embedding table is otherwise not touched.
        self.step_weight_bytes = (self.L * self.layer_params + self.V * self.H + self.H) * elem
        self.elem = elem
        self.kv_bytes_per_token = 2 * self.L * self.nkv * self.d * elem

    def decode_step_bytes(self, batch: int, mean_context: float) -> float:
        """What a decode step has to read: every weight it uses once and the live requests'
        cache."""
        return (self.step_weight_bytes + batch * self.H * self.elem
                + batch * mean_context * self.kv_bytes_per_token)

    def prefill_flops(self, T: int) -> float:
        linear = 2.0 * T * self.L * (self.layer_params - 2 * self.H)
        attention = 4.0 * self.L * self.nh * self.d * T * (T + 1) / 2
        return linear + attention + 2.0 * self.V * self.H


def build_model(name: str, dtype: str, layers, longest: int):
    import torch
    from rust_llm_inference_server_amd.config import preset_dict
    from rust_llm_inference_server_amd.engine import random_model
    cfg = preset_dict(name)
    full_layers = cfg["num_hidden_layers"]
    if layers:
        cfg["num_hidden_layers"] = layers
    cfg["max_position_embeddings"] = min(cfg["max_position_embeddings"], longest + 64)
    t0 = time.time()
    model = random_model(cfg, seed=0, dtype=dtype, max_positions=cfg["max_position_embeddings"])
    torch.cuda.synchronize()
    say(f"{name} ready in {time.time() - t0:.1f}s")
    return model, cfg, full_layers


def run_requests(model, shape: Shape, reqs, new_tokens: int, budget: int, trials: int = 2) -> dict:
    """``reqs`` through the engine under continuous batching with a token budget of ``budget``
    (chunked prefill), ``new_tokens`` each with seeded temperature sampling; timed from the
    first arrival to the last end (best of ``trials``) on an engine that has captured its
    decode steps before the first arrival, as a server does when it starts (``warm_up_s``).
    Steps that only decode, with every request live, are also timed on their own."""
    import torch
    from rust_llm_inference_server_amd.config import EngineConfig
    from rust_llm_inference_server_amd.engine import Engine
    from rust_llm_inference_server_amd.sampling import SamplingParams
    lens = [len(r) for r in reqs]
    pages = sum(-(-(n + new_tokens) // PAGE) + 1 for n in lens) + 64
    sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True, temperature=0.8, seed=1)
    best = None
    for trial in range(trials):
        engine = Engine(model, EngineConfig(
            max_num_seqs=len(reqs), max_batched_tokens=max(budget, len(reqs)), num_pages=pages,
            block_size=PAGE, max_seq_len=max(lens) + new_tokens + 8))
        torch.cuda.synchronize()
        t_warm = time.perf_counter()
        engine.warm_up()
        torch.cuda.synchronize()
        t_warm = time.perf_counter() - t_warm
        for r in reqs:
            engine.add_request(r, sp)
        decode_s = prefill_s = 0.0
        decode_steps = decode_tokens = 0
        context_sum = 0.0
        torch.cuda.synchronize()
        t0 = last = time.perf_counter()
        while engine.has_work():
            before = copy.copy(engine.stats())
            running = engine.scheduler.num_running
            engine.step()                      # ends with the sampled tokens on the host
            now = time.perf_counter()
            after = engine.stats()
            made = after.generated_tokens - before.generated_tokens
            if after.prefill_tokens != before.prefill_tokens:
                prefill_s += now - last
            elif running == len(reqs) and made == len(reqs):
                decode_s += now - last
                decode_steps += 1
                decode_tokens += made
                context_sum += (sum(lens) + after.generated_tokens) / len(reqs)
            last = now
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        stats = engine.stats()
        generated = stats.generated_tokens
        say(f"  run {trial}: {dt:.3f}s, {stats.steps} steps, {stats.preemptions} preemptions "
            f"(decode steps captured beforehand in {t_warm:.2f}s)")
        result = {
            "seconds": dt, "generated": generated, "prompt_tokens": sum(lens), "steps": stats.steps,
            "preemptions": stats.preemptions, "tok_s": generated / dt, "warm_up_s": t_warm,
            "total_tok_s": (generated + sum(lens)) / dt,
            "prefill_tok_s": stats.prefill_tokens / prefill_s if prefill_s else 0.0,
            "decode_steps": decode_steps,
            "decode_tok_s": decode_tokens / decode_s if decode_s else 0.0,
            "decode_ms": decode_s / decode_steps * 1e3 if decode_steps else 0.0,
        }
        if decode_steps:
            step_bytes = shape.decode_step_bytes(len(reqs), context_sum / decode_steps)
            result["decode_context"] = context_sum / decode_steps
            result["decode_frac"] = step_bytes / (decode_s / decode_steps) / 1e9 / HBM_GBPS
        if best is None or result["seconds"] < best["seconds"]:
            best = result
        del engine
    return best


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
    ap.add_argument("--points-context", type=int, default=512,
                    help="prompt length of the decode points at batch 1, 8, 32 and 64")
    ap.add_argument("--points-new-tokens", type=int, default=256,
                    help="timed decode steps of each of those points")
    ap.add_argument("--skip-points", action="store_true")
    ap.add_argument("--skip-prefill", action="store_true")
    ap.add_argument("--skip-extra", action="store_true",
                    help="leave out the 3B serving run and the 8B long-context run")
    ap.add_argument("--extra-seconds", type=float, default=150.0,
                    help="an extra workload starts only while the run is younger than this")
    ap.add_argument("--max-batched-tokens", type=int, default=8192,
                    help="token budget of the engine steps that prefill the decode runs")
    ap.add_argument("--serve", action="store_true",
                    help="time a batch of requests through the engine instead")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--min-prompt", type=int, default=128)
    ap.add_argument("--max-prompt", type=int, default=2048)
    ap.add_argument("--new-tokens", type=int, default=256)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (single-GPU engine)")
        return 2
    started = time.time()

    import torch
    from rust_llm_inference_server_amd.config import EngineConfig
    from rust_llm_inference_server_amd.engine import Engine, ModelRunner, StepEntry
    from rust_llm_inference_server_amd.ops import lib
    from rust_llm_inference_server_amd.sampling import SamplingParams

    torch.cuda.set_device(0)
    lib.load()
    K, W = args.steps, args.warmup
    elem = 2 if args.dtype == "bfloat16" else 4
    g = torch.Generator().manual_seed(0)

    def prompts(n, length, vocab):
        return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(n)]

    def random_requests(n, lo, hi, vocab):
        lens = torch.randint(lo, hi + 1, (n,), generator=g).tolist()
        return [torch.randint(0, vocab, (m,), generator=g).tolist() for m in lens]

    if args.serve:
        # ---- one workload of requests through the engine, alone ------------------------------
        model, cfg, full_layers = build_model(args.model, args.dtype, args.layers,
                                              args.max_prompt + args.new_tokens)
        shape = Shape(cfg, elem)
        reqs = random_requests(args.requests, args.min_prompt, args.max_prompt, shape.V)
        r = run_requests(model, shape, reqs, args.new_tokens, args.max_batched_tokens)
        print(json.dumps({
            "metric": f"served tok/s, {args.requests} requests ({args.model} shape)",
            "value": round(r["tok_s"], 1), "unit": "generated tokens/s", "n_gpus": 1,
            "seconds": round(r["seconds"], 4), "higher_is_better": True,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
            "config": {"model": args.model, "layers": shape.L, "layers_full": full_layers,
                       "requests": args.requests, "min_prompt": args.min_prompt,
                       "max_prompt": args.max_prompt, "new_tokens": args.new_tokens,
                       "max_batched_tokens": args.max_batched_tokens, "page_size": PAGE,
                       "prompt_tokens": r["prompt_tokens"], "generated_tokens": r["generated"],
                       "steps": r["steps"], "preemptions": r["preemptions"]},
            "total_tokens_per_s": round(r["total_tok_s"], 1),
            "prefill_tokens_per_s": round(r["prefill_tok_s"], 1),
            "warm_up_seconds": round(r["warm_up_s"], 3),
            "decode": {"steps": r["decode_steps"], "tokens_per_s": round(r["decode_tok_s"], 1),
                       "ms_per_step": round(r["decode_ms"], 4),
                       "context": round(r.get("decode_context", 0.0), 1),
                       "hbm_frac": round(r.get("decode_frac", 0.0), 4)},
        }))
        return 0

    # room for the timed steps themselves when they are more than the context holds
    longest = max(args.context, args.prefill_tokens, 4096, K + W + 128)
    model, cfg, full_layers = build_model(args.model, args.dtype, args.layers, longest)
    shape = Shape(cfg, elem)

    def decode_run(batch, context, steps, warmup, prompt_len=None):
        """tokens/s, ms/step and mean context of `steps` decode steps of `batch` requests, none
        of which goes beyond `context` (or, with `prompt_len`, after prompts of that length).
        Prompts are prefilled in portions under the engine's
        token budget while earlier requests already decode, so every request is given room for
        the steps that the prefill of the others takes; the timed steps are pure decode steps."""
        budget = max(args.max_batched_tokens, batch)
        if prompt_len is not None:
            budget = max(budget, batch * prompt_len)      # all prompts in one step
            context = prompt_len
        prefill_steps = -(-batch * context // budget) + 1
        new_tokens = steps + warmup + prefill_steps + 1
        if prompt_len is not None:
            context = prompt_len + new_tokens
        else:
            context = max(context, new_tokens + 16)       # more steps than the context holds
            prompt_len = context - new_tokens
        pages = batch * (-(-context // PAGE) + 1) + 8
        engine = Engine(model, EngineConfig(max_num_seqs=max(batch, 1), max_batched_tokens=budget,
                                            num_pages=pages, block_size=PAGE,
                                            max_seq_len=context + 8, watermark_pages=0))
        sp = SamplingParams(max_tokens=new_tokens, ignore_eos=True)
        # the decode steps' graphs are captured before the first request arrives, as a server
        # does when it starts (Engine.warm_up): the warm-up steps below are then replays
        engine.runner.capture_decode_steps(longest=context + 8, max_batch=batch)
        for p in prompts(batch, prompt_len, shape.V):
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

    # ---- prefill: one prompt of T tokens in one step, last-row logits ------------------
    T = args.prefill_tokens
    runner = ModelRunner(model, num_pages=-(-T // PAGE) + 1, page_size=PAGE, max_num_seqs=1)
    prompt = prompts(1, T, shape.V)[0]
    times = []
    # (eight: the engine captures a step whose shape has come back three times and replays it
    # from then on, as it does for a server that sees prompts of one length)
    for i in range(1 if args.skip_prefill else 8):
        runner.reserve(0, T)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry(0, prompt, [T - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.free(0)
    prefill_s = min(times[1:] or times)
    prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
               "frac": round(shape.prefill_flops(T) / prefill_s / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}
    del runner
    say(f"prefill {prefill}")

    # ---- headline: batch B near the benchmark context ------------------------------------
    value, ms_per_step, mean_ctx = decode_run(args.batch, args.context, K, W)
    achieved = shape.decode_step_bytes(args.batch, mean_ctx) / (ms_per_step * 1e-3) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_GBPS, 4)}
    say(f"decode b{args.batch}: {value:.0f} tok/s, {ms_per_step:.3f} ms/step, "
        f"{roofline['frac']:.3f} of HBM")

    points = {}
    if not args.skip_points:
        # the metric's own workload: 512-token prompts, then 256 new tokens at batch 1, 8, 32 and 64
        # (after W untimed decode steps, so the timed steps' mean context is 640 + W)
        for b in (1, 8, 32, 64):
            v, ms, mean = decode_run(b, 0, args.points_new_tokens, W, prompt_len=args.points_context)
            frac = shape.decode_step_bytes(b, mean) / (ms * 1e-3) / 1e9 / HBM_GBPS
            name = f"decode_b{b}" if b != args.batch else f"decode_b{b}_p{args.points_context}"
            points[name] = round(v, 1)
            points[name + "_frac"] = round(frac, 4)
            points[name + "_ctx"] = round(mean, 1)
            say(f"decode b{b}, {args.points_new_tokens} new tokens after {args.points_context}-token "
                f"prompts: {v:.0f} tok/s, {ms:.3f} ms/step, {frac:.3f} of HBM at mean context {mean:.0f}")

    # ---- the larger workloads, each in a model of its own ------------------------------------
    extras = [] if args.skip_extra or args.skip_points or args.layers else [
        ("serve_3b", "llama-3.2-3b", dict(n=64, lo=128, hi=2048, new=256, budget=512)),
        ("long_8b", "llama-3.1-8b", dict(n=32, lo=8192, hi=8192, new=128, budget=8192)),
    ]
    if extras:
        extras.append(("deep_8b", "llama-3.1-8b", None))
    for key, name, wl in extras:
        if time.time() - started > args.extra_seconds:
            say(f"{key}: left out, the run is older than {args.extra_seconds:.0f}s")
            continue
        if wl is None:
            # the whole 8B shape: decode at batch 4 with 32,768 positions, a prompt of 8,192
            cmd = [sys.executable, os.path.abspath(__file__), "--model", name, "--dtype", args.dtype,
                   "--batch", "4", "--context", "32768", "--prefill-tokens", "8192", "--steps", "32",
                   "--warmup", "4", "--skip-points"]
            try:
                child = subprocess.run(cmd, stdout=subprocess.PIPE, text=True, timeout=240)
                line = (child.stdout.strip().splitlines() or [""])[-1]
                if child.returncode != 0 or not line.startswith("{"):
                    raise RuntimeError(f"exit code {child.returncode}")
                r = json.loads(line)
                points[f"{key}_b4_ctx32k_tok_s"] = r["value"]
                points[f"{key}_b4_ctx32k_ms"] = r["ms_per_step"]
                points[f"{key}_b4_ctx32k_frac"] = r["roofline"]["frac"]
                points[f"{key}_prefill8192_tok_s"] = r["prefill"]["value"]
                points[f"{key}_prefill8192_frac"] = r["prefill"]["frac"]
                say(f"{key}: batch 4 at 32,768 positions {r['ms_per_step']:.2f} ms/step, "
                    f"{r['roofline']['frac']:.3f} of HBM; prefill of 8,192 tokens "
                    f"{r['prefill']['value']:.0f} tok/s, {r['prefill']['frac']:.3f} of the matrix peak")
            except Exception as exc:
                say(f"{key} failed: {type(exc).__name__}: {exc}")
            continue
        # A process of its own: whatever happens there, the headline below is printed.
        cmd = [sys.executable, os.path.abspath(__file__), "--serve", "--model", name, "--dtype",
               args.dtype, "--requests", str(wl["n"]), "--min-prompt", str(wl["lo"]), "--max-prompt",
               str(wl["hi"]), "--new-tokens", str(wl["new"]), "--max-batched-tokens",
               str(wl["budget"])]
        try:
            child = subprocess.run(cmd, stdout=subprocess.PIPE, text=True, timeout=240)
            line = (child.stdout.strip().splitlines() or [""])[-1]
            if child.returncode != 0 or not line.startswith("{"):
                raise RuntimeError(f"exit code {child.returncode}")
            r = json.loads(line)
            points[f"{key}_tok_s"] = r["value"]
            points[f"{key}_total_tok_s"] = r["total_tokens_per_s"]
            points[f"{key}_prefill_tok_s"] = r["prefill_tokens_per_s"]
            points[f"{key}_decode_tok_s"] = r["decode"]["tokens_per_s"]
            points[f"{key}_decode_ms"] = r["decode"]["ms_per_step"]
            points[f"{key}_decode_frac"] = r["decode"]["hbm_frac"]
            say(f"{key}: {r['value']:.0f} generated tok/s in {r['seconds']:.2f}s; decode steps "
                f"{r['decode']['ms_per_step']:.2f} ms, {r['decode']['tokens_per_s']:.0f} tok/s, "
                f"{r['decode']['hbm_frac']:.3f} of HBM at context {r['decode']['context']:.0f}; "
                f"prompts {r['prefill_tokens_per_s']:.0f} tok/s")
        except Exception as exc:
            say(f"{key} failed: {type(exc).__name__}: {exc}")

    print(json.dumps({
        "metric": f"decode tok/s at batch {args.batch} ({args.model} shape)", "value": round(value, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
        "config": {"model": args.model, "layers": shape.L, "layers_full": full_layers,
                   "hidden": shape.H, "heads": shape.nh, "kv_heads": shape.nkv, "head_dim": shape.d,
                   "intermediate": shape.I, "vocab": shape.V, "global_batch": args.batch,
                   "seq_len": args.context, "page_size": PAGE, "prefill_tokens": T,
                   "points_prompt": args.points_context, "points_new_tokens": args.points_new_tokens,
                   "parallelism": "single GPU"},
        "prefill": prefill, "roofline": roofline, "points": points,
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())
