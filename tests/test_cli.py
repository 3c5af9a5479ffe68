"""The command line: option names and defaults are the reference's
(crates/server/src/main.rs:31-127), and both subcommands run a tiny random model on the GPU."""
import json
import os
import subprocess
import sys

import pytest

import plain_llama as plain
from rust_llm_inference_server_amd import cli

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_option_names_and_defaults_are_the_references():
    ap = cli.build_parser()
    g = ap.parse_args(["generate", "--model", "m", "--prompt-ids", "1 2"])
    # main.rs:46-61 (model), 63-86 (generate), 106-127 (engine)
    assert (g.max_seq_len, g.max_tokens, g.temperature, g.top_p, g.top_k, g.repetition_penalty,
            g.seed) == (2048, 128, 0.0, 1.0, 0, 1.0, None)
    assert (g.kv_cache_gb, g.block_size, g.max_num_seqs, g.max_batched_tokens, g.scheduler,
            g.attention, g.no_prefix_caching) == (1.0, 16, 64, 2048, "continuous", "v2", False)
    p = ap.parse_args(["perplexity", "--model", "m", "--ids-file", "f"])
    assert (p.ctx, p.max_windows) == (512, 0)             # main.rs:31-43
    assert ap.parse_args(["generate", "--page-size", "8", "--scheduler", "static"]).block_size == 8


@pytest.mark.parametrize("argv,message", [
    (["generate", "--dtype", "f16"], "f16"),
    (["generate", "--scheduler", "fair"], "invalid choice"),
    (["serve"], "invalid choice"),
])
def test_refused_options(argv, message, capsys):
    with pytest.raises(SystemExit):
        cli.build_parser().parse_args(argv)
    assert message in capsys.readouterr().err


def test_refused_runs():
    with pytest.raises(SystemExit, match="GPU only"):
        cli.main(["generate", "--device", "cpu", "--model", "m", "--prompt-ids", "1"])
    with pytest.raises(SystemExit, match="--random-weights needs --config"):
        cli.main(["generate", "--random-weights", "--prompt-ids", "1"])
    with pytest.raises(SystemExit, match="--model is required"):
        cli.main(["generate", "--prompt-ids", "1"])


@pytest.mark.gpu
def test_generate_prints_the_greedy_tokens(tiny_folders, capsys):
    folder = tiny_folders["b"]
    w, c = plain.read_weights(folder), plain.read_config(folder)
    prompt = [5, 17, 3, 99, 250, 7, 7, 12, 300]
    rc = cli.main(["generate", "--model", folder, "--dtype", "f32", "--max-seq-len", "128",
                   "--num-pages", "32", "--block-size", "8", "--max-tokens", "6",
                   "--prompt-ids", ",".join(map(str, prompt))])
    out = capsys.readouterr()
    assert rc == 0
    assert [int(t) for t in out.out.split()] == plain.greedy_generate(w, c, prompt, 6)
    assert "prompt 9 tok | output 6 tok (length) | ttft" in out.err and "tok/s" in out.err


@pytest.mark.gpu
def test_the_program_generates_and_scores(tiny_folders, tmp_path):
    """``bin/rlis`` as a child process: generation with a seeded temperature twice (the same
    tokens), and the perplexity report as JSON on standard output."""
    folder = tiny_folders["a"]
    w, c = plain.read_weights(folder), plain.read_config(folder)
    base = [sys.executable, os.path.join(ROOT, "bin", "rlis")]
    common = ["--model", folder, "--dtype", "f32", "--max-seq-len", "128"]
    runs = [subprocess.run(base + ["generate"] + common + [
        "--num-pages", "16", "--prompt-ids", "3 1 4 1 5", "--max-tokens", "5",
        "--temperature", "0.8", "--seed", "11"], capture_output=True, text=True, timeout=300)
        for _ in range(2)]
    assert all(r.returncode == 0 for r in runs), runs[0].stderr
    assert runs[0].stdout.split() == runs[1].stdout.split() and len(runs[0].stdout.split()) == 5
    tokens = [(7 * i + 3) % c["vocab_size"] for i in range(50)]
    ids = tmp_path / "ids.txt"
    ids.write_text(" ".join(map(str, tokens)))
    r = subprocess.run(base + ["perplexity"] + common + ["--ids-file", str(ids), "--ctx", "16",
                                                          "--bos", "1"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    report = json.loads(r.stdout.strip().splitlines()[-1])
    want = plain.perplexity(w, c, tokens, bos=1, ctx=16)
    assert report["windows"] == 3 and report["tokens_scored"] == want["tokens_scored"]
    assert abs(report["ppl"] - want["ppl"]) < 1e-4 * want["ppl"]
    assert "PPL = " in r.stderr


def test_bench_measures_one_gpu_only():
    """For more than one GPU bench.py prints one line that says so and exits with 2."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert len(r.stdout.strip().splitlines()) == 1 and "one GPU" in r.stdout


@pytest.mark.gpu
def test_bench_line_has_the_agreed_fields():
    """A short run at a reduced number of layers: one JSON line with the fields of the
    contract, a flat configuration of at most 20 keys that names both layer counts."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "2",
                        "--steps", "4", "--warmup", "2", "--context", "256"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "prefill", "roofline", "points"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 4 and rec["warmup"] == 2
    cfg = rec["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 2 and cfg["layers_full"] == 16
    assert set(rec["prefill"]) == {"value", "tokens", "ms", "frac"} and rec["prefill"]["tokens"] == 2048
    assert rec["roofline"]["bound"] == "hbm" and rec["roofline"]["peak"] == 8000.0
    assert abs(rec["roofline"]["frac"] - rec["roofline"]["achieved"] / 8000.0) < 1e-3
    assert {"decode_b1", "decode_b32", "decode_b64", "decode_b8_p512"} <= set(rec["points"])
    assert all(isinstance(v, (int, float)) for v in rec["points"].values())
    for name in ("decode_b1", "decode_b32", "decode_b64", "decode_b8_p512"):
        assert 0 < rec["points"][name + "_frac"] < 1
        # the metric's own workload whatever --steps says: 256 new tokens after prompts of
        # 512, timed after the warm-up steps, so a mean context of 512 + 2 + 129
        assert abs(rec["points"][name + "_ctx"] - 643) <= 1
    assert cfg["points_prompt"] == 512 and cfg["points_new_tokens"] == 256
    assert abs(rec["value"] - 8 / rec["ms_per_step"] * 1e3) < 0.01 * rec["value"]


@pytest.mark.gpu
def test_bench_serves_a_batch_of_requests():
    """The mode that the larger workloads run in (as child processes of the default run): a
    few requests through the engine, one JSON line with the decode steps timed on their own."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--serve", "--layers", "2",
                        "--requests", "6", "--min-prompt", "20", "--max-prompt", "90",
                        "--new-tokens", "24", "--max-batched-tokens", "64"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    assert rec["config"]["generated_tokens"] == 6 * 24 and rec["config"]["requests"] == 6
    assert rec["value"] > 0 and rec["total_tokens_per_s"] > rec["value"]
    assert rec["decode"]["steps"] > 0 and 0 < rec["decode"]["hbm_frac"] < 1
    assert 20 < rec["decode"]["context"] < 90 + 24


@pytest.mark.gpu
def test_smoke_entry_point(capsys):
    import __graft_entry__ as entry
    entry.smoke()
    assert "smoke ok" in capsys.readouterr().out
