"""Zepolix on the GPU as a user runs it: ``bin/trace_run`` as a subprocess over the same requests whole, with a
decoded tail, in changing portions and mixed with others on a pool so small that pages and state slots are used
again; float32 against the plain implementation, bfloat16 against what the plain implementation loses when it rounds
where 16-bit kernels round; long decoding from the first token; greedy generation through the entry point."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_zepolix as plain
import traces
from helpers import random_tokens, relative_error
from tiny_zepolix import CASES, model_folder, plain_logits, plain_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu
BF16 = plain.rounding_to(torch.bfloat16)


def check_rounding(engine_errors, rounded_errors, what, factor=1.25):
    """A bfloat16 run against what the plain implementation loses when it rounds where 16-bit kernels round, position by
    position on the same sequences.  Routed experts make the spread heavy-tailed: where two router logits lie a rounding
    apart, either run may choose the other expert, each at places of its own, and such a place is off by many times the
    usual error, and so are the places behind it that attend to it: a handful of such events decides the tail of a few
    thousand places, so the two tails differ by a factor of two between seeds.  The median is therefore held tightly
    (within ``factor``), the 90th percentile within 1.3 times that, and the tail by its weight: at most 2.5 times as many
    places far off (ten times the rounded oracle's median) as the rounded oracle has, and two in a hundred."""
    engine, rounded = np.asarray(engine_errors, dtype=np.float64), np.asarray(rounded_errors, dtype=np.float64)
    assert np.isfinite(engine).all() and len(engine) >= 48, what
    middle = float(np.median(rounded))
    figures = {"median": (np.median(engine), middle, factor), "90th percentile": (np.quantile(engine, 0.9), np.quantile(rounded, 0.9), 1.3 * factor)}
    far = (float(np.mean(engine > 10 * middle)), float(np.mean(rounded > 10 * middle)))
    print(f"  {what}: " + ", ".join(f"{name} {ours:.2e} / {theirs:.2e}" for name, (ours, theirs, _) in figures.items()) +
          f", far off {far[0]:.3f} / {far[1]:.3f}", flush=True)
    for name, (ours, theirs, allowed) in figures.items():
        assert ours <= allowed * theirs, f"{what}: {name} error {ours:.3e} is more than {allowed} x the rounded oracle's {theirs:.3e}"
    assert far[0] <= 2.5 * far[1] + 0.02, f"{what}: {far[0]:.3f} of the places are far off, {far[1]:.3f} of the rounded oracle's"


def rounded_logits(case, tokens):
    raw, tensors = plain_model(case)
    return plain.forward(raw, tensors, list(tokens), r=BF16).numpy()


def run_trace(case, dtype, steps, tmp_path, max_tokens, page_size):
    out = tmp_path / f"out-{case}-{dtype}"
    command = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder(case), "--dtype", dtype,
               "--out", str(out), "--max-tokens", str(max_tokens), "--page-size", str(page_size)]
    done = subprocess.run(command, input=traces.to_lines(steps), capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    assert done.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    return traces.collect(steps, str(out), CASES[case][0]["vocab"])


def build_trace(case):
    vocab = CASES[case][0]["vocab"]
    requests, steps = {}, []

    def add(prefix, lengths, maker, seed0):
        mine = {f"{prefix}{i}": random_tokens(vocab, n, seed0 + i) for i, n in enumerate(lengths)}
        requests.update(mine)
        for step in maker(mine):
            step["step"] = len(steps)
            steps.append(step)

    base = (70, 33, 100, 1, 2)
    add("w", base, traces.whole, 100)
    add("t", base, lambda r: traces.tail_decoded(r, 32), 100)
    add("p", base, lambda r: traces.changing_portions(r, sizes=(2, 7, 1, 3, 33, 2, 2, 16, 5)), 100)
    add("m", (5, 17, 33, 70, 100, 41, 64, 1, 90, 130, 20, 77), lambda r: traces.mixed(r, seed=7, budget_tokens=256), 200)
    return steps, requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", sorted(CASES))
def test_all_schedules_match_the_plain_implementation(case, dtype, tmp_path):
    print(f"replay {case} {dtype}", flush=True)
    steps, requests = build_trace(case)
    results = run_trace(case, dtype, steps, tmp_path, traces.peak_tokens(steps), CASES[case][2])
    assert len(results) == sum(len(t) for t in requests.values())
    errors, lost = [], []
    for (rid, position), logits in results.items():
        expected = plain_logits(case, tuple(requests[rid]))[position].numpy()
        if dtype == "float32":
            np.testing.assert_allclose(logits, expected, atol=3e-5, rtol=2e-4, err_msg=f"{rid} position {position}")
        else:
            errors.append(relative_error(logits, expected))
    if errors:
        for rid, tokens in requests.items():
            exact = plain_logits(case, tuple(tokens)).numpy()
            lost += [relative_error(row, want) for row, want in zip(rounded_logits(case, tuple(tokens)), exact)]
        check_rounding(errors, lost, f"case {case} against the plain implementation")
    # the same request cut differently agrees with itself
    between = []
    for index in range(5):
        for position in range(len(requests[f"w{index}"])):
            for other in ("t", "p"):
                a, b = results[(f"w{index}", position)], results[(f"{other}{index}", position)]
                if dtype == "float32":
                    assert float(np.abs(a - b).max()) <= 1e-4 * max(1.0, float(np.abs(a).max())), (index, other, position)
                else:
                    between.append(relative_error(b, a))
    if between:
        check_rounding(between, lost, f"case {case} between two cuts of the same request", factor=2.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_from_the_first_token(dtype, tmp_path):
    """A one-token prompt decoded for 600 tokens: past the contexts that a workgroup merges itself, across many pages."""
    print(f"long decoding {dtype}", flush=True)
    case = "ZD"
    tokens = random_tokens(CASES[case][0]["vocab"], 601, 31)
    steps = traces.tail_decoded({"long": tokens}, tail=600)
    results = run_trace(case, dtype, steps, tmp_path, 640, 16)
    expected = plain_logits(case, tuple(tokens)).numpy()
    errors = []
    for position in range(601):
        if dtype == "float32":
            np.testing.assert_allclose(results[("long", position)], expected[position], atol=3e-5, rtol=2e-4, err_msg=f"position {position}")
        else:
            errors.append(relative_error(results[("long", position)], expected[position]))
    if errors:
        lost = [relative_error(row, want) for row, want in zip(rounded_logits(case, tuple(tokens)), expected)]
        check_rounding(errors, lost, "long decoding")


def test_greedy_generation_through_the_entry_point():
    from llmserver_amd.entrypoints import generate
    print("generation", flush=True)
    raw, tensors = plain_model("ZB")
    prompts = [random_tokens(130, n, 700 + n) for n in (19, 3, 41, 8, 1, 27)]
    expected = [plain.greedy_generate(raw, tensors, prompt, 7) for prompt in prompts]
    got = generate(model_folder("ZB"), prompts, max_new_tokens=7, dtype="float32", device="cuda", block_size=8, num_blocks=26,
                   max_batch_size=3, max_num_batched_tokens=24, prefill_chunk_size=16)
    assert got == expected
    rounded = generate(model_folder("ZB"), prompts, max_new_tokens=7, dtype="bfloat16", device="cuda", block_size=8)
    same = sum(a == b for g, e in zip(rounded, expected) for a, b in zip(g, e))
    assert same >= 0.6 * sum(len(e) for e in expected), (rounded, expected)


def test_the_benchmark_command_line_and_the_design_option_of_bench(tmp_path, capsys):
    """The framework's command line serves a Zepolix folder like any other (matrix of prompt lengths and batch sizes, one
    prompt's tokens equal to the oracle's; the mixed workload); ``bench.py --design zepolix`` prints one JSON line with
    every named size beside its dense neighbour (two layers each here)."""
    import json
    import subprocess

    from llmserver_amd.cli import benchmark
    print("command lines", flush=True)
    folder, raw = model_folder("ZD"), CASES["ZD"][0]
    report = tmp_path / "report.json"
    assert benchmark.main(["--model", folder, "--dtype", "float32", "--prompt-tokens", "9,40", "--batch-sizes", "1,3", "--output-tokens", "6",
                           "--repeats", "1", "--block-size", "16", "--json", str(report)]) == 0
    results = json.loads(report.read_text())["results"]
    assert [(r["prompt_tokens"], r["batch"]) for r in results] == [(9, 1), (9, 3), (40, 1), (40, 3)]
    config, tensors = plain_model("ZD")
    prompt = benchmark.matrix_prompts(raw["vocab"], 9, 1, "whole-run", 0, 0)[0]
    assert results[0]["tokens"][0] == plain.greedy_generate(config, tensors, prompt, 6)
    capsys.readouterr()
    assert benchmark.main(["--model", folder, "--mixed-requests", "6", "--mixed-prompt-range", "4,40", "--shared-prefix-tokens", "16",
                           "--output-tokens", "5", "--block-size", "8", "--max-num-batched-tokens", "64"]) == 0
    assert "mixed: 6 requests" in capsys.readouterr().out
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--design", "zepolix", "--layers", "2", "--steps", "4", "--warmup", "1",
                           "--prefill-tokens", "256"], capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-3000:]
    lines = [line for line in done.stdout.splitlines() if line.strip()]
    assert len(lines) == 1
    record = json.loads(lines[0])
    assert set(record["sizes"]) == {"zepolix-2k", "dense-2k", "zepolix-4k", "dense-4k"} and record["value"] > 0
    assert all(entry["layers"] == 2 and entry["decode_b8_tok_s"] > 0 and entry["prefill_256_ms"] > 0 for entry in record["sizes"].values())
