"""Zepolix through the engine's own step function, cache manager, scheduler and entry point on the CPU (torch twins
of the kernels) against the plain implementation: configuration and weights, each mechanism, every way of cutting
and batching, pages and state slots used again, and greedy generation."""
import io
import json

import numpy as np
import pytest
import torch

import plain_zepolix as plain
import traces
from helpers import random_tokens
from llmserver_amd.config import ConfigError, UnsupportedModelError, config_from_dict
from llmserver_amd.engine.batch import StepEntry
from llmserver_amd.engine.replay import make_runner, replay
from llmserver_amd.parts import PagedAndStateSpec
from llmserver_amd.weights import build_model
from tiny_zepolix import CASES, ZA, ZB, model_folder, plain_logits, plain_model
from torch_ops import TorchOps


def runner_for(case, max_tokens, page=None, live=4):
    return make_runner(model_folder(case), "float32", max_tokens, page or CASES[case][2], device="cpu", ops=TorchOps(), max_live=live)


def run(case, steps, tmp_path, page=None):
    runner = runner_for(case, traces.peak_tokens(steps), page)
    report = io.StringIO()
    replay(runner, traces.to_lines(steps).splitlines(), str(tmp_path), report)
    runner.cache.check_invariants()
    assert not runner.cache.requests and runner.cache.state_slots_free() in (None, 4)
    assert all(free == group.pool.num_pages for free, group in zip(runner.cache.available_pages(), runner.cache.groups))
    return traces.collect(steps, str(tmp_path), CASES[case][0]["vocab"])


def check(case, results, requests, atol=3e-5):
    for (rid, position), logits in results.items():
        expected = plain_logits(case, tuple(requests[rid]))[position].numpy()
        np.testing.assert_allclose(logits, expected, atol=atol, rtol=2e-4, err_msg=f"{case} {rid} position {position}")
    assert len(results) == sum(len(tokens) for tokens in requests.values())


def requests_of(case, lengths, seed0=300):
    return {f"q{i}": random_tokens(CASES[case][0]["vocab"], n, seed0 + i) for i, n in enumerate(lengths)}


# -- configuration and weights ---------------------------------------------------------------------------------------
def test_the_configuration_reads_back_and_refuses_what_is_not_built():
    config = config_from_dict(dict(ZB))
    assert config_from_dict(config.to_dict()) == config
    assert config.canon_taps == 4 and config.layers[1].mlp is None and config.layers[0].mixer.rot_dims == 4
    assert config.layers[2].mlp.top == 4 and config.norm_eps == 1e-6
    other = json.loads(json.dumps(ZA))
    other["layers"][1]["type"] = "something else"
    with pytest.raises(UnsupportedModelError, match="something else"):
        config_from_dict(other)
    other = json.loads(json.dumps(ZA))
    del other["layers"][0]["mixer"]["kv_rank"]
    with pytest.raises(ConfigError, match="kv_rank"):
        config_from_dict(other)
    other = json.loads(json.dumps(ZA))
    other["layers"][0]["mixer"]["kv_rank"] = 300
    with pytest.raises(UnsupportedModelError, match="256"):
        config_from_dict(other)


def test_the_model_declares_the_checkpoints_tensors_and_its_caches():
    model = build_model(config_from_dict(dict(ZB)))
    names = set(model.param_specs())
    assert {"embed", "embed.norm", "final.norm", "head", "l0.mix.q", "l0.mix.dkv.norm", "l0.mix.sink", "l0.mix.g", "l0.canon1",
            "l0.ls1", "l0.ls2", "l0.dwa", "l0.mlp.router", "l0.mlp.e2.down", "l2.mlp.e3.gate", "l1.norm1"} <= names
    assert not {"l1.norm2", "l1.ls2", "l1.mlp.router", "l0.mlp.e3.gate"} & names
    assert model.param_specs()["l2.dwa"].shape == (4,) and model.param_specs()["l0.canon1"].shape == (64, 4)
    specs = model.cache_specs()
    assert all(isinstance(spec, PagedAndStateSpec) and spec.state.shape == (3, 64) for spec in specs.values())
    assert [spec.paged.head_dim for spec in specs.values()] == [48, 16, 48] and all(spec.paged.n_kv_heads == 1 for spec in specs.values())


# -- schedules ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("case", sorted(CASES))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_every_schedule_matches_the_plain_implementation(case, schedule, tmp_path):
    lengths = (5, 17, 33, 70, 41, 1, 64, 90, 20, 2) if schedule == "mixed" else (70, 33, 1, 2)
    requests = requests_of(case, lengths)
    if schedule == "whole":
        steps = traces.whole(requests)
    elif schedule == "tail":
        steps = traces.tail_decoded(requests, 32)
    elif schedule == "portions":
        steps = traces.changing_portions(requests, sizes=(2, 7, 1, 3, 33, 2, 2, 16, 5))
    else:
        steps = traces.mixed(requests, seed=11, budget_tokens=256)
        assert max(len(s["entries"]) for s in steps) >= 3 and sum(lengths) > traces.peak_tokens(steps)
    check(case, run(case, steps, tmp_path), requests)


def test_prefill_equals_token_by_token_decoding_from_the_first_token(tmp_path):
    """Every token alone, from position 0: the convolution's state, the cache rows and the sink all start from nothing."""
    requests = requests_of("ZB", (40,))
    check("ZB", run("ZB", traces.tail_decoded(requests, 64), tmp_path), requests)


@pytest.mark.parametrize("page", [4, 8, 64])
def test_page_sizes_and_page_borders(page, tmp_path):
    requests = requests_of("ZA", (2 * page + 1, page, page - 1, page + 1))
    steps = traces.changing_portions(requests, sizes=(page - 1, 2, page, 1, page + 1))
    check("ZA", run("ZA", steps, tmp_path, page=page), requests)


def test_state_slots_and_pages_are_used_again_in_any_order(tmp_path):
    """Eight requests through four slots: a slot's next holder must find zeros, not its predecessor's last inputs."""
    runner = runner_for("ZD", 4 * 64, live=4)
    tokens = {i: random_tokens(200, 30 + i, 900 + i) for i in range(8)}
    got = {}
    for first in (0, 4):
        live = list(range(first, first + 4))
        for rid in live:
            runner.cache.open(rid)
        slots = [runner.cache.record(rid).state_slot for rid in live]
        assert sorted(slots) == [0, 1, 2, 3]
        done = {rid: 0 for rid in live}
        turn = 0
        while any(done[rid] < len(tokens[rid]) for rid in live):
            entries = []
            for rid in live[::-1] if turn % 2 else live:
                size = (1, 3, 2, 7)[(rid + turn) % 4]
                if done[rid] < len(tokens[rid]):
                    piece = tokens[rid][done[rid]:done[rid] + size]
                    entries.append(StepEntry(rid, piece, list(range(len(piece)))))
            logits = runner.step(entries)
            row = 0
            for entry in entries:
                for _ in entry.tokens:
                    got[(entry.request_id, done[entry.request_id])] = logits[row].numpy()
                    done[entry.request_id] += 1
                    row += 1
            turn += 1
        for rid in live[::-1]:
            runner.cache.close(rid)
    for (rid, position), logits in got.items():
        expected = plain_logits("ZD", tuple(tokens[rid]))[position].numpy()
        np.testing.assert_allclose(logits, expected, atol=3e-5, rtol=2e-4, err_msg=f"{rid} {position}")


# -- mechanisms that random weights could hide ---------------------------------------------------------------------
def sharpened(case, change):
    """The case's tensors with ``change(tensors)`` applied, written to a folder of its own; (folder, config, tensors)."""
    import os
    import tempfile

    from safetensors.torch import save_file
    raw, tensors = plain_model(case)
    tensors = {name: tensor.clone() for name, tensor in tensors.items()}
    change(tensors)
    folder = tempfile.mkdtemp(prefix="llmserver_amd_test_sharp_")
    save_file({name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    return (folder, *plain.read_folder(folder))


def logits_of(folder, tokens, cuts, page=8):
    runner = make_runner(folder, "float32", 64 * (-(-len(tokens) // 64)), page, device="cpu", ops=TorchOps())
    runner.cache.open("r")
    rows, start = [], 0
    for size in cuts:
        piece = tokens[start:start + size]
        if not piece:
            break
        rows.append(runner.step([StepEntry("r", piece, list(range(len(piece))))]).clone())
        start += len(piece)
    assert start == len(tokens)
    return torch.cat(rows).numpy()


def test_a_far_key_among_hundreds_decides_and_is_found():
    """Queries and the shared rotated key part are scaled up so that attention is sharp: single keys far back decide
    the output, in a prompt and for decoded tokens."""
    def change(tensors):
        tensors["l0.mix.q"] *= 6.0
        tensors["l0.mix.dkv"] *= 3.0
    folder, raw, tensors = sharpened("ZA", change)
    tokens = random_tokens(97, 400, 5)
    expected = plain.forward(raw, tensors, tokens).numpy()
    blunt = plain.forward(*plain_model("ZA"), tokens).numpy()
    assert np.abs(expected - blunt).max() > 0.1
    for cuts in ([400], [380] + [1] * 20, [3, 250, 2, 100, 45]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=2e-4, rtol=5e-4)


def test_the_sink_takes_its_share_once():
    """Sinks far above the scores swallow a head's output, sinks far below change nothing; both against the oracle,
    and the two differ, so a sink that is left out (or counted per key range) shows."""
    results = []
    for value in (12.0, -40.0):
        def change(tensors, value=value):
            for index in range(3):
                tensors[f"l{index}.mix.sink"][:] = value
                tensors[f"l{index}.mix.sink"][0] = 0.5
        folder, raw, tensors = sharpened("ZA", change)
        tokens = random_tokens(97, 150, 6)
        expected = plain.forward(raw, tensors, tokens).numpy()
        for cuts in ([150], [120] + [1] * 30, [2, 70, 3, 75]):
            np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=5e-5, rtol=3e-4)
        results.append(expected)
    assert np.abs(results[0] - results[1]).max() > 0.05


def test_the_convolutions_reach_across_steps_and_starts():
    """Large taps: what a token reads of its predecessors decides the logits, whatever step the predecessors came in."""
    def change(tensors):
        tensors["l0.canon1"] = torch.tensor([[1.5, -2.0, 0.7, 1.1, 0.9]] * 32, dtype=torch.float64) * torch.linspace(0.5, 1.5, 32, dtype=torch.float64)[:, None]
    folder, raw, tensors = sharpened("ZE", change)
    tokens = random_tokens(50, 60, 9)
    expected = plain.forward(raw, tensors, tokens).numpy()
    assert np.abs(expected - plain.forward(*plain_model("ZE"), tokens).numpy()).max() > 0.05
    for cuts in ([60], [1] * 60, [2, 1, 3, 4, 5, 1, 1, 6, 2, 35], [4, 56], [5, 55], [3, 2, 55]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=5e-5, rtol=3e-4, err_msg=str(cuts))


def test_depth_weights_layer_scales_and_norm_offsets_matter_and_match():
    def change(tensors):
        tensors["l2.dwa"] = torch.tensor([0.9, -0.6, 0.4, 1.3], dtype=torch.float64)
        tensors["l1.dwa"] = torch.tensor([-0.5, 0.25, 1.5], dtype=torch.float64)
        tensors["l0.ls2"] *= 3.0
        tensors["l1.norm1"] -= 0.5
    folder, raw, tensors = sharpened("ZB", change)
    tokens = random_tokens(130, 50, 10)
    expected = plain.forward(raw, tensors, tokens).numpy()
    assert np.abs(expected - plain.forward(*plain_model("ZB"), tokens).numpy()).max() > 0.05
    for cuts in ([50], [20] + [1] * 30):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=5e-5, rtol=3e-4)


def test_router_choices_and_weights_follow_the_oracle():
    """A router scaled up makes the softmax over the chosen logits far from even; every token's experts are the oracle's."""
    def change(tensors):
        for index in range(3):
            tensors[f"l{index}.mlp.router"] *= 4.0
    folder, raw, tensors = sharpened("ZA", change)
    tokens = random_tokens(97, 80, 12)
    np.testing.assert_allclose(logits_of(folder, tokens, [33, 2, 45]), plain.forward(raw, tensors, tokens).numpy(), atol=5e-5, rtol=3e-4)


# -- the oracle itself -------------------------------------------------------------------------------------------------
def test_the_oracles_mechanisms_by_hand():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(plain.norm_around_zero(x, torch.tensor([0.0, 1.0], dtype=torch.float64), 0.0), torch.tensor([[3.0, 8.0]], dtype=torch.float64) / 12.5 ** 0.5)
    h = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    assert plain.short_convolution(h, torch.tensor([[1.0, 2.0, 3.0]], dtype=torch.float64)).flatten().tolist() == [3.0, 32.0, 321.0]
    quarter = plain.rotate_pairs(torch.tensor([[1.0, 0.0, 5.0]], dtype=torch.float64), torch.tensor([1]), 10.0, 2, torch.float64)
    assert torch.allclose(quarter, torch.tensor([[np.cos(1.0), np.sin(1.0), 5.0]], dtype=torch.float64))
    weights = plain.softmax_with_sink(torch.tensor([[0.0, float("-inf")]], dtype=torch.float64), torch.tensor([0.0], dtype=torch.float64))
    assert weights.tolist() == [[0.5, 0.0]]
    indices, shares = plain.route(torch.tensor([[1.0, 0.0]], dtype=torch.float64), torch.tensor([[1.0, 0], [3.0, 0], [2.0, 0]], dtype=torch.float64), 2)
    assert indices.tolist() == [[1, 2]] and torch.allclose(shares, torch.softmax(torch.tensor([[3.0, 2.0]], dtype=torch.float64), dim=-1))
    # a shift of all positions changes no score: the rotation enters through position differences only
    q, k = torch.randn(4, 6, dtype=torch.float64), torch.randn(4, 6, dtype=torch.float64)
    near = plain.rotate_pairs(q, torch.arange(4), 50.0, 6, torch.float64) @ plain.rotate_pairs(k, torch.arange(4), 50.0, 6, torch.float64).T
    far = plain.rotate_pairs(q, torch.arange(4) + 900, 50.0, 6, torch.float64) @ plain.rotate_pairs(k, torch.arange(4) + 900, 50.0, 6, torch.float64).T
    assert torch.allclose(near, far, atol=1e-9)


# -- generation through the entry point, the scheduler and the engine ------------------------------------------------------
def test_greedy_generation_through_the_entry_point_equals_the_oracles():
    """More requests than places, prompts cut into portions by the token budget, a pool so small that requests wait
    for pages: the engine's own scheduler, cache manager, step function and sampler produce the oracle's tokens."""
    from llmserver_amd.entrypoints import generate
    raw, tensors = plain_model("ZB")
    prompts = [random_tokens(130, n, 700 + n) for n in (19, 3, 41, 8, 1, 27)]
    expected = [plain.greedy_generate(raw, tensors, prompt, 7) for prompt in prompts]
    got = generate(model_folder("ZB"), prompts, max_new_tokens=7, dtype="float32", device="cpu", block_size=8, num_blocks=26,
                   max_batch_size=3, max_num_batched_tokens=24, prefill_chunk_size=16, ops=TorchOps())
    assert got == expected


def test_the_per_head_products_made_inside_the_kernels_give_the_same(tmp_path):
    """Steps of few tokens let the kernels around attention multiply with the heads' matrices themselves; the twins of
    that dataflow match the oracle like the batched products do."""
    ops = TorchOps()
    ops.inside = True
    requests = requests_of("ZB", (40, 9))
    steps = traces.tail_decoded(requests, 12)
    runner = make_runner(model_folder("ZB"), "float32", traces.peak_tokens(steps), 8, device="cpu", ops=ops)
    replay(runner, traces.to_lines(steps).splitlines(), str(tmp_path), io.StringIO())
    check("ZB", traces.collect(steps, str(tmp_path), CASES["ZB"][0]["vocab"]), requests)
